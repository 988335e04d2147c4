// NNEF tensor files (".dat") for the tensors of this path: f32 / f16 tensors and Q4_0 / Q8 block-quantised
// values, as tract reads and writes them (nnef/src/tensors.rs).  Host code only; it is what
// save_to / load_from of a cache state use so that a quantised cache round-trips without being
// dequantised.
//
//   header  : 128 bytes, little endian (tensors.rs:10-25): magic 4E EF, version 1.0, data_size_bytes,
//             rank, dims[8], bits_per_item, item_type, item_type_vendor, 32 + 44 bytes of zeros
//   f32/f16 : vendor 0, item_type 0, bits 32 / 16, payload = the elements (tensors.rs:96-99, 196-233)
//   Q4_0    : vendor 'TR' (0x5452), item_type 0x3040, bits 0xFFFFFFFF, shape flattened to
//             [product of the leading dims, last dim], payload = the 18-byte blocks (tensors.rs:300-322).
//             item_type 0x2040 is the older nibble order, converted on read (tensors.rs:250-273, 290-292).
//   Q8      : tract's 8-bit block format is Q8_1 (36-byte blocks: d, sum, 32 codes).  Its writer emits
//             item_type 0x3081 (tensors.rs:319) while its reader accepts 0x3080 (tensors.rs:278); this
//             code writes what the writer writes and reads both.  The cache's Q8_0 blocks are Q8_1
//             blocks without the sum; on the way out the sum is recomputed from the codes (d * sum of
//             codes, rounded to f16) -- tract computes it from the unquantised values, which a cache
//             no longer has, and never reads it back (q8_1.rs:52-59).
#include <string.h>
#include "common.h"

namespace trocm {
namespace {

struct DatHeader {
    uint8_t magic[2];
    uint8_t version_maj, version_min;
    uint32_t data_size_bytes;
    uint32_t rank;
    uint32_t dims[8];
    uint32_t bits_per_item;
    uint16_t item_type;
    uint16_t item_type_vendor;
    uint8_t item_type_params_deprecated[32];
    uint32_t padding[11];
};
static_assert(sizeof(DatHeader) == 128, "the NNEF tensor header is 128 bytes");   // tensors.rs:333-335

constexpr uint16_t kVendorTract = ((uint16_t)'T' << 8) | (uint16_t)'R';   // tensors.rs:8

}  // namespace
}  // namespace trocm

using namespace trocm;

extern "C" {

int trocm_dat_header_write(void *dst128, int item, int rank, const int64_t *dims, size_t data_bytes) {
    TROCM_NOT_NULL(dst128);
    TROCM_NOT_NULL(dims);
    TROCM_REQUIRE(rank >= 0 && rank <= 8, "Only rank up to 8 are supported");   // tensors.rs:191-193
    DatHeader h;
    memset(&h, 0, sizeof(h));
    h.magic[0] = 0x4e, h.magic[1] = 0xef, h.version_maj = 1, h.version_min = 0;
    uint64_t len = 1;
    for (int d = 0; d < rank; d++) {
        TROCM_REQUIRE(dims[d] >= 0 && dims[d] <= 0xffffffffll, "dat: dimension %d out of range", d);
        len *= (uint64_t)dims[d];
    }
    TROCM_REQUIRE(data_bytes <= 0xffffffffull, "dat: %zu bytes do not fit the header's 32-bit size", data_bytes);
    if (item == TROCM_F32 || item == TROCM_F16) {
        const uint64_t es = item == TROCM_F32 ? 4 : 2;
        TROCM_REQUIRE(len * es == data_bytes, "dat: shape and size mismatch (%llu elements, %zu bytes)",
                      (unsigned long long)len, data_bytes);
        h.rank = (uint32_t)rank;
        for (int d = 0; d < rank; d++) h.dims[d] = (uint32_t)dims[d];
        h.bits_per_item = (uint32_t)(es * 8);
        h.item_type = 0, h.item_type_vendor = 0;
    } else if (item == TROCM_Q4_0 || item == TROCM_Q8_0) {
        TROCM_REQUIRE(rank >= 1, "dat: a block-quantised value needs rank >= 1");
        const uint64_t k = (uint64_t)dims[rank - 1], m = k ? len / k : 0;
        const uint64_t bb = item == TROCM_Q4_0 ? 18 : 36;
        TROCM_REQUIRE(k % 32 == 0, "dat: the last dimension (%llu) must be a multiple of the block length 32",
                      (unsigned long long)k);
        TROCM_REQUIRE(m * k / 32 * bb == data_bytes, "dat: shape and size mismatch (%llu blocks of %llu bytes, %zu bytes)",
                      (unsigned long long)(m * k / 32), (unsigned long long)bb, data_bytes);
        h.rank = 2;                                       // tensors.rs:305-311: flattened to [m, k]
        h.dims[0] = (uint32_t)m, h.dims[1] = (uint32_t)k;
        h.bits_per_item = 0xffffffffu;                    // tensors.rs:312
        h.item_type_vendor = kVendorTract;
        h.item_type = item == TROCM_Q4_0 ? 0x3040 : 0x3081;   // tensors.rs:316
    } else {
        return fail("dat: unsupported item kind %d", item);
    }
    h.data_size_bytes = (uint32_t)data_bytes;
    memcpy(dst128, &h, sizeof(h));
    return 0;
}

int trocm_dat_header_read(const void *src128, int *item, int *rank, int64_t *dims8, size_t *data_bytes, int *flags) {
    TROCM_NOT_NULL(src128);
    TROCM_NOT_NULL(item);
    TROCM_NOT_NULL(rank);
    TROCM_NOT_NULL(dims8);
    TROCM_NOT_NULL(data_bytes);
    DatHeader h;
    memcpy(&h, src128, sizeof(h));
    TROCM_REQUIRE(h.magic[0] == 0x4e && h.magic[1] == 0xef, "Wrong magic number");                 // tensors.rs:48-50
    TROCM_REQUIRE(!(h.version_maj != 1 && h.version_min != 0), "Wrong version number");            // tensors.rs:51-53
    TROCM_REQUIRE(h.rank <= 8, "Wrong tensor rank %u", h.rank);                                    // tensors.rs:54-56
    uint64_t len = 1;
    for (uint32_t d = 0; d < h.rank; d++) {
        dims8[d] = h.dims[d];
        len *= h.dims[d];
    }
    TROCM_REQUIRE(h.item_type_vendor == 0 || h.item_type_vendor == kVendorTract, "Unknownn item type vendor %u",
                  h.item_type_vendor);                                                             // tensors.rs:91-93
    int fl = 0;
    if (h.item_type_vendor == 0 && h.item_type == 0 && (h.bits_per_item == 32 || h.bits_per_item == 16)) {
        *item = h.bits_per_item == 32 ? TROCM_F32 : TROCM_F16;
        TROCM_REQUIRE(len * (h.bits_per_item / 8) == h.data_size_bytes, "Shape and len mismatch: bits_per_item:%u, bytes:%u",
                      h.bits_per_item, h.data_size_bytes);                                         // tensors.rs:78-89
    } else if (h.item_type_vendor == kVendorTract && (h.item_type == 0x2040 || h.item_type == 0x3040 ||
                                                       h.item_type == 0x3080 || h.item_type == 0x3081)) {
        const bool q4 = h.item_type == 0x2040 || h.item_type == 0x3040;
        *item = q4 ? TROCM_Q4_0 : TROCM_Q8_0;
        if (h.item_type == 0x2040) fl |= TROCM_DAT_LEGACY_Q4_PACKING;
        if (!q4) fl |= TROCM_DAT_Q8_1_BLOCKS;
        TROCM_REQUIRE(h.rank >= 2, "block-quantised value of rank %u", h.rank);                   // tensors.rs:282
        const uint64_t m = h.dims[0], k = m ? len / m : 0;
        TROCM_REQUIRE(k % 32 == 0, "block-quantised row of %llu elements", (unsigned long long)k); // tensors.rs:288
        TROCM_REQUIRE(m * k / 32 * (q4 ? 18 : 36) == h.data_size_bytes, "block-quantised value: %u bytes for shape",
                      h.data_size_bytes);                                                          // tensors.rs:289-295
    } else {
        return fail("Unsupported type in tensor type:%u bits_per_item:%u", h.item_type, h.bits_per_item);  // tensors.rs:147-151
    }
    *rank = (int)h.rank;
    *data_bytes = h.data_size_bytes;
    if (flags) *flags = fl;
    return 0;
}

// tract_to_gguf_q4_0_packing (tensors.rs:250-273): the older files keep element i of a block in nibble
// i % 2 of byte i / 2; the current layout keeps element j in the low and element j + 16 in the high
// nibble of byte j.  In place.
int trocm_dat_q4_0_legacy_to_gguf(void *blocks, size_t bytes) {
    TROCM_REQUIRE(bytes % 18 == 0, "%zu bytes is not a whole number of Q4_0 blocks", bytes);
    if (bytes == 0) return 0;
    TROCM_NOT_NULL(blocks);
    uint8_t *p = (uint8_t *)blocks;
    for (size_t b = 0; b < bytes / 18; b++) {
        uint8_t *nib = p + b * 18 + 2;
        uint8_t elems[32];
        for (int i = 0; i < 32; i++) elems[i] = (i % 2 == 0) ? (nib[i / 2] & 0x0f) : (nib[i / 2] >> 4);
        for (int j = 0; j < 16; j++) nib[j] = (uint8_t)(elems[j] | (elems[j + 16] << 4));
    }
    return 0;
}

// Q8_1 blocks (36 bytes: d, sum, codes) <-> the cache's Q8_0 blocks (34 bytes: d, codes).  Host memory.
int trocm_q8_1_to_q8_0(const void *src, void *dst, size_t n_blocks) {
    if (n_blocks == 0) return 0;
    TROCM_NOT_NULL(src);
    TROCM_NOT_NULL(dst);
    const uint8_t *s = (const uint8_t *)src;
    uint8_t *d = (uint8_t *)dst;
    for (size_t b = 0; b < n_blocks; b++) {
        memcpy(d + b * 34, s + b * 36, 2);
        memcpy(d + b * 34 + 2, s + b * 36 + 4, 32);
    }
    return 0;
}

int trocm_q8_0_to_q8_1(const void *src, void *dst, size_t n_blocks) {
    if (n_blocks == 0) return 0;
    TROCM_NOT_NULL(src);
    TROCM_NOT_NULL(dst);
    const uint8_t *s = (const uint8_t *)src;
    uint8_t *d = (uint8_t *)dst;
    for (size_t b = 0; b < n_blocks; b++) {
        _Float16 scale;
        memcpy(&scale, s + b * 34, 2);
        int sum = 0;
        for (int i = 0; i < 32; i++) sum += (int8_t)s[b * 34 + 2 + i];
        const _Float16 hs = (_Float16)((float)scale * (float)sum);
        memcpy(d + b * 36, &scale, 2);
        memcpy(d + b * 36 + 2, &hs, 2);
        memcpy(d + b * 36 + 4, s + b * 34 + 2, 32);
    }
    return 0;
}

}  // extern "C"
