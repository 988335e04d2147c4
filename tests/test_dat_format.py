"""NNEF tensor files: the library's host-side header functions against the reference's fixture files,
a `struct` restatement of nnef/src/tensors.rs, and closed forms.  No GPU needed."""
import os
import struct

import numpy as np
import pytest

import tract_amd
from oracle import oracle as orc
from tract_amd import dat

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
V0 = os.path.join(GOLD, "ref_sdpa", "simple-mask-f32", "v0.dat")
Q40 = os.path.join(GOLD, "nnef_dat", "linear__var0_q4_0.dat")


def test_reference_f32_fixture():
    data = open(V0, "rb").read()
    h = orc.dat_header_fields(data)
    assert h == {"magic": (0x4E, 0xEF), "version": (1, 0), "data_size_bytes": 8, "rank": 2, "dims": (2, 1),
                 "bits_per_item": 32, "item_type": 0, "item_type_vendor": 0, "rest_is_zero": True}
    item, shape, arr = dat.read_tensor(data)
    assert item == tract_amd.F32 and shape == (2, 1) and arr.dtype == np.float32
    assert arr.tobytes() == data[128:]
    # writing it back gives the file, byte for byte (the reference wrote it with write_tensor)
    assert dat.write_tensor(arr) == data == orc.dat_write_plain(arr)


def test_reference_q4_0_fixture_header_and_legacy_packing():
    data = open(Q40, "rb").read()
    h = orc.dat_header_fields(data)
    assert h["item_type_vendor"] == 0x5452 and h["item_type"] == 0x2040 and h["bits_per_item"] == 0xFFFFFFFF
    assert h["rank"] == 2 and h["dims"] == (16, 96) and h["data_size_bytes"] == 16 * 96 // 32 * 18 == len(data) - 128
    item, shape, blocks = dat.read_tensor(data)
    assert item == tract_amd.Q4_0 and shape == (16, 96) and blocks.size == 864
    # the older nibble order is converted on read: same bytes as the statement-by-statement restatement
    raw = np.frombuffer(data[128:], np.uint8)
    assert blocks.tobytes() == orc.q4_0_legacy_to_gguf(raw).tobytes() != raw.tobytes()
    assert blocks.reshape(-1, 18)[:, :2].tobytes() == raw.reshape(-1, 18)[:, :2].tobytes()   # scales untouched
    # The file holds the weight arange(16 * 96) quantised to Q4_0: after the conversion every element
    # dequantises to its own index within one quantisation step, in order.  (Without the conversion, or
    # with nibbles paired the wrong way, neighbouring elements land 16 apart.)
    w = orc.dequant(orc.FMT_Q4_0, blocks).reshape(-1, 32)
    step = np.abs(blocks.reshape(-1, 18)[:, :2].copy().view(np.float16).astype(np.float32))
    index = np.arange(16 * 96, dtype=np.float32).reshape(-1, 32)
    assert np.all(np.abs(w - index) <= step)
    unconverted = orc.dequant(orc.FMT_Q4_0, raw).reshape(-1, 32)
    assert not np.all(np.abs(unconverted - index) <= step)


def test_legacy_packing_is_sequential_nibbles():
    """Independent of the restated loop: build a block whose element i has code (i * 5) % 16 in the
    older layout (element i in nibble i % 2 of byte i / 2) and check, with the Q4_0 dequantiser that
    is pinned on the reference's known answers, that the converted block holds them in order."""
    codes = np.array([(i * 5) % 16 for i in range(32)], np.uint8)
    legacy = np.zeros(18, np.uint8)
    legacy[:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    for i, c in enumerate(codes):
        legacy[2 + i // 2] |= c << (4 * (i % 2))
    buf = legacy.copy()
    tract_amd._lib.call("trocm_dat_q4_0_legacy_to_gguf", buf.ctypes.data, buf.size)
    assert np.array_equal(orc.dequant(orc.FMT_Q4_0, buf), (codes.astype(np.float32) - 8) * 0.5)
    assert buf.tobytes() == orc.q4_0_legacy_to_gguf(legacy).tobytes()


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("shape", [(3,), (2, 8, 5, 64), (1, 1, 0, 4), ()])
def test_plain_round_trip_and_header_bytes(dt, shape):
    a = np.random.default_rng(1).standard_normal(shape).astype(dt)
    data = dat.write_tensor(a)
    assert data == orc.dat_write_plain(a)
    item, shp, back = dat.read_tensor(data)
    assert shp == tuple(shape) and back.dtype == dt and back.tobytes() == a.tobytes()


def test_block_quant_files():
    x = np.random.default_rng(2).standard_normal((2, 3, 5, 64)).astype(np.float32)
    q4 = orc.quant(orc.FMT_Q4_0, x)
    data = dat.write_block_quant(tract_amd.Q4_0, q4, x.shape)
    assert data == orc.dat_write_block_quant(0x3040, q4.tobytes(), x.shape)
    h = orc.dat_header_fields(data)
    assert h["rank"] == 2 and h["dims"] == (30, 64) and h["bits_per_item"] == 0xFFFFFFFF   # tensors.rs:305-312
    item, shape, blocks = dat.read_tensor(data)
    assert (item, shape) == (tract_amd.Q4_0, (30, 64)) and blocks.tobytes() == q4.tobytes()
    # Q8: the cache's 34-byte blocks go out as Q8_1 blocks of 36 bytes under the writer's item type
    q8 = orc.quant(orc.FMT_Q8_0, x)
    data = dat.write_block_quant(tract_amd.Q8_0, q8, x.shape)
    h = orc.dat_header_fields(data)
    assert h["item_type"] == 0x3081 and h["data_size_bytes"] == x.size // 32 * 36
    on_disk = np.frombuffer(data[128:], np.uint8).reshape(-1, 36)
    assert on_disk[:, :2].tobytes() == q8.reshape(-1, 34)[:, :2].tobytes()
    assert on_disk[:, 4:].tobytes() == q8.reshape(-1, 34)[:, 2:].tobytes()
    d = on_disk[:, :2].copy().view(np.float16).astype(np.float32)[:, 0]
    sums = on_disk[:, 4:].view(np.int8).astype(np.int32).sum(1)
    assert on_disk[:, 2:4].copy().view(np.float16)[:, 0].tobytes() == (d * sums).astype(np.float16).tobytes()
    item, shape, blocks = dat.read_tensor(data)
    assert item == tract_amd.Q8_0 and blocks.tobytes() == q8.tobytes()
    # ... and a file under the item type the reference's reader expects is read the same way
    alt = bytearray(data)
    struct.pack_into("<H", alt, 48, 0x3080)
    assert dat.read_tensor(bytes(alt))[2].tobytes() == q8.tobytes()
    # a real Q8_1 block from the oracle (sum of the unquantised values) loses only its sum
    q81 = orc.quant(orc.FMT_Q8_1, x)
    f = orc.dat_write_block_quant(0x3081, q81.tobytes(), x.shape)
    assert dat.read_tensor(f)[2].tobytes() == q8.tobytes()


def test_header_errors():
    good = bytearray(dat.write_tensor(np.zeros((2, 2), np.float32)))
    bad = bytearray(good)
    bad[0] = 0
    with pytest.raises(tract_amd.TractRocmError, match="Wrong magic number"):
        dat.read_tensor(bytes(bad))
    bad = bytearray(good)
    struct.pack_into("<I", bad, 8, 9)
    with pytest.raises(tract_amd.TractRocmError, match="Wrong tensor rank"):
        dat.read_tensor(bytes(bad))
    bad = bytearray(good)
    struct.pack_into("<I", bad, 4, 12)
    with pytest.raises(tract_amd.TractRocmError, match="Shape and len mismatch"):
        dat.read_tensor(bytes(bad))
    bad = bytearray(good)
    struct.pack_into("<H", bad, 48, 1)   # unsigned integers: not a tensor of this path
    with pytest.raises(tract_amd.TractRocmError, match="Unsupported type in tensor"):
        dat.read_tensor(bytes(bad))
    bad = bytearray(good)
    struct.pack_into("<H", bad, 50, 7)
    with pytest.raises(tract_amd.TractRocmError, match="item type vendor"):
        dat.read_tensor(bytes(bad))
    with pytest.raises(tract_amd.TractRocmError, match="truncated"):
        dat.read_tensor(bytes(good[:100]))
    with pytest.raises(tract_amd.TractRocmError, match="multiple of the block length"):
        dat.write_block_quant(tract_amd.Q4_0, np.zeros(18, np.uint8), (1, 33))
