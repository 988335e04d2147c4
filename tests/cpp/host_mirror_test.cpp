// C++ twin of tract's unit tests for the in-place KV cache and the fused op
// (transformers/src/ops/inplace_kv_cache.rs:366-418, 456-491, 595-658, 898-942), run against
// the rocm library through the C++ host mirror.  References are written in the test, as the
// reference's own tests do: plain concatenation and naive f32 attention.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>
#include "tract_rocm.hpp"

using namespace trocm;

#define EXPECT(cond)                                                          \
    do {                                                                      \
        if (!(cond)) {                                                        \
            std::fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            return 1;                                                         \
        }                                                                     \
    } while (0)

// deterministic filler (seq_tensor of the reference tests)
static std::vector<float> seq_tensor(size_t n, float start) {
    std::vector<float> v(n);
    for (size_t i = 0; i < n; i++) v[i] = start + 0.001f * (float)(i % 977) - 0.3f * (float)(i % 7);
    return v;
}

// naive GQA attention over [B,H,S,D] f32, causal bottom-right aligned
static std::vector<float> naive(const std::vector<float> &q, const std::vector<float> &k, const std::vector<float> &v,
                                int B, int Hq, int Hkv, int Sq, int Sk, int D, bool causal) {
    std::vector<float> out((size_t)B * Hq * Sq * D);
    const float scale = 1.0f / std::sqrt((float)D);
    std::vector<float> s(Sk);
    for (int b = 0; b < B; b++)
        for (int h = 0; h < Hq; h++) {
            int kh = h / (Hq / Hkv);
            for (int i = 0; i < Sq; i++) {
                float mx = -INFINITY;
                int vis = causal ? std::min(Sk, i + (Sk - Sq) + 1) : Sk;
                for (int j = 0; j < vis; j++) {
                    float a = 0;
                    for (int d = 0; d < D; d++) a += q[(((size_t)b * Hq + h) * Sq + i) * D + d] * k[(((size_t)b * Hkv + kh) * Sk + j) * D + d];
                    s[j] = a * scale;
                    mx = std::fmax(mx, s[j]);
                }
                float sum = 0;
                for (int j = 0; j < vis; j++) sum += (s[j] = std::exp(s[j] - mx));
                for (int d = 0; d < D; d++) {
                    float a = 0;
                    for (int j = 0; j < vis; j++) a += s[j] * v[(((size_t)b * Hkv + kh) * Sk + j) * D + d];
                    out[(((size_t)b * Hq + h) * Sq + i) * D + d] = a / sum;
                }
            }
        }
    return out;
}

// concat along axis 2 of [B,H,*,D]
static void concat(std::vector<float> &acc, int &len, const std::vector<float> &x, int B, int H, int n, int D) {
    std::vector<float> out((size_t)B * H * (len + n) * D);
    for (int bh = 0; bh < B * H; bh++) {
        std::memcpy(&out[(size_t)bh * (len + n) * D], acc.data() + (size_t)bh * len * D, sizeof(float) * len * D);
        std::memcpy(&out[((size_t)bh * (len + n) + len) * D], x.data() + (size_t)bh * n * D, sizeof(float) * n * D);
    }
    acc.swap(out);
    len += n;
}

int main() {
    try {
        Runtime rt = runtime_for_name("rocm");
        rt.check();
        bool threw = false;
        try {
            runtime_for_name("cuda");
        } catch (const Error &) {
            threw = true;
        }
        EXPECT(threw);

        // inplace_matches_concat + realloc count (inplace_kv_cache.rs:366-418)
        {
            const int B = 1, H = 4, D = 16;
            InPlaceKvCache c(2);
            std::vector<float> ref;
            int len = 0;
            for (int step = 0; step < 1024; step++) {
                auto x = seq_tensor((size_t)B * H * D, (float)step);
                c.push(DeviceTensor::from_host(x.data(), {B, H, 1, D}, DatumType::F32));
                if (step < 70 || step == 1023) concat(ref, len, x, B, H, 1, D);
            }
            EXPECT(c.len() == 1024 && c.capacity() == 1024 && c.reallocs() <= 12);
            InPlaceKvCache c2(2);
            std::vector<float> ref2;
            int len2 = 0;
            int chunks[] = {3, 1, 7, 1, 30, 2};
            for (int n : chunks) {
                auto x = seq_tensor((size_t)B * H * n * D, (float)n);
                c2.push(DeviceTensor::from_host(x.data(), {B, H, n, D}, DatumType::F32));
                concat(ref2, len2, x, B, H, n, D);
                auto got = c2.valid_contiguous();
                EXPECT(got.size() == ref2.size() * 4 && std::memcmp(got.data(), ref2.data(), got.size()) == 0);
            }
            EXPECT(c2.len() == 44 && c2.capacity() == 84);  // 3 -> 6 -> 12 -> 42 -> 84
            // truncate + clone (dyn_kv_cache.rs:112-119, :262-272)
            InPlaceKvCache frozen = c2.clone();
            c2.truncate(10);
            EXPECT(c2.len() == 10 && frozen.len() == 44);
            bool bad = false;
            try {
                c2.truncate(11);
            } catch (const Error &) {
                bad = true;
            }
            EXPECT(bad);
        }

        // fused op vs {concat, naive attention}, GQA + causal, decode loop (inplace_kv_cache.rs:595-658)
        {
            const int B = 2, Hq = 8, Hkv = 2, D = 64;
            InPlaceKvSdpaState st = InPlaceKvSdpa{2, true, std::nullopt}.state();
            std::vector<float> kc, vc;
            int klen = 0, vlen = 0;
            double worst = 0;
            int lens[] = {40, 1, 1, 1, 5, 1};
            for (int n : lens) {
                auto q = seq_tensor((size_t)B * Hq * n * D, 0.1f * n), k = seq_tensor((size_t)B * Hkv * n * D, 0.2f * n),
                     v = seq_tensor((size_t)B * Hkv * n * D, 0.3f * n);
                for (auto &x : q) x *= 0.05f;
                for (auto &x : k) x *= 0.1f;
                DeviceTensor out = st.eval(DeviceTensor::from_host(q.data(), {B, Hq, n, D}, DatumType::F32),
                                           DeviceTensor::from_host(k.data(), {B, Hkv, n, D}, DatumType::F32),
                                           DeviceTensor::from_host(v.data(), {B, Hkv, n, D}, DatumType::F32));
                concat(kc, klen, k, B, Hkv, n, D);
                concat(vc, vlen, v, B, Hkv, n, D);
                std::vector<float> got(out.len());
                out.to_host(got.data());
                auto want = naive(q, kc, vc, B, Hq, Hkv, n, klen, D, true);
                for (size_t i = 0; i < got.size(); i++) worst = std::fmax(worst, std::fabs((double)got[i] - want[i]));
            }
            EXPECT(worst < 1e-3);
            // save / load resume is exact (inplace_kv_cache.rs:898-942)
            std::vector<std::vector<uint8_t>> saved;
            st.save_to(saved);
            EXPECT(saved.size() == 2 && saved[0].size() == kc.size() * 4);
            EXPECT(std::memcmp(saved[0].data(), kc.data(), saved[0].size()) == 0);
            EXPECT(std::memcmp(saved[1].data(), vc.data(), saved[1].size()) == 0);
            InPlaceKvSdpaState st2 = InPlaceKvSdpa{2, true, std::nullopt}.state();
            st2.load_from(DeviceTensor::from_host(saved[0].data(), {B, Hkv, klen, D}, DatumType::F32),
                          DeviceTensor::from_host(saved[1].data(), {B, Hkv, klen, D}, DatumType::F32));
            EXPECT(st2.k.len() == klen && st2.k.valid_contiguous() == saved[0]);
        }

        // Sdpa: mask rejected when causal (sdpa.rs:297-299)
        {
            auto x = seq_tensor(2 * 4 * 8, 0.f);
            DeviceTensor t = DeviceTensor::from_host(x.data(), {1, 2, 4, 8}, DatumType::F32);
            Sdpa op{std::nullopt, true};
            bool bad = false;
            try {
                op.eval(t, t, t, &t);
            } catch (const Error &e) {
                bad = std::string(e.what()).find("Mask cannot be provided") != std::string::npos;
            }
            EXPECT(bad);
            Sdpa nc{1.3f, false};
            DeviceTensor o = nc.eval(t, t, t);
            std::vector<float> got(o.len());
            o.to_host(got.data());
            EXPECT(std::isfinite(got[0]));
        }
        // window_holds_last_w_as_a_set + prefill_chunk_larger_than_window_keeps_last_w (window_kv_cache.rs:342-374)
        {
            const int w = 4;
            InPlaceKvCache c = InPlaceKvCache::window(2, w);
            for (int t = 0; t < 10; t++) {
                float x = (float)t;
                c.push(DeviceTensor::from_host(&x, {1, 1, 1, 1}, DatumType::F32));
                EXPECT(c.len() <= w);
                auto bytes = c.valid_contiguous();
                std::vector<float> got(bytes.size() / 4);
                std::memcpy(got.data(), bytes.data(), bytes.size());
                std::sort(got.begin(), got.end());
                for (size_t i = 0; i < got.size(); i++) EXPECT(got[i] == (float)(t + 1 - (int)got.size() + (int)i));
            }
            EXPECT(c.capacity() == w && c.cursor() == 10 % w);
            InPlaceKvCache big = InPlaceKvCache::window(2, 3);
            float chunk[7] = {0, 1, 2, 3, 4, 5, 6};
            big.push(DeviceTensor::from_host(chunk, {1, 1, 7, 1}, DatumType::F32));
            auto bytes = big.valid_contiguous();
            float got[3];
            std::memcpy(got, bytes.data(), 12);
            EXPECT(got[0] == 4.f && got[1] == 5.f && got[2] == 6.f && big.cursor() == 0);
        }

        // window_sdpa_decode_matches_last_w_in_model (window_kv_cache.rs:468-527)
        {
            const int B = 1, H = 2, D = 16, W = 5;
            WindowKvSdpaState st = WindowKvSdpa{2, W, std::nullopt}.state();
            auto mk = [&](float base) {
                std::vector<float> v((size_t)B * H * D);
                for (size_t i = 0; i < v.size(); i++) v[i] = base + std::sin((float)i * 0.013f);
                return v;
            };
            std::vector<float> kf, vf;
            int len = 0, vlen = 0;
            for (int t = 0; t < 15; t++) {
                auto q = mk(9.0f + t * 0.1f), k = mk(1.0f + t * 0.07f), v = mk(5.0f - t * 0.05f);
                DeviceTensor o = st.eval(DeviceTensor::from_host(q.data(), {B, H, 1, D}, DatumType::F32),
                                         DeviceTensor::from_host(k.data(), {B, H, 1, D}, DatumType::F32),
                                         DeviceTensor::from_host(v.data(), {B, H, 1, D}, DatumType::F32));
                std::vector<float> got(o.len());
                o.to_host(got.data());
                concat(kf, len, k, B, H, 1, D);
                concat(vf, vlen, v, B, H, 1, D);
                const int n = std::min(len, W);
                std::vector<float> kl((size_t)B * H * n * D), vl(kl.size());
                for (int bh = 0; bh < B * H; bh++)
                    for (int j = 0; j < n; j++) {
                        std::memcpy(&kl[((size_t)bh * n + j) * D], &kf[((size_t)bh * len + len - n + j) * D], sizeof(float) * D);
                        std::memcpy(&vl[((size_t)bh * n + j) * D], &vf[((size_t)bh * len + len - n + j) * D], sizeof(float) * D);
                    }
                auto want = naive(q, kl, vl, B, H, H, 1, n, D, false);
                for (size_t i = 0; i < want.size(); i++) EXPECT(std::fabs(want[i] - got[i]) <= 1e-3f);
            }
        }

        // test_rotate_half (apply_rope.rs:257-277) and ApplyRope against its definition
        {
            const int R = 10, C = 64;
            std::vector<float> x((size_t)R * C), cs(x.size()), sn(x.size());
            for (size_t i = 0; i < x.size(); i++) x[i] = (float)i, cs[i] = std::cos((float)i), sn[i] = std::sin((float)i);
            DeviceTensor dx = DeviceTensor::from_host(x.data(), {R, C}, DatumType::F32);
            DeviceTensor twice = RotateHalf{}.eval(RotateHalf{}.eval(dx));
            std::vector<float> back(x.size());
            twice.to_host(back.data());
            for (size_t i = 0; i < x.size(); i++) EXPECT(-back[i] == x[i]);
            DeviceTensor y = ApplyRope{}.eval(dx, DeviceTensor::from_host(cs.data(), {R, C}, DatumType::F32),
                                              DeviceTensor::from_host(sn.data(), {R, C}, DatumType::F32));
            std::vector<float> got(x.size());
            y.to_host(got.data());
            for (int r = 0; r < R; r++)
                for (int c = 0; c < C; c++) {
                    size_t i = (size_t)r * C + c;
                    float rot = c < C / 2 ? -x[i + C / 2] : x[i - C / 2];
                    volatile float a = x[i] * cs[i];   // each operation rounded on its own, like the CPU op
                    volatile float b = rot * sn[i];
                    EXPECT(got[i] == a + b);
                }
            DeviceTensor h = Cast{DatumType::F16}.eval(dx);
            DeviceTensor f = Cast{DatumType::F32}.eval(h);
            std::vector<float> rt2(x.size());
            f.to_host(rt2.data());
            for (size_t i = 0; i < x.size(); i++) EXPECT(rt2[i] == x[i]);   // integers up to 2048 are exact in f16
        }
        // Q4_0 weights x activations: every block holds the nibbles i % 16 (the table of q4_0.rs:722-739),
        // so sums over whole blocks and single elements are known in closed form
        {
            const int N = 4, K = 96;
            const float scales[N] = {0.5f, 0.25f, 1.0f, 2.0f};
            const uint16_t scale_bits[N] = {0x3800, 0x3400, 0x3C00, 0x4000};
            std::vector<uint8_t> blocks((size_t)N * (K / 32) * 18);
            for (int j = 0; j < N; j++)
                for (int b = 0; b < K / 32; b++) {
                    uint8_t *blk = &blocks[((size_t)j * (K / 32) + b) * 18];
                    blk[0] = (uint8_t)(scale_bits[j] & 0xff), blk[1] = (uint8_t)(scale_bits[j] >> 8);
                    for (int i = 0; i < 16; i++) blk[2 + i] = (uint8_t)((i % 16) | (((16 + i) % 16) << 4));
                }
            Q40Weights w(blocks.data(), 1, N, K);
            std::vector<float> ones(K, 1.0f), e(K, 0.0f), got(N);
            GgmlGemm{}.eval(DeviceTensor::from_host(ones.data(), {1, 1, K}, DatumType::F32), w).to_host(got.data());
            for (int j = 0; j < N; j++) EXPECT(got[j] == scales[j] * -48.0f);   // 3 blocks x sum(i % 16 - 8) = 3 x -16
            e[37] = 1.0f;   // block 1, element 5: (5 - 8) * d
            GgmlGemm{}.eval(DeviceTensor::from_host(e.data(), {1, 1, K}, DatumType::F32), w).to_host(got.data());
            for (int j = 0; j < N; j++) EXPECT(got[j] == scales[j] * -3.0f);
            e[37] = 0.0f, e[16] = 1.0f;   // a high nibble: element 16 has code 0
            GgmlGemm{}.eval(DeviceTensor::from_host(e.data(), {1, 1, K}, DatumType::F32), w).to_host(got.data());
            for (int j = 0; j < N; j++) EXPECT(got[j] == scales[j] * -8.0f);
        }
        // quant_cache_accumulates_near_lossless_int8 (quant_dyn_kv_cache.rs:728-756): 40 single-token steps through the
        // quantised cache op, Values then Keys; every output is the concatenation so far within SuperApproximate
        // (atol 0.1, rtol 0.05), and here within half an 8-bit step of data in [-0.5, 0.5)
        for (int per_channel = 0; per_channel < 2; per_channel++) {
            const int B = 1, H = 2, D = 8;
            QuantizedDynKvCacheState st = QuantizedDynKeyValueCache{"kv0", 2, 8, per_channel != 0}.state();
            uint64_t lcg = 3;
            auto nf = [&]() {
                lcg = lcg * 6364136223846793005ull + 1;
                return (float)(lcg >> 40) / (float)(1ull << 24) - 0.5f;
            };
            std::vector<float> acc;
            int len = 0;
            for (int t = 0; t < 40; t++) {
                std::vector<float> step((size_t)B * H * D);
                for (auto &x : step) x = nf();
                DeviceTensor out = st.eval(DeviceTensor::from_host(step.data(), {B, H, 1, D}, DatumType::F32));
                concat(acc, len, step, B, H, 1, D);
                EXPECT(out.shape()[2] == len && st.resolve_symbols() == len);
                std::vector<float> got(out.len());
                out.to_host(got.data());
                for (size_t i = 0; i < got.size(); i++) {
                    EXPECT(std::fabs(got[i] - acc[i]) <= 0.1f + 0.05f * std::fabs(acc[i]));
                    EXPECT(std::fabs(got[i] - acc[i]) <= 0.5f / 255.0f + 1e-6f);
                }
                if (t < 4) for (size_t i = 0; i < got.size(); i++) EXPECT(got[i] == acc[i]);   // sink tokens are kept in f32
            }
            QuantizedDynKvCacheState frozen = st.freeze();
            EXPECT(frozen.resolve_symbols() == 40);
        }
        // quantized_kv_sdpa_runs_in_model (kv_quant.rs:568-650): 10 decode steps of the fused op against f32 attention
        // over the growing cache, within SuperApproximate
        {
            const int B = 1, H = 2, D = 16;
            QuantizedKvSdpaState st = QuantizedKvSdpa{2, std::nullopt}.state();
            auto mk = [&](float base) {
                std::vector<float> v((size_t)B * H * D);
                for (size_t i = 0; i < v.size(); i++) v[i] = base + std::sin((float)i * 0.013f);
                return v;
            };
            std::vector<float> kf, vf;
            int len = 0, vlen = 0;
            for (int t = 0; t < 10; t++) {
                auto q = mk(9.0f + t * 0.1f), k = mk(1.0f + t * 0.07f), v = mk(5.0f - t * 0.05f);
                DeviceTensor o = st.eval(DeviceTensor::from_host(q.data(), {B, H, 1, D}, DatumType::F32),
                                         DeviceTensor::from_host(k.data(), {B, H, 1, D}, DatumType::F32),
                                         DeviceTensor::from_host(v.data(), {B, H, 1, D}, DatumType::F32));
                std::vector<float> got(o.len());
                o.to_host(got.data());
                concat(kf, len, k, B, H, 1, D);
                concat(vf, vlen, v, B, H, 1, D);
                auto want = naive(q, kf, vf, B, H, H, 1, len, D, false);
                for (size_t i = 0; i < want.size(); i++) EXPECT(std::fabs(want[i] - got[i]) <= 0.1f + 0.05f * std::fabs(want[i]));
            }
            EXPECT(st.k.memory_bytes() == (size_t)B * H * (10 * D + D * 8));    // memory_bytes, kv_quant.rs:233-235
            EXPECT(st.v.memory_bytes() == (size_t)B * H * (10 * D + 10 * 8));   // kv_quant.rs:160-162
        }
        std::printf("host_mirror_test: all checks passed\n");
        return 0;
    } catch (const std::exception &e) {
        std::fprintf(stderr, "host_mirror_test: exception: %s\n", e.what());
        return 2;
    }
}
