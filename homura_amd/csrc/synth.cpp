// Deterministic synthetic tensors for tests and benchmarks (host side, no GPU involved).
//
// Counter-based: output n of a stream is mix64(seed + (n + 1) * GOLDEN), i.e. the n-th value
// of the splitmix64 sequence started at `seed`, so any slice can be produced independently
// and in parallel. A "normal" variate is the centred sum of twelve 16-bit uniform fields
// (Irwin-Hall; mean 0, variance 1 - 2^-32, support +-6) evaluated in integer arithmetic, so
// the bits are identical on every platform and compiler.
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>

#include "../../include/homura_amd_bench.h"

namespace {

constexpr uint64_t GOLDEN = 0x9E3779B97F4A7C15ULL;

inline uint64_t mix64(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}
inline uint64_t stream_at(uint64_t seed, uint64_t n) { return mix64(seed + (n + 1) * GOLDEN); }

inline int sum16(uint64_t v) {
    return (int)(v & 0xFFFF) + (int)((v >> 16) & 0xFFFF) + (int)((v >> 32) & 0xFFFF) +
           (int)(v >> 48);
}

inline float normal_at(uint64_t seed, uint64_t i) {
    const int s = sum16(stream_at(seed, 3 * i)) + sum16(stream_at(seed, 3 * i + 1)) +
                  sum16(stream_at(seed, 3 * i + 2));
    return (float)(s - 393210) * (1.0f / 65536.0f);  // exact in f32
}

template <typename F>
void parallel_for(size_t n, F f) {
    unsigned hw = std::thread::hardware_concurrency();
    unsigned nt = std::max(1u, std::min(hw ? hw : 1u, 16u));
    if (n < (size_t)1 << 16) nt = 1;
    if (nt == 1) {
        f((size_t)0, n);
        return;
    }
    std::vector<std::thread> th;
    const size_t per = (n + nt - 1) / nt;
    for (unsigned t = 0; t < nt; t++) {
        const size_t b = std::min(n, per * t), e = std::min(n, per * (t + 1));
        if (b < e) th.emplace_back([=] { f(b, e); });
    }
    for (auto &t : th) t.join();
}

}  // namespace

extern "C" {

uint16_t hm_f32_to_bf16_rne(float v) {
    uint32_t u;
    std::memcpy(&u, &v, 4);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu)) return (uint16_t)((u >> 16) | 0x40u);
    const uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

uint16_t hm_f32_to_f16_rne(float v) {
    uint32_t u;
    std::memcpy(&u, &v, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const uint32_t absu = u & 0x7FFFFFFFu;
    if (absu >= 0x7F800000u)  // inf / NaN
        return (uint16_t)(sign | 0x7C00u | (absu > 0x7F800000u ? 0x200u : 0u));
    if (absu >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);  // rounds to inf
    if (absu < 0x33000001u) return (uint16_t)sign;              // rounds to zero (<= 2^-25)
    const int exp = (int)(absu >> 23) - 127;
    uint32_t mant = (absu & 0x007FFFFFu) | 0x00800000u;  // 24-bit significand
    int shift;                                           // bits dropped from the significand
    uint32_t base;
    if (exp < -14) {  // subnormal half
        shift = 13 + (-14 - exp);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(exp + 15) << 10;
        mant &= 0x007FFFFFu;
    }
    uint32_t q = mant >> shift;
    const uint32_t rem = mant & ((1u << shift) - 1u);
    const uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q++;
    return (uint16_t)(sign | (base + q));  // a carry out of the mantissa bumps the exponent
}

void hm_synth_normal_f32(uint64_t seed, uint64_t first, size_t n, float scale, float *out) {
    parallel_for(n, [=](size_t b, size_t e) {
        for (size_t i = b; i < e; i++) out[i] = normal_at(seed, first + i) * scale;
    });
}

void hm_synth_normal_bf16(uint64_t seed, uint64_t first, size_t n, float scale, uint16_t *out) {
    parallel_for(n, [=](size_t b, size_t e) {
        for (size_t i = b; i < e; i++) out[i] = hm_f32_to_bf16_rne(normal_at(seed, first + i) * scale);
    });
}

void hm_synth_token_ids(uint64_t seed, size_t n, int vocab, int64_t *out) {
    for (size_t i = 0; i < n; i++)
        out[i] = (int64_t)(((stream_at(seed, i) >> 32) * (uint64_t)vocab) >> 32);
}

void hm_synth_q8_0(uint64_t seed, size_t n_blocks, float d_scale, uint8_t *out) {
    const uint64_t seed_d = seed ^ 0xD5CA1E5ULL;
    parallel_for(n_blocks, [=](size_t b0, size_t b1) {
        for (size_t b = b0; b < b1; b++) {
            uint8_t *blk = out + b * 34;
            float d = normal_at(seed_d, b) * d_scale;
            if (d < 0) d = -d;
            const uint16_t h = hm_f32_to_f16_rne(d);
            blk[0] = (uint8_t)(h & 0xFF);
            blk[1] = (uint8_t)(h >> 8);
            for (int w = 0; w < 8; w++) {
                const uint64_t r = stream_at(seed, b * 8 + w);
                for (int f = 0; f < 4; f++) {
                    const uint32_t u = (uint32_t)(r >> (16 * f)) & 0xFFFFu;
                    const int q = (int)((u * 255u) >> 16) - 127;  // uniform over [-127, 127]
                    blk[2 + w * 4 + f] = (uint8_t)(int8_t)q;
                }
            }
        }
    });
}

void hm_synth_q4_0(uint64_t seed, size_t n_blocks, float d_scale, uint8_t *out) {
    const uint64_t seed_d = seed ^ 0xD5CA1E5ULL;
    parallel_for(n_blocks, [=](size_t b0, size_t b1) {
        for (size_t b = b0; b < b1; b++) {
            uint8_t *blk = out + b * 18;
            float d = normal_at(seed_d, b) * d_scale;
            if (d < 0) d = -d;
            const uint16_t h = hm_f32_to_f16_rne(d);
            blk[0] = (uint8_t)(h & 0xFF);
            blk[1] = (uint8_t)(h >> 8);
            for (int w = 0; w < 2; w++) {
                const uint64_t r = stream_at(seed, b * 2 + w);  // 16 uniform nibbles
                std::memcpy(blk + 2 + w * 8, &r, 8);
            }
        }
    });
}

}  // extern "C"
