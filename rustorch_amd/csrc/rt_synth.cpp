// Seeded synthetic GGUF tensor payloads (host code, no GPU involved).
//
// Every 64-bit word is a pure function of (seed, tensor_id, block index, word
// index):   key = mix(seed ^ mix(tensor_id));   r(b, w) = mix(key + 32*b + w)
// with mix = the splitmix64 finaliser applied to (z + 0x9E3779B97F4A7C15).
// Field maps (u24(v) = (v & 0xFFFFFF) / 2^24 in double; a scale is
// f16_rne((float)(lo + (hi - lo) * u))):
//   Q8_0 : w0 -> d from u24(r);  w1..w8 -> 32 x u16 v, qs = ((v * 255) >> 16) - 127        Q8_1 : the same draw, plus s = f16(d * sum qs)
//   Q4_0 : w0 -> d;  w1,w2 -> the 16 qs bytes verbatim
//   Q4_1 : w0 -> d from u24(r), m = -8 d' with d' from u24(r >> 32);  w1,w2 -> qs
//   Q5_0 : w0 -> d, qh = bits 32..63 of r;  w1,w2 -> qs        Q5_1 : w0 -> d, m = -16 d';  w1,w2 -> qs;  w3 -> qh (low 32 bits)
//   Q2_K : w0,w1 -> the 16 scale bytes verbatim;  w2..w9 -> qs;  w10 -> d from u24(r), dmin from u24(r >> 32)
//   Q3_K : w0..w3 -> hmask;  w4..w11 -> qs;  w12 and the low half of w13 -> the 12 scale bytes verbatim;  w14 -> d
//   Q4_K : w0 -> d from u24(r), dmin from u24(r >> 32);  w1 -> 8 scales (byte & 63);
//          w2 -> 8 mins (byte & 63), packed into the 12-byte field;  w3..w18 -> qs
//   Q5_K : w0..w2 as Q4_K;  w3..w6 -> qh;  w7..w22 -> qs
//   Q6_K : w0..w15 -> ql;  w16..w23 -> qh;  w24,w25 -> scales = (byte & 63) - 32;  w26 -> d
// The block layouts are the public ggml ones; the byte sizes match
// GGMLType::type_size (example-cli/src/model/formats/gguf.rs:125-144).
#include "../../include/rustorch_hip.h"

#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

namespace {

inline uint64_t mix(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

inline uint64_t make_key(uint64_t seed, uint64_t tensor_id) { return mix(seed ^ mix(tensor_id)); }

inline double u24(uint64_t v) { return (double)(v & 0xFFFFFFull) / 16777216.0; }

// binary32 -> binary16, round to nearest even.
inline uint16_t f32_to_f16(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u, exp = (x >> 23) & 0xFFu, man = x & 0x7FFFFFu;
    if (exp == 255) return (uint16_t)(sign | 0x7C00u | (man ? (0x200u | (man >> 13)) : 0));
    int e = (int)exp - 112;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        int shift = 14 - e;
        uint32_t hm = man >> shift, rem = man & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (hm & 1u))) hm++;
        return (uint16_t)(sign | hm);
    }
    uint32_t h = ((uint32_t)e << 10) | (man >> 13), rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

// binary16 -> binary32 (exact).
inline float f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
    uint32_t x;
    if (exp == 0) {
        if (man == 0) x = sign;
        else {                                     // subnormal: renormalise
            int e = -1;
            uint32_t m = man;
            do { e++; m <<= 1; } while ((m & 0x400u) == 0);
            x = sign | ((uint32_t)(112 - e) << 23) | ((m & 0x3FFu) << 13);
        }
    } else if (exp == 31) x = sign | 0x7F800000u | (man << 13);
    else x = sign | ((exp + 112u) << 23) | (man << 13);
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}

inline uint16_t scale_f16(double lo, double hi, double u) { return f32_to_f16((float)(lo + (hi - lo) * u)); }

inline void put16(uint8_t *p, uint16_t v) { p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); }
inline void put64(uint8_t *p, uint64_t v) { std::memcpy(p, &v, 8); }

// 8 six-bit scales + 8 six-bit mins -> the 12 packed bytes of a Q4_K super-block.
void pack_q4k_scales(const uint8_t sc[8], const uint8_t mn[8], uint8_t out[12]) {
    for (int j = 0; j < 4; j++) {
        out[j] = (uint8_t)((sc[j] & 63) | ((sc[j + 4] >> 4) << 6));
        out[j + 4] = (uint8_t)((mn[j] & 63) | ((mn[j + 4] >> 4) << 6));
        out[j + 8] = (uint8_t)((sc[j + 4] & 0x0F) | ((mn[j + 4] & 0x0F) << 4));
    }
}

void gen_block(int type, uint64_t key, uint64_t b, double lo, double hi, uint8_t *o) {
    uint64_t base = key + 32ull * b;
    switch (type) {
    case RT_GGML_Q8_0: {
        put16(o, scale_f16(lo, hi, u24(mix(base))));
        for (int w = 0; w < 8; w++) {
            uint64_t r = mix(base + 1 + w);
            for (int i = 0; i < 4; i++) {
                uint32_t v = (uint32_t)((r >> (16 * i)) & 0xFFFFu);
                o[2 + 4 * w + i] = (uint8_t)(int8_t)((int)((v * 255u) >> 16) - 127);
            }
        }
        break;
    }
    case RT_GGML_Q8_1: {       // the Q8_0 draw with the format's second field, d * sum of the quants (rounded to fp16), filled in
        const uint16_t dh = scale_f16(lo, hi, u24(mix(base)));
        put16(o, dh);
        int sum = 0;
        for (int w = 0; w < 8; w++) {
            uint64_t r = mix(base + 1 + w);
            for (int i = 0; i < 4; i++) {
                uint32_t v = (uint32_t)((r >> (16 * i)) & 0xFFFFu);
                const int q = (int)((v * 255u) >> 16) - 127;
                o[4 + 4 * w + i] = (uint8_t)(int8_t)q;
                sum += q;
            }
        }
        put16(o + 2, f32_to_f16(f16_to_f32(dh) * (float)sum));
        break;
    }
    case RT_GGML_Q4_0: {
        put16(o, scale_f16(lo, hi, u24(mix(base))));
        put64(o + 2, mix(base + 1));
        put64(o + 10, mix(base + 2));
        break;
    }
    case RT_GGML_Q4_1: {       // the offset sits where a symmetric format would put it (m of the order of -8 d)
        uint64_t r0 = mix(base);
        put16(o, scale_f16(lo, hi, u24(r0)));
        put16(o + 2, scale_f16(-8.0 * lo, -8.0 * hi, u24(r0 >> 32)));
        put64(o + 4, mix(base + 1));
        put64(o + 12, mix(base + 2));
        break;
    }
    case RT_GGML_Q5_0: {
        uint64_t r0 = mix(base);
        put16(o, scale_f16(lo, hi, u24(r0)));
        uint32_t qh = (uint32_t)(r0 >> 32);
        std::memcpy(o + 2, &qh, 4);
        put64(o + 6, mix(base + 1));
        put64(o + 14, mix(base + 2));
        break;
    }
    case RT_GGML_Q5_1: {
        uint64_t r0 = mix(base);
        put16(o, scale_f16(lo, hi, u24(r0)));
        put16(o + 2, scale_f16(-16.0 * lo, -16.0 * hi, u24(r0 >> 32)));
        uint32_t qh = (uint32_t)mix(base + 3);
        std::memcpy(o + 4, &qh, 4);
        put64(o + 8, mix(base + 1));
        put64(o + 16, mix(base + 2));
        break;
    }
    case RT_GGML_Q2_K: {
        for (int w = 0; w < 10; w++) put64(o + 8 * w, mix(base + w));
        uint64_t r = mix(base + 10);
        put16(o + 80, scale_f16(lo, hi, u24(r)));
        put16(o + 82, scale_f16(lo, hi, u24(r >> 32)));
        break;
    }
    case RT_GGML_Q3_K: {
        for (int w = 0; w < 12; w++) put64(o + 8 * w, mix(base + w));
        put64(o + 96, mix(base + 12));
        uint32_t tail = (uint32_t)mix(base + 13);
        std::memcpy(o + 104, &tail, 4);
        put16(o + 108, scale_f16(lo, hi, u24(mix(base + 14))));
        break;
    }
    case RT_GGML_Q4_K: {
        uint64_t r0 = mix(base);
        put16(o, scale_f16(lo, hi, u24(r0)));
        put16(o + 2, scale_f16(lo, hi, u24(r0 >> 32)));
        uint64_t r1 = mix(base + 1), r2 = mix(base + 2);
        uint8_t sc[8], mn[8];
        for (int j = 0; j < 8; j++) {
            sc[j] = (uint8_t)((r1 >> (8 * j)) & 63);
            mn[j] = (uint8_t)((r2 >> (8 * j)) & 63);
        }
        pack_q4k_scales(sc, mn, o + 4);
        for (int w = 0; w < 16; w++) put64(o + 16 + 8 * w, mix(base + 3 + w));
        break;
    }
    case RT_GGML_Q5_K: {       // as Q4_K, then 4 words of fifth bits and 16 words of nibbles
        uint64_t r0 = mix(base);
        put16(o, scale_f16(lo, hi, u24(r0)));
        put16(o + 2, scale_f16(lo, hi, u24(r0 >> 32)));
        uint64_t r1 = mix(base + 1), r2 = mix(base + 2);
        uint8_t sc[8], mn[8];
        for (int j = 0; j < 8; j++) {
            sc[j] = (uint8_t)((r1 >> (8 * j)) & 63);
            mn[j] = (uint8_t)((r2 >> (8 * j)) & 63);
        }
        pack_q4k_scales(sc, mn, o + 4);
        for (int w = 0; w < 20; w++) put64(o + 16 + 8 * w, mix(base + 3 + w));
        break;
    }
    case RT_GGML_Q6_K: {
        for (int w = 0; w < 24; w++) put64(o + 8 * w, mix(base + w));
        for (int w = 0; w < 2; w++) {
            uint64_t r = mix(base + 24 + w);
            for (int j = 0; j < 8; j++) o[192 + 8 * w + j] = (uint8_t)(int8_t)((int)((r >> (8 * j)) & 63) - 32);
        }
        put16(o + 208, scale_f16(lo, hi, u24(mix(base + 26))));
        break;
    }
    }
}

template <class F> void parallel_for(size_t n, size_t grain, F f) {
    unsigned hw = std::thread::hardware_concurrency();
    size_t nt = hw ? hw : 1;
    if (nt > 16) nt = 16;
    if (n < grain * 2 || nt == 1) { f(0, n); return; }
    if (nt > n / grain) nt = n / grain;
    std::vector<std::thread> th;
    size_t chunk = (n + nt - 1) / nt;
    for (size_t t = 0; t < nt; t++) {
        size_t a = t * chunk, b = a + chunk < n ? a + chunk : n;
        if (a >= b) break;
        th.emplace_back([=] { f(a, b); });
    }
    for (auto &t : th) t.join();
}

}  // namespace

extern "C" {

int rt_synth_blocks(int ggml_type, uint64_t seed, uint64_t tensor_id, size_t n_blocks, float d_lo, float d_hi,
                    void *out) {
    size_t bb = rt_hip_type_block_bytes(ggml_type);
    if (!out || bb == 0 || ggml_type == RT_GGML_F32 || ggml_type == RT_GGML_F16) return RT_HIP_ERR_UNSUPPORTED_TYPE;
    uint64_t key = make_key(seed, tensor_id);
    uint8_t *o = (uint8_t *)out;
    double lo = d_lo, hi = d_hi;
    parallel_for(n_blocks, 4096, [=](size_t a, size_t b) {
        for (size_t i = a; i < b; i++) gen_block(ggml_type, key, i, lo, hi, o + bb * i);
    });
    return RT_HIP_OK;
}

// Box-Muller on two 53-bit uniforms per pair; element 2i uses the cosine branch, 2i+1 the sine branch.
int rt_synth_normal_f32(uint64_t seed, uint64_t tensor_id, size_t n, float mean, float std, float *out) {
    if (!out) return RT_HIP_ERR_INVALID_ARG;
    uint64_t key = make_key(seed, tensor_id);
    parallel_for((n + 1) / 2, 1 << 14, [=](size_t a, size_t b) {
        for (size_t i = a; i < b; i++) {
            double u1 = ((double)(mix(key + 2 * i) >> 11) + 1.0) / 9007199254740992.0; /* (0,1] */
            double u2 = (double)(mix(key + 2 * i + 1) >> 11) / 9007199254740992.0;
            double r = std::sqrt(-2.0 * std::log(u1));
            double t = 6.283185307179586476925286766559 * u2;
            out[2 * i] = (float)((double)mean + (double)std * r * std::cos(t));
            if (2 * i + 1 < n) out[2 * i + 1] = (float)((double)mean + (double)std * r * std::sin(t));
        }
    });
    return RT_HIP_OK;
}

int rt_synth_tokens(uint64_t seed, uint64_t tensor_id, size_t n, int vocab, int *out) {
    if (!out || vocab <= 0) return RT_HIP_ERR_INVALID_ARG;
    uint64_t key = make_key(seed, tensor_id);
    for (size_t i = 0; i < n; i++) out[i] = (int)(((mix(key + i) >> 32) * (uint64_t)vocab) >> 32);
    return RT_HIP_OK;
}

}  // extern "C"
