// Device-side helpers shared by the kernel files.
#pragma once
#include <hip/hip_fp16.h>
#include "common.hpp"

namespace cg {

__device__ __forceinline__ uint32_t fastdiv(uint32_t n, const FastDiv &f) {
    uint32_t t = __umulhi(f.m, n);
    return (t + ((n - t) >> f.s1)) >> f.s2;
}

__device__ __forceinline__ float asf(uint32_t b) { return __uint_as_float(b); }
__device__ __forceinline__ uint32_t asu(float f) { return __float_as_uint(f); }

// The f32 word of one element of a narrow format, and back (exact: a word that is stored narrow holds a value of the format).
__device__ __forceinline__ uint32_t f8_word_of_dev(uint8_t b);
__device__ __forceinline__ uint8_t f8_byte_of_dev(uint32_t u);

// VEC consecutive elements (element stride o.is) of a NARROW operand, widened to f32 words.  VEC 4 or 8 with unit stride:
// one load of 8 or 16 bytes (16-bit formats), of 4 or 8 bytes (fp8); the planner has checked the alignment.
template <int VEC>
__device__ __forceinline__ void load_narrow(const Operand &o, int64_t off, uint32_t (&r)[VEC]) {
    if (o.fmt == kFmtF8) {
        const uint8_t *p = reinterpret_cast<const uint8_t *>(o.ptr) + off;
        if (VEC >= 4 && o.is == 1) {
            uint32_t t[VEC >= 8 ? 2 : 1];
            if (VEC >= 8) {
                const uint2 q = *reinterpret_cast<const uint2 *>(p);
                t[0] = q.x;
                t[VEC >= 8 ? 1 : 0] = q.y;
            } else {
                t[0] = *reinterpret_cast<const uint32_t *>(p);
            }
#pragma unroll
            for (int j = 0; j < VEC; j++) r[j] = f8_word_of_dev((uint8_t)(t[j / 4] >> (8 * (j % 4))));
        } else if (o.is == 0) {
            const uint32_t t = f8_word_of_dev(*p);
#pragma unroll
            for (int j = 0; j < VEC; j++) r[j] = t;
        } else {
#pragma unroll
            for (int j = 0; j < VEC; j++) r[j] = f8_word_of_dev(p[(int64_t)j * o.is]);
        }
        return;
    }
    const uint16_t *p = reinterpret_cast<const uint16_t *>(o.ptr) + off;
    uint16_t h[VEC];
    if (VEC >= 4 && o.is == 1) {
        uint32_t t[VEC / 2 > 0 ? VEC / 2 : 1];
        if (VEC >= 8) {
            const uint4 q = *reinterpret_cast<const uint4 *>(p);
            t[0] = q.x;
            t[1 % (VEC / 2 > 0 ? VEC / 2 : 1)] = q.y;
            t[2 % (VEC / 2 > 0 ? VEC / 2 : 1)] = q.z;
            t[3 % (VEC / 2 > 0 ? VEC / 2 : 1)] = q.w;
        } else {
            const uint2 q = *reinterpret_cast<const uint2 *>(p);
            t[0] = q.x;
            t[1 % (VEC / 2 > 0 ? VEC / 2 : 1)] = q.y;
        }
#pragma unroll
        for (int j = 0; j < VEC; j++) h[j] = (uint16_t)(t[j / 2] >> (16 * (j % 2)));
    } else if (o.is == 0) {
        const uint16_t t = *p;
#pragma unroll
        for (int j = 0; j < VEC; j++) h[j] = t;
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++) h[j] = p[(int64_t)j * o.is];
    }
#pragma unroll
    for (int j = 0; j < VEC; j++)
        r[j] = o.fmt == kFmtBF16 ? (uint32_t)h[j] << 16 : __float_as_uint(__half2float(__ushort_as_half(h[j])));
}

// f32 words that hold values of a narrow format, stored as that format's patterns.
template <int VEC, bool STREAM = false>
__device__ __forceinline__ void store_narrow(const Operand &o, int64_t off, const uint32_t (&r)[VEC]) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    typedef uint32_t u2 __attribute__((ext_vector_type(2)));
    if (o.fmt == kFmtF8) {
        uint8_t *p = reinterpret_cast<uint8_t *>(const_cast<char *>(o.ptr)) + off;
        if (VEC >= 4 && o.is == 1) {
            uint32_t t[VEC >= 8 ? 2 : 1] = {};
#pragma unroll
            for (int j = 0; j < VEC; j++) t[j / 4] |= (uint32_t)f8_byte_of_dev(r[j]) << (8 * (j % 4));
            if (VEC >= 8) {
                const u2 v = {t[0], t[VEC >= 8 ? 1 : 0]};
                if (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<u2 *>(p));
                else *reinterpret_cast<u2 *>(p) = v;
            } else {
                *reinterpret_cast<uint32_t *>(p) = t[0];
            }
        } else {
#pragma unroll
            for (int j = 0; j < VEC; j++) p[(int64_t)j * o.is] = f8_byte_of_dev(r[j]);
        }
        return;
    }
    uint16_t h[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++)
        h[j] = o.fmt == kFmtBF16 ? (uint16_t)(r[j] >> 16) : __half_as_ushort(__float2half_rn(__uint_as_float(r[j])));
    uint16_t *p = reinterpret_cast<uint16_t *>(const_cast<char *>(o.ptr)) + off;
    if (VEC >= 4 && o.is == 1) {
        constexpr int W = VEC / 2 > 0 ? VEC / 2 : 1;
        uint32_t t[W];
#pragma unroll
        for (int j = 0; j < W; j++) t[j] = (uint32_t)h[(2 * j) % VEC] | ((uint32_t)h[(2 * j + 1) % VEC] << 16);
        if (VEC >= 8) {
            const u4 v = {t[0], t[1 % W], t[2 % W], t[3 % W]};
            if (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<u4 *>(p));
            else *reinterpret_cast<u4 *>(p) = v;
        } else {
            const u2 v = {t[0], t[1 % W]};
            if (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<u2 *>(p));
            else *reinterpret_cast<u2 *>(p) = v;
        }
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++) p[(int64_t)j * o.is] = h[j];
    }
}

// WORDS: the caller knows that the operand lies in 32-bit words (kernels compiled for launches whose operands all do:
// without the narrow formats' code between its loads a program keeps them all in flight).
template <int VEC, bool STREAM = false, bool WORDS = false>
__device__ __forceinline__ void load_words(const Operand &o, int64_t off, uint32_t (&r)[VEC]) {
    if (o.uniform) {
#pragma unroll
        for (int j = 0; j < VEC; j++) r[j] = o.ubits;
        return;
    }
    if (!WORDS && o.fmt != kFmtWords) { // (the same for every lane: the format is a launch parameter)
        load_narrow<VEC>(o, off, r);
        return;
    }
    const uint32_t *p = reinterpret_cast<const uint32_t *>(o.ptr) + off;
    if (VEC >= 4 && o.is == 1) {
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int q = 0; q < VEC / 4; q++) {
            const u4 t = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const u4 *>(p) + q) : reinterpret_cast<const u4 *>(p)[q];
            r[(4 * q) % VEC] = t[0];
            r[(4 * q + 1) % VEC] = t[1];
            r[(4 * q + 2) % VEC] = t[2];
            r[(4 * q + 3) % VEC] = t[3];
        }
    } else if (o.is == 0) {
        uint32_t t = *p;
#pragma unroll
        for (int j = 0; j < VEC; j++) r[j] = t;
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++) r[j] = p[(int64_t)j * o.is];
    }
}

// STREAM: the output is far larger than the caches; non-temporal stores keep it from
// evicting the operands that are still being read.
template <int VEC, bool STREAM = false, bool WORDS = false>
__device__ __forceinline__ void store_words(const Operand &o, int64_t off, const uint32_t (&r)[VEC]) {
    if (!WORDS && o.fmt != kFmtWords) {
        store_narrow<VEC, STREAM>(o, off, r);
        return;
    }
    uint32_t *p = reinterpret_cast<uint32_t *>(const_cast<char *>(o.ptr)) + off;
    if (VEC >= 4 && o.is == 1) {
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int q = 0; q < VEC / 4; q++) {
            const u4 v = {r[(4 * q) % VEC], r[(4 * q + 1) % VEC], r[(4 * q + 2) % VEC], r[(4 * q + 3) % VEC]};
            if (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<u4 *>(p) + q);
            else reinterpret_cast<u4 *>(p)[q] = v;
        }
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++) p[(int64_t)j * o.is] = r[j];
    }
}


// Rust `f32 as u32` (ndarray.rs:155): truncate, saturate, NaN -> 0.
__device__ __forceinline__ uint32_t f32_as_u32(float v) {
    if (!(v == v) || v <= 0.0f) return 0u;
    if (v >= 4294967296.0f) return 0xFFFFFFFFu;
    return (uint32_t)v;
}

__device__ __forceinline__ uint32_t wrapping_pow(uint32_t a, uint32_t e) {
    uint32_t acc = 1;
    while (e) {
        if (e & 1) acc *= a;
        a *= a;
        e >>= 1;
    }
    return acc;
}

// f32 bits -> bits of the nearest bfloat16 value (ties to even), as f32; NaNs stay NaNs (quiet)
__host__ __device__ __forceinline__ uint32_t round_bf16_bits(uint32_t u) {
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u | 0x00400000u) & 0xFFFF0000u;
    return (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
}

// fp8 = E4M3 (float8::F8E4M3): 4 exponent bits with bias 7, 3 mantissa bits, no infinities, 0x7F the NaN, largest
// finite value 448, subnormals m * 2^-9.  f32 bits -> f32 bits of the nearest such value (ties to even); 448 and
// beyond, infinities included, give +-448 (the crate's saturating conversion); NaN stays NaN.
__host__ __device__ __forceinline__ uint32_t round_f8_bits(uint32_t u) {
    const uint32_t sign = u & 0x80000000u, a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return sign | 0x7FC00000u;
    if (a >= 0x43E00000u) return sign | 0x43E00000u; // 448
    if (a < 0x3C800000u) {                           // below 2^-6: whole multiples of 2^-9
        const float units = rintf(__builtin_bit_cast(float, a) * 512.0f);
        return sign | __builtin_bit_cast(uint32_t, units * (1.0f / 512.0f));
    }
    const uint32_t r = (a + 0x7FFFFu + ((a >> 20) & 1u)) & 0xFFF00000u; // a carry runs into the exponent
    return sign | (r > 0x43E00000u ? 0x43E00000u : r);
}
// the byte of a representable value, and back
__host__ __device__ __forceinline__ uint8_t f8_byte_of(uint32_t u) {
    const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return sign | 0x7Fu;
    if (a >= 0x3C800000u) return sign | (uint8_t)((((a >> 23) - 120u) << 3) | ((a >> 20) & 7u));
    return sign | (uint8_t)(uint32_t)(__builtin_bit_cast(float, a) * 512.0f);
}
__host__ __device__ __forceinline__ uint32_t f8_word_of(uint8_t b) {
    const uint32_t sign = (uint32_t)(b & 0x80u) << 24, e = (b >> 3) & 0xFu, m = b & 7u;
    if (e == 0xFu && m == 7u) return sign | 0x7FC00000u;
    if (e != 0) return sign | ((e + 120u) << 23) | (m << 20);
    return sign | __builtin_bit_cast(uint32_t, (float)m * (1.0f / 512.0f));
}

__device__ __forceinline__ uint32_t f8_word_of_dev(uint8_t b) { return f8_word_of(b); }
__device__ __forceinline__ uint8_t f8_byte_of_dev(uint32_t u) { return f8_byte_of(u); }

// One scalar application of OP on raw 32-bit words.  F = operands are f32.
template <int OP, bool F>
__device__ __forceinline__ uint32_t apply(uint32_t a, uint32_t b, uint32_t c, uint32_t *fault) {
    (void)b;
    (void)c;
    (void)fault;
    if constexpr (OP == kCopy) return a;
    if constexpr (OP == kCastF2U) return f32_as_u32(asf(a));
    if constexpr (OP == kCastU2F) return asu((float)a); // round to nearest even
    if constexpr (OP == kWhere) return F ? (asf(a) > 0.0f ? b : c) : (a != 0 ? b : c);
    if constexpr (F) {
        float x = asf(a), y = asf(b);
        if constexpr (OP == kNeg) return a ^ 0x80000000u;
        if constexpr (OP == kSin) return asu(sinf(x));
        if constexpr (OP == kCos) return asu(cosf(x));
        if constexpr (OP == kExp) return asu(expf(x));
        if constexpr (OP == kLog) return asu(logf(x));
        if constexpr (OP == kFloor) return asu(floorf(x));
        if constexpr (OP == kRound) return asu(rintf(x)); // ties to even (ndarray.rs:646-648)
        if constexpr (OP == kRoundBF16) return round_bf16_bits(a);
        if constexpr (OP == kRoundF16) return asu(__half2float(__float2half_rn(x))); // v_cvt_f16_f32: nearest even, overflow -> inf
        if constexpr (OP == kRoundF8) return round_f8_bits(a);
        if constexpr (OP == kAdd) return asu(x + y);
        if constexpr (OP == kSub) return asu(x - y);
        if constexpr (OP == kMul) return asu(x * y);
        if constexpr (OP == kDiv) return asu(x / y);
        if constexpr (OP == kPow) return asu(powf(x, y));
        if constexpr (OP == kLt) return asu(x < y ? 1.0f : 0.0f);
        if constexpr (OP == kGt) return asu(x > y ? 1.0f : 0.0f);
        if constexpr (OP == kGte) return asu(x >= y ? 1.0f : 0.0f);
        if constexpr (OP == kLte) return asu(x <= y ? 1.0f : 0.0f);
        if constexpr (OP == kEq) return asu(x == y ? 1.0f : 0.0f);
    } else {
        if constexpr (OP == kNeg) return 0u - a;
        if constexpr (OP == kAdd) return a + b;
        if constexpr (OP == kSub) return a - b;
        if constexpr (OP == kMul) return a * b;
        if constexpr (OP == kDiv) {
            if (b == 0) {
                *fault = kFaultDivZero; // reported by the next waiting call
                return 0u;
            }
            return a / b;
        }
        if constexpr (OP == kPow) return wrapping_pow(a, b);
        if constexpr (OP == kLt) return a < b;
        if constexpr (OP == kGt) return a > b;
        if constexpr (OP == kGte) return a >= b;
        if constexpr (OP == kLte) return a <= b;
        if constexpr (OP == kEq) return a == b;
    }
    return 0u;
}

// Offset (in elements) of row `row` of a view whose outer axes are described by
// (od, odiv, os), innermost first.
__device__ __forceinline__ int64_t row_offset(uint32_t row, uint32_t nouter, const uint32_t *od, const FastDiv *odiv,
                                              const int64_t *os) {
    int64_t off = 0;
    for (uint32_t d = 0; d < nouter; d++) {
        uint32_t q = fastdiv(row, odiv[d]);
        off += (int64_t)(row - q * od[d]) * os[d];
        row = q;
    }
    return off;
}

} // namespace cg
