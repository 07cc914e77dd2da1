// Device-side helpers shared by the kernel files.
#pragma once
#include "common.hpp"

namespace cg {

__device__ __forceinline__ uint32_t fastdiv(uint32_t n, const FastDiv &f) {
    uint32_t t = __umulhi(f.m, n);
    return (t + ((n - t) >> f.s1)) >> f.s2;
}

__device__ __forceinline__ float asf(uint32_t b) { return __uint_as_float(b); }
__device__ __forceinline__ uint32_t asu(float f) { return __float_as_uint(f); }

template <int VEC> __device__ __forceinline__ void load_words(const Operand &o, int64_t off, uint32_t (&r)[VEC]) {
    if (o.uniform) {
#pragma unroll
        for (int j = 0; j < VEC; j++) r[j] = o.ubits;
        return;
    }
    const uint32_t *p = reinterpret_cast<const uint32_t *>(o.ptr) + off;
    if (VEC == 4 && o.is == 1) {
        uint4 t = *reinterpret_cast<const uint4 *>(p);
        r[0] = t.x;
        r[1 % VEC] = t.y;
        r[2 % VEC] = t.z;
        r[3 % VEC] = t.w;
    } else if (o.is == 0) {
        uint32_t t = *p;
#pragma unroll
        for (int j = 0; j < VEC; j++) r[j] = t;
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++) r[j] = p[(int64_t)j * o.is];
    }
}

template <int VEC> __device__ __forceinline__ void store_words(const Operand &o, int64_t off, const uint32_t (&r)[VEC]) {
    uint32_t *p = reinterpret_cast<uint32_t *>(const_cast<char *>(o.ptr)) + off;
    if (VEC == 4 && o.is == 1) {
        *reinterpret_cast<uint4 *>(p) = make_uint4(r[0], r[1 % VEC], r[2 % VEC], r[3 % VEC]);
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++) p[(int64_t)j * o.is] = r[j];
    }
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
