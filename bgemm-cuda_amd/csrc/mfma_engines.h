// Matrix-core "engines": how a 256-bit K-tile of packed bits becomes MFMA operands.
#pragma once
#include "common.h"

namespace bgemm {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

// int8 engine: a 256-bit K-tile is eight 32-deep steps of v_mfma_i32_32x32x32_i8;
// byte c of word q at step s is bit 8c+s.
struct EngI8 {
    typedef v16i Acc;
    typedef v4i Frag;
    static constexpr int STEPS = 8;
    __device__ static __forceinline__ Frag expand(const uint4 w, const int s)
    {
        Frag r;
        r.x = (w.x >> s) & 0x01010101u; r.y = (w.y >> s) & 0x01010101u;
        r.z = (w.z >> s) & 0x01010101u; r.w = (w.w >> s) & 0x01010101u;
        return r;
    }
    __device__ static __forceinline__ unsigned expand1(const unsigned w, const int s) { return (w >> s) & 0x01010101u; }
    __device__ static __forceinline__ Frag make(const unsigned (&f)[4])
    {
        Frag r = {(int)f[0], (int)f[1], (int)f[2], (int)f[3]};
        return r;
    }
    __device__ static __forceinline__ Acc mma(const Frag a, const Frag b, const Acc c)
    {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
    }
    __device__ static __forceinline__ int to_int(const Acc& c, const int v) { return c[v]; }
};

// fp4 engine: the same tile is four 64-deep steps of v_mfma_f32_32x32x64_f8f6f4 with E2M1
// operands; nibble c of word q at step s is bit 4c+s, moved to nibble bit 1 (0b0010 = 1.0).
// Products are 0 or 1 and the fp32 accumulator holds integers below 2^24, so it stays exact.
struct EngF4 {
    typedef v16f Acc;
    typedef v8i Frag;
    static constexpr int STEPS = 4;
    __device__ static __forceinline__ unsigned nib(const unsigned w, const int s)
    {
        return (s == 0 ? (w << 1) : (w >> (s - 1))) & 0x22222222u;
    }
    __device__ static __forceinline__ Frag expand(const uint4 w, const int s)
    {
        Frag r = {0, 0, 0, 0, 0, 0, 0, 0};
        r[0] = nib(w.x, s); r[1] = nib(w.y, s); r[2] = nib(w.z, s); r[3] = nib(w.w, s);
        return r;
    }
    __device__ static __forceinline__ unsigned expand1(const unsigned w, const int s) { return nib(w, s); }
    __device__ static __forceinline__ Frag make(const unsigned (&f)[4])
    {
        Frag r = {(int)f[0], (int)f[1], (int)f[2], (int)f[3], 0, 0, 0, 0};
        return r;
    }
    __device__ static __forceinline__ Acc mma(const Frag a, const Frag b, const Acc c)
    {
        return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 4, 4, 0, 0, 0, 0);
    }
    __device__ static __forceinline__ int to_int(const Acc& c, const int v) { return (int)c[v]; }
};

__device__ __forceinline__ int popc4(const uint4 w)
{
    return __popc(w.x) + __popc(w.y) + __popc(w.z) + __popc(w.w);
}

}  // namespace bgemm
