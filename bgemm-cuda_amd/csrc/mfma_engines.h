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
    // both operands expand alike
    __device__ static __forceinline__ Frag expand_w(const uint4 w, const int s) { return expand(w, s); }
    __device__ static __forceinline__ Frag expand_x(const uint4 w, const int s) { return expand(w, s); }
    __device__ static __forceinline__ unsigned expand1_w(const unsigned w, const int s) { return expand1(w, s); }
    __device__ static __forceinline__ unsigned expand1_x(const unsigned w, const int s) { return expand1(w, s); }
    // a K of at most 64 bits: only the first two words of a lane hold any
    __device__ static __forceinline__ Frag expand_w2(const uint4 w, const int s)
    {
        Frag r = {(int)expand1(w.x, s), (int)expand1(w.y, s), 0, 0};
        return r;
    }
    __device__ static __forceinline__ Frag expand_x2(const uint4 w, const int s) { return expand_w2(w, s); }
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
    __device__ static __forceinline__ float to_float(const Acc& c, const int v) { return (float)c[v]; }
};

// fp4 engine: the same tile is four 64-deep steps of v_mfma_f32_32x32x64_f8f6f4 with E2M1
// operands; nibble c of word q at step s is bit 4c+s.  E2M1 has three single-bit values,
// 0b0001 = 0.5, 0b0010 = 1.0, 0b0100 = 2.0, so a bit can often stay where it is: the weight side
// keeps bits 0..2 in place (0.5, 1, 2: one AND per step) and the activation side moves the same
// bits to the reciprocal values (2, 1, 0.5), so every product of set bits is exactly 1; bit 3
// (the sign position) is shifted to 1.0 on both sides.  Five VALU ops per weight word and six
// per activation word instead of seven and seven.  Products are 0 or 1 and the fp32 accumulator
// holds integers below 2^24, so it stays exact.
struct EngF4 {
    typedef v16f Acc;
    typedef v8i Frag;
    static constexpr int STEPS = 4;
    __device__ static __forceinline__ unsigned expand1_w(const unsigned w, const int s)
    {
        return s == 3 ? (w >> 2) & 0x22222222u : w & (0x11111111u << s);
    }
    __device__ static __forceinline__ unsigned expand1_x(const unsigned w, const int s)
    {
        return s == 0 ? (w << 2) & 0x44444444u : s == 1 ? w & 0x22222222u : (w >> 2) & (s == 2 ? 0x11111111u : 0x22222222u);
    }
    __device__ static __forceinline__ Frag expand_w(const uint4 w, const int s)
    {
        Frag r = {0, 0, 0, 0, 0, 0, 0, 0};
        r[0] = expand1_w(w.x, s); r[1] = expand1_w(w.y, s); r[2] = expand1_w(w.z, s); r[3] = expand1_w(w.w, s);
        return r;
    }
    __device__ static __forceinline__ Frag expand_x(const uint4 w, const int s)
    {
        Frag r = {0, 0, 0, 0, 0, 0, 0, 0};
        r[0] = expand1_x(w.x, s); r[1] = expand1_x(w.y, s); r[2] = expand1_x(w.z, s); r[3] = expand1_x(w.w, s);
        return r;
    }
    // a K of at most 64 bits: only the first two words of a lane hold any
    __device__ static __forceinline__ Frag expand_w2(const uint4 w, const int s)
    {
        Frag r = {(int)expand1_w(w.x, s), (int)expand1_w(w.y, s), 0, 0, 0, 0, 0, 0};
        return r;
    }
    __device__ static __forceinline__ Frag expand_x2(const uint4 w, const int s)
    {
        Frag r = {(int)expand1_x(w.x, s), (int)expand1_x(w.y, s), 0, 0, 0, 0, 0, 0};
        return r;
    }
    __device__ static __forceinline__ Frag make(const unsigned (&f)[4])
    {
        Frag r = {(int)f[0], (int)f[1], (int)f[2], (int)f[3], 0, 0, 0, 0};
        return r;
    }
    // Binary weight x ternary activation with SIGNED operands: one MFMA where the AND-dot needs two (one per bit plane of
    // the activations) and rank-one terms.  A nibble is a sign (bit 3) and one value bit.  Activation: the nonzero plane's
    // bit stays where it is at steps 0..2 (0.5, 1, 2; at step 3 it moves to 1.0) under the bit of the sign plane (a sign
    // over a zero value adds nothing); weight: its sign bit over the reciprocal value (2, 1, 0.5, 1), so a product is -1, 0
    // or +1 and the accumulator holds the layer's output itself.  Three VALU ops per activation register, seven per four
    // weight registers.
    __device__ static __forceinline__ unsigned tern_x(const unsigned z, const unsigned zs, const int s)
    {
        return s == 3 ? (zs & 0x88888888u) | ((z >> 2) & 0x22222222u) : ((zs << (3 - s)) & 0x88888888u) | (z & (0x11111111u << s));
    }
    // (mask in place, then one v_lshl_or_b32 with the value constant in a scalar register: written as the instruction,
    // because the compiler turns the expression into shift, AND and OR, a literal each, which this ISA cannot fold.  Step 3
    // needs no shift: one v_and_or_b32, whose second constant has to sit in a vector register, `c1` = tern_const().)
    __device__ static __forceinline__ unsigned tern_const()
    {
        unsigned c = 0x22222222u;
        asm volatile("" : "+v"(c));          // kept in a register: as a literal it would be a second constant operand
        return c;
    }
    __device__ static __forceinline__ unsigned tern_w(const unsigned w, const int s, const unsigned c1)
    {
        unsigned r;
        if (s == 3) {
            asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(w), "s"(0x88888888u), "v"(c1));
            return r;
        }
        const unsigned m = w & (0x11111111u << s), c = 0x44444444u >> s;
        if (s == 0) asm("v_lshl_or_b32 %0, %1, 3, %2" : "=v"(r) : "v"(m), "s"(c));
        else if (s == 1) asm("v_lshl_or_b32 %0, %1, 2, %2" : "=v"(r) : "v"(m), "s"(c));
        else asm("v_lshl_or_b32 %0, %1, 1, %2" : "=v"(r) : "v"(m), "s"(c));
        return r;
    }
    // a = activation-side fragment, b = weight-side fragment
    __device__ static __forceinline__ Acc mma(const Frag a, const Frag b, const Acc c)
    {
        return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 4, 4, 0, 0, 0, 0);
    }
    __device__ static __forceinline__ int to_int(const Acc& c, const int v) { return (int)c[v]; }
    __device__ static __forceinline__ float to_float(const Acc& c, const int v) { return c[v]; }
};

__device__ __forceinline__ int popc4(const uint4 w)
{
    return __popc(w.x) + __popc(w.y) + __popc(w.z) + __popc(w.w);
}

}  // namespace bgemm
