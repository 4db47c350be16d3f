// Element-to-bit helpers shared by the pack kernels and by the GEMM kernels that read
// unpacked activations themselves.
#pragma once
#include "common.h"

namespace bgemm {

__device__ __forceinline__ uint16_t half_bits(const float f)
{
    return __half_as_ushort(__float2half_rn(f));
}

// Sign (and nonzero) bits of eight fp16 bit patterns, element e at bit 7 - e.
__device__ __forceinline__ void bits8(const uint16_t (&h)[8], uint32_t& sg, uint32_t& nz)
{
    sg = 0; nz = 0;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        sg |= (uint32_t)(h[e] >> 15) << (7 - e);
        nz |= (uint32_t)((h[e] & 0x7fff) != 0) << (7 - e);
    }
}

// The same for eight fp16 as they come out of one 16-byte load (element 2i in the low half of word i),
// two halves at a time: a half is nonzero iff adding 0x7fff to its low 15 bits reaches bit 15.
__device__ __forceinline__ void bits8(const uint4 v, uint32_t& sg, uint32_t& nz)
{
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
    sg = 0; nz = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t s = d[i] & 0x80008000u;
        const uint32_t u = d[i] & 0x7fff7fffu;
        const uint32_t z = ((u + 0x7fff7fffu) | u) & 0x80008000u;
        sg |= (s >> (8 + 2 * i)) | (s >> (25 + 2 * i));          // low half -> bit 7 - 2i, high half -> bit 6 - 2i
        nz |= (z >> (8 + 2 * i)) | (z >> (25 + 2 * i));
    }
    sg &= 0xffu; nz &= 0xffu;
}

// fp16 bit patterns of elements k0 .. k0 + 7 of one source row (fp16, or fp32 rounded to fp16 as
// `.to(torch.half)` rounds), after subtracting the zero point if there is one; elements from K on
// read as +0.0.  `row` points at the row's first element.
__device__ __forceinline__ void load8_as_half(const void* row, const bool f32, const int64_t k0, const int64_t K,
                                              const bool centred, const float zf, uint16_t (&h)[8])
{
#pragma unroll
    for (int e = 0; e < 8; e++) h[e] = 0;
    if (k0 >= K) return;
    if (f32) {
        const float* p = reinterpret_cast<const float*>(row) + k0;
        if (k0 + 8 <= K && (((uintptr_t)p) & 15) == 0) {
            const float4 u = *reinterpret_cast<const float4*>(p), v = *reinterpret_cast<const float4*>(p + 4);
            const float f[8] = {u.x, u.y, u.z, u.w, v.x, v.y, v.z, v.w};
#pragma unroll
            for (int e = 0; e < 8; e++) h[e] = half_bits(centred ? __fsub_rn(f[e], zf) : f[e]);
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) if (k0 + e < K) h[e] = half_bits(centred ? __fsub_rn(p[e], zf) : p[e]);
        }
    } else {
        const uint16_t* p = reinterpret_cast<const uint16_t*>(row) + k0;
        if (k0 + 8 <= K && (((uintptr_t)p) & 15) == 0) {
            const uint4 v = *reinterpret_cast<const uint4*>(p);
            h[0] = v.x & 0xffff; h[1] = v.x >> 16; h[2] = v.y & 0xffff; h[3] = v.y >> 16;
            h[4] = v.z & 0xffff; h[5] = v.z >> 16; h[6] = v.w & 0xffff; h[7] = v.w >> 16;
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) if (k0 + e < K) h[e] = p[e];
        }
        if (centred) {
#pragma unroll
            for (int e = 0; e < 8; e++)
                if (k0 + e < K) h[e] = half_bits(__fsub_rn(__half2float(__ushort_as_half(h[e])), zf));
        }
    }
}

// Byte of the tile that holds elements 8c .. 8c + 7 of tile row 0 (add 16 per row): word c >> 2 of the
// row goes to slot h * 32 + r, position q; the row's first element is the word's most significant bit,
// i.e. byte 3 of the little-endian word.
__device__ __forceinline__ int tile_byte_of_chunk(const int c)
{
    return (((c >> 4) * 32) * 4 + ((c >> 2) & 3)) * 4 + (3 - (c & 3));
}

}  // namespace bgemm
