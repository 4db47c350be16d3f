// Skinny GEMM for decode-like shapes: the activation side fits one 32-row MFMA operand
// (N <= 32 binary rows, or N <= 16 ternary rows whose two planes share the operand), so the
// work is one pass over the packed weights and the kernel is HBM-bound.
//
// A block owns RT weight row tiles; its KW waves split K between them (the in-kernel split-K:
// no workspace, no second launch, no atomics on global memory) and meet in LDS, where the
// partial accumulators are summed, the rank-one terms applied and the rows stored.
#include "common.h"
#include "mfma_engines.h"

namespace bgemm {

template <typename Eng, int RT, int KW>
__global__ __launch_bounds__(KW * 64) void gemm_skinny_kernel(const GemmArgs a, const int groups)
{
    __shared__ int sAcc[KW][RT][16][64];
    __shared__ int sPa[RT][32], sPb[32];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = lane >> 5, r = lane & 31;
    const int b = blockIdx.x / groups, grp = blockIdx.x % groups;
    const bool two = a.mc.planes == 2;

    if (threadIdx.x < 32) {
        sPb[threadIdx.x] = 0;
#pragma unroll
        for (int t = 0; t < RT; t++) sPa[t][threadIdx.x] = 0;
    }

    int kt0, kt1;
    split_range(a.KT, KW, wave, &kt0, &kt1);

    // activation operand: one tile row; with two planes rows 0..15 come from the nonzero plane
    // and rows 16..31 from the sign&nonzero plane (both hold at most 16 real rows)
    const uint4* xp = (two && r >= 16 ? a.X2 + (h * 32 + r - 16) : a.X + lane) + (int64_t)b * a.strideX;
    const uint4* wp[RT];
#pragma unroll
    for (int t = 0; t < RT; t++) {
        const int64_t rt = min((int64_t)grp * RT + t, (int64_t)a.MT - 1);
        wp[t] = a.W + (int64_t)b * a.strideW + rt * a.KT * TILE_U4 + lane;
    }

    typename Eng::Acc acc[RT];
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][v] = 0;
    int pa[RT], pb = 0;
#pragma unroll
    for (int t = 0; t < RT; t++) pa[t] = 0;

    // all of this wave's K range is requested up front: the ranges are short (K/KW) and the
    // kernel lives on memory-level parallelism
    constexpr int MAXT = 4;                      // K-tiles kept in flight per wave
    for (int kb = kt0; kb < kt1; kb += MAXT) {
        uint4 xq[MAXT], wq[MAXT][RT];
#pragma unroll
        for (int q = 0; q < MAXT; q++) {
            const int64_t off = (int64_t)min(kb + q, kt1 - 1) * TILE_U4;
            xq[q] = xp[off];
#pragma unroll
            for (int t = 0; t < RT; t++) wq[q][t] = wp[t][off];
        }
#pragma unroll
        for (int q = 0; q < MAXT; q++) {
            if (kb + q >= kt1) break;
            pb += popc4(xq[q]);
#pragma unroll
            for (int t = 0; t < RT; t++) pa[t] += popc4(wq[q][t]);
#pragma unroll
            for (int s = 0; s < Eng::STEPS; s++) {
                const typename Eng::Frag ax = Eng::expand(xq[q], s);
#pragma unroll
                for (int t = 0; t < RT; t++) acc[t] = Eng::mma(ax, Eng::expand(wq[q][t], s), acc[t]);
            }
        }
    }

    // ---- meet in LDS ---------------------------------------------------------------------------
    pb += __shfl_xor(pb, 32);
#pragma unroll
    for (int t = 0; t < RT; t++) pa[t] += __shfl_xor(pa[t], 32);
    __syncthreads();                 // popcount arrays are zeroed
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) sAcc[wave][t][v][lane] = Eng::to_int(acc[t], v);
    if (lane < 32) {
        atomicAdd(&sPb[lane], pb);
#pragma unroll
        for (int t = 0; t < RT; t++) atomicAdd(&sPa[t][lane], pa[t]);
    }
    __syncthreads();

    // ---- reduce, apply the mode's rank-one terms, store -------------------------------------------
    const ModeCoef mc = a.mc;
    const int out_rows = two ? 8 : 16;           // accumulator rows that carry outputs
    const int kbits = (int)a.K;
    for (int job = wave; job < RT * out_rows; job += KW) {
        const int t = job / out_rows, v = job % out_rows;
        int d = 0, d2 = 0;
#pragma unroll
        for (int w = 0; w < KW; w++) {
            d += sAcc[w][t][v][lane];
            if (two) d2 += sAcc[w][t][v + 8][lane];
        }
        const int n = 8 * (v >> 2) + 4 * h + (v & 3);
        const int64_t m = ((int64_t)grp * RT + t) * 32 + r;
        int val = __mul24(mc.c0, kbits) + __mul24(mc.ca, sPa[t][r]) + __mul24(mc.cb, sPb[n]) + __mul24(mc.cd, d);
        if (two) val += __mul24(mc.cb2, sPb[n + 16]) + __mul24(mc.cd2, d2);
        if (n < a.N && m < a.M) store_out(a, (int64_t)b * a.strideC + (int64_t)n * a.M, m, val);
    }
}

bool gemm_skinny_eligible(const GemmArgs& a)
{
    return a.mc.planes == 2 ? a.N <= 16 : a.N <= 32;
}

template <typename Eng, int RT>
static int launch_rt(const GemmArgs& a, hipStream_t st)
{
    const int groups = (int)cdiv(a.MT, RT);
    const int64_t blocks = (int64_t)a.batch * groups;
    if (blocks > 0x7fffffffLL) return fail(BGEMM_EINVAL, "gemm_skinny: grid of %lld blocks", (long long)blocks);
    // K ways per block: at least what the caller asked for, more when the grid alone would leave the
    // chip mostly idle (about four waves per SIMD wanted), never more than there are K-tiles
    constexpr int KW_MAX = 8 / RT;               // the LDS meeting area is KW * RT * 4 KiB
    int kw = 1;
    while (kw < KW_MAX && (kw < a.splitK || blocks * kw < 4096) && kw * 2 <= a.KT) kw *= 2;
    const dim3 g((unsigned)blocks);
    if (kw == 1) hipLaunchKernelGGL((gemm_skinny_kernel<Eng, RT, 1>), g, dim3(64), 0, st, a, groups);
    else if (kw == 2) hipLaunchKernelGGL((gemm_skinny_kernel<Eng, RT, 2>), g, dim3(128), 0, st, a, groups);
    else if (kw == 4) hipLaunchKernelGGL((gemm_skinny_kernel<Eng, RT, 4>), g, dim3(256), 0, st, a, groups);
    else if constexpr (KW_MAX >= 8) hipLaunchKernelGGL((gemm_skinny_kernel<Eng, RT, 8>), g, dim3(512), 0, st, a, groups);
    return check_launch("gemm_skinny");
}

int launch_gemm_skinny(const GemmArgs& a, hipStream_t st, bool fp4)
{
    // two row tiles per block share one expansion of the activation fragment once there are
    // enough row tiles to keep every CU busy anyway
    const bool rt2 = (int64_t)a.batch * a.MT >= 2048;
    if (fp4) return rt2 ? launch_rt<EngF4, 2>(a, st) : launch_rt<EngF4, 1>(a, st);
    return rt2 ? launch_rt<EngI8, 2>(a, st) : launch_rt<EngI8, 1>(a, st);
}

}  // namespace bgemm
