// Design (b): AND-dot on the int8 matrix cores.
//
// CDNA4 has no 1-bit MFMA.  Every mode reduces to the AND-dot D[n,m] = popc(a_m & b_n)
// plus rank-one terms in the row popcounts (see ModeCoef), and D is an ordinary int8
// GEMM of {0,1} matrices.  The operands stay bit-packed all the way into registers:
// one 16-byte load per lane fetches a 32-row x 256-bit tile in exactly the order
// v_mfma_i32_32x32x32_i8 wants its fragments (lane = half*32 + row), and the eight
// 32-deep MFMA steps of the tile are produced by (word >> j) & 0x01010101, which turns
// bit (8c+j) of each word into byte c.  Both operands use the same rule, so the
// K permutation it implies cancels.  Waves never exchange data: no LDS, no barriers
// in the main loop.  Row popcounts for the rank-one terms are accumulated from the
// same registers (4 v_bcnt per fragment per tile).
#include "common.h"

namespace bgemm {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

__device__ __forceinline__ v4i expand_bits(const uint4 w, const int j)
{
    v4i r;
    r.x = (w.x >> j) & 0x01010101u; r.y = (w.y >> j) & 0x01010101u;
    r.z = (w.z >> j) & 0x01010101u; r.w = (w.w >> j) & 0x01010101u;
    return r;
}

__device__ __forceinline__ int popc4(const uint4 w)
{
    return __popc(w.x) + __popc(w.y) + __popc(w.z) + __popc(w.w);
}

// Block = WGN x WGM waves, each wave owns WN x WM tiles of 32x32 outputs, PL activation planes.
template <int WGN, int WGM, int WN, int WM, int PL>
__global__ __launch_bounds__(WGN* WGM * 64) void gemm_mfma_kernel(const GemmArgs a, const int tiles_n,
                                                                   const int tiles_m)
{
    constexpr int NW = WGN * WGM;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wn = wave / WGM, wm = wave % WGM;

    // XCD-aware decode: hardware deals workgroups round-robin over the 8 XCDs, so give
    // each XCD a contiguous run of logical ids (neighbouring tiles then share one L2).
    const unsigned G = gridDim.x;
    unsigned bid = blockIdx.x;
    {
        const unsigned per = G / 8, rem = G % 8, x = bid % 8, y = bid / 8;
        bid = x * per + (x < rem ? x : rem) + y;
    }
    const int per_gemm = tiles_n * tiles_m;
    const int tile_id = bid % per_gemm;
    const int bs = bid / per_gemm;
    const int split = bs % a.splitK, b = bs / a.splitK;
    // group tiles in bands of 8 along n so a band reuses its weight panels
    const int band = 8;
    const int band_id = tile_id / (band * tiles_m), in_band = tile_id % (band * tiles_m);
    const int band_n0 = band_id * band;
    const int band_h = min(band, tiles_n - band_n0);
    const int tn = band_n0 + in_band % band_h, tm = in_band / band_h;

    int kt0, kt1;
    split_range(a.KT, a.splitK, split, &kt0, &kt1);

    const int nt0 = (tn * WGN + wn) * WN, mt0 = (tm * WGM + wm) * WM;
    const uint4* Wb = a.W + (int64_t)b * a.strideW;
    const uint4* Xb = a.X + (int64_t)b * a.strideX;
    const uint4* X2b = PL == 2 ? a.X2 + (int64_t)b * a.strideX : nullptr;

    // per-fragment base pointers (row tile clamped so ragged edges re-read a valid tile)
    const uint4* xp[PL][WN];
    const uint4* wp[WM];
#pragma unroll
    for (int i = 0; i < WN; i++) {
        const int64_t rt = min(nt0 + i, a.NT - 1);
        xp[0][i] = Xb + (rt * a.KT) * TILE_U4 + lane;
        if (PL == 2) xp[PL - 1][i] = X2b + (rt * a.KT) * TILE_U4 + lane;
    }
#pragma unroll
    for (int j = 0; j < WM; j++) {
        const int64_t rt = min(mt0 + j, a.MT - 1);
        wp[j] = Wb + (rt * a.KT) * TILE_U4 + lane;
    }

    v16i acc[PL][WN][WM];
#pragma unroll
    for (int p = 0; p < PL; p++)
#pragma unroll
        for (int i = 0; i < WN; i++)
#pragma unroll
            for (int j = 0; j < WM; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[p][i][j][v] = 0;
    int pa[WM], pb[PL][WN];
#pragma unroll
    for (int j = 0; j < WM; j++) pa[j] = 0;
#pragma unroll
    for (int p = 0; p < PL; p++)
#pragma unroll
        for (int i = 0; i < WN; i++) pb[p][i] = 0;

    uint4 xf[PL][WN], wf[WM], xn[PL][WN], wn_[WM];
    if (kt0 < kt1) {
#pragma unroll
        for (int p = 0; p < PL; p++)
#pragma unroll
            for (int i = 0; i < WN; i++) xn[p][i] = xp[p][i][(int64_t)kt0 * TILE_U4];
#pragma unroll
        for (int j = 0; j < WM; j++) wn_[j] = wp[j][(int64_t)kt0 * TILE_U4];
    }
    for (int kt = kt0; kt < kt1; kt++) {
#pragma unroll
        for (int p = 0; p < PL; p++)
#pragma unroll
            for (int i = 0; i < WN; i++) xf[p][i] = xn[p][i];
#pragma unroll
        for (int j = 0; j < WM; j++) wf[j] = wn_[j];
        if (kt + 1 < kt1) {
#pragma unroll
            for (int p = 0; p < PL; p++)
#pragma unroll
                for (int i = 0; i < WN; i++) xn[p][i] = xp[p][i][(int64_t)(kt + 1) * TILE_U4];
#pragma unroll
            for (int j = 0; j < WM; j++) wn_[j] = wp[j][(int64_t)(kt + 1) * TILE_U4];
        }
#pragma unroll
        for (int j = 0; j < WM; j++) pa[j] += popc4(wf[j]);
#pragma unroll
        for (int p = 0; p < PL; p++)
#pragma unroll
            for (int i = 0; i < WN; i++) pb[p][i] += popc4(xf[p][i]);
#pragma unroll
        for (int s = 0; s < 8; s++) {
            v4i bw[WM];
#pragma unroll
            for (int j = 0; j < WM; j++) bw[j] = expand_bits(wf[j], s);
#pragma unroll
            for (int p = 0; p < PL; p++)
#pragma unroll
                for (int i = 0; i < WN; i++) {
                    const v4i ax = expand_bits(xf[p][i], s);
#pragma unroll
                    for (int j = 0; j < WM; j++)
                        acc[p][i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ax, bw[j], acc[p][i][j], 0, 0, 0);
                }
        }
    }

    // ---- epilogue: rank-one terms, then store or split-K accumulate -----------------
    const int64_t kbit0 = (int64_t)kt0 * TILE_KBITS;
    int64_t kbit1 = (int64_t)kt1 * TILE_KBITS;
    if (kbit1 > a.K) kbit1 = a.K;
    const int bits = kbit1 > kbit0 ? (int)(kbit1 - kbit0) : 0;
#pragma unroll
    for (int j = 0; j < WM; j++) pa[j] += __shfl_xor(pa[j], 32);
#pragma unroll
    for (int p = 0; p < PL; p++)
#pragma unroll
        for (int i = 0; i < WN; i++) pb[p][i] += __shfl_xor(pb[p][i], 32);

    const ModeCoef mc = a.mc;
    const int col = lane & 31, half = lane >> 5;
    const bool direct = a.splitK == 1;
    int* accum = direct ? nullptr : a.ws_acc + (int64_t)b * a.N * a.M;
    char* outb = reinterpret_cast<char*>(a.out);
    const int64_t out_off = (int64_t)b * a.strideC;
#pragma unroll
    for (int i = 0; i < WN; i++) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int nrow = 8 * (v >> 2) + 4 * half + (v & 3);
            const int pbv = __shfl(pb[0][i], nrow);
            const int pbv2 = PL == 2 ? __shfl(pb[PL - 1][i], nrow) : 0;
            const int64_t n = (int64_t)(nt0 + i) * 32 + nrow;
#pragma unroll
            for (int j = 0; j < WM; j++) {
                const int64_t m = (int64_t)(mt0 + j) * 32 + col;
                int val = mc.c0 * bits + mc.ca * pa[j] + mc.cb * pbv + mc.cd * acc[0][i][j][v];
                if (PL == 2) val += mc.cb2 * pbv2 + mc.cd2 * acc[PL - 1][i][j][v];
                if (n < a.N && m < a.M) {
                    if (direct) store_out(outb, a.out_f16, out_off + n * a.M + m, val);
                    else atomicAdd(accum + n * a.M + m, val);
                }
            }
        }
    }
    if (direct) return;

    // ---- split-K: the last split to arrive on this output tile publishes it ---------
    __shared__ int s_last;
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned t = atomicAdd(a.ws_cnt + (int64_t)b * per_gemm + tile_id, 1u);
        s_last = (t == (unsigned)a.splitK - 1u);
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    constexpr int BN = WGN * WN * 32, BM = WGM * WM * 32;
    const int64_t n_base = (int64_t)tn * BN, m_base = (int64_t)tm * BM;
    for (int e = threadIdx.x; e < BN * BM; e += NW * 64) {
        const int64_t n = n_base + e / BM, m = m_base + e % BM;
        if (n < a.N && m < a.M) {
            const int v = atomicExch(accum + n * a.M + m, 0);   // read the sum and leave zero behind
            store_out(outb, a.out_f16, out_off + n * a.M + m, v);
        }
    }
    if (threadIdx.x == 0) atomicExch(a.ws_cnt + (int64_t)b * per_gemm + tile_id, 0u);
}

struct TileCfg { int bn, bm; };

template <int WGN, int WGM, int WN, int WM>
static int launch_cfg(const GemmArgs& a, hipStream_t st)
{
    constexpr int BN = WGN * WN * 32, BM = WGM * WM * 32;
    const int tiles_n = (int)cdiv(a.N, BN), tiles_m = (int)cdiv(a.M, BM);
    const int64_t grid = (int64_t)a.batch * a.splitK * tiles_n * tiles_m;
    if (grid <= 0 || grid > 0x7fffffffLL) return fail(BGEMM_EINVAL, "gemm_mfma: grid of %lld blocks", (long long)grid);
    if (a.mc.planes == 2) {
        // two accumulator sets: only the tiles whose registers fit are built for two planes
        if constexpr (WN * WM <= 4)
            hipLaunchKernelGGL((gemm_mfma_kernel<WGN, WGM, WN, WM, 2>), dim3((unsigned)grid), dim3(WGN * WGM * 64), 0,
                               st, a, tiles_n, tiles_m);
        else
            return fail(BGEMM_EINVAL, "gemm_mfma: tile not built for two planes");
    } else
        hipLaunchKernelGGL((gemm_mfma_kernel<WGN, WGM, WN, WM, 1>), dim3((unsigned)grid), dim3(WGN * WGM * 64), 0, st,
                           a, tiles_n, tiles_m);
    return check_launch("gemm_mfma");
}

// Tile choice: the largest tile that still yields about two blocks per CU.
static int pick_cfg(const GemmArgs& a)
{
    const int64_t want = 512;
    auto blocks = [&](int bn, int bm) { return (int64_t)a.batch * a.splitK * cdiv(a.N, bn) * cdiv(a.M, bm); };
    if (a.mc.planes == 1 && blocks(256, 256) >= want) return 0;
    if (blocks(128, 128) >= want) return 1;
    if (blocks(64, 128) >= want || a.N > 32) return 2;
    return 3;
}

size_t gemm_mfma_ws_bytes(int64_t batch, int64_t M, int64_t N, int64_t K, int splitK, int planes)
{
    (void)K; (void)planes;
    if (splitK <= 1) return 0;
    // running sums + one counter per smallest tile (32 x 128 outputs), rounded to 256 bytes
    const size_t accb = (size_t)batch * N * M * 4;
    const size_t cnt = (size_t)batch * cdiv(N, 32) * cdiv(M, 128) * 4;
    return ((accb + 255) / 256) * 256 + ((cnt + 255) / 256) * 256;
}

int launch_gemm_mfma(const GemmArgs& a, hipStream_t st)
{
    switch (pick_cfg(a)) {
    case 0: return launch_cfg<2, 2, 4, 4>(a, st);    // 256 x 256
    case 1: return launch_cfg<2, 2, 2, 2>(a, st);    // 128 x 128
    case 2: return launch_cfg<1, 4, 2, 1>(a, st);    // 64 x 128
    default: return launch_cfg<1, 4, 1, 1>(a, st);   // 32 x 128
    }
}

}  // namespace bgemm
