// Design (a): AND + popcount on the vector ALU (v_and_b32 + v_bcnt_u32_b32).
//
// A general register-tiled kernel: a 256-thread block owns 64 x 64 outputs, stages one
// 256-bit K-tile of both operands through LDS in the tiled order (so the 16-byte LDS
// reads of neighbouring lanes are contiguous) and every thread accumulates a 4 x 4
// patch.  Like the MFMA kernel it computes the AND-dot and applies the mode's integer
// epilogue from the row popcounts, which the loading threads collect for free.
#include "common.h"

namespace bgemm {

__device__ __forceinline__ int popc4v(const uint4 w)
{
    return __popc(w.x) + __popc(w.y) + __popc(w.z) + __popc(w.w);
}

__device__ __forceinline__ int and_popc(const uint4 a, const uint4 b, int acc)
{
    acc += __popc(a.x & b.x); acc += __popc(a.y & b.y);
    acc += __popc(a.z & b.z); acc += __popc(a.w & b.w);
    return acc;
}

template <int PL>
__global__ __launch_bounds__(256) void gemm_valu_kernel(const GemmArgs a, const int tiles_n, const int tiles_m)
{
    __shared__ uint4 sX[PL][2][128];     // [plane][buffer][row tile (2) x slot (64)]
    __shared__ uint4 sW[2][128];
    __shared__ int sPopX[PL][64], sPopW[64];
    __shared__ int s_last;

    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int per_gemm = tiles_n * tiles_m;
    const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int split = bid % a.splitK;
    const unsigned rest = bid / a.splitK;
    const int tile_id = rest % per_gemm, b = rest / per_gemm;
    if (b >= a.batch) return;                    // padding blocks of a split-K grid
    const int tn = tile_id / tiles_m, tm = tile_id % tiles_m;
    int kt0, kt1;
    split_range(a.KT, a.splitK, split, &kt0, &kt1);

    // loader role: threads 0..127 fetch the activation tile slots, 128..255 the weight ones
    const bool loadsX = tid < 128;
    const int lslot = tid & 127, lrt = lslot >> 6;
    const uint4* lsrc; const uint4* lsrc2 = nullptr;
    if (loadsX) {
        const int64_t rt = min((int64_t)tn * 2 + lrt, (int64_t)a.NT - 1);
        lsrc = a.X + (int64_t)b * a.strideX + rt * a.KT * TILE_U4 + (lslot & 63);
        if (PL == 2) lsrc2 = a.X2 + (int64_t)b * a.strideX + rt * a.KT * TILE_U4 + (lslot & 63);
    } else {
        const int64_t rt = min((int64_t)tm * 2 + lrt, (int64_t)a.MT - 1);
        lsrc = a.W + (int64_t)b * a.strideW + rt * a.KT * TILE_U4 + (lslot & 63);
    }
    if (tid < 64) { sPopW[tid] = 0; for (int p = 0; p < PL; p++) sPopX[p][tid] = 0; }
    __syncthreads();

    int acc[PL][4][4];
#pragma unroll
    for (int p = 0; p < PL; p++)
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[p][i][j] = 0;
    int mypop = 0, mypop2 = 0;

    // LDS slot of row `row` (0..63) for K half h: tiled order inside each 32-row tile
    auto slot_of = [](int row, int h) { return (row >> 5) * 64 + h * 32 + (row & 31); };

    uint4 g0 = make_uint4(0, 0, 0, 0), g1 = g0;
    if (kt0 < kt1) { g0 = lsrc[(int64_t)kt0 * TILE_U4]; if (PL == 2 && loadsX) g1 = lsrc2[(int64_t)kt0 * TILE_U4]; }
    for (int kt = kt0; kt < kt1; kt++) {
        const int buf = (kt - kt0) & 1;
        if (loadsX) { sX[0][buf][lslot] = g0; if (PL == 2) sX[PL - 1][buf][lslot] = g1; }
        else sW[buf][lslot] = g0;
        mypop += popc4v(g0);
        if (PL == 2) mypop2 += popc4v(g1);
        if (kt + 1 < kt1) {
            g0 = lsrc[(int64_t)(kt + 1) * TILE_U4];
            if (PL == 2 && loadsX) g1 = lsrc2[(int64_t)(kt + 1) * TILE_U4];
        }
        __syncthreads();   // one barrier per K-tile: the two LDS buffers alternate
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint4 w[4];
#pragma unroll
            for (int j = 0; j < 4; j++) w[j] = sW[buf][slot_of(tx + 16 * j, h)];
#pragma unroll
            for (int p = 0; p < PL; p++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint4 x = sX[p][buf][slot_of(ty + 16 * i, h)];
#pragma unroll
                    for (int j = 0; j < 4; j++) acc[p][i][j] = and_popc(x, w[j], acc[p][i][j]);
                }
        }
    }
    // row popcounts: each loader owns (row, half) of one operand
    {
        const int row = lrt * 32 + (lslot & 31);
        if (loadsX) { atomicAdd(&sPopX[0][row], mypop); if (PL == 2) atomicAdd(&sPopX[PL - 1][row], mypop2); }
        else atomicAdd(&sPopW[row], mypop);
    }
    __syncthreads();

    const int64_t kbit0 = (int64_t)kt0 * TILE_KBITS;
    int64_t kbit1 = (int64_t)kt1 * TILE_KBITS;
    if (kbit1 > a.K) kbit1 = a.K;
    const int bits = kbit1 > kbit0 ? (int)(kbit1 - kbit0) : 0;
    const ModeCoef mc = a.mc;
    int val[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int t = mc.c0 * bits + mc.ca * sPopW[tx + 16 * j] + mc.cb * sPopX[0][ty + 16 * i] + mc.cd * acc[0][i][j];
            if (PL == 2) t += mc.cb2 * sPopX[PL - 1][ty + 16 * i] + mc.cd2 * acc[PL - 1][i][j];
            val[i][j] = t;
        }
    if (a.splitK > 1) {
        // partial tiles in register order; the last split to arrive adds the others to its own
        int4* tile_base = reinterpret_cast<int4*>(a.ws_part) + ((int64_t)b * per_gemm + tile_id) * a.splitK * 1024;
        int4* mine = tile_base + (int64_t)split * 1024 + tid;
#pragma unroll
        for (int i = 0; i < 4; i++) mine[i * 256] = make_int4(val[i][0], val[i][1], val[i][2], val[i][3]);
        if (!splitk_arrive(a.ws_cnt + (int64_t)b * per_gemm + tile_id, (unsigned)a.splitK, &s_last)) return;
        for (int s = 0; s < a.splitK; s++) {
            if (s == split) continue;
            const int4* other = tile_base + (int64_t)s * 1024;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int4 o = load_partial(other, (unsigned)(tid + i * 256) * 16u);
                val[i][0] += o.x; val[i][1] += o.y; val[i][2] += o.z; val[i][3] += o.w;
            }
        }
    }
    const int64_t out_off = (int64_t)b * a.strideC;
    if (bits_kind(a.out_kind)) {
        // a wave holds rows ty = 4w .. 4w+3 (16 lanes each); columns tx + 16 j: two j make one 32-bit word
        const int lane = tid & 63, g = lane >> 4;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int64_t n = (int64_t)tn * 64 + ty + 16 * i;
#pragma unroll
            for (int jj = 0; jj < 2; jj++) {
                unsigned field[2];
#pragma unroll
                for (int q = 0; q < 2; q++) {
                    const int64_t m = (int64_t)tm * 64 + tx + 16 * (2 * jj + q);
                    const bool real = n < a.N && m < a.M;
                    const unsigned long long bal = __ballot(real && next_sign_bit(a, m, val[i][2 * jj + q]) != 0);
                    field[q] = (unsigned)(bal >> (16 * g)) & 0xffffu;
                }
                const int64_t m32 = (int64_t)tm * 64 + 32 * jj;
                if (tx == 0 && n < a.N && m32 < a.M)
                    reinterpret_cast<uint32_t*>(a.out)[out_off + tiled_word_offset(n, m32 >> 5, k_tiles(a.M))] =
                        __brev(field[0] | (field[1] << 16));
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int64_t n = (int64_t)tn * 64 + ty + 16 * i;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int64_t m = (int64_t)tm * 64 + tx + 16 * j;
            if (n < a.N && m < a.M) store_out(a, out_off + n * a.M, m, val[i][j]);
        }
    }
}

void gemm_valu_ws(int64_t batch, int64_t M, int64_t N, int64_t K, int splitK, int planes, size_t* part_bytes, size_t* counters)
{
    (void)planes;
    const int64_t tiles = batch * cdiv(N, 64) * cdiv(M, 64);
    const int s = effective_split(tiles, splitK, (int)k_tiles(K));       // as launch_gemm_valu will split
    *part_bytes = s > 1 ? (size_t)tiles * s * 64 * 64 * 4 : 0;
    *counters = s > 1 ? (size_t)tiles : 0;
}

int launch_gemm_valu(const GemmArgs& a_in, hipStream_t st)
{
    GemmArgs a = a_in;
    const int tiles_n = (int)cdiv(a.N, 64), tiles_m = (int)cdiv(a.M, 64);
    a.splitK = effective_split((int64_t)a.batch * tiles_n * tiles_m, a.splitK, a.KT);
    const int64_t grid = splitk_grid((int64_t)a.batch * a.splitK * tiles_n * tiles_m, a.splitK);
    if (grid <= 0 || grid > 0x7fffffffLL) return fail(BGEMM_EINVAL, "gemm_valu: grid of %lld blocks", (long long)grid);
    if (a.mc.planes == 2)
        hipLaunchKernelGGL((gemm_valu_kernel<2>), dim3((unsigned)grid), dim3(256), 0, st, a, tiles_n, tiles_m);
    else
        hipLaunchKernelGGL((gemm_valu_kernel<1>), dim3((unsigned)grid), dim3(256), 0, st, a, tiles_n, tiles_m);
    return check_launch("gemm_valu");
}

}  // namespace bgemm
