// Skinny GEMM for decode-like shapes: the activation side fits one 32-row MFMA operand
// (N <= 32 binary rows, or N <= 16 ternary rows whose two planes share the operand), so the
// work is one pass over the packed weights and the kernels are HBM-bound.  Weight tiles are
// read once and streamed past the caches (non-temporal loads); the activation tiles are
// re-read by every wave and stay cached.
//
// Three kernels:
//  * gemm_skinny_stream_kernel: every wave owns RT weight row tiles over the whole K and keeps
//    its accumulators to the end: no LDS, no barriers, nothing shared between waves.  Used when
//    there are enough row tiles (a batch of weight matrices, a very tall one) to fill the chip.
//  * gemm_skinny_splitk_kernel: a block owns one row tile and its KW waves split K between them
//    (the in-kernel split-K: no workspace, no second launch, no atomics on global memory); the
//    partial sums meet in LDS through ds_add.  Used for a single decode-size matrix, which has
//    too few row tiles to occupy every SIMD otherwise, and, one 32 x 32 piece of the output per
//    block, for outputs of up to about a thousand such pieces.
//  * gemm_skinny_splitk_quad_kernel: the same with a 64 x 64 piece per block (four accumulators a
//    wave), for a few thousand pieces over a long K.
#include "common.h"
#include "mfma_engines.h"
#include "pack_bits.h"
#include <type_traits>

namespace bgemm {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// Weight tiles are used exactly once: keep them out of the way of the activation tiles.
__device__ __forceinline__ uint4 load_stream(const uint4* p)
{
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

// Pointer to this lane's slot of the activation operand's first K-tile.  With two planes, rows
// 0..15 of the operand come from the nonzero plane and rows 16..31 from the sign&nonzero plane
// (both hold at most 16 real rows), so one MFMA yields both dots.
// `half` picks rows 0..15 or 16..31 of the activation tile row for the two-plane operand.
__device__ __forceinline__ const uint4* skinny_x_ptr(const GemmArgs& a, const int b, const int lane, const int half = 0)
{
    const int h = lane >> 5, r = lane & 31;
    if (a.mc.planes != 2) return a.X + lane + (int64_t)b * a.strideX;
    return (r >= 16 ? a.X2 : a.X) + (h * 32 + half * 16 + (r & 15)) + (int64_t)b * a.strideX;
}

// ---- streaming kernel --------------------------------------------------------------------------
template <typename Eng, int RT>
__global__ __launch_bounds__(256, 2) void gemm_skinny_stream_kernel(const GemmArgs a, const int groups)
{
    constexpr int CH = 2;                        // K-tiles per chunk; two chunks are in flight
    const int lane = threadIdx.x & 63;
    const int h = lane >> 5, r = lane & 31;
    const int64_t gid = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int b = (int)(gid / groups), grp = (int)(gid % groups);
    if (b >= a.batch) return;                    // whole wave leaves together
    const bool two = a.mc.planes == 2;

    const uint4* xp = skinny_x_ptr(a, b, lane);
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

    // a chunk that starts inside K is fetched whole: K-tiles past the end are read again from the
    // last one and skipped when the chunk is consumed
    const int kt_last = a.KT - 1;
    uint4 xq0[CH], xq1[CH], wq0[CH][RT], wq1[CH][RT];
    auto fetch = [&](uint4 (&xq)[CH], uint4 (&wq)[CH][RT], const int kb) {
        if (kb > kt_last) return;
#pragma unroll
        for (int q = 0; q < CH; q++) {
            const int64_t off = (int64_t)min(kb + q, kt_last) * TILE_U4;
            xq[q] = xp[off];
#pragma unroll
            for (int t = 0; t < RT; t++) wq[q][t] = load_stream(wp[t] + off);
        }
    };
    auto consume = [&](const uint4 (&xq)[CH], const uint4 (&wq)[CH][RT], const int kb) {
#pragma unroll
        for (int q = 0; q < CH; q++) {
            if (kb + q > kt_last) break;
            pb += popc4(xq[q]);
#pragma unroll
            for (int t = 0; t < RT; t++) pa[t] += popc4(wq[q][t]);
#pragma unroll
            for (int s = 0; s < Eng::STEPS; s++) {
                const typename Eng::Frag ax = Eng::expand_x(xq[q], s);
#pragma unroll
                for (int t = 0; t < RT; t++) acc[t] = Eng::mma(ax, Eng::expand_w(wq[q][t], s), acc[t]);
            }
        }
    };
    fetch(xq0, wq0, 0);
    for (int kb = 0; kb < a.KT; kb += 2 * CH) {
        fetch(xq1, wq1, kb + CH);
        consume(xq0, wq0, kb);
        fetch(xq0, wq0, kb + 2 * CH);
        consume(xq1, wq1, kb + CH);
    }

    // ---- rank-one terms and store, straight from the accumulators ---------------------------------
    // The vector ALU is shared by the waves of a SIMD, so what a wave spends here is not hidden behind
    // the others' loads: row terms and addresses are formed once, and the plain kinds get loops of
    // their own with nothing but a multiply-add, a conversion and the store per output.
    pb += __shfl_xor(pb, 32);                    // lane r (either half) now holds the popcount of operand row r
#pragma unroll
    for (int t = 0; t < RT; t++) pa[t] += __shfl_xor(pa[t], 32);
    const ModeCoef mc = a.mc;
    const int NV = two ? 8 : 16;                 // rows 16..31 of a two-plane operand are the second plane
    int colterm[RT];
    bool col_ok[RT];
#pragma unroll
    for (int t = 0; t < RT; t++) {
        colterm[t] = mc.c0 * (int)a.K + mc.ca * pa[t];
        col_ok[t] = ((int64_t)grp * RT + t) * 32 + r < a.M;
    }
    const int64_t m0 = (int64_t)grp * RT * 32 + r;                        // column of tile 0
    const int64_t out_row0 = (int64_t)b * a.strideC;
    auto row_of = [&](const int v) { return 8 * (v >> 2) + 4 * h + (v & 3); };
    auto value = [&](const int v, const int t, const int rowterm) {
        const int base = colterm[t] + rowterm;
        return two ? base + dot_terms2(mc, Eng::to_int(acc[t], v), Eng::to_int(acc[t], (v + 8) & 15)) : base + dot_term(mc, Eng::to_int(acc[t], v));
    };
    // row terms: the popcounts sit in lanes 0..31; both candidates (lane half 0 / 1) are read as
    // scalars and selected, which costs no LDS round trip
    auto row_term = [&](const int v) {
        const int n0 = 8 * (v >> 2) + (v & 3), n1 = n0 + 4;
        int t0 = mc.cb * __builtin_amdgcn_readlane(pb, n0), t1 = mc.cb * __builtin_amdgcn_readlane(pb, n1);
        if (two) {
            t0 += mc.cb2 * __builtin_amdgcn_readlane(pb, (n0 + 16) & 31);
            t1 += mc.cb2 * __builtin_amdgcn_readlane(pb, (n1 + 16) & 31);
        }
        return h ? t1 : t0;
    };
    if (a.out_kind == BGEMM_OUT_I32 || a.out_kind == BGEMM_OUT_F16) {
        const bool wide = a.out_kind == BGEMM_OUT_I32;
        // from a handful of rows on the output is a noticeable share of the traffic and is written past the
        // caches (timed: 5 to 7 % at 6 to 16 rows, while at 1 to 4 rows ordinary stores are 3 % faster)
        const bool past_cache = wide && a.N > 4;
        const int sh = wide ? 2 : 1;
        const int64_t row_bytes = a.M << sh;
        char* const base = reinterpret_cast<char*>(a.out) + ((out_row0 + m0) << sh) + 4 * h * row_bytes;
        if (RT == 2 && wide && a.N <= 4 && ((int64_t)grp * RT + RT) * 32 <= a.M) {
            // Up to four rows live in lane half 0 alone (rows 4 .. 7 would be half 1's): the second tile's value moves
            // over to half 1, and a row's 64 outputs leave as ONE 256-byte store of all lanes instead of two 128-byte
            // stores of half of them (64 matrices x 4 rows in a launch: 67.1 -> 65.2 us, 0.69 -> 0.71 of 8 TB/s).
            // (With more rows both halves hold outputs and would have to swap one value each per store for the same effect:
            // 64 matrices x 16 rows 78.3 us that way against 73.1 with the two 128-byte pieces per store below.)
            char* const row0 = reinterpret_cast<char*>(a.out) + ((out_row0 + (m0 - r)) << 2) + lane * 4;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                int rowterm = mc.cb * __builtin_amdgcn_readlane(pb, v);
                if (two) rowterm += mc.cb2 * __builtin_amdgcn_readlane(pb, v + 16);
                const int v0 = value(v, 0, rowterm), v1 = value(v, 1, rowterm);
                const int moved = __shfl(v1, lane & 31);
                if (v < a.N) *reinterpret_cast<int*>(row0 + v * row_bytes) = h ? moved : v0;
            }
            return;
        }
#pragma unroll
        for (int v = 0; v < 16; v++) {
            if (v >= NV) break;
            const int rowterm = row_term(v);
            if (row_of(v) >= a.N) continue;
            char* const rowp = base + (8 * (v >> 2) + (v & 3)) * row_bytes;       // uniform offset from the lane's base
#pragma unroll
            for (int t = 0; t < RT; t++) {
                if (!col_ok[t]) continue;
                const int val = value(v, t, rowterm);
                if (past_cache) __builtin_nontemporal_store(val, reinterpret_cast<int*>(rowp + t * 128));
                else if (wide) *reinterpret_cast<int*>(rowp + t * 128) = val;
                else *reinterpret_cast<__half*>(rowp + t * 64) = __float2half_rn((float)val);
            }
        }
        return;
    }
#pragma unroll
    for (int v = 0; v < 16; v++) {
        if (v >= NV) break;
        const int n = row_of(v);
        const int rowterm = row_term(v);
        if (n >= a.N) continue;
#pragma unroll
        for (int t = 0; t < RT; t++) {
            const int64_t m = m0 + t * 32;
            const int val = value(v, t, rowterm);
            if (bits_kind(a.out_kind))          // a half-wave holds the 32 columns of this row tile for row n
                store_bits_word(a, b, n, m - r, m < a.M ? next_sign_bit(a, m, val) : 0u);
            else if (m < a.M)
                store_out(a, out_row0 + (int64_t)n * a.M, m, val);
        }
    }
}

// ---- split-K kernel ----------------------------------------------------------------------------
// One block per (weight row tile, activation tile row): a 32 x 32 piece of the output, with K split over
// the block's KW waves.  blockIdx.y walks the activation tile rows, so outputs of a few hundred such pieces
// (a batch of 128 rows against a thousand weight rows, 512 x 512 with a long K) put KW waves on every piece,
// each on a short K range with all of its loads in flight, instead of a few waves walking all of K.
// FUSEX: the activations arrive unpacked (fp16 or fp32 rows, optionally minus a zero point): every wave
// builds the activation tiles of its own K range itself, in LDS, while its weight loads are in flight,
// which saves the separate pack launch of a decode step (a third of its time).  One tile row, batch == 1.
// Two bit planes (a ternary operand): 16 rows of both planes share one 32-row operand, rows 0..15 from the
// nonzero plane and 16..31 from the sign plane, so one MFMA yields both dots; up to 32 rows are taken that way,
// 16 a block (blockIdx.y & 1 picks the half of the tile row).  PL2: more rows than that; every block takes 32
// rows of each plane as two operands against one expansion of the weight tile, two accumulators, which halves
// the blocks and the weight traffic (64 to 128 rows: 8 to 15 % faster; up to 32 rows the half blocks win by
// 10 to 20 %, twice the blocks with half the matrix-core chain each).
template <typename Eng, int KW, bool FUSEX = false, bool PL2 = false>
__global__ __launch_bounds__(KW * 64, FUSEX && KW <= 8 ? 4 : 2) void gemm_skinny_splitk_kernel(const GemmArgs a)
{
    static_assert(!(FUSEX && PL2), "in-kernel activation packing is built for up to four rows");
    constexpr int NT = KW * 64, NP = PL2 ? 2 : 1;
    constexpr int MAXT = FUSEX ? 2 : 4;
    __shared__ int sAcc[NP][16][64];             // accumulator layout of the MFMA: [v][lane]
    __shared__ int sPa[32], sPb[NP][32];
    __shared__ __align__(16) unsigned char sX[FUSEX ? KW : 1][FUSEX ? MAXT : 1][FUSEX ? 1024 : 16];

    // the wave index as a scalar: the wave's K range and every address derived from it stay on the scalar unit
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rt = blockIdx.x, b = blockIdx.z;   // weight row tile, matrix of the batch
    const bool two = !PL2 && a.mc.planes == 2;   // both planes in one operand, 16 rows a block
    const int nt = two ? blockIdx.y >> 1 : blockIdx.y, nbase = two ? blockIdx.y * 16 : blockIdx.y * 32;

    int kt0, kt1;
    split_range(a.KT, KW, wave, &kt0, &kt1);

    const uint4* const xp = FUSEX ? nullptr
                            : (PL2 ? a.X + lane + (int64_t)b * a.strideX : skinny_x_ptr(a, b, lane, blockIdx.y & 1)) + (int64_t)nt * a.KT * TILE_U4;
    const uint4* const xp2 = PL2 ? a.X2 + lane + (int64_t)b * a.strideX + (int64_t)nt * a.KT * TILE_U4 : nullptr;
    const uint4* wp = a.W + (int64_t)b * a.strideW + (int64_t)rt * a.KT * TILE_U4 + lane;

    typename Eng::Acc acc, acc2;                 // acc2: the second plane's dots (PL2)
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = acc2[v] = 0;
    int pa = 0, pb = 0, pb2 = 0;

    // FUSEX: the activation tiles of this wave's K-tiles are built by the wave in its own LDS area: row n of
    // the source goes to operand row n (sign bits) or, with two planes, its nonzero bits to row n and
    // sign & nonzero to row n + 16; everything else in a tile is zero.  Lane (c = lane & 31, lane >> 5) takes
    // elements 8c .. 8c + 7 of rows (lane >> 5) + 2j.  The loads of the first four rows go out BEFORE the
    // weight loads (loads return in order: behind them they could only be used once the weights are in),
    // and are turned into bits while the weights are in flight.
    float xzf = 0.f;
    if (FUSEX && a.xzp)
        xzf = a.xsrc_f32 ? *reinterpret_cast<const float*>(a.xzp) : __half2float(*reinterpret_cast<const __half*>(a.xzp));
    const int xc = lane & 31, xb0 = tile_byte_of_chunk(xc), xr = lane >> 5;
    const bool xfast = FUSEX && !a.xsrc_f32 && (a.K & 7) == 0 && ((((uintptr_t)a.xsrc) | (uintptr_t)(a.xld * 2)) & 15) == 0;
    auto x_put_bits = [&](unsigned char* const t, const int n, const uint32_t sg, const uint32_t nz) {
        if (two) {
            t[xb0 + n * 16] = (unsigned char)nz;
            t[xb0 + (n + 16) * 16] = (unsigned char)(sg & nz);
        } else
            t[xb0 + n * 16] = (unsigned char)sg;
    };
    auto x_put = [&](unsigned char* const t, const int n, uint16_t (&hb)[8]) {
        uint32_t sg, nz;
        bits8(hb, sg, nz);
        if (two) {
            t[xb0 + n * 16] = (unsigned char)nz;
            t[xb0 + (n + 16) * 16] = (unsigned char)(sg & nz);
        } else
            t[xb0 + n * 16] = (unsigned char)sg;
    };
    auto x_rows_slow = [&](unsigned char* const t, const int kt, const int n_from) {
        const int64_t esz = a.xsrc_f32 ? 4 : 2;
        for (int n = n_from + xr; n < (int)a.N; n += 2) {
            uint16_t hb[8];
            load8_as_half(reinterpret_cast<const char*>(a.xsrc) + (int64_t)n * a.xld * esz, a.xsrc_f32 != 0,
                          (int64_t)kt * TILE_KBITS + 8 * xc, a.K, a.xzp != nullptr, xzf, hb);
            x_put(t, n, hb);
        }
    };

    // the wave's K range is short (K / KW) and requested MAXT K-tiles at a time: the kernel lives
    // on memory-level parallelism
    // (FUSEX: the source rows of the first four activation rows are requested one round of K-tiles ahead, the first
    // round before the loop, so that a wave with several rounds does not pay the trip to memory once per round:
    // W[4096,11008] x 4 ternary rows 9.5 -> 8.6 us, and 7.2 with sixteen ways a block, see launch_splitk_fusex)
    typedef uint4 XRaw[FUSEX ? MAXT : 1][FUSEX ? 2 : 1];
    XRaw xraw;
    auto x_request = [&](XRaw& to, const int kb) {
#pragma unroll
        for (int q = 0; q < MAXT; q++)
#pragma unroll
            for (int jr = 0; jr < 2; jr++) {
                const int n = xr + 2 * jr;
                const int64_t k0 = (int64_t)(kb + q) * TILE_KBITS + 8 * xc;
                to[FUSEX ? q : 0][FUSEX ? jr : 0] = (kb + q < kt1 && n < (int)a.N && k0 < a.K)
                                  ? *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(a.xsrc) + (int64_t)n * a.xld + k0)
                                  : make_uint4(0u, 0u, 0u, 0u);
            }
    };
    if (FUSEX && xfast) x_request(xraw, kt0);
    // the operand rows that carry activation rows: every other lane's share of a tile built in LDS is zero and is
    // not read (nor cleared) there
    const bool x_real_row = (lane & 31) < (int)a.N || (two && (lane & 31) >= 16 && (lane & 31) - 16 < (int)a.N);
    for (int kb = kt0; kb < kt1 || kb == kt0; kb += MAXT) {
        uint4 xq[MAXT], xq2[PL2 ? MAXT : 1], wq[MAXT];
        XRaw xahead;
        if (kb < kt1) {
#pragma unroll
            for (int q = 0; q < MAXT; q++) {
                if (kb + q >= kt1) break;                       // wave-uniform: no load for a K-tile past the range
                const int64_t off = (int64_t)(kb + q) * TILE_U4;
                if (!FUSEX) xq[q] = xp[off];
                if (PL2) xq2[q] = xp2[off];
                wq[q] = load_stream(wp + off);
            }
            if (FUSEX && xfast && kb + MAXT < kt1) x_request(xahead, kb + MAXT);
            if (FUSEX) {
#pragma unroll
                for (int q = 0; q < MAXT; q++) {
                    if (kb + q >= kt1) break;
                    unsigned char* const t = sX[wave][q];
                    if (xfast) {
#pragma unroll
                        for (int jr = 0; jr < 2; jr++) {
                            const int n = xr + 2 * jr;
                            const uint4 v = xraw[q][jr];
                            if (n >= (int)a.N) continue;
                            if (a.xzp && (int64_t)(kb + q) * TILE_KBITS + 8 * xc < a.K) {
                                uint16_t hb[8] = {(uint16_t)(v.x & 0xffff), (uint16_t)(v.x >> 16), (uint16_t)(v.y & 0xffff), (uint16_t)(v.y >> 16),
                                                  (uint16_t)(v.z & 0xffff), (uint16_t)(v.z >> 16), (uint16_t)(v.w & 0xffff), (uint16_t)(v.w >> 16)};
#pragma unroll
                                for (int e = 0; e < 8; e++) hb[e] = half_bits(__fsub_rn(__half2float(__ushort_as_half(hb[e])), xzf));
                                x_put(t, n, hb);
                            } else {
                                uint32_t sg, nz;
                                bits8(v, sg, nz);
                                x_put_bits(t, n, sg, nz);
                            }
                        }
                        x_rows_slow(t, kb + q, 4);               // rows from the fifth on, if any
                    } else
                        x_rows_slow(t, kb + q, 0);
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int q = 0; q < MAXT; q++)
                    xq[q] = x_real_row ? reinterpret_cast<const uint4*>(sX[wave][min(q, kt1 - 1 - kb)])[lane] : make_uint4(0u, 0u, 0u, 0u);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");      // the next chunk overwrites the area
                __builtin_amdgcn_wave_barrier();
                if (xfast && kb + MAXT < kt1) {
#pragma unroll
                    for (int q = 0; q < MAXT; q++)
#pragma unroll
                        for (int jr = 0; jr < 2; jr++) xraw[FUSEX ? q : 0][FUSEX ? jr : 0] = xahead[FUSEX ? q : 0][FUSEX ? jr : 0];
                }
            }
        }
        if (kb == kt0) {
            // clear the meeting area while the first loads are in flight: every wave gets here at
            // once, so this barrier costs next to nothing
            for (int i = threadIdx.x; i < NP * 16 * 64; i += NT) (&sAcc[0][0][0])[i] = 0;
            if (threadIdx.x < 32) {
                sPa[threadIdx.x] = sPb[0][threadIdx.x] = 0;
                if (PL2) sPb[NP - 1][threadIdx.x] = 0;
            }
            __syncthreads();
        }
        if (kb < kt1) {
#pragma unroll
            for (int q = 0; q < MAXT; q++) {
                if (kb + q >= kt1) break;
                pa += popc4(wq[q]);
                pb += popc4(xq[q]);
                if (PL2) pb2 += popc4(xq2[q]);
#pragma unroll
                for (int s = 0; s < Eng::STEPS; s++) {
                    const typename Eng::Frag bw = Eng::expand_w(wq[q], s);
                    acc = Eng::mma(Eng::expand_x(xq[q], s), bw, acc);
                    if (PL2) acc2 = Eng::mma(Eng::expand_x(xq2[PL2 ? q : 0], s), bw, acc2);
                }
            }
        }
    }

    // ---- meet in LDS: integer adds of the accumulator rows that carry outputs ------------------------
    pa += __shfl_xor(pa, 32);
    pb += __shfl_xor(pb, 32);
    if (PL2) pb2 += __shfl_xor(pb2, 32);
    if (kt0 < kt1) {
        // accumulator registers 4g .. 4g + 3 hold operand rows 8g .. 8g + 7: whole groups past the last real row
        // are skipped (a branch the wave takes as one), rows past it inside a group are added and never read
        const int nrows = (int)a.N - nbase;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            if (8 * (two ? (g & 1) : g) >= nrows) continue;
#pragma unroll
            for (int v = 4 * g; v < 4 * g + 4; v++) {
                atomicAdd(&sAcc[0][v][lane], Eng::to_int(acc, v));
                if (PL2) atomicAdd(&sAcc[NP - 1][v][lane], Eng::to_int(acc2, v));
            }
        }
        if (lane < 32) {
            atomicAdd(&sPa[lane], pa);
            atomicAdd(&sPb[0][lane], pb);
            if (PL2) atomicAdd(&sPb[NP - 1][lane], pb2);
        }
    }
    __syncthreads();

    // ---- rank-one terms and store: one output per thread and step, consecutive threads on one row ----
    const ModeCoef mc = a.mc;
    const int kbits = (int)a.K;
    const int nout = min((int)a.N - nbase, two ? 16 : 32) * 32;
    // one copy of the loop per output kind: the kind's own addressing and parameters only
    auto outputs = [&](auto store) {
        for (int o = threadIdx.x; o < nout; o += NT) {
            const int nl = o >> 5, c = o & 31;
            const int v = 4 * (nl >> 3) + (nl & 3), hh = (nl >> 2) & 1;   // accumulator slot of operand row nl
            const int d = sAcc[0][v][hh * 32 + c];
            const int d2 = PL2 ? sAcc[NP - 1][v][hh * 32 + c] : two ? sAcc[0][v + 8][hh * 32 + c] : 0;
            const int rb2 = PL2 ? sPb[NP - 1][nl] : two ? sPb[0][nl + 16] : 0;
            store(nbase + nl, rt * 32 + c, skinny_value(mc, two || PL2, kbits, sPa[c], sPb[0][nl], rb2, d, d2));
        }
    };
    const int64_t out0 = (int64_t)b * a.strideC;
    const int M = (int)a.M;
    auto elements = [&](auto kind) {
        outputs([&](const int n, const int m, const int val) {
            if (m < M) store_out_as<decltype(kind)::value>(a, out0 + (int64_t)n * M, m, val);
        });
    };
    switch (a.out_kind) {
    case BGEMM_OUT_I32:     // written past the caches: nothing here reads it again (1 to 4 % on 16 to 64 rows)
        outputs([&](const int n, const int m, const int val) {
            if (m < M) __builtin_nontemporal_store(val, reinterpret_cast<int*>(a.out) + out0 + (int64_t)n * M + m);
        });
        break;
    case BGEMM_OUT_F16: elements(std::integral_constant<int, BGEMM_OUT_F16>{}); break;
    case BGEMM_OUT_F32_SCALED: elements(std::integral_constant<int, BGEMM_OUT_F32_SCALED>{}); break;
    case BGEMM_OUT_F16_SCALED: elements(std::integral_constant<int, BGEMM_OUT_F16_SCALED>{}); break;
    default:        // the bits kinds: every lane takes part in the ballot
        outputs([&](const int n, const int m, const int val) {
            store_bits_word(a, b, n, (int64_t)rt * 32, m < M ? next_sign_bit(a, m, val) : 0u);
        });
    }
}

// ---- split-K kernel on the vector ALU: one or two activation vectors ------------------------------
// With one or two rows the matrix cores have nothing to amortise the bit expansion over (13 vector-ALU
// instructions per MFMA, of whose 32 output rows a few are used).  Here a lane keeps the weight words of
// its row and K-half and ANDs them with the same words of each activation vector (NVEC = rows x bit planes,
// TWO = two planes: vector 2n is row n's nonzero plane, 2n + 1 its sign plane; all lanes of a half-wave read
// one address), popcounts accumulate per lane, and the meeting in LDS is one integer per lane and vector
// instead of a 32 x 32 accumulator.  Same grid, K split and epilogue as the matrix-core kernel above.
// FUSEX: the activations arrive unpacked.  A wave walks its K range 512 elements at a time: lane L loads
// elements 8L .. 8L + 7 of every row, turns them into a byte of sign (and nonzero) bits, and the 64 bytes of
// a vector, stored through the wave's own 64 bytes of LDS in big-endian word order, are the sixteen packed
// words of two K-tiles, which every lane reads back as the two 16-byte pieces its K-half needs.
template <int KW, int NVEC, bool TWO, bool FUSEX>
__global__ __launch_bounds__(KW * 64) void gemm_skinny_popc_kernel(const GemmArgs a)
{
    static_assert(!TWO || NVEC % 2 == 0, "two planes come in pairs of vectors");
    constexpr int NT = KW * 64, MAXT = FUSEX ? 2 : 4, ROWS = TWO ? NVEC / 2 : NVEC;
    __shared__ int sD[NVEC][32], sPa[32], sPb[NVEC];
    __shared__ __align__(16) unsigned char sXb[FUSEX ? KW : 1][FUSEX ? NVEC : 1][64];

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5;
    const int rt = blockIdx.x, b = blockIdx.z;
    int kt0, kt1;
    split_range(a.KT, KW, wave, &kt0, &kt1);

    const uint4* const wp = a.W + (int64_t)b * a.strideW + (int64_t)rt * a.KT * TILE_U4 + lane;
    const uint4* xp[NVEC];
#pragma unroll
    for (int j = 0; j < NVEC; j++) {             // a vector past the last row reads the last row again and is not stored
        const int n = min(TWO ? j >> 1 : j, (int)a.N - 1);
        xp[j] = FUSEX ? nullptr : ((TWO && (j & 1)) ? a.X2 : a.X) + (int64_t)b * a.strideX + h * 32 + n;
    }
    float xzf = 0.f;
    if (FUSEX && a.xzp)
        xzf = a.xsrc_f32 ? *reinterpret_cast<const float*>(a.xzp) : __half2float(*reinterpret_cast<const __half*>(a.xzp));
    const bool xfast = FUSEX && !a.xsrc_f32 && !a.xzp && (a.K & 7) == 0 && ((((uintptr_t)a.xsrc) | (uintptr_t)(a.xld * 2)) & 15) == 0;
    int d[NVEC], pb[NVEC], pa = 0;
#pragma unroll
    for (int j = 0; j < NVEC; j++) d[j] = pb[j] = 0;

    // FUSEX, aligned fp16 rows without a zero point: the 16 bytes a lane turns into bits are requested one pair of
    // K-tiles ahead (the first pair before the loop, ahead of the weight loads: loads return in order), so that a wave
    // with several pairs pays the trip to memory once
    uint4 xraw[FUSEX ? ROWS : 1];
    auto x_request = [&](uint4 (&to)[FUSEX ? ROWS : 1], const int kb) {
        const int64_t k0 = (int64_t)kb * TILE_KBITS + 8 * lane;
        const bool mine = kb + h < kt1;                         // the second K-tile of the pair may be another wave's
#pragma unroll
        for (int rr = 0; rr < ROWS; rr++) {
            const int n = min(rr, (int)a.N - 1);
            to[FUSEX ? rr : 0] = (mine && k0 < a.K) ? *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(a.xsrc) + (int64_t)n * a.xld + k0)
                                                    : make_uint4(0u, 0u, 0u, 0u);
        }
    };
    if (FUSEX && xfast) x_request(xraw, kt0);
    for (int kb = kt0; kb < kt1 || kb == kt0; kb += MAXT) {
        uint4 wq[MAXT], xq[MAXT][NVEC], xahead[FUSEX ? ROWS : 1];
        if (kb < kt1) {
#pragma unroll
            for (int q = 0; q < MAXT; q++) {
                if (kb + q >= kt1) break;                       // wave-uniform: no load for a K-tile past the range
                const int64_t off = (int64_t)(kb + q) * TILE_U4;
                if (!FUSEX) {
#pragma unroll
                    for (int j = 0; j < NVEC; j++) xq[q][j] = xp[j][off];
                }
                wq[q] = load_stream(wp + off);
            }
            if (FUSEX && xfast && kb + MAXT < kt1) x_request(xahead, kb + MAXT);
            uint32_t xbyte[NVEC];
            if (FUSEX) {
                const int64_t k0 = (int64_t)kb * TILE_KBITS + 8 * lane;
                const bool mine = kb + h < kt1;
#pragma unroll
                for (int rr = 0; rr < ROWS; rr++) {
                    const int n = min(rr, (int)a.N - 1);
                    uint32_t sg, nz;
                    if (xfast) {
                        bits8(xraw[FUSEX ? rr : 0], sg, nz);
                        if (kb + MAXT < kt1) xraw[FUSEX ? rr : 0] = xahead[FUSEX ? rr : 0];
                    } else {
                        uint16_t hb[8];
                        load8_as_half(reinterpret_cast<const char*>(a.xsrc) + (int64_t)n * a.xld * (a.xsrc_f32 ? 4 : 2), a.xsrc_f32 != 0,
                                      mine ? k0 : a.K, a.K, a.xzp != nullptr, xzf, hb);
                        bits8(hb, sg, nz);
                    }
                    if (TWO) { xbyte[2 * rr] = nz; xbyte[TWO ? 2 * rr + 1 : 0] = sg & nz; }
                    else xbyte[rr] = sg;
                }
#pragma unroll
                for (int j = 0; j < NVEC; j++) sXb[wave][j][lane ^ 3] = (unsigned char)xbyte[j];
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int q = 0; q < MAXT; q++)
#pragma unroll
                    for (int j = 0; j < NVEC; j++) xq[q][j] = *reinterpret_cast<const uint4*>(&sXb[wave][j][32 * q + 16 * h]);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");      // the next pair overwrites the area
                __builtin_amdgcn_wave_barrier();
            }
        }
        if (kb == kt0) {                                        // cleared while the first loads are in flight
            if (threadIdx.x < 32) {
                sPa[threadIdx.x] = 0;
#pragma unroll
                for (int j = 0; j < NVEC; j++) sD[j][threadIdx.x] = 0;
                if (threadIdx.x < NVEC) sPb[threadIdx.x] = 0;
            }
            __syncthreads();
        }
        if (kb < kt1) {
#pragma unroll
            for (int q = 0; q < MAXT; q++) {
                if (kb + q >= kt1) break;
                const uint4 w = wq[q];
                pa += popc4(w);
#pragma unroll
                for (int j = 0; j < NVEC; j++) {
                    const uint4 x = xq[q][j];
                    pb[j] += popc4(x);
                    d[j] += popc4(make_uint4(w.x & x.x, w.y & x.y, w.z & x.z, w.w & x.w));
                }
            }
        }
    }

    // ---- meet in LDS: lane r of either half now adds what its wave found for weight row r -----------
    pa += __shfl_xor(pa, 32);
#pragma unroll
    for (int j = 0; j < NVEC; j++) {
        d[j] += __shfl_xor(d[j], 32);
        pb[j] += __shfl_xor(pb[j], 32);
    }
    if (kt0 < kt1 && lane < 32) {
        atomicAdd(&sPa[lane], pa);
#pragma unroll
        for (int j = 0; j < NVEC; j++) {
            atomicAdd(&sD[j][lane], d[j]);
            if (lane == 0) atomicAdd(&sPb[j], pb[j]);
        }
    }
    __syncthreads();

    // ---- rank-one terms and store: one output per thread ----------------------------------------------
    const ModeCoef mc = a.mc;
    const int kbits = (int)a.K;
    const int nout = (int)a.N * 32;
    auto outputs = [&](auto store) {
        for (int o = threadIdx.x; o < nout; o += NT) {
            const int nl = o >> 5, c = o & 31, j = TWO ? 2 * nl : nl, j2 = TWO ? j + 1 : j;
            store(nl, rt * 32 + c, skinny_value(mc, TWO, kbits, sPa[c], sPb[j], sPb[j2], sD[j][c], sD[j2][c]));
        }
    };
    const int64_t out0 = (int64_t)b * a.strideC;
    const int M = (int)a.M;
    auto elements = [&](auto kind) {
        outputs([&](const int n, const int m, const int val) {
            if (m < M) store_out_as<decltype(kind)::value>(a, out0 + (int64_t)n * M, m, val);
        });
    };
    switch (a.out_kind) {
    case BGEMM_OUT_I32: elements(std::integral_constant<int, BGEMM_OUT_I32>{}); break;
    case BGEMM_OUT_F16: elements(std::integral_constant<int, BGEMM_OUT_F16>{}); break;
    case BGEMM_OUT_F32_SCALED: elements(std::integral_constant<int, BGEMM_OUT_F32_SCALED>{}); break;
    case BGEMM_OUT_F16_SCALED: elements(std::integral_constant<int, BGEMM_OUT_F16_SCALED>{}); break;
    default:        // the bits kinds: every lane takes part in the ballot
        outputs([&](const int n, const int m, const int val) {
            store_bits_word(a, b, n, (int64_t)rt * 32, m < M ? next_sign_bit(a, m, val) : 0u);
        });
    }
}

// ---- split-K kernel, four pieces a block ---------------------------------------------------------
// The same scheme for outputs of a few thousand pieces (a few hundred activation rows against a few
// thousand weight rows): a block owns two weight row tiles and two activation tile rows, a 64 x 64 piece
// of the output, and every wave runs four accumulators over its K range.  Each expanded fragment then
// feeds two matrix-core instructions instead of one and every tile is fetched by half as many blocks:
// the 32 x 32 scheme spends more vector-ALU time on expansion than the matrix cores spend on the
// products.  One bit plane only.  The K range is walked two K-tiles at a time with the next pair in flight.
// TWO: a ternary operand; the block's two activation tiles are the two bit planes of ONE tile row (32 rows), so a
// block is a 32 x 64 piece of the output and the two accumulators of a weight tile combine in the epilogue.
template <typename Eng, int KW, bool TWO = false>
__global__ __launch_bounds__(KW * 64, 2) void gemm_skinny_splitk_quad_kernel(const GemmArgs a)
{
    constexpr int NT = KW * 64, CH = 2;
    __shared__ int sAcc[2][2][16][64];           // [weight tile][activation tile], then the MFMA's [v][lane]
    __shared__ int sPa[2][32], sPb[2][32];

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rt0 = blockIdx.x * 2, nt0 = TWO ? blockIdx.y : blockIdx.y * 2, b = blockIdx.z;
    const bool has_w1 = rt0 + 1 < a.MT, has_x1 = TWO || nt0 + 1 < a.NT;      // the second tiles exist (else: the first again, unused)
    int kt0, kt1;
    split_range(a.KT, KW, wave, &kt0, &kt1);

    const int64_t tile_row = (int64_t)a.KT * TILE_U4;
    const uint4* const wp0 = a.W + (int64_t)b * a.strideW + rt0 * tile_row + lane;
    const uint4* const wp1 = wp0 + (has_w1 ? tile_row : 0);
    const uint4* const xp0 = a.X + (int64_t)b * a.strideX + nt0 * tile_row + lane;
    const uint4* const xp1 = TWO ? a.X2 + (int64_t)b * a.strideX + nt0 * tile_row + lane : xp0 + (has_x1 ? tile_row : 0);

    typename Eng::Acc acc[2][2];
#pragma unroll
    for (int v = 0; v < 16; v++) acc[0][0][v] = acc[0][1][v] = acc[1][0][v] = acc[1][1][v] = 0;
    int pa[2] = {0, 0}, pb[2] = {0, 0};

    uint4 wA[CH][2], xA[CH][2], wB[CH][2], xB[CH][2], wC[CH][2], xC[CH][2];
    // Every fetch issues all of its loads, a K-tile past the range as the range's last one again (a cache hit,
    // never multiplied): with loads under a branch the compiler can no longer count how many are in flight
    // at a use and waits for all of them, the pairs requested ahead included.
    auto fetch = [&](uint4 (&wq)[CH][2], uint4 (&xq)[CH][2], const int kb) {
#pragma unroll
        for (int q = 0; q < CH; q++) {
            const int64_t off = (int64_t)min(kb + q, kt1 - 1) * TILE_U4;
            xq[q][0] = xp0[off]; xq[q][1] = xp1[off];
            wq[q][0] = wp0[off]; wq[q][1] = wp1[off];
        }
    };
    auto consume = [&](const uint4 (&wq)[CH][2], const uint4 (&xq)[CH][2], const int kb) {
#pragma unroll
        for (int q = 0; q < CH; q++) {
            if (kb + q >= kt1) break;
            pa[0] += popc4(wq[q][0]); pa[1] += popc4(wq[q][1]);
            pb[0] += popc4(xq[q][0]); pb[1] += popc4(xq[q][1]);
#pragma unroll
            for (int s = 0; s < Eng::STEPS; s++) {
                const typename Eng::Frag bw0 = Eng::expand_w(wq[q][0], s), bw1 = Eng::expand_w(wq[q][1], s);
                const typename Eng::Frag ax0 = Eng::expand_x(xq[q][0], s), ax1 = Eng::expand_x(xq[q][1], s);
                acc[0][0] = Eng::mma(ax0, bw0, acc[0][0]);
                acc[1][0] = Eng::mma(ax0, bw1, acc[1][0]);
                acc[0][1] = Eng::mma(ax1, bw0, acc[0][1]);
                acc[1][1] = Eng::mma(ax1, bw1, acc[1][1]);
            }
        }
    };
    fetch(wA, xA, kt0);
    // the meeting area is cleared while the first loads are in flight
    for (int i = threadIdx.x; i < 4 * 16 * 64; i += NT) (&sAcc[0][0][0][0])[i] = 0;
    if (threadIdx.x < 64) (&sPa[0][0])[threadIdx.x] = (&sPb[0][0])[threadIdx.x] = 0;
    __syncthreads();
    fetch(wB, xB, kt0 + CH);
    for (int kb = kt0; kb < kt1; kb += 3 * CH) {       // two pairs ahead of the one being multiplied
        fetch(wC, xC, kb + 2 * CH);
        consume(wA, xA, kb);
        fetch(wA, xA, kb + 3 * CH);
        consume(wB, xB, kb + CH);
        fetch(wB, xB, kb + 4 * CH);
        consume(wC, xC, kb + 2 * CH);
    }

    // ---- meet in LDS ------------------------------------------------------------------------------
#pragma unroll
    for (int i = 0; i < 2; i++) {
        pa[i] += __shfl_xor(pa[i], 32);
        pb[i] += __shfl_xor(pb[i], 32);
    }
    if (kt0 < kt1) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int nrows = (int)a.N - (nt0 + (TWO ? 0 : j)) * 32;      // accumulator registers 4g .. 4g + 3 hold operand rows 8g .. 8g + 7
#pragma unroll
            for (int i = 0; i < 2; i++) {
                if (i && !has_w1) continue;
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    if (8 * g >= nrows) continue;
#pragma unroll
                    for (int v = 4 * g; v < 4 * g + 4; v++) atomicAdd(&sAcc[i][j][v][lane], Eng::to_int(acc[i][j], v));
                }
            }
        }
        if (lane < 32) {
            atomicAdd(&sPa[0][lane], pa[0]); atomicAdd(&sPa[1][lane], pa[1]);
            atomicAdd(&sPb[0][lane], pb[0]); atomicAdd(&sPb[1][lane], pb[1]);
        }
    }
    __syncthreads();

    // ---- rank-one terms and store: a wave takes one output row of the piece, 64 consecutive columns ----
    const ModeCoef mc = a.mc;
    const int kbits = (int)a.K;
    // A thread keeps its column (one of the piece's 64, so its weight-row count is read once) and walks the rows
    // KW apart, four at a time with their LDS reads issued together.
    const int nrows_out = min((int)a.N - nt0 * 32, TWO ? 32 : 64);
    auto outputs = [&](auto store) {
        const int mm = threadIdx.x & 63, i = mm >> 5, c = mm & 31;
        const int pa_c = sPa[i][c];
        for (int n0 = threadIdx.x >> 6; n0 < nrows_out; n0 += 4 * KW) {
            int d[4], d2[4], pbv[4], pb2[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int nn = min(n0 + u * KW, nrows_out - 1);
                const int j = TWO ? 0 : nn >> 5, nl = nn & 31;
                const int v = 4 * (nl >> 3) + (nl & 3), hh = (nl >> 2) & 1;   // accumulator slot of operand row nl
                d[u] = sAcc[i][j][v][hh * 32 + c];
                d2[u] = TWO ? sAcc[i][1][v][hh * 32 + c] : 0;
                pbv[u] = sPb[j][nl];
                pb2[u] = TWO ? sPb[1][nl] : 0;
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int nn = n0 + u * KW;
                if (nn < nrows_out)
                    store(nt0 * 32 + nn, rt0 * 32 + mm, i, skinny_value(mc, TWO, kbits, pa_c, pbv[u], pb2[u], d[u], d2[u]));
            }
        }
    };
    const int64_t out0 = (int64_t)b * a.strideC;
    const int M = (int)a.M;
    auto elements = [&](auto kind) {
        outputs([&](const int n, const int m, const int, const int val) {
            if (m < M) store_out_as<decltype(kind)::value>(a, out0 + (int64_t)n * M, m, val);
        });
    };
    switch (a.out_kind) {
    case BGEMM_OUT_I32:
        if (a.nt_store)     // a small output that nothing here reads again: written past the caches
            outputs([&](const int n, const int m, const int, const int val) {
                if (m < M) __builtin_nontemporal_store(val, reinterpret_cast<int*>(a.out) + out0 + (int64_t)n * M + m);
            });
        else
            elements(std::integral_constant<int, BGEMM_OUT_I32>{});
        break;
    case BGEMM_OUT_F16: elements(std::integral_constant<int, BGEMM_OUT_F16>{}); break;
    case BGEMM_OUT_F32_SCALED: elements(std::integral_constant<int, BGEMM_OUT_F32_SCALED>{}); break;
    case BGEMM_OUT_F16_SCALED: elements(std::integral_constant<int, BGEMM_OUT_F16_SCALED>{}); break;
    default:        // the bits kinds: a half-wave holds the 32 columns of one weight row tile, every lane takes part
        outputs([&](const int n, const int m, const int i, const int val) {
            store_bits_word(a, b, n, (int64_t)(rt0 + i) * 32, m < M ? next_sign_bit(a, m, val) : 0u);
        });
    }
}

// Shapes the four-pieces kernel takes (pieces = 32 x 32 outputs, blocks of 2 x 2 pieces, or of one tile row of both planes
// x two weight tiles): at least two tile rows on either side, one round of blocks (192 / 256 to 512: fewer leave compute
// units idle, more are a second round, where the general kernel's tiles re-read less), and a K long enough for the shared
// expansions to outweigh the larger meeting area: one plane up to 1024 pieces from 16 K-tiles, 2048 from 24; two planes
// from 24 K-tiles.  `bench.py --only thresholds` times it against both neighbours.
static bool skinny_quad_shape(int planes, int64_t batch, int64_t M, int64_t N, int64_t KT)
{
    const int64_t MT = row_tiles(M), NT = row_tiles(N);
    // (two planes of up to 16 rows share ONE operand on the one-piece kernel: half the matrix-core work)
    if (MT < 2 || (planes == 2 ? N <= 16 : NT < 2)) return false;
    if (batch > 1 && KT < 24) return false;      // (a batch of small products: operands that were just written, see gemm_skinny_shape)
    if (planes == 2 && two_plane_tile_128(batch, M, N, KT)) return false;      // (the general kernel's pipelined tile is ahead there)
    const int64_t blocks = batch * cdiv(MT, 2) * (planes == 2 ? NT : cdiv(NT, 2));
    if (blocks < (KT >= 40 ? 192 : 256) || blocks > 512) return false;
    if (planes == 2) return KT >= 24;
    return batch * MT * NT <= (KT >= 24 ? 2048 : KT >= 16 ? 1024 : 0);
}

// Shapes the skinny kernels take: one group of activation rows always (32 rows, or 16 rows of two bit planes).  More
// groups where splitting K inside the block buys more than the general kernel's 32 x 128 tiles do (pieces = 32 x 32 outputs):
// up to 1024 pieces from eight K-tiles on (512 for a batch of products: attention-shaped work on operands that were just
// written and sit in the caches, where the general kernel keeps up); on four to seven K-tiles up to 512 pieces of two bit
// planes, or few tile rows of activations.  The bounds are set by weights that come from HBM (a model's layers): there the
// general kernel's serial K loop pays the full memory latency per step.  Beyond, the four-pieces kernel where that pays,
// else the general one.
bool gemm_skinny_shape(int planes, int64_t batch, int64_t M, int64_t N, int64_t K)
{
    if (batch > 65535) return false;             // these kernels walk the batch in the grid's third dimension
    if (N <= (planes == 2 ? 16 : 32)) return true;
    const int64_t NT = row_tiles(N), pieces = batch * row_tiles(M) * NT, KT = k_tiles(K);
    if (skinny_quad_shape(planes, batch, M, N, KT)) return true;
    if (KT >= 8) return pieces <= (batch > 1 ? 512 : 1024);
    if (KT < 4) return false;
    if (planes == 2) return pieces <= 512 || (NT <= 2 && pieces <= 1024);
    if (NT > 2) return NT <= 4 && pieces <= 512;      // (an MLP's first layer at batch 128)
    return pieces <= 1024 && (KT >= 6 || pieces > 384);
}

template <typename Eng>
static int launch_splitk_fusex(const GemmArgs& a, hipStream_t st)
{
    const int64_t blocks = (int64_t)a.MT;
    int kw = 1;
    while (kw < 8 && (kw < a.splitK || blocks * kw < 4096) && kw * 2 <= a.KT) kw *= 2;
    const dim3 g((unsigned)blocks);
    // few row tiles against a long K: sixteen ways, as for packed activations (launch_splitk), and more to gain here,
    // where every K-tile of a wave's range costs it the packing as well
    if (kw == 8 && blocks * 8 < 2048 && a.KT >= 32) {
        hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 16, true>), g, dim3(1024), 0, st, a);
        return check_launch("gemm_skinny");
    }
    if (kw == 1) hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 1, true>), g, dim3(64), 0, st, a);
    else if (kw == 2) hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 2, true>), g, dim3(128), 0, st, a);
    else if (kw == 4) hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 4, true>), g, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 8, true>), g, dim3(512), 0, st, a);
    return check_launch("gemm_skinny");
}

static bool skinny_quad(const GemmArgs& a) { return skinny_quad_shape(a.mc.planes, a.batch, a.M, a.N, a.KT); }

template <typename Eng, bool TWO>
static int launch_splitk_quad(const GemmArgs& a, hipStream_t st)
{
    const int64_t gx = cdiv(a.MT, 2), gy = TWO ? a.NT : cdiv(a.NT, 2);
    if (gy > 65535 || a.batch > 65535)
        return fail(BGEMM_EINVAL, "gemm_skinny: grid of %lld x %lld x %lld blocks", (long long)gx, (long long)gy, (long long)a.batch);
    // K ways per block.  The kernel's registers allow two waves a SIMD, eight a CU: eight ways are one block a CU, which is
    // what up to 256 blocks want; beyond that every block more on a CU is a round more, and four ways (two blocks a CU, each
    // wave on twice the K range, half as many meetings in LDS and store loops per unit of work) are faster; two ways where
    // four blocks a CU are one full round (769 to 1024 blocks).
    const int64_t blocks = gx * gy * a.batch;
    int kw = blocks <= 256 ? 8 : blocks > 768 && blocks <= 1024 ? 2 : 4;
    while (kw > 1 && kw > a.KT) kw /= 2;
    const dim3 g((unsigned)gx, (unsigned)gy, (unsigned)a.batch);
    if (kw == 1) hipLaunchKernelGGL((gemm_skinny_splitk_quad_kernel<Eng, 1, TWO>), g, dim3(64), 0, st, a);
    else if (kw == 2) hipLaunchKernelGGL((gemm_skinny_splitk_quad_kernel<Eng, 2, TWO>), g, dim3(128), 0, st, a);
    else if (kw == 4) hipLaunchKernelGGL((gemm_skinny_splitk_quad_kernel<Eng, 4, TWO>), g, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((gemm_skinny_splitk_quad_kernel<Eng, 8, TWO>), g, dim3(512), 0, st, a);
    return check_launch("gemm_skinny");
}

template <typename Eng>
static int launch_splitk(const GemmArgs& a, hipStream_t st)
{
    const int64_t blocks = (int64_t)a.batch * a.MT;
    const bool pl2 = a.mc.planes == 2 && a.N > 32;      // two operands a block
    const int64_t groups = a.mc.planes == 2 && !pl2 ? cdiv(a.N, 16) : a.NT;      // 16 rows of two planes a block, else 32 rows
    if (groups > 65535 || a.batch > 65535)
        return fail(BGEMM_EINVAL, "gemm_skinny: grid of %lld x %lld x %lld blocks", (long long)a.MT, (long long)groups, (long long)a.batch);
    // K ways per block: at least what the caller asked for, more when the grid alone would leave the
    // chip mostly idle (about four waves per SIMD wanted), never more than there are K-tiles
    int kw = 1;
    while (kw < 8 && (kw < a.splitK || blocks * groups * kw < 4096) && kw * 2 <= a.KT) kw *= 2;
    const dim3 g((unsigned)a.MT, (unsigned)groups, (unsigned)a.batch);
    // few row tiles against a long K (W[4096,11008]: 128 blocks): eight ways leave under two waves a SIMD, each on
    // a long serial range; sixteen ways are faster there
    if (!pl2 && kw == 8 && blocks * groups * 8 < 2048 && a.KT >= 32) {
        hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 16>), g, dim3(1024), 0, st, a);
        return check_launch("gemm_skinny");
    }
    if (pl2) {
        if (kw == 1) hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 1, false, true>), g, dim3(64), 0, st, a);
        else if (kw == 2) hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 2, false, true>), g, dim3(128), 0, st, a);
        else if (kw == 4) hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 4, false, true>), g, dim3(256), 0, st, a);
        else hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 8, false, true>), g, dim3(512), 0, st, a);
    } else if (kw == 1) hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 1>), g, dim3(64), 0, st, a);
    else if (kw == 2) hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 2>), g, dim3(128), 0, st, a);
    else if (kw == 4) hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 4>), g, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((gemm_skinny_splitk_kernel<Eng, 8>), g, dim3(512), 0, st, a);
    return check_launch("gemm_skinny");
}

// Vector-ALU kernel: one matrix of the batch per grid plane, one block per weight row tile.
template <int NVEC, bool TWO, bool FUSEX>
static int launch_popc(const GemmArgs& a, hipStream_t st)
{
    const int64_t blocks = (int64_t)a.batch * a.MT;
    if (a.batch > 65535) return fail(BGEMM_EINVAL, "gemm_skinny: grid of %lld x 1 x %lld blocks", (long long)a.MT, (long long)a.batch);
    int kw = 1;
    while (kw < 8 && (kw < a.splitK || blocks * kw < 4096) && kw * 2 <= a.KT) kw *= 2;
    const dim3 g((unsigned)a.MT, 1u, (unsigned)a.batch);
    if (kw == 8 && blocks * 8 < 2048 && a.KT >= 32) {      // few row tiles, long K: sixteen ways (see launch_splitk)
        hipLaunchKernelGGL((gemm_skinny_popc_kernel<16, NVEC, TWO, FUSEX>), g, dim3(1024), 0, st, a);
        return check_launch("gemm_skinny");
    }
    if (kw == 1) hipLaunchKernelGGL((gemm_skinny_popc_kernel<1, NVEC, TWO, FUSEX>), g, dim3(64), 0, st, a);
    else if (kw == 2) hipLaunchKernelGGL((gemm_skinny_popc_kernel<2, NVEC, TWO, FUSEX>), g, dim3(128), 0, st, a);
    else if (kw == 4) hipLaunchKernelGGL((gemm_skinny_popc_kernel<4, NVEC, TWO, FUSEX>), g, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((gemm_skinny_popc_kernel<8, NVEC, TWO, FUSEX>), g, dim3(512), 0, st, a);
    return check_launch("gemm_skinny");
}

// One or two vectors (rows x bit planes), packed or not.  From three on the matrix-core kernels are faster:
// with unpacked activations every further row costs this kernel about a microsecond (all waves of the grid
// fetch the same few lines of the row at once).
template <bool FUSEX>
static bool launch_popc_for(const GemmArgs& a, hipStream_t st, int* rc)
{
    const int64_t nvec = a.N * a.mc.planes;
    if (nvec > 2) return false;
    if (a.mc.planes == 2) *rc = launch_popc<2, true, FUSEX>(a, st);
    else *rc = nvec == 1 ? launch_popc<1, false, FUSEX>(a, st) : launch_popc<2, false, FUSEX>(a, st);
    return true;
}

template <typename Eng, int RT>
static int launch_stream(const GemmArgs& a, hipStream_t st)
{
    const int groups = (int)cdiv(a.MT, RT);
    const int64_t blocks = cdiv((int64_t)a.batch * groups, 4);
    if (blocks > 0x7fffffffLL) return fail(BGEMM_EINVAL, "gemm_skinny: grid of %lld blocks", (long long)blocks);
    hipLaunchKernelGGL((gemm_skinny_stream_kernel<Eng, RT>), dim3((unsigned)blocks), dim3(256), 0, st, a, groups);
    return check_launch("gemm_skinny");
}

// Shapes whose activations the decode kernel packs itself: one matrix, up to four activation rows (a
// decode step; every wave packs the rows for its own K range, and all waves of a SIMD share its vector
// ALU, so beyond four rows the separate pack launch is faster), few enough weight row tiles that K is
// split inside the block.
bool gemm_skinny_fusex_shape(int planes, int64_t M, int64_t N)
{
    (void)planes;
    return N >= 1 && N <= 4 && row_tiles(M) < 4096;
}

// Which of the kernels above a shape gets (BGEMM_KERNEL_* ids).
int gemm_skinny_kernel_id(const GemmArgs& a, bool fp4)
{
    // a few vectors: the vector ALU does it with less work than the expansion costs (the int8-engine variant
    // keeps the matrix-core kernels for every row count)
    const int64_t row_tiles = (int64_t)a.batch * a.MT, nvec = a.N * a.mc.planes;
    if (a.xsrc) return fp4 && nvec <= 2 ? BGEMM_KERNEL_SKINNY_POPC : BGEMM_KERNEL_SKINNY_SPLITK;
    if (fp4 && row_tiles < 4096 && nvec <= 2) return BGEMM_KERNEL_SKINNY_POPC;
    // Enough row tiles for about four waves on every SIMD: no K split needed (the result does not
    // depend on it).
    if ((a.mc.planes == 2 ? a.N <= 16 : a.NT <= 1) && row_tiles >= 4096) return BGEMM_KERNEL_SKINNY_STREAM;
    return skinny_quad(a) ? BGEMM_KERNEL_SKINNY_QUAD : BGEMM_KERNEL_SKINNY_SPLITK;
}

int launch_gemm_skinny(const GemmArgs& a, hipStream_t st, bool fp4)
{
    int rc;
    const int id = a.force >= 0 ? a.force : gemm_skinny_kernel_id(a, fp4);
    switch (id) {
    case BGEMM_KERNEL_SKINNY_POPC:
        if (a.xsrc ? launch_popc_for<true>(a, st, &rc) : launch_popc_for<false>(a, st, &rc)) return rc;
        return fail(BGEMM_EINVAL, "gemm_skinny: the vector-ALU decode kernel takes one or two vectors");
    case BGEMM_KERNEL_SKINNY_STREAM:
        if (a.xsrc || !(a.mc.planes == 2 ? a.N <= 16 : a.NT <= 1))
            return fail(BGEMM_EINVAL, "gemm_skinny: the streaming kernel takes one group of packed activation rows");
        // two row tiles per wave share one expansion of the activation tiles
        if ((int64_t)a.batch * a.MT >= 8192) return fp4 ? launch_stream<EngF4, 2>(a, st) : launch_stream<EngI8, 2>(a, st);
        return fp4 ? launch_stream<EngF4, 1>(a, st) : launch_stream<EngI8, 1>(a, st);
    case BGEMM_KERNEL_SKINNY_QUAD:
        if (a.xsrc) return fail(BGEMM_EINVAL, "gemm_skinny: the four-pieces kernel takes packed activations");
        if (a.mc.planes == 2) return fp4 ? launch_splitk_quad<EngF4, true>(a, st) : launch_splitk_quad<EngI8, true>(a, st);
        return fp4 ? launch_splitk_quad<EngF4, false>(a, st) : launch_splitk_quad<EngI8, false>(a, st);
    case BGEMM_KERNEL_SKINNY_SPLITK:
        if (a.xsrc) return fp4 ? launch_splitk_fusex<EngF4>(a, st) : launch_splitk_fusex<EngI8>(a, st);
        return fp4 ? launch_splitk<EngF4>(a, st) : launch_splitk<EngI8>(a, st);
    default:
        return fail(BGEMM_EINVAL, "gemm_skinny: no kernel %d", id);
    }
}

}  // namespace bgemm
