// Design (b): AND-dot on the matrix cores.
//
// CDNA4 has no 1-bit MFMA.  Every mode reduces to the AND-dot D[n,m] = popc(a_m & b_n)
// plus rank-one terms in the row popcounts (see ModeCoef), and D is an ordinary GEMM of
// {0,1} matrices.  The operands stay bit-packed all the way into registers: one 16-byte
// load per lane fetches a 32-row x 256-bit tile in exactly the order the 32x32 MFMA wants
// its fragments (lane = half*32 + row), and the MFMA steps of the tile are produced by a
// mask (and for some steps a shift) per register.  Both operands map bits to steps by the same
// rule, so the K permutation it implies cancels.  Waves never exchange data: no LDS, no barriers in the main loop.  Row
// popcounts for the rank-one terms come from the same registers (4 v_bcnt per fragment).
#include "common.h"
#include "mfma_engines.h"
#include <type_traits>

namespace bgemm {

// Block = WGN x WGM waves, each wave owns WN x WM tiles of 32x32 outputs, PL activation planes.
// COUNTED (pipelined tiles only): the operands' row popcounts come with the call (GemmArgs::cntW / cntX) and the main
// loop counts nothing: a sixth of its vector instructions on the 256 x 128 tile.
// TERN (pipelined, fp4 engine, PL = 1): binary weights x ternary activations with signed operands (EngF4::tern_x / tern_w):
// a slot of the activation side is made of both planes' raw words, one MFMA does what takes the AND-dot two, and the
// accumulators hold the output itself: no popcounts, no rank-one terms.
template <typename Eng, int WGN, int WGM, int WN, int WM, int PL, bool PIPE, bool COUNTED = false, bool TERN = false>
// (Second launch bound: from two waves a SIMD on, a wave's register budget is the 256 architected registers, and the
// compiler then keeps the accumulators there instead of in the accumulation registers, which the epilogue could
// only reach through one copy per value.)
__global__ __launch_bounds__(WGN* WGM * 64, (WN * WM * PL <= 8 ? 2 : 1)) void gemm_mfma_kernel(const GemmArgs a, const int tiles_n,
                                                                   const int tiles_m)
{
    // the wave index as a scalar: tile coordinates and operand bases stay on the scalar unit
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wn = wave / WGM, wm = wave % WGM;

    // logical block id: XCD-contiguous (see xcd_contiguous_id)
    const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int per_gemm = tiles_n * tiles_m;
    const int tile_id = bid % per_gemm, b = bid / per_gemm;
    // Tiles are walked in bands along n, so that the blocks in flight share their weight panels: eight tile rows, or two
    // of the 128- and 256-row tiles on fewer than 32 K-tiles (blocks that run together then write 16 KiB and more of every
    // output row they touch instead of 4 KiB, which is what large outputs on a short K wait for; two tile rows of the small
    // tiles are slower), four from 32 K-tiles on, where the operands' reuse in L2 weighs as much.
    const int band = WGN * WN * 32 >= 128 && a.KT < 128 ? (a.KT < 32 ? 2 : 4) : 8;
    int tn_block, tm;
    int sn = a.KT < 16 ? 4 : 2;
    // (the other way round where only that divides, below 32 K-tiles)
    if (a.KT < 32 && (tiles_n % sn != 0 || tiles_m % (8 / sn) != 0)) sn = 8 / sn;
    const int sm = 8 / sn;
    if (WGN * WN * 32 >= 128 && gridDim.x == (unsigned)per_gemm && tiles_n % sn == 0 && tiles_m % sm == 0) {
        // One GEMM on the tall tiles whose tile grid splits evenly: XCD x (the hardware's block id modulo 8) takes a
        // sub-rectangle of the grid, 1/2 x 1/4 of it (1/4 x 1/2 on a short K), and walks that in bands: its L2 then
        // needs a half and a quarter of the operands instead of an eighth of one and all of the other.
        const int x = blockIdx.x % 8, y = blockIdx.x / 8, sub_n = tiles_n / sn, sub_m = tiles_m / sm;
        const int bd = y / (band * sub_m), ib = y % (band * sub_m);
        const int n0 = bd * band, bh = min(band, sub_n - n0);
        tn_block = (x / sm) * sub_n + n0 + ib % bh;
        tm = (x % sm) * sub_m + ib / bh;
    } else {
        const int band_id = tile_id / (band * tiles_m), in_band = tile_id % (band * tiles_m);
        const int band_n0 = band_id * band;
        const int band_h = min(band, tiles_n - band_n0);
        tn_block = band_n0 + in_band % band_h;
        tm = in_band / band_h;
    }

    // K is never split across blocks here: outputs of so few tiles that a K split would pay go to the kernel
    // that splits K among the waves of a block (gemm_skinny_shape)
    const int kt0 = 0, kt1 = a.KT;

    const int mt0 = (tm * WGM + wm) * WM;
    const uint4* Wb = a.W + (int64_t)b * a.strideW;
    const uint4* Xb = a.X + (int64_t)b * a.strideX;
    const uint4* X2b = PL == 2 || TERN ? a.X2 + (int64_t)b * a.strideX : nullptr;
    constexpr int ROW_I = WM * 32 + 8;       // staged row stride in ints (+8 keeps the two lane halves on
                                             // different LDS banks)
    __shared__ __align__(16) int rowp[WGN * WGM * WN * 32];
    __shared__ __align__(16) int stage[WGN * WGM * 32 * ROW_I];
    // The tile's work is a function object of its own: written straight into the kernel body the same code came
    // out with 10 to 25 % more registers (113 against 89 for the 64 x 128 tile: three waves a SIMD instead of four).
  auto do_tile = [&](const int tn) {
    const int nt0 = (tn * WGN + wn) * WN;
    // Pipelined tiles: the two waves of a block that share their activation fragments (same wn) keep them in
    // slots rotated by half against each other, slot i of wave wm holding tile row nt0 + (i ^ xs): each wave then
    // counts the bits of its first WN / 2 slots only, which are different rows for the two, and they swap the
    // counts through LDS before the epilogue (half the activation side's popcounts: 0.25 vector instructions a MFMA).
    static_assert(!PIPE || PL == 2 || (WGM == 2 && WN % 2 == 0), "the popcount split is laid out for two waves along M");
    const int xs = PIPE && PL == 1 && !TERN ? wm * (WN / 2) : 0;      // (two bit planes: every wave counts all its activation slots)
    auto x_tile = [&](const int i) { return nt0 + (i ^ xs); };

    // per-fragment base pointers (row tile clamped so ragged edges re-read a valid tile)
    const uint4* xp[PL][WN];
    const uint4* wp[WM];
#pragma unroll
    for (int i = 0; i < WN; i++) {
        const int64_t rt = min(nt0 + i, a.NT - 1);
        xp[0][i] = Xb + (rt * a.KT) * TILE_U4 + lane;
        if (PL == 2) xp[PL - 1][i] = X2b + (rt * a.KT) * TILE_U4 + lane;
    }
    // Plain fp16 output on a tile with an even number of weight tiles per wave: the two weight fragments of a
    // pair take the even and the odd rows of the pair's 64 weight rows (lane l: rows 2l and 2l + 1), so that a
    // lane ends up with two neighbouring outputs of a row, one 4-byte store of two halves, and a half-wave
    // with a whole 128-byte line (see the epilogue).  The popcounts travel with the lane, nothing else changes.
    const bool pair_cols = !PIPE && WM % 2 == 0 && a.out_kind == BGEMM_OUT_F16 && a.vec_store == 8 &&
                           a.K <= (1 << 20) && a.M < (1 << 28);
#pragma unroll
    for (int j = 0; j < WM; j++) {
        if (pair_cols) {
            const int r = 2 * (lane & 31) + (j & 1);                                  // row within the pair's 64
            const int64_t rt = min(mt0 + (j & ~1) + (r >> 5), a.MT - 1);
            wp[j] = Wb + (rt * a.KT) * TILE_U4 + (lane & 32) + (r & 31);
        } else {
            const int64_t rt = min(mt0 + j, a.MT - 1);
            wp[j] = Wb + (rt * a.KT) * TILE_U4 + lane;
        }
    }

    typename Eng::Acc acc[PL][WN][WM];
    int pa[WM], pb[PL][WN];
    if constexpr (PIPE) {           // (the other loop starts every sum with its first K-tile)
#pragma unroll
        for (int p = 0; p < PL; p++)
#pragma unroll
            for (int i = 0; i < WN; i++)
#pragma unroll
                for (int j = 0; j < WM; j++)
#pragma unroll
                    for (int v = 0; v < 16; v++) acc[p][i][j][v] = 0;
    }

    if constexpr (PIPE) {
        // ---- main loop, software-pipelined by hand -------------------------------------------------
        // One MFMA is followed by the two-register slice of the NEXT step's bit expansion (four VALU
        // ops that fit in the MFMA's shadow); a scheduling barrier after each such group keeps the
        // compiler from clustering them.  Two raw tile buffers ping-pong: while K-tile kt is consumed
        // from A, B holds kt+1, and A is refilled with kt+2 during kt's last step.
        // Two bit planes: the activation slots are the WN tile rows of the first plane, then the same rows of the second
        // (XN = PL * WN slots); a 128 x 128 tile of two planes has the fragments and accumulators of a 256 x 128 tile of one.
        constexpr int XN = PL * WN, NF = XN + WM, ND = NF * 4, NM = XN * WM, STEPS = Eng::STEPS;
        static_assert(ND % NM == 0 && NF <= NM && STEPS % 2 == 0, "tile shape does not pipeline");
        constexpr int DPG = ND / NM;                       // expanded registers produced per MFMA
        // Both operands have one layout and the two expansions are each other's mirror (every product of set bits
        // is 1 either way round), so the side with more fragments a wave gets the cheaper one (five instructions a
        // word against six): the activation side's four fragments on the 256 x 128 tile.
        constexpr bool XS_FIRST = XN <= WM;                // true: activation fragments take the activation-side expansion
        // Every fragment's row of K-tiles is a buffer of its own (a wave-uniform base in scalar registers, KT KiB
        // long), so all loads of a K-tile share ONE per-lane offset, lane * 16 + kt * 1024: no address arithmetic
        // per load, and K-tiles past the range read as zero bits (a buffer load out of range returns 0; zero bits
        // add nothing to the dot or the popcounts), so the loop can always run whole pairs of K-tiles.  Buffer
        // loads also return in order, which lets the compiler wait for the K-tile it needs and no more (flat
        // loads, as a pointer that may point at a zero tile made them, are waited for down to the last one).
        __amdgpu_buffer_rsrc_t rs[NF];
#pragma unroll
        for (int f = 0; f < NF; f++) {
            const int64_t rt = f < XN ? min(x_tile(f % WN), a.NT - 1) : min(mt0 + (f - XN), a.MT - 1);
            const uint4* base = (f < WN ? Xb : f < XN ? X2b : Wb) + rt * a.KT * TILE_U4;
            rs[f] = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4*>(base), 0, a.KT * (TILE_U4 * 16), 0x00020000);
        }
        // Raw K-tiles in flight: two buffers (a K-tile requested one tile ahead of its first use), or three where the
        // registers allow (two tiles ahead: the 256 x 128 tile's 32 MFMAs a K-tile are half a microsecond, less
        // than a trip to a far L2 takes under load; on the 128 x 128 tile likewise: 3072 x 1024 x 8192 17.0 -> 15.3 us,
        // 11008 x 640 x 8192 28.3 -> 25.8)
        constexpr int NBUF = (NM == 8 || NM == 4) && STEPS == 4 && !TERN ? 3 : 2;       // (the int8 engine's eight steps a tile, and the second plane's raw words, leave no registers for it)
        unsigned rawA[NF][4], rawB[NF][4], rawC[NBUF == 3 ? NF : 1][4], buf[2][NF][4];
        constexpr int XN2 = TERN ? XN : 1;                 // TERN: the sign plane's raw words of every activation slot
        unsigned rawA2[XN2][4], rawB2[XN2][4];
        __amdgpu_buffer_rsrc_t rs2[XN2];
        if constexpr (TERN) {
#pragma unroll
            for (int f = 0; f < XN; f++)
                rs2[f] = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4*>(X2b + min((int64_t)x_tile(f), (int64_t)a.NT - 1) * a.KT * TILE_U4), 0,
                                                           a.KT * (TILE_U4 * 16), 0x00020000);
        }
        int pop[NF];
#pragma unroll
        for (int f = 0; f < NF; f++) pop[f] = 0;
        auto load_frag = [&](unsigned (&r)[4], const int f, const int kt) {
            const v4i v = __builtin_amdgcn_raw_buffer_load_b128(rs[f], lane * 16 + kt * (TILE_U4 * 16), 0, 0);
            r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
        };
        auto load_frag2 = [&](unsigned (&r)[4], const int f, const int kt) {
            const v4i v = __builtin_amdgcn_raw_buffer_load_b128(rs2[f], lane * 16 + kt * (TILE_U4 * 16), 0, 0);
            r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
        };
        unsigned tern_c1 = 0;
        if constexpr (TERN) tern_c1 = Eng::tern_const();
        // register d of fragment f at step s, from the raw words of the K-tile it belongs to
        auto expand_reg = [&](const unsigned (&R)[NF][4], const unsigned (&R2)[XN2][4], const int f, const int c, const int s) -> unsigned {
            if constexpr (TERN) return f < XN ? Eng::tern_x(R[f][c], R2[f < XN2 ? f : 0][c], s) : Eng::tern_w(R[f][c], s, tern_c1);
            else return (f < XN) == XS_FIRST ? Eng::expand1_x(R[f][c], s) : Eng::expand1_w(R[f][c], s);
        };
        auto k_tile = [&](unsigned (&A)[NF][4], unsigned (&B)[NF][4], unsigned (&A2)[XN2][4], unsigned (&B2)[XN2][4], const int kt) {
#pragma unroll
            for (int s = 0; s < STEPS; s++) {
                unsigned (&cur)[NF][4] = buf[s & 1];
                unsigned (&nxt)[NF][4] = buf[(s + 1) & 1];
#pragma unroll
                for (int q = 0; q < NM; q++) {
                    const int u = q / WM, j = q % WM;              // activation slot: plane u / WN, tile row u % WN
                    acc[u / WN][u % WN][j] = Eng::mma(Eng::make(cur[u]), Eng::make(cur[XN + j]), acc[u / WN][u % WN][j]);
#pragma unroll
                    for (int d = q * DPG; d < (q + 1) * DPG; d++)      // fragments 0 .. XN-1 are the activation side
                        nxt[d / 4][d % 4] = s + 1 < STEPS ? expand_reg(A, A2, d / 4, d % 4, s + 1) : expand_reg(B, B2, d / 4, d % 4, 0);
                    if (!COUNTED && !TERN && s == 0 && (q < (PL == 1 ? WN / 2 : XN) || (q >= XN && q < NF))) {     // v_bcnt adds into its accumulator: four instructions a fragment, written out
#pragma unroll                                  // because the compiler prefers four counts and two three-way adds
                        for (int c = 0; c < 4; c++) asm("v_bcnt_u32_b32 %0, %1, %0" : "+v"(pop[q]) : "v"(A[q][c]));
                    }
                    if (s == STEPS - 1 && q < NF) load_frag(A[q], q, kt + NBUF);   // A is dead after step STEPS-2
                    if constexpr (TERN) {
                        if (s == STEPS - 1 && q >= NM - XN) load_frag2(A2[q - (NM - XN)], q - (NM - XN), kt + NBUF);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        if (kt0 < kt1) {
#pragma unroll
            for (int f = 0; f < NF; f++) {
                load_frag(rawA[f], f, kt0); load_frag(rawB[f], f, kt0 + 1);
                if constexpr (NBUF == 3) load_frag(rawC[f], f, kt0 + 2);
                if constexpr (TERN) {
                    if (f < XN) { load_frag2(rawA2[f < XN ? f : 0], f, kt0); load_frag2(rawB2[f < XN ? f : 0], f, kt0 + 1); }
                }
            }
#pragma unroll
            for (int f = 0; f < NF; f++)
#pragma unroll
                for (int c = 0; c < 4; c++) buf[0][f][c] = expand_reg(rawA, rawA2, f, c, 0);
            if constexpr (NBUF == 3) {
                // whole rounds of three, then what is left in the same rotation (a K-tile past the range multiplies zeros)
                int kt = kt0;
                for (; kt + 3 <= kt1; kt += 3) {
                    k_tile(rawA, rawB, rawA2, rawB2, kt);
                    k_tile(rawB, rawC, rawA2, rawB2, kt + 1);
                    k_tile(rawC, rawA, rawA2, rawB2, kt + 2);
                }
                if (kt < kt1) {
                    k_tile(rawA, rawB, rawA2, rawB2, kt);
                    if (kt + 1 < kt1) k_tile(rawB, rawC, rawA2, rawB2, kt + 1);
                }
            } else {
                for (int kt = kt0; kt < kt1; kt += 2) {
                    k_tile(rawA, rawB, rawA2, rawB2, kt);
                    k_tile(rawB, rawA, rawB2, rawA2, kt + 1);
                }
            }
        }
        if constexpr (TERN) {          // nothing was counted and nothing is needed
#pragma unroll
            for (int i = 0; i < WN; i++) pb[0][i] = 0;
#pragma unroll
            for (int j = 0; j < WM; j++) pa[j] = 0;
        } else if constexpr (COUNTED) {
            // the lane's row of every fragment, read where the caller keeps the counts (rows past the end: any valid one,
            // their outputs are never stored); halved below by nothing: these are whole rows, not K-halves
            const int64_t cx = a.strideX ? (int64_t)b * a.N : 0, cw = a.strideW ? (int64_t)b * a.M : 0;
#pragma unroll
            for (int i = 0; i < WN; i++) pb[0][i] = a.cntX[cx + min((int64_t)x_tile(i) * 32 + (lane & 31), a.N - 1)];
#pragma unroll
            for (int j = 0; j < WM; j++) pa[j] = a.cntW[cw + min((int64_t)(mt0 + j) * 32 + (lane & 31), a.M - 1)];
        } else if constexpr (PL == 2) {
#pragma unroll
            for (int u = 0; u < XN; u++) pb[u / WN][u % WN] = pop[u] + __shfl_xor(pop[u], 32);
#pragma unroll
            for (int j = 0; j < WM; j++) pa[j] = pop[XN + j] + __shfl_xor(pop[XN + j], 32);
        } else {
            // the two K-halves of a row meet, then the two waves that share these rows exchange what each counted
            __shared__ int xcnt[WGN][WN][32];
#pragma unroll
            for (int i = 0; i < WN / 2; i++) {
                const int n = pop[i] + __shfl_xor(pop[i], 32);
                if (lane < 32) xcnt[wn][i ^ xs][lane] = n;
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < WN; i++) pb[0][i] = xcnt[wn][i ^ xs][lane & 31];
#pragma unroll
            for (int j = 0; j < WM; j++) pa[j] = pop[WN + j] + __shfl_xor(pop[WN + j], 32);
        }
    } else {
    // ---- main loop: raw tiles are prefetched one K-tile ahead ----------------------------------
    // The first K-tile is a copy of its own: its first MFMA step takes a constant zero as the sum to add to (no
    // accumulator is cleared beforehand) and the popcounts start from it; and when all of K is at most 64 bits
    // (attention scores at head size 64) only the first two words of a lane hold any, so two words a fragment
    // are expanded instead of four.  A launch with one K-tile is mostly prologue and epilogue, and every wave
    // pays them: instructions saved here are a fifth of such a launch.
    uint4 xf[PL][WN], wf[WM], xn[PL][WN], wn_[WM];
#pragma unroll
    for (int p = 0; p < PL; p++)
#pragma unroll
        for (int i = 0; i < WN; i++) xn[p][i] = xp[p][i][(int64_t)kt0 * TILE_U4];
#pragma unroll
    for (int j = 0; j < WM; j++) wn_[j] = wp[j][(int64_t)kt0 * TILE_U4];
    const bool two_words = a.K <= 64;
    // (the two expansions mirror each other, so the side with more fragments a wave takes the cheaper one)
    constexpr bool XS_FIRST = WN * PL <= WM;
    auto k_tile = [&](auto first_c, auto two_c, const int kt) {
        constexpr bool FIRST = decltype(first_c)::value, TWO = decltype(two_c)::value;
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
        auto count = [](const uint4 w) { return TWO ? __popc(w.x) + __popc(w.y) : popc4(w); };
#pragma unroll
        for (int j = 0; j < WM; j++) pa[j] = (FIRST ? 0 : pa[j]) + count(wf[j]);
#pragma unroll
        for (int p = 0; p < PL; p++)
#pragma unroll
            for (int i = 0; i < WN; i++) pb[p][i] = (FIRST ? 0 : pb[p][i]) + count(xf[p][i]);
        typename Eng::Acc zero;
#pragma unroll
        for (int v = 0; v < 16; v++) zero[v] = 0;
#pragma unroll
        for (int s = 0; s < Eng::STEPS; s++) {
            typename Eng::Frag bw[WM];
#pragma unroll
            for (int j = 0; j < WM; j++)
                bw[j] = XS_FIRST ? (TWO ? Eng::expand_w2(wf[j], s) : Eng::expand_w(wf[j], s))
                                 : (TWO ? Eng::expand_x2(wf[j], s) : Eng::expand_x(wf[j], s));
#pragma unroll
            for (int p = 0; p < PL; p++)
#pragma unroll
                for (int i = 0; i < WN; i++) {
                    const typename Eng::Frag ax = XS_FIRST ? (TWO ? Eng::expand_x2(xf[p][i], s) : Eng::expand_x(xf[p][i], s))
                                                           : (TWO ? Eng::expand_w2(xf[p][i], s) : Eng::expand_w(xf[p][i], s));
#pragma unroll
                    for (int j = 0; j < WM; j++) acc[p][i][j] = Eng::mma(ax, bw[j], FIRST && s == 0 ? zero : acc[p][i][j]);
                }
        }
    };
    if (two_words) k_tile(std::true_type{}, std::true_type{}, kt0);
    else k_tile(std::true_type{}, std::false_type{}, kt0);
    for (int kt = kt0 + 1; kt < kt1; kt++) k_tile(std::false_type{}, std::false_type{}, kt);

    }

    // ---- epilogue: rank-one terms turn the AND-dot into C -----------------------------------------
    const int bits = (int)a.K;
    if constexpr (!COUNTED && !PIPE) {        // a lane counted its K-half of the row (the pipelined loop has summed already)
#pragma unroll
        for (int j = 0; j < WM; j++) pa[j] += __shfl_xor(pa[j], 32);
#pragma unroll
        for (int p = 0; p < PL; p++)
#pragma unroll
            for (int i = 0; i < WN; i++) pb[p][i] += __shfl_xor(pb[p][i], 32);
    }

    // Per-element terms go through the full-rate unsigned 24-bit multiply (dot_term: the dots stay below
    // 2^24); v_mul_lo_u32 would cost four times as much per element, and is used for the few row and
    // column terms only.
    const ModeCoef mc = a.mc;
    const int col = lane & 31, half = lane >> 5;
    int capa[WM];
#pragma unroll
    for (int j = 0; j < WM; j++) capa[j] = mc.c0 * bits + mc.ca * pa[j];
    // Row terms go through a small LDS table of the wave's own, so that a strip fetches its 16 with four
    // vector reads issued together (sixteen dependent lane permutes cost a strip two thousand cycles).
    // All LDS traffic of the epilogue is private to the wave: LDS executes one wave's accesses in
    // order, so compiler-level wave fences are all the synchronisation it needs, and the waves of a
    // block drift apart freely (one computes a strip while another's stores drain).
    int* const rp = rowp + wave * (WN * 32);
    auto wave_sync = [] {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    if (half == 0) {
#pragma unroll
        for (int i = 0; i < WN; i++) {
            int rowterm = mc.cb * pb[0][i];
            if (PL == 2) rowterm += mc.cb2 * pb[PL - 1][i];
            rp[i * 32 + col] = rowterm;
        }
    }
    wave_sync();
    // C for tile row i
    auto tile_row_vals = [&](const int i, int (&val)[WM][16]) {
        int4 r4[4];
#pragma unroll
        for (int g = 0; g < 4; g++) r4[g] = *reinterpret_cast<const int4*>(rp + i * 32 + 8 * g + 4 * half);
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int4 q = r4[v >> 2];
            const int rowterm = (v & 3) == 0 ? q.x : (v & 3) == 1 ? q.y : (v & 3) == 2 ? q.z : q.w;
#pragma unroll
            for (int j = 0; j < WM; j++) {
                if constexpr (TERN) val[j][v] = Eng::to_int(acc[0][i][j], v);
                else
                val[j][v] = capa[j] + rowterm + (PL == 2 ? dot_terms2(mc, Eng::to_int(acc[0][i][j], v), Eng::to_int(acc[PL - 1][i][j], v))
                                                          : dot_term(mc, Eng::to_int(acc[0][i][j], v)));
            }
        }
    };

    // ---- int32 output: straight from the accumulators ---------------------------------------------
    // In the accumulator layout of the 32 x 32 MFMA a lane holds one output column (weight row m) of sixteen
    // output rows, and the lanes of a half-wave hold 32 consecutive columns: one 4-byte store instruction
    // writes two whole 128-byte lines, one per half-wave, and needs no transposition.  The address is a
    // wave-uniform base (strip row, weight tile: scalar registers) plus one fixed 32-bit offset per lane.
    if (a.out_kind == BGEMM_OUT_I32 && a.M < (1 << 28)) {
        const int64_t row_b = a.M * 4;
        char* const out_b = reinterpret_cast<char*>(a.out) + (int64_t)b * a.strideC * 4;
        const uint32_t voff = (uint32_t)(half * 4 * row_b + col * 4);
        auto rows_out = [&](auto past_cache) {
#pragma unroll
            for (int i = 0; i < WN; i++) {
                const int64_t nrow0 = (int64_t)x_tile(i) * 32;
                if (nrow0 >= a.N) continue;                       // the whole strip lies past the last row
                int val[WM][16];
                tile_row_vals(i, val);
                auto put = [&](int* const to, const int v) {
                    if constexpr (decltype(past_cache)::value) __builtin_nontemporal_store(v, to);
                    else *to = v;
                };
                char* const ub = out_b + nrow0 * row_b + (int64_t)mt0 * 128;      // uniform: scalar registers
                if (nrow0 + 32 <= a.N && (int64_t)(mt0 + WM) * 32 <= a.M) {
                    // the strip exists as a whole: no test per store, one scalar base per row, the weight tile in
                    // the instruction's immediate offset (a lone wave on its SIMD issues an instruction every
                    // 2.3 ns at best, so the epilogue costs what it counts in instructions, scalar ones included)
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        int* const row = reinterpret_cast<int*>(ub + (8 * (v >> 2) + (v & 3)) * row_b + voff);
#pragma unroll
                        for (int j = 0; j < WM; j++) put(row + j * 32, val[j][v]);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < WM; j++) {
                        if ((int64_t)(mt0 + j) * 32 + col >= a.M) continue;
#pragma unroll
                        for (int v = 0; v < 16; v++) {
                            const int r = 8 * (v >> 2) + (v & 3);      // the lane's row is r + 4 * half
                            if (nrow0 + r + 4 * half < a.N) put(reinterpret_cast<int*>(ub + r * row_b + voff) + j * 32, val[j][v]);
                        }
                    }
                }
            }
        };
        // Past the caches: outputs of up to 32 MiB (a.nt_store), and larger ones on 8 to 31 K-tiles, where the operands a
        // block's neighbours still need would otherwise leave the L2 for the output lines (weights rotating through HBM:
        // 16384 x 8192 x 4096 198.1 -> 184.4 us, 8192^2 x 2048 63.5 -> 61.0, 11008 x 2048 x 4096 40.8 -> 39.5; on four K-tiles
        // ordinary stores are 7 % ahead, 8192^2 x 1024 49.0 against 52.4, from 32 on there is no difference)
        if (a.nt_store || (a.KT >= 8 && a.KT < 32)) rows_out(std::true_type{});
        else rows_out(std::false_type{});
        return;
    }

    // ---- plain fp16 from paired columns: straight from the accumulators ---------------------------
    // With the weight rows dealt as above, a lane's accumulators 2p and 2p + 1 are the outputs (n, m) and
    // (n, m + 1): rounded together (v_cvt_pk_f16_f32) they are one 4-byte store, 32 lanes one 128-byte line, as in
    // the int32 case.  The arithmetic runs in fp32, where it is exact: every term is an integer below 2^24 for
    // K <= 2^20, so the rounding to fp16 starts from the same number as on the integer path.
    if constexpr (!PIPE && WM % 2 == 0) {
        if (pair_cols) {
            typedef _Float16 h2v __attribute__((ext_vector_type(2)));
            typedef float f2v __attribute__((ext_vector_type(2)));
            const float cdf = (float)mc.cd, cd2f = (float)mc.cd2;
            float capaf[WM];
#pragma unroll
            for (int j = 0; j < WM; j++) capaf[j] = (float)capa[j];
            const int64_t row_b = a.M * 2;
            char* const out_b = reinterpret_cast<char*>(a.out) + (int64_t)b * a.strideC * 2;
            const uint32_t voff = (uint32_t)(half * 4 * row_b + col * 4);
#pragma unroll
            for (int i = 0; i < WN; i++) {
                const int64_t nrow0 = (int64_t)x_tile(i) * 32;
                if (nrow0 >= a.N) continue;                       // the whole strip lies past the last row
                int4 r4[4];
#pragma unroll
                for (int g = 0; g < 4; g++) r4[g] = *reinterpret_cast<const int4*>(rp + i * 32 + 8 * g + 4 * half);
                char* const ub = out_b + nrow0 * row_b + (int64_t)mt0 * 64;       // uniform: scalar registers
                const bool whole = nrow0 + 32 <= a.N && (int64_t)(mt0 + WM) * 32 <= a.M;
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int4 q = r4[v >> 2];
                    const float rowterm = (float)((v & 3) == 0 ? q.x : (v & 3) == 1 ? q.y : (v & 3) == 2 ? q.z : q.w);
                    const int r = 8 * (v >> 2) + (v & 3);         // the lane's row is r + 4 * half
                    unsigned* const row = reinterpret_cast<unsigned*>(ub + r * row_b + voff);
#pragma unroll
                    for (int pr = 0; pr < WM / 2; pr++) {
                        f2v f;
#pragma unroll
                        for (int e = 0; e < 2; e++) {
                            const int j = 2 * pr + e;
                            float t = fmaf(cdf, Eng::to_float(acc[0][i][j], v), capaf[j] + rowterm);
                            if (PL == 2) t = fmaf(cd2f, Eng::to_float(acc[PL - 1][i][j], v), t);
                            f[e] = t;
                        }
                        const unsigned w = __builtin_bit_cast(unsigned, __builtin_convertvector(f, h2v));
                        if (whole || ((int64_t)(mt0 + 2 * pr) * 32 + 2 * col < a.M && nrow0 + r + 4 * half < a.N))
                            __builtin_nontemporal_store(w, row + pr * 32);
                    }
                }
            }
            return;
        }
    }

    // ---- store ------------------------------------------------------------------------------
    // Every 32-row strip of the wave's tile is transposed through the wave's own LDS area, so that
    // lanes own consecutive outputs of one row.  Only the plain int32 case with 16-byte-aligned rows
    // is unrolled; the conversions of the other output kinds sit in rolled loops after the staging,
    // which keeps them out of the fully unrolled part of the kernel.
    const int esz_shift = out_elem_shift(a.out_kind);
    const int64_t out_off = (int64_t)b * a.strideC;
    char* const out_base = reinterpret_cast<char*>(a.out) + (out_off << esz_shift);
    const int64_t row_bytes = a.M << esz_shift;
    int* const st = stage + wave * (32 * ROW_I);
    // Stores past the caches (non-temporal) where timing favours them: always for the 2-byte kinds, for the
    // 4-byte kinds on outputs of up to 32 MiB (a.nt_store) and on larger ones on 8 to 31 K-tiles (see the int32 path above;
    // fp32 scaled: 16384 x 8192 x 4096 252.2 -> 238.3 us, 4096^3 36.0 -> 34.6); else ordinary stores are faster.
    // (The non-temporal store is written as an instruction: as a builtin next to an ordinary store of the same
    // value the optimiser merges the two into one ordinary store.  The s_nop belongs to it: a store of more
    // than 64 bits must not be followed at once by a vector-ALU write to its data registers, and the compiler,
    // which pads that hazard for its own stores, does not look inside an asm statement.)
    auto store16 = [&](char* const to, const int4 v, const bool past_cache) {
        if (past_cache) {
            const v4i x = {v.x, v.y, v.z, v.w};
            asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" : : "v"(to), "v"(x) : "memory");
        } else
            *reinterpret_cast<int4*>(to) = v;
    };
    // Plain fp16 with rows a multiple of eight long: the integers are rounded once, staged as halves, and a
    // lane reads back the eight it stores with one 16-byte LDS read (no conversion behind the staging).
    if (a.out_kind == BGEMM_OUT_F16 && a.vec_store == 8) {
        constexpr int ROW_H = WM * 32 + 8;       // staged row stride in halves (+8: rows four apart, the two
                                                 // lane halves, fall on different LDS banks)
        constexpr int C8 = WM * 4, RSTEP = 64 / C8;              // lanes per staged row, rows per store instruction
        __half* const sh = reinterpret_cast<__half*>(st);
        const int c8 = lane % C8, row0 = lane / C8;
        const int64_t m = (int64_t)mt0 * 32 + c8 * 8;
#pragma unroll
        for (int i = 0; i < WN; i++) {
            const int64_t nrow0 = (int64_t)x_tile(i) * 32;
            if (nrow0 >= a.N) continue;                           // the whole strip lies past the last row
            int val[WM][16];
            tile_row_vals(i, val);
#pragma unroll
            for (int v = 0; v < 16; v++)
#pragma unroll
                for (int j = 0; j < WM; j++)
                    sh[(8 * (v >> 2) + 4 * half + (v & 3)) * ROW_H + j * 32 + col] = __float2half_rn((float)val[j][v]);
            wave_sync();
            if (m < a.M) {
                char* dst = out_base + (nrow0 + row0) * row_bytes + (m << 1);
                const __half* sp = sh + row0 * ROW_H + c8 * 8;
#pragma unroll
                for (int row = row0; row < 32; row += RSTEP, sp += RSTEP * ROW_H, dst += RSTEP * row_bytes)
                    if (nrow0 + row < a.N) store16(dst, *reinterpret_cast<const int4*>(sp), true);
            }
            wave_sync();                                 // the next strip overwrites the staging area
        }
        return;
    }
    // fp16 scaled, eight elements a lane: the lane's eight columns are the same for every strip, so their parameters are
    // fetched once, before the strips (inside the strip loop the stores between them keep the compiler from reusing them)
    ColParams cp8[8];
    float saf8 = 0.f;
    if (a.vec_store == 8 && a.out_kind == BGEMM_OUT_F16_SCALED) {
        saf8 = ep_scalar(a.out_kind, a.ep_sa);
#pragma unroll
        for (int e = 0; e < 8; e++) cp8[e] = col_params(a, (int64_t)mt0 * 32 + (lane % (WM * 4)) * 8 + e);
    }
    // (the same for the scaled kinds stored four elements a lane: fp32, and fp16 rows that are no multiple of eight long)
    ColParams cp4[4];
    if (a.vec_store && a.vec_store != 8 && (a.out_kind == BGEMM_OUT_F32_SCALED || a.out_kind == BGEMM_OUT_F16_SCALED)) {
        saf8 = ep_scalar(a.out_kind, a.ep_sa);
#pragma unroll
        for (int e = 0; e < 4; e++) cp4[e] = col_params(a, (int64_t)mt0 * 32 + (lane % (WM * 8)) * 4 + e);
    }
#pragma unroll
    for (int i = 0; i < WN; i++) {
        int val[WM][16];
        tile_row_vals(i, val);
#pragma unroll
        for (int v = 0; v < 16; v++)
#pragma unroll
            for (int j = 0; j < WM; j++) st[(8 * (v >> 2) + 4 * half + (v & 3)) * ROW_I + j * 32 + col] = val[j][v];
        wave_sync();
        const int64_t nrow0 = (int64_t)x_tile(i) * 32, mcol0 = (int64_t)mt0 * 32;
        constexpr int C4 = WM * 8;               // int4 per staged row
        constexpr int NP = 32 * C4 / 64;
        if (a.vec_store && a.out_kind == BGEMM_OUT_I32) {
            // 16-byte stores: one instruction covers 64 * 4 consecutive elements of the strip.  Eight
            // LDS reads are issued together, then their stores; the address advances by whole rows.
            constexpr int RSTEP = 64 / C4, CHUNK = NP < 8 ? NP : 8;
            const int c4 = lane % C4, row0 = lane / C4;
            const int* sp = st + row0 * ROW_I + c4 * 4;
            const int64_t m = mcol0 + c4 * 4, dstep = RSTEP * row_bytes;
            char* dst = out_base + (nrow0 + row0) * row_bytes + (m << 2);
            if (m < a.M) {
                if (nrow0 + 32 <= a.N) {             // uniform: the whole strip exists, nothing to mask
#pragma unroll
                    for (int p0 = 0; p0 < NP; p0 += CHUNK) {
                        int4 q[CHUNK];
#pragma unroll
                        for (int p = 0; p < CHUNK; p++) q[p] = *reinterpret_cast<const int4*>(sp + (p0 + p) * RSTEP * ROW_I);
                        if (a.nt_store || (a.KT >= 8 && a.KT < 32)) {
#pragma unroll
                            for (int p = 0; p < CHUNK; p++, dst += dstep) store16(dst, q[p], true);
                        } else {
#pragma unroll
                            for (int p = 0; p < CHUNK; p++, dst += dstep) store16(dst, q[p], false);
                        }
                    }
                } else {
                    for (int row = row0; nrow0 + row < a.N; row += RSTEP, sp += RSTEP * ROW_I, dst += dstep)
                        store16(dst, *reinterpret_cast<const int4*>(sp), (a.nt_store != 0 || (a.KT >= 8 && a.KT < 32)));
                }
            }
        } else if (a.vec_store == 8) {
            // fp16 kinds, rows a multiple of eight long: eight elements and one 16-byte store per lane
            constexpr int C8 = WM * 4, RSTEP = 64 / C8;          // lanes per staged row, rows per step
            const int c8 = lane % C8, row0 = lane / C8;
            const int64_t m = mcol0 + c8 * 8;
            const int* sp = st + row0 * ROW_I + c8 * 8;
            char* dst = out_base + (nrow0 + row0) * row_bytes + (m << 1);
            const int64_t dstep = RSTEP * row_bytes;
            const bool scaled = a.out_kind == BGEMM_OUT_F16_SCALED;
            const ColParams (&cp)[8] = cp8;      // this lane's eight columns, the same for every row of every strip
            const float saf = saf8;
            const bool has_bias = a.ep_bias != nullptr;
            // The scaled kind's two multiplications and its addition run on fp16 pairs.  scaled_f16 spells every step out as
            // fp32 arithmetic on fp16 values rounded back to fp16 (what torch's kernels do); with 24 >= 2 * 11 + 2 significand
            // bits in between, that double rounding gives the correctly rounded fp16 result for a product or a sum of two fp16
            // values, which is what the fp16 instructions return.
            __half2 swh[4], biash[4];
            const __half2 sah = __float2half2_rn(saf);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                swh[e] = scaled ? __floats2half2_rn(cp[2 * e].sw, cp[2 * e + 1].sw) : sah;
                biash[e] = scaled && has_bias ? __floats2half2_rn(cp[2 * e].bias, cp[2 * e + 1].bias) : sah;
            }
            auto put8 = [&](const int4 q0, const int4 q1, char* const to, const bool sc) {
#pragma clang fp contract(off)
                const int q[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
                union { __half h[8]; __half2 h2[4]; uint4 u; } pk;
#pragma unroll
                for (int e = 0; e < 8; e++) pk.h[e] = __float2half_rn((float)q[e]);
                if (sc) {
#pragma unroll
                    for (int e = 0; e < 4; e++) pk.h2[e] = __hmul2(__hmul2(pk.h2[e], swh[e]), sah);
                    if (has_bias) {
#pragma unroll
                        for (int e = 0; e < 4; e++) pk.h2[e] = __hadd2(pk.h2[e], biash[e]);
                    }
                }
                store16(to, make_int4((int)pk.u.x, (int)pk.u.y, (int)pk.u.z, (int)pk.u.w), true);
            };
            if (m < a.M) {
                if (nrow0 + 32 <= a.N) {             // uniform: whole strip: reads issued in pairs of rows
#pragma unroll
                    for (int r = 0; r < 32 / RSTEP; r += 2, dst += 2 * dstep) {
                        const int* s0 = sp + r * RSTEP * ROW_I, * s1 = s0 + RSTEP * ROW_I;
                        const int4 a0 = *reinterpret_cast<const int4*>(s0), a1 = *reinterpret_cast<const int4*>(s0 + 4);
                        const int4 b0 = *reinterpret_cast<const int4*>(s1), b1 = *reinterpret_cast<const int4*>(s1 + 4);
                        put8(a0, a1, dst, scaled);
                        put8(b0, b1, dst + dstep, scaled);
                    }
                } else {
#pragma unroll 2
                    for (int row = row0; row < 32 && nrow0 + row < a.N; row += RSTEP, sp += RSTEP * ROW_I, dst += dstep)
                        put8(*reinterpret_cast<const int4*>(sp), *reinterpret_cast<const int4*>(sp + 4), dst, scaled);
                }
            }
        } else if (a.vec_store) {
            // four elements per lane; the address advances by whole rows from step to step
            constexpr int RSTEP = 64 / C4;
            const int c4 = lane % C4, row0 = lane / C4;
            const int64_t m = mcol0 + c4 * 4;
            const int* sp = st + row0 * ROW_I + c4 * 4;
            char* dst = out_base + (nrow0 + row0) * row_bytes + (m << esz_shift);
            const int64_t dstep = RSTEP * row_bytes;
            const bool has_bias = a.ep_bias != nullptr;
            const ColParams (&cp)[4] = cp4;
            const float saf = saf8;
            if (m < a.M) {
#pragma unroll 2
                for (int row = row0; row < 32 && nrow0 + row < a.N; row += RSTEP, sp += RSTEP * ROW_I, dst += dstep) {
                    const int4 q = *reinterpret_cast<const int4*>(sp);
                    union { __half h[4]; uint2 u; } pk;
                    switch (a.out_kind) {
                    case BGEMM_OUT_I32:
                        store16(dst, q, (a.nt_store != 0 || (a.KT >= 8 && a.KT < 32)));
                        break;
                    case BGEMM_OUT_F16:
                        pk.h[0] = __float2half_rn((float)q.x); pk.h[1] = __float2half_rn((float)q.y);
                        pk.h[2] = __float2half_rn((float)q.z); pk.h[3] = __float2half_rn((float)q.w);
                        *reinterpret_cast<uint2*>(dst) = pk.u;
                        break;
                    case BGEMM_OUT_F32_SCALED:
                        store16(dst, make_int4(__float_as_int(scaled_f32(q.x, cp[0], saf, has_bias)), __float_as_int(scaled_f32(q.y, cp[1], saf, has_bias)),
                                               __float_as_int(scaled_f32(q.z, cp[2], saf, has_bias)), __float_as_int(scaled_f32(q.w, cp[3], saf, has_bias))),
                                (a.nt_store != 0 || (a.KT >= 8 && a.KT < 32)));
                        break;
                    default:
                        pk.h[0] = scaled_f16(q.x, cp[0], saf, has_bias); pk.h[1] = scaled_f16(q.y, cp[1], saf, has_bias);
                        pk.h[2] = scaled_f16(q.z, cp[2], saf, has_bias); pk.h[3] = scaled_f16(q.w, cp[3], saf, has_bias);
                        *reinterpret_cast<uint2*>(dst) = pk.u;
                        break;
                    }
                }
            }
        } else {
            // ragged or unaligned rows, and the bits kinds: one element per lane and step.  A lane meets one
            // column (two where the strip is 128 wide), whose parameters it fetches once.
            constexpr int NC = WM == 4 ? 2 : 1;
            const bool bits = bits_kind(a.out_kind);
            const bool has_bias = a.ep_bias != nullptr;
            ColParams cp[NC];
            float saf = 0.f, zpf = 0.f;
            if (bits) {
                saf = ep_scalar(a.out_kind, a.ep_sa);
                if (a.ep_zp) zpf = ep_scalar(a.out_kind, a.ep_zp);
#pragma unroll
                for (int k = 0; k < NC; k++) cp[k] = col_params(a, mcol0 + (lane + 64 * k) % (32 * WM));
            }
            if (bits) {
                // half-waves hold 32 consecutive columns of one row: a ballot makes the output word.  The strip
                // starts on a row tile of the output operand, so its words sit at fixed steps from one base.
                uint32_t* const obase = reinterpret_cast<uint32_t*>(a.out) + (int64_t)b * a.strideC;
                const int64_t okt = k_tiles(a.M);
                int64_t wbase[NC];
                bool col_ok[NC], word_ok[NC];
#pragma unroll
                for (int k = 0; k < NC; k++) {
                    const int c = (lane + 64 * k) % (32 * WM);
                    col_ok[k] = mcol0 + c < a.M;
                    word_ok[k] = mcol0 + (c & ~31) < a.M;
                    wbase[k] = tiled_word_offset(nrow0, (mcol0 + c) >> 5, okt);
                }
#pragma unroll 4
                for (int p = 0; p < 16 * WM; p++) {
                    const int idx = p * 64 + lane, row = idx / (32 * WM), c = idx % (32 * WM), k = NC == 2 ? (p & 1) : 0;
                    const bool row_ok = nrow0 + row < a.N;
                    const unsigned bit = next_sign_bit(a.out_kind, st[row * ROW_I + c], cp[k], saf, has_bias, zpf);
                    const unsigned long long bal = __ballot(bit != 0 && row_ok && col_ok[k]);
                    const unsigned w = __brev((unsigned)(lane < 32 ? bal : bal >> 32));
                    if ((lane & 31) == 0 && row_ok && word_ok[k]) obase[wbase[k] + row * 4] = w;
                }
            } else {
#pragma unroll 4
                for (int p = 0; p < 16 * WM; p++) {
                    const int idx = p * 64 + lane, row = idx / (32 * WM), c = idx % (32 * WM);
                    const int64_t n = nrow0 + row, m = mcol0 + c;
                    if (n < a.N && m < a.M) store_out(a, out_off + n * a.M, m, st[row * ROW_I + c]);
                }
            }
        }
        wave_sync();                                 // the next strip overwrites the staging area
    }
  };
    do_tile(tn_block);
}

// ---- host side ---------------------------------------------------------------------------
struct MfmaCfg { int id, bn, bm; };

// Tile choice.  Every rule below separates two tiles whose timings cross at that point; `bench.py --only thresholds`
// re-times every tile on shapes either side of each rule and reports how far this function's choice is from the fastest
// kernel (the default run carries a summary).  The terms: `blocks` of a tile shape, `filled` = the share of a tiling's
// matrix-core work that lands on real outputs, K-tiles of 256 bits, 256 compute units holding one 256 x 256 block, two
// 256 x 128 blocks or three 128 x 128 blocks each.
//   * 256 x 256: one wave a SIMD and the cheapest loop per MFMA, but its epilogue is exposed: two rounds of blocks and a
//     very long K (128 K-tiles).
//   * 256 x 128: two resident blocks a unit, one storing while the other multiplies: from two blocks a unit; on 16 K-tiles
//     or more already from half a block a unit, since its loop is so much cheaper per MFMA than the smaller tiles', except
//     where a few units would run two blocks while the rest run one (257 to 384 blocks), or a last round would leave most
//     of the GPU idle.
//   * 128 x 128: runs the same hand-pipelined loop from 8 K-tiles on; from 192 blocks (144 on 16 K-tiles or more).
//   * 32 x 256: a short K into 2-byte outputs or into int32 rows a power of two long (many small blocks drift apart and
//     spread their stores over the memory channels), and two bit planes (one weight expansion feeds both planes).
//   * 64 x 128, 32 x 128: whatever is left, so that every unit gets a block; 64-column tiles for outputs of at most 64
//     columns.
//   * 128 x 256 signed (a ternary operand on the fp4 engine): half the matrix-core work of the two-plane tiles; from more
//     than half a block a unit on (ahead of every two-plane kernel from there, level with the best of them at 128 blocks),
//     two K-tiles or more (its loop runs whole pairs of them).
static MfmaCfg pick_cfg(int64_t batch, int64_t M, int64_t N, int64_t KT, int planes, int out_shift, bool fp4)
{
    auto blocks = [&](int bn, int bm) { return batch * cdiv(N, bn) * cdiv(M, bm); };
    auto filled = [&](int bn, int bm) { return (double)(N * M) / (double)(cdiv(N, bn) * bn * cdiv(M, bm) * bm); };
    auto round_fill = [](int64_t b, int64_t places) { return (double)b / (double)(cdiv(b, places) * places); };
    const int64_t out_elems = batch * N * M, b32 = blocks(32, 256), b21 = blocks(256, 128), b11 = blocks(128, 128);
    if (M <= 64) return blocks(128, 64) >= 1024 ? MfmaCfg{BGEMM_KERNEL_MFMA_128x64, 128, 64} : MfmaCfg{BGEMM_KERNEL_MFMA_64x64, 64, 64};
    // one K-tile: all store path.  2-byte outputs, or more int32 output than the memory-side cache holds
    if (KT < 2 && M >= 512 && b32 >= 512 && (out_shift == 1 || out_elems > (64 << 20))) return {BGEMM_KERNEL_MFMA_32x256, 32, 256};
    // up to six K-tiles into int32 rows of a power of two in bytes, up to 64 MiB of output
    if (batch == 1 && planes == 1 && out_shift == 2 && KT <= 6 && M >= 1024 && M <= 16384 && (M & (M - 1)) == 0 &&
        N * M <= (16 << 20) && b32 >= 1024)
        return {BGEMM_KERNEL_MFMA_32x256, 32, 256};
    if (planes == 1 && blocks(256, 256) >= 512 && KT >= 128 && filled(256, 256) >= 0.8) return {BGEMM_KERNEL_MFMA_256x256, 256, 256};
    // 256 x 128 unless its last round would leave most of the GPU idle where 128 x 128 fills its own
    const bool last_round_idle = KT >= 8 && (KT <= 16 || b21 <= 600) && b21 > 256 &&
                                 round_fill(b11, 768) >= round_fill(b21, 512) + 0.15 && filled(128, 128) >= 0.6;
    const bool few_blocks_ok = KT >= 16 && b21 >= 132 && (b21 < 192 || KT >= 24) && !(b21 > 256 && b21 <= 384);
    // (on 8 to 11 K-tiles the smaller tile's extra blocks hide more of the stores than its dearer loop costs)
    const bool k_long_enough = KT >= 12 || (out_shift == 2 && KT >= 4 && out_elems >= (64 << 20)) || b11 < 512;
    if (planes == 1 && !last_round_idle && (b21 >= 512 || few_blocks_ok) && k_long_enough && filled(256, 128) >= 0.75)
        return {BGEMM_KERNEL_MFMA_256x128, 256, 128};
    // 128 x 128: two rounds' worth of blocks, or (one plane, pipelined loop) from 192 / 144 blocks, not where some units
    // would run two blocks and the rest one on a short K
    const bool pipelined_ok = planes == 1 && KT >= 8 && b11 >= (KT >= 16 ? 144 : 192) &&
                              (b11 >= 192 || KT >= 24 || filled(128, 128) >= 0.85) && !(KT < 12 && b11 > 256 && b11 < 416);
    if (planes == 2 && fp4 && KT >= 2 && blocks(128, 256) > 128 && filled(128, 256) >= 0.7) return {BGEMM_KERNEL_MFMA_128x256T, 128, 256};
    if ((b11 >= 512 || pipelined_ok) && filled(128, 128) >= 0.6) return {BGEMM_KERNEL_MFMA_128x128, 128, 128};
    if (planes == 2 && two_plane_tile_128(batch, M, N, KT)) return {BGEMM_KERNEL_MFMA_128x128, 128, 128};
    if (planes == 2 && b32 >= (KT >= 8 ? 96 : 160)) return {BGEMM_KERNEL_MFMA_32x256, 32, 256};
    if (blocks(64, 128) >= 512 && filled(64, 128) >= 0.6) return {BGEMM_KERNEL_MFMA_64x128, 64, 128};
    return {BGEMM_KERNEL_MFMA_32x128, 32, 128};
}

template <typename Eng, int WGN, int WGM, int WN, int WM>
static int launch_cfg(const GemmArgs& a, hipStream_t st)
{
    constexpr int BN = WGN * WN * 32, BM = WGM * WM * 32;
    const int tiles_n = (int)cdiv(a.N, BN), tiles_m = (int)cdiv(a.M, BM);
    const int64_t grid = (int64_t)a.batch * tiles_n * tiles_m;
    if (grid <= 0 || grid > 0x7fffffffLL) return fail(BGEMM_EINVAL, "gemm_mfma: grid of %lld blocks", (long long)grid);
    if (a.mc.planes == 2) {
        // two accumulator sets: only the tiles whose registers fit are built for two planes
        if constexpr (WN * WM <= 4) {
            // 128 x 128 of two planes has the fragments and accumulators of 256 x 128 of one and runs its hand-pipelined
            // loop, from the same K on as the one-plane tile; so does 32 x 256 (a wave: one tile row of both planes against
            // two weight tiles, four MFMAs a step; W[11008,4096] x 128 ternary rows 10.3 -> 9.1 us, W[22016,4096] x 128 17.5 ->
            // 14.8, W[11008,8192] x 320 28.5 -> 24.0)
            if constexpr ((WGN == 2 && WGM == 2 && WN == 2 && WM == 2) || (WGN == 1 && WGM == 4 && WN == 1 && WM == 2)) {
                const bool pairs2 = a.out_kind == BGEMM_OUT_F16 && a.vec_store == 8;
                if (a.KT >= 8 && (!pairs2 || a.KT >= 16)) {
                    hipLaunchKernelGGL((gemm_mfma_kernel<Eng, WGN, WGM, WN, WM, 2, true>), dim3((unsigned)grid),
                                       dim3(WGN * WGM * 64), 0, st, a, tiles_n, tiles_m);
                    return check_launch("gemm_mfma");
                }
            }
            hipLaunchKernelGGL((gemm_mfma_kernel<Eng, WGN, WGM, WN, WM, 2, false>), dim3((unsigned)grid),
                               dim3(WGN * WGM * 64), 0, st, a, tiles_n, tiles_m);
        } else
            return fail(BGEMM_EINVAL, "gemm_mfma: tile not built for two planes");
    } else {
        // The hand-pipelined loop: always on the tiles of eight and sixteen MFMA tiles a wave; on 128 x 128 from eight
        // K-tiles on (11008 x 640 x 8192: 31.6 against 34.9 us, 8192^2 x 2048: 90.5 against 98.6; at four K-tiles the plain
        // loop is 4 % ahead); where the output is fp16 pairs, which only the plain loop stores straight from registers, from
        // sixteen K-tiles on (5120 x 2048 x 8192 -> fp16: 33.5 against 37.3 us, 6144 x 3072 x 4096: 31.2 against 33.8; level at eight).
        constexpr bool MUST_PIPE = WN * WM >= 8, CAN_PIPE = WN * WM >= 4 && WGM == 2 && WN % 2 == 0;
        const bool pairs = a.out_kind == BGEMM_OUT_F16 && a.vec_store == 8 && WM % 2 == 0;
        const dim3 g((unsigned)grid), blk(WGN * WGM * 64);
        if constexpr (CAN_PIPE) {
            if (MUST_PIPE || (a.KT >= 8 && (!pairs || a.KT >= 16))) {
                if (a.cntW && a.cntX)
                    hipLaunchKernelGGL((gemm_mfma_kernel<Eng, WGN, WGM, WN, WM, 1, true, true>), g, blk, 0, st, a, tiles_n, tiles_m);
                else
                    hipLaunchKernelGGL((gemm_mfma_kernel<Eng, WGN, WGM, WN, WM, 1, true>), g, blk, 0, st, a, tiles_n, tiles_m);
                return check_launch("gemm_mfma");
            }
        }
        if constexpr (!MUST_PIPE)
            hipLaunchKernelGGL((gemm_mfma_kernel<Eng, WGN, WGM, WN, WM, 1, false>), g, blk, 0, st, a, tiles_n, tiles_m);
    }
    return check_launch("gemm_mfma");
}

// Binary weights x ternary activations with signed operands on a 128 x 256 tile (a wave: two activation tile rows, the dearer
// side to expand, against four weight tiles): fp4 engine only.
template <typename Eng>
static int launch_tern(const GemmArgs& a, hipStream_t st)
{
    if constexpr (std::is_same<Eng, EngF4>::value) {
        if (a.mc.planes != 2) return fail(BGEMM_EINVAL, "gemm_mfma: the signed tile takes a ternary activation operand");
        const int tiles_n = (int)cdiv(a.N, 128), tiles_m = (int)cdiv(a.M, 256);
        const int64_t grid = (int64_t)a.batch * tiles_n * tiles_m;
        if (grid <= 0 || grid > 0x7fffffffLL) return fail(BGEMM_EINVAL, "gemm_mfma: grid of %lld blocks", (long long)grid);
        hipLaunchKernelGGL((gemm_mfma_kernel<EngF4, 2, 2, 2, 4, 1, true, false, true>), dim3((unsigned)grid), dim3(256), 0, st, a, tiles_n, tiles_m);
        return check_launch("gemm_mfma");
    } else
        return fail(BGEMM_EINVAL, "gemm_mfma: the signed ternary tile runs on the fp4 engine");
}

int gemm_mfma_kernel_id(int64_t batch, int64_t M, int64_t N, int64_t KT, int planes, int out_shift, bool fp4)
{
    return pick_cfg(batch, M, N, KT, planes, out_shift, fp4).id;
}

template <typename Eng>
static int launch_eng(const GemmArgs& a, hipStream_t st)
{
    const int id = a.force >= 0 ? a.force : pick_cfg(a.batch, a.M, a.N, a.KT, a.mc.planes, out_elem_shift(a.out_kind), std::is_same<Eng, EngF4>::value).id;
    switch (id) {
    case BGEMM_KERNEL_MFMA_256x256: return launch_cfg<Eng, 2, 2, 4, 4>(a, st);
    case BGEMM_KERNEL_MFMA_256x128: return launch_cfg<Eng, 2, 2, 4, 2>(a, st);    // two blocks per CU
    case BGEMM_KERNEL_MFMA_64x64: return launch_cfg<Eng, 2, 2, 1, 1>(a, st);
    case BGEMM_KERNEL_MFMA_128x64: return launch_cfg<Eng, 2, 2, 2, 1>(a, st);
    case BGEMM_KERNEL_MFMA_128x128: return launch_cfg<Eng, 2, 2, 2, 2>(a, st);
    case BGEMM_KERNEL_MFMA_64x128: return launch_cfg<Eng, 1, 4, 2, 1>(a, st);
    case BGEMM_KERNEL_MFMA_32x128: return launch_cfg<Eng, 1, 4, 1, 1>(a, st);
    case BGEMM_KERNEL_MFMA_32x256: return launch_cfg<Eng, 1, 4, 1, 2>(a, st);
    case BGEMM_KERNEL_MFMA_128x256T: return launch_tern<Eng>(a, st);
    default: return fail(BGEMM_EINVAL, "gemm_mfma: no kernel %d", id);
    }
}

int launch_gemm_mfma(const GemmArgs& a, hipStream_t st, bool fp4)
{
    return fp4 ? launch_eng<EngF4>(a, st) : launch_eng<EngI8>(a, st);
}

}  // namespace bgemm
