// fp16 / fp32 -> bit-plane packing and logical <-> tiled re-layout.  HBM-bound byte work.
// Tiled output: a wave packs one 32-row x 256-bit tile, with all of its 16-byte loads in
// flight at once; each lane turns eight elements into a byte of sign (and nonzero) bits, the
// bytes are put in tile order through LDS, and the tile leaves as one 16-byte store per lane.
// Logical output (the reference's row-major words): a wave packs 512 elements of one row.
#include "common.h"
#include "pack_bits.h"
#include <type_traits>
#include <string.h>

namespace bgemm {

// One operand to pack.  mode bit3: tiled output written by the row-segment waves (small operands:
// sixteen times as many, shorter waves).  mode bit0: also write the (sign & nonzero) plane and make plane 0 the
// nonzero plane.  mode bit1: write the logical layout instead of the tiled one.  mode bit2: the
// source is fp32 (rounded to fp16 first, as the layers' `.to(torch.half)` does).
// zp: device scalar of the source type subtracted before that rounding, or null.
// A job may hold nmat = outer x inner matrices of `rows` rows each (tiled output only): matrix (o, i) starts
// so * o + si * i elements into src and fills its own mtiles row tiles of the output, one matrix after the other.
struct PackJob {
    const void* src; int64_t rows, K, ld;
    uint32_t* dst0; uint32_t* dst1; int mode;
    const void* zp;
    int64_t rows_out, nseg, KT, Kw, waves;
    int64_t nmat, inner, so, si, mtiles;
};

// Element offset of output row `row` in the source, or -1 for a row of padding.
__device__ __forceinline__ int64_t source_row(const PackJob& j, const int64_t row)
{
    if (j.nmat == 1) return row < j.rows ? row * j.ld : -1;
    const int64_t mpad = j.mtiles * TILE_ROWS, b = row / mpad, rl = row - b * mpad;
    if (rl >= j.rows) return -1;
    const int64_t o = b / j.inner, i = b - o * j.inner;
    return o * j.so + i * j.si + rl * j.ld;
}

// Logical output: one wave packs 512 consecutive K elements of one row (16 words).
__device__ __forceinline__ void pack_wave(const PackJob& j, const int64_t gw, const int lane)
{
    const int64_t row = gw / j.nseg, seg = gw - row * j.nseg;
    if (row >= j.rows_out) return;        // whole wave leaves together
    const int64_t k0 = seg * 512 + 8 * lane;

    uint16_t h[8];                        // fp16 bit patterns; elements past K stay +0.0
#pragma unroll
    for (int e = 0; e < 8; e++) h[e] = 0;
    const int64_t soff = source_row(j, row);
    if (soff >= 0 && k0 < j.K) {
        if (j.mode & 4) {
            const float* p = reinterpret_cast<const float*>(j.src) + soff + k0;
            const float z = j.zp ? *reinterpret_cast<const float*>(j.zp) : 0.f;
            if (k0 + 8 <= j.K && (((uintptr_t)p) & 15) == 0) {
                const float4 u = *reinterpret_cast<const float4*>(p), v = *reinterpret_cast<const float4*>(p + 4);
                const float f[8] = {u.x, u.y, u.z, u.w, v.x, v.y, v.z, v.w};
#pragma unroll
                for (int e = 0; e < 8; e++) h[e] = half_bits(j.zp ? __fsub_rn(f[e], z) : f[e]);
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) if (k0 + e < j.K) h[e] = half_bits(j.zp ? __fsub_rn(p[e], z) : p[e]);
            }
        } else {
            const uint16_t* p = reinterpret_cast<const uint16_t*>(j.src) + soff + k0;
            if (k0 + 8 <= j.K && (((uintptr_t)p) & 15) == 0) {
                const uint4 v = *reinterpret_cast<const uint4*>(p);
                h[0] = v.x & 0xffff; h[1] = v.x >> 16; h[2] = v.y & 0xffff; h[3] = v.y >> 16;
                h[4] = v.z & 0xffff; h[5] = v.z >> 16; h[6] = v.w & 0xffff; h[7] = v.w >> 16;
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) if (k0 + e < j.K) h[e] = p[e];
            }
            if (j.zp) {
                const float z = __half2float(*reinterpret_cast<const __half*>(j.zp));
#pragma unroll
                for (int e = 0; e < 8; e++)
                    if (k0 + e < j.K) h[e] = half_bits(__fsub_rn(__half2float(__ushort_as_half(h[e])), z));
            }
        }
    }
    uint32_t sg = 0, nz = 0;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        sg |= (uint32_t)(h[e] >> 15) << (7 - e);
        nz |= (uint32_t)((h[e] & 0x7fff) != 0) << (7 - e);
    }
    const bool ternary = j.mode & 1;
    uint32_t p0 = ternary ? nz : sg, p1 = sg & nz;
    const int sh = 8 * (3 - (lane & 3));
    p0 <<= sh; p1 <<= sh;
    p0 |= __shfl_xor(p0, 1); p0 |= __shfl_xor(p0, 2);
    if (ternary) { p1 |= __shfl_xor(p1, 1); p1 |= __shfl_xor(p1, 2); }
    if (lane & 3) return;
    const int64_t jw = seg * 16 + (lane >> 2);
    if (j.mode & 2) {
        if (row < j.rows && jw < j.Kw) { j.dst0[row * j.Kw + jw] = p0; if (ternary) j.dst1[row * j.Kw + jw] = p1; }
    } else if (jw < j.KT * 8) {
        const int64_t o = tiled_word_offset(row, jw, j.KT);
        j.dst0[o] = p0;
        if (ternary) j.dst1[o] = p1;
    }
}

// One wave packs tile (rt, kt) = gw of the tiled layout.  Lane (c = lane & 31, lane >> 5) takes
// elements 256 kt + 8c .. + 7 of rows 2 jj + (lane >> 5), jj = 0..15.  lds: 2 KiB of this wave's own.
__device__ __forceinline__ void pack_tile(const PackJob& j, const int64_t gw, const int lane, unsigned char* lds)
{
    const int64_t rt = gw / j.KT, kt = gw - rt * j.KT;
    if (rt * TILE_ROWS >= j.rows_out) return;              // whole wave leaves together
    const int c = lane & 31, rsub = lane >> 5;
    const int64_t k0 = kt * TILE_KBITS + 8 * c;
    // where the tile's first row lies in the source, and how many source rows there are from it on
    int64_t off0 = rt * TILE_ROWS * j.ld, rows_left = j.rows - rt * TILE_ROWS;
    if (j.nmat > 1) {
        const int64_t b = rt / j.mtiles, rtl = rt - b * j.mtiles, o = b / j.inner, i = b - o * j.inner;
        off0 = o * j.so + i * j.si + rtl * TILE_ROWS * j.ld;
        rows_left = j.rows - rtl * TILE_ROWS;
    }
    const bool ternary = j.mode & 1, f32 = j.mode & 4;
    // byte of (row r, lane c) inside the tile: word c >> 2 of the row goes to slot h * 32 + r, position q;
    // the row's first element is the word's most significant bit, i.e. byte 3 of the little-endian word
    const int byte0 = (((c >> 4) * 32) * 4 + ((c >> 2) & 3)) * 4 + (3 - (c & 3));
    float zf = 0.f;
    if (j.zp) zf = f32 ? *reinterpret_cast<const float*>(j.zp) : __half2float(*reinterpret_cast<const __half*>(j.zp));
    auto emit = [&](const int r, uint16_t (&h)[8], const int valid) {
        if (j.zp && !f32) {
#pragma unroll
            for (int e = 0; e < 8; e++)
                if (e < valid) h[e] = half_bits(__fsub_rn(__half2float(__ushort_as_half(h[e])), zf));
        }
        uint32_t sg, nz;
        bits8(h, sg, nz);
        lds[byte0 + r * 16] = (unsigned char)(ternary ? nz : sg);
        if (ternary) lds[1024 + byte0 + r * 16] = (unsigned char)(sg & nz);
    };
    // the whole tile lies inside the source and every row is 16-byte aligned: plain vector loads, all in flight
    const int64_t esz = f32 ? 4 : 2;
    const bool rows_in = rows_left >= TILE_ROWS &&
                         ((((uintptr_t)j.src) | (uintptr_t)(j.ld * esz) | (uintptr_t)(j.so * esz) | (uintptr_t)(j.si * esz)) & 15) == 0;
    const bool interior = rows_in && kt * TILE_KBITS + TILE_KBITS <= j.K;
    if (!f32 && rows_in && (interior || (j.K & 7) == 0)) {
        // also the last K-tile of a K that is a multiple of eight (head size 64: the only tile).  The lanes are
        // spread over as many 8-element chunks as the tile's rows have here (8, 16 or 32), so a short row
        // does not leave most of the wave idle: CW lanes per row, 64 / CW rows per step.
        const int64_t left = j.K - kt * TILE_KBITS;
        auto rows_by = [&](auto cw_tag) {
            constexpr int CW = decltype(cw_tag)::value, RI = 64 / CW, STEPS = TILE_ROWS / RI;
            const int cc = lane & (CW - 1), rs = lane / CW;
            const int b0 = (((cc >> 4) * 32) * 4 + ((cc >> 2) & 3)) * 4 + (3 - (cc & 3));
            const uint16_t* p = reinterpret_cast<const uint16_t*>(j.src) + off0 + rs * j.ld + kt * TILE_KBITS + 8 * cc;
            const bool live = 8 * cc < left;
            uint4 raw[STEPS];
#pragma unroll
            for (int jj = 0; jj < STEPS; jj++)
                raw[jj] = live ? *reinterpret_cast<const uint4*>(p + (int64_t)(RI * jj) * j.ld) : make_uint4(0u, 0u, 0u, 0u);
            if (CW < 32)                           // the bytes of the chunks this tile does not have
                for (int i = lane; i < (ternary ? 512 : 256); i += 64) reinterpret_cast<uint32_t*>(lds)[i] = 0u;
#pragma unroll
            for (int jj = 0; jj < STEPS; jj++) {
                const uint4 v = raw[jj];
                uint16_t h[8] = {(uint16_t)(v.x & 0xffff), (uint16_t)(v.x >> 16), (uint16_t)(v.y & 0xffff), (uint16_t)(v.y >> 16),
                                 (uint16_t)(v.z & 0xffff), (uint16_t)(v.z >> 16), (uint16_t)(v.w & 0xffff), (uint16_t)(v.w >> 16)};
                const int r = RI * jj + rs;
                uint32_t sg, nz;
                if (j.zp && live) {
#pragma unroll
                    for (int e = 0; e < 8; e++) h[e] = half_bits(__fsub_rn(__half2float(__ushort_as_half(h[e])), zf));
                    bits8(h, sg, nz);
                } else
                    bits8(v, sg, nz);
                lds[b0 + r * 16] = (unsigned char)(ternary ? nz : sg);
                if (ternary) lds[1024 + b0 + r * 16] = (unsigned char)(sg & nz);
            }
        };
        if (left <= 64) rows_by(std::integral_constant<int, 8>{});
        else if (left <= 128) rows_by(std::integral_constant<int, 16>{});
        else rows_by(std::integral_constant<int, 32>{});
    } else if (interior) {
        const float* p = reinterpret_cast<const float*>(j.src) + off0 + rsub * j.ld + k0;
#pragma unroll
        for (int g = 0; g < 2; g++) {
            float4 lo[8], hi[8];
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {
                const float* q = p + (int64_t)(2 * (8 * g + jj)) * j.ld;
                lo[jj] = *reinterpret_cast<const float4*>(q);
                hi[jj] = *reinterpret_cast<const float4*>(q + 4);
            }
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {
                const float f[8] = {lo[jj].x, lo[jj].y, lo[jj].z, lo[jj].w, hi[jj].x, hi[jj].y, hi[jj].z, hi[jj].w};
                uint16_t h[8];
#pragma unroll
                for (int e = 0; e < 8; e++) h[e] = half_bits(j.zp ? __fsub_rn(f[e], zf) : f[e]);
                emit(2 * (8 * g + jj) + rsub, h, 8);
            }
        }
    } else {
        // edge tiles and unaligned sources: element loads, rows and columns past the end read as +0.0
        for (int jj = 0; jj < 16; jj++) {
            const int row = 2 * jj + rsub;
            uint16_t h[8];
#pragma unroll
            for (int e = 0; e < 8; e++) h[e] = 0;
            int valid = 0;
            if (row < rows_left && k0 < j.K) {
                valid = (int)(j.K - k0 < 8 ? j.K - k0 : 8);
                if (f32) {
                    const float* q = reinterpret_cast<const float*>(j.src) + off0 + row * j.ld + k0;
#pragma unroll
                    for (int e = 0; e < 8; e++) if (e < valid) h[e] = half_bits(j.zp ? __fsub_rn(q[e], zf) : q[e]);
                } else {
                    const uint16_t* q = reinterpret_cast<const uint16_t*>(j.src) + off0 + row * j.ld + k0;
#pragma unroll
                    for (int e = 0; e < 8; e++) if (e < valid) h[e] = q[e];
                }
            }
            emit(2 * jj + rsub, h, valid);
        }
    }
    __builtin_amdgcn_wave_barrier();       // the tile was written by this wave alone: LDS keeps its order
    reinterpret_cast<uint4*>(j.dst0)[gw * TILE_U4 + lane] = reinterpret_cast<const uint4*>(lds)[lane];
    if (ternary) reinterpret_cast<uint4*>(j.dst1)[gw * TILE_U4 + lane] = reinterpret_cast<const uint4*>(lds + 1024)[lane];
}

// Up to two operands per launch (the fp16 entry point packs weights and activations together).
__global__ __launch_bounds__(256) void pack_f16_kernel(const PackJob j0, const PackJob j1)
{
    __shared__ __align__(16) unsigned char s_tile[4][2048];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int64_t gw = (int64_t)blockIdx.x * 4 + wave;
    const bool first = gw < j0.waves;
    const PackJob& j = first ? j0 : j1;
    if (!first) gw -= j0.waves;
    if (gw >= j.waves) return;
    if (j.mode & (2 | 8)) pack_wave(j, gw, lane);
    else pack_tile(j, gw, lane, s_tile[wave]);
}

// dir 0: logical -> tiled (zero padding), dir 1: tiled -> logical.  One thread per tiled word.
__global__ __launch_bounds__(256) void relayout_kernel(
    const uint32_t* __restrict__ src, uint32_t* __restrict__ dst, int64_t rows, int64_t Kw,
    int64_t KT, int64_t total, int dir)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    // decode tiled word index i -> (row, jw)
    const int64_t q = i & 3, slot = (i >> 2) & 63, tile = i >> 8;
    const int64_t kt = tile % KT, rt = tile / KT;
    const int64_t row = rt * 32 + (slot & 31), jw = kt * 8 + (slot >> 5) * 4 + q;
    const bool real = row < rows && jw < Kw;
    if (dir == 0) dst[i] = real ? src[row * Kw + jw] : 0u;
    else if (real) dst[row * Kw + jw] = src[i];
}

static int make_job(PackJob* j, const void* src, int64_t rows, int64_t K, int64_t ld, void* d0, void* d1, int mode,
                    const void* zp, const char* who, int64_t outer = 1, int64_t inner = 1, int64_t so = 0, int64_t si = 0)
{
    if (rows < 0 || K < 0 || ld < K) return fail(BGEMM_EINVAL, "%s: bad shape rows=%lld K=%lld ld=%lld", who,
                                                 (long long)rows, (long long)K, (long long)ld);
    if (outer < 0 || inner < 0 || so < 0 || si < 0 || ((mode & 2) && outer * inner != 1))
        return fail(BGEMM_EINVAL, "%s: bad batch %lld x %lld, strides %lld, %lld", who, (long long)outer,
                    (long long)inner, (long long)so, (long long)si);
    memset(j, 0, sizeof *j);
    if (rows == 0 || K == 0 || outer * inner == 0) return BGEMM_OK;
    if (!src || !d0 || ((mode & 1) && !d1)) return fail(BGEMM_ENULL, "%s: null pointer", who);
    if (((uintptr_t)d0 & 15) || ((uintptr_t)d1 & 15)) return fail(BGEMM_EALIGN, "%s: destination not 16-byte aligned", who);
    j->src = src; j->zp = zp; j->rows = rows; j->K = K; j->ld = ld;
    j->dst0 = (uint32_t*)d0; j->dst1 = (uint32_t*)d1; j->mode = mode;
    j->KT = k_tiles(K); j->Kw = cdiv(K, 32);
    j->nmat = outer * inner; j->inner = inner; j->so = so; j->si = si; j->mtiles = row_tiles(rows);
    j->rows_out = (mode & 2) ? rows : j->nmat * j->mtiles * TILE_ROWS;
    j->nseg = cdiv(j->KT * TILE_KBITS, 512);
    // a wave per tile streams best, but an operand of a few hundred tiles would leave most SIMDs without one
    // (measured crossover: 500 to 700 tiles)
    if (!(mode & 2) && j->nmat * j->mtiles * j->KT < 640) j->mode |= 8;
    j->waves = (j->mode & (2 | 8)) ? j->rows_out * j->nseg : j->nmat * j->mtiles * j->KT;
    return BGEMM_OK;
}

static int launch_jobs(const PackJob& j0, const PackJob& j1, hipStream_t st, const char* who)
{
    const int64_t blocks = cdiv(j0.waves + j1.waves, 4);
    if (blocks == 0) return BGEMM_OK;
    if (blocks > 0x7fffffffLL) return fail(BGEMM_EINVAL, "%s: operand too large", who);
    hipLaunchKernelGGL(pack_f16_kernel, dim3((unsigned)blocks), dim3(256), 0, st, j0, j1);
    return check_launch(who);
}

static int pack_common(const void* src, int64_t rows, int64_t K, int64_t ld, void* d0, void* d1,
                       int mode, const void* zp, hipStream_t st, const char* who,
                       int64_t outer = 1, int64_t inner = 1, int64_t so = 0, int64_t si = 0)
{
    PackJob j0, j1;
    memset(&j1, 0, sizeof j1);
    const int rc = make_job(&j0, src, rows, K, ld, d0, d1, mode, zp, who, outer, inner, so, si);
    return rc ? rc : launch_jobs(j0, j1, st, who);
}

// Sign-packs two fp16 operands into their tiled buffers with one launch.
int pack_sign_pair(const void* srcA, int64_t rowsA, void* dstA, const void* srcB, int64_t rowsB, void* dstB,
                   int64_t K, hipStream_t st, const char* who)
{
    PackJob j0, j1;
    int rc = make_job(&j0, srcA, rowsA, K, K, dstA, nullptr, 0, nullptr, who);
    if (!rc) rc = make_job(&j1, srcB, rowsB, K, K, dstB, nullptr, 0, nullptr, who);
    return rc ? rc : launch_jobs(j0, j1, st, who);
}

}  // namespace bgemm

using namespace bgemm;

extern "C" int64_t bgemm_tiled_words(int64_t rows, int64_t K)
{
    if (rows <= 0 || K <= 0) return 0;
    return row_tiles(rows) * k_tiles(K) * TILE_WORDS;
}

extern "C" int bgemm_pack_sign_f16(const void* src, int64_t rows, int64_t K, int64_t ld,
                                   void* dst_tiled, void* stream)
{
    return pack_common(src, rows, K, ld, dst_tiled, nullptr, 0, nullptr, (hipStream_t)stream, "bgemm_pack_sign_f16");
}

extern "C" int bgemm_pack_sign_f16_logical(const void* src, int64_t rows, int64_t K, int64_t ld,
                                           uint32_t* dst_logical, void* stream)
{
    return pack_common(src, rows, K, ld, dst_logical, nullptr, 2, nullptr, (hipStream_t)stream, "bgemm_pack_sign_f16_logical");
}

extern "C" int bgemm_pack_ternary_f16(const void* src, int64_t rows, int64_t K, int64_t ld,
                                      void* nz_tiled, void* sg_tiled, void* stream)
{
    return pack_common(src, rows, K, ld, nz_tiled, sg_tiled, 1, nullptr, (hipStream_t)stream, "bgemm_pack_ternary_f16");
}

extern "C" int bgemm_pack_sign_centered(const void* src, int src_dtype, int64_t rows, int64_t K, int64_t ld,
                                        const void* zero_point, void* dst_tiled, void* stream)
{
    if (src_dtype != BGEMM_SRC_F16 && src_dtype != BGEMM_SRC_F32)
        return fail(BGEMM_EINVAL, "bgemm_pack_sign_centered: unknown source type %d", src_dtype);
    return pack_common(src, rows, K, ld, dst_tiled, nullptr, src_dtype == BGEMM_SRC_F32 ? 4 : 0, zero_point,
                       (hipStream_t)stream, "bgemm_pack_sign_centered");
}

extern "C" int bgemm_pack_batched(const void* src, int src_dtype, int ternary, const void* zero_point,
                                  int64_t batch_outer, int64_t batch_inner, int64_t rows, int64_t K, int64_t ld,
                                  int64_t stride_outer, int64_t stride_inner, void* dst0_tiled, void* dst1_tiled,
                                  void* stream)
{
    if (src_dtype != BGEMM_SRC_F16 && src_dtype != BGEMM_SRC_F32)
        return fail(BGEMM_EINVAL, "bgemm_pack_batched: unknown source type %d", src_dtype);
    if (ternary && zero_point) return fail(BGEMM_EINVAL, "bgemm_pack_batched: a zero point goes with the sign pack only");
    return pack_common(src, rows, K, ld, dst0_tiled, ternary ? dst1_tiled : nullptr,
                       (ternary ? 1 : 0) | (src_dtype == BGEMM_SRC_F32 ? 4 : 0), zero_point, (hipStream_t)stream,
                       "bgemm_pack_batched", batch_outer, batch_inner, stride_outer, stride_inner);
}

namespace bgemm {

// Transposed source ([K][rows] in memory): a wave builds one 32-row x 256-bit tile.  For each of its
// four words, lane (h, k') reads the 32 consecutive fp16 of source row k = 256 kt + 128 h + 32 q + k'
// (four 16-byte loads when the source allows, all sixteen in flight), gathers their sign bits into a
// word (bit r = row r), and the 32 x 32 bit matrix held by the 32 lanes of a wave half is transposed
// in registers with five masked exchanges: lane r then holds the word of row r, bit k' = column k'.
__device__ __forceinline__ unsigned transpose32(unsigned w, const int lane)
{
#pragma unroll
    for (int j = 16; j >= 1; j >>= 1) {
        const unsigned m = j == 16 ? 0x0000ffffu : j == 8 ? 0x00ff00ffu : j == 4 ? 0x0f0f0f0fu : j == 2 ? 0x33333333u : 0x55555555u;
        const unsigned other = __shfl_xor(w, j);
        w = (lane & j) ? (w & (m << j)) | ((other >> j) & m) : (w & m) | ((other & m) << j);
    }
    return w;
}

template <bool F32>
__global__ __launch_bounds__(256) void pack_transposed_kernel(const void* __restrict__ src_, const int64_t rows,
                                                              const int64_t K, const int64_t ld, const int64_t inner,
                                                              const int64_t so, const int64_t si,
                                                              uint4* __restrict__ dst, const int64_t tiles_per_matrix,
                                                              const int64_t KT, const int64_t total_tiles)
{
    typedef typename std::conditional<F32, uint32_t, uint16_t>::type E;
    constexpr int EB = sizeof(E), NV = 32 * EB / 16;       // 16-byte loads per 32 elements
    const int lane = threadIdx.x & 63, h = lane >> 5, kk = lane & 31;
    const int64_t tile = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tile >= total_tiles) return;             // whole wave leaves together
    const int64_t b = tile / tiles_per_matrix, t = tile - b * tiles_per_matrix, rt = t / KT, kt = t - rt * KT;
    const int64_t o = b / inner, i = b - o * inner;
    const int64_t r0 = rt * 32, k0 = kt * TILE_KBITS + h * 128 + kk;
    const E* p = reinterpret_cast<const E*>(src_) + o * so + i * si + k0 * ld + r0;
    const bool vec = r0 + 32 <= rows &&
                     (((uintptr_t)src_ | (uintptr_t)(ld * EB) | (uintptr_t)(so * EB) | (uintptr_t)(si * EB)) & 15) == 0;
    unsigned w[4];
    if (vec) {
        uint4 raw[4][NV];
#pragma unroll
        for (int q = 0; q < 4; q++)
#pragma unroll
            for (int c = 0; c < NV; c++)
                raw[q][c] = k0 + q * 32 < K ? reinterpret_cast<const uint4*>(p + (int64_t)q * 32 * ld)[c] : make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
        for (int q = 0; q < 4; q++) {
            unsigned x = 0;
#pragma unroll
            for (int c = 0; c < NV; c++) {
                const unsigned d[4] = {raw[q][c].x, raw[q][c].y, raw[q][c].z, raw[q][c].w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    if (F32)
                        x |= (d[e] >> 31) << (4 * c + e);
                    else {
                        const unsigned sb = d[e] & 0x80008000u;          // sign bits of two halves
                        x |= (((sb >> 15) | (sb >> 30)) & 3u) << (8 * c + 2 * e);
                    }
                }
            }
            w[q] = x;
        }
    } else {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            unsigned x = 0;
            if (k0 + q * 32 < K)
                for (int r = 0; r < 32; r++)
                    if (r0 + r < rows) x |= (unsigned)(p[(int64_t)q * 32 * ld + r] >> (8 * EB - 1)) << r;
            w[q] = x;
        }
    }
    // lane r of each half now takes row r; element k' of a word goes to bit 31 - k'
#pragma unroll
    for (int q = 0; q < 4; q++) w[q] = __brev(transpose32(w[q], lane));
    dst[tile * TILE_U4 + lane] = make_uint4(w[0], w[1], w[2], w[3]);
}

}  // namespace bgemm

extern "C" int bgemm_pack_transposed_batched(const void* src, int src_dtype, int64_t batch_outer, int64_t batch_inner,
                                             int64_t rows, int64_t K, int64_t ld, int64_t stride_outer,
                                             int64_t stride_inner, void* dst_tiled, void* stream)
{
    const char* who = "bgemm_pack_transposed_batched";
    if (src_dtype != BGEMM_SRC_F16 && src_dtype != BGEMM_SRC_F32) return fail(BGEMM_EINVAL, "%s: unknown source type %d", who, src_dtype);
    if (batch_outer < 0 || batch_inner < 0 || rows < 0 || K < 0 || ld < rows || stride_outer < 0 || stride_inner < 0)
        return fail(BGEMM_EINVAL, "%s: bad shape batch=%lld x %lld rows=%lld K=%lld ld=%lld", who, (long long)batch_outer,
                    (long long)batch_inner, (long long)rows, (long long)K, (long long)ld);
    const int64_t batch = batch_outer * batch_inner;
    if (batch == 0 || rows == 0 || K == 0) return BGEMM_OK;
    if (!src || !dst_tiled) return fail(BGEMM_ENULL, "%s: null pointer", who);
    const bool f32 = src_dtype == BGEMM_SRC_F32;
    if (((uintptr_t)src & (f32 ? 3 : 1)) || ((uintptr_t)dst_tiled & 15))
        return fail(BGEMM_EALIGN, "%s: source must be aligned to its elements, destination to 16 bytes", who);
    const int64_t KT = k_tiles(K), per = row_tiles(rows) * KT, total = batch * per, blocks = cdiv(total, 4);
    if (blocks > 0x7fffffffLL) return fail(BGEMM_EINVAL, "%s: operand too large", who);
    if (f32)
        hipLaunchKernelGGL(pack_transposed_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, src, rows,
                           K, ld, batch_inner, stride_outer, stride_inner, reinterpret_cast<uint4*>(dst_tiled), per, KT, total);
    else
        hipLaunchKernelGGL(pack_transposed_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, src, rows,
                           K, ld, batch_inner, stride_outer, stride_inner, reinterpret_cast<uint4*>(dst_tiled), per, KT, total);
    return check_launch(who);
}

extern "C" int bgemm_pack_sign_f16_transposed(const void* src, int64_t batch, int64_t rows, int64_t K, int64_t ld,
                                              int64_t src_batch_stride, void* dst_tiled, void* stream)
{
    return bgemm_pack_transposed_batched(src, BGEMM_SRC_F16, 1, batch, rows, K, ld, 0, src_batch_stride, dst_tiled, stream);
}

static int relayout(const void* src, void* dst, int64_t rows, int64_t K, int dir, void* stream, const char* who)
{
    if (rows < 0 || K < 0) return fail(BGEMM_EINVAL, "%s: bad shape", who);
    if (rows == 0 || K == 0) return BGEMM_OK;
    if (!src || !dst) return fail(BGEMM_ENULL, "%s: null pointer", who);
    const int64_t total = bgemm_tiled_words(rows, K), blocks = cdiv(total, 256);
    if (blocks > 0x7fffffffLL) return fail(BGEMM_EINVAL, "%s: operand too large", who);
    hipLaunchKernelGGL(relayout_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const uint32_t*)src, (uint32_t*)dst, rows, cdiv(K, 32), k_tiles(K), total, dir);
    return check_launch(who);
}

// Row popcounts of a tiled operand: one block of sixteen waves per 32-row tile row, wave w takes K-tiles w, w + 16, ...
// (two 16-byte loads in flight a lane: a launch of this size is one memory round trip), lanes 0-31 and 32-63 of a
// wave hold the two K-halves of a row; the partial counts of a row meet in LDS.
__global__ __launch_bounds__(1024) void row_popcount_kernel(const uint4* __restrict__ tiled, int32_t* __restrict__ counts,
                                                            const int64_t rows, const int64_t KT, const int64_t stride_u4)
{
    __shared__ int part[1024];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t rt = blockIdx.x, b = blockIdx.y;
    const uint4* base = tiled + b * stride_u4 + rt * KT * TILE_U4 + lane;
    int n = 0;
    int64_t kt = wave;
    for (; kt + 16 < KT; kt += 32) {
        const uint4 v0 = base[kt * TILE_U4], v1 = base[(kt + 16) * TILE_U4];
        n += __popc(v0.x) + __popc(v0.y) + __popc(v0.z) + __popc(v0.w) + __popc(v1.x) + __popc(v1.y) + __popc(v1.z) + __popc(v1.w);
    }
    if (kt < KT) {
        const uint4 v = base[kt * TILE_U4];
        n += __popc(v.x) + __popc(v.y) + __popc(v.z) + __popc(v.w);
    }
    part[threadIdx.x] = n;
    __syncthreads();
    if (threadIdx.x < 32) {
        int t = 0;
#pragma unroll
        for (int w = 0; w < 32; w++) t += part[w * 32 + threadIdx.x];     // 16 waves x 2 K-halves
        const int64_t row = rt * 32 + threadIdx.x;
        if (row < rows) counts[b * rows + row] = t;
    }
}

extern "C" int bgemm_row_popcounts(const void* tiled, int64_t batch, int64_t rows, int64_t K, int64_t stride_words,
                                   void* counts, void* stream)
{
    if (batch < 0 || rows < 0 || K < 0 || K >= (1LL << 24) || stride_words < 0 || (stride_words & 3))
        return fail(BGEMM_EINVAL, "bgemm_row_popcounts: bad shape batch=%lld rows=%lld K=%lld stride=%lld", (long long)batch,
                    (long long)rows, (long long)K, (long long)stride_words);
    if (batch == 0 || rows == 0) return BGEMM_OK;
    if (!counts || (K > 0 && !tiled)) return fail(BGEMM_ENULL, "bgemm_row_popcounts: null pointer");
    if (((uintptr_t)tiled & 15) || ((uintptr_t)counts & 3)) return fail(BGEMM_EALIGN, "bgemm_row_popcounts: operand not aligned");
    if (batch > 65535 || row_tiles(rows) > 0x7fffffffLL) return fail(BGEMM_EINVAL, "bgemm_row_popcounts: operand too large");
    if (batch > 1 && stride_words < bgemm_tiled_words(rows, K))
        return fail(BGEMM_EINVAL, "bgemm_row_popcounts: stride %lld smaller than one operand", (long long)stride_words);
    hipLaunchKernelGGL(row_popcount_kernel, dim3((unsigned)row_tiles(rows), (unsigned)batch), dim3(1024), 0, (hipStream_t)stream,
                       (const uint4*)tiled, (int32_t*)counts, rows, k_tiles(K), stride_words / 4);
    return check_launch("bgemm_row_popcounts");
}

extern "C" int bgemm_tile_from_logical(const uint32_t* logical, int64_t rows, int64_t K,
                                       void* dst_tiled, void* stream)
{
    return relayout(logical, dst_tiled, rows, K, 0, stream, "bgemm_tile_from_logical");
}

extern "C" int bgemm_logical_from_tiled(const void* tiled, int64_t rows, int64_t K,
                                        uint32_t* dst_logical, void* stream)
{
    return relayout(tiled, dst_logical, rows, K, 1, stream, "bgemm_logical_from_tiled");
}
