// Shared definitions for the gfx950 BGEMM library (host + device).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/bgemm_mi355x.h"

namespace bgemm {

// Tiled operand geometry: a tile is 32 rows x 256 K-bits = 64 slots of 16 bytes.
constexpr int TILE_ROWS = 32;
constexpr int TILE_KBITS = 256;
constexpr int TILE_U4 = 64;      // uint4 slots per tile
constexpr int TILE_WORDS = 256;  // uint32 words per tile

__host__ __device__ static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline int64_t row_tiles(int64_t rows) { return cdiv(rows, TILE_ROWS); }
__host__ __device__ static inline int64_t k_tiles(int64_t K) { return cdiv(K, TILE_KBITS); }

// Word offset of logical word jw of `row` inside a tiled operand with KT k-tiles.
__host__ __device__ static inline int64_t tiled_word_offset(int64_t row, int64_t jw, int64_t KT)
{
    const int64_t rt = row >> 5, r = row & 31, kt = jw >> 3, h = (jw >> 2) & 1, q = jw & 3;
    return ((rt * KT + kt) * TILE_U4 + h * 32 + r) * 4 + q;
}

// Records a message for bgemm_last_error() and returns `code`.
int fail(int code, const char* fmt, ...);
// Maps a pending HIP error after a launch to BGEMM_ELAUNCH.
int check_launch(const char* what);

// Integer epilogue applied to the AND-dot D of a K range holding `bits` valid positions:
//   C = c0*bits + ca*pa[m] + cb*pb[n] + cd*D (+ cb2*pb2[n] + cd2*D2 for the second plane)
// pa / pb = popcounts of the weight-side / activation-side rows over the same range.
struct ModeCoef { int c0, ca, cb, cd, cb2, cd2, planes; };

static inline bool mode_coef(int mode, ModeCoef* mc)
{
    switch (mode) {
    case BGEMM_MODE_AND:    *mc = {0,  0,  0, 1, 0, 0, 1}; return true;
    case BGEMM_MODE_XOR:    *mc = {1, -2, -2, 4, 0, 0, 1}; return true;   // K - 2 popc(a^b)
    case BGEMM_MODE_ATTN:   *mc = {1, -1, -2, 2, 0, 0, 1}; return true;   // sum (1-a)(1-2b)
    case BGEMM_MODE_ATTN_X: *mc = {1, -2, -1, 2, 0, 0, 1}; return true;   // sum (1-b)(1-2a)
    case BGEMM_MODE_BWTA:   *mc = {0,  0,  1, -2, -2, 4, 2}; return true; // pz - 2pzs - 2D(a,z) + 4D(a,zs)
    default: return false;
    }
}

// Rank-one terms on the device.  K, the row popcounts and the AND-dot all reach 2^24 - 1, past the SIGNED
// 24-bit operands of __mul24 (which would read 2^23 as -2^23).  The few per-row and per-column terms use the
// plain 32-bit multiply.  The per-element term keeps a full-rate multiply-add through the UNSIGNED 24-bit
// one, whose operand range the dots fit; the signs of its coefficients are fixed by the number of planes
// (one plane: cd > 0; two planes, BWTA: cd < 0 < cd2), which mode_coef's table obeys.
__device__ __forceinline__ int dot_term(const ModeCoef& mc, const int d)
{
    return (int)__umul24((unsigned)mc.cd, (unsigned)d);
}
__device__ __forceinline__ int dot_terms2(const ModeCoef& mc, const int d, const int d2)
{
    return (int)__umul24((unsigned)mc.cd2, (unsigned)d2) - (int)__umul24((unsigned)-mc.cd, (unsigned)d);
}

// Output of one (activation row, weight row) pair from the AND-dots d (and d2 of the second plane).
__device__ __forceinline__ int skinny_value(const ModeCoef& mc, const bool two, const int kbits, const int pa,
                                            const int pb, const int pb2, const int d, const int d2)
{
    const int val = mc.c0 * kbits + mc.ca * pa + mc.cb * pb;
    return two ? val + mc.cb2 * pb2 + dot_terms2(mc, d, d2) : val + dot_term(mc, d);
}

struct GemmArgs {
    const uint4* W; const uint4* X; const uint4* X2;
    void* out; int out_kind;       // BGEMM_OUT_*
    const void* ep_sw; const void* ep_sa; const void* ep_bias;   // scaled output kinds: per-column scale, scalar, bias
    const void* ep_zp;    // bits kinds: the next layer's zero point (null = 0)
    int nt_store;         // general kernel: 4-byte outputs are stored past the caches (set for outputs of up to 32 MiB)
    int vec_store;        // 0, or the elements per lane the epilogue may store at once: 4 (rows of `out` 16-byte aligned
                          // for int32, 8-byte for fp16) or 8 (fp16 kinds with rows of a multiple of 8)
    int64_t M, N, K;
    int MT, NT, KT;
    int64_t strideW, strideX, strideC;   // uint4 units for W/X, elements for C
    int batch, splitK;
    int force;            // BGEMM_KERNEL_* the caller insists on (BGEMM_FORCE_KERNEL), or -1: chosen by shape
    const int32_t* cntW; const int32_t* cntX;   // row popcounts of W and X ([batch][rows], a shared operand once), or null:
                                                // the pipelined tiles then count nothing themselves
    ModeCoef mc;
    // activations not packed yet (the decode kernel packs them itself): X/X2 are null and these describe
    // the [N][K] source; with two planes the ternary planes of sign(x) are formed
    const void* xsrc; int64_t xld; int xsrc_f32; const void* xzp;
    int32_t* ws_part;     // split-K partial tiles, [batch][tile][split] in register order (scratch)
    uint32_t* ws_cnt;     // split-K arrival counters, one per output tile, zero between calls
};

// Contiguous split-K ranges over k-tiles: the first (KT - avg*splitK) splits get one extra.
__host__ __device__ static inline void split_range(int KT, int splitK, int s, int* k0, int* k1)
{
    const int avg = KT / splitK, extra = KT - avg * splitK;
    const int n = avg + (s < extra ? 1 : 0);
    const int st = avg * s + (s < extra ? s : extra);
    *k0 = st; *k1 = st + n;
}

// Hardware deals workgroups round-robin over the 8 XCDs (workgroup i runs on XCD i % 8, each XCD
// with its own L2).  This maps the hardware id to a logical id such that every XCD owns one
// contiguous run of logical ids: neighbouring tiles then share an L2.
__device__ __forceinline__ unsigned xcd_contiguous_id(const unsigned hw_id, const unsigned grid)
{
    const unsigned per = grid / 8, rem = grid % 8, x = hw_id % 8, y = hw_id / 8;
    return x * per + (x < rem ? x : rem) + y;
}

// Split-K hand-over between the blocks that share an output tile.  The grid is laid out so that
// these blocks carry the same hardware id modulo 8, i.e. run on one XCD and meet in one L2: the
// partial tile only has to have reached that L2 (stores complete) before the arrival ticket is
// taken, and the last block reads it with device-scope loads that bypass its L1.  A block that
// finds itself on another XCD than its id implies says so in the ticket and falls back to
// device-scope fences (whole-L2 write-back / invalidate, far slower), as does the reader then.
// Returns true in every thread of the block that arrived last.  Counters return to zero.
__device__ __forceinline__ bool splitk_arrive(unsigned* counter, const unsigned splits, int* s_flag)
{
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");     // this thread's partial stores have been acknowledged
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned xcc = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 0xf;    // XCC_ID[3:0]
        const bool home = xcc == (blockIdx.x & 7u);
        if (!home) __threadfence();
        const unsigned t = atomicAdd(counter, home ? 1u : 0x10001u);
        const int last = (t & 0xffffu) == splits - 1u;
        if (last) {
            atomicExch(counter, 0u);
            if (!home || (t >> 16)) __threadfence();
        }
        *s_flag = last;
    }
    __syncthreads();
    return *s_flag != 0;
}

// Device-scope 16-byte load of one partial-tile vector: `sc1` makes it miss the reader's L1 and
// take the line from the L2 the writer's stores went to.  `base` is uniform across the wave
// (a buffer resource is built from it), `byte_off` is this lane's offset from it.
__device__ __forceinline__ int4 load_partial(const void* base, const unsigned byte_off)
{
    typedef int v4i __attribute__((ext_vector_type(4)));
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7fffffff, 0x00020000);
    const v4i v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)byte_off, 0, 16 /* sc1 */);
    return make_int4(v.x, v.y, v.z, v.w);
}

// Split-K grids are padded to a multiple of 8 * splitK blocks and numbered split-fastest, so
// the splits of a tile fall into one XCD's contiguous run of logical ids.
static inline int64_t splitk_grid(int64_t real_blocks, int splitK)
{
    return splitK > 1 ? cdiv(real_blocks, 8 * (int64_t)splitK) * 8 * splitK : real_blocks;
}
// The result does not depend on the split, so the caller's value is treated as an upper bound.
// More K ranges than it takes to give every compute unit a block only add hand-over traffic (a
// grid that already has one block per unit gets slower when split), and a hand-over costs three
// dependent trips to the L2 (store, ticket, load: about 4 us), as much as a few dozen K-tiles of
// main loop: shorter ranges are not worth it.
static inline int effective_split(int64_t tiles, int splitK, int KT)
{
    int s = splitK;
    while (s > 1 && (tiles * s > 384 || KT / s < 24)) s--;
    return s;
}

// Output kinds: the int32 accumulator itself; fp16 = the integer rounded to nearest even (exact
// through fp32 because |v| < 2^24); or the binary Linear's scaling fused in, op for op as torch
// evaluates `half(acc) * sw * sa (+ bias)` (tests/python/bgemm_linear.py:482-484): with fp32
// parameters every step is an fp32 op, with fp16 parameters every step rounds to fp16.  No step
// may be contracted into an FMA: the functions switch contraction off and use plain operators (the
// __fmul_rn / __fadd_rn wrappers are ordinary inline functions compiled with contraction allowed, so
// a multiply and an add that come out of them can still be fused after inlining).
__device__ __forceinline__ float scaled_f32(const GemmArgs& a, const int64_t m, const int v)
{
#pragma clang fp contract(off)      // every step rounds by itself, as torch's separate kernels do
    float r = (__half2float(__float2half_rn((float)v)) * reinterpret_cast<const float*>(a.ep_sw)[m]);
    r = (r * *reinterpret_cast<const float*>(a.ep_sa));
    if (a.ep_bias) r = (r + reinterpret_cast<const float*>(a.ep_bias)[m]);
    return r;
}
__device__ __forceinline__ __half scaled_f16(const GemmArgs& a, const int64_t m, const int v)
{
#pragma clang fp contract(off)      // every step rounds by itself, as torch's separate kernels do
    // fp16 instructions: correctly rounded, hence equal to torch's fp32 operation rounded back to fp16
    _Float16 r = (_Float16)(float)v;
    r = r * reinterpret_cast<const _Float16*>(a.ep_sw)[m];
    r = r * *reinterpret_cast<const _Float16*>(a.ep_sa);
    if (a.ep_bias) r = r + reinterpret_cast<const _Float16*>(a.ep_bias)[m];
    __half_raw h; h.data = r;
    return __half(h);
}
// The same with the column's parameters already in registers (a store loop walks rows of fixed columns:
// the parameters are fetched once per column, not once per element), fp16 parameters widened to fp32.
struct ColParams { float sw, bias; };
__device__ __forceinline__ bool f32_params(const int kind) { return kind == BGEMM_OUT_F32_SCALED || kind == BGEMM_OUT_BITS_F32; }
__device__ __forceinline__ float ep_scalar(const int kind, const void* p)
{
    return f32_params(kind) ? *reinterpret_cast<const float*>(p) : __half2float(*reinterpret_cast<const __half*>(p));
}
__device__ __forceinline__ ColParams col_params(const GemmArgs& a, const int64_t m)
{
    ColParams c = {0.f, 0.f};
    if (m < a.M && a.ep_sw) {
        if (f32_params(a.out_kind)) {
            c.sw = reinterpret_cast<const float*>(a.ep_sw)[m];
            if (a.ep_bias) c.bias = reinterpret_cast<const float*>(a.ep_bias)[m];
        } else {
            c.sw = __half2float(reinterpret_cast<const __half*>(a.ep_sw)[m]);
            if (a.ep_bias) c.bias = __half2float(reinterpret_cast<const __half*>(a.ep_bias)[m]);
        }
    }
    return c;
}
__device__ __forceinline__ float scaled_f32(const int v, const ColParams c, const float sa, const bool has_bias)
{
#pragma clang fp contract(off)      // every step rounds by itself, as torch's separate kernels do
    float r = (__half2float(__float2half_rn((float)v)) * c.sw);
    r = (r * sa);
    if (has_bias) r = (r + c.bias);
    return r;
}
// fp16 parameters: every step is one fp16 instruction (v_mul_f16 / v_add_f16), whose result is the correctly rounded
// fp16 value, i.e. what torch's kernels get from an fp32 operation on fp16 values rounded back to fp16 (24 >= 2 * 11 + 2
// significand bits in between).  The steps must not be written as fp32 arithmetic on the widened parameters: the
// compiler turns `half(float(r) * sw)` with an fp32 `sw` into `v_fma_mixlo_f16 r, sw, 0`, and the +0 it adds makes a
// zero accumulator times a negative scale +0 where the multiplication gives -0 (one output in 80 at K = 1024).
// c.sw, c.bias and sa were widened from fp16, so narrowing them again is exact; the narrowing does not depend on the
// element and leaves a store loop.
__device__ __forceinline__ __half scaled_f16(const int v, const ColParams c, const float sa, const bool has_bias)
{
#pragma clang fp contract(off)      // every step rounds by itself, as torch's separate kernels do
    _Float16 r = (_Float16)(float)v;
    r = r * (_Float16)c.sw;
    r = r * (_Float16)sa;
    if (has_bias) r = r + (_Float16)c.bias;
    __half_raw h; h.data = r;
    return __half(h);
}
// sign bit of half_rn(y - zp) for the bits kinds, y as above
__device__ __forceinline__ unsigned next_sign_bit(const int kind, const int v, const ColParams c, const float sa,
                                                  const bool has_bias, const float zp)
{
#pragma clang fp contract(off)      // every step rounds by itself, as torch's separate kernels do
    const float y = kind == BGEMM_OUT_BITS_F32 ? scaled_f32(v, c, sa, has_bias) : __half2float(scaled_f16(v, c, sa, has_bias));
    return __float_as_uint((y - zp)) >> 31;
}
__host__ __device__ __forceinline__ int out_elem_shift(const int kind) { return (kind == BGEMM_OUT_F16 || kind == BGEMM_OUT_F16_SCALED) ? 1 : 2; }

// Bits kinds: the scaled output is not stored; the next binary layer's operand is, i.e. the sign bit
// of half_rn(y - zp) with y evaluated as above.  The subtraction is exact enough for its sign to
// survive the rounding to fp16, so the sign bit of the fp32 difference is taken.
__device__ __forceinline__ bool bits_kind(const int kind) { return kind >= BGEMM_OUT_BITS_F32; }
__device__ __forceinline__ unsigned next_sign_bit(const GemmArgs& a, const int64_t m, const int v)
{
#pragma clang fp contract(off)      // every step rounds by itself, as torch's separate kernels do
    float d;
    if (a.out_kind == BGEMM_OUT_BITS_F32)
        d = scaled_f32(a, m, v) - (a.ep_zp ? *reinterpret_cast<const float*>(a.ep_zp) : 0.f);
    else
        d = __half2float(scaled_f16(a, m, v)) - (a.ep_zp ? __half2float(*reinterpret_cast<const __half*>(a.ep_zp)) : 0.f);
    return __float_as_uint(d) >> 31;
}
// One word of the tiled output: the 32 lanes of a half-wave hold the bits of columns m32 .. m32 + 31
// (m32 a multiple of 32) of output row n, bit = 0 where the column does not exist.  Every lane of the
// wave calls this; column i lands at bit 31 - i.
__device__ __forceinline__ void store_bits_word(const GemmArgs& a, const int b, const int64_t n, const int64_t m32,
                                                const unsigned bit)
{
    const int lane = threadIdx.x & 63;
    const unsigned long long bal = __ballot(bit != 0);
    const unsigned w = __brev((unsigned)(lane < 32 ? bal : bal >> 32));
    if ((lane & 31) == 0 && n < a.N && m32 < a.M)
        reinterpret_cast<uint32_t*>(a.out)[(int64_t)b * a.strideC + tiled_word_offset(n, m32 >> 5, k_tiles(a.M))] = w;
}

// Final store of one output element (column m of a row whose first element has index row0).
template <int KIND>
__device__ __forceinline__ void store_out_as(const GemmArgs& a, const int64_t row0, const int64_t m, const int v)
{
    if constexpr (KIND == BGEMM_OUT_I32) reinterpret_cast<int*>(a.out)[row0 + m] = v;
    else if constexpr (KIND == BGEMM_OUT_F16) reinterpret_cast<__half*>(a.out)[row0 + m] = __float2half_rn((float)v);
    else if constexpr (KIND == BGEMM_OUT_F32_SCALED) reinterpret_cast<float*>(a.out)[row0 + m] = scaled_f32(a, m, v);
    else reinterpret_cast<__half*>(a.out)[row0 + m] = scaled_f16(a, m, v);
}
__device__ __forceinline__ void store_out(const GemmArgs& a, const int64_t row0, const int64_t m, const int v)
{
    switch (a.out_kind) {
    case BGEMM_OUT_I32: store_out_as<BGEMM_OUT_I32>(a, row0, m, v); break;
    case BGEMM_OUT_F16: store_out_as<BGEMM_OUT_F16>(a, row0, m, v); break;
    case BGEMM_OUT_F32_SCALED: store_out_as<BGEMM_OUT_F32_SCALED>(a, row0, m, v); break;
    default: store_out_as<BGEMM_OUT_F16_SCALED>(a, row0, m, v); break;
    }
}

// Sign-packs two fp16 [rows][K] operands (row stride K) into tiled buffers with one launch.
int pack_sign_pair(const void* srcA, int64_t rowsA, void* dstA, const void* srcB, int64_t rowsB, void* dstB,
                   int64_t K, hipStream_t st, const char* who);

// Kernel families (each in its own translation unit).
int launch_gemm_mfma(const GemmArgs& a, hipStream_t st, bool fp4);
int gemm_mfma_kernel_id(int64_t batch, int64_t M, int64_t N, int64_t KT, int planes, int out_shift, bool fp4);     // BGEMM_KERNEL_MFMA_* by shape
// A ternary operand's two planes on the general kernel's pipelined 128 x 128 tile (two resident blocks per CU): from two
// thirds of a block per CU on 16 K-tiles or more, except between one block per CU and one and two thirds, which would
// leave the launch waiting for the CUs that run two, and only where most of the tiles land on real outputs.
static inline bool two_plane_tile_128(int64_t batch, int64_t M, int64_t N, int64_t KT)
{
    const int64_t b = batch * cdiv(N, 128) * cdiv(M, 128);
    const double filled = (double)(N * M) / (double)(cdiv(N, 128) * 128 * cdiv(M, 128) * 128);
    return KT >= 16 && b >= 172 && !(b > 256 && b < 416) && filled >= 0.75;
}
int gemm_skinny_kernel_id(const GemmArgs& a, bool fp4);                                   // BGEMM_KERNEL_SKINNY_* by shape
int launch_gemm_valu(const GemmArgs& a, hipStream_t st);
// Skinny shapes (few activation rows): K is split inside the block, no workspace.
bool gemm_skinny_shape(int planes, int64_t batch, int64_t M, int64_t N, int64_t K);
bool gemm_skinny_fusex_shape(int planes, int64_t M, int64_t N);
int launch_gemm_skinny(const GemmArgs& a, hipStream_t st, bool fp4);
// Split-K needs of each family for a shape: bytes of partial-tile scratch, number of counters.
// (for the split that will actually be used: zero when the shape is not split at all)
void gemm_valu_ws(int64_t batch, int64_t M, int64_t N, int64_t K, int splitK, int planes, size_t* part_bytes, size_t* counters);

}  // namespace bgemm
