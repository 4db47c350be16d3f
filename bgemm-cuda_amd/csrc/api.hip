// C ABI: argument checking, workspace carving, variant dispatch.
#include "common.h"
#include <string.h>
#include <mutex>

namespace bgemm {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what)
{
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(BGEMM_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
    return BGEMM_OK;
}

static size_t round256(size_t x) { return (x + 255) / 256 * 256; }

// Shape policy.  The matrix-core path wins whenever there is enough work per weight tile to
// amortise the bit expansion; the fp4 engine runs at twice the int8 rate.
static int pick_variant(int mode, int64_t batch, int64_t M, int64_t N, int64_t K)
{
    (void)mode; (void)batch; (void)M; (void)N; (void)K;
    return BGEMM_VARIANT_MFMA_F4;
}

// `variant` = kernel family in the low byte, BGEMM_FORCE_KERNEL(id) above it.
static bool split_variant(int variant, int* family, int* force)
{
    *family = variant & 0xff;
    *force = (variant >> 8) - 1;
    if (variant < 0 || (variant >> 16) || *family > BGEMM_VARIANT_MFMA_F4) return false;
    if (*force < 0) return true;
    if (*family == BGEMM_VARIANT_VALU) return false;
    switch (*force) {
    case BGEMM_KERNEL_MFMA_256x256: case BGEMM_KERNEL_MFMA_128x128: case BGEMM_KERNEL_MFMA_64x128:
    case BGEMM_KERNEL_MFMA_32x128: case BGEMM_KERNEL_MFMA_256x128: case BGEMM_KERNEL_MFMA_32x256: case BGEMM_KERNEL_MFMA_64x64:
    case BGEMM_KERNEL_MFMA_128x64: case BGEMM_KERNEL_MFMA_128x256T: case BGEMM_KERNEL_SKINNY_STREAM: case BGEMM_KERNEL_SKINNY_SPLITK:
    case BGEMM_KERNEL_SKINNY_QUAD: case BGEMM_KERNEL_SKINNY_POPC: return true;
    default: return false;
    }
}

static void ws_needs(int variant, int planes, int64_t batch, int64_t M, int64_t N, int64_t K, int splitK,
                     size_t* part, size_t* counters)
{
    // Only the VALU family splits K across blocks.  The matrix-core family splits K among the waves of a block
    // for outputs of few tiles (gemm_skinny_shape) and not at all for the rest, which fill the chip without.
    *part = *counters = 0;
    if (variant == BGEMM_VARIANT_VALU) gemm_valu_ws(batch, M, N, K, splitK, planes, part, counters);
}

// one thread per counter
__global__ void clear_counters_kernel(uint32_t* c, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) c[i] = 0u;
}

}  // namespace bgemm

using namespace bgemm;

extern "C" const char* bgemm_last_error(void) { return g_err; }
extern "C" int bgemm_abi_version(void) { return 10; }

static bool ws_query(int mode, int64_t batch, int64_t M, int64_t N, int64_t K, int splitK, int variant,
                     size_t* part, size_t* counters)
{
    ModeCoef mc;
    *part = *counters = 0;
    if (!mode_coef(mode, &mc) || splitK <= 1 || batch <= 0 || M <= 0 || N <= 0 || K <= 0) return false;
    int family, force;
    if (!split_variant(variant, &family, &force)) return false;
    const int v = family == BGEMM_VARIANT_AUTO ? pick_variant(mode, batch, M, N, K) : family;
    ws_needs(v, mc.planes, batch, M, N, K, splitK, part, counters);
    return true;
}

extern "C" size_t bgemm_packed_workspace_bytes(int mode, int64_t batch, int64_t M, int64_t N, int64_t K,
                                               int splitK, int variant)
{
    size_t part, cnt;
    ws_query(mode, batch, M, N, K, splitK, variant, &part, &cnt);
    return round256(part);
}

extern "C" size_t bgemm_packed_counter_bytes(int mode, int64_t batch, int64_t M, int64_t N, int64_t K,
                                             int splitK, int variant)
{
    size_t part, cnt;
    ws_query(mode, batch, M, N, K, splitK, variant, &part, &cnt);
    return round256(cnt * 4);
}

// Fills a whole [batch][N][M] output with one value per column: what every mode gives for K = 0
// (an empty sum), after the output kind's scaling.  A kernel rather than a memset node, so the
// call can be captured in a HIP graph.
__global__ void fill_empty_sum_kernel(const GemmArgs a)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= a.N * a.M) return;
    for (int64_t b = blockIdx.y; b < a.batch; b += gridDim.y) store_out(a, b * a.strideC + (i / a.M) * a.M, i % a.M, 0);
}

// K = 0 with a bits kind: one thread per output word, the 32 columns in turn.
__global__ void fill_empty_bits_kernel(const GemmArgs a)
{
    const int64_t Mw = cdiv(a.M, 32), i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= a.N * Mw) return;
    const int64_t n = i / Mw, jw = i % Mw;
    unsigned w = 0;
    for (int c = 0; c < 32; c++)
        if (jw * 32 + c < a.M) w |= next_sign_bit(a, jw * 32 + c, 0) << (31 - c);
    for (int64_t b = blockIdx.y; b < a.batch; b += gridDim.y)
        reinterpret_cast<uint32_t*>(a.out)[b * a.strideC + tiled_word_offset(n, jw, k_tiles(a.M))] = w;
}

// Unpacked activations for the decode kernel that packs them itself (null = X_tiled / X2_tiled are used).
struct RawActivations { const void* src; int f32; int64_t ld; const void* zero_point; };
// Row popcounts the caller brings for both operands (one bit plane), or null.
struct RowCounts { const void* w; const void* x; };

static int packed_forward(int mode, const void* W_tiled, const void* X_tiled, const void* X2_tiled,
                          void* out, int out_dtype, int64_t batch, int64_t M, int64_t N, int64_t K,
                          int64_t strideW, int64_t strideX, int64_t strideC,
                          int splitK, int variant, void* ws, size_t ws_bytes,
                          void* counters, size_t counter_bytes,
                          const void* sw, const void* sa, const void* bias, const void* zp, void* stream,
                          const RawActivations* raw = nullptr, const bool kernel_id_only = false,
                          const RowCounts* counts = nullptr)
{
    g_err[0] = 0;
    GemmArgs a;
    memset(&a, 0, sizeof a);
    if (!mode_coef(mode, &a.mc)) return fail(BGEMM_EINVAL, "bgemm_packed_forward: unknown mode %d", mode);
    if (out_dtype < BGEMM_OUT_I32 || out_dtype > BGEMM_OUT_BITS_F16)
        return fail(BGEMM_EINVAL, "bgemm_packed_forward: unknown output dtype %d", out_dtype);
    const bool bits = out_dtype == BGEMM_OUT_BITS_F32 || out_dtype == BGEMM_OUT_BITS_F16;
    const bool scaled = bits || out_dtype == BGEMM_OUT_F32_SCALED || out_dtype == BGEMM_OUT_F16_SCALED;
    int family, force;
    if (!split_variant(variant, &family, &force))
        return fail(BGEMM_EINVAL, "bgemm_packed_forward: unknown variant %d", variant);
    if (batch < 0 || M < 0 || N < 0 || K < 0 || splitK < 1 || splitK > 65535)
        return fail(BGEMM_EINVAL, "bgemm_packed_forward: bad shape batch=%lld M=%lld N=%lld K=%lld splitK=%d",
                    (long long)batch, (long long)M, (long long)N, (long long)K, splitK);
    if (K >= (1LL << 24))   // keeps |C| below 2^24: exact in fp32 (fp16 store, fp4 engine accumulator)
        return fail(BGEMM_EINVAL, "bgemm_packed_forward: K=%lld exceeds 2^24-1", (long long)K);
    if (batch > 0x7fffffff || M > 0x7fffffff || N > 0x7fffffff)
        return fail(BGEMM_EINVAL, "bgemm_packed_forward: dimension too large");
    if (strideW < 0 || strideX < 0 || strideC < 0 || (strideW & 3) || (strideX & 3))
        return fail(BGEMM_EINVAL, "bgemm_packed_forward: operand strides must be non-negative multiples of 4 words");
    if (batch == 0 || M == 0 || N == 0)
        return kernel_id_only ? fail(BGEMM_EINVAL, "bgemm_packed_kernel_id: an empty output runs no kernel") : BGEMM_OK;
    if (!out) return fail(BGEMM_ENULL, "bgemm_packed_forward: out is NULL");
    if (scaled && (!sw || !sa)) return fail(BGEMM_ENULL, "bgemm_packed_forward_scaled: sw or sa is NULL");
    if (batch > 1 && strideC < (bits ? bgemm_tiled_words(N, M) : M * N))
        return fail(BGEMM_EINVAL, "bgemm_packed_forward: output stride %lld smaller than one output", (long long)strideC);
    if (bits && ((uintptr_t)out & 3)) return fail(BGEMM_EALIGN, "bgemm_packed_forward_bits: output not 4-byte aligned");
    if (!bits && ((uintptr_t)out & ((1u << out_elem_shift(out_dtype)) - 1)))
        return fail(BGEMM_EALIGN, "bgemm_packed_forward: output not aligned to its element size");
    a.out = out; a.out_kind = out_dtype;
    a.ep_sw = sw; a.ep_sa = sa; a.ep_bias = bias; a.ep_zp = zp;
    a.M = M; a.N = N; a.K = K;
    a.strideC = strideC;
    a.batch = (int)batch;
    a.force = force;
    if (K == 0) {   // empty sum: every mode gives 0
        if (cdiv(N * M, 256) > 0x7fffffffLL) return fail(BGEMM_EINVAL, "bgemm_packed_forward: output too large");
        const unsigned gy = (unsigned)(batch < 65535 ? batch : 65535);      // the kernels walk the rest of the batch
        if (kernel_id_only) return fail(BGEMM_EINVAL, "bgemm_packed_kernel_id: K = 0 runs no GEMM kernel");
        if (bits)
            hipLaunchKernelGGL(fill_empty_bits_kernel, dim3((unsigned)cdiv(N * cdiv(M, 32), 256), gy), dim3(256), 0,
                               (hipStream_t)stream, a);
        else
            hipLaunchKernelGGL(fill_empty_sum_kernel, dim3((unsigned)cdiv(N * M, 256), gy), dim3(256), 0,
                               (hipStream_t)stream, a);
        return check_launch("bgemm_packed_forward: fill");
    }
    if (raw) {
        if (!W_tiled || !raw->src) return fail(BGEMM_ENULL, "bgemm_packed_weight_forward: operand pointer is NULL");
        if (raw->ld < K) return fail(BGEMM_EINVAL, "bgemm_packed_weight_forward: row stride %lld < K", (long long)raw->ld);
        if (batch != 1 || !gemm_skinny_fusex_shape(a.mc.planes, M, N) || family == BGEMM_VARIANT_VALU)
            return fail(BGEMM_EINVAL, "bgemm_packed_weight_forward: shape M=%lld N=%lld not taken by the decode kernel "
                                      "(see bgemm_packed_weight_forward_supported)", (long long)M, (long long)N);
        if ((uintptr_t)raw->src & (raw->f32 ? 3 : 1))
            return fail(BGEMM_EALIGN, "bgemm_packed_weight_forward: activations not aligned to their element size");
        a.xsrc = raw->src; a.xsrc_f32 = raw->f32; a.xld = raw->ld; a.xzp = raw->zero_point;
    } else if (!W_tiled || !X_tiled || (a.mc.planes == 2 && !X2_tiled))
        return fail(BGEMM_ENULL, "bgemm_packed_forward: operand pointer is NULL");
    if (((uintptr_t)W_tiled & 15) || ((uintptr_t)X_tiled & 15) || ((uintptr_t)X2_tiled & 15))
        return fail(BGEMM_EALIGN, "bgemm_packed_forward: operands must be 16-byte aligned");

    if (counts) {
        if (!counts->w || !counts->x) return fail(BGEMM_ENULL, "bgemm_packed_forward_counted: a count array is NULL");
        if (((uintptr_t)counts->w & 3) || ((uintptr_t)counts->x & 3))
            return fail(BGEMM_EALIGN, "bgemm_packed_forward_counted: count arrays must be 4-byte aligned");
        if (a.mc.planes != 1) return fail(BGEMM_EINVAL, "bgemm_packed_forward_counted: modes of one bit plane only");
        a.cntW = (const int32_t*)counts->w; a.cntX = (const int32_t*)counts->x;
    }
    a.W = (const uint4*)W_tiled; a.X = (const uint4*)X_tiled; a.X2 = (const uint4*)X2_tiled;
    a.MT = (int)row_tiles(M); a.NT = (int)row_tiles(N); a.KT = (int)k_tiles(K);
    a.strideW = strideW / 4; a.strideX = strideX / 4;
    a.splitK = splitK;
    a.vec_store = !bits && (M % 4 == 0) && (strideC % 4 == 0) && (((uintptr_t)out & 15) == 0) ? 4 : 0;
    if (a.vec_store && out_elem_shift(a.out_kind) == 1 && M % 8 == 0 && strideC % 8 == 0) a.vec_store = 8;
    a.nt_store = batch * N * M * 4 <= (32LL << 20);
    const int v = family == BGEMM_VARIANT_AUTO ? pick_variant(mode, batch, M, N, K) : family;
    const bool fp4 = v == BGEMM_VARIANT_MFMA_F4;
    if (raw) {
        if (force >= 0 && force < BGEMM_KERNEL_SKINNY_STREAM)
            return fail(BGEMM_EINVAL, "bgemm_packed_weight_forward: kernel %d does not pack activations", force);
        return launch_gemm_skinny(a, (hipStream_t)stream, fp4);
    }
    const bool skinny = force >= 0 ? force >= BGEMM_KERNEL_SKINNY_STREAM
                                   : v != BGEMM_VARIANT_VALU && gemm_skinny_shape(a.mc.planes, batch, M, N, K);
    if (skinny && batch > 65535)
        return fail(BGEMM_EINVAL, "bgemm_packed_forward: the decode kernels take batches of up to 65535");
    if (kernel_id_only)
        return v == BGEMM_VARIANT_VALU ? BGEMM_KERNEL_VALU
               : force >= 0            ? force
               : skinny                ? gemm_skinny_kernel_id(a, fp4)
                                       : gemm_mfma_kernel_id(batch, M, N, a.KT, a.mc.planes, out_elem_shift(a.out_kind), fp4);
    if (splitK > 1 && v == BGEMM_VARIANT_VALU) {
        size_t part, cnt;
        ws_needs(v, a.mc.planes, batch, M, N, K, splitK, &part, &cnt);
        if (part) {       // this shape will really be split (splitK is an upper bound)
            if (!ws || !counters)
                return fail(BGEMM_EWORKSPACE, "bgemm_packed_forward: splitK=%d needs %zu workspace and %zu counter bytes",
                            splitK, round256(part), round256(cnt * 4));
            if (ws_bytes < part) return fail(BGEMM_EWORKSPACE, "bgemm_packed_forward: workspace %zu < %zu bytes", ws_bytes, part);
            if (counter_bytes < cnt * 4)
                return fail(BGEMM_EWORKSPACE, "bgemm_packed_forward: counters %zu < %zu bytes", counter_bytes, cnt * 4);
            if (((uintptr_t)ws & 15) || ((uintptr_t)counters & 3))
                return fail(BGEMM_EALIGN, "bgemm_packed_forward: workspace must be 16-byte aligned");
            a.ws_part = (int32_t*)ws;
            a.ws_cnt = (uint32_t*)counters;
        }
    }
    if (v == BGEMM_VARIANT_VALU) return launch_gemm_valu(a, (hipStream_t)stream);
    if (skinny) return launch_gemm_skinny(a, (hipStream_t)stream, fp4);
    return launch_gemm_mfma(a, (hipStream_t)stream, fp4);
}

extern "C" int bgemm_packed_kernel_id(int mode, int out_dtype, int64_t batch, int64_t M, int64_t N, int64_t K, int splitK,
                                      int variant)
{
    // the same checks and the same choice as a call, with stand-in pointers that are never dereferenced
    // and a workspace that is never too small
    alignas(16) static char stand_in[16];
    return packed_forward(mode, stand_in, stand_in, stand_in, stand_in, out_dtype, batch, M, N, K, 0, 0, M * N,
                          splitK, variant, stand_in, (size_t)-1, stand_in, (size_t)-1, stand_in, stand_in, nullptr, nullptr,
                          nullptr, nullptr, true);
}

extern "C" int bgemm_packed_forward(int mode, const void* W_tiled, const void* X_tiled, const void* X2_tiled,
                                    void* out, int out_dtype, int64_t batch, int64_t M, int64_t N, int64_t K,
                                    int64_t strideW, int64_t strideX, int64_t strideC,
                                    int splitK, int variant, void* ws, size_t ws_bytes,
                                    void* counters, size_t counter_bytes, void* stream)
{
    if (out_dtype != BGEMM_OUT_I32 && out_dtype != BGEMM_OUT_F16)
        return fail(BGEMM_EINVAL, "bgemm_packed_forward: unknown output dtype %d", out_dtype);
    return packed_forward(mode, W_tiled, X_tiled, X2_tiled, out, out_dtype, batch, M, N, K, strideW, strideX, strideC,
                          splitK, variant, ws, ws_bytes, counters, counter_bytes, nullptr, nullptr, nullptr, nullptr, stream);
}

extern "C" int bgemm_packed_forward_counted(int mode, const void* W_tiled, const void* X_tiled, const void* W_counts,
                                            const void* X_counts, void* out, int out_dtype, int64_t batch, int64_t M,
                                            int64_t N, int64_t K, int64_t strideW, int64_t strideX, int64_t strideC,
                                            int variant, void* stream)
{
    if (out_dtype != BGEMM_OUT_I32 && out_dtype != BGEMM_OUT_F16)
        return fail(BGEMM_EINVAL, "bgemm_packed_forward_counted: unknown output dtype %d", out_dtype);
    int family, force;
    if (split_variant(variant, &family, &force) && family == BGEMM_VARIANT_VALU)
        return fail(BGEMM_EINVAL, "bgemm_packed_forward_counted: the matrix-core kernels only");
    const RowCounts counts = {W_counts, X_counts};
    return packed_forward(mode, W_tiled, X_tiled, nullptr, out, out_dtype, batch, M, N, K, strideW, strideX, strideC, 1,
                          variant, nullptr, 0, nullptr, 0, nullptr, nullptr, nullptr, nullptr, stream, nullptr, false, &counts);
}

extern "C" int bgemm_packed_forward_scaled(int mode, const void* W_tiled, const void* X_tiled, const void* X2_tiled,
                                           void* out, int out_dtype, int64_t batch, int64_t M, int64_t N, int64_t K,
                                           int64_t strideW, int64_t strideX, int64_t strideC,
                                           int splitK, int variant, void* ws, size_t ws_bytes,
                                           void* counters, size_t counter_bytes,
                                           const void* sw, const void* sa, const void* bias, void* stream)
{
    if (out_dtype != BGEMM_OUT_F32_SCALED && out_dtype != BGEMM_OUT_F16_SCALED)
        return fail(BGEMM_EINVAL, "bgemm_packed_forward_scaled: output dtype must be BGEMM_OUT_F32_SCALED or "
                                  "BGEMM_OUT_F16_SCALED, got %d", out_dtype);
    return packed_forward(mode, W_tiled, X_tiled, X2_tiled, out, out_dtype, batch, M, N, K, strideW, strideX, strideC,
                          splitK, variant, ws, ws_bytes, counters, counter_bytes, sw, sa, bias, nullptr, stream);
}

extern "C" int bgemm_packed_forward_bits(int mode, const void* W_tiled, const void* X_tiled, const void* X2_tiled,
                                         void* out_tiled, int out_dtype, int64_t batch, int64_t M, int64_t N, int64_t K,
                                         int64_t strideW, int64_t strideX, int64_t strideOut,
                                         int splitK, int variant, void* ws, size_t ws_bytes,
                                         void* counters, size_t counter_bytes,
                                         const void* sw, const void* sa, const void* bias, const void* zero_point,
                                         void* stream)
{
    if (out_dtype != BGEMM_OUT_BITS_F32 && out_dtype != BGEMM_OUT_BITS_F16)
        return fail(BGEMM_EINVAL, "bgemm_packed_forward_bits: output dtype must be BGEMM_OUT_BITS_F32 or "
                                  "BGEMM_OUT_BITS_F16, got %d", out_dtype);
    return packed_forward(mode, W_tiled, X_tiled, X2_tiled, out_tiled, out_dtype, batch, M, N, K, strideW, strideX,
                          strideOut, splitK, variant, ws, ws_bytes, counters, counter_bytes, sw, sa, bias, zero_point, stream);
}

extern "C" int bgemm_packed_weight_forward_supported(int mode, int64_t M, int64_t N, int64_t K)
{
    ModeCoef mc;
    return mode_coef(mode, &mc) && M >= 1 && K >= 1 && K < (1LL << 24) && gemm_skinny_fusex_shape(mc.planes, M, N);
}

extern "C" int bgemm_packed_weight_forward(int mode, const void* W_tiled, const void* x, int x_dtype, int64_t ldx,
                                           const void* x_zero_point, void* out, int out_dtype,
                                           int64_t M, int64_t N, int64_t K, int variant,
                                           const void* sw, const void* sa, const void* bias,
                                           const void* next_zero_point, void* stream)
{
    if (x_dtype != BGEMM_SRC_F16 && x_dtype != BGEMM_SRC_F32)
        return fail(BGEMM_EINVAL, "bgemm_packed_weight_forward: unknown activation type %d", x_dtype);
    if (K == 0 || M == 0 || N == 0)      // nothing to pack: the packed entry point's empty cases
        return packed_forward(mode, W_tiled, nullptr, nullptr, out, out_dtype, 1, M, N, K, 0, 0, 0, 1, variant, nullptr, 0,
                              nullptr, 0, sw, sa, bias, next_zero_point, stream);
    const RawActivations raw = {x, x_dtype == BGEMM_SRC_F32, ldx, x_zero_point};
    return packed_forward(mode, W_tiled, nullptr, nullptr, out, out_dtype, 1, M, N, K, 0, 0, 0, 1, variant, nullptr, 0,
                          nullptr, 0, sw, sa, bias, next_zero_point, stream, &raw);
}

// ---- fp16-operand call: pack both operands into the workspace, then the packed GEMM ----
// Workspace layout: [counters] [partial tiles] [W tiled] [X tiled], each rounded to 256 bytes.
extern "C" size_t bgemm_f16_workspace_bytes(int64_t M, int64_t N, int64_t K, int splitK)
{
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    return bgemm_packed_counter_bytes(BGEMM_MODE_XOR, 1, M, N, K, splitK, BGEMM_VARIANT_AUTO) +
           bgemm_packed_workspace_bytes(BGEMM_MODE_XOR, 1, M, N, K, splitK, BGEMM_VARIANT_AUTO) +
           round256((size_t)bgemm_tiled_words(M, K) * 4) + round256((size_t)bgemm_tiled_words(N, K) * 4);
}

extern "C" int bgemm_f16_forward(const void* W, const void* X, void* C, int64_t M, int64_t N, int64_t K,
                                 void* ws, size_t ws_bytes, int splitK, int INSTR, void* stream)
{
    g_err[0] = 0;
    if (INSTR < BGEMM_MODE_AND || INSTR > BGEMM_MODE_ATTN)
        return fail(BGEMM_EINVAL, "bgemm_f16_forward: INSTR must be 0 (and), 1 (xor) or 2 (attn), got %d", INSTR);
    if (M < 0 || N < 0 || K < 0 || splitK < 1)
        return fail(BGEMM_EINVAL, "bgemm_f16_forward: bad shape M=%lld N=%lld K=%lld splitK=%d", (long long)M,
                    (long long)N, (long long)K, splitK);
    if (M == 0 || N == 0) return BGEMM_OK;
    if (!C) return fail(BGEMM_ENULL, "bgemm_f16_forward: C is NULL");
    if (K == 0)
        return bgemm_packed_forward(INSTR, nullptr, nullptr, nullptr, C, BGEMM_OUT_F16, 1, M, N, 0, 0, 0, 0, 1,
                                    BGEMM_VARIANT_AUTO, nullptr, 0, nullptr, 0, stream);
    if (!W || !X) return fail(BGEMM_ENULL, "bgemm_f16_forward: operand pointer is NULL");
    const size_t need = bgemm_f16_workspace_bytes(M, N, K, splitK);
    if (!ws || ws_bytes < need)
        return fail(BGEMM_EWORKSPACE, "bgemm_f16_forward: workspace of %zu bytes required, %zu given", need,
                    ws ? ws_bytes : (size_t)0);
    if ((uintptr_t)ws & 255) return fail(BGEMM_EALIGN, "bgemm_f16_forward: workspace must be 256-byte aligned");
    const size_t cb = bgemm_packed_counter_bytes(INSTR, 1, M, N, K, splitK, BGEMM_VARIANT_AUTO);
    const size_t pb = bgemm_packed_workspace_bytes(INSTR, 1, M, N, K, splitK, BGEMM_VARIANT_AUTO);
    char* cnt = (char*)ws;
    char* part = cnt + cb;
    char* wt = part + pb;
    char* xt = wt + round256((size_t)bgemm_tiled_words(M, K) * 4);
    if (cb) {   // a fill kernel rather than a memset node, so the call can be captured in a HIP graph
        const int64_t n = (int64_t)(cb / 4);
        hipLaunchKernelGGL(clear_counters_kernel, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, (hipStream_t)stream,
                           (uint32_t*)cnt, n);
        int rc = check_launch("bgemm_f16_forward: clear counters");
        if (rc) return rc;
    }
    int rc = pack_sign_pair(W, M, wt, X, N, xt, K, (hipStream_t)stream, "bgemm_f16_forward: pack");
    if (rc) return rc;
    return bgemm_packed_forward(INSTR, wt, xt, nullptr, C, BGEMM_OUT_F16, 1, M, N, K, 0, 0, 0, splitK,
                                BGEMM_VARIANT_AUTO, part, pb, cnt, cb, stream);
}

// ---- the same call for callers that cannot allocate -------------------------------------------
// The workspace of bgemm_f16_forward (the two packed operands, split-K state) lives in a device array of the
// library's own instead of a buffer the caller brings.  Every GPU holds its own copy of the array at its own
// address; the array's name is only a host-side handle for hipGetSymbolAddress, never an address itself.
static __device__ __align__(256) unsigned char scratch[BGEMM_STATIC_SCRATCH_BYTES];

static int static_scratch(void** ptr)
{
    constexpr int MAX_DEVICES = 64;
    static std::mutex mu;
    static void* per_device[MAX_DEVICES] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(BGEMM_ELAUNCH, "bgemm_f16_forward_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= MAX_DEVICES) return fail(BGEMM_EINVAL, "bgemm_f16_forward_static: device %d out of range", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!per_device[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));       // the address of THIS device's copy
        if (e != hipSuccess || !p)
            return fail(BGEMM_ELAUNCH, "bgemm_f16_forward_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        per_device[dev] = p;
    }
    *ptr = per_device[dev];
    return BGEMM_OK;
}

extern "C" int bgemm_f16_forward_static(const void* W, const void* X, void* C, int64_t M, int64_t N, int64_t K,
                                        int splitK, int INSTR, void* stream)
{
    g_err[0] = 0;
    if (M < 0 || N < 0 || K < 0 || splitK < 1)
        return fail(BGEMM_EINVAL, "bgemm_f16_forward_static: bad shape M=%lld N=%lld K=%lld splitK=%d", (long long)M,
                    (long long)N, (long long)K, splitK);
    const size_t need = bgemm_f16_workspace_bytes(M, N, K, splitK);
    if (need > (size_t)BGEMM_STATIC_SCRATCH_BYTES)
        return fail(BGEMM_EWORKSPACE, "bgemm_f16_forward_static: M=%lld N=%lld K=%lld needs %zu bytes of scratch, the "
                                      "library's own array holds %zu: use bgemm_f16_forward with a workspace",
                    (long long)M, (long long)N, (long long)K, need, (size_t)BGEMM_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    if (need) {     // (an empty problem touches no scratch and needs no device)
        const int rc = static_scratch(&ws);
        if (rc) return rc;
    }
    // Nothing in the scratch has to start at zero: the pack kernels write whole tiles, padding included, and
    // the call clears the split-K counters it uses (with a kernel, not a memset node) before the GEMM.
    return bgemm_f16_forward(W, X, C, M, N, K, ws, need ? (size_t)BGEMM_STATIC_SCRATCH_BYTES : 0, splitK, INSTR, stream);
}
