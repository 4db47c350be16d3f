/*
 * bgemm_mi355x.h -- C ABI of the MI355X (gfx950) binary-GEMM library.
 *
 * Plain C, plain pointers and sizes: no torch, no C++ types.  Every entry point is
 * asynchronous on the HIP stream it is given (NULL = the null stream), never
 * allocates or frees device memory, keeps no global state apart from a
 * thread-local error string, and returns 0 or a negative BGEMM_E* code.
 * All device pointers are borrowed for the duration of the enqueued work.
 *
 * Citations name the reference interface each entry point stands in for
 * (paths relative to the reference tree).
 *
 * Operand semantics (reference: lowbit_kernel/csrc/include/utils_core.cuh:242-303,
 * ptx_mma.cuh:196-250,299-336).  With a = sign bit of the weight-side element,
 * b = sign bit of the activation-side element (1 = negative, -0.0 included):
 *   BGEMM_MODE_AND   C[n,m] = #{k : a=1 and b=1}
 *   BGEMM_MODE_XOR   C[n,m] = K - 2*#{k : a != b}            ({-1,1} x {-1,1})
 *   BGEMM_MODE_ATTN  C[n,m] = sum_k (1-a)(1-2b)              ({0,1} weight side x {-1,1})
 *   BGEMM_MODE_BWTA  C[n,m] = sum_k t(1-2a), t in {-1,0,1} given as two planes
 *                    (nonzero, sign&nonzero) on the activation side
 *   BGEMM_MODE_ATTN_X  as ATTN with the roles swapped: {0,1} on the activation side
 * The output is row-major [N][M] (kernel_matmul.cuh:534-545), int32 or fp16 where
 * fp16 = the exact integer rounded to nearest even (kernel_matmul.cuh:540).
 */
#ifndef BGEMM_MI355X_H
#define BGEMM_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* INSTR values 0..2 are the reference's API (configs.h:70-72); 3 and 4 are supersets. */
enum { BGEMM_MODE_AND = 0, BGEMM_MODE_XOR = 1, BGEMM_MODE_ATTN = 2, BGEMM_MODE_BWTA = 3,
       BGEMM_MODE_ATTN_X = 4 };
/* Output kinds.  I32 = the accumulator; F16 = the integer rounded to nearest even.
 * F32_SCALED / F16_SCALED = the binary Linear's scaling fused into the store (see
 * bgemm_packed_forward_scaled): fp32 resp. fp16 output, parameters of the same type. */
enum { BGEMM_OUT_I32 = 0, BGEMM_OUT_F16 = 1, BGEMM_OUT_F32_SCALED = 2, BGEMM_OUT_F16_SCALED = 3,
       /* the scaled value's sign bit after the next layer's centring, written as a tiled operand
        * (see bgemm_packed_forward_bits); parameters fp32 resp. fp16 */
       BGEMM_OUT_BITS_F32 = 4, BGEMM_OUT_BITS_F16 = 5 };
/* Element type of a floating-point source operand. */
enum { BGEMM_SRC_F16 = 0, BGEMM_SRC_F32 = 1 };
/* Kernel family: AUTO picks per shape; VALU = and + popcount on the vector ALU;
 * MFMA = bit planes expanded to int8 in registers feeding v_mfma_i32_32x32x32_i8;
 * MFMA_F4 = bit planes expanded to E2M1 nibbles feeding v_mfma_f32_32x32x64_f8f6f4
 * (products are 0/1 and the fp32 accumulator stays below 2^24, so it is exact too). */
enum { BGEMM_VARIANT_AUTO = 0, BGEMM_VARIANT_VALU = 1, BGEMM_VARIANT_MFMA = 2, BGEMM_VARIANT_MFMA_F4 = 3 };

/* The kernels behind bgemm_packed_forward*, as bgemm_packed_kernel_id() names them: the general matrix-core
 * kernel by its block tile (activation rows x weight rows), the decode-shaped kernels, the VALU kernel. */
enum { BGEMM_KERNEL_MFMA_256x256 = 0, BGEMM_KERNEL_MFMA_128x128 = 1, BGEMM_KERNEL_MFMA_64x128 = 2,
       BGEMM_KERNEL_MFMA_32x128 = 3, BGEMM_KERNEL_MFMA_256x128 = 4, BGEMM_KERNEL_MFMA_32x256 = 5,
       BGEMM_KERNEL_MFMA_64x64 = 6,
       BGEMM_KERNEL_MFMA_128x64 = 7,
       BGEMM_KERNEL_MFMA_128x256T = 8,   /* ternary activations as signed operands: BGEMM_MODE_BWTA on the fp4 engine only */
       BGEMM_KERNEL_SKINNY_STREAM = 16, BGEMM_KERNEL_SKINNY_SPLITK = 17, BGEMM_KERNEL_SKINNY_QUAD = 18,
       BGEMM_KERNEL_SKINNY_POPC = 19,
       BGEMM_KERNEL_VALU = 32 };
/* Test and benchmark aid, OR-ed into a `variant` argument whose family is one of the matrix-core ones (or AUTO):
 * the call runs kernel `id` instead of the one chosen by shape, or returns BGEMM_EINVAL where that kernel
 * cannot take the shape (two bit planes on a tile built for one; the decode kernels beyond their row counts).
 * Results never depend on it. */
#define BGEMM_FORCE_KERNEL(id) (((id) + 1) << 8)

enum {
    BGEMM_OK = 0,
    BGEMM_EINVAL = -1,      /* bad shape, mode, dtype, variant or splitK            */
    BGEMM_ENULL = -2,       /* a required pointer is NULL                            */
    BGEMM_EWORKSPACE = -3,  /* workspace missing or smaller than *_workspace_bytes() */
    BGEMM_ELAUNCH = -4,     /* HIP reported an error at launch                       */
    BGEMM_EALIGN = -5,      /* a pointer is not 16-byte aligned                      */
    BGEMM_ETIMEOUT = -6     /* a chain launch gave up waiting (bgemm_chain_status)   */
};

/* Message for the last error returned on the calling thread ("" if none). */
const char* bgemm_last_error(void);
/* ABI version; bumped when a signature or the tiled layout changes. */
int bgemm_abi_version(void);

/* ---- packed operand layout -------------------------------------------------------
 * "Logical" format = the reference's (weight_prepacking.h:181-230): uint32 [rows][ceil(K/32)],
 * bit (31-i) of word j = sign bit of element 32*j+i, unused tail bits 0.
 * "Tiled" format = what the kernels stream: tiles of 32 rows x 256 K-bits, 1 KiB each,
 * tile (rt, kt) at word offset (rt*KT + kt)*256, inside a tile 64 slots of 16 bytes,
 * slot h*32 + r = logical words 8*kt + 4*h .. +3 of row 32*rt + r.  Rows and K are
 * zero-padded to whole tiles (zero bits contribute nothing in any mode).
 */
/* Number of uint32 words of a tiled operand of `rows` x K bits. */
int64_t bgemm_tiled_words(int64_t rows, int64_t K);

/* fp16 [rows][K] (row stride ld elements) -> tiled sign bits.
 * Replaces the in-kernel sign packing (ptx_mma.cuh:341-380) and the host routine
 * bin_matrix_prepacking_to_uint32 (weight_prepacking.h:203-230); this is the weight
 * prepack entry point that binary_weight_prepacking_cuda (fp6_linear.cu:519-542) stubs. */
int bgemm_pack_sign_f16(const void* src, int64_t rows, int64_t K, int64_t ld,
                        void* dst_tiled, void* stream);
/* fp16 -> logical format exactly as weight_prepacking.h:181-230 defines it. */
int bgemm_pack_sign_f16_logical(const void* src, int64_t rows, int64_t K, int64_t ld,
                                uint32_t* dst_logical, void* stream);
/* fp16 -> two tiled planes: nonzero, and sign&nonzero (ternary = torch.sign,
 * tests/python/bgemm_linear.py:222-241). */
int bgemm_pack_ternary_f16(const void* src, int64_t rows, int64_t K, int64_t ld,
                           void* nz_tiled, void* sg_tiled, void* stream);
/* Centre-and-pack in one pass: bit = sign bit of half_rn(src[r][k] - *zero_point), the
 * operand the binary Linear layers hand to the kernel (tests/python/bgemm_linear.py:479-482:
 * `x - zpa` resp. `weight - zpw`, then `.to(torch.half)`, then the sign pack of
 * ptx_mma.cuh:341-380).  src is fp16 or fp32 (BGEMM_SRC_*) with row stride ld elements;
 * zero_point is a DEVICE pointer to one scalar of the source type (so a zero point that
 * was computed on the GPU needs no host read-back), or NULL for 0. */
int bgemm_pack_sign_centered(const void* src, int src_dtype, int64_t rows, int64_t K, int64_t ld,
                             const void* zero_point, void* dst_tiled, void* stream);
/* Sign pack of the TRANSPOSE of a batch of fp16 matrices: src holds `batch` matrices of
 * [K][rows] (element (k, r) at src[b*src_batch_stride + k*ld + r]); matrix b of the result
 * is the tiled operand of `rows` x K bits at dst_tiled + b*bgemm_tiled_words(rows, K) words.
 * The right-hand operand of `matA @ matB` (tests/python/bgemm_linear.py:19-25) and the value
 * operand of `attn @ value` (:55-60), which the reference brings into [rows][K] order with
 * `.transpose(0, 1).contiguous()` before its kernel can read it, are packed as they lie. */
int bgemm_pack_sign_f16_transposed(const void* src, int64_t batch, int64_t rows, int64_t K, int64_t ld,
                                   int64_t src_batch_stride, void* dst_tiled, void* stream);
/* The pack entry points above over a batch of batch_outer x batch_inner matrices in one launch, each of
 * `rows` x K elements with rows ld elements apart; matrix (o, i) starts stride_outer*o + stride_inner*i
 * elements into src and its tiled operand is written bgemm_tiled_words(rows, K) words after the one before it
 * (o-major).  This reads the [B, H, S, d] views attention works on where they lie, e.g. the
 * `permute(0, 2, 1, 3)` view of a [B, S, H*d] projection (tests/python/bert/bert.py:216-220: strides S*H*d, d
 * and row stride H*d), for which the reference's 2-D kernel call needs a `.contiguous()` copy per matrix
 * (tests/python/bgemm_linear.py:25, :60).  src_dtype BGEMM_SRC_F16 or BGEMM_SRC_F32 (an fp32 source is rounded
 * to fp16 first, as `.to(torch.half)` does; the sign bit is the same).  ternary != 0 writes the (nonzero,
 * sign & nonzero) planes to dst0 / dst1, otherwise dst1 is ignored; zero_point as in bgemm_pack_sign_centered
 * (sign pack only), or NULL. */
int bgemm_pack_batched(const void* src, int src_dtype, int ternary, const void* zero_point,
                       int64_t batch_outer, int64_t batch_inner, int64_t rows, int64_t K, int64_t ld,
                       int64_t stride_outer, int64_t stride_inner, void* dst0_tiled, void* dst1_tiled, void* stream);
/* bgemm_pack_sign_f16_transposed over an outer x inner batch, fp16 or fp32 source: element (k, r) of matrix
 * (o, i) is at src[stride_outer*o + stride_inner*i + k*ld + r]. */
int bgemm_pack_transposed_batched(const void* src, int src_dtype, int64_t batch_outer, int64_t batch_inner,
                                  int64_t rows, int64_t K, int64_t ld, int64_t stride_outer, int64_t stride_inner,
                                  void* dst_tiled, void* stream);
/* logical <-> tiled re-layout of already packed bits (device buffers). */
int bgemm_tile_from_logical(const uint32_t* logical, int64_t rows, int64_t K,
                            void* dst_tiled, void* stream);
int bgemm_logical_from_tiled(const void* tiled, int64_t rows, int64_t K,
                             uint32_t* dst_logical, void* stream);

/* ---- GEMM on packed operands -------------------------------------------------------
 * Replaces bin_pack_linear_kernel + SplitK_Reduction (fp6_linear.cu:275-337,
 * kernel_reduction.cuh:29-48) for operands that are already bit-packed.
 *   W_tiled  : weight side, M rows.   X_tiled : activation side, N rows.
 *   X2_tiled : BWTA only, the sign&nonzero plane (X_tiled is the nonzero plane).
 *   batch    : number of independent GEMMs; strides in uint32 words / output elements
 *              (a stride of 0 shares that operand across the batch).
 *   splitK   : >= 1, an upper bound on the number of contiguous K ranges (partitioned as in
 *              kernel_matmul.cuh:397-404) that are reduced inside the same launch with integer
 *              adds, so the result does not depend on it.  K is only split where the output
 *              tiles alone leave compute units idle: the matrix-core kernels then split it
 *              among the waves of a block (no workspace); the VALU family splits it across
 *              blocks while every range stays long enough to pay for the hand-over.
 *   ws       : scratch for split-K partial tiles, bgemm_packed_workspace_bytes() bytes for the
 *              same arguments (0 when the shape will not be split across blocks: always for
 *              BGEMM_VARIANT_AUTO and the matrix-core variants), no initialisation needed
 *              (NULL when that is 0).
 *   counters : split-K arrival counters, bgemm_packed_counter_bytes() bytes.  Must be
 *              zero-filled once before first use; every call leaves them zero again.
 *              Calls that share counters must not overlap in time.
 */
size_t bgemm_packed_workspace_bytes(int mode, int64_t batch, int64_t M, int64_t N, int64_t K,
                                    int splitK, int variant);
size_t bgemm_packed_counter_bytes(int mode, int64_t batch, int64_t M, int64_t N, int64_t K,
                                  int splitK, int variant);
int bgemm_packed_forward(int mode, const void* W_tiled, const void* X_tiled, const void* X2_tiled,
                         void* out, int out_dtype, int64_t batch, int64_t M, int64_t N, int64_t K,
                         int64_t strideW, int64_t strideX, int64_t strideC,
                         int splitK, int variant, void* ws, size_t ws_bytes,
                         void* counters, size_t counter_bytes, void* stream);
/* The kernel (BGEMM_KERNEL_*) the three bgemm_packed_forward* entry points run for these arguments (out_dtype:
 * any BGEMM_OUT_* kind; 2-byte and 4-byte outputs can take different tiles), or a negative BGEMM_E* code for
 * arguments they would reject.  The reference's dispatch is the N-bucket switch
 * of bin_pack_linear_kernel (fp6_linear.cu:292-330), which lands on one tile for every shape; here the
 * choice depends on the shape, and tests and benchmarks ask which kernel they are looking at. */
int bgemm_packed_kernel_id(int mode, int out_dtype, int64_t batch, int64_t M, int64_t N, int64_t K, int splitK,
                           int variant);

/* Row popcounts of a tiled operand, counts[b * rows + r] (int32) = set bits in row r of batch entry b
 * (stride_words between entries; 0 with batch 1).  Every mode but AND needs them for its rank-one terms
 * (bits - 2 popc(a) - 2 popc(b) + 4 popc(a & b) is the XOR form of ptx_mma.cuh:212-250); the kernels count
 * while they multiply unless the caller brings the counts along, below.  They belong to a prepacked operand
 * like its bits: computed once per weight (the reference's weight_prepacking.h has no such field; its kernel
 * re-derives everything per call). */
int bgemm_row_popcounts(const void* tiled, int64_t batch, int64_t rows, int64_t K, int64_t stride_words,
                        void* counts, void* stream);
/* bgemm_packed_forward for the modes of one bit plane, with the row popcounts of both operands supplied
 * (W_counts [batch][M] or [M] when strideW is 0, X_counts likewise): same results; the large tiles leave the
 * counting out of their main loop (a sixth of its vector instructions; 4 % of an 8192^3 launch), the other
 * kernels ignore the counts.  Matrix-core families only; K is never split, no workspace. */
int bgemm_packed_forward_counted(int mode, const void* W_tiled, const void* X_tiled, const void* W_counts,
                                 const void* X_counts, void* out, int out_dtype, int64_t batch, int64_t M,
                                 int64_t N, int64_t K, int64_t strideW, int64_t strideX, int64_t strideC,
                                 int variant, void* stream);

/* The same GEMM with the binary Linear's output scaling fused into the store, replacing the
 * separate elementwise kernels of `bgemm(...) * sw * sa (+ bias)`
 * (tests/python/bgemm_linear.py:482-484).  Every step is evaluated and rounded exactly as
 * torch evaluates that expression: h = fp16_rn(C[n,m]); then, for BGEMM_OUT_F32_SCALED
 * (fp32 parameters, fp32 output) out = (float(h) * sw[m]) * sa + bias[m] in fp32; for
 * BGEMM_OUT_F16_SCALED (fp16 parameters, fp16 output) the same with every step rounded to
 * fp16.  sw: M per-output-channel scales; sa: one scalar; bias: M values or NULL; all are
 * DEVICE pointers of the output's element type. */
int bgemm_packed_forward_scaled(int mode, const void* W_tiled, const void* X_tiled, const void* X2_tiled,
                                void* out, int out_dtype, int64_t batch, int64_t M, int64_t N, int64_t K,
                                int64_t strideW, int64_t strideX, int64_t strideC,
                                int splitK, int variant, void* ws, size_t ws_bytes,
                                void* counters, size_t counter_bytes,
                                const void* sw, const void* sa, const void* bias, void* stream);

/* A binary Linear whose output feeds another binary Linear, with nothing but bits in between: the
 * scaled output y = half(acc) * sw * sa (+ bias) is evaluated as in bgemm_packed_forward_scaled,
 * then centred and sign-packed as the next layer would do it (tests/python/bgemm_linear.py:479-482
 * followed by :140-141 and the pack of ptx_mma.cuh:341-380): bit = sign bit of half_rn(y - *zero_point).
 * out_tiled receives the tiled operand of N rows x M bits (bgemm_tiled_words(N, M) words per batch
 * entry, strideOut words apart).  Only real bits are written: the padding of the last row tile and
 * K-tile must already be zero (zero-fill the buffer once; calls of the same shape keep it valid).
 * out_dtype: BGEMM_OUT_BITS_F32 (fp32 sw, sa, bias, zero_point) or BGEMM_OUT_BITS_F16 (fp16); all
 * are DEVICE pointers, bias may be NULL, zero_point NULL means 0.  No counterpart in the reference,
 * which materialises the fp16 activations between layers. */
int bgemm_packed_forward_bits(int mode, const void* W_tiled, const void* X_tiled, const void* X2_tiled,
                              void* out_tiled, int out_dtype, int64_t batch, int64_t M, int64_t N, int64_t K,
                              int64_t strideW, int64_t strideX, int64_t strideOut,
                              int splitK, int variant, void* ws, size_t ws_bytes,
                              void* counters, size_t counter_bytes,
                              const void* sw, const void* sa, const void* bias, const void* zero_point,
                              void* stream);

/* Decode step with the activations as they come out of the previous layer: prepacked weights x
 * fp16 or fp32 activations [N][K] (row stride ldx elements), one launch.  The kernel forms the sign bits
 * (with BGEMM_MODE_BWTA the ternary planes of sign(x)) itself, from `x - *x_zero_point` rounded to fp16
 * when a zero point is given: bgemm_pack_sign_centered / bgemm_pack_ternary_f16 followed by the packed
 * entry point (tests/python/bgemm_linear.py:479-484 for a batch of a few rows), without the pack launch.
 * Any output kind: out_dtype BGEMM_OUT_I32 / F16 (sw, sa, bias, next_zero_point NULL), the scaled kinds
 * (sw, sa; bias optional) or the bits kinds (also next_zero_point, optional).  Only shapes the decode
 * kernel takes this way (N <= 4 rows, M < 131072): ask _supported() first; other shapes
 * return BGEMM_EINVAL and go through the pack entry points and bgemm_packed_forward*. */
int bgemm_packed_weight_forward_supported(int mode, int64_t M, int64_t N, int64_t K);
int bgemm_packed_weight_forward(int mode, const void* W_tiled, const void* x, int x_dtype, int64_t ldx,
                                const void* x_zero_point, void* out, int out_dtype,
                                int64_t M, int64_t N, int64_t K, int variant,
                                const void* sw, const void* sa, const void* bias,
                                const void* next_zero_point, void* stream);

/* ---- fp16-operand call, the drop-in for the reference launcher -----------------------
 * Same argument meaning as bin_pack_linear_kernel (fp6_linear.cu:275-286):
 * W = weights half [M][K], X = in_feats half [N][K], C = half [N][M], INSTR in {0,1,2}.
 * Differences: any M, N, K >= 1 (the reference asserts M%32, N%32, K%128); the
 * workspace is bytes of scratch (packed operands + split-K state, no initialisation
 * needed: the call clears its own counters) instead of fp32 partial planes.
 */
size_t bgemm_f16_workspace_bytes(int64_t M, int64_t N, int64_t K, int splitK);
int bgemm_f16_forward(const void* W, const void* X, void* C, int64_t M, int64_t N, int64_t K,
                      void* ws, size_t ws_bytes, int splitK, int INSTR, void* stream);

/* bgemm_f16_forward for callers that cannot allocate device memory or bring a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference (whose
 * wrapper allocates its output and workspace with torch::empty on every call, fp6_linear.cu:580-586).
 * The scratch is a device array of BGEMM_STATIC_SCRATCH_BYTES inside the library, one copy per GPU, held
 * until the process ends; the call allocates and frees nothing.  Shapes whose
 * bgemm_f16_workspace_bytes(M, N, K, splitK) exceeds that size return BGEMM_EWORKSPACE (32 MiB covers
 * (M + N) * K up to about 2^28 bits, e.g. 8192 x 8192 against 8192 x 8192).  All calls on one GPU share the
 * one array: calls that overlap in time on the same GPU (two streams, two threads) race; serialise them, or
 * use bgemm_f16_forward with a workspace each.  The first call on a GPU looks the array's address up
 * (hipGetSymbolAddress): make it outside stream capture.  Same results as bgemm_f16_forward. */
#define BGEMM_STATIC_SCRATCH_BYTES (32u << 20)
int bgemm_f16_forward_static(const void* W, const void* X, void* C, int64_t M, int64_t N, int64_t K,
                             int splitK, int INSTR, void* stream);

/* ---- a chain of dependent decode-shaped layers in one launch ------------------------------------
 * Layer l computes acc = MODE(W_l [M_l][K_l], x_l [N][K_l]) and hands layer l + 1 the bits of
 * half_rn(y - *next_zero_point), y = half(acc) * sw * sa (+ bias) evaluated as in bgemm_packed_forward_scaled
 * (tests/python/bgemm_linear.py:479-484: one BGEMMLinear feeding the next): sign bits for the modes of one
 * plane, (nonzero, sign & nonzero) planes for BGEMM_MODE_BWTA (ternary = torch.sign, :222-241).  K_{l+1} = M_l.
 * The last layer writes `out` [N][M_last] as out_dtype I32, F16 or a scaled kind.  The reference runs such a
 * stack as one kernel launch (plus elementwise kernels) per layer and cannot run N < 32 at all
 * (fp6_linear.cu:288-290); here one block per compute unit stays resident, requests a layer's weights
 * while the layer before it is computed, and the layers exchange nothing but tagged bits.
 *   layers      : HOST array of n_layers entries; every pointer in it is a DEVICE pointer of param_dtype
 *                 (BGEMM_SRC_F16 / BGEMM_SRC_F32) elements: sw [M], bias [M] or NULL, sa one scalar,
 *                 next_zero_point one scalar or NULL (0; unused in the last layer)
 *   layers_dev  : the same array copied to the device by the caller (n_layers * 64 bytes)
 *   X_tiled     : the first layer's operand (X2_tiled: its sign & nonzero plane for BWTA), N rows:
 *                 N <= 32, with BWTA N <= 16
 *   ws          : bgemm_chain_workspace_bytes() bytes, ZERO-FILLED ONCE before its first use and then left
 *                 to the library; calls that share a workspace, or run on one GPU at the same time, must not
 *                 overlap (each holds every compute unit until its last layer is done)
 *   flags       : 0, or 1 / 2 to insist on the one-level / two-level exchange; 4 = block 0 leaves wall-clock stamps
 *                 (100 MHz ticks: start, then per layer operand ready / next layer requested / own K-tiles done /
 *                 partial sums met / outputs published) in the last (1 + 5 * 128) * 8 bytes of the workspace; bits 8.. = number of blocks (tests;
 *                 0 = one per compute unit)
 * Layers of up to 3 row tiles a block with K <= 4096, 2 with K <= 12288, 1 with K <= 16384 (a row tile is
 * 32 rows; blocks = compute units); others return BGEMM_EINVAL.  A block that waits longer than a quarter of
 * a second for its predecessors gives up; bgemm_chain_status() (synchronises the stream) then returns
 * BGEMM_ETIMEOUT once (it clears the mark, the workspace stays usable) and that call's output is undefined. */
typedef struct bgemm_chain_layer {
    const void* W_tiled;
    const void* sw;
    const void* bias;
    const void* sa;
    const void* next_zero_point;
    int64_t M, K;
    int64_t reserved;
} bgemm_chain_layer;
size_t bgemm_chain_workspace_bytes(int mode, const bgemm_chain_layer* layers, int n_layers, int64_t N);
int bgemm_chain_forward(int mode, const bgemm_chain_layer* layers, const void* layers_dev, int n_layers,
                        const void* X_tiled, const void* X2_tiled, int64_t N, void* out, int out_dtype,
                        int param_dtype, void* ws, size_t ws_bytes, int flags, void* stream);
int bgemm_chain_status(void* ws, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BGEMM_MI355X_H */
