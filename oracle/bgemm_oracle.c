/*
 * CPU oracle for the BGEMM / BWTA hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic of the reference's binary GEMM
 * path so that the HIP kernels can be checked bit for bit.  It is never linked
 * into, loaded by or called from the product library: only tests, the smoke
 * check and the CPU-baseline leg of the benchmark may use it.
 *
 * Reference anchors (paths relative to the reference tree):
 *   pack rule        lowbit_kernel/csrc/utils/weight_prepacking.h:181-230
 *                    lowbit_kernel/csrc/include/ptx_mma.cuh:341-380
 *   mode arithmetic  lowbit_kernel/csrc/include/utils_core.cuh:242-303
 *                    lowbit_kernel/csrc/include/ptx_mma.cuh:196-250,299-336
 *   split-K ranges   lowbit_kernel/csrc/include/kernel_matmul.cuh:391-404
 *   output layout    lowbit_kernel/csrc/include/kernel_matmul.cuh:529-546
 *   split-K reduce   lowbit_kernel/csrc/include/kernel_reduction.cuh:29-48
 *   host launcher    lowbit_kernel/csrc/fp6_linear.cu:275-337,561-616
 *
 * Parity status.  The reference holds no golden vectors for this path, its
 * device code is PTX and cannot be built here, and its host pack header needs
 * cuda_fp16.h (absent), so nothing of the reference is compiled.  Every function
 * below is instead pinned by tests/test_oracle.py against what the mathematics
 * fixes: dense integer matmuls on de-binarised operands (numpy), brute-force
 * loops, algebraic identities between the modes, numpy's IEEE float16 rounding
 * and hand-computed bit patterns.
 */
#include <stdint.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_AND  0   /* configs.h:70  AND_POP */
#define ORACLE_XOR  1   /* configs.h:71  XOR_POP */
#define ORACLE_ATTN 2   /* configs.h:72  ATTN_MM */

static inline int popc32(uint32_t x) { return __builtin_popcount(x); }

/* Number of 32-bit words that hold K sign bits. */
static inline int64_t words_for(int64_t K) { return (K + 31) / 32; }

/*
 * Sign-pack fp16 rows into 32-bit words, most significant bit first:
 * bit (31 - i) of word j of a row = IEEE sign bit of element 32*j + i.
 * weight_prepacking.h:181-190 builds it with shifts of (x & 0x8000); the device
 * routine ptx_mma.cuh:371-379 pairs element i with i+16 and lands on the same
 * bit positions.  -0.0 therefore packs as 1 and NaNs pack by their sign bit.
 * The reference asserts K % 128 == 0 (weight_prepacking.h:206); here a ragged
 * tail leaves the unused low bits of the last word at 0.
 * src: rows x K halves with row stride ld (in elements); dst: rows x ceil(K/32).
 */
void oracle_pack_sign_f16(const uint16_t* src, int64_t rows, int64_t K, int64_t ld,
                          uint32_t* dst)
{
    const int64_t Kw = words_for(K);
    for (int64_t r = 0; r < rows; r++) {
        for (int64_t j = 0; j < Kw; j++) {
            uint32_t w = 0;
            for (int i = 0; i < 32; i++) {
                const int64_t k = 32 * j + i;
                if (k < K && (src[r * ld + k] & 0x8000u)) w |= 1u << (31 - i);
            }
            dst[r * Kw + j] = w;
        }
    }
}

/*
 * Ternary pack for the binary-weight x ternary-activation product.  The reference
 * CPU path ternarises with torch.sign (tests/python/bgemm_linear.py:222-241), so
 * +-0 -> 0, negative -> -1, positive -> +1.  Two bit planes, same bit order as
 * oracle_pack_sign_f16:  nz = (magnitude bits != 0),  sg = nz & sign bit.
 */
void oracle_pack_ternary_f16(const uint16_t* src, int64_t rows, int64_t K, int64_t ld,
                             uint32_t* nz, uint32_t* sg)
{
    const int64_t Kw = words_for(K);
    for (int64_t r = 0; r < rows; r++) {
        for (int64_t j = 0; j < Kw; j++) {
            uint32_t z = 0, s = 0;
            for (int i = 0; i < 32; i++) {
                const int64_t k = 32 * j + i;
                if (k >= K) continue;
                const uint16_t h = src[r * ld + k];
                if (h & 0x7fffu) {
                    z |= 1u << (31 - i);
                    if (h & 0x8000u) s |= 1u << (31 - i);
                }
            }
            nz[r * Kw + j] = z;
            sg[r * Kw + j] = s;
        }
    }
}

/* Mask of the valid (high) bits of word j when only K bits of the row are real. */
static inline uint32_t valid_mask(int64_t j, int64_t K)
{
    const int64_t left = K - 32 * j;
    if (left >= 32) return 0xffffffffu;
    if (left <= 0) return 0u;
    return 0xffffffffu << (32 - left);
}

/*
 * One word of one mode, as the reference accumulates it per 128-bit slice
 * (utils_core.cuh:273-296):
 *   AND   c += popc(a & b)                              ptx_mma.cuh:196-210
 *   XOR   c += bits - 2*popc(a ^ b)                     ptx_mma.cuh:212-250 (bits = 128 there)
 *   ATTN  c += popc(~a & ~b) - popc(~a & b)             ptx_mma.cuh:299-336
 * a = weight-side word, b = activation-side word, vm = valid-bit mask.
 */
static inline int32_t mode_word(int mode, uint32_t a, uint32_t b, uint32_t vm)
{
    switch (mode) {
    case ORACLE_AND:  return popc32(a & b & vm);
    case ORACLE_XOR:  return popc32(vm) - 2 * popc32((a ^ b) & vm);
    default:          return popc32(~a & ~b & vm) - popc32(~a & b & vm);
    }
}

/*
 * Packed-operand BGEMM.  Wp: M x Kw words, Xp: N x Kw words (logical MSB-first
 * format above), C: int32, row-major [N][M] (kernel_matmul.cuh:534-545 writes
 * C[m + n*M]).  Accumulation range [w0, w1) in words lets the split-K path reuse it.
 */
static void bgemm_words(int mode, const uint32_t* Wp, const uint32_t* Xp, int32_t* C,
                        int64_t M, int64_t N, int64_t K, int64_t w0, int64_t w1)
{
    const int64_t Kw = words_for(K);
    for (int64_t n = 0; n < N; n++)
        for (int64_t m = 0; m < M; m++) {
            int32_t acc = 0;
            for (int64_t j = w0; j < w1; j++)
                acc += mode_word(mode, Wp[m * Kw + j], Xp[n * Kw + j], valid_mask(j, K));
            C[n * M + m] = acc;
        }
}

int oracle_bgemm_packed(int mode, const uint32_t* Wp, const uint32_t* Xp, int32_t* C,
                        int64_t M, int64_t N, int64_t K)
{
    if (mode < 0 || mode > 2) return -1;
    bgemm_words(mode, Wp, Xp, C, M, N, K, 0, words_for(K));
    return 0;
}

/*
 * Binary weight x ternary activation:  C[n][m] = sum_k t(X[n,k]) * s(W[m,k]),
 * t in {-1,0,+1}, s = -1 where the weight sign bit is set.  In bit planes
 * (a = weight sign word, z = nonzero plane, s = sign plane):
 *     C += popc(z) - 2*popc((a ^ s) & z)
 * which is the XOR rule restricted to the positions where the activation is
 * nonzero; with z = all ones it is the XOR mode, and with z = ~a_attn it is ATTN.
 */
void oracle_bwta_packed(const uint32_t* Wp, const uint32_t* Xnz, const uint32_t* Xsg,
                        int32_t* C, int64_t M, int64_t N, int64_t K)
{
    const int64_t Kw = words_for(K);
    for (int64_t n = 0; n < N; n++)
        for (int64_t m = 0; m < M; m++) {
            int32_t acc = 0;
            for (int64_t j = 0; j < Kw; j++) {
                const uint32_t vm = valid_mask(j, K);
                const uint32_t z = Xnz[n * Kw + j] & vm;
                acc += popc32(z) - 2 * popc32((Wp[m * Kw + j] ^ Xsg[n * Kw + j]) & z);
            }
            C[n * M + m] = acc;
        }
}

/* float -> IEEE binary16, round to nearest even, overflow to infinity. */
static uint16_t f32_to_f16_rn(float f)
{
    uint32_t x; memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) return sign | (absx > 0x7f800000u ? 0x7e00u : 0x7c00u);
    if (absx >= 0x477ff000u) return sign | 0x7c00u;        /* >= 65520 rounds to inf */
    if (absx < 0x33000001u) return sign;                   /* <= 2^-25 rounds to 0   */
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x7fffffu) | 0x800000u;
    int shift = (e < -14) ? (13 + (-14 - e)) : 13;         /* subnormal halves lose more bits */
    uint32_t half_man = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man++;
    uint32_t bits = (e < -14) ? half_man : (((uint32_t)(e + 15) << 10) + (half_man - 0x400u));
    return sign | (uint16_t)bits;
}

/*
 * int32 accumulator -> fp16 as the reference stores it: __int2half_rn
 * (kernel_matmul.cuh:540) when splitK == 1, else fp32 sum then __float2half_rn
 * (kernel_reduction.cuh:42,47).  Both are the correctly rounded integer while
 * |v| < 2^24, which every supported K satisfies.
 */
uint16_t oracle_int_to_f16(int32_t v) { return f32_to_f16_rn((float)v); }

/*
 * The whole reference call restated:  bin_pack_linear_kernel (fp6_linear.cu:275-337)
 * = sign-pack both fp16 operands, run the mode arithmetic over split-K ranges of
 * 128-bit K-tiles, write fp32 partial planes [splitK][N][M], sum them in fp32 and
 * round to fp16.  Partition (kernel_matmul.cuh:397-404): T = number of 128-bit
 * tiles, avg = T / splitK, the first T - avg*splitK splits get one extra tile,
 * ranges are contiguous.  The reference asserts M%32, N%32, K%128 == 0
 * (fp6_linear.cu:288-290); this restatement also accepts ragged shapes, a ragged
 * last tile simply counting fewer bits.
 * W: M x K halves, X: N x K halves.  out_f16 (N x M halves) and out_i32 (N x M)
 * may each be NULL.  Returns 0, or -1 on bad arguments, -2 on allocation failure.
 */
int oracle_bgemm_f16(const uint16_t* W, const uint16_t* X, uint16_t* out_f16, int32_t* out_i32,
                     int64_t M, int64_t N, int64_t K, int splitK, int mode)
{
    if (mode < 0 || mode > 2 || splitK < 1 || M < 0 || N < 0 || K < 0) return -1;
    const int64_t Kw = words_for(K), MN = M * N;
    if (MN == 0) return 0;
    uint32_t* Wp = (uint32_t*)calloc((size_t)(M * Kw) + 1, 4);
    uint32_t* Xp = (uint32_t*)calloc((size_t)(N * Kw) + 1, 4);
    int32_t* part = (int32_t*)malloc((size_t)MN * 4);
    float* ws = (float*)calloc((size_t)MN * (size_t)splitK, 4);
    if (!Wp || !Xp || !part || !ws) { free(Wp); free(Xp); free(part); free(ws); return -2; }
    oracle_pack_sign_f16(W, M, K, K, Wp);
    oracle_pack_sign_f16(X, N, K, K, Xp);
    const int64_t T = (K + 127) / 128, avg = T / splitK, extra = T - avg * splitK;
    for (int64_t s = 0; s < splitK; s++) {
        const int64_t n_it = avg + (s < extra ? 1 : 0);
        const int64_t t0 = avg * s + (s < extra ? s : extra);
        int64_t w0 = 4 * t0, w1 = 4 * (t0 + n_it);
        if (w1 > Kw) w1 = Kw;
        if (w0 > Kw) w0 = Kw;
        bgemm_words(mode, Wp, Xp, part, M, N, K, w0, w1);
        for (int64_t i = 0; i < MN; i++) ws[s * MN + i] = (float)part[i];
    }
    for (int64_t i = 0; i < MN; i++) {
        float sum = 0.0f;
        for (int64_t s = 0; s < splitK; s++) sum += ws[s * MN + i];
        if (out_f16) out_f16[i] = f32_to_f16_rn(sum);
        if (out_i32) out_i32[i] = (int32_t)sum;
    }
    free(Wp); free(Xp); free(part); free(ws);
    return 0;
}
