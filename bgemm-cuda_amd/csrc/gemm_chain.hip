// A chain of dependent decode-shaped layers in ONE launch.
//
// A decode step of a model is a sequence of small binary-weight products, each of which needs the whole
// output of the one before: layer l + 1's activation bits are the signs (ternary: sign and nonzero planes) of
// half(y_l - zp), y_l = half(acc_l) * sw * sa (+ bias) (tests/python/bgemm_linear.py:479-484).  Launched one
// by one, every layer pays a kernel launch and the first trip of its weights from HBM (about 4 us for 5.6 MB
// of weights, of which the transfer is under one).  Here one block per compute unit stays resident for the
// whole chain:
//   * block b owns weight row tiles b, b + G, ... of every layer; a wave of it owns K-tiles wave, wave + 8, ...
//     of those tiles, and requests layer l + 1's tiles (buffer loads, kept in registers) before it starts on
//     layer l, so the weights of a layer are in the compute unit before its activations exist;
//   * the activation operand of a layer (one tile row: up to 32 sign rows, or 16 rows of two planes) lives in
//     LDS; the partial sums of the waves meet in LDS through integer adds;
//   * a block publishes the 32-bit words of the next operand it is responsible for as 8-byte units
//     {tag, word} with device-scope stores, tag = a number that is new for every layer of every call; the
//     consumers poll the data itself, so an exchange is one store and one load through the memory fabric
//     (0.5 to 0.6 us between two compute units) and needs no counter, no fence and no second trip.
//     With many units (rows x K / 32 x planes) the 256 blocks would all pull every unit through the fabric;
//     then a block first fetches only its 1/32 share and re-publishes it in a replica that belongs to its
//     XCD (blocks b, b + 8, ... share an XCD and its L2), from which the 32 blocks of that XCD read.
// Every wait is bounded by a wall-clock budget: a block that runs out of it raises the error word of the
// workspace and leaves, and so, in turn, does every other block; no wave can wait for ever.
#include "common.h"
#include "mfma_engines.h"
#include "pack_bits.h"
#include <string.h>
#include <algorithm>
#include <type_traits>

namespace bgemm {

constexpr int CHAIN_THREADS = 512, CHAIN_WAVES = 8;
constexpr int CHAIN_MAX_LAYERS = 128;
constexpr int CHAIN_POLL_CH = 8;             // units a thread keeps in flight while it polls

// One layer as the device sees it: the caller's bgemm_chain_layer, 64 bytes.
struct ChainLayerDev { const uint4* W; const void* sw; const void* bias; const void* sa; const void* zp; int64_t M, K, pad; };
static_assert(sizeof(ChainLayerDev) == sizeof(bgemm_chain_layer), "the device table is the caller's array");

struct ChainArgs {
    const ChainLayerDev* layers; int n_layers;
    ModeCoef mc;
    int N;
    const uint4* X; const uint4* X2;          // the first layer's activation operand, one tile row
    void* out; int out_kind;                  // the last layer's output
    unsigned* state;                          // [0] tag base, [1] blocks done, [2] error
    unsigned long long* xg;                   // [2][u_max] units every block can see
    unsigned long long* xl;                   // [8][2][u_max] per-XCD replicas, or null: one level
    int u_max, kt_max;
    long long* trace;                         // null, or [1 + 5 * n_layers] wall-clock stamps written by thread 0 of block 0: start; per layer
                                              // operand in LDS, next layer requested, own K-tiles done, partial sums met, outputs published
    long long budget;                         // ticks of the 100 MHz wall clock a wait may take, from the kernel's start
    int mute_block0;                          // test hook: block 0 publishes nothing, so every wait for it runs out of budget
    unsigned e_magic;                         // ceil(2^32 / E), E = planes * N units per word (unused for E = 1)
};

__device__ __forceinline__ unsigned long long unit_load(const unsigned long long* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void unit_store(unsigned long long* p, const unsigned tag, const unsigned word)
{
    __hip_atomic_store(p, ((unsigned long long)tag << 32) | word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Polls units u0, u0 + stride, ... below U of `src` until each carries `tag` and hands (u, word) to `sink`.  A thread
// takes CHAIN_POLL_CH units at a time and asks for ALL of them that are still missing in every round of loads, so a round
// trip through the memory fabric is paid once per round and not once per unit.  Returns false when the budget ran out (the
// wall clock is a slow read: looked at once in 64 rounds).
template <typename Sink>
__device__ __forceinline__ bool poll_units(const unsigned long long* src, const int u0, const int stride, const int U, const unsigned tag,
                                           const long long t0, const long long budget, Sink sink)
{
    for (int base = u0; base < U; base += CHAIN_POLL_CH * stride) {
        unsigned pending = 0;
#pragma unroll
        for (int c = 0; c < CHAIN_POLL_CH; c++)
            if (base + c * stride < U) pending |= 1u << c;
        for (unsigned tries = 1; pending; tries++) {
            unsigned long long v[CHAIN_POLL_CH];
#pragma unroll
            for (int c = 0; c < CHAIN_POLL_CH; c++) {
                v[c] = 0;
                if (pending >> c & 1) v[c] = unit_load(src + base + c * stride);
            }
#pragma unroll
            for (int c = 0; c < CHAIN_POLL_CH; c++)
                if ((pending >> c & 1) && (unsigned)(v[c] >> 32) == tag) {
                    sink(base + c * stride, (unsigned)v[c]);
                    pending &= ~(1u << c);
                }
            if (pending && (tries & 63u) == 0 && wall_clock64() - t0 > budget) return false;
        }
    }
    return true;
}

template <int NTM, int KSM, bool F32>
__global__ __launch_bounds__(CHAIN_THREADS, 1) void gemm_chain_kernel(const ChainArgs a)
{
    typedef EngF4 Eng;
    extern __shared__ __align__(16) unsigned char smem[];
    uint4* const acts = reinterpret_cast<uint4*>(smem);                                    // [kt_max][64]
    int* const red = reinterpret_cast<int*>(smem + (size_t)a.kt_max * 1024);               // [2][NTM][16][64]
    int* const sPa = red + 2 * NTM * 1024;                                                 // [2][NTM][32]
    int* const sPb = sPa + 2 * NTM * 32;                                                   // [2][32]
    float* const sPar = reinterpret_cast<float*>(sPb + 64);                                // [2][NTM * 64 + 4]: sw, bias per row; sa, zp
    int* const sFlag = reinterpret_cast<int*>(sPar + 2 * (NTM * 64 + 4));                  // [4]
    ChainLayerDev* const sL = reinterpret_cast<ChainLayerDev*>(sFlag + 4);                 // [n_layers]
    constexpr int PAR = NTM * 64 + 4;

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int G = gridDim.x, b = blockIdx.x, L = a.n_layers;
    const long long t0 = wall_clock64();
    const bool two = a.mc.planes == 2;
    const int N = a.N, E = a.mc.planes * N;
    const ModeCoef mc = a.mc;

    for (int i = tid; i < L * 4; i += CHAIN_THREADS) reinterpret_cast<uint4*>(sL)[i] = reinterpret_cast<const uint4*>(a.layers)[i];
    for (int i = tid; i < 2 * NTM * 1024 + 2 * NTM * 32 + 64; i += CHAIN_THREADS) red[i] = 0;
    if (tid < 4) sFlag[tid] = 0;
    const unsigned epoch = __hip_atomic_load(a.state, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();

    // ---- what a thread requests one layer ahead ------------------------------------------------------
    // Weight tiles: tile i of the block is row tile b + i * G; slot j of the wave is K-tile wave + 8 * j.  Every
    // request is issued: loads under a branch would make the compiler wait for ALL outstanding loads at the first
    // use of any.  A slot that does not exist (a layer with fewer tiles than the kernel is built for) reads the
    // layer's first tile instead, which is always there and stays in the cache; its registers are never used.
    // Parameters: thread i * 32 + c holds sw and bias of row c of tile i, thread NTM * 32 the two scalars; lanes
    // without a parameter read the tag base instead.
    uint4 wq[NTM][KSM], wnext[NTM][KSM];      // this layer's tiles, the next layer's
    auto request_weights = [&](uint4 (&to)[NTM][KSM], const int l) {
        const ChainLayerDev& d = sL[l];
        const int MT = __builtin_amdgcn_readfirstlane((int)((d.M + 31) >> 5)), KT = __builtin_amdgcn_readfirstlane((int)((d.K + 255) >> 8));
        // (readfirstlane returns a signed int: it is narrowed to unsigned BEFORE it is widened, or a low word with bit 31
        // set would smear ones over the pointer's upper half)
        const uintptr_t wlo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(uintptr_t)d.W);
        const uintptr_t whi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)((uintptr_t)d.W >> 32));
        const uint4* const W = reinterpret_cast<const uint4*>(wlo | (whi << 32));
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4*>(W), 0, MT * KT * 1024, 0x00020000);
#pragma unroll
        for (int i = 0; i < NTM; i++)
#pragma unroll
            for (int j = 0; j < KSM; j++) {
                const int rt = b + i * G, kt = wave + CHAIN_WAVES * j;
                const unsigned off = (rt < MT && kt < KT ? (unsigned)(rt * KT + kt) * 1024u : 0u) + lane * 16u;
                const v4i v = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off, 0, 2 /* read once */);
                to[i][j] = make_uint4(v.x, v.y, v.z, v.w);
            }
    };
    typedef typename std::conditional<F32, float, __half>::type P;
    auto request_params = [&](P& pa_, P& pb_, const int l) {
        const ChainLayerDev& d = sL[l];
        const P* const dummy = reinterpret_cast<const P*>(a.state);
        const int i = tid >> 5, c = tid & 31;
        const int64_t m = (int64_t)(b + i * G) * 32 + c;
        const P* p0 = dummy; const P* p1 = dummy;
        if (tid < NTM * 32 && m < d.M) {          // (a last layer with a plain output may come without scales)
            if (d.sw) p0 = reinterpret_cast<const P*>(d.sw) + m;
            if (d.bias) p1 = reinterpret_cast<const P*>(d.bias) + m;
        } else if (tid == NTM * 32) {
            if (d.sa) p0 = reinterpret_cast<const P*>(d.sa);
            if (d.zp) p1 = reinterpret_cast<const P*>(d.zp);
        }
        // global (not flat) loads: they return in order with the weight requests that follow, so waiting for them
        // does not wait for those
        typedef typename std::conditional<F32, unsigned, unsigned short>::type R;
        typedef const __attribute__((address_space(1))) R* GP;
        const R r0 = *(GP)(const R*)p0, r1 = *(GP)(const R*)p1;
        __builtin_memcpy(&pa_, &r0, sizeof r0);
        __builtin_memcpy(&pb_, &r1, sizeof r1);
    };
    auto keep_params = [&](const P pa_, const P pb_, const int l, const int S) {
        const ChainLayerDev& d = sL[l];
        if (tid <= NTM * 32) {
            const bool second = tid < NTM * 32 ? d.bias != nullptr : d.zp != nullptr;
            sPar[S * PAR + 2 * tid] = (float)pa_;
            sPar[S * PAR + 2 * tid + 1] = second ? (float)pb_ : 0.f;
        }
    };

    // ---- layer 0: operand from the caller, weights and parameters requested now -----------------------
    {
        P p0, p1;
        request_params(p0, p1, 0);
        request_weights(wq, 0);
        const int KT0 = (int)((sL[0].K + 255) >> 8);
        for (int s = tid; s < a.kt_max * 64; s += CHAIN_THREADS) {
            const int kt = s >> 6, h = (s >> 5) & 1, prow = s & 31;
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (kt < KT0) {
                if (two) {
                    if ((prow & 15) < N) v = (prow < 16 ? a.X : a.X2)[kt * 64 + h * 32 + (prow & 15)];
                } else if (prow < N)
                    v = a.X[s];
            }
            acts[s] = v;
            const int p = popc4(v);
            if (p) atomicAdd(&sPb[prow], p);
        }
        keep_params(p0, p1, 0, 0);
        __builtin_amdgcn_s_waitcnt(0x0f70);          // vmcnt(0): layer 0's weights are waited for here, once
        __syncthreads();
    }

    bool aborted = false;
    const bool tracing = a.trace != nullptr && b == 0 && tid == 0;
    const long long c0 = tracing ? clock64() : 0;
    if (tracing) a.trace[0] = t0;
    // One body for every layer (the LDS areas alternate by the layer's parity S, the registers are handed on at the end):
    // a copy per parity would double the code, and the whole chain's code should stay in the instruction cache.
    auto body = [&](const int l) -> bool {
        const int S = l & 1;
        const ChainLayerDev& d = sL[l];
        const int M = __builtin_amdgcn_readfirstlane((int)d.M), K = __builtin_amdgcn_readfirstlane((int)d.K);
        const int MT = (M + 31) >> 5, KT = (K + 255) >> 8;
        const bool last = l + 1 == L;
        const int ntb = MT > b ? (MT - b + G - 1) / G : 0;            // row tiles this block owns
        const bool has_bias = d.bias != nullptr;

        if (tracing) a.trace[1 + 5 * l] = wall_clock64();
        // (1) the next layer's parameters and weights are requested before this layer is touched
        P np0, np1;
        request_params(np0, np1, last ? l : l + 1);
        request_weights(wnext, last ? l : l + 1);

        if (tracing) a.trace[2 + 5 * l] = wall_clock64();
        // (2) this wave's K-tiles of the block's row tiles against the operand in LDS
        typename Eng::Acc acc[NTM];
        int pa[NTM];
#pragma unroll
        for (int i = 0; i < NTM; i++) {
            pa[i] = 0;
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][v] = 0;
        }
#pragma unroll
        for (int j = 0; j < KSM; j++) {
            const int kt = wave + CHAIN_WAVES * j;
            if (kt >= KT || ntb == 0) continue;
            const uint4 xq = acts[kt * 64 + lane];
#pragma unroll
            for (int s = 0; s < Eng::STEPS; s++) {
                const typename Eng::Frag ax = Eng::expand_x(xq, s);
#pragma unroll
                for (int i = 0; i < NTM; i++)
                    if (i < ntb) acc[i] = Eng::mma(ax, Eng::expand_w(wq[i][j], s), acc[i]);
            }
#pragma unroll
            for (int i = 0; i < NTM; i++)
                if (i < ntb) pa[i] += popc4(wq[i][j]);
        }

        if (tracing) a.trace[3 + 5 * l] = wall_clock64();
        // (3) the waves' partial sums meet in LDS (accumulator registers 4g .. 4g + 3 hold operand rows 8g .. 8g + 7)
        if (wave < KT) {
#pragma unroll
            for (int i = 0; i < NTM; i++) {
                if (i >= ntb) continue;
                int* const r = red + (S * NTM + i) * 1024;
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    if (8 * (two ? (g & 1) : g) >= N) continue;
#pragma unroll
                    for (int v = 4 * g; v < 4 * g + 4; v++) atomicAdd(&r[v * 64 + lane], Eng::to_int(acc[i], v));
                }
                const int p = pa[i] + __shfl_xor(pa[i], 32);
                if (lane < 32) atomicAdd(&sPa[(S * NTM + i) * 32 + lane], p);
            }
        }
        __syncthreads();
        if (tracing) a.trace[4 + 5 * l] = wall_clock64();

        // (4) epilogue.  The areas of the other parity and the operand are cleared for the next layer, whose
        // parameters (requested in (1), before the weights, so they are here first) go to LDS.
        keep_params(np0, np1, last ? l : l + 1, S ^ 1);
        if (!last) {
            const int KTn = (M + 255) >> 8;                        // the next layer's K is this layer's M
            for (int s = tid; s < KTn * 64; s += CHAIN_THREADS) acts[s] = make_uint4(0u, 0u, 0u, 0u);
            for (int i = tid; i < NTM * 1024; i += CHAIN_THREADS) red[(S ^ 1) * NTM * 1024 + i] = 0;
            if (tid < NTM * 32) sPa[(S ^ 1) * NTM * 32 + tid] = 0;
            if (tid < 32) sPb[(S ^ 1) * 32 + tid] = 0;
        }
        const float sa = sPar[S * PAR + NTM * 64], zp = sPar[S * PAR + NTM * 64 + 1];
        const unsigned tag = epoch + (unsigned)l + 1u;
        unsigned long long* const pub = a.xg + (size_t)((l + 1) & 1) * a.u_max;
        const int total = ntb * N * 32;
        for (int o0 = wave * 64; o0 < total; o0 += CHAIN_THREADS) {
            const int o = o0 + lane, q = o >> 5, c = o & 31;
            const int i = (q >= N) + (q >= 2 * N), nl = q - i * N;
            const bool valid = o < total;
            const int64_t m = (int64_t)(b + i * G) * 32 + c;
            int val = 0;
            ColParams cp = {0.f, 0.f};
            if (valid) {
                const int v = 4 * (nl >> 3) + (nl & 3), hh = (nl >> 2) & 1;
                const int* const r = red + (S * NTM + i) * 1024;
                const int dd = r[v * 64 + hh * 32 + c], d2 = two ? r[(v + 8) * 64 + hh * 32 + c] : 0;
                val = skinny_value(mc, two, K, sPa[(S * NTM + i) * 32 + c], sPb[S * 32 + nl], two ? sPb[S * 32 + nl + 16] : 0, dd, d2);
                cp.sw = sPar[S * PAR + 2 * (i * 32 + c)];
                cp.bias = sPar[S * PAR + 2 * (i * 32 + c) + 1];
            }
            if (last) {
                if (valid && m < M) {
                    const int64_t at = (int64_t)nl * M + m;
                    switch (a.out_kind) {
                    case BGEMM_OUT_I32: reinterpret_cast<int*>(a.out)[at] = val; break;
                    case BGEMM_OUT_F16: reinterpret_cast<__half*>(a.out)[at] = __float2half_rn((float)val); break;
                    case BGEMM_OUT_F32_SCALED: reinterpret_cast<float*>(a.out)[at] = scaled_f32(val, cp, sa, has_bias); break;
                    default: reinterpret_cast<__half*>(a.out)[at] = scaled_f16(val, cp, sa, has_bias); break;
                    }
                }
            } else {
                unsigned sg = 0, nz = 0;
                if (valid && m < M) {
#pragma clang fp contract(off)
                    const float y = F32 ? scaled_f32(val, cp, sa, has_bias) : __half2float(scaled_f16(val, cp, sa, has_bias));
                    const uint16_t hb = half_bits((y - zp));
                    sg = hb >> 15; nz = (hb & 0x7fff) != 0;
                }
                const unsigned long long bs = __ballot(sg != 0 && (!two || nz != 0)), bz = __ballot(nz != 0);
                const unsigned ws = __brev((unsigned)(lane < 32 ? bs : bs >> 32)), wz = __brev((unsigned)(lane < 32 ? bz : bz >> 32));
                if (c == 0 && valid && !(a.mute_block0 && b == 0)) {
                    const int jw = b + i * G;
                    if (two) {
                        unit_store(pub + (jw * 2 + 0) * N + nl, tag, wz);
                        unit_store(pub + (jw * 2 + 1) * N + nl, tag, ws);
                    } else
                        unit_store(pub + jw * N + nl, tag, ws);
                }
            }
        }
        __syncthreads();
        if (tracing) a.trace[5 + 5 * l] = wall_clock64();
        if (last) return true;

        // (5) the next layer's operand: MT words a row and plane, E units a word
        const int U = MT * E;
        const unsigned long long* src = a.xg + (size_t)((l + 1) & 1) * a.u_max;
        bool ok = true;
        if (a.xl) {
            const int x = b & 7, j = b >> 3, nb = G >> 3, per = (U + nb - 1) / nb;
            unsigned long long* const rep = a.xl + (size_t)(x * 2 + ((l + 1) & 1)) * a.u_max;
            const int hi = min(U, (j + 1) * per);
            ok = poll_units(src, j * per + tid, CHAIN_THREADS, hi, tag, t0, a.budget, [&](const int u, const unsigned w) { unit_store(rep + u, tag, w); });
            src = rep;
        }
        if (ok)
            ok = poll_units(src, tid, CHAIN_THREADS, U, tag, t0, a.budget, [&](const int u, const unsigned w) {
                const int jw = E == 1 ? u : (int)__umulhi((unsigned)u, a.e_magic), e = u - jw * E;
                const int prow = two ? (e >= N ? 16 + e - N : e) : e;
                reinterpret_cast<unsigned*>(acts)[(jw >> 3) * 256 + ((jw >> 2) & 1) * 128 + prow * 4 + (jw & 3)] = w;
                const int p = __popc(w);
                if (p) atomicAdd(&sPb[(S ^ 1) * 32 + prow], p);
            });
        if (!ok) sFlag[0] = 1;
        // Loads return in order, so the polls above have also seen the next layer's weights arrive; saying so keeps
        // the compiler from waiting for the requests of the NEXT body when this one's registers are first used.
        __builtin_amdgcn_s_waitcnt(0x0f70);          // vmcnt(0)
#pragma unroll
        for (int i = 0; i < NTM; i++)
#pragma unroll
            for (int j = 0; j < KSM; j++) wq[i][j] = wnext[i][j];
        __syncthreads();
        return sFlag[0] == 0;
    };
    for (int l = 0; l < L; l++)
        if (!body(l)) { aborted = true; break; }

    if (tracing) {          // shader-clock ticks and wall-clock ticks of the whole launch: their ratio is the clock the launch ran at
        a.trace[1 + 5 * CHAIN_MAX_LAYERS - 2] = clock64() - c0;
        a.trace[1 + 5 * CHAIN_MAX_LAYERS - 1] = wall_clock64() - t0;
    }
    // The last block to get here moves the tag base past this call's tags and re-arms the counter.
    if (tid == 0) {
        if (aborted) __hip_atomic_store(a.state + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned n = __hip_atomic_fetch_add(a.state + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (n == (unsigned)G - 1u) {
            __hip_atomic_store(a.state + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(a.state, epoch + (unsigned)L + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

}  // namespace bgemm

// ---- host side -----------------------------------------------------------------------------------
namespace bgemm {

struct ChainShape { int ntm, ksm, kt_max, u_max; };

static int chain_grid(int forced)
{
    if (forced > 0) return forced;
    static int cus[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (!cus[dev]) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cus[dev] = n;
    }
    return cus[dev];
}

// Checks a chain and derives what the kernel needs of it.  0 or a BGEMM_E* code (message recorded).
static int chain_shape(int mode, const bgemm_chain_layer* layers, int n_layers, int64_t N, int G, ChainShape* cs, ModeCoef* mc)
{
    if (!mode_coef(mode, mc)) return fail(BGEMM_EINVAL, "bgemm_chain: unknown mode %d", mode);
    if (!layers) return fail(BGEMM_ENULL, "bgemm_chain: layers is NULL");
    if (n_layers < 1 || n_layers > CHAIN_MAX_LAYERS - 1) return fail(BGEMM_EINVAL, "bgemm_chain: 1 to %d layers, got %d", CHAIN_MAX_LAYERS - 1, n_layers);
    if (N < 1 || N > (mc->planes == 2 ? 16 : 32))
        return fail(BGEMM_EINVAL, "bgemm_chain: N=%lld activation rows; one operand tile row holds up to %d", (long long)N, mc->planes == 2 ? 16 : 32);
    if (G < 1) return fail(BGEMM_ELAUNCH, "bgemm_chain: cannot read the number of compute units");
    *cs = {1, 1, 1, 1};
    for (int l = 0; l < n_layers; l++) {
        const bgemm_chain_layer& d = layers[l];
        if (d.M < 1 || d.K < 1 || d.K >= (1LL << 24)) return fail(BGEMM_EINVAL, "bgemm_chain: layer %d is %lld x %lld", l, (long long)d.M, (long long)d.K);
        if (l && d.K != layers[l - 1].M)
            return fail(BGEMM_EINVAL, "bgemm_chain: layer %d reads K=%lld values, layer %d writes M=%lld", l, (long long)d.K, l - 1, (long long)layers[l - 1].M);
        if (!d.W_tiled) return fail(BGEMM_ENULL, "bgemm_chain: layer %d has no weights", l);
        if ((uintptr_t)d.W_tiled & 15) return fail(BGEMM_EALIGN, "bgemm_chain: layer %d: weights must be 16-byte aligned", l);
        const int64_t MT = row_tiles(d.M), KT = k_tiles(d.K);
        if (MT * KT * 1024 >= (1LL << 31)) return fail(BGEMM_EINVAL, "bgemm_chain: layer %d holds 2 GiB of weights or more", l);
        cs->ntm = (int)std::max<int64_t>(cs->ntm, cdiv(MT, G));
        cs->ksm = (int)std::max<int64_t>(cs->ksm, cdiv(KT, CHAIN_WAVES));
        cs->kt_max = (int)std::max<int64_t>(cs->kt_max, KT);
        if (l + 1 < n_layers) cs->u_max = (int)std::max<int64_t>(cs->u_max, MT * mc->planes * N);
    }
    if (cs->ntm > 3 || cs->ksm > 8 || (cs->ntm > 1 && cs->ksm > 6) || (cs->ntm > 2 && cs->ksm > 2))
        return fail(BGEMM_EINVAL, "bgemm_chain: a layer needs %d row tiles a block and %d K-tiles a wave; the kernel is built for up to "
                                  "3 x 2, 2 x 6 and 1 x 8 (run such a layer through bgemm_packed_forward)", cs->ntm, cs->ksm);
    return BGEMM_OK;
}

static size_t chain_trace_bytes() { return (1 + 5 * CHAIN_MAX_LAYERS) * 8; }
static size_t chain_ws_bytes(const ChainShape& cs) { return 256 + (size_t)18 * cs.u_max * 8 + chain_trace_bytes(); }

template <int NTM, int KSM, bool F32>
static int chain_launch(const ChainArgs& a, int G, hipStream_t st)
{
    const size_t lds = (size_t)a.kt_max * 1024 + 2 * NTM * 4096 + 2 * NTM * 128 + 256 + 2 * (NTM * 64 + 4) * 4 + 16 + (size_t)a.n_layers * 64;
    if (lds > 160 * 1024) return fail(BGEMM_EINVAL, "bgemm_chain: %zu bytes of LDS needed, 160 KiB there", lds);
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_chain_kernel<NTM, KSM, F32>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return fail(BGEMM_ELAUNCH, "bgemm_chain: cannot reserve %zu bytes of LDS", lds);
    }
    hipLaunchKernelGGL((gemm_chain_kernel<NTM, KSM, F32>), dim3((unsigned)G), dim3(CHAIN_THREADS), lds, st, a);
    return check_launch("bgemm_chain");
}

}  // namespace bgemm

using namespace bgemm;

extern "C" size_t bgemm_chain_workspace_bytes(int mode, const bgemm_chain_layer* layers, int n_layers, int64_t N)
{
    ChainShape cs; ModeCoef mc;
    if (chain_shape(mode, layers, n_layers, N, chain_grid(0), &cs, &mc) != BGEMM_OK) return 0;
    return chain_ws_bytes(cs);
}

extern "C" int bgemm_chain_forward(int mode, const bgemm_chain_layer* layers, const void* layers_dev, int n_layers,
                                   const void* X_tiled, const void* X2_tiled, int64_t N, void* out, int out_dtype, int param_dtype,
                                   void* ws, size_t ws_bytes, int flags, void* stream)
{
    ChainShape cs; ModeCoef mc;
    const int G = chain_grid(flags >> 8);
    const int rc = chain_shape(mode, layers, n_layers, N, G, &cs, &mc);
    if (rc != BGEMM_OK) return rc;
    if (!layers_dev || !X_tiled || !out || !ws || (mc.planes == 2 && !X2_tiled)) return fail(BGEMM_ENULL, "bgemm_chain_forward: a required pointer is NULL");
    if (((uintptr_t)X_tiled | (uintptr_t)X2_tiled | (uintptr_t)layers_dev | (uintptr_t)ws) & 15)
        return fail(BGEMM_EALIGN, "bgemm_chain_forward: operands, layer table and workspace must be 16-byte aligned");
    if (ws_bytes < chain_ws_bytes(cs)) return fail(BGEMM_EWORKSPACE, "bgemm_chain_forward: workspace %zu < %zu bytes", ws_bytes, chain_ws_bytes(cs));
    if (out_dtype < BGEMM_OUT_I32 || out_dtype > BGEMM_OUT_F16_SCALED) return fail(BGEMM_EINVAL, "bgemm_chain_forward: output kind %d", out_dtype);
    if (param_dtype != BGEMM_SRC_F16 && param_dtype != BGEMM_SRC_F32) return fail(BGEMM_EINVAL, "bgemm_chain_forward: parameter type %d", param_dtype);
    if ((out_dtype == BGEMM_OUT_F32_SCALED && param_dtype != BGEMM_SRC_F32) || (out_dtype == BGEMM_OUT_F16_SCALED && param_dtype != BGEMM_SRC_F16))
        return fail(BGEMM_EINVAL, "bgemm_chain_forward: a scaled output has the parameters' type");
    for (int l = 0; l < n_layers; l++) {
        const bool scaled = l + 1 < n_layers || out_dtype >= BGEMM_OUT_F32_SCALED;
        if (scaled && (!layers[l].sw || !layers[l].sa)) return fail(BGEMM_ENULL, "bgemm_chain_forward: layer %d has no sw or sa", l);
    }
    const int levels = flags & 3;
    if (levels == 3 || (flags & 0xf0)) return fail(BGEMM_EINVAL, "bgemm_chain_forward: flags");
    ChainArgs a;
    memset(&a, 0, sizeof a);
    a.layers = (const ChainLayerDev*)layers_dev; a.n_layers = n_layers;
    a.mc = mc; a.N = (int)N;
    a.X = (const uint4*)X_tiled; a.X2 = (const uint4*)X2_tiled;
    a.out = out; a.out_kind = out_dtype;
    a.state = (unsigned*)ws;
    a.xg = (unsigned long long*)((char*)ws + 256);
    // one level up to a few hundred units a layer (every block pulls every unit through the fabric), two beyond
    const bool two_level = G % 8 == 0 && (levels == 2 || (levels == 0 && cs.u_max > 4096));
    a.xl = two_level ? a.xg + (size_t)2 * cs.u_max : nullptr;
    a.u_max = cs.u_max; a.kt_max = cs.kt_max;
    a.trace = (flags & 4) ? (long long*)((char*)ws + 256 + (size_t)18 * cs.u_max * 8) : nullptr;
    a.budget = 25000000LL;          // a quarter of a second
    if (flags & 8) { a.mute_block0 = 1; a.budget = 100000LL; }      // (tests of the time-out path: a millisecond)
    const unsigned E = (unsigned)(mc.planes * N);
    a.e_magic = E > 1 ? (unsigned)(((1ULL << 32) + E - 1) / E) : 0;
    const bool f32 = param_dtype == BGEMM_SRC_F32;
    hipStream_t st = (hipStream_t)stream;
    if (cs.ntm <= 1 && cs.ksm > 6) return f32 ? chain_launch<1, 8, true>(a, G, st) : chain_launch<1, 8, false>(a, G, st);
    if (cs.ksm <= 2) return f32 ? chain_launch<3, 2, true>(a, G, st) : chain_launch<3, 2, false>(a, G, st);
    return f32 ? chain_launch<2, 6, true>(a, G, st) : chain_launch<2, 6, false>(a, G, st);
}

extern "C" int bgemm_chain_status(void* ws, void* stream)
{
    if (!ws) return fail(BGEMM_ENULL, "bgemm_chain_status: ws is NULL");
    unsigned st[4] = {0, 0, 0, 0};
    if (hipMemcpyAsync(st, ws, sizeof st, hipMemcpyDeviceToHost, (hipStream_t)stream) != hipSuccess || hipStreamSynchronize((hipStream_t)stream) != hipSuccess) {
        (void)hipGetLastError();
        return fail(BGEMM_ELAUNCH, "bgemm_chain_status: cannot read the workspace");
    }
    if (st[2]) {
        // reported once: the word is cleared so that the workspace can be used again
        const unsigned zero = 0;
        if (hipMemcpyAsync((char*)ws + 8, &zero, 4, hipMemcpyHostToDevice, (hipStream_t)stream) != hipSuccess || hipStreamSynchronize((hipStream_t)stream) != hipSuccess)
            (void)hipGetLastError();
        return fail(BGEMM_ETIMEOUT, "bgemm_chain: a block waited longer than its budget for the layer before it "
                                    "(calls that share a GPU at the same time can starve each other of compute units)");
    }
    return BGEMM_OK;
}
