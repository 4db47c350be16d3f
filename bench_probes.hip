// Measurement probes for bench.py (not part of the GEMM library): what the hardware allows the
// kernels of the library, measured on the GPU the benchmark runs on.
//   * the cost of launching a kernel that does nothing, and of reading a buffer once (the floor under a
//     decode-size launch, whose weights are one 5.6 MB read);
//   * the rate the matrix cores reach on the two MFMA instructions the library issues when nothing else
//     happens (no memory traffic, no bit expansion): the measured peak beside the datasheet one, following
//     the protocol of the reference's drivers (lowbit_kernel/csrc/kernel_test.h:10-11: warm-up launches, then
//     timed launches between two events, which bench.py does around these entry points);
//   * the same with a number of independent vector-ALU instructions after every MFMA, which is what the
//     in-register bit expansion costs the matrix-core kernels;
//   * what one all-to-all exchange of a few bytes per block costs blocks that stay resident (one per compute
//     unit): the floor under a layer of the chain kernel, to be set against the cost of a kernel boundary.
// Built into libbench_probes.so beside bench.py.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

__global__ void probe_empty_kernel(unsigned* out)
{
    if (out == reinterpret_cast<unsigned*>(1)) out[0] = 0;      // never true: nothing is done
}

// Grid-stride read of n_u4 16-byte words, four loads in flight per thread; the xor of everything
// read is compared with a value it never takes, so the loads stay and nothing is written.
__global__ __launch_bounds__(512) void probe_read_kernel(const uint4* __restrict__ src, int64_t n_u4, unsigned* out)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    unsigned acc = 0;
    for (; i + 3 * stride < n_u4; i += 4 * stride) {
        uint4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) v[u] = src[i + u * stride];
#pragma unroll
        for (int u = 0; u < 4; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < n_u4; i += stride) { const uint4 v = src[i]; acc ^= v.x ^ v.y ^ v.z ^ v.w; }
    if (acc == 0x12345678u && out == reinterpret_cast<unsigned*>(1)) out[0] = acc;
}

// NACC independent accumulators per wave keep the matrix pipe full.  The MFMAs read two sets of eight operand
// registers in turn, and after every MFMA exactly VALU vector-ALU instructions rewrite registers of the set it has just
// read, which the MFMA after next reads: as in the software-pipelined bit expansion, no MFMA waits for a register
// written just before it.  PERM: each is a v_perm_b32 (two vector registers and a scalar read); else a v_and_b32 of a
// vector register with a scalar, the form of most of the expansion.  The count per MFMA in the generated loop is VALU.
template <bool FP4, int NACC, int VALU, bool PERM>
__global__ __launch_bounds__(256) void probe_mfma_kernel(unsigned* out, const int iters, const unsigned seed)
{
    unsigned raw[8], op[16];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        if (i < 8) raw[i] = threadIdx.x * 2654435761u + i * 0x9e3779b9u + seed;
        op[i] = (threadIdx.x * 40503u + i) & (FP4 ? 0x22222222u : 0x01010101u);
    }
    typename std::conditional<FP4, v16f, v16i>::type acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[i][v] = 0;
    for (int it = 0; it < iters; it++) {
        const unsigned sel = 0x07020500u ^ ((seed + it) & 0x03030303u);           // scalar unit; bytes of either source
        const unsigned msk = (FP4 ? 0x33333333u : 0x01010101u) ^ ((seed + it) & (FP4 ? 0x44444444u : 0x02020202u));
#pragma unroll
        for (int i = 0; i < NACC; i++) {
            const int s = (i & 1) * 8;
            if constexpr (FP4) {
                const v8i a = {(int)op[s + 0], (int)op[s + 1], (int)op[s + 2], (int)op[s + 3], 0, 0, 0, 0};
                const v8i b = {(int)op[s + 4], (int)op[s + 5], (int)op[s + 6], (int)op[s + 7], 0, 0, 0, 0};
                acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[i], 4, 4, 0, 0, 0, 0);
            } else {
                const v4i a = {(int)op[s + 0], (int)op[s + 1], (int)op[s + 2], (int)op[s + 3]};
                const v4i b = {(int)op[s + 4], (int)op[s + 5], (int)op[s + 6], (int)op[s + 7]};
                acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[i], 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < VALU; u++) {
                const int j = ((i >> 1) * VALU + u) & 7;
                if constexpr (PERM) op[s + j] = __builtin_amdgcn_perm(op[s + j], raw[j], sel);
                else op[s + j] = raw[j] & (msk * (unsigned)(2 * i + 1));                              // the mask: scalar unit
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    unsigned sum = 0;
#pragma unroll
    for (int i = 0; i < NACC; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) sum += (unsigned)acc[i][v];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = sum;
}

}  // namespace

// All return 0, -1 for bad arguments, or the hipError_t of the launch.
// What sharing expanded fragments through LDS would make of the 256 x 128 tile's loop, at its most favourable: a wave
// expands three of its six fragments itself (two vector-ALU instructions per MFMA, half of today's expansion), writes
// them to LDS for the wave that needs the same ones and reads that wave's three: per step of eight MFMAs three
// ds_write_b128 and three ds_read_b128 a wave, straight from and into operand registers, and no barrier or flag
// between writer and reader (a real kernel needs one per K-tile).  Same accumulators, operand sets, grid and launch
// bounds as probe_mfma_kernel<true, 8, 2, false>, whose loop this is plus the six LDS instructions.
__global__ __launch_bounds__(256) void probe_mfma_lds_kernel(unsigned* out, const int iters, const unsigned seed)
{
    __shared__ uint4 sh[4][3][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    unsigned raw[8], op[16];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        if (i < 8) raw[i] = threadIdx.x * 2654435761u + i * 0x9e3779b9u + seed;
        op[i] = (threadIdx.x * 40503u + i) & 0x22222222u;
    }
#pragma unroll
    for (int i = 0; i < 3; i++) sh[wave][i][lane] = make_uint4(op[0], op[1], op[2], op[3]);
    __syncthreads();
    v16f acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[i][v] = 0;
    for (int it = 0; it < iters; it++) {
        const unsigned msk = 0x33333333u ^ ((seed + it) & 0x44444444u);                 // scalar unit
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int s = (i & 1) * 8;
            const v8i a = {(int)op[s + 0], (int)op[s + 1], (int)op[s + 2], (int)op[s + 3], 0, 0, 0, 0};
            const v8i b = {(int)op[s + 4], (int)op[s + 5], (int)op[s + 6], (int)op[s + 7], 0, 0, 0, 0};
            acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[i], 4, 4, 0, 0, 0, 0);
            if (i < 6 && (i & 1) == 0) {                          // own fragment: expanded in registers, then published
#pragma unroll
                for (int u = 0; u < 4; u++) op[s + u] = raw[u] & (msk * (unsigned)(2 * i + 1));
                sh[wave][i >> 1][lane] = make_uint4(op[s + 0], op[s + 1], op[s + 2], op[s + 3]);
            } else if (i < 6) {                                   // the other wave's fragment: read, not expanded
                const uint4 r = sh[wave ^ 1][i >> 1][lane];
                op[s + 4] = r.x; op[s + 5] = r.y; op[s + 6] = r.z; op[s + 7] = r.w;
            } else {                                              // the remaining expansion of the step (16 in all)
#pragma unroll
                for (int u = 0; u < 2; u++) op[s + 4 * (i & 1) + u] = raw[4 + u] & (msk * (unsigned)(2 * i + 1));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    unsigned sum = 0;
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) sum += (unsigned)acc[i][v];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = sum;
}

// `rounds` all-to-all exchanges among the blocks of the grid: every round, every block stores `units` 8-byte
// {tag, payload} units with device-scope stores into each of `copies` replicas and then polls every unit of replica
// blockIdx % copies until it carries the round's tag.  Waits are bounded (0.2 s of the 100 MHz wall clock); a block
// that runs out sets err[0] and leaves, a wrong payload counts in err[1].
__global__ __launch_bounds__(512) void probe_exchange_kernel(unsigned long long* buf, const int units, const int copies, const int rounds,
                                                            const unsigned epoch, unsigned long long* err, const int stride)
{
    const int G = gridDim.x, b = blockIdx.x, t = threadIdx.x, U = G * units;
    const long long t0 = wall_clock64();
    for (int r = 0; r < rounds; r++) {
        unsigned long long* cur = buf + (size_t)(r & 1) * copies * stride;
        const unsigned tag = epoch + r;
        for (int i = t; i < units * copies; i += 512)
            __hip_atomic_store(&cur[(size_t)(i / units) * stride + b * units + i % units],
                               ((unsigned long long)tag << 32) | (unsigned)(b * 131 + i % units + r), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long* mine = cur + (size_t)(b % copies) * stride;
        // a thread asks for all of its units that are still missing in every round of loads (up to four units a thread)
        int bad = 0;
        for (int base = t; base < U && !bad; base += 4 * 512) {
            unsigned pending = 0;
#pragma unroll
            for (int c = 0; c < 4; c++)
                if (base + c * 512 < U) pending |= 1u << c;
            for (unsigned tries = 1; pending; tries++) {
                unsigned long long v[4];
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    v[c] = 0;
                    if (pending >> c & 1) v[c] = __hip_atomic_load(&mine[base + c * 512], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int c = 0; c < 4; c++)
                    if ((pending >> c & 1) && (unsigned)(v[c] >> 32) == tag) {
                        const int i = base + c * 512;
                        if ((unsigned)v[c] != (unsigned)((i / units) * 131 + i % units + r)) atomicAdd(err + 1, 1ull);
                        pending &= ~(1u << c);
                    }
                if (pending && (tries & 63) == 0 && wall_clock64() - t0 > 20000000ll) { bad = 1; break; }
            }
        }
        if (__syncthreads_or(bad)) { if (t == 0) atomicAdd(err, 1ull); return; }
    }
}

extern "C" int bench_probe_empty(int blocks, int threads, void* scratch, void* stream)
{
    if (blocks <= 0 || threads <= 0 || threads > 1024) return -1;
    hipLaunchKernelGGL(probe_empty_kernel, dim3(blocks), dim3(threads), 0, (hipStream_t)stream, (unsigned*)scratch);
    return (int)hipGetLastError();
}

extern "C" int bench_probe_read(const void* src, int64_t bytes, int blocks, int threads, void* scratch, void* stream)
{
    if (!src || bytes < 16 || blocks <= 0 || threads <= 0 || threads > 512 || ((uintptr_t)src & 15)) return -1;
    hipLaunchKernelGGL(probe_read_kernel, dim3(blocks), dim3(threads), 0, (hipStream_t)stream, (const uint4*)src,
                       bytes / 16, (unsigned*)scratch);
    return (int)hipGetLastError();
}

// buf: 2 * copies * stride units of 8 bytes, zero before the first call, stride >= blocks * units; epoch: a number that
// is new for every call on the same buffer (advance it by `rounds`, starting at 1); err: two zeroed 8-byte counters.
extern "C" int bench_probe_exchange(void* buf, int blocks, int units, int copies, int rounds, unsigned epoch, void* err, int stride, void* stream)
{
    if (!buf || !err || blocks <= 0 || units <= 0 || copies <= 0 || rounds <= 0 || stride < blocks * units) return -1;
    hipLaunchKernelGGL(probe_exchange_kernel, dim3(blocks), dim3(512), 0, (hipStream_t)stream, (unsigned long long*)buf, units, copies, rounds,
                       epoch, (unsigned long long*)err, stride);
    return (int)hipGetLastError();
}

// One launch of `blocks` blocks of four waves, each wave issuing iters * 8 MFMAs (fp4 != 0:
// v_mfma_f32_32x32x64_f8f6f4 with E2M1 operands, 2 * 32 * 32 * 64 ops each; else v_mfma_i32_32x32x32_i8,
// 2 * 32 * 32 * 32 ops each) with `valu` in 0 .. 8 vector-ALU instructions after every one (v_and_b32; 100 + valu, fp4 only: v_perm_b32); fp4 with valu = -1: two
// vector-ALU instructions and the LDS traffic of fragments shared between the waves of a block (probe_mfma_lds_kernel).
// out: blocks * 256 words.
extern "C" int bench_probe_mfma(int fp4, int valu, int blocks, int iters, void* out, void* stream)
{
    if (blocks <= 0 || iters <= 0 || !out) return -1;
    const dim3 g(blocks), b(256);
    hipStream_t st = (hipStream_t)stream;
    unsigned* o = (unsigned*)out;
    if (fp4 && valu == -1) hipLaunchKernelGGL(probe_mfma_lds_kernel, g, b, 0, st, o, iters, 1u);      // fragments shared through LDS
    else {
#define PROBE_CASE(V) case V: if (fp4) hipLaunchKernelGGL((probe_mfma_kernel<true, 8, V, false>), g, b, 0, st, o, iters, 1u); \
                              else hipLaunchKernelGGL((probe_mfma_kernel<false, 8, V, false>), g, b, 0, st, o, iters, 1u); break; \
                      case 100 + V: if (!fp4) return -1; hipLaunchKernelGGL((probe_mfma_kernel<true, 8, V, true>), g, b, 0, st, o, iters, 1u); break;
        switch (valu) {
            PROBE_CASE(0) PROBE_CASE(1) PROBE_CASE(2) PROBE_CASE(3) PROBE_CASE(4) PROBE_CASE(5) PROBE_CASE(6) PROBE_CASE(7) PROBE_CASE(8)
            default: return -1;
        }
#undef PROBE_CASE
    }
    return (int)hipGetLastError();
}
