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

// NACC independent accumulators per wave keep the matrix pipe full; VALU masks of live registers after
// every MFMA stand in for the bit expansion (their results feed the next round's operands, so they stay).
template <bool FP4, int NACC, int VALU>
__global__ __launch_bounds__(256) void probe_mfma_kernel(unsigned* out, const int iters)
{
    unsigned m[8];
#pragma unroll
    for (int i = 0; i < 8; i++) m[i] = threadIdx.x * 2654435761u + i;
    typename std::conditional<FP4, v16f, v16i>::type acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[i][v] = 0;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < NACC; i++) {
            if constexpr (FP4) {
                const v8i a = {(int)(m[0] & 0x22222222u), (int)(m[1] & 0x22222222u), (int)(m[2] & 0x22222222u), (int)(m[3] & 0x22222222u), 0, 0, 0, 0};
                const v8i b = {(int)(m[4] & 0x22222222u), (int)(m[5] & 0x22222222u), (int)(m[6] & 0x22222222u), (int)(m[7] & 0x22222222u), 0, 0, 0, 0};
                acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[i], 4, 4, 0, 0, 0, 0);
            } else {
                const v4i a = {(int)(m[0] & 0x01010101u), (int)(m[1] & 0x01010101u), (int)(m[2] & 0x01010101u), (int)(m[3] & 0x01010101u)};
                const v4i b = {(int)(m[4] & 0x01010101u), (int)(m[5] & 0x01010101u), (int)(m[6] & 0x01010101u), (int)(m[7] & 0x01010101u)};
                acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[i], 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < VALU; u++) m[(i * VALU + u) & 7] = (m[(i * VALU + u) & 7] >> 1) ^ (it + u);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    unsigned s = 0;
#pragma unroll
    for (int i = 0; i < NACC; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) s += (unsigned)acc[i][v];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace

// All return 0, -1 for bad arguments, or the hipError_t of the launch.
// What sharing expanded fragments through LDS would make of the 256 x 128 tile's loop: per MFMA two vector-ALU
// instructions (half of today's expansion: every fragment expanded once per block instead of once per wave that needs it)
// plus the traffic that replaces the other half: of a K-tile's 32 MFMAs a wave, 24 ds_read_b128 (its six fragments x four
// steps) and 12 ds_write_b128 (its quarter of the block's twelve fragments), i.e. three reads and one and a half writes per
// four MFMAs.  Same accumulators, grid and launch bounds as the MFMA-only probe.
__global__ __launch_bounds__(256) void probe_mfma_lds_kernel(unsigned* out, const int iters)
{
    __shared__ uint4 s[4][8][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    unsigned m[8];
#pragma unroll
    for (int i = 0; i < 8; i++) m[i] = threadIdx.x * 2654435761u + i;
#pragma unroll
    for (int i = 0; i < 8; i++) s[wave][i][lane] = make_uint4(m[0], m[1], m[2], m[3]);
    __syncthreads();
    v16f acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[i][v] = 0;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const v8i a = {(int)(m[0] & 0x22222222u), (int)(m[1] & 0x22222222u), (int)(m[2] & 0x22222222u), (int)(m[3] & 0x22222222u), 0, 0, 0, 0};
            const v8i b = {(int)(m[4] & 0x22222222u), (int)(m[5] & 0x22222222u), (int)(m[6] & 0x22222222u), (int)(m[7] & 0x22222222u), 0, 0, 0, 0};
            acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[i], 4, 4, 0, 0, 0, 0);
            if ((i & 3) != 3) {                                  // three reads per four MFMAs: another wave's fragment
                const uint4 r = s[(wave + 1) & 3][i][lane];
                m[(i & 1) * 4 + 0] ^= r.x; m[(i & 1) * 4 + 1] ^= r.y; m[(i & 1) * 4 + 2] ^= r.z; m[(i & 1) * 4 + 3] ^= r.w;
            }
            if ((i & 3) == 1 || (i & 7) == 3)                    // one and a half writes per four MFMAs: this wave's own
                s[wave][i][lane] = make_uint4(m[0] + it, m[1], m[2], m[3]);
            m[i] = (m[i] >> 1) ^ (it + i);                       // the two vector-ALU instructions that stay
            m[(i + 3) & 7] = (m[(i + 3) & 7] >> 1) ^ it;
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
// 2 * 32 * 32 * 32 ops each) with `valu` in {0, 2, 4} vector-ALU instructions after every one; fp4 with valu = -1: two
// vector-ALU instructions and the LDS traffic of fragments shared between the waves of a block (probe_mfma_lds_kernel).
// out: blocks * 256 words.
extern "C" int bench_probe_mfma(int fp4, int valu, int blocks, int iters, void* out, void* stream)
{
    if (blocks <= 0 || iters <= 0 || !out) return -1;
    const dim3 g(blocks), b(256);
    hipStream_t st = (hipStream_t)stream;
    unsigned* o = (unsigned*)out;
    if (fp4 && valu == -1) hipLaunchKernelGGL(probe_mfma_lds_kernel, g, b, 0, st, o, iters);      // fragments shared through LDS
    else if (fp4) {
        if (valu == 0) hipLaunchKernelGGL((probe_mfma_kernel<true, 8, 0>), g, b, 0, st, o, iters);
        else if (valu == 2) hipLaunchKernelGGL((probe_mfma_kernel<true, 8, 2>), g, b, 0, st, o, iters);
        else if (valu == 4) hipLaunchKernelGGL((probe_mfma_kernel<true, 8, 4>), g, b, 0, st, o, iters);
        else return -1;
    } else {
        if (valu == 0) hipLaunchKernelGGL((probe_mfma_kernel<false, 8, 0>), g, b, 0, st, o, iters);
        else if (valu == 2) hipLaunchKernelGGL((probe_mfma_kernel<false, 8, 2>), g, b, 0, st, o, iters);
        else if (valu == 4) hipLaunchKernelGGL((probe_mfma_kernel<false, 8, 4>), g, b, 0, st, o, iters);
        else return -1;
    }
    return (int)hipGetLastError();
}
