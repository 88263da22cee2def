// Diagnostics of the device, not of the BitLinear arithmetic: what a chain of dependent kernel launches costs on the
// current device when the kernels do nothing, and when they only read the bytes a decode launch reads.  A token step
// at batch 1 is a chain of 120 launches in which every launch needs the result of the one before it; these figures are
// the floor such a chain cannot go below, measured in the same process as the benchmark of the real chain.
// No counterpart in the reference (its CPU path has no launches).
#include "common.hpp"
#include "tiledot.hpp"

namespace bitnet {
namespace {

__global__ void diag_empty_kernel(unsigned *sink)
{
    (void)sink;  // an argument buffer to fetch, as every real launch has, and nothing else
}

// Streams n16 16-byte words once, every load with the non-temporal hint the decode GEMV gives its weight tiles, and keeps
// nothing: the xor of what was read is stored only if it equals a value that random bytes give once in 2^32 launches.
__global__ __launch_bounds__(256) void diag_stream_read_kernel(const uint4 *src, size_t n16, unsigned *sink)
{
    const size_t stride = (size_t)gridDim.x * 256;
    uint4 acc = make_uint4(0, 0, 0, 0);
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) {
        const uint4 v = load_weight_slot(src + i);
        acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w;
    }
    const unsigned r = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (r == 0x9e3779b9u) sink[blockIdx.x & 63] = r;
}

// ---- hand-over inside one launch ---------------------------------------------------------------------------------------
// The alternative to a chain of launches is one launch whose workgroups stay resident and hand a vector from step to step
// through memory.  This kernel measures what one such hand-over ("hop") costs: `values` 8-byte words (value, hop number)
// are produced by the workgroups in equal shares (device-scope stores, written through to where every XCD reads them), and
// every workgroup must have seen all words of hop h before it produces its share of hop h + 1 (each new value is the
// neighbouring old value plus one, so after H hops every value is H: the result is checked).
//   flat:      every workgroup polls all words with device-scope loads.
//   two-level: the first workgroup of each XCD (workgroup ids go to the XCDs in turn) polls them and copies them into a
//              buffer of its XCD with plain stores; the other workgroups of the XCD poll that copy in their own L2
//              (invalidating their compute unit's L1 before every look).
// Every wait is bounded: a thread that does not see its word within the spin limit records a failure and goes on, so the
// kernel ends whatever happens.  Writers are at most one hop ahead of the slowest reader, hence two buffers by hop parity.
constexpr int HOP_THREADS = 256;

__device__ __forceinline__ unsigned long long hop_load_device(const unsigned long long *ptr)
{
    return __hip_atomic_load(ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void hop_store_device(unsigned long long *ptr, unsigned long long v)
{
    __hip_atomic_store(ptr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <bool TWO_LEVEL>
__global__ __launch_bounds__(HOP_THREADS) void diag_hop_kernel(unsigned long long *pub /* [2][values] */,
                                                               unsigned long long *local /* [8][2][values] */, int values, int hops,
                                                               int spin_limit, unsigned *status /* [0]: failures, [1]: wrong values */)
{
    extern __shared__ unsigned vec[];  // the vector of the current hop, as every workgroup holds it
    const int tid = threadIdx.x, wg = blockIdx.x, nwg = gridDim.x;
    const int xcd = wg & 7;
    const bool leader = wg < 8;
    const int share = (values + nwg - 1) / nwg, first = wg * share, last = min(values, first + share);
    for (int i = tid; i < values; i += HOP_THREADS) vec[i] = 0u;  // hop 0: all zero, known to everybody
    __syncthreads();
    unsigned failures = 0;
    for (int h = 1; h <= hops; ++h) {
        unsigned long long *buf = pub + (size_t)(h & 1) * values;
        // produce this workgroup's share of hop h from the vector of hop h - 1
        for (int i = first + tid; i < last; i += HOP_THREADS)
            hop_store_device(buf + i, (unsigned long long)(vec[(i + 1) % values] + 1u) | ((unsigned long long)(unsigned)h << 32));
        __syncthreads();  // vec is read above and overwritten below
        if (!TWO_LEVEL || leader) {
            for (int i = tid; i < values; i += HOP_THREADS) {
                unsigned long long w = 0;
                int spin = 0;
                const int limit = failures ? 1 : spin_limit;  // after a wait that ran out, look once and go on
                for (; spin < limit; ++spin) {
                    w = hop_load_device(buf + i);
                    if ((unsigned)(w >> 32) == (unsigned)h) break;
                }
                if (spin == limit) ++failures;
                vec[i] = (unsigned)w;
                if (TWO_LEVEL) local[((size_t)xcd * 2 + (h & 1)) * values + i] = w;  // plain store: into this XCD's L2
            }
        } else {
            const unsigned long long *mine = local + ((size_t)xcd * 2 + (h & 1)) * values;
            for (int i = tid; i < values; i += HOP_THREADS) {
                unsigned long long w = 0;
                int spin = 0;
                const int limit = failures ? 1 : spin_limit;
                for (; spin < limit; ++spin) {
                    asm volatile("buffer_inv sc0" ::: "memory");  // drop this compute unit's L1 copy: the load below reads L2
                    w = *reinterpret_cast<const volatile unsigned long long *>(mine + i);
                    if ((unsigned)(w >> 32) == (unsigned)h) break;
                }
                if (spin == limit) ++failures;
                vec[i] = (unsigned)w;
            }
        }
        __syncthreads();
    }
    unsigned wrong = 0;
    for (int i = tid; i < values; i += HOP_THREADS) wrong += vec[i] != (unsigned)hops;
    if (failures) atomicAdd(&status[0], failures);
    if (wrong) atomicAdd(&status[1], wrong);
}

struct ChainResources {
    hipStream_t cs = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hipEvent_t e[2] = {nullptr, nullptr};
    unsigned *sink = nullptr;
    ~ChainResources()
    {
        if (exec) (void)hipGraphExecDestroy(exec);
        if (graph) (void)hipGraphDestroy(graph);
        if (cs) (void)hipStreamDestroy(cs);
        for (hipEvent_t v : e)
            if (v) (void)hipEventDestroy(v);
        if (sink) (void)hipFree(sink);
    }
};

}  // namespace
}  // namespace bitnet

using namespace bitnet;

extern "C" int bitnet_hip_measure_launch_chain(const void *buf, const size_t *bytes_per_launch, size_t pattern_len,
                                               size_t launches, size_t replays, double *us_per_replay, void *stream)
{
    if (!us_per_replay) return fail(BITNET_HIP_NULL_POINTER, "measure_launch_chain: the result pointer is required");
    *us_per_replay = 0.0;
    if (launches == 0 || launches > 100000 || replays == 0)
        return fail(BITNET_HIP_INVALID_CONFIG, "measure_launch_chain: %zu launches, %zu replays", launches, replays);
    const bool reads = buf != nullptr;
    if (reads && (!bytes_per_launch || pattern_len == 0))
        return fail(BITNET_HIP_NULL_POINTER, "measure_launch_chain: a buffer needs the bytes each launch reads");
    if (reads && (reinterpret_cast<uintptr_t>(buf) & 15) != 0)
        return fail(BITNET_HIP_INVALID_CONFIG, "measure_launch_chain: the buffer must be 16-byte aligned");
    if (reads)
        for (size_t i = 0; i < pattern_len; ++i)
            if (bytes_per_launch[i] % 16 != 0)
                return fail(BITNET_HIP_INVALID_CONFIG, "measure_launch_chain: launch %zu reads %zu bytes, not a multiple of 16", i,
                            bytes_per_launch[i]);
    ChainResources r;
    BITNET_HIP_TRY(hipMalloc(reinterpret_cast<void **>(&r.sink), 64 * sizeof(unsigned)));
    BITNET_HIP_TRY(hipStreamCreateWithFlags(&r.cs, hipStreamNonBlocking));
    BITNET_HIP_TRY(hipEventCreate(&r.e[0]));
    BITNET_HIP_TRY(hipEventCreate(&r.e[1]));
    // The chain, recorded: launch i reads the bytes behind those of launch i - 1 (distinct memory every launch, as the
    // projections of a stack are), in stream order, so each launch starts when the one before it has finished.
    BITNET_HIP_TRY(hipStreamBeginCapture(r.cs, hipStreamCaptureModeThreadLocal));
    const uint8_t *at = static_cast<const uint8_t *>(buf);
    for (size_t i = 0; i < launches; ++i) {
        if (!reads) {
            hipLaunchKernelGGL(diag_empty_kernel, dim3(256), dim3(256), 0, r.cs, r.sink);
        } else {
            const size_t n16 = bytes_per_launch[i % pattern_len] / 16;
            const size_t blocks = (n16 + 255) / 256;
            const unsigned grid = (unsigned)(blocks < 1 ? 1 : (blocks > 2048 ? 2048 : blocks));
            hipLaunchKernelGGL(diag_stream_read_kernel, dim3(grid), dim3(256), 0, r.cs, reinterpret_cast<const uint4 *>(at), n16,
                               r.sink);
            at += n16 * 16;
        }
    }
    hipError_t launch_err = hipGetLastError();
    hipError_t end_err = hipStreamEndCapture(r.cs, &r.graph);  // always ends the recording
    if (launch_err != hipSuccess)
        return fail(BITNET_HIP_KERNEL_ERROR, "measure_launch_chain: a launch failed: %s", hipGetErrorString(launch_err));
    BITNET_HIP_TRY(end_err);
    BITNET_HIP_TRY(hipGraphInstantiate(&r.exec, r.graph, nullptr, nullptr, 0));
    hipStream_t s = as_stream(stream);
    for (int i = 0; i < 2; ++i) BITNET_HIP_TRY(hipGraphLaunch(r.exec, s));  // untimed: first touch, clocks
    BITNET_HIP_TRY(hipStreamSynchronize(s));
    BITNET_HIP_TRY(hipEventRecord(r.e[0], s));
    for (size_t i = 0; i < replays; ++i) BITNET_HIP_TRY(hipGraphLaunch(r.exec, s));
    BITNET_HIP_TRY(hipEventRecord(r.e[1], s));
    BITNET_HIP_TRY(hipEventSynchronize(r.e[1]));
    float ms = 0.0f;
    BITNET_HIP_TRY(hipEventElapsedTime(&ms, r.e[0], r.e[1]));
    *us_per_replay = (double)ms * 1e3 / (double)replays;
    return BITNET_HIP_OK;
}

extern "C" int bitnet_hip_measure_hop(int two_level, size_t values, size_t hops, int spin_limit, double *us_per_hop, int *intact,
                                      void *stream)
{
    if (!us_per_hop || !intact) return fail(BITNET_HIP_NULL_POINTER, "measure_hop: the result pointers are required");
    *us_per_hop = 0.0;
    *intact = 0;
    if (values == 0 || values > 16384 || hops == 0 || hops > 100000)
        return fail(BITNET_HIP_INVALID_CONFIG, "measure_hop: %zu values (1 .. 16384), %zu hops (1 .. 100000)", values, hops);
    int device = 0, units = 0;
    BITNET_HIP_TRY(hipGetDevice(&device));
    BITNET_HIP_TRY(hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device));
    // one workgroup per compute unit at most, so that all of them are resident at once (they wait for each other)
    const int nwg = (units < 256 ? units : 256) / 8 * 8;
    if (nwg < 8) return fail(BITNET_HIP_UNSUPPORTED, "measure_hop: %d compute units", units);
    struct Buffers {
        unsigned long long *pub = nullptr, *local = nullptr;
        unsigned *status = nullptr;
        hipEvent_t e[2] = {nullptr, nullptr};
        ~Buffers()
        {
            if (pub) (void)hipFree(pub);
            if (local) (void)hipFree(local);
            if (status) (void)hipFree(status);
            for (hipEvent_t v : e)
                if (v) (void)hipEventDestroy(v);
        }
    } b;
    BITNET_HIP_TRY(hipMalloc(reinterpret_cast<void **>(&b.pub), 2 * values * sizeof(unsigned long long)));
    BITNET_HIP_TRY(hipMalloc(reinterpret_cast<void **>(&b.local), 16 * values * sizeof(unsigned long long)));
    BITNET_HIP_TRY(hipMalloc(reinterpret_cast<void **>(&b.status), 2 * sizeof(unsigned)));
    BITNET_HIP_TRY(hipEventCreate(&b.e[0]));
    BITNET_HIP_TRY(hipEventCreate(&b.e[1]));
    hipStream_t s = as_stream(stream);
    // default: some milliseconds, far beyond any hand-over that works; a thread whose wait runs out looks only once from then on
    if (spin_limit <= 0 || spin_limit > 100000) spin_limit = 20000;
    const size_t lds = values * sizeof(unsigned);
    float ms = 0.0f;
    for (int pass = 0; pass < 2; ++pass) {  // the first pass is untimed (same length)
        BITNET_HIP_TRY(hipMemsetAsync(b.pub, 0, 2 * values * sizeof(unsigned long long), s));
        BITNET_HIP_TRY(hipMemsetAsync(b.local, 0, 16 * values * sizeof(unsigned long long), s));
        BITNET_HIP_TRY(hipMemsetAsync(b.status, 0, 2 * sizeof(unsigned), s));
        BITNET_HIP_TRY(hipEventRecord(b.e[0], s));
        if (two_level)
            hipLaunchKernelGGL((diag_hop_kernel<true>), dim3(nwg), dim3(HOP_THREADS), lds, s, b.pub, b.local, (int)values, (int)hops,
                               spin_limit, b.status);
        else
            hipLaunchKernelGGL((diag_hop_kernel<false>), dim3(nwg), dim3(HOP_THREADS), lds, s, b.pub, b.local, (int)values, (int)hops,
                               spin_limit, b.status);
        BITNET_HIP_CHECK_LAUNCH("diag_hop_kernel");
        BITNET_HIP_TRY(hipEventRecord(b.e[1], s));
        BITNET_HIP_TRY(hipEventSynchronize(b.e[1]));
        BITNET_HIP_TRY(hipEventElapsedTime(&ms, b.e[0], b.e[1]));
    }
    unsigned status[2] = {1, 1};
    BITNET_HIP_TRY(hipMemcpy(status, b.status, sizeof status, hipMemcpyDeviceToHost));
    *intact = status[0] == 0 && status[1] == 0;
    *us_per_hop = (double)ms * 1e3 / (double)hops;
    return BITNET_HIP_OK;
}
