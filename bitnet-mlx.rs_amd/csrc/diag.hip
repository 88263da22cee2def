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
