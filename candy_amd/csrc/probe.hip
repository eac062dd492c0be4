// Read-only streaming probe: what this device delivers to a kernel that does nothing but read, per launch,
// so that the matvec's bytes per second can be quoted against an achievable figure measured in the same run
// as well as against the published peak.  No counterpart in the reference.
#include "blocks.h"
#include "internal.h"

namespace candy {

// Every thread issues U independent 16-byte loads (consecutive threads read consecutive chunks, a wavefront's
// U loads are 4 KB apart: all of them in flight before the first use), folds them into one word and stores
// it only if it equals a value the zero-filled buffer cannot produce, which keeps the loads alive.
template <int U>
__global__ __launch_bounds__(256) void k_stream_read(const u32x4 *__restrict__ src, size_t chunks, uint32_t *sink) {
    const size_t base = (size_t)blockIdx.x * (256 * U) + threadIdx.x;
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const size_t c = base + (size_t)u * 256;
        v[u] = src[c < chunks ? c : chunks - 1];
    }
    uint32_t acc = 0;
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    if (acc == 0x9E3779B9u) *sink = acc;
}

__global__ void k_empty() {}

// One 16-byte load per lane and wavefront, the wavefronts `stride` chunks apart (the rows of a weight): what a launch
// costs when it touches memory once - dispatch, first address, one round trip, end of kernel - and streams nothing.
__global__ __launch_bounds__(256) void k_one_load(const u32x4 *__restrict__ src, size_t stride, uint32_t *sink) {
    const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const u32x4 v = src[wave * stride + (threadIdx.x & 63)];
    const uint32_t acc = v.x ^ v.y ^ v.z ^ v.w;
    if (acc == 0x9E3779B9u) *sink = acc;
}

}  // namespace candy

using namespace candy;

extern "C" int candy_hip_stream_probe(candy_hip_device *dev, size_t bytes_per_launch, size_t span_bytes, int iters,
                                      float *elapsed_ms) {
    CANDY_REQUIRE(dev && elapsed_ms, "nil argument");
    CANDY_REQUIRE(iters > 0, "invalid iteration count");
    CANDY_REQUIRE(bytes_per_launch % 16 == 0, "bytes per launch must be a multiple of 16");
    CANDY_REQUIRE(bytes_per_launch == 0 || span_bytes >= bytes_per_launch, "the span must hold at least one launch");
    CANDY_REQUIRE(span_bytes <= (size_t(8) << 30), "span too large");
    if (int rc = use_device(dev)) return rc;
    constexpr int U = 8;
    void *buf = nullptr;
    uint32_t *sink = nullptr;
    size_t regions = 1;
    if (bytes_per_launch) {
        regions = span_bytes / bytes_per_launch;
        if (int rc = candy_hip_alloc(dev, regions * bytes_per_launch + 16, &buf)) return rc;
        int rc = candy_hip_alloc(dev, 16, (void **)&sink);
        if (!rc) rc = candy_hip_zero(dev, buf, regions * bytes_per_launch);
        if (rc) {
            (void)candy_hip_free(dev, buf);
            if (sink) (void)candy_hip_free(dev, sink);
            return rc;
        }
    }
    const size_t chunks = bytes_per_launch / 16;
    const size_t grid = (chunks + 256 * U - 1) / (256 * U);
    auto launch = [&](int i) {
        if (bytes_per_launch == 0) {
            hipLaunchKernelGGL(k_empty, dim3(1), dim3(64), 0, dev->stream);
        } else {
            const u32x4 *src = (const u32x4 *)((const uint8_t *)buf + (size_t)(i % regions) * bytes_per_launch);
            hipLaunchKernelGGL((k_stream_read<U>), dim3((unsigned)grid), dim3(256), 0, dev->stream, src, chunks, sink);
        }
    };
    hipError_t e = hipSuccess;
    if (grid > 0x7FFFFFFF) {
        e = hipErrorInvalidValue;
    } else {
        for (int i = 0; i < 3 && i < iters; ++i) launch(i);  // warm-up: code object, page tables
        e = hipEventRecord(dev->ev_start, dev->stream);
        for (int i = 0; i < iters; ++i) launch(i + 3);
        if (e == hipSuccess) e = hipGetLastError();
        if (e == hipSuccess) e = hipEventRecord(dev->ev_stop, dev->stream);
        if (e == hipSuccess) e = hipEventSynchronize(dev->ev_stop);
        if (e == hipSuccess) e = hipEventElapsedTime(elapsed_ms, dev->ev_start, dev->ev_stop);
    }
    if (buf) (void)candy_hip_free(dev, buf);
    if (sink) (void)candy_hip_free(dev, sink);
    if (e != hipSuccess) return fail(CANDY_HIP_ERR_HIP, "stream probe failed: %s", hipGetErrorString(e));
    return CANDY_HIP_OK;
}

// Where the fixed part of a launch goes (no counterpart in the reference).  `iters` launches back to back on the
// handle's stream of: kind 0 an empty kernel of one wavefront; 1 an empty kernel of 1024 workgroups x 256 threads
// (the grid of a 4096-row batch-1 contraction); 2 the same grid with every wavefront issuing ONE 16-byte load per
// lane, 6192 bytes apart (the rows of a Q4_K weight with 11008 columns), the same lines every launch (they stay in
// the caches); 3 the same, every launch in a region of its own out of 640 MiB (translation and HBM cold).
extern "C" int candy_hip_launch_probe(candy_hip_device *dev, int kind, int iters, float *elapsed_ms) {
    CANDY_REQUIRE(dev && elapsed_ms, "nil argument");
    CANDY_REQUIRE(kind >= 0 && kind <= 3 && iters > 0, "invalid probe kind or iteration count");
    if (int rc = use_device(dev)) return rc;
    constexpr size_t ROW = 6192, ROWS = 4096, REGION = ROW * ROWS, SPAN = size_t(640) << 20;
    const size_t regions = kind == 3 ? SPAN / REGION : 1;
    void *buf = nullptr;
    uint32_t *sink = nullptr;
    if (kind >= 2) {
        if (int rc = candy_hip_alloc(dev, regions * REGION + 1024, &buf)) return rc;
        int rc = candy_hip_alloc(dev, 16, (void **)&sink);
        if (!rc) rc = candy_hip_zero(dev, buf, regions * REGION + 1024);
        if (rc) {
            (void)candy_hip_free(dev, buf);
            if (sink) (void)candy_hip_free(dev, sink);
            return rc;
        }
    }
    auto launch = [&](int i) {
        if (kind == 0) hipLaunchKernelGGL(k_empty, dim3(1), dim3(64), 0, dev->stream);
        else if (kind == 1) hipLaunchKernelGGL(k_empty, dim3(ROWS / 4), dim3(256), 0, dev->stream);
        else
            hipLaunchKernelGGL(k_one_load, dim3(ROWS / 4), dim3(256), 0, dev->stream,
                               (const u32x4 *)((const uint8_t *)buf + (size_t)(i % regions) * REGION), ROW / 16, sink);
    };
    for (int i = 0; i < 20 && i < iters; ++i) launch(i);
    hipError_t e = hipEventRecord(dev->ev_start, dev->stream);
    for (int i = 0; i < iters; ++i) launch(i + 20);
    if (e == hipSuccess) e = hipGetLastError();
    if (e == hipSuccess) e = hipEventRecord(dev->ev_stop, dev->stream);
    if (e == hipSuccess) e = hipEventSynchronize(dev->ev_stop);
    if (e == hipSuccess) e = hipEventElapsedTime(elapsed_ms, dev->ev_start, dev->ev_stop);
    if (buf) (void)candy_hip_free(dev, buf);
    if (sink) (void)candy_hip_free(dev, sink);
    if (e != hipSuccess) return fail(CANDY_HIP_ERR_HIP, "launch probe failed: %s", hipGetErrorString(e));
    return CANDY_HIP_OK;
}
