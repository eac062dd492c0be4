// Host-side internals shared by the translation units of libcandy_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/candy_hip.h"

namespace candy {

// Thread-local failure text behind candy_hip_last_error().
void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define CANDY_HIP_TRY(expr)                                                              \
    do {                                                                                 \
        hipError_t _e = (expr);                                                          \
        if (_e != hipSuccess)                                                            \
            return ::candy::fail(_e == hipErrorOutOfMemory ? CANDY_HIP_ERR_OOM : CANDY_HIP_ERR_HIP, \
                                 "%s failed: %s", #expr, hipGetErrorString(_e));         \
    } while (0)

#define CANDY_REQUIRE(cond, ...)                                                          \
    do {                                                                                 \
        if (!(cond)) return ::candy::fail(CANDY_HIP_ERR_INVALID, __VA_ARGS__);           \
    } while (0)

// Check the launch that was just enqueued.
#define CANDY_LAUNCH_CHECK() CANDY_HIP_TRY(hipGetLastError())

struct FormatInfo {
    int elems;
    int bytes;
};
FormatInfo format_info(int fmt);  // {0,0} if unknown

// Planar Q8_0 activations: the matvec / MFMA kernels read the int8 quants and the
// per-32 scale separately so every load is naturally aligned.
struct Q8Scale {
    float d;       // fp16-rounded scale, widened back to f32 (what a Q8_0 block stores)
    int32_t bsum;  // sum of the block's 32 quants (for the `min` term of Q4_K)
};

}  // namespace candy

struct candy_hip_device {
    int ordinal = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    int num_cus = 0;
    char name[256] = {0};
    // Workspace for quantized activations (grown on demand, never shrunk).
    void *ws = nullptr;
    size_t ws_bytes = 0;
};

struct candy_hip_qtensor {
    candy_hip_device *dev = nullptr;
    int fmt = 0;
    int64_t rows = 0, cols = 0;
    size_t nbytes = 0;
    void *data = nullptr;
    bool owned = false;
};

struct candy_hip_qact {
    candy_hip_device *dev = nullptr;
    int64_t max_m = 0, max_cols = 0;  // capacity
    int64_t m = 0, cols = 0;          // shape of what it currently holds
    int8_t *qs = nullptr;             // [m, cols] int8
    candy::Q8Scale *scales = nullptr; // [m, cols/32]
};

namespace candy {

// Makes dev's GPU current for the calling thread (cgo may move goroutines between threads).
int use_device(const candy_hip_device *dev);
// Returns a workspace of at least `bytes` bytes (256-byte aligned).
int workspace(candy_hip_device *dev, size_t bytes, void **out);

// quant.hip: x[rows, cols] -> planar int8 quants + scales; optionally also 34-byte blocks.
int launch_quantize_q8(candy_hip_device *dev, const float *x, int64_t rows, int64_t cols,
                       int8_t *qs, Q8Scale *scales, void *blocks);
// quant.hip: Q8_0 blocks -> planar form.
int launch_q8_blocks_to_planar(candy_hip_device *dev, const void *blocks, int64_t n_blocks,
                               int8_t *qs, Q8Scale *scales);
// matvec.hip: y[m, rows] for m in 1..15 from planar activations.
int launch_matvec(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs,
                  const Q8Scale *scales, int64_t m, float *y);
// mmq.hip: MFMA tile kernel for m >= 16. half_ws: mmq_m_pad(m) * cols fp16 values of scratch.
int64_t mmq_m_pad(int64_t m);
int launch_mmq(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs,
               const Q8Scale *scales, int64_t m, float *y, void *half_ws);
// Workspace carved for one contraction: planar quants, scales and (m >= 16) fp16 activations.
struct ActWorkspace {
    int8_t *qs;
    Q8Scale *scales;
    void *half_ws;
};
int act_workspace(candy_hip_device *dev, int64_t m, int64_t cols, bool need_quants, ActWorkspace *out);

}  // namespace candy
