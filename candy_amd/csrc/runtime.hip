// Library runtime: error text, device handles, raw memory, timing.
// Stands behind candy.BackendDevice (device.go:49-82) and the storage plumbing of
// candy.BackendStorage (backend.go:4-16).
#include <cstring>

#include "internal.h"

namespace candy {

static thread_local std::string g_last_error;

void set_error(const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
}

int fail(int status, const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return status;
}

FormatInfo format_info(int fmt) {
    switch (fmt) {
    case CANDY_HIP_Q4_0:
    case CANDY_HIP_Q4_0_GGML: return {32, 18};
    case CANDY_HIP_Q8_0: return {32, 34};
    case CANDY_HIP_Q4_K: return {256, 144};
    case CANDY_HIP_Q6_K: return {256, 210};
    case CANDY_HIP_Q4_1:
    case CANDY_HIP_Q4_1_GGML: return {32, 20};
    case CANDY_HIP_Q5_0: return {32, 22};
    case CANDY_HIP_Q5_1: return {32, 24};
    case CANDY_HIP_Q2_K: return {256, 84};
    case CANDY_HIP_Q3_K: return {256, 110};
    case CANDY_HIP_Q5_K: return {256, 176};
    case CANDY_HIP_Q8_K: return {256, 292};
    default: return {0, 0};
    }
}

int use_device(const candy_hip_device *dev) {
    if (!dev) return fail(CANDY_HIP_ERR_INVALID, "device handle is nil");
    CANDY_HIP_TRY(hipSetDevice(dev->ordinal));
    return CANDY_HIP_OK;
}

int check_fault(candy_hip_device *dev) {
    volatile int *f = dev->fault;
    if (f && *f) {
        *f = 0;
        return fail(CANDY_HIP_ERR_INVALID, "an index-select on this device met an id outside its table (indexing.go:8-26 "
                                           "panics there); the rows it selected are not valid");
    }
    return CANDY_HIP_OK;
}

int workspace(candy_hip_device *dev, size_t bytes, void **out) {
    if (bytes > dev->ws_bytes) {
        // Work already enqueued may still read the old buffer.
        CANDY_HIP_TRY(hipStreamSynchronize(dev->stream));
        if (dev->ws) CANDY_HIP_TRY(hipFree(dev->ws));
        dev->ws = nullptr;
        dev->ws_bytes = 0;
        size_t want = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
        CANDY_HIP_TRY(hipMalloc(&dev->ws, want));
        dev->ws_bytes = want;
    }
    *out = dev->ws;
    return CANDY_HIP_OK;
}

int splitk_workspace(candy_hip_device *dev, size_t bytes, void **out) {
    if (bytes > dev->ws_split_bytes) {
        CANDY_HIP_TRY(hipStreamSynchronize(dev->stream));
        if (dev->ws_split) CANDY_HIP_TRY(hipFree(dev->ws_split));
        dev->ws_split = nullptr;
        dev->ws_split_bytes = 0;
        size_t want = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
        CANDY_HIP_TRY(hipMalloc(&dev->ws_split, want));
        dev->ws_split_bytes = want;
    }
    *out = dev->ws_split;
    return CANDY_HIP_OK;
}

__global__ __launch_bounds__(256) void k_zero_bytes(uint8_t *p, size_t bytes) {
    // 16 bytes per thread where aligned, byte stores for the ragged head and tail
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 16;
    if (i >= bytes) return;
    if ((((uintptr_t)p + i) & 15) == 0 && i + 16 <= bytes) {
        *(uint4 *)(p + i) = make_uint4(0, 0, 0, 0);
    } else {
        for (size_t j = i; j < i + 16 && j < bytes; ++j) p[j] = 0;
    }
}

int launch_zero(candy_hip_device *dev, void *dptr, size_t bytes) {
    if (bytes == 0) return CANDY_HIP_OK;
    const size_t threads = (bytes + 15) / 16;
    const size_t grid = (threads + 255) / 256;
    CANDY_REQUIRE(grid <= 0x7FFFFFFF, "buffer too large to zero in one launch");
    hipLaunchKernelGGL(k_zero_bytes, dim3((unsigned)grid), dim3(256), 0, dev->stream, (uint8_t *)dptr, bytes);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

}  // namespace candy

using namespace candy;

extern "C" {

const char *candy_hip_last_error(void) { return g_last_error.c_str(); }

const char *candy_hip_version(void) { return "candy-hip 0.1 (gfx950)"; }

int candy_hip_device_count(int *count) {
    CANDY_REQUIRE(count, "count is nil");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        *count = 0;
        return fail(CANDY_HIP_ERR_HIP, "hipGetDeviceCount failed: %s", hipGetErrorString(e));
    }
    *count = n;
    return CANDY_HIP_OK;
}

int candy_hip_open(int ordinal, candy_hip_device **out) {
    CANDY_REQUIRE(out, "out is nil");
    *out = nullptr;
    int n = 0;
    CANDY_HIP_TRY(hipGetDeviceCount(&n));
    CANDY_REQUIRE(ordinal >= 0 && ordinal < n, "device ordinal %d out of range (have %d)", ordinal, n);
    CANDY_HIP_TRY(hipSetDevice(ordinal));
    hipDeviceProp_t props;
    CANDY_HIP_TRY(hipGetDeviceProperties(&props, ordinal));
    if (strncmp(props.gcnArchName, "gfx950", 6) != 0)
        return fail(CANDY_HIP_ERR_UNSUPPORTED, "device %d is %s; this library holds gfx950 code only", ordinal,
                    props.gcnArchName);
    candy_hip_device *dev = new candy_hip_device();
    dev->ordinal = ordinal;
    dev->num_cus = props.multiProcessorCount;
    snprintf(dev->name, sizeof(dev->name), "%s (%s)", props.name, props.gcnArchName);
    hipError_t e = hipStreamCreateWithFlags(&dev->stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreate(&dev->ev_start);
    if (e == hipSuccess) e = hipEventCreate(&dev->ev_stop);
    if (e == hipSuccess) e = hipHostMalloc((void **)&dev->fault, 64, hipHostMallocDefault);  // pinned: kernels store to it
    if (e == hipSuccess) *dev->fault = 0;
    if (e != hipSuccess) {
        candy_hip_close(dev);
        return fail(CANDY_HIP_ERR_HIP, "creating stream/events failed: %s", hipGetErrorString(e));
    }
    if (int rc = noalloc_scratch_init(dev)) {  // this GPU is current: its copy of the scratch array
        candy_hip_close(dev);
        return rc;
    }
    *out = dev;
    return CANDY_HIP_OK;
}

int candy_hip_close(candy_hip_device *dev) {
    if (!dev) return CANDY_HIP_OK;
    (void)hipSetDevice(dev->ordinal);
    if (dev->stream) (void)hipStreamSynchronize(dev->stream);
    if (dev->ws) (void)hipFree(dev->ws);
    if (dev->ws_split) (void)hipFree(dev->ws_split);
    if (dev->fault) (void)hipHostFree(dev->fault);
    if (dev->ev_start) (void)hipEventDestroy(dev->ev_start);
    if (dev->ev_stop) (void)hipEventDestroy(dev->ev_stop);
    if (dev->stream) (void)hipStreamDestroy(dev->stream);
    delete dev;
    return CANDY_HIP_OK;
}

int candy_hip_device_ordinal(const candy_hip_device *dev, int *ordinal) {
    CANDY_REQUIRE(dev && ordinal, "nil argument");
    *ordinal = dev->ordinal;
    return CANDY_HIP_OK;
}

int candy_hip_device_name(const candy_hip_device *dev, char *buf, size_t buf_len) {
    CANDY_REQUIRE(dev && buf && buf_len > 0, "nil argument");
    snprintf(buf, buf_len, "%s", dev->name);
    return CANDY_HIP_OK;
}

int candy_hip_synchronize(candy_hip_device *dev) {
    if (int rc = use_device(dev)) return rc;
    CANDY_HIP_TRY(hipStreamSynchronize(dev->stream));
    return check_fault(dev);
}

int candy_hip_alloc(candy_hip_device *dev, size_t bytes, void **dptr) {
    CANDY_REQUIRE(dptr, "dptr is nil");
    *dptr = nullptr;
    if (int rc = use_device(dev)) return rc;
    if (bytes == 0) bytes = 1;  // a zero-length storage still gets a distinct address
    CANDY_HIP_TRY(hipMalloc(dptr, bytes));
    return CANDY_HIP_OK;
}

int candy_hip_free(candy_hip_device *dev, void *dptr) {
    if (!dptr) return CANDY_HIP_OK;
    if (int rc = use_device(dev)) return rc;
    CANDY_HIP_TRY(hipStreamSynchronize(dev->stream));  // kernels in flight may still use it
    CANDY_HIP_TRY(hipFree(dptr));
    return CANDY_HIP_OK;
}

int candy_hip_zero(candy_hip_device *dev, void *dptr, size_t bytes) {
    if (bytes == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(dptr, "dptr is nil");
    if (int rc = use_device(dev)) return rc;
    // a fill kernel rather than a memset node: callers may capture this into a HIP graph
    size_t done = 0;
    while (done < bytes) {
        const size_t chunk = bytes - done < (size_t(1) << 36) ? bytes - done : (size_t(1) << 36);
        if (int rc = launch_zero(dev, (uint8_t *)dptr + done, chunk)) return rc;
        done += chunk;
    }
    return CANDY_HIP_OK;
}

int candy_hip_h2d(candy_hip_device *dev, void *dst_dev, const void *src_host, size_t bytes) {
    if (bytes == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(dst_dev && src_host, "nil pointer");
    if (int rc = use_device(dev)) return rc;
    // Pageable host memory: the copy is complete (staged) when this returns, so the caller's
    // buffer is not referenced afterwards.
    CANDY_HIP_TRY(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, dev->stream));
    CANDY_HIP_TRY(hipStreamSynchronize(dev->stream));
    return CANDY_HIP_OK;
}

int candy_hip_d2h(candy_hip_device *dev, void *dst_host, const void *src_dev, size_t bytes) {
    if (bytes == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(dst_host && src_dev, "nil pointer");
    if (int rc = use_device(dev)) return rc;
    CANDY_HIP_TRY(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, dev->stream));
    CANDY_HIP_TRY(hipStreamSynchronize(dev->stream));
    return check_fault(dev);
}

int candy_hip_d2d(candy_hip_device *dev, void *dst_dev, const void *src_dev, size_t bytes) {
    if (bytes == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(dst_dev && src_dev, "nil pointer");
    if (int rc = use_device(dev)) return rc;
    CANDY_HIP_TRY(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, dev->stream));
    return CANDY_HIP_OK;
}

int candy_hip_block_elems(int fmt) { return format_info(fmt).elems; }
int candy_hip_block_bytes(int fmt) { return format_info(fmt).bytes; }

size_t candy_hip_qweight_bytes(int fmt, int64_t rows, int64_t cols) {
    FormatInfo fi = format_info(fmt);
    if (fi.elems == 0 || rows < 0 || cols < 0 || cols % fi.elems != 0) return 0;
    return (size_t)rows * (size_t)(cols / fi.elems) * (size_t)fi.bytes;
}

static int qtensor_check(candy_hip_device *dev, int fmt, int64_t rows, int64_t cols, size_t nbytes, bool exact = true) {
    FormatInfo fi = format_info(fmt);
    CANDY_REQUIRE(dev, "device handle is nil");
    CANDY_REQUIRE(fi.elems != 0, "unknown quantized format %d", fmt);
    CANDY_REQUIRE(rows > 0 && cols > 0, "invalid matrix dimensions %lld x %lld", (long long)rows, (long long)cols);
    CANDY_REQUIRE(cols % fi.elems == 0, "cols %lld is not a multiple of the block size %d", (long long)cols, fi.elems);
    size_t want = candy_hip_qweight_bytes(fmt, rows, cols);
    CANDY_REQUIRE(exact ? nbytes == want : nbytes >= want, "weight has %zu bytes, %lld x %lld blocks of format %d need %zu",
                  nbytes, (long long)rows, (long long)cols, fmt, want);
    return CANDY_HIP_OK;
}

int candy_hip_qtensor_upload(candy_hip_device *dev, int fmt, int64_t rows, int64_t cols, const void *host_blocks,
                             size_t nbytes, candy_hip_qtensor **out) {
    CANDY_REQUIRE(out, "out is nil");
    *out = nullptr;
    if (int rc = qtensor_check(dev, fmt, rows, cols, nbytes)) return rc;
    CANDY_REQUIRE(host_blocks, "host_blocks is nil");
    void *d = nullptr;
    // 64 bytes of slack after the last block: the matvec kernels read whole 16-byte vectors.
    if (int rc = candy_hip_alloc(dev, nbytes + 64, &d)) return rc;
    if (int rc = candy_hip_h2d(dev, d, host_blocks, nbytes)) {
        (void)hipFree(d);
        return rc;
    }
    candy_hip_qtensor *q = new candy_hip_qtensor();
    q->dev = dev; q->fmt = fmt; q->rows = rows; q->cols = cols; q->nbytes = nbytes; q->data = d; q->owned = true;
    q->padded = true;
    *out = q;
    return CANDY_HIP_OK;
}

int candy_hip_qtensor_wrap(candy_hip_device *dev, int fmt, int64_t rows, int64_t cols, void *dev_blocks,
                           size_t nbytes, candy_hip_qtensor **out) {
    CANDY_REQUIRE(out, "out is nil");
    *out = nullptr;
    if (int rc = qtensor_check(dev, fmt, rows, cols, nbytes, /*exact=*/false)) return rc;
    CANDY_REQUIRE(dev_blocks, "dev_blocks is nil");
    CANDY_REQUIRE(((uintptr_t)dev_blocks & 15) == 0, "device blocks must be 16-byte aligned");
    candy_hip_qtensor *q = new candy_hip_qtensor();
    const size_t want = candy_hip_qweight_bytes(fmt, rows, cols);
    q->dev = dev; q->fmt = fmt; q->rows = rows; q->cols = cols; q->nbytes = want; q->data = dev_blocks; q->owned = false;
    q->padded = nbytes >= want + 16;  // room for the widest load that starts inside the last block
    *out = q;
    return CANDY_HIP_OK;
}

int candy_hip_qtensor_free(candy_hip_qtensor *q) {
    if (!q) return CANDY_HIP_OK;
    int rc = CANDY_HIP_OK;
    if (q->owned && q->data) rc = candy_hip_free(q->dev, q->data);
    delete q;
    return rc;
}

int candy_hip_qtensor_info(const candy_hip_qtensor *q, int *fmt, int64_t *rows, int64_t *cols, size_t *nbytes,
                           void **dev_blocks) {
    CANDY_REQUIRE(q, "qtensor is nil");
    if (fmt) *fmt = q->fmt;
    if (rows) *rows = q->rows;
    if (cols) *cols = q->cols;
    if (nbytes) *nbytes = q->nbytes;
    if (dev_blocks) *dev_blocks = q->data;
    return CANDY_HIP_OK;
}

namespace {
struct OptionKey {
    const char *key;
    int candy::Options::*field;
    int lo, hi;
};
// every key of candy_hip_set_option with the range it accepts
const OptionKey OPTION_KEYS[] = {
    {"matvec.span", &candy::Options::matvec_span, 0, 1},
    {"matvec.small_batch_kernel", &candy::Options::small_batch_kernel, 0, 1},
    {"matvec.even_two_rows", &candy::Options::even_two_rows, 0, 1},
    {"mmq.i8_min_m", &candy::Options::i8_min_m, 0, 1 << 20},
    {"mmq.min_m", &candy::Options::mmq_min_m, 16, 1 << 20},
    {"mmq.f16_big_min_m", &candy::Options::f16_big_min_m, 16, 1 << 30},
    {"mmq.f16_api_min_m", &candy::Options::f16_api_min_m, 16, 1 << 30},
    {"mmq.fp16_only", &candy::Options::mmq_fp16_only, 0, 1},
    {"mmq.i8_grid_split", &candy::Options::i8_grid_split, 0, 1},
    {"mmq.f16_shape", &candy::Options::f16_shape, 0, 4},
    {"mmq.f16_split", &candy::Options::f16_split, 0, 16},
    {"mmv.min_m", &candy::Options::mmv_min_m, 2, 32},
    {"mmv.max_m", &candy::Options::mmv_max_m, 0, 32},
    {"mmv.variant", &candy::Options::mmv_variant, 0, 2},
    {"fused.pair_rows", &candy::Options::pair_rows, 0, 32},
    {"fused.rms_rows", &candy::Options::rms_rows, 0, 24},
    {"prefill.qkv_group", &candy::Options::prefill_qkv_group, 0, 1},
    {"prefill.fold_split_sums", &candy::Options::prefill_fold_split_sums, 0, 1},
    {"prefill.attention_valu", &candy::Options::prefill_attention_valu, 0, 1},
    {"llama.graph", &candy::Options::llama_graph, 0, 1},
    {"fused.wide", &candy::Options::fused_wide, 0, 1},
    {"fused.wide_waves", &candy::Options::wide_waves, 8, 16},
    {"fused.down_quant", &candy::Options::down_quant, 0, 1},
    {"prefill.attention_groups", &candy::Options::prefill_attention_groups, 0, 2},
    {"attention.splits", &candy::Options::attn_splits, 0, 64},
};
const OptionKey *find_option(const char *key) {
    for (const OptionKey &k : OPTION_KEYS)
        if (strcmp(k.key, key) == 0) return &k;
    return nullptr;
}
}  // namespace

int candy_hip_set_option(candy_hip_device *dev, const char *key, int64_t value) {
    CANDY_REQUIRE(dev && key, "nil argument");
    const OptionKey *k = find_option(key);
    CANDY_REQUIRE(k, "unknown option \"%s\"", key);
    CANDY_REQUIRE(value >= k->lo && value <= k->hi, "option %s takes %d .. %d, got %lld", key, k->lo, k->hi, (long long)value);
    dev->opt.*(k->field) = (int)value;
    ++dev->opt_epoch;  // decoders notice and capture their step again under the new options
    return CANDY_HIP_OK;
}

int candy_hip_get_option(const candy_hip_device *dev, const char *key, int64_t *value) {
    CANDY_REQUIRE(dev && key && value, "nil argument");
    // read-only: what the handle's grow-only workspaces hold at the moment
    if (strcmp(key, "runtime.workspace_bytes") == 0) { *value = (int64_t)dev->ws_bytes; return CANDY_HIP_OK; }
    if (strcmp(key, "runtime.split_workspace_bytes") == 0) { *value = (int64_t)dev->ws_split_bytes; return CANDY_HIP_OK; }
    const OptionKey *k = find_option(key);
    CANDY_REQUIRE(k, "unknown option \"%s\"", key);
    *value = dev->opt.*(k->field);
    return CANDY_HIP_OK;
}

int candy_hip_timer_start(candy_hip_device *dev) {
    if (int rc = use_device(dev)) return rc;
    CANDY_HIP_TRY(hipEventRecord(dev->ev_start, dev->stream));
    return CANDY_HIP_OK;
}

int candy_hip_timer_stop(candy_hip_device *dev, float *elapsed_ms) {
    CANDY_REQUIRE(elapsed_ms, "elapsed_ms is nil");
    if (int rc = use_device(dev)) return rc;
    CANDY_HIP_TRY(hipEventRecord(dev->ev_stop, dev->stream));
    CANDY_HIP_TRY(hipEventSynchronize(dev->ev_stop));
    CANDY_HIP_TRY(hipEventElapsedTime(elapsed_ms, dev->ev_start, dev->ev_stop));
    return CANDY_HIP_OK;
}

}  // extern "C"
