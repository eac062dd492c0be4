// candy_hip.hpp -- host-side mirror of candy's backend interfaces over libcandy_hip.so.
//
// candy is Go; where no Go toolchain exists this header is the host layer above the C ABI
// (include/candy_hip.h). It keeps candy's names, argument meaning and error behaviour:
//   HipDevice      <- candy.BackendDevice  (device.go:49-82)
//   HipStorage<T>  <- candy.BackendStorage (backend.go:4-238), the methods a Llama block calls
//   Layout / Shape <- candy.Layout (layout.go:10-176), as far as MatMul and the ops need it
//   QTensor/QMatMul <- the quantized Linear built on the operator hook (tensor/ops.go:10-47)
// Every fallible call returns Result<T> = (value, error) like the Go code; error strings follow
// tensor/internal/cpu/storage.go where a CPU counterpart exists.
#pragma once

#include <cstdint>
#include <memory>
#include <numeric>
#include <string>
#include <utility>
#include <vector>

#include "../../include/candy_hip.h"

namespace candy {

struct Error {
    std::string msg;  // empty = nil
    explicit operator bool() const { return !msg.empty(); }
};
inline Error Ok() { return {}; }
inline Error Errorf(std::string m) { return Error{std::move(m)}; }
inline Error Wrap(const std::string &what, const Error &e) { return Error{what + ": " + e.msg}; }  // fmt.Errorf("%w")

template <class T>
struct Result {
    T value{};
    Error err;
    bool ok() const { return !err; }
};

enum class DeviceLocation { Cpu, Gpu, Metal };  // device.go:26-32

// ---------------------------------------------------------------- Layout (layout.go)
class Layout {
public:
    Layout() = default;
    Layout(std::vector<int> dims, std::vector<int> stride, int start) : dims_(std::move(dims)), stride_(std::move(stride)), start_(start) {}
    static Layout Contiguous(std::vector<int> dims) {  // layout.go:30
        std::vector<int> st(dims.size(), 1);
        for (int i = (int)dims.size() - 2; i >= 0; --i) st[i] = st[i + 1] * dims[i + 1];
        return Layout(std::move(dims), std::move(st), 0);
    }
    int Rank() const { return (int)dims_.size(); }
    const std::vector<int> &Dims() const { return dims_; }
    std::vector<int> Stride() const { return stride_; }  // a copy, like layout.go:46-48
    int StartOffset() const { return start_; }
    int Numel() const { return std::accumulate(dims_.begin(), dims_.end(), 1, [](int a, int b) { return a * b; }); }
    bool IsContiguous() const {  // layout.go:134
        int expect = 1;
        for (int i = Rank() - 1; i >= 0; --i) {
            if (dims_[i] != 1 && stride_[i] != expect) return false;
            expect *= dims_[i];
        }
        return true;
    }
    Result<Layout> Transpose(int d1, int d2) const {  // layout.go:160: strides swapped, no copy
        const int r = Rank();
        if (d1 < 0) d1 += r;
        if (d2 < 0) d2 += r;
        if (d1 < 0 || d1 >= r || d2 < 0 || d2 >= r) return {Layout(), Errorf("dimension out of range")};
        Layout l = *this;
        std::swap(l.dims_[d1], l.dims_[d2]);
        std::swap(l.stride_[d1], l.stride_[d2]);
        return {l, Ok()};
    }

private:
    std::vector<int> dims_, stride_;
    int start_ = 0;
};

// ---------------------------------------------------------------- device
inline Error last_error(int status, const char *what) {
    if (status == CANDY_HIP_OK) return Ok();
    return Errorf(std::string(what) + ": " + candy_hip_last_error());
}

class HipDevice {
public:
    static Result<std::shared_ptr<HipDevice>> New(int ordinal) {
        candy_hip_device *h = nullptr;
        if (Error e = last_error(candy_hip_open(ordinal, &h), "open hip device")) return {nullptr, e};
        return {std::shared_ptr<HipDevice>(new HipDevice(h, ordinal)), Ok()};
    }
    ~HipDevice() { candy_hip_close(h_); }
    HipDevice(const HipDevice &) = delete;
    DeviceLocation Location() const { return DeviceLocation::Gpu; }
    bool IsSame(const HipDevice &o) const { return o.ordinal_ == ordinal_; }
    Error Synchronize() { return last_error(candy_hip_synchronize(h_), "synchronize"); }
    Error SetSeed(uint64_t) { return Errorf("cannot seed the HIP rng with set_seed"); }  // as cpu/device.go:49-51
    candy_hip_device *handle() const { return h_; }
    int ordinal() const { return ordinal_; }

private:
    HipDevice(candy_hip_device *h, int o) : h_(h), ordinal_(o) {}
    candy_hip_device *h_;
    int ordinal_;
};
using DevicePtr = std::shared_ptr<HipDevice>;

// ---------------------------------------------------------------- storage
template <class T>
class HipStorage {
public:
    using Ptr = std::shared_ptr<HipStorage<T>>;

    // BackendDevice.StorageFromSlice (device.go:57): alloc + h2d
    static Result<Ptr> FromSlice(const DevicePtr &dev, const std::vector<T> &data) {
        auto r = Alloc(dev, data.size());
        if (!r.ok()) return r;
        if (Error e = last_error(candy_hip_h2d(dev->handle(), r.value->ptr_, data.data(), data.size() * sizeof(T)), "h2d"))
            return {nullptr, e};
        return r;
    }
    // BackendDevice.Alloc / Zeros (device.go:69-72): zero-initialised
    static Result<Ptr> Alloc(const DevicePtr &dev, size_t n) {
        void *p = nullptr;
        if (Error e = last_error(candy_hip_alloc(dev->handle(), n * sizeof(T), &p), "alloc")) return {nullptr, e};
        Ptr s(new HipStorage<T>(dev, p, n));
        if (Error e = last_error(candy_hip_zero(dev->handle(), p, n * sizeof(T)), "zero")) return {nullptr, e};
        return {s, Ok()};
    }
    ~HipStorage() { candy_hip_free(dev_->handle(), ptr_); }
    HipStorage(const HipStorage &) = delete;

    // backend.go:8-9 "Data returns a copy": a device-to-host copy here
    std::vector<T> Data() const {
        std::vector<T> out(n_);
        if (n_) candy_hip_d2h(dev_->handle(), out.data(), ptr_, n_ * sizeof(T));
        return out;
    }
    const DevicePtr &Device() const { return dev_; }  // backend.go:12
    size_t Len() const { return n_; }
    void *ptr() const { return ptr_; }

    Result<Ptr> Clone() const {  // backend.go:6
        auto r = Alloc(dev_, n_);
        if (!r.ok()) return r;
        if (Error e = last_error(candy_hip_d2d(dev_->handle(), r.value->ptr_, ptr_, n_ * sizeof(T)), "d2d")) return {nullptr, e};
        return r;
    }

    // backend.go:78; validation and messages of cpu/storage.go:867-879
    Result<Ptr> MatMul(const Layout *lhsLayout, const Ptr &rhs, const Layout *rhsLayout, int b, int m, int n, int k) const {
        if (!rhs) return {nullptr, Errorf("rhs storage must be HipStorage")};
        if (!lhsLayout || !rhsLayout) return {nullptr, Errorf("layouts cannot be nil")};
        if (m <= 0 || n <= 0 || k <= 0) return {nullptr, Errorf("invalid matrix dimensions")};
        auto out = Alloc(dev_, (size_t)b * m * n);
        if (!out.ok()) return out;
        const float *lp = (const float *)ptr_ + lhsLayout->StartOffset(), *rp = (const float *)rhs->ptr_ + rhsLayout->StartOffset();
        int rc;
        if (lhsLayout->IsContiguous() && rhsLayout->IsContiguous()) {
            rc = candy_hip_matmul_f32(dev_->handle(), lp, rp, (float *)out.value->ptr_, b, m, n, k, 0);
        } else if (b == 1) {
            // one batch through the last two strides of each layout (cpu/storage.go:893-910); Linear's W^T view,
            // strides {1, k} (nn/linear.go:65), is the case on the hot path
            auto ls = lhsLayout->Stride(), rs = rhsLayout->Stride();
            const int lr = lhsLayout->Rank(), rr = rhsLayout->Rank();
            if (lr < 2 || rr < 2) return {nullptr, Errorf("MatMul operands must have at least two dimensions")};
            if (ls[lr - 2] < 0 || ls[lr - 1] < 0 || rs[rr - 2] < 0 || rs[rr - 1] < 0)
                return {nullptr, Errorf("negative strides are not supported on the HIP backend")};
            rc = candy_hip_matmul_f32_strided(dev_->handle(), lp, rp, (float *)out.value->ptr_, m, n, k, ls[lr - 2], ls[lr - 1],
                                              rs[rr - 2], rs[rr - 1]);
        } else {
            // cpu/storage.go:911-926 multiplies such operands as if they were contiguous; that is a wrong answer,
            // not a behaviour to keep
            return {nullptr, Errorf("batched MatMul needs contiguous operands on the HIP backend")};
        }
        if (Error e = last_error(rc, "matmul")) return {nullptr, e};
        return out;
    }

    // backend.go:150; cpu/storage.go:2328-2345
    Result<Ptr> FastRmsNorm(const Layout *layout, const Ptr &alpha, const Layout *alphaLayout, T eps) const {
        if (!layout) return {nullptr, Errorf("layout cannot be nil")};
        if ((size_t)layout->Numel() != n_) return {nullptr, Errorf("layout element count does not match storage size")};
        if (!alpha) return {nullptr, Errorf("alpha must be HIP storage")};
        if (!alphaLayout || !alphaLayout->IsContiguous()) return {nullptr, Errorf("alpha must be contiguous")};
        const int cols = layout->Dims().back();
        auto out = Alloc(dev_, n_);
        if (!out.ok()) return out;
        if (Error e = last_error(candy_hip_rms_norm(dev_->handle(), (const float *)ptr_, (const float *)alpha->ptr_, (float)eps,
                                                    layout->Numel() / cols, cols, (float *)out.value->ptr_), "rms_norm"))
            return {nullptr, e};
        return out;
    }

    // backend.go:159; checks of cpu/storage.go:2502-2546. cos/sin are [t, d/2] or [b, t, d/2].
    Result<Ptr> Rope(const Layout *layout, const Ptr &cos, const Layout *cosLayout, const Ptr &sin, const Layout *sinLayout) const {
        return rope_variant(0, layout, cos, cosLayout, sin, sinLayout);
    }
    // backend.go:156 (adjacent pairs; input [b, h, t, d]); checks of cpu/storage.go:2428-2470
    Result<Ptr> RopeI(const Layout *layout, const Ptr &cos, const Layout *cosLayout, const Ptr &sin, const Layout *sinLayout) const {
        return rope_variant(1, layout, cos, cosLayout, sin, sinLayout);
    }
    // backend.go:162 (input [b, t, h, d]); checks of cpu/storage.go:2577-2620
    Result<Ptr> RopeThd(const Layout *layout, const Ptr &cos, const Layout *cosLayout, const Ptr &sin, const Layout *sinLayout) const {
        return rope_variant(2, layout, cos, cosLayout, sin, sinLayout);
    }

  private:
    Result<Ptr> rope_variant(int variant, const Layout *layout, const Ptr &cos, const Layout *cosLayout, const Ptr &sin,
                             const Layout *sinLayout) const {
        if (!layout) return {nullptr, Errorf("layout cannot be nil")};
        if (!cosLayout) return {nullptr, Errorf("cos layout cannot be nil")};
        if (!sinLayout) return {nullptr, Errorf("sin layout cannot be nil")};
        if (n_ == 0) return {nullptr, Errorf("source storage is empty")};
        if (!cosLayout->IsContiguous()) return {nullptr, Errorf("input cos must be contiguous")};
        if (!sinLayout->IsContiguous()) return {nullptr, Errorf("input sin must be contiguous")};
        if ((size_t)layout->Numel() != n_) return {nullptr, Errorf("layout element count does not match storage size")};
        if (!cos) return {nullptr, Errorf("cos must be HIP storage")};
        if (!sin) return {nullptr, Errorf("sin must be HIP storage")};
        if (layout->Rank() != 4) return {nullptr, Errorf("input must be 4D for RoPE")};
        const int b = layout->Dims()[0];
        const int h = layout->Dims()[variant == 2 ? 2 : 1], t = layout->Dims()[variant == 2 ? 1 : 2], d = layout->Dims()[3];
        const int per_batch = t * d / 2;
        int64_t stride_b = 0;
        if (cosLayout->Numel() == b * per_batch && b > 1) stride_b = (int64_t)h * t * d;  // one table per batch entry
        else if (cosLayout->Numel() != per_batch)
            return {nullptr, Errorf("cos size mismatch: expected " + std::to_string(b * per_batch) + ", got " + std::to_string(cosLayout->Numel()))};
        if (sinLayout->Numel() != cosLayout->Numel())
            return {nullptr, Errorf("sin size mismatch: expected " + std::to_string(cosLayout->Numel()) + ", got " + std::to_string(sinLayout->Numel()))};
        auto out = Alloc(dev_, n_);
        if (!out.ok()) return out;
        const float *x = (const float *)ptr_, *c = (const float *)cos->ptr_, *sn = (const float *)sin->ptr_;
        float *y = (float *)out.value->ptr_;
        int rc;
        if (variant == 0) rc = candy_hip_rope(dev_->handle(), x, c, sn, (int64_t)b * h, (int64_t)t * d, d, stride_b, y);
        else if (variant == 1) rc = candy_hip_rope_i(dev_->handle(), x, c, sn, (int64_t)b * h, (int64_t)t * d, stride_b, y);
        else rc = candy_hip_rope_thd(dev_->handle(), x, c, sn, b, t, h, d, stride_b, y);
        if (Error e = last_error(rc, "rope")) return {nullptr, e};
        return out;
    }

  public:

    // backend.go:147; cpu/storage.go:2304-2325
    Result<Ptr> FastSoftmax(const Layout *layout) const {
        if (!layout) return {nullptr, Errorf("layout cannot be nil")};
        if ((size_t)layout->Numel() != n_) return {nullptr, Errorf("layout element count does not match storage size")};
        const int cols = layout->Dims().back();
        auto out = Alloc(dev_, n_);
        if (!out.ok()) return out;
        if (Error e = last_error(candy_hip_softmax(dev_->handle(), (const float *)ptr_, cols ? layout->Numel() / cols : 0, cols,
                                                   (float *)out.value->ptr_), "softmax"))
            return {nullptr, e};
        return out;
    }

    // backend.go:228
    Result<Ptr> Silu(const Layout *layout) const {
        if (!layout) return {nullptr, Errorf("layout cannot be nil")};
        if ((size_t)layout->Numel() != n_) return {nullptr, Errorf("layout element count does not match storage size")};
        auto out = Alloc(dev_, n_);
        if (!out.ok()) return out;
        if (Error e = last_error(candy_hip_silu(dev_->handle(), (const float *)ptr_, n_, (float *)out.value->ptr_), "silu")) return {nullptr, e};
        return out;
    }

    // backend.go:21, :27 for contiguous same-shape operands
    Result<Ptr> Add(const Ptr &rhs, const Layout *l, const Layout *r, const Layout *res) const { return binary(rhs, l, r, res, true); }
    Result<Ptr> Mul(const Ptr &rhs, const Layout *l, const Layout *r, const Layout *res) const { return binary(rhs, l, r, res, false); }

    // backend.go:129
    Result<std::shared_ptr<HipStorage<uint32_t>>> FastArgmax(const Layout *layout) const {
        using U = HipStorage<uint32_t>;
        if (!layout) return {nullptr, Errorf("layout cannot be nil")};
        if ((size_t)layout->Numel() != n_) return {nullptr, Errorf("layout element count does not match storage size")};
        const int cols = layout->Dims().back();
        const int rows = cols ? layout->Numel() / cols : 0;
        auto out = U::Alloc(dev_, rows);
        if (!out.ok()) return out;
        if (Error e = last_error(candy_hip_argmax(dev_->handle(), (const float *)ptr_, rows, cols, (uint32_t *)out.value->ptr()), "argmax"))
            return {nullptr, e};
        return out;
    }

private:
    template <class U> friend class HipStorage;
    HipStorage(DevicePtr dev, void *p, size_t n) : dev_(std::move(dev)), ptr_(p), n_(n) {}
    Result<Ptr> binary(const Ptr &rhs, const Layout *l, const Layout *r, const Layout *res, bool add) const {
        if (!rhs) return {nullptr, Errorf("rhs storage must be HipStorage")};
        if (!l || !r || !res) return {nullptr, Errorf("layouts cannot be nil")};
        if (!l->IsContiguous() || !r->IsContiguous() || l->Numel() != r->Numel() || (size_t)l->Numel() != n_ || rhs->n_ != n_)
            return {nullptr, Errorf("operands must be contiguous and of the same shape on the HIP backend")};
        auto out = Alloc(dev_, n_);
        if (!out.ok()) return out;
        const int st = add ? candy_hip_add(dev_->handle(), (const float *)ptr_, (const float *)rhs->ptr_, n_, (float *)out.value->ptr_)
                           : candy_hip_mul(dev_->handle(), (const float *)ptr_, (const float *)rhs->ptr_, n_, (float *)out.value->ptr_);
        if (Error e = last_error(st, add ? "add" : "mul")) return {nullptr, e};
        return out;
    }
    DevicePtr dev_;
    void *ptr_;
    size_t n_;
};

// ---------------------------------------------------------------- quantized weight + op
enum class QFormat {
    Q4_0 = CANDY_HIP_Q4_0, Q8_0 = CANDY_HIP_Q8_0, Q4_K = CANDY_HIP_Q4_K, Q6_K = CANDY_HIP_Q6_K, Q4_0_GGML = CANDY_HIP_Q4_0_GGML,
    Q4_1 = CANDY_HIP_Q4_1, Q4_1_GGML = CANDY_HIP_Q4_1_GGML, Q5_0 = CANDY_HIP_Q5_0, Q5_1 = CANDY_HIP_Q5_1,
    Q2_K = CANDY_HIP_Q2_K, Q3_K = CANDY_HIP_Q3_K, Q5_K = CANDY_HIP_Q5_K, Q8_K = CANDY_HIP_Q8_K
};

class QTensor {
public:
    using Ptr = std::shared_ptr<QTensor>;
    // blocks: candy's original block layout (kernels/quantized.go:8-75), row-major
    static Result<Ptr> New(const DevicePtr &dev, QFormat f, int rows, int cols, const std::vector<uint8_t> &blocks) {
        candy_hip_qtensor *h = nullptr;
        if (Error e = last_error(candy_hip_qtensor_upload(dev->handle(), (int)f, rows, cols, blocks.data(), blocks.size(), &h),
                                 "upload quantized weight"))
            return {nullptr, e};
        return {Ptr(new QTensor(dev, h, f, rows, cols)), Ok()};
    }
    // Quantize f32 [rows, cols] on the device into blocks of f (the kernels candy only names,
    // tensor/internal/metal/kernels/kernels.go:563-592); the QTensor owns the block buffer.
    static Result<Ptr> Quantize(const DevicePtr &dev, QFormat f, const HipStorage<float>::Ptr &x, int rows, int cols) {
        if (!x) return {nullptr, Errorf("quantize: input must live on the HIP device")};
        if (rows <= 0 || cols <= 0 || (size_t)rows * cols != x->Len()) return {nullptr, Errorf("quantize: shape mismatch")};
        const size_t nbytes = candy_hip_qweight_bytes((int)f, rows, cols);
        if (nbytes == 0) return {nullptr, Errorf("quantize: cols is not a multiple of the block size")};
        void *blocks = nullptr;
        const size_t room = nbytes + 64;  // spare bytes after the blocks: every tile kernel may take the weight
        if (Error e = last_error(candy_hip_alloc(dev->handle(), room, &blocks), "quantize")) return {nullptr, e};
        int rc = (int)f == CANDY_HIP_Q8_0 ? candy_hip_quantize_q8_0(dev->handle(), (const float *)x->ptr(), rows, cols, blocks)
                                          : candy_hip_quantize(dev->handle(), (int)f, (const float *)x->ptr(), rows, cols, blocks);
        candy_hip_qtensor *h = nullptr;
        if (!rc) rc = candy_hip_qtensor_wrap(dev->handle(), (int)f, rows, cols, blocks, room, &h);
        if (Error e = last_error(rc, "quantize")) {
            candy_hip_free(dev->handle(), blocks);
            return {nullptr, e};
        }
        Ptr q(new QTensor(dev, h, f, rows, cols));
        q->owned_blocks_ = blocks;
        return {q, Ok()};
    }
    ~QTensor() {
        candy_hip_qtensor_free(h_);
        if (owned_blocks_) candy_hip_free(dev_->handle(), owned_blocks_);
    }
    QTensor(const QTensor &) = delete;
    int Rows() const { return rows_; }
    int Cols() const { return cols_; }
    QFormat Format() const { return f_; }

    Result<HipStorage<float>::Ptr> Dequantize() const {
        auto out = HipStorage<float>::Alloc(dev_, (size_t)rows_ * cols_);
        if (!out.ok()) return out;
        if (Error e = last_error(candy_hip_dequantize(dev_->handle(), h_, (float *)out.value->ptr()), "dequantize")) return {nullptr, e};
        return out;
    }

    // The float64 twin of Dequantize (kernels/quantized.go:96-104, 119-128, 139-144: Q4_0, Q4_1, Q8_0 only)
    Result<HipStorage<double>::Ptr> DequantizeF64() const {
        auto out = HipStorage<double>::Alloc(dev_, (size_t)rows_ * cols_);
        if (!out.ok()) return out;
        void *blocks = nullptr;
        if (Error e = last_error(candy_hip_qtensor_info(h_, nullptr, nullptr, nullptr, nullptr, &blocks), "dequantize")) return {nullptr, e};
        const int64_t nb = (int64_t)rows_ * cols_ / candy_hip_block_elems((int)f_);
        if (Error e = last_error(candy_hip_dequantize_blocks_f64(dev_->handle(), (int)f_, blocks, nb, (double *)out.value->ptr()), "dequantize"))
            return {nullptr, e};
        return out;
    }
    // fp16 output (kernels.go:486-505 dequantize_block_*_f16); the storage holds the IEEE half bits
    Result<HipStorage<uint16_t>::Ptr> DequantizeF16() const {
        auto out = HipStorage<uint16_t>::Alloc(dev_, (size_t)rows_ * cols_);
        if (!out.ok()) return out;
        if (Error e = last_error(candy_hip_dequantize_f16(dev_->handle(), h_, out.value->ptr()), "dequantize")) return {nullptr, e};
        return out;
    }
    // y[Rows] = dequantize(W) . x with f32 activations (quantized.cu:1251-1345, :1550-1693, :1810-1911): what the CPU
    // backend's Dequantize + MatMul gives, without the Q8_0 rounding of x that QMatMul carries
    Result<HipStorage<float>::Ptr> DequantizeMulMatVec(const HipStorage<float>::Ptr &x) const {
        if (!x) return {nullptr, Errorf("dmmv: lhs must live on the HIP device")};
        if ((int64_t)x->Len() != cols_) return {nullptr, Errorf("dmmv: shape mismatch, lhs has " + std::to_string(x->Len()) + " values, weight [" +
                                                               std::to_string(rows_) + " " + std::to_string(cols_) + "]")};
        auto out = HipStorage<float>::Alloc(dev_, (size_t)rows_);
        if (!out.ok()) return out;
        if (Error e = last_error(candy_hip_dmmv(dev_->handle(), h_, (const float *)x->ptr(), (float *)out.value->ptr()), "dmmv")) return {nullptr, e};
        return out;
    }

    // y[m, Rows] = x[m, Cols] . W^T; x contiguous f32 on the same device
    Result<HipStorage<float>::Ptr> QMatMul(const HipStorage<float>::Ptr &x, const Layout *xLayout) const {
        if (!x) return {nullptr, Errorf("qmatmul: lhs must live on the HIP device")};
        if (!xLayout) return {nullptr, Errorf("layouts cannot be nil")};
        if (!xLayout->IsContiguous()) return {nullptr, Errorf("qmatmul: lhs must be contiguous")};
        if (xLayout->Rank() < 1 || xLayout->Dims().back() != cols_)
            return {nullptr, Errorf("qmatmul: shape mismatch, lhs last dim " + std::to_string(xLayout->Rank() ? xLayout->Dims().back() : 0) +
                                    ", weight [" + std::to_string(rows_) + " " + std::to_string(cols_) + "]")};
        const int m = xLayout->Numel() / cols_;
        if (m <= 0) return {nullptr, Errorf("invalid matrix dimensions")};
        auto out = HipStorage<float>::Alloc(dev_, (size_t)m * rows_);
        if (!out.ok()) return out;
        if (Error e = last_error(candy_hip_qmatmul(dev_->handle(), h_, (const float *)x->ptr(), m, (float *)out.value->ptr()), "qmatmul"))
            return {nullptr, Wrap("qmatmul", e)};
        return out;
    }

private:
    QTensor(DevicePtr dev, candy_hip_qtensor *h, QFormat f, int r, int c) : dev_(std::move(dev)), h_(h), f_(f), rows_(r), cols_(c) {}
    DevicePtr dev_;
    candy_hip_qtensor *h_;
    QFormat f_;
    int rows_, cols_;
    void *owned_blocks_ = nullptr;
};

}  // namespace candy
