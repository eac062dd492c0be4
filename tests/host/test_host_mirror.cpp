// GPU test of the C++ host mirror (candy_amd/host/candy_hip.hpp) written the way candy's own
// table-driven tests read (tensor/internal/cpu/kernels/*_test.go): expected values come from the
// reference's test vectors or from the CPU oracle on the same seeded inputs.
// Exit code 0 = all checks passed; every failure prints a line.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "../../candy_amd/host/candy_hip.hpp"
#include "../../oracle/candy_oracle.h"

using namespace candy;
using F = HipStorage<float>;

static int g_fail = 0;
#define CHECK(cond, ...)                                  \
    do {                                                  \
        if (!(cond)) {                                    \
            ++g_fail;                                     \
            std::printf("FAIL %s:%d: ", __FILE__, __LINE__); \
            std::printf(__VA_ARGS__);                     \
            std::printf("\n");                            \
        }                                                 \
    } while (0)

static bool close_vec(const std::vector<float> &a, const std::vector<float> &b, double tol) {
    if (a.size() != b.size()) return false;
    for (size_t i = 0; i < a.size(); ++i)
        if (std::fabs((double)a[i] - (double)b[i]) >= tol) return false;
    return true;
}
static double rel_err(const std::vector<float> &got, const std::vector<float> &want) {
    double num = 0, den = 0;
    for (size_t i = 0; i < got.size(); ++i) {
        num = std::fmax(num, std::fabs((double)got[i] - want[i]));
        den = std::fmax(den, std::fabs((double)want[i]));
    }
    return num / den;
}

int main() {
    auto dr = HipDevice::New(0);
    if (!dr.ok()) { std::printf("FAIL open: %s\n", dr.err.msg.c_str()); return 1; }
    DevicePtr dev = dr.value;
    CHECK(dev->Location() == DeviceLocation::Gpu, "location");
    CHECK(dev->IsSame(*dev), "IsSame");
    CHECK((bool)dev->SetSeed(1), "SetSeed must be an error, as on the CPU device");
    CHECK((bool)HipDevice::New(99).err, "opening a missing device must fail");

    // ---- MatMul: conv_test.go:11-65 vectors
    {
        struct Case { const char *name; int m, n, k; std::vector<float> a, b, want; };
        std::vector<Case> cases = {
            {"Basic 2x2", 2, 2, 2, {1, 2, 3, 4}, {5, 6, 7, 8}, {19, 22, 43, 50}},
            {"Dot product", 1, 1, 4, {1, 2, 3, 4}, {4, 3, 2, 1}, {20}},
            {"Random 3x4 from 3x2 * 2x4", 3, 4, 2,
             {0.33669036626815796f, 0.12880940735340118f, 0.23446236550807953f, 0.23033303022384644f, -1.1228563785552979f, -0.18632829189300537f},
             {2.2082014083862305f, -0.637997031211853f, 0.46165722608566284f, 0.2673508822917938f, 0.5349046587944031f, 0.809357225894928f, 1.110290288925171f, -1.6897989511489868f},
             {0.8123809099197388f, -0.11055462807416916f, 0.29845139384269714f, -0.1276475340127945f, 0.6409463286399841f, 0.03683541342616081f, 0.3639777600765228f, -0.326532781124115f, -2.5791609287261963f, 0.5655729174613953f, -0.7252532243728638f, 0.014660704880952835f}},
        };
        for (auto &c : cases) {
            auto a = F::FromSlice(dev, c.a).value, b = F::FromSlice(dev, c.b).value;
            Layout la = Layout::Contiguous({c.m, c.k}), lb = Layout::Contiguous({c.k, c.n});
            auto r = a->MatMul(&la, b, &lb, 1, c.m, c.n, c.k);
            CHECK(r.ok() && close_vec(r.value->Data(), c.want, 1e-6), "MatMul %s", c.name);
        }
        auto a = F::FromSlice(dev, {1, 2, 3, 4}).value;
        Layout l = Layout::Contiguous({2, 2});
        CHECK(a->MatMul(&l, nullptr, &l, 1, 2, 2, 2).err.msg == "rhs storage must be HipStorage", "rhs nil");
        CHECK(a->MatMul(nullptr, a, &l, 1, 2, 2, 2).err.msg == "layouts cannot be nil", "nil layout");  // cpu/storage.go:873-875
        CHECK(a->MatMul(&l, a, &l, 1, 0, 2, 2).err.msg == "invalid matrix dimensions", "m <= 0");       // cpu/storage.go:877-879
    }
    // ---- Linear's call shape (nn/linear.go:58-112): x [m,k] times the transposed view of W [n,k]
    {
        std::mt19937 rng(1);
        std::normal_distribution<float> nd;
        const int m = 3, n = 70, k = 130;
        std::vector<float> x(m * k), w(n * k), want(m * n);
        for (auto &v : x) v = nd(rng);
        for (auto &v : w) v = nd(rng);
        const int64_t as[3] = {0, k, 1}, bs[3] = {0, 1, k}, cs[3] = {0, n, 1};
        co_naive_batched_matmul_strided_f32(1, m, n, k, x.data(), w.data(), want.data(), as, bs, cs);
        auto xs = F::FromSlice(dev, x).value, ws = F::FromSlice(dev, w).value;
        Layout lx = Layout::Contiguous({m, k});
        Layout lwt = Layout::Contiguous({n, k}).Transpose(-1, -2).value;  // dims [k,n], strides {1,k}
        CHECK(!lwt.IsContiguous() && lwt.Stride()[0] == 1 && lwt.Stride()[1] == k, "transpose view");
        auto r = xs->MatMul(&lx, ws, &lwt, 1, m, n, k);
        CHECK(r.ok() && rel_err(r.value->Data(), want) < 1e-5, "Linear-shaped MatMul");
    }
    // ---- other strided views of one batch, with start offsets: a column-major lhs window inside a larger buffer
    //      times a row-strided rhs window (cpu/storage.go:893-910 takes the last two strides; its missing
    //      StartOffset is not reproduced); a batched strided operand is an error, not a silent contiguous read
    {
        std::mt19937 rng(2);
        std::normal_distribution<float> nd;
        const int m = 5, n = 9, k = 17, a_off = 3, b_off = 7;
        std::vector<float> abuf(a_off + k * m + 4), bbuf(b_off + k * (2 * n) + 4), want(m * n);
        for (auto &v : abuf) v = nd(rng);
        for (auto &v : bbuf) v = nd(rng);
        // a[i, l] at a_off + i + l * m (strides {1, m}); b[l, j] at b_off + l * 2n + j * 2 (strides {2n, 2})
        const int64_t as[3] = {0, 1, m}, bs[3] = {0, 2 * n, 2}, cs[3] = {0, n, 1};
        co_naive_batched_matmul_strided_f32(1, m, n, k, abuf.data() + a_off, bbuf.data() + b_off, want.data(), as, bs, cs);
        auto sa = F::FromSlice(dev, abuf).value, sb = F::FromSlice(dev, bbuf).value;
        Layout la({m, k}, {1, m}, a_off), lb({k, n}, {2 * n, 2}, b_off);
        auto r = sa->MatMul(&la, sb, &lb, 1, m, n, k);
        CHECK(r.ok() && r.value->Data() == want, "strided MatMul with start offsets equals the CPU loop bit for bit");
        Layout l3({2, m, k}, {m * k, 1, m}, 0), r3 = Layout::Contiguous({2, k, n});
        CHECK(sa->MatMul(&l3, sb, &r3, 2, m, n, k).err.msg == "batched MatMul needs contiguous operands on the HIP backend",
              "batched strided MatMul is refused");
    }
    // ---- FastRmsNorm: reduce_test.go:1909-1971
    {
        auto x = F::FromSlice(dev, {1, 2, 3, 4, 5, 6}).value;
        auto alpha = F::FromSlice(dev, {0.5f, 0.5f, 0.5f}).value;
        Layout l = Layout::Contiguous({2, 3}), la = Layout::Contiguous({3});
        auto r = x->FastRmsNorm(&l, alpha, &la, 1e-5f);
        CHECK(r.ok() && close_vec(r.value->Data(), {0.2314547747373581f, 0.4629095494747162f, 0.6943643093109131f, 0.39477095007896423f, 0.4934636950492859f, 0.5921564102172852f}, 1e-6), "FastRmsNorm with alpha");
        CHECK(x->FastRmsNorm(nullptr, alpha, &la, 1e-5f).err.msg == "layout cannot be nil", "rmsnorm nil layout");
        Layout bad = Layout::Contiguous({7});
        CHECK(x->FastRmsNorm(&bad, alpha, &la, 1e-5f).err.msg == "layout element count does not match storage size", "rmsnorm size");
    }
    // ---- Rope: reduce_test.go:2775-2832 (first case) as a [1,1,1,4] tensor
    {
        auto x = F::FromSlice(dev, {1, 2, 3, 4}).value;
        auto c = F::FromSlice(dev, {1, 0}).value, s = F::FromSlice(dev, {0, 1}).value;
        Layout l = Layout::Contiguous({1, 1, 1, 4}), lc = Layout::Contiguous({1, 2});
        auto r = x->Rope(&l, c, &lc, s, &lc);
        CHECK(r.ok() && close_vec(r.value->Data(), {1, -4, 3, 2}, 1e-6), "Rope");
        Layout l3 = Layout::Contiguous({1, 1, 4});
        CHECK(x->Rope(&l3, c, &lc, s, &lc).err.msg == "input must be 4D for RoPE", "rope rank");
        Layout lbad = Layout::Contiguous({3});
        auto c3 = F::FromSlice(dev, {1, 0, 1}).value;
        CHECK(x->Rope(&l, c3, &lbad, s, &lc).err.msg.rfind("cos size mismatch", 0) == 0, "rope cos size");
    }
    // ---- RopeI / RopeThd: reduce_test.go:2507-2560 and 3033-3094 (first and second cases)
    {
        auto c = F::FromSlice(dev, {1, 0}).value, s = F::FromSlice(dev, {0, 1}).value;
        Layout l = Layout::Contiguous({1, 1, 1, 4}), lc = Layout::Contiguous({1, 2});
        auto xi = F::FromSlice(dev, {1, 3, 2, 4}).value;
        auto ri = xi->RopeI(&l, c, &lc, s, &lc);
        CHECK(ri.ok() && close_vec(ri.value->Data(), {1, 3, -4, 2}, 1e-6), "RopeI");
        auto xt = F::FromSlice(dev, {1, 2, 3, 4, 5, 6, 7, 8}).value;
        auto c2 = F::FromSlice(dev, {1, 0, 0.5f, 0.5f}).value, s2 = F::FromSlice(dev, {0, 1, 0.5f, 0.5f}).value;
        Layout lt = Layout::Contiguous({1, 2, 1, 4}), lc2 = Layout::Contiguous({2, 2});
        auto rt = xt->RopeThd(&lt, c2, &lc2, s2, &lc2);
        CHECK(rt.ok() && close_vec(rt.value->Data(), {1, -4, 3, 2, -1, -1, 6, 7}, 1e-6), "RopeThd");
        Layout l3 = Layout::Contiguous({1, 1, 4});
        CHECK(xi->RopeI(&l3, c, &lc, s, &lc).err.msg == "input must be 4D for RoPE", "rope_i rank");
    }
    // ---- FastSoftmax / Silu / Add / Mul / FastArgmax
    {
        auto x = F::FromSlice(dev, {1, 2, 3, 4, 5, 6}).value;
        Layout l = Layout::Contiguous({2, 3});
        CHECK(close_vec(x->FastSoftmax(&l).value->Data(), {0.09003057f, 0.24472848f, 0.66524094f, 0.09003057f, 0.24472848f, 0.66524094f}, 1e-6), "FastSoftmax");
        auto y = F::FromSlice(dev, {0, 1, -1}).value;
        Layout l3 = Layout::Contiguous({3});
        CHECK(close_vec(y->Silu(&l3).value->Data(), {0.0f, (float)(1 / (1 + std::exp(-1.0))), (float)(-1 / (1 + std::exp(1.0)))}, 1e-6), "Silu");
        auto a = F::FromSlice(dev, {1.5f, -2, 3}).value, b = F::FromSlice(dev, {0.25f, 4, -1}).value;
        CHECK(close_vec(a->Add(b, &l3, &l3, &l3).value->Data(), {1.75f, 2, 2}, 0.0 + 1e-12), "Add");
        CHECK(close_vec(a->Mul(b, &l3, &l3, &l3).value->Data(), {0.375f, -8, -3}, 0.0 + 1e-12), "Mul");
        auto am = F::FromSlice(dev, {3, 3, 2, 4}).value;
        Layout l22 = Layout::Contiguous({2, 2});
        auto idx = am->FastArgmax(&l22).value->Data();
        CHECK(idx.size() == 2 && idx[0] == 0 && idx[1] == 1, "FastArgmax ties take the first");
        auto cl = a->Clone().value->Data();
        CHECK(cl == a->Data(), "Clone");
    }
    // ---- QTensor / QMatMul against the CPU oracle on the same bytes
    {
        std::mt19937 rng(7);
        std::normal_distribution<float> nd;
        struct Fm { QFormat f; int id; } fmts[] = {{QFormat::Q4_K, CO_Q4_K}, {QFormat::Q8_0, CO_Q8_0}, {QFormat::Q6_K, CO_Q6_K}, {QFormat::Q4_0, CO_Q4_0}};
        for (auto fm : fmts) {
            const int rows = 96, cols = 1024;
            const size_t nbytes = (size_t)rows * (cols / co_block_elems(fm.id)) * co_block_bytes(fm.id);
            std::vector<uint8_t> blocks(nbytes);
            for (auto &v : blocks) v = (uint8_t)(rng() & 0xFF);
            // sane fp16 scales: overwrite the d (and dmin) fields with small positive halves
            const int bs = co_block_bytes(fm.id);
            for (size_t b = 0; b < nbytes / bs; ++b) {
                uint16_t d = co_f32_to_fp16(0.01f + 0.01f * (float)(rng() % 100) / 100.f);
                uint8_t *p = blocks.data() + b * bs;
                if (fm.id == CO_Q6_K) std::memcpy(p + 208, &d, 2);
                else { std::memcpy(p, &d, 2); if (fm.id == CO_Q4_K) std::memcpy(p + 2, &d, 2); }
            }
            auto q = QTensor::New(dev, fm.f, rows, cols, blocks);
            CHECK(q.ok(), "QTensor::New");
            // dequantize: bit-exact
            std::vector<float> want_dq((size_t)rows * cols);
            co_dequantize(fm.id, blocks.data(), rows * cols / co_block_elems(fm.id), want_dq.data());
            auto dq = q.value->Dequantize().value->Data();
            CHECK(std::memcmp(dq.data(), want_dq.data(), dq.size() * 4) == 0, "Dequantize bit-exact fmt %d", fm.id);
            {   // the other outputs: float64 where the CPU kernels have a twin (for these formats it is the f32 value
                // widened: an fp16 scale times at most 8 bits is exact in both), fp16 = the f32 value rounded once
                auto d64 = q.value->DequantizeF64();
                if (fm.id == CO_Q8_0 || fm.id == CO_Q4_0) {
                    bool same = d64.ok();
                    if (same) { auto v = d64.value->Data(); for (size_t i = 0; i < v.size() && same; ++i) same = v[i] == (double)want_dq[i]; }
                    CHECK(same, "DequantizeF64 fmt %d", fm.id);
                } else {
                    CHECK(!d64.ok(), "DequantizeF64 refuses fmt %d", fm.id);
                }
                auto h16 = q.value->DequantizeF16();
                bool same = h16.ok();
                if (same) { auto v = h16.value->Data(); for (size_t i = 0; i < v.size() && same; ++i) same = v[i] == co_f32_to_fp16(want_dq[i]); }
                CHECK(same, "DequantizeF16 fmt %d", fm.id);
                // f32-activation matvec against Dequantize + the naive loop
                std::vector<float> x1(cols), want1(rows);
                for (auto &v : x1) v = nd(rng);
                for (int r = 0; r < rows; ++r) { float a = 0; for (int k = 0; k < cols; ++k) a += want_dq[(size_t)r * cols + k] * x1[k]; want1[r] = a; }
                auto y1 = q.value->DequantizeMulMatVec(F::FromSlice(dev, x1).value);
                CHECK(y1.ok() && rel_err(y1.value->Data(), want1) <= 2e-5, "DequantizeMulMatVec fmt %d", fm.id);
            }
            for (int m : {1, 5, 32}) {
                std::vector<float> x((size_t)m * cols), want((size_t)m * rows);
                for (auto &v : x) v = nd(rng);
                co_qmatmul(fm.id, blocks.data(), rows, cols, x.data(), m, want.data());
                auto xs = F::FromSlice(dev, x).value;
                Layout lx = Layout::Contiguous({m, cols});
                auto y = q.value->QMatMul(xs, &lx);
                CHECK(y.ok() && rel_err(y.value->Data(), want) <= 1e-3, "QMatMul fmt %d m %d", fm.id, m);  // the 1e-3 bar
            }
            Layout lbad = Layout::Contiguous({2, 512});
            auto xs = F::FromSlice(dev, std::vector<float>(1024)).value;
            CHECK(q.value->QMatMul(xs, &lbad).err.msg.rfind("qmatmul: shape mismatch", 0) == 0, "qmatmul shape error");
        }
        CHECK((bool)QTensor::New(dev, QFormat::Q4_K, 4, 100, std::vector<uint8_t>(10)).err, "cols not a multiple of the block");
        // ---- QTensor::Quantize: the device's blocks dequantize to what the CPU restatement's blocks do, bit for bit
        struct Qm { QFormat f; int id; } qfm[] = {{QFormat::Q4_0, CO_Q4_0}, {QFormat::Q8_0, CO_Q8_0}, {QFormat::Q4_K, CO_Q4_K}, {QFormat::Q6_K, CO_Q6_K}};
        for (auto fm : qfm) {
            const int rows = 6, cols = 768;
            std::vector<float> xw((size_t)rows * cols);
            for (auto &v : xw) v = 0.02f * nd(rng);
            std::vector<uint8_t> cpu_blocks((size_t)rows * (cols / co_block_elems(fm.id)) * co_block_bytes(fm.id));
            CHECK(co_quantize(fm.id, xw.data(), rows, cols, cpu_blocks.data()) == 0, "co_quantize fmt %d", fm.id);
            std::vector<float> want((size_t)rows * cols);
            co_dequantize(fm.id, cpu_blocks.data(), rows * cols / co_block_elems(fm.id), want.data());
            auto q = QTensor::Quantize(dev, fm.f, F::FromSlice(dev, xw).value, rows, cols);
            CHECK(q.ok(), "QTensor::Quantize fmt %d", fm.id);
            if (q.ok()) {
                auto got = q.value->Dequantize().value->Data();
                CHECK(std::memcmp(got.data(), want.data(), got.size() * 4) == 0, "Quantize -> Dequantize bit-exact fmt %d", fm.id);
            }
        }
        CHECK((bool)QTensor::Quantize(dev, QFormat::Q4_K, F::FromSlice(dev, std::vector<float>(300)).value, 3, 100).err, "quantize: cols off the block");
    }
    CHECK(!dev->Synchronize(), "Synchronize");
    std::printf(g_fail ? "host mirror: %d check(s) FAILED\n" : "host mirror: all checks passed\n", g_fail);
    return g_fail ? 1 : 0;
}
