// HipQ8Backend implementation: routing, scratch ownership and error reporting
// around the qw3::ported launchers.  Mirrors the reference's CUDA backend for
// these ops (src/kernels_cuda.cu, lines cited per function).
//
// Deviations from the reference's routing, all inside what it allows a backend
// to choose:
//   * q8_0_matmul with batch == 8 stays on the GEMV (Q8_1 activations); the
//     reference sends exactly batch 8 to its MMA tile with the D4 quantizer
//     (src/kernels_cuda.cu:12598-12629) while every other batch <= 8 entry point
//     uses the GEMV.  Here all batch <= 8 routes agree.
//   * q8_0_matvec_fanout fuses up to four weights into one launch at batch 1
//     (the reference pairs only same-shape neighbours, :11261-11290).
//   * batch-1 ops on rows of at most 8192 columns run as one launch that quantizes the
//     activations inside the GEMV; the outputs are the same bits as the two-step form.
//   * rms_norm sums the squares in a fixed order and takes an IEEE root (the reference's order
//     follows its block size and its root is rsqrtf); rms_norm_q8_0_matmul_fanout fuses the norm
//     into the quantizer (batch <= 8) or into the GEMV itself (batch 1) for Q8_0 weights, where
//     the reference runs rms_norm_batch and q8_0_matmul_fanout one after the other.
//   * strided batch > 8 (in_stride != cols or out_stride != rows), which the
//     reference serves with a legacy kernel outside this path, runs as GEMV
//     slices of eight rows.
//   * q8_0_matmul_silu_mul is served for Q8_0 (the reference declines it and the executor
//     falls back to two matmuls and silu_mul_n); q8_0_matmul_add above eight rows and bf16
//     outputs of q8_0_matmul take the tile kernel's fused store where it has one.
//   * a norm and the projections that read its output share work: rms_norm / rms_norm_batch of
//     up to eight rows also leave the rows' Q8_1 blocks in the scratch, and the operator called
//     next reads them instead of quantizing again; a one-row rms_norm is held back one call and
//     runs inside the GEMV when that call is a batch-1 projection of its output (PendingNorm
//     in the header); an fp32 add / add_n is held back one call and runs inside the rms_norm_batch
//     of its sum when that is the next call (PendingAdd).  Same bits either way.
#include "hip_q8_backend.hpp"

#include <cstdio>
#include <cstring>

#include "qw3_ported.hpp"

namespace qw3 {
namespace {

thread_local char g_msg[256];

using OwnerRef = std::shared_ptr<HipQ8Backend::Owner>;
void tell_owner(const OwnerRef &owner, const void *ptr) {
    if (owner && owner->backend && ptr) owner->backend->released(ptr);
}

struct HipTensor final : DeviceTensor {
    void *ptr = nullptr;
    OwnerRef owner;
    ~HipTensor() override {
        tell_owner(owner, ptr);
        if (ptr) (void)hipFree(ptr);
    }
    float *f32() const { return static_cast<float *>(ptr); }
    uint16_t *bf16() const { return static_cast<uint16_t *>(ptr); }
    bool is_bf16() const { return dtype == DeviceTensorDType::BF16; }
};

struct HipWeight final : DeviceWeight {
    uint8_t *ptr = nullptr;
    uint64_t bytes = 0;
    OwnerRef owner;
    ~HipWeight() override {
        tell_owner(owner, ptr);
        if (ptr) (void)hipFree(ptr);
    }
};

struct HipArgmaxBuffer final : DeviceArgmaxBuffer {
    q8mi_argmax_pair *ptr = nullptr;
    ~HipArgmaxBuffer() override {
        if (ptr) (void)hipFree(ptr);
    }
};

const HipTensor &T(const DeviceTensor &t) { return static_cast<const HipTensor &>(t); }
HipTensor &T(DeviceTensor &t) { return static_cast<HipTensor &>(t); }
const HipWeight &W(const DeviceWeight &w) { return static_cast<const HipWeight &>(w); }

DeviceStatus hip_status(hipError_t e, const char *where) {
    if (e == hipSuccess) return {};
    std::snprintf(g_msg, sizeof(g_msg), "%s: %s", where, hipGetErrorString(e));
    return {false, g_msg};
}

std::unique_ptr<DeviceTensor> make_tensor(uint64_t count, uint32_t elem_size, DeviceTensorDType dtype, const OwnerRef &owner) {
    auto t = std::make_unique<HipTensor>();
    t->owner = owner;
    t->count = count;
    t->elem_size = elem_size;
    t->dtype = dtype;
    if (hipMalloc(&t->ptr, count ? count * elem_size : 1) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return t;
}

}  // namespace

HipQ8Backend::HipQ8Backend() : owner_(std::make_shared<Owner>()) {
    owner_->backend = this;
    (void)hipSetDevice(0);
    // one non-blocking exec stream at the default priority (src/kernels_cuda.cu:9675-9679)
    (void)hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking);
}

HipQ8Backend::~HipQ8Backend() {
    owner_->backend = nullptr;   // tensors and weights that outlive the backend have nobody to tell
    if (stream_) (void)hipStreamSynchronize(stream_);
    for (Scratch *s : {&q8_1_, &d4_, &argmax_partial_, &argmax_result_, &lm_head_, &lm_rows_, &out_f32_, &row_ids_}) {
        if (s->ptr) (void)hipFree(s->ptr);
    }
    if (argmax_dev_) (void)hipFree(argmax_dev_);
    if (lm_host_) (void)hipHostFree(lm_host_);
    if (argmax_host_) (void)hipHostFree(argmax_host_);
    if (graph_exec_) (void)hipGraphExecDestroy(graph_exec_);
    if (graph_) (void)hipGraphDestroy(graph_);
    if (stream_) (void)hipStreamDestroy(stream_);
}

DeviceStatus HipQ8Backend::end() { return synchronize(); }

DeviceStatus HipQ8Backend::synchronize() {
    if (auto st = flush_norm(); !st.ok) return st;
    return hip_status(hipStreamSynchronize(stream_), "hip synchronize");
}

// ---- graph capture (src/kernels_cuda.cu:9958-9980) -------------------------------
bool HipQ8Backend::begin_capture() {
    if (capturing_) return false;
    if (!flush_norm().ok) return false;   // a norm from before the capture runs before it
    if (hipStreamBeginCapture(stream_, hipStreamCaptureModeThreadLocal) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    capturing_ = true;
    return true;
}

DeviceStatus HipQ8Backend::end_capture() {
    if (!capturing_) return {false, "end_capture without begin_capture"};
    const DeviceStatus flushed = flush_norm();   // a norm still held back belongs to the graph
    capturing_ = false;
    if (graph_exec_) { (void)hipGraphExecDestroy(graph_exec_); graph_exec_ = nullptr; }
    if (graph_) { (void)hipGraphDestroy(graph_); graph_ = nullptr; }
    if (auto st = hip_status(hipStreamEndCapture(stream_, &graph_), "hip end capture"); !st.ok) return st;
    if (!flushed.ok) return flushed;
    return hip_status(hipGraphInstantiate(&graph_exec_, graph_, nullptr, nullptr, 0), "hip graph instantiate");
}

DeviceStatus HipQ8Backend::replay_graph() {
    if (!graph_exec_) return {false, "replay_graph: nothing captured"};
    if (auto st = flush_norm(); !st.ok) return st;   // eager work still held back comes before the graph
    return hip_status(hipGraphLaunch(graph_exec_, stream_), "hip graph launch");
}

// ---- tensors / weights -------------------------------------------------------------
// (A new tensor may reuse the address of a freed one: whatever the scratch holds for that address is stale.)
std::unique_ptr<DeviceTensor> HipQ8Backend::tensor_f32(uint64_t count, const char *) {
    forget_quantized();
    return make_tensor(count, 4, DeviceTensorDType::F32, owner_);
}

std::unique_ptr<DeviceTensor> HipQ8Backend::tensor_bf16(uint64_t count, const char *) {
    forget_quantized();
    return make_tensor(count, 2, DeviceTensorDType::BF16, owner_);
}

std::unique_ptr<DeviceWeight> HipQ8Backend::weight_f32(const float *data, uint64_t count, const char *) {
    auto w = std::make_unique<HipWeight>();
    w->owner = owner_;
    w->rows = 1;
    w->cols = count;
    w->format = DeviceWeightFormat::F32;
    w->bytes = count * 4;
    if (hipMalloc(reinterpret_cast<void **>(&w->ptr), w->bytes ? w->bytes : 1) != hipSuccess ||
        hipMemcpy(w->ptr, data, w->bytes, hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return w;
}

// src/kernels_cuda.cu:1566-1594, 10158-10160: repack on the host, one upload
std::unique_ptr<DeviceWeight> HipQ8Backend::weight_q8_0(const void *data, uint64_t rows, uint64_t cols,
                                                        const char *) {
    if (cols % 32 != 0) return nullptr;
    auto w = std::make_unique<HipWeight>();
    w->owner = owner_;
    w->rows = rows;
    w->cols = cols;
    w->format = DeviceWeightFormat::Q8_0;
    w->bytes = rows * (cols / 32) * 34;
    std::vector<uint8_t> staged(w->bytes);
    if (q8mi_repack_q8_0_split_host(data, rows, cols, staged.data()) != Q8MI_OK) return nullptr;
    if (hipMalloc(reinterpret_cast<void **>(&w->ptr), w->bytes ? w->bytes : 1) != hipSuccess ||
        hipMemcpy(w->ptr, staged.data(), w->bytes, hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return w;
}

DeviceStatus HipQ8Backend::copy_bytes_from_host(DeviceTensor &x, uint64_t byte_offset, const void *host,
                                                uint64_t bytes) {
    auto &t = T(x);
    if (byte_offset + bytes > t.count * t.elem_size) return {false, "copy_bytes_from_host out of range"};
    if (auto st = flush_norm(); !st.ok) return st;
    forget_quantized();
    if (auto st = hip_status(hipMemcpyAsync(static_cast<uint8_t *>(t.ptr) + byte_offset, host, bytes,
                                            hipMemcpyHostToDevice, stream_), "copy_bytes_from_host"); !st.ok)
        return st;
    return synchronize();
}

DeviceStatus HipQ8Backend::copy_bytes_to_host(const DeviceTensor &x, void *host, uint64_t byte_offset,
                                              uint64_t bytes) {
    const auto &t = T(x);
    if (byte_offset + bytes > t.count * t.elem_size) return {false, "copy_bytes_to_host out of range"};
    if (auto st = flush_norm(); !st.ok) return st;
    if (auto st = hip_status(hipMemcpyAsync(host, static_cast<const uint8_t *>(t.ptr) + byte_offset, bytes,
                                            hipMemcpyDeviceToHost, stream_), "copy_bytes_to_host"); !st.ok)
        return st;
    return synchronize();
}

DeviceStatus HipQ8Backend::copy_to_host(const DeviceTensor &x, float *host, uint64_t offset, uint64_t count) {
    if (T(x).dtype != DeviceTensorDType::F32) return {false, "copy_to_host expects an fp32 tensor"};
    return copy_bytes_to_host(x, host, offset * 4, count * 4);
}

DeviceStatus HipQ8Backend::zero_tensor(DeviceTensor &x) {
    auto &t = T(x);
    // memset nodes are kept out of captured graphs
    if (capturing_) return {false, "zero_tensor is not available during graph capture"};
    if (auto st = flush_norm(); !st.ok) return st;
    forget_quantized();
    return hip_status(hipMemsetAsync(t.ptr, 0, t.count * t.elem_size, stream_), "zero_tensor");
}

// ---- helpers -------------------------------------------------------------------------
// grow-only scratch (src/kernels_cuda.cu:14479-14507)
DeviceStatus HipQ8Backend::ensure(Scratch &s, size_t need, const char *what) {
    if (need <= s.capacity) return {};
    if (capturing_) return {false, "scratch would grow during graph capture: run the op eagerly once first"};
    if (&s == &q8_1_) forget_quantized();
    if (s.ptr) {
        (void)hipStreamSynchronize(stream_);
        (void)hipFree(s.ptr);
        s.ptr = nullptr;
        s.capacity = 0;
    }
    if (auto st = hip_status(hipMalloc(&s.ptr, need), what); !st.ok) return st;
    s.capacity = need;
    return {};
}

DeviceStatus HipQ8Backend::launch_status(const char *where) { return hip_status(hipGetLastError(), where); }

DeviceStatus HipQ8Backend::failed(const char *where) {
    std::snprintf(g_msg, sizeof(g_msg), "%s: %s", where, q8mi_last_error());
    (void)hipGetLastError();
    return {false, g_msg};
}

// The Q8_1 blocks of `batch` rows at x, in the scratch: quantized now, unless the norm that wrote
// those rows has left them there already.
DeviceStatus HipQ8Backend::quantize_q8_1(const float *x, uint32_t batch, uint32_t cols, uint32_t stride) {
    if (quantized_.src == x && quantized_.batch == batch && quantized_.cols == cols && quantized_.stride == stride)
        return {};
    forget_quantized();
    if (auto st = ensure(q8_1_, ported::q8_1_scratch_bytes(batch, cols), "q8_1 scratch alloc"); !st.ok) return st;
    if (!ported::launch_quantize_q8_1(x, q8_1_.ptr, batch, cols, stride, stream_))
        return failed("quantize_q8_1");
    return {};
}

// Runs the norm that rms_norm_batch held back, with the quantizer in the same pass.
DeviceStatus HipQ8Backend::flush_add() {
    if (!pending_add_.active) return {};
    const PendingAdd p = pending_add_;
    pending_add_.active = false;
    if (q8mi_add(p.out, p.a, p.b, p.count, 0, stream_) != Q8MI_OK) return failed("add");
    return launch_status("hip add");
}

DeviceStatus HipQ8Backend::flush_norm() {
    if (auto st = flush_add(); !st.ok) return st;
    if (!pending_.active) return {};
    const PendingNorm n = pending_;
    pending_.active = false;
    forget_quantized();
    if (auto st = ensure(q8_1_, ported::q8_1_scratch_bytes(1, n.cols), "q8_1 scratch alloc"); !st.ok) return st;
    if (q8mi_rms_norm_quantize_q8_1(n.x, n.weight, n.out, q8_1_.ptr, 1, n.cols, n.cols, n.cols, n.eps, stream_) != Q8MI_OK)
        return failed("rms_norm_quantize_q8_1");
    quantized_ = QuantizedRows{n.out, 1, n.cols, n.cols};
    return launch_status("hip rms_norm");
}

void HipQ8Backend::released(const void *ptr) {
    if (ptr == quantized_.src) forget_quantized();
    if (pending_add_.active) {
        if (ptr == pending_add_.out) pending_add_.active = false;   // nobody can read the sum any more
        else if (ptr == pending_add_.a || ptr == pending_add_.b) (void)flush_add();
    }
    if (!pending_.active) return;
    if (ptr == pending_.out) pending_.active = false;
    else if (ptr == pending_.x || ptr == pending_.weight) (void)flush_norm();
}

// Whether a batch-1 projection of x (cols floats) whose first output is out0 can run the held-back
// norm inside its own launch: x is that norm's output, and the launch writes neither the norm's
// input (every workgroup reads it) nor its output (workgroup 0 writes it).
bool HipQ8Backend::absorbs_norm(const float *x, uint32_t cols, const void *out0) const {
    return pending_.active && x == pending_.out && cols == pending_.cols && out0 != pending_.x && out0 != pending_.out;
}

// Batch 1 on rows of up to 8192 columns: one launch that quantizes the activations inside the GEMV
// (measured on MI355X: 10.2 against 3.3 + 9.3 us for the QKV fan-out, 9.3 against 3.3 + 7.8 us for the O
// projection).  Longer rows (the down projection's 17408 columns) and batches above 1 are faster
// with the stand-alone quantizer in front (3.5 + 18.0 against 23.7 us).  The fused entry point may
// still decline a shape; the two-step form below then runs.  Rows whose Q8_1 blocks a norm has
// already left in the scratch take the two-step form without its first step.
bool HipQ8Backend::fuse_quantizer(const float *x, uint32_t batch, uint32_t cols, uint32_t stride) const {
    if (quantized_.src == x && quantized_.batch == batch && quantized_.cols == cols && quantized_.stride == stride)
        return false;
    return batch == 1 && cols % 256 == 0 && cols <= 8192;
}

// dispatch_q8_matvec, src/kernels_cuda.cu:14617-14658: any batch as GEMV slices of <= 8 rows
DeviceStatus HipQ8Backend::gemv_route(float *out, const DeviceWeight &weight, const float *x, uint32_t batch,
                                      uint32_t in_stride, uint32_t out_stride) {
    const auto &w = W(weight);
    const uint32_t cols = static_cast<uint32_t>(w.cols), rows = static_cast<uint32_t>(w.rows);
    const uint32_t xs = (batch == 1 && in_stride == 0) ? cols : in_stride;
    const uint32_t os = (batch == 1 && out_stride == 0) ? rows : out_stride;
    if (fuse_quantizer(x, batch, cols, xs) &&
        q8mi_qgemv(w.ptr, x, xs, out, 0, rows, cols, 1, os, stream_) == Q8MI_OK)
        return launch_status("hip q8_0_matvec fused");
    for (uint32_t j0 = 0; j0 < batch; j0 += 8) {
        const uint32_t m = batch - j0 < 8 ? batch - j0 : 8;
        if (auto st = quantize_q8_1(x + static_cast<uint64_t>(j0) * xs, m, cols, xs); !st.ok) return st;
        if (!ported::launch_mmvq_q8_0(w.ptr, q8_1_.ptr, out + static_cast<uint64_t>(j0) * os, rows, cols, m, os,
                                      stream_))
            return failed("mmvq_q8_0");
    }
    return launch_status("hip q8_0_matvec");
}

// D4 records of `batch` rows of x in the scratch (src/kernels_cuda.cu:14493-14507)
DeviceStatus HipQ8Backend::quantize_d4(const float *x, uint32_t batch, uint32_t cols, uint32_t stride) {
    if (auto st = ensure(d4_, ported::q8_1_mmq_scratch_bytes(batch, cols), "q8_1_mmq scratch alloc"); !st.ok) return st;
    if (!ported::launch_quantize_mmq_q8_1(x, d4_.ptr, batch, cols, stride, stream_)) return failed("quantize_mmq_q8_1");
    return {};
}

// ---- decode-side ops --------------------------------------------------------------------
// src/kernels_cuda.cu:10764-10888
DeviceStatus HipQ8Backend::q8_0_matvec(DeviceTensor &out, const DeviceWeight &weight, const DeviceTensor &x) {
    const auto &w = W(weight);
    auto &o = T(out);
    if (w.format != DeviceWeightFormat::Q8_0) return {false, "q8_0_matvec: weight is not Q8_0"};
    const uint32_t cols = static_cast<uint32_t>(w.cols), rows = static_cast<uint32_t>(w.rows);
    const float *xin = T(x).f32();
    if (absorbs_norm(xin, cols, o.ptr)) {   // norm, quantizer and GEMV in one launch
        const int rc = q8mi_nqgemv(w.ptr, pending_.x, pending_.weight, pending_.eps, pending_.out, o.ptr,
                                   o.is_bf16() ? 1 : 0, rows, cols, 1, stream_);
        if (rc == Q8MI_OK) {
            pending_.active = false;
            wrote(o.ptr);
            return launch_status("hip rms_norm + q8_0_matvec");
        }
        if (rc != Q8MI_REJECTED) return failed("nqgemv");
    }
    if (auto st = flush_norm(); !st.ok) return st;
    wrote(o.ptr);
    if (o.is_bf16()) {
        if (fuse_quantizer(xin, 1, cols, cols) &&
            q8mi_qgemv(w.ptr, xin, cols, o.bf16(), 1, rows, cols, 1, rows, stream_) == Q8MI_OK)
            return launch_status("hip q8_0_matvec bf16 fused");
        if (auto st = quantize_q8_1(xin, 1, cols, cols); !st.ok) return st;
        if (!ported::launch_mmvq_q8_0_bf16(w.ptr, q8_1_.ptr, o.bf16(), rows, cols, 1, rows, stream_))
            return failed("mmvq_q8_0_bf16");
        return launch_status("hip q8_0_matvec bf16");
    }
    return gemv_route(o.f32(), weight, xin, 1, 0, 0);
}

// src/kernels_cuda.cu:12035-12069
DeviceStatus HipQ8Backend::q8_0_matvec_add(DeviceTensor &accum, const DeviceWeight &weight, const DeviceTensor &x) {
    const auto &w = W(weight);
    auto &o = T(accum);
    if (w.format != DeviceWeightFormat::Q8_0) return {false, "q8_0_matvec_add: weight is not Q8_0"};
    if (auto st = flush_norm(); !st.ok) return st;
    wrote(o.ptr);
    const uint32_t cols = static_cast<uint32_t>(w.cols), rows = static_cast<uint32_t>(w.rows);
    const float *xin = T(x).f32();
    if (fuse_quantizer(xin, 1, cols, cols) &&
        q8mi_qgemv_add(w.ptr, xin, cols, o.ptr, o.is_bf16() ? 1 : 0, rows, cols, 1, rows, stream_) == Q8MI_OK)
        return launch_status("hip q8_0_matvec_add fused");
    if (auto st = quantize_q8_1(xin, 1, cols, cols); !st.ok) return st;
    const bool ok = o.is_bf16()
        ? ported::launch_mmvq_q8_0_add_bf16(w.ptr, q8_1_.ptr, o.bf16(), rows, cols, 1, rows, stream_)
        : ported::launch_mmvq_q8_0_add(w.ptr, q8_1_.ptr, o.f32(), rows, cols, 1, rows, stream_);
    if (!ok) return failed("mmvq_q8_0_add");
    return launch_status("hip q8_0_matvec_add");
}

// src/kernels_cuda.cu:12227-12258
DeviceStatus HipQ8Backend::q8_0_matvec_silu_mul(DeviceTensor &out, const DeviceWeight &weight_gate,
                                                const DeviceWeight &weight_up, const DeviceTensor &x) {
    const auto &g = W(weight_gate);
    return q8_0_matmul_silu_mul(out, weight_gate, weight_up, x, 1, static_cast<uint32_t>(g.cols),
                                static_cast<uint32_t>(g.rows));
}

// src/kernels_cuda.cu:11244-11302: quantize once, then as few launches as possible
DeviceStatus HipQ8Backend::q8_0_matvec_fanout(DeviceTensor *const *outs, const DeviceWeight *const *weights,
                                              uint32_t n, const DeviceTensor &x) {
    std::vector<uint32_t> os(n);
    for (uint32_t i = 0; i < n; ++i) os[i] = static_cast<uint32_t>(W(*weights[i]).rows);
    return q8_0_matmul_fanout(outs, weights, os.data(), n, x, 1, n ? static_cast<uint32_t>(W(*weights[0]).cols) : 0);
}

// ---- prefill / verify ops -----------------------------------------------------------------
// src/kernels_cuda.cu:12552-12630 and mmq_q8 (:14559-14615)
DeviceStatus HipQ8Backend::q8_0_matmul(DeviceTensor &out, const DeviceWeight &weight, const DeviceTensor &x,
                                       uint32_t batch, uint32_t in_stride, uint32_t out_stride) {
    const auto &w = W(weight);
    auto &o = T(out);
    if (batch == 0) return {};
    if (w.format != DeviceWeightFormat::Q8_0) return {false, "q8_0_matmul: weight is not Q8_0"};
    if (batch == 1 && (in_stride == 0 || in_stride == w.cols) && (out_stride == 0 || out_stride == w.rows))
        return q8_0_matvec(out, weight, x);
    if (auto st = flush_norm(); !st.ok) return st;
    wrote(o.ptr);
    const uint32_t cols = static_cast<uint32_t>(w.cols), rows = static_cast<uint32_t>(w.rows);
    const uint64_t out_count = static_cast<uint64_t>(batch) * (out_stride ? out_stride : rows);
    const float *xin = T(x).f32();
    const bool contiguous = in_stride == cols && out_stride == rows;
    const bool tiles = batch > 8 && contiguous && cols % 32 == 0;
    const bool d4 = rows >= 128 && cols % 128 == 0;   // layout rule of src/kernels_cuda.cu:14545-14552
    if (tiles && d4 && o.is_bf16()) {   // the tile kernel rounds to bf16 in its store where it can
        if (auto st = quantize_d4(xin, batch, cols, cols); !st.ok) return st;
        const int rc = q8mi_gemm_bf16(w.ptr, d4_.ptr, o.bf16(), rows, cols, batch, rows, stream_);
        if (rc == Q8MI_OK) return launch_status("hip q8_0_matmul mmq bf16");
        if (rc != Q8MI_REJECTED) return failed("gemm_bf16");
    }
    float *dst = o.f32();
    if (o.is_bf16()) {   // compute in fp32, convert at the end (src/kernels_cuda.cu:14509-14530)
        if (auto st = ensure(out_f32_, out_count * 4, "q8 fp32 output workspace"); !st.ok) return st;
        dst = static_cast<float *>(out_f32_.ptr);
    }
    auto finish = [&](DeviceStatus st) -> DeviceStatus {
        if (!st.ok || !o.is_bf16()) return st;
        if (q8mi_f32_to_bf16(dst, o.bf16(), out_count, stream_) != Q8MI_OK) return failed("f32_to_bf16");
        return launch_status("hip q8 fp32->bf16 output");
    };
    if (tiles) {
        if (d4) {
            if (!o.is_bf16()) {   // (quantized above otherwise)
                if (auto st = quantize_d4(xin, batch, cols, cols); !st.ok) return st;
            }
            const bool medium = batch >= 12 && batch <= 64;   // vmed range, src/kernels_cuda.cu:14566
            const bool ok = medium
                ? ported::launch_mmq_q8_0_medium(w.ptr, d4_.ptr, dst, rows, cols, batch, rows, stream_)
                : ported::launch_mmq_q8_0(w.ptr, d4_.ptr, dst, rows, cols, batch, rows, stream_);
            if (!ok) return failed("mmq_q8_0");
            return finish(launch_status("hip q8_0_matmul mmq"));
        }
        if (auto st = quantize_q8_1(xin, batch, cols, cols); !st.ok) return st;
        if (!ported::launch_mmq_q8_0(w.ptr, q8_1_.ptr, dst, rows, cols, batch, rows, stream_))
            return failed("mmq_q8_0 (q8_1 layout)");
        return finish(launch_status("hip q8_0_matmul mmq small"));
    }
    return finish(gemv_route(dst, weight, xin, batch, in_stride, out_stride));
}

// norm (already applied or to be applied inside the first launch) + projections of up to eight rows:
// shared by rms_norm_q8_0_matmul_fanout and by a fan-out that follows a held-back one-row norm.
// xin: the rows before the norm; nrm: where the normalised rows go; add: a held-back add whose sum xin is
// (batch >= 2), to run inside the norm's launch.
DeviceStatus HipQ8Backend::fanout_normed(float *nrm, const float *xin, const float *nwp, float eps,
                                         DeviceTensor *const *outs, const DeviceWeight *const *weights,
                                         const uint32_t *out_strides, uint32_t fanout, uint32_t batch, uint32_t cols,
                                         const PendingAdd *add) {
    auto group = [&](uint32_t i0, const uint8_t *(&wp)[4], float *(&op)[4], uint32_t (&r)[4], uint32_t (&s)[4]) {
        for (uint32_t k = 0; k < 4; ++k) { wp[k] = nullptr; op[k] = nullptr; r[k] = 0; s[k] = 0; }
        for (uint32_t i = i0; i < fanout && i < i0 + 4; ++i) {
            wp[i - i0] = W(*weights[i]).ptr;
            op[i - i0] = T(*outs[i]).f32();
            r[i - i0] = static_cast<uint32_t>(W(*weights[i]).rows);
            s[i - i0] = out_strides[i];
        }
    };
    const uint8_t *wp[4];
    float *op[4];
    uint32_t r[4], s[4];
    uint32_t first = 0;
    bool quantized = false;
    forget_quantized();
    if (batch == 1 && nrm != xin) {   // the first four weights: norm + quantizer inside the GEMV, which also leaves
                                      // `normalized` (not in place: every workgroup reads x)
        group(0, wp, op, r, s);
        bool dense = true;            // the one-launch form writes dense rows
        for (uint32_t k = 0; k < 4; ++k) dense = dense && (r[k] == 0 || s[k] == r[k]);
        if (dense) {
            const int rc = q8mi_nqgemv_fanout4(wp[0], wp[1], wp[2], wp[3], xin, nwp, eps, nrm, op[0], op[1], op[2], op[3],
                                               r[0], r[1], r[2], r[3], cols, 1, stream_);
            if (rc == Q8MI_OK) first = 4;
            else if (rc != Q8MI_REJECTED) return failed("nqgemv_fanout4");
        }
    }
    if (first == 0) {
        if (auto st = ensure(q8_1_, ported::q8_1_scratch_bytes(batch, cols), "q8_1 scratch alloc"); !st.ok) return st;
        if (add != nullptr) {
            if (q8mi_add_rms_norm(add->a, add->b, add->out, nwp, nrm, q8_1_.ptr, batch, cols, cols, cols, eps, stream_) != Q8MI_OK)
                return failed("add_rms_norm");
        } else if (q8mi_rms_norm_quantize_q8_1(xin, nwp, nrm, q8_1_.ptr, batch, cols, cols, cols, eps, stream_) != Q8MI_OK) {
            return failed("rms_norm_quantize_q8_1");
        }
        quantized = true;
    }
    for (uint32_t i0 = first; i0 < fanout; i0 += 4) {
        group(i0, wp, op, r, s);
        if (!quantized) {   // batch 1, weights beyond the fourth: quantize `normalized` inside the GEMV
            if (q8mi_qgemv_fanout4(wp[0], wp[1], wp[2], wp[3], nrm, cols, op[0], op[1], op[2], op[3], r[0], r[1], r[2],
                                   r[3], cols, 1, s[0], s[1], s[2], s[3], stream_) != Q8MI_OK)
                return failed("qgemv_fanout4");
            continue;
        }
        if (!ported::launch_mmvq_q8_0_fanout4_batch(wp[0], wp[1], wp[2], wp[3], q8_1_.ptr, op[0], op[1], op[2], op[3],
                                                    r[0], r[1], r[2], r[3], cols, batch, s[0], s[1], s[2], s[3],
                                                    stream_))
            return failed("mmvq_q8_0_fanout4_batch");
    }
    if (quantized) quantized_ = QuantizedRows{nrm, batch, cols, cols};   // the next projection of these rows reads the blocks
    for (uint32_t i = 0; i < fanout; ++i) wrote(T(*outs[i]).ptr);
    return launch_status("hip rms_norm_q8_0_matmul_fanout");
}

// src/kernels_cuda.cu:11551-11613
DeviceStatus HipQ8Backend::q8_0_matmul_fanout(DeviceTensor *const *outs, const DeviceWeight *const *weights,
                                              const uint32_t *out_strides, uint32_t n, const DeviceTensor &x,
                                              uint32_t batch, uint32_t in_stride) {
    if (n == 0 || batch == 0) return {};
    const uint32_t cols = static_cast<uint32_t>(W(*weights[0]).cols);
    bool fast = batch <= 8 && in_stride == cols && cols % 32 == 0;
    for (uint32_t i = 0; i < n && fast; ++i) {
        const auto &w = W(*weights[i]);
        fast = w.format == DeviceWeightFormat::Q8_0 && w.cols == cols && !T(*outs[i]).is_bf16();
    }
    const float *xin = T(x).f32();
    if (fast && batch == 1 && pending_.active) {   // a held-back norm of x: inside the first launch
        bool absorb = true;
        for (uint32_t i = 0; i < n; ++i) absorb = absorb && absorbs_norm(xin, cols, T(*outs[i]).ptr);
        if (absorb) {
            const PendingNorm pn = pending_;
            pending_.active = false;
            return fanout_normed(pn.out, pn.x, pn.weight, pn.eps, outs, weights, out_strides, n, 1, cols);
        }
    }
    if (auto st = flush_norm(); !st.ok) return st;
    if (!fast) {   // base-class behaviour: one q8_0_matmul per weight
        for (uint32_t i = 0; i < n; ++i) {
            if (auto st = q8_0_matmul(*outs[i], *weights[i], x, batch, in_stride, out_strides[i]); !st.ok) return st;
        }
        return {};
    }
    const bool fused = fuse_quantizer(xin, batch, cols, in_stride);
    if (!fused) {
        if (auto st = quantize_q8_1(xin, batch, cols, in_stride); !st.ok) return st;
    }
    for (uint32_t i0 = 0; i0 < n; i0 += 4) {
        const uint8_t *wp[4] = {nullptr, nullptr, nullptr, nullptr};
        float *op[4] = {nullptr, nullptr, nullptr, nullptr};
        uint32_t r[4] = {0, 0, 0, 0}, s[4] = {0, 0, 0, 0};
        for (uint32_t i = i0; i < n && i < i0 + 4; ++i) {
            wp[i - i0] = W(*weights[i]).ptr;
            op[i - i0] = T(*outs[i]).f32();
            r[i - i0] = static_cast<uint32_t>(W(*weights[i]).rows);
            s[i - i0] = out_strides[i];
        }
        if (fused) {
            if (q8mi_qgemv_fanout4(wp[0], wp[1], wp[2], wp[3], xin, in_stride, op[0], op[1], op[2], op[3], r[0],
                                   r[1], r[2], r[3], cols, batch, s[0], s[1], s[2], s[3], stream_) != Q8MI_OK)
                return failed("qgemv_fanout4");
            continue;
        }
        if (!ported::launch_mmvq_q8_0_fanout4_batch(wp[0], wp[1], wp[2], wp[3], q8_1_.ptr, op[0], op[1], op[2], op[3],
                                                    r[0], r[1], r[2], r[3], cols, batch, s[0], s[1], s[2], s[3],
                                                    stream_))
            return failed("mmvq_q8_0_fanout4_batch");
    }
    for (uint32_t i = 0; i < n; ++i) wrote(T(*outs[i]).ptr);
    return launch_status("hip q8_0_matmul_fanout");
}

// ---- RMS norm ------------------------------------------------------------------------------
// src/kernels_cuda.cu:14748-14779
DeviceStatus HipQ8Backend::rms_norm(DeviceTensor &out, const DeviceTensor &x, const DeviceWeight &weight, float eps) {
    return rms_norm_batch(out, x, weight, 1, static_cast<uint32_t>(T(x).count), eps);
}

// src/kernels_cuda.cu:14781-14816.  Up to eight rows (what a GEMV takes) also leave their Q8_1 blocks
// in the scratch for the projection that follows; one row of a length the fused GEMVs serve is held
// back for that projection's own launch (flush_norm runs it if something else comes first).
DeviceStatus HipQ8Backend::rms_norm_batch(DeviceTensor &out, const DeviceTensor &x, const DeviceWeight &weight,
                                          uint32_t batch, uint32_t n, float eps) {
    if (batch == 0) return {};
    const auto &w = W(weight);
    if (T(out).is_bf16()) return {false, "hip rms_norm_batch BF16 output is not implemented"};
    if (T(x).is_bf16()) return {false, "hip rms_norm_batch BF16 input is outside the Q8_0 path"};
    if (w.format != DeviceWeightFormat::F32 || w.cols < n) return {false, "rms_norm_batch: norm weight is not fp32 [n]"};
    if (T(x).count < static_cast<uint64_t>(batch) * n || T(out).count < static_cast<uint64_t>(batch) * n)
        return {false, "rms_norm_batch: tensor smaller than batch * n"};
    const float *xin = T(x).f32();
    const float *nwp = reinterpret_cast<const float *>(w.ptr);
    float *nrm = T(out).f32();
    auto aligned16 = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const bool hold_back = norm_shortcuts_ && batch == 1 && n % 256 == 0 && n <= 6144 && nrm != xin && aligned16(xin) &&
                           aligned16(nwp) && aligned16(nrm);
    // the add that produced these rows is still held back: one launch for add, norm (and quantizer)
    if (pending_add_.active && !hold_back && xin == pending_add_.out &&
        pending_add_.count == static_cast<uint64_t>(batch) * n && nrm != pending_add_.out && nrm != pending_add_.a &&
        nrm != pending_add_.b) {
        const PendingAdd pa = pending_add_;
        pending_add_.active = false;
        forget_quantized();
        const bool quant = batch <= 8 && n % 32 == 0;
        if (quant)
            if (auto st = ensure(q8_1_, ported::q8_1_scratch_bytes(batch, n), "q8_1 scratch alloc"); !st.ok) return st;
        if (q8mi_add_rms_norm(pa.a, pa.b, pa.out, nwp, nrm, quant ? q8_1_.ptr : nullptr, batch, n, n, n, eps, stream_) !=
            Q8MI_OK)
            return failed("add_rms_norm");
        if (quant) quantized_ = QuantizedRows{nrm, batch, n, n};
        return launch_status("hip add + rms_norm_batch");
    }
    if (auto st = flush_norm(); !st.ok) return st;
    wrote(T(out).ptr);
    if (hold_back) {
        pending_ = PendingNorm{true, xin, nwp, nrm, n, eps};
        return {};
    }
    if (norm_shortcuts_ && batch <= 8 && n % 32 == 0) {
        forget_quantized();
        if (auto st = ensure(q8_1_, ported::q8_1_scratch_bytes(batch, n), "q8_1 scratch alloc"); !st.ok) return st;
        if (q8mi_rms_norm_quantize_q8_1(xin, nwp, nrm, q8_1_.ptr, batch, n, n, n, eps, stream_) != Q8MI_OK)
            return failed("rms_norm_quantize_q8_1");
        quantized_ = QuantizedRows{nrm, batch, n, n};
        return launch_status("hip rms_norm_batch");
    }
    if (q8mi_rms_norm(xin, nwp, nrm, batch, n, n, n, eps, stream_) != Q8MI_OK) return failed("rms_norm");
    return launch_status("hip rms_norm_batch");
}

void HipQ8Backend::set_norm_shortcuts(bool on) {
    if (!on) (void)invalidate_norm_state();
    norm_shortcuts_ = on;
}

DeviceStatus HipQ8Backend::invalidate_norm_state() {
    forget_quantized();
    return flush_norm();
}

// include/qw3/device_backend.hpp:421-444
DeviceStatus HipQ8Backend::rms_norm_q8_0_matmul_fanout(DeviceTensor &normalized, DeviceTensor *const *outs,
                                                       const DeviceWeight *const *weights, const uint32_t *out_strides,
                                                       uint32_t fanout, const DeviceTensor &x,
                                                       const DeviceWeight &norm_weight, uint32_t batch,
                                                       uint32_t in_stride, float eps) {
    if (fanout == 0 || batch == 0) return {};
    const auto &nw = W(norm_weight);
    const uint32_t cols = in_stride;
    bool fast = batch <= 8 && cols % 32 == 0 && !T(x).is_bf16() && !T(normalized).is_bf16() &&
                nw.format == DeviceWeightFormat::F32 && nw.cols == cols &&
                T(x).count >= static_cast<uint64_t>(batch) * cols &&
                T(normalized).count >= static_cast<uint64_t>(batch) * cols;
    for (uint32_t i = 0; i < fanout && fast; ++i) {
        const auto &w = W(*weights[i]);
        fast = w.format == DeviceWeightFormat::Q8_0 && w.cols == cols && !T(*outs[i]).is_bf16() &&
               out_strides[i] >= w.rows && T(*outs[i]).count >= static_cast<uint64_t>(batch) * out_strides[i];
    }
    if (!fast) {   // base-class behaviour
        if (auto st = rms_norm_batch(normalized, x, norm_weight, batch, in_stride, eps); !st.ok) return st;
        return q8_0_matmul_fanout(outs, weights, out_strides, fanout, normalized, batch, in_stride);
    }
    // a held-back add whose sum these rows are (the add_n that ends the layer before): inside the norm's launch
    PendingAdd add;
    float *nrm = T(normalized).f32();
    if (pending_add_.active && batch >= 2 && T(x).f32() == pending_add_.out &&
        pending_add_.count == static_cast<uint64_t>(batch) * cols && nrm != pending_add_.out && nrm != pending_add_.a &&
        nrm != pending_add_.b) {
        add = pending_add_;
        pending_add_.active = false;
    }
    if (auto st = flush_norm(); !st.ok) return st;
    wrote(nrm);
    return fanout_normed(nrm, T(x).f32(), reinterpret_cast<const float *>(nw.ptr), eps, outs, weights, out_strides, fanout,
                         batch, cols, add.active ? &add : nullptr);
}

// src/kernels_cuda.cu:14818-14862: elementwise out = a + b over the first `count` elements; the
// three tensors are all fp32 or all bf16
DeviceStatus HipQ8Backend::add(DeviceTensor &out, const DeviceTensor &a, const DeviceTensor &b) {
    return add_n(out, a, b, out.count);
}

DeviceStatus HipQ8Backend::add_n(DeviceTensor &out, const DeviceTensor &a, const DeviceTensor &b, uint64_t count) {
    auto &o = T(out);
    const auto &aa = T(a), &bb = T(b);
    if (count > o.count || count > aa.count || count > bb.count) return {false, "hip add_n count exceeds tensor size"};
    if (o.is_bf16() || aa.is_bf16() || bb.is_bf16()) {
        if (!o.is_bf16()) return {false, "hip add_n BF16 input with FP32 output"};
        if (!aa.is_bf16()) return {false, "hip add_n BF16 output with FP32 lhs"};
        if (!bb.is_bf16()) return {false, "hip add_n BF16 output with FP32 rhs"};
    }
    if (auto st = flush_norm(); !st.ok) return st;
    wrote(o.ptr);
    if (norm_shortcuts_ && !o.is_bf16() && count > 0) {   // held back for the norm that may follow
        pending_add_ = PendingAdd{true, o.f32(), aa.f32(), bb.f32(), count};
        return {};
    }
    if (q8mi_add(o.ptr, aa.ptr, bb.ptr, count, o.is_bf16() ? 1 : 0, stream_) != Q8MI_OK) return failed("add");
    return launch_status("hip add");
}

// src/kernels_cuda.cu:14880-14900
DeviceStatus HipQ8Backend::silu_mul(DeviceTensor &out, const DeviceTensor &gate, const DeviceTensor &up) {
    return silu_mul_n(out, gate, up, out.count);
}

DeviceStatus HipQ8Backend::silu_mul_n(DeviceTensor &out, const DeviceTensor &gate, const DeviceTensor &up,
                                      uint64_t count) {
    auto &o = T(out);
    const auto &g = T(gate), &u = T(up);
    if (count > o.count || count > g.count || count > u.count) return {false, "hip silu_mul_n count exceeds tensor size"};
    if (o.is_bf16() || g.is_bf16() || u.is_bf16()) return {false, "hip silu_mul_n: fp32 tensors only"};
    if (auto st = flush_norm(); !st.ok) return st;
    wrote(o.ptr);
    if (q8mi_silu_mul(o.f32(), g.f32(), u.f32(), count, stream_) != Q8MI_OK) return failed("silu_mul");
    return launch_status("hip silu_mul");
}

// src/kernels_cuda.cu:11919-11957: in-place residual add for batch <= 8; above, the tile kernel
// adds the residual in its store where it can, else matmul + add
DeviceStatus HipQ8Backend::q8_0_matmul_add(DeviceTensor &out, const DeviceTensor &residual, DeviceTensor &matmul_tmp,
                                           const DeviceWeight &weight, const DeviceTensor &x, uint32_t batch,
                                           uint32_t in_stride, uint32_t out_stride) {
    const auto &w = W(weight);
    auto &o = T(out);
    const uint32_t cols = static_cast<uint32_t>(w.cols), rows = static_cast<uint32_t>(w.rows);
    const bool shapes_ok = w.format == DeviceWeightFormat::Q8_0 && cols % 32 == 0 && batch >= 1 && in_stride == cols &&
                           o.count >= static_cast<uint64_t>(batch) * out_stride;
    const bool fast = shapes_ok && o.ptr == T(residual).ptr && batch <= 8;
    if (auto st = flush_norm(); !st.ok) return st;
    if (!fast) {
        if (shapes_ok && batch > 8 && out_stride == rows && rows >= 128 && cols % 256 == 0 && !o.is_bf16() &&
            !T(residual).is_bf16() && !T(matmul_tmp).is_bf16() &&
            T(residual).count >= static_cast<uint64_t>(batch) * out_stride &&
            T(matmul_tmp).count >= static_cast<uint64_t>(batch) * out_stride) {
            wrote(o.ptr);
            wrote(T(matmul_tmp).ptr);
            if (auto st = quantize_d4(T(x).f32(), batch, cols, cols); !st.ok) return st;
            const int rc = q8mi_gemm_add(w.ptr, d4_.ptr, T(residual).f32(), o.f32(), rows, cols, batch, rows, stream_);
            if (rc == Q8MI_OK) return launch_status("hip q8_0_matmul_add mmq");
            if (rc != Q8MI_REJECTED) return failed("gemm_add");
            // a shape the tile kernel sums from two halves of K: the same records, then the add
            if (!ported::launch_mmq_q8_0(w.ptr, d4_.ptr, T(matmul_tmp).f32(), rows, cols, batch, rows, stream_))
                return failed("mmq_q8_0");
            if (q8mi_add(o.ptr, T(residual).ptr, T(matmul_tmp).ptr, static_cast<uint64_t>(batch) * rows, 0, stream_) != Q8MI_OK)
                return failed("add");
            return launch_status("hip q8_0_matmul_add mmq + add");
        }
        // include/qw3/device_backend.hpp:529-540: the matmul into the temporary, then out = residual + tmp
        if (auto st = q8_0_matmul(matmul_tmp, weight, x, batch, in_stride, out_stride); !st.ok) return st;
        return add(out, residual, matmul_tmp);
    }
    wrote(o.ptr);
    if (auto st = quantize_q8_1(T(x).f32(), batch, cols, in_stride); !st.ok) return st;
    const bool ok = o.is_bf16()
        ? ported::launch_mmvq_q8_0_add_bf16(w.ptr, q8_1_.ptr, o.bf16(), rows, cols, batch, out_stride, stream_)
        : ported::launch_mmvq_q8_0_add(w.ptr, q8_1_.ptr, o.f32(), rows, cols, batch, out_stride, stream_);
    if (!ok) return failed("mmvq_q8_0_add");
    return launch_status("hip q8_0_matmul_add");
}

// include/qw3/device_backend.hpp:330-336 (batch 1: src/kernels_cuda.cu:12227-12258).  One GEMV launch
// for up to eight rows; above, D4 records once and one launch of the dual-weight tiles; shapes
// neither serves run as GEMV slices of eight rows.
DeviceStatus HipQ8Backend::q8_0_matmul_silu_mul(DeviceTensor &out, const DeviceWeight &weight_gate,
                                                const DeviceWeight &weight_up, const DeviceTensor &x,
                                                uint32_t batch, uint32_t in_stride, uint32_t out_stride) {
    const auto &g = W(weight_gate), &u = W(weight_up);
    auto &o = T(out);
    if (batch == 0) return {};
    if (g.format != DeviceWeightFormat::Q8_0 || u.format != DeviceWeightFormat::Q8_0)
        return {false, "q8_0_matmul_silu_mul: weights are not Q8_0"};
    if (g.rows != u.rows || g.cols != u.cols) return {false, "q8_0_matmul_silu_mul: gate/up shapes differ"};
    if (o.is_bf16() || T(x).is_bf16()) return {false, "q8_0_matmul_silu_mul: fp32 tensors only"};
    const uint32_t cols = static_cast<uint32_t>(g.cols), rows = static_cast<uint32_t>(g.rows);
    if (cols % 32 != 0) return {false, "q8_0_matmul_silu_mul: cols not a multiple of 32"};
    if (in_stride < cols || out_stride < rows) return {false, "q8_0_matmul_silu_mul: stride shorter than a row"};
    if (T(x).count < static_cast<uint64_t>(batch - 1) * in_stride + cols ||
        o.count < static_cast<uint64_t>(batch - 1) * out_stride + rows)
        return {false, "q8_0_matmul_silu_mul: tensor smaller than the batch"};
    const float *xin = T(x).f32();
    if (batch == 1 && absorbs_norm(xin, cols, o.ptr)) {   // norm, quantizer and SwiGLU GEMV in one launch
        const int rc = q8mi_nqgemv_silu_mul(g.ptr, u.ptr, pending_.x, pending_.weight, pending_.eps, pending_.out,
                                            o.f32(), rows, cols, 1, stream_);
        if (rc == Q8MI_OK) {
            pending_.active = false;
            wrote(o.ptr);
            return launch_status("hip rms_norm + q8_0_matvec_silu_mul");
        }
        if (rc != Q8MI_REJECTED) return failed("nqgemv_silu_mul");
    }
    if (auto st = flush_norm(); !st.ok) return st;
    wrote(o.ptr);
    if (fuse_quantizer(xin, batch, cols, in_stride) &&
        q8mi_qgemv_silu_mul(g.ptr, u.ptr, xin, in_stride, o.f32(), rows, cols, 1, out_stride, stream_) == Q8MI_OK)
        return launch_status("hip q8_0_matvec_silu_mul fused");
    if (batch > 8 && rows >= 128 && cols % 256 == 0) {
        if (auto st = quantize_d4(xin, batch, cols, in_stride); !st.ok) return st;
        const int rc = q8mi_gemm_silu_mul(g.ptr, u.ptr, d4_.ptr, o.f32(), rows, cols, batch, out_stride, stream_);
        if (rc == Q8MI_OK) return launch_status("hip q8_0_matmul_silu_mul mmq");
        if (rc != Q8MI_REJECTED) return failed("gemm_silu_mul");
    }
    for (uint32_t j0 = 0; j0 < batch; j0 += 8) {
        const uint32_t m = batch - j0 < 8 ? batch - j0 : 8;
        if (auto st = quantize_q8_1(xin + static_cast<uint64_t>(j0) * in_stride, m, cols, in_stride); !st.ok) return st;
        if (!ported::launch_mmvq_q8_0_silu_mul(g.ptr, u.ptr, q8_1_.ptr, o.f32() + static_cast<uint64_t>(j0) * out_stride,
                                               rows, cols, m, out_stride, stream_))
            return failed("mmvq_q8_0_silu_mul");
    }
    return launch_status("hip q8_0_matmul_silu_mul");
}

// ---- argmax (src/kernels_cuda.cu:20733-20850) ------------------------------------------------
DeviceStatus HipQ8Backend::argmax_launch(const DeviceTensor &x) {
    const auto &t = T(x);
    if (auto st = flush_norm(); !st.ok) return st;
    if (!argmax_dev_) {
        if (capturing_) return {false, "argmax buffers must exist before capture"};
        if (auto st = hip_status(hipMalloc(reinterpret_cast<void **>(&argmax_dev_), 8), "argmax alloc"); !st.ok)
            return st;
    }
    if (!argmax_host_) {
        if (capturing_) return {false, "argmax buffers must exist before capture"};
        if (auto st = hip_status(hipHostMalloc(reinterpret_cast<void **>(&argmax_host_), 8, hipHostMallocDefault),
                                 "argmax pinned alloc"); !st.ok)
            return st;
        argmax_host_[0] = -1;
        argmax_host_[1] = 0;
    }
    if (q8mi_argmax(t.f32(), t.count, argmax_dev_, stream_) != Q8MI_OK) return failed("argmax");
    if (auto st = hip_status(hipMemcpyAsync(argmax_host_, argmax_dev_, 8, hipMemcpyDeviceToHost, stream_),
                             "argmax copy"); !st.ok)
        return st;
    return launch_status("hip argmax_launch");
}

DeviceArgmax HipQ8Backend::argmax_collect() {
    DeviceArgmax best;
    if (!argmax_host_) return best;
    (void)hipStreamSynchronize(stream_);
    best.token = argmax_host_[0];
    std::memcpy(&best.logit, &argmax_host_[1], sizeof(float));
    return best;
}

DeviceArgmax HipQ8Backend::argmax(const DeviceTensor &x) {
    if (auto st = argmax_launch(x); !st.ok) return {};
    return argmax_collect();
}

std::unique_ptr<DeviceArgmaxBuffer> HipQ8Backend::argmax_buffer(uint64_t count) {
    if (count == 0) return nullptr;
    auto b = std::make_unique<HipArgmaxBuffer>();
    b->count = count;
    if (hipMalloc(reinterpret_cast<void **>(&b->ptr), count * sizeof(q8mi_argmax_pair)) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return b;
}

DeviceStatus HipQ8Backend::argmax_to_buffer(const DeviceTensor &x, DeviceArgmaxBuffer &out, uint32_t index) {
    auto &dst = static_cast<HipArgmaxBuffer &>(out);
    if (index >= dst.count) return {false, "argmax_to_buffer index oob"};
    if (auto st = flush_norm(); !st.ok) return st;
    if (q8mi_argmax_to_pair(T(x).f32(), T(x).count, dst.ptr, index, stream_) != Q8MI_OK)
        return failed("argmax_to_pair");
    return launch_status("hip argmax_to_buffer");
}

DeviceStatus HipQ8Backend::q8_0_get_row(DeviceTensor &out, const DeviceWeight &weight, uint64_t row) {
    const auto &w = W(weight);
    auto &o = T(out);
    if (w.format != DeviceWeightFormat::Q8_0) return {false, "row lookup requires Q8_0 weight"};
    if (o.count < w.cols) return {false, "q8_0_get_row: output smaller than a row"};
    if (row >= w.rows) return {false, "q8_0_get_row: row outside the matrix"};
    if (auto st = flush_norm(); !st.ok) return st;
    wrote(o.ptr);
    if (q8mi_get_row(w.ptr, row, w.rows, w.cols, o.ptr, o.is_bf16() ? 1 : 0, stream_) != Q8MI_OK)
        return failed("get_row");
    return launch_status("hip q8_0_get_row");
}

DeviceStatus HipQ8Backend::q8_0_get_row_from_argmax(DeviceTensor &out, const DeviceWeight &weight,
                                                    const DeviceArgmaxBuffer &argmaxes, uint32_t index) {
    const auto &w = W(weight);
    auto &o = T(out);
    const auto &a = static_cast<const HipArgmaxBuffer &>(argmaxes);
    if (index >= a.count) return {false, "q8_0_get_row_from_argmax index oob"};
    if (w.format != DeviceWeightFormat::Q8_0) return {false, "argmax row lookup requires Q8_0 weight"};
    if (o.is_bf16()) return {false, "q8_0_get_row_from_argmax: fp32 output only"};
    if (o.count < w.cols) return {false, "q8_0_get_row_from_argmax: output smaller than a row"};
    if (auto st = flush_norm(); !st.ok) return st;
    wrote(o.ptr);
    if (q8mi_get_row_from_argmax(w.ptr, a.ptr, index, w.rows, w.cols, o.f32(), stream_) != Q8MI_OK)
        return failed("get_row_from_argmax");
    return launch_status("hip q8_0_get_row_from_argmax");
}

DeviceStatus HipQ8Backend::q8_0_get_rows_batch(DeviceTensor &out, const DeviceWeight &weight,
                                               const uint64_t *rows, uint32_t batch) {
    if (batch == 0) return {};
    const auto &w = W(weight);
    auto &o = T(out);
    if (w.format != DeviceWeightFormat::Q8_0) return {false, "batched row lookup requires Q8_0 weight"};
    if (o.count < static_cast<uint64_t>(batch) * w.cols) return {false, "q8_0_get_rows_batch: output too small"};
    if (auto st = flush_norm(); !st.ok) return st;
    wrote(o.ptr);
    // grow-only device copy of the ids (src/kernels_cuda.cu:10722-10727)
    if (auto st = ensure(row_ids_, batch * sizeof(uint64_t), "row id buffer"); !st.ok) return st;
    if (auto st = hip_status(hipMemcpyAsync(row_ids_.ptr, rows, batch * sizeof(uint64_t), hipMemcpyHostToDevice,
                                            stream_), "row id upload"); !st.ok)
        return st;
    if (q8mi_get_rows(w.ptr, static_cast<const uint64_t *>(row_ids_.ptr), batch, w.rows, w.cols, o.ptr,
                      o.is_bf16() ? 1 : 0, stream_) != Q8MI_OK)
        return failed("get_rows");
    return launch_status("hip q8_0_get_rows_batch");
}

DeviceStatus HipQ8Backend::copy_argmax_buffer_to_host(const DeviceArgmaxBuffer &src, DeviceArgmax *host,
                                                      uint32_t count) {
    const auto &s = static_cast<const HipArgmaxBuffer &>(src);
    if (count > s.count) return {false, "copy_argmax_buffer_to_host count oob"};
    std::vector<q8mi_argmax_pair> tmp(count);
    if (auto st = hip_status(hipMemcpyAsync(tmp.data(), s.ptr, count * sizeof(q8mi_argmax_pair),
                                            hipMemcpyDeviceToHost, stream_), "copy_argmax_buffer_to_host"); !st.ok)
        return st;
    if (auto st = synchronize(); !st.ok) return st;
    for (uint32_t i = 0; i < count; ++i) host[i] = {tmp[i].index, tmp[i].value};
    return {};
}

DeviceStatus HipQ8Backend::argmax_batch(const DeviceTensor &x, uint32_t batch, uint32_t row_stride,
                                        std::vector<DeviceArgmax> &out) {
    const auto &t = T(x);
    out.assign(batch, DeviceArgmax{});
    if (batch == 0) return {};
    if (auto st = flush_norm(); !st.ok) return st;
    const uint32_t blocks_per_row = (row_stride + 255) / 256;
    if (row_stride == 0 || blocks_per_row > 1024 || t.count < static_cast<uint64_t>(batch) * row_stride) {
        // the reference's host scan (include/qw3/device_backend.hpp:2477-2497)
        std::vector<float> host(static_cast<size_t>(batch) * row_stride);
        if (auto st = copy_to_host(x, host.data(), 0, host.size()); !st.ok) return st;
        for (uint32_t row = 0; row < batch; ++row) {
            DeviceArgmax best;
            best.logit = -__builtin_inff();
            for (uint32_t c = 0; c < row_stride; ++c) {
                const float v = host[static_cast<size_t>(row) * row_stride + c];
                if (v > best.logit) { best.logit = v; best.token = static_cast<int>(c); }
            }
            out[row] = best;
        }
        return {};
    }
    if (auto st = ensure(argmax_partial_, q8mi_argmax_rows_scratch_bytes(batch, row_stride), "argmax partial alloc");
        !st.ok) return st;
    if (auto st = ensure(argmax_result_, batch * sizeof(q8mi_argmax_pair), "argmax result alloc"); !st.ok) return st;
    auto *res = static_cast<q8mi_argmax_pair *>(argmax_result_.ptr);
    if (q8mi_argmax_rows(t.f32(), batch, row_stride, argmax_partial_.ptr, res, stream_) != Q8MI_OK)
        return failed("argmax_rows");
    std::vector<q8mi_argmax_pair> host(batch);
    if (auto st = hip_status(hipMemcpyAsync(host.data(), res, batch * sizeof(q8mi_argmax_pair),
                                            hipMemcpyDeviceToHost, stream_), "argmax batch copy"); !st.ok)
        return st;
    if (auto st = synchronize(); !st.ok) return st;
    for (uint32_t i = 0; i < batch; ++i) out[i] = {host[i].index, host[i].value};
    return {};
}

// ---- fused verify tail ----------------------------------------------------------------------------
DeviceStatus HipQ8Backend::lm_head_verify(const DeviceWeight &w_out, const DeviceTensor &norm, uint32_t batch,
                                          uint32_t in_stride, const int32_t *drafts, uint32_t n_drafts, int32_t eos,
                                          std::vector<DeviceArgmax> &rows_out, uint32_t &accepted,
                                          int32_t &next_token) {
    const auto &w = W(w_out);
    if (w.format != DeviceWeightFormat::Q8_0) return {false, "lm_head_verify: weight is not Q8_0"};
    if (batch == 0 || batch > 8 || n_drafts + 1 != batch) return {false, "lm_head_verify: batch must be drafts + 1, <= 8"};
    if (auto st = flush_norm(); !st.ok) return st;
    const uint32_t cols = static_cast<uint32_t>(w.cols), vocab = static_cast<uint32_t>(w.rows);
    if (auto st = ensure(lm_head_, q8mi_lm_head_scratch_bytes(vocab, cols, batch), "lm head scratch alloc"); !st.ok)
        return st;
    // eight row pairs and {accepted, next} side by side on the device, and a pinned mirror: one copy back
    constexpr size_t kResultBytes = 8 * sizeof(q8mi_argmax_pair) + 2 * sizeof(int32_t);
    if (auto st = ensure(lm_rows_, kResultBytes, "lm head rows alloc"); !st.ok) return st;
    if (!lm_host_) {
        if (capturing_) return {false, "lm_head_verify: first call must run outside graph capture"};
        if (auto st = hip_status(hipHostMalloc(reinterpret_cast<void **>(&lm_host_), kResultBytes, hipHostMallocDefault),
                                 "lm head pinned mirror"); !st.ok)
            return st;
    }
    if (auto st = quantize_q8_1(T(norm).f32(), batch, cols, in_stride ? in_stride : cols); !st.ok) return st;
    auto *rows_dev = static_cast<q8mi_argmax_pair *>(lm_rows_.ptr);
    auto *accept_dev = reinterpret_cast<int32_t *>(rows_dev + 8);
    if (q8mi_lm_head_argmax_accept(w.ptr, q8_1_.ptr, vocab, cols, batch, drafts, 0, eos, rows_dev, accept_dev,
                                   nullptr, vocab, lm_head_.ptr, stream_) != Q8MI_OK)
        return failed("lm_head_argmax_accept");
    if (auto st = hip_status(hipMemcpyAsync(lm_host_, rows_dev, kResultBytes, hipMemcpyDeviceToHost, stream_),
                             "lm head result copy"); !st.ok)
        return st;
    if (auto st = synchronize(); !st.ok) return st;
    const auto *host_rows = reinterpret_cast<const q8mi_argmax_pair *>(lm_host_);
    const auto *host_acc = reinterpret_cast<const int32_t *>(host_rows + 8);
    rows_out.assign(batch, DeviceArgmax{});
    for (uint32_t i = 0; i < batch; ++i) rows_out[i] = {host_rows[i].index, host_rows[i].value};
    accepted = static_cast<uint32_t>(host_acc[0]);
    next_token = host_acc[1];
    return {};
}

}  // namespace qw3
