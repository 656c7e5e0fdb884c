// HipQ8Backend: the Q8_0 linear + argmax slice of qw3's device operator API on
// one MI355X.
//
// The reference executor drives every device op through the virtuals of
// `qw3::DeviceBackend` (include/qw3/device_backend.hpp:88-).  This class
// implements, with the same names, arguments and DeviceStatus conventions, the
// ones that lie on the Q8_0 hot path:
//   weight_q8_0 (:215), q8_0_matvec (:300), q8_0_matvec_add (:309),
//   q8_0_matvec_silu_mul (:322), q8_0_matmul_silu_mul (:332),
//   q8_0_matvec_fanout (:372), q8_0_matmul (:387), q8_0_matmul_fanout (:406),
//   q8_0_matmul_add (:529), argmax (:2456), argmax_buffer / argmax_to_buffer /
//   copy_argmax_buffer_to_host (:2458-2473), argmax_batch (:2477),
//   argmax_launch / argmax_collect (:2503-2509), begin/end_capture, replay_graph
//   (:120-122), weight_f32 (:214), rms_norm / rms_norm_batch (:624-638) and
//   rms_norm_q8_0_matmul_fanout with its recurrent / attention twins (:421-523),
//   plus the handful of tensor calls a test needs.
// Routing follows the reference's CUDA backend (src/kernels_cuda.cu:10764-12630,
// 14559-14658) except where noted in the .cpp; one op is new: lm_head_verify.
//
// The small value types below repeat the reference's declarations
// (device_backend.hpp:24-69) so this header stands alone; inside the reference
// tree a maintainer deletes them, includes the real header and derives from
// DeviceBackend.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <memory>
#include <vector>

namespace qw3 {

struct DeviceStatus {
    bool ok = true;
    const char *message = "";
};

enum class DeviceTensorDType { F32, F16, BF16, I32, Q8_KV, FP8_E4M3 };

struct DeviceTensor {
    virtual ~DeviceTensor() = default;
    uint64_t count = 0;
    uint32_t elem_size = 4;
    DeviceTensorDType dtype = DeviceTensorDType::F32;
};

enum class DeviceWeightFormat { F32, BF16, FP8_E4M3, Q8_0, NVFP4_E2M1 };

struct DeviceWeight {
    virtual ~DeviceWeight() = default;
    uint64_t rows = 0;
    uint64_t cols = 0;
    DeviceWeightFormat format = DeviceWeightFormat::F32;
};

struct DeviceArgmax {
    int token = -1;
    float logit = 0.0f;
};

struct DeviceArgmaxBuffer {
    virtual ~DeviceArgmaxBuffer() = default;
    uint64_t count = 0;
};

class HipQ8Backend {
public:
    HipQ8Backend();
    ~HipQ8Backend();
    HipQ8Backend(const HipQ8Backend &) = delete;
    HipQ8Backend &operator=(const HipQ8Backend &) = delete;

    const char *name() const { return "hip-q8 (gfx950)"; }
    DeviceStatus begin() { return {}; }
    DeviceStatus end();           // drains the exec stream (src/kernels_cuda.cu:9807-9823)
    DeviceStatus synchronize();
    // The shortcuts around rms_norm_batch (a one-row norm held back for the projection that reads
    // it; the Q8_1 blocks a 2..8-row norm leaves for the projections that follow; an fp32 add / add_n
    // held back for the norm that reads its sum) rely on this backend seeing every read and write of
    // the tensors involved.  A host that lets other code touch those tensors in between (kernels of
    // its own on exec_stream(), views that alias them) either calls invalidate_norm_state() before
    // such an access or turns the shortcuts off; results are the same bits either way, only the
    // launch count changes.
    void set_norm_shortcuts(bool on);
    bool norm_shortcuts() const { return norm_shortcuts_; }
    DeviceStatus invalidate_norm_state();   // runs a held-back add or norm, forgets the cached blocks
    // Called by the destructors of this backend's tensors and weights, before they free `ptr`: a
    // held-back norm that reads it runs now, one that only writes it is dropped (nobody can read
    // the result), cached blocks of its rows are forgotten.
    void released(const void *ptr);
    // What those objects keep of the backend: cleared when the backend goes first.
    struct Owner {
        HipQ8Backend *backend = nullptr;
    };
    hipStream_t exec_stream() const { return stream_; }

    // HIP-graph capture of whatever is launched between begin_capture and end_capture
    bool begin_capture();
    DeviceStatus end_capture();
    DeviceStatus replay_graph();

    // tensors / weights
    std::unique_ptr<DeviceTensor> tensor_f32(uint64_t count, const char *label);
    std::unique_ptr<DeviceTensor> tensor_bf16(uint64_t count, const char *label);
    // fp32 vector (norm weights): rows = 1, cols = count (src/kernels_cuda.cu: weight_f32)
    std::unique_ptr<DeviceWeight> weight_f32(const float *data, uint64_t count, const char *label);
    // `data`: interleaved GGUF Q8_0 blocks (34 B); stored split-plane on the device
    std::unique_ptr<DeviceWeight> weight_q8_0(const void *data, uint64_t rows, uint64_t cols, const char *label);
    DeviceStatus copy_bytes_from_host(DeviceTensor &x, uint64_t byte_offset, const void *host, uint64_t bytes);
    DeviceStatus copy_to_host(const DeviceTensor &x, float *host, uint64_t offset, uint64_t count);
    DeviceStatus copy_bytes_to_host(const DeviceTensor &x, void *host, uint64_t byte_offset, uint64_t bytes);
    DeviceStatus zero_tensor(DeviceTensor &x);

    // decode-side linear ops (batch 1)
    DeviceStatus q8_0_matvec(DeviceTensor &out, const DeviceWeight &weight, const DeviceTensor &x);
    DeviceStatus q8_0_matvec_add(DeviceTensor &accum, const DeviceWeight &weight, const DeviceTensor &x);
    DeviceStatus q8_0_matvec_silu_mul(DeviceTensor &out, const DeviceWeight &weight_gate,
                                      const DeviceWeight &weight_up, const DeviceTensor &x);
    DeviceStatus q8_0_matvec_fanout(DeviceTensor *const *outs, const DeviceWeight *const *weights, uint32_t n,
                                    const DeviceTensor &x);

    // prefill / verify linear ops
    DeviceStatus q8_0_matmul(DeviceTensor &out, const DeviceWeight &weight, const DeviceTensor &x, uint32_t batch,
                             uint32_t in_stride, uint32_t out_stride);
    DeviceStatus q8_0_matmul_fanout(DeviceTensor *const *outs, const DeviceWeight *const *weights,
                                    const uint32_t *out_strides, uint32_t n, const DeviceTensor &x, uint32_t batch,
                                    uint32_t in_stride);
    // elementwise out = a + b (include/qw3/device_backend.hpp:639-646): what the batched
    // q8_0_matmul_add ends with when its fused in-place form does not apply
    DeviceStatus add(DeviceTensor &out, const DeviceTensor &a, const DeviceTensor &b);
    DeviceStatus add_n(DeviceTensor &out, const DeviceTensor &a, const DeviceTensor &b, uint64_t count);
    DeviceStatus q8_0_matmul_add(DeviceTensor &out, const DeviceTensor &residual, DeviceTensor &matmul_tmp,
                                 const DeviceWeight &weight, const DeviceTensor &x, uint32_t batch,
                                 uint32_t in_stride, uint32_t out_stride);
    // out[j][r] = silu(gate row r . x[j]) * (up row r . x[j]) for `batch` rows of x
    // (include/qw3/device_backend.hpp:330-336): one GEMV launch up to eight rows, one tile launch
    // above (the reference's CUDA backend declines Q8_0 here and the executor runs two matmuls and
    // silu_mul_n, src/kernels_cuda.cu:12323-12333, src/qwen_executor.cpp:6669-6685)
    DeviceStatus q8_0_matmul_silu_mul(DeviceTensor &out, const DeviceWeight &weight_gate,
                                      const DeviceWeight &weight_up, const DeviceTensor &x, uint32_t batch,
                                      uint32_t in_stride, uint32_t out_stride);
    // elementwise out = silu(gate) * up over the whole of `out` / its first `count` elements
    // (include/qw3/device_backend.hpp:652-663, src/kernels_cuda.cu:14880-14900); fp32 tensors
    DeviceStatus silu_mul(DeviceTensor &out, const DeviceTensor &gate, const DeviceTensor &up);
    DeviceStatus silu_mul_n(DeviceTensor &out, const DeviceTensor &gate, const DeviceTensor &up, uint64_t count);

    // RMS norm in front of the projections.  rms_norm normalises the whole tensor as one row
    // (src/kernels_cuda.cu:14748-14779), rms_norm_batch `batch` dense rows of n (:14781-14816).
    DeviceStatus rms_norm(DeviceTensor &out, const DeviceTensor &x, const DeviceWeight &weight, float eps);
    DeviceStatus rms_norm_batch(DeviceTensor &out, const DeviceTensor &x, const DeviceWeight &weight, uint32_t batch,
                                uint32_t n, float eps);
    // norm, then several projections of the normalised rows (include/qw3/device_backend.hpp:421-444;
    // the reference's CUDA override fuses FP8 weights only and runs the two steps for Q8_0,
    // src/kernels_cuda.cu:11615-11658).  Here a batch of one row is one launch (norm and quantizer
    // inside the fan-out GEMV), up to eight rows are a fused norm + quantizer and one GEMV launch per
    // four weights; `normalized` receives the fp32 rows either way.
    DeviceStatus rms_norm_q8_0_matmul_fanout(DeviceTensor &normalized, DeviceTensor *const *outs,
                                             const DeviceWeight *const *weights, const uint32_t *out_strides,
                                             uint32_t fanout, const DeviceTensor &x, const DeviceWeight &norm_weight,
                                             uint32_t batch, uint32_t in_stride, float eps);
    DeviceStatus rms_norm_q8_0_matmul_recurrent_fanout(DeviceTensor &normalized, DeviceTensor *const *outs,
                                                       const DeviceWeight *const *weights, const uint32_t *out_strides,
                                                       uint32_t fanout, const DeviceTensor &x,
                                                       const DeviceWeight &norm_weight, uint32_t batch,
                                                       uint32_t in_stride, float eps) {
        return rms_norm_q8_0_matmul_fanout(normalized, outs, weights, out_strides, fanout, x, norm_weight, batch,
                                           in_stride, eps);
    }
    DeviceStatus rms_norm_q8_0_matmul_attention_fanout(DeviceTensor &normalized, DeviceTensor *const *outs,
                                                       const DeviceWeight *const *weights, const uint32_t *out_strides,
                                                       uint32_t fanout, const DeviceTensor &x,
                                                       const DeviceWeight &norm_weight, uint32_t batch,
                                                       uint32_t in_stride, float eps) {
        return rms_norm_q8_0_matmul_fanout(normalized, outs, weights, out_strides, fanout, x, norm_weight, batch,
                                           in_stride, eps);
    }

    // argmax
    DeviceArgmax argmax(const DeviceTensor &x);
    DeviceStatus argmax_launch(const DeviceTensor &x);
    DeviceArgmax argmax_collect();
    std::unique_ptr<DeviceArgmaxBuffer> argmax_buffer(uint64_t count);
    DeviceStatus argmax_to_buffer(const DeviceTensor &x, DeviceArgmaxBuffer &out, uint32_t index);
    DeviceStatus copy_argmax_buffer_to_host(const DeviceArgmaxBuffer &src, DeviceArgmax *host, uint32_t count);
    DeviceStatus argmax_batch(const DeviceTensor &x, uint32_t batch, uint32_t row_stride,
                              std::vector<DeviceArgmax> &out);

    // embedding lookup: dequantized rows of a Q8_0 matrix
    // (include/qw3/device_backend.hpp:276-299, src/kernels_cuda.cu:10613-10755).
    // `out` may be fp32 or bf16; the argmax variant is fp32 only and yields zeros
    // when the slot holds no valid token.  `rows` of the batch variant is a HOST array.
    DeviceStatus q8_0_get_row(DeviceTensor &out, const DeviceWeight &weight, uint64_t row);
    DeviceStatus q8_0_get_row_from_argmax(DeviceTensor &out, const DeviceWeight &weight,
                                          const DeviceArgmaxBuffer &argmaxes, uint32_t index);
    DeviceStatus q8_0_get_rows_batch(DeviceTensor &out, const DeviceWeight &weight, const uint64_t *rows,
                                     uint32_t batch);

    // Format-neutral forwards with the reference's default bodies
    // (include/qw3/device_backend.hpp:541-607): the executor calls these; for Q8_0
    // weights they are the q8_0_* operators.
    DeviceStatus linear_get_row(DeviceTensor &out, const DeviceWeight &weight, uint64_t row) {
        return q8_0_get_row(out, weight, row);
    }
    DeviceStatus linear_get_row_from_argmax(DeviceTensor &out, const DeviceWeight &weight,
                                            const DeviceArgmaxBuffer &argmaxes, uint32_t index) {
        return q8_0_get_row_from_argmax(out, weight, argmaxes, index);
    }
    DeviceStatus linear_get_rows_batch(DeviceTensor &out, const DeviceWeight &weight, const uint64_t *rows,
                                       uint32_t batch) {
        return q8_0_get_rows_batch(out, weight, rows, batch);
    }
    // include/qw3/device_backend.hpp:609-622: linear_matmul into the temporary, then add
    DeviceStatus linear_matmul_add(DeviceTensor &out, const DeviceTensor &residual, DeviceTensor &matmul_tmp,
                                   const DeviceWeight &weight, const DeviceTensor &x, uint32_t batch,
                                   uint32_t in_stride, uint32_t out_stride) {
        if (auto st = q8_0_matmul(matmul_tmp, weight, x, batch, in_stride, out_stride); !st.ok) return st;
        return add(out, residual, matmul_tmp);
    }
    DeviceStatus linear_matvec(DeviceTensor &out, const DeviceWeight &weight, const DeviceTensor &x) {
        return q8_0_matvec(out, weight, x);
    }
    DeviceStatus linear_matvec_add(DeviceTensor &accum, const DeviceWeight &weight, const DeviceTensor &x) {
        return q8_0_matvec_add(accum, weight, x);
    }
    DeviceStatus linear_matvec_silu_mul(DeviceTensor &out, const DeviceWeight &weight_gate,
                                        const DeviceWeight &weight_up, const DeviceTensor &x) {
        return q8_0_matvec_silu_mul(out, weight_gate, weight_up, x);
    }
    DeviceStatus linear_matvec_fanout(DeviceTensor *const *outs, const DeviceWeight *const *weights, uint32_t n,
                                      const DeviceTensor &x) {
        for (uint32_t i = 0; i < n; ++i)
            if (auto st = linear_matvec(*outs[i], *weights[i], x); !st.ok) return st;
        return {};
    }
    DeviceStatus linear_matmul(DeviceTensor &out, const DeviceWeight &weight, const DeviceTensor &x, uint32_t batch,
                               uint32_t in_stride, uint32_t out_stride) {
        return q8_0_matmul(out, weight, x, batch, in_stride, out_stride);
    }
    DeviceStatus linear_matmul_fanout(DeviceTensor *const *outs, const DeviceWeight *const *weights,
                                      const uint32_t *out_strides, uint32_t n, const DeviceTensor &x,
                                      uint32_t batch, uint32_t in_stride) {
        for (uint32_t i = 0; i < n; ++i)
            if (auto st = linear_matmul(*outs[i], *weights[i], x, batch, in_stride, out_strides[i]); !st.ok) return st;
        return {};
    }

    // New op (no counterpart in the reference): the whole verify tail in one pass
    // over the LM-head weights.  Equivalent to q8_0_matmul(logits, w_out, norm, batch,
    // in_stride, vocab) + argmax_batch + the greedy accept loop
    // (src/qwen_executor.cpp:6779-6821, src/qwen_native_backend.cpp:15948-15960,
    // 16048-16052).  rows_out[i] gates drafts[i]; `accepted` is the number of
    // leading drafts equal to their row's token; `next_token` = token of row
    // `accepted` (eos if that row has none).
    DeviceStatus lm_head_verify(const DeviceWeight &w_out, const DeviceTensor &norm, uint32_t batch,
                                uint32_t in_stride, const int32_t *drafts, uint32_t n_drafts, int32_t eos,
                                std::vector<DeviceArgmax> &rows_out, uint32_t &accepted, int32_t &next_token);

private:
    struct Scratch {
        void *ptr = nullptr;
        size_t capacity = 0;
    };
    // A one-row rms_norm whose launch is held back until the next call: when that call is a
    // batch-1 projection of the normalised row, norm, quantizer and GEMV run as one launch (which
    // also writes the normalised row); any other call runs the norm first.  Nothing a caller can
    // observe depends on which of the two happened.
    struct PendingNorm {
        bool active = false;
        const float *x = nullptr;
        const float *weight = nullptr;
        float *out = nullptr;
        uint32_t cols = 0;
        float eps = 0.0f;
    };
    // An fp32 add / add_n whose launch is held back until the next call: when that call is the
    // rms_norm_batch of exactly the rows it sums (the batched layer loop's add_n + rms_norm_batch,
    // src/qwen_executor.cpp:6642-6668), add, norm and quantizer run as one launch; any other call
    // runs the add first.  Never active together with a PendingNorm.
    struct PendingAdd {
        bool active = false;
        float *out = nullptr;
        const float *a = nullptr, *b = nullptr;
        uint64_t count = 0;
    };
    // What the Q8_1 scratch holds: the blocks of `batch` rows of `cols` floats at `src`, written by
    // the norm that produced those rows.  Valid only until the next call that writes a tensor or
    // the scratch: the projections that follow a norm read them instead of quantizing again.
    struct QuantizedRows {
        const float *src = nullptr;
        uint32_t batch = 0, cols = 0, stride = 0;
    };
    DeviceStatus flush_norm();   // runs whatever is held back (an add, or a norm)
    DeviceStatus flush_add();
    void forget_quantized() { quantized_ = QuantizedRows{}; }
    bool absorbs_norm(const float *x, uint32_t cols, const void *out0) const;
    DeviceStatus ensure(Scratch &s, size_t need, const char *what);
    DeviceStatus launch_status(const char *where);
    DeviceStatus failed(const char *where);
    void wrote(const void *tensor) {   // a call that writes `tensor`: its rows' blocks in the scratch are stale
        if (tensor == quantized_.src) forget_quantized();
    }
    bool fuse_quantizer(const float *x, uint32_t batch, uint32_t cols, uint32_t stride) const;
    DeviceStatus quantize_q8_1(const float *x, uint32_t batch, uint32_t cols, uint32_t stride);
    DeviceStatus quantize_d4(const float *x, uint32_t batch, uint32_t cols, uint32_t stride);
    DeviceStatus fanout_normed(float *nrm, const float *xin, const float *nwp, float eps, DeviceTensor *const *outs,
                               const DeviceWeight *const *weights, const uint32_t *out_strides, uint32_t fanout,
                               uint32_t batch, uint32_t cols, const PendingAdd *add = nullptr);
    DeviceStatus gemv_route(float *out, const DeviceWeight &w, const float *x, uint32_t batch, uint32_t in_stride,
                            uint32_t out_stride);

    hipStream_t stream_ = nullptr;
    PendingNorm pending_;
    PendingAdd pending_add_;
    bool norm_shortcuts_ = true;
    std::shared_ptr<Owner> owner_;
    QuantizedRows quantized_;
    Scratch q8_1_, d4_, argmax_partial_, argmax_result_, lm_head_, lm_rows_, out_f32_, row_ids_;
    int32_t *argmax_dev_ = nullptr;    // {token, logit bits}
    int32_t *argmax_host_ = nullptr;   // pinned mirror
    uint8_t *lm_host_ = nullptr;       // pinned mirror of lm_head_verify's row pairs and {accepted, next}
    hipGraph_t graph_ = nullptr;
    hipGraphExec_t graph_exec_ = nullptr;
    bool capturing_ = false;
};

}  // namespace qw3
