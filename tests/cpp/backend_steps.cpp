// The linear operators of one transformer layer driven through qw3::HipQ8Backend in the order the
// reference's executors call them, for bench.py (loaded with ctypes): what a drop-in backend is
// asked to do per layer, as opposed to the hand-picked C-ABI launch sequence of the headline step.
//
//   decode (batch 1), src/qwen_executor.cpp:5514-5746:
//       rms_norm(attn_norm) -> q8_0_matvec_fanout(q, k, v) -> [attention] -> q8_0_matvec_add(o)
//       -> rms_norm(ffn_norm) -> q8_0_matvec_silu_mul(gate, up) -> q8_0_matvec_add(down)
//   verify / prefill chunk (batch m), order 0 = src/qwen_executor.cpp:6459-6693:
//       rms_norm_q8_0_matmul_fanout(q, k, v) -> [attention] -> q8_0_matmul(o) + add_n
//       -> rms_norm_batch(ffn_norm) -> q8_0_matmul_silu_mul(gate, up) -> q8_0_matmul(down) + add_n
//   order 1 = the continuous-batching verifier, src/qwen_native_backend.cpp:7091-7207:
//       rms_norm_batch -> q8_0_matmul_fanout -> [attention] -> q8_0_matmul_add(o, in place)
//       -> rms_norm_batch -> q8_0_matmul_silu_mul -> q8_0_matmul_add(down, in place)
//   head: rms_norm_batch(output_norm) -> lm_head_verify (the fused form of q8_0_matmul + argmax_batch
//       + the accept loop, src/qwen_executor.cpp:6779-6821)
// Attention itself is outside this library: its output is a fixed random tensor.
#include <cstdint>
#include <cstring>
#include <memory>
#include <vector>

#include "../../kvmem-qw3_amd/host/hip_q8_backend.hpp"

namespace {

struct Layer {
    std::unique_ptr<qw3::DeviceWeight> q, k, v, o, gate, up, down;
};

struct Steps {
    qw3::HipQ8Backend backend;
    uint32_t hidden = 0, qdim = 0, kvdim = 0, attn_out = 0, ffn = 0, vocab = 0;
    std::vector<Layer> layers;
    std::unique_ptr<qw3::DeviceWeight> head, norm_w;
    uint32_t batch = 0;
    std::unique_ptr<qw3::DeviceTensor> h, norm, q, k, v, mid, ffn_mid, tmp_h;
    char error[256] = "";
};

bool fail(Steps *s, const qw3::DeviceStatus &st) {
    std::strncpy(s->error, st.message ? st.message : "", sizeof(s->error) - 1);
    return false;
}

#define TRY(expr)                                  \
    do {                                           \
        const qw3::DeviceStatus st_ = (expr);      \
        if (!st_.ok) return fail(s, st_);          \
    } while (0)

bool decode_layer(Steps *s, const Layer &l) {
    auto &b = s->backend;
    const float eps = 1e-6f;
    TRY(b.rms_norm(*s->norm, *s->h, *s->norm_w, eps));
    qw3::DeviceTensor *outs[3] = {s->q.get(), s->k.get(), s->v.get()};
    const qw3::DeviceWeight *ws[3] = {l.q.get(), l.k.get(), l.v.get()};
    TRY(b.q8_0_matvec_fanout(outs, ws, 3, *s->norm));
    TRY(b.q8_0_matvec_add(*s->h, *l.o, *s->mid));
    TRY(b.rms_norm(*s->norm, *s->h, *s->norm_w, eps));
    TRY(b.q8_0_matvec_silu_mul(*s->ffn_mid, *l.gate, *l.up, *s->norm));
    TRY(b.q8_0_matvec_add(*s->h, *l.down, *s->ffn_mid));
    return true;
}

bool verify_layer(Steps *s, const Layer &l, uint32_t m, int order) {
    auto &b = s->backend;
    const float eps = 1e-6f;
    qw3::DeviceTensor *outs[3] = {s->q.get(), s->k.get(), s->v.get()};
    const qw3::DeviceWeight *ws[3] = {l.q.get(), l.k.get(), l.v.get()};
    const uint32_t strides[3] = {s->qdim, s->kvdim, s->kvdim};
    const uint64_t hn = static_cast<uint64_t>(m) * s->hidden;
    if (order == 0) {
        TRY(b.rms_norm_q8_0_matmul_fanout(*s->norm, outs, ws, strides, 3, *s->h, *s->norm_w, m, s->hidden, eps));
        TRY(b.q8_0_matmul(*s->tmp_h, *l.o, *s->mid, m, s->attn_out, s->hidden));
        TRY(b.add_n(*s->h, *s->h, *s->tmp_h, hn));
    } else {
        TRY(b.rms_norm_batch(*s->norm, *s->h, *s->norm_w, m, s->hidden, eps));
        TRY(b.q8_0_matmul_fanout(outs, ws, strides, 3, *s->norm, m, s->hidden));
        TRY(b.q8_0_matmul_add(*s->h, *s->h, *s->tmp_h, *l.o, *s->mid, m, s->attn_out, s->hidden));
    }
    TRY(b.rms_norm_batch(*s->norm, *s->h, *s->norm_w, m, s->hidden, eps));
    TRY(b.q8_0_matmul_silu_mul(*s->ffn_mid, *l.gate, *l.up, *s->norm, m, s->hidden, s->ffn));
    if (order == 0) {
        TRY(b.q8_0_matmul(*s->tmp_h, *l.down, *s->ffn_mid, m, s->ffn, s->hidden));
        TRY(b.add_n(*s->h, *s->h, *s->tmp_h, hn));
    } else {
        TRY(b.q8_0_matmul_add(*s->h, *s->h, *s->tmp_h, *l.down, *s->ffn_mid, m, s->ffn, s->hidden));
    }
    return true;
}

}  // namespace

extern "C" {

void *bsteps_create(uint32_t hidden, uint32_t qdim, uint32_t kvdim, uint32_t attn_out, uint32_t ffn) {
    auto *s = new Steps();
    s->hidden = hidden; s->qdim = qdim; s->kvdim = kvdim; s->attn_out = attn_out; s->ffn = ffn;
    const std::vector<float> ones(hidden, 1.0f);
    s->norm_w = s->backend.weight_f32(ones.data(), hidden, "norm.weight");
    return s;
}

void bsteps_destroy(void *handle) { delete static_cast<Steps *>(handle); }

const char *bsteps_error(void *handle) { return static_cast<Steps *>(handle)->error; }

// The seven weights of a layer as interleaved GGUF Q8_0 blocks (host memory).  Returns the layer's index, -1 on failure.
int bsteps_add_layer(void *handle, const void *q, const void *k, const void *v, const void *o, const void *gate,
                     const void *up, const void *down) {
    auto *s = static_cast<Steps *>(handle);
    auto &b = s->backend;
    Layer l;
    l.q = b.weight_q8_0(q, s->qdim, s->hidden, "attn_q");
    l.k = b.weight_q8_0(k, s->kvdim, s->hidden, "attn_k");
    l.v = b.weight_q8_0(v, s->kvdim, s->hidden, "attn_v");
    l.o = b.weight_q8_0(o, s->hidden, s->attn_out, "attn_output");
    l.gate = b.weight_q8_0(gate, s->ffn, s->hidden, "ffn_gate");
    l.up = b.weight_q8_0(up, s->ffn, s->hidden, "ffn_up");
    l.down = b.weight_q8_0(down, s->hidden, s->ffn, "ffn_down");
    if (!l.q || !l.k || !l.v || !l.o || !l.gate || !l.up || !l.down) return -1;
    s->layers.push_back(std::move(l));
    return static_cast<int>(s->layers.size()) - 1;
}

int bsteps_set_head(void *handle, const void *blocks, uint32_t vocab) {
    auto *s = static_cast<Steps *>(handle);
    s->head = s->backend.weight_q8_0(blocks, vocab, s->hidden, "output");
    s->vocab = vocab;
    return s->head ? 0 : -1;
}

// Tensors for `batch` rows; h and mid (the residual stream and the attention output) from host floats.
int bsteps_prepare(void *handle, uint32_t batch, const float *h, const float *mid) {
    auto *s = static_cast<Steps *>(handle);
    auto &b = s->backend;
    s->batch = batch;
    const uint64_t m = batch;
    s->h = b.tensor_f32(m * s->hidden, "h");
    s->norm = b.tensor_f32(m * s->hidden, "norm");
    s->q = b.tensor_f32(m * s->qdim, "q");
    s->k = b.tensor_f32(m * s->kvdim, "k");
    s->v = b.tensor_f32(m * s->kvdim, "v");
    s->mid = b.tensor_f32(m * s->attn_out, "mid");
    s->ffn_mid = b.tensor_f32(m * s->ffn, "ffn_mid");
    s->tmp_h = b.tensor_f32(m * s->hidden, "tmp");
    if (!s->h || !s->norm || !s->q || !s->k || !s->v || !s->mid || !s->ffn_mid || !s->tmp_h) return -1;
    if (!b.copy_bytes_from_host(*s->h, 0, h, m * s->hidden * 4).ok) return -1;
    if (!b.copy_bytes_from_host(*s->mid, 0, mid, m * s->attn_out * 4).ok) return -1;
    return 0;
}

// One layer step (order < 0: the decode order, batch 1).  0 on success.
int bsteps_layer(void *handle, uint32_t layer, int order) {
    auto *s = static_cast<Steps *>(handle);
    if (layer >= s->layers.size()) return -1;
    const bool ok = order < 0 ? decode_layer(s, s->layers[layer]) : verify_layer(s, s->layers[layer], s->batch, order);
    return ok ? 0 : -1;
}

// Device milliseconds per step of `steps` layer steps over the layers in turn (events on the backend's
// stream), after `warmup` untimed ones.  Negative on failure.
double bsteps_time_layers(void *handle, int order, uint32_t steps, uint32_t warmup) {
    auto *s = static_cast<Steps *>(handle);
    const uint32_t nl = static_cast<uint32_t>(s->layers.size());
    if (nl == 0 || steps == 0) return -1.0;
    for (uint32_t i = 0; i < warmup; ++i)
        if (bsteps_layer(handle, i % nl, order) != 0) return -1.0;
    if (!s->backend.synchronize().ok) return -1.0;
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return -1.0;
    (void)hipEventRecord(e0, s->backend.exec_stream());
    bool ok = true;
    for (uint32_t i = 0; i < steps && ok; ++i) ok = bsteps_layer(handle, (warmup + i) % nl, order) == 0;
    ok = ok && s->backend.synchronize().ok;   // also launches a norm still held back
    (void)hipEventRecord(e1, s->backend.exec_stream());
    (void)hipEventSynchronize(e1);
    float ms = 0.0f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return ok ? static_cast<double>(ms) / steps : -1.0;
}

// Final norm + fused LM head on the current residual rows.  The operator ends in a host read of the
// accept result, so the stream time between the first and the last call includes a host round trip
// per call: milliseconds per call as a decoder would see them.
double bsteps_time_head(void *handle, uint32_t calls, uint32_t warmup, int32_t *accepted_out, int32_t *next_out) {
    auto *s = static_cast<Steps *>(handle);
    if (!s->head || s->batch == 0 || s->batch > 8) return -1.0;
    auto &b = s->backend;
    std::vector<int32_t> drafts(s->batch > 1 ? s->batch - 1 : 0, 0);
    std::vector<qw3::DeviceArgmax> rows;
    uint32_t accepted = 0;
    int32_t next = -1;
    auto once = [&]() {
        return b.rms_norm_batch(*s->norm, *s->h, *s->norm_w, s->batch, s->hidden, 1e-6f).ok &&
               b.lm_head_verify(*s->head, *s->norm, s->batch, s->hidden, drafts.data(), s->batch - 1, 0, rows, accepted, next).ok;
    };
    for (uint32_t i = 0; i < warmup; ++i)
        if (!once()) return -1.0;
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return -1.0;
    (void)hipEventRecord(e0, b.exec_stream());
    bool ok = true;
    for (uint32_t i = 0; i < calls && ok; ++i) ok = once();
    (void)hipEventRecord(e1, b.exec_stream());
    (void)hipEventSynchronize(e1);
    float ms = 0.0f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (accepted_out) *accepted_out = static_cast<int32_t>(accepted);
    if (next_out) *next_out = next;
    return ok ? static_cast<double>(ms) / calls : -1.0;
}

}  // extern "C"
