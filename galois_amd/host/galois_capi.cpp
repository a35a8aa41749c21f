// Flat C handles over the C++ host mirror so that pytest can drive it with ctypes.
#include <cstring>
#include <string>

#include "galois.hpp"
#include "gguf.hpp"
#include "llama.hpp"

using namespace galois;

static thread_local std::string g_last_error;
static thread_local int g_last_kind = 0;
static int fail(const GResult &r) {
    g_last_error = r.msg;
    g_last_kind = (int)r.kind;
    return (int)r.kind;
}

extern "C" {
// GError kind of the failure galois_host_last_error() describes (for functions that return a handle)
int galois_host_last_error_kind() { return g_last_kind; }

const char *galois_host_last_error() { return g_last_error.c_str(); }

void *galois_host_device_new(int ordinal) {
    auto *d = new Device();
    GResult r = CudaDevice::create(ordinal, &d->gpu);
    if (!r.ok()) {
        fail(r);
        delete d;
        return nullptr;
    }
    return d;
}
void *galois_host_device_cpu() { return new Device(); }
// galois_hip_set_option on the device's context (a Cpu device has none)
int galois_host_device_set_option(void *d, int option, int value) {
    auto *dev = (Device *)d;
    if (!dev->is_gpu()) return fail(GError{GError::Unimplemented, "set_option: a Cpu device has no options"});
    GResult r = dev->gpu->check(galois_hip_set_option(dev->gpu->ctx(), option, value));
    return r.ok() ? 0 : fail(r);
}
void galois_host_device_free(void *d) { delete (Device *)d; }

void *galois_host_tensor_from_raw(void *dev, const void *bytes, size_t nbytes, size_t n_dims, const size_t *shape, int dtype) {
    auto *t = new Tensor();
    GResult r = Tensor::from_raw(bytes, nbytes, n_dims, shape, (GGmlType)dtype, *(Device *)dev, t);
    if (!r.ok()) {
        fail(r);
        delete t;
        return nullptr;
    }
    return t;
}
void *galois_host_tensor_zeros(void *dev, size_t n_dims, const size_t *shape, int dtype) {
    auto *t = new Tensor();
    GResult r = Tensor::zeros(n_dims, shape, (GGmlType)dtype, *(Device *)dev, t);
    if (!r.ok()) {
        fail(r);
        delete t;
        return nullptr;
    }
    return t;
}
void *galois_host_tensor_view(void *src, size_t elem_offset, size_t n_dims, const size_t *shape) {
    auto *t = new Tensor();
    GResult r = ((Tensor *)src)->view(elem_offset, n_dims, shape, t);
    if (!r.ok()) {
        fail(r);
        delete t;
        return nullptr;
    }
    return t;
}
int galois_host_tensor_to_cpu(void *src, void *out, size_t nbytes) {
    Tensor c;
    GResult r = ((Tensor *)src)->to_cpu_tensor(&c);
    if (!r.ok()) return fail(r);
    if (nbytes != c.nbytes()) return fail(GError{GError::ShapeError, "to_cpu: byte count mismatch"});
    memcpy(out, c.data(), nbytes);
    return 0;
}
size_t galois_host_tensor_nbytes(void *t) { return ((Tensor *)t)->nbytes(); }
void galois_host_tensor_free(void *t) { delete (Tensor *)t; }

int galois_host_matmul(void *a, void *b, void *dst) {
    GResult r = galois_matmul(*(Tensor *)a, *(Tensor *)b, *(Tensor *)dst);
    return r.ok() ? 0 : fail(r);
}
int galois_host_rms_norm(void *src, void *dst, float eps) {
    GResult r = galois_rms_norm(*(Tensor *)src, *(Tensor *)dst, eps);
    return r.ok() ? 0 : fail(r);
}
int galois_host_rope_custom(size_t n_dims, int mode, int n_ctx, float freq_base, float freq_scale, float xpos_base,
                            int xpos_down, void *src0, void *src1, void *dst) {
    RopeCustomOption op;
    op.n_dims = n_dims, op.mode = mode, op.n_ctx = n_ctx, op.freq_base = freq_base, op.freq_scale = freq_scale;
    op.xpos_base = xpos_base, op.xpos_down = xpos_down != 0;
    GResult r = galois_rope_custom(op, *(Tensor *)src0, *(Tensor *)src1, *(Tensor *)dst);
    return r.ok() ? 0 : fail(r);
}
int galois_host_soft_max(void *src, void *dst) {
    GResult r = galois_soft_max(*(Tensor *)src, *(Tensor *)dst);
    return r.ok() ? 0 : fail(r);
}

void *galois_host_tensor_view_strided(void *src, size_t elem_offset, size_t n_dims, const size_t *shape, const size_t *stride) {
    auto *t = new Tensor();
    GResult r = ((Tensor *)src)->view_strided(elem_offset, n_dims, shape, stride, t);
    if (!r.ok()) {
        fail(r);
        delete t;
        return nullptr;
    }
    return t;
}
int galois_host_tensor_write(void *t, const void *bytes, size_t nbytes) {
    GResult r = ((Tensor *)t)->write(bytes, nbytes);
    return r.ok() ? 0 : fail(r);
}
void *galois_host_tensor_data(void *t) { return ((Tensor *)t)->data(); }

int galois_host_add(void *a, void *b, void *dst) {
    GResult r = galois_add(*(Tensor *)a, *(Tensor *)b, *(Tensor *)dst);
    return r.ok() ? 0 : fail(r);
}
int galois_host_mul(void *a, void *b, void *dst) {
    GResult r = galois_mul(*(Tensor *)a, *(Tensor *)b, *(Tensor *)dst);
    return r.ok() ? 0 : fail(r);
}
int galois_host_unary_silu(void *src, void *dst) {
    GResult r = galois_unary(*(Tensor *)src, *(Tensor *)dst, UnaryOp::Silu);
    return r.ok() ? 0 : fail(r);
}
int galois_host_scale(void *src0, void *src1, void *dst) {
    GResult r = galois_scale(*(Tensor *)src0, *(Tensor *)src1, *(Tensor *)dst);
    return r.ok() ? 0 : fail(r);
}
int galois_host_cpy(void *src, void *dst) {
    GResult r = galois_cpy(*(Tensor *)src, *(Tensor *)dst);
    return r.ok() ? 0 : fail(r);
}
int galois_host_cont(void *src, void *dst) {
    GResult r = galois_cont(*(Tensor *)src, *(Tensor *)dst);
    return r.ok() ? 0 : fail(r);
}
int galois_host_get_rows(void *src0, void *src1, void *dst) {
    GResult r = galois_get_rows(*(Tensor *)src0, *(Tensor *)src1, *(Tensor *)dst);
    return r.ok() ? 0 : fail(r);
}

// ---- LLaMA decode driver -------------------------------------------------------------------------
void *galois_host_llama_new(void *dev, size_t n_vocab, size_t n_embd, size_t n_head, size_t n_layer, size_t n_ff,
                            size_t n_ctx, float rms_eps, float freq_base) {
    LlamaHParams hp;
    hp.n_vocab = n_vocab, hp.n_embd = n_embd, hp.n_head = n_head, hp.n_layer = n_layer, hp.n_ff = n_ff, hp.n_ctx = n_ctx;
    hp.rms_eps = rms_eps, hp.freq_base = freq_base;
    std::unique_ptr<LlamaDecoder> m;
    GResult r = LlamaDecoder::create(hp, *(Device *)dev, &m);
    if (!r.ok()) {
        fail(r);
        return nullptr;
    }
    return m.release();
}
// the same with a choice of KV cache: bit 0 of kv_flags = f16, bit 1 = kept head-major
void *galois_host_llama_new_kv(void *dev, size_t n_vocab, size_t n_embd, size_t n_head, size_t n_layer, size_t n_ff,
                               size_t n_ctx, float rms_eps, float freq_base, int kv_flags) {
    LlamaHParams hp;
    hp.n_vocab = n_vocab, hp.n_embd = n_embd, hp.n_head = n_head, hp.n_layer = n_layer, hp.n_ff = n_ff, hp.n_ctx = n_ctx;
    hp.rms_eps = rms_eps, hp.freq_base = freq_base, hp.kv_f16 = (kv_flags & 1) != 0, hp.kv_head_major = (kv_flags & 2) != 0;
    std::unique_ptr<LlamaDecoder> m;
    GResult r = LlamaDecoder::create(hp, *(Device *)dev, &m);
    if (!r.ok()) {
        fail(r);
        return nullptr;
    }
    return m.release();
}
void galois_host_llama_free(void *m) { delete (LlamaDecoder *)m; }
// borrowed handle: valid while the decoder lives, never passed to galois_host_tensor_free
void *galois_host_llama_tensor(void *m, const char *name, int layer) {
    Tensor *t = ((LlamaDecoder *)m)->tensor(name, layer);
    if (!t) fail(GError{GError::Unexpected, std::string("no tensor named ") + name});
    return t;
}
void *galois_host_llama_logits(void *m) { return (void *)&((LlamaDecoder *)m)->logits(); }
size_t galois_host_llama_ops_per_step(void *m) { return ((LlamaDecoder *)m)->ops_per_step(); }
int galois_host_llama_decode(void *m, int32_t token, int32_t n_past, int fused) {
    GResult r = ((LlamaDecoder *)m)->decode(token, n_past, fused);
    return r.ok() ? 0 : fail(r);
}
int galois_host_llama_prefill(void *m, const int32_t *tokens, size_t n, int32_t n_past) {
    GResult r = ((LlamaDecoder *)m)->prefill(tokens, n, n_past);
    return r.ok() ? 0 : fail(r);
}
size_t galois_host_llama_ops_per_prefill(void *m) { return ((LlamaDecoder *)m)->ops_per_prefill(); }
// `reps` prefills of the same tokens between two events; milliseconds for all of them in *ms
int galois_host_llama_time_prefill(void *m, void *dev, const int32_t *tokens, size_t n, int32_t n_past, int reps, float *ms) {
    galois_hip_ctx *ctx = ((Device *)dev)->gpu->ctx();
    galois_hip_event *e0 = nullptr, *e1 = nullptr;
    int32_t st = galois_hip_event_create(ctx, &e0);
    if (!st) st = galois_hip_event_create(ctx, &e1);
    if (!st) st = galois_hip_event_record(ctx, e0);
    GResult r;
    for (int i = 0; i < reps && !st && r.ok(); i++) r = ((LlamaDecoder *)m)->prefill(tokens, n, n_past);
    if (!st) st = galois_hip_event_record(ctx, e1);
    if (!st) st = galois_hip_event_elapsed_ms(ctx, e0, e1, ms);
    galois_hip_event_destroy(ctx, e0);
    galois_hip_event_destroy(ctx, e1);
    if (!r.ok()) return fail(r);
    if (st) return fail(((Device *)dev)->gpu->check(st));
    return 0;
}
int galois_host_llama_capture(void *m, int32_t token, int32_t n_past, int fused) {
    GResult r = ((LlamaDecoder *)m)->capture(token, n_past, fused);
    return r.ok() ? 0 : fail(r);
}
int galois_host_llama_replay(void *m) {
    GResult r = ((LlamaDecoder *)m)->replay();
    return r.ok() ? 0 : fail(r);
}
// replays the captured step `n` times between two events; milliseconds for all n in *ms
int galois_host_llama_time_replays(void *m, void *dev, int n, float *ms) {
    galois_hip_ctx *ctx = ((Device *)dev)->gpu->ctx();
    galois_hip_event *e0 = nullptr, *e1 = nullptr;
    int32_t st = galois_hip_event_create(ctx, &e0);
    if (!st) st = galois_hip_event_create(ctx, &e1);
    if (!st) st = galois_hip_event_record(ctx, e0);
    GResult r;
    for (int i = 0; i < n && !st && r.ok(); i++) r = ((LlamaDecoder *)m)->replay();
    if (!st) st = galois_hip_event_record(ctx, e1);
    if (!st) st = galois_hip_event_elapsed_ms(ctx, e0, e1, ms);
    galois_hip_event_destroy(ctx, e0);
    galois_hip_event_destroy(ctx, e1);
    if (!r.ok()) return fail(r);
    return st ? fail(GError{GError::DeviceError, galois_hip_last_error(ctx)}) : 0;
}
// same for eager steps (op-by-op launches)
int galois_host_llama_time_steps(void *m, void *dev, int32_t token, int32_t n_past, int fused, int n, float *ms) {
    galois_hip_ctx *ctx = ((Device *)dev)->gpu->ctx();
    galois_hip_event *e0 = nullptr, *e1 = nullptr;
    int32_t st = galois_hip_event_create(ctx, &e0);
    if (!st) st = galois_hip_event_create(ctx, &e1);
    if (!st) st = galois_hip_event_record(ctx, e0);
    GResult r;
    for (int i = 0; i < n && !st && r.ok(); i++) r = ((LlamaDecoder *)m)->decode(token, n_past, fused);
    if (!st) st = galois_hip_event_record(ctx, e1);
    if (!st) st = galois_hip_event_elapsed_ms(ctx, e0, e1, ms);
    galois_hip_event_destroy(ctx, e0);
    galois_hip_event_destroy(ctx, e1);
    if (!r.ok()) return fail(r);
    return st ? fail(GError{GError::DeviceError, galois_hip_last_error(ctx)}) : 0;
}

// ---- GGUF model files -----------------------------------------------------------------------------
// Functions returning a handle return null on failure, functions returning int the GError kind (0 = ok);
// galois_host_last_error() then holds the message.
void *galois_host_gguf_open(const char *path) {
    std::unique_ptr<GgufFile> f;
    GResult r = GgufFile::open(path, &f);
    if (!r.ok()) {
        fail(r);
        return nullptr;
    }
    return f.release();
}
void galois_host_gguf_close(void *f) { delete (GgufFile *)f; }
uint32_t galois_host_gguf_version(void *f) { return ((GgufFile *)f)->version(); }
size_t galois_host_gguf_alignment(void *f) { return ((GgufFile *)f)->alignment(); }
size_t galois_host_gguf_data_start(void *f) { return ((GgufFile *)f)->data_start(); }
size_t galois_host_gguf_n_tensors(void *f) { return ((GgufFile *)f)->tensors().size(); }
size_t galois_host_gguf_n_kv(void *f) { return ((GgufFile *)f)->metadata().size(); }
// name (borrowed, valid while the file is open), n_dims, shape[4], ggml type id, offset, nbytes, supported
const char *galois_host_gguf_tensor_info(void *f, size_t idx, size_t *n_dims, size_t *shape, uint32_t *ggml_type,
                                         uint64_t *offset, size_t *nbytes, int *supported) {
    const auto &ts = ((GgufFile *)f)->tensors();
    if (idx >= ts.size()) {
        fail(GError{GError::Unexpected, "gguf: tensor index out of range"});
        return nullptr;
    }
    const GgufTensorInfo &t = ts[idx];
    *n_dims = t.n_dims;
    for (int d = 0; d < 4; d++) shape[d] = t.shape[d];
    *ggml_type = t.ggml_type, *offset = t.offset, *nbytes = t.nbytes, *supported = t.supported ? 1 : 0;
    return t.name.c_str();
}
int galois_host_gguf_get_uint(void *f, const char *key, uint64_t *out) { return ((GgufFile *)f)->get_uint(key, out) ? 1 : 0; }
int galois_host_gguf_get_float(void *f, const char *key, double *out) { return ((GgufFile *)f)->get_float(key, out) ? 1 : 0; }
// copies at most cap - 1 bytes and a terminator; returns the string's length, or -1 when the key is no string
long galois_host_gguf_get_string(void *f, const char *key, char *buf, size_t cap) {
    std::string s;
    if (!((GgufFile *)f)->get_string(key, &s)) return -1;
    if (cap > 0) {
        const size_t n = s.size() < cap - 1 ? s.size() : cap - 1;
        memcpy(buf, s.data(), n);
        buf[n] = 0;
    }
    return (long)s.size();
}
// number of elements of a string array and the length of element i (copied like get_string); -1 = no such array
long galois_host_gguf_string_array(void *f, const char *key, size_t i, char *buf, size_t cap) {
    std::vector<std::string> v;
    GResult r = ((GgufFile *)f)->get_string_array(key, &v);
    if (!r.ok()) {
        fail(r);
        return -1;
    }
    if (!buf) return (long)v.size();
    if (i >= v.size()) return -1;
    const size_t n = cap == 0 ? 0 : (v[i].size() < cap - 1 ? v[i].size() : cap - 1);
    if (cap > 0) {
        memcpy(buf, v[i].data(), n);
        buf[n] = 0;
    }
    return (long)v[i].size();
}
void *galois_host_gguf_load_tensor(void *f, const char *name, void *dev) {
    Tensor *t = new Tensor();
    GResult r = ((GgufFile *)f)->load_tensor(name, *(Device *)dev, t);
    if (!r.ok()) {
        delete t;
        fail(r);
        return nullptr;
    }
    return t;
}
// hp[6] = n_vocab, n_embd, n_head, n_layer, n_ff, n_ctx; fp[3] = rms_eps, freq_base, freq_scale
int galois_host_gguf_llama_hparams(void *f, size_t n_ctx_max, size_t *hp, float *fp) {
    LlamaHParams h;
    GResult r = llama_hparams_from_gguf(*(GgufFile *)f, n_ctx_max, &h);
    if (!r.ok()) return fail(r);
    hp[0] = h.n_vocab, hp[1] = h.n_embd, hp[2] = h.n_head, hp[3] = h.n_layer, hp[4] = h.n_ff, hp[5] = h.n_ctx;
    fp[0] = h.rms_eps, fp[1] = h.freq_base, fp[2] = h.freq_scale;
    return 0;
}
void *galois_host_llama_from_gguf(void *f, void *dev, size_t n_ctx_max) {
    std::unique_ptr<LlamaDecoder> m;
    GResult r = llama_from_gguf(*(GgufFile *)f, *(Device *)dev, n_ctx_max, &m);
    if (!r.ok()) {
        fail(r);
        return nullptr;
    }
    return m.release();
}

}  // extern "C"
