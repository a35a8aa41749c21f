// LLaMA decode step over the galois op mirror (see llama.hpp).
#include "llama.hpp"

#include <cstring>

#include <cmath>

namespace galois {

static GError err(GError::Kind k, const std::string &m) { return GError{k, m}; }

#define G_TRY(expr)              \
    do {                         \
        GResult r__ = (expr);    \
        if (!r__.ok()) return r__; \
    } while (0)

GResult galois_rms_norm_mul(const Tensor &src, const Tensor &weight, Tensor &dst, float eps) {
    if (!src.device().is_gpu() || !weight.device().is_gpu() || !dst.device().is_gpu())
        return err(GError::Unimplemented, "galois_rms_norm_mul: only (Gpu, Gpu, Gpu)");
    if (src.dtype() != GGmlType::F32 || weight.dtype() != GGmlType::F32 || dst.dtype() != GGmlType::F32)
        return err(GError::Unimplemented, "galois_rms_norm_mul: F32 only");
    if (weight.dim().elem_count() != src.dim().shape[0] || src.dim().elem_count() != dst.dim().elem_count())
        return err(GError::ShapeError, "rms_norm_mul: weight must have ne00 elements, dst the shape of src");
    if (!src.dim().ggml_is_contiguous(src.dtype()) || !dst.dim().ggml_is_contiguous(dst.dtype()) ||
        !weight.dim().ggml_is_contiguous(weight.dtype()))
        return err(GError::Unimplemented, "galois_rms_norm_mul: contiguous operands only (the kernel walks whole rows)");
    const auto &dev = src.device().gpu;
    return dev->check(galois_hip_rms_norm_mul_f32(dev->ctx(), (const float *)src.data(), (const float *)weight.data(),
                                                  (float *)dst.data(), (int32_t)src.dim().shape[0],
                                                  (int32_t)src.dim().nrows(), eps));
}

GResult galois_silu_mul(const Tensor &gate, const Tensor &up, Tensor &dst) {
    if (!gate.device().is_gpu() || !up.device().is_gpu() || !dst.device().is_gpu())
        return err(GError::Unimplemented, "galois_silu_mul: only (Gpu, Gpu, Gpu)");
    if (gate.dtype() != GGmlType::F32 || up.dtype() != GGmlType::F32 || dst.dtype() != GGmlType::F32)
        return err(GError::Unimplemented, "galois_silu_mul: F32 only");
    if (gate.dim().elem_count() != up.dim().elem_count() || gate.dim().elem_count() != dst.dim().elem_count())
        return err(GError::ShapeError, "silu_mul: shapes differ");
    const auto &dev = gate.device().gpu;
    return dev->check(galois_hip_silu_mul_f32(dev->ctx(), (const float *)gate.data(), (const float *)up.data(),
                                              (float *)dst.data(), (int64_t)gate.dim().elem_count()));
}

// Checks the products and writes them as the C ABI's items (at most 8); dev receives their device.
static GResult matvec_items(const std::vector<MatvecItem> &items, galois_hip_gemv_item *it, std::shared_ptr<CudaDevice> &dev) {
    if (items.empty() || items.size() > 8) return err(GError::ShapeError, "galois_matvec_group: 1 to 8 products");
    memset(it, 0, 8 * sizeof(*it));
    for (size_t i = 0; i < items.size(); i++) {
        const MatvecItem &m = items[i];
        if (!m.w || !m.x || !m.dst) return err(GError::Unexpected, "galois_matvec_group: w, x and dst are required");
        for (const Tensor *t : {m.w, m.w_up, m.x, m.norm_weight, m.residual, (const Tensor *)m.dst, (const Tensor *)m.dst_scaled,
                                m.scale_weight, (const Tensor *)m.sumsq_out, m.sumsq_in}) {
            if (!t) continue;
            if (!t->device().is_gpu()) return err(GError::Unimplemented, "galois_matvec_group: Gpu tensors only");
            if (!dev) dev = t->device().gpu;
            if (t->device().gpu != dev) return err(GError::Unimplemented, "galois_matvec_group: one device");
            if (!t->dim().ggml_is_contiguous(t->dtype())) return err(GError::Unimplemented, "galois_matvec_group: contiguous tensors only");
        }
        if (m.w->dtype() != GGmlType::Q4_0 || (m.w_up && m.w_up->dtype() != GGmlType::Q4_0))
            return err(GError::Unimplemented, "galois_matvec_group: Q4_0 matrices only");
        for (const Tensor *t : {m.x, m.norm_weight, m.residual, (const Tensor *)m.dst, (const Tensor *)m.dst_scaled, m.scale_weight,
                                (const Tensor *)m.sumsq_out, m.sumsq_in})
            if (t && t->dtype() != GGmlType::F32) return err(GError::Unimplemented, "galois_matvec_group: F32 vectors only");
        const size_t K = m.w->dim().shape[0], N = m.w->dim().shape[1];
        if (m.w->dim().elem_count() != K * N || m.x->dim().elem_count() != K || m.dst->dim().elem_count() != N ||
            (m.w_up && (m.w_up->dim().shape[0] != K || m.w_up->dim().elem_count() != K * N)) ||
            (m.norm_weight && m.norm_weight->dim().elem_count() != K) || (m.residual && m.residual->dim().elem_count() != N))
            return err(GError::ShapeError, "galois_matvec_group: w [K, N], w_up [K, N], x and norm_weight K, dst and residual N elements");
        if ((m.dst_scaled && m.dst_scaled->dim().elem_count() != N) || (m.scale_weight && m.scale_weight->dim().elem_count() != N) ||
            (m.sumsq_out && m.sumsq_out->dim().elem_count() < (N + 15) / 16) || (m.sumsq_in && m.sumsq_in->dim().elem_count() < (K + 15) / 16))
            return err(GError::ShapeError, "galois_matvec_group: dst_scaled and scale_weight N elements, sumsq_out ceil(N / 16), sumsq_in ceil(K / 16)");
        it[i].dst_scaled = m.dst_scaled ? (float *)m.dst_scaled->data() : nullptr;
        it[i].scale_weight = m.scale_weight ? (const float *)m.scale_weight->data() : nullptr;
        it[i].sumsq_out = m.sumsq_out ? (float *)m.sumsq_out->data() : nullptr;
        it[i].sumsq_in = m.sumsq_in ? (const float *)m.sumsq_in->data() : nullptr;
        it[i].vx = m.w->data(), it[i].vx_up = m.w_up ? m.w_up->data() : nullptr, it[i].y = (const float *)m.x->data();
        it[i].norm_weight = m.norm_weight ? (const float *)m.norm_weight->data() : nullptr;
        it[i].residual = m.residual ? (const float *)m.residual->data() : nullptr;
        it[i].dst = (float *)m.dst->data(), it[i].ncols = (int32_t)K, it[i].nrows = (int32_t)N, it[i].norm_eps = m.eps;
    }
    return GError{};
}

GResult galois_matvec_group(const std::vector<MatvecItem> &items) {
    galois_hip_gemv_item it[8];
    std::shared_ptr<CudaDevice> dev;
    G_TRY(matvec_items(items, it, dev));
    return dev->check(galois_hip_dequantize_mul_mat_vec_q4_0_group(dev->ctx(), it, (int32_t)items.size()));
}

// The checks both attention calls share; dev receives the tensors' device.
// head_major_n_ctx receives 0 for caches [n_embd, n_ctx] and n_ctx for caches [head_dim, n_ctx, n_head].
static GResult attn_check(const RopeCustomOption &op, const Tensor &q, const Tensor &k, const Tensor &v, Tensor &k_cache,
                          Tensor &v_cache, const Tensor &pos, Tensor &out, size_t n_head, int32_t n_past,
                          std::shared_ptr<CudaDevice> &dev, int32_t *head_major_n_ctx) {
    for (const Tensor *t : {&q, &k, &v, (const Tensor *)&k_cache, (const Tensor *)&v_cache, &pos, (const Tensor *)&out}) {
        if (!t->device().is_gpu()) return err(GError::Unimplemented, "galois_attn_decode: Gpu tensors only");
        if (!dev) dev = t->device().gpu;
        if (t->device().gpu != dev) return err(GError::Unimplemented, "galois_attn_decode: one device");
        if (!t->dim().ggml_is_contiguous(t->dtype())) return err(GError::Unimplemented, "galois_attn_decode: contiguous tensors only");
        const bool cache = t == (const Tensor *)&k_cache || t == (const Tensor *)&v_cache;
        const GGmlType want = t == &pos ? GGmlType::I32 : (cache ? k_cache.dtype() : GGmlType::F32);
        if (t->dtype() != want || (cache && want != GGmlType::F32 && want != GGmlType::F16))
            return err(GError::Unimplemented, "galois_attn_decode: F32 vectors, I32 pos, both caches F32 or both F16");
    }
    if (op.mode != 0) return err(GError::Unimplemented, "galois_attn_decode: rope mode 0 only (src/cuda.rs:1336-1340)");
    const size_t E = q.dim().elem_count();
    if (n_head == 0 || E % n_head != 0 || op.n_dims != E / n_head || k.dim().elem_count() != E || v.dim().elem_count() != E ||
        out.dim().elem_count() != E || pos.dim().elem_count() != 1 || n_past < 0 || (size_t)n_past >= k_cache.dim().shape[1] ||
        (size_t)n_past >= v_cache.dim().shape[1])
        return err(GError::ShapeError, "galois_attn_decode: q, k, v, out of n_head * n_dims elements, n_past < n_ctx");
    const bool head_major = k_cache.dim().n_dims == 3;
    for (const Tensor *c : {(const Tensor *)&k_cache, (const Tensor *)&v_cache}) {
        const Dim &d = c->dim();
        const bool ok = head_major ? (d.n_dims == 3 && d.shape[0] == E / n_head && d.shape[2] == n_head && d.shape[1] == k_cache.dim().shape[1])
                                   : (d.n_dims == 2 && d.shape[0] == E);
        if (!ok) return err(GError::ShapeError, "galois_attn_decode: both caches [n_embd, n_ctx] or both [head_dim, n_ctx, n_head]");
    }
    *head_major_n_ctx = head_major ? (int32_t)k_cache.dim().shape[1] : 0;
    return GError{};
}

GResult galois_attn_decode(const RopeCustomOption &op, const Tensor &q, const Tensor &k, const Tensor &v, Tensor &k_cache,
                           Tensor &v_cache, const Tensor &pos, Tensor &out, size_t n_head, int32_t n_past, float scale) {
    std::shared_ptr<CudaDevice> dev;
    int32_t hm = 0;
    G_TRY(attn_check(op, q, k, v, k_cache, v_cache, pos, out, n_head, n_past, dev, &hm));
    const size_t E = q.dim().elem_count();
    const float theta_scale = powf(op.freq_base, -2.0f / (float)op.n_dims);  // as galois_rope_custom derives it (src/cuda.rs:1327)
    if (k_cache.dtype() == GGmlType::F16)
        return dev->check(galois_hip_attn_decode_f16kv(dev->ctx(), (const float *)q.data(), (const float *)k.data(),
                                                       (const float *)v.data(), k_cache.data(), v_cache.data(), (float *)out.data(),
                                                       (int32_t)n_head, (int32_t)(E / n_head), n_past, (const int32_t *)pos.data(),
                                                       op.freq_scale, theta_scale, scale, hm));
    return dev->check(galois_hip_attn_decode_f32(dev->ctx(), (const float *)q.data(), (const float *)k.data(), (const float *)v.data(),
                                                 (float *)k_cache.data(), (float *)v_cache.data(), (float *)out.data(), (int32_t)n_head,
                                                 (int32_t)(E / n_head), n_past, (const int32_t *)pos.data(), op.freq_scale, theta_scale, scale, hm));
}

GResult galois_qkv_attn_decode(const RopeCustomOption &op, const std::vector<MatvecItem> &qkv, Tensor &k_cache, Tensor &v_cache,
                               const Tensor &pos, Tensor &out, size_t n_head, int32_t n_past, float scale) {
    if (qkv.size() != 3) return err(GError::ShapeError, "galois_qkv_attn_decode: the three products q, k, v");
    galois_hip_gemv_item it[8];
    std::shared_ptr<CudaDevice> dev, adev;
    G_TRY(matvec_items(qkv, it, dev));
    int32_t hm = 0;
    G_TRY(attn_check(op, *qkv[0].dst, *qkv[1].dst, *qkv[2].dst, k_cache, v_cache, pos, out, n_head, n_past, adev, &hm));
    if (adev != dev) return err(GError::Unimplemented, "galois_qkv_attn_decode: one device");
    const size_t E = out.dim().elem_count();
    const float theta_scale = powf(op.freq_base, -2.0f / (float)op.n_dims);
    if (k_cache.dtype() == GGmlType::F16)
        return dev->check(galois_hip_qkv_attn_decode_f16kv(dev->ctx(), it, k_cache.data(), v_cache.data(), (float *)out.data(),
                                                           (int32_t)n_head, (int32_t)(E / n_head), n_past,
                                                           (const int32_t *)pos.data(), op.freq_scale, theta_scale, scale, hm));
    return dev->check(galois_hip_qkv_attn_decode_f32(dev->ctx(), it, (float *)k_cache.data(), (float *)v_cache.data(),
                                                     (float *)out.data(), (int32_t)n_head, (int32_t)(E / n_head), n_past,
                                                     (const int32_t *)pos.data(), op.freq_scale, theta_scale, scale, hm));
}

static GResult mk(Tensor *t, GGmlType ty, const Device &dev, size_t ne0, size_t ne1 = 0, size_t ne2 = 0) {
    const size_t shape[3] = {ne0, ne1, ne2};
    return Tensor::zeros(ne2 ? 3 : (ne1 ? 2 : 1), shape, ty, dev, t);
}

GResult LlamaDecoder::create(const LlamaHParams &hp, const Device &dev, std::unique_ptr<LlamaDecoder> *out) {
    if (!dev.is_gpu()) return err(GError::Unimplemented, "LlamaDecoder: Gpu device only");
    if (hp.n_head == 0 || hp.n_embd % hp.n_head != 0 || (hp.n_embd / hp.n_head) % 2 != 0)
        return err(GError::ShapeError, "LlamaDecoder: n_embd must split into n_head even-sized heads");
    if (hp.n_embd % 32 != 0 || hp.n_ff % 32 != 0) return err(GError::ShapeError, "LlamaDecoder: n_embd and n_ff must be multiples of 32");
    std::unique_ptr<LlamaDecoder> m(new LlamaDecoder());
    m->hp_ = hp;
    m->dev_ = dev;
    const size_t E = hp.n_embd, F = hp.n_ff, V = hp.n_vocab, C = hp.n_ctx, H = hp.n_head, D = E / H;
    const GGmlType Q = GGmlType::Q4_0, F32 = GGmlType::F32;
    G_TRY(mk(&m->tok_embd_, Q, dev, E, V));
    G_TRY(mk(&m->out_norm_, F32, dev, E));
    G_TRY(mk(&m->output_, Q, dev, E, V));
    m->layers_.resize(hp.n_layer);
    for (Layer &l : m->layers_) {
        G_TRY(mk(&l.attn_norm, F32, dev, E));
        G_TRY(mk(&l.ffn_norm, F32, dev, E));
        G_TRY(mk(&l.wq, Q, dev, E, E));
        G_TRY(mk(&l.wk, Q, dev, E, E));
        G_TRY(mk(&l.wv, Q, dev, E, E));
        G_TRY(mk(&l.wo, Q, dev, E, E));
        G_TRY(mk(&l.w_gate, Q, dev, E, F));
        G_TRY(mk(&l.w_up, Q, dev, E, F));
        G_TRY(mk(&l.w_down, Q, dev, F, E));
        const GGmlType ct = hp.kv_f16 ? GGmlType::F16 : F32;
        if (hp.kv_head_major) {
            G_TRY(mk(&l.k_cache, ct, dev, D, C, H));
            G_TRY(mk(&l.v_cache, ct, dev, D, C, H));
        } else {
            G_TRY(mk(&l.k_cache, ct, dev, E, C));
            G_TRY(mk(&l.v_cache, ct, dev, E, C));
        }
    }
    G_TRY(mk(&m->tok_id_, GGmlType::I32, dev, 1));
    G_TRY(mk(&m->pos_, GGmlType::I32, dev, 1));
    G_TRY(mk(&m->scale_, F32, Device{}, 1));
    *(float *)m->scale_.data() = 1.0f / sqrtf((float)D);
    for (Tensor *t : {&m->x_, &m->t_, &m->a_, &m->q_, &m->k_, &m->v_, &m->ao_, &m->x1_, &m->f_, &m->d_}) G_TRY(mk(t, F32, dev, E, 1));
    G_TRY(mk(&m->qr_, F32, dev, D, H, 1));
    G_TRY(mk(&m->kr_, F32, dev, D, H, 1));
    G_TRY(mk(&m->s_, F32, dev, C, 1, H));
    G_TRY(mk(&m->p_, F32, dev, C, 1, H));
    G_TRY(mk(&m->o_, F32, dev, D, 1, H));
    for (Tensor *t : {&m->g_, &m->u_, &m->h_}) G_TRY(mk(t, F32, dev, F, 1));
    G_TRY(mk(&m->logits_, F32, dev, V, 1));
    G_TRY(mk(&m->ssq_, F32, dev, (E + 15) / 16));
    G_TRY(mk(&m->ssq1_, F32, dev, (E + 15) / 16));
    *out = std::move(m);
    return GError{};
}

LlamaDecoder::~LlamaDecoder() {
    if (graph_) galois_hip_graph_destroy(dev_.gpu->ctx(), graph_);
}

Tensor *LlamaDecoder::tensor(const std::string &name, int layer) {
    if (layer < 0) {
        if (name == "tok_embd") return &tok_embd_;
        if (name == "out_norm") return &out_norm_;
        if (name == "output") return &output_;
        return nullptr;
    }
    if ((size_t)layer >= layers_.size()) return nullptr;
    Layer &l = layers_[layer];
    const std::pair<const char *, Tensor *> names[] = {
        {"attn_norm", &l.attn_norm}, {"ffn_norm", &l.ffn_norm}, {"wq", &l.wq}, {"wk", &l.wk}, {"wv", &l.wv}, {"wo", &l.wo},
        {"w_gate", &l.w_gate}, {"w_up", &l.w_up}, {"w_down", &l.w_down}, {"k_cache", &l.k_cache}, {"v_cache", &l.v_cache}};
    for (const auto &n : names)
        if (name == n.first) return n.second;
    return nullptr;
}

GResult LlamaDecoder::set_inputs(int32_t token, int32_t n_past) {
    if (token < 0 || (size_t)token >= hp_.n_vocab) return err(GError::ShapeError, "decode: token id out of range");
    if (n_past < 0 || (size_t)n_past >= hp_.n_ctx) return err(GError::ShapeError, "decode: n_past must be below n_ctx");
    if (token != last_token_) G_TRY(tok_id_.write(&token, sizeof(token)));  // synchronous copies: only when they change
    if (n_past != last_pos_) G_TRY(pos_.write(&n_past, sizeof(n_past)));
    last_token_ = token, last_pos_ = n_past;
    return GError{};
}

// The op sequence of one token.  Shapes in ggml order [ne0, ne1, ne2]; L = n_past + 1 keys are visible,
// so the softmax needs no mask.
GResult LlamaDecoder::step(int32_t n_past, int fused) {
    if (hp_.kv_f16 && fused < 3)
        return err(GError::Unimplemented, "LlamaDecoder: an f16 KV cache runs with the fused attention only (fused = 3)");
    // the grouped launches take vectors of a multiple of 64 up to 12288 elements (one pass through LDS)
    if (fused >= 2 && (hp_.n_embd % 64 != 0 || hp_.n_ff % 64 != 0 || hp_.n_embd > 12288 || hp_.n_ff > 12288))
        return err(GError::Unimplemented, "LlamaDecoder: the grouped launch plans (fused >= 2) need n_embd and n_ff to be "
                                          "multiples of 64 no larger than 12288; use fused = 0 or 1");
    const size_t E = hp_.n_embd, H = hp_.n_head, D = E / H, L = (size_t)n_past + 1, C = hp_.n_ctx;
    if (fused >= 5 && (D != 128 || E > 11776))
        return err(GError::Unimplemented, "LlamaDecoder: the launch that carries q | k | v and the attention (fused = 5) needs heads of 128 "
                                          "and n_embd up to 11776");
    RopeCustomOption rope;
    rope.n_dims = D, rope.mode = 0, rope.n_ctx = (int32_t)C, rope.freq_base = hp_.freq_base, rope.freq_scale = hp_.freq_scale;
    size_t ops = 0;
    auto norm = [&](const Tensor &src, const Tensor &w, Tensor &dst) -> GResult {
        if (fused) {
            ops += 1;
            return galois_rms_norm_mul(src, w, dst, hp_.rms_eps);
        }
        ops += 2;
        G_TRY(galois_rms_norm(src, t_, hp_.rms_eps));
        return galois_mul(t_, w, dst);
    };
    // views that depend on L: the first L scores of every head are packed as [L, 1, H]
    Tensor s, p, q3, k_row, v_row;
    {
        const size_t sh[3] = {L, 1, H};
        G_TRY(s_.view(0, 3, sh, &s));
        G_TRY(p_.view(0, 3, sh, &p));
        const size_t qs[3] = {D, 1, H};
        G_TRY(qr_.view(0, 3, qs, &q3));
    }
    G_TRY(galois_get_rows(tok_embd_, tok_id_, x_)); ops++;
    const bool grouped = fused >= 2;
    auto item = [&](const Tensor &w, const Tensor &x, Tensor &dst) {
        MatvecItem m;
        m.w = &w, m.x = &x, m.dst = &dst, m.eps = hp_.rms_eps;
        return m;
    };
    for (Layer &l : layers_) {
        const size_t li = (size_t)(&l - &layers_[0]);
        const bool split = fused >= 4;       // norms split over producer and consumer launches
        const bool qkv_attn = fused >= 5;    // the three projections and the attention in one launch
        if (grouped) {  // rms_norm * weight + the three projections: one launch
            MatvecItem mq = item(l.wq, x_, q_), mk_ = item(l.wk, x_, k_), mv = item(l.wv, x_, v_);
            if (split && li > 0) {  // the previous layer's last launch left x * attn_norm in a_ and the sums of squares of x
                mq.x = mk_.x = mv.x = &a_;
                mq.sumsq_in = mk_.sumsq_in = mv.sumsq_in = &ssq_;
            } else {
                mq.norm_weight = mk_.norm_weight = mv.norm_weight = &l.attn_norm;
            }
            if (qkv_attn) {
                G_TRY(galois_qkv_attn_decode(rope, {mq, mk_, mv}, l.k_cache, l.v_cache, pos_, ao_, H, n_past, *(const float *)scale_.data()));
            } else {
                G_TRY(galois_matvec_group({mq, mk_, mv}));
            }
            ops++;
        } else {
            G_TRY(norm(x_, l.attn_norm, a_));
            G_TRY(galois_matmul(l.wq, a_, q_));
            G_TRY(galois_matmul(l.wk, a_, k_));
            G_TRY(galois_matmul(l.wv, a_, v_)); ops += 3;
        }
        if (fused >= 3) {  // the eight attention ops as one launch, then the grouped tail of the layer
            if (!qkv_attn) {
                G_TRY(galois_attn_decode(rope, q_, k_, v_, l.k_cache, l.v_cache, pos_, ao_, H, n_past, *(const float *)scale_.data()));
                ops++;
            }
            MatvecItem mo = item(l.wo, ao_, x1_);
            mo.residual = &x_;
            if (split) mo.dst_scaled = &f_, mo.scale_weight = &l.ffn_norm, mo.sumsq_out = &ssq1_;
            G_TRY(galois_matvec_group({mo})); ops++;
            MatvecItem mg = item(l.w_gate, split ? f_ : x1_, h_);
            mg.w_up = &l.w_up;
            if (split)
                mg.sumsq_in = &ssq1_;
            else
                mg.norm_weight = &l.ffn_norm;
            G_TRY(galois_matvec_group({mg})); ops++;
            MatvecItem md = item(l.w_down, h_, x_);
            md.residual = &x1_;
            if (split)  // x times the weight of the norm that reads it next: the next layer's, or the output norm
                md.dst_scaled = &a_, md.scale_weight = li + 1 < layers_.size() ? &layers_[li + 1].attn_norm : &out_norm_, md.sumsq_out = &ssq_;
            G_TRY(galois_matvec_group({md})); ops++;
            continue;
        }
        Tensor qv, kv;
        const size_t hs[3] = {D, H, 1};
        G_TRY(q_.view(0, 3, hs, &qv));
        G_TRY(k_.view(0, 3, hs, &kv));
        G_TRY(galois_rope_custom(rope, qv, pos_, qr_));
        G_TRY(galois_rope_custom(rope, kv, pos_, kr_)); ops += 2;
        // append this position to the cache: row n_past of [n_ctx][E], or row n_past of every head of [H][n_ctx][D]
        const size_t row[2] = {E, 1};
        const bool hm = hp_.kv_head_major;
        if (hm) {
            const size_t rsh[2] = {D, H}, rst[2] = {1, C * D};
            G_TRY(l.k_cache.view_strided((size_t)n_past * D, 2, rsh, rst, &k_row));
            G_TRY(l.v_cache.view_strided((size_t)n_past * D, 2, rsh, rst, &v_row));
            Tensor kr2, v2;
            G_TRY(kr_.view(0, 2, rsh, &kr2));
            G_TRY(v_.view(0, 2, rsh, &v2));
            G_TRY(galois_cpy(kr2, k_row));
            G_TRY(galois_cpy(v2, v_row));
        } else {
            G_TRY(l.k_cache.view((size_t)n_past * E, 2, row, &k_row));
            G_TRY(l.v_cache.view((size_t)n_past * E, 2, row, &v_row));
            Tensor kr_flat;
            G_TRY(kr_.view(0, 2, row, &kr_flat));
            G_TRY(galois_cpy(kr_flat, k_row));
            G_TRY(galois_cpy(v_, v_row));
        }
        ops += 2;
        // scores = K^T q per head: K seen as [D, L, H] with strides (1, E, D), or (1, D, n_ctx * D) in a head-major cache
        Tensor kc, vc;
        const size_t ksh[3] = {D, L, H}, kst[3] = {1, hm ? D : E, hm ? C * D : D};
        G_TRY(l.k_cache.view_strided(0, 3, ksh, kst, &kc));
        G_TRY(galois_matmul(kc, q3, s));
        G_TRY(galois_scale(s, scale_, s));
        G_TRY(galois_soft_max(s, p)); ops += 3;
        // out = V p per head: V seen as [L, D, H] with strides (E, 1, D), or (D, 1, n_ctx * D)
        const size_t vsh[3] = {L, D, H}, vst[3] = {hm ? D : E, 1, hm ? C * D : D};
        G_TRY(l.v_cache.view_strided(0, 3, vsh, vst, &vc));
        G_TRY(galois_matmul(vc, p, o_)); ops++;
        Tensor o_flat;
        G_TRY(o_.view(0, 2, row, &o_flat));
        if (grouped) {
            MatvecItem mo = item(l.wo, o_flat, x1_);  // x1 = wo . o + x
            mo.residual = &x_;
            G_TRY(galois_matvec_group({mo})); ops++;
            MatvecItem mg = item(l.w_gate, x1_, h_);  // h = silu(w_gate . n) * (w_up . n), n = rms_norm(x1) * ffn_norm
            mg.w_up = &l.w_up, mg.norm_weight = &l.ffn_norm;
            G_TRY(galois_matvec_group({mg})); ops++;
            MatvecItem md = item(l.w_down, h_, x_);   // x = w_down . h + x1
            md.residual = &x1_;
            G_TRY(galois_matvec_group({md})); ops++;
            continue;
        }
        G_TRY(galois_matmul(l.wo, o_flat, ao_));
        G_TRY(galois_add(ao_, x_, x1_)); ops += 2;
        G_TRY(norm(x1_, l.ffn_norm, f_));
        G_TRY(galois_matmul(l.w_gate, f_, g_));
        G_TRY(galois_matmul(l.w_up, f_, u_)); ops += 2;
        if (fused) {
            G_TRY(galois_silu_mul(g_, u_, h_)); ops++;
        } else {
            G_TRY(galois_unary(g_, h_, UnaryOp::Silu));
            G_TRY(galois_mul(h_, u_, h_)); ops += 2;
        }
        G_TRY(galois_matmul(l.w_down, h_, d_));
        G_TRY(galois_add(d_, x1_, x_)); ops += 2;
    }
    if (grouped) {
        MatvecItem ml = item(output_, x_, logits_);
        if (fused >= 4)
            ml.x = &a_, ml.sumsq_in = &ssq_;
        else
            ml.norm_weight = &out_norm_;
        G_TRY(galois_matvec_group({ml})); ops++;
    } else {
        G_TRY(norm(x_, out_norm_, a_));
        G_TRY(galois_matmul(output_, a_, logits_)); ops++;
    }
    n_ops_ = ops;
    return GError{};
}

GResult LlamaDecoder::decode(int32_t token, int32_t n_past, int fused) {
    G_TRY(set_inputs(token, n_past));
    return step(n_past, fused);
}

GResult LlamaDecoder::capture(int32_t token, int32_t n_past, int fused) {
    galois_hip_ctx *ctx = dev_.gpu->ctx();
    if (graph_) {
        G_TRY(dev_.gpu->check(galois_hip_graph_destroy(ctx, graph_)));
        graph_ = nullptr;
    }
    G_TRY(set_inputs(token, n_past));
    G_TRY(dev_.gpu->check(galois_hip_graph_begin_capture(ctx)));
    GResult r = step(n_past, fused);
    galois_hip_graph *g = nullptr;
    GResult e = dev_.gpu->check(galois_hip_graph_end_capture(ctx, &g));  // always close the capture
    if (!r.ok()) {
        if (g) galois_hip_graph_destroy(ctx, g);
        return r;
    }
    G_TRY(e);
    graph_ = g;
    return GError{};
}

GResult LlamaDecoder::replay() {
    if (!graph_) return err(GError::Unexpected, "replay: no step has been captured");
    return dev_.gpu->check(galois_hip_graph_launch(dev_.gpu->ctx(), graph_));
}

}  // namespace galois
