// Prefill of the LLaMA driver: many tokens through the graph in one pass (see llama.hpp).
#include <cmath>
#include <cstring>

#include "llama.hpp"

namespace galois {

static GError err(GError::Kind k, const std::string &m) { return GError{k, m}; }

#define G_TRY(expr)              \
    do {                         \
        GResult r__ = (expr);    \
        if (!r__.ok()) return r__; \
    } while (0)

size_t galois_panel_elems(size_t K, size_t M) { return (M + 15) / 16 * 16 * K; }

// src [K, M] f32 contiguous on the Gpu, panel F16 with room for its panel: returns the device, K and M.
static GResult panel_operands(const Tensor &src, const Tensor &panel, std::shared_ptr<CudaDevice> *dev, size_t *K, size_t *M,
                              const char *what) {
    if (!src.device().is_gpu() || !panel.device().is_gpu() || src.device().gpu != panel.device().gpu)
        return err(GError::Unimplemented, std::string(what) + ": Gpu tensors on one device");
    if (src.dtype() != GGmlType::F32 || panel.dtype() != GGmlType::F16)
        return err(GError::Unimplemented, std::string(what) + ": F32 source, F16 panel");
    if (!src.dim().ggml_is_contiguous(src.dtype()) || !panel.dim().ggml_is_contiguous(panel.dtype()))
        return err(GError::Unimplemented, std::string(what) + ": contiguous tensors only");
    *K = src.dim().shape[0], *M = src.dim().nrows();
    if (panel.dim().elem_count() < galois_panel_elems(*K, *M))
        return err(GError::ShapeError, std::string(what) + ": the panel tensor is smaller than galois_panel_elems(K, M)");
    *dev = src.device().gpu;
    return GError{};
}

GResult galois_rms_norm_mul_panel(const Tensor &src, const Tensor &weight, Tensor &panel, float eps) {
    std::shared_ptr<CudaDevice> dev;
    size_t K, M;
    G_TRY(panel_operands(src, panel, &dev, &K, &M, "galois_rms_norm_mul_panel"));
    if (!weight.device().is_gpu() || weight.dtype() != GGmlType::F32 || weight.dim().elem_count() != K)
        return err(GError::ShapeError, "galois_rms_norm_mul_panel: weight must be ne00 F32 elements on the Gpu");
    return dev->check(galois_hip_rms_norm_mul_f16_panel(dev->ctx(), (const float *)src.data(), (const float *)weight.data(),
                                                        panel.data(), (int32_t)K, (int32_t)M, eps));
}

GResult galois_silu_mul_panel(const Tensor &gate, const Tensor &up, Tensor &panel) {
    std::shared_ptr<CudaDevice> dev;
    size_t K, M;
    G_TRY(panel_operands(gate, panel, &dev, &K, &M, "galois_silu_mul_panel"));
    if (!up.device().is_gpu() || up.dtype() != GGmlType::F32 || up.dim().elem_count() != gate.dim().elem_count() ||
        !up.dim().ggml_is_contiguous(up.dtype()))
        return err(GError::ShapeError, "galois_silu_mul_panel: up must have the shape of gate");
    return dev->check(galois_hip_silu_mul_f16_panel(dev->ctx(), (const float *)gate.data(), (const float *)up.data(), panel.data(),
                                                    (int32_t)K, (int32_t)M));
}

GResult galois_to_panel(const Tensor &src, Tensor &panel) {
    std::shared_ptr<CudaDevice> dev;
    size_t K, M;
    G_TRY(panel_operands(src, panel, &dev, &K, &M, "galois_to_panel"));
    return dev->check(galois_hip_f32_to_f16_panel(dev->ctx(), (const float *)src.data(), panel.data(), (int32_t)K, (int32_t)M));
}

GResult galois_matmul_panel(const std::vector<PanelMatmulItem> &items, const Tensor &panel, size_t K, size_t M) {
    if (items.empty() || items.size() > 4) return err(GError::ShapeError, "galois_matmul_panel: 1 to 4 matrices");
    if (!panel.device().is_gpu() || panel.dtype() != GGmlType::F16 || panel.dim().elem_count() < galois_panel_elems(K, M))
        return err(GError::ShapeError, "galois_matmul_panel: an F16 Gpu panel of galois_panel_elems(K, M) elements");
    const auto &dev = panel.device().gpu;
    galois_hip_gemm_item it[4];
    memset(it, 0, sizeof(it));
    for (size_t j = 0; j < items.size(); j++) {
        const Tensor *w = items[j].w;
        Tensor *d = items[j].dst;
        if (!w || !d) return err(GError::Unexpected, "galois_matmul_panel: w and dst are required");
        if (!w->device().is_gpu() || !d->device().is_gpu() || w->device().gpu != dev || d->device().gpu != dev)
            return err(GError::Unimplemented, "galois_matmul_panel: Gpu tensors on the panel's device");
        if (w->dtype() != GGmlType::Q4_0 || d->dtype() != GGmlType::F32 || !w->dim().ggml_is_contiguous(w->dtype()) ||
            !d->dim().ggml_is_contiguous(d->dtype()))
            return err(GError::Unimplemented, "galois_matmul_panel: contiguous Q4_0 matrices and F32 results");
        const size_t N = w->dim().shape[1];
        if (w->dim().shape[0] != K || w->dim().elem_count() != K * N || d->dim().elem_count() != N * M)
            return err(GError::ShapeError, "galois_matmul_panel: w [K, N], dst [N, M]");
        it[j].W = w->data(), it[j].Y = (float *)d->data(), it[j].N = (int32_t)N;
    }
    return dev->check(galois_hip_mul_mat_q4_0_f16_panel(dev->ctx(), it, (int32_t)items.size(), panel.data(), (int32_t)K, (int32_t)M));
}

GResult galois_matmul_panel_add(const Tensor &w, const Tensor &panel, const Tensor *residual, Tensor &dst, size_t K, size_t M,
                                Tensor *workspace) {
    if (!panel.device().is_gpu() || panel.dtype() != GGmlType::F16 || panel.dim().elem_count() < galois_panel_elems(K, M))
        return err(GError::ShapeError, "galois_matmul_panel_add: an F16 Gpu panel of galois_panel_elems(K, M) elements");
    const auto &dev = panel.device().gpu;
    for (const Tensor *t : {&w, (const Tensor *)&dst, residual, (const Tensor *)workspace})
        if (t && (!t->device().is_gpu() || t->device().gpu != dev))
            return err(GError::Unimplemented, "galois_matmul_panel_add: Gpu tensors on the panel's device");
    if (w.dtype() != GGmlType::Q4_0 || dst.dtype() != GGmlType::F32 || !w.dim().ggml_is_contiguous(w.dtype()) ||
        !dst.dim().ggml_is_contiguous(dst.dtype()))
        return err(GError::Unimplemented, "galois_matmul_panel_add: a contiguous Q4_0 matrix and an F32 result");
    const size_t N = w.dim().shape[1];
    if (w.dim().shape[0] != K || w.dim().elem_count() != K * N || dst.dim().elem_count() != N * M)
        return err(GError::ShapeError, "galois_matmul_panel_add: w [K, N], dst [N, M]");
    if (residual && (residual->dtype() != GGmlType::F32 || !residual->dim().ggml_is_contiguous(residual->dtype()) ||
                     residual->dim().elem_count() != N * M))
        return err(GError::ShapeError, "galois_matmul_panel_add: residual F32 [N, M]");
    if (workspace && (workspace->dtype() != GGmlType::F32 || !workspace->dim().ggml_is_contiguous(workspace->dtype())))
        return err(GError::ShapeError, "galois_matmul_panel_add: workspace contiguous F32");
    return dev->check(galois_hip_mul_mat_q4_0_f16_panel_add(
        dev->ctx(), w.data(), panel.data(), residual ? (const float *)residual->data() : nullptr, (float *)dst.data(), (int32_t)K,
        (int32_t)N, (int32_t)M, workspace ? workspace->data() : nullptr,
        workspace ? (int64_t)(workspace->dim().elem_count() * sizeof(float)) : 0));
}

GResult galois_matmul_swiglu_panel(const Tensor &w_gate, const Tensor &w_up, const Tensor &panel, Tensor &panel_out, size_t K, size_t M) {
    if (!panel.device().is_gpu() || panel.dtype() != GGmlType::F16 || panel.dim().elem_count() < galois_panel_elems(K, M))
        return err(GError::ShapeError, "galois_matmul_swiglu_panel: an F16 Gpu panel of galois_panel_elems(K, M) elements");
    const auto &dev = panel.device().gpu;
    for (const Tensor *t : {&w_gate, &w_up, (const Tensor *)&panel_out})
        if (!t->device().is_gpu() || t->device().gpu != dev)
            return err(GError::Unimplemented, "galois_matmul_swiglu_panel: Gpu tensors on the panel's device");
    const size_t N = w_gate.dim().shape[1];
    for (const Tensor *w : {&w_gate, &w_up})
        if (w->dtype() != GGmlType::Q4_0 || !w->dim().ggml_is_contiguous(w->dtype()) || w->dim().shape[0] != K ||
            w->dim().elem_count() != K * N)
            return err(GError::ShapeError, "galois_matmul_swiglu_panel: w_gate and w_up contiguous Q4_0 [K, N]");
    if (panel_out.dtype() != GGmlType::F16 || !panel_out.dim().ggml_is_contiguous(panel_out.dtype()) ||
        panel_out.dim().elem_count() < galois_panel_elems(N, M) || panel_out.data() == panel.data())
        return err(GError::ShapeError, "galois_matmul_swiglu_panel: panel_out a second F16 tensor of galois_panel_elems(N, M) elements");
    return dev->check(galois_hip_mul_mat_q4_0_swiglu_f16_panel(dev->ctx(), w_gate.data(), w_up.data(), panel.data(), panel_out.data(),
                                                               (int32_t)K, (int32_t)N, (int32_t)M));
}

GResult galois_matmul_panel_shares(const Tensor &w, const Tensor &panel, Tensor &shares, size_t K, size_t M, int32_t *n_shares) {
    if (!n_shares) return err(GError::Unexpected, "galois_matmul_panel_shares: n_shares is required");
    if (!panel.device().is_gpu() || panel.dtype() != GGmlType::F16 || panel.dim().elem_count() < galois_panel_elems(K, M))
        return err(GError::ShapeError, "galois_matmul_panel_shares: an F16 Gpu panel of galois_panel_elems(K, M) elements");
    const auto &dev = panel.device().gpu;
    if (!w.device().is_gpu() || w.device().gpu != dev || !shares.device().is_gpu() || shares.device().gpu != dev)
        return err(GError::Unimplemented, "galois_matmul_panel_shares: Gpu tensors on the panel's device");
    if (w.dtype() != GGmlType::Q4_0 || shares.dtype() != GGmlType::F32 || !w.dim().ggml_is_contiguous(w.dtype()) ||
        !shares.dim().ggml_is_contiguous(shares.dtype()))
        return err(GError::Unimplemented, "galois_matmul_panel_shares: a contiguous Q4_0 matrix and an F32 tensor for the shares");
    const size_t N = w.dim().shape[1];
    if (w.dim().shape[0] != K || w.dim().elem_count() != K * N || shares.dim().elem_count() < N * M)
        return err(GError::ShapeError, "galois_matmul_panel_shares: w [K, N], shares of at least N * M elements");
    return dev->check(galois_hip_mul_mat_q4_0_f16_panel_shares(dev->ctx(), w.data(), panel.data(), (float *)shares.data(),
                                                               (int64_t)(shares.dim().elem_count() * sizeof(float)), (int32_t)K,
                                                               (int32_t)N, (int32_t)M, n_shares));
}

GResult galois_add_rms_norm_mul_panel(const Tensor &shares, int32_t n_shares, const Tensor *residual, Tensor &sum_out,
                                      const Tensor &weight, Tensor &panel, float eps) {
    std::shared_ptr<CudaDevice> dev;
    size_t K, M;
    G_TRY(panel_operands(sum_out, panel, &dev, &K, &M, "galois_add_rms_norm_mul_panel"));
    if (n_shares < 1 || n_shares > 2) return err(GError::ShapeError, "galois_add_rms_norm_mul_panel: one or two shares");
    if (!shares.device().is_gpu() || shares.device().gpu != dev || shares.dtype() != GGmlType::F32 ||
        !shares.dim().ggml_is_contiguous(shares.dtype()) || shares.dim().elem_count() < (size_t)n_shares * K * M)
        return err(GError::ShapeError, "galois_add_rms_norm_mul_panel: shares F32 on the Gpu, n_shares results of sum_out's size");
    if (residual && (!residual->device().is_gpu() || residual->device().gpu != dev || residual->dtype() != GGmlType::F32 ||
                     !residual->dim().ggml_is_contiguous(residual->dtype()) || residual->dim().elem_count() != K * M))
        return err(GError::ShapeError, "galois_add_rms_norm_mul_panel: residual F32 of sum_out's shape");
    if (!weight.device().is_gpu() || weight.dtype() != GGmlType::F32 || weight.dim().elem_count() != K)
        return err(GError::ShapeError, "galois_add_rms_norm_mul_panel: weight must be ne00 F32 elements on the Gpu");
    const float *a = (const float *)shares.data();
    return dev->check(galois_hip_add_rms_norm_mul_f16_panel(dev->ctx(), a, n_shares == 2 ? a + K * M : nullptr,
                                                            residual ? (const float *)residual->data() : nullptr, (float *)sum_out.data(),
                                                            (const float *)weight.data(), panel.data(), (int32_t)K, (int32_t)M, eps));
}

GResult galois_rope_qk_append(const RopeCustomOption &op, const Tensor &q, const Tensor &k, const Tensor *v, const Tensor &pos,
                              Tensor &q_out, Tensor &k_rows, Tensor *v_rows) {
    if ((v == nullptr) != (v_rows == nullptr)) return err(GError::Unexpected, "galois_rope_qk_append: v and v_rows together or neither");
    const auto &dev = q.device().gpu;
    for (const Tensor *t : {&q, &k, v, &pos, (const Tensor *)&q_out, (const Tensor *)&k_rows, (const Tensor *)v_rows})
        if (t && (!t->device().is_gpu() || t->device().gpu != dev || !t->dim().ggml_is_contiguous(t->dtype())))
            return err(GError::Unimplemented, "galois_rope_qk_append: contiguous Gpu tensors on one device");
    if (op.mode != 0) return err(GError::Unimplemented, "galois_rope_qk_append: mode 0");
    if (q.dtype() != GGmlType::F32 || k.dtype() != GGmlType::F32 || q_out.dtype() != GGmlType::F32 || (v && v->dtype() != GGmlType::F32) ||
        pos.dtype() != GGmlType::I32)
        return err(GError::Unimplemented, "galois_rope_qk_append: F32 q, k, v, q_out and I32 positions");
    const GGmlType ct = k_rows.dtype();
    if ((ct != GGmlType::F32 && ct != GGmlType::F16) || (v_rows && v_rows->dtype() != ct))
        return err(GError::Unimplemented, "galois_rope_qk_append: cache rows both F32 or both F16");
    const size_t D = q.dim().shape[0], H = q.dim().shape[1], n = q.dim().shape[2], total = D * H * n;
    if (q.dim().n_dims != 3 || op.n_dims != D || D % 4 != 0 || D > 256 || pos.dim().shape[0] != n)
        return err(GError::ShapeError, "galois_rope_qk_append: q [head_dim, n_head, n] with n_dims = head_dim (a multiple of 4 up to 256), one position per token");
    for (const Tensor *t : {&k, v, (const Tensor *)&q_out, (const Tensor *)&k_rows, (const Tensor *)v_rows})
        if (t && t->dim().elem_count() != total) return err(GError::ShapeError, "galois_rope_qk_append: every tensor has q's element count");
    const float theta_scale = powf(op.freq_base, -2.0f / (float)op.n_dims);  // as galois_rope_custom derives it (src/cuda.rs:1327)
    return dev->check(galois_hip_rope_qk_append(dev->ctx(), (const float *)q.data(), (const float *)k.data(),
                                                v ? (const float *)v->data() : nullptr, (float *)q_out.data(), k_rows.data(),
                                                v_rows ? v_rows->data() : nullptr, ct == GGmlType::F16, (int32_t)D, (int32_t)H, (int32_t)n,
                                                (const int32_t *)pos.data(), op.freq_scale, theta_scale));
}

GResult galois_attn_prefill(const Tensor &q, const Tensor &k_cache, const Tensor &v_cache, Tensor &dst, size_t n_head,
                            int32_t n_past, float scale) {
    for (const Tensor *t : {&q, &k_cache, &v_cache, (const Tensor *)&dst})
        if (!t->device().is_gpu() || t->device().gpu != q.device().gpu)
            return err(GError::Unimplemented, "galois_attn_prefill: Gpu tensors on one device");
    if (q.dtype() != GGmlType::F32 || !q.dim().ggml_is_contiguous(q.dtype()))
        return err(GError::Unimplemented, "galois_attn_prefill: q contiguous F32");
    if (k_cache.dtype() != v_cache.dtype() || (k_cache.dtype() != GGmlType::F32 && k_cache.dtype() != GGmlType::F16) ||
        !k_cache.dim().ggml_is_contiguous(k_cache.dtype()) || !v_cache.dim().ggml_is_contiguous(v_cache.dtype()))
        return err(GError::Unimplemented, "galois_attn_prefill: contiguous caches, both F32 or both F16");
    const size_t E = q.dim().shape[0], n = q.dim().nrows();
    if (n_head == 0 || E % n_head != 0 || n_past < 0) return err(GError::ShapeError, "galois_attn_prefill: n_embd = n_head * head_dim");
    if (k_cache.dim().shape[0] != E || v_cache.dim().shape[0] != E || k_cache.dim().nrows() < (size_t)n_past + n ||
        v_cache.dim().nrows() < (size_t)n_past + n)
        return err(GError::ShapeError, "galois_attn_prefill: caches [n_embd, >= n_past + n]");
    float *out = nullptr;
    void *panel = nullptr;
    if (dst.dtype() == GGmlType::F32 && dst.dim().ggml_is_contiguous(dst.dtype()) && dst.dim().elem_count() == E * n)
        out = (float *)dst.data();
    else if (dst.dtype() == GGmlType::F16 && dst.dim().ggml_is_contiguous(dst.dtype()) && dst.dim().elem_count() >= galois_panel_elems(E, n))
        panel = dst.data();
    else
        return err(GError::ShapeError, "galois_attn_prefill: dst is F32 [n_embd, n] or an F16 panel of galois_panel_elems(n_embd, n)");
    const auto &dev = q.device().gpu;
    if (k_cache.dtype() == GGmlType::F16)
        return dev->check(galois_hip_attn_prefill_f16kv(dev->ctx(), (const float *)q.data(), k_cache.data(), v_cache.data(), out, panel,
                                                        (int32_t)n_head, (int32_t)(E / n_head), (int32_t)n, n_past, scale));
    return dev->check(galois_hip_attn_prefill_f32(dev->ctx(), (const float *)q.data(), (const float *)k_cache.data(),
                                                  (const float *)v_cache.data(), out, panel, (int32_t)n_head, (int32_t)(E / n_head),
                                                  (int32_t)n, n_past, scale));
}

static GResult mk(Tensor *t, GGmlType ty, const Device &dev, size_t ne0, size_t ne1 = 0, size_t ne2 = 0) {
    const size_t shape[3] = {ne0, ne1, ne2};
    return Tensor::zeros(ne2 ? 3 : (ne1 ? 2 : 1), shape, ty, dev, t);
}

GResult LlamaDecoder::prefill_buffers(size_t n, size_t keys) {
    const size_t E = hp_.n_embd, F = hp_.n_ff, H = hp_.n_head, D = E / H;
    const bool op_sequence = D != 128;              // the attention as single ops needs the scores and the permuted copies
    const bool single_ropes = D % 4 != 0 || D > 256;  // the rotations and the append as single ops need a rotated k
    if (n <= pf_.rows && (keys <= pf_.keys || !op_sequence)) return GError{};
    const size_t rows = n > pf_.rows ? n : pf_.rows, kk = keys > pf_.keys ? keys : pf_.keys;
    // The old buffers are released when b replaces them at the end; an earlier call may still be queued on them, so the
    // stream is drained first.
    Prefill b;
    G_TRY(dev_.gpu->check(galois_hip_synchronize(dev_.gpu->ctx())));
    const GGmlType F32 = GGmlType::F32;
    G_TRY(mk(&b.tok, GGmlType::I32, dev_, rows));
    G_TRY(mk(&b.pos, GGmlType::I32, dev_, rows));
    for (Tensor *t : {&b.x, &b.x1, &b.q, &b.k}) G_TRY(mk(t, F32, dev_, E, rows));
    if (hp_.kv_f16) G_TRY(mk(&b.v, F32, dev_, E, rows));  // an f32 cache takes the values straight from the product
    G_TRY(mk(&b.qr, F32, dev_, D, H, rows));
    if (single_ropes && hp_.kv_f16) G_TRY(mk(&b.kr, F32, dev_, D, H, rows));
    if (op_sequence) {
        G_TRY(mk(&b.ao, F32, dev_, E, rows));
        G_TRY(mk(&b.q3, F32, dev_, D, rows, H));
        G_TRY(mk(&b.o, F32, dev_, D, rows, H));
        G_TRY(mk(&b.s, F32, dev_, kk, rows, H));
        G_TRY(mk(&b.p, F32, dev_, kk, rows, H));
    }
    G_TRY(mk(&b.panel_e, GGmlType::F16, dev_, galois_panel_elems(E, rows)));
    G_TRY(mk(&b.panel_f, GGmlType::F16, dev_, galois_panel_elems(F, rows)));
    G_TRY(mk(&b.split_ws, F32, dev_, 2 * E * rows));
    b.rows = rows, b.keys = kk;
    pf_ = std::move(b);
    return GError{};
}

GResult LlamaDecoder::prefill(const int32_t *tokens, size_t n, int32_t n_past) {
    const size_t E = hp_.n_embd, F = hp_.n_ff, H = hp_.n_head, D = E / H, C = hp_.n_ctx;
    if (!tokens || n == 0) return err(GError::ShapeError, "prefill: at least one token");
    if (n_past < 0 || (size_t)n_past + n > C) return err(GError::ShapeError, "prefill: n_past + n must not exceed n_ctx");
    if (E % 256 != 0 || F % 256 != 0)
        return err(GError::Unimplemented, "prefill: the fp16 panels need n_embd and n_ff to be multiples of 256; decode token by token");
    if (hp_.kv_head_major) return err(GError::Unimplemented, "prefill: caches [n_embd, n_ctx] only");
    for (size_t i = 0; i < n; i++)
        if (tokens[i] < 0 || (size_t)tokens[i] >= hp_.n_vocab) return err(GError::ShapeError, "prefill: token id out of range");
    const size_t P = (size_t)n_past, L = P + n;
    G_TRY(prefill_buffers(n, L));
    Prefill &b = pf_;
    galois_hip_ctx *ctx = dev_.gpu->ctx();
    // views of the buffers at this call's n and L (the buffers may be larger)
    Tensor tok, pos, x, x1, q, k, v, ao, qr, kr, q3, o, s, p;
    {
        const size_t one[1] = {n}, en[2] = {E, n}, dhn[3] = {D, H, n}, dnh[3] = {D, n, H}, lnh[3] = {L, n, H};
        G_TRY(b.tok.view(0, 1, one, &tok));
        G_TRY(b.pos.view(0, 1, one, &pos));
        for (auto pr : {std::make_pair(&b.x, &x), std::make_pair(&b.x1, &x1), std::make_pair(&b.q, &q), std::make_pair(&b.k, &k)})
            G_TRY(pr.first->view(0, 2, en, pr.second));
        if (hp_.kv_f16) G_TRY(b.v.view(0, 2, en, &v));
        G_TRY(b.qr.view(0, 3, dhn, &qr));
        if (hp_.kv_f16 && (D % 4 != 0 || D > 256)) G_TRY(b.kr.view(0, 3, dhn, &kr));
        if (D != 128) {
            G_TRY(b.ao.view(0, 2, en, &ao));
            G_TRY(b.q3.view(0, 3, dnh, &q3));
            G_TRY(b.o.view(0, 3, dnh, &o));
            G_TRY(b.s.view(0, 3, lnh, &s));
            G_TRY(b.p.view(0, 3, lnh, &p));
        }
    }
    std::vector<int32_t> positions(n);
    for (size_t i = 0; i < n; i++) positions[i] = n_past + (int32_t)i;
    G_TRY(tok.write(tokens, n * sizeof(int32_t)));
    G_TRY(pos.write(positions.data(), n * sizeof(int32_t)));
    last_token_ = last_pos_ = -1;  // the pass ends in buffers of the decode step (x_, a_, logits_): the next decode sets its inputs anew

    RopeCustomOption rope;
    rope.n_dims = D, rope.mode = 0, rope.n_ctx = (int32_t)C, rope.freq_base = hp_.freq_base, rope.freq_scale = hp_.freq_scale;
    size_t ops = 0;
    const bool one_launch = D == 128;  // the attention of a layer as one launch (galois_attn_prefill)
    const float attn_scale = 1.0f / sqrtf((float)D);
    G_TRY(galois_get_rows(tok_embd_, tok, x)); ops++;
    // the first layer's attention norm; every later one rides on the pass that adds the down projection's shares
    G_TRY(galois_rms_norm_mul_panel(x, layers_[0].attn_norm, b.panel_e, hp_.rms_eps)); ops++;
    for (size_t li = 0; li < layers_.size(); li++) {
        Layer &l = layers_[li];
        // attention block: (norm -> panel, above or at the end of the layer before) q | k | v in one launch
        Tensor q_heads, k_heads;
        {
            const size_t dhn[3] = {D, H, n};
            G_TRY(q.view(0, 3, dhn, &q_heads));
            G_TRY(k.view(0, 3, dhn, &k_heads));
        }
        const size_t en[2] = {E, n};
        Tensor k_rows, v_rows;  // rows n_past .. n_past + n - 1 of both caches: one contiguous piece each
        G_TRY(l.k_cache.view(P * E, 2, en, &k_rows));
        G_TRY(l.v_cache.view(P * E, 2, en, &v_rows));
        if (D % 4 == 0 && D <= 256) {
            // both rotations and the append in one launch; an f32 cache takes the values straight from the product
            if (!hp_.kv_f16) {
                G_TRY(galois_matmul_panel({{&l.wq, &q}, {&l.wk, &k}, {&l.wv, &v_rows}}, b.panel_e, E, n));
                G_TRY(galois_rope_qk_append(rope, q_heads, k_heads, nullptr, pos, qr, k_rows, nullptr));
            } else {
                G_TRY(galois_matmul_panel({{&l.wq, &q}, {&l.wk, &k}, {&l.wv, &v}}, b.panel_e, E, n));
                G_TRY(galois_rope_qk_append(rope, q_heads, k_heads, &v, pos, qr, k_rows, &v_rows));
            }
            ops += 2;
        } else if (!hp_.kv_f16) {
            Tensor kr_cache;
            const size_t dhn[3] = {D, H, n};
            G_TRY(k_rows.view(0, 3, dhn, &kr_cache));
            G_TRY(galois_matmul_panel({{&l.wq, &q}, {&l.wk, &k}, {&l.wv, &v_rows}}, b.panel_e, E, n)); ops++;
            G_TRY(galois_rope_custom(rope, q_heads, pos, qr));
            G_TRY(galois_rope_custom(rope, k_heads, pos, kr_cache)); ops += 2;
        } else {
            G_TRY(galois_matmul_panel({{&l.wq, &q}, {&l.wk, &k}, {&l.wv, &v}}, b.panel_e, E, n)); ops++;
            G_TRY(galois_rope_custom(rope, q_heads, pos, qr));
            G_TRY(galois_rope_custom(rope, k_heads, pos, kr)); ops += 2;
            Tensor kr_flat;
            G_TRY(kr.view(0, 2, en, &kr_flat));
            G_TRY(galois_cpy(kr_flat, k_rows));
            G_TRY(galois_cpy(v, v_rows)); ops += 2;
        }
        if (one_launch) {
            Tensor qr_flat;
            G_TRY(qr.view(0, 2, en, &qr_flat));
            G_TRY(galois_attn_prefill(qr_flat, l.k_cache, l.v_cache, b.panel_e, H, n_past, attn_scale)); ops++;
        } else {
            // q as [D, n, H] (a head's queries contiguous), scores = K^T q per head over all L keys, causal soft_max
            {
                const size_t sh[3] = {D, n, H}, st[3] = {1, E, D};
                Tensor q_by_head;
                G_TRY(qr.view_strided(0, 3, sh, st, &q_by_head));
                G_TRY(galois_cpy(q_by_head, q3)); ops++;
            }
            Tensor kc, vc;
            const size_t ksh[3] = {D, L, H}, kst[3] = {1, E, D};
            G_TRY(l.k_cache.view_strided(0, 3, ksh, kst, &kc));
            G_TRY(galois_matmul(kc, q3, s));
            G_TRY(galois_scale(s, scale_, s)); ops += 2;
            // row m of head h keeps the keys 0 .. n_past + m (the index mask of galois_hip_soft_max_causal_f32)
            G_TRY(dev_.gpu->check(galois_hip_soft_max_causal_f32(ctx, (const float *)s.data(), (float *)p.data(), (int32_t)L,
                                                                 (int32_t)n, (int32_t)(n * H), n_past))); ops++;
            const size_t vsh[3] = {L, D, H}, vst[3] = {E, 1, D};
            G_TRY(l.v_cache.view_strided(0, 3, vsh, vst, &vc));
            G_TRY(galois_matmul(vc, p, o)); ops++;
            // back to [E, n] (token-major) and into the panel of the output projection
            {
                const size_t sh[3] = {D, H, n}, st[3] = {1, n * D, D};
                Tensor o_by_token, ao3;
                G_TRY(o.view_strided(0, 3, sh, st, &o_by_token));
                G_TRY(ao.view(0, 3, sh, &ao3));
                G_TRY(galois_cpy(o_by_token, ao3)); ops++;
            }
            G_TRY(galois_to_panel(ao, b.panel_e)); ops++;
        }
        // output projection as its shares of k (narrow for the device: two); the pass that adds them and the residual
        // stream also writes the feed-forward norm's panel
        int32_t shares = 0;
        G_TRY(galois_matmul_panel_shares(l.wo, b.panel_e, b.split_ws, E, n, &shares));
        G_TRY(galois_add_rms_norm_mul_panel(b.split_ws, shares, &x, x1, l.ffn_norm, b.panel_e, hp_.rms_eps)); ops += 2;
        // feed-forward block: gate | up with the SwiGLU in one launch -> panel, down as shares; the adding pass writes the next
        // layer's attention norm (after the last layer there is no next norm: the plain adding pass)
        G_TRY(galois_matmul_swiglu_panel(l.w_gate, l.w_up, b.panel_e, b.panel_f, E, n)); ops++;
        if (li + 1 < layers_.size()) {
            G_TRY(galois_matmul_panel_shares(l.w_down, b.panel_f, b.split_ws, F, n, &shares));
            G_TRY(galois_add_rms_norm_mul_panel(b.split_ws, shares, &x1, x, layers_[li + 1].attn_norm, b.panel_e, hp_.rms_eps)); ops += 2;
        } else {
            G_TRY(galois_matmul_panel_add(l.w_down, b.panel_f, &x1, x, F, n, &b.split_ws)); ops++;
        }
    }
    // the last token's logits, by the decode step's own tail
    {
        const size_t e1[2] = {E, 1};
        Tensor last;
        G_TRY(x.view((n - 1) * E, 2, e1, &last));
        G_TRY(galois_cpy(last, x_));
        G_TRY(galois_rms_norm_mul(x_, out_norm_, a_, hp_.rms_eps));
        G_TRY(galois_matmul(output_, a_, logits_)); ops += 3;
    }
    n_prefill_ops_ = ops;
    return GError{};
}

}  // namespace galois
