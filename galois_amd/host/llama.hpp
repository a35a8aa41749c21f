// One-token decode step of a LLaMA-architecture model written with the galois ops of galois.hpp.
//
// The reference ships no model graph (its consumer is external, example/src/main.rs:4); the op set it
// registers (src/kernels.rs:5-20) is the ggml-era LLaMA graph, and this driver issues exactly that
// sequence: get_rows, rms_norm, mul, matmul (Q4_0 and f32), rope_custom, cpy, scale, soft_max, unary
// (Silu) and add.  Linear weights are Q4_0, norms and the KV cache f32.  The step can be issued op by
// op or recorded once and replayed as a HIP graph.
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "galois.hpp"

namespace galois {

struct LlamaHParams {
    size_t n_vocab = 32000, n_embd = 4096, n_head = 32, n_layer = 32, n_ff = 11008, n_ctx = 2048;
    float rms_eps = 1e-6f, freq_base = 10000.0f, freq_scale = 1.0f;
    bool kv_f16 = false;  // KV cache in f16 (as the reference keeps it on the GPU); needs the fused attention (fused = 3)
    bool kv_head_major = false;  // caches kept [head_dim, n_ctx, n_head] instead of [n_embd, n_ctx]: a head's keys contiguous
};

class LlamaDecoder {
   public:
    // Allocates zeroed weights, the KV cache ([n_embd, n_ctx] f32 per layer, for K and for V) and every
    // intermediate of a step, so that decode() itself allocates nothing.
    static GResult create(const LlamaHParams &hp, const Device &dev, std::unique_ptr<LlamaDecoder> *out);
    ~LlamaDecoder();

    // Weights by name: "tok_embd" [n_embd, n_vocab] Q4_0, "out_norm" [n_embd] F32, "output" [n_embd, n_vocab] Q4_0
    // (layer = -1), and per layer "attn_norm", "ffn_norm" F32, "wq", "wk", "wv", "wo" [n_embd, n_embd],
    // "w_gate", "w_up" [n_embd, n_ff], "w_down" [n_ff, n_embd] Q4_0, "k_cache", "v_cache" [n_embd, n_ctx] F32 or F16
    // ([head_dim, n_ctx, n_head] with kv_head_major).
    Tensor *tensor(const std::string &name, int layer);

    // Enqueues one step for `token` at position n_past (attention over n_past + 1 keys); logits() holds the
    // result once the stream is synchronised (to_cpu_tensor does that).  fused = use the library's fused
    // rms_norm*weight and silu*up kernels instead of two ops each.
    // fused = 2 additionally sends the Q4_0 matrix-vector products out in grouped launches (q | k | v together,
    // gate | up as a SwiGLU pair) with the norms, silu * up and the residual adds riding along: 12 launches per layer;
    // fused = 3 also replaces the eight attention ops of a layer by galois_attn_decode: 5 launches per layer;
    // fused = 4 splits the norms that follow a residual add over the launch that produces the residual stream (it
    // also writes the stream times the next norm weight and its partial sums of squares) and the launch that consumes
    // it (it fetches one vector instead of two and waits for no reduction): the same 5 launches per layer.
    // fused = 5 sends the q | k | v products and the attention out as one launch (galois_qkv_attn_decode; heads of
    // 128): 4 launches per layer.
    // fused >= 3 are the plans that run with an f16 KV cache.
    GResult decode(int32_t token, int32_t n_past, int fused);
    // Records the same step as a graph / replays the recorded step.
    GResult capture(int32_t token, int32_t n_past, int fused);
    GResult replay();
    // Prefill: `n` tokens at positions n_past .. n_past + n - 1 in one pass (llama_prefill.cpp).  The same graph as n
    // decode steps, issued with the many-row ops: the Q4_0 products through the prefill matmul on fp16 panels that the
    // norms and the SwiGLU write directly (q | k | v and gate | up one launch each), rope_custom over all positions,
    // the n new rows of both caches appended at once, scores = K^T Q and out = V P per head on the matrix cores with
    // a causal soft_max between them (heads of 128: galois_attn_prefill instead, one launch that writes the panel of
    // the output projection; f32 caches receive the rotated keys and the values directly); the output and down
    // projections add the residual stream where they store (galois_matmul_panel_add).  Afterwards the caches hold positions 0 .. n_past + n - 1 and logits() the last
    // token's.  n_embd and n_ff must be multiples of 256; caches [n_embd, n_ctx] (not head-major), f32 or f16.
    // Intermediates are sized for the largest n and n_past + n seen so far (this call allocates when they grow).
    GResult prefill(const int32_t *tokens, size_t n, int32_t n_past);
    size_t ops_per_prefill() const { return n_prefill_ops_; }  // library calls of the last prefill (a call is one or two launches)
    const Tensor &logits() const { return logits_; }
    const LlamaHParams &hparams() const { return hp_; }
    size_t ops_per_step() const { return n_ops_; }

   private:
    struct Layer {
        Tensor attn_norm, ffn_norm, wq, wk, wv, wo, w_gate, w_up, w_down, k_cache, v_cache;
    };
    GResult set_inputs(int32_t token, int32_t n_past);
    GResult step(int32_t n_past, int fused);

    LlamaHParams hp_;
    Device dev_;
    Tensor tok_embd_, out_norm_, output_;
    std::vector<Layer> layers_;
    Tensor tok_id_, pos_, scale_;                                    // I32 [1], I32 [1], host f32 [1]
    Tensor x_, t_, a_, q_, k_, v_, qr_, kr_, s_, p_, o_, ao_, x1_, f_, g_, u_, h_, d_, logits_;
    Tensor ssq_, ssq1_;  // partial sums of squares of x and x1 (fused = 4)
    struct Prefill {  // intermediates of prefill(), for up to `rows` tokens attending over up to `keys` positions
        size_t rows = 0, keys = 0;
        Tensor tok, pos, x, x1, q, k, v, qr, kr, q3, s, p, o, ao, panel_e, panel_f, split_ws;
    };
    GResult prefill_buffers(size_t n, size_t keys);
    Prefill pf_;
    galois_hip_graph *graph_ = nullptr;
    size_t n_ops_ = 0, n_prefill_ops_ = 0;
    int32_t last_token_ = -1, last_pos_ = -1;
};

// Extensions used by the fused mode (no counterpart in the reference's op list): rms_norm followed by the
// weight multiply, and silu(gate) * up, each as one kernel.
GResult galois_rms_norm_mul(const Tensor &src, const Tensor &weight, Tensor &dst, float eps);
GResult galois_silu_mul(const Tensor &gate, const Tensor &up, Tensor &dst);

// Several Q4_0 matrix-vector products in one launch (galois_hip_dequantize_mul_mat_vec_q4_0_group): per product
// dst = w . x, where x is first replaced by rms_norm(x, eps) * norm_weight when norm_weight is set, the result
// becomes silu(w . x) * (w_up . x) when w_up is set, and residual is added when set (it may be dst).
// A norm can be split over two calls: the call that produces a vector also writes dst_scaled = dst * scale_weight and
// sumsq_out (the sums of squares of dst per 16 elements); the call that consumes it passes x = that dst_scaled,
// sumsq_in = that sumsq_out and eps, and gets w . (rms_norm(dst, eps) * scale_weight) up to rounding.
struct MatvecItem {
    const Tensor *w = nullptr, *w_up = nullptr, *x = nullptr, *norm_weight = nullptr, *residual = nullptr;
    Tensor *dst = nullptr;
    float eps = 0.0f;
    Tensor *dst_scaled = nullptr, *sumsq_out = nullptr;
    const Tensor *scale_weight = nullptr, *sumsq_in = nullptr;
};
GResult galois_matvec_group(const std::vector<MatvecItem> &items);

// The prefill matmul's fp16 panel (galois_hip_*_f16_panel): `panel` is an F16 tensor of galois_panel_elems(K, M)
// elements.  The producers write rms_norm(src, eps) * weight, silu(gate) * up, or src itself, for src = [K, M] f32;
// galois_matmul_panel multiplies one to four Q4_0 matrices [K, N_j] by it in one launch, dst_j = [N_j, M] f32.
size_t galois_panel_elems(size_t K, size_t M);
GResult galois_rms_norm_mul_panel(const Tensor &src, const Tensor &weight, Tensor &panel, float eps);
GResult galois_silu_mul_panel(const Tensor &gate, const Tensor &up, Tensor &panel);
GResult galois_to_panel(const Tensor &src, Tensor &panel);
struct PanelMatmulItem {
    const Tensor *w = nullptr;
    Tensor *dst = nullptr;
};
GResult galois_matmul_panel(const std::vector<PanelMatmulItem> &items, const Tensor &panel, size_t K, size_t M);
// dst = residual + w . panel (galois_hip_mul_mat_q4_0_f16_panel_add); residual may be null or dst.  workspace: an F32
// tensor the call may overwrite (2 * N * M elements let a narrow matrix run as two shares of k), or null.
GResult galois_matmul_panel_add(const Tensor &w, const Tensor &panel, const Tensor *residual, Tensor &dst, size_t K, size_t M,
                                Tensor *workspace);

// Attention of one decode step in one launch (galois_hip_attn_decode_f32): rope_custom of q and k at position
// pos[0] = n_past, append of k and v to row n_past of the caches ([n_embd, n_ctx], both f32 or both f16), scores = K^T q scaled
// by `scale`, soft_max over the n_past + 1 keys and out = V p, for n_head heads of q.dim / n_head elements.
GResult galois_attn_decode(const RopeCustomOption &op, const Tensor &q, const Tensor &k, const Tensor &v, Tensor &k_cache,
                           Tensor &v_cache, const Tensor &pos, Tensor &out, size_t n_head, int32_t n_past, float scale);

// panel_out = the panel of silu(w_gate . x) * (w_up . x) for x given as `panel` ([K, M] operand), one launch
// (galois_hip_mul_mat_q4_0_swiglu_f16_panel); w_gate, w_up [K, N] Q4_0, panel_out of galois_panel_elems(N, M) elements.
GResult galois_matmul_swiglu_panel(const Tensor &w_gate, const Tensor &w_up, const Tensor &panel, Tensor &panel_out, size_t K, size_t M);
// The product alone as its one or two shares of k (galois_hip_mul_mat_q4_0_f16_panel_shares): shares is an F32 tensor of
// at least N * M elements (2 * N * M let a narrow matrix run as two shares); *n_shares says how many partial results
// it now holds, N * M elements apart.
GResult galois_matmul_panel_shares(const Tensor &w, const Tensor &panel, Tensor &shares, size_t K, size_t M, int32_t *n_shares);
// sum_out = the n_shares partial results in `shares` + residual (may be null), and rms_norm(sum_out, eps) * weight into
// the panel, in one launch (galois_hip_add_rms_norm_mul_f16_panel).  sum_out: F32 [ncols, nrows]; it may be residual.
GResult galois_add_rms_norm_mul_panel(const Tensor &shares, int32_t n_shares, const Tensor *residual, Tensor &sum_out,
                                      const Tensor &weight, Tensor &panel, float eps);

// rope_custom (mode 0, n_dims = head_dim) of q and k ([head_dim, n_head, n] f32, positions pos) and the append to the
// caches' rows of those tokens, one launch (galois_hip_rope_qk_append): q rotated to q_out; k rotated to k_rows and, when
// v is given, v to v_rows -- contiguous views of the caches' rows, [n_embd, n], both F32 or both F16.
GResult galois_rope_qk_append(const RopeCustomOption &op, const Tensor &q, const Tensor &k, const Tensor *v, const Tensor &pos,
                              Tensor &q_out, Tensor &k_rows, Tensor *v_rows);

// Causal attention of all rows of q ([n_embd, n] f32, rotated) over caches ([n_embd, n_ctx], both f32 or both f16) that
// already hold positions 0 .. n_past + n - 1, in one launch (galois_hip_attn_prefill_f32 / _f16kv; heads of 128).
// dst is either an F32 tensor [n_embd, n] or an F16 panel of galois_panel_elems(n_embd, n) elements.
GResult galois_attn_prefill(const Tensor &q, const Tensor &k_cache, const Tensor &v_cache, Tensor &dst, size_t n_head,
                            int32_t n_past, float scale);

// The three products q | k | v (as galois_matvec_group takes them; plain or normalising) and the attention that
// consumes them (galois_attn_decode on their dst tensors) in one launch (galois_hip_qkv_attn_decode_f32 / _f16kv).
GResult galois_qkv_attn_decode(const RopeCustomOption &op, const std::vector<MatvecItem> &qkv, Tensor &k_cache, Tensor &v_cache,
                               const Tensor &pos, Tensor &out, size_t n_head, int32_t n_past, float scale);

}  // namespace galois
