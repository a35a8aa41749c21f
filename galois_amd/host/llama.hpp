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
    galois_hip_graph *graph_ = nullptr;
    size_t n_ops_ = 0;
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

// Attention of one decode step in one launch (galois_hip_attn_decode_f32): rope_custom of q and k at position
// pos[0] = n_past, append of k and v to row n_past of the caches ([n_embd, n_ctx], both f32 or both f16), scores = K^T q scaled
// by `scale`, soft_max over the n_past + 1 keys and out = V p, for n_head heads of q.dim / n_head elements.
GResult galois_attn_decode(const RopeCustomOption &op, const Tensor &q, const Tensor &k, const Tensor &v, Tensor &k_cache,
                           Tensor &v_cache, const Tensor &pos, Tensor &out, size_t n_head, int32_t n_past, float scale);

// The three products q | k | v (as galois_matvec_group takes them; plain or normalising) and the attention that
// consumes them (galois_attn_decode on their dst tensors) in one launch (galois_hip_qkv_attn_decode_f32 / _f16kv).
GResult galois_qkv_attn_decode(const RopeCustomOption &op, const std::vector<MatvecItem> &qkv, Tensor &k_cache, Tensor &v_cache,
                               const Tensor &pos, Tensor &out, size_t n_head, int32_t n_past, float scale);

}  // namespace galois
