// Reader for GGUF model files (versions 2 and 3), the container the ggml ecosystem stores Q4_0 models in,
// feeding Tensor::from_raw (src/lib.rs:2477-2523) and the LLaMA decode driver of llama.hpp.
//
// The reference has no file loader: its consumer hands raw tensor bytes to Tensor::from_raw.  This is
// the piece that sits in front of that call, so that a real model file replaces random weights.  The file
// is memory-mapped; nothing is copied until a tensor is sent to a device.  A malformed or truncated file
// yields a GError, never a crash: every length read from the file is checked against the mapping.
//
// Layout read here (little-endian): "GGUF", u32 version, u64 tensor_count, u64 kv_count; kv_count times
// { string key, u32 value_type, value }; tensor_count times { string name, u32 n_dims, u64 ne[n_dims]
// (ne[0] innermost, as in ggml), u32 ggml_type, u64 offset }; padding to `general.alignment` (default 32);
// tensor data, each tensor at data_start + offset.  A string is u64 length + bytes (no terminator).
#pragma once
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "galois.hpp"
#include "llama.hpp"

namespace galois {

enum class GgufType : uint32_t {
    U8 = 0, I8 = 1, U16 = 2, I16 = 3, U32 = 4, I32 = 5, F32 = 6, Bool = 7, String = 8, Array = 9, U64 = 10, I64 = 11, F64 = 12
};

struct GgufValue {
    GgufType type = GgufType::U8;
    uint64_t u = 0;   // unsigned integers and Bool
    int64_t i = 0;    // signed integers
    double f = 0.0;   // F32, F64
    std::string s;    // String
    // Array: element type, count, and where the elements lie in the mapping (not decoded until asked for)
    GgufType elem_type = GgufType::U8;
    uint64_t count = 0;
    const uint8_t *elems = nullptr;
    size_t elems_bytes = 0;
};

struct GgufTensorInfo {
    std::string name;
    size_t n_dims = 0;
    size_t shape[4] = {1, 1, 1, 1};  // ne0 (innermost) first
    uint32_t ggml_type = 0;          // type id as stored in the file
    bool supported = false;          // F32, F16 or Q4_0: the types this backend computes with
    GGmlType dtype = GGmlType::F32;  // valid when supported
    uint64_t offset = 0;             // from the start of the data section
    size_t nbytes = 0;               // 0 when the file's type id is not in the size table
};

class GgufFile {
   public:
    static GResult open(const std::string &path, std::unique_ptr<GgufFile> *out);
    ~GgufFile();
    GgufFile(const GgufFile &) = delete;
    GgufFile &operator=(const GgufFile &) = delete;

    uint32_t version() const { return version_; }
    size_t alignment() const { return alignment_; }
    size_t data_start() const { return data_start_; }
    const std::map<std::string, GgufValue> &metadata() const { return kv_; }
    const std::vector<GgufTensorInfo> &tensors() const { return tensors_; }

    const GgufValue *find(const std::string &key) const;
    // Integer / float / string metadata; false when the key is absent or of another kind.
    bool get_uint(const std::string &key, uint64_t *out) const;
    bool get_float(const std::string &key, double *out) const;
    bool get_string(const std::string &key, std::string *out) const;
    // Elements of a string array (a tokenizer's token list)
    GResult get_string_array(const std::string &key, std::vector<std::string> *out) const;

    const GgufTensorInfo *tensor(const std::string &name) const;
    // Bytes of a tensor inside the mapping
    const uint8_t *tensor_data(const GgufTensorInfo &t) const { return base_ + data_start_ + t.offset; }
    // Tensor::from_raw on the tensor's bytes
    GResult load_tensor(const std::string &name, const Device &dev, Tensor *out) const;

   private:
    GgufFile() = default;
    GResult parse();

    const uint8_t *base_ = nullptr;
    size_t size_ = 0;
    int fd_ = -1;
    uint32_t version_ = 0;
    size_t alignment_ = 32, data_start_ = 0;
    std::map<std::string, GgufValue> kv_;
    std::vector<GgufTensorInfo> tensors_;
    std::map<std::string, size_t> by_name_;
};

// Hyper-parameters of a `general.architecture = "llama"` file (llama.block_count, llama.embedding_length,
// llama.feed_forward_length, llama.attention.head_count, llama.attention.layer_norm_rms_epsilon,
// llama.rope.freq_base, llama.context_length; n_vocab from token_embd.weight).  n_ctx = min(n_ctx_max, the
// file's context length).  Models this driver cannot run (grouped-query attention, partial rotary dimensions)
// are refused.
GResult llama_hparams_from_gguf(const GgufFile &f, size_t n_ctx_max, LlamaHParams *hp);

// Creates a decoder for the file's hyper-parameters and fills its weights from the file: token_embd.weight,
// output_norm.weight, output.weight (token_embd.weight again when the file ties them), and per layer
// blk.N.{attn_norm, attn_q, attn_k, attn_v, attn_output, ffn_norm, ffn_gate, ffn_up, ffn_down}.weight.
// Linear weights must be Q4_0 and norms F32, with exactly the shapes the decoder allocates.
GResult llama_from_gguf(const GgufFile &f, const Device &dev, size_t n_ctx_max, std::unique_ptr<LlamaDecoder> *out);

}  // namespace galois
