// GGUF reader: see gguf.hpp.  Every length taken from the file is checked against the mapping before use.
#include "gguf.hpp"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cmath>
#include <cstring>

namespace galois {
namespace {

GError err(GError::Kind k, const std::string &m) { return GError{k, m}; }

struct Cursor {
    const uint8_t *p;
    size_t size, pos = 0;
    size_t left() const { return size - pos; }
    template <class T>
    bool read(T *v) {
        if (left() < sizeof(T)) return false;
        memcpy(v, p + pos, sizeof(T));
        pos += sizeof(T);
        return true;
    }
    bool read_string(std::string *s) {
        uint64_t n;
        if (!read(&n) || n > left()) return false;
        s->assign(reinterpret_cast<const char *>(p + pos), (size_t)n);
        pos += (size_t)n;
        return true;
    }
    bool skip_string() {
        uint64_t n;
        if (!read(&n) || n > left()) return false;
        pos += (size_t)n;
        return true;
    }
};

// bytes of a fixed-size metadata value; 0 for String and Array
size_t scalar_size(GgufType t) {
    switch (t) {
        case GgufType::U8: case GgufType::I8: case GgufType::Bool: return 1;
        case GgufType::U16: case GgufType::I16: return 2;
        case GgufType::U32: case GgufType::I32: case GgufType::F32: return 4;
        case GgufType::U64: case GgufType::I64: case GgufType::F64: return 8;
        default: return 0;
    }
}

bool read_scalar(Cursor &c, GgufType t, GgufValue *v) {
    switch (t) {
        case GgufType::U8: { uint8_t x; if (!c.read(&x)) return false; v->u = x; return true; }
        case GgufType::Bool: { uint8_t x; if (!c.read(&x)) return false; v->u = x != 0; return true; }
        case GgufType::I8: { int8_t x; if (!c.read(&x)) return false; v->i = x; return true; }
        case GgufType::U16: { uint16_t x; if (!c.read(&x)) return false; v->u = x; return true; }
        case GgufType::I16: { int16_t x; if (!c.read(&x)) return false; v->i = x; return true; }
        case GgufType::U32: { uint32_t x; if (!c.read(&x)) return false; v->u = x; return true; }
        case GgufType::I32: { int32_t x; if (!c.read(&x)) return false; v->i = x; return true; }
        case GgufType::U64: { uint64_t x; if (!c.read(&x)) return false; v->u = x; return true; }
        case GgufType::I64: { int64_t x; if (!c.read(&x)) return false; v->i = x; return true; }
        case GgufType::F32: { float x; if (!c.read(&x)) return false; v->f = x; return true; }
        case GgufType::F64: { double x; if (!c.read(&x)) return false; v->f = x; return true; }
        default: return false;
    }
}

// (bytes per block, elements per block) of the ggml tensor types whose size is fixed by the format
bool ggml_type_sizes(uint32_t id, size_t *type_size, size_t *blck) {
    struct Row { uint32_t id; size_t ts, bs; };
    static const Row rows[] = {{0, 4, 1},     {1, 2, 1},     {2, 18, 32},   {3, 20, 32},   {6, 22, 32},   {7, 24, 32},
                               {8, 34, 32},   {9, 36, 32},   {10, 84, 256}, {11, 110, 256}, {12, 144, 256}, {13, 176, 256},
                               {14, 210, 256}, {15, 292, 256}, {24, 1, 1},   {25, 2, 1},    {26, 4, 1},    {27, 8, 1},
                               {28, 8, 1},    {30, 2, 1}};
    for (const Row &r : rows)
        if (r.id == id) {
            *type_size = r.ts, *blck = r.bs;
            return true;
        }
    return false;
}

}  // namespace

GgufFile::~GgufFile() {
    if (base_) munmap(const_cast<uint8_t *>(base_), size_);
    if (fd_ >= 0) close(fd_);
}

GResult GgufFile::open(const std::string &path, std::unique_ptr<GgufFile> *out) {
    std::unique_ptr<GgufFile> f(new GgufFile());
    f->fd_ = ::open(path.c_str(), O_RDONLY);
    if (f->fd_ < 0) return err(GError::Unexpected, "gguf: cannot open " + path);
    struct stat st;
    if (fstat(f->fd_, &st) != 0 || st.st_size < 24) return err(GError::ShapeError, "gguf: " + path + " is shorter than a header");
    f->size_ = (size_t)st.st_size;
    void *m = mmap(nullptr, f->size_, PROT_READ, MAP_PRIVATE, f->fd_, 0);
    if (m == MAP_FAILED) return err(GError::Unexpected, "gguf: mmap of " + path + " failed");
    f->base_ = static_cast<const uint8_t *>(m);
    GResult r = f->parse();
    if (!r.ok()) return r;
    *out = std::move(f);
    return GResult{};
}

GResult GgufFile::parse() {
    Cursor c{base_, size_};
    uint32_t magic;
    uint64_t n_tensors, n_kv;
    if (!c.read(&magic) || magic != 0x46554747u) return err(GError::ShapeError, "gguf: bad magic");
    if (!c.read(&version_)) return err(GError::ShapeError, "gguf: truncated header");
    if (version_ != 2 && version_ != 3)
        return err(GError::Unimplemented, "gguf: version " + std::to_string(version_) + " (2 and 3 are read)");
    if (!c.read(&n_tensors) || !c.read(&n_kv)) return err(GError::ShapeError, "gguf: truncated header");
    // a key-value pair takes at least 13 bytes and a tensor record 24: larger counts cannot be honest
    if (n_kv > size_ / 13 || n_tensors > size_ / 24) return err(GError::ShapeError, "gguf: counts exceed the file size");

    for (uint64_t k = 0; k < n_kv; k++) {
        std::string key;
        uint32_t t;
        if (!c.read_string(&key) || !c.read(&t)) return err(GError::ShapeError, "gguf: truncated metadata");
        if (t > (uint32_t)GgufType::F64) return err(GError::ShapeError, "gguf: unknown value type of key " + key);
        GgufValue v;
        v.type = (GgufType)t;
        if (v.type == GgufType::String) {
            if (!c.read_string(&v.s)) return err(GError::ShapeError, "gguf: truncated string value of key " + key);
        } else if (v.type == GgufType::Array) {
            uint32_t et;
            if (!c.read(&et) || !c.read(&v.count)) return err(GError::ShapeError, "gguf: truncated array header of key " + key);
            if (et > (uint32_t)GgufType::F64 || et == (uint32_t)GgufType::Array)
                return err(GError::Unimplemented, "gguf: array element type of key " + key);
            v.elem_type = (GgufType)et;
            const size_t start = c.pos;
            if (v.elem_type == GgufType::String) {
                if (v.count > c.left() / 8) return err(GError::ShapeError, "gguf: array count of key " + key + " exceeds the file");
                for (uint64_t i = 0; i < v.count; i++)
                    if (!c.skip_string()) return err(GError::ShapeError, "gguf: truncated string array of key " + key);
            } else {
                const size_t es = scalar_size(v.elem_type);
                if (v.count > c.left() / es) return err(GError::ShapeError, "gguf: array count of key " + key + " exceeds the file");
                c.pos += (size_t)v.count * es;
            }
            v.elems = base_ + start, v.elems_bytes = c.pos - start;
        } else if (!read_scalar(c, v.type, &v)) {
            return err(GError::ShapeError, "gguf: truncated value of key " + key);
        }
        kv_[key] = std::move(v);
    }

    uint64_t al;
    if (get_uint("general.alignment", &al)) {
        if (al == 0 || al > (1u << 20) || (al & (al - 1)) != 0)
            return err(GError::ShapeError, "gguf: general.alignment must be a power of two up to 1 MiB");
        alignment_ = (size_t)al;
    }

    tensors_.reserve((size_t)n_tensors);
    for (uint64_t i = 0; i < n_tensors; i++) {
        GgufTensorInfo t;
        uint32_t nd;
        if (!c.read_string(&t.name) || !c.read(&nd)) return err(GError::ShapeError, "gguf: truncated tensor record");
        if (nd < 1 || nd > 4) return err(GError::ShapeError, "gguf: tensor " + t.name + " has " + std::to_string(nd) + " dimensions");
        t.n_dims = nd;
        uint64_t elems = 1;
        for (uint32_t d = 0; d < nd; d++) {
            uint64_t ne;
            if (!c.read(&ne)) return err(GError::ShapeError, "gguf: truncated tensor record");
            if (ne == 0 || ne > ((uint64_t)1 << 40) || elems > ((uint64_t)1 << 48) / ne)
                return err(GError::ShapeError, "gguf: tensor " + t.name + " has an impossible shape");
            elems *= ne;
            t.shape[d] = (size_t)ne;
        }
        if (!c.read(&t.ggml_type) || !c.read(&t.offset)) return err(GError::ShapeError, "gguf: truncated tensor record");
        size_t ts, bs;
        if (ggml_type_sizes(t.ggml_type, &ts, &bs)) {
            if (t.shape[0] % bs != 0)
                return err(GError::ShapeError, "gguf: row length of tensor " + t.name + " is not a multiple of its block size");
            t.nbytes = (size_t)(elems / bs) * ts;
        }
        if (t.ggml_type <= 2) t.supported = true, t.dtype = (GGmlType)t.ggml_type;
        if (by_name_.count(t.name)) return err(GError::ShapeError, "gguf: tensor name " + t.name + " appears twice");
        by_name_[t.name] = tensors_.size();
        tensors_.push_back(std::move(t));
    }

    data_start_ = (c.pos + alignment_ - 1) / alignment_ * alignment_;
    if (n_tensors > 0 && data_start_ > size_) return err(GError::ShapeError, "gguf: no data section");
    for (const GgufTensorInfo &t : tensors_) {
        if (t.offset % alignment_ != 0) return err(GError::ShapeError, "gguf: tensor " + t.name + " is not aligned");
        if (t.offset > size_ - data_start_ || t.nbytes > size_ - data_start_ - t.offset)
            return err(GError::ShapeError, "gguf: tensor " + t.name + " reaches past the end of the file");
    }
    return GResult{};
}

const GgufValue *GgufFile::find(const std::string &key) const {
    auto it = kv_.find(key);
    return it == kv_.end() ? nullptr : &it->second;
}

bool GgufFile::get_uint(const std::string &key, uint64_t *out) const {
    const GgufValue *v = find(key);
    if (!v) return false;
    switch (v->type) {
        case GgufType::U8: case GgufType::U16: case GgufType::U32: case GgufType::U64: case GgufType::Bool:
            *out = v->u;
            return true;
        case GgufType::I8: case GgufType::I16: case GgufType::I32: case GgufType::I64:
            if (v->i < 0) return false;
            *out = (uint64_t)v->i;
            return true;
        default: return false;
    }
}

bool GgufFile::get_float(const std::string &key, double *out) const {
    const GgufValue *v = find(key);
    if (!v || (v->type != GgufType::F32 && v->type != GgufType::F64)) return false;
    *out = v->f;
    return true;
}

bool GgufFile::get_string(const std::string &key, std::string *out) const {
    const GgufValue *v = find(key);
    if (!v || v->type != GgufType::String) return false;
    *out = v->s;
    return true;
}

GResult GgufFile::get_string_array(const std::string &key, std::vector<std::string> *out) const {
    const GgufValue *v = find(key);
    if (!v || v->type != GgufType::Array || v->elem_type != GgufType::String)
        return err(GError::Unexpected, "gguf: " + key + " is not a string array");
    Cursor c{v->elems, v->elems_bytes};
    out->clear();
    out->reserve((size_t)v->count);
    for (uint64_t i = 0; i < v->count; i++) {
        std::string s;
        if (!c.read_string(&s)) return err(GError::ShapeError, "gguf: truncated string array " + key);
        out->push_back(std::move(s));
    }
    return GResult{};
}

const GgufTensorInfo *GgufFile::tensor(const std::string &name) const {
    auto it = by_name_.find(name);
    return it == by_name_.end() ? nullptr : &tensors_[it->second];
}

GResult GgufFile::load_tensor(const std::string &name, const Device &dev, Tensor *out) const {
    const GgufTensorInfo *t = tensor(name);
    if (!t) return err(GError::Unexpected, "gguf: no tensor named " + name);
    if (!t->supported)
        return err(GError::Unimplemented, "gguf: tensor " + name + " has ggml type " + std::to_string(t->ggml_type) +
                                              " (F32, F16 and Q4_0 are loaded)");
    return Tensor::from_raw(tensor_data(*t), t->nbytes, t->n_dims, t->shape, t->dtype, dev, out);
}

GResult llama_hparams_from_gguf(const GgufFile &f, size_t n_ctx_max, LlamaHParams *hp) {
    std::string arch;
    if (!f.get_string("general.architecture", &arch)) return err(GError::ShapeError, "gguf: general.architecture is missing");
    if (arch != "llama") return err(GError::Unimplemented, "gguf: architecture " + arch + " (this driver runs llama)");
    uint64_t n_layer, n_embd, n_ff, n_head, v;
    if (!f.get_uint("llama.block_count", &n_layer) || !f.get_uint("llama.embedding_length", &n_embd) ||
        !f.get_uint("llama.feed_forward_length", &n_ff) || !f.get_uint("llama.attention.head_count", &n_head))
        return err(GError::ShapeError, "gguf: llama.block_count / embedding_length / feed_forward_length / attention.head_count missing");
    if (n_layer == 0 || n_embd == 0 || n_ff == 0 || n_head == 0 || n_embd % n_head != 0)
        return err(GError::ShapeError, "gguf: impossible llama hyper-parameters");
    if (f.get_uint("llama.attention.head_count_kv", &v) && v != n_head)
        return err(GError::Unimplemented, "gguf: grouped-query attention (head_count_kv != head_count)");
    if (f.get_uint("llama.rope.dimension_count", &v) && v != n_embd / n_head)
        return err(GError::Unimplemented, "gguf: rotary dimensions other than the head size");
    const GgufTensorInfo *emb = f.tensor("token_embd.weight");
    if (!emb || emb->n_dims != 2 || emb->shape[0] != n_embd)
        return err(GError::ShapeError, "gguf: token_embd.weight is missing or not [embedding_length, n_vocab]");
    LlamaHParams h;
    h.n_vocab = emb->shape[1], h.n_embd = (size_t)n_embd, h.n_head = (size_t)n_head, h.n_layer = (size_t)n_layer;
    h.n_ff = (size_t)n_ff;
    uint64_t n_ctx_file = 0;
    const bool has_ctx = f.get_uint("llama.context_length", &n_ctx_file) && n_ctx_file > 0;
    h.n_ctx = has_ctx && n_ctx_file < n_ctx_max ? (size_t)n_ctx_file : n_ctx_max;
    if (h.n_ctx == 0) return err(GError::ShapeError, "gguf: context length 0");
    double d;
    h.rms_eps = f.get_float("llama.attention.layer_norm_rms_epsilon", &d) ? (float)d : 1e-5f;
    h.freq_base = f.get_float("llama.rope.freq_base", &d) ? (float)d : 10000.0f;
    h.freq_scale = 1.0f;
    std::string scaling;
    if (f.get_string("llama.rope.scaling.type", &scaling) && scaling != "none") {
        if (scaling != "linear") return err(GError::Unimplemented, "gguf: rope scaling type " + scaling);
        if (f.get_float("llama.rope.scaling.factor", &d) && d > 0.0) h.freq_scale = (float)(1.0 / d);
    } else if (f.get_float("llama.rope.scale_linear", &d) && d > 0.0) {
        h.freq_scale = (float)(1.0 / d);
    }
    if (!std::isfinite(h.rms_eps) || !std::isfinite(h.freq_base) || h.freq_base <= 0.0f)
        return err(GError::ShapeError, "gguf: rms epsilon or rope base is not a usable number");
    *hp = h;
    return GResult{};
}

namespace {

GResult fill(const GgufFile &f, const std::string &file_name, Tensor *dst, const char *what) {
    const GgufTensorInfo *t = f.tensor(file_name);
    if (!t) return err(GError::ShapeError, "gguf: tensor " + file_name + " is missing");
    if (!dst) return err(GError::Unexpected, std::string("llama decoder has no tensor ") + what);
    if (!t->supported || t->dtype != dst->dtype())
        return err(GError::Unimplemented, "gguf: tensor " + file_name + " has ggml type " + std::to_string(t->ggml_type) +
                                              ", the decoder holds " + what + " as type " + std::to_string((int)dst->dtype()));
    bool same = t->nbytes == dst->nbytes();
    for (int d = 0; d < 4; d++) same = same && t->shape[d] == dst->dim().shape[d];
    if (!same) return err(GError::ShapeError, "gguf: tensor " + file_name + " does not have the shape of " + what);
    return dst->write(f.tensor_data(*t), t->nbytes);
}

}  // namespace

GResult llama_from_gguf(const GgufFile &f, const Device &dev, size_t n_ctx_max, std::unique_ptr<LlamaDecoder> *out) {
    LlamaHParams hp;
    GResult r = llama_hparams_from_gguf(f, n_ctx_max, &hp);
    if (!r.ok()) return r;
    std::unique_ptr<LlamaDecoder> m;
    r = LlamaDecoder::create(hp, dev, &m);
    if (!r.ok()) return r;
    r = fill(f, "token_embd.weight", m->tensor("tok_embd", -1), "tok_embd");
    if (!r.ok()) return r;
    r = fill(f, "output_norm.weight", m->tensor("out_norm", -1), "out_norm");
    if (!r.ok()) return r;
    r = fill(f, f.tensor("output.weight") ? "output.weight" : "token_embd.weight", m->tensor("output", -1), "output");
    if (!r.ok()) return r;
    static const char *const pairs[][2] = {{"attn_norm", "attn_norm"}, {"attn_q", "wq"},       {"attn_k", "wk"},
                                           {"attn_v", "wv"},           {"attn_output", "wo"},  {"ffn_norm", "ffn_norm"},
                                           {"ffn_gate", "w_gate"},     {"ffn_up", "w_up"},     {"ffn_down", "w_down"}};
    for (size_t l = 0; l < hp.n_layer; l++)
        for (const auto &p : pairs) {
            r = fill(f, "blk." + std::to_string(l) + "." + p[0] + ".weight", m->tensor(p[1], (int)l), p[1]);
            if (!r.ok()) return r;
        }
    *out = std::move(m);
    return GResult{};
}

}  // namespace galois
