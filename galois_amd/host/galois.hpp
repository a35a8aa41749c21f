// C++ host mirror of galois's tensor / op interface for the Q4_0 hot path, written above the C ABI
// of include/galois_hip.h exactly as a rewritten src/cuda.rs would sit above it.
//
// Same names and argument meaning as the reference: Tensor::from_raw (src/lib.rs:2477-2491),
// Tensor::to_cpu_tensor (src/lib.rs:2279-2341), GGmlType numbering (src/lib.rs:278-300), ggml
// shapes [ne0 innermost .. ne3] with strides in storage elements (src/shape.rs:422-430), and the op
// entry points galois_matmul / galois_rms_norm / galois_rope_custom / galois_soft_max
// (src/op.rs:3093-3341).  Where the reference panics (todo!(), assert!) this layer returns a GError.
#pragma once
#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "../../include/galois_hip.h"

namespace galois {

enum class GGmlType : int { F32 = 0, F16 = 1, Q4_0 = 2, I32 = 18 };  // src/lib.rs:278-300

// GS_TYPE_SIZE / GS_BLCK_SIZE, src/lib.rs:358-400
size_t type_size(GGmlType t);
size_t blck_size(GGmlType t);

struct GError {
    enum Kind { Ok = 0, Unimplemented, ShapeError, DeviceError, Unexpected } kind = Ok;
    std::string msg;
    bool ok() const { return kind == Ok; }
};
using GResult = GError;  // GResult<()> of src/error.rs:14

// Dim { n_dims, shape, stride }, src/shape.rs
struct Dim {
    size_t n_dims = 0;
    size_t shape[4] = {1, 1, 1, 1};
    size_t stride[4] = {1, 1, 1, 1};  // in storage elements (blocks for quantized types)
    static Dim contiguous(size_t n_dims, const size_t *shape, GGmlType t);  // Shape::ggml_stride
    size_t nrows() const { return shape[1] * shape[2] * shape[3]; }
    size_t elem_count() const { return shape[0] * shape[1] * shape[2] * shape[3]; }
    bool ggml_is_contiguous(GGmlType t) const;
};

// CudaDevice, src/cuda.rs:213-229: one ordinal + one stream, shared by clones.
class CudaDevice {
   public:
    static GResult create(int ordinal, std::shared_ptr<CudaDevice> *out);  // CudaDevice::new + init_cuda_function
    ~CudaDevice();
    galois_hip_ctx *ctx() const { return ctx_; }
    GResult check(int32_t status) const;

   private:
    galois_hip_ctx *ctx_ = nullptr;
};

// Device::{Cpu, Gpu(CudaDevice)}, src/lib.rs:267-270
struct Device {
    std::shared_ptr<CudaDevice> gpu;  // null = Cpu
    bool is_gpu() const { return gpu != nullptr; }
};

class Tensor {
   public:
    // Tensor::from_raw(bytes, n_dims, shape, dtype, &device): copies the bytes to the device
    static GResult from_raw(const void *bytes, size_t nbytes, size_t n_dims, const size_t *shape, GGmlType dtype,
                            const Device &dev, Tensor *out);
    // Tensor::zeros / from_elem(0)
    static GResult zeros(size_t n_dims, const size_t *shape, GGmlType dtype, const Device &dev, Tensor *out);
    // to_cpu_tensor(): synchronises the stream and returns a host copy
    GResult to_cpu_tensor(Tensor *out) const;
    // view with another shape over the same storage (view_tensor): offset in storage elements
    GResult view(size_t elem_offset, size_t n_dims, const size_t *shape, Tensor *out) const;
    // view with explicit strides in storage elements (what permute / transpose produce in the reference)
    GResult view_strided(size_t elem_offset, size_t n_dims, const size_t *shape, const size_t *stride, Tensor *out) const;
    // overwrite the tensor's bytes from host memory (synchronous)
    GResult write(const void *bytes, size_t nbytes);

    GGmlType dtype() const { return dtype_; }
    const Dim &dim() const { return dim_; }
    const Device &device() const { return dev_; }
    size_t nbytes() const { return dim_.elem_count() / blck_size(dtype_) * type_size(dtype_); }
    const void *data() const { return ptr_; }  // host pointer (Cpu) or device pointer (Gpu)
    void *data() { return ptr_; }

   private:
    struct Storage;  // owns host vector or device allocation
    std::shared_ptr<Storage> storage_;
    void *ptr_ = nullptr;
    size_t avail_ = 0;  // bytes from ptr_ to the end of the storage
    GGmlType dtype_ = GGmlType::F32;
    Dim dim_;
    Device dev_;
};

// RopeCustomOption, src/op.rs:3294-3302
struct RopeCustomOption {
    size_t n_dims = 0;
    int32_t mode = 0;
    int32_t n_ctx = 0;
    float freq_base = 10000.0f;
    float freq_scale = 1.0f;
    float xpos_base = 0.0f;
    bool xpos_down = false;
};

GResult galois_matmul(const Tensor &a, const Tensor &b, Tensor &dst);                                   // op.rs:3093-3111
GResult galois_rms_norm(const Tensor &src, Tensor &dst, float eps);                                      // op.rs:3155-3169
GResult galois_rope_custom(const RopeCustomOption &op, const Tensor &src0, const Tensor &src1, Tensor &dst);  // op.rs:3304-3341
GResult galois_soft_max(const Tensor &src, Tensor &dst);                                                  // op.rs:3216-3230

enum class UnaryOp { Silu };  // the only arm the reference implements, src/op.rs:3232-3256
GResult galois_add(const Tensor &a, const Tensor &b, Tensor &dst);          // op.rs:3073-3091
GResult galois_mul(const Tensor &a, const Tensor &b, Tensor &dst);          // op.rs:3113-3127
GResult galois_unary(const Tensor &src, Tensor &dst, UnaryOp op);           // op.rs:3232-3256
GResult galois_scale(const Tensor &src0, const Tensor &src1, Tensor &dst);  // op.rs:3258-3279 (src1: one f32, Cpu or Gpu)
GResult galois_cpy(const Tensor &src, Tensor &dst);                         // op.rs:3171-3185
GResult galois_cont(const Tensor &src, Tensor &dst);                        // op.rs:3187-3201
GResult galois_get_rows(const Tensor &src0, const Tensor &src1, Tensor &dst);  // op.rs:3281-3292 (Gpu arm is todo!() there)

}  // namespace galois
