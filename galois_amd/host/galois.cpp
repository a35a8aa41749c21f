// Host mirror of galois's op layer over the C ABI (see galois.hpp).  The launch logic follows
// src/cuda.rs: dtype dispatch of CudaMap2::map (:476-521), the batch-slice loops of
// CudaMatMul::f_q_f32_f32 (:994-1139), and the one-kernel launchers of the row ops.
#include "galois.hpp"

#include <cmath>
#include <cstring>

namespace galois {

size_t type_size(GGmlType t) {
    switch (t) {
        case GGmlType::F32: return 4;
        case GGmlType::F16: return 2;
        case GGmlType::Q4_0: return 18;
        case GGmlType::I32: return 4;
    }
    return 0;
}
size_t blck_size(GGmlType t) { return t == GGmlType::Q4_0 ? 32 : 1; }

static GError err(GError::Kind k, const std::string &m) { return GError{k, m}; }
static GError ok() { return GError{}; }

Dim Dim::contiguous(size_t n_dims, const size_t *shape, GGmlType t) {
    Dim d;
    d.n_dims = n_dims;
    for (size_t i = 0; i < 4; i++) d.shape[i] = i < n_dims ? shape[i] : 1;
    d.stride[0] = 1;
    d.stride[1] = d.shape[0] / blck_size(t);
    for (size_t i = 2; i < 4; i++) d.stride[i] = d.stride[i - 1] * d.shape[i - 1];
    return d;
}

bool Dim::ggml_is_contiguous(GGmlType t) const {
    return stride[0] == 1 && stride[1] == shape[0] / blck_size(t) && stride[2] == stride[1] * shape[1] &&
           stride[3] == stride[2] * shape[2];
}

GResult CudaDevice::create(int ordinal, std::shared_ptr<CudaDevice> *out) {
    galois_hip_ctx *ctx = nullptr;
    int32_t st = galois_hip_create(ordinal, &ctx);
    if (st != 0) return err(GError::DeviceError, std::string("CudaDevice::new: ") + galois_hip_status_string(st));
    int32_t n = 0;
    if (galois_hip_abi_version() != GALOIS_HIP_ABI_VERSION) {
        galois_hip_destroy(ctx);
        return err(GError::DeviceError, "libgalois_hip: ABI version differs from the header this mirror was built against");
    }
    st = galois_hip_init_functions(ctx, GALOIS_HIP_ABI_VERSION, &n);
    if (st != 0) {
        galois_hip_destroy(ctx);
        return err(GError::DeviceError, "init_cuda_function: ABI mismatch");
    }
    auto d = std::shared_ptr<CudaDevice>(new CudaDevice());
    d->ctx_ = ctx;
    *out = d;
    return ok();
}
CudaDevice::~CudaDevice() {
    if (ctx_) galois_hip_destroy(ctx_);
}
GResult CudaDevice::check(int32_t st) const {
    if (st == 0) return ok();
    return err(GError::DeviceError, std::string("galois_hip status ") + std::to_string(st) + ": " + galois_hip_last_error(ctx_));
}

struct Tensor::Storage {
    std::vector<uint8_t> host;
    void *dev = nullptr;
    std::shared_ptr<CudaDevice> gpu;
    ~Storage() {
        if (dev && gpu) galois_hip_free(gpu->ctx(), dev);
    }
};

GResult Tensor::zeros(size_t n_dims, const size_t *shape, GGmlType dtype, const Device &dev, Tensor *out) {
    if (n_dims == 0 || n_dims > 4) return err(GError::ShapeError, "rank must be 1..4");
    Tensor t;
    t.dtype_ = dtype;
    t.dim_ = Dim::contiguous(n_dims, shape, dtype);
    t.dev_ = dev;
    if (t.dim_.shape[0] % blck_size(dtype) != 0) return err(GError::ShapeError, "ne0 is not a multiple of the block size");
    t.storage_ = std::make_shared<Storage>();
    const size_t nb = t.nbytes();
    if (dev.is_gpu()) {
        t.storage_->gpu = dev.gpu;
        GResult r = dev.gpu->check(galois_hip_alloc_zeros(dev.gpu->ctx(), nb, &t.storage_->dev));
        if (!r.ok()) return r;
        t.ptr_ = t.storage_->dev;
    } else {
        t.storage_->host.assign(nb, 0);
        t.ptr_ = t.storage_->host.data();
    }
    t.avail_ = nb;
    *out = t;
    return ok();
}

GResult Tensor::from_raw(const void *bytes, size_t nbytes, size_t n_dims, const size_t *shape, GGmlType dtype,
                         const Device &dev, Tensor *out) {
    Tensor t;
    GResult r = zeros(n_dims, shape, dtype, dev, &t);
    if (!r.ok()) return r;
    if (nbytes != t.nbytes()) return err(GError::ShapeError, "from_raw: byte count does not match the shape");
    if (dev.is_gpu())
        r = dev.gpu->check(galois_hip_htod_sync_copy(dev.gpu->ctx(), t.ptr_, bytes, nbytes));
    else
        memcpy(t.ptr_, bytes, nbytes);
    if (!r.ok()) return r;
    *out = t;
    return ok();
}

GResult Tensor::to_cpu_tensor(Tensor *out) const {
    if (!dim_.ggml_is_contiguous(dtype_)) return err(GError::Unimplemented, "to_cpu_tensor of a strided view");
    Tensor t;
    GResult r = zeros(dim_.n_dims, dim_.shape, dtype_, Device{}, &t);
    if (!r.ok()) return r;
    if (dev_.is_gpu())
        r = dev_.gpu->check(galois_hip_dtoh_sync_copy(dev_.gpu->ctx(), t.ptr_, ptr_, nbytes()));
    else
        memcpy(t.ptr_, ptr_, nbytes());
    if (!r.ok()) return r;
    *out = t;
    return ok();
}

GResult Tensor::view(size_t elem_offset, size_t n_dims, const size_t *shape, Tensor *out) const {
    Tensor t = *this;
    t.dim_ = Dim::contiguous(n_dims, shape, dtype_);
    if (elem_offset % blck_size(dtype_) != 0) return err(GError::ShapeError, "view offset splits a block");
    const size_t off_bytes = elem_offset / blck_size(dtype_) * type_size(dtype_);
    if (off_bytes + t.nbytes() > avail_) return err(GError::ShapeError, "view exceeds the tensor");
    t.avail_ = avail_ - off_bytes;
    t.ptr_ = (uint8_t *)ptr_ + off_bytes;
    *out = t;
    return ok();
}

GResult Tensor::view_strided(size_t elem_offset, size_t n_dims, const size_t *shape, const size_t *stride,
                             Tensor *out) const {
    if (n_dims == 0 || n_dims > 4) return err(GError::ShapeError, "rank must be 1..4");
    if (blck_size(dtype_) != 1) return err(GError::Unimplemented, "strided views of quantized tensors");
    Tensor t = *this;
    t.dim_ = Dim();
    t.dim_.n_dims = n_dims;
    size_t last = 0;  // largest element offset the view reaches
    for (size_t i = 0; i < 4; i++) {
        t.dim_.shape[i] = i < n_dims ? shape[i] : 1;
        t.dim_.stride[i] = i < n_dims ? stride[i] : (i ? t.dim_.stride[i - 1] * t.dim_.shape[i - 1] : 1);
        if (t.dim_.shape[i] == 0) return err(GError::ShapeError, "view with an empty dimension");
        last += (t.dim_.shape[i] - 1) * t.dim_.stride[i];
    }
    const size_t ts = type_size(dtype_);
    if ((elem_offset + last + 1) * ts > avail_) return err(GError::ShapeError, "view exceeds the tensor");
    t.avail_ = avail_ - elem_offset * ts;
    t.ptr_ = (uint8_t *)ptr_ + elem_offset * ts;
    *out = t;
    return ok();
}

GResult Tensor::write(const void *bytes, size_t n) {
    if (!dim_.ggml_is_contiguous(dtype_)) return err(GError::Unimplemented, "write into a strided view");
    if (n != nbytes()) return err(GError::ShapeError, "write: byte count does not match the shape");
    if (dev_.is_gpu()) return dev_.gpu->check(galois_hip_htod_sync_copy(dev_.gpu->ctx(), ptr_, bytes, n));
    memcpy(ptr_, bytes, n);
    return ok();
}

// ---- ops ----------------------------------------------------------------------------------------

static bool all_gpu(std::initializer_list<const Tensor *> ts, std::shared_ptr<CudaDevice> *dev) {
    for (const Tensor *t : ts) {
        if (!t->device().is_gpu()) return false;
        if (*dev && t->device().gpu != *dev) return false;
        *dev = t->device().gpu;
    }
    return true;
}

// f32 x f32 arm (the products over the KV cache).  The reference routes this case to a todo!()
// (src/cuda.rs:994-1010) after a cuBLAS sgemm path for F16 weights (:698-782); here src0 may be
// any strided 3-D view, so a permuted cache needs no cont() copy first.
// (F32 | F16, F32) -> F32 over strided views of src0.
static GResult matmul_f32(const CudaDevice &dev, const Tensor &a, const Tensor &b, Tensor &dst) {
    const Dim &ad = a.dim(), &bd = b.dim(), &dd = dst.dim();
    if (ad.shape[0] != bd.shape[0]) return err(GError::ShapeError, "matmul: ne00 != ne10");
    if (dd.shape[0] != ad.shape[1] || dd.shape[1] != bd.shape[1] || dd.shape[2] != bd.shape[2] || dd.shape[3] != bd.shape[3])
        return err(GError::ShapeError, "matmul: dst shape must be [ne01, ne11, ne12, ne13]");
    if (ad.shape[3] != 1 || bd.shape[3] != 1) return err(GError::Unimplemented, "matmul f32: 4-D batches");
    if (ad.shape[2] == 0 || bd.shape[2] % ad.shape[2] != 0) return err(GError::ShapeError, "matmul: src0 must broadcast over ne12");
    if (!bd.ggml_is_contiguous(b.dtype()) || !dd.ggml_is_contiguous(dst.dtype()))
        return err(GError::Unimplemented, "matmul f32: src1 and dst must be contiguous");
    // an F16 src0 is the (F16, F32) -> F32 arm that the reference hands to cuBLAS (CudaMatMul::f_x_y_y,
    // src/cuda.rs:881-992): the same views, the a operand widened exactly
    const int32_t K = (int32_t)ad.shape[0], N = (int32_t)ad.shape[1], M = (int32_t)bd.shape[1];
    const int32_t ne02 = (int32_t)ad.shape[2], ne12 = (int32_t)bd.shape[2];
    const int64_t s0 = (int64_t)ad.stride[0], s1 = (int64_t)ad.stride[1], s2 = (int64_t)ad.stride[2];
    if (a.dtype() == GGmlType::F16)
        return dev.check(galois_hip_mul_mat_f16_f32(dev.ctx(), a.data(), (const float *)b.data(), (float *)dst.data(), K, N, M,
                                                    ne02, ne12, s0, s1, s2));
    return dev.check(galois_hip_mul_mat_f32(dev.ctx(), (const float *)a.data(), (const float *)b.data(), (float *)dst.data(),
                                            K, N, M, ne02, ne12, s0, s1, s2));
}

// galois_matmul, src/op.rs:3093-3111 -> CudaMatMul.map -> f_q_f32_f32 (src/cuda.rs:994-1139).
GResult galois_matmul(const Tensor &a, const Tensor &b, Tensor &dst) {
    std::shared_ptr<CudaDevice> dev;
    if (!all_gpu({&a, &b, &dst}, &dev))
        return err(GError::Unimplemented, "galois_matmul: only (Gpu, Gpu, Gpu) operands on one device (the reference's other arms are todo!() or CPU)");
    if ((a.dtype() == GGmlType::F32 || a.dtype() == GGmlType::F16) && b.dtype() == GGmlType::F32 && dst.dtype() == GGmlType::F32)
        return matmul_f32(*dev, a, b, dst);
    if (!(a.dtype() == GGmlType::Q4_0 && b.dtype() == GGmlType::F32 && dst.dtype() == GGmlType::F32))
        return err(GError::Unimplemented, "galois_matmul: only (Q4_0 | F16 | F32, F32) -> F32 (CudaMap2::map, src/cuda.rs:476-521)");
    const Dim &ad = a.dim(), &bd = b.dim(), &dd = dst.dim();
    const size_t ne00 = ad.shape[0], ne01 = ad.shape[1], ne02 = ad.shape[2], ne03 = ad.shape[3];
    const size_t ne10 = bd.shape[0], ne11 = bd.shape[1], ne12 = bd.shape[2], ne13 = bd.shape[3];
    const size_t ne0 = dd.shape[0], ne1 = dd.shape[1];
    // the asserts of src/op.rs:1422-1435, 1473-1474 as errors
    if (ne00 != ne10) return err(GError::ShapeError, "matmul: ne00 != ne10");
    if (ne0 != ne01 || ne1 != ne11 || dd.shape[2] != ne12 || dd.shape[3] != ne13)
        return err(GError::ShapeError, "matmul: dst shape must be [ne01, ne11, ne12, ne13]");
    if (ne02 == 0 || ne03 == 0 || ne12 % ne02 != 0 || ne13 % ne03 != 0)
        return err(GError::ShapeError, "matmul: src0 must broadcast over src1's batch dims");
    if (ne03 != 1 && ne03 != ne13) return err(GError::Unimplemented, "matmul: broadcast over ne03");
    if (!ad.ggml_is_contiguous(a.dtype()) || !bd.ggml_is_contiguous(b.dtype()) || !dd.ggml_is_contiguous(dst.dtype()))
        return err(GError::Unimplemented, "matmul: strided operands (the reference copies them first, src/cuda.rs:1049-1122)");
    if (ne00 % 32 != 0) return err(GError::ShapeError, "matmul: ne00 must be a multiple of 32");
    const size_t i02_divisor = ne12 / ne02;
    const uint8_t *w = (const uint8_t *)a.data();
    const float *x = (const float *)b.data();
    float *y = (float *)dst.data();
    // Batch slices of a decode product (ne11 == 1): the reference launches one kernel per slice (the loop at
    // src/cuda.rs:1026-1034); here up to eight slices go out per launch when the grouped kernel takes the shape
    // (a launch gap costs as much as streaming ~15 MB of weights).  Same results bit for bit.
    const size_t nslices = ne13 * ne12;
    if (ne11 == 1 && nslices > 1 && ne00 % 64 == 0 && ne00 <= 12288 && ((uintptr_t)w % 4) == 0 && ((uintptr_t)x % 8) == 0 &&
        (ne01 * (ne00 / 32) * 18) % 4 == 0 && (ne10 * sizeof(float)) % 8 == 0) {
        for (size_t i0 = 0; i0 < nslices; i0 += 8) {
            galois_hip_gemv_item items[8];
            const size_t n = nslices - i0 < 8 ? nslices - i0 : 8;
            memset(items, 0, sizeof(items));
            for (size_t j = 0; j < n; j++) {
                items[j].vx = w + ((i0 + j) / i02_divisor) * ne01 * (ne00 / 32) * 18;
                items[j].y = x + (i0 + j) * ne10;
                items[j].dst = y + (i0 + j) * ne0;
                items[j].ncols = (int32_t)ne00, items[j].nrows = (int32_t)ne01;
            }
            GResult r = dev->check(galois_hip_dequantize_mul_mat_vec_q4_0_group(dev->ctx(), items, (int32_t)n));
            if (!r.ok()) return r;
        }
        return ok();
    }
    for (size_t i0 = 0; i0 < nslices; i0++) {  // src/cuda.rs:1026-1034 and :1076-1134
        const uint8_t *wi = w + (i0 / i02_divisor) * ne01 * (ne00 / 32) * 18;
        const float *xi = x + i0 * ne11 * ne10;
        float *yi = y + i0 * ne1 * ne0;
        int32_t st;
        if (ne11 == 1)  // GEMV branch: ne11 == 1 && ne00 % GGML_CUDA_DMMV_X == 0
            st = galois_hip_dequantize_mul_mat_vec_q4_0(dev->ctx(), wi, xi, yi, (int32_t)ne00, (int32_t)ne01);
        else
            st = galois_hip_mul_mat_q4_0_f32(dev->ctx(), wi, xi, yi, (int32_t)ne00, (int32_t)ne01, (int32_t)ne11);
        GResult r = dev->check(st);
        if (!r.ok()) return r;
    }
    return ok();
}

// galois_rms_norm, src/op.rs:3155-3169 -> CudaRmsNorm::f (src/cuda.rs:1146-1181).
GResult galois_rms_norm(const Tensor &src, Tensor &dst, float eps) {
    std::shared_ptr<CudaDevice> dev;
    if (!all_gpu({&src, &dst}, &dev)) return err(GError::Unimplemented, "galois_rms_norm: only (Gpu, Gpu)");
    if (src.dtype() != GGmlType::F32 || dst.dtype() != GGmlType::F32) return err(GError::Unimplemented, "galois_rms_norm: F32 only");
    if (src.dim().elem_count() != dst.dim().elem_count() || src.dim().shape[0] != dst.dim().shape[0])
        return err(GError::ShapeError, "rms_norm: src and dst shapes differ");
    if (!src.dim().ggml_is_contiguous(src.dtype()) || !dst.dim().ggml_is_contiguous(dst.dtype()))
        return err(GError::Unimplemented, "galois_rms_norm: contiguous operands only (the kernel walks whole rows)");
    return dev->check(galois_hip_rms_norm_f32(dev->ctx(), (const float *)src.data(), (float *)dst.data(),
                                              (int32_t)src.dim().shape[0], (int32_t)src.dim().nrows(), eps));
}

// galois_rope_custom, src/op.rs:3304-3341 -> CudaRope::f_x_y_x (src/cuda.rs:1300-1356).
GResult galois_rope_custom(const RopeCustomOption &op, const Tensor &src0, const Tensor &src1, Tensor &dst) {
    std::shared_ptr<CudaDevice> dev;
    if (!all_gpu({&src0, &src1, &dst}, &dev)) return err(GError::Unimplemented, "galois_rope_custom: only (Gpu, Gpu, Gpu)");
    if (src0.dtype() != GGmlType::F32 || dst.dtype() != GGmlType::F32) return err(GError::Unimplemented, "rope: F32 only");
    if ((op.mode & 2) != 0 || (op.mode & 4) != 0) return err(GError::Unimplemented, "rope: NeoX / GLM modes (todo!() at src/cuda.rs:1336-1340)");
    if ((op.mode & 1) == 0) {
        if (src1.dtype() != GGmlType::I32) return err(GError::ShapeError, "rope: positions must be I32");
        if (src1.dim().shape[0] != dst.dim().shape[2]) return err(GError::ShapeError, "rope: one position per ne2");
    }
    if (op.n_dims == 0 || op.n_dims % 2 != 0 || src0.dim().shape[0] % 2 != 0)
        return err(GError::ShapeError, "rope: n_dims and ne00 must be even");
    if (src0.dim().elem_count() != dst.dim().elem_count()) return err(GError::ShapeError, "rope: src and dst shapes differ");
    if (!src0.dim().ggml_is_contiguous(src0.dtype()) || !dst.dim().ggml_is_contiguous(dst.dtype()))
        return err(GError::Unimplemented, "galois_rope_custom: contiguous operands only (the kernel walks whole rows)");
    const float theta_scale = powf(op.freq_base, -2.0f / (float)op.n_dims);  // src/cuda.rs:1327
    return dev->check(galois_hip_rope_f32(dev->ctx(), (const float *)src0.data(), (float *)dst.data(),
                                          (int32_t)src0.dim().shape[0], (int32_t)src0.dim().nrows(),
                                          (const int32_t *)src1.data(), op.freq_scale, (int32_t)src0.dim().shape[1],
                                          theta_scale));
}

// galois_soft_max, src/op.rs:3216-3230 -> CudaSoftMax::f (src/cuda.rs:1642-1663).
GResult galois_soft_max(const Tensor &src, Tensor &dst) {
    std::shared_ptr<CudaDevice> dev;
    if (!all_gpu({&src, &dst}, &dev)) return err(GError::Unimplemented, "galois_soft_max: only (Gpu, Gpu)");
    if (src.dtype() != GGmlType::F32 || dst.dtype() != GGmlType::F32) return err(GError::Unimplemented, "soft_max: F32 only");
    if (src.dim().elem_count() != dst.dim().elem_count() || src.dim().shape[0] != dst.dim().shape[0])
        return err(GError::ShapeError, "soft_max: src and dst shapes differ");
    if (!src.dim().ggml_is_contiguous(src.dtype()) || !dst.dim().ggml_is_contiguous(dst.dtype()))
        return err(GError::Unimplemented, "galois_soft_max: contiguous operands only (the kernel walks whole rows)");
    return dev->check(galois_hip_soft_max_f32(dev->ctx(), (const float *)src.data(), (float *)dst.data(),
                                              (int32_t)src.dim().shape[0], (int32_t)src.dim().nrows()));
}

// galois_add / galois_mul, src/op.rs:3073-3127 -> CudaAdd / CudaMul (src/cuda.rs:1190-1250):
// kx = elements of src0, ky = ne10 * ne11 of src1, dst[i] = src0[i] op src1[i % ky].
static GResult binary(const char *name, bool is_add, const Tensor &a, const Tensor &b, Tensor &dst) {
    std::shared_ptr<CudaDevice> dev;
    if (!all_gpu({&a, &b, &dst}, &dev)) return err(GError::Unimplemented, std::string(name) + ": only (Gpu, Gpu, Gpu)");
    if (a.dtype() != GGmlType::F32 || b.dtype() != GGmlType::F32 || dst.dtype() != GGmlType::F32)
        return err(GError::Unimplemented, std::string(name) + ": F32 only");
    if (!a.dim().ggml_is_contiguous(a.dtype()) || !b.dim().ggml_is_contiguous(b.dtype()) ||
        !dst.dim().ggml_is_contiguous(dst.dtype()))
        return err(GError::Unimplemented, std::string(name) + ": contiguous operands only");
    const int64_t kx = (int64_t)a.dim().elem_count(), ky = (int64_t)(b.dim().shape[0] * b.dim().shape[1]);
    if ((int64_t)dst.dim().elem_count() != kx) return err(GError::ShapeError, std::string(name) + ": dst must have src0's element count");
    auto fn = is_add ? galois_hip_add_f32 : galois_hip_mul_f32;
    return dev->check(fn(dev->ctx(), (const float *)a.data(), (const float *)b.data(), (float *)dst.data(), kx, ky));
}
GResult galois_add(const Tensor &a, const Tensor &b, Tensor &dst) { return binary("galois_add", true, a, b, dst); }
GResult galois_mul(const Tensor &a, const Tensor &b, Tensor &dst) { return binary("galois_mul", false, a, b, dst); }

// galois_unary, src/op.rs:3232-3256 -> CudaSilu (src/cuda.rs:1665-1690).
GResult galois_unary(const Tensor &src, Tensor &dst, UnaryOp op) {
    std::shared_ptr<CudaDevice> dev;
    if (!all_gpu({&src, &dst}, &dev)) return err(GError::Unimplemented, "galois_unary: only (Gpu, Gpu)");
    if (op != UnaryOp::Silu) return err(GError::Unimplemented, "galois_unary: only Silu");
    if (src.dtype() != GGmlType::F32 || dst.dtype() != GGmlType::F32) return err(GError::Unimplemented, "galois_unary: F32 only");
    if (src.dim().elem_count() != dst.dim().elem_count()) return err(GError::ShapeError, "unary: src and dst shapes differ");
    if (!src.dim().ggml_is_contiguous(src.dtype()) || !dst.dim().ggml_is_contiguous(dst.dtype()))
        return err(GError::Unimplemented, "galois_unary: contiguous operands only");
    return dev->check(galois_hip_silu_f32(dev->ctx(), (const float *)src.data(), (float *)dst.data(),
                                          (int64_t)src.dim().elem_count()));
}

// galois_scale, src/op.rs:3258-3279 -> CudaScale::f_g_c (src/cuda.rs:1621-1638): the factor is the first
// element of src1.  The reference's (Gpu, Gpu, Gpu) arm would read device memory from the host; only the
// (Gpu, Cpu, Gpu) arm is meaningful and kept.
GResult galois_scale(const Tensor &src0, const Tensor &src1, Tensor &dst) {
    std::shared_ptr<CudaDevice> dev;
    if (!all_gpu({&src0, &dst}, &dev) || src1.device().is_gpu())
        return err(GError::Unimplemented, "galois_scale: only (Gpu, Cpu, Gpu)");
    if (src0.dtype() != GGmlType::F32 || src1.dtype() != GGmlType::F32 || dst.dtype() != GGmlType::F32)
        return err(GError::Unimplemented, "galois_scale: F32 only");
    if (src1.dim().elem_count() == 0) return err(GError::ShapeError, "scale: empty factor tensor");
    if (src0.dim().elem_count() != dst.dim().elem_count()) return err(GError::ShapeError, "scale: src and dst shapes differ");
    if (!src0.dim().ggml_is_contiguous(src0.dtype()) || !dst.dim().ggml_is_contiguous(dst.dtype()))
        return err(GError::Unimplemented, "galois_scale: contiguous operands only");
    return dev->check(galois_hip_scale_f32(dev->ctx(), (const float *)src0.data(), (float *)dst.data(),
                                           *(const float *)src1.data(), (int64_t)src0.dim().elem_count()));
}

// galois_cpy / galois_cont, src/op.rs:3171-3201 -> CudaCpy (src/cuda.rs:1382-1595): element i of the source
// (in its own ne0/ne1/ne2 order and byte strides) goes to element i of the destination.
GResult galois_cpy(const Tensor &src, Tensor &dst) {
    std::shared_ptr<CudaDevice> dev;
    if (!all_gpu({&src, &dst}, &dev)) return err(GError::Unimplemented, "galois_cpy: only (Gpu, Gpu)");
    if (src.dtype() != GGmlType::F32 || (dst.dtype() != GGmlType::F32 && dst.dtype() != GGmlType::F16))
        return err(GError::Unimplemented, "galois_cpy: F32 -> F32 | F16 only");
    const Dim &sd = src.dim(), &dd = dst.dim();
    if (sd.elem_count() != dd.elem_count()) return err(GError::ShapeError, "cpy: element counts differ");
    if (sd.shape[3] != 1 || dd.shape[3] != 1) return err(GError::Unimplemented, "cpy: 4-D tensors (the kernel indexes three dims, cpy.cu:79-110)");
    const int64_t ss = 4, ds = (int64_t)type_size(dst.dtype());
    return dev->check(galois_hip_cpy_f32(dev->ctx(), src.data(), dst.data(), dst.dtype() == GGmlType::F16,
                                         (int64_t)sd.elem_count(), (int64_t)sd.shape[0], (int64_t)sd.shape[1],
                                         (int64_t)sd.stride[0] * ss, (int64_t)sd.stride[1] * ss, (int64_t)sd.stride[2] * ss,
                                         (int64_t)dd.shape[0], (int64_t)dd.shape[1], (int64_t)dd.stride[0] * ds,
                                         (int64_t)dd.stride[1] * ds, (int64_t)dd.stride[2] * ds));
}
GResult galois_cont(const Tensor &src, Tensor &dst) {
    if (!dst.dim().ggml_is_contiguous(dst.dtype())) return err(GError::ShapeError, "cont: dst must be contiguous");
    return galois_cpy(src, dst);
}

// galois_get_rows, src/op.rs:3281-3292 -> GetRows::f_q_x_f32 (src/op.rs:2546-2571), on the device.
GResult galois_get_rows(const Tensor &src0, const Tensor &src1, Tensor &dst) {
    std::shared_ptr<CudaDevice> dev;
    if (!all_gpu({&src0, &src1, &dst}, &dev)) return err(GError::Unimplemented, "galois_get_rows: only (Gpu, Gpu, Gpu)");
    if (src0.dtype() != GGmlType::Q4_0 || src1.dtype() != GGmlType::I32 || dst.dtype() != GGmlType::F32)
        return err(GError::Unimplemented, "galois_get_rows: (Q4_0, I32) -> F32 only");
    const size_t nc = src0.dim().shape[0], nr = src1.dim().elem_count();
    if (dst.dim().shape[0] != nc || dst.dim().elem_count() != nc * nr) return err(GError::ShapeError, "get_rows: dst must be [ne00, n_ids]");
    if (!src0.dim().ggml_is_contiguous(src0.dtype()) || !dst.dim().ggml_is_contiguous(dst.dtype()))
        return err(GError::Unimplemented, "galois_get_rows: contiguous operands only");
    return dev->check(galois_hip_get_rows_q4_0(dev->ctx(), src0.data(), (const int32_t *)src1.data(), (float *)dst.data(),
                                               (int32_t)nc, (int32_t)nr, (int32_t)src0.dim().shape[1]));
}

}  // namespace galois
