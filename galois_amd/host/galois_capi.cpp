// Flat C handles over the C++ host mirror so that pytest can drive it with ctypes.
#include <cstring>
#include <string>

#include "galois.hpp"

using namespace galois;

static thread_local std::string g_last_error;
static int fail(const GResult &r) {
    g_last_error = r.msg;
    return (int)r.kind;
}

extern "C" {

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

}  // extern "C"
