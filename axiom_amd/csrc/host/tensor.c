/* Refcounted storage and tensor views (the subset of Axiom's src/core/tensor.c the GEMM path
 * uses).  Device memory is never touched here: allocation, release and copies go through the
 * hooks of the backend that owns the device (src/core/tensor.c:201-286, 1016-1085). */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "axiom/compute.h"
#include "axiom/internal/backend_ops.h"
#include "axiom/rng.h"
#include "axiom/tensor.h"

static _Thread_local ax_device_t tl_default_device = AX_DEVICE_CPU;

void ax_set_default_device(ax_device_t dev) { tl_default_device = dev; }
ax_device_t ax_get_default_device(void) { return tl_default_device; }
void ax_set_seed(unsigned int seed) { ax_rng_seed((uint64_t)seed); }

/* zeroed = false: the caller overwrites everything (host memory is never cleared here either way) */
static ax_storage_t *storage_create(size_t size_bytes, ax_device_t device, bool zeroed) {
    ax_storage_t *s = calloc(1, sizeof *s);
    if (!s) {
        ax_err_set(AX_ERR_ALLOC, "ax_storage_create: out of memory");
        return NULL;
    }
    if (device == AX_DEVICE_CPU) {
        size_t rounded = (size_bytes + 63) & ~(size_t)63;
        s->data = aligned_alloc(64, rounded ? rounded : 64);
        if (!s->data) ax_err_set(AX_ERR_ALLOC, "ax_storage_create: %zu host bytes", size_bytes);
    } else {
        const ax_backend_ops_t *ops = ax_backend_for_device(device);
        if (!ops || !ops->storage_alloc) {
            ax_err_set(AX_ERR_BACKEND, "no backend registered for device %d", (int)device);
            free(s);
            return NULL;
        }
        /* the hooks report their own failures */
        s->data = (!zeroed && ops->storage_alloc_uninit) ? ops->storage_alloc_uninit(size_bytes)
                                                         : ops->storage_alloc(size_bytes);
    }
    if (!s->data) {
        free(s);
        return NULL;
    }
    s->size_bytes = size_bytes;
    atomic_init(&s->refcount, 1);
    s->device = device;
    s->is_arena_temp = false;
    s->generation = 1;
    return s;
}

ax_storage_t *ax_storage_create(size_t size_bytes, ax_device_t device) { return storage_create(size_bytes, device, true); }

void ax_storage_retain(ax_storage_t *s) {
    if (s) atomic_fetch_add(&s->refcount, 1);
}

void ax_storage_release(ax_storage_t *s) {
    if (!s || s->is_arena_temp) return;
    if (atomic_fetch_sub(&s->refcount, 1) > 1) return;
    if (s->device == AX_DEVICE_CPU) {
        free(s->data);
    } else {
        const ax_backend_ops_t *ops = ax_backend_for_device(s->device);
        if (ops && ops->storage_free) ops->storage_free(s->data);
    }
    free(s);
}

static int64_t numel_of(const int64_t *shape, int ndim) {
    int64_t n = 1;
    for (int i = 0; i < ndim; i++) {
        if (shape[i] < 0) return -1;
        if (shape[i] != 0 && n > INT64_MAX / shape[i]) return -1;
        n *= shape[i];
    }
    return n;
}

static void set_contiguous(ax_tensor_t *t, const int64_t *shape, int ndim) {
    int64_t stride = 1;
    t->ndim = ndim;
    for (int i = ndim - 1; i >= 0; i--) {
        t->shape[i] = shape[i];
        t->strides[i] = stride;
        stride *= shape[i];
    }
}

static ax_tensor_t *tensor_create(const int64_t *shape, int ndim, ax_dtype_t dtype, bool zeroed) {
    if (!shape || ndim < 0 || ndim > AX_MAX_DIMS) {
        ax_err_set(AX_ERR_INVALID_SHAPE, "tensor_create: bad shape (ndim=%d)", ndim);
        return NULL;
    }
    size_t esz = ax_dtype_size(dtype);
    int64_t n = numel_of(shape, ndim);
    if (!esz || n < 0 || (uint64_t)n > (SIZE_MAX >> 1) / esz) {          /* n * esz must not wrap */
        ax_err_set(esz ? AX_ERR_INVALID_SHAPE : AX_ERR_INVALID_DTYPE, "tensor_create: bad dtype or extent");
        return NULL;
    }
    ax_tensor_t *t = calloc(1, sizeof *t);
    if (!t) {
        ax_err_set(AX_ERR_ALLOC, "tensor_create: out of memory");
        return NULL;
    }
    t->storage = storage_create((size_t)n * esz, tl_default_device, zeroed);
    if (!t->storage) {
        free(t);
        return NULL;
    }
    t->dtype = dtype;
    set_contiguous(t, shape, ndim);
    return t;
}

ax_tensor_t *ax_tensor_create(const int64_t *shape, int ndim, ax_dtype_t dtype) {
    return tensor_create(shape, ndim, dtype, false);
}

static ax_status_t write_from_host(ax_tensor_t *t, const void *src, size_t bytes) {
    if (!bytes) return AX_OK;
    char *dst = (char *)t->storage->data + (size_t)t->offset * ax_dtype_size(t->dtype);
    if (t->storage->device == AX_DEVICE_CPU) {
        memcpy(dst, src, bytes);
        return AX_OK;
    }
    const ax_backend_ops_t *ops = ax_backend_for_device(t->storage->device);
    if (!ops || !ops->memcpy_h2d) {
        ax_err_set(AX_ERR_BACKEND, "no h2d copy for device %d", (int)t->storage->device);
        return AX_ERR_BACKEND;
    }
    return ops->memcpy_h2d(dst, src, bytes);
}

ax_tensor_t *ax_tensor_zeros(const int64_t *shape, int ndim, ax_dtype_t dtype) {
    ax_tensor_t *t = tensor_create(shape, ndim, dtype, true);
    if (!t) return NULL;
    /* device allocations arrive zero-filled from storage_alloc; host memory is cleared here */
    if (t->storage->device == AX_DEVICE_CPU) memset(t->storage->data, 0, t->storage->size_bytes);
    return t;
}

ax_tensor_t *ax_tensor_from_array(const void *host_data, const int64_t *shape, int ndim, ax_dtype_t dtype) {
    if (!host_data) {
        ax_err_set(AX_ERR_NULL_ARG, "tensor_from_array: NULL data");
        return NULL;
    }
    ax_tensor_t *t = ax_tensor_create(shape, ndim, dtype);
    if (!t) return NULL;
    if (write_from_host(t, host_data, t->storage->size_bytes) != AX_OK) {
        ax_tensor_destroy(t);
        return NULL;
    }
    return t;
}

ax_tensor_t *ax_tensor_rand(const int64_t *shape, int ndim, float low, float high) {
    ax_tensor_t *t = ax_tensor_create(shape, ndim, AX_FLOAT32);
    if (!t) return NULL;
    int64_t n = ax_tensor_numel(t);
    float *host = t->storage->device == AX_DEVICE_CPU ? (float *)t->storage->data
                                                      : malloc((size_t)(n ? n : 1) * sizeof(float));
    if (!host) {
        ax_err_set(AX_ERR_ALLOC, "tensor_rand: out of memory");
        ax_tensor_destroy(t);
        return NULL;
    }
    for (int64_t i = 0; i < n; i++) host[i] = ax_rng_uniform(low, high);
    if (t->storage->device != AX_DEVICE_CPU) {
        ax_status_t st = write_from_host(t, host, (size_t)n * sizeof(float));
        free(host);
        if (st != AX_OK) {
            ax_tensor_destroy(t);
            return NULL;
        }
    }
    return t;
}

void ax_tensor_destroy(ax_tensor_t *t) {
    if (!t) return;
    ax_storage_release(t->storage);
    free(t);
}

int64_t ax_tensor_numel(const ax_tensor_t *t) { return t ? numel_of(t->shape, t->ndim) : 0; }

bool ax_tensor_is_contiguous(const ax_tensor_t *t) {
    if (!t) return false;
    int64_t expect = 1;
    for (int i = t->ndim - 1; i >= 0; i--) {
        if (t->shape[i] != 1 && t->strides[i] != expect) return false;
        expect *= t->shape[i];
    }
    return true;
}

ax_tensor_t *ax_tensor_reshape(ax_tensor_t *t, const int64_t *new_shape, int new_ndim) {
    if (!t || !new_shape) {
        ax_err_set(AX_ERR_NULL_ARG, "reshape: NULL");
        return NULL;
    }
    if (new_ndim < 0 || new_ndim > AX_MAX_DIMS || numel_of(new_shape, new_ndim) != ax_tensor_numel(t)) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "reshape: element count differs");
        return NULL;
    }
    if (!ax_tensor_is_contiguous(t)) {
        ax_err_set(AX_ERR_NOT_IMPLEMENTED, "reshape of a non-contiguous tensor");
        return NULL;
    }
    ax_tensor_t *v = calloc(1, sizeof *v);
    if (!v) {
        ax_err_set(AX_ERR_ALLOC, "reshape: out of memory");
        return NULL;
    }
    *v = *t;
    v->grad = NULL;
    v->grad_fn = NULL;
    set_contiguous(v, new_shape, new_ndim);
    ax_storage_retain(v->storage);
    return v;
}

ax_status_t ax_tensor_write(ax_tensor_t *t, const void *host_src, size_t bytes) {
    if (!t || !t->storage || !host_src) {
        ax_err_set(AX_ERR_NULL_ARG, "tensor_write: NULL");
        return AX_ERR_NULL_ARG;
    }
    if (!ax_tensor_is_contiguous(t) || bytes > (size_t)ax_tensor_numel(t) * ax_dtype_size(t->dtype)) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "tensor_write: non-contiguous tensor or too many bytes");
        return AX_ERR_SHAPE_MISMATCH;
    }
    ax_status_t st = write_from_host(t, host_src, bytes);
    if (st == AX_OK) t->storage->generation++;
    return st;
}

ax_status_t ax_tensor_read(const ax_tensor_t *t, void *host_dst, size_t bytes) {
    if (!t || !host_dst) {
        ax_err_set(AX_ERR_NULL_ARG, "tensor_read: NULL");
        return AX_ERR_NULL_ARG;
    }
    size_t esz = ax_dtype_size(t->dtype);
    if (!ax_tensor_is_contiguous(t) || bytes > (size_t)ax_tensor_numel(t) * esz) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "tensor_read: non-contiguous tensor or too many bytes");
        return AX_ERR_SHAPE_MISMATCH;
    }
    const char *src = (const char *)t->storage->data + (size_t)t->offset * esz;
    if (t->storage->device == AX_DEVICE_CPU) {
        memcpy(host_dst, src, bytes);
        return AX_OK;
    }
    const ax_backend_ops_t *ops = ax_backend_for_device(t->storage->device);
    if (!ops || !ops->memcpy_d2h) {
        ax_err_set(AX_ERR_BACKEND, "no d2h copy for device %d", (int)t->storage->device);
        return AX_ERR_BACKEND;
    }
    return ops->memcpy_d2h(host_dst, src, bytes);
}

ax_tensor_t *ax_tensor_to_device(ax_tensor_t *t, ax_device_t dev) {
    if (!t) {
        ax_err_set(AX_ERR_NULL_ARG, "to_device: NULL tensor");
        return NULL;
    }
    if (!ax_tensor_is_contiguous(t)) {
        ax_err_set(AX_ERR_NOT_IMPLEMENTED, "to_device of a non-contiguous tensor");
        return NULL;
    }
    const size_t esz = ax_dtype_size(t->dtype);
    const size_t bytes = (size_t)ax_tensor_numel(t) * esz;
    ax_device_t prev = tl_default_device;
    tl_default_device = dev;
    ax_tensor_t *out = ax_tensor_create(t->shape, t->ndim, t->dtype);
    tl_default_device = prev;
    if (!out) return NULL;
    ax_status_t st = AX_OK;
    const char *src = (const char *)t->storage->data + (size_t)t->offset * esz;
    if (t->storage->device == AX_DEVICE_CPU) {
        st = write_from_host(out, src, bytes);
    } else if (dev == AX_DEVICE_CPU) {
        st = ax_tensor_read(t, out->storage->data, bytes);
    } else if (dev == t->storage->device) {
        const ax_backend_ops_t *ops = ax_backend_for_device(dev);
        st = (ops && ops->memcpy_d2d) ? ops->memcpy_d2d(out->storage->data, src, bytes) : AX_ERR_BACKEND;
    } else {
        ax_err_set(AX_ERR_NOT_IMPLEMENTED, "copy between two non-CPU devices");
        st = AX_ERR_NOT_IMPLEMENTED;
    }
    if (st != AX_OK) {
        ax_tensor_destroy(out);
        return NULL;
    }
    out->layout = t->layout;
    return out;
}

ax_tensor_t *ax_tensor_to_cpu(ax_tensor_t *t) { return ax_tensor_to_device(t, AX_DEVICE_CPU); }
