/* axiom/tensor.h — refcounted storage + strided tensor view.  Field order and types of
 * ax_storage_t / ax_tensor_t follow Axiom (include/axiom/tensor.h:29-70) exactly: backend
 * objects built here are handed tensors created by the reference library and vice versa. */
#ifndef AX_TENSOR_H
#define AX_TENSOR_H

#include "error.h"
#include "types.h"
#ifndef __cplusplus
#include <stdatomic.h>
#endif

typedef struct {
    void *data;             /* host pointer, or a device pointer owned by the device's backend */
    size_t size_bytes;
#ifdef __cplusplus
    int refcount;
#else
    atomic_int refcount;
#endif
    ax_device_t device;
    bool is_arena_temp;     /* always false here (no arenas); kept for layout */
    uint64_t generation;    /* bumped on every write through the dispatch layer */
} ax_storage_t;

typedef struct ax_tensor {
    ax_storage_t *storage;
    int64_t shape[AX_MAX_DIMS];
    int64_t strides[AX_MAX_DIMS];   /* in elements */
    int ndim;
    ax_dtype_t dtype;
    int64_t offset;                 /* in elements */
    bool requires_grad;             /* autograd fields: carried, never used (inference only) */
    struct ax_tensor *grad;
    void *grad_fn;
    ax_layout_t layout;
} ax_tensor_t;

#ifdef __cplusplus
extern "C" {
#endif

/* storage: device memory comes from the owning backend's storage_alloc hook (zero-filled) */
ax_storage_t *ax_storage_create(size_t size_bytes, ax_device_t device);
void          ax_storage_retain(ax_storage_t *s);
void          ax_storage_release(ax_storage_t *s);

/* constructors allocate on the thread's default device; NULL + ax_err on failure */
ax_tensor_t *ax_tensor_create(const int64_t *shape, int ndim, ax_dtype_t dtype);   /* contents undefined */
ax_tensor_t *ax_tensor_zeros(const int64_t *shape, int ndim, ax_dtype_t dtype);
ax_tensor_t *ax_tensor_from_array(const void *host_data, const int64_t *shape, int ndim, ax_dtype_t dtype);
ax_tensor_t *ax_tensor_rand(const int64_t *shape, int ndim, float low, float high); /* fp32 U[low,high) */
void         ax_tensor_destroy(ax_tensor_t *t);
void         ax_set_seed(unsigned int seed);

int64_t      ax_tensor_numel(const ax_tensor_t *t);
bool         ax_tensor_is_contiguous(const ax_tensor_t *t);
ax_tensor_t *ax_tensor_reshape(ax_tensor_t *t, const int64_t *new_shape, int new_ndim);  /* view */

/* device placement */
void         ax_set_default_device(ax_device_t dev);
ax_device_t  ax_get_default_device(void);
ax_tensor_t *ax_tensor_to_device(ax_tensor_t *t, ax_device_t dev);   /* contiguous copy */
ax_tensor_t *ax_tensor_to_cpu(ax_tensor_t *t);
/* copy a contiguous tensor's elements to host memory, whatever device holds them */
ax_status_t  ax_tensor_read(const ax_tensor_t *t, void *host_dst, size_t bytes);
/* the reverse: fill a contiguous tensor from host memory (what the model loader uses to place
 * parameters on a device; the reference's loader memcpy()s into host storage, serialize.c:690) */
ax_status_t  ax_tensor_write(ax_tensor_t *t, const void *host_src, size_t bytes);

#ifdef __cplusplus
}
#endif
#endif
