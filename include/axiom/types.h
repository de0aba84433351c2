/* axiom/types.h — scalar types, status codes and device ids of the Axiom C API, as far as the
 * GEMM path needs them.  Numeric values follow Axiom 0.10.0 (include/axiom/types.h:52-110) so
 * objects built against either header agree; AX_DEVICE_HIP is appended after the
 * reference's last device id. */
#ifndef AX_TYPES_H
#define AX_TYPES_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#define AX_MAX_DIMS 8

typedef enum {
    AX_FLOAT32 = 0, AX_FLOAT64, AX_INT32, AX_INT64, AX_UINT8, AX_BOOL, AX_DTYPE_COUNT
} ax_dtype_t;

static inline size_t ax_dtype_size(ax_dtype_t dt) {
    switch (dt) {
        case AX_FLOAT32: case AX_INT32: return 4;
        case AX_FLOAT64: case AX_INT64: return 8;
        case AX_UINT8: case AX_BOOL: return 1;
        default: return 0;
    }
}

typedef enum {
    AX_OK = 0,
    AX_ERR_NULL_ARG,
    AX_ERR_ALLOC,
    AX_ERR_SHAPE_MISMATCH,
    AX_ERR_DTYPE_MISMATCH,
    AX_ERR_INVALID_AXIS,
    AX_ERR_INVALID_SHAPE,
    AX_ERR_INVALID_DTYPE,
    AX_ERR_OUT_OF_BOUNDS,
    AX_ERR_BACKEND,
    AX_ERR_NOT_IMPLEMENTED,
    AX_ERR_INTERNAL,
    AX_STATUS_COUNT
} ax_status_t;

const char *ax_status_name(ax_status_t s);

typedef enum {
    AX_DEVICE_CPU = 0,
    AX_DEVICE_CUDA,        /* kept so numeric values match; no CUDA code exists here */
    AX_DEVICE_HIP,         /* MI355X through libaxhip */
    AX_DEVICE_COUNT
} ax_device_t;

typedef enum { AX_LAYOUT_NCHW = 0, AX_LAYOUT_NHWC = 1, AX_LAYOUT_COUNT } ax_layout_t;

#endif
