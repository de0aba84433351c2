/* Weight initialisers (Axiom's src/core/init.c:30-94): draw on the host in element order,
 * then hand the buffer to the tensor's device through the backend's h2d hook. */
#include <math.h>
#include <stdlib.h>

#include "axiom/compute.h"
#include "axiom/init.h"
#include "axiom/internal/backend_ops.h"
#include "axiom/rng.h"

typedef float (*draw_fn)(float p0, float p1);

static void fill_with(ax_tensor_t *t, draw_fn draw, float p0, float p1) {
    if (!t || !t->storage || t->dtype != AX_FLOAT32) return;
    const int64_t n = ax_tensor_numel(t);
    const bool on_host = t->storage->device == AX_DEVICE_CPU;
    float *buf = on_host ? (float *)t->storage->data + t->offset : malloc((size_t)(n ? n : 1) * sizeof(float));
    if (!buf) return;
    for (int64_t i = 0; i < n; i++) buf[i] = draw(p0, p1);
    if (!on_host) {
        const ax_backend_ops_t *ops = ax_backend_for_device(t->storage->device);
        if (ops && ops->memcpy_h2d)
            ops->memcpy_h2d((float *)t->storage->data + t->offset, buf, (size_t)n * sizeof(float));
        free(buf);
    }
    t->storage->generation++;
}

void ax_init_kaiming_uniform(ax_tensor_t *t, int64_t fan_in) {
    const float limit = sqrtf(6.0f / (float)fan_in);
    fill_with(t, ax_rng_uniform, -limit, limit);
}

void ax_init_xavier_uniform(ax_tensor_t *t, int64_t fan_in, int64_t fan_out) {
    const float limit = sqrtf(6.0f / (float)(fan_in + fan_out));
    fill_with(t, ax_rng_uniform, -limit, limit);
}

void ax_init_uniform(ax_tensor_t *t, float low, float high) { fill_with(t, ax_rng_uniform, low, high); }
void ax_init_normal(ax_tensor_t *t, float mean, float std) { fill_with(t, ax_rng_normal_params, mean, std); }
