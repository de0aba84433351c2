/* axiom/axiom.h — master include of the GEMM-path subset of the Axiom C API (plus layers, model
 * container and model files around it). */
#ifndef AXIOM_H
#define AXIOM_H
#include "attention.h"
#include "compute.h"
#include "device.h"
#include "error.h"
#include "init.h"
#include "layer.h"
#include "model.h"
#include "ops.h"
#include "quantize.h"
#include "rng.h"
#include "serialize.h"
#include "tensor.h"
#include "types.h"
#ifdef __cplusplus
extern "C" {
#endif
ax_status_t ax_init(void);       /* = ax_compute_init (include/axiom/axiom.h:102) */
void        ax_shutdown(void);
#ifdef __cplusplus
}
#endif
#endif
