/* axiom/init.h — weight initialisers used by Dense and the attention layer (include/axiom/init.h,
 * src/core/init.c:60-94).
 * Values are drawn on the host in element order and copied to the tensor's device. */
#ifndef AX_INIT_H
#define AX_INIT_H
#include "tensor.h"
#ifdef __cplusplus
extern "C" {
#endif
void ax_init_kaiming_uniform(ax_tensor_t *t, int64_t fan_in);     /* U(+-sqrt(6/fan_in)) */
void ax_init_xavier_uniform(ax_tensor_t *t, int64_t fan_in, int64_t fan_out);   /* U(+-sqrt(6/(in+out))), init.c:60-70 */
void ax_init_normal(ax_tensor_t *t, float mean, float std);
void ax_init_uniform(ax_tensor_t *t, float low, float high);
#ifdef __cplusplus
}
#endif
#endif
