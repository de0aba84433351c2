/* axiom/device.h — device queries routed through the owning backend (include/axiom/device.h). */
#ifndef AX_DEVICE_H
#define AX_DEVICE_H
#include "tensor.h"
#include "types.h"
#ifdef __cplusplus
extern "C" {
#endif
int  ax_device_count(ax_device_t device);
void ax_device_synchronize(ax_device_t device);
int  ax_device_is_available(ax_device_t device);
#ifdef __cplusplus
}
#endif
#endif
