/* axiom/serialize.h — model and tensor files (include/axiom/serialize.h, src/core/serialize.c).
 *
 * Files are the reference's, byte for byte (little-endian, no padding):
 *   .axt  u32 "AXT0" | u32 dtype | u32 ndim | i64 shape[ndim] | raw data
 *   .axm  u32 "AXON" | u32 version (4) | u32 n_layers
 *         per layer: u32 type | u32 n_params | u32 n_buffers | type-specific descriptor
 *         per parameter (then buffer) of each layer, in order: the tensor record of .axt without
 *         the magic
 *         u32 CRC-32 (zlib polynomial) of everything before it
 * ax_model_load builds the layers on the thread's default device and copies each parameter
 * there, so a model trained and saved by the reference runs on the GPU as loaded; ax_model_save
 * reads parameters back from whatever device holds them.  Layer types with a forward pass in
 * this library are accepted (Dense, the activation layers, LayerNorm, MHA); a file that names any
 * other type is refused with AX_ERR_NOT_IMPLEMENTED.  Every count and extent read from a file is
 * validated before it is used (serialize.c:189-260, 560-585).
 *
 * The reference has no file form for quantized weights; .axq is defined here:
 *   u32 "AXQ0" | i64 N | i64 K | f32 scales[N] | i8 data[N*K] | u32 CRC-32 of everything before */
#ifndef AX_SERIALIZE_H
#define AX_SERIALIZE_H
#include "model.h"
#include "quantize.h"
#ifdef __cplusplus
extern "C" {
#endif

#define AX_MAGIC 0x41584F4E          /* "AXON" */
#define AX_FORMAT_VERSION 4

ax_status_t  ax_model_save(ax_model_t *model, const char *path);
ax_model_t  *ax_model_load(const char *path);
ax_status_t  ax_tensor_save(ax_tensor_t *t, const char *path);
ax_tensor_t *ax_tensor_load(const char *path);

ax_status_t   ax_qweight_save(const ax_qweight_t *host_qw, const char *path);
ax_qweight_t *ax_qweight_load(const char *path);     /* host copy; ax_qweight_to_device() to place it */

#ifdef __cplusplus
}
#endif
#endif
