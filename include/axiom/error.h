/* axiom/error.h — per-thread status + message, the error convention of the Axiom C API
 * (include/axiom/error.h:13-33): functions return ax_status_t (or NULL) and never abort. */
#ifndef AX_ERROR_H
#define AX_ERROR_H

#include "types.h"

#ifdef __cplusplus
extern "C" {
#endif

#define AX_ERR_MSG_MAX 256

void        ax_err_set(ax_status_t status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void        ax_err_clear(void);
ax_status_t ax_err_last_status(void);
const char *ax_err_last_message(void);     /* "" when no error; valid until the next set/clear */

#ifdef __cplusplus
}
#endif
#endif
