/* Thread-local error state (the convention of Axiom's src/core/error.c). */
#include <stdarg.h>
#include <stdio.h>

#include "axiom/error.h"

static _Thread_local ax_status_t tl_status = AX_OK;
static _Thread_local char tl_message[AX_ERR_MSG_MAX] = "";

void ax_err_set(ax_status_t status, const char *fmt, ...) {
    tl_status = status;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(tl_message, sizeof tl_message, fmt ? fmt : "", ap);
    va_end(ap);
}

void ax_err_clear(void) {
    tl_status = AX_OK;
    tl_message[0] = '\0';
}

ax_status_t ax_err_last_status(void) { return tl_status; }
const char *ax_err_last_message(void) { return tl_message; }

const char *ax_status_name(ax_status_t s) {
    static const char *const names[AX_STATUS_COUNT] = {
        "ok", "null argument", "allocation failed", "shape mismatch", "dtype mismatch",
        "invalid axis", "invalid shape", "invalid dtype", "out of bounds", "backend error",
        "not implemented", "internal error"};
    return ((int)s >= 0 && s < AX_STATUS_COUNT) ? names[s] : "unknown error";
}
