/* Status names, structured errors and checked integer helpers used on the attention
 * path (behaviour of src/core/status.c and include/yvex/internal/core.h:289-295). */
#include "private.h"

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

const char *yvex_status_name(yvex_status status)
{
    switch (status) {
    case YVEX_OK: return "YVEX_OK";
    case YVEX_ERR: return "YVEX_ERR";
    case YVEX_ERR_NOMEM: return "YVEX_ERR_NOMEM";
    case YVEX_ERR_IO: return "YVEX_ERR_IO";
    case YVEX_ERR_FORMAT: return "YVEX_ERR_FORMAT";
    case YVEX_ERR_UNSUPPORTED: return "YVEX_ERR_UNSUPPORTED";
    case YVEX_ERR_BACKEND: return "YVEX_ERR_BACKEND";
    case YVEX_ERR_BOUNDS: return "YVEX_ERR_BOUNDS";
    case YVEX_ERR_STATE: return "YVEX_ERR_STATE";
    case YVEX_ERR_CANCELLED: return "YVEX_ERR_CANCELLED";
    case YVEX_ERR_INVALID_ARG: return "YVEX_ERR_INVALID_ARG";
    case YVEX_ERR_TIMEOUT: return "YVEX_ERR_TIMEOUT";
    }
    return "YVEX_STATUS_UNKNOWN";
}

void yvex_error_clear(yvex_error *err)
{
    if (!err) return;
    err->code = YVEX_OK;
    err->where[0] = '\0';
    err->message[0] = '\0';
}

void yvex_core_text_copy(char *destination, size_t capacity, const char *source)
{
    size_t n;
    if (!destination || !capacity) return;
    if (!source) source = "";
    n = strlen(source);
    if (n >= capacity) n = capacity - 1u;
    memcpy(destination, source, n);
    destination[n] = '\0';
}

void yvex_error_set(yvex_error *err, yvex_status code, const char *where, const char *message)
{
    if (!err) return;
    err->code = code;
    yvex_core_text_copy(err->where, sizeof(err->where), where);
    yvex_core_text_copy(err->message, sizeof(err->message), message);
}

void yvex_error_setf(yvex_error *err, yvex_status code, const char *where, const char *fmt, ...)
{
    char text[YVEX_ERROR_MESSAGE_CAP];
    va_list args;
    va_start(args, fmt);
    vsnprintf(text, sizeof(text), fmt ? fmt : "", args);
    va_end(args);
    yvex_error_set(err, code, where, text);
}

int yvex_core_u64_add(unsigned long long left, unsigned long long right, unsigned long long *out)
{
    if (!out || left > ULLONG_MAX - right) return 0;
    *out = left + right;
    return 1;
}

int yvex_core_u64_mul(unsigned long long left, unsigned long long right, unsigned long long *out)
{
    if (!out || (left != 0ull && right > ULLONG_MAX / left)) return 0;
    *out = left * right;
    return 1;
}
