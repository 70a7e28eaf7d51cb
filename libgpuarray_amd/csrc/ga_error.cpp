// Error records and the static message table.
// Behaviour follows the reference's src/util/error.c:8-43 (per-context and
// process-global records, printf-style setters returning the code) and
// src/gpuarray_error.c:7-29 (one fixed string per code).
#include "private.hpp"

static ga_errrec g_global_err_storage = {{0}, 0};
ga_errrec *ga_global_err = &g_global_err_storage;

int ga_err_set(ga_errrec *e, int code, const char *msg) {
  e->code = code;
  snprintf(e->msg, GA_ERROR_MSGBUF_LEN, "%s", msg);
  return code;
}

int ga_err_fmt(ga_errrec *e, int code, const char *fmt, ...) {
  va_list ap;
  e->code = code;
  va_start(ap, fmt);
  vsnprintf(e->msg, GA_ERROR_MSGBUF_LEN, fmt, ap);
  va_end(ap);
  return code;
}

extern "C" const char *gpuarray_error_str(int err) {
  static const char *const table[] = {
      "No error",
      "Out of memory",
      "Value invalid or out of range",
      "Unknown device error",
      "Invalid value or operation",
      "Unsupported operation",
      nullptr, /* GA_SYS_ERROR: strerror(errno) */
      "Could not execute helper program",
      "Device does not support operation",
      "Buffer is read-only",
      "Buffer is write-only",
      "Error in BLAS call",
      "Unaligned array",
      "Copy is needed but disallowed by parameters",
      "No devices are available",
      "Undeterminate error",
      "Error in collectives call",
      "Input size too large for operation",
      "Error loading library",
  };
  if (err == GA_SYS_ERROR) return strerror(errno);
  if (err < 0 || err >= (int)(sizeof(table) / sizeof(table[0])))
    return "Unknown GA error";
  return table[err];
}
