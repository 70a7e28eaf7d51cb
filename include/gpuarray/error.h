/* Error codes shared by every entry point.
 * Values and order are ABI: reference src/gpuarray/error.h:19-41.
 * Message table: reference src/gpuarray_error.c:7-29. */
#ifndef GPUARRAY_ERROR_H
#define GPUARRAY_ERROR_H

#include <gpuarray/config.h>

#ifdef __cplusplus
extern "C" {
#endif

enum ga_error {
  GA_NO_ERROR = 0,
  GA_MEMORY_ERROR = 1,
  GA_VALUE_ERROR = 2,
  GA_IMPL_ERROR = 3,        /* backend failure; the context message has details */
  GA_INVALID_ERROR = 4,
  GA_UNSUPPORTED_ERROR = 5,
  GA_SYS_ERROR = 6,         /* errno has details */
  GA_RUN_ERROR = 7,
  GA_DEVSUP_ERROR = 8,
  GA_READONLY_ERROR = 9,
  GA_WRITEONLY_ERROR = 10,
  GA_BLAS_ERROR = 11,
  GA_UNALIGNED_ERROR = 12,
  GA_COPY_ERROR = 13,
  GA_NODEV_ERROR = 14,
  GA_MISC_ERROR = 15,
  GA_COMM_ERROR = 16,
  GA_XLARGE_ERROR = 17,
  GA_LOAD_ERROR = 18
};

/* Static description of an error code (never NULL). */
GPUARRAY_PUBLIC const char *gpuarray_error_str(int err);

#ifdef __cplusplus
}
#endif
#endif
