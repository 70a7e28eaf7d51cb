/* Named backend hooks (ref src/gpuarray/extension.h:1-37,
 * src/gpuarray_extension.c:32-52).  The "hip" backend publishes the names
 * listed in gpuarray/ext_hip.h; unknown names give NULL. */
#ifndef GPUARRAY_EXTENSIONS_H
#define GPUARRAY_EXTENSIONS_H

#include <gpuarray/config.h>

#ifdef __cplusplus
extern "C" {
#endif

GPUARRAY_PUBLIC void *gpuarray_get_extension(const char *name);

#ifdef __cplusplus
}
#endif
#endif
