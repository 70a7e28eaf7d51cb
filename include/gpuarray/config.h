/* Build configuration visible to callers.
 * Mirrors the contract of the reference's src/gpuarray/config.h:1-43
 * (API version 2, GPUARRAY_PUBLIC export macro, fixed-width integer types,
 * ssize_t).  Linux/gfx950 only: there is no Windows branch here. */
#ifndef GPUARRAY_CONFIG
#define GPUARRAY_CONFIG

#include <gpuarray/abi_version.h>
#define GPUARRAY_API_VERSION 2

#if defined(GPUARRAY_SHARED) || defined(GPUARRAY_BUILDING_DLL)
#define GPUARRAY_PUBLIC __attribute__((visibility("default")))
#else
#define GPUARRAY_PUBLIC
#endif

#include <stddef.h>
#include <stdint.h>
#include <sys/types.h>

#endif
