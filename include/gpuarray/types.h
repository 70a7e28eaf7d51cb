/* Element type codes.  The numbering is ABI and follows numpy's dtype.num on
 * LP64 Linux: reference src/gpuarray/types.h:45-131 (table in
 * src/gpuarray_types.c:107-189). */
#ifndef GPUARRAY_TYPES_H
#define GPUARRAY_TYPES_H

#include <gpuarray/config.h>

#ifdef __cplusplus
extern "C" {
#endif

/* One row of the type table: device-side spelling, byte size, alignment. */
typedef struct _gpuarray_type {
  const char *cluda_name;
  size_t size;
  size_t align;
  int typecode;
} gpuarray_type;

enum GPUARRAY_TYPES {
  GA_BUFFER = -1,
  GA_BOOL = 0, GA_BYTE = 1, GA_UBYTE = 2, GA_SHORT = 3, GA_USHORT = 4,
  GA_INT = 5, GA_UINT = 6, GA_LONG = 7, GA_ULONG = 8,
  GA_LONGLONG = 9, GA_ULONGLONG = 10,
  GA_FLOAT = 11, GA_DOUBLE = 12, GA_QUAD = 13,
  GA_CFLOAT = 14, GA_CDOUBLE = 15, GA_CQUAD = 16,
  /* 17..22 are holes kept for numpy compatibility */
  GA_HALF = 23, GA_SIZE = 24, GA_SSIZE = 25,
  GA_NBASE = 26,

  GA_DELIM = 255,

  /* short vector types, 256.. */
  GA_BYTE2 = 256, GA_UBYTE2 = 257, GA_BYTE3 = 258, GA_UBYTE3 = 259,
  GA_BYTE4 = 260, GA_UBYTE4 = 261, GA_BYTE8 = 262, GA_UBYTE8 = 263,
  GA_BYTE16 = 264, GA_UBYTE16 = 265,
  GA_SHORT2 = 266, GA_USHORT2 = 267, GA_SHORT3 = 268, GA_USHORT3 = 269,
  GA_SHORT4 = 270, GA_USHORT4 = 271, GA_SHORT8 = 272, GA_USHORT8 = 273,
  GA_SHORT16 = 274, GA_USHORT16 = 275,
  GA_INT2 = 276, GA_UINT2 = 277, GA_INT3 = 278, GA_UINT3 = 279,
  GA_INT4 = 280, GA_UINT4 = 281, GA_INT8 = 282, GA_UINT8 = 283,
  GA_INT16 = 284, GA_UINT16 = 285,
  GA_LONG2 = 286, GA_ULONG2 = 287, GA_LONG3 = 288, GA_ULONG3 = 289,
  GA_LONG4 = 290, GA_ULONG4 = 291, GA_LONG8 = 292, GA_ULONG8 = 293,
  GA_LONG16 = 294, GA_ULONG16 = 295,
  GA_FLOAT2 = 296, GA_FLOAT4 = 297, GA_FLOAT8 = 298, GA_FLOAT16 = 299,
  GA_DOUBLE2 = 300, GA_DOUBLE4 = 301, GA_DOUBLE8 = 302, GA_DOUBLE16 = 303,
  GA_HALF2 = 304, GA_HALF4 = 305, GA_HALF8 = 306, GA_HALF16 = 307,
  GA_NVEC = 308,

  GA_ENDVEC = 512   /* user-registered types start here */
};

#ifdef __cplusplus
}
#endif
#endif
