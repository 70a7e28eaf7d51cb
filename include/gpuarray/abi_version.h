/* ABI number of the shared library: 1000*major + minor.
 * The reference writes this file from its build (src/CMakeLists.txt:118-127,
 * library VERSION 3.0 at :110); the replacement keeps the same number so
 * callers that test GPUARRAY_ABI_VERSION keep working. */
#ifndef GPUARRAY_ABI_VERSION
#define GPUARRAY_ABI_VERSION 3000
#endif
