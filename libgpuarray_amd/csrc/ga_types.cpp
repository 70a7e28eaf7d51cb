// Type table: device spelling, size and alignment per typecode.
// Contents follow the reference's generated src/gpuarray_types.c:107-189
// (sizes are the device sizes: ga_long is 8 bytes, ga_longlong/ga_quad 16,
// vector types carry alignment 0) and the lookup rules of
// src/gpuarray_util.c:24-60 (GA_BUFFER row, no_type row for holes,
// user types from 512).
#include "private.hpp"

#include <mutex>
#include <vector>

namespace {

template <typename T> struct align_probe { char c; T x; };
#define ALIGN_OF(T) (sizeof(align_probe<T>) - sizeof(T))

struct q16 { uint64_t a, b; };            // 16-byte scalars (longlong, quad)
struct cf8 { float r, i; };               // complex float
struct cd16 { double r, i; };             // complex double
struct cq32 { q16 r, i; };                // complex quad

const gpuarray_type k_none = {nullptr, 0, 0, -1};
const gpuarray_type k_buffer = {nullptr, sizeof(GpuArray *), ALIGN_OF(GpuArray *),
                                GA_BUFFER};

const gpuarray_type k_scalar[GA_NBASE] = {
    {"ga_bool", 1, ALIGN_OF(uint8_t), GA_BOOL},
    {"ga_byte", 1, ALIGN_OF(int8_t), GA_BYTE},
    {"ga_ubyte", 1, ALIGN_OF(uint8_t), GA_UBYTE},
    {"ga_short", 2, ALIGN_OF(int16_t), GA_SHORT},
    {"ga_ushort", 2, ALIGN_OF(uint16_t), GA_USHORT},
    {"ga_int", 4, ALIGN_OF(int32_t), GA_INT},
    {"ga_uint", 4, ALIGN_OF(uint32_t), GA_UINT},
    {"ga_long", 8, ALIGN_OF(int64_t), GA_LONG},
    {"ga_ulong", 8, ALIGN_OF(uint64_t), GA_ULONG},
    {"ga_longlong", 16, ALIGN_OF(q16), GA_LONGLONG},
    {"ga_ulonglong", 16, ALIGN_OF(q16), GA_ULONGLONG},
    {"ga_float", 4, ALIGN_OF(float), GA_FLOAT},
    {"ga_double", 8, ALIGN_OF(double), GA_DOUBLE},
    {"ga_quad", 16, ALIGN_OF(q16), GA_QUAD},
    {"ga_cfloat", 8, ALIGN_OF(cf8), GA_CFLOAT},
    {"ga_cdouble", 16, ALIGN_OF(cd16), GA_CDOUBLE},
    {"ga_cquad", 32, ALIGN_OF(cq32), GA_CQUAD},
    {nullptr, 0, 0, -1}, {nullptr, 0, 0, -1}, {nullptr, 0, 0, -1},
    {nullptr, 0, 0, -1}, {nullptr, 0, 0, -1}, {nullptr, 0, 0, -1},
    {"ga_half", 2, ALIGN_OF(uint16_t), GA_HALF},
    {"ga_size", sizeof(size_t), ALIGN_OF(size_t), GA_SIZE},
    {"ga_ssize", sizeof(ssize_t), ALIGN_OF(ssize_t), GA_SSIZE},
};

// Vector rows are regular: base name, element size and lane counts.
struct vec_family { const char *base; size_t elsize; int first; int lanes[5]; int nl; bool paired; };
const vec_family k_families[] = {
    {"byte", 1, GA_BYTE2, {2, 3, 4, 8, 16}, 5, true},
    {"short", 2, GA_SHORT2, {2, 3, 4, 8, 16}, 5, true},
    {"int", 4, GA_INT2, {2, 3, 4, 8, 16}, 5, true},
    {"long", 8, GA_LONG2, {2, 3, 4, 8, 16}, 5, true},
    {"float", 4, GA_FLOAT2, {2, 4, 8, 16, 0}, 4, false},
    {"double", 8, GA_DOUBLE2, {2, 4, 8, 16, 0}, 4, false},
    {"half", 2, GA_HALF2, {2, 4, 8, 16, 0}, 4, false},
};

struct vec_table {
  gpuarray_type rows[GA_NVEC - 256];
  char names[GA_NVEC - 256][16];
  vec_table() {
    for (auto &r : rows) r = k_none;
    for (const auto &f : k_families) {
      int code = f.first;
      for (int l = 0; l < f.nl; l++) {
        int lanes = f.lanes[l];
        // integer families come as signed/unsigned pairs: ga_int4, ga_uint4
        for (int u = 0; u < (f.paired ? 2 : 1); u++, code++) {
          int idx = code - 256;
          snprintf(names[idx], sizeof(names[idx]), "ga_%s%s%d", u ? "u" : "",
                   f.base, lanes);
          rows[idx] = {names[idx], f.elsize * (size_t)lanes, 0, code};
        }
      }
    }
  }
};
const vec_table &vectors() { static const vec_table t; return t; }

std::mutex g_custom_mu;
std::vector<gpuarray_type *> g_custom;

}  // namespace

extern "C" int gpuarray_register_type(gpuarray_type *t, int *ret) {
  if (t == nullptr) {
    if (ret) *ret = GA_VALUE_ERROR;
    return -1;
  }
  std::lock_guard<std::mutex> lk(g_custom_mu);
  t->typecode = GA_ENDVEC + (int)g_custom.size();
  g_custom.push_back(t);
  return t->typecode;
}

extern "C" const gpuarray_type *gpuarray_get_type(int typecode) {
  if (typecode == GA_BUFFER) return &k_buffer;
  if (typecode < 0) return &k_none;
  if (typecode < GA_NBASE) return &k_scalar[typecode];
  if (typecode < 256) return &k_none;
  if (typecode < GA_NVEC) return &vectors().rows[typecode - 256];
  if (typecode < GA_ENDVEC) return &k_none;
  std::lock_guard<std::mutex> lk(g_custom_mu);
  size_t i = (size_t)(typecode - GA_ENDVEC);
  return i < g_custom.size() ? g_custom[i] : &k_none;
}

extern "C" size_t gpuarray_get_elsize(int typecode) {
  return gpuarray_get_type(typecode)->size;
}
