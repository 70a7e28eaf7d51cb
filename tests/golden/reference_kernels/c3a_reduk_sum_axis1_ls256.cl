
#include "cluda.h"



#define REDUCE(a, b) (a + b)

KERNEL void reduk(const unsigned int n, GLOBAL_MEM ga_float * out,
                    const unsigned int out_off
                    , const unsigned int dim0
                    , const unsigned int dim1
                    , GLOBAL_MEM ga_float * a_data
                    , const unsigned int a_offset
                    , const int a_str_0
                    , const int a_str_1
) {
  LOCAL_MEM ga_float ldata[256];
  const unsigned int lid = LID_0;
  unsigned int i;
  GLOBAL_MEM char *tmp;

  tmp = (GLOBAL_MEM char *)a_data; tmp += a_offset;
  a_data = (GLOBAL_MEM ga_float *)tmp;
  tmp = (GLOBAL_MEM char *)out; tmp += out_off;
  out = (GLOBAL_MEM ga_float *)tmp;

  i = GID_0;
  const unsigned int pos0 = i;

  ga_float acc = 0;

  for (i = lid; i < n; i += LDIM_0) {
    int ii = i;
    int pos;
        GLOBAL_MEM char *a_p = (GLOBAL_MEM char *)a_data;
        pos = ii % dim1;
        ii = ii / dim1;
        a_p += pos * a_str_1;
        a_p += pos0 * a_str_0;
    GLOBAL_MEM ga_float * a = (GLOBAL_MEM ga_float *)a_p;
    acc = REDUCE((acc), (a[0]));
  }
  ldata[lid] = acc;

    local_barrier();
    if (lid < 128) {
      ldata[lid] = REDUCE(ldata[lid], ldata[lid+128]);
    }
    local_barrier();
    if (lid < 64) {
      ldata[lid] = REDUCE(ldata[lid], ldata[lid+64]);
    }
    local_barrier();
    if (lid < 32) {
      ldata[lid] = REDUCE(ldata[lid], ldata[lid+32]);
    }
    local_barrier();
    if (lid < 16) {
      ldata[lid] = REDUCE(ldata[lid], ldata[lid+16]);
    }
    local_barrier();
    if (lid < 8) {
      ldata[lid] = REDUCE(ldata[lid], ldata[lid+8]);
    }
    local_barrier();
    if (lid < 4) {
      ldata[lid] = REDUCE(ldata[lid], ldata[lid+4]);
    }
    local_barrier();
    if (lid < 2) {
      ldata[lid] = REDUCE(ldata[lid], ldata[lid+2]);
    }
    local_barrier();
    if (lid < 1) {
      ldata[lid] = REDUCE(ldata[lid], ldata[lid+1]);
    }
  local_barrier();
  if (lid == 0) out[GID_0] = ldata[0];
}
