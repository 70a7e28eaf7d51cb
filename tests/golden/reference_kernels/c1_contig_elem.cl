#include "cluda.h"

KERNEL void elem(const ga_size n, GLOBAL_MEM ga_float *a_p,  const ga_size a_offset, GLOBAL_MEM ga_float *b_p,  const ga_size b_offset, GLOBAL_MEM ga_float *c_p,  const ga_size c_offset) {
const ga_size idx = LDIM_0 * GID_0 + LID_0;
const ga_size numThreads = LDIM_0 * GDIM_0;
ga_size i;
GLOBAL_MEM char *tmp;

tmp = (GLOBAL_MEM char *)a_p;tmp += a_offset; a_p = (GLOBAL_MEM ga_float *)tmp;tmp = (GLOBAL_MEM char *)b_p;tmp += b_offset; b_p = (GLOBAL_MEM ga_float *)tmp;tmp = (GLOBAL_MEM char *)c_p;tmp += c_offset; c_p = (GLOBAL_MEM ga_float *)tmp;for (i = idx; i < n; i += numThreads) {
ga_float a;
a = a_p[i];
ga_float b;
b = b_p[i];
ga_float c;
c = a*b + 0.5f;
c_p[i] = c;
}
}
