#include "cluda.h"

KERNEL void elem(const ga_size n, const ga_size dim0, const ga_size dim1, GLOBAL_MEM ga_float *a_data, const ga_size a_offset, const ga_ssize a_str_0, const ga_ssize a_str_1, GLOBAL_MEM ga_float *b_data, const ga_size b_offset, const ga_ssize b_str_0, const ga_ssize b_str_1, GLOBAL_MEM ga_float *c_data, const ga_size c_offset, const ga_ssize c_str_0, const ga_ssize c_str_1, GLOBAL_MEM ga_float *out_data, const ga_size out_offset, const ga_ssize out_str_0, const ga_ssize out_str_1) {
const ga_uint idx = LDIM_0 * GID_0 + LID_0;
const ga_uint numThreads = LDIM_0 * GDIM_0;
ga_uint i;
for(i = idx; i < n; i += numThreads) {
ga_uint ii = i;
ga_uint pos;
ga_uint a_p = a_offset;
ga_uint b_p = b_offset;
ga_uint c_p = c_offset;
ga_uint out_p = out_offset;
pos = ii % (ga_uint)dim1;
ii = ii / (ga_uint)dim1;
a_p += pos * (ga_int)a_str_1;
b_p += pos * (ga_int)b_str_1;
c_p += pos * (ga_int)c_str_1;
out_p += pos * (ga_int)out_str_1;
pos = ii;
a_p += pos * (ga_int)a_str_0;
b_p += pos * (ga_int)b_str_0;
c_p += pos * (ga_int)c_str_0;
out_p += pos * (ga_int)out_str_0;
ga_float a;a = *(GLOBAL_MEM ga_float *)(((GLOBAL_MEM char *)a_data) + a_p);
ga_float b;b = *(GLOBAL_MEM ga_float *)(((GLOBAL_MEM char *)b_data) + b_p);
ga_float c;c = *(GLOBAL_MEM ga_float *)(((GLOBAL_MEM char *)c_data) + c_p);
ga_float out;out = a + b*c;
*(GLOBAL_MEM ga_float *)(((GLOBAL_MEM char *)out_data) + out_p) = out;
}
}
