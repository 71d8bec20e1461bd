// top_k for 64-bit elements (double, int64): the kernels and host code of topk.hip, compiled as
// a translation unit of their own.
#define DLFX_TOPK_PART 1
#include "topk.hip"
