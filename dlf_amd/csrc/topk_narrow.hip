// top_k for 16-bit elements (IEEE half, int16): the kernels and host code of topk.hip, compiled
// as a translation unit of their own.
#define DLFX_TOPK_PART 2
#include "topk.hip"
