#include "common.hip.h"
extern "C" size_t dlfx_top_k_scratch_bytes(int, int64_t, int64_t, int64_t) { return 0; }
extern "C" int dlfx_top_k(dlfx_stream_t, int64_t, int, int, int, int, const int64_t*, const int64_t*, const void*, int64_t, const int64_t*, void*, int64_t, const int64_t*, void*, int64_t, const int64_t*, void*, size_t) { return DLFX_ERR_UNKNOWN_OP; }
