#include "common.hip.h"
extern "C" size_t dlfx_sort_scratch_bytes(int, int64_t, int64_t) { return 0; }
extern "C" int dlfx_sort(dlfx_stream_t, int, int, int, const int64_t*, const void*, int64_t, const int64_t*, void*, int64_t, const int64_t*, void*, size_t) { return DLFX_ERR_UNKNOWN_OP; }
extern "C" size_t dlfx_argsort_scratch_bytes(int, int64_t, int64_t) { return 0; }
extern "C" int dlfx_argsort(dlfx_stream_t, int, int, int, int, const int64_t*, const void*, int64_t, const int64_t*, void*, int64_t, const int64_t*, void*, int64_t, const int64_t*, void*, size_t) { return DLFX_ERR_UNKNOWN_OP; }
