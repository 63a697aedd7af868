#include "common.h"
extern "C" size_t ga_gat_workspace_bytes(int64_t, int64_t, int64_t) { return 0; }
extern "C" int ga_gat_aggregate(const int32_t *, const int32_t *, const int32_t *, const float *, const float *, const void *, void *, int64_t, int64_t, int64_t, int64_t, float, int, void *, size_t, ga_stream_t) { return GA_EUNSUPPORTED; }
