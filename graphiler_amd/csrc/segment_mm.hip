#include "common.h"
extern "C" int ga_segment_mm(const int32_t *, int64_t, const void *, const void *, void *, int64_t, int64_t, int64_t, int64_t, int, ga_stream_t) { return GA_EUNSUPPORTED; }
