// Temporary: chunked backward entry points not built yet.
#include "common.h"
extern "C" int mrx_linear_attn_bwd(void *, const void *, const void *, const void *, const void *, const void *, const void *, const void *, void *, void *, void *, void *, int64_t, int64_t, int64_t, int64_t, int64_t, int, int, int) { return MRX_ERR_UNSUPPORTED; }
extern "C" int mrx_delta_rule_bwd(void *, const void *, const void *, const void *, const void *, const void *, const void *, const void *, const void *, void *, void *, void *, void *, void *, int64_t, int64_t, int64_t, int64_t, int64_t, int, int) { return MRX_ERR_UNSUPPORTED; }
