#include "common.h"
extern "C" {
int ptj_attn_fwd(const void*, const void*, const void*, const uint8_t*, void*, float*, float*, int64_t, int64_t,
                 int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int, int64_t,
                 int, void*) { return ptj_set_error(PTJ_ERR_INVALID, "attn_fwd: not built yet"); }
int ptj_attn_bwd(const void*, const void*, const void*, const void*, const void*, const float*, const float*,
                 const uint8_t*, void*, void*, void*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,
                 int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,
                 int64_t, int64_t, int, int64_t, int, void*) { return ptj_set_error(PTJ_ERR_INVALID, "attn_bwd: not built yet"); }
}
