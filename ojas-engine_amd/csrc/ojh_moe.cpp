// MoE op seam: router and grouped expert FFN.
#include "ojh_internal.h"

extern "C" int ojh_moe_route(ojh_device *, const ojh_buf *, uint32_t, uint32_t, uint32_t, ojh_buf *, ojh_buf *) {
    return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_moe_route: not built yet");
}

extern "C" int ojh_moe_ffn(ojh_device *, const ojh_buf *, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t,
                           const ojh_buf *, const ojh_buf *, const ojh_lin *, const ojh_lin *, const ojh_lin *,
                           ojh_buf *, int, int) {
    return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_moe_ffn: not built yet");
}
