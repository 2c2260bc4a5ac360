// The planned table-driven kernels (conv_planned.h): float16 instantiations (values held as half,
// computed in float; the backward over sender rows only, as half values have no float atomics).

#include "conv_planned.h"

namespace e3j_amd {

int launch_plan_build_f16(const e3j_amd_conv_params &p, const void *coef, bool cols_ji, int32_t *plan,
                          hipStream_t stream) {
    return launch_plan_build_t<half_t>(p, coef, cols_ji, plan, stream);
}

int launch_planned_fwd_f16(const e3j_amd_conv_params &p, const int32_t *plan, const void *x, const void *y,
                           const void *s, const int32_t *other, const int32_t *row_ptr, const int32_t *perm,
                           void *out, hipStream_t stream) {
    return launch_planned_fwd_t<half_t>(p, plan, x, y, s, other, row_ptr, perm, out, stream);
}

int launch_planned_bwd_f16(const e3j_amd_conv_params &p, bool group_is_receiver, const int32_t *plan, const void *x,
                           const void *y, const void *s, const void *dm, const int32_t *other,
                           const int32_t *row_ptr, const int32_t *perm, void *dx, void *dy, void *ds,
                           hipStream_t stream) {
    return launch_planned_bwd_t<half_t>(p, group_is_receiver, plan, x, y, s, dm, other, row_ptr, perm, dx, dy, ds,
                                        stream);
}

}  // namespace e3j_amd
