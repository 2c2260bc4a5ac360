// The planned table-driven kernels (conv_planned.h): float32 instantiations and the entry points
// the rest of the library calls.

#include "conv_planned.h"

namespace e3j_amd {

bool plan_takes(const e3j_amd_conv_params &p) {
    return (p.val_dtype == E3J_AMD_F32 || p.val_dtype == E3J_AMD_F16) && plan_sizes_fit(p);
}

size_t plan_bytes(const e3j_amd_conv_params &p) { return sizeof(int32_t) * plan_words(p); }

int launch_plan_build(const e3j_amd_conv_params &p, const void *coef, bool cols_ji, int32_t *plan,
                      hipStream_t stream) {
    return p.val_dtype == E3J_AMD_F16 ? launch_plan_build_f16(p, coef, cols_ji, plan, stream)
                                      : launch_plan_build_t<float>(p, coef, cols_ji, plan, stream);
}

int launch_planned_fwd(const e3j_amd_conv_params &p, const int32_t *plan, const void *x, const void *y,
                       const void *s, const int32_t *other, const int32_t *row_ptr, const int32_t *perm,
                       void *out, hipStream_t stream) {
    return p.val_dtype == E3J_AMD_F16
               ? launch_planned_fwd_f16(p, plan, x, y, s, other, row_ptr, perm, out, stream)
               : launch_planned_fwd_t<float>(p, plan, x, y, s, other, row_ptr, perm, out, stream);
}

int launch_planned_bwd(const e3j_amd_conv_params &p, bool group_is_receiver, const int32_t *plan, const void *x,
                       const void *y, const void *s, const void *dm, const int32_t *other,
                       const int32_t *row_ptr, const int32_t *perm, void *dx, void *dy, void *ds,
                       hipStream_t stream) {
    return p.val_dtype == E3J_AMD_F16
               ? launch_planned_bwd_f16(p, group_is_receiver, plan, x, y, s, dm, other, row_ptr, perm, dx, dy, ds,
                                        stream)
               : launch_planned_bwd_t<float>(p, group_is_receiver, plan, x, y, s, dm, other, row_ptr, perm, dx, dy,
                                             ds, stream);
}

}  // namespace e3j_amd

extern "C" int e3j_amd_table_plan_status(const e3j_amd_conv_params *p, const void *coef, int32_t coef_cols_ji,
                                         int32_t *status, void *stream_) {
    using namespace e3j_amd;
    if (p == nullptr || status == nullptr || (coef == nullptr && p->num_coef > 0))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "table_plan_status: null operand");
    status[0] = status[1] = status[2] = status[3] = 0;
    if (!plan_takes(*p)) return E3J_AMD_OK;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    void *mem = p->table_plan;  // the caller's memory: the plan is built there and stays
    const bool own = mem == nullptr;
    int rc = E3J_AMD_OK;
    if (own) rc = check_hip(hipMalloc(&mem, plan_bytes(*p)), "table_plan_status: hipMalloc");
    else if (reinterpret_cast<uintptr_t>(mem) % alignof(int32_t) != 0)
        rc = set_error(E3J_AMD_INVALID_ARGUMENT, "table_plan_status: table_plan must be 4-byte aligned");
    if (rc) return rc;
    rc = launch_plan_build(*p, coef, coef_cols_ji != 0, static_cast<int32_t *>(mem), stream);
    int32_t header[kHeaderWords] = {0};
    if (!rc) rc = check_hip(hipMemcpyAsync(header, mem, sizeof(header), hipMemcpyDeviceToHost, stream),
                            "table_plan_status: copy");
    if (!rc) rc = check_hip(hipStreamSynchronize(stream), "table_plan_status: synchronize");
    if (own) (void)hipFree(mem);
    if (rc) return rc;
    status[0] = header[kEligible];
    status[1] = header[kNumCells];
    status[2] = __builtin_popcount((unsigned)header[kChunkMask]);
    status[3] = header[kNumZeroL];
    return E3J_AMD_OK;
}

extern "C" size_t e3j_amd_table_plan_bytes(const e3j_amd_conv_params *p) {
    using namespace e3j_amd;
    return (p != nullptr && plan_takes(*p)) ? plan_bytes(*p) : 0;
}
