// Shared declarations of the gfx950 convolution library (internal).
#ifndef E3J_AMD_CSRC_COMMON_H_
#define E3J_AMD_CSRC_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <string>
#include <vector>

#include "../../include/e3j_amd.h"

namespace e3j_amd {

constexpr int kWave = 64;  // gfx950 wavefront width

// Packed coefficient entry: the struct behind the opaque `coef` operand
// (field order and padding of lib/e3j_ops/cuda/convolution.cuh:31-44).
template <typename Idx, typename Val> struct CoefAlign;
template <> struct CoefAlign<uint8_t, float>  { static constexpr int value = 8; };
template <> struct CoefAlign<int32_t, float>  { static constexpr int value = 32; };
template <> struct CoefAlign<uint8_t, double> { static constexpr int value = 16; };
template <> struct CoefAlign<int32_t, double> { static constexpr int value = 32; };
typedef _Float16 half_t;  // float16 values: arithmetic in half precision
template <> struct CoefAlign<uint8_t, half_t>  { static constexpr int value = 8; };
template <> struct CoefAlign<int32_t, half_t>  { static constexpr int value = 32; };

template <typename Idx, typename Val>
struct alignas(CoefAlign<Idx, Val>::value) Coef4D {
    Val val;
    Idx i, j, k, l;
};
static_assert(sizeof(Coef4D<uint8_t, float>) == 8, "packed size");
static_assert(sizeof(Coef4D<int32_t, float>) == 32, "packed size");
static_assert(sizeof(Coef4D<uint8_t, double>) == 16, "packed size");
static_assert(sizeof(Coef4D<int32_t, double>) == 32, "packed size");
static_assert(sizeof(Coef4D<uint8_t, half_t>) == 8, "packed size");
static_assert(sizeof(Coef4D<int32_t, half_t>) == 32, "packed size");

// Sum over the 64 lanes of a wave (half values travel as float).
template <typename Val>
__device__ inline Val wave_sum(Val v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
template <>
__device__ inline half_t wave_sum<half_t>(half_t v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += (half_t)__shfl_xor((float)v, off, kWave);
    return v;
}
inline size_t val_bytes(int val_dtype) {
    return val_dtype == E3J_AMD_F64 ? 8 : val_dtype == E3J_AMD_F16 ? 2 : 4;
}

// Element strides of a (rows, dim, channels) operand in either layout.
struct RowLayout {
    int64_t row;   // elements between consecutive rows
    int32_t dim;   // stride of the irreps coordinate
    int32_t chan;  // stride of the channel
};

inline RowLayout make_layout(int layout, int dim, int channels) {
    RowLayout r;
    r.row = (int64_t)dim * channels;
    if (layout == E3J_AMD_LAYOUT_TRAILING) { r.dim = channels; r.chan = 1; }
    else                                   { r.dim = 1;        r.chan = dim; }
    return r;
}

// Error reporting ------------------------------------------------------
int set_error(int code, const std::string &msg);
int check_hip(hipError_t err, const char *what);

// Entry point shared by the C ABI and the XLA-FFI handlers.
int run_backward(const e3j_amd_conv_params *p, bool group_is_receiver, const void *coef,
                 const void *x, const void *y, const void *s, const void *dm,
                 const int32_t *other, const int32_t *row_ptr, const int32_t *edge_perm,
                 void *dx, void *dy, void *ds, hipStream_t stream, bool coef_cols_ji);

// Table-driven kernels (conv_generic.hip) ---------------------------------
int launch_generic_fwd(const e3j_amd_conv_params &p, const void *coef, const void *x, const void *y,
                       const void *s, const int32_t *other, const int32_t *row_ptr,
                       const int32_t *edge_perm, void *out, hipStream_t stream);
int launch_generic_bwd(const e3j_amd_conv_params &p, bool group_is_receiver, const void *coef,
                       const void *x, const void *y, const void *s, const void *dm,
                       const int32_t *other, const int32_t *row_ptr, const int32_t *edge_perm,
                       void *dx, void *dy, void *ds, hipStream_t stream,
                       bool coef_cols_ji = false);
int launch_fill_zero(void *ptr, size_t bytes, hipStream_t stream);
// Table-driven kernels over a plan of the table (conv_planned.hip): float32 tables within the
// plan's limits.  The plan is built on the device; its first word says whether the table could
// be taken, and the kernels with and without plan both look at it.
bool plan_takes(const e3j_amd_conv_params &p);
size_t plan_bytes(const e3j_amd_conv_params &p);
int launch_plan_build(const e3j_amd_conv_params &p, const void *coef, bool cols_ji, int32_t *plan,
                      hipStream_t stream);
int launch_planned_fwd(const e3j_amd_conv_params &p, const int32_t *plan, const void *x, const void *y,
                       const void *s, const int32_t *other, const int32_t *row_ptr, const int32_t *perm,
                       void *out, hipStream_t stream);
int launch_planned_bwd(const e3j_amd_conv_params &p, bool group_is_receiver, const int32_t *plan, const void *x,
                       const void *y, const void *s, const void *dm, const int32_t *other,
                       const int32_t *row_ptr, const int32_t *perm, void *dx, void *dy, void *ds,
                       hipStream_t stream);
std::atomic<int> &table_plans();  // 1: plan the tables that can be planned (default); 0: never
// Zero the dy/ds rows of padding edges (float32 operands).
int launch_zero_padding(const e3j_amd_conv_params &p, const int32_t *other, const int32_t *row_ptr,
                        const int32_t *perm, float *dy, float *ds, hipStream_t stream);
int launch_zero_padding(const e3j_amd_conv_params &p, const int32_t *other, const int32_t *row_ptr,
                        const int32_t *perm, double *dy, double *ds, hipStream_t stream);
int launch_zero_padding(const e3j_amd_conv_params &p, const int32_t *other, const int32_t *row_ptr,
                        const int32_t *perm, half_t *dy, half_t *ds, hipStream_t stream);

// Launch-shape variants of the unrolled kernels, from E3J_AMD_FWD_VARIANT /
// E3J_AMD_BWD_VARIANT (read once; 0 = default).  For tuning runs.
// The two numbers are read by every launch and may be set from another thread: relaxed atomics
// (a launch sees the old or the new shape, never a torn value).
struct Tuning {
    std::atomic<int> fwd_variant{0};
    std::atomic<int> bwd_variant{0};
};
const Tuning &tuning();

// Atomic-free backward of the unrolled kernels: instead of float atomics, a wave stores the dx
// contribution of every CSR position as one row of `u` and, when several waves share an
// edge, its dy sums into slot (position, wave) of `dy_slots`; fixed-order reductions follow
// (`reduce_ordered_dx`, `reduce_ordered_dy`).  The launcher fills in `slots` and `covered`.
constexpr int kMaxDySlots = 16;
// upper bound for a channel count: at most four parts times the 64-channel slices
inline int max_dy_slots(int channels) {
    const int slots = 4 * ((channels + 63) / 64);
    return slots < kMaxDySlots ? slots : kMaxDySlots;
}
struct OrderedBwd {
    float *u;                 // (num_edges, X * K)
    float *dy_slots;          // (num_edges, slots, Y)
    int slots;                // waves per edge of the launched variant (1: dy written directly)
    unsigned long long covered;  // x coordinates some coefficient touches (bit per coordinate)
};
// keys[pos] = other[pos] for the positions the kernels visit (inside a CSR row, endpoint in
// range), INT32_MAX otherwise (graph.hip).
int launch_live_keys(const int32_t *other, const int32_t *row_ptr, int32_t num_nodes,
                     int64_t num_edges, int32_t *keys, hipStream_t stream);
// rows[pos] = CSR row of every position (INT32_MAX past the last row); out[i] = inner[outer[i]]
// (inner null: identity) (graph.hip).
int launch_expand_rows(const int32_t *row_ptr, int32_t num_nodes, int64_t num_edges, int32_t *rows,
                       hipStream_t stream);
int launch_compose_perm(const int32_t *outer, const int32_t *inner, int64_t n, int32_t *out, hipStream_t stream);
int reduce_ordered_dx(const e3j_amd_conv_params &p, const float *u, const int32_t *sender_ptr,
                      const int32_t *sender_pos, unsigned long long covered, float *dx,
                      hipStream_t stream);
int reduce_ordered_dy(const e3j_amd_conv_params &p, const float *dy_slots, int slots,
                      const int32_t *perm, float *dy, hipStream_t stream);

// Compile-time-unrolled kernels (generated, sig_*.hip) ----------------------
struct Signature {
    const char *name;
    int32_t num_x, num_y, num_out, num_scalars, num_coef;
    int32_t channels;  // channel count the kernels were built for
    int32_t layout;
    const float *val;      // (num_coef) forward table, as float32
    const uint8_t *idx;    // (num_coef, 4) i, j, k, l
    int (*fwd)(const e3j_amd_conv_params &p, const float *x, const float *y, const float *s,
               const int32_t *sender, const int32_t *receiver_ptr, const int32_t *edge_perm,
               float *out, hipStream_t stream);
    int (*bwd)(const e3j_amd_conv_params &p, const float *x, const float *y, const float *s,
               const float *dm, const int32_t *sender, const int32_t *receiver_ptr,
               const int32_t *edge_perm, float *dx, float *dy, float *ds, hipStream_t stream,
               OrderedBwd *ordered);  // ordered: nullptr = dx (and shared dy) by float atomics
    // backward over tiles of receivers (nullptr: none) and the LDS bytes it needs per tile row
    int (*bwd_tiled)(const e3j_amd_conv_params &p, const float *x, const float *y, const float *s,
                     const float *dm, const e3j_amd_tile_schedule &schedule, float *dx, float *dy,
                     float *ds, hipStream_t stream);
    int (*tile_row_bytes)();
    int (*tile_rows_default)();  // receivers per tile the launch variant is tuned for
    // backward on the sender-grouped adjacency (receiver per position, row pointer by sender): dx
    // owned by the rows, no atomics on it (nullptr: none, the table-driven kernel serves that grouping)
    int (*bwd_sender)(const e3j_amd_conv_params &p, const float *x, const float *y, const float *s,
                      const float *dm, const int32_t *receiver_t, const int32_t *sender_ptr,
                      const int32_t *edge_perm, float *dx, float *dy, float *ds, hipStream_t stream);
    // float64 kernels (trailing layout, receiver rows; nullptr: none).  They read one coefficient
    // per class of entries of equal magnitude from e3j_amd_conv_params.coef_classes: coef_class
    // (num_coef) names the class of every entry, num_classes <= kF64Classes.
    int32_t num_classes;
    const uint8_t *coef_class;
    int (*fwd_f64)(const e3j_amd_conv_params &p, const double *x, const double *y, const double *s,
                   const int32_t *sender, const int32_t *receiver_ptr, const int32_t *edge_perm, double *out,
                   hipStream_t stream);
    int (*bwd_f64)(const e3j_amd_conv_params &p, const double *x, const double *y, const double *s,
                   const double *dm, const int32_t *sender, const int32_t *receiver_ptr,
                   const int32_t *edge_perm, double *dx, double *dy, double *ds, hipStream_t stream);
    // float16 kernels (trailing layout, receiver rows; nullptr: none): values held as half, the float
    // kernels' arithmetic, literals and scale factor
    int (*fwd_f16)(const e3j_amd_conv_params &p, const half_t *x, const half_t *y, const half_t *s,
                   const int32_t *sender, const int32_t *receiver_ptr, const int32_t *edge_perm, half_t *out,
                   hipStream_t stream);
    int (*bwd_f16)(const e3j_amd_conv_params &p, const half_t *x, const half_t *y, const half_t *s,
                   const half_t *dm, const int32_t *sender, const int32_t *receiver_ptr,
                   const int32_t *edge_perm, half_t *dx, half_t *dy, half_t *ds, hipStream_t stream);
};
// the coefficient classes of a float64 launch, passed to the kernel by value
constexpr int kF64Classes = E3J_AMD_F64_CLASSES;
struct F64Coefs {
    double v[kF64Classes];
};
// built-in signatures (generated/registry.hip), then the ones registered at run time (capi.hip)
// A table entry on the host, and the lookup of a table among the signatures (capi.hip): the
// tables are compared as sets of entries, up to one positive factor and one sign per y component.
struct TableEntry {
    float val;
    int32_t idx[4];  // i, j, k, l
};
std::vector<TableEntry> unpack_entries(const void *packed_host, int32_t coef_idx_bytes, int32_t num_coef,
                                       bool columns_ji);
int match_signature(std::vector<TableEntry> entries, int32_t num_x, int32_t num_y, int32_t num_out,
                    int32_t num_scalars, int32_t channels, int32_t layout, float *coef_scale,
                    uint32_t *y_flip, double tolerance = 4e-7, bool float16_kernels = false);
// the same for tables of half values (float16 kernels) and of double values (float64 kernels: the
// table's own magnitudes per class of the signature's entries into coef_classes[kF64Classes])
int match_signature_f16(const void *coef_host, int32_t coef_idx_bytes, int32_t num_coef, int32_t num_x,
                        int32_t num_y, int32_t num_out, int32_t num_scalars, int32_t channels, int32_t layout,
                        bool columns_ji, float *coef_scale, uint32_t *y_flip);
int match_signature_f64(const void *coef_host, int32_t coef_idx_bytes, int32_t num_coef, int32_t num_x,
                        int32_t num_y, int32_t num_out, int32_t num_scalars, int32_t channels, int32_t layout,
                        bool columns_ji, double *coef_classes, uint32_t *y_flip);
int num_builtin_signatures();
const Signature &builtin_signature(int id);
int num_signatures();
const Signature &signature(int id);

}  // namespace e3j_amd
#endif
