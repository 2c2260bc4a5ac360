// C-ABI entry points: argument validation, kernel selection, error reporting.

#include <cmath>
#include <cstdlib>
#include <cstring>

#include <cstdint>
#include <deque>
#include <initializer_list>
#include <algorithm>
#include <mutex>
#include <vector>

#include "common.h"
#include "tuning_api.h"
#include "row_pieces.h"

namespace e3j_amd {

static thread_local std::string g_last_error;

int set_error(int code, const std::string &msg) {
    const char *cls = code == E3J_AMD_INVALID_ARGUMENT ? "InvalidArgument"
                    : code == E3J_AMD_UNIMPLEMENTED    ? "Unimplemented"
                                                       : "Internal";
    g_last_error = std::string("E3J_AMD_ERROR[") + cls + "]: " + msg;
    return code;
}

int check_hip(hipError_t err, const char *what) {
    if (err == hipSuccess) return E3J_AMD_OK;
    return set_error(E3J_AMD_INTERNAL, std::string(what) + ": " + hipGetErrorString(err));
}

namespace {
Tuning &mutable_tuning() {
    static Tuning t;
    static const bool from_environment = [] {
        if (const char *e = std::getenv("E3J_AMD_FWD_VARIANT")) t.fwd_variant.store(std::atoi(e));
        if (const char *e = std::getenv("E3J_AMD_BWD_VARIANT")) t.bwd_variant.store(std::atoi(e));
        return true;
    }();
    (void)from_environment;
    return t;
}
}  // namespace

const Tuning &tuning() { return mutable_tuning(); }

std::atomic<int> &table_plans() {
    static std::atomic<int> on{[] {
        const char *e = std::getenv("E3J_AMD_TABLE_PLANS");
        return e == nullptr || std::atoi(e) != 0 ? 1 : 0;
    }()};
    return on;
}

// Signatures registered at run time live behind the built-in ones.  The list only grows and
// a deque never moves its elements, so ids and references stay valid.
namespace {
std::mutex g_registry_mutex;
std::deque<const Signature *> g_registered;
}  // namespace

int num_signatures() {
    std::lock_guard<std::mutex> lock(g_registry_mutex);
    return num_builtin_signatures() + (int)g_registered.size();
}

const Signature &signature(int id) {
    if (id < num_builtin_signatures()) return builtin_signature(id);
    std::lock_guard<std::mutex> lock(g_registry_mutex);
    return *g_registered[id - num_builtin_signatures()];
}

namespace {

int validate(const e3j_amd_conv_params *p, const char *op) {
    const std::string name(op);
    if (p == nullptr) return set_error(E3J_AMD_INVALID_ARGUMENT, name + ": null params");
    if (p->num_nodes < 0 || p->num_edges < 0 || p->num_coef < 0)
        return set_error(E3J_AMD_INVALID_ARGUMENT, name + ": negative size");
    if (p->num_x < 1 || p->num_y < 1 || p->num_out < 1 || p->num_scalars < 1 || p->channels < 1)
        return set_error(E3J_AMD_INVALID_ARGUMENT,
                         name + ": num_x, num_y, num_out, num_scalars and channels must be >= 1");
    if (p->layout != E3J_AMD_LAYOUT_LEADING && p->layout != E3J_AMD_LAYOUT_TRAILING)
        return set_error(E3J_AMD_INVALID_ARGUMENT, name + ": unknown layout " + std::to_string(p->layout));
    if (p->val_dtype != E3J_AMD_F32 && p->val_dtype != E3J_AMD_F64 && p->val_dtype != E3J_AMD_F16)
        return set_error(E3J_AMD_INVALID_ARGUMENT, name + ": unsupported (IDX, VAL) dtype pair");
    if (p->coef_idx_bytes != 1 && p->coef_idx_bytes != 4)
        return set_error(E3J_AMD_INVALID_ARGUMENT, name + ": unsupported (IDX, VAL) dtype pair");
    if (p->num_edges > 0x7fffffffLL)
        return set_error(E3J_AMD_INVALID_ARGUMENT, name + ": edge positions are int32");
    if (p->signature >= num_signatures())
        return set_error(E3J_AMD_INVALID_ARGUMENT,
                         name + ": unknown signature id " + std::to_string(p->signature));
    if (p->signature < 0 && p->y_flip != 0)
        return set_error(E3J_AMD_INVALID_ARGUMENT,
                         name + ": y_flip needs an unrolled kernel (the table-driven kernels take "
                                "the signs in the table)");
    if (p->signature >= 0) {
        const Signature &sg = signature(p->signature);
        const bool dtype_served = p->val_dtype == E3J_AMD_F32 ||
                                  (p->val_dtype == E3J_AMD_F64 && sg.fwd_f64 != nullptr && sg.bwd_f64 != nullptr) ||
                                  (p->val_dtype == E3J_AMD_F16 && sg.fwd_f16 != nullptr && sg.bwd_f16 != nullptr);
        if (!dtype_served || sg.num_x != p->num_x || sg.num_y != p->num_y ||
            sg.num_out != p->num_out || sg.num_scalars != p->num_scalars ||
            sg.channels != p->channels || sg.layout != p->layout)
            return set_error(E3J_AMD_INVALID_ARGUMENT,
                             name + ": operand shapes or value dtype do not match signature " + sg.name);
        if (p->val_dtype == E3J_AMD_F64 && p->coef_classes == nullptr)
            return set_error(E3J_AMD_INVALID_ARGUMENT,
                             name + ": float64 operands on an unrolled kernel need coef_classes "
                                    "(e3j_amd_find_signature_f64)");
    }
    return E3J_AMD_OK;
}

bool missing(const void *ptr, int64_t count) { return count > 0 && ptr == nullptr; }

// The unrolled kernels move rows in pieces of up to 16 bytes (whole blocks in the leading layout,
// several channels per lane and the fixed-order dx reduction in the trailing one): operands that
// are not 16-byte aligned (a view at an odd element offset) take the table-driven kernels.
bool aligned16(std::initializer_list<const void *> ptrs) {
    for (const void *ptr : ptrs)
        if (reinterpret_cast<uintptr_t>(ptr) % 16 != 0) return false;
    return true;
}
bool signature_fits(const e3j_amd_conv_params *p, std::initializer_list<const void *> ptrs) {
    return p->signature >= 0 && p->val_dtype == E3J_AMD_F32 && aligned16(ptrs);
}
// float64 operands on the float64 kernels of a signature (validate() has checked that they exist);
// rows are moved as 8-byte elements, so any float64 array is aligned enough
bool signature_fits_f64(const e3j_amd_conv_params *p) {
    return p->signature >= 0 && p->val_dtype == E3J_AMD_F64;
}
bool signature_fits_f16(const e3j_amd_conv_params *p) {
    return p->signature >= 0 && p->val_dtype == E3J_AMD_F16;
}
int f64_receiver_rows_only(const char *op) {
    return set_error(E3J_AMD_UNIMPLEMENTED,
                     std::string(op) + ": the float64 and float16 unrolled kernels serve the forward pass and the "
                                       "receiver-grouped backward; pass signature = -1 for the table-driven kernel");
}
// Falling back to the table-driven kernel is only right when no sign flip was asked for.
int flip_without_kernel(const e3j_amd_conv_params *p, const char *op) {
    if (p->y_flip == 0) return E3J_AMD_OK;
    return set_error(E3J_AMD_INVALID_ARGUMENT,
                     std::string(op) + ": y_flip needs the unrolled kernel, which these operands "
                                       "(alignment or grouping) cannot use");
}

int finish(const e3j_amd_conv_params *p, hipStream_t stream, int rc, const char *op) {
    if (rc != E3J_AMD_OK || p->debug <= 0) return rc;
    return check_hip(hipStreamSynchronize(stream), op);
}

}  // namespace

int run_backward(const e3j_amd_conv_params *p, bool group_is_receiver, const void *coef,
                 const void *x, const void *y, const void *s, const void *dm,
                 const int32_t *other, const int32_t *row_ptr, const int32_t *edge_perm,
                 void *dx, void *dy, void *ds, hipStream_t stream, bool coef_cols_ji) {
    const char *op = group_is_receiver ? "convolution_bwd_receiver" : "convolution_bwd";
    int rc = validate(p, op);
    if (rc) return rc;
    if (p->num_nodes == 0 && p->num_edges == 0) return E3J_AMD_OK;
    if (missing(x, p->num_nodes) || missing(dm, p->num_nodes) || missing(dx, p->num_nodes) ||
        row_ptr == nullptr || missing(other, p->num_edges) || missing(y, p->num_edges) ||
        missing(s, p->num_edges) || missing(dy, p->num_edges) || missing(ds, p->num_edges) ||
        (p->signature < 0 && missing(coef, p->num_coef)))
        return set_error(E3J_AMD_INVALID_ARGUMENT, std::string(op) + ": null operand");
    if (p->num_nodes == 0) return E3J_AMD_OK;
    if (signature_fits_f64(p)) {
        if (!group_is_receiver) return f64_receiver_rows_only(op);
        rc = signature(p->signature).bwd_f64(*p, static_cast<const double *>(x), static_cast<const double *>(y),
                                             static_cast<const double *>(s), static_cast<const double *>(dm),
                                             other, row_ptr, edge_perm, static_cast<double *>(dx),
                                             static_cast<double *>(dy), static_cast<double *>(ds), stream);
        if (rc == E3J_AMD_OK)
            rc = launch_zero_padding(*p, other, row_ptr, edge_perm, static_cast<double *>(dy),
                                     static_cast<double *>(ds), stream);
    } else if (signature_fits_f16(p)) {
        if (!group_is_receiver) return f64_receiver_rows_only(op);
        rc = signature(p->signature).bwd_f16(*p, static_cast<const half_t *>(x), static_cast<const half_t *>(y),
                                             static_cast<const half_t *>(s), static_cast<const half_t *>(dm),
                                             other, row_ptr, edge_perm, static_cast<half_t *>(dx),
                                             static_cast<half_t *>(dy), static_cast<half_t *>(ds), stream);
        if (rc == E3J_AMD_OK)
            rc = launch_zero_padding(*p, other, row_ptr, edge_perm, static_cast<half_t *>(dy),
                                     static_cast<half_t *>(ds), stream);
    } else if (group_is_receiver && signature_fits(p, {x, s, dm, dx, ds}) &&
        signature(p->signature).bwd != nullptr) {
        rc = signature(p->signature).bwd(*p, static_cast<const float *>(x),
                                         static_cast<const float *>(y), static_cast<const float *>(s),
                                         static_cast<const float *>(dm), other, row_ptr, edge_perm,
                                         static_cast<float *>(dx), static_cast<float *>(dy),
                                         static_cast<float *>(ds), stream, nullptr);
        if (rc == E3J_AMD_OK)
            rc = launch_zero_padding(*p, other, row_ptr, edge_perm, static_cast<float *>(dy),
                                     static_cast<float *>(ds), stream);
    } else if (!group_is_receiver && p->layout == E3J_AMD_LAYOUT_TRAILING && signature_fits(p, {x, s, dm, dx, ds}) &&
               signature(p->signature).bwd_sender != nullptr) {
        // the reference's grouping on the unrolled kernels: rows own their dx (no atomics)
        rc = signature(p->signature).bwd_sender(*p, static_cast<const float *>(x), static_cast<const float *>(y),
                                                static_cast<const float *>(s), static_cast<const float *>(dm),
                                                other, row_ptr, edge_perm, static_cast<float *>(dx),
                                                static_cast<float *>(dy), static_cast<float *>(ds), stream);
        if (rc == E3J_AMD_OK)
            rc = launch_zero_padding(*p, other, row_ptr, edge_perm, static_cast<float *>(dy),
                                     static_cast<float *>(ds), stream);
    } else {
        if ((rc = flip_without_kernel(p, op))) return rc;
        if (coef == nullptr && p->num_coef > 0)
            return set_error(E3J_AMD_INVALID_ARGUMENT,
                             std::string(op) + ": this grouping runs the table-driven kernel and needs `coef`");
        rc = launch_generic_bwd(*p, group_is_receiver, coef, x, y, s, dm, other, row_ptr, edge_perm,
                                dx, dy, ds, stream, coef_cols_ji);
    }
    return finish(p, stream, rc, op);
}

// ---- table lookup ---------------------------------------------------------------------------
std::vector<TableEntry> unpack_entries(const void *packed, int32_t coef_idx_bytes, int32_t num_coef,
                                       bool columns_ji) {
    const size_t item = coef_idx_bytes == 1 ? sizeof(Coef4D<uint8_t, float>) : sizeof(Coef4D<int32_t, float>);
    const unsigned char *bytes = static_cast<const unsigned char *>(packed);
    std::vector<TableEntry> entries((size_t)num_coef);
    for (int n = 0; n < num_coef; n++) {
        TableEntry &e = entries[n];
        std::memcpy(&e.val, bytes + n * item, sizeof(float));
        for (int t = 0; t < 4; t++) {
            if (coef_idx_bytes == 1) e.idx[t] = bytes[n * item + 4 + t];
            else std::memcpy(&e.idx[t], bytes + n * item + 4 + 4 * t, 4);
        }
        if (columns_ji) std::swap(e.idx[0], e.idx[1]);  // (j, i, k, l) of a dx table -> (i, j, k, l)
    }
    return entries;
}

namespace {
bool entry_less(const TableEntry &a, const TableEntry &b) {
    for (int t = 0; t < 4; t++)
        if (a.idx[t] != b.idx[t]) return a.idx[t] < b.idx[t];
    return false;
}
}  // namespace

// The tables are compared as sets of entries (both sorted by their coordinates): the reference
// permutes the rows of a table when it balances them over warps (src/e3j/ops/convolution.py:178-208).
int match_signature(std::vector<TableEntry> entries, int32_t num_x, int32_t num_y, int32_t num_out,
                    int32_t num_scalars, int32_t channels, int32_t layout, float *coef_scale,
                    uint32_t *y_flip, double tolerance, bool float16_kernels) {
    if (coef_scale) *coef_scale = 1.0f;
    if (y_flip) *y_flip = 0;
    const int num_coef = (int)entries.size();
    if (num_coef == 0) return -1;
    std::stable_sort(entries.begin(), entries.end(), entry_less);
    const bool signs_allowed = y_flip != nullptr && num_y <= 32;
    std::vector<TableEntry> own((size_t)num_coef);
    for (int id = 0; id < num_signatures(); id++) {
        const Signature &sg = signature(id);
        if (sg.num_coef != num_coef || sg.num_x != num_x || sg.num_y != num_y ||
            sg.num_out != num_out || sg.num_scalars != num_scalars || sg.channels != channels ||
            sg.layout != layout)
            continue;
        if (float16_kernels && (sg.fwd_f16 == nullptr || sg.bwd_f16 == nullptr)) continue;
        for (int n = 0; n < num_coef; n++) {
            own[n].val = sg.val[n];
            for (int t = 0; t < 4; t++) own[n].idx[t] = sg.idx[4 * n + t];
        }
        std::stable_sort(own.begin(), own.end(), entry_less);
        // One uniform positive factor is allowed between the tables; its magnitude is taken
        // from the entry of largest magnitude and every entry must agree to float32 rounding.
        // A negative ratio is a sign flip of that entry's y component, which must then hold
        // for every entry of the component.
        int big = 0;
        for (int n = 1; n < num_coef; n++)
            if (std::fabs(own[n].val) > std::fabs(own[big].val)) big = n;
        const double scale = std::fabs((double)entries[big].val / (double)own[big].val);
        bool same = scale > 0.0 && std::isfinite(scale);
        uint32_t flip = 0, seen = 0;
        for (int n = 0; n < num_coef && same; n++) {
            const int32_t *idx = entries[n].idx;
            for (int t = 0; t < 4 && same; t++) same = idx[t] == own[n].idx[t];
            if (!same) break;
            const double v = entries[n].val, want = scale * (double)own[n].val;
            const bool plus = std::fabs(v - want) <= tolerance * std::fabs(want);
            const bool minus = std::fabs(v + want) <= tolerance * std::fabs(want);
            if (plus) {
                same = !signs_allowed || !((seen >> idx[2]) & 1u) || !((flip >> idx[2]) & 1u);
            } else if (minus && signs_allowed) {
                same = !((seen >> idx[2]) & 1u) || ((flip >> idx[2]) & 1u);
                flip |= 1u << idx[2];
            } else {
                same = false;
            }
            if (signs_allowed) seen |= 1u << idx[2];
        }
        if (same) {
            if (coef_scale) *coef_scale = (float)scale;
            if (y_flip) *y_flip = flip;
            return id;
        }
    }
    return -1;
}

}  // namespace e3j_amd

using namespace e3j_amd;

extern "C" {

const char *e3j_amd_last_error(void) { return g_last_error.c_str(); }

const char *e3j_amd_version(void) { return "e3j_amd 0.1 (gfx950)"; }

int e3j_amd_register_signature(const void *entry) {
    const Signature *sg = static_cast<const Signature *>(entry);
    if (sg == nullptr || sg->fwd == nullptr || sg->bwd == nullptr || sg->val == nullptr ||
        sg->idx == nullptr || sg->num_coef <= 0) {
        set_error(E3J_AMD_INVALID_ARGUMENT, "register_signature: incomplete entry");
        return -1;
    }
    std::lock_guard<std::mutex> lock(g_registry_mutex);
    g_registered.push_back(sg);
    return num_builtin_signatures() + (int)g_registered.size() - 1;
}

void e3j_amd_set_table_plans(int32_t on) { table_plans().store(on ? 1 : 0, std::memory_order_relaxed); }

void e3j_amd_set_launch_variant(int32_t fwd_variant, int32_t bwd_variant) {
    mutable_tuning().fwd_variant.store(fwd_variant, std::memory_order_relaxed);
    mutable_tuning().bwd_variant.store(bwd_variant, std::memory_order_relaxed);
}

int e3j_amd_convolution_fwd(const e3j_amd_conv_params *p, const void *coef, const void *x,
                            const void *y, const void *s, const int32_t *sender,
                            const int32_t *receiver_ptr, const int32_t *edge_perm, void *out,
                            void *stream_) {
    int rc = validate(p, "convolution");
    if (rc) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (p->num_nodes == 0) return E3J_AMD_OK;
    if (missing(out, p->num_nodes) || missing(x, p->num_nodes) || receiver_ptr == nullptr ||
        missing(sender, p->num_edges) || missing(y, p->num_edges) || missing(s, p->num_edges) ||
        (p->signature < 0 && missing(coef, p->num_coef)))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: null operand");
    if (signature_fits_f64(p)) {
        if (p->row_cap != 0 || p->segments != nullptr)
            return set_error(E3J_AMD_UNIMPLEMENTED, "convolution: row_cap / segments are taken by the float32 "
                                                    "unrolled kernels only");
        rc = signature(p->signature).fwd_f64(*p, static_cast<const double *>(x), static_cast<const double *>(y),
                                             static_cast<const double *>(s), sender, receiver_ptr, edge_perm,
                                             static_cast<double *>(out), stream);
        return finish(p, stream, rc, "convolution");
    }
    if (signature_fits_f16(p)) {
        if (p->row_cap != 0 || p->segments != nullptr)
            return set_error(E3J_AMD_UNIMPLEMENTED, "convolution: row_cap / segments are taken by the float32 "
                                                    "unrolled kernels only");
        rc = signature(p->signature).fwd_f16(*p, static_cast<const half_t *>(x), static_cast<const half_t *>(y),
                                             static_cast<const half_t *>(s), sender, receiver_ptr, edge_perm,
                                             static_cast<half_t *>(out), stream);
        return finish(p, stream, rc, "convolution");
    }
    const bool split_rows = p->row_cap > 0 || p->segments != nullptr;
    if (p->row_cap < 0 || p->max_segments < 0 || p->row_piece < 0 || p->row_piece > p->row_cap)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: row_cap / row_piece / max_segments");
    if (split_rows && !(signature_fits(p, {x, s, out}) && p->layout == E3J_AMD_LAYOUT_TRAILING))
        return set_error(E3J_AMD_UNIMPLEMENTED,
                         "convolution: row_cap / segments are taken by the unrolled kernels of the "
                         "trailing layout only (16-byte aligned operands)");
    if (signature_fits(p, {x, s, out}) && p->segments != nullptr && p->partials != nullptr) {
        // the pieces of long rows in a fixed order: every piece sums into a scratch row of its own
        // (the launch names the piece's number as its row), then the rows of a receiver's pieces
        // are added to its output row one after another
        const int64_t row_floats = (int64_t)p->num_out * p->channels;
        if (reinterpret_cast<uintptr_t>(p->partials) % 16 != 0)
            return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: partials must be 16-byte aligned");
        rc = launch_prepare_partials(p->segments, p->max_segments, row_floats, p->partials, stream);
        if (rc == E3J_AMD_OK) {
            e3j_amd_conv_params numbered = *p;
            numbered.segments = row_partials_list(p->partials, p->max_segments, row_floats);
            numbered.partials = nullptr;
            rc = signature(p->signature).fwd(numbered, static_cast<const float *>(x), static_cast<const float *>(y),
                                             static_cast<const float *>(s), sender, receiver_ptr, edge_perm,
                                             p->partials, stream);
        }
        if (rc == E3J_AMD_OK)
            rc = launch_combine_pieces(p->segments, receiver_ptr, p->max_segments,
                                       p->row_piece > 0 ? p->row_piece : p->row_cap, row_floats, p->partials,
                                       static_cast<float *>(out), stream);
    } else if (signature_fits(p, {x, s, out})) {
        rc = signature(p->signature).fwd(*p, static_cast<const float *>(x), static_cast<const float *>(y),
                                         static_cast<const float *>(s), sender, receiver_ptr,
                                         edge_perm, static_cast<float *>(out), stream);
    } else {
        if ((rc = flip_without_kernel(p, "convolution"))) return rc;
        if (missing(coef, p->num_coef))
            return set_error(E3J_AMD_INVALID_ARGUMENT,
                             "convolution: operands are not 16-byte aligned, which runs the "
                             "table-driven kernel and needs `coef`");
        rc = launch_generic_fwd(*p, coef, x, y, s, sender, receiver_ptr, edge_perm, out, stream);
    }
    return finish(p, stream, rc, "convolution");
}

int e3j_amd_convolution_bwd_sender(const e3j_amd_conv_params *p, const void *coef, const void *x,
                                   const void *y, const void *s, const void *dm,
                                   const int32_t *receiver_t, const int32_t *sender_ptr,
                                   const int32_t *edge_perm, void *dx, void *dy, void *ds,
                                   void *stream) {
    return run_backward(p, false, coef, x, y, s, dm, receiver_t, sender_ptr, edge_perm, dx, dy, ds,
                        static_cast<hipStream_t>(stream), false);
}

int e3j_amd_convolution_bwd_receiver(const e3j_amd_conv_params *p, const void *coef, const void *x,
                                     const void *y, const void *s, const void *dm,
                                     const int32_t *sender, const int32_t *receiver_ptr,
                                     const int32_t *edge_perm, void *dx, void *dy, void *ds,
                                     void *stream) {
    return run_backward(p, true, coef, x, y, s, dm, sender, receiver_ptr, edge_perm, dx, dy, ds,
                        static_cast<hipStream_t>(stream), false);
}

size_t e3j_amd_row_partials_bytes(int64_t max_segments, int32_t num_out, int32_t channels) {
    if (num_out <= 0 || channels <= 0) return 0;
    return row_partials_bytes(max_segments, (int64_t)num_out * channels);
}

int e3j_amd_num_signatures(void) { return num_signatures(); }

const char *e3j_amd_signature_name(int id) {
    if (id < 0 || id >= num_signatures()) return "";
    return signature(id).name;
}

namespace {
size_t align256(size_t n) { return (n + 255) / 256 * 256; }
struct OrderedWorkspace {
    size_t keys, pos, scratch, ptr, csr, u, slots, total;
    explicit OrderedWorkspace(const e3j_amd_conv_params &p) {
        const size_t e = (size_t)p.num_edges, n = (size_t)p.num_nodes;
        size_t at = 0;
        auto take = [&](size_t bytes) { const size_t here = at; at += align256(bytes); return here; };
        keys = take(4 * e);
        pos = take(4 * e);
        scratch = take(4 * e);
        ptr = take(4 * (n + 1));
        csr = take(e3j_amd_csr_workspace_bytes(p.num_nodes, p.num_edges));
        u = take(4 * e * (size_t)p.num_x * (size_t)p.channels);
        slots = take(4 * e * (size_t)max_dy_slots(p.channels) * (size_t)p.num_y);
        total = at;
    }
};
}  // namespace

size_t e3j_amd_convolution_bwd_ordered_workspace_bytes(const e3j_amd_conv_params *p) {
    if (p == nullptr || p->num_nodes < 0 || p->num_edges < 0 || p->num_x < 1 || p->num_y < 1 ||
        p->channels < 1)
        return 0;
    return OrderedWorkspace(*p).total + 256;
}

int e3j_amd_convolution_bwd_ordered(const e3j_amd_conv_params *p, const void *coef, const void *x,
                                    const void *y, const void *s, const void *dm,
                                    const int32_t *sender, const int32_t *receiver_ptr,
                                    const int32_t *edge_perm, void *dx, void *dy, void *ds,
                                    void *workspace, void *stream_) {
    (void)coef;
    const char *op = "convolution_bwd_ordered";
    int rc = validate(p, op);
    if (rc) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (p->num_nodes == 0 && p->num_edges == 0) return E3J_AMD_OK;
    if (missing(x, p->num_nodes) || missing(dm, p->num_nodes) || missing(dx, p->num_nodes) ||
        receiver_ptr == nullptr || missing(sender, p->num_edges) || missing(y, p->num_edges) ||
        missing(s, p->num_edges) || missing(dy, p->num_edges) || missing(ds, p->num_edges) ||
        workspace == nullptr)
        return set_error(E3J_AMD_INVALID_ARGUMENT, std::string(op) + ": null operand");
    if (p->num_nodes == 0) return E3J_AMD_OK;
    if (p->signature >= 0 && !aligned16({x, s, dm, dx, ds, workspace}))
        return set_error(E3J_AMD_INVALID_ARGUMENT, std::string(op) + ": operands must be 16-byte aligned");
    if (!signature_fits(p, {x, s, dm, dx, ds}) || signature(p->signature).bwd == nullptr)
        return set_error(E3J_AMD_UNIMPLEMENTED,
                         std::string(op) + ": needs a compile-time-unrolled kernel for the table; "
                                           "e3j_amd_convolution_bwd_sender is the atomic-free "
                                           "table-driven backward");
    char *base = static_cast<char *>(workspace);
    base += (256 - reinterpret_cast<uintptr_t>(base) % 256) % 256;
    const OrderedWorkspace w(*p);
    int32_t *keys = reinterpret_cast<int32_t *>(base + w.keys);
    int32_t *pos = reinterpret_cast<int32_t *>(base + w.pos);
    int32_t *scratch = reinterpret_cast<int32_t *>(base + w.scratch);
    int32_t *sender_ptr = reinterpret_cast<int32_t *>(base + w.ptr);
    // positions grouped by sender, ascending within a sender (stable sort): the summation order
    rc = launch_live_keys(sender, receiver_ptr, p->num_nodes, p->num_edges, keys, stream);
    if (rc) return rc;
    rc = e3j_amd_sort_edges(keys, keys, p->num_edges, p->num_nodes, pos, scratch, sender_ptr,
                            base + w.csr, stream);
    if (rc) return rc;
    OrderedBwd ordered{reinterpret_cast<float *>(base + w.u), reinterpret_cast<float *>(base + w.slots), 0, 0};
    rc = signature(p->signature).bwd(*p, static_cast<const float *>(x), static_cast<const float *>(y),
                                     static_cast<const float *>(s), static_cast<const float *>(dm),
                                     sender, receiver_ptr, edge_perm, static_cast<float *>(dx),
                                     static_cast<float *>(dy), static_cast<float *>(ds), stream, &ordered);
    if (rc == E3J_AMD_OK)
        rc = reduce_ordered_dx(*p, ordered.u, sender_ptr, pos, ordered.covered, static_cast<float *>(dx), stream);
    if (rc == E3J_AMD_OK && ordered.slots > 1)
        rc = reduce_ordered_dy(*p, ordered.dy_slots, ordered.slots, edge_perm, static_cast<float *>(dy), stream);
    if (rc == E3J_AMD_OK)
        rc = launch_zero_padding(*p, sender, receiver_ptr, edge_perm, static_cast<float *>(dy),
                                 static_cast<float *>(ds), stream);
    return finish(p, stream, rc, op);
}

int32_t e3j_amd_tile_rows(int32_t sig) {
    if (sig < 0 || sig >= num_signatures()) return 0;
    const Signature &sg = signature(sig);
    if (sg.bwd_tiled == nullptr || sg.tile_row_bytes == nullptr) return 0;
    const int bytes = sg.tile_row_bytes();
    return bytes > 0 ? (int32_t)(160 * 1024 / bytes) : 0;
}

int32_t e3j_amd_tile_rows_default(int32_t sig) {
    const int32_t limit = e3j_amd_tile_rows(sig);
    if (limit <= 0) return 0;
    const int32_t want = signature(sig).tile_rows_default ? signature(sig).tile_rows_default() : limit;
    return want < 1 ? 1 : want > limit ? limit : want;
}

int e3j_amd_convolution_bwd_tiled(const e3j_amd_conv_params *p, const void *x, const void *y,
                                  const void *s, const void *dm, const int32_t *sender,
                                  const int32_t *receiver_ptr, const int32_t *edge_perm,
                                  const e3j_amd_tile_schedule *schedule, void *dx, void *dy, void *ds,
                                  void *stream_) {
    const char *op = "convolution_bwd_tiled";
    int rc = validate(p, op);
    if (rc) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (p->num_nodes == 0 && p->num_edges == 0) return E3J_AMD_OK;
    if (missing(x, p->num_nodes) || missing(dm, p->num_nodes) || missing(dx, p->num_nodes) ||
        receiver_ptr == nullptr || missing(sender, p->num_edges) || missing(y, p->num_edges) ||
        missing(s, p->num_edges) || missing(dy, p->num_edges) || missing(ds, p->num_edges) ||
        schedule == nullptr)
        return set_error(E3J_AMD_INVALID_ARGUMENT, std::string(op) + ": null operand");
    if (p->num_nodes == 0) return E3J_AMD_OK;
    if (p->signature < 0 || p->val_dtype != E3J_AMD_F32 || signature(p->signature).bwd_tiled == nullptr)
        return set_error(E3J_AMD_UNIMPLEMENTED,
                         std::string(op) + ": needs a float32 compile-time-unrolled kernel of the trailing layout "
                                           "with at least 64 channels; e3j_amd_convolution_bwd_receiver "
                                           "serves the other cases");
    if (!aligned16({x, s, dm, dx, ds}))
        return set_error(E3J_AMD_INVALID_ARGUMENT, std::string(op) + ": operands must be 16-byte aligned");
    if (schedule->num_work < 0 || (schedule->num_work > 0 && schedule->work == nullptr) ||
        missing(schedule->sender, p->num_edges) || missing(schedule->edge, p->num_edges) ||
        missing(schedule->local, p->num_edges))
        return set_error(E3J_AMD_INVALID_ARGUMENT, std::string(op) + ": incomplete schedule");
    rc = signature(p->signature).bwd_tiled(*p, static_cast<const float *>(x), static_cast<const float *>(y),
                                           static_cast<const float *>(s), static_cast<const float *>(dm),
                                           *schedule, static_cast<float *>(dx), static_cast<float *>(dy),
                                           static_cast<float *>(ds), stream);
    if (rc == E3J_AMD_OK)
        rc = launch_zero_padding(*p, sender, receiver_ptr, edge_perm, static_cast<float *>(dy),
                                 static_cast<float *>(ds), stream);
    return finish(p, stream, rc, op);
}

int e3j_amd_find_signature(const void *coef_host, int32_t coef_idx_bytes, int32_t val_dtype,
                           int32_t num_coef, int32_t num_x, int32_t num_y, int32_t num_out,
                           int32_t num_scalars, int32_t channels, int32_t layout,
                           float *coef_scale, uint32_t *y_flip) {
    if (coef_scale) *coef_scale = 1.0f;
    if (y_flip) *y_flip = 0;
    if (coef_host == nullptr || (val_dtype != E3J_AMD_F32 && val_dtype != E3J_AMD_F16) || num_coef <= 0) return -1;
    if (coef_idx_bytes != 1 && coef_idx_bytes != 4) return -1;
    if (val_dtype == E3J_AMD_F16)
        return match_signature_f16(coef_host, coef_idx_bytes, num_coef, num_x, num_y, num_out, num_scalars, channels,
                                   layout, false, coef_scale, y_flip);
    const std::vector<TableEntry> entries = unpack_entries(coef_host, coef_idx_bytes, num_coef, false);
    return match_signature(entries, num_x, num_y, num_out, num_scalars, channels, layout, coef_scale, y_flip);
}

int e3j_amd_find_signature_f64(const void *coef_host, int32_t coef_idx_bytes, int32_t num_coef,
                               int32_t num_x, int32_t num_y, int32_t num_out, int32_t num_scalars,
                               int32_t channels, int32_t layout, double *coef_classes, uint32_t *y_flip) {
    return match_signature_f64(coef_host, coef_idx_bytes, num_coef, num_x, num_y, num_out, num_scalars, channels,
                               layout, false, coef_classes, y_flip);
}

}  // extern "C"

namespace e3j_amd {

int match_signature_f16(const void *coef_host, int32_t coef_idx_bytes, int32_t num_coef, int32_t num_x,
                        int32_t num_y, int32_t num_out, int32_t num_scalars, int32_t channels, int32_t layout,
                        bool columns_ji, float *coef_scale, uint32_t *y_flip) {
    // a table of half values: every entry within half rounding (2^-11) of the built-in table times one
    // factor; the float16 kernels then compute with the built-in float values
    const size_t item = coef_idx_bytes == 1 ? sizeof(Coef4D<uint8_t, half_t>) : sizeof(Coef4D<int32_t, half_t>);
    const unsigned char *bytes = static_cast<const unsigned char *>(coef_host);
    std::vector<TableEntry> entries((size_t)num_coef);
    for (int n = 0; n < num_coef; n++) {
        half_t h;
        std::memcpy(&h, bytes + n * item, sizeof(h));
        entries[n].val = (float)h;
        for (int t = 0; t < 4; t++) {
            if (coef_idx_bytes == 1) entries[n].idx[t] = bytes[n * item + 2 + t];
            else std::memcpy(&entries[n].idx[t], bytes + n * item + 4 + 4 * t, 4);
        }
        if (columns_ji) std::swap(entries[n].idx[0], entries[n].idx[1]);  // (j, i, k, l) of a dx table -> (i, j, k, l)
    }
    // (an entry and the entry the factor is taken from are each off by up to 2^-11: 2^-10 between them)
    return match_signature(entries, num_x, num_y, num_out, num_scalars, channels, layout, coef_scale, y_flip,
                           1.5 / 1024.0, true);
}

int match_signature_f64(const void *coef_host, int32_t coef_idx_bytes, int32_t num_coef, int32_t num_x,
                        int32_t num_y, int32_t num_out, int32_t num_scalars, int32_t channels, int32_t layout,
                        bool columns_ji, double *coef_classes, uint32_t *y_flip) {
    if (y_flip) *y_flip = 0;
    if (coef_host == nullptr || coef_classes == nullptr || num_coef <= 0) return -1;
    if (coef_idx_bytes != 1 && coef_idx_bytes != 4) return -1;
    struct Entry {
        double val;
        int32_t idx[4];
        int32_t cls;
    };
    auto less = [](const Entry &a, const Entry &b) {
        for (int t = 0; t < 4; t++)
            if (a.idx[t] != b.idx[t]) return a.idx[t] < b.idx[t];
        return false;
    };
    const size_t item = coef_idx_bytes == 1 ? sizeof(Coef4D<uint8_t, double>) : sizeof(Coef4D<int32_t, double>);
    const unsigned char *bytes = static_cast<const unsigned char *>(coef_host);
    std::vector<Entry> given((size_t)num_coef), own((size_t)num_coef);
    for (int n = 0; n < num_coef; n++) {
        std::memcpy(&given[n].val, bytes + n * item, sizeof(double));
        for (int t = 0; t < 4; t++) {
            if (coef_idx_bytes == 1) given[n].idx[t] = bytes[n * item + 8 + t];
            else std::memcpy(&given[n].idx[t], bytes + n * item + 8 + 4 * t, 4);
        }
        if (columns_ji) std::swap(given[n].idx[0], given[n].idx[1]);  // (j, i, k, l) of a dx table -> (i, j, k, l)
    }
    std::stable_sort(given.begin(), given.end(), less);
    const bool signs_allowed = y_flip != nullptr && num_y <= 32;
    for (int id = 0; id < num_signatures(); id++) {
        const Signature &sg = signature(id);
        if (sg.fwd_f64 == nullptr || sg.bwd_f64 == nullptr || sg.coef_class == nullptr ||
            sg.num_classes < 1 || sg.num_classes > kF64Classes)
            continue;
        if (sg.num_coef != num_coef || sg.num_x != num_x || sg.num_y != num_y || sg.num_out != num_out ||
            sg.num_scalars != num_scalars || sg.channels != channels || sg.layout != layout)
            continue;
        for (int n = 0; n < num_coef; n++) {
            own[n].val = sg.val[n];
            own[n].cls = sg.coef_class[n];
            for (int t = 0; t < 4; t++) own[n].idx[t] = sg.idx[4 * n + t];
        }
        std::stable_sort(own.begin(), own.end(), less);
        // Same coordinates; the sign of every entry equal to the built-in one, or opposite for all
        // entries of a y component; one magnitude per class of the built-in table.
        double mags[kF64Classes];
        bool have[kF64Classes] = {false};
        uint32_t flip = 0, seen = 0;
        bool same = true;
        for (int n = 0; n < num_coef && same; n++) {
            for (int t = 0; t < 4 && same; t++) same = given[n].idx[t] == own[n].idx[t];
            if (!same) break;
            const double v = given[n].val;
            if (own[n].val == 0.0f || own[n].cls >= sg.num_classes) {  // (no built-in table holds zeros)
                same = v == 0.0;
                continue;
            }
            if (v == 0.0 || !std::isfinite(v)) { same = false; break; }
            const int m = own[n].cls;
            const double mag = std::fabs(v);
            if (!have[m]) { mags[m] = mag; have[m] = true; }
            else same = std::fabs(mag - mags[m]) <= 1e-13 * mags[m];
            const bool opposite = (v < 0.0) != (own[n].val < 0.0f);
            const int k = given[n].idx[2];
            if (!signs_allowed) {
                same = same && !opposite;
            } else if ((seen >> k) & 1u) {
                same = same && (((flip >> k) & 1u) != 0) == opposite;
            } else {
                seen |= 1u << k;
                if (opposite) flip |= 1u << k;
            }
        }
        if (!same) continue;
        for (int m = 0; m < kF64Classes; m++) coef_classes[m] = m < sg.num_classes && have[m] ? mags[m] : 0.0;
        if (y_flip) *y_flip = flip;
        return id;
    }
    return -1;
}

}  // namespace e3j_amd
