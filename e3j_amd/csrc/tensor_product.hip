// Row-wise sparse tensor product z[r] = sum_n c_n x[r, j_n] (*) y[r, k_n] -> z[r, i_n] for
// gfx950: table-driven kernels for any coefficient table, the three channel modes, both
// layouts, float32/float64.  Same math as the convolution without gather and scatter
// (lib/e3j_ops/cuda/tensor_product.cuh:40-118; channel modes of
// lib/e3j_ops/cuda/tensor_product/trailing_channels.cuh and leading_channels.cuh):
//   OUTER  z[r, i, cx, cy] += c x[r, j, cx] y[r, k, cy]   (either side may have no channel axis)
//   INNER  z[r, i]         += c sum_c x[r, j, c] y[r, k, c]
//   MAP    z[r, i, c]      += c x[r, j, c] y[r, k, c]
//
// Mapping: a lane owns one output column (r, cz) (INNER: one channel of a row), copies the
// X + Y operand values of its column into a private column of LDS, which the table then
// indexes dynamically; coefficients are wave-uniform and travel through scalar loads.  Runs
// of equal output index are summed in a register and stored once.

#include <cmath>
#include <cstring>
#include <deque>
#include <initializer_list>
#include <mutex>

#include "tp_unrolled.h"

namespace e3j_amd {

// Signatures registered at run time live behind the built-in ones.  The list only grows and a
// deque never moves its elements, so ids and references stay valid.
namespace {
std::mutex g_tp_registry_mutex;
std::deque<const TpSignature *> g_tp_registered;
}  // namespace

int num_tp_signatures() {
    std::lock_guard<std::mutex> lock(g_tp_registry_mutex);
    return num_builtin_tp_signatures() + (int)g_tp_registered.size();
}

const TpSignature &tp_signature(int id) {
    if (id < num_builtin_tp_signatures()) return builtin_tp_signature(id);
    std::lock_guard<std::mutex> lock(g_tp_registry_mutex);
    return *g_tp_registered[id - num_builtin_tp_signatures()];
}

namespace {

// Packed (val, i, j, k) entry: field order and padding of
// lib/e3j_ops/cuda/tensor_product.cuh:98-111.
template <typename Idx, typename Val> struct Coef3Align;
template <> struct Coef3Align<uint8_t, float>  { static constexpr int value = 8; };
template <> struct Coef3Align<int32_t, float>  { static constexpr int value = 16; };
template <> struct Coef3Align<uint8_t, double> { static constexpr int value = 16; };
template <> struct Coef3Align<int32_t, double> { static constexpr int value = 32; };
template <> struct Coef3Align<uint8_t, half_t> { static constexpr int value = 8; };
template <> struct Coef3Align<int32_t, half_t> { static constexpr int value = 16; };
template <typename Idx, typename Val>
struct alignas(Coef3Align<Idx, Val>::value) Coef3 {
    Val val;
    Idx i, j, k;
};
static_assert(sizeof(Coef3<uint8_t, float>) == 8, "packed size");
static_assert(sizeof(Coef3<int32_t, float>) == 16, "packed size");
static_assert(sizeof(Coef3<uint8_t, double>) == 16, "packed size");
static_assert(sizeof(Coef3<int32_t, double>) == 32, "packed size");
static_assert(sizeof(Coef3<uint8_t, half_t>) == 8, "packed size");
static_assert(sizeof(Coef3<int32_t, half_t>) == 16, "packed size");

// One operand or the result: base pointer strides and channel count.
struct Side {
    RowLayout l;
    int dim;       // irreps coordinates
    int channels;  // 1 when the operand has no channel axis
};

// OUTER and MAP: a lane per output column.  `kSorted`: equal output indices are contiguous
// and ascending, so every output coordinate is stored exactly once (zeros for coordinates
// no coefficient reaches); otherwise the column is zero-filled first and runs are added.
template <typename Idx, typename Val, bool kSorted>
__global__ void tp_columns_kernel(const Coef3<Idx, Val> *__restrict__ coef, int num_coef,
                                  const Val *__restrict__ x, Side sx, const Val *__restrict__ y, Side sy,
                                  Val *__restrict__ z, Side sz, int64_t num_cols, int map_mode) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int lane = threadIdx.x, wave = threadIdx.y;
    const int64_t col = ((int64_t)blockIdx.x * blockDim.y + wave) * kWave + lane;
    const bool active = col < num_cols;
    const int64_t cc = active ? col : 0;
    const int64_t r = cc / sz.channels;
    const int cz = (int)(cc % sz.channels);
    const int cx = map_mode ? cz : cz / sy.channels;
    const int cy = map_mode ? cz : cz % sy.channels;

    Val *xs = reinterpret_cast<Val *>(smem_raw) + (size_t)wave * (sx.dim + sy.dim) * kWave + lane;
    Val *ys = xs + (size_t)sx.dim * kWave;
    const Val *xr = x + r * sx.l.row + (int64_t)cx * sx.l.chan;
    const Val *yr = y + r * sy.l.row + (int64_t)cy * sy.l.chan;
    for (int j = 0; j < sx.dim; j++) xs[j * kWave] = xr[(int64_t)j * sx.l.dim];
    for (int k = 0; k < sy.dim; k++) ys[k * kWave] = yr[(int64_t)k * sy.l.dim];

    Val *zr = z + r * sz.l.row + (int64_t)cz * sz.l.chan;
    if (!kSorted && active)
        for (int i = 0; i < sz.dim; i++) zr[(int64_t)i * sz.l.dim] = Val(0);
    int cur = -1, next_row = 0;
    Val acc = Val(0);
    auto flush = [&]() {
        if (!active || cur < 0) return;
        if (kSorted) {
            for (; next_row < cur; next_row++) zr[(int64_t)next_row * sz.l.dim] = Val(0);
            zr[(int64_t)cur * sz.l.dim] = acc;
            next_row = cur + 1;
        } else {
            zr[(int64_t)cur * sz.l.dim] += acc;
        }
    };
    for (int n = 0; n < num_coef; n++) {
        const Coef3<Idx, Val> cf = coef[n];
        const int ci = (int)cf.i;
        if (ci != cur) {
            flush();
            cur = ci;
            acc = Val(0);
        }
        acc += (xs[(int)cf.j * kWave] * ys[(int)cf.k * kWave]) * cf.val;
    }
    flush();
    if (kSorted && active)
        for (; next_row < sz.dim; next_row++) zr[(int64_t)next_row * sz.l.dim] = Val(0);
}

// INNER: a wave per row; lanes walk the channels in chunks of 64 and keep one partial sum per
// output coordinate in their LDS column; the channel sum is a wave reduction per coordinate.
template <typename Idx, typename Val>
__global__ void tp_inner_kernel(const Coef3<Idx, Val> *__restrict__ coef, int num_coef,
                                const Val *__restrict__ x, Side sx, const Val *__restrict__ y, Side sy,
                                Val *__restrict__ z, int num_out, int64_t num_rows) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int lane = threadIdx.x, wave = threadIdx.y;
    const int64_t r = (int64_t)blockIdx.x * blockDim.y + wave;
    if (r >= num_rows) return;  // uniform per wave; no barriers below
    Val *zs = reinterpret_cast<Val *>(smem_raw) + (size_t)wave * (num_out + sx.dim + sy.dim) * kWave + lane;
    Val *xs = zs + (size_t)num_out * kWave;
    Val *ys = xs + (size_t)sx.dim * kWave;
    for (int i = 0; i < num_out; i++) zs[i * kWave] = Val(0);
    const int channels = sx.channels;
    for (int c0 = 0; c0 < channels; c0 += kWave) {
        const int c = c0 + lane;
        const bool active = c < channels;
        const Val *xr = x + r * sx.l.row + (int64_t)(active ? c : 0) * sx.l.chan;
        const Val *yr = y + r * sy.l.row + (int64_t)(active ? c : 0) * sy.l.chan;
        for (int j = 0; j < sx.dim; j++) xs[j * kWave] = active ? xr[(int64_t)j * sx.l.dim] : Val(0);
        for (int k = 0; k < sy.dim; k++) ys[k * kWave] = yr[(int64_t)k * sy.l.dim];
        for (int n = 0; n < num_coef; n++) {
            const Coef3<Idx, Val> cf = coef[n];
            zs[(int)cf.i * kWave] += (xs[(int)cf.j * kWave] * ys[(int)cf.k * kWave]) * cf.val;
        }
    }
    Val *zr = z + r * num_out;
    for (int i = 0; i < num_out; i++) {
        const Val total = wave_sum(zs[i * kWave]);
        if (lane == 0) zr[i] = total;
    }
}

constexpr int kMaxLds = 64 * 1024;  // per block, without opting in to more

template <typename Idx, typename Val>
int launch_typed(int mode, bool sorted, const void *coef, int num_coef, const void *x, Side sx,
                 const void *y, Side sy, void *z, Side sz, int64_t num_rows, hipStream_t stream) {
    using C = Coef3<Idx, Val>;
    if (num_rows == 0) return E3J_AMD_OK;
    if (mode == E3J_AMD_MODE_INNER) {
        const size_t per_wave = (size_t)(sz.dim + sx.dim + sy.dim) * kWave * sizeof(Val);
        if (per_wave > kMaxLds)
            return set_error(E3J_AMD_UNIMPLEMENTED,
                             "tensor_product: INNER mode keeps num_x + num_y + num_out values per lane in "
                             "LDS; these sizes need " + std::to_string(per_wave) + " bytes per wave");
        int waves = (int)(kMaxLds / per_wave);
        waves = waves > 4 ? 4 : waves;
        const int64_t blocks = (num_rows + waves - 1) / waves;
        if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "tensor_product: too many rows");
        hipLaunchKernelGGL((tp_inner_kernel<Idx, Val>), dim3((unsigned)blocks), dim3(kWave, waves),
                           per_wave * waves, stream, static_cast<const C *>(coef), num_coef,
                           static_cast<const Val *>(x), sx, static_cast<const Val *>(y), sy,
                           static_cast<Val *>(z), sz.dim, num_rows);
        return check_hip(hipGetLastError(), "tensor_product (INNER) launch");
    }
    const size_t per_wave = (size_t)(sx.dim + sy.dim) * kWave * sizeof(Val);
    if (per_wave > kMaxLds)
        return set_error(E3J_AMD_UNIMPLEMENTED, "tensor_product: num_x + num_y too large for the LDS columns");
    int waves = (int)(kMaxLds / per_wave);
    waves = waves > 4 ? 4 : waves;
    const int64_t num_cols = num_rows * sz.channels;
    const int64_t blocks = (num_cols + (int64_t)waves * kWave - 1) / ((int64_t)waves * kWave);
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "tensor_product: too many columns");
    const int map_mode = mode == E3J_AMD_MODE_MAP;
    if (sorted)
        hipLaunchKernelGGL((tp_columns_kernel<Idx, Val, true>), dim3((unsigned)blocks), dim3(kWave, waves),
                           per_wave * waves, stream, static_cast<const C *>(coef), num_coef,
                           static_cast<const Val *>(x), sx, static_cast<const Val *>(y), sy,
                           static_cast<Val *>(z), sz, num_cols, map_mode);
    else
        hipLaunchKernelGGL((tp_columns_kernel<Idx, Val, false>), dim3((unsigned)blocks), dim3(kWave, waves),
                           per_wave * waves, stream, static_cast<const C *>(coef), num_coef,
                           static_cast<const Val *>(x), sx, static_cast<const Val *>(y), sy,
                           static_cast<Val *>(z), sz, num_cols, map_mode);
    return check_hip(hipGetLastError(), "tensor_product launch");
}

Side make_side(int layout, int dim, int channels) { return Side{make_layout(layout, dim, channels), dim, channels}; }

int out_channels(int mode, int cx, int cy) {
    return mode == E3J_AMD_MODE_OUTER ? cx * cy : mode == E3J_AMD_MODE_INNER ? 1 : cx;
}

// One product with explicit operand sizes: the forward pass and both halves of the backward.
int launch_product(const e3j_amd_tp_params *p, int mode, const void *coef, const void *a, int dim_a, int ch_a,
                   const void *b, int dim_b, int ch_b, void *out, int dim_out, hipStream_t stream) {
    const Side sa = make_side(p->layout, dim_a, ch_a), sb = make_side(p->layout, dim_b, ch_b);
    const Side so = make_side(p->layout, dim_out, out_channels(mode, ch_a, ch_b));
    const bool sorted = p->coef_sorted != 0;
    const bool u8 = p->coef_idx_bytes == 1;
    if (p->val_dtype == E3J_AMD_F16)
        return u8 ? launch_typed<uint8_t, half_t>(mode, sorted, coef, p->num_coef, a, sa, b, sb, out, so, p->num_rows, stream)
                  : launch_typed<int32_t, half_t>(mode, sorted, coef, p->num_coef, a, sa, b, sb, out, so, p->num_rows, stream);
    if (p->val_dtype == E3J_AMD_F32)
        return u8 ? launch_typed<uint8_t, float>(mode, sorted, coef, p->num_coef, a, sa, b, sb, out, so, p->num_rows, stream)
                  : launch_typed<int32_t, float>(mode, sorted, coef, p->num_coef, a, sa, b, sb, out, so, p->num_rows, stream);
    return u8 ? launch_typed<uint8_t, double>(mode, sorted, coef, p->num_coef, a, sa, b, sb, out, so, p->num_rows, stream)
              : launch_typed<int32_t, double>(mode, sorted, coef, p->num_coef, a, sa, b, sb, out, so, p->num_rows, stream);
}

int validate_tp(const e3j_amd_tp_params *p, const char *op) {
    const std::string name(op);
    if (p == nullptr) return set_error(E3J_AMD_INVALID_ARGUMENT, name + ": null params");
    if (p->num_rows < 0 || p->num_coef < 0) return set_error(E3J_AMD_INVALID_ARGUMENT, name + ": negative size");
    if (p->num_x < 1 || p->num_y < 1 || p->num_out < 1 || p->channels_x < 1 || p->channels_y < 1)
        return set_error(E3J_AMD_INVALID_ARGUMENT,
                         name + ": num_x, num_y, num_out, channels_x and channels_y must be >= 1");
    if (p->layout != E3J_AMD_LAYOUT_LEADING && p->layout != E3J_AMD_LAYOUT_TRAILING)
        return set_error(E3J_AMD_INVALID_ARGUMENT, name + ": unknown layout " + std::to_string(p->layout));
    if (p->mode != E3J_AMD_MODE_OUTER && p->mode != E3J_AMD_MODE_INNER && p->mode != E3J_AMD_MODE_MAP)
        return set_error(E3J_AMD_INVALID_ARGUMENT, name + ": unknown mode " + std::to_string(p->mode));
    if (p->mode != E3J_AMD_MODE_OUTER && p->channels_x != p->channels_y)
        return set_error(E3J_AMD_INVALID_ARGUMENT,
                         name + ": MAP and INNER modes require same number of LHS and RHS channels, got (" +
                             std::to_string(p->channels_x) + ", " + std::to_string(p->channels_y) + ")");
    if ((p->val_dtype != E3J_AMD_F32 && p->val_dtype != E3J_AMD_F64 && p->val_dtype != E3J_AMD_F16) ||
        (p->coef_idx_bytes != 1 && p->coef_idx_bytes != 4))
        return set_error(E3J_AMD_INVALID_ARGUMENT, name + ": unsupported (IDX, VAL) dtype pair");
    if (p->signature >= num_tp_signatures())
        return set_error(E3J_AMD_INVALID_ARGUMENT, name + ": unknown signature id " + std::to_string(p->signature));
    if (p->signature >= 0) {
        const TpSignature &sg = tp_signature(p->signature);
        const bool mode_ok = sg.uniform_y == 1 ? (p->mode == E3J_AMD_MODE_OUTER && p->channels_y == 1)
                           : sg.uniform_y == 2 ? (p->mode == E3J_AMD_MODE_INNER && p->channels_y == p->channels_x)
                                               : (p->mode == E3J_AMD_MODE_MAP && p->channels_y == p->channels_x);
        const bool channels_ok = sg.layout == E3J_AMD_LAYOUT_TRAILING
                                     ? sg.channels == p->channels_x
                                     : (tp_leading_channels_ok(p->channels_x, sg.uniform_y) &&
                                        p->num_rows * p->channels_x >= kWave);
        const bool dtype_ok = p->val_dtype == E3J_AMD_F32 || (p->val_dtype == E3J_AMD_F16 && sg.fwd_f16 != nullptr) ||
                              (p->val_dtype == E3J_AMD_F64 && sg.fwd_f64 != nullptr);
        if (!mode_ok || !channels_ok || !dtype_ok || p->layout != sg.layout ||
            sg.num_x != p->num_x || sg.num_y != p->num_y || sg.num_out != p->num_out)
            return set_error(E3J_AMD_INVALID_ARGUMENT,
                             name + ": operands do not match signature " + sg.name);
        if (p->val_dtype == E3J_AMD_F64 && p->coef_classes == nullptr)
            return set_error(E3J_AMD_INVALID_ARGUMENT,
                             name + ": a float64 signature needs coef_classes (e3j_amd_tp_find_signature_f64)");
    }
    return E3J_AMD_OK;
}

bool absent(const void *ptr, int64_t count) { return count > 0 && ptr == nullptr; }

// the coefficient classes of a float64 launch, from the caller's host array
F64Coefs tp_classes(const e3j_amd_tp_params *p) {
    F64Coefs c;
    std::memcpy(c.v, p->coef_classes, sizeof(c.v));
    return c;
}

// The unrolled kernels of the leading layout move columns in 16-byte pieces.
const char *const kUnaligned = "tensor_product: the unrolled kernels of the leading layout need 16-byte "
                               "aligned operands (pass signature -1 for the table-driven kernels)";
bool pieces_aligned(const e3j_amd_tp_params *p, std::initializer_list<const void *> ptrs) {
    if (p->layout != E3J_AMD_LAYOUT_LEADING) return true;
    for (const void *ptr : ptrs)
        if (reinterpret_cast<uintptr_t>(ptr) % 16 != 0) return false;
    return true;
}

int finish_tp(const e3j_amd_tp_params *p, hipStream_t stream, int rc, const char *op) {
    if (rc != E3J_AMD_OK || p->debug <= 0) return rc;
    return check_hip(hipStreamSynchronize(stream), op);
}

}  // namespace
}  // namespace e3j_amd

using namespace e3j_amd;

extern "C" int e3j_amd_tensor_product_fwd(const e3j_amd_tp_params *p, const void *coef, const void *x,
                                          const void *y, void *z, void *stream_ptr) {
    hipStream_t stream = static_cast<hipStream_t>(stream_ptr);
    if (int rc = validate_tp(p, "tensor_product")) return rc;
    if (absent(x, p->num_rows) || absent(y, p->num_rows) || absent(z, p->num_rows) ||
        (p->signature < 0 && absent(coef, (int64_t)p->num_coef * p->num_rows)))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "tensor_product: null operand");
    if (p->signature >= 0) {
        if (!pieces_aligned(p, {x, y, z})) return set_error(E3J_AMD_INVALID_ARGUMENT, kUnaligned);
        const TpSignature &sg = tp_signature(p->signature);
        int rc;
        if (p->val_dtype == E3J_AMD_F16)
            rc = sg.fwd_f16(p->num_rows, p->channels_x, p->coef_scale, static_cast<const half_t *>(x),
                            static_cast<const half_t *>(y), static_cast<half_t *>(z), stream);
        else if (p->val_dtype == E3J_AMD_F64)
            rc = sg.fwd_f64(p->num_rows, p->channels_x, tp_classes(p), static_cast<const double *>(x),
                            static_cast<const double *>(y), static_cast<double *>(z), stream);
        else
            rc = sg.fwd(p->num_rows, p->channels_x, p->coef_scale, static_cast<const float *>(x),
                        static_cast<const float *>(y), static_cast<float *>(z), stream);
        return finish_tp(p, stream, rc, "tensor_product");
    }
    const int rc = launch_product(p, p->mode, coef, x, p->num_x, p->channels_x, y, p->num_y, p->channels_y, z,
                                  p->num_out, stream);
    return finish_tp(p, stream, rc, "tensor_product");
}

extern "C" int e3j_amd_tensor_product_bwd(const e3j_amd_tp_params *p, const void *coef_bwd, const void *x,
                                          const void *y, const void *dz, void *dx, void *dy,
                                          void *stream_ptr) {
    hipStream_t stream = static_cast<hipStream_t>(stream_ptr);
    if (int rc = validate_tp(p, "tensor_product_bwd")) return rc;
    if (p->mode == E3J_AMD_MODE_OUTER && p->channels_x > 1 && p->channels_y > 1)
        return set_error(E3J_AMD_UNIMPLEMENTED,
                         "tensor_product_bwd: OUTER mode requires either LHS or RHS to have one channel, got (" +
                             std::to_string(p->channels_x) + ", " + std::to_string(p->channels_y) + ")");
    if (absent(x, p->num_rows) || absent(y, p->num_rows) || absent(dz, p->num_rows) || absent(dx, p->num_rows) ||
        absent(dy, p->num_rows) || (p->signature < 0 && absent(coef_bwd, (int64_t)p->num_coef * p->num_rows)))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "tensor_product_bwd: null operand");
    if (p->signature >= 0) {
        if (!pieces_aligned(p, {x, y, dz, dx, dy})) return set_error(E3J_AMD_INVALID_ARGUMENT, kUnaligned);
        const TpSignature &sg = tp_signature(p->signature);
        int rc;
        if (p->val_dtype == E3J_AMD_F16)
            rc = sg.bwd_f16(p->num_rows, p->channels_x, p->coef_scale, static_cast<const half_t *>(x),
                            static_cast<const half_t *>(y), static_cast<const half_t *>(dz),
                            static_cast<half_t *>(dx), static_cast<half_t *>(dy), stream);
        else if (p->val_dtype == E3J_AMD_F64)
            rc = sg.bwd_f64(p->num_rows, p->channels_x, tp_classes(p), static_cast<const double *>(x),
                            static_cast<const double *>(y), static_cast<const double *>(dz),
                            static_cast<double *>(dx), static_cast<double *>(dy), stream);
        else
            rc = sg.bwd(p->num_rows, p->channels_x, p->coef_scale, static_cast<const float *>(x),
                        static_cast<const float *>(y), static_cast<const float *>(dz), static_cast<float *>(dx),
                        static_cast<float *>(dy), stream);
        return finish_tp(p, stream, rc, "tensor_product_bwd");
    }
    // dx = product(table (j; i, k); dz, y), dy = product(table (k; i, j); dz, x).  The channel
    // mode of each half follows from where the channel axis of the forward pass went
    // (src/e3j/ops/tensor_product.py:503-529): u,u->u gives MAP twice; u,u->1 gives 1,u->u twice;
    // u,1->u gives u,1->u and u,u->1; 1,u->u gives u,u->1 and u,1->u.
    const int cx = p->channels_x, cy = p->channels_y;
    const int cz = out_channels(p->mode, cx, cy);
    int mode_x, mode_y;
    if (p->mode == E3J_AMD_MODE_MAP) mode_x = mode_y = E3J_AMD_MODE_MAP;
    else if (p->mode == E3J_AMD_MODE_INNER) mode_x = mode_y = E3J_AMD_MODE_OUTER;
    else if (cx > 1) { mode_x = E3J_AMD_MODE_OUTER; mode_y = E3J_AMD_MODE_INNER; }
    else if (cy > 1) { mode_x = E3J_AMD_MODE_INNER; mode_y = E3J_AMD_MODE_OUTER; }
    else mode_x = mode_y = E3J_AMD_MODE_OUTER;
    const size_t item = p->coef_idx_bytes == 1 ? (p->val_dtype == E3J_AMD_F64 ? 16 : 8)
                                               : (p->val_dtype == E3J_AMD_F64 ? 32 : 16);
    const void *coef_x = coef_bwd;
    const void *coef_y = static_cast<const unsigned char *>(coef_bwd) + item * (size_t)p->num_coef;
    int rc = launch_product(p, mode_x, coef_x, dz, p->num_out, cz, y, p->num_y, cy, dx, p->num_x, stream);
    if (rc == E3J_AMD_OK)
        rc = launch_product(p, mode_y, coef_y, dz, p->num_out, cz, x, p->num_x, cx, dy, p->num_y, stream);
    return finish_tp(p, stream, rc, "tensor_product_bwd");
}

extern "C" int e3j_amd_tp_num_signatures(void) { return num_tp_signatures(); }

extern "C" int e3j_amd_tp_register_signature(const void *entry) {
    const TpSignature *sg = static_cast<const TpSignature *>(entry);
    if (sg == nullptr || sg->fwd == nullptr || sg->bwd == nullptr || sg->val == nullptr || sg->idx == nullptr ||
        sg->num_coef <= 0 || sg->uniform_y < 0 || sg->uniform_y > 2) {
        set_error(E3J_AMD_INVALID_ARGUMENT, "tp_register_signature: incomplete entry");
        return -1;
    }
    std::lock_guard<std::mutex> lock(g_tp_registry_mutex);
    g_tp_registered.push_back(sg);
    return num_builtin_tp_signatures() + (int)g_tp_registered.size() - 1;
}

extern "C" const char *e3j_amd_tp_signature_name(int id) {
    return (id >= 0 && id < num_tp_signatures()) ? tp_signature(id).name : "";
}

namespace {

// entry n of a packed rank-3 table in host memory: value (as double) and the three indices
template <typename Val>
double tp_entry(const unsigned char *bytes, int coef_idx_bytes, int n, int32_t (&index)[3]) {
    if (coef_idx_bytes == 1) {
        Coef3<uint8_t, Val> e;
        std::memcpy(&e, bytes + (size_t)n * sizeof(e), sizeof(e));
        index[0] = e.i; index[1] = e.j; index[2] = e.k;
        return (double)e.val;
    }
    Coef3<int32_t, Val> e;
    std::memcpy(&e, bytes + (size_t)n * sizeof(e), sizeof(e));
    index[0] = e.i; index[1] = e.j; index[2] = e.k;
    return (double)e.val;
}

bool tp_sizes_match(const TpSignature &sg, int32_t num_coef, int32_t num_x, int32_t num_y, int32_t num_out,
                    int32_t channels, int32_t kind, int32_t layout) {
    if (sg.num_coef != num_coef || sg.num_x != num_x || sg.num_y != num_y || sg.num_out != num_out ||
        sg.layout != layout || sg.uniform_y != kind)
        return false;
    return sg.layout == E3J_AMD_LAYOUT_TRAILING ? sg.channels == channels : tp_leading_channels_ok(channels, kind);
}

// float32 and float16 tables: one uniform positive factor is allowed between the caller's table and
// the built-in one, taken from the entry of largest magnitude; every entry must agree with it
// within `tolerance` (float32 rounding; for half values the rounding of the entry and of the
// entry the factor is taken from)
template <typename Val>
int tp_find(const unsigned char *bytes, int32_t coef_idx_bytes, int32_t num_coef, int32_t num_x, int32_t num_y,
            int32_t num_out, int32_t channels, int32_t kind, int32_t layout, double tolerance, bool half_kernels,
            float *coef_scale) {
    for (int id = 0; id < num_tp_signatures(); id++) {
        const TpSignature &sg = tp_signature(id);
        if (!tp_sizes_match(sg, num_coef, num_x, num_y, num_out, channels, kind, layout)) continue;
        if (half_kernels && sg.fwd_f16 == nullptr) continue;
        int big = 0;
        for (int n = 1; n < num_coef; n++)
            if (std::fabs(sg.val[n]) > std::fabs(sg.val[big])) big = n;
        int32_t index[3];
        const double scale = tp_entry<Val>(bytes, coef_idx_bytes, big, index) / (double)sg.val[big];
        bool same = scale > 0.0 && std::isfinite(scale);
        for (int n = 0; n < num_coef && same; n++) {
            const double v = tp_entry<Val>(bytes, coef_idx_bytes, n, index);
            for (int t = 0; t < 3 && same; t++) same = index[t] == (int32_t)sg.idx[3 * n + t];
            const double want = scale * (double)sg.val[n];
            same = same && std::fabs(v - want) <= tolerance * std::fabs(want);
        }
        if (same) {
            if (coef_scale) *coef_scale = (float)scale;
            return id;
        }
    }
    return -1;
}

}  // namespace

extern "C" int e3j_amd_tp_find_signature(const void *coef_host, int32_t coef_idx_bytes, int32_t val_dtype,
                                         int32_t num_coef, int32_t num_x, int32_t num_y, int32_t num_out,
                                         int32_t channels, int32_t kind, int32_t layout,
                                         float *coef_scale) {
    if (coef_scale) *coef_scale = 1.0f;
    if (coef_host == nullptr || num_coef <= 0) return -1;
    if (coef_idx_bytes != 1 && coef_idx_bytes != 4) return -1;
    const unsigned char *bytes = static_cast<const unsigned char *>(coef_host);
    if (val_dtype == E3J_AMD_F32)
        return tp_find<float>(bytes, coef_idx_bytes, num_coef, num_x, num_y, num_out, channels, kind, layout, 4e-7,
                              false, coef_scale);
    if (val_dtype == E3J_AMD_F16)
        return tp_find<half_t>(bytes, coef_idx_bytes, num_coef, num_x, num_y, num_out, channels, kind, layout,
                               1.5 / 1024.0, true, coef_scale);
    return -1;
}

extern "C" int e3j_amd_tp_find_signature_f64(const void *coef_host, int32_t coef_idx_bytes, int32_t num_coef,
                                             int32_t num_x, int32_t num_y, int32_t num_out, int32_t channels,
                                             int32_t kind, int32_t layout, double *coef_classes) {
    if (coef_host == nullptr || coef_classes == nullptr || num_coef <= 0) return -1;
    if (coef_idx_bytes != 1 && coef_idx_bytes != 4) return -1;
    const unsigned char *bytes = static_cast<const unsigned char *>(coef_host);
    for (int id = 0; id < num_tp_signatures(); id++) {
        const TpSignature &sg = tp_signature(id);
        if (!tp_sizes_match(sg, num_coef, num_x, num_y, num_out, channels, kind, layout)) continue;
        if (sg.fwd_f64 == nullptr || sg.num_classes > kF64Classes) continue;
        // same entries in the same order, the sign of every entry as built in, and within a class
        // of equal built-in magnitude one magnitude (to float64 rounding): the kernels then
        // compute with the caller's own values
        double classes[kF64Classes];
        bool seen[kF64Classes] = {};
        for (int c = 0; c < kF64Classes; c++) classes[c] = 0.0;
        bool same = true;
        for (int n = 0; n < num_coef && same; n++) {
            int32_t index[3];
            const double v = tp_entry<double>(bytes, coef_idx_bytes, n, index);
            for (int t = 0; t < 3 && same; t++) same = index[t] == (int32_t)sg.idx[3 * n + t];
            const int c = sg.coef_class[n];
            same = same && c < sg.num_classes && std::isfinite(v) && v != 0.0 && (v < 0.0) == (sg.val[n] < 0.f);
            if (!same) break;
            if (!seen[c]) { seen[c] = true; classes[c] = std::fabs(v); }
            else same = std::fabs(std::fabs(v) - classes[c]) <= 1e-13 * classes[c];
        }
        if (same) {
            std::memcpy(coef_classes, classes, sizeof(classes));
            return id;
        }
    }
    return -1;
}
