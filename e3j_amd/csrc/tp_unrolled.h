// Kernel templates of the compile-time-unrolled row-wise tensor product (gfx950):
// trailing-channels layout for channel counts that are multiples of 64, or 16 or 32 (first
// part: float32, and for whole waves of channels float16, held as half and computed in float,
// and float64), and leading-channels layout (second part, float32).
//
// A generated `Sig` type supplies the straight-line Clebsch-Gordan arithmetic of one table
// (`fwd`, `bwd`); the templates supply the wave <-> (row, 64-channel slice) mapping and the
// row accesses.  A lane owns one channel: every access of a wave is one coalesced 256-byte
// piece of a row, touched once and therefore non-temporal.  Two channel modes:
//   MAP            z[r, i, c] = sum c_ijk x[r, j, c] y[r, k, c]      y (R, Y, K)
//   uniform y      z[r, i, c] = sum c_ijk x[r, j, c] y[r, k]         y (R, Y)   (OUTER, u x 1 -> u)
// In the uniform mode y is wave-uniform (scalar loads) and dy is a sum over the channels: one
// wave walks all slices of a row, keeps the per-lane partial sums and reduces them once.
#ifndef E3J_AMD_CSRC_TP_UNROLLED_H_
#define E3J_AMD_CSRC_TP_UNROLLED_H_

#include "unrolled.h"

namespace e3j_amd {

// Registry entry of one table at one channel count and channel mode (generated sources).
struct TpSignature {
    const char *name;
    int32_t num_x, num_y, num_out, num_coef;
    int32_t channels;     // trailing layout: the channel count the kernels were built for;
                          // leading layout: 0, the kernels take the channel count at run time
    int32_t uniform_y;    // channel mode: 0 MAP; 1 OUTER with a y without channel axis; 2 INNER
    int32_t layout;
    const float *val;     // (num_coef) table values as float32
    const uint8_t *idx;   // (num_coef, 3) i, j, k
    int (*fwd)(int64_t rows, int channels, float scale, const float *x, const float *y, float *z,
               hipStream_t stream);
    int (*bwd)(int64_t rows, int channels, float scale, const float *x, const float *y, const float *dz,
               float *dx, float *dy, hipStream_t stream);
    // float16 (values held as half) and float64 forms, or null.  The float64 kernels read one
    // coefficient per class of equal magnitude (`coef_class` of each entry, `num_classes` of them)
    // from `classes` instead of carrying the values as literals: tables of this structure are
    // served to float64 accuracy whatever their values were rounded to.
    int32_t num_classes;
    const uint8_t *coef_class;
    int (*fwd_f16)(int64_t rows, int channels, float scale, const half_t *x, const half_t *y, half_t *z,
                   hipStream_t stream);
    int (*bwd_f16)(int64_t rows, int channels, float scale, const half_t *x, const half_t *y, const half_t *dz,
                   half_t *dx, half_t *dy, hipStream_t stream);
    int (*fwd_f64)(int64_t rows, int channels, const F64Coefs &classes, const double *x, const double *y, double *z,
                   hipStream_t stream);
    int (*bwd_f64)(int64_t rows, int channels, const F64Coefs &classes, const double *x, const double *y,
                   const double *dz, double *dx, double *dy, hipStream_t stream);
};
// channel counts the leading-layout kernels take: MAP any multiple of 4 (16-byte pieces) with at
// least 64 columns in all; uniform y and INNER (channel sums): whole waves per row that fit a block
inline bool tp_leading_channels_ok(int channels, int kind) {
    if (channels < 4 || channels % 4 != 0) return false;
    return kind == 0 || channels == 64 || channels == 128 || channels == 256;
}
// built-in signatures (generated/tp_registry.hip), then the ones registered at run time
int num_builtin_tp_signatures();
const TpSignature &builtin_tp_signature(int id);
int num_tp_signatures();
const TpSignature &tp_signature(int id);

// What the generated arithmetic takes beside its operands: nothing (the coefficients are
// literals), or the coefficient classes of a float64 launch.
struct TpNoCoefs {};
// A: the type the arithmetic runs in for values held as V; Cf: the coefficient argument.
template <typename V> struct TpValue { using A = float; using Cf = TpNoCoefs; };
template <> struct TpValue<double> { using A = double; using Cf = F64Coefs; };
template <typename V> using tp_arith = typename TpValue<V>::A;
template <typename V> using tp_coefs = typename TpValue<V>::Cf;

// Row of a (rows, dim, K) array seen by one lane: coordinate I lives at p[I * K].
template <int K, typename V = float>
struct RowStore {
    V *p;
    bool on;  // lanes past the last row store nothing
    template <int I>
    __device__ __forceinline__ void put(tp_arith<V> v) const {
        if (on) __builtin_nontemporal_store((V)v, p + I * K);
    }
};
template <int K, typename V = float>
struct RowLoad {
    const V *p;
    tp_arith<V> scale;
    template <int I>
    __device__ __forceinline__ tp_arith<V> get() const {
        return (tp_arith<V>)__builtin_nontemporal_load(p + I * K) * scale;
    }
};

// Coordinates kept in registers (results of `fwd`, cotangents for `bwd`).
template <int Z, typename A = float>
struct RegStore {
    A *v;
    template <int I>
    __device__ __forceinline__ void put(A a) const { v[I] = a; }
};
template <int Z, typename A = float>
struct RegLoad {
    const A *v;
    template <int I>
    __device__ __forceinline__ A get() const { return v[I]; }
};

// The wave-uniform y of the uniform-y backward: float values are moved to vector registers (the
// arithmetic then never meets the limit of scalar operands per instruction); doubles stay where
// the compiler puts them, in scalar registers, which leaves the kernel 32 vector registers more
// (float64, l<=3, K=128, 262 144 rows: 10.1 ms instead of 11.8 ms).
__device__ __forceinline__ double tp_vgpr(double v) { return v; }
__device__ __forceinline__ float tp_vgpr(float v) { return to_vgpr(v); }

__device__ __forceinline__ int64_t tp_uniform(int64_t v) {
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)(v & 0xffffffffu));
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)((unsigned long long)v >> 32));
    return (int64_t)(((unsigned long long)hi << 32) | lo);
}

// Which row and channel a lane works on.  Whole waves per row for K >= 64; for 16 or 32
// channels the wave takes 64 / K consecutive rows side by side, one per group of K lanes.
template <int K>
struct TpTile {
    static constexpr int SUB = (K == 16 || K == 32) ? kWave / K : 1;
    static constexpr int SL = K >= kWave ? K / kWave : 1;
    static_assert(SUB > 1 || K % kWave == 0, "64-channel slices, or 16 / 32 channels");
    int64_t r;  // row (clamped to the last one on lanes past the end)
    int c0;     // channel
    bool on;    // the lane has a row
    __device__ __forceinline__ TpTile(int64_t item, int lane, int64_t rows) {
        if (SUB > 1) {
            const int64_t rr = item * SUB + lane / K;
            on = rr < rows;
            r = on ? rr : rows - 1;
            c0 = lane % K;
        } else {
            r = item / SL;
            c0 = (int)(item % SL) * kWave + lane;
            on = true;
        }
    }
    __host__ __device__ static int64_t items(int64_t rows) { return SUB > 1 ? (rows + SUB - 1) / SUB : rows * SL; }
};

template <typename Sig, int K, int WPB, bool kUniformY, typename V = float>
__global__ __launch_bounds__(kWave * WPB) void tp_unrolled_fwd_kernel(
    const V *__restrict__ x, const V *__restrict__ y, V *__restrict__ z, int64_t rows, tp_arith<V> scale,
    tp_coefs<V> cf) {
    using A = tp_arith<V>;
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z;
    const int64_t item = tp_uniform((int64_t)blockIdx.x * WPB + threadIdx.y);
    if (item >= TpTile<K>::items(rows)) return;
    const TpTile<K> t(item, threadIdx.x, rows);
    const int64_t r = t.r;
    const int c0 = t.c0;
    A xv[X], yv[Y];
    const V *xr = x + r * (X * K) + c0;
#pragma unroll
    for (int j = 0; j < X; j++) xv[j] = (A)__builtin_nontemporal_load(xr + j * K) * scale;
    if (kUniformY) {
        const V *yr = y + r * Y;
#pragma unroll
        for (int k = 0; k < Y; k++) yv[k] = (A)yr[k];
    } else {
        const V *yr = y + r * (Y * K) + c0;
#pragma unroll
        for (int k = 0; k < Y; k++) yv[k] = (A)__builtin_nontemporal_load(yr + k * K);
    }
    Sig::fwd(xv, yv, RowStore<K, V>{z + r * (Z * K) + c0, t.on}, cf);
}

// MAP backward: dz is read once for both cotangents.
template <typename Sig, int K, int WPB, typename V = float>
__global__ __launch_bounds__(kWave * WPB) void tp_unrolled_bwd_map_kernel(
    const V *__restrict__ x, const V *__restrict__ y, const V *__restrict__ dz,
    V *__restrict__ dx, V *__restrict__ dy, int64_t rows, tp_arith<V> scale, tp_coefs<V> cf) {
    using A = tp_arith<V>;
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z;
    const int64_t item = tp_uniform((int64_t)blockIdx.x * WPB + threadIdx.y);
    if (item >= TpTile<K>::items(rows)) return;
    const TpTile<K> t(item, threadIdx.x, rows);
    const int64_t r = t.r;
    const int c0 = t.c0;
    A xv[X], yv[Y], dxv[X], dyv[Y];
    const V *xr = x + r * (X * K) + c0;
    const V *yr = y + r * (Y * K) + c0;
#pragma unroll
    for (int j = 0; j < X; j++) { xv[j] = (A)__builtin_nontemporal_load(xr + j * K); dxv[j] = A(0); }
#pragma unroll
    for (int k = 0; k < Y; k++) { yv[k] = (A)__builtin_nontemporal_load(yr + k * K); dyv[k] = A(0); }
    Sig::bwd(xv, yv, RowLoad<K, V>{dz + r * (Z * K) + c0, scale}, dxv, dyv, cf);
    if (!t.on) return;
    V *dxr = dx + r * (X * K) + c0;
    V *dyr = dy + r * (Y * K) + c0;
#pragma unroll
    for (int j = 0; j < X; j++) __builtin_nontemporal_store((V)dxv[j], dxr + j * K);
#pragma unroll
    for (int k = 0; k < Y; k++) __builtin_nontemporal_store((V)dyv[k], dyr + k * K);
}

// Uniform-y backward: a wave per (row, slice); dy (rows, Y) is the channel sum: every wave
// reduces its 64 channels, the slices of a row sit in one block and meet in LDS, and the
// first of them stores the row (fixed order, no atomics).
template <int K>
struct TpUniformGeometry {
    static constexpr int SL = K >= kWave ? K / kWave : 1;  // waves per row
    static constexpr int RPB = SL >= 4 ? 1 : 4 / SL;       // rows per block
    static constexpr int WPB = SL * RPB;
};

// (float64, l<=3: more than 256 registers, one wave per SIMD resident; bounded to 256 it spills
// and takes twice the time)
template <typename Sig, int K, typename V = float>
__global__ __launch_bounds__(kWave * TpUniformGeometry<K>::WPB) void tp_unrolled_bwd_uniform_kernel(
    const V *__restrict__ x, const V *__restrict__ y, const V *__restrict__ dz,
    V *__restrict__ dx, V *__restrict__ dy, int64_t rows, tp_arith<V> scale, tp_coefs<V> cf) {
    using A = tp_arith<V>;
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z;
    using G = TpUniformGeometry<K>;
    using Red = WaveReduceBlocks<Y, kWave, A>;
    __shared__ A partial[G::WPB][Red::P];
    const int wave = threadIdx.y, lane = threadIdx.x;
    const int slice = wave % G::SL;
    const int64_t r = tp_uniform((int64_t)blockIdx.x * G::RPB + wave / G::SL);
    const bool valid = r < rows;  // uniform per wave; every wave reaches the barrier
    if (valid) {
        A yv[Y], dyv[Red::P], xv[X], dxv[X];
        const V *yr = y + r * Y;
#pragma unroll
        for (int k = 0; k < Y; k++) yv[k] = tp_vgpr((A)yr[k]);
#pragma unroll
        for (int k = 0; k < Red::P; k++) dyv[k] = A(0);
        const int c0 = slice * kWave + lane;
        const V *xr = x + r * (X * K) + c0;
#pragma unroll
        for (int j = 0; j < X; j++) { xv[j] = (A)__builtin_nontemporal_load(xr + j * K); dxv[j] = A(0); }
        Sig::bwd(xv, yv, RowLoad<K, V>{dz + r * (Z * K) + c0, scale}, dxv, dyv, cf);
        V *dxr = dx + r * (X * K) + c0;
#pragma unroll
        for (int j = 0; j < X; j++) __builtin_nontemporal_store((V)dxv[j], dxr + j * K);
        A *mine = partial[wave];
        Red::run(dyv, lane, [&](int k, A total) { mine[k] = total; });
    }
    __syncthreads();
    if (valid && slice == 0 && lane < Y) {
        A total = partial[wave][lane];
#pragma unroll
        for (int s2 = 1; s2 < G::SL; s2++) total += partial[wave + s2][lane];
        dy[r * Y + lane] = (V)total;
    }
}

// INNER mode, z[r, i] = sum over the channels: a wave per (row, slice) runs the MAP arithmetic
// on registers, reduces its 64 channels sixteen coordinates at a time, and the slices of a row
// meet in LDS as in the uniform-y backward.  Its backward is the MAP backward with a
// wave-uniform cotangent (scalar loads).
template <int Z, typename V = float>
struct UniformLoad {
    const V *p;
    tp_arith<V> scale;
    template <int I>
    __device__ __forceinline__ tp_arith<V> get() const { return (tp_arith<V>)p[I] * scale; }
};

// sums of zv[0..Z) over the lanes of the wave into out[0..Z) (LDS, one row per wave)
template <int Z, typename A = float>
__device__ __forceinline__ void tp_reduce_columns(const A *zv, A *out, int lane) {
    using Red = WaveReduceBlocks<Z, kWave, A>;
    A padded[Red::P];
#pragma unroll
    for (int t = 0; t < Red::P; t++) padded[t] = t < Z ? zv[t] : A(0);
    Red::run(padded, lane, [&](int i, A total) { out[i] = total; });
}

template <typename Sig, int K, typename V = float>
__global__ __launch_bounds__(kWave * TpUniformGeometry<K>::WPB) void tp_unrolled_fwd_inner_kernel(
    const V *__restrict__ x, const V *__restrict__ y, V *__restrict__ z, int64_t rows, tp_arith<V> scale,
    tp_coefs<V> cf) {
    using A = tp_arith<V>;
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z;
    using G = TpUniformGeometry<K>;
    __shared__ A partial[G::WPB][Z];
    const int wave = threadIdx.y, lane = threadIdx.x;
    const int slice = wave % G::SL;
    const int64_t r = tp_uniform((int64_t)blockIdx.x * G::RPB + wave / G::SL);
    const bool valid = r < rows;  // uniform per wave; every wave reaches the barrier
    if (valid) {
        const int c0 = slice * kWave + lane;
        A xv[X], yv[Y], zv[Z];
        const V *xr = x + r * (X * K) + c0;
        const V *yr = y + r * (Y * K) + c0;
#pragma unroll
        for (int j = 0; j < X; j++) xv[j] = (A)__builtin_nontemporal_load(xr + j * K) * scale;
#pragma unroll
        for (int k = 0; k < Y; k++) yv[k] = (A)__builtin_nontemporal_load(yr + k * K);
        Sig::fwd(xv, yv, RegStore<Z, A>{zv}, cf);
        tp_reduce_columns<Z, A>(zv, partial[wave], lane);
    }
    __syncthreads();
    if (valid && slice == 0) {
        for (int i = lane; i < Z; i += kWave) {
            A total = partial[wave][i];
#pragma unroll
            for (int s2 = 1; s2 < G::SL; s2++) total += partial[wave + s2][i];
            z[r * Z + i] = (V)total;
        }
    }
}

template <typename Sig, int K, int WPB, typename V = float>
__global__ __launch_bounds__(kWave * WPB) void tp_unrolled_bwd_inner_kernel(
    const V *__restrict__ x, const V *__restrict__ y, const V *__restrict__ dz,
    V *__restrict__ dx, V *__restrict__ dy, int64_t rows, tp_arith<V> scale, tp_coefs<V> cf) {
    using A = tp_arith<V>;
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z;
    const int64_t item = tp_uniform((int64_t)blockIdx.x * WPB + threadIdx.y);
    if (item >= TpTile<K>::items(rows)) return;
    const TpTile<K> t(item, threadIdx.x, rows);
    const int64_t r = t.r;
    const int c0 = t.c0;
    A xv[X], yv[Y], dxv[X], dyv[Y];
    const V *xr = x + r * (X * K) + c0;
    const V *yr = y + r * (Y * K) + c0;
#pragma unroll
    for (int j = 0; j < X; j++) { xv[j] = (A)__builtin_nontemporal_load(xr + j * K); dxv[j] = A(0); }
#pragma unroll
    for (int k = 0; k < Y; k++) { yv[k] = (A)__builtin_nontemporal_load(yr + k * K); dyv[k] = A(0); }
    Sig::bwd(xv, yv, UniformLoad<Z, V>{dz + r * Z, scale}, dxv, dyv, cf);
    if (!t.on) return;
    V *dxr = dx + r * (X * K) + c0;
    V *dyr = dy + r * (Y * K) + c0;
#pragma unroll
    for (int j = 0; j < X; j++) __builtin_nontemporal_store((V)dxv[j], dxr + j * K);
#pragma unroll
    for (int k = 0; k < Y; k++) __builtin_nontemporal_store((V)dyv[k], dyr + k * K);
}

// 16 or 32 channels, kinds that sum over the channels: the groups of K lanes reduce on their
// own and store their own row; no slices to combine.
template <typename Sig, int K, int WPB>
__global__ __launch_bounds__(kWave * WPB) void tp_unrolled_bwd_uniform_narrow_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ dz,
    float *__restrict__ dx, float *__restrict__ dy, int64_t rows, float scale) {
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z;
    using Red = WaveReduceBlocks<Y, K>;
    const int64_t item = tp_uniform((int64_t)blockIdx.x * WPB + threadIdx.y);
    if (item >= TpTile<K>::items(rows)) return;
    const int lane = threadIdx.x;
    const TpTile<K> t(item, lane, rows);
    const int64_t r = t.r;
    float yv[Y], dyv[Red::P], xv[X], dxv[X];
    const float *yr = y + r * Y;
#pragma unroll
    for (int k = 0; k < Y; k++) yv[k] = yr[k];
#pragma unroll
    for (int k = 0; k < Red::P; k++) dyv[k] = 0.f;
    const float *xr = x + r * (X * K) + t.c0;
#pragma unroll
    for (int j = 0; j < X; j++) { xv[j] = __builtin_nontemporal_load(xr + j * K); dxv[j] = 0.f; }
    Sig::bwd(xv, yv, RowLoad<K>{dz + r * (Z * K) + t.c0, scale}, dxv, dyv);
    if (t.on) {
        float *dxr = dx + r * (X * K) + t.c0;
#pragma unroll
        for (int j = 0; j < X; j++) __builtin_nontemporal_store(dxv[j], dxr + j * K);
    }
    const bool on = t.on;
    float *dyr = dy + r * Y;
    Red::run(dyv, lane, [&](int k, float total) { if (on) dyr[k] = total; });
}

template <typename Sig, int K, int WPB>
__global__ __launch_bounds__(kWave * WPB) void tp_unrolled_fwd_inner_narrow_kernel(
    const float *__restrict__ x, const float *__restrict__ y, float *__restrict__ z, int64_t rows, float scale) {
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z;
    using Red = WaveReduceBlocks<Z, K>;
    const int64_t item = tp_uniform((int64_t)blockIdx.x * WPB + threadIdx.y);
    if (item >= TpTile<K>::items(rows)) return;
    const int lane = threadIdx.x;
    const TpTile<K> t(item, lane, rows);
    const int64_t r = t.r;
    float xv[X], yv[Y], zv[Red::P];
    const float *xr = x + r * (X * K) + t.c0;
    const float *yr = y + r * (Y * K) + t.c0;
#pragma unroll
    for (int j = 0; j < X; j++) xv[j] = __builtin_nontemporal_load(xr + j * K) * scale;
#pragma unroll
    for (int k = 0; k < Y; k++) yv[k] = __builtin_nontemporal_load(yr + k * K);
#pragma unroll
    for (int i = Z; i < Red::P; i++) zv[i] = 0.f;
    Sig::fwd(xv, yv, RegStore<Z>{zv});
    const bool on = t.on;
    float *zr = z + r * Z;
    Red::run(zv, lane, [&](int i, float total) { if (on) zr[i] = total; });
}

inline int tp_grid(int64_t items, int wpb, unsigned *blocks) {
    const int64_t b = (items + wpb - 1) / wpb;
    if (b > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "tensor_product: too many rows for one launch");
    *blocks = (unsigned)b;
    return E3J_AMD_OK;
}

// kKind: 0 MAP, 1 OUTER with a channel-free y, 2 INNER; V: the type the values are held in
template <typename Sig, int K, int kKind, typename V>
int launch_tp_unrolled_fwd_t(int64_t rows, tp_arith<V> scale, const tp_coefs<V> &cf, const V *x, const V *y, V *z,
                             hipStream_t stream) {
    constexpr int WPB = 4;
    if (rows == 0) return E3J_AMD_OK;
    unsigned blocks;
    if constexpr (kKind == 2 && TpTile<K>::SUB > 1) {
        static_assert(std::is_same<V, float>::value, "16 / 32 channels: float32 only");
        if (int rc = tp_grid(TpTile<K>::items(rows), WPB, &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_fwd_inner_narrow_kernel<Sig, K, WPB>), dim3(blocks), dim3(kWave, WPB), 0,
                           stream, x, y, z, rows, scale);
    } else if constexpr (kKind == 2) {
        using G = TpUniformGeometry<K>;
        if (int rc = tp_grid(rows, G::RPB, &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_fwd_inner_kernel<Sig, K, V>), dim3(blocks), dim3(kWave, G::WPB), 0, stream,
                           x, y, z, rows, scale, cf);
    } else {
        if (int rc = tp_grid(TpTile<K>::items(rows), WPB, &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_fwd_kernel<Sig, K, WPB, kKind == 1, V>), dim3(blocks), dim3(kWave, WPB), 0,
                           stream, x, y, z, rows, scale, cf);
    }
    return check_hip(hipGetLastError(), "tensor_product (unrolled) launch");
}

template <typename Sig, int K, int kKind, typename V>
int launch_tp_unrolled_bwd_t(int64_t rows, tp_arith<V> scale, const tp_coefs<V> &cf, const V *x, const V *y,
                             const V *dz, V *dx, V *dy, hipStream_t stream) {
    constexpr int WPB = 4;
    if (rows == 0) return E3J_AMD_OK;
    unsigned blocks;
    if constexpr (kKind == 2) {
        if (int rc = tp_grid(TpTile<K>::items(rows), WPB, &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_bwd_inner_kernel<Sig, K, WPB, V>), dim3(blocks), dim3(kWave, WPB), 0, stream,
                           x, y, dz, dx, dy, rows, scale, cf);
    } else if constexpr (kKind == 1 && TpTile<K>::SUB > 1) {
        static_assert(std::is_same<V, float>::value, "16 / 32 channels: float32 only");
        if (int rc = tp_grid(TpTile<K>::items(rows), WPB, &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_bwd_uniform_narrow_kernel<Sig, K, WPB>), dim3(blocks), dim3(kWave, WPB), 0,
                           stream, x, y, dz, dx, dy, rows, scale);
    } else if constexpr (kKind == 1) {
        using G = TpUniformGeometry<K>;
        if (int rc = tp_grid(rows, G::RPB, &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_bwd_uniform_kernel<Sig, K, V>), dim3(blocks), dim3(kWave, G::WPB), 0, stream,
                           x, y, dz, dx, dy, rows, scale, cf);
    } else {
        if (int rc = tp_grid(TpTile<K>::items(rows), WPB, &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_bwd_map_kernel<Sig, K, WPB, V>), dim3(blocks), dim3(kWave, WPB), 0, stream,
                           x, y, dz, dx, dy, rows, scale, cf);
    }
    return check_hip(hipGetLastError(), "tensor_product_bwd (unrolled) launch");
}

// the registry's entry points: float32, float16 (whole waves of channels), float64 (the same; the
// uniform factor of the table is part of its coefficient classes)
template <typename Sig, int K, int kKind>
int launch_tp_unrolled_fwd(int64_t rows, int, float scale, const float *x, const float *y, float *z,
                           hipStream_t stream) {
    return launch_tp_unrolled_fwd_t<Sig, K, kKind, float>(rows, scale, TpNoCoefs{}, x, y, z, stream);
}
template <typename Sig, int K, int kKind>
int launch_tp_unrolled_bwd(int64_t rows, int, float scale, const float *x, const float *y, const float *dz,
                           float *dx, float *dy, hipStream_t stream) {
    return launch_tp_unrolled_bwd_t<Sig, K, kKind, float>(rows, scale, TpNoCoefs{}, x, y, dz, dx, dy, stream);
}
template <typename Sig, int K, int kKind>
int launch_tp_unrolled_fwd_f16(int64_t rows, int, float scale, const half_t *x, const half_t *y, half_t *z,
                               hipStream_t stream) {
    return launch_tp_unrolled_fwd_t<Sig, K, kKind, half_t>(rows, scale, TpNoCoefs{}, x, y, z, stream);
}
template <typename Sig, int K, int kKind>
int launch_tp_unrolled_bwd_f16(int64_t rows, int, float scale, const half_t *x, const half_t *y, const half_t *dz,
                               half_t *dx, half_t *dy, hipStream_t stream) {
    return launch_tp_unrolled_bwd_t<Sig, K, kKind, half_t>(rows, scale, TpNoCoefs{}, x, y, dz, dx, dy, stream);
}
template <typename Sig, int K, int kKind>
int launch_tp_unrolled_fwd_f64(int64_t rows, int, const F64Coefs &classes, const double *x, const double *y,
                               double *z, hipStream_t stream) {
    return launch_tp_unrolled_fwd_t<Sig, K, kKind, double>(rows, 1.0, classes, x, y, z, stream);
}
template <typename Sig, int K, int kKind>
int launch_tp_unrolled_bwd_f64(int64_t rows, int, const F64Coefs &classes, const double *x, const double *y,
                               const double *dz, double *dx, double *dy, hipStream_t stream) {
    return launch_tp_unrolled_bwd_t<Sig, K, kKind, double>(rows, 1.0, classes, x, y, dz, dx, dy, stream);
}

// ---------------------------------------------------------------------------
// Leading-channels layout: x (R, K, X), y (R, K, Y) or (R, Y), z (R, K, Z).  The columns
// (r, c) are consecutive blocks of X (Y, Z) floats, so a wave takes 64 consecutive columns
// whatever the channel count: it moves their contiguous block with coalesced 16-byte
// accesses and turns it through its strip of LDS (odd row stride: conflict-free column
// access), runs the same generated arithmetic on registers, and turns the results back.
// The last tile is moved back to end at the last column; the columns it shares with the
// tile before receive the same values from both.  The register budgets in the launch bounds
// (resident waves per SIMD) are the measured optima: a fourth wave pays for the uniform-y
// forward and a third for the MAP backward despite a few spilled registers, nowhere else.
// ---------------------------------------------------------------------------
template <int X, int Y, int Z>
struct TpLeadingGeometry {
    static constexpr int PX = odd_stride(X), PY = odd_stride(Y), PZ = odd_stride(Z);
    static constexpr int XR = round4(kWave * PX), YR = round4(kWave * PY);
    static constexpr int GC = 16;  // columns of z / dz that pass through the strip at a time
    static constexpr int ZR = round4(GC * PZ);
    static constexpr int REGION = XR + YR > ZR ? XR + YR : ZR;
};

__device__ __forceinline__ int64_t tp_tile_start(int64_t tile, int64_t cols) {
    const int64_t c = tile * kWave;
    return c + kWave <= cols ? c : cols - kWave;
}

// columns of this wave into registers (x scaled); y from its strip, or per row when uniform
template <typename Sig, bool kUniformY>
__device__ __forceinline__ void tp_leading_operands(const float *__restrict__ x, const float *__restrict__ y,
                                                    int64_t col0, int K, float scale, float *strip, int lane,
                                                    float *xv, float *yv) {
    using G = TpLeadingGeometry<Sig::X, Sig::Y, Sig::Z>;
    float *strip_x = strip, *strip_y = strip + G::XR;
    LinearBlock<kWave * Sig::X> xl;
    xl.template load<true>(x + col0 * Sig::X, lane);
    xl.template to_strip<Sig::X, G::PX>(strip_x, lane);
    if (!kUniformY) {
        LinearBlock<kWave * Sig::Y> yl;
        yl.template load<true>(y + col0 * Sig::Y, lane);
        yl.template to_strip<Sig::Y, G::PY>(strip_y, lane);
    }
    strip_fence();
#pragma unroll
    for (int j = 0; j < Sig::X; j++) xv[j] = strip_x[lane * G::PX + j] * scale;
    if (kUniformY) {
        const float *yr = y + ((col0 + lane) / K) * Sig::Y;
#pragma unroll
        for (int k = 0; k < Sig::Y; k++) yv[k] = yr[k];
    } else {
#pragma unroll
        for (int k = 0; k < Sig::Y; k++) yv[k] = strip_y[lane * G::PY + k];
    }
}

template <typename Sig, int WPB, bool kUniformY>
__global__ __launch_bounds__(kWave * WPB, kUniformY ? 4 : 1) void tp_unrolled_fwd_leading_kernel(
    const float *__restrict__ x, const float *__restrict__ y, float *__restrict__ z, int64_t cols, int K,
    float scale) {
    constexpr int Z = Sig::Z;
    using G = TpLeadingGeometry<Sig::X, Sig::Y, Z>;
    __shared__ __attribute__((aligned(16))) float strips[WPB * G::REGION];
    float *strip = strips + threadIdx.y * G::REGION;
    const int lane = threadIdx.x;
    const int64_t tile = tp_uniform((int64_t)blockIdx.x * WPB + threadIdx.y);
    if (tile >= (cols + kWave - 1) / kWave) return;  // uniform per wave; no block barrier below
    const int64_t col0 = tp_tile_start(tile, cols);
    float xv[Sig::X], yv[Sig::Y], zv[Z];
    tp_leading_operands<Sig, kUniformY>(x, y, col0, K, scale, strip, lane, xv, yv);
    Sig::fwd(xv, yv, RegStore<Z>{zv});
#pragma unroll
    for (int q = 0; q < kWave / G::GC; q++) {
        strip_fence();  // the reads of the strip so far are done
        if (lane / G::GC == q) {
#pragma unroll
            for (int i = 0; i < Z; i++) strip[(lane % G::GC) * G::PZ + i] = zv[i];
        }
        strip_fence();
        LinearBlock<G::GC * Z> ol;
        ol.template from_strip<Z, G::PZ>(strip, lane);
        ol.store(z + (col0 + q * G::GC) * Z, lane);
    }
}

// cotangent columns of this wave into registers (scaled), 16 columns at a time through the strip
template <typename Sig>
__device__ __forceinline__ void tp_leading_cotangent(const float *__restrict__ dz, int64_t col0, float scale,
                                                     float *strip, int lane, float *dzv) {
    constexpr int Z = Sig::Z;
    using G = TpLeadingGeometry<Sig::X, Sig::Y, Z>;
#pragma unroll
    for (int q = 0; q < kWave / G::GC; q++) {
        LinearBlock<G::GC * Z> dl;
        dl.template load<true>(dz + (col0 + q * G::GC) * Z, lane);
        strip_fence();
        dl.template to_strip<Z, G::PZ>(strip, lane);
        strip_fence();
        if (lane / G::GC == q) {
#pragma unroll
            for (int i = 0; i < Z; i++) dzv[i] = strip[(lane % G::GC) * G::PZ + i] * scale;
        }
    }
}

// kInner: the cotangent is (rows, Z), one row per column's row (INNER mode)
template <typename Sig, int WPB, bool kInner>
__global__ __launch_bounds__(kWave * WPB, kInner ? 1 : 3) void tp_unrolled_bwd_map_leading_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ dz,
    float *__restrict__ dx, float *__restrict__ dy, int64_t cols, int K, float scale) {
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z;
    using G = TpLeadingGeometry<X, Y, Z>;
    __shared__ __attribute__((aligned(16))) float strips[WPB * G::REGION];
    float *strip = strips + threadIdx.y * G::REGION;
    const int lane = threadIdx.x;
    const int64_t tile = tp_uniform((int64_t)blockIdx.x * WPB + threadIdx.y);
    if (tile >= (cols + kWave - 1) / kWave) return;
    const int64_t col0 = tp_tile_start(tile, cols);
    float xv[X], yv[Y], dzv[Z], dxv[X], dyv[Y];
    tp_leading_operands<Sig, false>(x, y, col0, K, 1.f, strip, lane, xv, yv);
    if (kInner) {
        const float *zr = dz + ((col0 + lane) / K) * Z;
#pragma unroll
        for (int i = 0; i < Z; i++) dzv[i] = zr[i] * scale;
    } else {
        tp_leading_cotangent<Sig>(dz, col0, scale, strip, lane, dzv);
    }
#pragma unroll
    for (int j = 0; j < X; j++) dxv[j] = 0.f;
#pragma unroll
    for (int k = 0; k < Y; k++) dyv[k] = 0.f;
    Sig::bwd(xv, yv, RegLoad<Z>{dzv}, dxv, dyv);
    float *strip_x = strip, *strip_y = strip + G::XR;
    strip_fence();
#pragma unroll
    for (int j = 0; j < X; j++) strip_x[lane * G::PX + j] = dxv[j];
#pragma unroll
    for (int k = 0; k < Y; k++) strip_y[lane * G::PY + k] = dyv[k];
    strip_fence();
    LinearBlock<kWave * X> xl;
    xl.template from_strip<X, G::PX>(strip_x, lane);
    xl.store(dx + col0 * X, lane);
    LinearBlock<kWave * Y> yl;
    yl.template from_strip<Y, G::PY>(strip_y, lane);
    yl.store(dy + col0 * Y, lane);
}

// Uniform y, K = 64 * SL with SL in {1, 2, 4}: the SL tiles of a row sit in one block; each
// wave reduces its 64 channels and the first wave of the row adds the partial sums in a fixed order.
template <typename Sig, int WPB>
__global__ __launch_bounds__(kWave * WPB) void tp_unrolled_bwd_uniform_leading_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ dz,
    float *__restrict__ dx, float *__restrict__ dy, int64_t rows, int K, float scale) {
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z;
    using G = TpLeadingGeometry<X, Y, Z>;
    using Red = WaveReduceBlocks<Y>;
    __shared__ __attribute__((aligned(16))) float strips[WPB * G::REGION];
    __shared__ float partial[WPB][Red::P];
    float *strip = strips + threadIdx.y * G::REGION;
    const int lane = threadIdx.x, wave = threadIdx.y;
    const int sl = K / kWave, rpb = WPB / sl;
    const int slice = wave % sl;
    const int64_t r = tp_uniform((int64_t)blockIdx.x * rpb + wave / sl);
    const bool valid = r < rows;  // uniform per wave; every wave reaches the barrier
    if (valid) {
        const int64_t col0 = r * K + (int64_t)slice * kWave;
        float xv[X], yv[Y], dzv[Z], dxv[X], dyv[Red::P];
        tp_leading_operands<Sig, true>(x, y, col0, K, 1.f, strip, lane, xv, yv);
        tp_leading_cotangent<Sig>(dz, col0, scale, strip, lane, dzv);
#pragma unroll
        for (int j = 0; j < X; j++) dxv[j] = 0.f;
#pragma unroll
        for (int k = 0; k < Red::P; k++) dyv[k] = 0.f;
        Sig::bwd(xv, yv, RegLoad<Z>{dzv}, dxv, dyv);
        strip_fence();
#pragma unroll
        for (int j = 0; j < X; j++) strip[lane * G::PX + j] = dxv[j];
        strip_fence();
        LinearBlock<kWave * X> xl;
        xl.template from_strip<X, G::PX>(strip, lane);
        xl.store(dx + col0 * X, lane);
        float *mine = partial[wave];
        Red::run(dyv, lane, [&](int k, float total) { mine[k] = total; });
    }
    __syncthreads();
    if (valid && slice == 0 && lane < Y) {
        float total = partial[wave][lane];
        for (int s2 = 1; s2 < sl; s2++) total += partial[wave + s2][lane];
        dy[r * Y + lane] = total;
    }
}

// The same with the cotangent tile resident in LDS (64 columns x Z floats per wave) and read
// where the arithmetic needs it, instead of Z more registers per lane: three times the resident
// waves.  Two waves per block (25 KB each at Z = 99), so rows of at most 128 channels.
template <int X, int Y, int Z, int WPB>
struct TpCotangentTile {
    using G = TpLeadingGeometry<X, Y, Z>;
    static constexpr int TILE = round4(kWave * G::PZ);
    static constexpr int REGION = TILE > G::REGION ? TILE : G::REGION;
    static constexpr bool FITS = WPB * REGION * sizeof(float) <= 60 * 1024;  // static LDS of a block
};

template <int Z>
struct StripLoad {
    const float *column;
    float scale;
    template <int I>
    __device__ __forceinline__ float get() const { return column[I] * scale; }
};

template <typename Sig, int WPB>
__global__ __launch_bounds__(kWave * WPB) void tp_unrolled_bwd_uniform_leading_lds_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ dz,
    float *__restrict__ dx, float *__restrict__ dy, int64_t rows, int K, float scale) {
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z;
    using G = TpLeadingGeometry<X, Y, Z>;
    using Red = WaveReduceBlocks<Y>;
    using T = TpCotangentTile<X, Y, Z, WPB>;
    constexpr int REGION = T::REGION;
    if constexpr (!T::FITS) return;  // (never launched: the launcher takes the register form)
    __shared__ __attribute__((aligned(16))) float strips[T::FITS ? WPB * REGION : 4];
    __shared__ float partial[WPB][Red::P];
    float *strip = strips + threadIdx.y * REGION;
    const int lane = threadIdx.x, wave = threadIdx.y;
    const int sl = K / kWave, rpb = WPB / sl;
    const int slice = wave % sl;
    const int64_t r = tp_uniform((int64_t)blockIdx.x * rpb + wave / sl);
    const bool valid = r < rows;  // uniform per wave; every wave reaches the barrier
    if (valid) {
        const int64_t col0 = r * K + (int64_t)slice * kWave;
        float xv[X], yv[Y], dxv[X], dyv[Red::P];
        tp_leading_operands<Sig, true>(x, y, col0, K, 1.f, strip, lane, xv, yv);
        strip_fence();  // the operand columns are in registers: the strip takes the cotangent tile
#pragma unroll
        for (int q = 0; q < kWave / G::GC; q++) {
            LinearBlock<G::GC * Z> dl;
            dl.template load<true>(dz + (col0 + q * G::GC) * Z, lane);
            dl.template to_strip<Z, G::PZ>(strip + q * G::GC * G::PZ, lane);
        }
        strip_fence();
#pragma unroll
        for (int j = 0; j < X; j++) dxv[j] = 0.f;
#pragma unroll
        for (int k = 0; k < Red::P; k++) dyv[k] = 0.f;
        Sig::bwd(xv, yv, StripLoad<Z>{strip + lane * G::PZ, scale}, dxv, dyv);
        strip_fence();
#pragma unroll
        for (int j = 0; j < X; j++) strip[lane * G::PX + j] = dxv[j];
        strip_fence();
        LinearBlock<kWave * X> xl;
        xl.template from_strip<X, G::PX>(strip, lane);
        xl.store(dx + col0 * X, lane);
        float *mine = partial[wave];
        Red::run(dyv, lane, [&](int k, float total) { mine[k] = total; });
    }
    __syncthreads();
    if (valid && slice == 0 && lane < Y) {
        float total = partial[wave][lane];
        for (int s2 = 1; s2 < sl; s2++) total += partial[wave + s2][lane];
        dy[r * Y + lane] = total;
    }
}

// INNER forward, K = 64 * SL with SL in {1, 2, 4}: as the uniform-y backward, the tiles of a
// row sit in one block and their channel sums meet in LDS.
template <typename Sig, int WPB>
__global__ __launch_bounds__(kWave * WPB) void tp_unrolled_fwd_inner_leading_kernel(
    const float *__restrict__ x, const float *__restrict__ y, float *__restrict__ z, int64_t rows, int K,
    float scale) {
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z;
    using G = TpLeadingGeometry<X, Y, Z>;
    __shared__ __attribute__((aligned(16))) float strips[WPB * G::REGION];
    __shared__ float partial[WPB][Z];
    float *strip = strips + threadIdx.y * G::REGION;
    const int lane = threadIdx.x, wave = threadIdx.y;
    const int sl = K / kWave, rpb = WPB / sl;
    const int slice = wave % sl;
    const int64_t r = tp_uniform((int64_t)blockIdx.x * rpb + wave / sl);
    const bool valid = r < rows;  // uniform per wave; every wave reaches the barrier
    if (valid) {
        float xv[X], yv[Y], zv[Z];
        tp_leading_operands<Sig, false>(x, y, r * K + (int64_t)slice * kWave, K, scale, strip, lane, xv, yv);
        Sig::fwd(xv, yv, RegStore<Z>{zv});
        tp_reduce_columns<Z>(zv, partial[wave], lane);
    }
    __syncthreads();
    if (valid && slice == 0) {
        for (int i = lane; i < Z; i += kWave) {
            float total = partial[wave][i];
            for (int s2 = 1; s2 < sl; s2++) total += partial[wave + s2][i];
            z[r * Z + i] = total;
        }
    }
}

template <typename Sig, int kKind>
int launch_tp_unrolled_fwd_leading(int64_t rows, int channels, float scale, const float *x, const float *y,
                                   float *z, hipStream_t stream) {
    constexpr int WPB = 4;
    const int64_t cols = rows * channels;
    if (cols < kWave || !tp_leading_channels_ok(channels, kKind))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "tensor_product: channel count outside the leading-layout "
                                                   "kernels (a multiple of 4, at least 64 columns in all; "
                                                   "64, 128 or 256 where channels are summed)");
    unsigned blocks;
    if (kKind == 2) {
        if (int rc = tp_grid(rows, WPB / (channels / kWave), &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_fwd_inner_leading_kernel<Sig, WPB>), dim3(blocks), dim3(kWave, WPB), 0,
                           stream, x, y, z, rows, channels, scale);
    } else {
        if (int rc = tp_grid((cols + kWave - 1) / kWave, WPB, &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_fwd_leading_kernel<Sig, WPB, kKind == 1>), dim3(blocks), dim3(kWave, WPB), 0,
                           stream, x, y, z, cols, channels, scale);
    }
    return check_hip(hipGetLastError(), "tensor_product (unrolled, leading) launch");
}

template <typename Sig, int kKind>
int launch_tp_unrolled_bwd_leading(int64_t rows, int channels, float scale, const float *x, const float *y,
                                   const float *dz, float *dx, float *dy, hipStream_t stream) {
    constexpr int WPB = 4;
    const int64_t cols = rows * channels;
    if (cols < kWave || !tp_leading_channels_ok(channels, kKind))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "tensor_product_bwd: channel count outside the "
                                                   "leading-layout kernels");
    unsigned blocks;
    constexpr int PAIR = 2;  // waves per block of the kernel that keeps the cotangent tile in LDS
    if (kKind == 1 && channels <= PAIR * kWave && TpCotangentTile<Sig::X, Sig::Y, Sig::Z, PAIR>::FITS) {
        if (int rc = tp_grid(rows, PAIR / (channels / kWave), &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_bwd_uniform_leading_lds_kernel<Sig, PAIR>), dim3(blocks),
                           dim3(kWave, PAIR), 0, stream, x, y, dz, dx, dy, rows, channels, scale);
    } else if (kKind == 1) {
        if (int rc = tp_grid(rows, WPB / (channels / kWave), &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_bwd_uniform_leading_kernel<Sig, WPB>), dim3(blocks), dim3(kWave, WPB), 0,
                           stream, x, y, dz, dx, dy, rows, channels, scale);
    } else {
        if (int rc = tp_grid((cols + kWave - 1) / kWave, WPB, &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_bwd_map_leading_kernel<Sig, WPB, kKind == 2>), dim3(blocks),
                           dim3(kWave, WPB), 0, stream, x, y, dz, dx, dy, cols, channels, scale);
    }
    return check_hip(hipGetLastError(), "tensor_product_bwd (unrolled, leading) launch");
}

}  // namespace e3j_amd
#endif
