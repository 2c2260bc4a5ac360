// Kernel templates of the compile-time-unrolled row-wise tensor product (gfx950, float32,
// trailing-channels layout, channel counts that are multiples of 64).
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
    int32_t channels;
    int32_t uniform_y;    // 1: y has no channel axis (OUTER); 0: MAP
    const float *val;     // (num_coef) table values as float32
    const uint8_t *idx;   // (num_coef, 3) i, j, k
    int (*fwd)(int64_t rows, float scale, const float *x, const float *y, float *z, hipStream_t stream);
    int (*bwd)(int64_t rows, float scale, const float *x, const float *y, const float *dz, float *dx,
               float *dy, hipStream_t stream);
};
int num_tp_signatures();
const TpSignature &tp_signature(int id);

// Row of a (rows, dim, K) array seen by one lane: coordinate I lives at p[I * K].
template <int K>
struct RowStore {
    float *p;
    template <int I>
    __device__ __forceinline__ void put(float v) const { __builtin_nontemporal_store(v, p + I * K); }
};
template <int K>
struct RowLoad {
    const float *p;
    float scale;
    template <int I>
    __device__ __forceinline__ float get() const { return __builtin_nontemporal_load(p + I * K) * scale; }
};

__device__ __forceinline__ int64_t tp_uniform(int64_t v) {
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)(v & 0xffffffffu));
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)((unsigned long long)v >> 32));
    return (int64_t)(((unsigned long long)hi << 32) | lo);
}

template <typename Sig, int K, int WPB, bool kUniformY>
__global__ __launch_bounds__(kWave * WPB) void tp_unrolled_fwd_kernel(
    const float *__restrict__ x, const float *__restrict__ y, float *__restrict__ z, int64_t rows, float scale) {
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z, SL = K / kWave;
    static_assert(K % kWave == 0, "whole 64-channel slices");
    const int64_t item = tp_uniform((int64_t)blockIdx.x * WPB + threadIdx.y);
    if (item >= rows * SL) return;
    const int64_t r = item / SL;
    const int c0 = (int)(item % SL) * kWave + threadIdx.x;
    float xv[X], yv[Y];
    const float *xr = x + r * (X * K) + c0;
#pragma unroll
    for (int j = 0; j < X; j++) xv[j] = __builtin_nontemporal_load(xr + j * K) * scale;
    if (kUniformY) {
        const float *yr = y + r * Y;
#pragma unroll
        for (int k = 0; k < Y; k++) yv[k] = yr[k];
    } else {
        const float *yr = y + r * (Y * K) + c0;
#pragma unroll
        for (int k = 0; k < Y; k++) yv[k] = __builtin_nontemporal_load(yr + k * K);
    }
    Sig::fwd(xv, yv, RowStore<K>{z + r * (Z * K) + c0});
}

// MAP backward: dz is read once for both cotangents.
template <typename Sig, int K, int WPB>
__global__ __launch_bounds__(kWave * WPB) void tp_unrolled_bwd_map_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ dz,
    float *__restrict__ dx, float *__restrict__ dy, int64_t rows, float scale) {
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z, SL = K / kWave;
    const int64_t item = tp_uniform((int64_t)blockIdx.x * WPB + threadIdx.y);
    if (item >= rows * SL) return;
    const int64_t r = item / SL;
    const int c0 = (int)(item % SL) * kWave + threadIdx.x;
    float xv[X], yv[Y], dxv[X], dyv[Y];
    const float *xr = x + r * (X * K) + c0;
    const float *yr = y + r * (Y * K) + c0;
#pragma unroll
    for (int j = 0; j < X; j++) { xv[j] = __builtin_nontemporal_load(xr + j * K); dxv[j] = 0.f; }
#pragma unroll
    for (int k = 0; k < Y; k++) { yv[k] = __builtin_nontemporal_load(yr + k * K); dyv[k] = 0.f; }
    Sig::bwd(xv, yv, RowLoad<K>{dz + r * (Z * K) + c0, scale}, dxv, dyv);
    float *dxr = dx + r * (X * K) + c0;
    float *dyr = dy + r * (Y * K) + c0;
#pragma unroll
    for (int j = 0; j < X; j++) __builtin_nontemporal_store(dxv[j], dxr + j * K);
#pragma unroll
    for (int k = 0; k < Y; k++) __builtin_nontemporal_store(dyv[k], dyr + k * K);
}

// Uniform-y backward: a wave per (row, slice); dy (rows, Y) is the channel sum: every wave
// reduces its 64 channels, the slices of a row sit in one block and meet in LDS, and the
// first of them stores the row (fixed order, no atomics).
template <int K>
struct TpUniformGeometry {
    static constexpr int SL = K / kWave;              // waves per row
    static constexpr int RPB = SL >= 4 ? 1 : 4 / SL;  // rows per block
    static constexpr int WPB = SL * RPB;
};

template <typename Sig, int K>
__global__ __launch_bounds__(kWave * TpUniformGeometry<K>::WPB) void tp_unrolled_bwd_uniform_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ dz,
    float *__restrict__ dx, float *__restrict__ dy, int64_t rows, float scale) {
    constexpr int X = Sig::X, Y = Sig::Y, Z = Sig::Z;
    using G = TpUniformGeometry<K>;
    using Red = WaveReduce<Y>;
    __shared__ float partial[G::WPB][Red::P];
    const int wave = threadIdx.y, lane = threadIdx.x;
    const int slice = wave % G::SL;
    const int64_t r = tp_uniform((int64_t)blockIdx.x * G::RPB + wave / G::SL);
    const bool valid = r < rows;  // uniform per wave; every wave reaches the barrier
    if (valid) {
        float yv[Y], dyv[Red::P], xv[X], dxv[X];
        const float *yr = y + r * Y;
#pragma unroll
        for (int k = 0; k < Y; k++) yv[k] = to_vgpr(yr[k]);
#pragma unroll
        for (int k = 0; k < Red::P; k++) dyv[k] = 0.f;
        const int c0 = slice * kWave + lane;
        const float *xr = x + r * (X * K) + c0;
#pragma unroll
        for (int j = 0; j < X; j++) { xv[j] = __builtin_nontemporal_load(xr + j * K); dxv[j] = 0.f; }
        Sig::bwd(xv, yv, RowLoad<K>{dz + r * (Z * K) + c0, scale}, dxv, dyv);
        float *dxr = dx + r * (X * K) + c0;
#pragma unroll
        for (int j = 0; j < X; j++) __builtin_nontemporal_store(dxv[j], dxr + j * K);
        const float total = Red::run(dyv, lane);
        if (lane < 16) partial[wave][Red::slot(lane)] = total;
    }
    __syncthreads();
    if (valid && slice == 0 && lane < Y) {
        float total = partial[wave][lane];
#pragma unroll
        for (int s2 = 1; s2 < G::SL; s2++) total += partial[wave + s2][lane];
        dy[r * Y + lane] = total;
    }
}

inline int tp_grid(int64_t items, int wpb, unsigned *blocks) {
    const int64_t b = (items + wpb - 1) / wpb;
    if (b > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "tensor_product: too many rows for one launch");
    *blocks = (unsigned)b;
    return E3J_AMD_OK;
}

template <typename Sig, int K, bool kUniformY>
int launch_tp_unrolled_fwd(int64_t rows, float scale, const float *x, const float *y, float *z,
                           hipStream_t stream) {
    constexpr int WPB = 4;
    if (rows == 0) return E3J_AMD_OK;
    unsigned blocks;
    if (int rc = tp_grid(rows * (K / kWave), WPB, &blocks)) return rc;
    hipLaunchKernelGGL((tp_unrolled_fwd_kernel<Sig, K, WPB, kUniformY>), dim3(blocks), dim3(kWave, WPB), 0, stream,
                       x, y, z, rows, scale);
    return check_hip(hipGetLastError(), "tensor_product (unrolled) launch");
}

template <typename Sig, int K, bool kUniformY>
int launch_tp_unrolled_bwd(int64_t rows, float scale, const float *x, const float *y, const float *dz,
                           float *dx, float *dy, hipStream_t stream) {
    constexpr int WPB = 4;
    if (rows == 0) return E3J_AMD_OK;
    unsigned blocks;
    if (kUniformY) {
        using G = TpUniformGeometry<K>;
        if (int rc = tp_grid(rows, G::RPB, &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_bwd_uniform_kernel<Sig, K>), dim3(blocks), dim3(kWave, G::WPB), 0, stream,
                           x, y, dz, dx, dy, rows, scale);
    } else {
        if (int rc = tp_grid(rows * (K / kWave), WPB, &blocks)) return rc;
        hipLaunchKernelGGL((tp_unrolled_bwd_map_kernel<Sig, K, WPB>), dim3(blocks), dim3(kWave, WPB), 0, stream,
                           x, y, dz, dx, dy, rows, scale);
    }
    return check_hip(hipGetLastError(), "tensor_product_bwd (unrolled) launch");
}

}  // namespace e3j_amd
#endif
