// Kernel templates of the compile-time-unrolled convolution (gfx950, float32).
//
// A generated `Sig` type supplies the straight-line Clebsch-Gordan arithmetic of
// one irreps signature (`edge_fwd`, `edge_bwd`); the templates here supply
// everything around it: the wave <-> (node, channel slice) mapping, coalesced
// row loads with the next edge prefetched while the current one is computed,
// register-resident accumulation over a receiver's edge segment, the single
// row write-back, the channel reduction of dy and the float atomics of dx.
//
// Mapping (trailing-channels layout): one 64-lane wavefront owns one receiver
// and a slice of 64*CPL consecutive channels; a lane owns CPL consecutive
// channels, so every row access is one fully coalesced 256*CPL-byte load.
// Waves never communicate (no LDS, no barrier): a block is only a bundle of
// WPB independent waves.  Everything indexed by the edge is wave-uniform
// (scalar registers / scalar loads).
#ifndef E3J_AMD_CSRC_UNROLLED_H_
#define E3J_AMD_CSRC_UNROLLED_H_

#include "common.h"

namespace e3j_amd {

template <int C>
struct Vec {
    float v[C];
};

template <int C>
__device__ __forceinline__ Vec<C> vzero() {
    Vec<C> r;
#pragma unroll
    for (int t = 0; t < C; t++) r.v[t] = 0.f;
    return r;
}
template <int C>
__device__ __forceinline__ Vec<C> vmul(const Vec<C> &a, float w) {
    Vec<C> r;
#pragma unroll
    for (int t = 0; t < C; t++) r.v[t] = a.v[t] * w;
    return r;
}
template <int C>
__device__ __forceinline__ Vec<C> vfma(const Vec<C> &a, float w, const Vec<C> &c) {
    Vec<C> r;
#pragma unroll
    for (int t = 0; t < C; t++) r.v[t] = fmaf(a.v[t], w, c.v[t]);
    return r;
}
template <int C>
__device__ __forceinline__ Vec<C> vmulv(const Vec<C> &a, const Vec<C> &b) {
    Vec<C> r;
#pragma unroll
    for (int t = 0; t < C; t++) r.v[t] = a.v[t] * b.v[t];
    return r;
}
template <int C>
__device__ __forceinline__ Vec<C> vfmav(const Vec<C> &a, const Vec<C> &b, const Vec<C> &c) {
    Vec<C> r;
#pragma unroll
    for (int t = 0; t < C; t++) r.v[t] = fmaf(a.v[t], b.v[t], c.v[t]);
    return r;
}
template <int C>
__device__ __forceinline__ float hsum(const Vec<C> &a) {
    float r = a.v[0];
#pragma unroll
    for (int t = 1; t < C; t++) r += a.v[t];
    return r;
}

template <int C>
__device__ __forceinline__ Vec<C> load_vec(const float *p);
template <>
__device__ __forceinline__ Vec<1> load_vec<1>(const float *p) {
    Vec<1> r;
    r.v[0] = *p;
    return r;
}
template <>
__device__ __forceinline__ Vec<2> load_vec<2>(const float *p) {
    const float2 t = *reinterpret_cast<const float2 *>(p);
    Vec<2> r;
    r.v[0] = t.x; r.v[1] = t.y;
    return r;
}
template <>
__device__ __forceinline__ Vec<4> load_vec<4>(const float *p) {
    const float4 t = *reinterpret_cast<const float4 *>(p);
    Vec<4> r;
    r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
    return r;
}
template <int C>
__device__ __forceinline__ void store_vec(float *p, const Vec<C> &a);
template <>
__device__ __forceinline__ void store_vec<1>(float *p, const Vec<1> &a) { *p = a.v[0]; }
template <>
__device__ __forceinline__ void store_vec<2>(float *p, const Vec<2> &a) {
    *reinterpret_cast<float2 *>(p) = make_float2(a.v[0], a.v[1]);
}
template <>
__device__ __forceinline__ void store_vec<4>(float *p, const Vec<4> &a) {
    *reinterpret_cast<float4 *>(p) = make_float4(a.v[0], a.v[1], a.v[2], a.v[3]);
}

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

constexpr int next_pow2_c(int n) { return n <= 1 ? 1 : 2 * next_pow2_c((n + 1) / 2); }

// Sum NV per-lane values over the 64 lanes of a wave.  Halving exchange: at each
// step a lane keeps one half of its values and receives the partner's partial sums
// of that half, so NV values cost about 2*NV exchanges instead of 6*NV.  On return
// the total of value k sits in v[0] of every lane whose `slot(lane)` equals k.
template <int NV>
struct WaveReduce {
    static constexpr int P = next_pow2_c(NV) > 64 ? 64 : next_pow2_c(NV);
    static_assert(NV <= 64, "at most 64 values");
    __device__ static __forceinline__ int slot(int lane) {
        int k = 0;
        int off = 32;
#pragma unroll
        for (int n = P; n > 1; n >>= 1, off >>= 1) k = 2 * k + ((lane & off) ? 1 : 0);
        return k;
    }
    // number of low lane bits over which results are replicated
    static constexpr int replicated() { return 64 / P; }
    __device__ static __forceinline__ float run(float (&v)[P], int lane) {
        int off = 32;
#pragma unroll
        for (int n = P; n > 1; n >>= 1, off >>= 1) {
            const bool upper = (lane & off) != 0;
#pragma unroll
            for (int t = 0; t < n / 2; t++) {
                const float send = upper ? v[t] : v[t + n / 2];
                const float keep = upper ? v[t + n / 2] : v[t];
                v[t] = keep + __shfl_xor(send, off, kWave);
            }
        }
#pragma unroll
        for (; off > 0; off >>= 1) v[0] += __shfl_xor(v[0], off, kWave);
        return v[0];
    }
};

// ---------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------
template <typename Sig, int K, int CPL, int WPB>
__global__ __launch_bounds__(kWave *WPB) void unrolled_fwd_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ s,
    const int32_t *__restrict__ sender, const int32_t *__restrict__ row_ptr,
    const int32_t *__restrict__ perm, float *__restrict__ out, int num_nodes, float scale) {
    constexpr int X = Sig::X, Y = Sig::Y, S = Sig::S, Z = Sig::Z;
    constexpr int SLICE = kWave * CPL;
    constexpr int CW = (K + SLICE - 1) / SLICE;
    static_assert(K % CPL == 0, "channels must be a multiple of the per-lane vector width");
    using V = Vec<CPL>;

    const int lane = threadIdx.x;
    const int item = uniform(blockIdx.x * WPB + threadIdx.y);
    if (item >= num_nodes * CW) return;
    const int r = item / CW;
    const int c_raw = (item % CW) * SLICE + lane * CPL;
    // every lane owns channels when K fills whole slices: no predication in that case
    const bool active = (K % SLICE == 0) || c_raw < K;
    const int c0 = active ? c_raw : 0;  // idle lanes read channel 0 and never store

    V acc[Z];
#pragma unroll
    for (int i = 0; i < Z; i++) acc[i] = vzero<CPL>();

    int e = row_ptr[r];
    const int e1 = row_ptr[r + 1];

    V xn[X], sn[S];
    float yn[Y];
    bool valid_n = false;
    auto fetch = [&](int pos) {
        const int snd = sender[pos];
        valid_n = (unsigned)snd < (unsigned)num_nodes;
        const int row = valid_n ? snd : 0;
        const int64_t ee = perm ? (int64_t)perm[pos] : (int64_t)pos;
        const float *xr = x + (int64_t)row * (X * K) + c0;
        const float *sr = s + ee * (int64_t)(S * K) + c0;
        const float *yr = y + ee * Y;
#pragma unroll
        for (int j = 0; j < X; j++) xn[j] = load_vec<CPL>(xr + j * K);
#pragma unroll
        for (int l = 0; l < S; l++) sn[l] = load_vec<CPL>(sr + l * K);
#pragma unroll
        for (int k = 0; k < Y; k++) yn[k] = yr[k];
    };
    if (e < e1) fetch(e);
    while (e < e1) {
        V xc[X], sc[S];
        float yc[Y];
#pragma unroll
        for (int j = 0; j < X; j++) xc[j] = xn[j];
#pragma unroll
        for (int l = 0; l < S; l++) sc[l] = sn[l];
#pragma unroll
        for (int k = 0; k < Y; k++) yc[k] = yn[k];
        const bool valid = valid_n;
        e++;
        if (e < e1) fetch(e);
        if (valid) Sig::template edge_fwd<CPL>(xc, yc, sc, acc);
    }
    if (active) {
        float *orow = out + (int64_t)r * (Z * K) + c0;
#pragma unroll
        for (int i = 0; i < Z; i++) store_vec<CPL>(orow + i * K, vmul(acc[i], scale));
    }
}

// ---------------------------------------------------------------------------
// backward, receiver-grouped: dm row resident, x gathered, dx scattered by atomics
// ---------------------------------------------------------------------------
template <typename Sig, int K, int CPL, int WPB>
__global__ __launch_bounds__(kWave *WPB) void unrolled_bwd_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ s,
    const float *__restrict__ dm, const int32_t *__restrict__ sender,
    const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    float *__restrict__ dx, float *__restrict__ dy, float *__restrict__ ds, int num_nodes,
    float scale) {
    constexpr int X = Sig::X, Y = Sig::Y, S = Sig::S, Z = Sig::Z;
    constexpr int SLICE = kWave * CPL;
    constexpr int CW = (K + SLICE - 1) / SLICE;
    using V = Vec<CPL>;
    using Red = WaveReduce<Y>;

    const int lane = threadIdx.x;
    const int item = uniform(blockIdx.x * WPB + threadIdx.y);
    if (item >= num_nodes * CW) return;
    const int r = item / CW;
    const int c_raw = (item % CW) * SLICE + lane * CPL;
    const bool active = (K % SLICE == 0) || c_raw < K;
    const int c0 = active ? c_raw : 0;

    V dmr[Z];
    {
        const float *zr = dm + (int64_t)r * (Z * K) + c0;
#pragma unroll
        for (int i = 0; i < Z; i++) {
            dmr[i] = vmul(load_vec<CPL>(zr + i * K), scale);
            if (!active) dmr[i] = vzero<CPL>();  // idle lanes must add nothing to dy
        }
    }

    int e = row_ptr[r];
    const int e1 = row_ptr[r + 1];

    V xn[X], sn[S];
    float yn[Y];
    bool valid_n = false;
    int snd_n = 0;
    int64_t ee_n = 0;
    auto fetch = [&](int pos) {
        const int snd = sender[pos];
        valid_n = (unsigned)snd < (unsigned)num_nodes;
        snd_n = valid_n ? snd : 0;
        ee_n = perm ? (int64_t)perm[pos] : (int64_t)pos;
        const float *xr = x + (int64_t)snd_n * (X * K) + c0;
        const float *sr = s + ee_n * (int64_t)(S * K) + c0;
        const float *yr = y + ee_n * Y;
#pragma unroll
        for (int j = 0; j < X; j++) xn[j] = load_vec<CPL>(xr + j * K);
#pragma unroll
        for (int l = 0; l < S; l++) sn[l] = load_vec<CPL>(sr + l * K);
#pragma unroll
        for (int k = 0; k < Y; k++) yn[k] = yr[k];
    };
    if (e < e1) fetch(e);
    while (e < e1) {
        V xc[X], sc[S];
        float yc[Y];
#pragma unroll
        for (int j = 0; j < X; j++) xc[j] = xn[j];
#pragma unroll
        for (int l = 0; l < S; l++) sc[l] = sn[l];
#pragma unroll
        for (int k = 0; k < Y; k++) yc[k] = yn[k];
        const bool valid = valid_n;
        const int snd = snd_n;
        const int64_t ee = ee_n;
        e++;
        if (e < e1) fetch(e);
        if (!valid) continue;  // padding edge: its dy/ds rows are zero-filled separately

        V dxe[X];
        float dye[Red::P];
        Sig::template edge_bwd<CPL, K>(xc, yc, sc, dmr, dxe, dye, ds + ee * (int64_t)(S * K) + c0,
                                       active);
#pragma unroll
        for (int k = Y; k < Red::P; k++) dye[k] = 0.f;

        if (active) {
            float *dxr = dx + (int64_t)snd * (X * K) + c0;
#pragma unroll
            for (int j = 0; j < X; j++) {
#pragma unroll
                for (int t = 0; t < CPL; t++) unsafeAtomicAdd(dxr + j * K + t, dxe[j].v[t]);
            }
        }
        const float total = Red::run(dye, lane);
        const int k = Red::slot(lane);
        if ((lane & (Red::replicated() - 1)) == 0 && k < Y) {
            if (CW == 1) dy[ee * Y + k] = total;
            else unsafeAtomicAdd(dy + ee * Y + k, total);  // dy zero-filled by the launcher
        }
    }
}

template <typename Sig, int K, int CPL, int WPB>
int launch_unrolled_fwd(const e3j_amd_conv_params &p, const float *x, const float *y, const float *s,
                        const int32_t *sender, const int32_t *row_ptr, const int32_t *perm,
                        float *out, hipStream_t stream) {
    constexpr int CW = (K + kWave * CPL - 1) / (kWave * CPL);
    const int64_t items = (int64_t)p.num_nodes * CW;
    const int64_t blocks = (items + WPB - 1) / WPB;
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: grid too large");
    hipLaunchKernelGGL((unrolled_fwd_kernel<Sig, K, CPL, WPB>), dim3((unsigned)blocks),
                       dim3(kWave, WPB), 0, stream, x, y, s, sender, row_ptr, perm, out,
                       p.num_nodes, p.coef_scale);
    return check_hip(hipGetLastError(), "convolution forward launch");
}

template <typename Sig, int K, int CPL, int WPB>
int launch_unrolled_bwd(const e3j_amd_conv_params &p, const float *x, const float *y, const float *s,
                        const float *dm, const int32_t *sender, const int32_t *row_ptr,
                        const int32_t *perm, float *dx, float *dy, float *ds, hipStream_t stream) {
    constexpr int CW = (K + kWave * CPL - 1) / (kWave * CPL);
    int rc = launch_fill_zero(dx, sizeof(float) * (size_t)p.num_nodes * Sig::X * K, stream);
    if (rc) return rc;
    if (CW > 1) {
        rc = launch_fill_zero(dy, sizeof(float) * (size_t)p.num_edges * Sig::Y, stream);
        if (rc) return rc;
    }
    rc = launch_zero_padding(p, sender, row_ptr, perm, dy, ds, stream);
    if (rc) return rc;
    const int64_t items = (int64_t)p.num_nodes * CW;
    const int64_t blocks = (items + WPB - 1) / WPB;
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution_bwd: grid too large");
    hipLaunchKernelGGL((unrolled_bwd_kernel<Sig, K, CPL, WPB>), dim3((unsigned)blocks),
                       dim3(kWave, WPB), 0, stream, x, y, s, dm, sender, row_ptr, perm, dx, dy, ds,
                       p.num_nodes, p.coef_scale);
    return check_hip(hipGetLastError(), "convolution backward launch");
}

}  // namespace e3j_amd
#endif
