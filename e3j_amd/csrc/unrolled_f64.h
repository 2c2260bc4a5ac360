// float64 kernels of the compile-time-unrolled convolution (gfx950, trailing-channels layout).
//
// The same mapping as the float kernels of unrolled.h: one 64-lane wave owns one receiver, 64
// channels (a double per lane, which takes the registers of two float channels) and one part of
// the signature's paths; rows are whole 512-byte pieces, the next edge is fetched while the
// current one is computed, a receiver's segment is summed in registers and written once.  The
// backward gathers x, holds the receiver's dm rows and adds dx with float64 atomics.
//
// What differs is where the coefficients come from.  A float kernel carries the table's values as
// literals and takes one scale factor, which is exact to float32 rounding.  That is not good
// enough here: a table folded with a normalisation and stored in float32 (as the modules build
// it) is not a multiple of the built-in table to float64 accuracy.  The generated float64
// arithmetic (`edge_fwd_f64`, `edge_bwd_f64`) therefore reads one value per class of equal
// magnitude from a kernel argument (`F64Coefs`, at most 64 classes; the signs are structure),
// and the host fills it from the table at hand: any table with the structure of the signature is
// served exactly.
#ifndef E3J_AMD_CSRC_UNROLLED_F64_H_
#define E3J_AMD_CSRC_UNROLLED_F64_H_

#include "unrolled.h"

namespace e3j_amd {

using VD = Vec<1, double>;

__device__ __forceinline__ VD load_f64(const double *p) {
    VD r;
    r.v[0] = *p;
    return r;
}
__device__ __forceinline__ VD load_stream_f64(const double *p) {
    VD r;
    r.v[0] = __builtin_nontemporal_load(p);
    return r;
}
__device__ __forceinline__ void store_stream_f64(double *p, const VD &a) { __builtin_nontemporal_store(a.v[0], p); }

__device__ __forceinline__ double flip_sign(double v, unsigned flip, int k) {
    if (k >= 32) return v;  // the mask covers 32 components
    const unsigned long long bit = (unsigned long long)((flip >> k) & 1u) << 63;
    return __longlong_as_double((long long)((unsigned long long)__double_as_longlong(v) ^ bit));
}
__device__ __forceinline__ double to_vgpr(double v) {
    asm volatile("" : "+v"(v));
    return v;
}

// ---------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------
template <typename Part, int K>
__device__ __forceinline__ void unrolled_fwd_f64_part(
    const double *__restrict__ x, const double *__restrict__ y, const double *__restrict__ s,
    const int32_t *__restrict__ sender, const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    double *__restrict__ out, int num_nodes, unsigned y_flip, int r, int slice, int lane, const double *cf) {
    constexpr int NX = Part::NX, NS = Part::NS, NZ = Part::NZ, Y = Part::Y;
    constexpr int X = Part::X, S = Part::S, Z = Part::Z;
    const int c0 = slice * kWave + lane;

    VD acc[NZ];
#pragma unroll
    for (int i = 0; i < NZ; i++) acc[i] = vzero<1, double>();

    int e = row_ptr[r];
    const int e1 = row_ptr[r + 1];
    VD xn[NX], sn[NS];
    double yn[Y];
    bool valid_n = false;
    auto fetch = [&](int pos) {
        const int snd = sender[pos];
        valid_n = (unsigned)snd < (unsigned)num_nodes;
        const int row = valid_n ? snd : 0;
        const int64_t ee = perm ? (int64_t)perm[pos] : (int64_t)pos;
        const double *xr = x + (int64_t)row * (X * K) + c0;
        const double *sr = s + ee * (int64_t)(S * K) + c0;
        const double *yr = y + ee * Y;
#pragma unroll
        for (int j = 0; j < NX; j++) xn[j] = load_f64(xr + Part::kX[j] * K);
#pragma unroll
        for (int l = 0; l < NS; l++) sn[l] = load_stream_f64(sr + Part::kS[l] * K);
#pragma unroll
        for (int k = 0; k < Y; k++) yn[k] = yr[k];
    };
    if (e < e1) fetch(e);
    while (e < e1) {
        VD xc[NX], sc[NS];
        double yc[Y];
#pragma unroll
        for (int j = 0; j < NX; j++) xc[j] = xn[j];
#pragma unroll
        for (int l = 0; l < NS; l++) sc[l] = sn[l];
#pragma unroll
        for (int k = 0; k < Y; k++) yc[k] = to_vgpr(flip_sign(yn[k], y_flip, k));
        const bool valid = valid_n;
        e++;
        if (e < e1) fetch(e);
        if (valid) Part::edge_fwd_f64(xc, yc, sc, acc, cf);
    }
    double *orow = out + (int64_t)r * (Z * K) + c0;
#pragma unroll
    for (int i = 0; i < NZ; i++) store_stream_f64(orow + Part::kZ[i] * K, acc[i]);
}

template <int K, int I>
__device__ __forceinline__ void dispatch_fwd_f64(int, const double *, const double *, const double *, const int32_t *,
                                                 const int32_t *, const int32_t *, double *, int, unsigned, int, int,
                                                 int, const double *) {}
template <int K, int I, typename Part, typename... Rest>
__device__ __forceinline__ void dispatch_fwd_f64(int part, const double *x, const double *y, const double *s,
                                                 const int32_t *sender, const int32_t *row_ptr, const int32_t *perm,
                                                 double *out, int num_nodes, unsigned y_flip, int r, int slice,
                                                 int lane, const double *cf) {
    if (part == I)
        unrolled_fwd_f64_part<Part, K>(x, y, s, sender, row_ptr, perm, out, num_nodes, y_flip, r, slice, lane, cf);
    else
        dispatch_fwd_f64<K, I + 1, Rest...>(part, x, y, s, sender, row_ptr, perm, out, num_nodes, y_flip, r, slice,
                                            lane, cf);
}

// One wave per (receiver, 64 channels, part).  `scale` is unused (the coefficient classes carry
// the table's own values) and kept so that the argument list reads like the float kernels'.
template <int K, int WPB, typename... Parts>
__global__ __launch_bounds__(kWave *WPB) void unrolled_fwd_f64_kernel(
    const double *__restrict__ x, const double *__restrict__ y, const double *__restrict__ s,
    const int32_t *__restrict__ sender, const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ row_order, double *__restrict__ out, int num_nodes, double scale, unsigned y_flip,
    F64Coefs coefs) {
    static_assert(K % kWave == 0, "whole waves of channels");
    constexpr int NP = sizeof...(Parts);
    constexpr int CW = K / kWave;
    (void)scale;
    const int64_t item = logical_block() * WPB + threadIdx.y;
    if (item >= (int64_t)num_nodes * (CW * NP)) return;
    const int part = uniform((int)(item % NP));
    const int slice = uniform((int)((item / NP) % CW));
    const int q = uniform((int)(item / (NP * CW)));
    const int r = row_order ? row_order[q] : q;
    dispatch_fwd_f64<K, 0, Parts...>(part, x, y, s, sender, row_ptr, perm, out, num_nodes, y_flip, uniform(r), slice,
                                     threadIdx.x, coefs.v);
}

// ---------------------------------------------------------------------------
// backward, receiver-grouped
// ---------------------------------------------------------------------------
template <int K>
struct DsRowsF64 {
    double *row;
    template <int L>
    __device__ __forceinline__ void put(const VD &v) const {
        store_stream_f64(row + L * K, v);
    }
};

template <typename Part, int K, bool kAtomicDy>
__device__ __forceinline__ void unrolled_bwd_f64_part(
    const double *__restrict__ x, const double *__restrict__ y, const double *__restrict__ s,
    const double *__restrict__ dm, const int32_t *__restrict__ sender, const int32_t *__restrict__ row_ptr,
    const int32_t *__restrict__ perm, double *__restrict__ dx, double *__restrict__ dy, double *__restrict__ ds,
    int num_nodes, unsigned y_flip, int r, int slice, int lane, const double *cf) {
    constexpr int NX = Part::NX, NS = Part::NS, NZ = Part::NZ, Y = Part::Y;
    constexpr int X = Part::X, S = Part::S, Z = Part::Z;
    using Red = WaveReduceBlocks<Y, kWave, double>;
    const int c0 = slice * kWave + lane;

    VD dmr[NZ];
    {
        const double *zr = dm + (int64_t)r * (Z * K) + c0;
#pragma unroll
        for (int i = 0; i < NZ; i++) dmr[i] = load_stream_f64(zr + Part::kZ[i] * K);
    }
    int e = row_ptr[r];
    const int e1 = row_ptr[r + 1];

    VD xn[NX], sn[NS];
    double yn[Y];
    int snd_n = 0;
    int64_t ee_n = 0;
    auto fetch = [&](int pos) {
        snd_n = load_uniform(sender + pos);
        ee_n = perm ? (int64_t)load_uniform(perm + pos) : (int64_t)pos;
        const double *xr = x + (int64_t)snd_n * (X * K) + c0;
        const double *sr = s + ee_n * (int64_t)(S * K) + c0;
        const double *yr = y + ee_n * Y;
#pragma unroll
        for (int j = 0; j < NX; j++) xn[j] = load_f64(xr + Part::kX[j] * K);
#pragma unroll
        for (int l = 0; l < NS; l++) sn[l] = load_stream_f64(sr + Part::kS[l] * K);
#pragma unroll
        for (int k = 0; k < Y; k++) yn[k] = yr[k];
    };
    // padding edges (their dy / ds rows are zero-filled by the launcher) are stepped over on
    // wave-uniform values, so that the body is one straight line (see unrolled_bwd_part)
    auto next_edge = [&](int p) {
        while (p < e1 && !((unsigned)load_uniform(sender + p) < (unsigned)num_nodes)) p++;
        return p;
    };
    e = next_edge(e);
    if (e < e1) fetch(e);
    __builtin_amdgcn_s_waitcnt(kWaitVmcnt0);
    while (e < e1) {
        VD xc[NX], sc[NS];
        double yc[Y];
#pragma unroll
        for (int j = 0; j < NX; j++) xc[j] = xn[j];
#pragma unroll
        for (int l = 0; l < NS; l++) sc[l] = sn[l];
#pragma unroll
        for (int k = 0; k < Y; k++) yc[k] = to_vgpr(flip_sign(yn[k], y_flip, k));
        const int snd = snd_n;
        const int64_t ee = ee_n;
        e = next_edge(e + 1);
        if (e < e1) fetch(e);

        VD dxe[NX];
        double dye[Red::P];
        const DsRowsF64<K> ds_rows{ds + ee * (int64_t)(S * K) + c0};
        Part::edge_bwd_f64(xc, yc, sc, dmr, dxe, dye, ds_rows, cf);
#pragma unroll
        for (int k = Y; k < Red::P; k++) dye[k] = 0.0;

        double *dxr = dx + (int64_t)snd * (X * K) + c0;
#pragma unroll
        for (int j = 0; j < NX; j++) unsafeAtomicAdd(dxr + Part::kX[j] * K, dxe[j].v[0]);
        Red::run(dye, lane, [&](int k, double sum) {
            const double total = flip_sign(sum, y_flip, k);
            if (!kAtomicDy) dy[ee * Y + k] = total;
            else unsafeAtomicAdd(dy + ee * Y + k, total);  // dy zero-filled by the launcher
        });
    }
}

template <int K, bool A, int I>
__device__ __forceinline__ void dispatch_bwd_f64(int, const double *, const double *, const double *, const double *,
                                                 const int32_t *, const int32_t *, const int32_t *, double *,
                                                 double *, double *, int, unsigned, int, int, int, const double *) {}
template <int K, bool A, int I, typename Part, typename... Rest>
__device__ __forceinline__ void dispatch_bwd_f64(int part, const double *x, const double *y, const double *s,
                                                 const double *dm, const int32_t *sender, const int32_t *row_ptr,
                                                 const int32_t *perm, double *dx, double *dy, double *ds,
                                                 int num_nodes, unsigned y_flip, int r, int slice, int lane,
                                                 const double *cf) {
    if (part == I)
        unrolled_bwd_f64_part<Part, K, A>(x, y, s, dm, sender, row_ptr, perm, dx, dy, ds, num_nodes, y_flip, r,
                                          slice, lane, cf);
    else
        dispatch_bwd_f64<K, A, I + 1, Rest...>(part, x, y, s, dm, sender, row_ptr, perm, dx, dy, ds, num_nodes,
                                               y_flip, r, slice, lane, cf);
}

template <int K, int WPB, typename... Parts>
__global__ __launch_bounds__(kWave *WPB) void unrolled_bwd_f64_kernel(
    const double *__restrict__ x, const double *__restrict__ y, const double *__restrict__ s,
    const double *__restrict__ dm, const int32_t *__restrict__ sender, const int32_t *__restrict__ row_ptr,
    const int32_t *__restrict__ perm, const int32_t *__restrict__ row_order, double *__restrict__ dx,
    double *__restrict__ dy, double *__restrict__ ds, int num_nodes, double scale, unsigned y_flip,
    F64Coefs coefs) {
    static_assert(K % kWave == 0, "whole waves of channels");
    constexpr int NP = sizeof...(Parts);
    constexpr int CW = K / kWave;
    constexpr bool kAtomicDy = NP * CW > 1;  // several waves add into one dy row
    (void)scale;
    const int64_t item = logical_block() * WPB + threadIdx.y;
    if (item >= (int64_t)num_nodes * (CW * NP)) return;
    const int part = uniform((int)(item % NP));
    const int slice = uniform((int)((item / NP) % CW));
    const int q = uniform((int)(item / (NP * CW)));
    const int r = row_order ? row_order[q] : q;
    dispatch_bwd_f64<K, kAtomicDy, 0, Parts...>(part, x, y, s, dm, sender, row_ptr, perm, dx, dy, ds, num_nodes,
                                                y_flip, uniform(r), slice, threadIdx.x, coefs.v);
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
inline int f64_coefs(const e3j_amd_conv_params &p, F64Coefs *coefs, const char *op) {
    if (p.coef_classes == nullptr)
        return set_error(E3J_AMD_INVALID_ARGUMENT,
                         std::string(op) + ": float64 operands on an unrolled kernel need coef_classes (the values "
                                           "e3j_amd_find_signature_f64 returned for the table)");
    for (int m = 0; m < kF64Classes; m++) coefs->v[m] = p.coef_classes[m];
    return E3J_AMD_OK;
}

template <int K, int WPB, typename... Parts>
int launch_unrolled_fwd_f64(const e3j_amd_conv_params &p, const double *x, const double *y, const double *s,
                            const int32_t *sender, const int32_t *row_ptr, const int32_t *perm, double *out,
                            hipStream_t stream) {
    F64Coefs coefs;
    int rc = f64_coefs(p, &coefs, "convolution");
    if (rc) return rc;
    constexpr int64_t PER_NODE = (int64_t)(K / kWave) * sizeof...(Parts);
    const int64_t blocks = padded_grid(((int64_t)p.num_nodes * PER_NODE + WPB - 1) / WPB);
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: grid too large");
    if (blocks == 0) return E3J_AMD_OK;
    hipLaunchKernelGGL((unrolled_fwd_f64_kernel<K, WPB, Parts...>), dim3((unsigned)blocks), dim3(kWave, WPB), 0,
                       stream, x, y, s, sender, row_ptr, perm, p.row_order, out, p.num_nodes, 1.0, p.y_flip, coefs);
    return check_hip(hipGetLastError(), "convolution forward launch (float64)");
}

template <int K, int WPB, int Y, int X, typename... Parts>
int launch_unrolled_bwd_f64(const e3j_amd_conv_params &p, const double *x, const double *y, const double *s,
                            const double *dm, const int32_t *sender, const int32_t *row_ptr, const int32_t *perm,
                            double *dx, double *dy, double *ds, hipStream_t stream) {
    F64Coefs coefs;
    int rc = f64_coefs(p, &coefs, "convolution_bwd");
    if (rc) return rc;
    constexpr int64_t PER_NODE = (int64_t)(K / kWave) * sizeof...(Parts);
    rc = launch_fill_zero(dx, sizeof(double) * (size_t)p.num_nodes * X * K, stream);
    if (rc == E3J_AMD_OK && PER_NODE > 1) rc = launch_fill_zero(dy, sizeof(double) * (size_t)p.num_edges * Y, stream);
    if (rc) return rc;
    const int64_t blocks = padded_grid(((int64_t)p.num_nodes * PER_NODE + WPB - 1) / WPB);
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution_bwd: grid too large");
    if (blocks == 0) return E3J_AMD_OK;
    hipLaunchKernelGGL((unrolled_bwd_f64_kernel<K, WPB, Parts...>), dim3((unsigned)blocks), dim3(kWave, WPB), 0,
                       stream, x, y, s, dm, sender, row_ptr, perm, p.row_order, dx, dy, ds, p.num_nodes, 1.0,
                       p.y_flip, coefs);
    return check_hip(hipGetLastError(), "convolution backward launch (float64)");
}

}  // namespace e3j_amd
#endif
