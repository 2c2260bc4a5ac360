// float16 kernels of the compile-time-unrolled convolution (gfx950, trailing-channels layout).
//
// Values are held in memory as half and computed in float: the mapping, the generated
// Clebsch-Gordan arithmetic (`edge_fwd`, `edge_bwd` of the float kernels, literals and scale factor
// included) and the register-resident sums are those of unrolled.h; only the row accesses differ.  A
// lane holds CPL consecutive channels (two where the channel count is a multiple of 128: a wave
// moves 256-byte row pieces as half pairs; one at 64 channels) and converts on the way in and out.
// The reference computes in half (lib/e3j_ops/cuda/utils.cuh:108-112); float arithmetic on the
// half operands is at least as accurate.
//
// dx of the receiver-grouped backward is added with packed half atomics
// (global_atomic_pk_add_f16): a lane adds its two channels, or, with one channel per lane,
// neighbouring lanes pair up and the even lane adds both.  The
// dy row of an edge is stored directly when one wave covers the edge, else added with the same
// packed atomics by the lanes that hold the even components after the wave reduction.
#ifndef E3J_AMD_CSRC_UNROLLED_F16_H_
#define E3J_AMD_CSRC_UNROLLED_F16_H_

#include <hip/hip_fp16.h>

#include "unrolled.h"

namespace e3j_amd {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

template <int C>
__device__ __forceinline__ Vec<C> load_f16(const half_t *p);
template <>
__device__ __forceinline__ Vec<1> load_f16<1>(const half_t *p) {
    Vec<1> r;
    r.v[0] = (float)*p;
    return r;
}
template <>
__device__ __forceinline__ Vec<2> load_f16<2>(const half_t *p) {
    const half2_t h = *reinterpret_cast<const half2_t *>(p);
    Vec<2> r;
    r.v[0] = (float)h.x;
    r.v[1] = (float)h.y;
    return r;
}
template <int C>
__device__ __forceinline__ Vec<C> load_stream_f16(const half_t *p);
template <>
__device__ __forceinline__ Vec<1> load_stream_f16<1>(const half_t *p) {
    Vec<1> r;
    r.v[0] = (float)__builtin_nontemporal_load(p);
    return r;
}
template <>
__device__ __forceinline__ Vec<2> load_stream_f16<2>(const half_t *p) {
    const half2_t h = __builtin_nontemporal_load(reinterpret_cast<const half2_t *>(p));
    Vec<2> r;
    r.v[0] = (float)h.x;
    r.v[1] = (float)h.y;
    return r;
}
__device__ __forceinline__ void store_stream_f16(half_t *p, const Vec<1> &a) {
    __builtin_nontemporal_store((half_t)a.v[0], p);
}
__device__ __forceinline__ void store_stream_f16(half_t *p, const Vec<2> &a) {
    half2_t h;
    h.x = (half_t)a.v[0];
    h.y = (half_t)a.v[1];
    __builtin_nontemporal_store(h, reinterpret_cast<half2_t *>(p));
}
// Adds `mine` to p[0] and `next` to p[1] (p 4-byte aligned) in one packed request.
__device__ __forceinline__ void atomic_add_pair_f16(half_t *p, float mine, float next) {
    unsafeAtomicAdd(reinterpret_cast<__half2 *>(p), __floats2half2_rn(mine, next));
}

// Adds v to one half value whose row is only 2-byte aligned (dy rows of an odd number of
// components): compare-and-swap on the 32-bit word that holds it.
__device__ __forceinline__ void atomic_add_one_f16(half_t *p, float v) {
    const uintptr_t addr = reinterpret_cast<uintptr_t>(p);
    unsigned *word = reinterpret_cast<unsigned *>(addr & ~(uintptr_t)3);
    const bool upper = (addr & 2) != 0;
    unsigned seen = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    while (true) {
        const unsigned short bits = upper ? (unsigned short)(seen >> 16) : (unsigned short)(seen & 0xffffu);
        half_t cur;
        __builtin_memcpy(&cur, &bits, sizeof(cur));
        const half_t sum = (half_t)((float)cur + v);
        unsigned short out_bits;
        __builtin_memcpy(&out_bits, &sum, sizeof(sum));
        const unsigned want = upper ? (seen & 0xffffu) | ((unsigned)out_bits << 16) : (seen & 0xffff0000u) | out_bits;
        const unsigned prior = atomicCAS(word, seen, want);
        if (prior == seen) break;
        seen = prior;
    }
}

// ---------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------
template <typename Part, int K, int CPL>
__device__ __forceinline__ void unrolled_fwd_f16_part(
    const half_t *__restrict__ x, const half_t *__restrict__ y, const half_t *__restrict__ s,
    const int32_t *__restrict__ sender, const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    half_t *__restrict__ out, int num_nodes, float scale, unsigned y_flip, int r, int slice, int lane) {
    constexpr int NX = Part::NX, NS = Part::NS, NZ = Part::NZ, Y = Part::Y;
    constexpr int X = Part::X, S = Part::S, Z = Part::Z;
    using V = Vec<CPL>;
    const int c0 = (slice * kWave + lane) * CPL;

    V acc[NZ];
#pragma unroll
    for (int i = 0; i < NZ; i++) acc[i] = vzero<CPL>();

    int e = row_ptr[r];
    const int e1 = row_ptr[r + 1];
    V xn[NX], sn[NS];
    float yn[Y];
    bool valid_n = false;
    auto fetch = [&](int pos) {
        const int snd = sender[pos];
        valid_n = (unsigned)snd < (unsigned)num_nodes;
        const int row = valid_n ? snd : 0;
        const int64_t ee = perm ? (int64_t)perm[pos] : (int64_t)pos;
        const half_t *xr = x + (int64_t)row * (X * K) + c0;
        const half_t *sr = s + ee * (int64_t)(S * K) + c0;
        const half_t *yr = y + ee * Y;
#pragma unroll
        for (int j = 0; j < NX; j++) xn[j] = load_f16<CPL>(xr + Part::kX[j] * K);
#pragma unroll
        for (int l = 0; l < NS; l++) sn[l] = load_stream_f16<CPL>(sr + Part::kS[l] * K);
#pragma unroll
        for (int k = 0; k < Y; k++) yn[k] = (float)yr[k];
    };
    if (e < e1) fetch(e);
    while (e < e1) {
        V xc[NX], sc[NS];
        float yc[Y];
#pragma unroll
        for (int j = 0; j < NX; j++) xc[j] = xn[j];
#pragma unroll
        for (int l = 0; l < NS; l++) sc[l] = sn[l];
#pragma unroll
        for (int k = 0; k < Y; k++) yc[k] = to_vgpr(flip_sign(yn[k], y_flip, k));
        const bool valid = valid_n;
        e++;
        if (e < e1) fetch(e);
        if (valid) Part::template edge_fwd<CPL>(xc, yc, sc, acc);
    }
    half_t *orow = out + (int64_t)r * (Z * K) + c0;
#pragma unroll
    for (int i = 0; i < NZ; i++) store_stream_f16(orow + Part::kZ[i] * K, vmul(acc[i], scale));
}

template <int K, int CPL, int I>
__device__ __forceinline__ void dispatch_fwd_f16(int, const half_t *, const half_t *, const half_t *, const int32_t *,
                                                 const int32_t *, const int32_t *, half_t *, int, float, unsigned,
                                                 int, int, int) {}
template <int K, int CPL, int I, typename Part, typename... Rest>
__device__ __forceinline__ void dispatch_fwd_f16(int part, const half_t *x, const half_t *y, const half_t *s,
                                                 const int32_t *sender, const int32_t *row_ptr, const int32_t *perm,
                                                 half_t *out, int num_nodes, float scale, unsigned y_flip, int r,
                                                 int slice, int lane) {
    if (part == I)
        unrolled_fwd_f16_part<Part, K, CPL>(x, y, s, sender, row_ptr, perm, out, num_nodes, scale, y_flip, r, slice,
                                            lane);
    else
        dispatch_fwd_f16<K, CPL, I + 1, Rest...>(part, x, y, s, sender, row_ptr, perm, out, num_nodes, scale, y_flip, r,
                                            slice, lane);
}

template <int K, int CPL, int WPB, typename... Parts>
__global__ __launch_bounds__(kWave *WPB) void unrolled_fwd_f16_kernel(
    const half_t *__restrict__ x, const half_t *__restrict__ y, const half_t *__restrict__ s,
    const int32_t *__restrict__ sender, const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ row_order, half_t *__restrict__ out, int num_nodes, float scale, unsigned y_flip) {
    static_assert(K % (kWave * CPL) == 0, "whole waves of channels");
    constexpr int NP = sizeof...(Parts);
    constexpr int CW = K / (kWave * CPL);
    const int64_t item = logical_block() * WPB + threadIdx.y;
    if (item >= (int64_t)num_nodes * (CW * NP)) return;
    const int part = uniform((int)(item % NP));
    const int slice = uniform((int)((item / NP) % CW));
    const int q = uniform((int)(item / (NP * CW)));
    const int r = row_order ? row_order[q] : q;
    dispatch_fwd_f16<K, CPL, 0, Parts...>(part, x, y, s, sender, row_ptr, perm, out, num_nodes, scale, y_flip, uniform(r),
                                     slice, threadIdx.x);
}

// ---------------------------------------------------------------------------
// backward, receiver-grouped
// ---------------------------------------------------------------------------
template <int K, int CPL>
struct DsRowsF16 {
    half_t *row;
    template <int L>
    __device__ __forceinline__ void put(const Vec<CPL> &v) const {
        store_stream_f16(row + L * K, v);
    }
};

template <typename Part, int K, int CPL, bool kAtomicDy>
__device__ __forceinline__ void unrolled_bwd_f16_part(
    const half_t *__restrict__ x, const half_t *__restrict__ y, const half_t *__restrict__ s,
    const half_t *__restrict__ dm, const int32_t *__restrict__ sender, const int32_t *__restrict__ row_ptr,
    const int32_t *__restrict__ perm, half_t *__restrict__ dx, half_t *__restrict__ dy, half_t *__restrict__ ds,
    int num_nodes, float scale, unsigned y_flip, int r, int slice, int lane) {
    constexpr int NX = Part::NX, NS = Part::NS, NZ = Part::NZ, Y = Part::Y;
    constexpr int X = Part::X, S = Part::S, Z = Part::Z;
    using V = Vec<CPL>;
    using Red = WaveReduceBlocks<Y, kWave>;
    const int c0 = (slice * kWave + lane) * CPL;

    V dmr[NZ];
    {
        const half_t *zr = dm + (int64_t)r * (Z * K) + c0;
#pragma unroll
        for (int i = 0; i < NZ; i++) dmr[i] = vmul(load_stream_f16<CPL>(zr + Part::kZ[i] * K), scale);
    }
    int e = row_ptr[r];
    const int e1 = row_ptr[r + 1];

    V xn[NX], sn[NS];
    float yn[Y];
    int snd_n = 0;
    int64_t ee_n = 0;
    auto fetch = [&](int pos) {
        snd_n = load_uniform(sender + pos);
        ee_n = perm ? (int64_t)load_uniform(perm + pos) : (int64_t)pos;
        const half_t *xr = x + (int64_t)snd_n * (X * K) + c0;
        const half_t *sr = s + ee_n * (int64_t)(S * K) + c0;
        const half_t *yr = y + ee_n * Y;
#pragma unroll
        for (int j = 0; j < NX; j++) xn[j] = load_f16<CPL>(xr + Part::kX[j] * K);
#pragma unroll
        for (int l = 0; l < NS; l++) sn[l] = load_stream_f16<CPL>(sr + Part::kS[l] * K);
#pragma unroll
        for (int k = 0; k < Y; k++) yn[k] = (float)yr[k];
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
        V xc[NX], sc[NS];
        float yc[Y];
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

        V dxe[NX];
        float dye[Red::P];
        const DsRowsF16<K, CPL> ds_rows{ds + ee * (int64_t)(S * K) + c0};
        Part::template edge_bwd<CPL>(xc, yc, sc, dmr, dxe, dye, ds_rows);
#pragma unroll
        for (int k = Y; k < Red::P; k++) dye[k] = 0.f;

        half_t *dxr = dx + (int64_t)snd * (X * K) + c0;
#pragma unroll
        for (int j = 0; j < NX; j++) {
            if (CPL == 2) {  // the lane's two channels in one packed request
                atomic_add_pair_f16(dxr + Part::kX[j] * K, dxe[j].v[0], dxe[j].v[CPL - 1]);
            } else {  // the even lane of a pair adds both channels (quad_perm [1,0,3,2] brings the odd one's value)
                const float next = dpp_move<0xB1>(dxe[j].v[0]);
                if ((lane & 1) == 0) atomic_add_pair_f16(dxr + Part::kX[j] * K, dxe[j].v[0], next);
            }
        }
        if (!kAtomicDy) {
            Red::run(dye, lane, [&](int k, float sum) { dy[ee * Y + k] = (half_t)flip_sign(sum, y_flip, k); });
        } else if (Y % 2 == 0) {
            // after the reduction lane L < 16 of a block of 16 values holds component slot(L) (the bits of
            // L reversed): lanes 0..7 hold the even components, lane L + 8 the one after it
            Red::run(dye, lane, [&](int k, float sum) {
                const float total = flip_sign(sum, y_flip, k);
                const float next = __shfl_down(total, 8, 16);
                if ((k & 1) == 0) atomic_add_pair_f16(dy + ee * Y + k, total, next);
            });
        } else {  // rows of an odd number of components are 2-byte aligned: one value at a time
            Red::run(dye, lane, [&](int k, float sum) { atomic_add_one_f16(dy + ee * Y + k, flip_sign(sum, y_flip, k)); });
        }
    }
}

template <int K, int CPL, bool A, int I>
__device__ __forceinline__ void dispatch_bwd_f16(int, const half_t *, const half_t *, const half_t *, const half_t *,
                                                 const int32_t *, const int32_t *, const int32_t *, half_t *,
                                                 half_t *, half_t *, int, float, unsigned, int, int, int) {}
template <int K, int CPL, bool A, int I, typename Part, typename... Rest>
__device__ __forceinline__ void dispatch_bwd_f16(int part, const half_t *x, const half_t *y, const half_t *s,
                                                 const half_t *dm, const int32_t *sender, const int32_t *row_ptr,
                                                 const int32_t *perm, half_t *dx, half_t *dy, half_t *ds,
                                                 int num_nodes, float scale, unsigned y_flip, int r, int slice,
                                                 int lane) {
    if (part == I)
        unrolled_bwd_f16_part<Part, K, CPL, A>(x, y, s, dm, sender, row_ptr, perm, dx, dy, ds, num_nodes, scale,
                                               y_flip, r, slice, lane);
    else
        dispatch_bwd_f16<K, CPL, A, I + 1, Rest...>(part, x, y, s, dm, sender, row_ptr, perm, dx, dy, ds, num_nodes,
                                               scale, y_flip, r, slice, lane);
}

template <int K, int CPL, int WPB, typename... Parts>
__global__ __launch_bounds__(kWave *WPB) void unrolled_bwd_f16_kernel(
    const half_t *__restrict__ x, const half_t *__restrict__ y, const half_t *__restrict__ s,
    const half_t *__restrict__ dm, const int32_t *__restrict__ sender, const int32_t *__restrict__ row_ptr,
    const int32_t *__restrict__ perm, const int32_t *__restrict__ row_order, half_t *__restrict__ dx,
    half_t *__restrict__ dy, half_t *__restrict__ ds, int num_nodes, float scale, unsigned y_flip) {
    static_assert(K % (kWave * CPL) == 0, "whole waves of channels");
    constexpr int NP = sizeof...(Parts);
    constexpr int CW = K / (kWave * CPL);
    constexpr bool kAtomicDy = NP * CW > 1;  // several waves add into one dy row
    const int64_t item = logical_block() * WPB + threadIdx.y;
    if (item >= (int64_t)num_nodes * (CW * NP)) return;
    const int part = uniform((int)(item % NP));
    const int slice = uniform((int)((item / NP) % CW));
    const int q = uniform((int)(item / (NP * CW)));
    const int r = row_order ? row_order[q] : q;
    dispatch_bwd_f16<K, CPL, kAtomicDy, 0, Parts...>(part, x, y, s, dm, sender, row_ptr, perm, dx, dy, ds, num_nodes,
                                                scale, y_flip, uniform(r), slice, threadIdx.x);
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
template <int K, int CPL, int WPB, typename... Parts>
int launch_unrolled_fwd_f16(const e3j_amd_conv_params &p, const half_t *x, const half_t *y, const half_t *s,
                            const int32_t *sender, const int32_t *row_ptr, const int32_t *perm, half_t *out,
                            hipStream_t stream) {
    constexpr int64_t PER_NODE = (int64_t)(K / (kWave * CPL)) * sizeof...(Parts);
    if (CPL > 1 && (reinterpret_cast<uintptr_t>(x) % 4 != 0 || reinterpret_cast<uintptr_t>(s) % 4 != 0 ||
                    reinterpret_cast<uintptr_t>(out) % 4 != 0))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: float16 operands must be 4-byte aligned");
    const int64_t blocks = padded_grid(((int64_t)p.num_nodes * PER_NODE + WPB - 1) / WPB);
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: grid too large");
    if (blocks == 0) return E3J_AMD_OK;
    hipLaunchKernelGGL((unrolled_fwd_f16_kernel<K, CPL, WPB, Parts...>), dim3((unsigned)blocks), dim3(kWave, WPB), 0,
                       stream, x, y, s, sender, row_ptr, perm, p.row_order, out, p.num_nodes, p.coef_scale, p.y_flip);
    return check_hip(hipGetLastError(), "convolution forward launch (float16)");
}

template <int K, int CPL, int WPB, int Y, int X, typename... Parts>
int launch_unrolled_bwd_f16(const e3j_amd_conv_params &p, const half_t *x, const half_t *y, const half_t *s,
                            const half_t *dm, const int32_t *sender, const int32_t *row_ptr, const int32_t *perm,
                            half_t *dx, half_t *dy, half_t *ds, hipStream_t stream) {
    constexpr int64_t PER_NODE = (int64_t)(K / (kWave * CPL)) * sizeof...(Parts);
    if (reinterpret_cast<uintptr_t>(dx) % 4 != 0 || (PER_NODE > 1 && reinterpret_cast<uintptr_t>(dy) % 4 != 0))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution_bwd: float16 dx and dy must be 4-byte aligned "
                                                   "(packed atomics)");
    if (CPL > 1 && (reinterpret_cast<uintptr_t>(x) % 4 != 0 || reinterpret_cast<uintptr_t>(s) % 4 != 0 ||
                    reinterpret_cast<uintptr_t>(dm) % 4 != 0 || reinterpret_cast<uintptr_t>(ds) % 4 != 0))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution_bwd: float16 operands must be 4-byte aligned");
    int rc = launch_fill_zero(dx, sizeof(half_t) * (size_t)p.num_nodes * X * K, stream);
    if (rc == E3J_AMD_OK && PER_NODE > 1) rc = launch_fill_zero(dy, sizeof(half_t) * (size_t)p.num_edges * Y, stream);
    if (rc) return rc;
    const int64_t blocks = padded_grid(((int64_t)p.num_nodes * PER_NODE + WPB - 1) / WPB);
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution_bwd: grid too large");
    if (blocks == 0) return E3J_AMD_OK;
    hipLaunchKernelGGL((unrolled_bwd_f16_kernel<K, CPL, WPB, Parts...>), dim3((unsigned)blocks), dim3(kWave, WPB), 0,
                       stream, x, y, s, dm, sender, row_ptr, perm, p.row_order, dx, dy, ds, p.num_nodes, p.coef_scale,
                       p.y_flip);
    return check_hip(hipGetLastError(), "convolution backward launch (float16)");
}

}  // namespace e3j_amd
#endif
