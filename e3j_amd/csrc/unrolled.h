// Kernel templates of the compile-time-unrolled convolution (gfx950, float32).
//
// A generated `Sig` type supplies the straight-line Clebsch-Gordan arithmetic of
// one irreps signature (`edge_fwd`, `edge_bwd`); the templates here supply
// everything around it: the wave <-> (node, channel slice) mapping, coalesced
// row loads with the next edge prefetched while the current one is computed,
// register-resident accumulation over a receiver's edge segment, the single
// row write-back, the channel reduction of dy and the float atomics of dx.
//
// Mapping (trailing-channels layout): one 64-lane wavefront owns one receiver,
// a slice of 64*CPL channels and one part of the signature's paths; a lane owns
// CPL channels (consecutive in the forward, a wave apart in the backward), so
// every row access is a fully coalesced load of whole 256-byte row pieces.
// Waves never communicate (no LDS, no barrier): a block is only a bundle of
// WPB independent waves.  Everything indexed by the edge is wave-uniform
// (scalar registers / scalar loads).
//
// Mapping (leading-channels layout): the same arithmetic between two 90-degree
// turns of contiguous (channels, dim) blocks through LDS strips; see the
// section further down.
#ifndef E3J_AMD_CSRC_UNROLLED_H_
#define E3J_AMD_CSRC_UNROLLED_H_

#include <initializer_list>
#include <type_traits>

#include "common.h"

namespace e3j_amd {

// C values of scalar type T per lane (T = double: the float64 kernels of unrolled_f64.h, which
// share the generated arithmetic).
template <int C, typename T = float>
struct Vec {
    T v[C];
};
// (keeps a scalar argument out of template deduction: the vector operand fixes T)
template <typename T>
struct SameAs {
    using type = T;
};
template <typename T>
using same_t = typename SameAs<T>::type;
__device__ __forceinline__ float fma_t(float a, float b, float c) { return fmaf(a, b, c); }
__device__ __forceinline__ double fma_t(double a, double b, double c) { return fma(a, b, c); }

template <int C, typename T = float>
__device__ __forceinline__ Vec<C, T> vzero() {
    Vec<C, T> r;
#pragma unroll
    for (int t = 0; t < C; t++) r.v[t] = T(0);
    return r;
}
// Fixes the point in the instruction stream where `a` is computed: the value is an operand of
// an (empty) statement the compiler keeps in program order.  Without it the instruction
// selector emits a sum at its last use, and the operands of every term stay in registers
// until then.
template <int C, typename T>
__device__ __forceinline__ void pin(Vec<C, T> &a) {
#pragma unroll
    for (int t = 0; t < C; t++) asm volatile("" : "+v"(a.v[t]));
}
template <int C, typename T>
__device__ __forceinline__ Vec<C, T> vmul(const Vec<C, T> &a, same_t<T> w) {
    Vec<C, T> r;
#pragma unroll
    for (int t = 0; t < C; t++) r.v[t] = a.v[t] * w;
    return r;
}
template <int C, typename T>
__device__ __forceinline__ Vec<C, T> vfma(const Vec<C, T> &a, same_t<T> w, const Vec<C, T> &c) {
    Vec<C, T> r;
#pragma unroll
    for (int t = 0; t < C; t++) r.v[t] = fma_t(a.v[t], w, c.v[t]);
    return r;
}
template <int C, typename T>
__device__ __forceinline__ Vec<C, T> vmulv(const Vec<C, T> &a, const Vec<C, T> &b) {
    Vec<C, T> r;
#pragma unroll
    for (int t = 0; t < C; t++) r.v[t] = a.v[t] * b.v[t];
    return r;
}
template <int C, typename T>
__device__ __forceinline__ Vec<C, T> vfmav(const Vec<C, T> &a, const Vec<C, T> &b, const Vec<C, T> &c) {
    Vec<C, T> r;
#pragma unroll
    for (int t = 0; t < C; t++) r.v[t] = fma_t(a.v[t], b.v[t], c.v[t]);
    return r;
}
// sum over the channels of a lane of a * b (+ c): one fused multiply-add per channel
template <int C, typename T>
__device__ __forceinline__ T vdot(const Vec<C, T> &a, const Vec<C, T> &b, same_t<T> c) {
#pragma unroll
    for (int t = 0; t < C; t++) c = fma_t(a.v[t], b.v[t], c);
    return c;
}
template <int C, typename T>
__device__ __forceinline__ T vdot(const Vec<C, T> &a, const Vec<C, T> &b) {
    T c = a.v[0] * b.v[0];
#pragma unroll
    for (int t = 1; t < C; t++) c = fma_t(a.v[t], b.v[t], c);
    return c;
}
template <int C, typename T>
__device__ __forceinline__ T hsum(const Vec<C, T> &a) {
    T r = a.v[0];
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
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
// Loads and stores of data that is touched once (radial weights, output rows): marked
// non-temporal so that they do not displace the gathered sender rows from the L2.
template <int C>
__device__ __forceinline__ Vec<C> load_stream(const float *p);
template <>
__device__ __forceinline__ Vec<1> load_stream<1>(const float *p) {
    Vec<1> r;
    r.v[0] = __builtin_nontemporal_load(p);
    return r;
}
template <>
__device__ __forceinline__ Vec<2> load_stream<2>(const float *p) {
    const f32x2 t = __builtin_nontemporal_load(reinterpret_cast<const f32x2 *>(p));
    Vec<2> r;
    r.v[0] = t.x; r.v[1] = t.y;
    return r;
}
template <>
__device__ __forceinline__ Vec<4> load_stream<4>(const float *p) {
    const f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p));
    Vec<4> r;
    r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
    return r;
}
template <int C>
__device__ __forceinline__ void store_vec(float *p, const Vec<C> &a);
template <>
__device__ __forceinline__ void store_vec<1>(float *p, const Vec<1> &a) {
    *p = a.v[0];
}
template <>
__device__ __forceinline__ void store_vec<2>(float *p, const Vec<2> &a) {
    *reinterpret_cast<float2 *>(p) = make_float2(a.v[0], a.v[1]);
}
template <>
__device__ __forceinline__ void store_vec<4>(float *p, const Vec<4> &a) {
    *reinterpret_cast<float4 *>(p) = make_float4(a.v[0], a.v[1], a.v[2], a.v[3]);
}
template <int C>
__device__ __forceinline__ void store_stream(float *p, const Vec<C> &a);
template <>
__device__ __forceinline__ void store_stream<1>(float *p, const Vec<1> &a) {
    __builtin_nontemporal_store(a.v[0], p);
}
template <>
__device__ __forceinline__ void store_stream<2>(float *p, const Vec<2> &a) {
    f32x2 t;
    t.x = a.v[0]; t.y = a.v[1];
    __builtin_nontemporal_store(t, reinterpret_cast<f32x2 *>(p));
}
template <>
__device__ __forceinline__ void store_stream<4>(float *p, const Vec<4> &a) {
    f32x4 t;
    t.x = a.v[0]; t.y = a.v[1]; t.z = a.v[2]; t.w = a.v[3];
    __builtin_nontemporal_store(t, reinterpret_cast<f32x4 *>(p));
}

// Backward: the C channels of a lane lie a wave apart (lane, lane + 64, ...), so each of the C
// accesses of a wave is one coalesced 256-byte piece of a row and every float atomic request
// carries 16 values (atomics retire per 64-byte request, whatever it holds).
template <int C>
__device__ __forceinline__ Vec<C> load_apart(const float *p) {
    Vec<C> r;
#pragma unroll
    for (int t = 0; t < C; t++) r.v[t] = p[t * kWave];
    return r;
}
template <int C>
__device__ __forceinline__ Vec<C> load_apart_stream(const float *p) {
    Vec<C> r;
#pragma unroll
    for (int t = 0; t < C; t++) r.v[t] = __builtin_nontemporal_load(p + t * kWave);
    return r;
}
template <int C>
__device__ __forceinline__ void store_apart_stream(float *p, const Vec<C> &a) {
#pragma unroll
    for (int t = 0; t < C; t++) __builtin_nontemporal_store(a.v[t], p + t * kWave);
}

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// s_waitcnt operand on gfx9: vmcnt(0), the other counters left alone (expcnt 7, lgkmcnt 15).
constexpr int kWaitVmcnt0 = 0x0F70;

// One int32 at a wave-uniform address through the scalar data path, waited for on the spot.  For
// loads inside small search loops, which the compiler otherwise issues as vector loads whose wait
// (vmcnt is one in-order counter) would also wait for every store and atomic issued before.
__device__ __forceinline__ int load_uniform(const int32_t *p) {
    int v;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(p));
    return __builtin_amdgcn_readfirstlane(v);  // tells the compiler what the register class says
}

// Pin a wave-uniform value (scalar register) into a vector register.  A VALU operation
// reads at most one scalar or literal operand, so `literal * y` with y in a scalar
// register would make the compiler park every coefficient literal in a vector register
// for the whole kernel; with y in a vector register the literals stay inline.
// Negate v when bit k of `flip` is set (the parity signs of the y components when a kernel
// walks the edges of a symmetric graph in the reversed direction).
__device__ __forceinline__ float flip_sign(float v, unsigned flip, int k) {
    if (k >= 32) return v;  // the mask covers 32 components; tables with more carry their signs
    return __uint_as_float(__float_as_uint(v) ^ (((flip >> k) & 1u) << 31));
}

__device__ __forceinline__ float to_vgpr(float v) {
    asm volatile("" : "+v"(v));
    return v;
}

// Sum NV (<= 16) per-lane values over the 64 lanes of a wave with about 3*NV + 4
// VALU operations instead of 6*NV exchanges.  Halving exchange: at each of the four
// in-row steps a lane keeps one half of its values and adds the partner's partial sums
// of that half.  The partner comes from a DPP row permutation that flips the lane bit of
// the step and keeps the lower ones (xor 1, xor 2, rotate by 4, rotate by 8 within a row
// of 16), the half is picked with a bit-field insert under a per-lane
// mask (never a register-array select, which the compiler would lower to a chain of
// compares), and two cross-row exchanges finish the sum.  On return every lane holds
// in v[0] the total of value `slot(lane)`.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ double dpp_move(double v) {  // the two halves travel alike
    const int lo = __builtin_amdgcn_mov_dpp(__double2loint(v), CTRL, 0xf, 0xf, true);
    const int hi = __builtin_amdgcn_mov_dpp(__double2hiint(v), CTRL, 0xf, 0xf, true);
    return __hiloint2double(hi, lo);
}
// (a where mask is all ones, b where it is zero)
__device__ __forceinline__ float pick_bits(float a, float b, unsigned mask) {
    return __uint_as_float((__float_as_uint(a) & mask) | (__float_as_uint(b) & ~mask));
}
__device__ __forceinline__ double pick_bits(double a, double b, unsigned mask) {
    const unsigned long long m = (unsigned long long)(long long)(int)mask;
    return __longlong_as_double((long long)(((unsigned long long)__double_as_longlong(a) & m) |
                                            ((unsigned long long)__double_as_longlong(b) & ~m)));
}

template <int NV, int LANES = kWave, typename T = float>
struct WaveReduce {
    static_assert(NV >= 1 && NV <= 16, "at most 16 values");
    static_assert(LANES == 16 || LANES == 32 || LANES == 64, "sums run over groups of 16, 32 or 64 lanes");
    static constexpr int P = 16;  // values are padded to 16 by the caller
    __device__ static __forceinline__ int slot(int lane) {
        return ((lane & 1) << 3) | ((lane & 2) << 1) | ((lane & 4) >> 1) | ((lane & 8) >> 3);
    }
    template <int CTRL, int N>
    __device__ static __forceinline__ void level(T (&v)[P], unsigned upper) {
#pragma unroll
        for (int t = 0; t < N / 2; t++) {
            const T keep = pick_bits(v[t + N / 2], v[t], upper);
            const T send = pick_bits(v[t], v[t + N / 2], upper);
            v[t] = keep + dpp_move<CTRL>(send);
        }
    }
    __device__ static __forceinline__ T run(T (&v)[P], int lane) {
        level<0xB1, 16>(v, (lane & 1) ? ~0u : 0u);   // quad_perm [1,0,3,2]
        level<0x4E, 8>(v, (lane & 2) ? ~0u : 0u);    // quad_perm [2,3,0,1]
        level<0x124, 4>(v, (lane & 4) ? ~0u : 0u);   // row_ror:4 (the source lane differs in bit 2)
        level<0x128, 2>(v, (lane & 8) ? ~0u : 0u);   // row_ror:8 (= xor 8)
        if (LANES > 16) v[0] += __shfl_xor(v[0], 16, kWave);
        if (LANES > 32) v[0] += __shfl_xor(v[0], 32, kWave);
        return v[0];
    }
};

// Any number of values: sixteen at a time.  `sink(k, total)` is called on the first 16 lanes of
// every group of LANES lanes for the values k they hold (k < NV); `v` must be padded to a
// multiple of 16.
template <int NV, int LANES = kWave, typename T = float>
struct WaveReduceBlocks {
    static constexpr int P = (NV + 15) / 16 * 16;
    template <typename Sink>
    __device__ static __forceinline__ void run(T (&v)[P], int lane, const Sink &sink) {
        using Red = WaveReduce<16, LANES, T>;
#pragma unroll
        for (int base = 0; base < P; base += 16) {
            T part[16];
#pragma unroll
            for (int t = 0; t < 16; t++) part[t] = v[base + t];
            const T total = Red::run(part, lane);
            const int k = base + Red::slot(lane);
            if (lane % LANES < 16 && k < NV) sink(k, total);
        }
    }
};

// ---------------------------------------------------------------------------
// A generated `Part` covers a subset of the Clebsch-Gordan paths of a signature
// (all of them when the signature is not split).  It names the rows it touches:
//   kX[NX]  x coordinates it reads (and whose dx it produces)
//   kS[NS]  paths: rows of s it reads / of ds it writes
//   kZ[NZ]  output coordinates it accumulates (rows of out / dm)
// and supplies edge_fwd / edge_bwd on arrays indexed by those local positions.
// Splitting a signature over several waves divides the register-resident
// accumulators (out rows forward, dm rows backward) between them.
// ---------------------------------------------------------------------------

// Consecutive workgroups of a launch are dealt round-robin to the 8 XCDs, each with its own
// L2.  Logical block numbers are therefore handed out so that every XCD walks one contiguous
// eighth of the work list: rows that are neighbours in the list (and, with a locality-aware
// row order, in space) share an L2.  The grid is padded to a multiple of 8 blocks.
constexpr int kXcds = 8;
__device__ __forceinline__ int64_t logical_block() {
    const unsigned per_xcd = gridDim.x / kXcds;
    return (int64_t)(blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
}
inline int64_t padded_grid(int64_t blocks) { return (blocks + kXcds - 1) / kXcds * kXcds; }

template <int K, int CPL>
struct Slice {
    static constexpr int WIDTH = kWave * CPL;                 // channels per wave
    static constexpr int COUNT = (K + WIDTH - 1) / WIDTH;     // waves per row
    static constexpr bool FULL = (K % WIDTH) == 0;            // no idle lanes
    // Fewer channels than lanes (16 or 32, one per lane): the wave walks SUB edges of its row
    // side by side, one per group of K lanes, instead of idling the lanes past K.
    static constexpr int SUB = (CPL == 1 && (K == 16 || K == 32)) ? kWave / K : 1;
    static_assert(K % CPL == 0, "channels must be a multiple of the per-lane vector width");
};

template <typename First, typename...>
struct FirstOfParts {
    using type = First;
};

// ---------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------
template <typename Part, int K, int CPL>
__device__ __forceinline__ void unrolled_fwd_part(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ s,
    const int32_t *__restrict__ sender, const int32_t *__restrict__ row_ptr,
    const int32_t *__restrict__ perm, float *__restrict__ out, int num_nodes, float scale, unsigned y_flip, int r, int slice, int lane,
    int e, int e1, bool add) {
    // [e, e1): the positions of row r this wave sums; add: into `out` by float atomics (one of
    // several waves that share a long row) instead of storing the row
    constexpr int NX = Part::NX, NS = Part::NS, NZ = Part::NZ, Y = Part::Y;
    constexpr int X = Part::X, S = Part::S, Z = Part::Z;
    using V = Vec<CPL>;
    using SL = Slice<K, CPL>;
    constexpr int SUB = SL::SUB;

    const int sub = SUB > 1 ? lane / K : 0;  // which of the SUB edges walked side by side
    const int c_raw = SUB > 1 ? lane % K : slice * SL::WIDTH + lane * CPL;
    const bool active = SL::FULL || SUB > 1 || c_raw < K;
    const int c0 = active ? c_raw : 0;  // idle lanes read channel 0 and never store

    V acc[NZ];
#pragma unroll
    for (int i = 0; i < NZ; i++) acc[i] = vzero<CPL>();

    V xn[NX], sn[NS];
    float yn[Y];
    bool valid_n = false;
    auto fetch = [&](int base) {
        // SUB > 1: the group's own position; past the end of the row it re-reads the last
        // position and contributes nothing
        const bool inside = SUB == 1 || base + sub < e1;
        const int pos = SUB == 1 ? base : (inside ? base + sub : e1 - 1);
        const int snd = sender[pos];
        valid_n = inside && (unsigned)snd < (unsigned)num_nodes;
        const int row = valid_n ? snd : 0;
        const int64_t ee = perm ? (int64_t)perm[pos] : (int64_t)pos;
        const float *xr = x + (int64_t)row * (X * K) + c0;
        const float *sr = s + ee * (int64_t)(S * K) + c0;
        const float *yr = y + ee * Y;
#pragma unroll
        for (int j = 0; j < NX; j++) xn[j] = load_vec<CPL>(xr + Part::kX[j] * K);
#pragma unroll
        for (int l = 0; l < NS; l++) sn[l] = load_stream<CPL>(sr + Part::kS[l] * K);
#pragma unroll
        for (int k = 0; k < Y; k++) yn[k] = yr[k];
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
        e += SUB;
        if (e < e1) fetch(e);
        if (valid) Part::template edge_fwd<CPL>(xc, yc, sc, acc);
    }
    if (SUB > 1) {  // the groups hold partial sums over their edges: add them up
#pragma unroll
        for (int i = 0; i < NZ; i++) {
#pragma unroll
            for (int off = K; off < kWave; off *= 2) acc[i].v[0] += __shfl_xor(acc[i].v[0], off, kWave);
        }
    }
    if (active && sub == 0) {
        float *orow = out + (int64_t)r * (Z * K) + c0;
        if (!add) {
#pragma unroll
            for (int i = 0; i < NZ; i++) store_stream<CPL>(orow + Part::kZ[i] * K, vmul(acc[i], scale));
        } else {
#pragma unroll
            for (int i = 0; i < NZ; i++) {
#pragma unroll
                for (int t = 0; t < CPL; t++)
                    unsafeAtomicAdd(orow + Part::kZ[i] * K + t, acc[i].v[t] * scale);
            }
        }
    }
}

template <int K, int CPL, int I>
__device__ __forceinline__ void dispatch_fwd(int, const float *, const float *, const float *,
                                             const int32_t *, const int32_t *, const int32_t *,
                                             float *, int, float, unsigned, int, int, int, int, int,
                                             bool) {}
template <int K, int CPL, int I, typename Part, typename... Rest>
__device__ __forceinline__ void dispatch_fwd(int part, const float *x, const float *y, const float *s,
                                             const int32_t *sender, const int32_t *row_ptr,
                                             const int32_t *perm, float *out, int num_nodes,
                                             float scale, unsigned y_flip, int r, int slice, int lane,
                                             int e, int e1, bool add) {
    if (part == I)
        unrolled_fwd_part<Part, K, CPL>(x, y, s, sender, row_ptr, perm, out, num_nodes, scale, y_flip, r,
                                        slice, lane, e, e1, add);
    else
        dispatch_fwd<K, CPL, I + 1, Rest...>(part, x, y, s, sender, row_ptr, perm, out, num_nodes,
                                             scale, y_flip, r, slice, lane, e, e1, add);
}

// One wave per (receiver, channel slice, part); consecutive waves share a receiver.
// MINW: resident waves per SIMD the register allocation must leave room for (1 = no demand).
template <int K, int CPL, int WPB, int MINW, typename... Parts>
__global__ __launch_bounds__(kWave *WPB, MINW) void unrolled_fwd_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ s,
    const int32_t *__restrict__ sender, const int32_t *__restrict__ row_ptr,
    const int32_t *__restrict__ perm, const int32_t *__restrict__ row_order,
    float *__restrict__ out, int num_nodes, float scale, unsigned y_flip, int row_cap, int row_piece,
    const int32_t *__restrict__ segments, int max_segments) {
    // segments == nullptr: one item per row; a row longer than row_cap (> 0) is cut after
    // row_piece positions.
    // Otherwise the items are the listed pieces of long rows (count in segments[0], then
    // (row, begin, end) from segments[4] on), whose sums are added to `out`.
    constexpr int NP = sizeof...(Parts);
    constexpr int CW = Slice<K, CPL>::COUNT;
    const int64_t item = logical_block() * WPB + threadIdx.y;
    const int rows = segments ? min(segments[0], max_segments) : num_nodes;
    if (item >= (int64_t)rows * (CW * NP)) return;
    const int part = uniform((int)(item % NP));
    const int slice = uniform((int)((item / NP) % CW));
    const int q = uniform((int)(item / (NP * CW)));
    int r, e, e1;
    if (segments) {
        r = segments[4 + 3 * q];
        e = segments[5 + 3 * q];
        e1 = segments[6 + 3 * q];
    } else {
        r = row_order ? row_order[q] : q;
        e = row_ptr[r];
        e1 = row_ptr[r + 1];
        if (row_cap > 0 && e1 - e > row_cap) e1 = e + row_piece;
    }
    dispatch_fwd<K, CPL, 0, Parts...>(part, x, y, s, sender, row_ptr, perm, out, num_nodes, scale, y_flip,
                                      uniform(r), slice, threadIdx.x, uniform(e), uniform(e1),
                                      segments != nullptr);
}

// ---------------------------------------------------------------------------
// backward, receiver-grouped: dm rows resident, x gathered, dx scattered by atomics
// ---------------------------------------------------------------------------

// Where the generated arithmetic puts the ds value of path L (trailing layout: straight
// into the edge's row of ds).
template <int CPL, int K>
struct DsRows {
    float *row;
    bool active;
    template <int L>
    __device__ __forceinline__ void put(const Vec<CPL> &v) const {
        if (active) store_apart_stream<CPL>(row + L * K, v);
    }
};

template <typename Part, int K, int CPL, bool kAtomicDy, bool kOrdered>
__device__ __forceinline__ void unrolled_bwd_part(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ s,
    const float *__restrict__ dm, const int32_t *__restrict__ sender,
    const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    float *__restrict__ dx, float *__restrict__ dy, float *__restrict__ ds, int num_nodes,
    float scale, unsigned y_flip, int dy_slot, int dy_slots, int r, int slice, int lane) {
    // kOrdered: `dx` is the per-position contribution buffer and, when several waves share an
    // edge, `dy` the slot buffer (no atomics; fixed-order reductions follow)
    constexpr int NX = Part::NX, NS = Part::NS, NZ = Part::NZ, Y = Part::Y;
    constexpr int X = Part::X, S = Part::S, Z = Part::Z;
    using V = Vec<CPL>;
    using SL = Slice<K, CPL>;
    constexpr int SUB = SL::SUB;  // edges of the row walked side by side (channel counts below 64)
    using Red = WaveReduceBlocks<Y, kWave / SUB>;

    static_assert(CPL == 1 || SL::FULL, "several channels per lane need whole slices");
    const int sub = SUB > 1 ? lane / K : 0;
    const int c_raw = SUB > 1 ? lane % K : slice * SL::WIDTH + lane;  // further channels of the lane: + 64, + 128, ...
    const bool active = SL::FULL || SUB > 1 || c_raw < K;
    const int c0 = active ? c_raw : 0;

    V dmr[NZ];
    {
        const float *zr = dm + (int64_t)r * (Z * K) + c0;
#pragma unroll
        for (int i = 0; i < NZ; i++) {
            dmr[i] = vmul(load_apart_stream<CPL>(zr + Part::kZ[i] * K), scale);
            if (!active) dmr[i] = vzero<CPL>();  // idle lanes must add nothing to dy
        }
    }

    int e = row_ptr[r];
    const int e1 = row_ptr[r + 1];

    V xn[NX], sn[NS];
    float yn[Y];
    bool valid_n = false;
    int snd_n = 0, pos_n = 0;
    int64_t ee_n = 0;
    auto fetch = [&](int base) {
        // SUB > 1: the group's own position; past the end of the row it re-reads the last
        // position and does nothing with it
        const bool inside = SUB == 1 || base + sub < e1;
        const int pos = SUB == 1 ? base : (inside ? base + sub : e1 - 1);
        pos_n = pos;
        // (explicit scalar loads where the position is wave-uniform: see load_uniform)
        const int snd = SUB == 1 ? load_uniform(sender + pos) : sender[pos];
        valid_n = inside && (unsigned)snd < (unsigned)num_nodes;
        snd_n = valid_n ? snd : 0;
        ee_n = perm ? (int64_t)(SUB == 1 ? load_uniform(perm + pos) : perm[pos]) : (int64_t)pos;
        const float *xr = x + (int64_t)snd_n * (X * K) + c0;
        const float *sr = s + ee_n * (int64_t)(S * K) + c0;
        const float *yr = y + ee_n * Y;
#pragma unroll
        for (int j = 0; j < NX; j++) xn[j] = load_apart<CPL>(xr + Part::kX[j] * K);
#pragma unroll
        for (int l = 0; l < NS; l++) sn[l] = load_apart_stream<CPL>(sr + Part::kS[l] * K);
#pragma unroll
        for (int k = 0; k < Y; k++) yn[k] = yr[k];
    };
    // Padding edges (their dy/ds rows are zero-filled separately) are stepped over while looking
    // for the next edge, on wave-uniform values, so that the body below is one straight line
    // from the loads of the next edge to the stores and atomics of this one: the wait for those
    // loads at the top of the next turn then leaves the younger stores and atomics in flight.
    // (A branch around the body would make that wait a wait for everything, every edge.)
    auto next_edge = [&](int p) {
        if (SUB == 1)
            while (p < e1 && !((unsigned)load_uniform(sender + p) < (unsigned)num_nodes)) p++;
        return p;
    };
    e = next_edge(e);
    if (e < e1) fetch(e);
    // The first edge's operands are waited for here, before the loop: the loop is then entered
    // with nothing in flight, and the waits inside it are exact counts of what one turn issues.
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
        const bool valid = valid_n;
        const int snd = snd_n;
        const int64_t ee = ee_n;
        const int pos = pos_n;
        e = next_edge(e + SUB);
        if (e < e1) fetch(e);
        if (SUB > 1 && !valid) continue;  // (side-by-side edges: per group of lanes)

        V dxe[NX];
        float dye[Red::P];
        const DsRows<CPL, K> ds_rows{ds + ee * (int64_t)(S * K) + c0, active};
        Part::template edge_bwd<CPL>(xc, yc, sc, dmr, dxe, dye, ds_rows);
#pragma unroll
        for (int k = Y; k < Red::P; k++) dye[k] = 0.f;

        if (active) {
            if (kOrdered) {
                float *ur = dx + (int64_t)pos * (X * K) + c0;
#pragma unroll
                for (int j = 0; j < NX; j++) store_apart_stream<CPL>(ur + Part::kX[j] * K, dxe[j]);
            } else {
                float *dxr = dx + (int64_t)snd * (X * K) + c0;
#pragma unroll
                for (int j = 0; j < NX; j++) {
#pragma unroll
                    for (int t = 0; t < CPL; t++)
                        unsafeAtomicAdd(dxr + Part::kX[j] * K + t * kWave, dxe[j].v[t]);
                }
            }
        }
        Red::run(dye, lane, [&](int k, float sum) {
            const float total = flip_sign(sum, y_flip, k);
            if (!kAtomicDy) dy[ee * Y + k] = total;
            else if (kOrdered) dy[((int64_t)pos * dy_slots + dy_slot) * Y + k] = total;
            else unsafeAtomicAdd(dy + ee * Y + k, total);  // dy zero-filled by the launcher
        });
    }
}

template <int K, int CPL, bool A, bool O, int I>
__device__ __forceinline__ void dispatch_bwd(int, const float *, const float *, const float *,
                                             const float *, const int32_t *, const int32_t *,
                                             const int32_t *, float *, float *, float *, int, float,
                                             unsigned, int, int, int, int, int) {}
template <int K, int CPL, bool A, bool O, int I, typename Part, typename... Rest>
__device__ __forceinline__ void dispatch_bwd(int part, const float *x, const float *y, const float *s,
                                             const float *dm, const int32_t *sender,
                                             const int32_t *row_ptr, const int32_t *perm, float *dx,
                                             float *dy, float *ds, int num_nodes, float scale,
                                             unsigned y_flip, int dy_slot, int dy_slots,
                                             int r, int slice, int lane) {
    if (part == I)
        unrolled_bwd_part<Part, K, CPL, A, O>(x, y, s, dm, sender, row_ptr, perm, dx, dy, ds, num_nodes,
                                              scale, y_flip, dy_slot, dy_slots, r, slice, lane);
    else
        dispatch_bwd<K, CPL, A, O, I + 1, Rest...>(part, x, y, s, dm, sender, row_ptr, perm, dx, dy, ds,
                                                   num_nodes, scale, y_flip, dy_slot, dy_slots, r, slice,
                                                   lane);
}

template <int K, int CPL, int WPB, int MINW, bool kOrdered, typename... Parts>
__global__ __launch_bounds__(kWave *WPB, MINW)
void unrolled_bwd_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ s,
    const float *__restrict__ dm, const int32_t *__restrict__ sender,
    const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ row_order, float *__restrict__ dx, float *__restrict__ dy,
    float *__restrict__ ds, int num_nodes, float scale, unsigned y_flip) {
    constexpr int NP = sizeof...(Parts);
    constexpr int CW = Slice<K, CPL>::COUNT;
    constexpr bool kAtomicDy = NP * CW > 1;  // several waves add into one dy row
    const int64_t item = logical_block() * WPB + threadIdx.y;
    if (item >= (int64_t)num_nodes * (CW * NP)) return;
    const int part = uniform((int)(item % NP));
    const int slice = uniform((int)((item / NP) % CW));
    const int q = uniform((int)(item / (NP * CW)));
    const int r = row_order ? row_order[q] : q;
    dispatch_bwd<K, CPL, kAtomicDy, kOrdered, 0, Parts...>(part, x, y, s, dm, sender, row_ptr, perm, dx,
                                                           dy, ds, num_nodes, scale, y_flip,
                                                           part * CW + slice, NP * CW, r, slice,
                                                           threadIdx.x);
}

// ---------------------------------------------------------------------------
// backward, sender-grouped (the operands of the reference's "convolution_bwd"): the rows of the
// adjacency are senders.  A wave owns (sender, 64 channels): the sender's x row stays in
// registers, the dx sums of the row are kept in registers and stored once (no atomics, the
// same bits in every run), and the dm rows of every edge's receiver are gathered.  All parts
// of the signature run one after another in the wave (their dm rows are loaded per edge
// anyway), so an edge's dy is complete in the wave: stored directly at 64 channels and below,
// added by the K / 64 waves of an edge above (two addends at 128 channels: still the same
// bits in every run).  The gather of dm (Z rows per edge where the receiver-grouped kernels
// gather X) makes this the slower grouping; it needs no schedule, no workspace and no sort.
// ---------------------------------------------------------------------------
template <int K>
struct DsRowsScaled {  // one channel per lane: the edge's row of ds, values times `scale`
    float *row;
    bool active;
    float scale;
    template <int L>
    __device__ __forceinline__ void put(const Vec<1> &v) const {
        if (active) __builtin_nontemporal_store(v.v[0] * scale, row + L * K);
    }
};

template <typename Part, int K>
__device__ __forceinline__ void bwd_sender_stage(const Vec<1> *x_all, const float *yc, const float *sr,
                                                 const float *zr, Vec<1> *dx_all, float *dy_all,
                                                 const DsRowsScaled<K> &ds_rows, bool active) {
    constexpr int NX = Part::NX, NS = Part::NS, NZ = Part::NZ, Y = Part::Y;
    using V = Vec<1>;
    V xl[NX], dxl[NX], sl[NS], dml[NZ];
#pragma unroll
    for (int i = 0; i < NZ; i++) {
        dml[i] = load_vec<1>(zr + Part::kZ[i] * K);
        if (!active) dml[i] = vzero<1>();  // idle lanes must add nothing to dy
    }
#pragma unroll
    for (int l = 0; l < NS; l++) sl[l] = load_stream<1>(sr + Part::kS[l] * K);
#pragma unroll
    for (int j = 0; j < NX; j++) {
        xl[j] = x_all[Part::kX[j]];
        dxl[j] = dx_all[Part::kX[j]];
    }
    float dyp[Y];
    Part::template edge_bwd<1, true, false>(xl, yc, sl, dml, dxl, dyp, ds_rows);
#pragma unroll
    for (int j = 0; j < NX; j++) dx_all[Part::kX[j]] = dxl[j];
#pragma unroll
    for (int k = 0; k < Y; k++) dy_all[k] += dyp[k];
}

template <int K, int WPB, int MINW, typename... Parts>
__global__ __launch_bounds__(kWave *WPB, MINW) void unrolled_bwd_sender_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ s,
    const float *__restrict__ dm, const int32_t *__restrict__ receiver_t,
    const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ row_order, float *__restrict__ dx, float *__restrict__ dy,
    float *__restrict__ ds, int num_nodes, float scale, unsigned y_flip) {
    using P0 = typename FirstOfParts<Parts...>::type;
    constexpr int X = P0::X, Y = P0::Y, S = P0::S, Z = P0::Z;
    using SL = Slice<K, 1>;
    using V = Vec<1>;
    using Red = WaveReduceBlocks<Y, kWave>;
    constexpr int CW = SL::COUNT;
    const int64_t item = logical_block() * WPB + threadIdx.y;
    if (item >= (int64_t)num_nodes * CW) return;
    const int slice = uniform((int)(item % CW));
    const int q = uniform((int)(item / CW));
    const int r = uniform(row_order ? row_order[q] : q);
    const int lane = threadIdx.x;
    const int c_raw = slice * SL::WIDTH + lane;
    const bool active = SL::FULL || c_raw < K;
    const int c0 = active ? c_raw : 0;

    V xr[X], acc[X];
    {
        const float *xp = x + (int64_t)r * (X * K) + c0;
#pragma unroll
        for (int j = 0; j < X; j++) {
            xr[j] = load_vec<1>(xp + j * K);
            acc[j] = vzero<1>();
        }
    }
    const int e1 = row_ptr[r + 1];
    for (int pos = row_ptr[r]; pos < e1; pos++) {
        const int rcv = uniform(receiver_t[pos]);
        if (!((unsigned)rcv < (unsigned)num_nodes)) continue;  // padding edge: dy / ds zero-filled separately
        const int64_t ee = perm ? (int64_t)uniform(perm[pos]) : (int64_t)pos;
        const float *yr = y + ee * Y;
        float yc[Y], dye[Red::P];
#pragma unroll
        for (int k = 0; k < Y; k++) yc[k] = to_vgpr(flip_sign(yr[k], y_flip, k));
#pragma unroll
        for (int k = 0; k < Red::P; k++) dye[k] = 0.f;
        const DsRowsScaled<K> ds_rows{ds + ee * (int64_t)(S * K) + c0, active, scale};
        const float *sr = s + ee * (int64_t)(S * K) + c0;
        const float *zr = dm + (int64_t)rcv * (Z * K) + c0;
        (bwd_sender_stage<Parts, K>(xr, yc, sr, zr, acc, dye, ds_rows, active), ...);
        Red::run(dye, lane, [&](int k, float sum) {
            const float total = flip_sign(sum * scale, y_flip, k);
            if (CW == 1) dy[ee * Y + k] = total;
            else unsafeAtomicAdd(dy + ee * Y + k, total);  // dy zero-filled by the launcher
        });
    }
    if (active) {  // the row's dx, written once; coordinates no coefficient touches get zeros
        float *dxp = dx + (int64_t)r * (X * K) + c0;
#pragma unroll
        for (int j = 0; j < X; j++) dxp[j * K] = acc[j].v[0] * scale;
    }
}

// ---------------------------------------------------------------------------
// backward over tiles of receivers: dm rows of the tile resident in LDS, the tile's edges
// walked in sender order, dx summed in registers over the edges that share a sender
// ---------------------------------------------------------------------------
// Float atomics retire per 64-byte request at a fixed rate that bounds the receiver-grouped
// backward above.  Neighbouring receivers share most of their senders, so a block takes a
// tile of receivers that are consecutive in the row order (one part of the signature, one
// channel slice), keeps their dm rows in LDS, and walks the tile's edges sorted by sender
// (the schedule of `e3j_amd_tile_schedule_build`).  Its waves split that list at sender
// boundaries; a wave sums the dx contributions of the consecutive edges of one sender in
// registers and issues one set of atomics per (tile, sender) instead of one per edge, and
// gathers the sender's x row once.  dm is indexed from LDS by the edge's receiver, which
// also frees the registers the resident dm rows took.  ds and dy belong to the edge and
// are written as in the kernel above.  One barrier per block (after the tile is staged).

// The dm rows of one receiver of the tile as the generated arithmetic indexes them.
template <int CPL>
struct DmTile {
    const float *row;  // LDS: this lane's CPL values of the receiver's first staged row
    __device__ __forceinline__ Vec<CPL> operator[](int i) const {
        return load_vec<CPL>(row + i * (kWave * CPL));
    }
};

template <typename Part, int K, int CPL, bool kAtomicDy>
__device__ __forceinline__ void unrolled_bwd_tile_part(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ s,
    const float *__restrict__ dm, const int32_t *__restrict__ t_sender,
    const int32_t *__restrict__ t_edge, const int32_t *__restrict__ t_local,
    const int32_t *__restrict__ row_order, float *__restrict__ dx, float *__restrict__ dy,
    float *__restrict__ ds, int num_nodes, float scale, unsigned y_flip, int tile, int tile_rows,
    int begin, int end, int slice, float *tile_lds) {
    constexpr int NX = Part::NX, NS = Part::NS, NZ = Part::NZ, Y = Part::Y;
    constexpr int X = Part::X, S = Part::S, Z = Part::Z;
    using V = Vec<CPL>;
    using SL = Slice<K, CPL>;
    using Red = WaveReduceBlocks<Y, kWave>;
    constexpr int WIDTH = SL::WIDTH;
    static_assert(SL::SUB == 1, "the tile kernel takes whole waves of channels");
    static_assert(CPL == 1 || SL::FULL, "several channels per lane need whole slices");

    const int lane = threadIdx.x;
    const int wave = uniform(threadIdx.y), nw = blockDim.y;
    const int c_raw = slice * WIDTH + lane;  // further channels of the lane: + 64, + 128, ...
    const bool active = SL::FULL || c_raw < K;
    const int c0 = active ? c_raw : 0;

    // this wave's share of the list, cut at sender boundaries
    auto boundary = [&](int p) {
        if (p <= begin) return begin;
        while (p < end && load_uniform(t_sender + p) == load_uniform(t_sender + p - 1)) p++;
        return p;
    };
    const int n = end - begin;
    const int lo = boundary(begin + (int)((int64_t)n * wave / nw));
    int hi = boundary(begin + (int)((int64_t)n * (wave + 1) / nw));
    // padding edges (their dy/ds rows are zero-filled separately) are the tail of a tile's list:
    // the loop below never sees one, so its body is one straight line (see the kernel above)
    while (hi > lo && !((unsigned)load_uniform(t_sender + hi - 1) < (unsigned)num_nodes)) hi--;

    V xc[NX], xn[NX], sn[NS], acc[NX];
    float yn[Y];
    bool valid_n = false, newx_n = false;
    int snd_n = 0, loc_n = 0;
    int64_t ee_n = 0;
    // `held`: the sender whose x row the registers will hold when the fetched edge is computed
    // The indices of a position are read two positions ahead (scalar registers), so that the
    // loads of the next edge never wait for them.
    int snd_a = 0, ee_a = 0, loc_a = 0;
    auto read_indices = [&](int pos) {
        asm volatile("s_load_dword %0, %3, 0x0\n\ts_load_dword %1, %4, 0x0\n\ts_load_dword %2, %5, 0x0\n\t"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&s"(snd_a), "=&s"(ee_a), "=&s"(loc_a)
                     : "s"(t_sender + pos), "s"(t_edge + pos), "s"(t_local + pos));
        snd_a = uniform(snd_a);
        ee_a = uniform(ee_a);
        loc_a = uniform(loc_a);
    };
    auto fetch = [&](int held) {  // the edge whose indices were read last
        const int snd = snd_a;
        valid_n = true;  // (padding entries are cut off the range)
        snd_n = snd;
        ee_n = ee_a;
        loc_n = loc_a;
        newx_n = valid_n && snd != held;
        if (newx_n) {
            const float *xr = x + (int64_t)snd * (X * K) + c0;
#pragma unroll
            for (int j = 0; j < NX; j++) xn[j] = load_apart<CPL>(xr + Part::kX[j] * K);
        }
        const float *sr = s + ee_n * (int64_t)(S * K) + c0;
        const float *yr = y + ee_n * Y;
#pragma unroll
        for (int l = 0; l < NS; l++) sn[l] = load_apart_stream<CPL>(sr + Part::kS[l] * K);
#pragma unroll
        for (int k = 0; k < Y; k++) yn[k] = yr[k];
    };
    auto flush = [&](int snd) {
        if (!active) return;
        float *dxr = dx + (int64_t)snd * (X * K) + c0;
#pragma unroll
        for (int j = 0; j < NX; j++) {
#pragma unroll
            for (int t = 0; t < CPL; t++) unsafeAtomicAdd(dxr + Part::kX[j] * K + t * kWave, acc[j].v[t]);
        }
    };

    int held = -1, run = -1;
    if (lo < hi) {
        read_indices(lo);
        fetch(held);
        if (lo + 1 < hi) read_indices(lo + 1);
    }

    // stage the dm rows of the tile's receivers (scaled): row (t, i) at (t * NZ + i) * WIDTH
    {
        const int first = tile * tile_rows;
        const int rows = num_nodes - first < tile_rows ? num_nodes - first : tile_rows;
        for (int t = wave; t < rows; t += nw) {
            const int r = row_order ? row_order[first + t] : first + t;
            const float *zr = dm + (int64_t)r * (Z * K) + c0;
            float *dst = tile_lds + t * (NZ * WIDTH) + lane * CPL;
            V v[NZ];
#pragma unroll
            for (int i = 0; i < NZ; i++) v[i] = load_apart_stream<CPL>(zr + Part::kZ[i] * K);
#pragma unroll
            for (int i = 0; i < NZ; i++)  // idle lanes must add nothing to dy
                store_vec<CPL>(dst + i * WIDTH, active ? vmul(v[i], scale) : vzero<CPL>());
        }
    }
    __syncthreads();
    // entered with nothing in flight: the waits inside the loop are exact counts of one turn
    __builtin_amdgcn_s_waitcnt(kWaitVmcnt0);

    for (int pos = lo; pos < hi; pos++) {
        V sc[NS];
        float yc[Y];
        if (newx_n) {
#pragma unroll
            for (int j = 0; j < NX; j++) xc[j] = xn[j];
            held = snd_n;
        }
#pragma unroll
        for (int l = 0; l < NS; l++) sc[l] = sn[l];
#pragma unroll
        for (int k = 0; k < Y; k++) yc[k] = to_vgpr(flip_sign(yn[k], y_flip, k));
        const bool valid = valid_n;
        const int snd = snd_n, loc = loc_n;
        const int64_t ee = ee_n;
        if (pos + 1 < hi) {
            fetch(held);
            if (pos + 2 < hi) read_indices(pos + 2);
        }
        (void)valid;

        if (snd != run) {
            if (run >= 0) flush(run);
            run = snd;
#pragma unroll
            for (int j = 0; j < NX; j++) acc[j] = vzero<CPL>();
        }
        float dye[Red::P];
        const DsRows<CPL, K> ds_rows{ds + ee * (int64_t)(S * K) + c0, active};
        const DmTile<CPL> dm_rows{tile_lds + loc * (NZ * WIDTH) + lane * CPL};
        Part::template edge_bwd<CPL, true, true>(xc, yc, sc, dm_rows, acc, dye, ds_rows);  // adds to the run's sums
#pragma unroll
        for (int k = Y; k < Red::P; k++) dye[k] = 0.f;
        Red::run(dye, lane, [&](int k, float sum) {
            const float total = flip_sign(sum, y_flip, k);
            if (!kAtomicDy) dy[ee * Y + k] = total;
            else unsafeAtomicAdd(dy + ee * Y + k, total);  // dy zero-filled by the launcher
        });
    }
    if (run >= 0) flush(run);
}

template <int K, int CPL, bool A, int I>
__device__ __forceinline__ void dispatch_bwd_tile(int, const float *, const float *, const float *,
                                                  const float *, const int32_t *, const int32_t *,
                                                  const int32_t *, const int32_t *, float *, float *,
                                                  float *, int, float, unsigned, int, int, int, int, int,
                                                  float *) {}
template <int K, int CPL, bool A, int I, typename Part, typename... Rest>
__device__ __forceinline__ void dispatch_bwd_tile(int part, const float *x, const float *y, const float *s,
                                                  const float *dm, const int32_t *t_sender,
                                                  const int32_t *t_edge, const int32_t *t_local,
                                                  const int32_t *row_order, float *dx, float *dy,
                                                  float *ds, int num_nodes, float scale, unsigned y_flip,
                                                  int tile, int tile_rows, int begin, int end, int slice,
                                                  float *tile_lds) {
    if (part == I)
        unrolled_bwd_tile_part<Part, K, CPL, A>(x, y, s, dm, t_sender, t_edge, t_local, row_order, dx, dy,
                                                ds, num_nodes, scale, y_flip, tile, tile_rows, begin, end,
                                                slice, tile_lds);
    else
        dispatch_bwd_tile<K, CPL, A, I + 1, Rest...>(part, x, y, s, dm, t_sender, t_edge, t_local,
                                                     row_order, dx, dy, ds, num_nodes, scale, y_flip,
                                                     tile, tile_rows, begin, end, slice, tile_lds);
}

// One block per (work item, channel slice, part); a work item is a piece of one tile's edge list.
template <int K, int CPL, int WPB, int MINW, typename... Parts>
__global__ __launch_bounds__(kWave *WPB, MINW) void unrolled_bwd_tile_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ s,
    const float *__restrict__ dm, const int32_t *__restrict__ work,
    const int32_t *__restrict__ t_sender, const int32_t *__restrict__ t_edge,
    const int32_t *__restrict__ t_local, const int32_t *__restrict__ row_order,
    float *__restrict__ dx, float *__restrict__ dy, float *__restrict__ ds, int num_nodes,
    int tile_rows, int num_work, float scale, unsigned y_flip) {
    extern __shared__ __attribute__((aligned(16))) float tile_lds[];
    constexpr int NP = sizeof...(Parts);
    constexpr int CW = Slice<K, CPL>::COUNT;
    constexpr bool kAtomicDy = NP * CW > 1;  // several waves add into one dy row
    // The grid covers all num_work descriptors, of which the first work[3] are in use: those are
    // dealt to the XCDs in contiguous eighths (see logical_block), the surplus blocks leave.
    const int used = min(work[3], num_work);
    const int64_t items = (int64_t)used * (CW * NP);
    const int64_t per_xcd = (items + kXcds - 1) / kXcds;
    if ((int64_t)(blockIdx.x / kXcds) >= per_xcd) return;  // whole block: no barrier is left waiting
    const int64_t item = (int64_t)(blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
    if (item >= items) return;
    const int part = (int)(item % NP);
    const int slice = (int)((item / NP) % CW);
    const int64_t w = item / (NP * CW);
    const int tile = work[4 * w], begin = work[4 * w + 1], end = work[4 * w + 2];
    if (begin >= end) return;  // unused descriptor or a tile without edges (uniform over the block)
    dispatch_bwd_tile<K, CPL, kAtomicDy, 0, Parts...>(part, x, y, s, dm, t_sender, t_edge, t_local,
                                                      row_order, dx, dy, ds, num_nodes, scale, y_flip,
                                                      tile, tile_rows, begin, end, slice, tile_lds);
}

// ---------------------------------------------------------------------------
// Leading-channels layout: a row is (channels, dim), so the channels of a wave are one
// contiguous block of W * dim floats.  The wave moves such a block with coalesced 16-byte
// accesses and turns it through its private strip of LDS: lane c reads (or writes) the
// values of its channel there at an odd row stride, which is free of bank conflicts.
// The arithmetic between the two turns is the same generated code as for the trailing
// layout.  LDS operations of one wave complete in order, so the strip needs no barrier,
// only fences that keep the compiler from moving accesses across the turn.
// ---------------------------------------------------------------------------
constexpr int odd_stride(int n) { return (n % 2) ? n : n + 1; }

// f(std::integral_constant<int, I>) for I = FIRST .. LAST - 1
template <int FIRST, int LAST, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (FIRST < LAST) {
        f(std::integral_constant<int, FIRST>{});
        static_for<FIRST + 1, LAST>(f);
    }
}
constexpr int round4(int n) { return (n + 3) / 4 * 4; }

__device__ __forceinline__ void strip_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Block barrier that orders LDS accesses only.  `__syncthreads()` also waits for every global
// load, store and atomic of the wave (its fence covers all address spaces), which would drain
// the next edge's prefetch and the previous edge's stores at each barrier of the edge loop.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Position in a strip (rows of ROW values at stride PAD) of element g of the linear block.
template <int ROW, int PAD>
__device__ __forceinline__ int strip_index(int g) {
    return PAD == ROW ? g : g + (g / ROW) * (PAD - ROW);
}

template <int K, int X, int S, int Z>
struct LeadingGeometry {
    static constexpr int W = K < kWave ? K : kWave;  // channels per wave
    static constexpr int COUNT = K / W;              // waves per row
    static_assert(K % W == 0 && W % 4 == 0, "channel count must be a multiple of 4 and of 64 above 64");
    static constexpr int PX = odd_stride(X), PS = odd_stride(S), PZ = odd_stride(Z);
    static constexpr int XR = round4(W * PX);        // floats; keeps the s strip 16-byte aligned
    static constexpr int SR = round4(W * PS);
    static constexpr int REGION = XR + SR > 4 * PZ ? XR + SR : round4(4 * PZ);
    // out / dm rows pass through the whole strip in groups of GC channels
    static constexpr int group() {
        int g = W;
        while (g > 4 && g * PZ > REGION) g /= 2;
        return g;
    }
    static constexpr int GC = group();
    static_assert(W % GC == 0 && GC % 4 == 0, "channel groups must tile the wave");
};

// N floats (N % 4 == 0) at a 16-byte aligned address, dealt to NT threads in 16-byte pieces.
template <int N, int NT = kWave>
struct LinearBlock {
    static_assert(N % 4 == 0, "blocks are moved in 16-byte pieces");
    static constexpr int PIECES = N / 4;
    static constexpr int NV = (PIECES + NT - 1) / NT;
    static constexpr bool EXACT = NV * NT == PIECES;
    f32x4 v[NV];

    template <bool kStream>
    __device__ __forceinline__ void load(const float *src, int tid) {
        const f32x4 *p = reinterpret_cast<const f32x4 *>(src);
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int idx = i * NT + tid;
            if (EXACT || idx < PIECES) v[i] = kStream ? __builtin_nontemporal_load(p + idx) : p[idx];
        }
    }
    __device__ __forceinline__ void store(float *dst, int tid) const {
        f32x4 *p = reinterpret_cast<f32x4 *>(dst);
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int idx = i * NT + tid;
            if (EXACT || idx < PIECES) __builtin_nontemporal_store(v[i], p + idx);
        }
    }
    template <int ROW, int PAD>
    __device__ __forceinline__ void to_strip(float *strip, int tid) const {
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int idx = i * NT + tid;
            if (EXACT || idx < PIECES) {
                if (PAD == ROW) {
                    reinterpret_cast<f32x4 *>(strip)[idx] = v[i];
                } else {
#pragma unroll
                    for (int t = 0; t < 4; t++) strip[strip_index<ROW, PAD>(4 * idx + t)] = v[i][t];
                }
            }
        }
    }
    template <int ROW, int PAD>
    __device__ __forceinline__ void from_strip(const float *strip, int tid) {
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int idx = i * NT + tid;
            if (EXACT || idx < PIECES) {
                if (PAD == ROW) {
                    v[i] = reinterpret_cast<const f32x4 *>(strip)[idx];
                } else {
#pragma unroll
                    for (int t = 0; t < 4; t++) v[i][t] = strip[strip_index<ROW, PAD>(4 * idx + t)];
                }
            }
        }
    }

    // The same moves for a wave whose first thread index BASE is a compile-time constant (thread
    // = BASE + lane).  Whether a step's pieces exist is then known per wave when the code is
    // generated, and the global accesses of the loop are issued unconditionally: a step that
    // only part of the wave owns clamps the other lanes to the wave's last piece (they load it
    // again, and store the same values to the same place again).  With no global access under a
    // condition the compiler's wait counts stay exact.
    template <int BASE, int I>
    static constexpr int step_kind() {  // 0: no lane owns a piece, 1: every lane, 2: the first lanes
        return I * NT + BASE >= PIECES ? 0 : I * NT + BASE + kWave - 1 < PIECES ? 1 : 2;
    }
    template <int BASE, int I>
    __device__ static __forceinline__ int piece(int lane) {
        const int idx = I * NT + BASE + lane;
        return step_kind<BASE, I>() == 2 && idx >= PIECES ? PIECES - 1 : idx;
    }
    template <int BASE, bool kStream, int I = 0>
    __device__ __forceinline__ void load_at(const float *src, int lane) {
        if constexpr (I < NV) {
            if constexpr (step_kind<BASE, I>() != 0) {
                const f32x4 *p = reinterpret_cast<const f32x4 *>(src) + piece<BASE, I>(lane);
                v[I] = kStream ? __builtin_nontemporal_load(p) : *p;
            }
            load_at<BASE, kStream, I + 1>(src, lane);
        }
    }
    template <int BASE, int I = 0>
    __device__ __forceinline__ void store_at(float *dst, int lane) const {
        if constexpr (I < NV) {
            if constexpr (step_kind<BASE, I>() != 0)
                __builtin_nontemporal_store(v[I], reinterpret_cast<f32x4 *>(dst) + piece<BASE, I>(lane));
            store_at<BASE, I + 1>(dst, lane);
        }
    }
    template <int BASE, int ROW, int PAD, int I = 0>
    __device__ __forceinline__ void to_strip_at(float *strip, int lane) const {
        if constexpr (I < NV) {
            if constexpr (step_kind<BASE, I>() != 0) {
                const int idx = piece<BASE, I>(lane);  // clamped lanes rewrite the last piece with its own values
                if (PAD == ROW) {
                    reinterpret_cast<f32x4 *>(strip)[idx] = v[I];
                } else {
#pragma unroll
                    for (int t = 0; t < 4; t++) strip[strip_index<ROW, PAD>(4 * idx + t)] = v[I][t];
                }
            }
            to_strip_at<BASE, ROW, PAD, I + 1>(strip, lane);
        }
    }
    template <int BASE, int ROW, int PAD, int I = 0>
    __device__ __forceinline__ void from_strip_at(const float *strip, int lane) {
        if constexpr (I < NV) {
            if constexpr (step_kind<BASE, I>() != 0) {
                const int idx = piece<BASE, I>(lane);
                if (PAD == ROW) {
                    v[I] = reinterpret_cast<const f32x4 *>(strip)[idx];
                } else {
#pragma unroll
                    for (int t = 0; t < 4; t++) v[I][t] = strip[strip_index<ROW, PAD>(4 * idx + t)];
                }
            }
            from_strip_at<BASE, ROW, PAD, I + 1>(strip, lane);
        }
    }
};

// Bit i of the result: element i * NT + tid of a linear block of N values in rows of ROW
// lies in a column of `mask`.  Computed once per thread; the per-edge loops test one bit.
template <int N, int ROW, int NT>
__device__ __forceinline__ unsigned column_predicate(unsigned long long mask, int tid) {
    constexpr int STEPS = (N + NT - 1) / NT;
    static_assert(STEPS <= 32, "block too large for a 32-bit predicate");
    unsigned pred = 0;
#pragma unroll
    for (int i = 0; i < STEPS; i++) {
        const int g = i * NT + tid;
        if (g < N && ((mask >> (g % ROW)) & 1ull)) pred |= 1u << i;
    }
    return pred;
}

// forward ---------------------------------------------------------------------
template <typename Part, int K>
__device__ __forceinline__ void unrolled_fwd_leading(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ s,
    const int32_t *__restrict__ sender, const int32_t *__restrict__ row_ptr,
    const int32_t *__restrict__ perm, float *__restrict__ out, int num_nodes, float scale, unsigned y_flip, int r,
    int slice, int lane, float *strip) {
    constexpr int NX = Part::NX, NS = Part::NS, NZ = Part::NZ, Y = Part::Y;
    constexpr int X = Part::X, S = Part::S, Z = Part::Z;
    static_assert(NZ == Z, "the forward pass of the leading layout is not split into parts");
    using G = LeadingGeometry<K, X, S, Z>;
    using V = Vec<1>;
    constexpr int W = G::W, GC = G::GC;
    float *strip_x = strip, *strip_s = strip + G::XR;

    const bool active = lane < W;
    const int cl = active ? lane : 0;  // idle lanes (channel count below 64) mirror channel 0
    const int64_t ch0 = (int64_t)slice * W;

    V acc[NZ];
#pragma unroll
    for (int i = 0; i < NZ; i++) acc[i] = vzero<1>();

    int e = row_ptr[r];
    const int e1 = row_ptr[r + 1];

    LinearBlock<W * X> xl;
    LinearBlock<W * S> sl;
    float yn[Y];
    bool valid_n = false;
    auto fetch = [&](int pos) {
        const int snd = sender[pos];
        valid_n = (unsigned)snd < (unsigned)num_nodes;
        const int row = valid_n ? snd : 0;
        const int64_t ee = perm ? (int64_t)perm[pos] : (int64_t)pos;
        xl.template load<false>(x + ((int64_t)row * K + ch0) * X, lane);
        sl.template load<true>(s + (ee * K + ch0) * S, lane);
        const float *yr = y + ee * Y;
#pragma unroll
        for (int k = 0; k < Y; k++) yn[k] = yr[k];
    };
    if (e < e1) fetch(e);
    while (e < e1) {
        strip_fence();  // the column reads of the previous edge are done
        xl.template to_strip<X, G::PX>(strip_x, lane);
        sl.template to_strip<S, G::PS>(strip_s, lane);
        strip_fence();
        V xc[NX], sc[NS];
        float yc[Y];
#pragma unroll
        for (int j = 0; j < NX; j++) xc[j].v[0] = strip_x[cl * G::PX + Part::kX[j]];
#pragma unroll
        for (int l = 0; l < NS; l++) sc[l].v[0] = strip_s[cl * G::PS + Part::kS[l]];
#pragma unroll
        for (int k = 0; k < Y; k++) yc[k] = to_vgpr(flip_sign(yn[k], y_flip, k));
        const bool valid = valid_n;
        e++;
        if (e < e1) fetch(e);
        if (valid) Part::template edge_fwd<1>(xc, yc, sc, acc);
    }

    // write-back: GC channels at a time through the whole strip
    float *orow = out + ((int64_t)r * K + ch0) * Z;
#pragma unroll
    for (int q = 0; q < W / GC; q++) {
        strip_fence();
        if (active && lane / GC == q) {
#pragma unroll
            for (int i = 0; i < NZ; i++) strip[(lane % GC) * G::PZ + Part::kZ[i]] = acc[i].v[0] * scale;
        }
        strip_fence();
        LinearBlock<GC * Z> ol;
        ol.template from_strip<Z, G::PZ>(strip, lane);
        ol.store(orow + (int64_t)q * GC * Z, lane);
    }
}

template <int K, int WPB, typename Part>
__global__ __launch_bounds__(kWave *WPB) void unrolled_fwd_leading_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ s,
    const int32_t *__restrict__ sender, const int32_t *__restrict__ row_ptr,
    const int32_t *__restrict__ perm, const int32_t *__restrict__ row_order,
    float *__restrict__ out, int num_nodes, float scale, unsigned y_flip) {
    using G = LeadingGeometry<K, Part::X, Part::S, Part::Z>;
    __shared__ __attribute__((aligned(16))) float strips[WPB * G::REGION];
    const int64_t item = logical_block() * WPB + threadIdx.y;
    if (item >= (int64_t)num_nodes * G::COUNT) return;
    const int slice = uniform((int)(item % G::COUNT));
    const int q = uniform((int)(item / G::COUNT));
    const int r = row_order ? row_order[q] : q;
    unrolled_fwd_leading<Part, K>(x, y, s, sender, row_ptr, perm, out, num_nodes, scale, y_flip, r, slice,
                                  threadIdx.x, strips + threadIdx.y * G::REGION);
}

// backward --------------------------------------------------------------------
// One block per (receiver, channel slice); its waves are the parts of the signature.  They
// share the staged x and s blocks of an edge (each thread moves its pieces once), and their
// ds and dx values meet in a second pair of strips from which the block stores whole ds
// rows and issues the dx atomics in linear, coalesced order.  All waves of a block walk the
// same edge segment, so the two block barriers per edge are reached uniformly.
struct DsStrip {
    float *row;
    bool active;
    template <int L>
    __device__ __forceinline__ void put(const Vec<1> &v) const {
        if (active) row[L] = v.v[0];
    }
};

template <int K, int X, int S, int Z, int NP>
struct LeadingBwdGeometry : LeadingGeometry<K, X, S, Z> {
    using Base = LeadingGeometry<K, X, S, Z>;
    static constexpr int NT = kWave * NP;
    static constexpr int IN = Base::XR + Base::SR;  // staged operands, then as much again for results
    static constexpr int REGION = 2 * IN > 4 * Base::PZ ? 2 * IN : round4(4 * Base::PZ);
    static constexpr int group() {
        int g = Base::W;
        while (g > 4 && g * Base::PZ > REGION) g /= 2;
        return g;
    }
    static constexpr int GC = group();  // channels of dm rows staged at a time
};

template <typename Part, int K, int NP, int PART, unsigned long long kCoveredDx, bool kOrdered>
__device__ __forceinline__ void unrolled_bwd_leading(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ s,
    const float *__restrict__ dm, const int32_t *__restrict__ sender,
    const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    float *__restrict__ dx, float *__restrict__ dy, float *__restrict__ ds, int num_nodes,
    float scale, unsigned y_flip, int r, int slice, int lane, int tid, float *region) {
    // PART: this wave's index in the block (tid = PART * 64 + lane), a constant of the generated code
    constexpr int part = PART, BASE = PART * kWave;
    constexpr int NX = Part::NX, NS = Part::NS, NZ = Part::NZ, Y = Part::Y;
    constexpr int X = Part::X, S = Part::S, Z = Part::Z;
    static_assert(X <= 64 && S <= 64, "part masks hold 64 columns");
    using G = LeadingBwdGeometry<K, X, S, Z, NP>;
    using V = Vec<1>;
    using Red = WaveReduceBlocks<Y>;
    constexpr int W = G::W, GC = G::GC, NT = G::NT;
    constexpr int XN = W * X, SN = W * S;
    constexpr bool kAllDx = kCoveredDx == (X == 64 ? ~0ull : ((1ull << X) - 1));
    float *in_x = region, *in_s = in_x + G::XR, *out_x = in_s + G::SR, *out_s = out_x + G::XR;

    const bool active = lane < W;
    const int cl = active ? lane : 0;
    const int64_t ch0 = (int64_t)slice * W;

    // cotangent rows: GC channels at a time through the whole region
    V dmr[NZ];
    {
        const float *zr = dm + ((int64_t)r * K + ch0) * Z;
#pragma unroll
        for (int i = 0; i < NZ; i++) dmr[i] = vzero<1>();  // idle lanes must add nothing to dy
#pragma unroll
        for (int q = 0; q < W / GC; q++) {
            LinearBlock<GC * Z, NT> zl;
            zl.template load<true>(zr + (int64_t)q * GC * Z, tid);
            __syncthreads();  // the column reads of the previous group are done
            zl.template to_strip<Z, G::PZ>(region, tid);
            __syncthreads();
            if (active && lane / GC == q) {
#pragma unroll
                for (int i = 0; i < NZ; i++) dmr[i].v[0] = region[(lane % GC) * G::PZ + Part::kZ[i]] * scale;
            }
        }
        __syncthreads();
    }
    // x columns no coefficient touches take no dx (their rows stay zero)
    unsigned covered = ~0u;
    if (!kAllDx) covered = column_predicate<XN, X, NT>(kCoveredDx, tid);

    int e = row_ptr[r];
    const int e1 = row_ptr[r + 1];

    LinearBlock<XN, NT> xl;
    LinearBlock<SN, NT> sl;
    float yn[Y];
    int snd_n = 0;
    int64_t ee_n = 0;
    // Padding edges (their dy/ds rows are zero-filled separately) are stepped over here, so the
    // loop body is one straight line and its waits are exact counts (see the trailing kernel).
    auto next_edge = [&](int p) {
        while (p < e1 && !((unsigned)load_uniform(sender + p) < (unsigned)num_nodes)) p++;
        return p;
    };
    auto fetch = [&](int pos) {
        snd_n = load_uniform(sender + pos);
        ee_n = perm ? (int64_t)load_uniform(perm + pos) : (int64_t)pos;
        xl.template load_at<BASE, false>(x + ((int64_t)snd_n * K + ch0) * X, lane);
        sl.template load_at<BASE, true>(s + (ee_n * K + ch0) * S, lane);
        const float *yr = y + ee_n * Y;
#pragma unroll
        for (int k = 0; k < Y; k++) yn[k] = yr[k];
    };
    e = next_edge(e);
    if (e < e1) fetch(e);
    __builtin_amdgcn_s_waitcnt(kWaitVmcnt0);  // entered with nothing in flight
    while (e < e1) {
        // (the result strips of the previous edge are still being read by other waves: the
        // operand strips are separate, and the barrier below orders the next result writes)
        xl.template to_strip_at<BASE, X, G::PX>(in_x, lane);
        sl.template to_strip_at<BASE, S, G::PS>(in_s, lane);
        lds_barrier();
        V xc[NX], sc[NS];
        float yc[Y];
#pragma unroll
        for (int j = 0; j < NX; j++) xc[j].v[0] = in_x[cl * G::PX + Part::kX[j]];
#pragma unroll
        for (int l = 0; l < NS; l++) sc[l].v[0] = in_s[cl * G::PS + Part::kS[l]];
#pragma unroll
        for (int k = 0; k < Y; k++) yc[k] = to_vgpr(flip_sign(yn[k], y_flip, k));
        const int snd = snd_n;
        const int64_t ee = ee_n;
        const int pos = e;
        e = next_edge(e + 1);
        if (e < e1) fetch(e);

        float dye[Red::P];
        {
            V dxe[NX];
            const DsStrip ds_strip{out_s + cl * G::PS, active};
            Part::template edge_bwd<1>(xc, yc, sc, dmr, dxe, dye, ds_strip);
            if (active) {
#pragma unroll
                for (int j = 0; j < NX; j++) out_x[cl * G::PX + Part::kX[j]] = dxe[j].v[0];
            }
        }
        lds_barrier();  // operands consumed by every wave, results of every wave in place

        LinearBlock<SN, NT> dl;
        dl.template from_strip_at<BASE, S, G::PS>(out_s, lane);
        dl.template store_at<BASE>(ds + (ee * K + ch0) * S, lane);
        if (kOrdered) {  // the contribution of this position as one row of the buffer, no atomics
            LinearBlock<XN, NT> ul;
            ul.template from_strip_at<BASE, X, G::PX>(out_x, lane);
            ul.template store_at<BASE>(dx + ((int64_t)pos * K + ch0) * X, lane);
        } else {
            float *dx_block = dx + ((int64_t)snd * K + ch0) * X;
            static_for<0, (XN + NT - 1) / NT>([&](auto step) {
                constexpr int i = decltype(step)::value, first = i * NT + BASE;
                // does this wave own elements in this step: none, all (no condition left), some
                constexpr int kind = first >= XN ? 0 : first + kWave - 1 < XN ? 1 : 2;
                if constexpr (kind != 0) {
                    const int g = first + lane;
                    const bool mine = kAllDx ? (kind == 1 || g < XN) : (((covered >> i) & 1u) != 0);
                    if (mine) unsafeAtomicAdd(dx_block + g, out_x[strip_index<X, G::PX>(g)]);
                }
            });
        }

#pragma unroll
        for (int k = Y; k < Red::P; k++) dye[k] = 0.f;
        Red::run(dye, lane, [&](int k, float sum) {
            constexpr int SLOTS = NP * G::COUNT;
            const float total = flip_sign(sum, y_flip, k);
            if (SLOTS == 1) dy[ee * Y + k] = total;
            else if (kOrdered) dy[((int64_t)pos * SLOTS + part * G::COUNT + slice) * Y + k] = total;
            else unsafeAtomicAdd(dy + ee * Y + k, total);  // dy zero-filled by the launcher
        });
    }
}

template <int K, int NP, unsigned long long kCoveredDx, bool O, int I>
__device__ __forceinline__ void dispatch_bwd_leading(int, const float *, const float *, const float *,
                                                     const float *, const int32_t *, const int32_t *,
                                                     const int32_t *, float *, float *, float *, int,
                                                     float, unsigned, int, int, int, int, float *) {}
template <int K, int NP, unsigned long long kCoveredDx, bool O, int I, typename Part, typename... Rest>
__device__ __forceinline__ void dispatch_bwd_leading(int part, const float *x, const float *y,
                                                     const float *s, const float *dm,
                                                     const int32_t *sender, const int32_t *row_ptr,
                                                     const int32_t *perm, float *dx, float *dy,
                                                     float *ds, int num_nodes, float scale,
                                                     unsigned y_flip, int r, int slice, int lane,
                                                     int tid, float *region) {
    if (part == I)
        unrolled_bwd_leading<Part, K, NP, I, kCoveredDx, O>(x, y, s, dm, sender, row_ptr, perm, dx, dy, ds,
                                                            num_nodes, scale, y_flip, r, slice, lane, tid,
                                                            region);
    else
        dispatch_bwd_leading<K, NP, kCoveredDx, O, I + 1, Rest...>(part, x, y, s, dm, sender, row_ptr,
                                                                   perm, dx, dy, ds, num_nodes, scale,
                                                                   y_flip, r, slice, lane, tid, region);
}

template <typename First, typename...>
struct FirstOf {
    using type = First;
};

// The second launch bound asks for three resident waves per SIMD when the signature is split
// in three or more parts (at most 168 vector registers): a few registers above that line cost
// a third of the occupancy and 35 % of the run time.
template <int K, bool kOrdered, typename... Parts>
__global__ __launch_bounds__(kWave * sizeof...(Parts), sizeof...(Parts) >= 3 ? 3 : sizeof...(Parts))
void unrolled_bwd_leading_kernel(
    const float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ s,
    const float *__restrict__ dm, const int32_t *__restrict__ sender,
    const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ row_order, float *__restrict__ dx, float *__restrict__ dy,
    float *__restrict__ ds, int num_nodes, float scale, unsigned y_flip) {
    using P0 = typename FirstOf<Parts...>::type;
    constexpr int NP = sizeof...(Parts);
    using G = LeadingBwdGeometry<K, P0::X, P0::S, P0::Z, NP>;
    constexpr unsigned long long kCoveredDx = (Parts::kDxMask | ...);
    __shared__ __attribute__((aligned(16))) float region[G::REGION];
    const int64_t item = logical_block();
    if (item >= (int64_t)num_nodes * G::COUNT) return;  // whole block: no barrier is left waiting
    const int slice = (int)(item % G::COUNT);
    const int q = (int)(item / G::COUNT);
    const int r = row_order ? row_order[q] : q;
    const int part = uniform((int)threadIdx.y);
    dispatch_bwd_leading<K, NP, kCoveredDx, kOrdered, 0, Parts...>(
        part, x, y, s, dm, sender, row_ptr, perm, dx, dy, ds, num_nodes, scale, y_flip, r, slice,
        threadIdx.x, threadIdx.y * kWave + threadIdx.x, region);
}

template <int K, int CPL, int WPB, int MINW, typename... Parts>
int launch_unrolled_fwd(const e3j_amd_conv_params &p, const float *x, const float *y, const float *s,
                        const int32_t *sender, const int32_t *row_ptr, const int32_t *perm,
                        float *out, hipStream_t stream) {
    constexpr int64_t PER_NODE = (int64_t)Slice<K, CPL>::COUNT * sizeof...(Parts);
    const int64_t items = p.segments ? (int64_t)p.max_segments : (int64_t)p.num_nodes;
    const int64_t blocks = padded_grid((items * PER_NODE + WPB - 1) / WPB);
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: grid too large");
    if (blocks == 0) return E3J_AMD_OK;
    hipLaunchKernelGGL((unrolled_fwd_kernel<K, CPL, WPB, MINW, Parts...>), dim3((unsigned)blocks),
                       dim3(kWave, WPB), 0, stream, x, y, s, sender, row_ptr, perm, p.row_order, out,
                       p.num_nodes, p.coef_scale, p.y_flip, p.row_cap,
                       p.row_piece > 0 ? p.row_piece : p.row_cap, p.segments, p.max_segments);
    return check_hip(hipGetLastError(), "convolution forward launch");
}

// Where the backward kernels put dx and dy: float atomics into zero-filled results, or (ordered)
// the per-position buffers behind `ordered`, which is then told what the variant produced.
template <int X, int Y, int SLOTS, unsigned long long COVERED>
int prepare_bwd_targets(const e3j_amd_conv_params &p, OrderedBwd *ordered, int K, float *&dx, float *&dy,
                        hipStream_t stream) {
    static_assert(SLOTS <= kMaxDySlots, "more waves per edge than dy slots");
    if (ordered != nullptr) {
        ordered->slots = SLOTS;
        ordered->covered = COVERED;
        dx = ordered->u;
        if (SLOTS > 1) dy = ordered->dy_slots;
        return E3J_AMD_OK;
    }
    int rc = launch_fill_zero(dx, sizeof(float) * (size_t)p.num_nodes * X * K, stream);
    if (rc == E3J_AMD_OK && SLOTS > 1) rc = launch_fill_zero(dy, sizeof(float) * (size_t)p.num_edges * Y, stream);
    return rc;
}

template <int K, int CPL, int WPB, int MINW, int Y, int X, typename... Parts>
int launch_unrolled_bwd(const e3j_amd_conv_params &p, const float *x, const float *y, const float *s,
                        const float *dm, const int32_t *sender, const int32_t *row_ptr,
                        const int32_t *perm, float *dx, float *dy, float *ds, hipStream_t stream,
                        OrderedBwd *ordered) {
    constexpr int64_t PER_NODE = (int64_t)Slice<K, CPL>::COUNT * sizeof...(Parts);
    constexpr unsigned long long kCovered = (Parts::kDxMask | ...);
    int rc = prepare_bwd_targets<X, Y, (int)PER_NODE, kCovered>(p, ordered, K, dx, dy, stream);
    if (rc) return rc;
    const int64_t blocks = padded_grid(((int64_t)p.num_nodes * PER_NODE + WPB - 1) / WPB);
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution_bwd: grid too large");
    if (ordered != nullptr)
        hipLaunchKernelGGL((unrolled_bwd_kernel<K, CPL, WPB, MINW, true, Parts...>), dim3((unsigned)blocks),
                           dim3(kWave, WPB), 0, stream, x, y, s, dm, sender, row_ptr, perm, p.row_order,
                           dx, dy, ds, p.num_nodes, p.coef_scale, p.y_flip);
    else
        hipLaunchKernelGGL((unrolled_bwd_kernel<K, CPL, WPB, MINW, false, Parts...>), dim3((unsigned)blocks),
                           dim3(kWave, WPB), 0, stream, x, y, s, dm, sender, row_ptr, perm, p.row_order,
                           dx, dy, ds, p.num_nodes, p.coef_scale, p.y_flip);
    return check_hip(hipGetLastError(), "convolution backward launch");
}

template <int K, int WPB, int MINW, int Y, typename... Parts>
int launch_unrolled_bwd_sender(const e3j_amd_conv_params &p, const float *x, const float *y, const float *s,
                               const float *dm, const int32_t *receiver_t, const int32_t *row_ptr,
                               const int32_t *perm, float *dx, float *dy, float *ds, hipStream_t stream) {
    constexpr int CW = Slice<K, 1>::COUNT;
    if (CW > 1) {  // several waves add into one dy row
        const int rc = launch_fill_zero(dy, sizeof(float) * (size_t)p.num_edges * Y, stream);
        if (rc) return rc;
    }
    const int64_t blocks = padded_grid(((int64_t)p.num_nodes * CW + WPB - 1) / WPB);
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution_bwd: grid too large");
    if (blocks == 0) return E3J_AMD_OK;
    hipLaunchKernelGGL((unrolled_bwd_sender_kernel<K, WPB, MINW, Parts...>), dim3((unsigned)blocks),
                       dim3(kWave, WPB), 0, stream, x, y, s, dm, receiver_t, row_ptr, perm, p.row_order, dx, dy,
                       ds, p.num_nodes, p.coef_scale, p.y_flip);
    return check_hip(hipGetLastError(), "convolution backward (sender rows) launch");
}

constexpr int max_of(std::initializer_list<int> v) {
    int m = 0;
    for (int a : v) m = a > m ? a : m;
    return m;
}
constexpr size_t kMaxTileLds = 160 * 1024;  // LDS of a CU, all of which one block may take

// LDS bytes per receiver of a tile (the part with the most dm rows decides).
template <int CPL, typename... Parts>
constexpr int tile_row_bytes() {
    return max_of({Parts::NZ...}) * kWave * CPL * (int)sizeof(float);
}

template <int K, int CPL, int WPB, int MINW, int Y, int X, typename... Parts>
int launch_unrolled_bwd_tile(const e3j_amd_conv_params &p, const float *x, const float *y, const float *s,
                             const float *dm, const e3j_amd_tile_schedule &sch, float *dx, float *dy,
                             float *ds, hipStream_t stream) {
    constexpr int64_t PER_WORK = (int64_t)Slice<K, CPL>::COUNT * sizeof...(Parts);
    constexpr unsigned long long kCovered = (Parts::kDxMask | ...);
    const size_t lds = (size_t)tile_row_bytes<CPL, Parts...>() * (size_t)sch.tile_rows;
    if (sch.tile_rows < 1 || lds > kMaxTileLds)
        return set_error(E3J_AMD_INVALID_ARGUMENT,
                         "convolution_bwd_tiled: the schedule's tiles hold more receivers than fit the LDS "
                         "(e3j_amd_tile_rows gives the limit)");
    int rc = prepare_bwd_targets<X, Y, (int)PER_WORK, kCovered>(p, nullptr, K, dx, dy, stream);
    if (rc) return rc;
    const int64_t blocks = padded_grid((int64_t)sch.num_work * PER_WORK);
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution_bwd_tiled: grid too large");
    if (blocks == 0) return E3J_AMD_OK;
    auto kernel = unrolled_bwd_tile_kernel<K, CPL, WPB, MINW, Parts...>;
    rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxTileLds),
                   "hipFuncSetAttribute(bwd_tiled)");
    if (rc) return rc;
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(kWave, WPB), lds, stream, x, y, s, dm, sch.work,
                       sch.sender, sch.edge, sch.local, p.row_order, dx, dy, ds, p.num_nodes, sch.tile_rows,
                       sch.num_work, p.coef_scale, p.y_flip);
    return check_hip(hipGetLastError(), "convolution backward (tiled) launch");
}

template <int K, int WPB, typename Part>
int launch_unrolled_fwd_leading(const e3j_amd_conv_params &p, const float *x, const float *y,
                                const float *s, const int32_t *sender, const int32_t *row_ptr,
                                const int32_t *perm, float *out, hipStream_t stream) {
    using G = LeadingGeometry<K, Part::X, Part::S, Part::Z>;
    const int64_t blocks = padded_grid(((int64_t)p.num_nodes * G::COUNT + WPB - 1) / WPB);
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: grid too large");
    hipLaunchKernelGGL((unrolled_fwd_leading_kernel<K, WPB, Part>), dim3((unsigned)blocks),
                       dim3(kWave, WPB), 0, stream, x, y, s, sender, row_ptr, perm, p.row_order, out,
                       p.num_nodes, p.coef_scale, p.y_flip);
    return check_hip(hipGetLastError(), "convolution forward launch");
}

template <int K, int Y, int X, typename... Parts>
int launch_unrolled_bwd_leading(const e3j_amd_conv_params &p, const float *x, const float *y,
                                const float *s, const float *dm, const int32_t *sender,
                                const int32_t *row_ptr, const int32_t *perm, float *dx, float *dy,
                                float *ds, hipStream_t stream, OrderedBwd *ordered) {
    using P0 = typename FirstOf<Parts...>::type;
    constexpr int NP = sizeof...(Parts);
    using G = LeadingBwdGeometry<K, P0::X, P0::S, P0::Z, NP>;
    constexpr unsigned long long kCovered = (Parts::kDxMask | ...);
    int rc = prepare_bwd_targets<X, Y, G::COUNT * NP, kCovered>(p, ordered, K, dx, dy, stream);
    if (rc) return rc;
    const int64_t blocks = padded_grid((int64_t)p.num_nodes * G::COUNT);
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution_bwd: grid too large");
    if (ordered != nullptr)
        hipLaunchKernelGGL((unrolled_bwd_leading_kernel<K, true, Parts...>), dim3((unsigned)blocks),
                           dim3(kWave, NP), 0, stream, x, y, s, dm, sender, row_ptr, perm, p.row_order,
                           dx, dy, ds, p.num_nodes, p.coef_scale, p.y_flip);
    else
        hipLaunchKernelGGL((unrolled_bwd_leading_kernel<K, false, Parts...>), dim3((unsigned)blocks),
                           dim3(kWave, NP), 0, stream, x, y, s, dm, sender, row_ptr, perm, p.row_order,
                           dx, dy, ds, p.num_nodes, p.coef_scale, p.y_flip);
    return check_hip(hipGetLastError(), "convolution backward launch");
}

}  // namespace e3j_amd
#endif
