// Table-driven convolution kernels for gfx950: any coefficient table, any
// channel count, both layouts, float32/float64.  They are the fallback behind
// the compile-time-unrolled kernels and the carrier of every edge-case rule.
//
// Mapping: one 64-lane wavefront owns one CSR row (a node); a lane owns one
// channel of a 64-channel chunk.  Each lane keeps its operands and
// accumulators in a private column of LDS (dynamic indexing by the table's
// coordinates), so no barrier or cross-lane traffic is needed except the
// channel reduction of dy.  Coefficients, y and the adjacency are
// wave-uniform and travel through scalar loads.
//
// Semantics restated from lib/e3j_ops/cuda/convolution/fwd.cuh:289-403 and
// bwd.cuh:116-321: zero rows for nodes without live edges, padding edges
// skipped by a bounds check on the gathered endpoint, dy/ds of padding edges
// written as zeros, dx rows zero-filled before accumulation.

#include <type_traits>

#include "common.h"

namespace e3j_amd {
namespace {

// Value of lane `src` (a wave-uniform number) of a per-lane variable, as a wave-uniform value.
template <typename T>
__device__ __forceinline__ T lane_pick(T v, int src) {
    if constexpr (sizeof(T) == 2) {
        const uint32_t w = __builtin_amdgcn_readlane((uint32_t)__builtin_bit_cast(uint16_t, v), src);
        return __builtin_bit_cast(T, (uint16_t)w);
    } else {
        static_assert(sizeof(T) % 4 == 0, "whole registers");
        uint32_t w[sizeof(T) / 4];
        __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
        for (int q = 0; q < (int)(sizeof(T) / 4); q++) w[q] = __builtin_amdgcn_readlane(w[q], src);
        __builtin_memcpy(&v, w, sizeof(T));
        return v;
    }
}

template <typename Val>
struct CoefFields {  // one table entry, wave-uniform
    int i, j, k, l;
    Val val;
};

// Sixty-four consecutive entries of the table, one per lane (one coalesced vector load), handed
// out one at a time as wave-uniform values through lane reads: the coefficient stream costs
// no scalar-memory round trip per entry.
template <typename Idx, typename Val>
struct CoefChunk {
    Val val;
    uint32_t w[sizeof(Idx) == 1 ? 1 : 4];

    __device__ __forceinline__ void load(const Coef4D<Idx, Val> *__restrict__ coef, int n0, int num_coef, int lane) {
        int n = n0 + lane;
        if (n >= num_coef) n = num_coef - 1;
        const Coef4D<Idx, Val> c = coef[n];
        val = c.val;
        if constexpr (sizeof(Idx) == 1) {
            w[0] = (uint32_t)c.i | ((uint32_t)c.j << 8) | ((uint32_t)c.k << 16) | ((uint32_t)c.l << 24);
        } else {
            w[0] = (uint32_t)c.i; w[1] = (uint32_t)c.j; w[2] = (uint32_t)c.k; w[3] = (uint32_t)c.l;
        }
    }
    __device__ __forceinline__ CoefFields<Val> pick(int u) const {
        CoefFields<Val> f;
        f.val = lane_pick(val, u);
        if constexpr (sizeof(Idx) == 1) {
            const uint32_t a = __builtin_amdgcn_readlane(w[0], u);
            f.i = (int)(a & 255u); f.j = (int)((a >> 8) & 255u); f.k = (int)((a >> 16) & 255u); f.l = (int)(a >> 24);
        } else {
            f.i = (int)__builtin_amdgcn_readlane(w[0], u); f.j = (int)__builtin_amdgcn_readlane(w[1], u);
            f.k = (int)__builtin_amdgcn_readlane(w[2], u); f.l = (int)__builtin_amdgcn_readlane(w[3], u);
        }
        return f;
    }
};

// A strided row of global memory into a lane-private LDS column, sixteen loads in flight.
// `row` must be readable on every lane (lanes past the last channel pass the last channel's
// row); lanes that are not `active` store zeros.
template <typename Val>
__device__ __forceinline__ void stage_column(Val *col, const Val *row, int64_t stride, int n, bool active) {
    constexpr int B = 16;
    for (int j0 = 0; j0 < n; j0 += B) {
        Val t[B];
#pragma unroll
        for (int v = 0; v < B; v++) {
            const int j = j0 + v < n ? j0 + v : n - 1;
            t[v] = row[(int64_t)j * stride];
        }
#pragma unroll
        for (int v = 0; v < B; v++) {
            const int j = j0 + v < n ? j0 + v : n - 1;  // the tail rewrites the last element
            col[j * kWave] = active ? t[v] : Val(0);
        }
    }
}

// y of one edge for the coefficient loop: up to 64 components sit in one register (lane k
// holds y[k]) and are read as wave-uniform values; longer y rows are read from memory.
template <typename Val, bool kYLane>
struct EdgeY {
    Val reg;
    const Val *row;
    __device__ __forceinline__ EdgeY(const Val *ye, int num_y, int lane) : reg(Val(0)), row(ye) {
        if (kYLane && lane < num_y) reg = ye[lane];
    }
    __device__ __forceinline__ Val operator[](int k) const { return kYLane ? lane_pick(reg, k) : row[k]; }
};

constexpr int kCoefBatch = 8;  // table entries whose LDS reads are issued together

template <typename Idx, typename Val, bool kYLane>
__global__ void generic_fwd_kernel(const Coef4D<Idx, Val> *__restrict__ coef, int num_coef,
                                   const Val *__restrict__ x, RowLayout lx,
                                   const Val *__restrict__ y, int num_y,
                                   const Val *__restrict__ s, RowLayout ls,
                                   const int32_t *__restrict__ other,
                                   const int32_t *__restrict__ row_ptr,
                                   const int32_t *__restrict__ perm,
                                   const int32_t *__restrict__ row_order,
                                   Val *__restrict__ out, RowLayout lo,
                                   int num_nodes, int channels, int X, int S, int Z, int nchunks,
                                   const int32_t *__restrict__ served) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    if (served && *served) return;  // the kernel over the table's plan has taken the call
    const int lane = threadIdx.x;
    const int wave = threadIdx.y;
    const int64_t item = (int64_t)blockIdx.x * blockDim.y + wave;
    if (item >= (int64_t)num_nodes * nchunks) return;  // uniform per wave; no barriers below
    const int q = (int)(item / nchunks);
    const int r = row_order ? row_order[q] : q;
    const int c = (int)(item % nchunks) * kWave + lane;
    const bool active = c < channels;
    const int cr = active ? c : channels - 1;  // channel whose rows an idle lane reads

    Val *acc = reinterpret_cast<Val *>(smem_raw) + (size_t)wave * (Z + X + S) * kWave + lane;
    Val *xs = acc + (size_t)Z * kWave;
    Val *ss = xs + (size_t)X * kWave;
    for (int i = 0; i < Z; i++) acc[i * kWave] = Val(0);

    CoefChunk<Idx, Val> next;
    if (num_coef > 0) next.load(coef, 0, num_coef, lane);

    const int e0 = row_ptr[r], e1 = row_ptr[r + 1];
    for (int e = e0; e < e1; e++) {
        const int snd = other[e];
        if ((unsigned)snd >= (unsigned)num_nodes) continue;  // padding edge
        const int64_t ee = perm ? (int64_t)perm[e] : (int64_t)e;
        stage_column(xs, x + (int64_t)snd * lx.row + (int64_t)cr * lx.chan, lx.dim, X, active);
        stage_column(ss, s + ee * ls.row + (int64_t)cr * ls.chan, ls.dim, S, active);
        const EdgeY<Val, kYLane> ye(y + ee * num_y, num_y, lane);

        // runs of equal (output coordinate, path): the old accumulator and the path's scalar
        // are read when the run starts, so that its end is one LDS write
        int cur_i = -1, cur_l = 0;
        Val msg = Val(0), before = Val(0), scalar = Val(0);
        for (int n0 = 0; n0 < num_coef; n0 += kWave) {
            const CoefChunk<Idx, Val> chunk = next;
            next.load(coef, n0 + kWave < num_coef ? n0 + kWave : 0, num_coef, lane);
            const int nn = num_coef - n0 < kWave ? num_coef - n0 : kWave;
            for (int u = 0; u < nn; u += kCoefBatch) {
                CoefFields<Val> cf[kCoefBatch];
                Val xv[kCoefBatch], yv[kCoefBatch];
#pragma unroll
                for (int v = 0; v < kCoefBatch; v++) {
                    cf[v] = chunk.pick(u + v < nn ? u + v : nn - 1);
                    xv[v] = xs[cf[v].j * kWave];
                    yv[v] = ye[cf[v].k];
                }
#pragma unroll
                for (int v = 0; v < kCoefBatch; v++) {
                    if (u + v >= nn) break;
                    if (cf[v].i != cur_i || cf[v].l != cur_l) {
                        if (cur_i >= 0) acc[cur_i * kWave] = before + scalar * msg;
                        cur_i = cf[v].i; cur_l = cf[v].l; msg = Val(0);
                        before = acc[cur_i * kWave];
                        scalar = ss[cur_l * kWave];
                    }
                    msg += (xv[v] * yv[v]) * cf[v].val;
                }
            }
        }
        if (cur_i >= 0) acc[cur_i * kWave] = before + scalar * msg;
    }
    if (active) {
        Val *orow = out + (int64_t)r * lo.row + (int64_t)c * lo.chan;
        for (int i = 0; i < Z; i++) orow[(int64_t)i * lo.dim] = acc[i * kWave];
    }
}

// kGroupIsReceiver: rows are receivers (dm row fixed, x gathered, dx scattered with
// atomics into a zero-filled buffer).  Otherwise rows are senders (x row fixed, dm
// gathered, dx accumulated in place by the owning wave).
template <typename Idx, typename Val, bool kGroupIsReceiver, bool kYLane>
__global__ void generic_bwd_kernel(const Coef4D<Idx, Val> *__restrict__ coef, int num_coef,
                                   const Val *__restrict__ x, RowLayout lx,
                                   const Val *__restrict__ y, int num_y,
                                   const Val *__restrict__ s, RowLayout ls,
                                   const Val *__restrict__ dm, RowLayout lo,
                                   const int32_t *__restrict__ other,
                                   const int32_t *__restrict__ row_ptr,
                                   const int32_t *__restrict__ perm,
                                   const int32_t *__restrict__ row_order,
                                   Val *__restrict__ dx, Val *__restrict__ dy, Val *__restrict__ ds,
                                   int num_nodes, int channels, int X, int S, int Z, int nchunks,
                                   int cols_ji, const int32_t *__restrict__ served) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    if (served && *served) return;  // the kernel over the table's plan has taken the call
    const int lane = threadIdx.x;
    const int wave = threadIdx.y;
    const int64_t item = (int64_t)blockIdx.x * blockDim.y + wave;
    if (item >= (int64_t)num_nodes) return;
    const int g = row_order ? row_order[item] : (int)item;

    const int per_wave = Z + 2 * X + 2 * S + num_y;
    Val *zc = reinterpret_cast<Val *>(smem_raw) + (size_t)wave * per_wave * kWave + lane;
    Val *xc = zc + (size_t)Z * kWave;
    Val *sc = xc + (size_t)X * kWave;
    Val *dsc = sc + (size_t)S * kWave;
    Val *dxc = dsc + (size_t)S * kWave;
    Val *dyc = dxc + (size_t)X * kWave;

    if (!kGroupIsReceiver) {
        for (int q = 0; q < nchunks; q++) {
            const int c = q * kWave + lane;
            if (c < channels) {
                Val *row = dx + (int64_t)g * lx.row + (int64_t)c * lx.chan;
                for (int j = 0; j < X; j++) row[(int64_t)j * lx.dim] = Val(0);
            }
        }
    }

    CoefChunk<Idx, Val> next;
    if (num_coef > 0) next.load(coef, 0, num_coef, lane);

    const int e0 = row_ptr[g], e1 = row_ptr[g + 1];
    for (int e = e0; e < e1; e++) {
        const int o = other[e];
        if ((unsigned)o >= (unsigned)num_nodes) continue;  // padding edge: zero-filled separately
        const int64_t ee = perm ? (int64_t)perm[e] : (int64_t)e;
        const int xnode = kGroupIsReceiver ? o : g;
        const int znode = kGroupIsReceiver ? g : o;
        const EdgeY<Val, kYLane> ye(y + ee * num_y, num_y, lane);
        for (int k = 0; k < num_y; k++) dyc[k * kWave] = Val(0);

        for (int q = 0; q < nchunks; q++) {
            const int c = q * kWave + lane;
            const bool active = c < channels;
            const int cr = active ? c : channels - 1;  // channel whose rows an idle lane reads
            stage_column(zc, dm + (int64_t)znode * lo.row + (int64_t)cr * lo.chan, lo.dim, Z, active);
            stage_column(xc, x + (int64_t)xnode * lx.row + (int64_t)cr * lx.chan, lx.dim, X, active);
            stage_column(sc, s + ee * ls.row + (int64_t)cr * ls.chan, ls.dim, S, active);
            for (int j = 0; j < X; j++) dxc[j * kWave] = Val(0);
            for (int l = 0; l < S; l++) dsc[l * kWave] = Val(0);
            for (int n0 = 0; n0 < num_coef; n0 += kWave) {
                const CoefChunk<Idx, Val> chunk = next;
                next.load(coef, n0 + kWave < num_coef ? n0 + kWave : 0, num_coef, lane);
                const int nn = num_coef - n0 < kWave ? num_coef - n0 : kWave;
                for (int u = 0; u < nn; u += kCoefBatch) {
                    CoefFields<Val> cf[kCoefBatch];
                    Val dz[kCoefBatch], xv[kCoefBatch], sv[kCoefBatch], yv[kCoefBatch];
#pragma unroll
                    for (int v = 0; v < kCoefBatch; v++) {
                        cf[v] = chunk.pick(u + v < nn ? u + v : nn - 1);
                        // cols_ji: the table's first two columns hold (x, output) coordinates, as in
                        // the dx-transposed copy the reference passes (src/e3j/ops/convolution.py:367).
                        if (cols_ji) { const int t = cf[v].i; cf[v].i = cf[v].j; cf[v].j = t; }
                        dz[v] = zc[cf[v].i * kWave];
                        xv[v] = xc[cf[v].j * kWave];
                        sv[v] = sc[cf[v].l * kWave];
                        yv[v] = ye[cf[v].k];
                    }
#pragma unroll
                    for (int v = 0; v < kCoefBatch; v++) {
                        if (u + v >= nn) break;
                        const Val gz = dz[v] * sv[v];
                        const Val t = cf[v].val * yv[v];
                        // (LDS float adds retire far slower than a read, an add and a write)
                        dxc[cf[v].j * kWave] += t * gz;
                        dsc[cf[v].l * kWave] += (t * dz[v]) * xv[v];
                        dyc[cf[v].k * kWave] += (cf[v].val * gz) * xv[v];
                    }
                }
            }
            if (active) {
                Val *dsrow = ds + ee * ls.row + (int64_t)c * ls.chan;
                for (int l = 0; l < S; l++) dsrow[(int64_t)l * ls.dim] = dsc[l * kWave];
                Val *dxrow = dx + (int64_t)xnode * lx.row + (int64_t)c * lx.chan;
                for (int j = 0; j < X; j++) {
                    if constexpr (kGroupIsReceiver) unsafeAtomicAdd(dxrow + (int64_t)j * lx.dim, dxc[j * kWave]);
                    else dxrow[(int64_t)j * lx.dim] += dxc[j * kWave];
                }
            }
        }
        for (int k = 0; k < num_y; k++) {
            const Val total = wave_sum(dyc[k * kWave]);
            if (lane == 0) dy[ee * num_y + k] = total;
        }
    }
}

// dy/ds rows of padding edges: positions past the last row, or whose gathered
// endpoint is out of range (lib/e3j_ops/cuda/convolution/bwd.cuh:308-319).
// A wave inspects 64 positions at a time (one per lane) and then zeroes the rows of the
// padding positions among them together; live graphs have few, so this is one pass over
// the index array.
template <typename Val>
__global__ void zero_padding_edges_kernel(const int32_t *__restrict__ other,
                                          const int32_t *__restrict__ row_ptr,
                                          const int32_t *__restrict__ perm, int num_nodes,
                                          int64_t num_edges, Val *__restrict__ dy, int num_y,
                                          Val *__restrict__ ds, int64_t ds_row) {
    const int lane = threadIdx.x;
    const int64_t live_end = row_ptr[num_nodes];
    const int64_t stride = (int64_t)gridDim.x * blockDim.y * kWave;
    for (int64_t base = ((int64_t)blockIdx.x * blockDim.y + threadIdx.y) * kWave; base < num_edges;
         base += stride) {
        const int64_t e = base + lane;
        bool padding = false;
        if (e < num_edges) padding = e >= live_end || (unsigned)other[e] >= (unsigned)num_nodes;
        uint64_t mask = __ballot(padding);
        while (mask) {
            const int src = __ffsll((unsigned long long)mask) - 1;
            mask &= mask - 1;
            const int64_t pos = base + src;
            const int64_t ee = perm ? (int64_t)perm[pos] : pos;
            for (int k = lane; k < num_y; k += kWave) dy[ee * num_y + k] = Val(0);
            for (int64_t t = lane; t < ds_row; t += kWave) ds[ee * ds_row + t] = Val(0);
        }
    }
}

// n_words whole words, then `tail_halves` (0 or 1) two-byte values behind them
__global__ void fill_zero_kernel(uint32_t *__restrict__ p, size_t n_words, int tail_halves) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t first = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (size_t i = first; i < n_words; i += stride) p[i] = 0u;
    if (tail_halves && first == 0) *reinterpret_cast<uint16_t *>(p + n_words) = 0;
}

constexpr size_t kMaxLds = 160 * 1024;  // LDS per CU / per workgroup on gfx950

// waves per block such that the block's LDS stays within `budget`
int pick_waves(size_t per_wave_bytes, size_t budget) {
    int w = (int)(budget / per_wave_bytes);
    return w < 1 ? 1 : (w > 4 ? 4 : w);
}

template <typename Idx, typename Val>
int run_fwd(const e3j_amd_conv_params &p, const void *coef, const void *x, const void *y,
            const void *s, const int32_t *other, const int32_t *row_ptr, const int32_t *perm,
            void *out, hipStream_t stream, const int32_t *plan, bool plan_only) {
    const int nchunks = (p.channels + kWave - 1) / kWave;
    if (plan && plan_only)  // a plan the caller vouches for: the planned kernel alone
        return launch_planned_fwd(p, plan, x, y, s, other, row_ptr, perm, out, stream);
    const size_t per_wave = (size_t)(p.num_out + p.num_x + p.num_scalars) * kWave * sizeof(Val);
    if (per_wave > kMaxLds)  // (before anything is launched)
        return set_error(E3J_AMD_UNIMPLEMENTED, "convolution: num_out + num_x + num_scalars = " +
                         std::to_string(p.num_out + p.num_x + p.num_scalars) +
                         " exceeds the LDS capacity of the table-driven kernel");
    if (plan) {  // runs if the plan took the table; the kernel below runs if it did not
        int rc = launch_planned_fwd(p, plan, x, y, s, other, row_ptr, perm, out, stream);
        if (rc) return rc;
    }
    const int waves = pick_waves(per_wave, 64 * 1024);
    const size_t lds = per_wave * waves;
    // y rows of up to 64 components travel in a register of the wave
    auto kernel = p.num_y <= kWave ? generic_fwd_kernel<Idx, Val, true> : generic_fwd_kernel<Idx, Val, false>;
    if (lds > 64 * 1024) {
        int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                           "hipFuncSetAttribute(fwd)");
        if (rc) return rc;
    }
    const int64_t items = (int64_t)p.num_nodes * nchunks;
    const int64_t blocks = (items + waves - 1) / waves;
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: grid too large");
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(kWave, waves), lds, stream,
                       static_cast<const Coef4D<Idx, Val> *>(coef), p.num_coef,
                       static_cast<const Val *>(x), make_layout(p.layout, p.num_x, p.channels),
                       static_cast<const Val *>(y), p.num_y,
                       static_cast<const Val *>(s), make_layout(p.layout, p.num_scalars, p.channels),
                       other, row_ptr, perm, p.row_order,
                       static_cast<Val *>(out), make_layout(p.layout, p.num_out, p.channels),
                       p.num_nodes, p.channels, p.num_x, p.num_scalars, p.num_out, nchunks, plan);
    return check_hip(hipGetLastError(), "convolution forward launch");
}

template <typename Val>
int zero_padding(const e3j_amd_conv_params &p, const int32_t *other, const int32_t *row_ptr,
                 const int32_t *perm, Val *dy, Val *ds, hipStream_t stream) {
    if (p.num_edges == 0) return E3J_AMD_OK;
    const int64_t zblocks = std::min<int64_t>((p.num_edges + 4 * kWave - 1) / (4 * kWave), 2048);
    hipLaunchKernelGGL(zero_padding_edges_kernel<Val>, dim3((unsigned)zblocks), dim3(kWave, 4), 0,
                       stream, other, row_ptr, perm, p.num_nodes, p.num_edges, dy, p.num_y, ds,
                       (int64_t)p.num_scalars * p.channels);
    return check_hip(hipGetLastError(), "convolution backward padding launch");
}

template <typename Idx, typename Val>
int run_bwd(const e3j_amd_conv_params &p, bool group_is_receiver, const void *coef, const void *x,
            const void *y, const void *s, const void *dm, const int32_t *other,
            const int32_t *row_ptr, const int32_t *perm, void *dx, void *dy, void *ds,
            hipStream_t stream, bool cols_ji, const int32_t *plan, bool plan_only) {
    const int nchunks = (p.channels + kWave - 1) / kWave;
    if (std::is_same<Val, half_t>::value && group_is_receiver)
        // no float atomics on half values: rows must own their dx (sender-grouped)
        return set_error(E3J_AMD_UNIMPLEMENTED,
                         "convolution_bwd: float16 runs the sender-grouped backward only (dx by "
                         "float atomics has no half-precision form)");
    const size_t per_wave =
        (size_t)(p.num_out + 2 * p.num_x + 2 * p.num_scalars + p.num_y) * kWave * sizeof(Val);
    if (per_wave > kMaxLds && !(plan && plan_only))
        return set_error(E3J_AMD_UNIMPLEMENTED,
                         "convolution_bwd: irreps dimensions exceed the LDS capacity of the "
                         "table-driven kernel");
    const int waves = pick_waves(per_wave, 64 * 1024);
    const size_t lds = per_wave * waves;
    const int64_t blocks = ((int64_t)p.num_nodes + waves - 1) / waves;
    const RowLayout lx = make_layout(p.layout, p.num_x, p.channels);
    const RowLayout ls = make_layout(p.layout, p.num_scalars, p.channels);
    const RowLayout lo = make_layout(p.layout, p.num_out, p.channels);
    int rc = 0;
    if (group_is_receiver) {
        rc = launch_fill_zero(dx, (size_t)p.num_nodes * p.num_x * p.channels * sizeof(Val), stream);
        if (rc) return rc;
    }
    if (plan && group_is_receiver && nchunks > 1) {  // the waves of an edge add their dy parts
        rc = launch_fill_zero(dy, (size_t)p.num_edges * p.num_y * sizeof(Val), stream);
        if (rc) return rc;
    }
    rc = zero_padding<Val>(p, other, row_ptr, perm, static_cast<Val *>(dy), static_cast<Val *>(ds), stream);
    if (rc) return rc;
    if (plan) {  // runs if the plan took the table; the kernel below runs if it did not
        rc = launch_planned_bwd(p, group_is_receiver, plan, x, y, s, dm, other, row_ptr, perm, dx, dy, ds, stream);
        if (rc || plan_only) return rc;  // (a plan the caller vouches for: the planned kernel alone)
    }
#define E3J_LAUNCH_BWD(FLAG)                                                                      \
    do {                                                                                          \
        auto kernel = p.num_y <= kWave ? generic_bwd_kernel<Idx, Val, FLAG, true>                 \
                                       : generic_bwd_kernel<Idx, Val, FLAG, false>;               \
        if (lds > 64 * 1024) {                                                                    \
            rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),            \
                                               hipFuncAttributeMaxDynamicSharedMemorySize,        \
                                               (int)lds),                                         \
                           "hipFuncSetAttribute(bwd)");                                           \
            if (rc) return rc;                                                                    \
        }                                                                                         \
        hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(kWave, waves), lds, stream,       \
                           static_cast<const Coef4D<Idx, Val> *>(coef), p.num_coef,               \
                           static_cast<const Val *>(x), lx, static_cast<const Val *>(y), p.num_y, \
                           static_cast<const Val *>(s), ls, static_cast<const Val *>(dm), lo,     \
                           other, row_ptr, perm, p.row_order, static_cast<Val *>(dx),             \
                           static_cast<Val *>(dy),                                               \
                           static_cast<Val *>(ds), p.num_nodes, p.channels, p.num_x,              \
                           p.num_scalars, p.num_out, nchunks, cols_ji ? 1 : 0, plan);             \
    } while (0)
    if constexpr (std::is_same<Val, half_t>::value) {
        E3J_LAUNCH_BWD(false);
    } else {
        if (group_is_receiver) E3J_LAUNCH_BWD(true);
        else E3J_LAUNCH_BWD(false);
    }
#undef E3J_LAUNCH_BWD
    return check_hip(hipGetLastError(), "convolution backward launch");
}

// Atomic-free dx: sum the per-position contribution rows of every sender in ascending
// position order (a fixed order: the result is bit-reproducible).  One wave per (sender,
// 256-float piece of the row); x coordinates no coefficient touches read as zero.
__global__ __launch_bounds__(256) void reduce_ordered_dx_kernel(
    const float *__restrict__ u, const int32_t *__restrict__ sender_ptr,
    const int32_t *__restrict__ sender_pos, int num_nodes, int row_floats, int num_x,
    int channels, int trailing, unsigned long long covered, float *__restrict__ dx) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const int pieces = (row_floats + 255) / 256;
    const int64_t item = (int64_t)blockIdx.x * blockDim.y + threadIdx.y;
    if (item >= (int64_t)num_nodes * pieces) return;
    const int n = (int)(item / pieces);
    const int first = ((int)(item % pieces) * kWave + threadIdx.x) * 4;  // first float of the lane
    if (first >= row_floats) return;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    const int t1 = sender_ptr[n + 1];
    int t = sender_ptr[n];
    auto row = [&](int at) {
        return __builtin_nontemporal_load(
            reinterpret_cast<const f32x4 *>(u + (int64_t)sender_pos[at] * row_floats + first));
    };
    for (; t + 8 <= t1; t += 8) {  // eight rows in flight, added in position order
        f32x4 v[8];
#pragma unroll
        for (int q = 0; q < 8; q++) v[q] = row(t + q);
#pragma unroll
        for (int q = 0; q < 8; q++) acc += v[q];
    }
    for (; t < t1; t++) acc += row(t);
#pragma unroll
    for (int q = 0; q < 4; q++) {
        // trailing layout (X, K): coordinate = index / K; leading (K, X): coordinate = index % X
        const int coord = trailing ? (first + q) / channels : (first + q) % num_x;
        if (!((covered >> coord) & 1ull)) acc[q] = 0.f;
    }
    *reinterpret_cast<f32x4 *>(dx + (int64_t)n * row_floats + first) = acc;
}

// dy of every position from the slots its waves filled, in slot order.
__global__ void reduce_ordered_dy_kernel(const float *__restrict__ dy_slots, int slots, int num_y,
                                         int64_t num_edges, const int32_t *__restrict__ perm,
                                         float *__restrict__ dy) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < num_edges * num_y; i += stride) {
        const int64_t pos = i / num_y;
        const int k = (int)(i % num_y);
        float total = 0.f;
        for (int q = 0; q < slots; q++) total += dy_slots[(pos * slots + q) * num_y + k];
        const int64_t ee = perm ? (int64_t)perm[pos] : pos;
        dy[ee * num_y + k] = total;
    }
}

}  // namespace

int reduce_ordered_dx(const e3j_amd_conv_params &p, const float *u, const int32_t *sender_ptr,
                      const int32_t *sender_pos, unsigned long long covered, float *dx,
                      hipStream_t stream) {
    const int row_floats = p.num_x * p.channels;
    if (row_floats % 4 != 0 || p.num_x > 64)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution_bwd_ordered: unsupported row shape");
    if (p.num_nodes == 0) return E3J_AMD_OK;
    const int pieces = (row_floats + 255) / 256;
    const int64_t blocks = ((int64_t)p.num_nodes * pieces + 3) / 4;
    hipLaunchKernelGGL(reduce_ordered_dx_kernel, dim3((unsigned)blocks), dim3(kWave, 4), 0, stream, u,
                       sender_ptr, sender_pos, p.num_nodes, row_floats, p.num_x, p.channels,
                       p.layout == E3J_AMD_LAYOUT_TRAILING ? 1 : 0, covered, dx);
    return check_hip(hipGetLastError(), "ordered dx reduction launch");
}

int reduce_ordered_dy(const e3j_amd_conv_params &p, const float *dy_slots, int slots,
                      const int32_t *perm, float *dy, hipStream_t stream) {
    if (p.num_edges == 0) return E3J_AMD_OK;
    const int64_t total = p.num_edges * p.num_y;
    const unsigned blocks = (unsigned)std::min<int64_t>((total + 255) / 256, 8192);
    hipLaunchKernelGGL(reduce_ordered_dy_kernel, dim3(blocks), dim3(256), 0, stream, dy_slots, slots,
                       p.num_y, p.num_edges, perm, dy);
    return check_hip(hipGetLastError(), "ordered dy reduction launch");
}

int launch_fill_zero(void *ptr, size_t bytes, hipStream_t stream) {
    if (bytes == 0) return E3J_AMD_OK;
    // whole 32-bit words, and one trailing half value (an odd number of float16 elements)
    if (bytes % 2 != 0 || (reinterpret_cast<uintptr_t>(ptr) % 4) != 0)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "fill: buffer must be 4-byte aligned");
    const size_t words = bytes / 4;
    const size_t blocks = std::max<size_t>(1, std::min<size_t>((words + 255) / 256, 8192));
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                       static_cast<uint32_t *>(ptr), words, (int)(bytes % 4 / 2));
    return check_hip(hipGetLastError(), "fill launch");
}

int launch_zero_padding(const e3j_amd_conv_params &p, const int32_t *other, const int32_t *row_ptr,
                        const int32_t *perm, float *dy, float *ds, hipStream_t stream) {
    return zero_padding<float>(p, other, row_ptr, perm, dy, ds, stream);
}
int launch_zero_padding(const e3j_amd_conv_params &p, const int32_t *other, const int32_t *row_ptr,
                        const int32_t *perm, double *dy, double *ds, hipStream_t stream) {
    return zero_padding<double>(p, other, row_ptr, perm, dy, ds, stream);
}
int launch_zero_padding(const e3j_amd_conv_params &p, const int32_t *other, const int32_t *row_ptr,
                        const int32_t *perm, half_t *dy, half_t *ds, hipStream_t stream) {
    return zero_padding<half_t>(p, other, row_ptr, perm, dy, ds, stream);
}

// The plan of a table the planned kernels can take (conv_planned.hip): in the caller's memory
// (e3j_amd_conv_params.table_plan) or, without it, in memory of the stream's pool for the length
// of the call; none when the sizes are outside the plan's limits, when planning is switched off,
// and, for pool memory, when the stream is being captured into a graph (the call then allocates
// nothing) or when the pool gives nothing.
struct PlanScratch {
    int32_t *plan = nullptr;
    bool pooled = false;  // plan memory taken from the stream's pool (given back when the call returns)
    bool ready = false;   // the caller vouches for a plan built earlier that takes the table: no other kernel runs
    hipStream_t stream;
    int rc = E3J_AMD_OK;
    PlanScratch(const e3j_amd_conv_params &p, const void *coef, bool cols_ji, hipStream_t st) : stream(st) {
        if (p.table_plan_state == E3J_AMD_PLAN_NONE) return;
        if (p.table_plan_state != E3J_AMD_PLAN_BUILD && p.table_plan_state != E3J_AMD_PLAN_READY) {
            rc = set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: unknown table_plan_state");
            return;
        }
        if (!plan_takes(p) || !table_plans().load(std::memory_order_relaxed)) return;
        if (p.table_plan_state == E3J_AMD_PLAN_READY) {
            if (p.table_plan == nullptr || reinterpret_cast<uintptr_t>(p.table_plan) % alignof(int32_t) != 0) {
                rc = set_error(E3J_AMD_INVALID_ARGUMENT,
                               "convolution: table_plan_state says the plan is ready, table_plan holds none");
                return;
            }
            plan = p.table_plan;
            ready = true;
            return;
        }
        if (p.table_plan != nullptr) {  // the caller's memory: nothing allocated, fine under capture
            if (reinterpret_cast<uintptr_t>(p.table_plan) % alignof(int32_t) != 0) {
                rc = set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: table_plan must be 4-byte aligned");
                return;
            }
            plan = p.table_plan;
            rc = launch_plan_build(p, coef, cols_ji, plan, stream);
            return;
        }
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &capture) != hipSuccess) {
            (void)hipGetLastError();
            return;
        }
        if (capture != hipStreamCaptureStatusNone) return;
        void *mem = nullptr;
        if (hipMallocAsync(&mem, plan_bytes(p), stream) != hipSuccess) {
            (void)hipGetLastError();
            return;
        }
        plan = static_cast<int32_t *>(mem);
        pooled = true;
        rc = launch_plan_build(p, coef, cols_ji, plan, stream);
    }
    ~PlanScratch() {
        if (pooled) (void)hipFreeAsync(plan, stream);
    }
    PlanScratch(const PlanScratch &) = delete;
    PlanScratch &operator=(const PlanScratch &) = delete;
};

#define E3J_DISPATCH(CALL)                                                                  \
    if (p.val_dtype == E3J_AMD_F32 && p.coef_idx_bytes == 1) return CALL(uint8_t, float);   \
    if (p.val_dtype == E3J_AMD_F32 && p.coef_idx_bytes == 4) return CALL(int32_t, float);   \
    if (p.val_dtype == E3J_AMD_F64 && p.coef_idx_bytes == 1) return CALL(uint8_t, double);  \
    if (p.val_dtype == E3J_AMD_F64 && p.coef_idx_bytes == 4) return CALL(int32_t, double);  \
    if (p.val_dtype == E3J_AMD_F16 && p.coef_idx_bytes == 1) return CALL(uint8_t, half_t);  \
    if (p.val_dtype == E3J_AMD_F16 && p.coef_idx_bytes == 4) return CALL(int32_t, half_t);  \
    return set_error(E3J_AMD_INVALID_ARGUMENT, "unsupported (IDX, VAL) dtype pair")

int launch_generic_fwd(const e3j_amd_conv_params &p, const void *coef, const void *x, const void *y,
                       const void *s, const int32_t *other, const int32_t *row_ptr,
                       const int32_t *edge_perm, void *out, hipStream_t stream) {
    const PlanScratch scratch(p, coef, false, stream);
    if (scratch.rc) return scratch.rc;
    const int32_t *plan = scratch.plan;
#define E3J_FWD(I, V) run_fwd<I, V>(p, coef, x, y, s, other, row_ptr, edge_perm, out, stream, plan, scratch.ready)
    E3J_DISPATCH(E3J_FWD);
#undef E3J_FWD
}

int launch_generic_bwd(const e3j_amd_conv_params &p, bool group_is_receiver, const void *coef,
                       const void *x, const void *y, const void *s, const void *dm,
                       const int32_t *other, const int32_t *row_ptr, const int32_t *edge_perm,
                       void *dx, void *dy, void *ds, hipStream_t stream, bool coef_cols_ji) {
    const PlanScratch scratch(p, coef, coef_cols_ji, stream);
    if (scratch.rc) return scratch.rc;
    const int32_t *plan = scratch.plan;
#define E3J_BWD(I, V)                                                                            \
    run_bwd<I, V>(p, group_is_receiver, coef, x, y, s, dm, other, row_ptr, edge_perm, dx, dy, ds, \
                  stream, coef_cols_ji, plan, scratch.ready)
    E3J_DISPATCH(E3J_BWD);
#undef E3J_BWD
}

}  // namespace e3j_amd
