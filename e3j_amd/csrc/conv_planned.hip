// Table-driven convolution kernels over a plan of the table (float32; any table whose output
// coordinates each use one scalar, up to 128 output coordinates, 16 x coordinates, 64 y
// components).
//
// The contraction out[i] += c * x[j] * y[k] * s[l] (lib/e3j_ops/cuda/convolution/fwd.cuh:88-153)
// is regrouped per edge as out[i] += s[l(i)] * sum_j M[i][j] * x[j] with the channel-independent
// matrix M[i][j] = sum_k c_ijk * y[k].  A wave builds M once per edge in its strip of LDS (the
// lanes share the table's non-empty cells), and then every lane (one channel) runs loops over
// i and j whose bounds are compile-time numbers, so that x, the accumulators and the partial
// sums sit in registers under constant indices; M is read as wave-uniform 16-byte LDS
// broadcasts.  What depends on the table is data: the plan, built on the device by one
// workgroup per call (no read-back, no compiler at run time):
//   * the output coordinates in the order the loops visit them ("slots": sorted by the x
//     coordinates their path touches, then by scalar, so that rows of one scalar are adjacent
//     and blocks of 16 slots touch few groups of 4 x coordinates),
//   * a bit per (block of 16 slots, group of 4 x coordinates) that has a coefficient at all: the
//     loops skip the others with a wave-uniform branch,
//   * the non-empty cells (slot, j) with their (coefficient, k) lists in table order.
// The backward pass (lib/e3j_ops/cuda/convolution/bwd.cuh:116-321) uses the same M: ds from the
// forward's partial sums, dx[j] += M[i][j] * s[l(i)] * dm[i], and for dy the per-channel products
// x[j] * s * dm[i] of a block of 64 cells are summed over the 64 channels with a transposing
// butterfly (lane t ends with the total of cell t), multiplied with the cell's coefficients and
// added into the wave's dy row in LDS.
//
// Tables the plan cannot take (an output coordinate with two different scalars, sizes beyond the
// limits) run the kernels of conv_generic.hip: eligibility is a flag in the plan that both
// kernels read, so the host never waits for the device.

#include "common.h"

#ifndef E3J_ADDR_MODE
#define E3J_ADDR_MODE 1
#endif
#ifndef E3J_LBYTES
#define E3J_LBYTES 0
#endif

namespace e3j_amd {
namespace {

constexpr int kSlots = 128;     // output coordinates a plan holds (8 blocks of 16)
constexpr int kPlanX = 16;      // x coordinates (4 groups of 4)
constexpr int kCells = kSlots * kPlanX;
constexpr int kPlanMaxY = 64;
constexpr int kPlanMaxS = 64;       // scalars (their rows of one edge sit in the wave's LDS)
constexpr int kPlanMaxCoef = 2048;  // entries (the table sits in the workgroup's LDS; 11-bit fields)
constexpr int kPlanMaxRun = 255;    // entries of one cell
constexpr int kBuildThreads = 256;

// header words
enum { kEligible = 0, kNumCells = 1, kChunkMask = 2, kNumZeroL = 3, kMaxRun = 4, kHeaderWords = 8 };

struct PlanLayout {  // offsets in 32-bit words
    // slot_row, slot_l: output coordinate and scalar of a slot; first, count: the entries of a dense
    // cell (slot * 16 + j); cells: the non-empty cells packed as cell | first << 11 | count << 22;
    // pairs: (coefficient bits, k) of the entries, cell by cell; coef, k, t, cell_list: working arrays
    // of the builder; zero_l: scalars no entry uses
    // slot_l8, slot_row8: the same as bytes, four slots to a word, 255 = none
    int slot_row, slot_l, slot_l8, slot_row8, first, count, cell_list, cells, pairs, coef, k, t, zero_l, words;
    PlanLayout(int num_coef, int num_scalars) {
        int at = kHeaderWords;
        auto take = [&](int n) { const int here = at; at += (n + 3) / 4 * 4; return here; };
        slot_row = take(kSlots); slot_l = take(kSlots); slot_l8 = take(kSlots / 4); slot_row8 = take(kSlots / 4);
        first = take(kCells); count = take(kCells); cell_list = take(kCells); cells = take(kCells);
        pairs = take(2 * num_coef);
        coef = take(num_coef); k = take(num_coef); t = take(num_coef);
        zero_l = take(num_scalars);
        words = at;
    }
};

// words of LDS the staged table takes (cells, then pairs from an even word on)
__host__ __device__ inline int table_words(int num_coef) {
    const int cells = num_coef < kCells ? num_coef : kCells;
    return ((cells + 1) / 2 * 2 + 2 * num_coef + 3) / 4 * 4;
}

__device__ __forceinline__ int wave_max_int(int v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const int o = __shfl_xor(v, off, kWave);
        v = o > v ? o : v;
    }
    return v;
}

template <typename Idx>
__device__ inline void decode(const Coef4D<Idx, float> &c, int cols_ji, int &i, int &j, int &k, int &l) {
    i = (int)c.i; j = (int)c.j; k = (int)c.k; l = (int)c.l;
    if (cols_ji) { const int t = i; i = j; j = t; }
}

// One workgroup turns the table into the plan.
template <typename Idx>
__global__ __launch_bounds__(kBuildThreads) void plan_build_kernel(
    const Coef4D<Idx, float> *__restrict__ coef, int num_coef, int X, int Y, int Z, int S, int xg, int cols_ji,
    int32_t *__restrict__ plan, PlanLayout L) {
    __shared__ int lmin[kSlots], lmax[kSlots], support[kSlots], slot_of_row[kSlots];
    __shared__ int path_support[kPlanMaxS], referenced[kPlanMaxS];
    __shared__ int eligible, chunk_mask, num_cells, num_zero_l, max_run;
    __shared__ int scan[kBuildThreads];
    const int tid = threadIdx.x;
    if (tid == 0) { eligible = 1; chunk_mask = 0; num_cells = 0; num_zero_l = 0; max_run = 0; }
    for (int i = tid; i < kSlots; i += kBuildThreads) { lmin[i] = 0x7fffffff; lmax[i] = -1; support[i] = 0; }
    for (int l = tid; l < S; l += kBuildThreads) { path_support[l] = 0; referenced[l] = 0; }
    for (int c = tid; c < kCells; c += kBuildThreads) plan[L.count + c] = 0;
    __syncthreads();
    // rows: the scalars and the groups of x coordinates their entries use
    for (int n = tid; n < num_coef; n += kBuildThreads) {
        int i, j, k, l;
        decode(coef[n], cols_ji, i, j, k, l);
        if ((unsigned)i >= (unsigned)Z || (unsigned)j >= (unsigned)X || (unsigned)k >= (unsigned)Y ||
            (unsigned)l >= (unsigned)S) { eligible = 0; continue; }
        atomicMin(&lmin[i], l); atomicMax(&lmax[i], l); atomicOr(&support[i], 1 << (j >> 2));
    }
    __syncthreads();
    for (int i = tid; i < Z; i += kBuildThreads) {
        if (lmax[i] < 0) continue;
        if (lmin[i] != lmax[i]) { eligible = 0; continue; }
        atomicOr(&path_support[lmax[i]], support[i]);
        referenced[lmax[i]] = 1;
    }
    __syncthreads();
    // slots: rows sorted by (support of the row's scalar, scalar, row); rows without entries last
    auto key = [&](int i) {
        return lmax[i] < 0 ? (1 << 30) | i : (path_support[lmax[i]] << 24) | (lmax[i] << 8) | i;
    };
    for (int i = tid; i < kSlots; i += kBuildThreads) { plan[L.slot_row + i] = -1; plan[L.slot_l + i] = -1; }
    __syncthreads();
    for (int i = tid; i < Z; i += kBuildThreads) {
        const int mine = key(i);
        int rank = 0;
        for (int o = 0; o < Z; o++) rank += key(o) < mine ? 1 : 0;
        slot_of_row[i] = rank;
        plan[L.slot_row + rank] = i;
        plan[L.slot_l + rank] = lmax[i];
    }
    if (tid == 0) {  // scalars no row uses: their ds rows are zeros
        for (int l = 0; l < S; l++)
            if (!referenced[l]) plan[L.zero_l + num_zero_l++] = l;
    }
    __syncthreads();
    if (!eligible) {
        if (tid == 0) plan[kEligible] = 0;
        return;  // (uniform: `eligible` is shared and was last written before the barrier)
    }
    // cells: entry counts, then their places (an exclusive scan over the dense cell array)
    for (int n = tid; n < num_coef; n += kBuildThreads) {
        int i, j, k, l;
        decode(coef[n], cols_ji, i, j, k, l);
        atomicAdd(&plan[L.count + slot_of_row[i] * kPlanX + j], 1);
    }
    __syncthreads();
    constexpr int kPer = kCells / kBuildThreads;  // consecutive cells per thread
    int sum = 0, live = 0;
    for (int q = 0; q < kPer; q++) {
        const int c = plan[L.count + tid * kPer + q];
        sum += c; live += c > 0 ? 1 : 0;
    }
    // two scans with one buffer: entries (low 16 bits hold up to 8192) and live cells (high bits)
    scan[tid] = sum | (live << 16);
    __syncthreads();
    for (int off = 1; off < kBuildThreads; off *= 2) {
        const int add = tid >= off ? scan[tid - off] : 0;
        __syncthreads();
        scan[tid] += add;
        __syncthreads();
    }
    {
        const int before = tid ? scan[tid - 1] : 0;
        int at = before & 0xffff, cell_at = before >> 16;
        for (int q = 0; q < kPer; q++) {
            const int cell = tid * kPer + q;
            const int c = plan[L.count + cell];
            plan[L.first + cell] = at;
            at += c;
            if (c > 0) {
                plan[L.cell_list + cell_at++] = cell;
                atomicOr(&chunk_mask, 1 << ((cell / kPlanX / 16) * xg + (cell % kPlanX) / 4));
            }
        }
        if (tid == kBuildThreads - 1) num_cells = scan[tid] >> 16;
    }
    __syncthreads();
    // entries to their cells; table order inside a cell (a fixed summation order)
    for (int c = tid; c < kCells; c += kBuildThreads) plan[L.count + c] = 0;
    __syncthreads();
    for (int n = tid; n < num_coef; n += kBuildThreads) {
        int i, j, k, l;
        decode(coef[n], cols_ji, i, j, k, l);
        const int cell = slot_of_row[i] * kPlanX + j;
        const int at = plan[L.first + cell] + atomicAdd(&plan[L.count + cell], 1);
        plan[L.coef + at] = __float_as_int(coef[n].val);
        plan[L.k + at] = k;
        plan[L.t + at] = n;
    }
    __syncthreads();
    for (int cell = tid; cell < kCells; cell += kBuildThreads) {
        const int first = plan[L.first + cell], cnt = plan[L.count + cell];
        for (int a = 1; a < cnt; a++) {  // insertion sort by table position
            const int t = plan[L.t + first + a], cf = plan[L.coef + first + a], kk = plan[L.k + first + a];
            int b = a - 1;
            while (b >= 0 && plan[L.t + first + b] > t) {
                plan[L.t + first + b + 1] = plan[L.t + first + b];
                plan[L.coef + first + b + 1] = plan[L.coef + first + b];
                plan[L.k + first + b + 1] = plan[L.k + first + b];
                b--;
            }
            plan[L.t + first + b + 1] = t; plan[L.coef + first + b + 1] = cf; plan[L.k + first + b + 1] = kk;
        }
        if (cnt > kPlanMaxRun) eligible = 0;
        if (cnt > 0) atomicMax(&max_run, cnt);
    }
    for (int w = tid; w < kSlots / 4; w += kBuildThreads) {
        unsigned lw = 0, rw = 0;
        for (int q = 0; q < 4; q++) {
            const int l = plan[L.slot_l + 4 * w + q], row = plan[L.slot_row + 4 * w + q];
            lw |= (unsigned)(l < 0 ? 255 : l) << (8 * q);
            rw |= (unsigned)(row < 0 ? 255 : row) << (8 * q);
        }
        plan[L.slot_l8 + w] = (int)lw;
        plan[L.slot_row8 + w] = (int)rw;
    }
    __syncthreads();
    // the forms the kernels stage in LDS
    for (int q = tid; q < num_cells; q += kBuildThreads) {
        const int cell = plan[L.cell_list + q];
        plan[L.cells + q] = cell | (plan[L.first + cell] << 11) | (plan[L.count + cell] << 22);
    }
    for (int n = tid; n < num_coef; n += kBuildThreads) {
        plan[L.pairs + 2 * n] = plan[L.coef + n];
        plan[L.pairs + 2 * n + 1] = plan[L.k + n];
    }
    if (tid == 0) {
        plan[kEligible] = eligible; plan[kNumCells] = num_cells; plan[kChunkMask] = chunk_mask;
        plan[kNumZeroL] = num_zero_l; plan[kMaxRun] = max_run;
    }
}

// LDS traffic between the lanes of one wave: its LDS operations complete in program order, so
// only the compiler has to be kept from moving accesses across this point.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int kAhead = 32;  // scalar rows of the next edge a wave holds in registers

// The table part of the plan in LDS, shared by the waves of a workgroup: the packed cells, then
// (coefficient, k) pairs.  Every thread of the workgroup calls this (it holds a barrier).
// `dense` (backward): first | count << 11 of the first `dense_cells` dense cells behind them.
__device__ __forceinline__ void stage_table(const int32_t *__restrict__ plan, const PlanLayout &L, int num_cells,
                                            int num_coef, int32_t *tab, int dense_cells = 0) {
    const int tid = threadIdx.y * kWave + threadIdx.x, threads = blockDim.y * kWave;
    const int pairs = (num_cells + 1) & ~1;  // the pairs start at an even word
    for (int t = tid; t < num_cells; t += threads) tab[t] = plan[L.cells + t];
    for (int t = tid; t < 2 * num_coef; t += threads) tab[pairs + t] = plan[L.pairs + t];
    int32_t *dense = tab + table_words(num_coef);
    for (int t = tid; t < dense_cells; t += threads) {
        const int cnt = plan[L.count + t];  // (an empty cell behind the last entry has first = 2048: dropped)
        dense[t] = cnt > 0 ? plan[L.first + t] | (cnt << 11) : 0;
    }
    __syncthreads();
}

// M of one edge: lane q takes the cells q, q + 64, ... of the staged list; lane k of `yreg` holds y[k].
template <int XG>
__device__ __forceinline__ void build_edge_matrix(const int32_t *tab, int num_cells, int most, float yreg, float *M,
                                                  int lane) {
    const int pairs = (num_cells + 1) & ~1;
    for (int q0 = 0; q0 < num_cells; q0 += kWave) {  // (all lanes run the same trips: the lane reads below are shuffles)
        const int q = q0 + lane;
        const unsigned w = (unsigned)tab[q < num_cells ? q : 0];
        const int cell = (int)(w & 2047u), first = (int)((w >> 11) & 2047u);
        const int cnt = q < num_cells ? (int)(w >> 22) : 0;
        float sum = 0.f;
        for (int r = 0; r < most; r++) {
            const int at = r < cnt ? first + r : first;
            const int kk = tab[pairs + 2 * at + 1];
            const float cf = r < cnt ? __int_as_float(tab[pairs + 2 * at]) : 0.f;
            sum += cf * __shfl(yreg, kk, kWave);
        }
        if (cnt > 0) {
            const int slot = cell / kPlanX, j = cell % kPlanX;
            M[(slot * XG + (j >> 2)) * 4 + (j & 3)] = sum;
        }
    }
}

__device__ __forceinline__ int next_live(const int32_t *__restrict__ other, int e, int e1, int num_nodes) {
    while (e < e1 && (unsigned)other[e] >= (unsigned)num_nodes) e++;  // padding edges are stepped over
    return e;
}

// A row of an operand: `base` is wave-uniform, the lanes differ by a 32-bit offset, so that the
// load takes a scalar base and one offset register.
__device__ __forceinline__ const float *row_at(const float *base, int64_t row_stride, int row) {
    return base + (int64_t)row * row_stride;
}
// element `lane_off + row * stride` behind a wave-uniform base: one scalar base, one 32-bit offset
__device__ __forceinline__ float load_row(const float *base, unsigned lane_off, unsigned stride, int row) {
#if E3J_ADDR_MODE == 0
    return (base + lane_off)[(int64_t)row * stride];   // per-lane pointer, 64-bit row offset
#elif E3J_ADDR_MODE == 1
    return (base + (int64_t)row * stride)[lane_off];   // scalar row pointer, lane offset
#else
    return base[lane_off + (unsigned)row * stride];
#endif
}
// slot byte q of a packed word array held in scalar registers
#define E3J_SLOT_BYTE(words, slot) (((words)[(slot) / 4] >> (8 * ((slot) % 4))) & 255u)

template <int NB, int XG>
__global__ __launch_bounds__(256, 2) void planned_fwd_kernel(
    const int32_t *__restrict__ plan, PlanLayout L, const float *__restrict__ x, RowLayout lx,
    const float *__restrict__ y, int num_y, const float *__restrict__ s, RowLayout ls,
    const int32_t *__restrict__ other, const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ row_order, float *__restrict__ out, RowLayout lo, int num_nodes, int channels,
    int X, int S, int num_coef, int nchunks) {
    extern __shared__ __align__(16) float planned_lds[];
    if (plan[kEligible] == 0) return;  // (the whole grid) the table-driven kernel without a plan runs instead
    constexpr int kStrip = NB * 16 * XG * 4;
    const int lane = threadIdx.x, wave = __builtin_amdgcn_readfirstlane((int)threadIdx.y);  // (wave-uniform: in scalar registers)
    const int num_cells = plan[kNumCells];
    const unsigned chunk_mask = (unsigned)plan[kChunkMask];
    const int max_run = plan[kMaxRun];
    int32_t *tab = reinterpret_cast<int32_t *>(planned_lds);
    float *M = planned_lds + table_words(num_coef) + wave * (kStrip + S * kWave);
    float *sbuf = M + kStrip;
    for (int t = lane; t < kStrip; t += kWave) M[t] = 0.f;
    stage_table(plan, L, num_cells, num_coef, tab);
    const int64_t item = (int64_t)blockIdx.x * blockDim.y + wave;
    if (item >= (int64_t)num_nodes * nchunks) return;  // uniform per wave; no workgroup barrier below
    const int q = (int)(item / nchunks);
    const int r = row_order ? row_order[q] : q;
    const int c = (int)(item % nchunks) * kWave + lane;
    const bool active = c < channels;
    const int cr = active ? c : channels - 1;  // channel whose rows an idle lane reads
    const unsigned xoff = (unsigned)cr * (unsigned)lx.chan, soff = (unsigned)cr * (unsigned)ls.chan;
    unsigned lbytes[NB * 4];  // the scalar of every slot, a byte each
#pragma unroll
    for (int w = 0; w < NB * 4; w++) lbytes[w] = (unsigned)plan[L.slot_l8 + w];

    float acc[NB * 16];
#pragma unroll
    for (int t = 0; t < NB * 16; t++) acc[t] = 0.f;

    const int e1 = row_ptr[r + 1];
    int e = next_live(other, row_ptr[r], e1, num_nodes);
    // operands of the edge after the one in work, loaded while that one is computed
    float yn = 0.f, xn[XG * 4], sn[kAhead];
    int64_t een = 0;
    auto issue = [&](int at) {
        const int snd = other[at];
        een = perm ? (int64_t)perm[at] : (int64_t)at;
        yn = lane < num_y ? y[een * num_y + lane] : 0.f;
        const float *xbase = x + (int64_t)snd * lx.row;
#pragma unroll
        for (int j = 0; j < XG * 4; j++) xn[j] = load_row(xbase, xoff, (unsigned)lx.dim, j < X ? j : X - 1);  // (clamped, not skipped: straight-line loads)
        const float *sbase = s + een * ls.row;
#pragma unroll
        for (int t = 0; t < kAhead; t++) sn[t] = load_row(sbase, soff, (unsigned)ls.dim, t < S ? t : S - 1);
    };
    if (e < e1) issue(e);
    while (e < e1) {
        const float ycur = yn;
        const int64_t ee = een;
        float xv[XG * 4];
#pragma unroll
        for (int j = 0; j < XG * 4; j++) xv[j] = j < X ? xn[j] : 0.f;
        wave_lds_sync();  // the reads of the edge before are behind the writes below
#pragma unroll
        for (int t = 0; t < kAhead; t++) sbuf[(t < S ? t : S - 1) * kWave + lane] = sn[t];
        for (int t = kAhead; t < S; t++)  // (rows past the ones held ahead: read now)
            sbuf[t * kWave + lane] = load_row(s + ee * ls.row, soff, (unsigned)ls.dim, t);
        const int en = next_live(other, e + 1, e1, num_nodes);
        if (en < e1) issue(en);
        build_edge_matrix<XG>(tab, num_cells, max_run, ycur, M, lane);
        wave_lds_sync();
#pragma unroll
        for (int b = 0; b < NB; b++) {
            if (((chunk_mask >> (b * XG)) & ((1u << XG) - 1u)) == 0) continue;  // no coefficient in the block
            float sv[16], T[16];
#pragma unroll
            for (int u = 0; u < 16; u++) {
                // (a slot without entries reads row 0 of s; its output row is written as zero below)
#if E3J_LBYTES
                const unsigned l = E3J_SLOT_BYTE(lbytes, b * 16 + u);
#else
                const unsigned l = (unsigned)plan[L.slot_l + b * 16 + u] & 255u;
#endif
                sv[u] = sbuf[(l == 255u ? 0u : l) * kWave + lane];
                T[u] = 0.f;
            }
#pragma unroll
            for (int g = 0; g < XG; g++) {
                if (!((chunk_mask >> (b * XG + g)) & 1u)) continue;
#pragma unroll
                for (int u = 0; u < 16; u++) {
                    const f32x4 m = *reinterpret_cast<const f32x4 *>(&M[((b * 16 + u) * XG + g) * 4]);
                    T[u] = __builtin_fmaf(m.x, xv[4 * g], T[u]);
                    T[u] = __builtin_fmaf(m.y, xv[4 * g + 1], T[u]);
                    T[u] = __builtin_fmaf(m.z, xv[4 * g + 2], T[u]);
                    T[u] = __builtin_fmaf(m.w, xv[4 * g + 3], T[u]);
                }
            }
#pragma unroll
            for (int u = 0; u < 16; u++) acc[b * 16 + u] = __builtin_fmaf(sv[u], T[u], acc[b * 16 + u]);
        }
        e = en;
    }
    if (active) {
        float *obase = out + (int64_t)r * lo.row;
        const unsigned ooff = (unsigned)c * (unsigned)lo.chan;
#pragma unroll
        for (int t = 0; t < NB * 16; t++) {
            const unsigned row = ((unsigned)plan[L.slot_row8 + t / 4] >> (8 * (t % 4))) & 255u;
            const unsigned l = E3J_SLOT_BYTE(lbytes, t);
            if (row != 255u) (obase + (int64_t)row * lo.dim)[ooff] = l == 255u ? 0.f : acc[t];
        }
    }
}

// v[t] (t < 32) summed over the 64 lanes, the total of v[t] left in lanes t and t + 32.  Five
// halving steps inside each half of the wave (lanes whose bit N is clear keep the lower half of
// the values and hand the upper half to their partner), then the two halves are added.
template <int N>  // N pairs (p, p + N) are left; partner lanes differ in bit N
__device__ __forceinline__ void transpose_sum_step(float (&v)[32], int lane) {
    const bool upper = (lane & N) != 0;
#pragma unroll
    for (int p = 0; p < N; p++) {
        const float keep = upper ? v[p + N] : v[p];
        const float send = upper ? v[p] : v[p + N];
        v[p] = keep + __shfl_xor(send, N, kWave);
    }
}
__device__ __forceinline__ float transpose_sum(float (&v)[32], int lane) {
    transpose_sum_step<16>(v, lane); transpose_sum_step<8>(v, lane); transpose_sum_step<4>(v, lane);
    transpose_sum_step<2>(v, lane); transpose_sum_step<1>(v, lane);
    return v[0] + __shfl_xor(v[0], 32, kWave);
}

enum DyMode { kDyStore = 0, kDyAdd = 1, kDyAtomic = 2 };

template <int NB, int XG>
__global__ __launch_bounds__(256, 2) void planned_bwd_kernel(
    const int32_t *__restrict__ plan, PlanLayout L, const float *__restrict__ x, RowLayout lx,
    const float *__restrict__ y, int num_y, const float *__restrict__ s, RowLayout ls,
    const float *__restrict__ dm, RowLayout lo, const int32_t *__restrict__ other,
    const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ row_order, float *__restrict__ dx, float *__restrict__ dy,
    float *__restrict__ ds, int num_nodes, int channels, int X, int S, int num_coef, int nchunks,
    int group_is_receiver) {
    extern __shared__ __align__(16) float planned_lds[];
    if (plan[kEligible] == 0) return;
    constexpr int kStrip = NB * 16 * XG * 4;
    const int lane = threadIdx.x, wave = __builtin_amdgcn_readfirstlane((int)threadIdx.y);  // (wave-uniform: in scalar registers)
    const int num_cells = plan[kNumCells];
    const unsigned chunk_mask = (unsigned)plan[kChunkMask];
    const int max_run = plan[kMaxRun];
    const int num_zero_l = plan[kNumZeroL];
    int32_t *tab = reinterpret_cast<int32_t *>(planned_lds);
    const int32_t *dense = tab + table_words(num_coef);
    float *M = planned_lds + table_words(num_coef) + NB * 256 + wave * (kStrip + kPlanMaxY + S * kWave);
    float *dyl = M + kStrip;
    float *sbuf = dyl + kPlanMaxY;
    for (int t = lane; t < kStrip + kPlanMaxY; t += kWave) M[t] = 0.f;
    stage_table(plan, L, num_cells, num_coef, tab, NB * 256);
    const int pairs = (num_cells + 1) & ~1;
    const int64_t item = (int64_t)blockIdx.x * blockDim.y + wave;
    // receiver rows: a wave per (row, 64 channels), dx by float atomics, dy shared between the
    // waves of an edge; sender rows: a wave per row walks the channel chunks and owns dx and dy
    const int64_t items = group_is_receiver ? (int64_t)num_nodes * nchunks : (int64_t)num_nodes;
    if (item >= items) return;
    const int qrow = (int)(group_is_receiver ? item / nchunks : item);
    const int g = row_order ? row_order[qrow] : qrow;
    const int chunk0 = group_is_receiver ? (int)(item % nchunks) : 0;
    const int chunk1 = group_is_receiver ? chunk0 + 1 : nchunks;
    const int e0 = row_ptr[g], e1 = row_ptr[g + 1];

    for (int chunk = chunk0; chunk < chunk1; chunk++) {
        const int c = chunk * kWave + lane;
        const bool active = c < channels;
        const int cr = active ? c : channels - 1;
        const unsigned xoff = (unsigned)cr * (unsigned)lx.chan, soff = (unsigned)cr * (unsigned)ls.chan;
        const unsigned zoff = (unsigned)cr * (unsigned)lo.chan;
        const int dy_mode = group_is_receiver ? (nchunks > 1 ? kDyAtomic : kDyStore)
                                              : (chunk == 0 ? kDyStore : kDyAdd);
        float dxa[XG * 4];
#pragma unroll
        for (int j = 0; j < XG * 4; j++) dxa[j] = 0.f;
        int e = next_live(other, e0, e1, num_nodes);
        float yn = 0.f, xn[XG * 4], sn[kAhead];
        int64_t een = 0;
        int on = 0;
        auto issue = [&](int at) {
            on = other[at];
            een = perm ? (int64_t)perm[at] : (int64_t)at;
            yn = lane < num_y ? y[een * num_y + lane] : 0.f;
            const float *xbase = x + (int64_t)(group_is_receiver ? on : g) * lx.row;
#pragma unroll
            for (int j = 0; j < XG * 4; j++) xn[j] = load_row(xbase, xoff, (unsigned)lx.dim, j < X ? j : X - 1);  // (clamped, not skipped: straight-line loads)
            const float *sbase = s + een * ls.row;
#pragma unroll
            for (int t = 0; t < kAhead; t++) sn[t] = load_row(sbase, soff, (unsigned)ls.dim, t < S ? t : S - 1);
        };
        if (e < e1) issue(e);
        while (e < e1) {
            const float ycur = yn;
            const int64_t ee = een;
            const int o = on;
            const int xnode = group_is_receiver ? o : g;
            const int znode = group_is_receiver ? g : o;
            float xv[XG * 4];
#pragma unroll
            for (int j = 0; j < XG * 4; j++) xv[j] = (j < X && active) ? xn[j] : 0.f;  // (idle lanes add nothing to dy)
            wave_lds_sync();
#pragma unroll
            for (int t = 0; t < kAhead; t++) sbuf[(t < S ? t : S - 1) * kWave + lane] = sn[t];
            for (int t = kAhead; t < S; t++)
                sbuf[t * kWave + lane] = load_row(s + ee * ls.row, soff, (unsigned)ls.dim, t);
            const int en = next_live(other, e + 1, e1, num_nodes);
            if (en < e1) issue(en);
            build_edge_matrix<XG>(tab, num_cells, max_run, ycur, M, lane);
            wave_lds_sync();
            const float *zbase = dm + (int64_t)znode * lo.row;
            float *dsbase = ds + ee * ls.row;
            const unsigned dsoff = (unsigned)c * (unsigned)ls.chan;
            unsigned cur_l = 255u;
            float dsa = 0.f;
#pragma unroll
            for (int b = 0; b < NB; b++) {
                if (((chunk_mask >> (b * XG)) & ((1u << XG) - 1u)) == 0) continue;
                float sd[16], dz[16], T[16];
#pragma unroll
                for (int u = 0; u < 16; u++) {
                    const unsigned l = (unsigned)plan[L.slot_l + b * 16 + u] & 255u;  // (255: none)
                    const unsigned row = (unsigned)plan[L.slot_row + b * 16 + u] & 255u;
                    const float sv = sbuf[(l == 255u ? 0u : l) * kWave + lane];
                    dz[u] = load_row(zbase, zoff, (unsigned)lo.dim, row == 255u ? 0 : (int)row);
                    if (l == 255u || !active) dz[u] = 0.f;  // (wave-uniform or per lane: a select)
                    sd[u] = l == 255u ? 0.f : sv * dz[u];
                    T[u] = 0.f;
                }
#pragma unroll
                for (int gx = 0; gx < XG; gx++) {
                    if (!((chunk_mask >> (b * XG + gx)) & 1u)) continue;
                    // lane t ends with the channel sum of cell (slot 16 b + t / 4, x coordinate 4 gx + t % 4):
                    // the slots in two halves of eight, the first for lanes 0..31, the second for the rest
                    float total = 0.f;
#pragma unroll
                    for (int half = 0; half < 2; half++) {
                        float G[32];
#pragma unroll
                        for (int uu = 0; uu < 8; uu++) {
                            const int u = half * 8 + uu;
                            const f32x4 m = *reinterpret_cast<const f32x4 *>(&M[((b * 16 + u) * XG + gx) * 4]);
                            T[u] = __builtin_fmaf(m.x, xv[4 * gx], T[u]);
                            T[u] = __builtin_fmaf(m.y, xv[4 * gx + 1], T[u]);
                            T[u] = __builtin_fmaf(m.z, xv[4 * gx + 2], T[u]);
                            T[u] = __builtin_fmaf(m.w, xv[4 * gx + 3], T[u]);
                            dxa[4 * gx] = __builtin_fmaf(m.x, sd[u], dxa[4 * gx]);
                            dxa[4 * gx + 1] = __builtin_fmaf(m.y, sd[u], dxa[4 * gx + 1]);
                            dxa[4 * gx + 2] = __builtin_fmaf(m.z, sd[u], dxa[4 * gx + 2]);
                            dxa[4 * gx + 3] = __builtin_fmaf(m.w, sd[u], dxa[4 * gx + 3]);
#pragma unroll
                            for (int jj = 0; jj < 4; jj++) G[uu * 4 + jj] = sd[u] * xv[4 * gx + jj];
                        }
                        const float both = transpose_sum(G, lane);
                        if ((lane >> 5) == half) total = both;
                    }
                    const int where = dense[(b * 16 + lane / 4) * kPlanX + 4 * gx + lane % 4];
                    const int first = where & 2047, cnt = where >> 11;
                    for (int rr = 0; rr < cnt; rr++)
                        atomicAdd(&dyl[tab[pairs + 2 * (first + rr) + 1]],
                                  __int_as_float(tab[pairs + 2 * (first + rr)]) * total);
                }
                // ds: the slots of one scalar are adjacent; a scalar's sum is stored when the next begins
#pragma unroll
                for (int u = 0; u < 16; u++) {
                    const unsigned l = (unsigned)plan[L.slot_l + b * 16 + u] & 255u;
                    if (l != cur_l) {
                        if (cur_l != 255u && active) (dsbase + (int64_t)cur_l * ls.dim)[dsoff] = dsa;
                        cur_l = l;
                        dsa = 0.f;
                    }
                    dsa = __builtin_fmaf(dz[u], T[u], dsa);
                }
            }
            if (cur_l != 255u && active) (dsbase + (int64_t)cur_l * ls.dim)[dsoff] = dsa;
            if (active)
                for (int z = 0; z < num_zero_l; z++) (dsbase + (int64_t)plan[L.zero_l + z] * ls.dim)[dsoff] = 0.f;
            wave_lds_sync();
            if (lane < num_y) {
                const float v = dyl[lane];
                dyl[lane] = 0.f;
                float *at = dy + ee * num_y + lane;
                if (dy_mode == kDyStore) *at = v;
                else if (dy_mode == kDyAdd) *at += v;
                else unsafeAtomicAdd(at, v);
            }
            if (group_is_receiver) {
                if (active) {
                    float *dxbase = dx + (int64_t)xnode * lx.row;
#pragma unroll
                    for (int j = 0; j < XG * 4; j++)
                        if (j < X) unsafeAtomicAdd(dxbase + (int64_t)j * lx.dim + xoff, dxa[j]);
                }
#pragma unroll
                for (int j = 0; j < XG * 4; j++) dxa[j] = 0.f;
            }
            e = en;
        }
        if (!group_is_receiver && active) {
            float *dxbase = dx + (int64_t)g * lx.row;
#pragma unroll
            for (int j = 0; j < XG * 4; j++)
                if (j < X) (dxbase + (int64_t)j * lx.dim)[xoff] = dxa[j];
        }
    }
}

typedef void (*FwdKernel)(const int32_t *, PlanLayout, const float *, RowLayout, const float *, int, const float *,
                          RowLayout, const int32_t *, const int32_t *, const int32_t *, const int32_t *, float *,
                          RowLayout, int, int, int, int, int, int);
typedef void (*BwdKernel)(const int32_t *, PlanLayout, const float *, RowLayout, const float *, int, const float *,
                          RowLayout, const float *, RowLayout, const int32_t *, const int32_t *, const int32_t *,
                          const int32_t *, float *, float *, float *, int, int, int, int, int, int, int);

#ifdef E3J_PLANNED_ONE_SHAPE  // (a compile-time experiment: only the 7 x 4 shape)
#define E3J_ROW(K, NB) {K<7, 4>, K<7, 4>, K<7, 4>, K<7, 4>}
#else
#define E3J_ROW(K, NB) {K<NB, 1>, K<NB, 2>, K<NB, 3>, K<NB, 4>}
#endif
#define E3J_TABLE(K) {E3J_ROW(K, 1), E3J_ROW(K, 2), E3J_ROW(K, 3), E3J_ROW(K, 4), \
                      E3J_ROW(K, 5), E3J_ROW(K, 6), E3J_ROW(K, 7), E3J_ROW(K, 8)}
const FwdKernel kFwd[8][4] = E3J_TABLE(planned_fwd_kernel);
const BwdKernel kBwd[8][4] = E3J_TABLE(planned_bwd_kernel);
#undef E3J_TABLE
#undef E3J_ROW

constexpr int kWavesPerBlock = 4;

}  // namespace

bool plan_takes(const e3j_amd_conv_params &p) {
    return p.val_dtype == E3J_AMD_F32 && p.num_out >= 1 && p.num_out <= kSlots && p.num_x >= 1 &&
           p.num_x <= kPlanX && p.num_y >= 1 && p.num_y <= kPlanMaxY && p.num_scalars >= 1 &&
           p.num_scalars <= kPlanMaxS && p.num_coef >= 1 && p.num_coef <= kPlanMaxCoef && p.channels >= 1;
}

size_t plan_bytes(const e3j_amd_conv_params &p) {
    return sizeof(int32_t) * (size_t)PlanLayout(p.num_coef, p.num_scalars).words;
}

int launch_plan_build(const e3j_amd_conv_params &p, const void *coef, bool cols_ji, int32_t *plan,
                      hipStream_t stream) {
    const PlanLayout L(p.num_coef, p.num_scalars);
    const int xg = (p.num_x + 3) / 4;
    if (p.coef_idx_bytes == 1)
        hipLaunchKernelGGL(plan_build_kernel<uint8_t>, dim3(1), dim3(kBuildThreads), 0, stream,
                           static_cast<const Coef4D<uint8_t, float> *>(coef), p.num_coef, p.num_x, p.num_y,
                           p.num_out, p.num_scalars, xg, cols_ji ? 1 : 0, plan, L);
    else
        hipLaunchKernelGGL(plan_build_kernel<int32_t>, dim3(1), dim3(kBuildThreads), 0, stream,
                           static_cast<const Coef4D<int32_t, float> *>(coef), p.num_coef, p.num_x, p.num_y,
                           p.num_out, p.num_scalars, xg, cols_ji ? 1 : 0, plan, L);
    return check_hip(hipGetLastError(), "convolution plan launch");
}

int launch_planned_fwd(const e3j_amd_conv_params &p, const int32_t *plan, const void *x, const void *y,
                       const void *s, const int32_t *other, const int32_t *row_ptr, const int32_t *perm,
                       void *out, hipStream_t stream) {
    const int nb = (p.num_out + 15) / 16, xg = (p.num_x + 3) / 4;
    const int nchunks = (p.channels + kWave - 1) / kWave;
    const int64_t items = (int64_t)p.num_nodes * nchunks;
    const int64_t blocks = (items + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: grid too large");
    const size_t lds = sizeof(float) * ((size_t)table_words(p.num_coef) +
                                        (size_t)kWavesPerBlock * (nb * 16 * xg * 4 + p.num_scalars * kWave));
    if (lds > 64 * 1024) {
        const int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kFwd[nb - 1][xg - 1]),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                                 "hipFuncSetAttribute(planned fwd)");
        if (rc) return rc;
    }
    hipLaunchKernelGGL(kFwd[nb - 1][xg - 1], dim3((unsigned)blocks), dim3(kWave, kWavesPerBlock), lds, stream, plan,
                       PlanLayout(p.num_coef, p.num_scalars), static_cast<const float *>(x),
                       make_layout(p.layout, p.num_x, p.channels), static_cast<const float *>(y), p.num_y,
                       static_cast<const float *>(s), make_layout(p.layout, p.num_scalars, p.channels), other,
                       row_ptr, perm, p.row_order, static_cast<float *>(out),
                       make_layout(p.layout, p.num_out, p.channels), p.num_nodes, p.channels, p.num_x,
                       p.num_scalars, p.num_coef, nchunks);
    return check_hip(hipGetLastError(), "convolution forward launch (planned)");
}

int launch_planned_bwd(const e3j_amd_conv_params &p, bool group_is_receiver, const int32_t *plan, const void *x,
                       const void *y, const void *s, const void *dm, const int32_t *other,
                       const int32_t *row_ptr, const int32_t *perm, void *dx, void *dy, void *ds,
                       hipStream_t stream) {
    const int nb = (p.num_out + 15) / 16, xg = (p.num_x + 3) / 4;
    const int nchunks = (p.channels + kWave - 1) / kWave;
    const int64_t items = group_is_receiver ? (int64_t)p.num_nodes * nchunks : (int64_t)p.num_nodes;
    const int64_t blocks = (items + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution_bwd: grid too large");
    const size_t lds = sizeof(float) * ((size_t)table_words(p.num_coef) + (size_t)nb * 256 +
                                        (size_t)kWavesPerBlock * (nb * 16 * xg * 4 + kPlanMaxY + p.num_scalars * kWave));
    if (lds > 64 * 1024) {
        const int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kBwd[nb - 1][xg - 1]),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                                 "hipFuncSetAttribute(planned bwd)");
        if (rc) return rc;
    }
    hipLaunchKernelGGL(kBwd[nb - 1][xg - 1], dim3((unsigned)blocks), dim3(kWave, kWavesPerBlock), lds, stream, plan,
                       PlanLayout(p.num_coef, p.num_scalars), static_cast<const float *>(x),
                       make_layout(p.layout, p.num_x, p.channels), static_cast<const float *>(y), p.num_y,
                       static_cast<const float *>(s), make_layout(p.layout, p.num_scalars, p.channels),
                       static_cast<const float *>(dm), make_layout(p.layout, p.num_out, p.channels), other,
                       row_ptr, perm, p.row_order, static_cast<float *>(dx), static_cast<float *>(dy),
                       static_cast<float *>(ds), p.num_nodes, p.channels, p.num_x, p.num_scalars, p.num_coef, nchunks,
                       group_is_receiver ? 1 : 0);
    return check_hip(hipGetLastError(), "convolution backward launch (planned)");
}

}  // namespace e3j_amd

extern "C" int e3j_amd_table_plan_status(const e3j_amd_conv_params *p, const void *coef, int32_t coef_cols_ji,
                                         int32_t *status, void *stream_) {
    using namespace e3j_amd;
    if (p == nullptr || status == nullptr || (coef == nullptr && p->num_coef > 0))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "table_plan_status: null operand");
    status[0] = status[1] = status[2] = status[3] = 0;
    if (!plan_takes(*p)) return E3J_AMD_OK;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    void *mem = nullptr;
    int rc = check_hip(hipMalloc(&mem, plan_bytes(*p)), "table_plan_status: hipMalloc");
    if (rc) return rc;
    rc = launch_plan_build(*p, coef, coef_cols_ji != 0, static_cast<int32_t *>(mem), stream);
    int32_t header[kHeaderWords] = {0};
    if (!rc) rc = check_hip(hipMemcpyAsync(header, mem, sizeof(header), hipMemcpyDeviceToHost, stream),
                            "table_plan_status: copy");
    if (!rc) rc = check_hip(hipStreamSynchronize(stream), "table_plan_status: synchronize");
    (void)hipFree(mem);
    if (rc) return rc;
    status[0] = header[kEligible];
    status[1] = header[kNumCells];
    status[2] = __builtin_popcount((unsigned)header[kChunkMask]);
    status[3] = header[kNumZeroL];
    return E3J_AMD_OK;
}
