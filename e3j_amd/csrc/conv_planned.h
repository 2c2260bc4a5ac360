// Table-driven convolution kernels over a plan of the table (float32; any table whose output
// coordinates each use one scalar, up to 128 output coordinates, 16 x coordinates, 64 y
// components, 64 scalars, 2048 entries).
//
// The contraction out[i] += c * x[j] * y[k] * s[l] (lib/e3j_ops/cuda/convolution/fwd.cuh:88-153)
// is regrouped per edge as out[i] += s[l(i)] * sum_j M[i][j] * x[j] with the channel-independent
// matrix M[i][j] = sum_k c_ijk * y[k].  A wave builds M once per edge in its strip of LDS (the
// lanes share the table's non-empty cells), and then every lane (one channel) runs loops over
// i and j whose bounds are compile-time numbers, so that x, the accumulators and the partial
// sums sit in registers under constant indices; M is read four numbers to a 4-byte LDS read
// (lane t takes number t % 4) and used through DPP operands.  What depends on the table is data:
// the plan, built on the device by one workgroup per call (no read-back, no compiler at run
// time):
//   * the output coordinates in the order the loops visit them ("slots": sorted by the x
//     coordinates their path touches, then by scalar, so that rows of one scalar are adjacent
//     and blocks of 16 slots touch few groups of 4 x coordinates),
//   * a bit per (block of 16 slots, group of 4 x coordinates) that has a coefficient at all, and
//     inside those a bit per half of 8 slots: the loops skip the others with wave-uniform branches,
//   * the non-empty cells (slot, j) with their (coefficient, k) lists in table order.
// The backward pass (lib/e3j_ops/cuda/convolution/bwd.cuh:116-321) uses the same M: ds from the
// forward's partial sums, dx[j] += M[i][j] * s[l(i)] * dm[i], and for dy the channel sums of the
// products x[j] * (s * dm[i]) of a block of 16 slots, 16 x 16 cells, come from 16 matrix
// instructions whose summed index is the channel (operands moved through a tile of LDS); a lane per
// entry of the block then multiplies its cell's total with the coefficient and adds it into the
// wave's dy row in LDS.  Per edge a wave issues the loads of the edge's operands (the x row, the
// scalar rows, the first block of dm) together, builds M under them, and copies the scalar rows
// into its LDS strip (the loops read them by the slot's scalar, a number of the plan); the next
// edge's index, position and y are fetched one edge ahead.  The table part of the plan sits in the
// workgroup's LDS, the per-slot numbers in two vector registers of every wave that are read lane by
// lane.
//
// Tables the plan cannot take (an output coordinate with two different scalars, sizes beyond the
// limits) run the kernels of conv_generic.hip: eligibility is a flag in the plan that both
// kernels read, so the host never waits for the device.

#ifndef E3J_AMD_CSRC_CONV_PLANNED_H_
#define E3J_AMD_CSRC_CONV_PLANNED_H_

#include <type_traits>

#include "common.h"


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
enum { kEligible = 0, kNumCells = 1, kChunkMask = 2, kNumZeroL = 3, kMaxRun = 4, kHalfMask0 = 5, kHalfMask1 = 6,
       kHeaderWords = 8 };

// bit of (block b of 16 slots, group g of 4 x coordinates, half of 8 slots) in the 64-bit mask of halves
// that hold a coefficient (two header words)
template <int XG>
__device__ __forceinline__ bool half_live(unsigned mask0, unsigned mask1, int b, int g, int half) {
    const int bit = (b * XG + g) * 2 + half;
    return (((bit < 32 ? mask0 >> bit : mask1 >> (bit - 32))) & 1u) != 0;
}

struct PlanLayout {  // offsets in 32-bit words
    // slot_row, slot_l: output coordinate and scalar of a slot; first, count: the entries of a dense
    // cell (slot * 16 + j); cells: the non-empty cells packed as cell | first << 11 | count << 22;
    // pairs: (coefficient bits, k | cell within its block of 16 slots << 8) of the entries, cell by cell; coef, k, t, cell_list: working arrays
    // of the builder; zero_l: scalars no entry uses
    // slot_lw: 64 * scalar of the slot (the word offset of its row in a wave's LDS copy of s), 0 if none
    // block_first: the first entry of each block of 16 slots in `pairs` (the entries of a block are
    // adjacent: cells are numbered slot by slot), and the number of entries behind the last block
    int slot_row, slot_l, slot_lw, first, count, cell_list, cells, pairs, coef, k, t, zero_l, block_first, words;
    PlanLayout(int num_coef, int num_scalars) {
        int at = kHeaderWords;
        auto take = [&](int n) { const int here = at; at += (n + 3) / 4 * 4; return here; };
        slot_row = take(kSlots); slot_l = take(kSlots); slot_lw = take(kSlots);
        first = take(kCells); count = take(kCells); cell_list = take(kCells); cells = take(kCells);
        pairs = take(2 * num_coef);
        coef = take(num_coef); k = take(num_coef); t = take(num_coef);
        zero_l = take(num_scalars);
        block_first = take(kSlots / 16 + 1);
        words = at;
    }
};

// words of LDS the staged table takes (cells, then pairs from an even word on)
__host__ __device__ inline int table_words(int num_coef) {
    const int cells = num_coef < kCells ? num_coef : kCells;
    return ((cells + 1) / 2 * 2 + 2 * num_coef + 3) / 4 * 4;
}


template <typename Idx, typename Val>
__device__ inline void decode(const Coef4D<Idx, Val> &c, int cols_ji, int &i, int &j, int &k, int &l) {
    i = (int)c.i; j = (int)c.j; k = (int)c.k; l = (int)c.l;
    if (cols_ji) { const int t = i; i = j; j = t; }
}

// One workgroup turns the table into the plan.
template <typename Idx, typename Val>
__global__ __launch_bounds__(kBuildThreads) void plan_build_kernel(
    const Coef4D<Idx, Val> *__restrict__ coef, int num_coef, int X, int Y, int Z, int S, int xg, int cols_ji,
    int32_t *__restrict__ plan, PlanLayout L) {
    __shared__ int lmin[kSlots], lmax[kSlots], support[kSlots], slot_of_row[kSlots];
    __shared__ int path_support[kPlanMaxS], referenced[kPlanMaxS];
    __shared__ int eligible, chunk_mask, half_mask[2], num_cells, num_zero_l, max_run;
    __shared__ int scan[kBuildThreads];
    const int tid = threadIdx.x;
    if (tid == 0) { eligible = 1; chunk_mask = 0; half_mask[0] = half_mask[1] = 0; num_cells = 0; num_zero_l = 0; max_run = 0; }
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
                const int chunk = (cell / kPlanX / 16) * xg + (cell % kPlanX) / 4;
                const int half = 2 * chunk + (cell / kPlanX) % 16 / 8;
                atomicOr(&chunk_mask, 1 << chunk);
                atomicOr(&half_mask[half >> 5], 1 << (half & 31));
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
        plan[L.coef + at] = __float_as_int((float)coef[n].val);
        plan[L.k + at] = k | ((cell % (16 * kPlanX)) << 8);
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
    for (int q = tid; q < kSlots; q += kBuildThreads) {
        const int l = plan[L.slot_l + q];
        plan[L.slot_lw + q] = l < 0 ? 0 : l * kWave;
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
    if (tid <= kSlots / 16) plan[L.block_first + tid] = tid < kSlots / 16 ? plan[L.first + tid * 16 * kPlanX] : num_coef;
    if (tid == 0) {
        plan[kEligible] = eligible; plan[kNumCells] = num_cells; plan[kChunkMask] = chunk_mask;
        plan[kNumZeroL] = num_zero_l; plan[kMaxRun] = max_run;
        plan[kHalfMask0] = half_mask[0]; plan[kHalfMask1] = half_mask[1];
    }
}

// LDS traffic between the lanes of one wave: its LDS operations complete in program order, so
// only the compiler has to be kept from moving accesses across this point.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// acc += (m of lane K of the lane's group of four lanes) * v, one instruction (a DPP operand).  The
// loops read four wave-uniform numbers of M with one 4-byte LDS read (lane t takes number t % 4)
// instead of a 16-byte broadcast to every lane: a quarter of the LDS return traffic.  (m comes
// from an LDS read, never from a vector instruction just before, so no wait states are owed; the
// compiler's hazard pass does not look inside inline assembly, and e3j_amd/build.py reads the
// assembly listing of this file for a DPP operand written less than two wait states earlier.)
// Keeps the eight reads before it together (the values are all in registers here): without it the
// compiler moves each read next to its use and pays an LDS round trip per pair of values.
__device__ __forceinline__ void together(float (&m)[8]) {
    asm volatile("" : "+v"(m[0]), "+v"(m[1]), "+v"(m[2]), "+v"(m[3]), "+v"(m[4]), "+v"(m[5]), "+v"(m[6]), "+v"(m[7]));
}
// The reads before it are issued before the instructions behind it (the compiler would otherwise
// move a read down to its use, and the read ahead of the next eight numbers of M with it).
__device__ __forceinline__ void issued() { asm volatile("" ::: "memory"); }
// The eight slots' numbers of M of (block b, group g of x coordinates, half): lane t takes number t % 4.
template <int XG>
__device__ __forceinline__ void read_half(const float *M, int b, int g, int half, int lane, float (&m)[8]) {
#pragma unroll
    for (int uu = 0; uu < 8; uu++) m[uu] = M[((b * 16 + half * 8 + uu) * XG + g) * 4 + (lane & 3)];
}
template <int K>
__device__ __forceinline__ void fma_quad(float &acc, float m, float v) {
    asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[%3,%3,%3,%3] row_mask:0xf bank_mask:0xf"
        : "+v"(acc) : "v"(m), "v"(v), "n"(K));
}

// The table part of the plan in LDS, shared by the waves of a workgroup: the packed cells, then
// (coefficient, k) pairs.  Every thread of the workgroup calls this (it holds a barrier).
__device__ __forceinline__ void stage_table(const int32_t *__restrict__ plan, const PlanLayout &L, int num_cells,
                                            int num_coef, int32_t *tab) {
    const int tid = threadIdx.y * kWave + threadIdx.x, threads = blockDim.y * kWave;
    const int pairs = (num_cells + 1) & ~1;  // the pairs start at an even word
    for (int t = tid; t < num_cells; t += threads) tab[t] = plan[L.cells + t];
    for (int t = tid; t < 2 * num_coef; t += threads) tab[pairs + t] = plan[L.pairs + t];
    __syncthreads();
}

// M of one edge: lane q takes the cells q, q + 64, ... of the staged list; lane k of `yreg` holds y[k].
// `most`: the longest entry list of a cell (lanes with shorter lists add zeros).
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
            const int kk = tab[pairs + 2 * at + 1] & 255;
            const float cf = r < cnt ? __int_as_float(tab[pairs + 2 * at]) : 0.f;
            sum += cf * __shfl(yreg, kk, kWave);
        }
        if (cnt > 0) {
            const int slot = cell / kPlanX, j = cell % kPlanX;
            M[(slot * XG + (j >> 2)) * 4 + (j & 3)] = sum;
        }
    }
}

// The same with the lane's first kHeld cells of the list held in registers for all edges (their
// list words do not change from edge to edge) and their entry chains interleaved: the LDS round
// trips of the chains overlap instead of following each other.
constexpr int kHeld = 6;  // 384 cells
struct HeldCells {
    unsigned w[kHeld];
    __device__ __forceinline__ HeldCells(const int32_t *tab, int num_cells, int lane) {
#pragma unroll
        for (int it = 0; it < kHeld; it++) w[it] = it * kWave + lane < num_cells ? (unsigned)tab[it * kWave + lane] : 0u;
    }
};
template <int XG>
__device__ __forceinline__ void build_edge_matrix(const int32_t *tab, const HeldCells &held, int num_cells, int most,
                                                  float yreg, float *M, int lane) {
    const int pairs = (num_cells + 1) & ~1;
    float sum[kHeld];
#pragma unroll
    for (int it = 0; it < kHeld; it++) sum[it] = 0.f;
    for (int r = 0; r < most; r++) {
#pragma unroll
        for (int it = 0; it < kHeld; it++) {
            if (it * kWave >= num_cells) break;  // (wave-uniform)
            const int first = (int)((held.w[it] >> 11) & 2047u), cnt = (int)(held.w[it] >> 22);
            const int at = r < cnt ? first + r : first;
            const int kk = tab[pairs + 2 * at + 1] & 255;
            const float cf = r < cnt ? __int_as_float(tab[pairs + 2 * at]) : 0.f;
            sum[it] += cf * __shfl(yreg, kk, kWave);
        }
    }
#pragma unroll
    for (int it = 0; it < kHeld; it++) {
        if (it * kWave >= num_cells) break;
        if ((held.w[it] >> 22) > 0) {
            const int cell = (int)(held.w[it] & 2047u);
            const int slot = cell / kPlanX, j = cell % kPlanX;
            M[(slot * XG + (j >> 2)) * 4 + (j & 3)] = sum[it];
        }
    }
    for (int q0 = kHeld * kWave; q0 < num_cells; q0 += kWave) {  // cells past the held ones, one at a time
        const int q = q0 + lane;
        const unsigned w = (unsigned)tab[q < num_cells ? q : 0];
        const int cell = (int)(w & 2047u), first = (int)((w >> 11) & 2047u);
        const int cnt = q < num_cells ? (int)(w >> 22) : 0;
        float one = 0.f;
        for (int r = 0; r < most; r++) {
            const int at = r < cnt ? first + r : first;
            const int kk = tab[pairs + 2 * at + 1] & 255;
            const float cf = r < cnt ? __int_as_float(tab[pairs + 2 * at]) : 0.f;
            one += cf * __shfl(yreg, kk, kWave);
        }
        if (cnt > 0) {
            const int slot = cell / kPlanX, j = cell % kPlanX;
            M[(slot * XG + (j >> 2)) * 4 + (j & 3)] = one;
        }
    }
}

// Per-slot numbers of the plan, kept by a wave in two vector registers (lane t of register k
// holds the number of slot 64 k + t) and read as wave-uniform values with lane reads.
struct SlotWords {
    int lo, hi;
    __device__ __forceinline__ SlotWords(const int32_t *__restrict__ words, int lane)
        : lo(words[lane]), hi(words[kWave + lane]) {}
    __device__ __forceinline__ int operator[](int slot) const {
        return __builtin_amdgcn_readlane(slot < kWave ? lo : hi, slot % kWave);
    }
};

// A value every lane of the wave holds alike, moved to a scalar register (the compiler cannot
// know that a vector load of a wave-uniform address gives a wave-uniform value).
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }


// Rows of an operand behind a wave-uniform base: the lanes keep one 32-bit byte offset that
// moves from row to row by the row stride, so that a load takes a scalar base, one offset
// register and one vector addition.
// Values are held in memory as Val (float, or half: converted on the way in and out) and
// computed in float.
template <typename Val>
struct RowCursor {
    const char *base;   // wave-uniform
    unsigned at;        // byte offset of the lane's element in row 0
    unsigned step;      // bytes between rows
    __device__ __forceinline__ RowCursor(const Val *row0, unsigned lane_elems, unsigned stride_elems)
        : base(reinterpret_cast<const char *>(row0)), at((unsigned)sizeof(Val) * lane_elems),
          step((unsigned)sizeof(Val) * stride_elems) {}
    __device__ __forceinline__ Val raw(unsigned r) const {  // r wave-uniform; as held in memory
        return *reinterpret_cast<const Val *>((base + (size_t)r * step) + at);
    }
    __device__ __forceinline__ float row(unsigned r) const { return (float)raw(r); }
};
// the lane's element of row r of an output operand (same addressing)
template <typename Val>
__device__ __forceinline__ Val *element_at(Val *row0, unsigned lane_elems, unsigned stride_elems, unsigned r) {
    return reinterpret_cast<Val *>(reinterpret_cast<char *>(row0) +
                                   (unsigned)sizeof(Val) * (lane_elems + r * stride_elems));
}

// The scalar rows of one edge on their way into the wave's LDS copy: the loads of 24 rows are issued
// together with the edge's other loads, and the values are written to LDS once the edge's matrix is
// built (the matrix needs LDS only, so it is built while the loads are in flight).  Rows past 24
// follow in groups of eight.
constexpr int kRowsAhead = 24;
template <typename Val>
struct ScalarRows {
    Val v[kRowsAhead];  // (as loaded: a conversion here would wait for the load)
    __device__ __forceinline__ void load(const RowCursor<Val> &cur, int S) {
#pragma unroll
        for (int t = 0; t < 8; t++) v[t] = cur.raw((unsigned)(t < S ? t : S - 1));  // (clamped: straight-line)
        if (S > 8) {
#pragma unroll
            for (int t = 8; t < 16; t++) v[t] = cur.raw((unsigned)(t < S ? t : S - 1));
        }
        if (S > 16) {
#pragma unroll
            for (int t = 16; t < kRowsAhead; t++) v[t] = cur.raw((unsigned)(t < S ? t : S - 1));
        }
    }
    __device__ __forceinline__ void store(const RowCursor<Val> &cur, int S, float *sbuf, int lane) const {
#pragma unroll
        for (int t = 0; t < 8; t++) sbuf[(t < S ? t : S - 1) * kWave + lane] = (float)v[t];
        if (S > 8) {
#pragma unroll
            for (int t = 8; t < 16; t++) sbuf[(t < S ? t : S - 1) * kWave + lane] = (float)v[t];
        }
        if (S > 16) {
#pragma unroll
            for (int t = 16; t < kRowsAhead; t++) sbuf[(t < S ? t : S - 1) * kWave + lane] = (float)v[t];
        }
        for (int t0 = kRowsAhead; t0 < S; t0 += 8) {
            float w[8];
#pragma unroll
            for (int t = 0; t < 8; t++) w[t] = cur.row((unsigned)(t0 + t < S ? t0 + t : S - 1));
#pragma unroll
            for (int t = 0; t < 8; t++) sbuf[(t0 + t < S ? t0 + t : S - 1) * kWave + lane] = w[t];
        }
    }
};

// The edge a wave works on, fetched one edge ahead of its use: the other end, the position of the
// edge's operands and the wave's copy of y (lane k holds y[k]).
template <typename Val>
struct EdgeAhead {
    int other;
    int64_t at;
    Val y_held;  // (as loaded: a conversion here would wait for the load)
    __device__ __forceinline__ float y(int num_y, int lane) const { return lane < num_y ? (float)y_held : 0.f; }
    __device__ __forceinline__ static EdgeAhead fetch(const int32_t *__restrict__ other, const int32_t *__restrict__ perm,
                                                      const Val *__restrict__ y, int num_y, int e, int lane) {
        EdgeAhead a;
        a.other = uni(other[e]);
        a.at = perm ? (int64_t)uni(perm[e]) : (int64_t)e;
        a.y_held = y[a.at * num_y + (lane < num_y ? lane : 0)];
        return a;
    }
};

// Forward: a wave takes (row, 64 channels) and holds NB * 16 accumulators: up to three blocks of
// them leave room for three waves per SIMD (cfg2's table, 43 output coordinates: 0.35 ms with
// three, 0.43 ms with two), more for two.
template <typename Val, int NB, int XG>
__global__ __launch_bounds__(256, NB <= 3 ? 3 : 2) void planned_fwd_kernel(
    const int32_t *__restrict__ plan, PlanLayout L, const Val *__restrict__ x, RowLayout lx,
    const Val *__restrict__ y, int num_y, const Val *__restrict__ s, RowLayout ls,
    const int32_t *__restrict__ other, const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ row_order, Val *__restrict__ out, RowLayout lo, int num_nodes, int channels,
    int X, int S, int num_coef, int nchunks) {
    extern __shared__ __align__(16) float planned_lds[];
    if (plan[kEligible] == 0) return;  // (the whole grid) the table-driven kernel without a plan runs instead
    constexpr int kStrip = NB * 16 * XG * 4;
    const int lane = threadIdx.x, wave = __builtin_amdgcn_readfirstlane((int)threadIdx.y);
    const int num_cells = plan[kNumCells];
    const int max_run = plan[kMaxRun];
    int32_t *tab = reinterpret_cast<int32_t *>(planned_lds);
    float *M = planned_lds + table_words(num_coef) + wave * (kStrip + S * kWave);
    float *sbuf = M + kStrip;
    for (int t = lane; t < kStrip; t += kWave) M[t] = 0.f;
    stage_table(plan, L, num_cells, num_coef, tab);
    const int64_t item = (int64_t)blockIdx.x * blockDim.y + wave;
    if (item >= (int64_t)num_nodes * nchunks) return;  // uniform per wave; no workgroup barrier below
    const int q = (int)(item / nchunks);
    const int r = row_order ? uni(row_order[q]) : q;
    const int c = (int)(item % nchunks) * kWave + lane;
    const bool active = c < channels;
    const int cr = active ? c : channels - 1;  // channel whose rows an idle lane reads
    const unsigned xoff = (unsigned)cr * (unsigned)lx.chan, soff = (unsigned)cr * (unsigned)ls.chan;
    const unsigned chunk_mask = (unsigned)plan[kChunkMask];
    const unsigned half0 = (unsigned)plan[kHalfMask0], half1 = (unsigned)plan[kHalfMask1];
    const SlotWords slot_lw(plan + L.slot_lw, lane);
    const HeldCells held(tab, num_cells, lane);
    float acc[NB * 16];
#pragma unroll
    for (int t = 0; t < NB * 16; t++) acc[t] = 0.f;

    const int e0 = uni(row_ptr[r]), e1 = uni(row_ptr[r + 1]);
    EdgeAhead<Val> next = {0, 0, Val(0)};
    if (e0 < e1) next = EdgeAhead<Val>::fetch(other, perm, y, num_y, e0, lane);
    for (int e = e0; e < e1; e++) {
        const EdgeAhead<Val> edge = next;
        // this edge's loads, its matrix built under them (LDS only), then the next edge's numbers
        const bool live = (unsigned)edge.other < (unsigned)num_nodes;  // (wave-uniform) padding edges are stepped over
        const RowCursor<Val> sc(s + edge.at * ls.row, soff, (unsigned)ls.dim);
        ScalarRows<Val> rows;
        Val x_held[XG * 4];  // (as loaded; converted once the matrix is built)
        if (live) {
            const RowCursor<Val> xc(x + (int64_t)edge.other * lx.row, xoff, (unsigned)lx.dim);
#pragma unroll
            for (int j = 0; j < XG * 4; j++) x_held[j] = xc.raw((unsigned)(j < X ? j : X - 1));
            rows.load(sc, S);
            wave_lds_sync();  // the reads of the edge before are behind the writes below
            build_edge_matrix<XG>(tab, held, num_cells, max_run, edge.y(num_y, lane), M, lane);
        }
        next = EdgeAhead<Val>::fetch(other, perm, y, num_y, e + 1 < e1 ? e + 1 : e, lane);
        if (!live) continue;
        float xv[XG * 4];
#pragma unroll
        for (int j = 0; j < XG * 4; j++) xv[j] = j < X ? (float)x_held[j] : 0.f;
        rows.store(sc, S, sbuf, lane);
        wave_lds_sync();
#pragma unroll
        for (int b = 0; b < NB; b++) {
            if (((chunk_mask >> (b * XG)) & ((1u << XG) - 1u)) == 0) continue;  // no coefficient in the block
            float sv[16], T[16];
#pragma unroll
            for (int u = 0; u < 16; u++) {
                sv[u] = sbuf[slot_lw[b * 16 + u] + lane];
                T[u] = 0.f;
            }
#pragma unroll
            for (int g = 0; g < XG; g++) {
                if (!((chunk_mask >> (b * XG + g)) & 1u)) continue;
#pragma unroll
                for (int half = 0; half < 2; half++) {
                    if (!half_live<XG>(half0, half1, b, g, half)) continue;  // eight slots without a coefficient here
                    float m[8];  // (read together, used together: one LDS round trip per half)
                    read_half<XG>(M, b, g, half, lane, m);
                    together(m);
#pragma unroll
                    for (int uu = 0; uu < 8; uu++) {
                        const int u = half * 8 + uu;
                        fma_quad<0>(T[u], m[uu], xv[4 * g]);
                        fma_quad<1>(T[u], m[uu], xv[4 * g + 1]);
                        fma_quad<2>(T[u], m[uu], xv[4 * g + 2]);
                        fma_quad<3>(T[u], m[uu], xv[4 * g + 3]);
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < 16; u++) acc[b * 16 + u] = __builtin_fmaf(sv[u], T[u], acc[b * 16 + u]);
        }
    }
    {
        const SlotWords slot_row(plan + L.slot_row, lane), slot_l(plan + L.slot_l, lane);
        Val *obase = out + (int64_t)r * lo.row;
        const unsigned ooff = (unsigned)c * (unsigned)lo.chan;
#pragma unroll
        for (int t = 0; t < NB * 16; t++) {
            const int row = slot_row[t];
            // (a slot whose output coordinate no entry touches has read row 0 of s: it stores zero)
            if (row >= 0 && active)
                *element_at(obase, ooff, (unsigned)lo.dim, (unsigned)row) = (Val)(slot_l[t] < 0 ? 0.f : acc[t]);
        }
    }
}

// The channel sums of the per-lane products x[j] * s * dm[i] of a block of 16 slots, all 16 x 16 of
// them with 16 matrix instructions: a wave writes its 16 values per lane (one row of 64 channels per
// slot) to a tile of LDS and reads them back with lane t holding slot t % 16 of the channels
// 16 (t / 16) .. + 15 (four 16-byte reads; rows 68 words apart), which is the first operand of
// v_mfma_f32_16x16x4_f32 with the channels as the summed index; x of the edge, moved the same way
// once per edge, is the second.  Lane t then holds, in register r, the total of the cell
// (slot 4 (t / 16) + r, x coordinate t % 16).
constexpr int kTileStride = 68;
constexpr int kTileWords = 16 * kTileStride;
typedef float f32x4 __attribute__((ext_vector_type(4)));
struct ChannelOperand {
    f32x4 q[4];
    __device__ __forceinline__ void read(const float *tile, int lane) {
#pragma unroll
        for (int n = 0; n < 4; n++)
            q[n] = *reinterpret_cast<const f32x4 *>(&tile[(lane & 15) * kTileStride + 16 * (lane >> 4) + 4 * n]);
    }
};
__device__ __forceinline__ f32x4 channel_sums(const ChannelOperand &a, const ChannelOperand &b) {
    f32x4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int n = 0; n < 4; n++) {
        d = __builtin_amdgcn_mfma_f32_16x16x4f32(a.q[n].x, b.q[n].x, d, 0, 0, 0);
        d = __builtin_amdgcn_mfma_f32_16x16x4f32(a.q[n].y, b.q[n].y, d, 0, 0, 0);
        d = __builtin_amdgcn_mfma_f32_16x16x4f32(a.q[n].z, b.q[n].z, d, 0, 0, 0);
        d = __builtin_amdgcn_mfma_f32_16x16x4f32(a.q[n].w, b.q[n].w, d, 0, 0, 0);
    }
    return d;
}

enum DyMode { kDyStore = 0, kDyAdd = 1, kDyAtomic = 2 };

template <typename Val, int NB, int XG>
__global__ __launch_bounds__(256, 2) void planned_bwd_kernel(
    const int32_t *__restrict__ plan, PlanLayout L, const Val *__restrict__ x, RowLayout lx,
    const Val *__restrict__ y, int num_y, const Val *__restrict__ s, RowLayout ls,
    const Val *__restrict__ dm, RowLayout lo, const int32_t *__restrict__ other,
    const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ row_order, Val *__restrict__ dx, Val *__restrict__ dy,
    Val *__restrict__ ds, int num_nodes, int channels, int X, int S, int num_coef, int nchunks,
    int group_is_receiver) {
    extern __shared__ __align__(16) float planned_lds[];
    if (plan[kEligible] == 0) return;
    constexpr int kStrip = NB * 16 * XG * 4;
    const int lane = threadIdx.x, wave = __builtin_amdgcn_readfirstlane((int)threadIdx.y);
    const int num_cells = plan[kNumCells];
    const unsigned chunk_mask = (unsigned)plan[kChunkMask];
    const unsigned half0 = (unsigned)plan[kHalfMask0], half1 = (unsigned)plan[kHalfMask1];
    const int max_run = plan[kMaxRun];
    const int num_zero_l = plan[kNumZeroL];
    int32_t *tab = reinterpret_cast<int32_t *>(planned_lds);
    float *M = planned_lds + table_words(num_coef) + wave * (kStrip + kPlanMaxY + S * kWave + kTileWords);
    float *dyl = M + kStrip;
    float *sbuf = dyl + kPlanMaxY;
    float *tile = sbuf + S * kWave;
    for (int t = lane; t < kStrip + kPlanMaxY; t += kWave) M[t] = 0.f;
    stage_table(plan, L, num_cells, num_coef, tab);
    const int pairs = (num_cells + 1) & ~1;
    const int64_t item = (int64_t)blockIdx.x * blockDim.y + wave;
    // receiver rows: a wave per (row, 64 channels), dx by float atomics, dy shared between the
    // waves of an edge; sender rows: a wave per row walks the channel chunks and owns dx and dy
    const int64_t items = group_is_receiver ? (int64_t)num_nodes * nchunks : (int64_t)num_nodes;
    if (item >= items) return;
    const int qrow = (int)(group_is_receiver ? item / nchunks : item);
    const int g = row_order ? uni(row_order[qrow]) : qrow;
    const int chunk0 = group_is_receiver ? (int)(item % nchunks) : 0;
    const int chunk1 = group_is_receiver ? chunk0 + 1 : nchunks;
    const int e0 = uni(row_ptr[g]), e1 = uni(row_ptr[g + 1]);
    const SlotWords slot_l(plan + L.slot_l, lane), slot_row(plan + L.slot_row, lane);

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
        EdgeAhead<Val> next = {0, 0, Val(0)};
        if (e0 < e1) next = EdgeAhead<Val>::fetch(other, perm, y, num_y, e0, lane);
        for (int e = e0; e < e1; e++) {
            const EdgeAhead<Val> edge = next;
            const bool live = (unsigned)edge.other < (unsigned)num_nodes;  // (wave-uniform) padding edges are stepped over
            const int o = edge.other;
            const int64_t ee = edge.at;
            const int xnode = group_is_receiver ? o : g;
            const int znode = group_is_receiver ? g : o;
            // this edge's loads (x, scalars, the first block of dm), its matrix built under them (LDS
            // only), then the next edge's numbers
            const RowCursor<Val> sc(s + ee * ls.row, soff, (unsigned)ls.dim);
            const RowCursor<Val> zc(dm + (int64_t)(live ? znode : 0) * lo.row, zoff, (unsigned)lo.dim);
            ScalarRows<Val> rows;
            Val x_held[XG * 4];  // (as loaded; converted once the matrix is built)
            Val dz_held[16], dz_ahead[16];  // dm of the block at hand and of the block after it, as loaded
            auto load_dm = [&](int b, Val (&to)[16]) {
#pragma unroll
                for (int u = 0; u < 16; u++) {
                    const int row = slot_row[b * 16 + u];  // (-1: none)
                    to[u] = zc.raw((unsigned)(row < 0 ? 0 : row));
                }
            };
            if (live) {
                const RowCursor<Val> xc(x + (int64_t)xnode * lx.row, xoff, (unsigned)lx.dim);
#pragma unroll
                for (int j = 0; j < XG * 4; j++) x_held[j] = xc.raw((unsigned)(j < X ? j : X - 1));
                rows.load(sc, S);
                load_dm(0, dz_held);
                wave_lds_sync();  // the reads of the edge before are behind the writes below
                build_edge_matrix<XG>(tab, num_cells, max_run, edge.y(num_y, lane), M, lane);
            }
            next = EdgeAhead<Val>::fetch(other, perm, y, num_y, e + 1 < e1 ? e + 1 : e, lane);
            if (!live) continue;
            float xv[XG * 4];
#pragma unroll
            for (int j = 0; j < XG * 4; j++) xv[j] = j < X && active ? (float)x_held[j] : 0.f;  // (idle lanes add nothing to dy)
            rows.store(sc, S, sbuf, lane);
#pragma unroll
            for (int j = 0; j < 16; j++) tile[j * kTileStride + lane] = j < XG * 4 ? xv[j < XG * 4 ? j : 0] : 0.f;
            wave_lds_sync();
            ChannelOperand xop;
            xop.read(tile, lane);
            wave_lds_sync();  // (the tile is written again below)
            Val *dsrow0 = ds + ee * ls.row;
            const unsigned dsoff = (unsigned)c * (unsigned)ls.chan;
            int cur_l = -1;
            float dsa = 0.f;
#pragma unroll
            for (int b = 0; b < NB; b++) {
                if (b + 1 < NB) load_dm(b + 1, dz_ahead);
                const int entries0 = uni(plan[L.block_first + b]), entries1 = uni(plan[L.block_first + b + 1]);
                if (((chunk_mask >> (b * XG)) & ((1u << XG) - 1u)) == 0) {
#pragma unroll
                    for (int u = 0; u < 16; u++) dz_held[u] = dz_ahead[u];
                    continue;
                }
                float sd[16], dz[16], T[16];
#pragma unroll
                for (int u = 0; u < 16; u++) {
                    const int l = slot_l[b * 16 + u];  // (-1: none)
                    const float sv = sbuf[(l < 0 ? 0 : l) * kWave + lane];
                    dz[u] = l < 0 ? 0.f : (float)dz_held[u];
                    sd[u] = sv * dz[u];
                    T[u] = 0.f;
                }
                // the next half's numbers of M are read while the products of the one at hand run (read
                // whether or not the half holds a coefficient: the count of reads in flight stays a
                // compile-time number)
                float m[2][8];
                read_half<XG>(M, b, 0, 0, lane, m[0]);
#pragma unroll
                for (int it = 0; it < 2 * XG; it++) {
                    const int gx = it / 2, half = it % 2;
                    if (it + 1 < 2 * XG) read_half<XG>(M, b, (it + 1) / 2, (it + 1) % 2, lane, m[(it + 1) & 1]);
                    issued();
                    if (!half_live<XG>(half0, half1, b, gx, half)) continue;  // eight slots without a coefficient here
                    together(m[it & 1]);
#pragma unroll
                    for (int uu = 0; uu < 8; uu++) {
                        const int u = half * 8 + uu;
                        const float mu = m[it & 1][uu];
                        fma_quad<0>(T[u], mu, xv[4 * gx]);
                        fma_quad<1>(T[u], mu, xv[4 * gx + 1]);
                        fma_quad<2>(T[u], mu, xv[4 * gx + 2]);
                        fma_quad<3>(T[u], mu, xv[4 * gx + 3]);
                        fma_quad<0>(dxa[4 * gx], mu, sd[u]);
                        fma_quad<1>(dxa[4 * gx + 1], mu, sd[u]);
                        fma_quad<2>(dxa[4 * gx + 2], mu, sd[u]);
                        fma_quad<3>(dxa[4 * gx + 3], mu, sd[u]);
                    }
                }
                {   // dy: the channel sums of the block's cells, then the cells' entries
#pragma unroll
                    for (int u = 0; u < 16; u++) tile[u * kTileStride + lane] = sd[u];
                    wave_lds_sync();
                    ChannelOperand sdop;
                    sdop.read(tile, lane);
                    wave_lds_sync();  // (the tile is written again below)
                    const f32x4 sums = channel_sums(sdop, xop);
                    // the totals by cell in the tile, then a lane per entry of the block: coefficient x total
                    // of the entry's cell, added to dy[k] of the wave's row in LDS
#pragma unroll
                    for (int r = 0; r < 4; r++) tile[(4 * (lane >> 4) + r) * kPlanX + (lane & 15)] = sums[r];
                    wave_lds_sync();
                    for (int n0 = entries0; n0 < entries1; n0 += kWave) {
                        const int n = n0 + lane;
                        if (n < entries1) {
                            const int w = tab[pairs + 2 * n + 1];
                            atomicAdd(&dyl[w & 255], __int_as_float(tab[pairs + 2 * n]) * tile[w >> 8]);
                        }
                    }
                    wave_lds_sync();  // (the tile is written again by the next block)
                }
                // ds: the slots of one scalar are adjacent; a scalar's sum is stored when the next begins
#pragma unroll
                for (int u = 0; u < 16; u++) {
                    const int l = slot_l[b * 16 + u];
                    if (l != cur_l) {
                        if (cur_l >= 0 && active) *element_at(dsrow0, dsoff, (unsigned)ls.dim, (unsigned)cur_l) = (Val)dsa;
                        cur_l = l;
                        dsa = 0.f;
                    }
                    dsa = __builtin_fmaf(dz[u], T[u], dsa);
                }
#pragma unroll
                for (int u = 0; u < 16; u++) dz_held[u] = dz_ahead[u];
            }
            if (cur_l >= 0 && active) *element_at(dsrow0, dsoff, (unsigned)ls.dim, (unsigned)cur_l) = (Val)dsa;
            if (active)
                for (int z = 0; z < num_zero_l; z++)
                    *element_at(dsrow0, dsoff, (unsigned)ls.dim, (unsigned)plan[L.zero_l + z]) = Val(0);
            wave_lds_sync();
            if (lane < num_y) {
                const float v = dyl[lane];
                dyl[lane] = 0.f;
                Val *at = dy + ee * num_y + lane;
                if (dy_mode == kDyStore) *at = (Val)v;
                else if (dy_mode == kDyAdd) *at = (Val)((float)*at + v);
                else if constexpr (std::is_same<Val, float>::value) unsafeAtomicAdd(at, v);
            }
            if (group_is_receiver) {
                if constexpr (std::is_same<Val, float>::value) {  // (half values have no float atomics: sender rows only)
                    if (active) {
                        Val *dxrow0 = dx + (int64_t)xnode * lx.row;
#pragma unroll
                        for (int j = 0; j < XG * 4; j++)
                            if (j < X) unsafeAtomicAdd(element_at(dxrow0, xoff, (unsigned)lx.dim, (unsigned)j), dxa[j]);
                    }
                }
#pragma unroll
                for (int j = 0; j < XG * 4; j++) dxa[j] = 0.f;
            }
        }
        if (!group_is_receiver && active) {
            Val *dxrow0 = dx + (int64_t)g * lx.row;
#pragma unroll
            for (int j = 0; j < XG * 4; j++)
                if (j < X) *element_at(dxrow0, xoff, (unsigned)lx.dim, (unsigned)j) = (Val)dxa[j];
        }
    }
}

constexpr int kWavesPerBlock = 2;  // (120k edges, K = 128, l <= 3, before the skip of empty halves: forward 2.12 ms, backward 5.17 ms; four: 2.27 and 5.33; one: 2.10 and 6.07)

#define E3J_ROW(K, NB) {K<Val, NB, 1>, K<Val, NB, 2>, K<Val, NB, 3>, K<Val, NB, 4>}
#define E3J_TABLE(K) {E3J_ROW(K, 1), E3J_ROW(K, 2), E3J_ROW(K, 3), E3J_ROW(K, 4), \
                      E3J_ROW(K, 5), E3J_ROW(K, 6), E3J_ROW(K, 7), E3J_ROW(K, 8)}

template <typename Val>
int launch_plan_build_t(const e3j_amd_conv_params &p, const void *coef, bool cols_ji, int32_t *plan,
                        hipStream_t stream) {
    const PlanLayout L(p.num_coef, p.num_scalars);
    const int xg = (p.num_x + 3) / 4;
    if (p.coef_idx_bytes == 1)
        hipLaunchKernelGGL((plan_build_kernel<uint8_t, Val>), dim3(1), dim3(kBuildThreads), 0, stream,
                           static_cast<const Coef4D<uint8_t, Val> *>(coef), p.num_coef, p.num_x, p.num_y,
                           p.num_out, p.num_scalars, xg, cols_ji ? 1 : 0, plan, L);
    else
        hipLaunchKernelGGL((plan_build_kernel<int32_t, Val>), dim3(1), dim3(kBuildThreads), 0, stream,
                           static_cast<const Coef4D<int32_t, Val> *>(coef), p.num_coef, p.num_x, p.num_y,
                           p.num_out, p.num_scalars, xg, cols_ji ? 1 : 0, plan, L);
    return check_hip(hipGetLastError(), "convolution plan launch");
}

template <typename Val>
int launch_planned_fwd_t(const e3j_amd_conv_params &p, const int32_t *plan, const void *x, const void *y,
                         const void *s, const int32_t *other, const int32_t *row_ptr, const int32_t *perm,
                         void *out, hipStream_t stream) {
    typedef void (*Kernel)(const int32_t *, PlanLayout, const Val *, RowLayout, const Val *, int, const Val *,
                           RowLayout, const int32_t *, const int32_t *, const int32_t *, const int32_t *, Val *,
                           RowLayout, int, int, int, int, int, int);
    static const Kernel kernels[8][4] = E3J_TABLE(planned_fwd_kernel);
    const int nb = (p.num_out + 15) / 16, xg = (p.num_x + 3) / 4;
    const int nchunks = (p.channels + kWave - 1) / kWave;
    const int64_t items = (int64_t)p.num_nodes * nchunks;
    const int64_t blocks = (items + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution: grid too large");
    const size_t lds = sizeof(float) * ((size_t)table_words(p.num_coef) +
                                        (size_t)kWavesPerBlock * (nb * 16 * xg * 4 + p.num_scalars * kWave));
    if (lds > 64 * 1024) {
        const int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernels[nb - 1][xg - 1]),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                                 "hipFuncSetAttribute(planned fwd)");
        if (rc) return rc;
    }
    hipLaunchKernelGGL(kernels[nb - 1][xg - 1], dim3((unsigned)blocks), dim3(kWave, kWavesPerBlock), lds, stream, plan,
                       PlanLayout(p.num_coef, p.num_scalars), static_cast<const Val *>(x),
                       make_layout(p.layout, p.num_x, p.channels), static_cast<const Val *>(y), p.num_y,
                       static_cast<const Val *>(s), make_layout(p.layout, p.num_scalars, p.channels), other,
                       row_ptr, perm, p.row_order, static_cast<Val *>(out),
                       make_layout(p.layout, p.num_out, p.channels), p.num_nodes, p.channels, p.num_x,
                       p.num_scalars, p.num_coef, nchunks);
    return check_hip(hipGetLastError(), "convolution forward launch (planned)");
}

template <typename Val>
int launch_planned_bwd_t(const e3j_amd_conv_params &p, bool group_is_receiver, const int32_t *plan, const void *x,
                         const void *y, const void *s, const void *dm, const int32_t *other,
                         const int32_t *row_ptr, const int32_t *perm, void *dx, void *dy, void *ds,
                         hipStream_t stream) {
    typedef void (*Kernel)(const int32_t *, PlanLayout, const Val *, RowLayout, const Val *, int, const Val *,
                           RowLayout, const Val *, RowLayout, const int32_t *, const int32_t *, const int32_t *,
                           const int32_t *, Val *, Val *, Val *, int, int, int, int, int, int, int);
    static const Kernel kernels[8][4] = E3J_TABLE(planned_bwd_kernel);
    const int nb = (p.num_out + 15) / 16, xg = (p.num_x + 3) / 4;
    const int nchunks = (p.channels + kWave - 1) / kWave;
    const int64_t items = group_is_receiver ? (int64_t)p.num_nodes * nchunks : (int64_t)p.num_nodes;
    const int64_t blocks = (items + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "convolution_bwd: grid too large");
    const size_t lds = sizeof(float) * ((size_t)table_words(p.num_coef) +
                                        (size_t)kWavesPerBlock * (nb * 16 * xg * 4 + kPlanMaxY + p.num_scalars * kWave + kTileWords));
    if (lds > 64 * 1024) {
        const int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernels[nb - 1][xg - 1]),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                                 "hipFuncSetAttribute(planned bwd)");
        if (rc) return rc;
    }
    hipLaunchKernelGGL(kernels[nb - 1][xg - 1], dim3((unsigned)blocks), dim3(kWave, kWavesPerBlock), lds, stream, plan,
                       PlanLayout(p.num_coef, p.num_scalars), static_cast<const Val *>(x),
                       make_layout(p.layout, p.num_x, p.channels), static_cast<const Val *>(y), p.num_y,
                       static_cast<const Val *>(s), make_layout(p.layout, p.num_scalars, p.channels),
                       static_cast<const Val *>(dm), make_layout(p.layout, p.num_out, p.channels), other,
                       row_ptr, perm, p.row_order, static_cast<Val *>(dx), static_cast<Val *>(dy),
                       static_cast<Val *>(ds), p.num_nodes, p.channels, p.num_x, p.num_scalars, p.num_coef, nchunks,
                       group_is_receiver ? 1 : 0);
    return check_hip(hipGetLastError(), "convolution backward launch (planned)");
}
#undef E3J_TABLE
#undef E3J_ROW

// whether the sizes of a call fit a plan (the value type is the caller's question)
inline bool plan_sizes_fit(const e3j_amd_conv_params &p) {
    return p.num_out >= 1 && p.num_out <= kSlots && p.num_x >= 1 && p.num_x <= kPlanX && p.num_y >= 1 &&
           p.num_y <= kPlanMaxY && p.num_scalars >= 1 && p.num_scalars <= kPlanMaxS && p.num_coef >= 1 &&
           p.num_coef <= kPlanMaxCoef && p.channels >= 1;
}
inline size_t plan_words(const e3j_amd_conv_params &p) { return (size_t)PlanLayout(p.num_coef, p.num_scalars).words; }

}  // namespace

// The float16 instantiations are compiled in a unit of their own (conv_planned_f16.hip).
int launch_plan_build_f16(const e3j_amd_conv_params &p, const void *coef, bool cols_ji, int32_t *plan,
                          hipStream_t stream);
int launch_planned_fwd_f16(const e3j_amd_conv_params &p, const int32_t *plan, const void *x, const void *y,
                           const void *s, const int32_t *other, const int32_t *row_ptr, const int32_t *perm,
                           void *out, hipStream_t stream);
int launch_planned_bwd_f16(const e3j_amd_conv_params &p, bool group_is_receiver, const int32_t *plan, const void *x,
                           const void *y, const void *s, const void *dm, const int32_t *other,
                           const int32_t *row_ptr, const int32_t *perm, void *dx, void *dy, void *ds,
                           hipStream_t stream);

}  // namespace e3j_amd
#endif
