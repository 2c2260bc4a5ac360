// Graph preparation on the device: CSR row pointers and the stable edge sort
// behind the unsorted (GraphOrdering NONE) path and the transposed adjacency.
//
// Restates GraphCSR (src/e3j/data/graph.py:49-73): row_ptr = [0] +
// cumsum(bincount(key, length = N)) with out-of-range keys dropped, and
// sort = stable argsort by key.  The sort is rocPRIM's radix sort (via hipCUB)
// on unsigned keys, so sentinel and negative keys land after every live row.

#include <hipcub/hipcub.hpp>

#include <mutex>

#include "common.h"

namespace e3j_amd {
namespace {

// Histogram of the in-range keys into counts[key + 1].  A thread walks a short run of
// consecutive positions and issues one atomic per run of equal keys: sorted keys (the
// common case) then cost one atomic per thread instead of one per edge on a hot address.
constexpr int kCountChunk = 16;
__global__ void count_keys_kernel(const int32_t *__restrict__ key, int64_t num_edges, int num_nodes,
                                  int32_t *__restrict__ counts) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x * kCountChunk;
    for (int64_t base = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * kCountChunk;
         base < num_edges; base += stride) {
        const int64_t end = base + kCountChunk < num_edges ? base + kCountChunk : num_edges;
        int run_key = key[base], run = 1;
        for (int64_t e = base + 1; e < end; e++) {
            const int k = key[e];
            if (k == run_key) { run++; continue; }
            if ((unsigned)run_key < (unsigned)num_nodes) atomicAdd(&counts[run_key + 1], run);
            run_key = k; run = 1;
        }
        if ((unsigned)run_key < (unsigned)num_nodes) atomicAdd(&counts[run_key + 1], run);
    }
}

__global__ void iota_kernel(int32_t *__restrict__ out, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        out[i] = (int32_t)i;
}

__global__ void gather_kernel(const int32_t *__restrict__ src, const int32_t *__restrict__ perm,
                              int32_t *__restrict__ dst, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        dst[i] = src[perm[i]];
}

// One sweep of minimum-label propagation over a CSR adjacency:
// next[n] = min(cur[n], cur[m] for every m in row n).  One thread per row, no atomics.
// A row is read up to kLabelRowCap positions: the labels only steer which rows run together,
// and a thread that walked a hub's whole row would outlast the rest of the sweep many times.
constexpr int kLabelRowCap = 128;
constexpr int kLabelLanes = 4;  // lanes that share a row (its gathers then run four at a time)
__global__ void min_label_kernel(const int32_t *__restrict__ other,
                                 const int32_t *__restrict__ row_ptr, int num_nodes,
                                 const int32_t *__restrict__ cur, int32_t *__restrict__ next) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    const int n = t / kLabelLanes, part = t % kLabelLanes;
    const bool inside = n < num_nodes;  // (no early exit: the lanes of a group exchange below)
    // cur == nullptr: every node still carries its own id (the first sweep)
    int best = inside ? (cur ? cur[n] : n) : 0;
    if (inside) {
        const int begin = row_ptr[n];
        const int end = min(row_ptr[n + 1], begin + kLabelRowCap);
        for (int e = begin + part; e < end; e += kLabelLanes) {
            const int m = other[e];
            if ((unsigned)m < (unsigned)num_nodes) best = min(best, cur ? cur[m] : m);
        }
    }
#pragma unroll
    for (int off = 1; off < kLabelLanes; off *= 2) best = min(best, __shfl_xor(best, off, kWave));
    if (inside && part == 0) next[n] = best;
}

// key = (label after the second sweep, label after the first): one sort lists the coarse clusters
// and, inside them, the fine ones
__global__ void two_level_keys_kernel(const int32_t *__restrict__ coarse, const int32_t *__restrict__ fine,
                                      int num_nodes, int bits, uint32_t *__restrict__ keys,
                                      int32_t *__restrict__ vals) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= num_nodes) return;
    keys[i] = ((uint32_t)coarse[i] << bits) | (uint32_t)fine[i];
    vals[i] = i;
}

__global__ void copy_i32_kernel(const int32_t *__restrict__ src, int32_t *__restrict__ dst, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

// Rows with more than twice the mean number of edges ("long rows"): flag per list position.
__global__ void long_row_flags_kernel(const int32_t *__restrict__ order, const int32_t *__restrict__ row_ptr,
                                      int num_nodes, int32_t *__restrict__ flags) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= num_nodes) return;
    const int r = order[i];
    const int64_t degree = row_ptr[r + 1] - row_ptr[r];
    flags[i] = degree * num_nodes > 2 * (int64_t)row_ptr[num_nodes] ? 1 : 0;
}

// The kernels hand one contiguous eighth of the row list to each XCD and every XCD walks its
// eighth front to back.  Long rows started late leave the machine waiting for a few waves at
// the end, so they are dealt to the fronts of the eighths: eighth p takes the p-th eighth of the
// long rows, then the p-th eighth of the others, both in list order.  `rank` is the
// inclusive prefix sum of `flags`.  Without long rows the list is unchanged.
__global__ void deal_long_rows_kernel(const int32_t *__restrict__ order, const int32_t *__restrict__ flags,
                                      const int32_t *__restrict__ rank, int num_nodes,
                                      int32_t *__restrict__ dealt) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= num_nodes) return;
    constexpr int64_t kParts = 8;
    const int64_t num_long = rank[num_nodes - 1], num_short = num_nodes - num_long;
    const bool is_long = flags[i] != 0;
    const int64_t mine = is_long ? rank[i] - 1 : i - rank[i];  // position among the rows of its kind
    const int64_t kind = is_long ? num_long : num_short;
    int64_t part = 0;
    while (part < kParts - 1 && (part + 1) * kind / kParts <= mine) part++;
    const int64_t start = part * num_long / kParts + part * num_short / kParts;
    const int64_t longs_here = (part + 1) * num_long / kParts - part * num_long / kParts;
    const int64_t at = is_long ? start + (mine - part * num_long / kParts)
                               : start + longs_here + (mine - part * num_short / kParts);
    dealt[at] = order[i];
}

size_t align_up(size_t v, size_t a = 256) { return (v + a - 1) / a * a; }

unsigned grid_for(int64_t n) { return (unsigned)std::max<int64_t>(1, std::min<int64_t>((n + 255) / 256, 4096)); }

size_t scan_temp_bytes(int32_t num_nodes) {
    size_t bytes = 0;
    hipcub::DeviceScan::InclusiveSum(nullptr, bytes, (int32_t *)nullptr, (int32_t *)nullptr,
                                     num_nodes + 1);
    return bytes;
}

size_t sort_temp_bytes(int64_t num_edges) {
    size_t bytes = 0;
    hipcub::DeviceRadixSort::SortPairs(nullptr, bytes, (const uint32_t *)nullptr, (uint32_t *)nullptr,
                                       (const int32_t *)nullptr, (int32_t *)nullptr, (int)num_edges);
    return bytes;
}

int row_ptr_impl(const int32_t *key, int64_t num_edges, int32_t num_nodes, int32_t *row_ptr,
                 void *temp, size_t temp_bytes, hipStream_t stream) {
    int rc = launch_fill_zero(row_ptr, sizeof(int32_t) * ((size_t)num_nodes + 1), stream);
    if (rc) return rc;
    if (num_edges > 0) {
        hipLaunchKernelGGL(count_keys_kernel, dim3(grid_for((num_edges + kCountChunk - 1) / kCountChunk)),
                           dim3(256), 0, stream, key, num_edges, num_nodes, row_ptr);
        rc = check_hip(hipGetLastError(), "csr count launch");
        if (rc) return rc;
    }
    return check_hip(hipcub::DeviceScan::InclusiveSum(temp, temp_bytes, row_ptr, row_ptr,
                                                      num_nodes + 1, stream),
                     "csr scan");
}

// Global node ids of a sharded graph reduced to shard-local ids; the sentinel stays.
__global__ void wrap_index_kernel(const int32_t *__restrict__ index, int64_t n, int32_t num_nodes,
                                  int32_t *__restrict__ out) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const int32_t v = index[i];
        int32_t r = v;
        if (v != INT32_MAX) {
            r = v % num_nodes;          // Python semantics: the result takes the divisor's sign
            if (r < 0) r += num_nodes;
        }
        out[i] = r;
    }
}

__global__ void live_keys_kernel(const int32_t *__restrict__ other, const int32_t *__restrict__ row_ptr,
                                 int32_t num_nodes, int64_t num_edges, int32_t *__restrict__ keys) {
    const int64_t live_end = row_ptr[num_nodes];
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < num_edges; i += stride) {
        const int32_t v = other[i];
        keys[i] = (i < live_end && (unsigned)v < (unsigned)num_nodes) ? v : INT32_MAX;
    }
}


// ---- schedule of the backward over tiles of receivers ---------------------------------------
// Tiles are `tile_rows` consecutive entries of the row order.  A scan of the tiles' position
// counts places each tile's list; one wave per tile then writes the list, sorted by sender.

__global__ void tile_rank_kernel(const int32_t *__restrict__ row_order, int num_nodes,
                                 int32_t *__restrict__ rank) {
    const int q = blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= num_nodes) return;
    rank[row_order ? row_order[q] : q] = q;
}

// Per tile, two numbers that one prefix sum carries side by side in a 64-bit word: the positions
// of the tile (high half) and the work descriptors it is cut into (low half); both totals stay
// below 2^31, so the low half never carries into the high one.
__device__ inline int tile_start(uint64_t packed) { return (int)(packed >> 32); }
__device__ inline int tile_first_piece(uint64_t packed) { return (int)(uint32_t)packed; }

// packed[t + 1] = (positions of tile t, descriptors of tile t); packed[0] = 0
__global__ void tile_count_kernel(const int32_t *__restrict__ row_order, const int32_t *__restrict__ row_ptr,
                                  int num_nodes, int tile_rows, int num_tiles, int max_work_edges,
                                  uint64_t *__restrict__ packed) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t == 0) packed[0] = 0;
    if (t >= num_tiles) return;
    int total = 0;
    for (int q = t * tile_rows; q < (t + 1) * tile_rows && q < num_nodes; q++) {
        const int r = row_order ? row_order[q] : q;
        total += row_ptr[r + 1] - row_ptr[r];
    }
    const int pieces = total == 0 ? 1 : (total + max_work_edges - 1) / max_work_edges;
    packed[t + 1] = ((uint64_t)total << 32) | (uint64_t)pieces;
}

// The three lists of one tile, by one wave: the tile's positions (its rows in tile order, each
// row's positions ascending) are keyed by (sender, position), padding senders after the live
// ones, and sorted in LDS with a bitonic network when the tile has at most kTileSortLimit of
// them.  Longer tiles (hub rows) are not sorted by sender, only split into live positions first
// and padding positions last, which is all the kernel needs for correctness (it sums runs of
// equal senders wherever they occur); a hub's senders are mostly distinct anyway.
// The entries past the last row (padding positions that belong to no tile) are filled by all
// threads of the grid before they turn to their tiles.
constexpr int kTileSortLimit = 512;
__global__ __launch_bounds__(256) void tile_lists_kernel(
    const int32_t *__restrict__ other, const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ row_order, const uint64_t *__restrict__ packed, int num_nodes, int64_t num_edges,
    int tile_rows, int num_tiles, int32_t *__restrict__ t_sender, int32_t *__restrict__ t_edge,
    int32_t *__restrict__ t_local) {
    __shared__ uint64_t keys_all[4][kTileSortLimit];
    __shared__ uint16_t local_all[4][kTileSortLimit];
    {
        const int64_t stride = (int64_t)gridDim.x * blockDim.x;
        for (int64_t i = (int64_t)row_ptr[num_nodes] + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
             i < num_edges; i += stride) {
            t_sender[i] = -1; t_edge[i] = 0; t_local[i] = 0;
        }
    }
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int t = blockIdx.x * 4 + wave;
    if (t >= num_tiles) return;
    uint64_t *keys = keys_all[wave];
    uint16_t *locals = local_all[wave];
    const int begin = tile_start(packed[t]), m = tile_start(packed[t + 1]) - begin;
    if (m == 0) return;
    const int first = t * tile_rows;
    const int rows = num_nodes - first < tile_rows ? num_nodes - first : tile_rows;
    if (m <= kTileSortLimit) {
        int filled = 0;
        for (int i = 0; i < rows; i++) {
            const int r = row_order ? row_order[first + i] : first + i;
            const int b = row_ptr[r], d = row_ptr[r + 1] - b;
            for (int q = lane; q < d; q += 64) {
                const int snd = other[b + q];
                const uint64_t sk = (unsigned)snd < (unsigned)num_nodes ? (uint64_t)snd : (uint64_t)num_nodes;
                // (sender, position) orders the list; the row the position came from travels beside it
                keys[filled + q] = (sk << 32) | (uint64_t)(uint32_t)(b + q);
                locals[filled + q] = (uint16_t)i;
            }
            filled += d;
        }
        int padded = 64;
        while (padded < m) padded *= 2;
        for (int q = m + lane; q < padded; q += 64) { keys[q] = ~0ull; locals[q] = 0; }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        for (int k = 2; k <= padded; k *= 2) {
            for (int j = k / 2; j > 0; j /= 2) {
                // a lane per pair (q, q | j): q is the pair's number with a zero bit put in at j
                for (int pr = lane; pr < padded / 2; pr += 64) {
                    const int q = ((pr & ~(j - 1)) << 1) | (pr & (j - 1));
                    const int partner = q | j;
                    const uint64_t a = keys[q], c = keys[partner];
                    const bool ascending = (q & k) == 0;
                    if ((a > c) == ascending) {
                        keys[q] = c; keys[partner] = a;
                        const uint16_t la = locals[q];
                        locals[q] = locals[partner]; locals[partner] = la;
                    }
                }
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
        }
        for (int q = lane; q < m; q += 64) {
            const uint64_t key = keys[q];
            const int pos = (int)(uint32_t)key;
            const uint64_t sk = key >> 32;
            t_sender[begin + q] = sk == (uint64_t)num_nodes ? -1 : (int32_t)sk;
            t_edge[begin + q] = perm ? perm[pos] : pos;
            t_local[begin + q] = locals[q];
        }
        return;
    }
    // a long tile: live positions in tile order, then the padding positions
    int at = begin;
    for (int pass = 0; pass < 2; pass++) {
        for (int i = 0; i < rows; i++) {
            const int r = row_order ? row_order[first + i] : first + i;
            const int b = row_ptr[r], d = row_ptr[r + 1] - b;
            for (int q0 = 0; q0 < d; q0 += 64) {
                const int q = q0 + lane;
                const int snd = q < d ? other[b + q] : -1;
                const bool live = (unsigned)snd < (unsigned)num_nodes;
                const bool mine = q < d && (live == (pass == 0));
                const unsigned long long mask = __ballot(mine);
                if (mine) {
                    const int slot = at + __popcll(mask & ((1ull << lane) - 1ull));
                    t_sender[slot] = live ? snd : -1;
                    t_edge[slot] = perm ? perm[b + q] : b + q;
                    t_local[slot] = i;
                }
                at += __popcll(mask);
            }
        }
    }
}

// descriptors (tile, begin, end, 0), the first num_used of the num_work entries (a tile without
// positions takes one, with begin == end; the entries behind the used ones are not written),
// num_used in the fourth field of descriptor 0; `packed`: inclusive prefix sums, entry 0 = 0
__global__ void tile_work_kernel(const uint64_t *__restrict__ packed, int num_tiles, int max_work_edges,
                                 int32_t *__restrict__ work) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= num_tiles) return;
    const int begin = tile_start(packed[t]), end = tile_start(packed[t + 1]);
    int w = tile_first_piece(packed[t]);
    if (begin == end) {
        work[4 * w] = t; work[4 * w + 1] = begin; work[4 * w + 2] = begin; work[4 * w + 3] = 0;
    }
    for (int b = begin; b < end; b += max_work_edges, w++) {
        work[4 * w] = t;
        work[4 * w + 1] = b;
        work[4 * w + 2] = b + max_work_edges < end ? b + max_work_edges : end;
        work[4 * w + 3] = 0;
    }
    // the number of descriptors in use, for the kernel to deal them evenly to the XCDs (the
    // thread of tile 0 wrote descriptor 0 just above)
    if (t == 0) work[3] = tile_first_piece(packed[num_tiles]);
}

size_t scan64_temp_bytes(int32_t n) {
    size_t bytes = 0;
    hipcub::DeviceScan::InclusiveSum(nullptr, bytes, (uint64_t *)nullptr, (uint64_t *)nullptr, (int)std::max(n, 1));
    return bytes;
}

struct TileWorkspace {
    size_t temp, temp_bytes, packed, total;
    TileWorkspace(int32_t num_nodes, int32_t tile_rows) {
        const size_t n = (size_t)num_nodes;
        const size_t tiles = (n + (size_t)tile_rows - 1) / (size_t)tile_rows;
        size_t at = 0;
        auto take = [&](size_t bytes) { const size_t here = at; at += align_up(bytes); return here; };
        temp_bytes = scan64_temp_bytes((int32_t)tiles + 1);
        temp = take(temp_bytes);
        packed = take(8 * (tiles + 1));
        total = at;
    }
};


// rows[pos] = the CSR row that holds position pos; INT32_MAX past the last row
__global__ void expand_rows_kernel(const int32_t *__restrict__ row_ptr, int num_nodes, int64_t num_edges,
                                   int32_t *__restrict__ rows) {
    const int64_t live_end = row_ptr[num_nodes];
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t pos = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; pos < num_edges; pos += stride) {
        if (pos >= live_end) { rows[pos] = INT32_MAX; continue; }
        int lo = 0, hi = num_nodes;  // row_ptr[lo] <= pos < row_ptr[hi]
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (row_ptr[mid] <= pos) lo = mid; else hi = mid;
        }
        rows[pos] = lo;
    }
}

__global__ void compose_perm_kernel(const int32_t *__restrict__ outer, const int32_t *__restrict__ inner,
                                    int64_t n, int32_t *__restrict__ out) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        out[i] = inner ? inner[outer[i]] : outer[i];
}

// Pieces of the rows longer than `cap`, past their first `cap` positions: a row reserves its
// pieces with one atomic on the count (the order of the list is free).
__global__ void row_segments_kernel(const int32_t *__restrict__ row_ptr, int num_nodes, int cap, int piece,
                                    int max_segments, int32_t *__restrict__ segments) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= num_nodes) return;
    const int begin = row_ptr[r], end = row_ptr[r + 1];
    if (end - begin <= cap) return;
    const int extra = (end - begin - 1) / piece;  // pieces after the first
    const int at = atomicAdd(segments, extra);
    for (int k = 0; k < extra && at + k < max_segments; k++) {
        const int b = begin + (k + 1) * piece;
        int32_t *seg = segments + 4 + 3 * (at + k);
        seg[0] = r;
        seg[1] = b;
        seg[2] = b + piece < end ? b + piece : end;
    }
}

// ---- pairing of rows for the backward over tiles of two receivers ------------------------------
// Two rows that share most of their senders should sit in one tile: the tile then issues one set
// of dx atomics for every shared sender.  Every row picks, among the rows it has an edge from,
// the one with which it has the most senders in common; rows that pick each other are paired, the
// rest pick again among the rows still free (a few rounds of this greedy matching pair most rows
// of a radius graph).  Pairs are then listed first, in the order their earlier member had, each
// pair on an even and the following odd position; the unpaired rows follow in their old order.
constexpr int kPairMaxDegree = 128;  // rows with more edges (or none) stay unpaired
constexpr int kPairSlots = 256;      // hash slots per wave for the senders of its row
constexpr int kPairRounds = 4;

__device__ __forceinline__ unsigned pair_hash(int v) { return ((unsigned)v * 2654435761u) >> 24; }

// common[pos] = number of senders that the row of position pos and the row other[pos] share
// (-1: no candidate).  One wave per row; its senders go into a hash set in LDS, then every lane
// walks the row of one neighbour and counts hits.
__global__ __launch_bounds__(256) void pair_common_kernel(const int32_t *__restrict__ other,
                                                          const int32_t *__restrict__ row_ptr, int num_nodes,
                                                          int32_t *__restrict__ common) {
    __shared__ int32_t slots_all[4][kPairSlots];
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int i = blockIdx.x * 4 + wave;
    if (i >= num_nodes) return;
    int32_t *slots = slots_all[wave];
    const int begin = row_ptr[i], deg = row_ptr[i + 1] - begin;
    if (deg < 1) return;
    if (deg > kPairMaxDegree) {
        for (int q = lane; q < deg; q += 64) common[begin + q] = -1;
        return;
    }
    for (int t = lane; t < kPairSlots; t += 64) slots[t] = -1;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (int q = lane; q < deg; q += 64) {
        const int v = other[begin + q];
        if ((unsigned)v >= (unsigned)num_nodes) continue;
        unsigned h = pair_hash(v);
        for (int probe = 0; probe < kPairSlots; probe++) {
            const int old = atomicCAS(&slots[h], -1, v);
            if (old == -1 || old == v) break;
            h = (h + 1) % kPairSlots;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (int q = lane; q < deg; q += 64) {
        const int p = other[begin + q];
        int count = -1;
        if ((unsigned)p < (unsigned)num_nodes && p != i) {
            const int pb = row_ptr[p], pd = row_ptr[p + 1] - pb;
            if (pd >= 1 && pd <= kPairMaxDegree) {
                count = 0;
                for (int t = 0; t < pd; t++) {
                    const int v = other[pb + t];
                    if ((unsigned)v >= (unsigned)num_nodes) continue;
                    unsigned h = pair_hash(v);
                    for (int probe = 0; probe < kPairSlots; probe++) {
                        const int held = slots[h];
                        if (held == v) { count++; break; }
                        if (held == -1) break;
                        h = (h + 1) % kPairSlots;
                    }
                }
            }
        }
        common[begin + q] = count;
    }
}

// best[i] = the free row with the most senders in common with free row i (smaller id on ties), -1 if none
__global__ void pair_best_kernel(const int32_t *__restrict__ other, const int32_t *__restrict__ row_ptr,
                                 const int32_t *__restrict__ common, const int32_t *__restrict__ partner,
                                 int num_nodes, int32_t *__restrict__ best) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= num_nodes) return;
    int pick = -1, most = -1;
    const int begin = row_ptr[i], deg = row_ptr[i + 1] - begin;
    if (partner[i] < 0 && deg >= 1 && deg <= kPairMaxDegree) {
        for (int q = 0; q < deg; q++) {
            const int c = common[begin + q];
            if (c < 0) continue;
            const int p = other[begin + q];
            if (partner[p] >= 0) continue;
            if (c > most || (c == most && p < pick)) { most = c; pick = p; }
        }
    }
    best[i] = pick;
}

__global__ void pair_match_kernel(const int32_t *__restrict__ best, int num_nodes, int32_t *__restrict__ partner) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= num_nodes) return;
    const int p = best[i];
    if (p >= 0 && best[p] == i) partner[i] = p;  // (the thread of row p writes partner[p] = i)
}

__global__ void pair_keys_kernel(const int32_t *__restrict__ partner, const int32_t *__restrict__ rank,
                                 int num_nodes, uint32_t *__restrict__ keys, int32_t *__restrict__ vals) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= num_nodes) return;
    const int p = partner[i];
    const unsigned mine = rank ? rank[i] : i;
    vals[i] = i;
    if (p < 0) {
        keys[i] = 2u * (unsigned)num_nodes + mine;
    } else {
        const unsigned theirs = rank ? rank[p] : p;
        keys[i] = 2u * (mine < theirs ? mine : theirs) + (mine > theirs ? 1u : 0u);
    }
}

__global__ void fill_i32_kernel(int32_t *__restrict__ out, int64_t n, int32_t value) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = value;
}

}  // namespace

int launch_live_keys(const int32_t *other, const int32_t *row_ptr, int32_t num_nodes,
                     int64_t num_edges, int32_t *keys, hipStream_t stream) {
    if (num_edges == 0) return E3J_AMD_OK;
    hipLaunchKernelGGL(live_keys_kernel, dim3(grid_for(num_edges)), dim3(256), 0, stream, other, row_ptr,
                       num_nodes, num_edges, keys);
    return check_hip(hipGetLastError(), "live keys launch");
}

int launch_expand_rows(const int32_t *row_ptr, int32_t num_nodes, int64_t num_edges, int32_t *rows,
                       hipStream_t stream) {
    if (num_edges == 0) return E3J_AMD_OK;
    hipLaunchKernelGGL(expand_rows_kernel, dim3(grid_for(num_edges)), dim3(256), 0, stream, row_ptr, num_nodes,
                       num_edges, rows);
    return check_hip(hipGetLastError(), "expand rows launch");
}

int launch_compose_perm(const int32_t *outer, const int32_t *inner, int64_t n, int32_t *out, hipStream_t stream) {
    if (n == 0) return E3J_AMD_OK;
    hipLaunchKernelGGL(compose_perm_kernel, dim3(grid_for(n)), dim3(256), 0, stream, outer, inner, n, out);
    return check_hip(hipGetLastError(), "compose permutation launch");
}

}  // namespace e3j_amd

using namespace e3j_amd;

extern "C" {

size_t e3j_amd_csr_workspace_bytes(int32_t num_nodes, int64_t num_edges) {
    if (num_nodes < 0 || num_edges < 0) return 0;
    // [scan temp | sort temp | keys_out (E) | iota (E)]
    return align_up(scan_temp_bytes(num_nodes)) + align_up(sort_temp_bytes(num_edges)) +
           2 * align_up(sizeof(int32_t) * (size_t)num_edges) + 256;
}

int e3j_amd_csr_row_ptr(const int32_t *key, int64_t num_edges, int32_t num_nodes, int32_t *row_ptr,
                        void *workspace, void *stream_) {
    if (num_nodes < 0 || num_nodes >= INT32_MAX || num_edges < 0 || num_edges > 0x7fffffffLL)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "csr_row_ptr: bad sizes");
    if (row_ptr == nullptr || workspace == nullptr || (num_edges > 0 && key == nullptr))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "csr_row_ptr: null operand");
    return row_ptr_impl(key, num_edges, num_nodes, row_ptr, workspace, scan_temp_bytes(num_nodes),
                        static_cast<hipStream_t>(stream_));
}

// ---- row pointers without a workspace argument ------------------------------------------------
// The scan of e3j_amd_csr_row_ptr needs a few KB of temporary storage.  Callers that cannot
// allocate (code under graph capture, serving loops) get it from this array instead: device
// memory of the library's code object, one copy per GPU, held until the process ends.
constexpr size_t kStaticScratchBytes = 256 * 1024;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];  // address of `scratch` on each device, looked up once
// The device address of the array on the current device (the array's name is only a host-side
// handle of the symbol).
int static_scratch(void **ptr) {
    int device = 0;
    int rc = check_hip(hipGetDevice(&device), "csr_row_ptr_static: hipGetDevice");
    if (rc) return rc;
    if (device < 0 || device >= kMaxDevices)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "csr_row_ptr_static: device index out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[device] == nullptr) {
        void *address = nullptr;
        rc = check_hip(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)), "csr_row_ptr_static: hipGetSymbolAddress");
        if (rc) return rc;
        g_scratch_ptr[device] = address;
    }
    *ptr = g_scratch_ptr[device];
    return E3J_AMD_OK;
}
}  // namespace

int32_t e3j_amd_csr_row_ptr_static_max_nodes(void) {
    // the scan's temporary storage grows with the number of entries; largest count that fits
    int32_t lo = 0, hi = INT32_MAX - 1;
    while (lo < hi) {
        const int32_t mid = lo + (hi - lo + 1) / 2;
        if (scan_temp_bytes(mid) <= kStaticScratchBytes) lo = mid; else hi = mid - 1;
    }
    return lo;
}

int e3j_amd_csr_row_ptr_static(const int32_t *key, int64_t num_edges, int32_t num_nodes, int32_t *row_ptr,
                               void *stream_) {
    // (num_nodes + 1 entries are scanned: INT32_MAX nodes would overflow the count)
    if (num_nodes < 0 || num_nodes >= INT32_MAX || num_edges < 0 || num_edges > 0x7fffffffLL)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "csr_row_ptr_static: bad sizes");
    if (row_ptr == nullptr || (num_edges > 0 && key == nullptr))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "csr_row_ptr_static: null operand");
    const size_t need = scan_temp_bytes(num_nodes);
    if (need > kStaticScratchBytes)
        return set_error(E3J_AMD_INVALID_ARGUMENT,
                         "csr_row_ptr_static: " + std::to_string(num_nodes) + " nodes need " + std::to_string(need) +
                             " bytes of scan storage, the built-in scratch holds " +
                             std::to_string(kStaticScratchBytes) + " (use e3j_amd_csr_row_ptr with a workspace)");
    void *temp = nullptr;
    int rc = static_scratch(&temp);
    if (rc) return rc;
    return row_ptr_impl(key, num_edges, num_nodes, row_ptr, temp, need, static_cast<hipStream_t>(stream_));
}

int64_t e3j_amd_row_segments_max(int64_t num_edges, int32_t row_piece) {
    if (num_edges <= 0 || row_piece <= 0) return 0;
    return num_edges / row_piece;  // a piece after the first follows row_piece positions of its row
}

int e3j_amd_row_segments_build(const int32_t *receiver_ptr, int32_t num_nodes, int32_t row_cap,
                               int32_t row_piece, int32_t max_segments, int32_t *segments, void *stream_) {
    if (num_nodes < 0 || row_piece <= 0 || row_cap < row_piece || max_segments < 0)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "row_segments_build: bad sizes");
    if (segments == nullptr || (num_nodes > 0 && receiver_ptr == nullptr))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "row_segments_build: null operand");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int rc = launch_fill_zero(segments, sizeof(int32_t) * 4, stream);
    if (rc || num_nodes == 0) return rc;
    hipLaunchKernelGGL(row_segments_kernel, dim3(grid_for(num_nodes)), dim3(256), 0, stream, receiver_ptr,
                       num_nodes, row_cap, row_piece, max_segments, segments);
    return check_hip(hipGetLastError(), "row_segments_build");
}

int e3j_amd_wrap_index(const int32_t *index, int64_t n, int32_t num_nodes, int32_t *out,
                       void *stream_) {
    if (n < 0 || num_nodes <= 0)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "wrap_index: bad sizes");
    if (n == 0) return E3J_AMD_OK;
    if (index == nullptr || out == nullptr)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "wrap_index: null operand");
    hipLaunchKernelGGL(wrap_index_kernel, dim3(grid_for(n)), dim3(256), 0, (hipStream_t)stream_,
                       index, n, num_nodes, out);
    return check_hip(hipGetLastError(), "wrap_index");
}

namespace {
struct PairWorkspace {
    size_t temp, temp_bytes, common, best, partner, rank, keys_in, keys_out, vals_in, total;
    PairWorkspace(int32_t num_nodes, int64_t num_edges) {
        const size_t n = (size_t)num_nodes, e = (size_t)num_edges;
        size_t at = 0;
        auto take = [&](size_t bytes) { const size_t here = at; at += align_up(bytes); return here; };
        temp_bytes = sort_temp_bytes(num_nodes);
        temp = take(temp_bytes);
        common = take(4 * e);
        best = take(4 * n); partner = take(4 * n); rank = take(4 * n);
        keys_in = take(4 * n); keys_out = take(4 * n); vals_in = take(4 * n);
        total = at + 256;
    }
};
}  // namespace

size_t e3j_amd_pair_rows_workspace_bytes(int32_t num_nodes, int64_t num_edges) {
    if (num_nodes < 0 || num_edges < 0) return 0;
    return PairWorkspace(num_nodes, num_edges).total;
}

int e3j_amd_pair_rows(const int32_t *other, const int32_t *row_ptr, int32_t num_nodes, int64_t num_edges,
                      const int32_t *order_in, int32_t *order_out, void *workspace, void *stream_) {
    if (num_nodes < 0 || num_edges < 0 || num_edges > 0x7fffffffLL || num_nodes > 0x3fffffff)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "pair_rows: bad sizes");
    if (num_nodes == 0) return E3J_AMD_OK;
    if (order_out == nullptr || workspace == nullptr || row_ptr == nullptr || (num_edges > 0 && other == nullptr))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "pair_rows: null operand");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    unsigned char *ws = static_cast<unsigned char *>(workspace);
    const PairWorkspace w(num_nodes, num_edges);
    int32_t *common = reinterpret_cast<int32_t *>(ws + w.common);
    int32_t *best = reinterpret_cast<int32_t *>(ws + w.best);
    int32_t *partner = reinterpret_cast<int32_t *>(ws + w.partner);
    int32_t *rank = reinterpret_cast<int32_t *>(ws + w.rank);
    uint32_t *keys_in = reinterpret_cast<uint32_t *>(ws + w.keys_in);
    uint32_t *keys_out = reinterpret_cast<uint32_t *>(ws + w.keys_out);
    int32_t *vals_in = reinterpret_cast<int32_t *>(ws + w.vals_in);
    const unsigned rows_grid = (unsigned)((num_nodes + 255) / 256);

    hipLaunchKernelGGL(fill_i32_kernel, dim3(grid_for(num_nodes)), dim3(256), 0, stream, partner,
                       (int64_t)num_nodes, -1);
    hipLaunchKernelGGL(pair_common_kernel, dim3((unsigned)((num_nodes + 3) / 4)), dim3(256), 0, stream, other,
                       row_ptr, num_nodes, common);
    int rc = check_hip(hipGetLastError(), "pair_rows common");
    if (rc) return rc;
    for (int round = 0; round < kPairRounds; round++) {
        hipLaunchKernelGGL(pair_best_kernel, dim3(rows_grid), dim3(256), 0, stream, other, row_ptr, common, partner,
                           num_nodes, best);
        hipLaunchKernelGGL(pair_match_kernel, dim3(rows_grid), dim3(256), 0, stream, best, num_nodes, partner);
    }
    if (order_in != nullptr)
        hipLaunchKernelGGL(tile_rank_kernel, dim3(rows_grid), dim3(256), 0, stream, order_in, num_nodes, rank);
    hipLaunchKernelGGL(pair_keys_kernel, dim3(rows_grid), dim3(256), 0, stream, partner,
                       order_in != nullptr ? rank : nullptr, num_nodes, keys_in, vals_in);
    rc = check_hip(hipGetLastError(), "pair_rows keys");
    if (rc) return rc;
    int key_bits = 2;  // keys are below 3 * num_nodes
    while (key_bits < 32 && ((uint64_t)1 << key_bits) < 3ull * (uint64_t)num_nodes) key_bits++;
    size_t temp_bytes = w.temp_bytes;
    return check_hip(hipcub::DeviceRadixSort::SortPairs(ws + w.temp, temp_bytes, keys_in, keys_out, vals_in,
                                                        order_out, (int)num_nodes, 0, key_bits, stream),
                     "pair_rows sort");
}

size_t e3j_amd_order_workspace_bytes(int32_t num_nodes) {
    if (num_nodes < 0) return 0;
    // [sort / scan temp | label a | label b | keys in | keys out | order tmp]
    return align_up(std::max(sort_temp_bytes(num_nodes), scan_temp_bytes(num_nodes))) +
           5 * align_up(sizeof(int32_t) * (size_t)num_nodes) + 256;
}

int e3j_amd_locality_order(const int32_t *other, const int32_t *row_ptr, int32_t num_nodes,
                           int32_t rounds, int32_t *order, void *workspace, void *stream_) {
    if (num_nodes < 0 || rounds < 0 || rounds > 64)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "locality_order: bad sizes");
    if (num_nodes == 0) return E3J_AMD_OK;
    if (order == nullptr || workspace == nullptr || row_ptr == nullptr)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "locality_order: null operand");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    unsigned char *ws = static_cast<unsigned char *>(workspace);
    const size_t sort_bytes = std::max(sort_temp_bytes(num_nodes), scan_temp_bytes(num_nodes));
    const size_t vec = align_up(sizeof(int32_t) * (size_t)num_nodes);
    void *sort_temp = ws;
    int32_t *lab_a = reinterpret_cast<int32_t *>(ws + align_up(sort_bytes));
    int32_t *lab_b = reinterpret_cast<int32_t *>(ws + align_up(sort_bytes) + vec);
    uint32_t *keys_in = reinterpret_cast<uint32_t *>(ws + align_up(sort_bytes) + 2 * vec);
    uint32_t *keys_out = reinterpret_cast<uint32_t *>(ws + align_up(sort_bytes) + 3 * vec);
    int32_t *order_tmp = reinterpret_cast<int32_t *>(ws + align_up(sort_bytes) + 4 * vec);
    const unsigned ngrid = grid_for(num_nodes);
    const unsigned rows_grid = (unsigned)((num_nodes + 255) / 256);

    int rc = E3J_AMD_OK;
    const int32_t *listed = order;  // where the order stands before the long rows are dealt
    // Levels: after 1, 2, 4, 8, ... sweeps the labels name ever larger clusters.  The order is
    // refined from the finest level to the coarsest with stable sorts, so the coarsest clusters
    // are contiguous and, inside them, the finer ones.
    int done = 0;
    int label_bits = 1;  // labels are node ids: the sort passes stop at their highest bit
    while (label_bits < 32 && ((int64_t)1 << label_bits) < (int64_t)num_nodes) label_bits++;
    const unsigned label_grid = (unsigned)(((int64_t)num_nodes * kLabelLanes + 255) / 256);
    const bool two_levels = rounds == 2 && 2 * label_bits <= 32;
    if (two_levels) {
        // the two levels in one sort: same order as the two stable sorts below, half the passes
        hipLaunchKernelGGL(min_label_kernel, dim3(label_grid), dim3(256), 0, stream, other, row_ptr, num_nodes,
                           static_cast<const int32_t *>(nullptr), lab_b);
        hipLaunchKernelGGL(min_label_kernel, dim3(label_grid), dim3(256), 0, stream, other, row_ptr, num_nodes,
                           lab_b, lab_a);
        hipLaunchKernelGGL(two_level_keys_kernel, dim3(rows_grid), dim3(256), 0, stream, lab_a, lab_b, num_nodes,
                           label_bits, keys_in, order);
        rc = check_hip(hipGetLastError(), "locality_order sweeps");
        if (rc) return rc;
        size_t temp_bytes = sort_bytes;
        rc = check_hip(hipcub::DeviceRadixSort::SortPairs(sort_temp, temp_bytes, keys_in, keys_out, order, order_tmp,
                                                          (int)num_nodes, 0, 2 * label_bits, stream),
                       "locality_order sort");
        if (rc) return rc;
        listed = order_tmp;
        rounds = 0;  // done: skip the level loop
    } else {
        hipLaunchKernelGGL(iota_kernel, dim3(ngrid), dim3(256), 0, stream, lab_a, (int64_t)num_nodes);
        hipLaunchKernelGGL(iota_kernel, dim3(ngrid), dim3(256), 0, stream, order, (int64_t)num_nodes);
        rc = check_hip(hipGetLastError(), "locality_order init");
        if (rc) return rc;
    }
    for (int level = 1; level <= rounds; level *= 2) {
        for (; done < level; done++) {
            hipLaunchKernelGGL(min_label_kernel, dim3(label_grid), dim3(256), 0, stream, other, row_ptr,
                               num_nodes, lab_a, lab_b);
            int32_t *t = lab_a; lab_a = lab_b; lab_b = t;
        }
        hipLaunchKernelGGL(gather_kernel, dim3(ngrid), dim3(256), 0, stream, lab_a, order,
                           reinterpret_cast<int32_t *>(keys_in), (int64_t)num_nodes);
        rc = check_hip(hipGetLastError(), "locality_order sweep");
        if (rc) return rc;
        size_t temp_bytes = sort_bytes;
        rc = check_hip(hipcub::DeviceRadixSort::SortPairs(sort_temp, temp_bytes, keys_in, keys_out, order,
                                                          order_tmp, (int)num_nodes, 0, label_bits, stream),
                       "locality_order sort");
        if (rc) return rc;
        hipLaunchKernelGGL(copy_i32_kernel, dim3(ngrid), dim3(256), 0, stream, order_tmp, order,
                           (int64_t)num_nodes);
    }
    // long rows to the fronts of the eighths of the list
    int32_t *flags = reinterpret_cast<int32_t *>(keys_in), *rank = reinterpret_cast<int32_t *>(keys_out);
    hipLaunchKernelGGL(long_row_flags_kernel, dim3(rows_grid), dim3(256), 0, stream, listed, row_ptr, num_nodes,
                       flags);
    rc = check_hip(hipGetLastError(), "locality_order flags");
    if (rc) return rc;
    size_t scan_bytes = sort_bytes;
    rc = check_hip(hipcub::DeviceScan::InclusiveSum(sort_temp, scan_bytes, flags, rank, num_nodes, stream),
                   "locality_order scan");
    if (rc) return rc;
    if (listed == order_tmp) {  // dealt straight into the result
        hipLaunchKernelGGL(deal_long_rows_kernel, dim3(rows_grid), dim3(256), 0, stream, listed, flags, rank,
                           num_nodes, order);
    } else {
        hipLaunchKernelGGL(deal_long_rows_kernel, dim3(rows_grid), dim3(256), 0, stream, listed, flags, rank,
                           num_nodes, order_tmp);
        hipLaunchKernelGGL(copy_i32_kernel, dim3(ngrid), dim3(256), 0, stream, order_tmp, order,
                           (int64_t)num_nodes);
    }
    return check_hip(hipGetLastError(), "locality_order");
}

int64_t e3j_amd_tile_schedule_num_work(int32_t num_nodes, int64_t num_edges, int32_t tile_rows,
                                       int32_t max_work_edges) {
    if (num_nodes < 0 || num_edges < 0 || tile_rows < 1 || max_work_edges < 1) return 0;
    const int64_t tiles = ((int64_t)num_nodes + tile_rows - 1) / tile_rows;
    return tiles + num_edges / max_work_edges;  // sum over tiles of max(1, ceil(count / max)) at most
}

size_t e3j_amd_tile_schedule_workspace_bytes(int32_t num_nodes, int64_t num_edges, int32_t tile_rows) {
    if (num_nodes < 0 || num_edges < 0 || tile_rows < 1) return 0;
    (void)num_edges;
    return TileWorkspace(num_nodes, tile_rows).total + 256;
}

int e3j_amd_tile_schedule_build(const int32_t *other, const int32_t *row_ptr, const int32_t *edge_perm,
                                const int32_t *row_order, int32_t num_nodes, int64_t num_edges,
                                int32_t tile_rows, int32_t max_work_edges, int32_t *work,
                                int32_t *t_sender, int32_t *t_edge, int32_t *t_local, void *workspace,
                                void *stream_) {
    if (num_nodes < 0 || num_edges < 0 || num_edges > 0x7fffffffLL || tile_rows < 1 || tile_rows > 65535 ||
        max_work_edges < 1)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "tile_schedule_build: bad sizes");
    if (num_nodes == 0) return E3J_AMD_OK;
    if (row_ptr == nullptr || work == nullptr || workspace == nullptr ||
        (num_edges > 0 && (other == nullptr || t_sender == nullptr || t_edge == nullptr || t_local == nullptr)))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "tile_schedule_build: null operand");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    unsigned char *ws = static_cast<unsigned char *>(workspace);
    ws += (256 - reinterpret_cast<uintptr_t>(ws) % 256) % 256;
    const TileWorkspace w(num_nodes, tile_rows);
    uint64_t *packed = reinterpret_cast<uint64_t *>(ws + w.packed);
    const int num_tiles = (num_nodes + tile_rows - 1) / tile_rows;
    const unsigned tiles_grid = (unsigned)((num_tiles + 255) / 256);

    hipLaunchKernelGGL(tile_count_kernel, dim3(tiles_grid), dim3(256), 0, stream, row_order, row_ptr, num_nodes,
                       tile_rows, num_tiles, max_work_edges, packed);
    int rc = check_hip(hipGetLastError(), "tile schedule counts");
    if (rc) return rc;
    size_t temp_bytes = w.temp_bytes;
    rc = check_hip(hipcub::DeviceScan::InclusiveSum(ws + w.temp, temp_bytes, packed, packed, num_tiles + 1, stream),
                   "tile schedule scan");
    if (rc) return rc;
    hipLaunchKernelGGL(tile_work_kernel, dim3(tiles_grid), dim3(256), 0, stream, packed, num_tiles, max_work_edges,
                       work);
    rc = check_hip(hipGetLastError(), "tile schedule work");
    if (rc || num_edges == 0) return rc;
    // the lists: one wave per tile sorts its positions by sender in LDS
    hipLaunchKernelGGL(tile_lists_kernel, dim3((unsigned)((num_tiles + 3) / 4)), dim3(256), 0, stream, other, row_ptr,
                       edge_perm, row_order, packed, num_nodes, num_edges, tile_rows, num_tiles, t_sender, t_edge,
                       t_local);
    return check_hip(hipGetLastError(), "tile schedule lists");
}

int e3j_amd_sort_edges(const int32_t *key, const int32_t *other, int64_t num_edges,
                       int32_t num_nodes, int32_t *perm, int32_t *other_sorted, int32_t *row_ptr,
                       void *workspace, void *stream_) {
    if (num_nodes < 0 || num_edges < 0 || num_edges > 0x7fffffffLL)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "sort_edges: bad sizes");
    if (row_ptr == nullptr || workspace == nullptr ||
        (num_edges > 0 && (key == nullptr || other == nullptr || perm == nullptr || other_sorted == nullptr)))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "sort_edges: null operand");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    unsigned char *ws = static_cast<unsigned char *>(workspace);
    const size_t scan_bytes = scan_temp_bytes(num_nodes);
    const size_t sort_bytes = sort_temp_bytes(num_edges);
    void *scan_temp = ws;
    void *sort_temp = ws + align_up(scan_bytes);
    uint32_t *keys_out = reinterpret_cast<uint32_t *>(ws + align_up(scan_bytes) + align_up(sort_bytes));
    int32_t *iota = reinterpret_cast<int32_t *>(reinterpret_cast<unsigned char *>(keys_out) +
                                                align_up(sizeof(int32_t) * (size_t)num_edges));
    int rc = row_ptr_impl(key, num_edges, num_nodes, row_ptr, scan_temp, scan_bytes, stream);
    if (rc || num_edges == 0) return rc;
    hipLaunchKernelGGL(iota_kernel, dim3(grid_for(num_edges)), dim3(256), 0, stream, iota, num_edges);
    rc = check_hip(hipGetLastError(), "sort iota launch");
    if (rc) return rc;
    size_t temp_bytes = sort_bytes;
    rc = check_hip(hipcub::DeviceRadixSort::SortPairs(sort_temp, temp_bytes,
                                                      reinterpret_cast<const uint32_t *>(key), keys_out,
                                                      iota, perm, (int)num_edges, 0, 32, stream),
                   "edge sort");
    if (rc) return rc;
    hipLaunchKernelGGL(gather_kernel, dim3(grid_for(num_edges)), dim3(256), 0, stream, other, perm,
                       other_sorted, num_edges);
    return check_hip(hipGetLastError(), "sort gather launch");
}

}  // extern "C"
