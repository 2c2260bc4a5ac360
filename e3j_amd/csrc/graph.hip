// Graph preparation on the device: CSR row pointers and the stable edge sort
// behind the unsorted (GraphOrdering NONE) path and the transposed adjacency.
//
// Restates GraphCSR (src/e3j/data/graph.py:49-73): row_ptr = [0] +
// cumsum(bincount(key, length = N)) with out-of-range keys dropped, and
// sort = stable argsort by key.  The sort is rocPRIM's radix sort (via hipCUB)
// on unsigned keys, so sentinel and negative keys land after every live row.

#include <hipcub/hipcub.hpp>

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
__global__ void min_label_kernel(const int32_t *__restrict__ other,
                                 const int32_t *__restrict__ row_ptr, int num_nodes,
                                 const int32_t *__restrict__ cur, int32_t *__restrict__ next) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= num_nodes) return;
    int best = cur[n];
    for (int e = row_ptr[n]; e < row_ptr[n + 1]; e++) {
        const int m = other[e];
        if ((unsigned)m < (unsigned)num_nodes) best = min(best, cur[m]);
    }
    next[n] = best;
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

}  // namespace

int launch_live_keys(const int32_t *other, const int32_t *row_ptr, int32_t num_nodes,
                     int64_t num_edges, int32_t *keys, hipStream_t stream) {
    if (num_edges == 0) return E3J_AMD_OK;
    hipLaunchKernelGGL(live_keys_kernel, dim3(grid_for(num_edges)), dim3(256), 0, stream, other, row_ptr,
                       num_nodes, num_edges, keys);
    return check_hip(hipGetLastError(), "live keys launch");
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
    if (num_nodes < 0 || num_edges < 0 || num_edges > 0x7fffffffLL)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "csr_row_ptr: bad sizes");
    if (row_ptr == nullptr || workspace == nullptr || (num_edges > 0 && key == nullptr))
        return set_error(E3J_AMD_INVALID_ARGUMENT, "csr_row_ptr: null operand");
    return row_ptr_impl(key, num_edges, num_nodes, row_ptr, workspace, scan_temp_bytes(num_nodes),
                        static_cast<hipStream_t>(stream_));
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

    hipLaunchKernelGGL(iota_kernel, dim3(ngrid), dim3(256), 0, stream, lab_a, (int64_t)num_nodes);
    hipLaunchKernelGGL(iota_kernel, dim3(ngrid), dim3(256), 0, stream, order, (int64_t)num_nodes);
    int rc = check_hip(hipGetLastError(), "locality_order init");
    if (rc) return rc;
    // Levels: after 1, 2, 4, 8, ... sweeps the labels name ever larger clusters.  The order is
    // refined from the finest level to the coarsest with stable sorts, so the coarsest clusters
    // are contiguous and, inside them, the finer ones.
    int done = 0;
    for (int level = 1; level <= rounds; level *= 2) {
        for (; done < level; done++) {
            hipLaunchKernelGGL(min_label_kernel, dim3(rows_grid), dim3(256), 0, stream, other, row_ptr,
                               num_nodes, lab_a, lab_b);
            int32_t *t = lab_a; lab_a = lab_b; lab_b = t;
        }
        hipLaunchKernelGGL(gather_kernel, dim3(ngrid), dim3(256), 0, stream, lab_a, order,
                           reinterpret_cast<int32_t *>(keys_in), (int64_t)num_nodes);
        rc = check_hip(hipGetLastError(), "locality_order sweep");
        if (rc) return rc;
        size_t temp_bytes = sort_bytes;
        rc = check_hip(hipcub::DeviceRadixSort::SortPairs(sort_temp, temp_bytes, keys_in, keys_out, order,
                                                          order_tmp, (int)num_nodes, 0, 32, stream),
                       "locality_order sort");
        if (rc) return rc;
        hipLaunchKernelGGL(copy_i32_kernel, dim3(ngrid), dim3(256), 0, stream, order_tmp, order,
                           (int64_t)num_nodes);
    }
    // long rows to the fronts of the eighths of the list
    int32_t *flags = reinterpret_cast<int32_t *>(keys_in), *rank = reinterpret_cast<int32_t *>(keys_out);
    hipLaunchKernelGGL(long_row_flags_kernel, dim3(rows_grid), dim3(256), 0, stream, order, row_ptr, num_nodes,
                       flags);
    rc = check_hip(hipGetLastError(), "locality_order flags");
    if (rc) return rc;
    size_t scan_bytes = sort_bytes;
    rc = check_hip(hipcub::DeviceScan::InclusiveSum(sort_temp, scan_bytes, flags, rank, num_nodes, stream),
                   "locality_order scan");
    if (rc) return rc;
    hipLaunchKernelGGL(deal_long_rows_kernel, dim3(rows_grid), dim3(256), 0, stream, order, flags, rank,
                       num_nodes, order_tmp);
    hipLaunchKernelGGL(copy_i32_kernel, dim3(ngrid), dim3(256), 0, stream, order_tmp, order,
                       (int64_t)num_nodes);
    return check_hip(hipGetLastError(), "locality_order");
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
