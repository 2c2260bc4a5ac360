// Row regrouping around the per-degree channel mixing that follows a convolution.
//
// A convolution writes node rows (N, Z, K): for every output degree l its `mul` copies of 2l + 1
// components, rows base_l + u * dim_l + m.  The linear layer after it mixes copies and channels
// per degree, x'[n, m, c] = sum_{u, k} out[n, base_l + u * dim_l + m, k] W_l[u, k, c]: one plain
// matrix product per degree once the rows are regrouped as A_l[(n, m), (u, k)].  The kernel below
// moves every row of K values between the two arrangements in one launch, in whole 16-byte
// pieces, driven by two numbers per row: regrouped address of (n, i, k) = row_base[i] +
// n * row_stride[i] + k.  The products themselves are library matrix products (the one dense
// contraction of this step; src/e3j/core/linear.py of the reference does the same with an einsum).
// The backward pass uses the same kernel in the other direction, so the cotangent rows are
// written once (no zero fill, no additions of per-degree slices).
#include "common.h"

namespace e3j_amd {
namespace {

// VEC: elements per 16-byte piece
template <typename T, int VEC, bool kGather>
__global__ void rows_regroup_kernel(const T *__restrict__ src, T *__restrict__ dst, int64_t num_nodes,
                                    int32_t rows, int32_t channels, const int64_t *__restrict__ row_base,
                                    const int64_t *__restrict__ row_stride) {
    struct alignas(16) Piece { T v[VEC]; };
    const int32_t pieces = channels / VEC;
    const int64_t total = num_nodes * rows * pieces;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
        const int32_t q = (int32_t)(t % pieces);
        const int64_t row = t / pieces;  // n * rows + i
        const int32_t i = (int32_t)(row % rows);
        const int64_t n = row / rows;
        const int64_t plain = row * channels + (int64_t)q * VEC;
        const int64_t grouped = row_base[i] + n * row_stride[i] + (int64_t)q * VEC;
        if (kGather)   // plain (N, rows, K) -> regrouped
            *reinterpret_cast<Piece *>(dst + grouped) = *reinterpret_cast<const Piece *>(src + plain);
        else           // regrouped -> plain
            *reinterpret_cast<Piece *>(dst + plain) = *reinterpret_cast<const Piece *>(src + grouped);
    }
}

template <typename T>
int launch(const void *src, void *dst, int64_t num_nodes, int32_t rows, int32_t channels,
           const int64_t *row_base, const int64_t *row_stride, bool gather, hipStream_t stream) {
    constexpr int VEC = 16 / sizeof(T);
    const int64_t total = num_nodes * rows * (channels / VEC);
    const unsigned blocks = (unsigned)std::min<int64_t>((total + 255) / 256, 1 << 20);
    if (gather)
        hipLaunchKernelGGL((rows_regroup_kernel<T, VEC, true>), dim3(blocks), dim3(256), 0, stream,
                           static_cast<const T *>(src), static_cast<T *>(dst), num_nodes, rows, channels, row_base,
                           row_stride);
    else
        hipLaunchKernelGGL((rows_regroup_kernel<T, VEC, false>), dim3(blocks), dim3(256), 0, stream,
                           static_cast<const T *>(src), static_cast<T *>(dst), num_nodes, rows, channels, row_base,
                           row_stride);
    return check_hip(hipGetLastError(), "rows_regroup launch");
}

}  // namespace
}  // namespace e3j_amd

extern "C" int e3j_amd_rows_regroup(const void *src, void *dst, int64_t num_nodes, int32_t rows, int32_t channels,
                                    const int64_t *row_base, const int64_t *row_stride, int32_t to_plain,
                                    int32_t val_dtype, void *stream) {
    using namespace e3j_amd;
    if (num_nodes < 0 || rows < 0 || channels < 0)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "rows_regroup: negative size");
    if (num_nodes == 0 || rows == 0 || channels == 0) return E3J_AMD_OK;
    if (src == nullptr || dst == nullptr || row_base == nullptr || row_stride == nullptr)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "rows_regroup: null operand");
    const int vec = val_dtype == E3J_AMD_F64 ? 2 : 4;
    if (val_dtype != E3J_AMD_F32 && val_dtype != E3J_AMD_F64)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "rows_regroup: unsupported value dtype");
    if (channels % vec != 0 || reinterpret_cast<uintptr_t>(src) % 16 != 0 || reinterpret_cast<uintptr_t>(dst) % 16 != 0)
        return set_error(E3J_AMD_INVALID_ARGUMENT,
                         "rows_regroup: rows are moved in 16-byte pieces (channels a multiple of 4 floats / 2 "
                         "doubles, 16-byte aligned operands, row_base and row_stride multiples of that)");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (val_dtype == E3J_AMD_F32)
        return launch<float>(src, dst, num_nodes, rows, channels, row_base, row_stride, to_plain == 0, s);
    return launch<double>(src, dst, num_nodes, rows, channels, row_base, row_stride, to_plain == 0, s);
}
