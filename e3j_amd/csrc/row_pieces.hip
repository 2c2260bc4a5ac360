// Long rows of the forward pass, summed in a fixed order.  The pieces of a row longer than
// row_cap are summed by waves of their own (a second launch of the forward kernel over the list of
// pieces).  Instead of adding them to the output row with float atomics, whose order changes from
// run to run, every piece gets a row of a scratch array (the launch names the piece's own number
// as its "row" and adds into a zeroed row: one addition per element), and a last kernel adds the
// rows of a receiver's pieces to its output row in the order of their positions.  No counterpart
// in the reference, whose forward kernel walks the edges of a receiver one after another in one
// block (lib/e3j_ops/cuda/convolution/fwd.cuh:346-363) and is run-to-run reproducible for that
// reason (tests/test_ops/test_convolution_op.py:322-342); this keeps that property while sharing the row.

#include "row_pieces.h"

#include <algorithm>

#include "common.h"

namespace e3j_amd {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// block q: the numbered list entry of piece q and its zeroed row
__global__ __launch_bounds__(256) void prepare_partials_kernel(const int32_t *__restrict__ segments, int max_segments,
                                                               int64_t row_floats, float *__restrict__ partials,
                                                               int32_t *__restrict__ list) {
    const int count = min(segments[0], max_segments);
    if (blockIdx.x == 0 && threadIdx.x < 4) list[threadIdx.x] = threadIdx.x == 0 ? count : 0;
    const int q = blockIdx.x;
    if (q >= count) return;
    if (threadIdx.x == 0) {
        list[4 + 3 * q] = q;
        list[5 + 3 * q] = segments[5 + 3 * q];
        list[6 + 3 * q] = segments[6 + 3 * q];
    }
    float *row = partials + (int64_t)q * row_floats;
    for (int64_t t = threadIdx.x; t < row_floats; t += blockDim.x) row[t] = 0.f;
}

// Block (g, chunk) walks the pieces g, g + gridDim.x, ...: where a piece is the first listed piece of
// its row, the rows of all pieces of that row are added to 64 floats of the output row.  The four
// waves of the block each sum a quarter of the pieces (contiguous ranges, sixteen loads in flight),
// one after another in list order; the four sums are then added in order: the grouping is fixed by
// the list, so are the bits.  (The grid does not grow with the bound on the number of pieces: most
// graphs have none, and a launch of a block per possible piece and chunk would cost more than the
// sums.)
constexpr int kCombineWaves = 4;
constexpr int kCombineStride = 32;
__global__ __launch_bounds__(kWave *kCombineWaves) void combine_pieces_kernel(
    const int32_t *__restrict__ segments, const int32_t *__restrict__ row_ptr, int max_segments, int row_piece,
    int64_t row_floats, const float *__restrict__ partials, float *__restrict__ out) {
    __shared__ float sums[kCombineWaves][kWave];
    __shared__ int found[kWave * kCombineWaves][2], num_found;
    const int count = min(segments[0], max_segments);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int64_t t = (int64_t)blockIdx.y * kWave + lane;
    const bool inside = t < row_floats;
    const int64_t tt = inside ? t : 0;
    // the pieces g, g + gridDim.x, ... of this block, a thread each: which of them begin a row's run
    for (int base = blockIdx.x; base < count; base += gridDim.x * blockDim.x) {
        if (threadIdx.x == 0) num_found = 0;
        __syncthreads();
        const int q = base + (int)threadIdx.x * (int)gridDim.x;
        if (q < count) {
            const int r = segments[4 + 3 * q], b = segments[5 + 3 * q];
            const int begin = row_ptr[r], end = row_ptr[r + 1];
            if (b == begin + row_piece) {  // the first listed piece of row r
                const int at = atomicAdd(&num_found, 1);
                found[at][0] = q;
                found[at][1] = min((end - begin - 1) / row_piece, count - q);
            }
        }
        __syncthreads();
        const int n = num_found;
        for (int f = 0; f < n; f++) {
            const int first_piece = found[f][0], pieces = found[f][1];
            const int r = segments[4 + 3 * first_piece];
            const int first = first_piece + (int)((int64_t)pieces * wave / kCombineWaves);
            const int end = first_piece + (int)((int64_t)pieces * (wave + 1) / kCombineWaves);
            float sum = 0.f;
            int k = first;
            for (; k + 16 <= end; k += 16) {
                float v[16];
#pragma unroll
                for (int u = 0; u < 16; u++) v[u] = partials[(int64_t)(k + u) * row_floats + tt];
#pragma unroll
                for (int u = 0; u < 16; u++) sum += v[u];
            }
            for (; k < end; k++) sum += partials[(int64_t)k * row_floats + tt];
            sums[wave][lane] = sum;
            __syncthreads();
            if (wave == 0 && inside) {
                float total = out[(int64_t)r * row_floats + t];
#pragma unroll
                for (int w = 0; w < kCombineWaves; w++) total += sums[w][lane];
                out[(int64_t)r * row_floats + t] = total;
            }
            __syncthreads();  // `sums` is free for the next row
        }
    }
}

}  // namespace

size_t row_partials_bytes(int64_t max_segments, int64_t row_floats) {
    if (max_segments <= 0 || row_floats <= 0) return 0;
    return sizeof(float) * (size_t)max_segments * (size_t)row_floats + sizeof(int32_t) * (4 + 3 * (size_t)max_segments);
}

int32_t *row_partials_list(float *partials, int64_t max_segments, int64_t row_floats) {
    return reinterpret_cast<int32_t *>(partials + max_segments * row_floats);
}

int launch_prepare_partials(const int32_t *segments, int32_t max_segments, int64_t row_floats, float *partials,
                            hipStream_t stream) {
    if (max_segments <= 0) return E3J_AMD_OK;
    hipLaunchKernelGGL(prepare_partials_kernel, dim3((unsigned)max_segments), dim3(256), 0, stream, segments,
                       max_segments, row_floats, partials, row_partials_list(partials, max_segments, row_floats));
    return check_hip(hipGetLastError(), "row pieces: prepare");
}

int launch_combine_pieces(const int32_t *segments, const int32_t *row_ptr, int32_t max_segments, int32_t row_piece,
                          int64_t row_floats, const float *partials, float *out, hipStream_t stream) {
    if (max_segments <= 0) return E3J_AMD_OK;
    const int64_t chunks = (row_floats + kWave - 1) / kWave;
    if (chunks > 65535) return set_error(E3J_AMD_INVALID_ARGUMENT, "row pieces: output row too long");
    hipLaunchKernelGGL(combine_pieces_kernel, dim3((unsigned)std::min(max_segments, kCombineStride), (unsigned)chunks),
                       dim3(kWave * kCombineWaves), 0, stream, segments, row_ptr, max_segments, row_piece, row_floats,
                       partials, out);
    return check_hip(hipGetLastError(), "row pieces: combine");
}

}  // namespace e3j_amd
