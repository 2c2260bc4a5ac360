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

// ---------------------------------------------------------------------------
// The mixing itself in one launch (float32, 64 or 128 channels): no regrouped copies, no library
// calls.  A wave takes 32 nodes and one output row (degree l, component m) and runs
// v_mfma_f32_32x32x2_f32 with the nodes as rows: lane t holds, for node t % 32, the 32 consecutive
// channels 32 (t / 32) .. + 31 of a source row (one contiguous 128-byte read per lane: whole
// lines of the (N, Z, K) array), and step s of the product takes channel 32 (t / 32) + s from
// every lane, which is the layout of the instruction's first operand when its two summed
// indices are read as "channel s of the lower / of the upper half"; the second operand is the
// matching row of the weight, 32 consecutive output channels per half wave (served by the
// caches: a degree's weights are at most 7 x 16 KB at 64 channels).  Forward: the products of
// the mul copies of the degree accumulate into one output row.  Backward (weights transposed by
// the caller): the cotangent row is read once and gives one product per copy.
typedef float f32x16 __attribute__((ext_vector_type(16)));
constexpr int kMixDegrees = 8;
struct MixShape {
    int32_t degrees;
    int32_t mul[kMixDegrees], dim[kMixDegrees];
};

template <int K, bool kTranspose>
__global__ __launch_bounds__(256) void channel_mix_kernel(const float *__restrict__ src, float *__restrict__ dst,
                                                          const float *__restrict__ w, int64_t num_nodes,
                                                          MixShape shape, int32_t rows_plain, int32_t rows_mixed) {
    constexpr int KC = K / 64, KT = K / 32;   // chunks of 64 summed channels, tiles of 32 output channels
    const int lane = threadIdx.x, r = lane & 31, h = lane >> 5;
    const int64_t item = (int64_t)blockIdx.x * blockDim.y + threadIdx.y;
    const int64_t tiles = (num_nodes + 31) / 32;
    if (item >= tiles * rows_mixed) return;  // (uniform per wave)
    const int64_t tile = item / rows_mixed;
    const int xr = (int)(item % rows_mixed);
    // the degree and component of mixed row xr, the first plain row and the first weight of the degree
    int l = 0, zbase = 0, xbase = 0;
    int64_t wbase = 0;
    while (l < shape.degrees - 1 && xr >= xbase + shape.dim[l]) {
        zbase += shape.mul[l] * shape.dim[l];
        xbase += shape.dim[l];
        wbase += (int64_t)shape.mul[l] * K * K;
        l++;
    }
    const int m = xr - xbase, mul = shape.mul[l], dim = shape.dim[l];
    const int64_t node = tile * 32 + r;
    const int64_t node_read = node < num_nodes ? node : num_nodes - 1;  // (lanes past the end read the last node)
    // plain rows (N, rows_plain, K): the convolution's output / its cotangent; mixed rows (N, rows_mixed, K)
    const float *plain_in = src + node_read * ((int64_t)rows_plain * K) + 32 * h;
    const float *mixed_in = src + (node_read * rows_mixed + xr) * (int64_t)K + 32 * h;
    auto load_row = [&](const float *p, float (&a)[32]) {
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const float4 v = *reinterpret_cast<const float4 *>(p + 4 * q);
            a[4 * q] = v.x; a[4 * q + 1] = v.y; a[4 * q + 2] = v.z; a[4 * q + 3] = v.w;
        }
    };
    auto store_tile = [&](const f32x16 (&acc)[KT], float *row0, int64_t node_stride) {
        // register v of lane t: node 8 (v / 4) + 4 (t / 32) + v % 4 of the tile, output channel t % 32 of tile ct
#pragma unroll
        for (int ct = 0; ct < KT; ct++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int64_t n = tile * 32 + 8 * (v / 4) + 4 * h + v % 4;
                if (n < num_nodes) row0[n * node_stride + ct * 32 + r] = acc[ct][v];
            }
        }
    };
    f32x16 acc[KT];
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // One chunk of 64 summed channels: the weight rows of a block of steps are read together (a
    // read next to each product would leave the matrix unit waiting for it), then the products run.
    constexpr int SB = K == 64 ? 32 : 16;  // steps per block: SB * KT weight registers
    auto chunk = [&](const float (&a)[32], const float *wk) {
#pragma unroll
        for (int s0 = 0; s0 < 32; s0 += SB) {
            float b[SB][KT];
#pragma unroll
            for (int s = 0; s < SB; s++) {
#pragma unroll
                for (int ct = 0; ct < KT; ct++) b[s][ct] = wk[(int64_t)(s0 + s) * K + ct * 32];
            }
            asm volatile("" ::: "memory");  // (the reads above are issued before the products below)
#pragma unroll
            for (int s = 0; s < SB; s++) {
#pragma unroll
                for (int ct = 0; ct < KT; ct++)
                    acc[ct] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s0 + s], b[s][ct], acc[ct], 0, 0, 0);
            }
        }
    };
    if (!kTranspose) {
#pragma unroll
        for (int ct = 0; ct < KT; ct++) acc[ct] = zero;
        // (u, chunk) pairs in one sequence, the source row of the next pair read while the products of
        // the one at hand run
        const int pairs = mul * KC;
        float a[32], ahead[32];
        load_row(plain_in + (int64_t)(zbase + m) * K, a);
        for (int q = 0; q < pairs; q++) {
            const int u = q / KC, kc = q % KC;
            if (q + 1 < pairs) {
                const int un = (q + 1) / KC, kn = (q + 1) % KC;
                load_row(plain_in + (int64_t)(zbase + un * dim + m) * K + kn * 64, ahead);
            }
            chunk(a, w + wbase + (int64_t)u * K * K + (int64_t)(kc * 64 + 32 * h) * K + r);
#pragma unroll
            for (int s = 0; s < 32; s++) a[s] = ahead[s];
        }
        store_tile(acc, dst + (int64_t)xr * K, (int64_t)rows_mixed * K);
    } else {
        float a[KC][32];
#pragma unroll
        for (int kc = 0; kc < KC; kc++) load_row(mixed_in + kc * 64, a[kc]);
        for (int u = 0; u < mul; u++) {
            const float *wu = w + wbase + (int64_t)u * K * K;  // (transposed: [output channel c of the mixing][k])
#pragma unroll
            for (int ct = 0; ct < KT; ct++) acc[ct] = zero;
#pragma unroll
            for (int kc = 0; kc < KC; kc++) chunk(a[kc], wu + (int64_t)(kc * 64 + 32 * h) * K + r);
            store_tile(acc, dst + (int64_t)(zbase + u * dim + m) * K, (int64_t)rows_plain * K);
        }
    }
}

template <int K>
int launch_mix(const float *src, float *dst, const float *w, int64_t num_nodes, const MixShape &shape,
               int rows_plain, int rows_mixed, bool transpose, hipStream_t stream) {
    constexpr int kWavesPerBlock = 4;
    const int64_t items = (num_nodes + 31) / 32 * rows_mixed;
    const int64_t blocks = (items + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "channel_mix: too many nodes for one launch");
    if (transpose)
        hipLaunchKernelGGL((channel_mix_kernel<K, true>), dim3((unsigned)blocks), dim3(kWave, kWavesPerBlock), 0, stream,
                           src, dst, w, num_nodes, shape, rows_plain, rows_mixed);
    else
        hipLaunchKernelGGL((channel_mix_kernel<K, false>), dim3((unsigned)blocks), dim3(kWave, kWavesPerBlock), 0, stream,
                           src, dst, w, num_nodes, shape, rows_plain, rows_mixed);
    return check_hip(hipGetLastError(), "channel_mix launch");
}

}  // namespace
}  // namespace e3j_amd

extern "C" int e3j_amd_channel_mix(const void *src, void *dst, const void *weights, int64_t num_nodes,
                                   int32_t channels, int32_t num_degrees, const int32_t *mul, const int32_t *dim,
                                   int32_t transpose, void *stream) {
    using namespace e3j_amd;
    if (num_nodes < 0 || num_degrees < 1 || num_degrees > kMixDegrees || mul == nullptr || dim == nullptr)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "channel_mix: 1 to 8 degrees, their multiplicities and dimensions");
    if (channels != 64 && channels != 128)
        return set_error(E3J_AMD_UNIMPLEMENTED, "channel_mix: 64 or 128 channels (other counts: e3j_amd_rows_regroup "
                                                "around matrix products)");
    MixShape shape;
    shape.degrees = num_degrees;
    int rows_plain = 0, rows_mixed = 0;
    for (int l = 0; l < kMixDegrees; l++) {
        shape.mul[l] = l < num_degrees ? mul[l] : 0;
        shape.dim[l] = l < num_degrees ? dim[l] : 0;
        if (l < num_degrees && (mul[l] < 1 || dim[l] < 1))
            return set_error(E3J_AMD_INVALID_ARGUMENT, "channel_mix: multiplicities and dimensions must be >= 1");
        rows_plain += shape.mul[l] * shape.dim[l];
        rows_mixed += shape.dim[l];
    }
    if (num_nodes == 0) return E3J_AMD_OK;
    if (src == nullptr || dst == nullptr || weights == nullptr)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "channel_mix: null operand");
    if (reinterpret_cast<uintptr_t>(src) % 16 != 0 || reinterpret_cast<uintptr_t>(dst) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(weights) % 16 != 0)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "channel_mix: operands must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const float *a = static_cast<const float *>(src), *wt = static_cast<const float *>(weights);
    float *out = static_cast<float *>(dst);
    if (channels == 64) return launch_mix<64>(a, out, wt, num_nodes, shape, rows_plain, rows_mixed, transpose != 0, s);
    return launch_mix<128>(a, out, wt, num_nodes, shape, rows_plain, rows_mixed, transpose != 0, s);
}

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
