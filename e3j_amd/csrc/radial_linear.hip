// Last layer of the radial network that produces the per-edge, per-path weights of the
// convolution: s (E, N) = h (E, H) W (H, N) with N = paths * channels, float32, and the two
// products of its backward pass, dW = h^T ds and (from H = 64 on) dh = ds W^T.  The one dense
// contraction next to the convolution: it runs on the matrix cores.  H is small (8..128), so each
// pass is bound by the E * N stream it writes or reads; the tilings keep that stream at whole
// 128-byte lines and everything else (h, W) in registers or LDS.
//
// Register layout of one 32x32x2 product D += A B on a 64-lane wave (g = lane / 32, c = lane % 32):
// a lane supplies A[c][g] and B[g][c] and holds D[8 * (v / 4) + 4 * g + v % 4][c] in element v of
// its sixteen accumulators.  Which two inner indices a product takes is free as long as A and
// B agree: product j of a lane half takes the inner index g * (inner / 2) + j, so the operands of a
// lane are contiguous in memory.

#include <initializer_list>

#include "common.h"

namespace e3j_amd {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kTile = 32;        // rows and columns of a matrix-core tile
constexpr int kWaves = 4;        // waves per block

// s = h W.  A block takes kWaves * R * 32 consecutive edges, keeps their rows of h in registers
// as A operands and walks the columns of W in tiles of 32 that all its waves share through LDS
// (double buffered: the next tile is fetched while the current one is multiplied).
template <int H, int R>
__global__ __launch_bounds__(kWave * kWaves) void radial_linear_fwd_kernel(
    const float *__restrict__ h, const float *__restrict__ w, float *__restrict__ s, int64_t num_edges, int n) {
    constexpr int HH = H / 2;                        // inner indices per lane half
    constexpr int PIECES = H * kTile / 4;            // 16-byte pieces of a W tile
    constexpr int PER_THREAD = (PIECES + kWave * kWaves - 1) / (kWave * kWaves);
    static_assert(H % 8 == 0 && H <= 128, "inner size: a multiple of 8 up to 128");
    __shared__ __attribute__((aligned(16))) float tile[2][H * kTile];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int g = lane / kTile, c = lane % kTile;
    const int64_t e0 = ((int64_t)blockIdx.x * kWaves + wave) * (kTile * R);

    float a[R][HH];
#pragma unroll
    for (int r = 0; r < R; r++) {
        int64_t row = e0 + r * kTile + c;
        if (row >= num_edges) row = num_edges - 1;  // rows past the end are computed and not stored
        const f32x4 *p = reinterpret_cast<const f32x4 *>(h + row * H + g * HH);
#pragma unroll
        for (int q = 0; q < HH / 4; q++) {
            const f32x4 v = __builtin_nontemporal_load(p + q);
            a[r][4 * q] = v.x; a[r][4 * q + 1] = v.y; a[r][4 * q + 2] = v.z; a[r][4 * q + 3] = v.w;
        }
    }

    f32x4 staged[PER_THREAD];
    auto fetch = [&](int t) {  // columns [32 t, 32 t + 32) of W into registers
#pragma unroll
        for (int i = 0; i < PER_THREAD; i++) {
            const int piece = i * kWave * kWaves + tid;
            if (PIECES % (kWave * kWaves) == 0 || piece < PIECES)
                staged[i] = *reinterpret_cast<const f32x4 *>(w + (int64_t)(piece / 8) * n + t * kTile + (piece % 8) * 4);
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; i++) {
            const int piece = i * kWave * kWaves + tid;
            if (PIECES % (kWave * kWaves) == 0 || piece < PIECES)
                *reinterpret_cast<f32x4 *>(&tile[buf][piece * 4]) = staged[i];
        }
    };
    const int tiles = n / kTile;
    fetch(0);
    commit(0);
    __syncthreads();
    for (int t = 0; t < tiles; t++) {
        if (t + 1 < tiles) fetch(t + 1);
        float b[HH];
#pragma unroll
        for (int j = 0; j < HH; j++) b[j] = tile[t & 1][(g * HH + j) * kTile + c];
        f32x16 d[R];
#pragma unroll
        for (int r = 0; r < R; r++) d[r] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < HH; j++) {  // the R row tiles side by side: independent accumulator chains
#pragma unroll
            for (int r = 0; r < R; r++) d[r] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[r][j], b[j], d[r], 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            float *out = s + (e0 + r * kTile + 4 * g) * n + t * kTile + c;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = 8 * (v / 4) + v % 4;
                if (e0 + r * kTile + 4 * g + row < num_edges) __builtin_nontemporal_store(d[r][v], out + (int64_t)row * n);
            }
        }
        if (t + 1 < tiles) commit((t + 1) & 1);
        __syncthreads();
    }
}

// Inner sizes of 64 and more: at the float32 rate of the matrix cores (64 flop per cycle and
// SIMD) the products themselves would take longer than the stream, so they run at the bfloat16
// rate (16 times that) on operands split three ways: x = x1 + x2 + x3 with x1 the upper 8
// mantissa bits, x2 the next 8 and x3 the last 8 (each a bfloat16, the sum exact), and
// x y = x1 y1 + (x1 y2 + x2 y1) + (x1 y3 + x2 y2 + x3 y1) + O(2^-24 x y): six products whose
// partial products are exact and whose sum is kept in float32 accumulators, i.e. the accuracy
// of a float32 product at 6/16 of its cost.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct Split3 {
    bf16x8 term[3];
};

// eight floats into their three bfloat16 parts (truncation keeps every part exact)
__device__ __forceinline__ Split3 split3(const float (&x)[8]) {
    Split3 out;
    float rest[8];
#pragma unroll
    for (int m = 0; m < 8; m++) rest[m] = x[m];
#pragma unroll
    for (int t = 0; t < 3; t++) {
        u32x4 packed;
#pragma unroll
        for (int m = 0; m < 8; m += 2) {
            const uint32_t lo = __float_as_uint(rest[m]) & 0xffff0000u, hi = __float_as_uint(rest[m + 1]) & 0xffff0000u;
            packed[m / 2] = (lo >> 16) | hi;
            rest[m] -= __uint_as_float(lo);
            rest[m + 1] -= __uint_as_float(hi);
        }
        out.term[t] = __builtin_bit_cast(bf16x8, packed);
    }
    return out;
}

// One 32x32x16 product takes sixteen inner indices; a lane (g, c) supplies eight of them for
// row (A) or column (B) c: block q of the inner dimension gives it the indices 16 q + 8 g + m.
template <int H, int R>
__global__ __launch_bounds__(kWave * kWaves) void radial_linear_fwd_split_kernel(
    const float *__restrict__ h, const float *__restrict__ w, float *__restrict__ s, int64_t num_edges, int n) {
    constexpr int Q = H / 16;                         // inner blocks
    constexpr int SLOTS = 2 * Q * kTile;              // (q, g, c) operand slots of a W tile: 8 values each
    constexpr int PER_THREAD = (SLOTS + kWave * kWaves - 1) / (kWave * kWaves);
    static_assert(H % 16 == 0, "whole inner blocks");
    __shared__ __attribute__((aligned(16))) bf16x8 tile[2][3][SLOTS];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int g = lane / kTile, c = lane % kTile;
    const int64_t e0 = ((int64_t)blockIdx.x * kWaves + wave) * (kTile * R);

    Split3 a[R][Q];
#pragma unroll
    for (int r = 0; r < R; r++) {
        int64_t row = e0 + r * kTile + c;
        if (row >= num_edges) row = num_edges - 1;  // rows past the end are computed and not stored
#pragma unroll
        for (int q = 0; q < Q; q++) {
            const f32x4 *p = reinterpret_cast<const f32x4 *>(h + row * H + q * 16 + g * 8);
            const f32x4 v0 = __builtin_nontemporal_load(p), v1 = __builtin_nontemporal_load(p + 1);
            const float x[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
            a[r][q] = split3(x);
        }
    }

    // a thread stages whole operand slots: eight consecutive inner indices of one column
    float staged[PER_THREAD][8];
    auto fetch = [&](int t) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; i++) {
            const int slot = i * kWave * kWaves + tid;
            if (SLOTS % (kWave * kWaves) == 0 || slot < SLOTS) {
                const float *col = w + (int64_t)((slot / kTile) * 8) * n + t * kTile + slot % kTile;
#pragma unroll
                for (int m = 0; m < 8; m++) staged[i][m] = col[(int64_t)m * n];
            }
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; i++) {
            const int slot = i * kWave * kWaves + tid;
            if (SLOTS % (kWave * kWaves) == 0 || slot < SLOTS) {
                const Split3 parts = split3(staged[i]);
#pragma unroll
                for (int t = 0; t < 3; t++) tile[buf][t][slot] = parts.term[t];
            }
        }
    };
    const int tiles = n / kTile;
    fetch(0);
    commit(0);
    __syncthreads();
    for (int t = 0; t < tiles; t++) {
        if (t + 1 < tiles) fetch(t + 1);
        f32x16 d[R];
#pragma unroll
        for (int r = 0; r < R; r++) d[r] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < Q; q++) {
            bf16x8 b[3];
#pragma unroll
            for (int tb = 0; tb < 3; tb++) b[tb] = tile[t & 1][tb][(q * 2 + g) * kTile + c];
            // smallest partial products first
            constexpr int kPairs[6][2] = {{0, 2}, {1, 1}, {2, 0}, {0, 1}, {1, 0}, {0, 0}};
#pragma unroll
            for (int u = 0; u < 6; u++) {
#pragma unroll
                for (int r = 0; r < R; r++)
                    d[r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r][q].term[kPairs[u][0]], b[kPairs[u][1]], d[r], 0, 0, 0);
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            float *out = s + (e0 + r * kTile + 4 * g) * n + t * kTile + c;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = 8 * (v / 4) + v % 4;
                if (e0 + r * kTile + 4 * g + row < num_edges) __builtin_nontemporal_store(d[r][v], out + (int64_t)row * n);
            }
        }
        if (t + 1 < tiles) commit((t + 1) & 1);
        __syncthreads();
    }
}

template <int H>
int launch_fwd(const float *h, const float *w, float *s, int64_t num_edges, int n, hipStream_t stream) {
    constexpr int R = H >= 128 ? 1 : 2;  // row tiles per wave (their A operands stay in registers)
    const int64_t per_block = (int64_t)kWaves * R * kTile;
    const int64_t blocks = (num_edges + per_block - 1) / per_block;
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "radial_linear: too many edges");
    if constexpr (H >= 64)  // float32 matrix-core rate would bound these; the split form is bound by the stream
        hipLaunchKernelGGL((radial_linear_fwd_split_kernel<H, R>), dim3((unsigned)blocks), dim3(kWave * kWaves), 0,
                           stream, h, w, s, num_edges, n);
    else
        hipLaunchKernelGGL((radial_linear_fwd_kernel<H, R>), dim3((unsigned)blocks), dim3(kWave * kWaves), 0, stream,
                           h, w, s, num_edges, n);
    return check_hip(hipGetLastError(), "radial_linear launch");
}

// dW (H, n) = h^T ds, the contraction running over the edges.  Both operands are read the way the
// matrix cores want them: a lane (g, c) supplies A[c][k] = h[edge k][row tile * 32 + c] and
// B[k][c] = ds[edge k][column tile * 32 + c], so consecutive lanes read consecutive addresses.
// A block takes a slab of kSlab columns (kColTiles column tiles per wave) and one of `groups`
// ranges of the edges, keeps its part of dW in the accumulators and stores it as one slice of
// `partial (groups, H, n)`; a second kernel adds the slices in a fixed order.  The rows of h of a
// chunk of 64 edges (one contiguous block) are shared by the waves through LDS (double buffered).
// ds is read once; h once per slab (from the L2).
constexpr int kColTiles = 2;
constexpr int kSlab = kTile * kColTiles * kWaves;

template <int H>
__global__ __launch_bounds__(kWave * kWaves) void radial_linear_bwd_weight_kernel(
    const float *__restrict__ h, const float *__restrict__ ds, float *__restrict__ partial, int64_t num_edges,
    int n, int groups) {
    constexpr int RT = (H + kTile - 1) / kTile;  // row tiles of dW
    constexpr int HP = RT * kTile;               // rows padded to whole tiles (inner sizes 8, 16)
    constexpr int CHUNK = 64;                    // edges per step: 32 per lane half
    constexpr int HALF = CHUNK / 2;
    constexpr int PIECES = CHUNK * H / 4;        // 16-byte pieces of a chunk of h
    constexpr int PER_THREAD = (PIECES + kWave * kWaves - 1) / (kWave * kWaves);
    __shared__ __attribute__((aligned(16))) float rows[2][CHUNK * HP];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int g = lane / kTile, c = lane % kTile;
    const int slabs = (n + kSlab - 1) / kSlab;
    const int slab = blockIdx.x % slabs, group = blockIdx.x / slabs;
    const int col0 = slab * kSlab + wave * (kTile * kColTiles);  // first column of this wave
    const int64_t per_group = ((num_edges + groups - 1) / groups + CHUNK - 1) / CHUNK * CHUNK;
    const int64_t first = (int64_t)group * per_group;
    const int64_t last = first + per_group < num_edges ? first + per_group : num_edges;
    if (HP != H) {  // rows past the inner size multiply zeros
        for (int i = tid; i < 2 * CHUNK * HP; i += kWave * kWaves) (&rows[0][0])[i] = 0.f;
        __syncthreads();
    }

    f32x16 d[kColTiles][RT];
#pragma unroll
    for (int t = 0; t < kColTiles; t++)
#pragma unroll
        for (int rt = 0; rt < RT; rt++)
            d[t][rt] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    bool col_ok[kColTiles];                      // (n is a multiple of 32: whole tiles are in or out)
    const float *dcol[kColTiles];
#pragma unroll
    for (int t = 0; t < kColTiles; t++) {
        col_ok[t] = col0 + t * kTile < n;
        dcol[t] = ds + (col_ok[t] ? col0 + t * kTile + c : 0);
    }

    f32x4 staged[PER_THREAD];
    auto fetch = [&](int64_t e0) {  // rows [e0, e0 + 64) of h: edges past the range read as zeros
#pragma unroll
        for (int i = 0; i < PER_THREAD; i++) {
            const int piece = i * kWave * kWaves + tid;
            if (PIECES % (kWave * kWaves) == 0 || piece < PIECES) {
                const int64_t e = e0 + piece * 4 / H;
                staged[i] = e < last ? *reinterpret_cast<const f32x4 *>(h + e0 * H + (int64_t)piece * 4)
                                     : f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; i++) {
            const int piece = i * kWave * kWaves + tid;
            if (PIECES % (kWave * kWaves) == 0 || piece < PIECES) {
                const int at = piece * 4;
                *reinterpret_cast<f32x4 *>(&rows[buf][(at / H) * HP + at % H]) = staged[i];
            }
        }
    };
    if (first < last) {
        fetch(first);
        commit(0);
    }
    __syncthreads();
    int buf = 0;
    for (int64_t e0 = first; e0 < last; e0 += CHUNK, buf ^= 1) {
        const bool more = e0 + CHUNK < last;
        if (more) fetch(e0 + CHUNK);
        float b[kColTiles][HALF];
#pragma unroll
        for (int j = 0; j < HALF; j++) {
            const int64_t e = e0 + g * HALF + j;
            const bool in = e < last;            // edges past the range multiply zeros
            const int64_t ee = in ? e : last - 1;
#pragma unroll
            for (int t = 0; t < kColTiles; t++) b[t][j] = in ? __builtin_nontemporal_load(dcol[t] + ee * n) : 0.f;
        }
#pragma unroll
        for (int j = 0; j < HALF; j++) {
#pragma unroll
            for (int rt = 0; rt < RT; rt++) {
                const float a = rows[buf][(g * HALF + j) * HP + rt * kTile + c];
#pragma unroll
                for (int t = 0; t < kColTiles; t++)
                    d[t][rt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b[t][j], d[t][rt], 0, 0, 0);
            }
        }
        if (more) commit(buf ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int t = 0; t < kColTiles; t++) {
        if (!col_ok[t]) continue;
        float *out = partial + (int64_t)group * H * n + col0 + t * kTile + c;
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = rt * kTile + 8 * (v / 4) + 4 * g + v % 4;
                if (row < H) out[(int64_t)row * n] = d[t][rt][v];
            }
        }
    }
}

// The same from inner size 64 on, at the bfloat16 rate with both operands split three ways (see
// the forward kernel): h when a chunk is staged (an operand slot = eight consecutive edges of one
// row of dW), ds in registers as it arrives.
template <int H>
__global__ __launch_bounds__(kWave * kWaves) void radial_linear_bwd_weight_split_kernel(
    const float *__restrict__ h, const float *__restrict__ ds, float *__restrict__ partial, int64_t num_edges,
    int n, int groups) {
    constexpr int RT = H / kTile;                // row tiles of dW
    constexpr int CHUNK = 64, Q = CHUNK / 16;    // edges per step; inner blocks of 16 edges
    constexpr int SLOTS = 2 * Q * H;             // (q, g, row) operand slots of a chunk of h
    constexpr int PER_THREAD = SLOTS / (kWave * kWaves);
    static_assert(H % kTile == 0 && SLOTS % (kWave * kWaves) == 0, "whole tiles, whole rounds of slots");
    __shared__ __attribute__((aligned(16))) bf16x8 rows[2][3][SLOTS];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int g = lane / kTile, c = lane % kTile;
    const int slabs = (n + kSlab - 1) / kSlab;
    const int slab = blockIdx.x % slabs, group = blockIdx.x / slabs;
    const int col0 = slab * kSlab + wave * (kTile * kColTiles);
    const int64_t per_group = ((num_edges + groups - 1) / groups + CHUNK - 1) / CHUNK * CHUNK;
    const int64_t first = (int64_t)group * per_group;
    const int64_t last = first + per_group < num_edges ? first + per_group : num_edges;

    f32x16 d[kColTiles][RT];
#pragma unroll
    for (int t = 0; t < kColTiles; t++)
#pragma unroll
        for (int rt = 0; rt < RT; rt++)
            d[t][rt] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    bool col_ok[kColTiles];
    const float *dcol[kColTiles];
#pragma unroll
    for (int t = 0; t < kColTiles; t++) {
        col_ok[t] = col0 + t * kTile < n;
        dcol[t] = ds + (col_ok[t] ? col0 + t * kTile + c : 0);
    }

    float staged[PER_THREAD][8];
    auto fetch = [&](int64_t e0) {  // slot (q, g, row): h[e0 + 16 q + 8 g + m][row], m < 8
#pragma unroll
        for (int i = 0; i < PER_THREAD; i++) {
            const int slot = i * kWave * kWaves + tid;
            const int64_t e = e0 + (slot / H) * 8;
#pragma unroll
            for (int m = 0; m < 8; m++) staged[i][m] = e + m < last ? h[(e + m) * H + slot % H] : 0.f;
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; i++) {
            const Split3 parts = split3(staged[i]);
#pragma unroll
            for (int t = 0; t < 3; t++) rows[buf][t][i * kWave * kWaves + tid] = parts.term[t];
        }
    };
    if (first < last) {
        fetch(first);
        commit(0);
    }
    __syncthreads();
    // the eight ds values of a lane for the block of 16 edges at `e`: loaded one block ahead
    float xn[kColTiles][8];
    auto load_ds = [&](int64_t e) {
#pragma unroll
        for (int t = 0; t < kColTiles; t++)
#pragma unroll
            for (int m = 0; m < 8; m++) {
                const int64_t em = e + g * 8 + m;
                xn[t][m] = em < last ? __builtin_nontemporal_load(dcol[t] + em * n) : 0.f;
            }
    };
    if (first < last) load_ds(first);
    int buf = 0;
    for (int64_t e0 = first; e0 < last; e0 += CHUNK, buf ^= 1) {
        const bool more = e0 + CHUNK < last;
        if (more) fetch(e0 + CHUNK);
#pragma unroll 1
        for (int q = 0; q < Q; q++) {  // (not unrolled: the split operands of one block fill the registers)
            Split3 b[kColTiles];
#pragma unroll
            for (int t = 0; t < kColTiles; t++) b[t] = split3(xn[t]);
            if (e0 + (q + 1) * 16 < last) load_ds(e0 + (q + 1) * 16);
            constexpr int kPairs[6][2] = {{0, 2}, {1, 1}, {2, 0}, {0, 1}, {1, 0}, {0, 0}};
#pragma unroll
            for (int rt = 0; rt < RT; rt++) {
                bf16x8 a[3];
#pragma unroll
                for (int ta = 0; ta < 3; ta++) a[ta] = rows[buf][ta][(q * 2 + g) * H + rt * kTile + c];
#pragma unroll
                for (int u = 0; u < 6; u++) {
#pragma unroll
                    for (int t = 0; t < kColTiles; t++)
                        d[t][rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[kPairs[u][0]], b[t].term[kPairs[u][1]],
                                                                           d[t][rt], 0, 0, 0);
                }
            }
        }
        if (more) commit(buf ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int t = 0; t < kColTiles; t++) {
        if (!col_ok[t]) continue;
        float *out = partial + (int64_t)group * H * n + col0 + t * kTile + c;
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
#pragma unroll
            for (int v = 0; v < 16; v++) out[(int64_t)(rt * kTile + 8 * (v / 4) + 4 * g + v % 4) * n] = d[t][rt][v];
        }
    }
}

__global__ void radial_linear_sum_groups_kernel(const float *__restrict__ partial, float *__restrict__ dw,
                                                int64_t count, int groups) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float total = 0.f;
    for (int q = 0; q < groups; q++) total += partial[(int64_t)q * count + i];
    dw[i] = total;
}

// ranges of the edges: enough blocks to fill the machine several times over, at most 128 slices
int weight_groups(int64_t num_edges, int n) {
    const int slabs = (n + kSlab - 1) / kSlab;
    int64_t groups = (2048 + slabs - 1) / slabs;
    const int64_t most = (num_edges + 63) / 64;
    if (groups > most) groups = most;
    if (groups > 128) groups = 128;
    return groups < 1 ? 1 : (int)groups;
}

template <int H>
int launch_bwd_weight(const float *h, const float *ds, float *dw, float *partial, int64_t num_edges, int n,
                      hipStream_t stream) {
    const int groups = weight_groups(num_edges, n);
    const int slabs = (n + kSlab - 1) / kSlab;
    if constexpr (H >= 64)
        hipLaunchKernelGGL((radial_linear_bwd_weight_split_kernel<H>), dim3((unsigned)(slabs * groups)),
                           dim3(kWave * kWaves), 0, stream, h, ds, partial, num_edges, n, groups);
    else
        hipLaunchKernelGGL((radial_linear_bwd_weight_kernel<H>), dim3((unsigned)(slabs * groups)),
                           dim3(kWave * kWaves), 0, stream, h, ds, partial, num_edges, n, groups);
    int rc = check_hip(hipGetLastError(), "radial_linear_bwd_weight launch");
    if (rc) return rc;
    const int64_t count = (int64_t)H * n;
    hipLaunchKernelGGL(radial_linear_sum_groups_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream,
                       partial, dw, count, groups);
    return check_hip(hipGetLastError(), "radial_linear_bwd_weight reduction launch");
}

// dh (E, H) = ds W^T for inner sizes of 64 and more, with W^T passed as wt (n, H).  The
// contraction runs along the rows of ds, so a lane (which stands for an edge in the operand
// layout) would read its own row; instead a wave loads its tile of 32 R edges x 32 n the coalesced
// way (a row piece of 128 bytes per 8 lanes), splits it three ways and writes the parts to its
// private piece of LDS in operand order, from where every lane fetches its slots with 16-byte
// reads.  The rows of wt of the same 32 n, one contiguous block, are split and shared by the
// waves of the block.  ds is read once.
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int H, int R>
__global__ __launch_bounds__(kWave * kWaves) void radial_linear_bwd_input_split_kernel(
    const float *__restrict__ ds, const float *__restrict__ wt, float *__restrict__ dh, int64_t num_edges, int n) {
    constexpr int CT = H / kTile;                 // column tiles of dh
    constexpr int CHUNK = 32, Q = CHUNK / 16;     // n per step; inner blocks of 16
    constexpr int ROWS = R * kTile;               // edges of a wave
    constexpr int A_SLOTS = 2 * Q * ROWS;         // (q, g, edge) operand slots of a wave's tile
    constexpr int A_PIECES = ROWS * CHUNK / 4 / kWave;  // 16-byte pieces of the tile per lane
    constexpr int B_SLOTS = 2 * Q * H;            // (q, g, column) operand slots of the wt chunk
    constexpr int B_PER_THREAD = (B_SLOTS + kWave * kWaves - 1) / (kWave * kWaves);
    __shared__ __attribute__((aligned(16))) bf16x8 a_tile[kWaves][3][A_SLOTS];
    __shared__ __attribute__((aligned(16))) bf16x8 b_tile[3][B_SLOTS];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int g = lane / kTile, c = lane % kTile;
    const int64_t e0 = ((int64_t)blockIdx.x * kWaves + wave) * ROWS;

    // a lane moves A_PIECES pieces of 16 bytes of the tile: piece p = 64 i + lane is n-quad p % 8 of edge p / 8
    const float *src[A_PIECES];
    int half_slot[A_PIECES];  // where the piece goes: 8-byte half (p % 2) of slot (q, g, edge)
#pragma unroll
    for (int i = 0; i < A_PIECES; i++) {
        const int p = i * kWave + lane, edge = p / 8, quad = p % 8;
        int64_t row = e0 + edge;
        if (row >= num_edges) row = num_edges - 1;  // rows past the end are computed and not stored
        src[i] = ds + row * n + quad * 4;
        half_slot[i] = (((quad / 4) * 2 + (quad / 2) % 2) * ROWS + edge) * 2 + quad % 2;
    }
    f32x16 d[R][CT];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int ct = 0; ct < CT; ct++)
            d[r][ct] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    f32x4 a_next[A_PIECES];
    float b_next[B_PER_THREAD][8];
    auto fetch = [&](int t) {
#pragma unroll
        for (int i = 0; i < A_PIECES; i++)
            a_next[i] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src[i] + t * CHUNK));
#pragma unroll
        for (int i = 0; i < B_PER_THREAD; i++) {  // slot (q, g, column): wt[32 t + 16 q + 8 g + m][column]
            const int slot = i * kWave * kWaves + tid;
            if (B_SLOTS % (kWave * kWaves) == 0 || slot < B_SLOTS) {
                const float *col = wt + ((int64_t)t * CHUNK + (slot / H) * 8) * H + slot % H;
#pragma unroll
                for (int m = 0; m < 8; m++) b_next[i][m] = col[m * H];
            }
        }
    };
    auto commit = [&]() {
        u32x2 *halves[3] = {reinterpret_cast<u32x2 *>(a_tile[wave][0]), reinterpret_cast<u32x2 *>(a_tile[wave][1]),
                            reinterpret_cast<u32x2 *>(a_tile[wave][2])};
#pragma unroll
        for (int i = 0; i < A_PIECES; i++) {
            float rest[4] = {a_next[i].x, a_next[i].y, a_next[i].z, a_next[i].w};
#pragma unroll
            for (int t = 0; t < 3; t++) {  // the three parts of four values: see split3
                u32x2 packed;
#pragma unroll
                for (int m = 0; m < 4; m += 2) {
                    const uint32_t lo = __float_as_uint(rest[m]) & 0xffff0000u, hi = __float_as_uint(rest[m + 1]) & 0xffff0000u;
                    packed[m / 2] = (lo >> 16) | hi;
                    rest[m] -= __uint_as_float(lo);
                    rest[m + 1] -= __uint_as_float(hi);
                }
                halves[t][half_slot[i]] = packed;
            }
        }
#pragma unroll
        for (int i = 0; i < B_PER_THREAD; i++) {
            const int slot = i * kWave * kWaves + tid;
            if (B_SLOTS % (kWave * kWaves) == 0 || slot < B_SLOTS) {
                const Split3 parts = split3(b_next[i]);
#pragma unroll
                for (int t = 0; t < 3; t++) b_tile[t][slot] = parts.term[t];
            }
        }
    };
    const int chunks = n / CHUNK;
    fetch(0);
    for (int t = 0; t < chunks; t++) {
        commit();
        if (t + 1 < chunks) fetch(t + 1);
        __syncthreads();
        constexpr int kPairs[6][2] = {{0, 2}, {1, 1}, {2, 0}, {0, 1}, {1, 0}, {0, 0}};
#pragma unroll
        for (int q = 0; q < Q; q++) {
            bf16x8 a[R][3];
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int ta = 0; ta < 3; ta++) a[r][ta] = a_tile[wave][ta][(q * 2 + g) * ROWS + r * kTile + c];
#pragma unroll
            for (int ct = 0; ct < CT; ct++) {
                bf16x8 b[3];
#pragma unroll
                for (int tb = 0; tb < 3; tb++) b[tb] = b_tile[tb][(q * 2 + g) * H + ct * kTile + c];
#pragma unroll
                for (int u = 0; u < 6; u++) {
#pragma unroll
                    for (int r = 0; r < R; r++)
                        d[r][ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r][kPairs[u][0]], b[kPairs[u][1]], d[r][ct],
                                                                           0, 0, 0);
                }
            }
        }
        __syncthreads();  // every wave is done with the shared rows of wt before they are replaced
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int ct = 0; ct < CT; ct++) {
            float *out = dh + (e0 + r * kTile + 4 * g) * H + ct * kTile + c;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = 8 * (v / 4) + v % 4;
                if (e0 + r * kTile + 4 * g + row < num_edges) out[(int64_t)row * H] = d[r][ct][v];
            }
        }
    }
}

template <int H>
int launch_bwd_input(const float *ds, const float *wt, float *dh, int64_t num_edges, int n, hipStream_t stream) {
    constexpr int R = H >= 128 ? 1 : 2;  // row tiles per wave
    const int64_t per_block = (int64_t)kWaves * R * kTile;
    const int64_t blocks = (num_edges + per_block - 1) / per_block;
    if (blocks > 0x7fffffffLL) return set_error(E3J_AMD_INVALID_ARGUMENT, "radial_linear_bwd_input: too many edges");
    hipLaunchKernelGGL((radial_linear_bwd_input_split_kernel<H, R>), dim3((unsigned)blocks), dim3(kWave * kWaves), 0,
                       stream, ds, wt, dh, num_edges, n);
    return check_hip(hipGetLastError(), "radial_linear_bwd_input launch");
}

// The kernels move rows of the operands in 16-byte pieces.
int check_aligned(const char *what, std::initializer_list<const void *> ptrs) {
    for (const void *ptr : ptrs)
        if (reinterpret_cast<uintptr_t>(ptr) % 16 != 0)
            return set_error(E3J_AMD_INVALID_ARGUMENT, std::string(what) + ": operands must be 16-byte aligned");
    return E3J_AMD_OK;
}

int check_shapes(const char *what, int64_t num_edges, int32_t inner, int32_t n) {
    if (num_edges < 0 || inner <= 0 || n <= 0)
        return set_error(E3J_AMD_INVALID_ARGUMENT, std::string(what) + ": bad sizes");
    if (n % kTile != 0)
        return set_error(E3J_AMD_UNIMPLEMENTED, std::string(what) + ": paths * channels must be a multiple of 32");
    if (inner != 8 && inner != 16 && inner != 32 && inner != 64 && inner != 128)
        return set_error(E3J_AMD_UNIMPLEMENTED, std::string(what) + ": hidden size must be 8, 16, 32, 64 or 128");
    return E3J_AMD_OK;
}

}  // namespace

extern "C" int e3j_amd_radial_linear_fwd(const float *h, const float *w, float *s, int64_t num_edges,
                                         int32_t inner, int32_t n, void *stream_) {
    if (int rc = check_shapes("radial_linear", num_edges, inner, n)) return rc;
    if (num_edges == 0) return E3J_AMD_OK;
    if (h == nullptr || w == nullptr || s == nullptr)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "radial_linear: null operand");
    if (int rc = check_aligned("radial_linear", {h, w, s})) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    switch (inner) {
        case 8: return launch_fwd<8>(h, w, s, num_edges, n, stream);
        case 16: return launch_fwd<16>(h, w, s, num_edges, n, stream);
        case 32: return launch_fwd<32>(h, w, s, num_edges, n, stream);
        case 64: return launch_fwd<64>(h, w, s, num_edges, n, stream);
        default: return launch_fwd<128>(h, w, s, num_edges, n, stream);
    }
}

extern "C" size_t e3j_amd_radial_linear_bwd_weight_workspace_bytes(int64_t num_edges, int32_t inner, int32_t n) {
    if (num_edges <= 0 || inner <= 0 || n <= 0) return 0;
    return sizeof(float) * (size_t)weight_groups(num_edges, n) * inner * n;
}

extern "C" int e3j_amd_radial_linear_bwd_weight(const float *h, const float *ds, float *dw, void *workspace,
                                                int64_t num_edges, int32_t inner, int32_t n, void *stream_) {
    if (int rc = check_shapes("radial_linear_bwd_weight", num_edges, inner, n)) return rc;
    if (dw == nullptr) return set_error(E3J_AMD_INVALID_ARGUMENT, "radial_linear_bwd_weight: null operand");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (num_edges == 0) return launch_fill_zero(dw, sizeof(float) * (size_t)inner * n, stream);
    if (h == nullptr || ds == nullptr || workspace == nullptr)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "radial_linear_bwd_weight: null operand");
    if (int rc = check_aligned("radial_linear_bwd_weight", {h, ds, dw, workspace})) return rc;
    float *partial = static_cast<float *>(workspace);
    switch (inner) {
        case 8: return launch_bwd_weight<8>(h, ds, dw, partial, num_edges, n, stream);
        case 16: return launch_bwd_weight<16>(h, ds, dw, partial, num_edges, n, stream);
        case 32: return launch_bwd_weight<32>(h, ds, dw, partial, num_edges, n, stream);
        case 64: return launch_bwd_weight<64>(h, ds, dw, partial, num_edges, n, stream);
        default: return launch_bwd_weight<128>(h, ds, dw, partial, num_edges, n, stream);
    }
}

extern "C" int e3j_amd_radial_linear_bwd_input(const float *ds, const float *wt, float *dh, int64_t num_edges,
                                               int32_t inner, int32_t n, void *stream_) {
    if (int rc = check_shapes("radial_linear_bwd_input", num_edges, inner, n)) return rc;
    if (inner < 64)
        return set_error(E3J_AMD_UNIMPLEMENTED, "radial_linear_bwd_input: hidden sizes below 64 are left to the "
                                                "library product, which reads ds near the rate of the memory");
    if (num_edges == 0) return E3J_AMD_OK;
    if (ds == nullptr || wt == nullptr || dh == nullptr)
        return set_error(E3J_AMD_INVALID_ARGUMENT, "radial_linear_bwd_input: null operand");
    if (int rc = check_aligned("radial_linear_bwd_input", {ds, wt, dh})) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    return inner == 64 ? launch_bwd_input<64>(ds, wt, dh, num_edges, n, stream)
                       : launch_bwd_input<128>(ds, wt, dh, num_edges, n, stream);
}

}  // namespace e3j_amd
