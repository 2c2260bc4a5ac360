// Real spherical harmonics of edge vectors and their vector-Jacobian product, one thread per
// vector.  Counterpart of the polynomial evaluation behind `Harmonics.__call__`
// (src/e3j/core/harmonics.py:92-101, src/e3j/utils/spherical_harmonics.py:50-82), which XLA
// fuses on the reference's side; here it keeps the edge featurisation of a model (harmonics of
// about 1e5-1e6 vectors, forward and backward) to two launches.
//
// Degrees 0..l_max, m = -l..l within a degree; harmonic frame (X, Y, Z) = input (z, x, y).
// The functions are evaluated as homogeneous polynomials (no projection on the sphere unless
// `normalize` is set) from the recurrences of (X + iY)^m and of the associated Legendre
// polynomials divided by (1 - Z^2)^(m/2).  The backward pass runs the same recurrences on
// numbers that carry their gradient with respect to the three input components.
#include <cmath>

#include "common.h"

namespace e3j_amd {
namespace {

constexpr int kMaxDegree = 6;
constexpr int kMaxOut = (kMaxDegree + 1) * (kMaxDegree + 1);

// factor[l * l + l + m] for m >= 0: normalisation of Y_l^{+-m} (sqrt 2 included for m > 0)
struct Factors {
    double f[kMaxOut];
};

template <typename T>
struct Dual {  // value and gradient with respect to the input components (x, y, z)
    T v, g[3];
};
template <typename T>
__device__ __forceinline__ Dual<T> operator+(const Dual<T> &a, const Dual<T> &b) {
    return {a.v + b.v, {a.g[0] + b.g[0], a.g[1] + b.g[1], a.g[2] + b.g[2]}};
}
template <typename T>
__device__ __forceinline__ Dual<T> operator-(const Dual<T> &a, const Dual<T> &b) {
    return {a.v - b.v, {a.g[0] - b.g[0], a.g[1] - b.g[1], a.g[2] - b.g[2]}};
}
template <typename T>
__device__ __forceinline__ Dual<T> operator*(const Dual<T> &a, const Dual<T> &b) {
    return {a.v * b.v, {a.v * b.g[0] + a.g[0] * b.v, a.v * b.g[1] + a.g[1] * b.v, a.v * b.g[2] + a.g[2] * b.v}};
}
template <typename T>
__device__ __forceinline__ Dual<T> operator*(T s, const Dual<T> &a) {
    return {s * a.v, {s * a.g[0], s * a.g[1], s * a.g[2]}};
}
template <typename T>
__device__ __forceinline__ T constant(T, double c) { return (T)c; }
template <typename T>
__device__ __forceinline__ Dual<T> constant(Dual<T>, double c) { return {(T)c, {T(0), T(0), T(0)}}; }

// emit(index, value) receives every component; N is T or Dual<T>, S the scalar type
template <int L, typename S, typename N, typename Emit>
__device__ __forceinline__ void harmonics(const N &x_in, const N &y_in, const N &z_in, const Factors &fac,
                                          Emit emit) {
    const N X = z_in, Y = x_in, Z = y_in;
    const N r2 = X * X + Y * Y + Z * Z;
    N c[L + 1], s[L + 1];
    c[0] = constant(N{}, 1.0);
    s[0] = constant(N{}, 0.0);
#pragma unroll
    for (int m = 1; m <= L; m++) {
        c[m] = c[m - 1] * X - s[m - 1] * Y;
        s[m] = s[m - 1] * X + c[m - 1] * Y;
    }
    N q[L + 1][L + 1];
    double dfact = 1.0;  // (2m - 1)!!
#pragma unroll
    for (int m = 0; m <= L; m++) {
        if (m > 0) dfact *= (double)(2 * m - 1);
        q[m][m] = constant(N{}, dfact);
        if (m + 1 <= L) q[m + 1][m] = (S)(2 * m + 1) * (Z * q[m][m]);
#pragma unroll
        for (int l = m + 2; l <= L; l++)
            q[l][m] = (S)(1.0 / (l - m)) * ((S)(2 * l - 1) * (Z * q[l - 1][m]) - (S)(l + m - 1) * (r2 * q[l - 2][m]));
    }
#pragma unroll
    for (int l = 0; l <= L; l++) {
        const int base = l * l + l;
        emit(base, (S)fac.f[base] * q[l][0]);
#pragma unroll
        for (int m = 1; m <= l; m++) {
            const N qm = (S)fac.f[base + m] * q[l][m];
            emit(base + m, qm * c[m]);
            emit(base - m, qm * s[m]);
        }
    }
}

template <typename T>
__device__ __forceinline__ T safe_norm(T x, T y, T z) {
    const T n = sqrt(x * x + y * y + z * z);
    return n > T(0) ? n : T(1);
}

template <typename T, int L>
__global__ void harmonics_fwd_kernel(const T *__restrict__ vec, int64_t num, int normalize, Factors fac,
                                     T *__restrict__ out) {
    constexpr int NOUT = (L + 1) * (L + 1);
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < num; e += stride) {
        T x = vec[3 * e], y = vec[3 * e + 1], z = vec[3 * e + 2];
        if (normalize) {
            const T inv = T(1) / safe_norm(x, y, z);
            x *= inv; y *= inv; z *= inv;
        }
        T *row = out + e * NOUT;
        harmonics<L, T>(x, y, z, fac, [&](int index, T value) { row[index] = value; });
    }
}

template <typename T, int L>
__global__ void harmonics_bwd_kernel(const T *__restrict__ vec, const T *__restrict__ dout, int64_t num,
                                     int normalize, Factors fac, T *__restrict__ dvec) {
    constexpr int NOUT = (L + 1) * (L + 1);
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < num; e += stride) {
        T x = vec[3 * e], y = vec[3 * e + 1], z = vec[3 * e + 2];
        T inv = T(1);
        if (normalize) {
            inv = T(1) / safe_norm(x, y, z);
            x *= inv; y *= inv; z *= inv;
        }
        const Dual<T> dx{x, {T(1), T(0), T(0)}}, dy{y, {T(0), T(1), T(0)}}, dz{z, {T(0), T(0), T(1)}};
        const T *drow = dout + e * NOUT;
        T g[3] = {T(0), T(0), T(0)};
        harmonics<L, T>(dx, dy, dz, fac, [&](int index, const Dual<T> &value) {
            const T w = drow[index];
            g[0] += w * value.g[0];
            g[1] += w * value.g[1];
            g[2] += w * value.g[2];
        });
        if (normalize) {  // through r / |r|: (g - r (r . g)) / |r|
            const T dot = x * g[0] + y * g[1] + z * g[2];
            g[0] = (g[0] - x * dot) * inv;
            g[1] = (g[1] - y * dot) * inv;
            g[2] = (g[2] - z * dot) * inv;
        }
        dvec[3 * e] = g[0];
        dvec[3 * e + 1] = g[1];
        dvec[3 * e + 2] = g[2];
    }
}

double factorial(int n) {
    double f = 1.0;
    for (int i = 2; i <= n; i++) f *= i;
    return f;
}

// normalization: 0 integral, 1 component, 2 norm (src/e3j/core/harmonics.py:25-42)
bool make_factors(int l_max, int normalization, Factors *fac) {
    for (int l = 0; l <= l_max; l++) {
        double scale;
        if (normalization == 0) scale = 1.0;
        else if (normalization == 1) scale = std::sqrt(4.0 * M_PI);
        else if (normalization == 2) scale = std::sqrt(4.0 * M_PI / (2 * l + 1));
        else return false;
        for (int m = 0; m <= l; m++) {
            const double n_lm = std::sqrt((2 * l + 1) / (4.0 * M_PI) * factorial(l - m) / factorial(l + m));
            fac->f[l * l + l + m] = scale * n_lm * (m == 0 ? 1.0 : std::sqrt(2.0));
        }
    }
    return true;
}

template <typename T, int L>
int launch(bool backward, const void *vec, const void *dout, int64_t num, int normalize,
           const Factors &fac, void *result, hipStream_t stream) {
    const unsigned blocks = (unsigned)std::min<int64_t>((num + 255) / 256, 1 << 20);
    if (backward)
        hipLaunchKernelGGL((harmonics_bwd_kernel<T, L>), dim3(blocks), dim3(256), 0, stream,
                           static_cast<const T *>(vec), static_cast<const T *>(dout), num, normalize, fac,
                           static_cast<T *>(result));
    else
        hipLaunchKernelGGL((harmonics_fwd_kernel<T, L>), dim3(blocks), dim3(256), 0, stream,
                           static_cast<const T *>(vec), num, normalize, fac, static_cast<T *>(result));
    return check_hip(hipGetLastError(), backward ? "harmonics backward launch" : "harmonics launch");
}

template <typename T>
int dispatch_degree(int l_max, bool backward, const void *vec, const void *dout, int64_t num, int normalize,
                    const Factors &fac, void *result, hipStream_t stream) {
    switch (l_max) {
        case 0: return launch<T, 0>(backward, vec, dout, num, normalize, fac, result, stream);
        case 1: return launch<T, 1>(backward, vec, dout, num, normalize, fac, result, stream);
        case 2: return launch<T, 2>(backward, vec, dout, num, normalize, fac, result, stream);
        case 3: return launch<T, 3>(backward, vec, dout, num, normalize, fac, result, stream);
        case 4: return launch<T, 4>(backward, vec, dout, num, normalize, fac, result, stream);
        case 5: return launch<T, 5>(backward, vec, dout, num, normalize, fac, result, stream);
        default: return launch<T, 6>(backward, vec, dout, num, normalize, fac, result, stream);
    }
}

int run(bool backward, const void *vec, const void *dout, int64_t num, int32_t l_max, int32_t normalize,
        int32_t normalization, int32_t val_dtype, void *result, void *stream) {
    const char *op = backward ? "harmonics_bwd" : "harmonics";
    if (num < 0 || l_max < 0) return set_error(E3J_AMD_INVALID_ARGUMENT, std::string(op) + ": negative size");
    if (l_max > kMaxDegree)
        return set_error(E3J_AMD_UNIMPLEMENTED, std::string(op) + ": degrees above 6 are not built");
    Factors fac{};
    if (!make_factors(l_max, normalization, &fac))
        return set_error(E3J_AMD_INVALID_ARGUMENT, std::string(op) + ": unknown normalization");
    if (num == 0) return E3J_AMD_OK;
    if (vec == nullptr || result == nullptr || (backward && dout == nullptr))
        return set_error(E3J_AMD_INVALID_ARGUMENT, std::string(op) + ": null operand");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (val_dtype == E3J_AMD_F32)
        return dispatch_degree<float>(l_max, backward, vec, dout, num, normalize, fac, result, s);
    if (val_dtype == E3J_AMD_F64)
        return dispatch_degree<double>(l_max, backward, vec, dout, num, normalize, fac, result, s);
    return set_error(E3J_AMD_INVALID_ARGUMENT, std::string(op) + ": unsupported value dtype");
}

}  // namespace
}  // namespace e3j_amd

extern "C" {

int e3j_amd_harmonics(const void *vec, int64_t num, int32_t l_max, int32_t normalize,
                      int32_t normalization, int32_t val_dtype, void *out, void *stream) {
    return e3j_amd::run(false, vec, nullptr, num, l_max, normalize, normalization, val_dtype, out, stream);
}

int e3j_amd_harmonics_bwd(const void *vec, const void *dout, int64_t num, int32_t l_max,
                          int32_t normalize, int32_t normalization, int32_t val_dtype, void *dvec,
                          void *stream) {
    return e3j_amd::run(true, vec, dout, num, l_max, normalize, normalization, val_dtype, dvec, stream);
}

}  // extern "C"
