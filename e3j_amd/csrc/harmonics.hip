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

// ---- edge featurisation in one launch -----------------------------------------------------
// Everything a message-passing layer derives from the atom positions along an edge, per edge
// and in registers: the edge vector r_sender - r_receiver (+ lattice translation), its length,
// the harmonics of its direction, the radial basis (Bessel functions sqrt(2 / rc) sin(n pi r / rc) / r
// times the polynomial cutoff envelope 1 - 10 t^3 + 15 t^4 - 6 t^5, t = r / rc) and the hidden
// layer silu(basis W1) of the radial network of each of `layers` convolution layers.  The last
// layer of that network is e3j_amd_radial_linear_fwd, which writes the convolution's operand s.
// The backward pass recomputes all of it from the positions and adds the gradient of every edge
// vector to the positions of its two atoms.
struct EdgeFeatureSizes {
    int64_t num_edges;
    int32_t num_nodes, num_basis, hidden, layers;
    double cutoff;
};
constexpr int kMaxBasis = 16;

template <typename T>
__device__ __forceinline__ T sin_pi(T v);
template <>
__device__ __forceinline__ float sin_pi<float>(float v) { return sinpif(v); }
template <>
__device__ __forceinline__ double sin_pi<double>(double v) { return sinpi(v); }
template <typename T>
__device__ __forceinline__ T cos_pi(T v);
template <>
__device__ __forceinline__ float cos_pi<float>(float v) { return cospif(v); }
template <>
__device__ __forceinline__ double cos_pi<double>(double v) { return cospi(v); }

// basis[n] and, if kGrad, dbasis[n] / dr, n = 0 .. num_basis - 1, at distance r > 0
template <typename T, bool kGrad>
__device__ __forceinline__ void radial_basis(T r, T cutoff, int num_basis, T *basis, T *dbasis) {
    const T t = r / cutoff;
    const T tc = t < T(1) ? t : T(1);
    const T t2 = tc * tc, t3 = t2 * tc;
    const T env = T(1) - T(10) * t3 + T(15) * t3 * tc - T(6) * t3 * t2;
    const T denv = t < T(1) ? (T(-30) * t2 + T(60) * t3 - T(30) * t2 * t2) / cutoff : T(0);
    const T pref = sqrt(T(2) / cutoff);
    const T inv_r = T(1) / r;
    for (int n = 0; n < num_basis; n++) {
        const T k = T(n + 1);
        const T sn = sin_pi<T>(k * t);
        const T b = pref * sn * inv_r;
        basis[n] = b * env;
        if (kGrad) {
            const T cs = cos_pi<T>(k * t);
            const T db = pref * (k * T(M_PI) / cutoff * cs * inv_r - sn * inv_r * inv_r);
            dbasis[n] = db * env + b * denv;
        }
    }
}

template <typename T>
__device__ __forceinline__ T sigmoid(T v) { return T(1) / (T(1) + exp(-v)); }

template <typename T>
__device__ __forceinline__ bool edge_vector(const T *__restrict__ pos, const int32_t *__restrict__ sender,
                                            const int32_t *__restrict__ receiver, const T *__restrict__ shift,
                                            int64_t e, int32_t num_nodes, int &a, int &b, T (&v)[3]) {
    a = sender[e];
    b = receiver[e];
    if ((unsigned)a >= (unsigned)num_nodes || (unsigned)b >= (unsigned)num_nodes) return false;
#pragma unroll
    for (int d = 0; d < 3; d++) v[d] = pos[3 * (int64_t)a + d] - pos[3 * (int64_t)b + d] + (shift ? shift[3 * e + d] : T(0));
    return true;
}

template <typename T, int L>
__global__ void edge_features_fwd_kernel(const T *__restrict__ pos, const int32_t *__restrict__ sender,
                                         const int32_t *__restrict__ receiver, const T *__restrict__ shift,
                                         const T *__restrict__ w1, EdgeFeatureSizes sz, Factors fac,
                                         T *__restrict__ y, T *__restrict__ basis_out, T *__restrict__ h) {
    constexpr int NOUT = (L + 1) * (L + 1);
    const T cutoff = (T)sz.cutoff;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < sz.num_edges; e += stride) {
        int a, b;
        T v[3];
        T *yrow = y + e * NOUT;
        const bool live = edge_vector(pos, sender, receiver, shift, e, sz.num_nodes, a, b, v);
        const T r = live ? sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]) : T(0);
        if (!(r > T(0))) {  // padding edge, or two atoms on one point: no direction, no features
            for (int i = 0; i < NOUT; i++) yrow[i] = T(0);
            if (basis_out) for (int n = 0; n < sz.num_basis; n++) basis_out[e * sz.num_basis + n] = T(0);
            if (h) for (int l = 0; l < sz.layers; l++)
                for (int j = 0; j < sz.hidden; j++) h[((int64_t)l * sz.num_edges + e) * sz.hidden + j] = T(0);
            continue;
        }
        const T inv = T(1) / r;
        harmonics<L, T>(v[0] * inv, v[1] * inv, v[2] * inv, fac, [&](int index, T value) { yrow[index] = value; });
        T basis[kMaxBasis];
        radial_basis<T, false>(r, cutoff, sz.num_basis, basis, nullptr);
        if (basis_out) for (int n = 0; n < sz.num_basis; n++) basis_out[e * sz.num_basis + n] = basis[n];
        if (h) {
            for (int l = 0; l < sz.layers; l++) {
                const T *w = w1 + (int64_t)l * sz.num_basis * sz.hidden;
                T *hrow = h + ((int64_t)l * sz.num_edges + e) * sz.hidden;
                for (int j = 0; j < sz.hidden; j++) {
                    T pre = T(0);
                    for (int n = 0; n < sz.num_basis; n++) pre += basis[n] * w[n * sz.hidden + j];
                    hrow[j] = pre * sigmoid(pre);
                }
            }
        }
    }
}

template <typename T>
__device__ __forceinline__ void add_to(T *p, T v) { unsafeAtomicAdd(p, v); }

template <typename T, int L>
__global__ void edge_features_bwd_kernel(const T *__restrict__ pos, const int32_t *__restrict__ sender,
                                         const int32_t *__restrict__ receiver, const T *__restrict__ shift,
                                         const T *__restrict__ w1, const T *__restrict__ dy,
                                         const T *__restrict__ dbasis_in, const T *__restrict__ dh,
                                         EdgeFeatureSizes sz, Factors fac, T *__restrict__ dpos) {
    constexpr int NOUT = (L + 1) * (L + 1);
    const T cutoff = (T)sz.cutoff;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < sz.num_edges; e += stride) {
        int a, b;
        T v[3];
        if (!edge_vector(pos, sender, receiver, shift, e, sz.num_nodes, a, b, v)) continue;
        const T r = sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]);
        if (!(r > T(0))) continue;
        const T inv = T(1) / r;
        const T u[3] = {v[0] * inv, v[1] * inv, v[2] * inv};
        T g[3] = {T(0), T(0), T(0)};
        if (dy) {  // through the harmonics of the direction: (g - u (u . g)) / r
            const Dual<T> dx{u[0], {T(1), T(0), T(0)}}, dyy{u[1], {T(0), T(1), T(0)}}, dz{u[2], {T(0), T(0), T(1)}};
            const T *drow = dy + e * NOUT;
            harmonics<L, T>(dx, dyy, dz, fac, [&](int index, const Dual<T> &value) {
                const T w = drow[index];
                g[0] += w * value.g[0];
                g[1] += w * value.g[1];
                g[2] += w * value.g[2];
            });
            const T dot = u[0] * g[0] + u[1] * g[1] + u[2] * g[2];
#pragma unroll
            for (int d = 0; d < 3; d++) g[d] = (g[d] - u[d] * dot) * inv;
        }
        // through the length: the radial basis and the hidden layers fed by it
        T basis[kMaxBasis], dbdr[kMaxBasis], db[kMaxBasis];
        radial_basis<T, true>(r, cutoff, sz.num_basis, basis, dbdr);
        for (int n = 0; n < sz.num_basis; n++) db[n] = dbasis_in ? dbasis_in[e * sz.num_basis + n] : T(0);
        if (dh) {
            for (int l = 0; l < sz.layers; l++) {
                const T *w = w1 + (int64_t)l * sz.num_basis * sz.hidden;
                const T *drow = dh + ((int64_t)l * sz.num_edges + e) * sz.hidden;
                for (int j = 0; j < sz.hidden; j++) {
                    T pre = T(0);
                    for (int n = 0; n < sz.num_basis; n++) pre += basis[n] * w[n * sz.hidden + j];
                    const T sg = sigmoid(pre);
                    const T dpre = drow[j] * sg * (T(1) + pre * (T(1) - sg));
                    for (int n = 0; n < sz.num_basis; n++) db[n] += dpre * w[n * sz.hidden + j];
                }
            }
        }
        T dr = T(0);
        for (int n = 0; n < sz.num_basis; n++) dr += db[n] * dbdr[n];
#pragma unroll
        for (int d = 0; d < 3; d++) {
            const T total = g[d] + dr * u[d];
            add_to(dpos + 3 * (int64_t)a + d, total);
            add_to(dpos + 3 * (int64_t)b + d, -total);
        }
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

template <typename T, int L>
int launch_edge_features(bool backward, const void *pos, const int32_t *sender, const int32_t *receiver,
                         const void *shift, const void *w1, const void *a0, const void *a1, const void *a2,
                         const EdgeFeatureSizes &sz, const Factors &fac, void *r0, void *r1, void *r2,
                         hipStream_t stream) {
    const unsigned blocks = (unsigned)std::min<int64_t>((sz.num_edges + 255) / 256, 1 << 20);
    if (backward)
        hipLaunchKernelGGL((edge_features_bwd_kernel<T, L>), dim3(blocks), dim3(256), 0, stream,
                           static_cast<const T *>(pos), sender, receiver, static_cast<const T *>(shift),
                           static_cast<const T *>(w1), static_cast<const T *>(a0), static_cast<const T *>(a1),
                           static_cast<const T *>(a2), sz, fac, static_cast<T *>(r0));
    else
        hipLaunchKernelGGL((edge_features_fwd_kernel<T, L>), dim3(blocks), dim3(256), 0, stream,
                           static_cast<const T *>(pos), sender, receiver, static_cast<const T *>(shift),
                           static_cast<const T *>(w1), sz, fac, static_cast<T *>(r0), static_cast<T *>(r1),
                           static_cast<T *>(r2));
    return check_hip(hipGetLastError(), backward ? "edge_features backward launch" : "edge_features launch");
}

template <typename T>
int dispatch_edge_features(int l_max, bool backward, const void *pos, const int32_t *sender,
                           const int32_t *receiver, const void *shift, const void *w1, const void *a0,
                           const void *a1, const void *a2, const EdgeFeatureSizes &sz, const Factors &fac,
                           void *r0, void *r1, void *r2, hipStream_t stream) {
#define E3J_EDGE_CASE(L) \
    case L: return launch_edge_features<T, L>(backward, pos, sender, receiver, shift, w1, a0, a1, a2, sz, fac, r0, r1, r2, stream)
    switch (l_max) {
        E3J_EDGE_CASE(0); E3J_EDGE_CASE(1); E3J_EDGE_CASE(2); E3J_EDGE_CASE(3); E3J_EDGE_CASE(4); E3J_EDGE_CASE(5);
        default: return launch_edge_features<T, 6>(backward, pos, sender, receiver, shift, w1, a0, a1, a2, sz, fac,
                                                   r0, r1, r2, stream);
    }
#undef E3J_EDGE_CASE
}

int run_edge_features(bool backward, const e3j_amd_edge_features_params *p, const void *pos,
                      const int32_t *sender, const int32_t *receiver, const void *shift, const void *w1,
                      const void *a0, const void *a1, const void *a2, void *r0, void *r1, void *r2,
                      void *stream) {
    const std::string op = backward ? "edge_features_bwd" : "edge_features_fwd";
    if (p == nullptr) return set_error(E3J_AMD_INVALID_ARGUMENT, op + ": null params");
    if (p->num_edges < 0 || p->num_nodes < 0 || p->l_max < 0 || p->num_basis < 1 || p->hidden < 0 || p->layers < 0 ||
        !(p->cutoff > 0.0f))
        return set_error(E3J_AMD_INVALID_ARGUMENT, op + ": bad sizes");
    if (p->l_max > kMaxDegree) return set_error(E3J_AMD_UNIMPLEMENTED, op + ": degrees above 6 are not built");
    if (p->num_basis > kMaxBasis)
        return set_error(E3J_AMD_UNIMPLEMENTED, op + ": more than 16 radial basis functions are not built");
    Factors fac{};
    if (!make_factors(p->l_max, p->normalization, &fac))
        return set_error(E3J_AMD_INVALID_ARGUMENT, op + ": unknown normalization");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool hidden = p->hidden > 0 && p->layers > 0;
    if (backward) {  // a0 = dy, a1 = dbasis, a2 = dh (each optional), r0 = dpos
        if (p->num_nodes > 0 && r0 == nullptr) return set_error(E3J_AMD_INVALID_ARGUMENT, op + ": null dpos");
        const size_t elem = p->val_dtype == E3J_AMD_F64 ? 8 : 4;
        int rc = launch_fill_zero(r0, elem * 3 * (size_t)p->num_nodes, s);
        if (rc) return rc;
        if (!hidden) a2 = nullptr;
    } else if (p->num_edges > 0 && r0 == nullptr) {
        return set_error(E3J_AMD_INVALID_ARGUMENT, op + ": null y");
    }
    if (!hidden && !backward) r2 = nullptr;
    if (p->num_edges == 0) return E3J_AMD_OK;
    if (pos == nullptr || sender == nullptr || receiver == nullptr || ((backward ? a2 : r2) != nullptr && w1 == nullptr))
        return set_error(E3J_AMD_INVALID_ARGUMENT, op + ": null operand");
    const EdgeFeatureSizes sz{p->num_edges, p->num_nodes, p->num_basis, p->hidden, p->layers, (double)p->cutoff};
    if (p->val_dtype == E3J_AMD_F32)
        return dispatch_edge_features<float>(p->l_max, backward, pos, sender, receiver, shift, w1, a0, a1, a2, sz, fac,
                                             r0, r1, r2, s);
    if (p->val_dtype == E3J_AMD_F64)
        return dispatch_edge_features<double>(p->l_max, backward, pos, sender, receiver, shift, w1, a0, a1, a2, sz,
                                              fac, r0, r1, r2, s);
    return set_error(E3J_AMD_INVALID_ARGUMENT, op + ": unsupported value dtype");
}

}  // namespace
}  // namespace e3j_amd

extern "C" {

int e3j_amd_edge_features_fwd(const e3j_amd_edge_features_params *p, const void *positions,
                              const int32_t *sender, const int32_t *receiver, const void *shift,
                              const void *w1, void *y, void *basis, void *h, void *stream) {
    return e3j_amd::run_edge_features(false, p, positions, sender, receiver, shift, w1, nullptr, nullptr, nullptr,
                                      y, basis, h, stream);
}

int e3j_amd_edge_features_bwd(const e3j_amd_edge_features_params *p, const void *positions,
                              const int32_t *sender, const int32_t *receiver, const void *shift,
                              const void *w1, const void *dy, const void *dbasis, const void *dh,
                              void *dpositions, void *stream) {
    return e3j_amd::run_edge_features(true, p, positions, sender, receiver, shift, w1, dy, dbasis, dh, dpositions,
                                      nullptr, nullptr, stream);
}


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
