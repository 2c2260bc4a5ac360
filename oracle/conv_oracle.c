/* CPU restatement (plain C, float32) of the reference's convolution loops.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels and the timed
 * CPU baseline of bench.py.  Nothing in the product links or loads it.
 *
 * Forward follows cpu_convolution (lib/e3j_ops/tests/test_convolution.cpp:63-106)
 * with the operation order of the unfused path
 * (src/e3j/core/convolution.py:172-191, src/e3j/core/tensor_product.py:316-319):
 *   msg[i] += (x[send,j,c] * y[e,k]) * v ; out[recv,i,c] += s[e,l(i),c] * msg[i].
 * Backward follows cpu_convolution_bwd
 * (lib/e3j_ops/tests/test_convolution_bwd.cpp:111-182): ds, then g = s*dz, dx, dy.
 *
 * Edges arrive as COO (sender, receiver) in any order; an edge with an endpoint
 * outside [0, num_nodes) contributes nothing and keeps dy = ds = 0
 * (lib/e3j_ops/cuda/convolution/bwd.cuh:225-226,308-319).  Layout: trailing
 * channels, x (N, X, K), y (E, Y), s (E, S, K), out/dm (N, Z, K).
 * Rows are visited in a stable receiver-grouped order, so every sum runs in the
 * order of the reference loops; OpenMP only splits independent rows.
 * Pinned by tests/test_oracle.py against the numpy restatement, the literal
 * Python loops and the closed-form strip case.
 *
 * The loops live in conv_oracle_impl.h and are compiled twice: conv_oracle_fwd / conv_oracle_bwd in
 * float (above), conv_oracle_fwd_f64 / conv_oracle_bwd_f64 with every value in double (same loops,
 * same order): the exact reference the float32 results of full-size runs are compared with.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static int live(int32_t a, int32_t n) { return a >= 0 && a < n; }

/* stable counting sort of live edges by key; returns ptr (n+1) and order (count) */
static int64_t group_edges(const int32_t *key, const int32_t *other, int64_t num_edges,
                           int32_t num_nodes, int64_t *ptr, int64_t *order) {
    memset(ptr, 0, sizeof(int64_t) * ((size_t)num_nodes + 1));
    for (int64_t e = 0; e < num_edges; e++)
        if (live(key[e], num_nodes) && live(other[e], num_nodes)) ptr[key[e] + 1]++;
    for (int32_t n = 0; n < num_nodes; n++) ptr[n + 1] += ptr[n];
    int64_t *cursor = (int64_t *)malloc(sizeof(int64_t) * ((size_t)num_nodes + 1));
    memcpy(cursor, ptr, sizeof(int64_t) * ((size_t)num_nodes + 1));
    for (int64_t e = 0; e < num_edges; e++)
        if (live(key[e], num_nodes) && live(other[e], num_nodes)) order[cursor[key[e]]++] = e;
    free(cursor);
    return ptr[num_nodes];
}

#define REAL float
#define FN(name) name
#include "conv_oracle_impl.h"
#undef REAL
#undef FN

#define REAL double
#define FN(name) name##_f64
#include "conv_oracle_impl.h"
#undef REAL
#undef FN
