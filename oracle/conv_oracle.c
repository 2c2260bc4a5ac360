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

void conv_oracle_fwd(const int32_t *ci, const int32_t *cj, const int32_t *ck, const float *cv,
                     int32_t nnz, const int32_t *mix_idx,
                     const float *x, const float *y, const float *s,
                     const int32_t *sender, const int32_t *receiver,
                     int32_t num_nodes, int64_t num_edges,
                     int32_t X, int32_t Y, int32_t S, int32_t Z, int32_t K, float *out) {
    int64_t *ptr = (int64_t *)malloc(sizeof(int64_t) * ((size_t)num_nodes + 1));
    int64_t *order = (int64_t *)malloc(sizeof(int64_t) * (size_t)(num_edges > 0 ? num_edges : 1));
    group_edges(receiver, sender, num_edges, num_nodes, ptr, order);
    memset(out, 0, sizeof(float) * (size_t)num_nodes * Z * K);
#pragma omp parallel
    {
        float *msg = (float *)malloc(sizeof(float) * (size_t)Z);
#pragma omp for schedule(dynamic, 16)
        for (int32_t r = 0; r < num_nodes; r++) {
            for (int64_t p = ptr[r]; p < ptr[r + 1]; p++) {
                int64_t e = order[p];
                const float *xe = x + (size_t)sender[e] * X * K;
                const float *ye = y + (size_t)e * Y;
                const float *se = s + (size_t)e * S * K;
                float *orow = out + (size_t)r * Z * K;
                for (int32_t c = 0; c < K; c++) {
                    for (int32_t i = 0; i < Z; i++) msg[i] = 0.f;
                    for (int32_t n = 0; n < nnz; n++)
                        msg[ci[n]] += (xe[(size_t)cj[n] * K + c] * ye[ck[n]]) * cv[n];
                    for (int32_t i = 0; i < Z; i++)
                        orow[(size_t)i * K + c] += se[(size_t)mix_idx[i] * K + c] * msg[i];
                }
            }
        }
        free(msg);
    }
    free(ptr);
    free(order);
}

void conv_oracle_bwd(const int32_t *ci, const int32_t *cj, const int32_t *ck, const float *cv,
                     int32_t nnz, const int32_t *mix_idx,
                     const float *x, const float *y, const float *s, const float *dm,
                     const int32_t *sender, const int32_t *receiver,
                     int32_t num_nodes, int64_t num_edges,
                     int32_t X, int32_t Y, int32_t S, int32_t Z, int32_t K,
                     float *dx, float *dy, float *ds) {
    memset(dx, 0, sizeof(float) * (size_t)num_nodes * X * K);
    memset(dy, 0, sizeof(float) * (size_t)num_edges * Y);
    memset(ds, 0, sizeof(float) * (size_t)num_edges * S * K);
    /* edge-local cotangents: dy, ds */
#pragma omp parallel
    {
        float *g = (float *)malloc(sizeof(float) * (size_t)Z);
#pragma omp for schedule(dynamic, 64)
        for (int64_t e = 0; e < num_edges; e++) {
            if (!live(sender[e], num_nodes) || !live(receiver[e], num_nodes)) continue;
            const float *xe = x + (size_t)sender[e] * X * K;
            const float *ze = dm + (size_t)receiver[e] * Z * K;
            const float *ye = y + (size_t)e * Y;
            const float *se = s + (size_t)e * S * K;
            float *dse = ds + (size_t)e * S * K;
            float *dye = dy + (size_t)e * Y;
            for (int32_t c = 0; c < K; c++) {
                for (int32_t n = 0; n < nnz; n++)
                    dse[(size_t)mix_idx[ci[n]] * K + c] +=
                        ((cv[n] * xe[(size_t)cj[n] * K + c]) * ye[ck[n]]) * ze[(size_t)ci[n] * K + c];
                for (int32_t i = 0; i < Z; i++)
                    g[i] = se[(size_t)mix_idx[i] * K + c] * ze[(size_t)i * K + c];
                for (int32_t n = 0; n < nnz; n++)
                    dye[ck[n]] += (cv[n] * g[ci[n]]) * xe[(size_t)cj[n] * K + c];
            }
        }
        free(g);
    }
    /* dx: rows grouped by sender; within a row, edges in receiver-grouped order */
    int64_t *rptr = (int64_t *)malloc(sizeof(int64_t) * ((size_t)num_nodes + 1));
    int64_t *rorder = (int64_t *)malloc(sizeof(int64_t) * (size_t)(num_edges > 0 ? num_edges : 1));
    int64_t n_live = group_edges(receiver, sender, num_edges, num_nodes, rptr, rorder);
    int64_t *sptr = (int64_t *)malloc(sizeof(int64_t) * ((size_t)num_nodes + 1));
    int64_t *sorder = (int64_t *)malloc(sizeof(int64_t) * (size_t)(num_edges > 0 ? num_edges : 1));
    memset(sptr, 0, sizeof(int64_t) * ((size_t)num_nodes + 1));
    for (int64_t p = 0; p < n_live; p++) sptr[sender[rorder[p]] + 1]++;
    for (int32_t n = 0; n < num_nodes; n++) sptr[n + 1] += sptr[n];
    {
        int64_t *cursor = (int64_t *)malloc(sizeof(int64_t) * ((size_t)num_nodes + 1));
        memcpy(cursor, sptr, sizeof(int64_t) * ((size_t)num_nodes + 1));
        for (int64_t p = 0; p < n_live; p++) sorder[cursor[sender[rorder[p]]]++] = rorder[p];
        free(cursor);
    }
#pragma omp parallel
    {
        float *g = (float *)malloc(sizeof(float) * (size_t)Z);
#pragma omp for schedule(dynamic, 16)
        for (int32_t nd = 0; nd < num_nodes; nd++) {
            float *dxn = dx + (size_t)nd * X * K;
            for (int64_t p = sptr[nd]; p < sptr[nd + 1]; p++) {
                int64_t e = sorder[p];
                const float *ze = dm + (size_t)receiver[e] * Z * K;
                const float *ye = y + (size_t)e * Y;
                const float *se = s + (size_t)e * S * K;
                for (int32_t c = 0; c < K; c++) {
                    for (int32_t i = 0; i < Z; i++)
                        g[i] = se[(size_t)mix_idx[i] * K + c] * ze[(size_t)i * K + c];
                    for (int32_t n = 0; n < nnz; n++)
                        dxn[(size_t)cj[n] * K + c] += (cv[n] * g[ci[n]]) * ye[ck[n]];
                }
            }
        }
        free(g);
    }
    free(rptr); free(rorder); free(sptr); free(sorder);
}
