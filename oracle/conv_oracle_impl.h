/* The loops of conv_oracle.c, written once for the value type REAL; conv_oracle.c includes this
 * file for float (the reference's arithmetic: the checker and the timed CPU baseline) and for
 * double (the same loops as the exact reference of the full-size tests).
 * TEST INFRASTRUCTURE ONLY, like conv_oracle.c. */
void FN(conv_oracle_fwd)(const int32_t *ci, const int32_t *cj, const int32_t *ck, const REAL *cv,
                     int32_t nnz, const int32_t *mix_idx,
                     const REAL *x, const REAL *y, const REAL *s,
                     const int32_t *sender, const int32_t *receiver,
                     int32_t num_nodes, int64_t num_edges,
                     int32_t X, int32_t Y, int32_t S, int32_t Z, int32_t K, REAL *out) {
    int64_t *ptr = (int64_t *)malloc(sizeof(int64_t) * ((size_t)num_nodes + 1));
    int64_t *order = (int64_t *)malloc(sizeof(int64_t) * (size_t)(num_edges > 0 ? num_edges : 1));
    group_edges(receiver, sender, num_edges, num_nodes, ptr, order);
    memset(out, 0, sizeof(REAL) * (size_t)num_nodes * Z * K);
#pragma omp parallel
    {
        REAL *msg = (REAL *)malloc(sizeof(REAL) * (size_t)Z);
#pragma omp for schedule(dynamic, 16)
        for (int32_t r = 0; r < num_nodes; r++) {
            for (int64_t p = ptr[r]; p < ptr[r + 1]; p++) {
                int64_t e = order[p];
                const REAL *xe = x + (size_t)sender[e] * X * K;
                const REAL *ye = y + (size_t)e * Y;
                const REAL *se = s + (size_t)e * S * K;
                REAL *orow = out + (size_t)r * Z * K;
                for (int32_t c = 0; c < K; c++) {
                    for (int32_t i = 0; i < Z; i++) msg[i] = (REAL)0;
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

void FN(conv_oracle_bwd)(const int32_t *ci, const int32_t *cj, const int32_t *ck, const REAL *cv,
                     int32_t nnz, const int32_t *mix_idx,
                     const REAL *x, const REAL *y, const REAL *s, const REAL *dm,
                     const int32_t *sender, const int32_t *receiver,
                     int32_t num_nodes, int64_t num_edges,
                     int32_t X, int32_t Y, int32_t S, int32_t Z, int32_t K,
                     REAL *dx, REAL *dy, REAL *ds) {
    memset(dx, 0, sizeof(REAL) * (size_t)num_nodes * X * K);
    memset(dy, 0, sizeof(REAL) * (size_t)num_edges * Y);
    memset(ds, 0, sizeof(REAL) * (size_t)num_edges * S * K);
    /* edge-local cotangents: dy, ds */
#pragma omp parallel
    {
        REAL *g = (REAL *)malloc(sizeof(REAL) * (size_t)Z);
#pragma omp for schedule(dynamic, 64)
        for (int64_t e = 0; e < num_edges; e++) {
            if (!live(sender[e], num_nodes) || !live(receiver[e], num_nodes)) continue;
            const REAL *xe = x + (size_t)sender[e] * X * K;
            const REAL *ze = dm + (size_t)receiver[e] * Z * K;
            const REAL *ye = y + (size_t)e * Y;
            const REAL *se = s + (size_t)e * S * K;
            REAL *dse = ds + (size_t)e * S * K;
            REAL *dye = dy + (size_t)e * Y;
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
        REAL *g = (REAL *)malloc(sizeof(REAL) * (size_t)Z);
#pragma omp for schedule(dynamic, 16)
        for (int32_t nd = 0; nd < num_nodes; nd++) {
            REAL *dxn = dx + (size_t)nd * X * K;
            for (int64_t p = sptr[nd]; p < sptr[nd + 1]; p++) {
                int64_t e = sorder[p];
                const REAL *ze = dm + (size_t)receiver[e] * Z * K;
                const REAL *ye = y + (size_t)e * Y;
                const REAL *se = s + (size_t)e * S * K;
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
