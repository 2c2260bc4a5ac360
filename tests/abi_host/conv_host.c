/* A host program in plain C that drives the convolution through the C ABI alone (no Python, no
 * torch): what a binding in another host language does.  It reads a problem from a file, looks
 * the table up among the compiled signatures, builds the receiver CSR on the device, runs the
 * forward pass and the receiver-grouped backward pass and writes the results to a second file.
 * tests/test_gpu_abi_host.py writes the problem and checks the results against the CPU checker.
 *
 * problem file: int32[10] = {nodes, edges, channels, X, Y, Z, S, coefficients, index bytes, layout},
 * then the packed table, x, y, s, dm (float32) and sender, receiver (int32), in that order.
 * result file: out, dx, dy, ds (float32). */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "e3j_amd.h"

#define CHECK_HIP(call)                                                                    \
    do {                                                                                   \
        hipError_t err_ = (call);                                                          \
        if (err_ != hipSuccess) {                                                          \
            fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(err_));                  \
            return 3;                                                                      \
        }                                                                                  \
    } while (0)
#define CHECK_LIB(call)                                                                    \
    do {                                                                                   \
        int rc_ = (call);                                                                  \
        if (rc_ != E3J_AMD_OK) {                                                           \
            fprintf(stderr, "%s: code %d: %s\n", #call, rc_, e3j_amd_last_error());      \
            return 4;                                                                      \
        }                                                                                  \
    } while (0)

static void *read_block(FILE *f, size_t bytes) {
    void *p = malloc(bytes ? bytes : 1);
    if (p == NULL || fread(p, 1, bytes, f) != bytes) {
        fprintf(stderr, "short problem file\n");
        exit(2);
    }
    return p;
}

static int to_device(void **dev, const void *host, size_t bytes) {
    CHECK_HIP(hipMalloc(dev, bytes ? bytes : 4));
    if (bytes) CHECK_HIP(hipMemcpy(*dev, host, bytes, hipMemcpyHostToDevice));
    return 0;
}

static int from_device(FILE *f, const void *dev, size_t bytes) {
    void *host = malloc(bytes ? bytes : 1);
    if (host == NULL) return 2;
    if (bytes) CHECK_HIP(hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost));
    if (fwrite(host, 1, bytes, f) != bytes) return 2;
    free(host);
    return 0;
}

int main(int argc, char **argv) {
    if (argc != 3) {
        fprintf(stderr, "usage: %s problem.bin result.bin\n", argv[0]);
        return 2;
    }
    FILE *in = fopen(argv[1], "rb");
    if (in == NULL) { perror(argv[1]); return 2; }
    int32_t *h = (int32_t *)read_block(in, 10 * sizeof(int32_t));
    const int32_t N = h[0], K = h[2], X = h[3], Y = h[4], Z = h[5], S = h[6], nnz = h[7];
    const int32_t idx_bytes = h[8], layout = h[9];
    const int64_t E = h[1];
    const size_t entry = idx_bytes == 1 ? 8 : 32;  /* float32 values: packed entry size */
    const size_t nx = (size_t)N * X * K, ny = (size_t)E * Y, ns = (size_t)E * S * K, nz = (size_t)N * Z * K;
    void *coef = read_block(in, entry * nnz);
    float *x = (float *)read_block(in, 4 * nx), *y = (float *)read_block(in, 4 * ny);
    float *s = (float *)read_block(in, 4 * ns), *dm = (float *)read_block(in, 4 * nz);
    int32_t *sender = (int32_t *)read_block(in, 4 * (size_t)E);
    int32_t *receiver = (int32_t *)read_block(in, 4 * (size_t)E);
    fclose(in);

    e3j_amd_conv_params p;
    p.num_nodes = N; p.num_edges = E; p.num_coef = nnz; p.num_x = X; p.num_y = Y; p.num_out = Z;
    p.num_scalars = S; p.channels = K; p.layout = layout; p.val_dtype = E3J_AMD_F32;
    p.coef_idx_bytes = idx_bytes; p.debug = 1; p.coef_scale = 1.0f; p.y_flip = 0; p.row_order = NULL;
    p.signature = e3j_amd_find_signature(coef, idx_bytes, E3J_AMD_F32, nnz, X, Y, Z, S, K, layout,
                                         &p.coef_scale, &p.y_flip);
    printf("signature %d (%s)\n", p.signature,
           p.signature >= 0 ? e3j_amd_signature_name(p.signature) : "table-driven kernels");
    if (p.signature < 0) { p.coef_scale = 1.0f; p.y_flip = 0; }

    void *d_coef, *d_x, *d_y, *d_s, *d_dm, *d_sender, *d_receiver, *d_ptr, *d_ws;
    void *d_out, *d_dx, *d_dy, *d_ds;
    if (to_device(&d_coef, coef, entry * nnz) || to_device(&d_x, x, 4 * nx) || to_device(&d_y, y, 4 * ny) ||
        to_device(&d_s, s, 4 * ns) || to_device(&d_dm, dm, 4 * nz) ||
        to_device(&d_sender, sender, 4 * (size_t)E) || to_device(&d_receiver, receiver, 4 * (size_t)E))
        return 3;
    CHECK_HIP(hipMalloc(&d_ptr, 4 * ((size_t)N + 1)));
    CHECK_HIP(hipMalloc(&d_ws, e3j_amd_csr_workspace_bytes(N, E)));
    CHECK_HIP(hipMalloc(&d_out, 4 * nz + 4));
    CHECK_HIP(hipMalloc(&d_dx, 4 * nx + 4));
    CHECK_HIP(hipMalloc(&d_dy, 4 * ny + 4));
    CHECK_HIP(hipMalloc(&d_ds, 4 * ns + 4));

    hipStream_t stream;
    CHECK_HIP(hipStreamCreate(&stream));
    CHECK_LIB(e3j_amd_csr_row_ptr((const int32_t *)d_receiver, E, N, (int32_t *)d_ptr, d_ws, stream));
    CHECK_LIB(e3j_amd_convolution_fwd(&p, d_coef, d_x, d_y, d_s, (const int32_t *)d_sender,
                                      (const int32_t *)d_ptr, NULL, d_out, stream));
    CHECK_LIB(e3j_amd_convolution_bwd_receiver(&p, d_coef, d_x, d_y, d_s, d_dm, (const int32_t *)d_sender,
                                               (const int32_t *)d_ptr, NULL, d_dx, d_dy, d_ds, stream));
    CHECK_HIP(hipStreamSynchronize(stream));

    FILE *out = fopen(argv[2], "wb");
    if (out == NULL) { perror(argv[2]); return 2; }
    if (from_device(out, d_out, 4 * nz) || from_device(out, d_dx, 4 * nx) || from_device(out, d_dy, 4 * ny) ||
        from_device(out, d_ds, 4 * ns))
        return 3;
    fclose(out);
    CHECK_HIP(hipStreamDestroy(stream));
    return 0;
}
