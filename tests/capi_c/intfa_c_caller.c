/* A caller of libintfa.so that knows nothing of Python or torch: plain C, the HIP runtime for device memory, and the
 * entry points of include/intfa.h.  It reads q, k, v (int8 [B,H,N,D]), q_scale, k_scale (fp16 [B,H,N]) and v_scale
 * (fp16 [B,H]) from one binary file, runs intfa_fwd_full_int8 (optionally with split-KV and a workspace sized by
 * intfa_fwd_workspace_bytes) and writes the fp16 output [B,H,N,D] to another file.
 *
 *   intfa_c_caller <in.bin> <out.bin> B H N D causal num_splits
 *
 * The GPU test suite runs it and compares the file with what the Python wrapper returns for the same tensors. */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "intfa.h"

#define CHECK_HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); return 2; } } while (0)

static void* upload(FILE* f, size_t bytes) {
    void* host = malloc(bytes);
    void* dev = NULL;
    if (host == NULL || fread(host, 1, bytes, f) != bytes) { fprintf(stderr, "short input file\n"); exit(3); }
    if (hipMalloc(&dev, bytes) != hipSuccess || hipMemcpy(dev, host, bytes, hipMemcpyHostToDevice) != hipSuccess) {
        fprintf(stderr, "upload failed\n"); exit(2);
    }
    free(host);
    return dev;
}

int main(int argc, char** argv) {
    if (argc != 9) { fprintf(stderr, "usage: %s in.bin out.bin B H N D causal num_splits\n", argv[0]); return 1; }
    const int B = atoi(argv[3]), H = atoi(argv[4]), N = atoi(argv[5]), D = atoi(argv[6]);
    const int causal = atoi(argv[7]), splits = atoi(argv[8]);
    const size_t rows = (size_t)B * H * N, elems = rows * D;
    FILE* f = fopen(argv[1], "rb");
    if (f == NULL) { perror(argv[1]); return 1; }
    if (intfa_version() != INTFA_VERSION) { fprintf(stderr, "header/library version mismatch\n"); return 4; }

    intfa_fwd_params p = {0};
    p.q = upload(f, elems); p.k = upload(f, elems); p.v = upload(f, elems);
    p.q_scale = upload(f, rows * 2); p.k_scale = upload(f, rows * 2); p.v_scale = upload(f, (size_t)B * H * 2);
    fclose(f);
    void* out = NULL;
    CHECK_HIP(hipMalloc(&out, elems * 2));
    p.out = out;
    p.q_stride_b = p.k_stride_b = p.v_stride_b = p.o_stride_b = (int64_t)H * N * D;
    p.q_stride_h = p.k_stride_h = p.v_stride_h = p.o_stride_h = (int64_t)N * D;
    p.q_stride_n = p.k_stride_n = p.v_stride_n = p.o_stride_n = D;
    p.qs_stride_b = p.ks_stride_b = (int64_t)H * N; p.qs_stride_h = p.ks_stride_h = N; p.qs_stride_n = p.ks_stride_n = 1;
    p.vs_stride_b = H; p.vs_stride_h = 1;
    p.batch = B; p.heads = H; p.seqlen = N; p.head_dim = D;
    p.scale_dtype = INTFA_F16; p.io_dtype = INTFA_F16; p.causal = causal;
    p.sm_scale = 1.0f / sqrtf((float)D);
    p.p_round = INTFA_PROUND_RNE;
    p.num_splits = splits;
    if (splits > 1) {
        p.workspace_bytes = intfa_fwd_workspace_bytes(&p);
        CHECK_HIP(hipMalloc(&p.workspace, p.workspace_bytes));
    }
    hipStream_t stream;
    CHECK_HIP(hipStreamCreate(&stream));
    const int rc = intfa_fwd_full_int8(&p, (void*)stream);
    if (rc != 0) { fprintf(stderr, "intfa_fwd_full_int8: %d (%s)\n", rc, intfa_error_string(rc)); return 5; }
    CHECK_HIP(hipStreamSynchronize(stream));

    void* host_out = malloc(elems * 2);
    CHECK_HIP(hipMemcpy(host_out, out, elems * 2, hipMemcpyDeviceToHost));
    FILE* g = fopen(argv[2], "wb");
    if (g == NULL || fwrite(host_out, 1, elems * 2, g) != elems * 2) { perror(argv[2]); return 1; }
    fclose(g);
    printf("ok %zu elements, block_n %d\n", elems, intfa_fwd_block_n(INTFA_VARIANT_FULL_INT8, D));
    return 0;
}
