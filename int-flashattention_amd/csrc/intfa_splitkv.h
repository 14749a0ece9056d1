// Merge of split-KV partial results (algorithm of csrc/flash_fwd_kernel.h:1212-1235 and :1264-1283 in the
// reference, evaluated in base 2 because the forward kernels keep log2-domain statistics).
#pragma once
#include "intfa_device.h"

namespace intfa {

// One wavefront per output row: lane l owns head_dim/64 ... elements; 4 rows per 256-thread workgroup.
template <int D, int OUT_DT>
__global__ void __launch_bounds__(256) splitkv_combine_kernel(const KParams p) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t rows = (int64_t)p.batch * p.heads * p.seqlen;
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;
    if (row >= rows) return;
    const int ns = p.num_splits;
    // log-sum-exp over splits (every lane computes the same scalars)
    float lse_max = -INFINITY;
    for (int s = 0; s < ns; ++s) lse_max = fmaxf(lse_max, p.lse_part[(int64_t)s * rows + row]);
    if (lse_max == -INFINITY) lse_max = 0.f;
    float sum = 0.f;
    for (int s = 0; s < ns; ++s) sum += fast_exp2(p.lse_part[(int64_t)s * rows + row] - lse_max);
    const float lse = (sum == 0.f || sum != sum) ? INFINITY : __builtin_log2f(sum) + lse_max;
    constexpr int PER = D / 64;                     // consecutive elements per lane
    float acc[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) acc[i] = 0.f;
    for (int s = 0; s < ns; ++s) {
        const float w = fast_exp2(p.lse_part[(int64_t)s * rows + row] - lse);
        const float* op = p.o_part + ((int64_t)s * rows + row) * D + lane * PER;
#pragma unroll
        for (int i = 0; i < PER; ++i) acc[i] = fmaf(w, op[i], acc[i]);
    }
    const int64_t bh = row / p.seqlen, n = row % p.seqlen;
    const int64_t b = bh / p.heads, h = bh % p.heads;
    char* orow = p.out + b * p.o_sb + h * p.o_sh + n * p.o_sn + lane * PER * 2;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        if (OUT_DT == 0) {
            ((_Float16*)orow)[i] = (_Float16)acc[i];
        } else {
            ((uint16_t*)orow)[i] = (uint16_t)f32_to_bf16_bits(acc[i]);
        }
    }
    if (p.lse != nullptr && lane == 0) p.lse[row] = lse;
}

}  // namespace intfa
