// Merge of split-KV partial results (algorithm of csrc/flash_fwd_kernel.h:1212-1235 and :1264-1283 in the
// reference, evaluated in base 2 because the forward kernels keep log2-domain statistics).
#pragma once
#include "intfa_device.h"

namespace intfa {

// D / 4 lanes per output row (one 16-byte load per lane and split, one 8-byte store), 256 / (D / 4) rows per workgroup;
// the loads of four splits are in flight together.
template <int D, int OUT_DT>
__global__ void __launch_bounds__(256) splitkv_combine_kernel(const KParams p) {
    constexpr int LPR = D / 4, RPB = 256 / LPR;
    const int sub = threadIdx.x % LPR, rl = threadIdx.x / LPR;
    const int64_t rows = (int64_t)p.batch * p.heads * p.seqlen;
    const int64_t row = (int64_t)blockIdx.x * RPB + rl;
    if (row >= rows) return;
    const int ns = p.num_splits;
    // log-sum-exp over splits (every lane of a row computes the same scalars)
    float lse_max = -INFINITY;
    for (int s = 0; s < ns; ++s) lse_max = fmaxf(lse_max, p.lse_part[(int64_t)s * rows + row]);
    // A row no split saw a key for (an empty cache entry, a causal row above the first key): every partial is -inf and
    // the result is zeros with lse = -inf, the value the single-pass kernels write for such a row - the neutral element
    // for a caller that merges results by lse.
    const bool empty = lse_max == -INFINITY;
    if (empty) lse_max = 0.f;
    float sum = 0.f;
    for (int s = 0; s < ns; ++s) sum += fast_exp2(p.lse_part[(int64_t)s * rows + row] - lse_max);
    const float lse = empty ? -INFINITY : __builtin_log2f(sum) + lse_max;     // (a NaN partial propagates as NaN)
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    const float* op0 = p.o_part + row * D + sub * 4;
    const int64_t sstride = rows * D;
    for (int s0 = 0; s0 < ns; s0 += 4) {
        v4f part[4];
        float w[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int s = s0 + u < ns ? s0 + u : ns - 1;                 // clamped loads, zero weight past the end
            part[u] = *(const v4f*)(op0 + (int64_t)s * sstride);
            w[u] = (s0 + u < ns && !empty) ? fast_exp2(p.lse_part[(int64_t)s * rows + row] - lse) : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = fmaf(w[u], part[u][i], acc[i]);
    }
    const int64_t bh = row / p.seqlen, n = row % p.seqlen;
    const int64_t b = bh / p.heads, h = bh % p.heads;
    char* orow = p.out + b * p.o_sb + h * p.o_sh + n * p.o_sn + sub * 8;
    if (OUT_DT == 0) {
        v4h o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = (_Float16)acc[i];
        *(v4h*)orow = o;
    } else {
        v4s o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = f32_to_bf16(acc[i]);
        *(v4s*)orow = o;
    }
    if (p.lse != nullptr && sub == 0) p.lse[row] = lse;
}

}  // namespace intfa
