// Half-int8 and fp16/bf16 forward for few query rows per head (decoding against a key/value cache, Nq << Nk).
//
// Same arithmetic as fwd_f16pv_kernel (flash_atten_int8.py:9-66, flash_atten_fp.py:9-60 per 64-key block: S, running
// max, P = exp2(S c - m) cast to V's 16-bit type, fp32 accumulator scaled by alpha and P V added on top), other division
// of labour - the one of fwd_decode_full_int8_kernel.  One workgroup owns 32 query rows; its four waves share the keys.
//
// Head_dim 64: a step covers TWO consecutive 64-key blocks A and B (128 keys),
//   * wave w computes S^T for keys 32w .. 32w+31 of the step (waves 0, 1: block A; waves 2, 3: block B), dequantises and
//     takes the partial row maxima;
//   * the four partial maxima meet in LDS (barrier); every wave then knows both blocks' running maxima
//     m_A = max(m, max_A), m_B = max(m_A, max_B) and both factors alpha_A = 2^(m - m_A), alpha_B = 2^(m_A - m_B);
//   * wave w exponentiates its 32 keys against its block's maximum, casts to 16 bits and publishes two MFMA operands
//     in LDS (barrier);
//   * waves 0 and 1 own 32 output columns each: O = (O alpha_A + P_A V_A) alpha_B + P_B V_B with all eight operands.
// Head_dim 128 and 256: a step is ONE 64-key block.  Waves 0 and 1 compute S^T and P for its two 32-key sub-tiles,
// waves 2 and 3 only pass the barriers in that phase (the pass is bound by the stream of K and V, not by the arithmetic),
// every wave owns one (two at head_dim 256) 32-column output tile.  The smaller step is what the stream wants there: 24
// to 32 KiB of tiles per step let two or three workgroups share a compute unit at head_dim 128 (6.0 TB/s of K+V against
// 5.4 - 5.9 with 128-key steps and one workgroup), and at head_dim 256 two steps of 128 keys would not fit the LDS.
// Every block is evaluated with the same maximum, the same P and the same order of MFMA steps as in the general kernel;
// only the row sums are added in another order (per wave, joined in the epilogue).  K/V tiles of a step are
// double-buffered in LDS and the whole next step is requested at the start of a step.
#pragma once
#include "intfa_device.h"
#include "intfa_launch.h"
#include "intfa_fwd_f16pv.h"

namespace intfa {

// QK_INT8: int8 Q/K with per-token scales (half-int8) or 16-bit Q/K.  IO_DT: type of V, P and the output (and of Q/K
// when !QK_INT8): 0 fp16, 1 bf16.  The causal mask is a run-time switch here (p.causal).
template <bool QK_INT8, int D, int IO_DT, bool SPLIT>
__global__ void __launch_bounds__(kThreads, D == 256 ? 1 : (D == 128 && QK_INT8) ? 3 : 2) fwd_decode_f16pv_kernel(const KParams p) {
    static_assert(D == 64 || D == 128 || D == 256, "head dims 64, 128 and 256");
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass only needs the kernel's symbol
    constexpr int BNB = kBlockN16;                    // key block of the arithmetic
    constexpr int NBS = D <= 64 ? 2 : 1;              // key blocks per step
    constexpr int BN = NBS * BNB;                     // keys per step
    constexpr int QKW = BN / 32;                      // waves with a 32-key sub-tile of S^T (all four, or waves 0 and 1)
    constexpr int NG = BN / 16;                       // 16-key MFMA steps of P V per step (two per wave's sub-tile)
    constexpr int QB = QK_INT8 ? 1 : 2;               // bytes per Q/K element
    constexpr int KROW = D * QB, VROW = D * 2;
    constexpr int KS = KROW / 32;                     // MFMA k-steps of S^T
    constexpr int DT = D / 32;                        // 32-wide output tiles; wave w owns tiles w, w + 4 (head_dim 64: waves 0, 1)
    constexpr int DTW = (DT + 3) / 4;                 // output tiles per wave
    constexpr int KT = BN * KROW, VT = BN * VROW;
    constexpr int KCH = KROW / 16, VCH = VROW / 16;
    // LDS map (bytes)
    constexpr int OFF_KS = 0;                             // two fp32 k_scale vectors
    constexpr int OFF_XM = 2 * BN * 4;                    // 4 waves x 32 rows fp32: partial row maxima / row sums
    constexpr int OFF_XP = OFF_XM + 4 * 32 * 4;           // NG operands of 64 lanes x 16 bytes: the waves' 16-bit P
    static_assert(QKW == 4 || QKW == 2, "a step is four or two 32-key sub-tiles");
    constexpr int OFF_K = OFF_XP + NG * 1024;
    constexpr int OFF_V = OFF_K + 2 * KT;
    constexpr int LDS_BYTES = OFF_V + 2 * VT;
    static_assert(OFF_K % 256 == 0, "tiles keep the bank alignment the swizzles assume");
    static_assert(LDS_BYTES <= 160 * 1024, "one workgroup fits the LDS of a compute unit");
    __shared__ __attribute__((aligned(1024))) char smem[LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lq = lane & 31, lh = lane >> 5;

    // ---- block -> (head, 32-row query block, split)
    const int n_mblk = (p.seqlen + kDecodeRows - 1) / kDecodeRows;
    const int n_split = SPLIT ? p.num_splits : 1;
    const WorkgroupJob wg = deal_workgroup(p, blockIdx.x);
    const int rem = wg.rem, head = wg.b * p.heads + wg.h;
    const int mb = fast_div(rem, p.d_n_split), split = rem - mb * n_split;
    const int b = wg.b, h = wg.h;
    const int hk = wg.hk;

    const int seqlen_k = keys_of_batch(p, b);
    // causal: the row at position i sees keys 0 .. i + causal_off (mask aligned to the bottom right corner)
    // (causal_rows: the rows hold several query heads of one K/V group, causal_rows positions each)
    const int fold = p.causal_rows;
    const int causal_off = seqlen_k - (fold ? fold : p.seqlen);
    // (a split takes blocks_per_split 64-key blocks of the whole key range: every row of a decode-shaped problem sees
    // nearly all keys)
    const KeyBlocks kb = key_block_range<BNB>(seqlen_k, p.causal != 0, fold ? fold : mb * kDecodeRows + kDecodeRows, causal_off, SPLIT,
                                              n_split, split, false, p.blocks_per_split);
    const int nb_begin = kb.begin, nb_end = kb.end;
    const int key_end = nb_end * BNB < seqlen_k ? nb_end * BNB : seqlen_k;      // one past the last key of the range
    const int q_row = mb * kDecodeRows + lq;
    const bool q_valid = q_row < p.seqlen;
    const int q_ld = q_valid ? q_row : p.seqlen - 1;

    // ---- Q fragments (B operand of S^T = K Q^T), the same 32 rows in every wave
    v4i qreg[KS];
    {
        const char* qrow = p.q + b * p.q_sb + h * p.q_sh + (int64_t)q_ld * p.q_sn;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qreg[ks] = *(const v4i*)(qrow + ks * 32 + lh * 16);
    }
    const float qsc = QK_INT8 ? load_q_scale_log2(p, b, h, q_ld) : p.qk_scale_log2;

    float m_run = -INFINITY, l_run = 0.f;        // l_run: this wave's keys only
    v16f o_acc[DTW];
#pragma unroll
    for (int j = 0; j < DTW; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[j][r] = 0.f;

    // ---- global -> LDS copies (asynchronous, straight into LDS; the four waves split the instructions)
    const char* Kg = p.k + b * p.k_sb + hk * p.k_sh;
    const char* Vg = p.v + b * p.v_sb + hk * p.v_sh;
    const v4i k_rsrc = make_rsrc(Kg, (uint32_t)((seqlen_k - 1) * p.k_sn + KROW));
    const v4i v_rsrc = make_rsrc(Vg, (uint32_t)((seqlen_k - 1) * p.v_sn + VROW));
    const uint32_t k_sn = (uint32_t)p.k_sn, v_sn = (uint32_t)p.v_sn;
    const auto k_lane = tile_load_lane<KROW, SWZ_K, BN>(k_sn, wave, lane);
    const auto v_lane = tile_load_lane<VROW, SWZ_V16, BN>(v_sn, wave, lane);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    auto issue_loads = [&](int nb, int buf) __attribute__((always_inline)) {
        issue_tile_load<KROW, SWZ_K, BN>(k_rsrc, (uint32_t)(nb * BNB) * k_sn, k_sn, lds0 + OFF_K + buf * KT, wave, k_lane);
        issue_tile_load<VROW, SWZ_V16, BN>(v_rsrc, (uint32_t)(nb * BNB) * v_sn, v_sn, lds0 + OFF_V + buf * VT, wave, v_lane);
    };
    // k_scale of a step: thread t < 128 fetches the scale of key t; converted to fp32 when stored to LDS
    const KScaleSource ks_src(p, b, hk, seqlen_k);
    const bool ks_wave = wave < BN / 64;              // threads 0 .. BN-1 fetch one k_scale each (a scalar test: see fwd_full_int8_kernel)
    auto load_ks = [&](int nb) __attribute__((always_inline)) -> uint32_t {
        return (!QK_INT8 || !ks_wave) ? 0u : ks_src.load(nb * BNB + tid);
    };
    auto cvt_ks = [&](uint32_t raw) __attribute__((always_inline)) -> float { return ks_src.cvt(raw); };

    // ---- per-lane LDS offsets
    const int k_swz = swz_k<KROW>(lq) & (KCH - 1);
    uint32_t k_rd[KS];                            // this wave's 32 keys: row 32*wave + lq, chunk 2*ks + lh
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_rd[ks] = OFF_K + (32 * wave + lq) * KROW + (((2 * ks + lh) ^ k_swz) << 4);
    // V through ds_read_b64_tr_b16 (see fwd_f16pv_kernel): source lane s of a 16-lane group points at key row s >> 2 of a
    // run of four consecutive keys and at four head-dim values of the wave's output tile
    const int g16 = lane >> 4, s16 = lane & 15;
    const int v_row0 = 4 * lh + (s16 >> 2);           // + 8 for the second load, + 16 per MFMA step
    const int v_swz = swz_v16<VROW>(v_row0) & (VCH - 1);
    const bool own_tile = DT >= 4 || wave < DT;       // head_dim 64: waves 2 and 3 own no output tile
    const bool qk_wave = wave < QKW;                  // this wave computes a sub-tile of S^T and its P
    uint32_t v_rd[DTW];
#pragma unroll
    for (int j = 0; j < DTW; ++j) {
        const int dt = own_tile ? wave + 4 * j : 0;
        const int v_c = 4 * dt + 2 * (g16 & 1) + ((s16 & 3) >> 1);
        v_rd[j] = OFF_V + v_row0 * VROW + ((v_c ^ v_swz) << 4) + 8 * (s16 & 1);
    }
    const uint32_t ks_rd = OFF_KS + 4 * (32 * wave) + 16 * lh;       // + 4 * 8*a4 per read
    const uint32_t ks_wr = OFF_KS + 4 * (tid & (BN - 1));
    const uint32_t xm_wr = OFF_XM + 4 * (32 * wave + lq);
    const uint32_t xm_rd = OFF_XM + 4 * lq;                          // + 128 per wave
    const uint32_t xp_wr = OFF_XP + 2048 * wave + 16 * lane;         // + 1024 for the second operand
    const uint32_t xp_rd = OFF_XP + 16 * lane;                       // + 1024 per MFMA step
    // the smallest and this lane's own last visible key
    const int first_lim = p.causal ? (fold ? 0 : mb * kDecodeRows) + causal_off : 0x3fffffff;
    const int row_lim = p.causal ? (fold ? q_row % fold : q_row) + causal_off : 0x3fffffff;
    const bool blk_a = NBS == 1 || wave < 2;          // this wave's keys belong to the first block of a step

    auto mfma16 = [&](v4i a, v4i bb, v16f c) __attribute__((always_inline)) -> v16f {
        if (IO_DT == 0) return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, bb), c, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, bb), c, 0, 0, 0);
    };

    // One step: the 64-key blocks nb and nb + 1 (the second one may lie past the end of the range: its keys are masked)
    auto step = [&](auto buf_tag, int nb) __attribute__((always_inline)) {
        constexpr int BUF = decltype(buf_tag)::value ? 1 : 0;
        constexpr int KB = BUF * KT, VB = BUF * VT, SB = BUF * BN * 4;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();                                   // the tiles have landed; the other buffer and the exchange areas are free
        const bool more = nb + NBS < nb_end;
        uint32_t ks_next = 0;
        if (more) {
            issue_loads(nb + NBS, BUF ^ 1);
            ks_next = load_ks(nb + NBS);
        }
        // -------- S^T of this wave's 32 keys, dequantise, partial row maximum
        v4i fr[KS];
        v4f kk[4];
        v16i si = (v16i){0};
        v16f sf = (v16f){0};
        if (qk_wave) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) fr[ks] = *(const v4i*)(smem + k_rd[ks] + KB);
            if (QK_INT8) {
#pragma unroll
                for (int a4 = 0; a4 < 4; ++a4) kk[a4] = *(const v4f*)(smem + ks_rd + SB + 4 * 8 * a4);
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                if (QK_INT8) si = __builtin_amdgcn_mfma_i32_32x32x32_i8(fr[ks], qreg[ks], si, 0, 0, 0);
                else sf = mfma16(fr[ks], qreg[ks], sf);
            }
        }
        // V fragments of this wave's output tiles (all keys of the step) travel during the softmax
        v4i vf[DTW][NG];
        if (own_tile) {
#pragma unroll
            for (int j = 0; j < DTW; ++j)
#pragma unroll
                for (int g = 0; g < NG; ++g) {
                    const uint32_t a0 = v_rd[j] + VB + 16 * g * VROW;
                    const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)INTFA_LDS(smem + a0));
                    const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)INTFA_LDS(smem + a0 + 8 * VROW));
                    vf[j][g] = (v4i){__builtin_bit_cast(v2i, lo)[0], __builtin_bit_cast(v2i, lo)[1], __builtin_bit_cast(v2i, hi)[0], __builtin_bit_cast(v2i, hi)[1]};
                }
        }
        const int key0 = nb * BNB;
        // masked steps (wave-uniform test): keys past the end of the range, or past the first row's position
        const bool tail = key0 + BN > key_end || key0 + BN - 1 > first_lim;
        // keys of this lane with 8*a4 + b4 >= key_lim are hidden
        const int last_key = (row_lim < key_end - 1 ? row_lim : key_end - 1) - key0;
        const int key_lim = last_key + 1 - 32 * wave - 4 * lh;
        float x[16];
        float mx = -INFINITY;
        if (qk_wave) {
#pragma unroll
            for (int r = 0; r < 16; ++r) x[r] = QK_INT8 ? (float)si[r] * kk[r >> 2][r & 3] : sf[r];
            if (tail) {
                // (a branch of its own, kept one by the empty statement: see fwd_decode_full_int8_kernel)
                asm volatile("");
#pragma unroll
                for (int r = 0; r < 16; ++r) x[r] = hide_past(x[r], key_lim - 1, 8 * (r >> 2) + (r & 3));
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, x[r]);
            mx = half_pair_max(mx);
            if (lh == 0) *(float*)(smem + xm_wr) = mx;
        }
        __syncthreads();                                   // the partial maxima are in LDS
        const float mx_a = fmaxf(*(const float*)(smem + xm_rd), *(const float*)(smem + xm_rd + 128));
        const float m_a = fmaxf(m_run, mx_a * qsc);
        const float alpha_a = fast_exp2(m_run - m_a);
        float m_b = m_a, alpha_b = 1.f;                    // one block per step: no second factor
        if (NBS == 2) {
            const float mx_b = fmaxf(*(const float*)(smem + xm_rd + 256), *(const float*)(smem + xm_rd + 384));
            m_b = fmaxf(m_a, mx_b * qsc);
            alpha_b = fast_exp2(m_a - m_b);
        }
        m_run = m_b;
        // -------- P of this wave's keys in 16 bits; partial row sum
        const float m_own = blk_a ? m_a : m_b;
        float lsum = 0.f;
        if (qk_wave) {
            float e[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                e[r] = fast_exp2(fmaf(x[r], qsc, -m_own));
                lsum += e[r];
            }
#pragma unroll
            for (int u = 0; u < 2; ++u)
                *(v4i*)(smem + xp_wr + 1024 * u) = IO_DT == 0 ? __builtin_bit_cast(v4i, pack_p_f16(e + 8 * u))
                                                              : __builtin_bit_cast(v4i, pack_p_bf16(e + 8 * u));
        }
        __syncthreads();                                   // the P operands are in LDS
        // -------- this wave's output columns: O^T[d, q] = (O^T alpha_A + V_A^T P_A^T) alpha_B + V_B^T P_B^T
        if (own_tile) {
            v4i pall[NG];
#pragma unroll
            for (int g = 0; g < NG; ++g) pall[g] = *(const v4i*)(smem + xp_rd + 1024 * g);
#pragma unroll
            for (int j = 0; j < DTW; ++j) {
#pragma unroll
                for (int r = 0; r < 16; ++r) o_acc[j][r] *= alpha_a;
#pragma unroll
                for (int g = 0; g < NG / NBS; ++g) o_acc[j] = mfma16(vf[j][g], pall[g], o_acc[j]);
                if (NBS == 2) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) o_acc[j][r] *= alpha_b;
#pragma unroll
                    for (int g = NG / 2; g < NG; ++g) o_acc[j] = mfma16(vf[j][g], pall[g], o_acc[j]);
                }
            }
        }
        if (NBS == 1) l_run = fmaf(l_run, alpha_a, lsum);
        else l_run = blk_a ? fmaf(l_run, alpha_a, lsum) * alpha_b : fmaf(l_run * alpha_a, alpha_b, lsum);
        // (the raw scale is made opaque here, behind the step's last barrier: its conversion waits for the load, and with it
        // for the next step's tile copies that were issued ahead of it - that wait belongs at the end of the step)
        if (QK_INT8) asm volatile("" : "+v"(ks_next));
        if (QK_INT8 && more && ks_wave) *(float*)(smem + ks_wr + (BUF ^ 1) * BN * 4) = cvt_ks(ks_next);
    };

    if (nb_begin < nb_end) {
        issue_loads(nb_begin, 0);
        if (QK_INT8) {
            const uint32_t s0 = load_ks(nb_begin);
            if (ks_wave) *(float*)(smem + ks_wr) = cvt_ks(s0);
        }
        int nb = nb_begin;
        while (true) {
            step(BoolTag<false>{}, nb);
            nb += NBS;
            if (nb >= nb_end) break;
            step(BoolTag<true>{}, nb);
            nb += NBS;
            if (nb >= nb_end) break;
        }
    }

    // ---- epilogue: the waves' partial row sums meet in LDS; every wave scales and stores its own output columns
    __syncthreads();
    const float l_pair = half_pair_sum(l_run);
    if (lh == 0) *(float*)(smem + xm_wr) = l_pair;
    __syncthreads();
    const float l_tot = (*(const float*)(smem + xm_rd) + *(const float*)(smem + xm_rd + 128)) +
                        (*(const float*)(smem + xm_rd + 256) + *(const float*)(smem + xm_rd + 384));
    // false: an empty split range, an empty cache entry, or a causal row above the first key (zeros, lse = -inf; such a
    // row's accumulators hold NaN from exp2(-inf - -inf), hence the selects below)
    const bool seen = nb_begin < nb_end && m_run > -INFINITY;
    const float inv = seen ? 1.f / l_tot : 0.f;
    const float lse = seen ? m_run + __builtin_log2f(l_tot) : -INFINITY;
    if (!q_valid) return;
    if (SPLIT) {
        const int64_t row = ((int64_t)(split * p.batch + b) * p.heads + h) * p.seqlen + q_row;
        float* op = p.o_part + row * D;
        if (own_tile) {
#pragma unroll
            for (int j = 0; j < DTW; ++j)
#pragma unroll
                for (int a4 = 0; a4 < 4; ++a4) {
                    v4f o;
#pragma unroll
                    for (int b4 = 0; b4 < 4; ++b4) o[b4] = seen ? o_acc[j][4 * a4 + b4] * inv : 0.f;
                    *(v4f*)(op + 32 * (wave + 4 * j) + 8 * a4 + 4 * lh) = o;
                }
        }
        if (wave == 0 && lh == 0) p.lse_part[row] = lse;
        return;
    }
    char* orow = p.out + b * p.o_sb + h * p.o_sh + (int64_t)q_row * p.o_sn;
    if (own_tile) {
#pragma unroll
        for (int j = 0; j < DTW; ++j)
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                const int d0 = 32 * (wave + 4 * j) + 8 * a4 + 4 * lh;
                if (IO_DT == 0) {
                    v4h o;
#pragma unroll
                    for (int b4 = 0; b4 < 4; ++b4) o[b4] = (_Float16)(seen ? o_acc[j][4 * a4 + b4] * inv : 0.f);
                    *(v4h*)(orow + d0 * 2) = o;
                } else {
                    v4s o;
#pragma unroll
                    for (int b4 = 0; b4 < 4; ++b4) o[b4] = f32_to_bf16(seen ? o_acc[j][4 * a4 + b4] * inv : 0.f);
                    *(v4s*)(orow + d0 * 2) = o;
                }
            }
    }
    if (p.lse != nullptr && wave == 0 && lh == 0) p.lse[((int64_t)b * p.heads + h) * p.seqlen + q_row] = lse;
#endif  // __HIP_DEVICE_COMPILE__
}

}  // namespace intfa
