// Full-int8 forward for few query rows per head (decoding against a key/value cache, Nq << Nk).
//
// Same arithmetic as fwd_full_int8_kernel (flash_atten_full_int8.py:9-71 per 128-key block: int32 S, dequantise, running
// max, P = exp2(X c - m), P requantised with the fixed scale 127, int32 P V, fp32 accumulator), other division of labour.
// The general kernel gives each of its four waves 32 query rows; with one or a few query rows three of them would redo
// the first one's work on padding while the pass is bound by streaming K and V from HBM.  Here one workgroup owns 32
// query rows and its four waves share every key block:
//   * wave w computes S^T for keys 32w .. 32w+31 of the block (KS MFMAs), dequantises and takes the partial row maxima;
//   * the partial maxima meet in LDS (barrier), every wave then holds the block's row maximum;
//   * wave w exponentiates and requantises its 32 keys and publishes its P8 fragment in LDS (barrier);
//   * wave w multiplies the whole block's P (all four fragments) with ITS 32-column slice of V and updates its slice of
//     the fp32 output; the partial row sums of P meet once, in the epilogue.
// The int32 sums run over the same 128 keys as in the general kernel, so results agree with it up to the order of the
// fp32 additions of the row sums.  K/V tiles are double-buffered in LDS and the whole next tile is requested at the
// start of a block (the data comes from HBM, not from a cache shared with other query blocks).
// Head dims 64 and 256: the general kernels' key block is 64 there (the reference admits no key block longer than head_dim,
// flash_atten_full_int8.py:88; at 256 registers set the limit), so a 128-key step of this
// kernel covers TWO blocks A (waves 0, 1) and B (waves 2, 3): after the one exchange of partial maxima every wave knows
// m_A = max(m, max_A), m_B = max(m_A, max_B) and both factors alpha_A = 2^(m - m_A), alpha_B = 2^(m_A - m_B); each wave
// requantises its keys in its own block's frame, and an output tile is updated as
// O = (O alpha_A + P8_A V_A) alpha_B + P8_B V_B with one int32 sum per block - the blocks' arithmetic of that kernel.
#pragma once
#include "intfa_device.h"
#include "intfa_launch.h"

namespace intfa {

// Head_dim 128: one 128-key block per step, the block of the general kernel.  Head dims 64 and 256: two 64-key blocks.
template <int D, int OUT_DT /*0 f16, 1 bf16*/, int PROUND, bool SPLIT, bool VBLK>
__global__ void __launch_bounds__(kThreads, D <= 128 ? 2 : 1) fwd_decode_full_int8_kernel(const KParams p) {
    static_assert(D == 64 || D == 128 || D == 256, "head dims 64, 128, 256");
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass only needs the kernel's symbol
    constexpr int KS = D / 32;                   // k-steps of Q K^T
    constexpr int DT = D / 32;                   // 32-wide output tiles along head_dim; wave w owns tiles w, w+4, ...
    constexpr int DTW = (DT + 3) / 4;            // output tiles per wave
    constexpr int NST = 4, BN = 32 * NST;        // one 32-key sub-tile per wave
    constexpr int NBS = D == 128 ? 1 : 2;        // key blocks (of the arithmetic) per step
    constexpr int BNB = BN / NBS;                // key block of the arithmetic: intfa_fwd_block_n()
    constexpr int KT = BN * D, VT = BN * D;      // bytes of one K / V tile
    constexpr int CH = D / 16;                   // 16-byte chunks per row
    constexpr int SWM = CH - 1;                  // swizzle mask of V rows
    // LDS map (bytes)
    constexpr int OFF_KS = 0;                            // two fp32 k_scale vectors
    constexpr int OFF_XM = 2 * BN * 4;                   // 4 waves x 32 rows fp32: partial row maxima / row sums
    constexpr int OFF_XP = OFF_XM + 4 * 32 * 4;          // 4 waves x 64 lanes x 16 bytes: the waves' P8 fragments
    constexpr int OFF_VS = OFF_XP + 4 * 64 * 16;         // VBLK: two vectors of NBS * D fp32 channel scales (one row per block)
    constexpr int NV = NBS * D;                          // channel scales per step
    constexpr int OFF_K = OFF_VS + (VBLK ? 2 * NV * 4 : 0);
    constexpr int OFF_V = OFF_K + 2 * KT;
    constexpr int LDS_BYTES = OFF_V + 2 * VT;
    static_assert(OFF_K % 256 == 0, "tiles keep the bank alignment the swizzles assume");
    __shared__ __attribute__((aligned(1024))) char smem[LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lq = lane & 31, lh = lane >> 5;

    // ---- block -> (head, 32-row query block, split); whole K/V heads go to one XCD as in the general kernel
    const int n_mblk = (p.seqlen + kDecodeRows - 1) / kDecodeRows;
    const int n_split = SPLIT ? p.num_splits : 1;
    const WorkgroupJob wg = deal_workgroup(p, blockIdx.x);
    const int rem = wg.rem, head = wg.b * p.heads + wg.h;
    const int mb = fast_div(rem, p.d_n_split), split = rem - mb * n_split;
    const int b = wg.b, h = wg.h;
    const int hk = wg.hk;

    const int seqlen_k = keys_of_batch(p, b);
    // causal: row i sees keys 0 .. i + causal_off (mask aligned to the bottom right corner as in the general kernels: a few
    // new tokens against a cache); blocks past the last row's limit are not visited
    // (causal_rows: the rows hold several query heads of one K/V group, causal_rows positions each; a row's position is
    // then row % causal_rows and a 32-row block can hold every position)
    const int fold = p.causal_rows;
    const int causal_off = seqlen_k - (fold ? fold : p.seqlen);
    // (a split takes blocks_per_split blocks of the whole key range, masked or not: every row of a decode-shaped problem
    // sees nearly all keys)
    const KeyBlocks kb = key_block_range<BNB>(seqlen_k, p.causal != 0, fold ? fold : mb * kDecodeRows + kDecodeRows, causal_off, SPLIT,
                                             n_split, split, false, p.blocks_per_split);
    const int nb_begin = kb.begin, nb_end = kb.end;         // in blocks of BNB keys
    const int key_end = nb_end * BNB < seqlen_k ? nb_end * BNB : seqlen_k;      // one past the last key of the range
    const int q_row = mb * kDecodeRows + lq;
    const bool q_valid = q_row < p.seqlen;
    const int q_ld = q_valid ? q_row : p.seqlen - 1;

    // ---- Q fragment (B operand of S^T = K Q^T), the same 32 rows in every wave
    v4i qreg[KS];
    load_q8_fragments<KS>(qreg, p, b, h, q_ld, lh);
    const float qsc = load_q_scale_log2(p, b, h, q_ld);

    float m_run = -INFINITY, l_run = 0.f;        // l_run: this wave's keys only
    float o_acc[DTW][16];
#pragma unroll
    for (int j = 0; j < DTW; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[j][r] = 0.f;

    // ---- global -> LDS copies (asynchronous, straight into LDS; the four waves split the instructions)
    const char* Kg = p.k + b * p.k_sb + hk * p.k_sh;
    const char* Vg = p.v + b * p.v_sb + hk * p.v_sh;
    const v4i k_rsrc = make_rsrc(Kg, (uint32_t)((seqlen_k - 1) * p.k_sn + D));
    const v4i v_rsrc = make_rsrc(Vg, (uint32_t)((seqlen_k - 1) * p.v_sn + D));
    const uint32_t k_sn = (uint32_t)p.k_sn, v_sn = (uint32_t)p.v_sn;
    const auto k_lane = tile_load_lane<D, SWZ_K, BN>(k_sn, wave, lane);
    const auto v_lane = tile_load_lane<D, SWZ_V8, BN>(v_sn, wave, lane);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    auto issue_loads = [&](int nb, int buf) __attribute__((always_inline)) {
        issue_tile_load<D, SWZ_K, BN>(k_rsrc, (uint32_t)(nb * BNB) * k_sn, k_sn, lds0 + OFF_K + buf * KT, wave, k_lane);
        issue_tile_load<D, SWZ_V8, BN>(v_rsrc, (uint32_t)(nb * BNB) * v_sn, v_sn, lds0 + OFF_V + buf * VT, wave, v_lane);
    };
    // k_scale of a block: thread t < 128 fetches the scale of key t; converted to fp32 when stored to LDS
    const KScaleSource ks_src(p, b, hk, seqlen_k);
    auto load_ks = [&](int nb) __attribute__((always_inline)) -> uint32_t { return ks_src.load(nb * BNB + (tid & (BN - 1))); };
    auto cvt_ks = [&](uint32_t raw) __attribute__((always_inline)) -> float { return ks_src.cvt(raw); };
    // VBLK: fp32 channel scales of the step's key blocks, NV = NBS * D values.  Up to 128 values: thread 128 + i fetches
    // value i (block i / D, channel i % D); 512 values (head_dim 256): thread t fetches channel t of both blocks.
    // (per-wave tests, scalar branches: see fwd_full_int8_kernel)
    constexpr int VPT = NV > 128 ? NV / kThreads : 1;         // values per fetching thread
    const bool ks_wave = wave < BN / 64;
    const bool vs_thread = VBLK && (NV > 128 || (wave >= 2 && (wave - 2) * 64 < NV));
    const int vs_i = NV > 128 ? tid : (vs_thread ? tid - 128 : 0);
    const int vs_blk0 = NV > 128 ? 0 : vs_i / D;              // block (inside the step) of the thread's first value
    const float* Vsg = (const float*)p.v_scale + (b * p.vs_sb + hk * p.vs_sh + vs_i % D);
    const int vs_last_row = VBLK ? ((p.seqlen_k + BNB - 1) / BNB - 1) / p.vs_g : 0;
    // (a step's second block may lie past the end of the sequence: its keys are hidden, any scale row serves)
    auto load_vs = [&](int nb, int j) __attribute__((always_inline)) -> float {
        if (!VBLK) return 0.f;
        const int blk = nb + vs_blk0 + j;
        int row = p.vs_g == 1 ? blk : blk / p.vs_g;
        row = row < vs_last_row ? row : vs_last_row;
        return Vsg[(int64_t)row * p.vs_sblk];
    };

    // ---- per-lane LDS offsets
    const int k_swz = swz_k<D>(lq) & (CH - 1);
    uint32_t k_rd[KS];                            // this wave's 32 keys: row 32*wave + lq, chunk 2*ks + lh
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_rd[ks] = OFF_K + (32 * wave + lq) * D + (((2 * ks + lh) ^ k_swz) << 4);
    // V through the transposing 8-byte load (see fwd_full_int8_kernel): source lane s of a 16-lane group points at key
    // row 8*(j>>2) + 4*lh + (j&3), j = s/2 (+16 for the second load, +32 per sub-tile), 8-byte half s&1
    const int g16 = lane >> 4, i16 = lane & 15, jj = i16 >> 1;
    const int v_row0 = 8 * (jj >> 2) + 4 * lh + (jj & 3);
    const int v_swz = swz_v8<D>(v_row0) & SWM;
    uint32_t v_rd[DTW];
#pragma unroll
    for (int j = 0; j < DTW; ++j) {
        const int dt = (wave + 4 * j) % DT;          // (head_dim 64: waves 2 and 3 shadow tiles 0 and 1, see below)
        const int c = 2 * dt + (g16 & 1);
        v_rd[j] = OFF_V + v_row0 * D + 8 * (i16 & 1) + (((c & SWM) ^ v_swz) << 4) + ((c & ~SWM) << 4);
    }
    const uint32_t ks_rd = OFF_KS + 4 * (32 * wave) + 16 * lh;       // + 4 * 8*a4 per read
    const uint32_t ks_wr = OFF_KS + 4 * (tid & (BN - 1));
    const uint32_t xm_wr = OFF_XM + 4 * (32 * wave + lq);
    const uint32_t xm_rd = OFF_XM + 4 * lq;                          // + 128 per wave
    const uint32_t xp_wr = OFF_XP + 1024 * wave + 16 * lane;
    const uint32_t xp_rd = OFF_XP + 16 * lane;                       // + 1024 per wave
    const uint32_t vs_wr = OFF_VS + 4 * vs_i;                        // + 4 * kThreads per further value
    const uint32_t vs_rd = OFF_VS + 16 * lh;                         // + 4 * (D*blk + 32*dt + 8*a4) per read
    // head_dim 64 has two output tiles for four waves: waves 2 and 3 compute tiles 0 and 1 a second time and store
    // nothing (the same instruction stream for every wave; a run-time "owns a tile" test around the V fragments and the
    // accumulator update costs the owners a hundred register copies per step)
    // the last visible key of the first row of this query block, and of the lane's row
    const int first_lim = p.causal ? (fold ? 0 : mb * kDecodeRows) + causal_off : 0x3fffffff;
    const int row_lim = p.causal ? (fold ? q_row % fold : q_row) + causal_off : 0x3fffffff;
    const bool blk_a = NBS == 1 || wave < 2;                          // this wave's keys belong to the first block of a step

    auto step = [&](auto buf_tag, int nb) __attribute__((always_inline)) {
        constexpr int BUF = decltype(buf_tag)::value ? 1 : 0;
        constexpr int KB = BUF * KT, VB = BUF * VT, SB = BUF * BN * 4, VSB = BUF * NV * 4;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();                                   // tile nb has landed; the other buffer and the exchange areas are free
        const bool more = nb + NBS < nb_end;
        uint32_t ks_next = 0;
        float vs_next[VPT] = {};
        if (more) {
            issue_loads(nb + NBS, BUF ^ 1);
            if (ks_wave) ks_next = load_ks(nb + NBS);
            if (vs_thread) {
#pragma unroll
                for (int j = 0; j < VPT; ++j) vs_next[j] = load_vs(nb + NBS, j);
            }
        }
        // -------- S^T of this wave's 32 keys, dequantise, partial row maximum
        v4i fr[KS];
        v4f kk[4];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) fr[ks] = *(const v4i*)(smem + k_rd[ks] + KB);
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) kk[a4] = *(const v4f*)(smem + ks_rd + SB + 4 * 8 * a4);
        v16i sacc = (v16i){0};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) sacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fr[ks], qreg[ks], sacc, 0, 0, 0);
        // V fragments of this wave's output tiles travel during the softmax
        v4i vf[DTW][NST];
#pragma unroll
        for (int j = 0; j < DTW; ++j)
#pragma unroll
            for (int st = 0; st < NST; ++st) {
                const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                    (__attribute__((address_space(3))) v2i*)INTFA_LDS(smem + v_rd[j] + VB + (32 * st) * D));
                const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                    (__attribute__((address_space(3))) v2i*)INTFA_LDS(smem + v_rd[j] + VB + (32 * st + 16) * D));
                vf[j][st] = (v4i){lo[0], lo[1], hi[0], hi[1]};
            }
        float x[16];
        float mx = -INFINITY;
        // masked steps (wave-uniform test): keys past the end of the range (the ragged last block; with two blocks per
        // step, a second block that is not part of the range), or past the first row's position (the causal diagonal)
        const int key0 = nb * BNB;
        const bool tail = key0 + BN > key_end || key0 + BN - 1 > first_lim;
        // keys of this lane with 8*a4 + b4 >= key_lim are hidden: past the end of the range or past the lane's row
        const int last_key = (row_lim < key_end - 1 ? row_lim : key_end - 1) - key0;
        const int key_lim = last_key + 1 - 32 * wave - 4 * lh;
#pragma unroll
        for (int r = 0; r < 16; ++r) x[r] = (float)sacc[r] * kk[r >> 2][r & 3];
        if (tail) {
            // (a branch of its own, kept one by the empty statement: folded into the loop above, the test would put a
            // compare and a select on every element of every step)
            asm volatile("");
#pragma unroll
            for (int r = 0; r < 16; ++r) x[r] = hide_past(x[r], key_lim - 1, 8 * (r >> 2) + (r & 3));
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, x[r]);
        mx = half_pair_max(mx);
        if (lh == 0) *(float*)(smem + xm_wr) = mx;
        __syncthreads();                                   // the four partial maxima are in LDS
        // one block per step: alpha_b = 1 and m_a = m_b is the block's maximum; two blocks: the chain A, B
        const float mx_a = fmaxf(*(const float*)(smem + xm_rd), *(const float*)(smem + xm_rd + 128));
        const float mx_b = fmaxf(*(const float*)(smem + xm_rd + 256), *(const float*)(smem + xm_rd + 384));
        const float m_a = fmaxf(m_run, (NBS == 1 ? fmaxf(mx_a, mx_b) : mx_a) * qsc);
        const float alpha = fast_exp2(m_run - m_a);
        const float m_b = NBS == 1 ? m_a : fmaxf(m_a, mx_b * qsc);
        const float alpha_b = NBS == 1 ? 1.f : fast_exp2(m_a - m_b);
        m_run = m_b;
        // -------- P of this wave's keys, requantised in its block's frame; partial row sum
        const float bias = (PROUND == 0 ? kLog2_127 : 0.f) - (blk_a ? m_a : m_b);
        float lsum = 0.f;
        v4i p8;
        {
            float e[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                e[r] = fast_exp2(fmaf(x[r], qsc, bias));                         // RNE mode: 127 * p
                lsum += e[r];
            }
            if (PROUND == 0) {
#pragma unroll
                for (int w4 = 0; w4 < 4; ++w4) {
                    unsigned pk = 0;
#pragma unroll
                    for (int b4 = 0; b4 < 4; ++b4) pk = __builtin_amdgcn_cvt_pk_u8_f32(e[4 * w4 + b4], b4, pk);
                    p8[w4] = (int)pk;
                }
            } else {
                p8 = requant_p_reference16(e);                                   // the reference's fp16 chain
            }
        }
        *(v4i*)(smem + xp_wr) = p8;
        v4f vsc[NBS][DTW][4];                              // channel scales of the step's blocks for this wave's output tiles
        if (VBLK) {
#pragma unroll
            for (int blk = 0; blk < NBS; ++blk)
#pragma unroll
                for (int j = 0; j < DTW; ++j)
#pragma unroll
                    for (int a4 = 0; a4 < 4; ++a4)
                        vsc[blk][j][a4] = *(const v4f*)(smem + vs_rd + VSB + 4 * (D * blk + 32 * ((wave + 4 * j) % DT) + 8 * a4));
        }
        __syncthreads();                                   // the four P8 fragments are in LDS
        v4i pall[NST];
#pragma unroll
        for (int st = 0; st < NST; ++st) pall[st] = *(const v4i*)(smem + xp_rd + 1024 * st);
        // -------- this wave's output columns: O^T[d, q] += V^T[d, key] P^T[key, q] over the whole block
#pragma unroll
        for (int j = 0; j < DTW; ++j) {
            if (NBS == 1) {
                v16i acc = (v16i){0};
#pragma unroll
                for (int st = 0; st < NST; ++st) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf[j][st], pall[st], acc, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    if (VBLK) o_acc[j][r] = fmaf(o_acc[j][r], alpha, (float)acc[r] * vsc[0][j][r >> 2][r & 3]);
                    else o_acc[j][r] = fmaf(o_acc[j][r], alpha, (float)acc[r]);
                }
            } else {
                v16i acc_a = (v16i){0}, acc_b = (v16i){0};
#pragma unroll
                for (int st = 0; st < NST / 2; ++st) acc_a = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf[j][st], pall[st], acc_a, 0, 0, 0);
#pragma unroll
                for (int st = NST / 2; st < NST; ++st) acc_b = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf[j][st], pall[st], acc_b, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    if (VBLK) o_acc[j][r] = fmaf(fmaf(o_acc[j][r], alpha, (float)acc_a[r] * vsc[0][j][r >> 2][r & 3]), alpha_b,
                                                 (float)acc_b[r] * vsc[NBS - 1][j][r >> 2][r & 3]);
                    else o_acc[j][r] = fmaf(fmaf(o_acc[j][r], alpha, (float)acc_a[r]), alpha_b, (float)acc_b[r]);
                }
            }
        }
        if (NBS == 1) l_run = fmaf(l_run, alpha, lsum);
        else l_run = blk_a ? fmaf(l_run, alpha, lsum) * alpha_b : fmaf(l_run * alpha, alpha_b, lsum);
        // (the raw scale is made opaque here, behind the step's last barrier: its conversion waits for the load, and with it
        // for the next step's tile copies that were issued ahead of it - that wait belongs at the end of the step)
        asm volatile("" : "+v"(ks_next));
        if (more && ks_wave) *(float*)(smem + ks_wr + (BUF ^ 1) * BN * 4) = cvt_ks(ks_next);
        if (more && vs_thread) {
#pragma unroll
            for (int j = 0; j < VPT; ++j) *(float*)(smem + vs_wr + (BUF ^ 1) * NV * 4 + j * kThreads * 4) = vs_next[j];
        }
    };

    if (nb_begin < nb_end) {
        issue_loads(nb_begin, 0);
        if (ks_wave) *(float*)(smem + ks_wr) = cvt_ks(load_ks(nb_begin));
        if (vs_thread) {
#pragma unroll
            for (int j = 0; j < VPT; ++j) *(float*)(smem + vs_wr + j * kThreads * 4) = load_vs(nb_begin, j);
        }
        int nb = nb_begin;
        while (true) {
            if (nb >= nb_end) break;
            step(BoolTag<false>{}, nb);
            nb += NBS;
            if (nb >= nb_end) break;
            step(BoolTag<true>{}, nb);
            nb += NBS;
        }
    }

    // ---- epilogue: the waves' partial row sums meet in LDS; every wave scales and stores its own output columns
    __syncthreads();
    const float l_pair = half_pair_sum(l_run);
    if (lh == 0) *(float*)(smem + xm_wr) = l_pair;
    __syncthreads();
    const float l_tot = (*(const float*)(smem + xm_rd) + *(const float*)(smem + xm_rd + 128)) +
                        (*(const float*)(smem + xm_rd + 256) + *(const float*)(smem + xm_rd + 384));   // units of 1/127 when PROUND == 0
    const float vs = VBLK ? 1.f : load_scale(p.v_scale, b * p.vs_sb + hk * p.vs_sh, p.scale_dtype);
    // false: an empty split range, an empty cache entry, or a causal row above the first key (zeros, lse = -inf; such a
    // row's accumulators hold NaN from exp2(-inf - -inf), hence the selects below)
    const bool seen = nb_begin < nb_end && m_run > -INFINITY;
    const float out_scale = !seen ? 0.f : (PROUND == 0) ? (vs / l_tot) : (vs / (127.f * l_tot));
    const float l_true = (PROUND == 0) ? l_tot * (1.f / 127.f) : l_tot;
    const float lse = seen ? m_run + __builtin_log2f(l_true) : -INFINITY;
    if (!q_valid) return;
    if (SPLIT) {
        const int64_t row = ((int64_t)(split * p.batch + b) * p.heads + h) * p.seqlen + q_row;
        float* op = p.o_part + row * D;
#pragma unroll
        for (int j = 0; j < DTW; ++j) {
            const int dt = wave + 4 * j;
            if (dt >= DT) continue;
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                v4f o;
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) o[b4] = seen ? o_acc[j][4 * a4 + b4] * out_scale : 0.f;
                *(v4f*)(op + 32 * dt + 8 * a4 + 4 * lh) = o;
            }
        }
        if (wave == 0 && lh == 0) p.lse_part[row] = seen ? lse : -INFINITY;
        return;
    }
    char* orow = p.out + b * p.o_sb + h * p.o_sh + (int64_t)q_row * p.o_sn;
#pragma unroll
    for (int j = 0; j < DTW; ++j) {
        const int dt = wave + 4 * j;
        if (dt >= DT) continue;
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
            const int d0 = 32 * dt + 8 * a4 + 4 * lh;
            if (OUT_DT == 0) {
                v4h o;
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) o[b4] = (_Float16)(seen ? o_acc[j][4 * a4 + b4] * out_scale : 0.f);
                *(v4h*)(orow + d0 * 2) = o;
            } else {
                v4s o;
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) o[b4] = f32_to_bf16(seen ? o_acc[j][4 * a4 + b4] * out_scale : 0.f);
                *(v4s*)(orow + d0 * 2) = o;
            }
        }
    }
    if (p.lse != nullptr && wave == 0 && lh == 0) p.lse[((int64_t)b * p.heads + h) * p.seqlen + q_row] = lse;
#endif  // __HIP_DEVICE_COMPILE__
}

}  // namespace intfa
