// Forward kernel with P V on 16-bit floating-point MFMA: the half-int8 variant (int8 Q K^T with per-token
// scales, flash_atten_int8.py:9-66) and the fp16/bf16 variant (flash_atten_fp.py:9-60).
//
// Same tiling as the full-int8 kernel (4 waves x 32 query rows, S^T = K Q^T so that a lane owns one query
// column), but keys go in blocks of 64 (two 32-key sub-tiles) and P is cast to V's 16-bit type in registers
// and multiplied on v_mfma_f32_32x32x16_{f16,bf16}, whose fp32 accumulator IS the running output: the MFMA adds P V on
// top (acc = tl.dot(p, v, acc), flash_atten_int8.py:59); the rescaling by alpha of flash_atten_int8.py:48-52 happens only
// in the blocks where a row's maximum rises by more than kFrameSlack over the exponent's reference point (see below).
// V rows stay row-major in LDS; the transposing 8-byte load (ds_read_b64_tr_b16) delivers the A operand.
#pragma once
#include "intfa_device.h"
#include "intfa_fwd_int8.h"

namespace intfa {

constexpr int kBlockN16 = 64;      // key block of this kernel
constexpr float kFrameSlack = 8.f; // how far a row's block maximum may exceed the exponent's frame before the frame moves

__device__ __forceinline__ v8h pack_p_f16(const float* e) {
    v8h r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = (_Float16)e[i];
    return r;
}
__device__ __forceinline__ v8bf pack_p_bf16(const float* e) {
    v8bf r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = (__bf16)e[i];
    return r;
}

// QK_INT8: int8 Q/K with scales (half-int8) or 16-bit Q/K (fp16/bf16 variant).  IO_DT: type of V, P and the output
// (and of Q/K when !QK_INT8): 0 fp16, 1 bf16.
// Output columns one workgroup produces.  At head_dim 256 a full-width workgroup needs 128 fp32 output registers per lane:
// one wave per SIMD and spills.  This kernel can split the columns over two workgroups that each redo Q K^T and the
// softmax and multiply P with their half of V; the library does not instantiate it at head_dim 256 any more -
// fwd_f16pv_pair_kernel (intfa_fwd_f16pv_pair.h) divides the work between two waves of one workgroup instead.
template <int D> struct F16PvGeom {
    static constexpr int DV = D <= 128 ? D : 128;
    static constexpr int NHALF = D / DV;
};

// (16-bit K tiles at head_dim 256 are 32 KiB each: double-buffered beside the V tiles they leave room for one workgroup
// per compute unit, whatever the register count)
template <bool QK_INT8, int D, bool CAUSAL, int IO_DT, bool SPLIT>
// (head_dim 64: three waves per SIMD - the non-causal instances need 140-146 registers, the masked ones are held to 168
// and spill 7-9; 33 KiB / 25 KiB of LDS allow it)
__global__ void __launch_bounds__(kThreads, D > 128 ? (QK_INT8 ? 2 : 1) : (D == 64 ? 3 : 2)) fwd_f16pv_kernel(const KParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int BN = kBlockN16, NST = BN / 32;
    constexpr int QB = QK_INT8 ? 1 : 2;               // bytes per Q/K element
    constexpr int DV = F16PvGeom<D>::DV, NHALF = F16PvGeom<D>::NHALF;
    constexpr int KROW = D * QB, VROW = DV * 2;       // bytes per K row / per V row of this workgroup's columns
    constexpr int KS = KROW / 32;                     // MFMA k-steps of S^T (32 bytes of a row each)
    constexpr int DT = DV / 32;                       // 32-wide output tiles
    constexpr int KT = BN * KROW, VT = BN * VROW;
    constexpr int KCH = KROW / 16, VCH = VROW / 16;
    constexpr int OFF_KS = 0;
    constexpr int OFF_K = 2 * BN * 4;
    constexpr int OFF_V = OFF_K + 2 * KT;
    constexpr int LDS_BYTES = OFF_V + 2 * VT;
    __shared__ __attribute__((aligned(1024))) char smem[LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lq = lane & 31, lh = lane >> 5;

    const int n_mblk = (p.seqlen + kBlockM - 1) / kBlockM;      // the last query block may be partial
    const int n_split = SPLIT ? p.num_splits : 1;
    // Causal single-pass launches pair query block i with query block n-1-i in one workgroup (heavy one first): every
    // workgroup then walks the same number of key blocks and the launch has no tail of light workgroups.
    const bool pair = CAUSAL && !SPLIT && p.pair_mblocks != 0;
    const WorkgroupJob wg = deal_workgroup(p, blockIdx.x);
    const int rem = wg.rem, head = wg.b * p.heads + wg.h;
    const int half = rem % NHALF;                // column half of this workgroup (0 when the columns are not split)
    const int mb_idx = fast_div(rem / NHALF, p.d_n_split);
    const int split = rem / NHALF - mb_idx * n_split;
    const int njobs = pair ? 2 : 1;
#pragma clang loop unroll(disable)
    for (int job = 0; job < njobs; ++job) {
    if (job) __syncthreads();                    // every wave is done with the LDS tiles of the first query block
    int mb = mb_idx;
    if (CAUSAL) mb = (pair && job) ? mb_idx : n_mblk - 1 - mb_idx;     // heaviest query blocks first
    const int b = wg.b, h = wg.h;
    const int hk = wg.hk;                     // K/V head of this query head
    // ragged sequence lengths are handled as in the full-int8 kernel (zero-filled copies, masked last block, rows past
    // the end computed on clamped inputs and not stored)
    const int seqlen_k = keys_of_batch(p, b);
    // causal mask aligned to the bottom right corner as in the full-int8 kernel: row i sees keys 0 .. i + causal_off
    const int causal_off = seqlen_k - p.seqlen;
    const KeyBlocks kb = key_block_range<BN>(seqlen_k, CAUSAL, mb * kBlockM + kBlockM, causal_off, SPLIT, n_split, split, CAUSAL,
                                             p.blocks_per_split);
    const int nb_total = kb.total, nb_begin = kb.begin, nb_end = kb.end;
    const int q_row = mb * kBlockM + wave * 32 + lq;
    const bool q_valid = q_row < p.seqlen;
    const int q_ld = q_valid ? q_row : p.seqlen - 1;     // row read for lanes past the end

    // ---- Q fragments (B operand of S^T): 16 bytes per k-step
    v4i qreg[KS];
    {
        const char* qrow = p.q + b * p.q_sb + h * p.q_sh + (int64_t)q_ld * p.q_sn;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qreg[ks] = *(const v4i*)(qrow + ks * 32 + lh * 16);
    }
    // exponent scale of this lane's row: q_scale * sm_scale * log2(e) (int8 Q K^T) or sm_scale * log2(e)
    const float qsc = QK_INT8 ? load_scale(p.q_scale, b * p.qs_sb + h * p.qs_sh + (int64_t)q_ld * p.qs_sn, p.scale_dtype) * p.qk_scale_log2
                              : p.qk_scale_log2;
    float m_run = -INFINITY, l_run = 0.f;
    v16f o_acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[dt][r] = 0.f;

    // ---- global -> LDS copies
    const char* Kg = p.k + b * p.k_sb + hk * p.k_sh;
    const char* Vg = p.v + b * p.v_sb + hk * p.v_sh + half * DV * 2;
    const v4i k_rsrc = make_rsrc(Kg, (uint32_t)((seqlen_k - 1) * p.k_sn + KROW));
    const v4i v_rsrc = make_rsrc(Vg, (uint32_t)((seqlen_k - 1) * p.v_sn + VROW));
    const uint32_t k_sn = (uint32_t)p.k_sn, v_sn = (uint32_t)p.v_sn;
    const auto k_lane = tile_load_lane<KROW, SWZ_K, BN>(k_sn, wave, lane);
    const auto v_lane = tile_load_lane<VROW, SWZ_V16, BN>(v_sn, wave, lane);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    auto issue_loads = [&](int nb, int buf) __attribute__((always_inline)) {
        issue_tile_load<KROW, SWZ_K, BN>(k_rsrc, (uint32_t)(nb * BN) * k_sn, k_sn, lds0 + OFF_K + buf * KT, wave, k_lane);
        issue_tile_load<VROW, SWZ_V16, BN>(v_rsrc, (uint32_t)(nb * BN) * v_sn, v_sn, lds0 + OFF_V + buf * VT, wave, v_lane);
    };
    const KScaleSource ks_src(p, b, hk, seqlen_k);
    const bool ks_wave = wave == 0;                  // threads 0 .. 63 fetch one k_scale each (a scalar test: see fwd_full_int8_kernel)
    auto load_ks = [&](int nb) __attribute__((always_inline)) -> uint32_t {
        return (!QK_INT8 || !ks_wave) ? 0u : ks_src.load(nb * BN + tid);
    };
    auto cvt_ks = [&](uint32_t raw) __attribute__((always_inline)) -> float { return ks_src.cvt(raw); };

    // ---- per-lane LDS read offsets
    const int k_swz = swz_k<KROW>(lq) & (KCH - 1);
    uint32_t k_rd[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_rd[ks] = OFF_K + lq * KROW + (((2 * ks + lh) ^ k_swz) << 4);
    // V through ds_read_b64_tr_b16: inside a 16-lane group, result lane i element j comes from element i%4 of the
    // 8 bytes addressed by lane 4j + i/4.  Source lane s therefore points at key row (s >> 2) of a run of four
    // consecutive keys and at the four head-dim values d0 + 4*(s & 3) .. +3, d0 = 32*dt + 16*(group & 1).
    const int g16 = lane >> 4, s16 = lane & 15;
    const int v_row0 = 4 * lh + (s16 >> 2);           // + 8*w + 16*u + 32*st
    const int v_swz = swz_v16<VROW>(v_row0) & (VCH - 1);
    uint32_t v_rd[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const int c = 4 * dt + 2 * (g16 & 1) + ((s16 & 3) >> 1);
        v_rd[dt] = OFF_V + v_row0 * VROW + ((c ^ v_swz) << 4) + 8 * (s16 & 1);
    }
    const uint32_t ks_rd = OFF_KS + 16 * lh;
    const uint32_t ks_wr = OFF_KS + 4 * (tid & (BN - 1));

    auto mfma16 = [&](v4i a, v4i b, v16f c) __attribute__((always_inline)) -> v16f {
        if (IO_DT == 0) return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
    };

    // One key block out of LDS buffer BUF.  Inside the wave the work is software-pipelined and pinned with scheduling
    // barriers: the MFMAs of S^T sub-tile st+1 are issued one at a time between quarters of the vector work of sub-tile
    // st, the MFMAs of output d-tile dt between quarters of the rescaling of d-tile dt+1, and LDS operands are requested
    // one or two stages before the MFMA that consumes them.
    // DIAG selects the code instance with masking: keys whose index inside the block exceeds the lane's `lim` are masked
    // and sub-tiles st > gw (wave-uniform: the sub-tile of the largest lim in the wave) are skipped (causal diagonal:
    // lim = the lane's last visible key; ragged last block: the last valid key).
    auto compute = [&](auto buf_tag, auto diag_tag, int nb, int gw, int lim, int lim_lo) __attribute__((always_inline)) {
        constexpr int BUF = decltype(buf_tag)::value ? 1 : 0;
        constexpr bool DIAG = decltype(diag_tag)::value;
        constexpr int KB = BUF * KT, VB = BUF * VT, SB = BUF * BN * 4;
        static_assert(NST == 2, "the quarter interleave below assumes two sub-tiles of 32 keys");
        if (DIAG && gw < 0) return;                     // block entirely above the wave's rows
        const int nact = DIAG ? (gw + 1 < NST ? gw + 1 : NST) : NST;
        // -------- operands of both S^T sub-tiles
        v4i fr[NST][KS];
        v4f kk[NST][4];
#pragma unroll
        for (int st = 0; st < NST; ++st) {
            if (DIAG && st > gw) continue;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) fr[st][ks] = *(const v4i*)(smem + k_rd[ks] + KB + 32 * st * KROW);
            if (QK_INT8) {
#pragma unroll
                for (int a4 = 0; a4 < 4; ++a4) kk[st][a4] = *(const v4f*)(smem + ks_rd + SB + 4 * (32 * st + 8 * a4));
            }
        }
        auto load_vfrags = [&](v4i (&vf)[NST][2], int dt) __attribute__((always_inline)) {
#pragma unroll
            for (int st = 0; st < NST; ++st) {
                if (DIAG && st > gw) continue;
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const uint32_t a0 = v_rd[dt] + VB + (32 * st + 16 * u) * VROW;
                    const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)INTFA_LDS(smem + a0));
                    const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)INTFA_LDS(smem + a0 + 8 * VROW));
                    vf[st][u] = (v4i){__builtin_bit_cast(v2i, lo)[0], __builtin_bit_cast(v2i, lo)[1], __builtin_bit_cast(v2i, hi)[0], __builtin_bit_cast(v2i, hi)[1]};
                }
            }
        };
        // -------- pass 1: S^T sub-tiles, dequantise, running max
        v16i si[NST];                                       // int8 Q K^T accumulators
        v16f sf[NST];                                       // 16-bit Q K^T accumulators
        auto qk_mfma = [&](int st, int ks) __attribute__((always_inline)) {
            if (QK_INT8) si[st] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fr[st][ks], qreg[ks], ks ? si[st] : (v16i){0}, 0, 0, 0);
            else sf[st] = mfma16(fr[st][ks], qreg[ks], ks ? sf[st] : (v16f){0});
        };
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qk_mfma(0, ks);
        float t[NST][16];
        float mx = -INFINITY;
#pragma unroll
        for (int st = 0; st < NST; ++st) {
            if (DIAG && st > gw) {
#pragma unroll
                for (int r = 0; r < 16; ++r) t[st][r] = -INFINITY;
                continue;
            }
            const bool next = st + 1 < nact;
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                __builtin_amdgcn_sched_barrier(0);
                if (st + 1 < NST && next) {
#pragma unroll
                    for (int ks = a4 * KS / 4; ks < (a4 + 1) * KS / 4; ++ks) qk_mfma(st + 1, ks);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) {
                    const int r = 4 * a4 + b4;
                    float v = QK_INT8 ? (float)si[st][r] * kk[st][a4][b4] : sf[st][r];
                    if (DIAG && 32 * st + 31 > lim_lo && (32 * st + 8 * a4 + b4 + 4 * lh) > lim) v = -INFINITY;
                    t[st][r] = v;
                    mx = fmaxf(mx, v);
                }
            }
        }
        // V fragments of the first two d-tiles travel while the exponentials are evaluated
        v4i vf[2][NST][2];
        __builtin_amdgcn_sched_barrier(0);
        load_vfrags(vf[0], 0);
        if (1 < DT) load_vfrags(vf[1], 1);
        mx = half_pair_max(mx);
        // The exponent's reference point ("frame") follows the running maximum lazily: it moves, and the output and the row
        // sum are rescaled as the reference does in every block (flash_atten_int8.py:48-52), only when some row's block
        // maximum exceeds its frame by more than kFrameSlack.  P is a 16-bit FLOATING-point number here: p' = exp2(x - frame)
        // <= 2^kFrameSlack differs from the reference's p = exp2(x - m_new) by a factor that is the same for the numerator
        // sum p' v and for the row sum, so acc / l and m + log2(l) are unchanged; only the 16-bit rounding of the single
        // p' lands on other values (relative 2^-12, unbiased).  In the common case no vector instruction touches the output.
        const float mxs = mx * qsc;
        if (DIAG || __builtin_expect(__builtin_amdgcn_ballot_w64(mxs > m_run + kFrameSlack) != 0, 0)) {   // (the few masked blocks always move the frame: no branch around the rescale there)
            const float m_mv = fmaxf(m_run, mxs);
            const float a_mv = fast_exp2(m_run - m_mv);
            m_run = m_mv;
            l_run *= a_mv;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) o_acc[dt][r] *= a_mv;
        }
        const float m_new = m_run;
        // -------- pass 2: P = exp2(x*qsc - m), row sum, cast to the 16-bit type
        float lsum = 0.f;
        v4i pf[NST][2];                                   // B operands: 8 x 16-bit per 16-key step
#pragma unroll
        for (int st = 0; st < NST; ++st) {
            if (DIAG && st > gw) continue;
            __builtin_amdgcn_sched_barrier(0);
            float e[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) { e[r] = fast_exp2(fmaf(t[st][r], qsc, -m_new)); lsum += e[r]; }
#pragma unroll
            for (int u = 0; u < 2; ++u)
                pf[st][u] = IO_DT == 0 ? __builtin_bit_cast(v4i, pack_p_f16(e + 8 * u)) : __builtin_bit_cast(v4i, pack_p_bf16(e + 8 * u));
            asm volatile("" : "+v"(lsum));
        }
        l_run += lsum;
        // -------- O^T[d, q] += V^T[d, key] P^T[key, q] (the fp32 accumulators of the MFMAs are the running output)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                const int st = a4 >> 1, u = a4 & 1;
                __builtin_amdgcn_sched_barrier(0);
                if (!(DIAG && st > gw)) o_acc[dt] = mfma16(vf[dt & 1][st][u], pf[st][u], o_acc[dt]);
                __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (dt + 2 < DT) load_vfrags(vf[dt & 1], dt + 2);
        }
    };

    auto step = [&](auto buf_tag, auto diag_tag, int nb, int gw, int lim, int lim_lo) __attribute__((always_inline)) {
        constexpr int BUF = decltype(buf_tag)::value ? 1 : 0;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        const bool more = nb + 1 < nb_end;
        uint32_t ks_next = 0;
        if (more) { issue_loads(nb + 1, BUF ^ 1); ks_next = load_ks(nb + 1); }
        compute(buf_tag, diag_tag, nb, gw, lim, lim_lo);
        if (QK_INT8 && more && ks_wave) *(float*)(smem + ks_wr + (BUF ^ 1) * BN * 4) = cvt_ks(ks_next);
    };

    if (nb_begin < nb_end) {
        issue_loads(nb_begin, 0);
        if (QK_INT8) {
            const uint32_t s0 = load_ks(nb_begin);
            if (ks_wave) *(float*)(smem + ks_wr) = cvt_ks(s0);
        }
        const int diag_first = (mb * kBlockM + causal_off + 1) / BN;   // first block with a key hidden from the block's first row
        const int diag_begin = diag_first < 0 ? 0 : diag_first;
        const int tail_keys = seqlen_k - (nb_total - 1) * BN;        // valid keys of the last block (BN if it is full)
        const bool ragged = !CAUSAL && tail_keys < BN && nb_end == nb_total;
        const int plain_end = CAUSAL ? (nb_end > diag_begin ? diag_begin : nb_end) : (ragged ? nb_end - 1 : nb_end);
        int nb = nb_begin;
        while (true) {
            if (nb >= plain_end) break;
            step(BoolTag<false>{}, BoolTag<false>{}, nb++, 0, 0, 0);
            if (nb >= plain_end) break;
            step(BoolTag<true>{}, BoolTag<false>{}, nb++, 0, 0, 0);
        }
        // masked blocks: the blocks the causal diagonal of this query block crosses, or the ragged last block of a
        // non-causal pass
#pragma clang loop unroll(disable)
        for (; nb < nb_end; ++nb) {
            const int lim = CAUSAL ? q_row + causal_off - nb * BN : tail_keys - 1;
            const int gw = (CAUSAL ? mb * kBlockM + wave * 32 + 31 + causal_off - nb * BN : tail_keys - 1) >> 5;
            const int lim_lo = CAUSAL ? mb * kBlockM + wave * 32 + causal_off - nb * BN : tail_keys - 1;   // smallest lim in the wave
            if (((nb - nb_begin) & 1) == 0) step(BoolTag<false>{}, BoolTag<true>{}, nb, gw, lim, lim_lo);
            else step(BoolTag<true>{}, BoolTag<true>{}, nb, gw, lim, lim_lo);
        }
    }

    // ---- epilogue
    const KernargPtr pe = kernarg_block();
    const int e_heads = pe->heads, e_seqlen = pe->seqlen;
    const int eb = fast_div(head, pe->d_heads), eh = head - eb * e_heads;
    const float l_tot = half_pair_sum(l_run);
    // (no key at all - an empty cache entry - gives zeros and lse = -inf instead of 0 / 0)
    const bool any_key = nb_begin < nb_end && m_run > -INFINITY;      // (a causal row above the first key sees nothing)
    const float inv = any_key ? 1.f / l_tot : 0.f;
    const float lse = any_key ? m_run + __builtin_log2f(l_tot) : -INFINITY;
    if (SPLIT) {
        const int64_t row = ((int64_t)(split * pe->batch + eb) * e_heads + eh) * e_seqlen + q_row;
        float* op = pe->o_part + row * D + half * DV;
        // a row contributes nothing to this split when the split's range is empty for its workgroup, or when every
        // block of the range lies above the row's diagonal (its wave skipped them: the running max is still -inf)
        const bool seen = nb_begin < nb_end && m_run > -INFINITY;
        if (q_valid) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int a4 = 0; a4 < 4; ++a4) {
                    v4f o;
#pragma unroll
                    for (int b4 = 0; b4 < 4; ++b4) o[b4] = seen ? o_acc[dt][4 * a4 + b4] * inv : 0.f;
                    *(v4f*)(op + 32 * dt + 8 * a4 + 4 * lh) = o;
                }
            if (lh == 0 && half == 0) pe->lse_part[row] = seen ? lse : -INFINITY;
        }
        return;
    }
    {
    // 16-bit rows go out through LDS (whole lines per store instruction); the tiles are dead once every wave is here
    static_assert(4 * OutStage<DV>::BYTES <= LDS_BYTES, "output staging fits the tile memory");
    __syncthreads();
    // (an opaque copy of the lane index: the staging addresses depend on the lane only and would otherwise be computed
    // ahead of the main loop and held in registers through it)
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int lq_e = lane_e & 31, lh_e = lane_e >> 5;
    char* stage = smem + wave * OutStage<DV>::BYTES;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
            const int d0 = 32 * dt + 8 * a4 + 4 * lh_e;
            if (IO_DT == 0) {
                v4h o;
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) o[b4] = (_Float16)(any_key ? o_acc[dt][4 * a4 + b4] * inv : 0.f);
                out_stage_put<DV>(stage, lq_e, d0, __builtin_bit_cast(v2i, o));
            } else {
                v4s o;
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) o[b4] = f32_to_bf16(any_key ? o_acc[dt][4 * a4 + b4] * inv : 0.f);
                out_stage_put<DV>(stage, lq_e, d0, __builtin_bit_cast(v2i, o));
            }
        }
    const int row0 = mb * kBlockM + wave * 32;
    out_stage_flush<DV>(stage, pe->out + eb * pe->o_sb + eh * pe->o_sh + (int64_t)row0 * pe->o_sn + half * DV * 2, pe->o_sn,
                        e_seqlen - row0, lane_e);
    if (q_valid && pe->lse != nullptr && lh == 0 && half == 0) pe->lse[((int64_t)eb * e_heads + eh) * e_seqlen + q_row] = lse;
    }
    }   // job
#endif  // __HIP_DEVICE_COMPILE__
}

}  // namespace intfa
