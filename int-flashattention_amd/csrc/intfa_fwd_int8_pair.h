// Full-int8 forward at head_dim 256: eight waves per workgroup, two waves per 32 query rows.
//
// Same algorithm and the same key block (64 keys) as fwd_full_int8_kernel (flash_atten_full_int8.py:9-71), other
// division of labour.  A wave cannot hold 32 rows x 256 output columns in fp32 next to the S^T tile at two waves per
// SIMD, and giving the column halves to two independent workgroups makes both redo Q K^T and the whole softmax.  Here
// waves w and w + 4 (same SIMD) share the query rows 32w .. 32w+31:
//   * wave w + 4h computes S^T, the scaling, the row maxima, the exponentials and the int8 P of the keys 32h .. 32h+31
//     of the block (one 32-key sub-tile each);
//   * the two exchange their row maxima and their packed P fragments through LDS (the block's two workgroup barriers,
//     which also publish the V tile and the next block's K tile);
//   * wave w + 4h multiplies the whole P (64 keys) with the columns 128h .. 128h+127 of V and owns those output
//     columns; the row sum is kept per wave and added up in the epilogue.
// No vector instruction is issued twice for the same element.  Waves 0-3 copy the K tile of the next block, waves 4-7
// the V tile (both 64 rows x 256 bytes).
#pragma once
#include "intfa_device.h"

namespace intfa {

constexpr int kPairThreads = 512;

template <bool CAUSAL, int OUT_DT /*0 f16, 1 bf16*/, int PROUND, bool SPLIT, bool VBLK>
__global__ void __launch_bounds__(kPairThreads, 1) fwd_full_int8_pair_kernel(const KParams p) {
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass only needs the kernel's symbol
    constexpr int D = 256;
    constexpr int KS = D / 32;                   // k-steps of Q K^T
    constexpr int BN = 64;                       // keys per block
    constexpr int DVW = 128;                     // output columns of one wave
    constexpr int DT = DVW / 32;                 // 32-wide output tiles of one wave
    constexpr int KT = BN * D;                   // bytes of one K tile, and of one V tile
    // LDS map (bytes)
    constexpr int OFF_KS = 0;                    // two fp32 k_scale vectors
    constexpr int OFF_XM = OFF_KS + 2 * BN * 4;  // row maxima (and, in the epilogue, row sums): [wave][32]
    constexpr int OFF_VS = OFF_XM + 8 * 32 * 4;  // VBLK: two vectors of D fp32 channel scales
    constexpr int OFF_XP = OFF_VS + (VBLK ? 2 * D * 4 : 0);   // packed P fragments: [wave][lane] x 16 bytes
    constexpr int OFF_K = (OFF_XP + 8 * 64 * 16 + 1023) & ~1023;
    constexpr int OFF_V = OFF_K + 2 * KT;
    constexpr int LDS_BYTES = OFF_V + 2 * KT;
    __shared__ __attribute__((aligned(1024))) char smem[LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rw = wave & 3;                     // row group: query rows 32 rw .. 32 rw + 31 of the block
    const int hf = wave >> 2;                    // key sub-tile of the softmax work and column half of the output
    const int lq = lane & 31, lh = lane >> 5;

    // ---- block -> (head, m-block, split): whole K/V heads per XCD (as in fwd_full_int8_kernel)
    const int n_mblk = (p.seqlen + kBlockM - 1) / kBlockM;
    const int n_split = SPLIT ? p.num_splits : 1;
    const bool pair = CAUSAL && !SPLIT && p.pair_mblocks != 0;
    const WorkgroupJob wg = deal_workgroup(p, blockIdx.x);
    const int rem = wg.rem, head = wg.b * p.heads + wg.h;
    const int mb_idx = fast_div(rem, p.d_n_split);
    const int split = rem - mb_idx * n_split;
    const int njobs = pair ? 2 : 1;
#pragma clang loop unroll(disable)
    for (int job = 0; job < njobs; ++job) {
    if (job) __syncthreads();                    // every wave is done with the LDS of the first query block
    int mb = mb_idx;
    if (CAUSAL) mb = (pair && job) ? mb_idx : n_mblk - 1 - mb_idx;     // heaviest query blocks first
    const int b = wg.b, h = wg.h;
    const int hk = wg.hk;

    const int seqlen_k = keys_of_batch(p, b);
    // causal mask aligned to the bottom right corner: query row i sees keys 0 .. i + causal_off
    const int causal_off = seqlen_k - p.seqlen;
    const KeyBlocks kb = key_block_range<BN>(seqlen_k, CAUSAL, mb * kBlockM + kBlockM, causal_off, SPLIT, n_split, split, CAUSAL,
                                             p.blocks_per_split);
    const int nb_total = kb.total, nb_begin = kb.begin, nb_end = kb.end;
    const int q_row = mb * kBlockM + rw * 32 + lq;
    const bool q_valid = q_row < p.seqlen;
    const int q_ld = q_valid ? q_row : p.seqlen - 1;

    // ---- Q fragment (B operand of S^T = K Q^T), resident
    v4i qreg[KS];
    load_q8_fragments<KS>(qreg, p, b, h, q_ld, lh);
    const float qsc = load_q_scale_log2(p, b, h, q_ld);

    float m_run = -INFINITY, l_run = 0.f;        // l_run: this wave's keys only
    float o_acc[DT][16];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[dt][r] = 0.f;

    // ---- global -> LDS copies: waves 0-3 the K tile, waves 4-7 the V tile (same geometry, other swizzle and source)
    const char* Kg = p.k + b * p.k_sb + hk * p.k_sh;
    const char* Vg = p.v + b * p.v_sb + hk * p.v_sh;
    const uint32_t t_sn = __builtin_amdgcn_readfirstlane((uint32_t)(hf ? p.v_sn : p.k_sn));
    const v4i t_rsrc = make_rsrc(hf ? Vg : Kg, (uint32_t)((seqlen_k - 1) * (int64_t)t_sn + D));
    const auto k_lane = tile_load_lane<D, SWZ_K, BN>(t_sn, rw, lane);
    const auto v_lane = tile_load_lane<D, SWZ_V8, BN>(t_sn, rw, lane);
    TileLoadLane<D, SWZ_K, BN> t_lane;
    t_lane.off[0] = hf ? v_lane.off[0] : k_lane.off[0];
    static_assert(TileLoadLane<D, SWZ_K, BN>::NV == 1 && TileLoadLane<D, SWZ_V8, BN>::NV == 1, "one lane offset per tile");
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    const uint32_t t_lds = lds0 + (hf ? OFF_V : OFF_K);
    auto issue_loads = [&](int nb, int buf) __attribute__((always_inline)) {
        issue_tile_load<D, SWZ_K, BN>(t_rsrc, (uint32_t)(nb * BN) * t_sn, t_sn, t_lds + buf * KT, rw, t_lane);
    };
    // k_scale of a block: thread t < 64 fetches the scale of key t; converted to fp32 when stored to LDS
    const KScaleSource ks_src(p, b, hk, seqlen_k);
    const int ks_key = tid & (BN - 1);
    auto load_ks = [&](int nb) __attribute__((always_inline)) -> uint32_t { return ks_src.load(nb * BN + ks_key); };   // raw bits
    auto cvt_ks = [&](uint32_t raw) __attribute__((always_inline)) -> float { return ks_src.cvt(raw); };
    // VBLK: thread 256 + c fetches the fp32 scale of channel c of the key block's scale row (vs_g key blocks per row)
    // (Which threads fetch scales is decided per WAVE, from the wave index held in a scalar register: the branches
    // below are scalar branches that leave the exec mask alone.  A per-thread test of threadIdx would mask lanes off, and
    // a register spill or reload that the compiler places in the block where such lanes rejoin runs before the mask is
    // restored there: the lanes that were off lose the value.)
    const bool ks_wave = wave == 0;              // threads 0 .. 63: one k_scale each
    const int vs_c = tid - 256;
    const bool vs_thread = VBLK && hf == 1;      // threads 256 .. 511: one channel each
    const float* Vsg = (const float*)p.v_scale + (b * p.vs_sb + hk * p.vs_sh + (vs_thread ? vs_c : 0));
    auto load_vs = [&](int nb) __attribute__((always_inline)) -> float {
        if (!VBLK) return 0.f;
        const int row = p.vs_g == 1 ? nb : nb / p.vs_g;
        return Vsg[(int64_t)row * p.vs_sblk];
    };
    const uint32_t vs_wr = OFF_VS + 4 * (vs_thread ? vs_c : 0);
    const uint32_t vs_rd = OFF_VS + 4 * DVW * hf + 16 * lh;       // + 4 * (32*dt + 8*a4) per read

    // ---- per-lane LDS read offsets
    // K (A operand of S^T): row 32 hf + lq of the tile, chunk 2 ks + lh, XOR-swizzled by the row
    // (chunk (2 ks + lh) ^ swz = (2 ks) ^ (lh ^ swz): one base per lane, k-step ks flips 32 ks in it; the tile base
    // and the row offset are multiples of 256)
    const int k_swz = swz_k<D>(lq) & 15;
    const uint32_t k_rd0 = OFF_K + (32 * hf + lq) * D + ((lh ^ k_swz) << 4);
    static_assert(OFF_K % 256 == 0 && KT % 256 == 0, "k-step XOR assumes 256-byte aligned rows");
    auto k_rd = [&](int ks) __attribute__((always_inline)) -> uint32_t { return k_rd0 ^ (uint32_t)(32 * ks); };
    // V (A operand of O^T = V^T P^T) through the transposing 8-byte load; this wave's columns start at chunk 8 hf
    const int g16 = lane >> 4, i16 = lane & 15, jj = i16 >> 1;
    const int v_row0 = 8 * (jj >> 2) + 4 * lh + (jj & 3);
    const int v_swz = swz_v8<D>(v_row0) & 15;
    uint32_t v_rd[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const int c = 8 * hf + 2 * dt + (g16 & 1);
        v_rd[dt] = OFF_V + v_row0 * D + 8 * (i16 & 1) + ((c ^ v_swz) << 4);
    }
    const uint32_t v_own = 32 * hf * D, v_oth = 32 * (hf ^ 1) * D;      // sub-tile of this wave's P, of the partner's
    const uint32_t ks_rd = OFF_KS + 4 * 32 * hf + 16 * lh;              // + 32 * a4 per read
    const uint32_t ks_wr = OFF_KS + 4 * (tid & (BN - 1));
    const uint32_t xm_wr = OFF_XM + 4 * (wave * 32 + lq), xm_rd = OFF_XM + 4 * ((wave ^ 4) * 32 + lq);
    const uint32_t xp_wr = OFF_XP + 16 * (wave * 64 + lane), xp_rd = OFF_XP + 16 * ((wave ^ 4) * 64 + lane);


    // S^T accumulators of the block that is processed next (this wave's sub-tile): the MFMA chain of block nb+1 runs
    // under the accumulator update of block nb.
    v16i sacc;
    auto qk_loadfrags = [&](auto buf_tag, v4i (&fr)[KS]) __attribute__((always_inline)) {
        constexpr int KB = decltype(buf_tag)::value ? KT : 0;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) fr[ks] = *(const v4i*)(smem + (k_rd(ks) + KB));
    };
    uint32_t ks_next = 0;                        // raw k_scale of the next block (threads < 64)
    float vs_pend = 0.f;                         // VBLK: channel scale of the current block, not yet in LDS (threads >= 256)

    // One key block out of LDS buffer BUF.  Keys whose index inside the block exceeds the lane's `lim` are masked (causal
    // diagonal, or the keys past the end of the sequence in its last block); the test is skipped when the wave's
    // sub-tile lies at or below the smallest `lim` of the wave.  Two workgroup barriers per block, passed by every wave:
    //   B2 publishes the row maxima (and this block's V tile and channel scales),
    //   B3 publishes the packed P (and the next block's K tile and k_scale).
    // On entry the K tile and k_scale of this block are visible and `sacc` holds this wave's S^T sub-tile.
    auto compute = [&](auto buf_tag, int nb) __attribute__((always_inline)) {
        constexpr int BUF = decltype(buf_tag)::value ? 1 : 0;
        constexpr int VB = BUF * KT, SB = BUF * BN * 4;
        // last visible key relative to the block: smallest of the wave (uniform), and the lane's
        const int lim_lo = CAUSAL ? mb * kBlockM + rw * 32 + causal_off - nb * BN : seqlen_k - 1 - nb * BN;
        const int lim = CAUSAL ? lim_lo + lq : lim_lo;
        const bool more = nb + 1 < nb_end;
        auto load_vfrag = [&](uint32_t sub, int dt) __attribute__((always_inline)) -> v4i {
            const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                (__attribute__((address_space(3))) v2i*)INTFA_LDS(smem + v_rd[dt] + VB + sub));
            const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                (__attribute__((address_space(3))) v2i*)INTFA_LDS(smem + v_rd[dt] + VB + sub + 16 * D));
            return (v4i){lo[0], lo[1], hi[0], hi[1]};
        };
        // the K tile of the next block goes into the other buffer (last read one block ago)
        if (more && hf == 0) {
            issue_loads(nb + 1, BUF ^ 1);
            ks_next = load_ks(nb + 1);
        }
        // -------- pass 1: dequantise this wave's S^T sub-tile by k_scale, row maximum
        v4f kk[4];
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) kk[a4] = *(const v4f*)(smem + ks_rd + SB + 32 * a4);
        float t[16];
        float mx = -INFINITY;
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
            float xq[4];
#pragma unroll
            for (int b4 = 0; b4 < 4; ++b4) xq[b4] = (float)sacc[4 * a4 + b4] * kk[a4][b4];
            if (32 * hf + 31 > lim_lo) {                       // wave-uniform: some lane of the wave has a hidden key here
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4)
                    if ((32 * hf + 8 * a4 + b4 + 4 * lh) > lim) xq[b4] = -INFINITY;
            }
#pragma unroll
            for (int b4 = 0; b4 < 4; ++b4) {
                t[4 * a4 + b4] = xq[b4];
                mx = fmaxf(mx, xq[b4]);
            }
        }
        mx = half_pair_max(mx);
        *(float*)(smem + xm_wr) = mx;
        if (hf == 1) {                           // this block's V tile (requested one block ago) and channel scales
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (VBLK) *(float*)(smem + vs_wr + BUF * D * 4) = vs_pend;
        }
        __syncthreads();                         // ---- B2
        if (more && hf == 1) {                   // the other V buffer was last read before this barrier
            issue_loads(nb + 1, BUF ^ 1);
            if (VBLK) vs_pend = load_vs(nb + 1);
        }
        mx = fmaxf(mx, *(const float*)(smem + xm_rd));
        v4i vfo[2], vfp[2];
        vfo[0] = load_vfrag(v_own, 0);
        vfp[0] = load_vfrag(v_oth, 0);
        const float m_new = fmaxf(m_run, mx * qsc);
        float alpha = fast_exp2(m_run - m_new);
        // materialised here, well ahead of the hand-written v_fma_f32 that consumes it: the result of a transcendental
        // needs a wait state before its first use, which the compiler inserts for its own instructions only
        asm volatile("" : "+v"(alpha));
        m_run = m_new;
        // -------- pass 2: P = exp2(x*qsc - m) of this wave's keys, row sum, requantise
        float lsum = 0.f;
        v4i p8o;
        const float bias = (PROUND == 0 ? kLog2_127 : 0.f) - m_new;
        if (PROUND == 0) {
#pragma unroll
            for (int w4 = 0; w4 < 4; ++w4) {
                unsigned pk = 0;
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) {
                    const float e = fast_exp2(fmaf(t[4 * w4 + b4], qsc, bias));   // 127 * p
                    lsum += e;
                    pk = __builtin_amdgcn_cvt_pk_u8_f32(e, b4, pk);
                }
                p8o[w4] = (int)pk;
            }
        } else {
            float e[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                e[r] = fast_exp2(fmaf(t[r], qsc, bias));                          // p
                lsum += e[r];
            }
            p8o = requant_p_reference16(e);                                       // the reference's fp16 chain
        }
        *(v4i*)(smem + xp_wr) = p8o;
        // the chain of the first d-tile starts on this wave's own keys while the partner's P is on its way
        v16i oacc[2];
        oacc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(vfo[0], p8o, (v16i){0}, 0, 0, 0);
        vfo[1] = load_vfrag(v_own, 1);
        vfp[1] = load_vfrag(v_oth, 1);
        if (hf == 0) {                           // the next block's K tile and k_scale
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (more && ks_wave) *(float*)(smem + ks_wr + (BUF ^ 1) * BN * 4) = cvt_ks(ks_next);
        }
        __syncthreads();                         // ---- B3
        const v4i p8p = *(const v4i*)(smem + xp_rd);
        // K fragments of the next block (other buffer), four in flight: k-steps 2dt, 2dt+1 are consumed in stage dt and
        // their registers refilled with k-steps 2dt+4, 2dt+5
        constexpr int KBN = (BUF ^ 1) * KT;
        v4i fr[4];
        if (more) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) fr[ks] = *(const v4i*)(smem + (k_rd(ks) + KBN));
        }
        oacc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(vfp[0], p8p, oacc[0], 0, 0, 0);
        // -------- P V: O^T[d, q] += V^T[d, key] P^T[key, q]; the chain of d-tile dt+1 and a quarter of the next block's
        // Q K^T chain are issued before the accumulator update of d-tile dt
        constexpr int VSB = BUF * D * 4;
        v4f vsc[4];
        auto load_vsc = [&](int dt) __attribute__((always_inline)) {
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) vsc[a4] = *(const v4f*)(smem + vs_rd + VSB + 4 * (32 * dt + 8 * a4));
        };
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            __builtin_amdgcn_sched_barrier(0);
            if (VBLK) load_vsc(dt);
            if (dt + 1 < DT) {
                v16i& nacc = oacc[(dt + 1) & 1];
                nacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(vfo[(dt + 1) & 1], p8o, (v16i){0}, 0, 0, 0);
                nacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(vfp[(dt + 1) & 1], p8p, nacc, 0, 0, 0);
            }
            if (more) {
#pragma unroll
                for (int ks = 2 * dt; ks < 2 * dt + 2; ++ks) {
                    if (ks == 0) sacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fr[0], qreg[0], (v16i){0}, 0, 0, 0);
                    else sacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fr[ks & 3], qreg[ks], sacc, 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (more && 2 * dt + 4 < KS) {
#pragma unroll
                for (int ks = 2 * dt + 4; ks < 2 * dt + 6; ++ks) fr[ks & 3] = *(const v4i*)(smem + (k_rd(ks) + KBN));
            }
            if (dt + 2 < DT) {                   // fragments of d-tile dt+2 replace those of dt, whose chain has been issued
                vfo[dt & 1] = load_vfrag(v_own, dt + 2);
                vfp[dt & 1] = load_vfrag(v_oth, dt + 2);
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float pv = (float)oacc[dt & 1][r];
                if (VBLK) pv *= vsc[r >> 2][r & 3];
                asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(o_acc[dt][r]) : "v"(alpha), "v"(pv));
            }
        }
        l_run = fmaf(l_run, alpha, lsum);
    };

    if (nb_begin < nb_end) {
        // prologue: K tile, V tile, k_scale and channel scales of the first block; its Q K^T chain
        issue_loads(nb_begin, 0);
        {
            const uint32_t s0 = load_ks(nb_begin);
            if (ks_wave) *(float*)(smem + ks_wr) = cvt_ks(s0);
            if (vs_thread) vs_pend = load_vs(nb_begin);
        }
        if (hf == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        {
            v4i fr[KS];
            qk_loadfrags(BoolTag<false>{}, fr);
            sacc = (v16i){0};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) sacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fr[ks], qreg[ks], sacc, 0, 0, 0);
        }
        int nb = nb_begin;
        while (true) {
            if (nb >= nb_end) break;
            compute(BoolTag<false>{}, nb++);
            if (nb >= nb_end) break;
            compute(BoolTag<true>{}, nb++);
        }
    }

    // ---- epilogue
    const KernargPtr pe = kernarg_block();
    const int e_heads = pe->heads, e_seqlen = pe->seqlen;
    const int eb = fast_div(head, pe->d_heads), eh = head - eb * e_heads;
    // row sum: this wave's keys plus the partner's (the last block's barriers lie between the last use of the exchange
    // slots and this one)
    float l_tot = half_pair_sum(l_run);          // in units of 1/127 when PROUND == 0
    *(float*)(smem + xm_wr) = l_tot;
    __syncthreads();
    l_tot += *(const float*)(smem + xm_rd);
    const float vs = VBLK ? 1.f : load_scale(pe->v_scale, eb * pe->vs_sb + fast_div(eh, pe->d_kv_group) * pe->vs_sh, pe->scale_dtype);
    // (a row without a visible key gives zeros and lse = -inf; its accumulators hold NaN from exp2(-inf - -inf), hence
    // the selects)
    const bool any_key = nb_begin < nb_end && m_run > -INFINITY;
    const float out_scale = !any_key ? 0.f : (PROUND == 0) ? (vs / l_tot) : (vs / (127.f * l_tot));
    const float l_true = (PROUND == 0) ? l_tot * (1.f / 127.f) : l_tot;
    const float lse = any_key ? m_run + __builtin_log2f(l_true) : -INFINITY;
    if (SPLIT) {
        const int64_t row = ((int64_t)(split * pe->batch + eb) * e_heads + eh) * e_seqlen + q_row;
        float* op = pe->o_part + row * D + hf * DVW;
        if (q_valid) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int a4 = 0; a4 < 4; ++a4) {
                    v4f o;
#pragma unroll
                    for (int b4 = 0; b4 < 4; ++b4) o[b4] = any_key ? o_acc[dt][4 * a4 + b4] * out_scale : 0.f;
                    *(v4f*)(op + 32 * dt + 8 * a4 + 4 * lh) = o;
                }
            if (lh == 0 && hf == 0) pe->lse_part[row] = lse;
        }
        return;
    }
    {
    // 16-bit rows go out through LDS (whole lines per store instruction), staged in the tile memory: every wave has
    // passed the barrier of the row-sum exchange, so no tile is read any more
    static_assert(OFF_K + 8 * OutStage<DVW>::BYTES <= LDS_BYTES, "output staging fits the tile memory");
    // (an opaque copy of the lane index: the staging addresses depend on the lane only and would otherwise be computed
    // ahead of the main loop and held in registers through it)
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int lq_e = lane_e & 31, lh_e = lane_e >> 5;
    char* stage = smem + OFF_K + wave * OutStage<DVW>::BYTES;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
            const int d0 = 32 * dt + 8 * a4 + 4 * lh_e;
            if (OUT_DT == 0) {
                v4h o;
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) o[b4] = (_Float16)(any_key ? o_acc[dt][4 * a4 + b4] * out_scale : 0.f);
                out_stage_put<DVW>(stage, lq_e, d0, __builtin_bit_cast(v2i, o));
            } else {
                v4s o;
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) o[b4] = f32_to_bf16(any_key ? o_acc[dt][4 * a4 + b4] * out_scale : 0.f);
                out_stage_put<DVW>(stage, lq_e, d0, __builtin_bit_cast(v2i, o));
            }
        }
    const int row0 = mb * kBlockM + rw * 32;
    out_stage_flush<DVW>(stage, pe->out + eb * pe->o_sb + eh * pe->o_sh + (int64_t)row0 * pe->o_sn + hf * DVW * 2, pe->o_sn,
                         e_seqlen - row0, lane_e);
    if (q_valid && pe->lse != nullptr && lh == 0 && hf == 0) pe->lse[((int64_t)eb * e_heads + eh) * e_seqlen + q_row] = lse;
    }
    }   // job
#endif  // __HIP_DEVICE_COMPILE__
}

}  // namespace intfa
