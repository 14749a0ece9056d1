// Half-int8 and fp16/bf16 forward at head_dim 256: eight waves per workgroup, two waves per 32 query rows.
//
// Same algorithm and the same 64-key block as fwd_f16pv_kernel (flash_atten_int8.py:9-66, flash_atten_fp.py:9-60), with
// the division of labour of fwd_full_int8_pair_kernel: 32 rows x 256 fp32 output columns do not fit one wave at two
// waves per SIMD, and column halves in two independent workgroups make both redo Q K^T and the whole softmax.  Here
// waves w and w + 4 share the query rows 32w .. 32w+31:
//   * wave w + 4h computes S^T, the scaling, the row maxima, the exponentials and the 16-bit P of the keys
//     32h .. 32h+31 of the block (one 32-key sub-tile each);
//   * the two exchange their row maxima and their P fragments (32 bytes per lane) through LDS: the block's two workgroup
//     barriers, which also publish the V tile and the next block's K tile;
//   * wave w + 4h multiplies the whole P (64 keys) with the columns 128h .. 128h+127 of V on
//     v_mfma_f32_32x32x16_{f16,bf16}, whose fp32 accumulators are the running output of those columns (scaled by alpha
//     before each block's products are added); the row sum is kept per wave and added up in the epilogue.
// The Q K^T chain of block n+1 is issued between the P V chains of block n.  Waves 0-3 copy the K tile of the next
// block, waves 4-7 the V tile.
#pragma once
#include "intfa_device.h"
#include "intfa_fwd_f16pv.h"
#include "intfa_fwd_int8_pair.h"

namespace intfa {

template <bool QK_INT8, bool CAUSAL, int IO_DT /*0 f16, 1 bf16*/, bool SPLIT>
__global__ void __launch_bounds__(kPairThreads, 1) fwd_f16pv_pair_kernel(const KParams p) {
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass only needs the kernel's symbol
    constexpr int D = 256;
    constexpr int BN = kBlockN16;                // keys per block (64)
    constexpr int QB = QK_INT8 ? 1 : 2;          // bytes per Q/K element
    constexpr int KROW = D * QB, VROW = D * 2;   // bytes per K row / per V row
    constexpr int KS = KROW / 32;                // MFMA k-steps of S^T (32 bytes of a row each)
    constexpr int KPS = KS / 4;                  // k-steps of the next block's chain issued per output d-tile stage
    constexpr int DVW = 128;                     // output columns of one wave
    constexpr int DT = DVW / 32;                 // 32-wide output tiles of one wave
    constexpr int KT = BN * KROW, VT = BN * VROW;
    constexpr int KCH = KROW / 16, VCH = VROW / 16;
    static_assert(BN == 64 && DT == 4, "one 32-key sub-tile per wave of a pair, four output tiles per wave");
    // LDS map (bytes)
    constexpr int OFF_KS = 0;                    // two fp32 k_scale vectors
    constexpr int OFF_XM = OFF_KS + 2 * BN * 4;  // row maxima (and, in the epilogue, row sums): [wave][32]
    constexpr int OFF_XP = OFF_XM + 8 * 32 * 4;  // 16-bit P fragments: [16-key step][wave][lane] x 16 bytes
    constexpr int OFF_K = (OFF_XP + 8 * 64 * 32 + 1023) & ~1023;
    constexpr int OFF_V = OFF_K + 2 * KT;
    constexpr int LDS_BYTES = OFF_V + 2 * VT;
    static_assert(LDS_BYTES <= 160 * 1024, "one workgroup per compute unit");
    __shared__ __attribute__((aligned(1024))) char smem[LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rw = wave & 3;                     // row group: query rows 32 rw .. 32 rw + 31 of the block
    const int hf = wave >> 2;                    // key sub-tile of the softmax work and column half of the output
    const int lq = lane & 31, lh = lane >> 5;

    // ---- block -> (head, m-block, split): whole K/V heads per XCD
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
    const int nb_begin = kb.begin, nb_end = kb.end;
    const int q_row = mb * kBlockM + rw * 32 + lq;
    const bool q_valid = q_row < p.seqlen;
    const int q_ld = q_valid ? q_row : p.seqlen - 1;

    // ---- Q fragments (B operand of S^T = K Q^T), resident: 16 bytes per k-step
    v4i qreg[KS];
    load_q8_fragments<KS>(qreg, p, b, h, q_ld, lh);          // (byte addressing: serves 8- and 16-bit rows alike)
    // exponent scale of this lane's row: q_scale * sm_scale * log2(e) (int8 Q K^T) or sm_scale * log2(e)
    const float qsc = QK_INT8 ? load_q_scale_log2(p, b, h, q_ld) : p.qk_scale_log2;

    float m_run = -INFINITY, l_run = 0.f;        // l_run: this wave's keys only
    v16f o_acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[dt][r] = 0.f;

    // ---- global -> LDS copies: waves 0-3 the K tile, waves 4-7 the V tile
    const char* Kg = p.k + b * p.k_sb + hk * p.k_sh;
    const char* Vg = p.v + b * p.v_sb + hk * p.v_sh;
    const v4i k_rsrc = make_rsrc(Kg, (uint32_t)((seqlen_k - 1) * p.k_sn + KROW));
    const v4i v_rsrc = make_rsrc(Vg, (uint32_t)((seqlen_k - 1) * p.v_sn + VROW));
    const uint32_t k_sn = __builtin_amdgcn_readfirstlane((uint32_t)p.k_sn), v_sn = __builtin_amdgcn_readfirstlane((uint32_t)p.v_sn);
    const auto k_lane = tile_load_lane<KROW, SWZ_K, BN>(k_sn, rw, lane);
    const auto v_lane = tile_load_lane<VROW, SWZ_V16, BN>(v_sn, rw, lane);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    auto issue_k = [&](int nb, int buf) __attribute__((always_inline)) {
        issue_tile_load<KROW, SWZ_K, BN>(k_rsrc, (uint32_t)__builtin_amdgcn_readfirstlane((nb * BN) * (int)k_sn), k_sn, lds0 + OFF_K + buf * KT, rw, k_lane);
    };
    auto issue_v = [&](int nb, int buf) __attribute__((always_inline)) {
        issue_tile_load<VROW, SWZ_V16, BN>(v_rsrc, (uint32_t)__builtin_amdgcn_readfirstlane((nb * BN) * (int)v_sn), v_sn, lds0 + OFF_V + buf * VT, rw, v_lane);
    };
    // k_scale of a block: thread t < 64 fetches the scale of key t; converted to fp32 when stored to LDS
    const KScaleSource ks_src(p, b, hk, seqlen_k);
    const int ks_key = tid & (BN - 1);
    auto load_ks = [&](int nb) __attribute__((always_inline)) -> uint32_t { return QK_INT8 ? ks_src.load(nb * BN + ks_key) : 0u; };

    // ---- per-lane LDS read offsets
    // K (A operand of S^T): row 32 hf + lq of the tile, chunk 2 ks + lh, XOR-swizzled by the row
    // (chunk (2 ks + lh) ^ swz = (2 ks) ^ (lh ^ swz): one base per lane, k-step ks flips 32 ks in it; the tile base
    // and the row offset are multiples of the row length)
    const int k_swz = swz_k<KROW>(lq) & (KCH - 1);
    const uint32_t k_rd0 = OFF_K + (32 * hf + lq) * KROW + ((lh ^ k_swz) << 4);
    static_assert(OFF_K % 1024 == 0 && KT % 1024 == 0 && 32 * (KS - 1) < KROW, "k-step XOR stays inside the row");
    auto k_rd = [&](int ks) __attribute__((always_inline)) -> uint32_t { return k_rd0 ^ (uint32_t)(32 * ks); };
    // V (A operand of O^T = V^T P^T) through ds_read_b64_tr_b16: inside a 16-lane group, result lane i element j comes
    // from element i % 4 of the 8 bytes addressed by lane 4 j + i / 4.  Source lane s therefore points at key row s >> 2
    // of a run of four consecutive keys and at the four head-dim values d0 + 4 (s & 3) .. + 3,
    // d0 = 128 hf + 32 dt + 16 (group & 1).
    const int g16 = lane >> 4, s16 = lane & 15;
    const int v_row0 = 4 * lh + (s16 >> 2);           // + 8 for the second load, + 16 u + 32 (sub-tile)
    const int v_swz = swz_v16<VROW>(v_row0) & (VCH - 1);
    uint32_t v_rd[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const int c = 16 * hf + 4 * dt + 2 * (g16 & 1) + ((s16 & 3) >> 1);
        v_rd[dt] = OFF_V + v_row0 * VROW + ((c ^ v_swz) << 4) + 8 * (s16 & 1);
    }
    const uint32_t v_own = 32 * hf * VROW, v_oth = 32 * (hf ^ 1) * VROW;   // sub-tile of this wave's P, of the partner's
    const uint32_t ks_rd = OFF_KS + 4 * 32 * hf + 16 * lh;                 // + 32 * a4 per read
    const uint32_t ks_wr = OFF_KS + 4 * (tid & (BN - 1));
    const uint32_t xm_wr = OFF_XM + 4 * (wave * 32 + lq), xm_rd = OFF_XM + 4 * ((wave ^ 4) * 32 + lq);
    // (a lane's two fragments lie 8 KiB apart, so that consecutive lanes write consecutive 16 bytes: no bank conflicts)
    constexpr uint32_t XP_U = 8 * 64 * 16;
    const uint32_t xp_wr = OFF_XP + 16 * (wave * 64 + lane), xp_rd = OFF_XP + 16 * ((wave ^ 4) * 64 + lane);

    auto mfma16 = [&](v4i a, v4i b2, v16f c) __attribute__((always_inline)) -> v16f {
        if (IO_DT == 0) return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b2), c, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b2), c, 0, 0, 0);
    };
    // S^T accumulators of the block that is processed next (this wave's sub-tile): the chain of block nb+1 runs between
    // the P V chains of block nb.
    v16i si = {0};                               // int8 Q K^T
    v16f sf = {0};                               // 16-bit Q K^T
    auto qk_step = [&](v4i kf, int ks) __attribute__((always_inline)) {
        if (QK_INT8) si = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qreg[ks], ks ? si : (v16i){0}, 0, 0, 0);
        else sf = mfma16(kf, qreg[ks], ks ? sf : (v16f){0});
    };
    uint32_t ks_next = 0;                        // raw k_scale of the next block (threads < 64)

    // One key block out of LDS buffer BUF.  Keys whose index inside the block exceeds the lane's `lim` are masked (causal
    // diagonal, or the keys past the end of the sequence in its last block); the test is skipped when the wave's
    // sub-tile lies at or below the smallest `lim` of the wave.  Two workgroup barriers per block, passed by every wave:
    //   B2 publishes the row maxima (and this block's V tile),
    //   B3 publishes the P fragments (and the next block's K tile and k_scale).
    // On entry the K tile and k_scale of this block are visible and si / sf holds this wave's S^T sub-tile.
    auto compute = [&](auto buf_tag, int nb) __attribute__((always_inline)) {
        constexpr int BUF = decltype(buf_tag)::value ? 1 : 0;
        constexpr int VB = BUF * VT, SB = BUF * BN * 4;
        constexpr int KBN = (BUF ^ 1) * KT;
        // last visible key relative to the block: smallest of the wave (uniform), and the lane's
        const int lim_lo = CAUSAL ? mb * kBlockM + rw * 32 + causal_off - nb * BN : seqlen_k - 1 - nb * BN;
        const int lim = CAUSAL ? lim_lo + lq : lim_lo;
        const bool more = nb + 1 < nb_end;
        // fragment of d-tile dt for the 16 keys `u` of the sub-tile that starts at byte offset `sub`
        auto load_vfrag = [&](uint32_t sub, int dt, int u) __attribute__((always_inline)) -> v4i {
            const uint32_t a0 = v_rd[dt] + VB + sub + 16 * u * VROW;
            const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)INTFA_LDS(smem + a0));
            const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)INTFA_LDS(smem + a0 + 8 * VROW));
            return (v4i){__builtin_bit_cast(v2i, lo)[0], __builtin_bit_cast(v2i, lo)[1], __builtin_bit_cast(v2i, hi)[0], __builtin_bit_cast(v2i, hi)[1]};
        };
        // the K tile of the next block goes into the other buffer (last read two blocks ago)
        if (more && hf == 0) {
            issue_k(nb + 1, BUF ^ 1);
            ks_next = load_ks(nb + 1);
        }
        // -------- pass 1: this wave's S^T sub-tile (dequantised by k_scale), row maximum
        v4f kk[4];
        if (QK_INT8) {
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) kk[a4] = *(const v4f*)(smem + ks_rd + SB + 32 * a4);
        }
        float t[16];
        float mx = -INFINITY;
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
            float xq[4];
#pragma unroll
            for (int b4 = 0; b4 < 4; ++b4) xq[b4] = QK_INT8 ? (float)si[4 * a4 + b4] * kk[a4][b4] : sf[4 * a4 + b4];
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
        if (hf == 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // this block's V tile (requested one block ago)
        __syncthreads();                         // ---- B2
        if (more && hf == 1) issue_v(nb + 1, BUF ^ 1);                     // the other V buffer was last read before this barrier
        mx = fmaxf(mx, *(const float*)(smem + xm_rd));
        v4i vfo[2][2], vfp[2][2];                // V fragments of d-tile dt (buffer dt & 1): own keys, partner's keys; two k-steps each
#pragma unroll
        for (int u = 0; u < 2; ++u) { vfo[0][u] = load_vfrag(v_own, 0, u); vfp[0][u] = load_vfrag(v_oth, 0, u); }
        const float m_new = fmaxf(m_run, mx * qsc);
        const float alpha = fast_exp2(m_run - m_new);
        m_run = m_new;
        // -------- pass 2: P = exp2(x*qsc - m) of this wave's keys, row sum, cast to the 16-bit type
        float lsum = 0.f;
        float e[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) { e[r] = fast_exp2(fmaf(t[r], qsc, -m_new)); lsum += e[r]; }
        v4i pfo[2], pfp[2];                      // B operands: 8 x 16-bit per 16-key step (own keys, partner's keys)
#pragma unroll
        for (int u = 0; u < 2; ++u)
            pfo[u] = IO_DT == 0 ? __builtin_bit_cast(v4i, pack_p_f16(e + 8 * u)) : __builtin_bit_cast(v4i, pack_p_bf16(e + 8 * u));
        *(v4i*)(smem + xp_wr) = pfo[0];
        *(v4i*)(smem + xp_wr + XP_U) = pfo[1];
        l_run = fmaf(l_run, alpha, lsum);
        // the first d-tile is rescaled and its chain starts on this wave's own keys while the partner's P is on its way
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[0][r] *= alpha;
        o_acc[0] = mfma16(vfo[0][0], pfo[0], o_acc[0]);
        o_acc[0] = mfma16(vfo[0][1], pfo[1], o_acc[0]);
#pragma unroll
        for (int u = 0; u < 2; ++u) { vfo[1][u] = load_vfrag(v_own, 1, u); vfp[1][u] = load_vfrag(v_oth, 1, u); }
        if (hf == 0) {                           // the next block's K tile and k_scale
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (QK_INT8 && more && wave == 0) *(float*)(smem + ks_wr + (BUF ^ 1) * BN * 4) = ks_src.cvt(ks_next);
        }
        __syncthreads();                         // ---- B3
        pfp[0] = *(const v4i*)(smem + xp_rd);
        pfp[1] = *(const v4i*)(smem + xp_rd + XP_U);
        // K fragments of the next block (other buffer): the k-steps of stage dt + 1 are requested when those of stage dt
        // have been issued
        v4i fr[KPS];
        if (more) {
#pragma unroll
            for (int j = 0; j < KPS; ++j) fr[j] = *(const v4i*)(smem + (k_rd(j) + KBN));
        }
        // -------- P V: O^T[d, q] = alpha O^T + V^T[d, key] P^T[key, q].  Stage dt: the chain of d-tile dt (for d-tile 0
        // only its partner half is left), a quarter of the next block's Q K^T chain between its links, d-tile dt+1
        // rescaled under them.
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                __builtin_amdgcn_sched_barrier(0);
                if (a4 < 2) { if (dt > 0) o_acc[dt] = mfma16(vfo[dt & 1][a4], pfo[a4], o_acc[dt]); }
                else o_acc[dt] = mfma16(vfp[dt & 1][a4 - 2], pfp[a4 - 2], o_acc[dt]);
                if (more) {
#pragma unroll
                    for (int j = a4 * KPS / 4; j < (a4 + 1) * KPS / 4; ++j) qk_step(fr[j], dt * KPS + j);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (dt + 1 < DT) {
#pragma unroll
                    for (int b4 = 0; b4 < 4; ++b4) o_acc[dt + 1][4 * a4 + b4] *= alpha;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (more && dt + 1 < DT) {
#pragma unroll
                for (int j = 0; j < KPS; ++j) fr[j] = *(const v4i*)(smem + (k_rd((dt + 1) * KPS + j) + KBN));
            }
            if (dt + 2 < DT) {                   // fragments of d-tile dt+2 replace those of dt, whose chain has been issued
#pragma unroll
                for (int u = 0; u < 2; ++u) { vfo[dt & 1][u] = load_vfrag(v_own, dt + 2, u); vfp[dt & 1][u] = load_vfrag(v_oth, dt + 2, u); }
            }
        }
    };

    if (nb_begin < nb_end) {
        // prologue: K tile, V tile and k_scale of the first block; its Q K^T chain
        if (hf == 0) issue_k(nb_begin, 0); else issue_v(nb_begin, 0);
        if (QK_INT8) {
            const uint32_t s0 = load_ks(nb_begin);
            if (wave == 0) *(float*)(smem + ks_wr) = ks_src.cvt(s0);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qk_step(*(const v4i*)(smem + k_rd(ks)), ks);
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
    float l_tot = half_pair_sum(l_run);
    *(float*)(smem + xm_wr) = l_tot;
    __syncthreads();
    l_tot += *(const float*)(smem + xm_rd);
    // (a row without a visible key gives zeros and lse = -inf; its accumulators hold NaN from exp2(-inf - -inf), hence
    // the selects)
    const bool any_key = nb_begin < nb_end && m_run > -INFINITY;
    const float inv = any_key ? 1.f / l_tot : 0.f;
    const float lse = any_key ? m_run + __builtin_log2f(l_tot) : -INFINITY;
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
                    for (int b4 = 0; b4 < 4; ++b4) o[b4] = any_key ? o_acc[dt][4 * a4 + b4] * inv : 0.f;
                    *(v4f*)(op + 32 * dt + 8 * a4 + 4 * lh) = o;
                }
            if (lh == 0 && hf == 0) pe->lse_part[row] = lse;
        }
    } else {
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
                if (IO_DT == 0) {
                    v4h o;
#pragma unroll
                    for (int b4 = 0; b4 < 4; ++b4) o[b4] = (_Float16)(any_key ? o_acc[dt][4 * a4 + b4] * inv : 0.f);
                    out_stage_put<DVW>(stage, lq_e, d0, __builtin_bit_cast(v2i, o));
                } else {
                    v4s o;
#pragma unroll
                    for (int b4 = 0; b4 < 4; ++b4) o[b4] = f32_to_bf16(any_key ? o_acc[dt][4 * a4 + b4] * inv : 0.f);
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
