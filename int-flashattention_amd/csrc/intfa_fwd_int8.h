// Forward kernel with int8 Q K^T and int8 P V (full-int8).
//
// Algorithm restated from the reference tile loop (flash_atten_full_int8.py:9-71): per key block of BN keys
// (FullInt8Geom below), S = Q8 K8^T in int32; X = S * q_scale[row] * k_scale[col]; running max m in the exp2 domain;
// P = exp2(X * c - m_new); l sums the UNQUANTISED P; P is requantised to int8 with the fixed scale 127;
// acc = acc * alpha + P8 V8; output acc * v_scale / (127 l).
// Differences in evaluation order that stay within fp32 rounding: q_scale * c is folded into one per-row
// factor, v_scale / 127 is applied once in the epilogue, and (RNE mode) the factor 127 is folded into the
// exponent as exp2(x + log2 127).
//
// One workgroup (4 waves) owns 128 query rows of one (batch, head); wave w owns rows 32w..32w+31.
// LDS holds two K tiles, two V tiles and two k_scale vectors (double buffering); all LDS traffic uses
// integer offsets into ONE array so that operand addresses are a lane register plus an immediate.
#pragma once
#include "intfa_device.h"

namespace intfa {

// Key block length of the full-int8 kernels: 128 keys, or 64 at head_dim 256 (registers and LDS).  At head_dim 256 this
// kernel only serves the int32 S export; the forward itself is fwd_full_int8_pair_kernel (intfa_fwd_int8_pair.h), which
// spreads the 256 output columns of a query row over two waves.
template <int D> struct FullInt8Geom {
    static constexpr int NST = D == 128 ? 4 : 2;
    static constexpr int BN = 32 * NST;
    // occupancy the register budget is held to (a workgroup puts one wave on each SIMD: workgroups per compute unit)
    static constexpr int waves_per_simd(bool causal, int vblk) { return D == 64 ? (causal || vblk ? 3 : 4) : 2; }
};

// VBLK != 0: V carries one scale per key block and channel (layout of the reference's CUDA kernel,
// csrc/flash_fwd_kernel_full_qi8.h:156-160) instead of one per (batch, head): the int32 P V of a block is multiplied
// by the block's channel scales before it joins the accumulator (csrc/mask.h:313-340).  VBLK == 1: a scale row covers
// one or more whole key blocks of this kernel.  VBLK == 2: a scale row covers 64 keys, the key block of the reference's
// CUDA kernel (kBlockN = 64 at head_dim 128, csrc/flash_fwd_launch_template.h:514-519): the softmax still advances per
// 128-key block (the running maximum and P8 are those of intfa_fwd_block_n()), but P V is summed in int32 per 64-key
// half and each half is multiplied by its own scale row.
template <int D, bool CAUSAL, int OUT_DT /*0 f16, 1 bf16*/, int PROUND, bool DUMP_S, bool SPLIT, int VBLK = 0>
__global__ void __launch_bounds__(kThreads, FullInt8Geom<D>::waves_per_simd(CAUSAL, VBLK)) fwd_full_int8_kernel(const KParams p) {
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass only needs the kernel's symbol
    constexpr int KS = D / 32;                   // k-steps of Q K^T (32 bytes of head_dim each)
    static_assert(D <= 128 || DUMP_S, "head_dim 256 runs fwd_full_int8_pair_kernel");
    constexpr int DV = D;                        // output columns
    constexpr int DT = DV / 32;                  // 32-wide output tiles along head_dim
    constexpr int NST = FullInt8Geom<D>::NST;    // 32-key sub-tiles per key block
    constexpr int BN = FullInt8Geom<D>::BN;      // keys per block
    constexpr int KT = BN * D;                   // bytes of one K tile
    constexpr int VT = BN * DV;                  // bytes of one int8 V tile (this workgroup's columns)
    constexpr int CH = D / 16;                   // 16-byte chunks per K row
    constexpr int CHV = DV / 16;                 // 16-byte chunks per V row
    constexpr int SWM = (CHV < 8 ? CHV : 8) - 1; // swizzle mask of V rows
    // LDS map (bytes)
    constexpr int OFF_KS = 0;                    // two fp32 k_scale vectors
    constexpr int OFF_K = 2 * BN * 4;            // two K tiles
    constexpr int OFF_V = OFF_K + 2 * KT;        // two V tiles
    constexpr int VSUB = VBLK == 2 ? 2 : 1;      // V scale rows per key block
    static_assert(VBLK != 2 || NST == 4, "64-key V scale rows belong to the 128-key block");
    constexpr int OFF_VS = OFF_V + 2 * VT;       // VBLK: two vectors of VSUB * DV fp32 channel scales
    constexpr int LDS_BYTES = OFF_VS + (VBLK ? 2 * VSUB * DV * 4 : 0);
    __shared__ __attribute__((aligned(1024))) char smem[LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lq = lane & 31, lh = lane >> 5;

    // ---- block -> (head, m-block, split).  Workgroups are dealt round-robin to the 8 XCDs, each with its own
    // L2; give every XCD whole heads so that the K/V tiles of a head are re-read from one L2.
    const int n_mblk = (p.seqlen + kBlockM - 1) / kBlockM;      // the last query block may be partial
    const int n_split = SPLIT ? p.num_splits : 1;
    // Causal single-pass launches pair query block i with query block n-1-i in one workgroup (heavy one first): every
    // workgroup then walks the same number of key blocks and the launch has no tail of light workgroups.
    const bool pair = CAUSAL && !SPLIT && p.pair_mblocks != 0;
    const WorkgroupJob wg = deal_workgroup(p, blockIdx.x);
    const int rem = wg.rem, head = wg.b * p.heads + wg.h;
    const int mb_idx = fast_div(rem, p.d_n_split);
    const int split = rem - mb_idx * n_split;
    const int njobs = pair ? 2 : 1;
#pragma clang loop unroll(disable)
    for (int job = 0; job < njobs; ++job) {
    if (job) __syncthreads();                    // every wave is done with the LDS tiles of the first query block
    int mb = mb_idx;
    if (CAUSAL) mb = (pair && job) ? mb_idx : n_mblk - 1 - mb_idx;     // heaviest query blocks first
    const int b = wg.b, h = wg.h;
    const int hk = wg.hk;                     // K/V head of this query head

    // key-block range of this workgroup
    // Sequence lengths that are not a multiple of the block sizes: the copies of K/V rows past the end return zeros
    // (bounds-checked buffer loads), the last key block runs the masked code instance, query rows past the end are
    // computed on clamped inputs and not stored.
    const int seqlen_k = keys_of_batch(p, b);
    // Causal mask aligned to the bottom right corner: query row i sees keys 0 .. i + causal_off.  Equal lengths (the
    // reference's Python API) give causal_off = 0.
    const int causal_off = seqlen_k - p.seqlen;
    const KeyBlocks kb = key_block_range<BN>(seqlen_k, CAUSAL, mb * kBlockM + kBlockM, causal_off, SPLIT, n_split, split, CAUSAL,
                                             p.blocks_per_split);
    const int nb_total = kb.total, nb_begin = kb.begin, nb_end = kb.end;
    const int q_row = mb * kBlockM + wave * 32 + lq;     // this lane's query row
    const bool q_valid = q_row < p.seqlen;
    const int q_ld = q_valid ? q_row : p.seqlen - 1;     // row read for lanes past the end

    // ---- Q fragment (B operand of S^T = K Q^T): 16 bytes per k-step, resident for the whole kernel.
    v4i qreg[KS];
    load_q8_fragments<KS>(qreg, p, b, h, q_ld, lh);
    const float qsc = DUMP_S ? p.qk_scale_log2 : load_q_scale_log2(p, b, h, q_ld);

    float m_run = -INFINITY, l_run = 0.f;
    float o_acc[DT][16];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[dt][r] = 0.f;

    // ---- global -> LDS copies (asynchronous, straight into LDS)
    const char* Kg = p.k + b * p.k_sb + hk * p.k_sh;
    const char* Vg = DUMP_S ? Kg : p.v + b * p.v_sb + hk * p.v_sh;
    const v4i k_rsrc = make_rsrc(Kg, (uint32_t)((seqlen_k - 1) * p.k_sn + D));
    const v4i v_rsrc = make_rsrc(Vg, (uint32_t)((seqlen_k - 1) * p.v_sn + DV));
    const uint32_t k_sn = (uint32_t)p.k_sn, v_sn = (uint32_t)p.v_sn;
    const auto k_lane = tile_load_lane<D, SWZ_K, BN>(k_sn, wave, lane);
    const auto v_lane = tile_load_lane<DV, SWZ_V8, BN>(v_sn, wave, lane);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    auto issue_loads = [&](int nb, int buf) __attribute__((always_inline)) {
        issue_tile_load<D, SWZ_K, BN>(k_rsrc, (uint32_t)(nb * BN) * k_sn, k_sn, lds0 + OFF_K + buf * KT, wave, k_lane);
        if (!DUMP_S) issue_tile_load<DV, SWZ_V8, BN>(v_rsrc, (uint32_t)(nb * BN) * v_sn, v_sn, lds0 + OFF_V + buf * VT, wave, v_lane);
    };
    // The copy of the NEXT block is issued in slices spread over the stages of the current block (one K slice per
    // S^T sub-tile stage, one V slice per output d-tile stage) so that the waves do not queue behind a burst.
    constexpr int DMA_PARTS = TileLoadLane<D, SWZ_K, BN>::NINST / 4;
    constexpr int V_PARTS = TileLoadLane<DV, SWZ_V8, BN>::NINST / 4;
    // When there is no next block the slices are issued against an empty resource (num_records = 0: every access
    // is out of range and touches no memory), which keeps the stages free of branches.
    auto issue_k_slice = [&](v4i rsrc, int nb, int buf, int stage, int nstages) __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < DMA_PARTS; ++it)
            if (it * nstages / DMA_PARTS == stage)
                issue_tile_part<D, SWZ_K, BN>(rsrc, (uint32_t)(nb * BN) * k_sn, k_sn, lds0 + OFF_K + buf * KT, wave, k_lane, it);
    };
    auto issue_v_slice = [&](v4i rsrc, int nb, int buf, int stage, int nstages) __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < V_PARTS; ++it)
            if (it * nstages / V_PARTS == stage)
                issue_tile_part<DV, SWZ_V8, BN>(rsrc, (uint32_t)(nb * BN) * v_sn, v_sn, lds0 + OFF_V + buf * VT, wave, v_lane, it);
    };
    // k_scale of a block: thread t < 128 fetches the scale of key t; converted to fp32 when stored to LDS
    const KScaleSource ks_src(p, b, hk, seqlen_k);
    const int ks_key = tid & (BN - 1);
    auto load_ks = [&](int nb) __attribute__((always_inline)) -> uint32_t {           // raw bits
        return DUMP_S ? 0u : ks_src.load(nb * BN + ks_key);
    };
    auto cvt_ks = [&](uint32_t raw) __attribute__((always_inline)) -> float { return ks_src.cvt(raw); };
    // VBLK: channel scales of a key block; thread 128 + c fetches the scale of this workgroup's channel c.  A scale
    // row covers vs_g key blocks.
    // (Which threads fetch scales is decided per WAVE, from the wave index held in a scalar register: the branches
    // below are scalar branches that leave the exec mask alone.  A per-thread test of threadIdx would mask lanes off, and
    // a register spill or reload that the compiler places in the block where such lanes rejoin runs before the mask is
    // restored there: the lanes that were off lose the value.)
    const bool ks_wave = wave < BN / 64;             // threads 0 .. BN-1: one k_scale each
    const int vs_c = tid - 128;
    const bool vs_thread = VBLK && wave >= 2 && (wave - 2) * 64 < DV;   // threads 128 .. 128 + DV - 1: one channel each
    // (these scales are fp32 whatever the type of the per-token scales, as in the reference's kernel)
    const float* Vsg = (const float*)p.v_scale + (b * p.vs_sb + hk * p.vs_sh + (vs_thread ? vs_c : 0));
    // (VBLK == 2: scale rows 2 nb and 2 nb + 1; the second one does not exist when the sequence ends inside the block's
    // first half - its keys are masked, any row serves)
    const int vs_last_row = VBLK == 2 ? (p.seqlen_k + 63) / 64 - 1 : 0;
    auto load_vs = [&](int nb, int sub) __attribute__((always_inline)) -> float {
        if (!VBLK) return 0.f;
        int row = p.vs_g == 1 ? nb : nb / p.vs_g;
        if (VBLK == 2) { row = 2 * nb + sub; row = row < vs_last_row ? row : vs_last_row; }
        return Vsg[(int64_t)row * p.vs_sblk];
    };
    const uint32_t vs_wr = OFF_VS + 4 * (vs_thread ? vs_c : 0);     // + 4 * DV for the second scale row of a block
    const uint32_t vs_rd = OFF_VS + 16 * lh;       // + 4 * (DV * sub + 32*dt + 8*a4) per read

    // ---- per-lane LDS read offsets (everything else is an immediate)
    // K (A operand of S^T): lane reads row (32*st + lq), chunk (2*ks + lh), XOR-swizzled by the row
    const int k_swz = swz_k<D>(lq) & (CH - 1);
    uint32_t k_rd[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        k_rd[ks] = OFF_K + lq * D + (((2 * ks + lh) ^ k_swz) << 4);
    }
    // V (A operand of O^T = V^T P^T) through the transposing 8-byte load: source lane s of a 16-lane group points at
    // key row 8*(j>>2) + 4*lh + (j&3), j = s/2 (+16 for the second load, +32 per sub-tile), 8-byte half s&1
    const int g16 = lane >> 4, i16 = lane & 15, jj = i16 >> 1;
    const int v_row0 = 8 * (jj >> 2) + 4 * lh + (jj & 3);
    const int v_swz = swz_v8<DV>(v_row0) & SWM;
    uint32_t v_rd[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const int c = 2 * dt + (g16 & 1);
        v_rd[dt] = OFF_V + v_row0 * DV + 8 * (i16 & 1) + (((c & SWM) ^ v_swz) << 4) + ((c & ~SWM) << 4);
    }
    const uint32_t ks_rd = OFF_KS + 16 * lh;     // + 4 * (32*st + 8*a4) per read
    const uint32_t ks_wr = OFF_KS + 4 * (tid & (BN - 1));

    // One key block out of LDS buffer BUF.  DIAG selects the code for the block on the causal diagonal.
    // DIAG selects the code instance with masking: keys whose index inside the block exceeds the lane's `lim` are masked
    // and sub-tiles st > gw (wave-uniform, the sub-tile of the largest lim in the wave) are skipped.  Causal diagonal:
    // lim = the lane's last visible key; last block of a ragged sequence: lim = the last valid key.
    auto compute = [&](auto buf_tag, auto diag_tag, int nb, bool more, int gw_in, int lim, int lim_lo) __attribute__((always_inline)) {
        constexpr int BUF = decltype(buf_tag)::value ? 1 : 0;
        constexpr bool DIAG = decltype(diag_tag)::value;
        constexpr int KB = BUF * KT, VB = BUF * VT, SB = BUF * BN * 4;
        const int gw = gw_in;                              // wave-uniform; nact = active sub-tiles
        const int nact = DIAG ? (gw + 1 < NST ? gw + 1 : NST) : NST;
        if (DIAG && nact <= 0) return;                     // every key of this block is above the wave's rows
        v4i k_next = k_rsrc, v_next = v_rsrc;
        if (!more) { k_next[2] = 0; v_next[2] = 0; }
        // LDS operand fetches are issued one stage ahead of their MFMAs, in program order pinned by scheduling
        // barriers: the fragments of sub-tile st+1 (d-tile dt+1) are requested right after the MFMAs of st (dt)
        // have been issued and arrive while this wave does the vector work of st (dt).
        auto load_kfrags = [&](v4i (&fr)[KS], int st) __attribute__((always_inline)) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) fr[ks] = *(const v4i*)(smem + k_rd[ks] + KB + 32 * st * D);
        };
        auto load_vfrags = [&](v4i (&vf)[NST], int dt) __attribute__((always_inline)) {
#pragma unroll
            for (int st = 0; st < NST; ++st) {
                if (DIAG && st > gw && VBLK != 2) continue;     // (VBLK == 2 multiplies every sub-tile: P8 of a hidden one is 0)
                const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                    (__attribute__((address_space(3))) v2i*)INTFA_LDS(smem + v_rd[dt] + VB + (32 * st) * DV));
                const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                    (__attribute__((address_space(3))) v2i*)INTFA_LDS(smem + v_rd[dt] + VB + (32 * st + 16) * DV));
                vf[st] = (v4i){lo[0], lo[1], hi[0], hi[1]};
            }
        };
        // -------- pass 1: S^T sub-tiles, dequantise by k_scale, running row max.
        // Software pipeline inside the wave: the MFMA chain of sub-tile st+1 is issued before the vector work of
        // sub-tile st (the matrix core runs under the wave's own VALU instructions), and LDS operands are requested
        // two stages before the MFMA that consumes them (double-buffered fragments).
        float t[NST][16];
        float mx = -INFINITY;
        v4i fr[2][KS];
        v4i vf[2][NST];
        v16i sacc[2];
        // k_scale of the lane's keys, one quarter (4 keys) per register quad; a quad is refilled for the next sub-tile right
        // after the quarter that consumed it (three quarters of vector work ahead of its next use)
        v4f kk[4];
        auto load_kk = [&](int a4, int st) __attribute__((always_inline)) {
            kk[a4] = *(const v4f*)(smem + ks_rd + SB + 4 * (32 * st + 8 * a4));
        };
        auto qk_chain = [&](v16i& acc, const v4i (&f)[KS]) __attribute__((always_inline)) {
            acc = (v16i){0};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(f[ks], qreg[ks], acc, 0, 0, 0);
        };
        load_kfrags(fr[0], 0);
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) load_kk(a4, 0);
        if (1 < nact) load_kfrags(fr[1], 1);
        __builtin_amdgcn_sched_barrier(0);
        qk_chain(sacc[0], fr[0]);
        // The MFMAs of sub-tile st+1 are issued one at a time between quarters of the vector work of sub-tile st: each
        // quarter (4 keys: convert, scale, max) outlasts one MFMA, so the next MFMA of the dependent chain never
        // stalls the wave at issue and the matrix core runs entirely under this wave's own vector instructions.
#pragma unroll
        for (int st = 0; st < NST; ++st) {
            if (DIAG && st > gw) {                            // sub-tile entirely above the diagonal
#pragma unroll
                for (int r = 0; r < 16; ++r) t[st][r] = -INFINITY;
                continue;
            }
            const bool next = st + 1 < NST && st + 1 < nact;
            __builtin_amdgcn_sched_barrier(0);
            if (st + 2 < NST && st + 2 < nact) load_kfrags(fr[st & 1], st + 2);
            if (!DUMP_S && !DIAG) issue_k_slice(k_next, nb + 1, BUF ^ 1, st, NST);
            const v16i& acc = sacc[st & 1];
            v16i& nacc = sacc[(st + 1) & 1];
            if (DUMP_S) {
                const int key0 = nb * BN + 32 * st;
                int32_t* srow = p.s_dump + ((int64_t)(b * p.heads + h) * p.seqlen + q_ld) * p.seqlen_k + key0;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int kidx = 8 * (r >> 2) + 4 * lh + (r & 3);
                    if (q_valid && key0 + kidx < p.seqlen_k) srow[kidx] = acc[r];
                }
            }
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                __builtin_amdgcn_sched_barrier(0);
                if (next) {
#pragma unroll
                    for (int ks = a4 * KS / 4; ks < (a4 + 1) * KS / 4; ++ks) {
                        if (ks == 0) nacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fr[(st + 1) & 1][0], qreg[0], (v16i){0}, 0, 0, 0);
                        else nacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fr[(st + 1) & 1][ks], qreg[ks], nacc, 0, 0, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                float xq[4];
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) xq[b4] = (float)acc[4 * a4 + b4] * kk[a4][b4];
                if (next) load_kk(a4, st + 1);
                if (DIAG && 32 * st + 31 > lim_lo) {           // wave-uniform: some lane of the wave has a hidden key in this sub-tile
#pragma unroll
                    for (int b4 = 0; b4 < 4; ++b4)
                        if ((32 * st + 8 * a4 + b4 + 4 * lh) > lim) xq[b4] = -INFINITY;
                }
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) {
                    const float x = xq[b4];
                    t[st][4 * a4 + b4] = x;
                    mx = fmaxf(mx, x);
                }
            }
        }
        if (DUMP_S) return;
        // V fragments of the first two d-tiles travel while the exponentials are evaluated
        load_vfrags(vf[0], 0);
        if (1 < DT) load_vfrags(vf[1], 1);
        mx = half_pair_max(mx);
        const float m_new = fmaxf(m_run, mx * qsc);
        float alpha = fast_exp2(m_run - m_new);
        // materialised here, well ahead of the hand-written v_fma_f32 that consumes it: the result of a transcendental
        // needs a wait state before its first use, which the compiler inserts for its own instructions only
        asm volatile("" : "+v"(alpha));
        m_run = m_new;
        // -------- pass 2: P = exp2(x*qsc - m), row sum, requantise
        float lsum = 0.f;
        v4i p8[NST];
        v16i oacc[2];
        const float bias = (PROUND == 0 ? kLog2_127 : 0.f) - m_new;
#pragma unroll
        for (int st = 0; st < NST; ++st) {
            __builtin_amdgcn_sched_barrier(0);
            // V of the next block is requested here, well before the end of this block, so that the copy has landed
            // when the next block waits for it (its buffer was last read before this block's barrier)
            if (!DIAG) issue_v_slice(v_next, nb + 1, BUF ^ 1, st, NST);
            __builtin_amdgcn_sched_barrier(0);
            if (PROUND == 0) {
#pragma unroll
                for (int w4 = 0; w4 < 4; ++w4) {
                    unsigned pk = 0;
#pragma unroll
                    for (int b4 = 0; b4 < 4; ++b4) {
                        const float e = fast_exp2(fmaf(t[st][4 * w4 + b4], qsc, bias));   // 127 * p
                        lsum += e;
                        pk = __builtin_amdgcn_cvt_pk_u8_f32(e, b4, pk);
                    }
                    p8[st][w4] = (int)pk;
                }
            } else {
                // the reference's fp16 chain: fp16(p) * 127 -> fp16, + 0.5 -> fp16, truncate
                float e[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    e[r] = fast_exp2(fmaf(t[st][r], qsc, bias));                          // p
                    lsum += e[r];
                }
                p8[st] = requant_p_reference16(e);
            }
            asm volatile("" : "+v"(lsum));      // keep the row-sum chain inside its stage
            // the P V chain of the first d-tile advances by one MFMA as soon as this sub-tile's P8 is packed: it runs
            // under the exponentials of the next sub-tile instead of in a burst behind the pass
            if (VBLK == 2) {                     // keys 0..63 of the block only: the second half is a chain (and a scale row) of its own
                if (st == 0) oacc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf[0][0], p8[0], (v16i){0}, 0, 0, 0);
                if (st == 1) oacc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf[0][1], p8[1], oacc[0], 0, 0, 0);
            } else if (!(DIAG && st > gw)) {
                if (st == 0) oacc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf[0][0], p8[0], (v16i){0}, 0, 0, 0);
                else oacc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf[0][st], p8[st], oacc[0], 0, 0, 0);
            }
        }
        // -------- P V on int8 MFMA: O^T[d, q] += V^T[d, key] P^T[key, q]; the chain of d-tile dt+1 is issued
        // before the accumulator update of d-tile dt, its V fragments were requested two stages earlier.
        constexpr int VSB = BUF * VSUB * DV * 4;
        v4f vsc[2][4];                          // VBLK: channel scales of the d-tile being folded in / the next one
        if constexpr (VBLK == 2) {
            // Stage s = 2 dt + half: the int32 sum of d-tile dt over the keys 64 half .. 64 half + 63 of the block, times that
            // half's channel scales.  Stage 0 was multiplied during pass 2; the MFMAs of stage s + 1 are issued between the
            // quarters of the update of stage s.
            constexpr int NS = 2 * DT;
            // (one quad of channel scales per quarter, refilled for the next stage right after the quarter that used it)
            auto load_vsc2 = [&](int a4, int s2) __attribute__((always_inline)) {
                vsc[0][a4] = *(const v4f*)(smem + vs_rd + VSB + 4 * (DV * (s2 & 1) + 32 * (s2 >> 1) + 8 * a4));
            };
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) load_vsc2(a4, 0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s2 = 0; s2 < NS; ++s2) {
                const int dt = s2 >> 1, half = s2 & 1;
                const int dtn = (s2 + 1) >> 1, halfn = (s2 + 1) & 1;      // the stage whose MFMAs are issued here
                __builtin_amdgcn_sched_barrier(0);
                // V fragments of d-tile dt + 2 replace those of d-tile dt once its second half has been issued
                if (half == 1 && dt + 2 < DT) load_vfrags(vf[dt & 1], dt + 2);
                v16i& nacc = oacc[(s2 + 1) & 1];
#pragma unroll
                for (int a4 = 0; a4 < 4; ++a4) {
                    __builtin_amdgcn_sched_barrier(0);
                    if (s2 + 1 < NS && (a4 & 1) == 0) {
                        const int st = 2 * halfn + (a4 >> 1);
                        if (a4 == 0) nacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf[dtn & 1][st], p8[st], (v16i){0}, 0, 0, 0);
                        else nacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf[dtn & 1][st], p8[st], nacc, 0, 0, 0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int b4 = 0; b4 < 4; ++b4) {
                        const int r = 4 * a4 + b4;
                        const float pv = (float)oacc[s2 & 1][r] * vsc[0][a4][b4];
                        if (half == 0) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(o_acc[dt][r]) : "v"(alpha), "v"(pv));
                        else o_acc[dt][r] += pv;
                    }
                    if (s2 + 1 < NS) load_vsc2(a4, s2 + 1);
                }
            }
        } else {
        auto load_vsc = [&](v4f (&dst)[4], int dt) __attribute__((always_inline)) {
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) dst[a4] = *(const v4f*)(smem + vs_rd + VSB + 4 * (32 * dt + 8 * a4));
        };
        if (VBLK) load_vsc(vsc[0], 0);
        __builtin_amdgcn_sched_barrier(0);
        // As in pass 1: the MFMAs of d-tile dt+1 are issued one at a time between quarters of the accumulator update
        // of d-tile dt.
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            __builtin_amdgcn_sched_barrier(0);
            if (dt + 2 < DT) load_vfrags(vf[dt & 1], dt + 2);
            if (VBLK && dt + 1 < DT) load_vsc(vsc[(dt + 1) & 1], dt + 1);
            v16i& nacc = oacc[(dt + 1) & 1];
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                __builtin_amdgcn_sched_barrier(0);
                if (dt + 1 < DT) {
#pragma unroll
                    for (int st = a4 * NST / 4; st < (a4 + 1) * NST / 4; ++st) {
                        if (DIAG && st > gw) continue;
                        if (st == 0) nacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf[(dt + 1) & 1][0], p8[0], (v16i){0}, 0, 0, 0);
                        else nacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf[(dt + 1) & 1][st], p8[st], nacc, 0, 0, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) {
                    const int r = 4 * a4 + b4;
                    float pv = (float)oacc[dt & 1][r];
                    if (VBLK) pv *= vsc[dt & 1][a4][b4];
                    // o = o * alpha + pv, written as the three-operand instruction in place: left to the compiler the
                    // update is either sunk below the loop (no vector work beside the MFMAs of this stage) or, pinned
                    // here by an empty asm, emitted as v_fmac into the temporary plus a copy back (one instruction more
                    // per output element and block).
                    asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(o_acc[dt][r]) : "v"(alpha), "v"(pv));
                }
            }
        }
        }   // VBLK != 2
        l_run = fmaf(l_run, alpha, lsum);
    };

    // One pipeline step on LDS buffer BUF: wait for this block's tiles (issued one step earlier), make them
    // visible to all four waves, start the copy of the next block into the other buffer, compute.
    auto step = [&](auto buf_tag, auto diag_tag, int nb, int gw, int lim, int lim_lo) __attribute__((always_inline)) {
        constexpr int BUF = decltype(buf_tag)::value ? 1 : 0;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        const bool more = nb + 1 < nb_end;
        uint32_t ks_next = 0;
        float vs_next[VSUB] = {};
        constexpr bool DIAG = decltype(diag_tag)::value;
        if (more) {
            if (DUMP_S || DIAG) issue_loads(nb + 1, BUF ^ 1);      // (a diagonal block is the last one: more == false)
            ks_next = load_ks(nb + 1);
            if (vs_thread) {
#pragma unroll
                for (int sub = 0; sub < VSUB; ++sub) vs_next[sub] = load_vs(nb + 1, sub);
            }
        }
        compute(buf_tag, diag_tag, nb, more, gw, lim, lim_lo);
        if (more && ks_wave) *(float*)(smem + ks_wr + (BUF ^ 1) * BN * 4) = cvt_ks(ks_next);
        if (more && vs_thread) {
#pragma unroll
            for (int sub = 0; sub < VSUB; ++sub) *(float*)(smem + vs_wr + ((BUF ^ 1) * VSUB + sub) * DV * 4) = vs_next[sub];
        }
    };

    // ---- main loop: K/V tiles double-buffered in LDS, one barrier per key block.  The block on the causal
    // diagonal is always the last of the range and gets its own code instance after the loop.
    if (nb_begin < nb_end) {
        issue_loads(nb_begin, 0);
        {
            const uint32_t s0 = load_ks(nb_begin);
            if (ks_wave) *(float*)(smem + ks_wr) = cvt_ks(s0);
            if (vs_thread) {
#pragma unroll
                for (int sub = 0; sub < VSUB; ++sub) *(float*)(smem + vs_wr + sub * DV * 4) = load_vs(nb_begin, sub);
            }
        }
        // first key block that holds a key hidden from the first row of this query block (every block before it is
        // visible to all rows and runs without a mask)
        const int diag_first = (mb * kBlockM + causal_off + 1) / BN;
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
        // masked blocks: the blocks the causal diagonal of this query block crosses (kBlockM / BN of them when the lengths
        // are equal, one more when the offset is not a multiple of the block; keys past the end of a ragged sequence lie above
        // every valid row's diagonal), or the ragged last block of a non-causal pass
#pragma clang loop unroll(disable)
        for (; nb < nb_end; ++nb) {
            // lane: last visible key relative to the block; wave: sub-tile of the largest of them (negative: none)
            const int lim = CAUSAL ? q_row + causal_off - nb * BN : tail_keys - 1;
            const int gw = (CAUSAL ? mb * kBlockM + wave * 32 + 31 + causal_off - nb * BN : tail_keys - 1) >> 5;
            // smallest lim in the wave: sub-tiles that end at or below it need no per-key test
            const int lim_lo = CAUSAL ? mb * kBlockM + wave * 32 + causal_off - nb * BN : tail_keys - 1;
            if (((nb - nb_begin) & 1) == 0) step(BoolTag<false>{}, BoolTag<true>{}, nb, gw, lim, lim_lo);
            else step(BoolTag<true>{}, BoolTag<true>{}, nb, gw, lim, lim_lo);
        }
    }
    if (DUMP_S) return;

    // ---- epilogue.  Everything it needs from the parameter block is (re)loaded here, behind an opaque copy of the
    // kernel-argument pointer, so that these values do not occupy scalar registers during the main loop.
    const KernargPtr pe = kernarg_block();
    const int e_heads = pe->heads, e_seqlen = pe->seqlen;
    const int eb = fast_div(head, pe->d_heads), eh = head - eb * e_heads;
    const float l_tot = half_pair_sum(l_run);          // in units of 1/127 when PROUND == 0
    const float vs = VBLK ? 1.f : load_scale(pe->v_scale, eb * pe->vs_sb + fast_div(eh, pe->d_kv_group) * pe->vs_sh, pe->scale_dtype);
    // (no visible key at all - an empty cache entry, or a causal row above the first key when there are fewer keys than
    // queries - gives zeros and lse = -inf; such a row's accumulators hold NaN from exp2(-inf - -inf), hence the selects)
    const bool any_key = nb_begin < nb_end && m_run > -INFINITY;
    const float out_scale = !any_key ? 0.f : (PROUND == 0) ? (vs / l_tot) : (vs / (127.f * l_tot));
    const float l_true = (PROUND == 0) ? l_tot * (1.f / 127.f) : l_tot;
    const float lse = any_key ? m_run + __builtin_log2f(l_true) : -INFINITY;
    if (SPLIT) {
        const int64_t row = ((int64_t)(split * pe->batch + eb) * e_heads + eh) * e_seqlen + q_row;
        float* op = pe->o_part + row * D;
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
                    for (int b4 = 0; b4 < 4; ++b4) o[b4] = seen ? o_acc[dt][4 * a4 + b4] * out_scale : 0.f;
                    *(v4f*)(op + 32 * dt + 8 * a4 + 4 * lh) = o;
                }
            if (lh == 0) pe->lse_part[row] = seen ? lse : -INFINITY;
        }
        return;
    }
    if constexpr (!DUMP_S) {
    // 16-bit rows go out through LDS (whole lines per store instruction); the tiles are dead once every wave is here
    static_assert(4 * OutStage<DV>::BYTES <= LDS_BYTES, "output staging fits the tile memory");
    // (the last block's copy slices ran against an empty resource: they fetch nothing but still write zeros into the
    // other tile buffers, asynchronously - every wave awaits its own before the barrier)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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
            if (OUT_DT == 0) {
                v4h o;
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) o[b4] = (_Float16)(any_key ? o_acc[dt][4 * a4 + b4] * out_scale : 0.f);
                out_stage_put<DV>(stage, lq_e, d0, __builtin_bit_cast(v2i, o));
            } else {
                v4s o;
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) o[b4] = f32_to_bf16(any_key ? o_acc[dt][4 * a4 + b4] * out_scale : 0.f);
                out_stage_put<DV>(stage, lq_e, d0, __builtin_bit_cast(v2i, o));
            }
        }
    const int row0 = mb * kBlockM + wave * 32;
    out_stage_flush<DV>(stage, pe->out + eb * pe->o_sb + eh * pe->o_sh + (int64_t)row0 * pe->o_sn, pe->o_sn, e_seqlen - row0, lane_e);
    if (q_valid && pe->lse != nullptr && lh == 0) pe->lse[((int64_t)eb * e_heads + eh) * e_seqlen + q_row] = lse;
    }
    }   // job
#endif  // __HIP_DEVICE_COMPILE__
}

}  // namespace intfa
