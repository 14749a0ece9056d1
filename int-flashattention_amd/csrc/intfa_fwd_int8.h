// Forward kernels with int8 Q K^T: full-int8 (int8 P V) and half-int8 (fp16/bf16 P V).
//
// Algorithm restated from the reference tile loop (flash_atten_full_int8.py:9-71, flash_atten_int8.py:9-66):
// per key block of kBlockN keys, S = Q8 K8^T in int32; X = S * q_scale[row] * k_scale[col]; running max m in
// the exp2 domain; P = exp2(X * c - m_new); l sums the UNQUANTISED P; P is requantised to int8 with the fixed
// scale 127 (full) or cast to half precision (half); acc = acc * alpha + P V; output acc / l.
// Differences in evaluation order that stay within fp32 rounding: q_scale * c is folded into one per-row
// factor, v_scale / 127 is applied once in the epilogue, and (RNE mode) the factor 127 is folded into the
// exponent as exp2(x + log2 127).
#pragma once
#include "intfa_device.h"

namespace intfa {

enum { VAR_FULL = 0, VAR_HALF = 1 };

template <bool V> struct BoolTag { static constexpr bool value = V; };

template <int D> struct SmemInt8 {
    char k[2][kBlockN * D];
    char v[2][kBlockN * D * 2];     // sized for 16-bit V; the int8 variant uses the first half of each
    float ks[2][kBlockN];
};

// One workgroup = one (batch, head, 128-query block[, split]).
template <int VARIANT, int D, bool CAUSAL, int OUT_DT /*0 f16, 1 bf16*/, int PROUND, bool DUMP_S, bool SPLIT>
__global__ void __launch_bounds__(kThreads, 2) fwd_int8_kernel(const KParams p) {
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass only needs the kernel's symbol
    constexpr int KS = D / 32;                   // k-steps of Q K^T (32 bytes of head_dim each)
    constexpr int DT = D / 32;                   // 32-wide output tiles along head_dim
    constexpr int VB = (VARIANT == VAR_FULL) ? 1 : 2;   // bytes per V element
    constexpr int VROW = D * VB;

    __shared__ __attribute__((aligned(1024))) char sK0[kBlockN * D];
    __shared__ __attribute__((aligned(1024))) char sK1[kBlockN * D];
    __shared__ __attribute__((aligned(1024))) char sV0[kBlockN * VROW];
    __shared__ __attribute__((aligned(1024))) char sV1[kBlockN * VROW];
    __shared__ __attribute__((aligned(16))) float sKs0[kBlockN];
    __shared__ __attribute__((aligned(16))) float sKs1[kBlockN];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lq = lane & 31, lh = lane >> 5;

    // ---- block -> (head, m-block, split).  Workgroups are dealt round-robin to the 8 XCDs, each with its own
    // L2; give every XCD whole heads so that the K/V tiles of a head are re-read from one L2.
    const int n_mblk = p.seqlen / kBlockM;
    const int n_split = SPLIT ? p.num_splits : 1;
    const int per_head = n_mblk * n_split;
    const int n_heads = p.batch * p.heads;
    int bid = blockIdx.x;
    int head, rem;
    if ((n_heads & 7) == 0) {
        const int xcd = bid & 7, slot = bid >> 3;
        head = (slot / per_head) * 8 + xcd;
        rem = slot % per_head;
    } else {
        head = bid / per_head;
        rem = bid % per_head;
    }
    int mb = rem / n_split;
    const int split = rem % n_split;
    if (CAUSAL) mb = n_mblk - 1 - mb;            // heaviest query blocks first
    const int b = head / p.heads, h = head % p.heads;

    // key-block range of this workgroup
    int nb_begin = 0, nb_end = CAUSAL ? (mb + 1) : (p.seqlen / kBlockN);
    if (SPLIT) {
        nb_begin = split * p.blocks_per_split;
        const int e = nb_begin + p.blocks_per_split;
        nb_end = e < nb_end ? e : nb_end;
    }

    const char* Kg = p.k + b * p.k_sb + h * p.k_sh;
    const char* Vg = p.v + b * p.v_sb + h * p.v_sh;
    const char* Ksg = p.k_scale;
    const int64_t ks_base = b * p.ks_sb + h * p.ks_sh;
    const int q_row = mb * kBlockM + wave * 32 + lq;     // this lane's query row

    // ---- Q fragment (B operand of S^T = K Q^T): 16 bytes per k-step, resident for the whole kernel.
    v4i qreg[KS];
    {
        const char* qrow = p.q + b * p.q_sb + h * p.q_sh + (int64_t)q_row * p.q_sn;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qreg[ks] = *(const v4i*)(qrow + ks * 32 + lh * 16);
    }
    const float qs = DUMP_S ? 1.f : load_scale(p.q_scale, b * p.qs_sb + h * p.qs_sh + (int64_t)q_row * p.qs_sn, p.scale_dtype);
    const float qsc = qs * p.qk_scale_log2;

    float m_run = -INFINITY, l_run = 0.f;
    float o_acc[DT][16];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[dt][r] = 0.f;

    // per-lane pieces of the LDS read addresses
    // K (A operand of S^T): lane reads row (32*st + lq), chunk (2*ks + lh)
    const int k_swz = swz_k<D>(lq) & ((D / 16 < 8 ? D / 16 : 8) - 1);
    // V (A operand of O^T = V^T P^T) through the transposing 8-byte load; see intfa_device.h
    const int g16 = lane >> 4, i16 = lane & 15, jj = i16 >> 1;
    const int v_row0 = 8 * (jj >> 2) + 4 * lh + (jj & 3);          // + 16*w + 32*st
    const int v_sub = 8 * (i16 & 1);
    const int v_swz = swz_v<VROW>(v_row0) & ((VROW / 16 < 8 ? VROW / 16 : 8) - 1);

    const auto k_lane = tile_load_lane<D, false>((uint32_t)p.k_sn, wave, lane);
    const auto v_lane = tile_load_lane<VROW, true>((uint32_t)p.v_sn, wave, lane);
    const __amdgpu_buffer_rsrc_t k_rsrc = make_rsrc(Kg, (uint32_t)((p.seqlen - 1) * p.k_sn + D));
    const __amdgpu_buffer_rsrc_t v_rsrc = make_rsrc(DUMP_S ? Kg : Vg, (uint32_t)((p.seqlen - 1) * p.v_sn + VROW));
    auto issue_loads = [&](int nb, char* dK, char* dV) __attribute__((always_inline)) {
        issue_tile_load<D, false>(k_rsrc, (uint32_t)(nb * kBlockN) * (uint32_t)p.k_sn, (uint32_t)p.k_sn, dK, wave, k_lane);
        if (!DUMP_S) issue_tile_load<VROW, true>(v_rsrc, (uint32_t)(nb * kBlockN) * (uint32_t)p.v_sn, (uint32_t)p.v_sn, dV, wave, v_lane);
    };
    // k_scale of the block: thread t < 128 fetches the scale of key t, converted to fp32 when stored to LDS
    const int ks_esize = p.scale_dtype == 2 ? 4 : 2;
    const __amdgpu_buffer_rsrc_t ks_rsrc =
        make_rsrc(DUMP_S ? Kg : Ksg + ks_base * ks_esize, DUMP_S ? 0u : (uint32_t)(((p.seqlen - 1) * p.ks_sn + 1) * ks_esize));
    const uint32_t ks_lane = (uint32_t)(tid & (kBlockN - 1)) * (uint32_t)(p.ks_sn * ks_esize);
    auto load_ks = [&](int nb) __attribute__((always_inline)) -> uint32_t {           // raw bits; converted by cvt_ks
        if (DUMP_S) return 0u;
        const uint32_t so = (uint32_t)(nb * kBlockN) * (uint32_t)(p.ks_sn * ks_esize);
        if (p.scale_dtype == 2) return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(ks_rsrc, ks_lane, so, 0);
        return (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(ks_rsrc, ks_lane, so, 0);
    };
    auto cvt_ks = [&](uint32_t raw) __attribute__((always_inline)) -> float {
        if (p.scale_dtype == 0) return (float)__builtin_bit_cast(_Float16, (uint16_t)raw);
        if (p.scale_dtype == 1) return __builtin_bit_cast(float, raw << 16);
        return __builtin_bit_cast(float, raw);
    };

    // One key block.  DIAG selects the code for the block on the causal diagonal (mask + sub-tile skip).
    auto compute = [&](auto diag_tag, int nb, const char* cK, const char* cV, const float* cKs) __attribute__((always_inline)) {
        constexpr bool DIAG = decltype(diag_tag)::value;
        // Loop-invariant address pieces are re-derived per block from two opaque values, so the compiler does not
        // keep a register per (k-step, d-tile) variant alive across the whole loop.
        int ksw = k_swz, vsw = v_swz;
        asm volatile("" : "+v"(ksw), "+v"(vsw));
        // -------- pass 1: S^T sub-tiles, dequantise by k_scale, running row max
        float t[4][16];
        float mx = -INFINITY;
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            if (DIAG && st > wave) {                          // sub-tile entirely above the diagonal
#pragma unroll
                for (int r = 0; r < 16; ++r) t[st][r] = -INFINITY;
                continue;
            }
            __builtin_amdgcn_sched_barrier(0);
            v16i acc = {0};
            const char* krow = cK + (32 * st + lq) * D;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const v4i a = *(const v4i*)(krow + (((2 * ks + lh) ^ ksw) << 4));
                acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, qreg[ks], acc, 0, 0, 0);
            }
            if (DUMP_S) {
                int32_t* srow = p.s_dump + ((int64_t)(b * p.heads + h) * p.seqlen + q_row) * p.seqlen + nb * kBlockN + 32 * st;
#pragma unroll
                for (int r = 0; r < 16; ++r) srow[8 * (r >> 2) + 4 * lh + (r & 3)] = acc[r];
            }
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                const v4f kk = *(const v4f*)(cKs + 32 * st + 8 * a4 + 4 * lh);
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) {
                    float x = (float)acc[4 * a4 + b4] * kk[b4];
                    if (DIAG) {
                        // position of the key inside the 32x32 tile on the diagonal vs this lane's query
                        if (st == wave && (8 * a4 + b4) > lq - 4 * lh) x = -INFINITY;
                    }
                    t[st][4 * a4 + b4] = x;
                    mx = fmaxf(mx, x);
                }
            }
        }
        if (DUMP_S) return;
        mx = fmaxf(mx, wave_half_swap(mx));
        const float m_new = fmaxf(m_run, mx * qsc);
        const float alpha = fast_exp2(m_run - m_new);
        m_run = m_new;
        // -------- pass 2: P = exp2(x*qsc - m), row sum, requantise
        float lsum = 0.f;
        if (VARIANT == VAR_FULL) {
            v4i p8[4];
            const float bias = (PROUND == 0 ? kLog2_127 : 0.f) - m_new;
#pragma unroll
            for (int st = 0; st < 4; ++st) {
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int w4 = 0; w4 < 4; ++w4) {
                    unsigned pk = 0;
                    if (PROUND == 0) {
#pragma unroll
                        for (int b4 = 0; b4 < 4; ++b4) {
                            const float e = fast_exp2(fmaf(t[st][4 * w4 + b4], qsc, bias));   // 127 * p
                            lsum += e;
                            pk = __builtin_amdgcn_cvt_pk_u8_f32(e, b4, pk);
                        }
                    } else {
                        // the reference's fp16 chain: fp16(p) * 127 -> fp16, + 0.5 -> fp16, truncate
#pragma unroll
                        for (int b4 = 0; b4 < 4; ++b4) {
                            const float e = fast_exp2(fmaf(t[st][4 * w4 + b4], qsc, bias));   // p
                            lsum += e;
                            _Float16 hp = (_Float16)e;
                            hp = hp * (_Float16)127.0f;
                            hp = hp + (_Float16)0.5f;
                            const unsigned q8 = (unsigned)(int)hp;          // truncating convert, 0..127
                            pk |= q8 << (8 * b4);
                        }
                    }
                    p8[st][w4] = (int)pk;
                }
            }
            // -------- P V on int8 MFMA: O^T[d, q] += V^T[d, key] P^T[key, q]
            const char* vbase = cV + v_row0 * VROW + v_sub;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                __builtin_amdgcn_sched_barrier(0);
                v16i acc = {0};
                const int coff = ((2 * dt + (g16 & 1)) ^ vsw) << 4;
#pragma unroll
                for (int st = 0; st < 4; ++st) {
                    if (DIAG && st > wave) continue;
                    const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                        (__attribute__((address_space(3))) v2i*)INTFA_LDS(vbase + (32 * st) * VROW + coff));
                    const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                        (__attribute__((address_space(3))) v2i*)INTFA_LDS(vbase + (32 * st + 16) * VROW + coff));
                    const v4i a = {lo[0], lo[1], hi[0], hi[1]};
                    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, p8[st], acc, 0, 0, 0);
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) o_acc[dt][r] = fmaf(o_acc[dt][r], alpha, (float)acc[r]);
            }
        }
        l_run = fmaf(l_run, alpha, lsum);
    };
    // One pipeline step on LDS buffer BUF: wait for this block's tiles (issued one step earlier), make them
    // visible to all four waves, start the copy of the next block into the other buffer, compute.
    auto step = [&](auto buf_tag, auto diag_tag, int nb) __attribute__((always_inline)) {
        constexpr bool B1 = decltype(buf_tag)::value;
        char* cK = B1 ? sK1 : sK0; char* cV = B1 ? sV1 : sV0; float* cKs = B1 ? sKs1 : sKs0;
        char* nK = B1 ? sK0 : sK1; char* nV = B1 ? sV0 : sV1; float* nKs = B1 ? sKs0 : sKs1;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        const bool more = nb + 1 < nb_end;
        uint32_t ks_next = 0;
        if (more) { issue_loads(nb + 1, nK, nV); ks_next = load_ks(nb + 1); }
        compute(diag_tag, nb, cK, cV, cKs);
        if (more && tid < kBlockN) nKs[tid] = cvt_ks(ks_next);
    };

    // ---- main loop: K/V tiles double-buffered in LDS, one barrier per key block.  The block on the causal
    // diagonal is always the last of the range and gets its own code instance after the loop.
    if (nb_begin < nb_end) {
        issue_loads(nb_begin, sK0, sV0);
        {
            const uint32_t s0 = load_ks(nb_begin);
            if (tid < kBlockN) sKs0[tid] = cvt_ks(s0);
        }
        const bool has_diag = CAUSAL && (nb_end == mb + 1);
        const int plain_end = has_diag ? nb_end - 1 : nb_end;
        int nb = nb_begin;
        while (true) {
            if (nb >= plain_end) break;
            step(BoolTag<false>{}, BoolTag<false>{}, nb++);
            if (nb >= plain_end) break;
            step(BoolTag<true>{}, BoolTag<false>{}, nb++);
        }
        if (CAUSAL && has_diag) {
            if (((nb - nb_begin) & 1) == 0) step(BoolTag<false>{}, BoolTag<true>{}, nb);
            else step(BoolTag<true>{}, BoolTag<true>{}, nb);
        }
    }
    if (DUMP_S) return;

    // ---- epilogue
    const float l_tot = l_run + wave_half_swap(l_run);          // in units of 1/127 when PROUND == 0
    float out_scale;
    if (VARIANT == VAR_FULL) {
        const float vs = load_scale(p.v_scale, b * p.vs_sb + h * p.vs_sh, p.scale_dtype);
        out_scale = (PROUND == 0) ? (vs / l_tot) : (vs / (127.f * l_tot));
    } else {
        out_scale = 1.f / l_tot;
    }
    const float l_true = (VARIANT == VAR_FULL && PROUND == 0) ? l_tot * (1.f / 127.f) : l_tot;
    const float lse = m_run + __builtin_log2f(l_true);
    if (SPLIT) {
        const int64_t row = ((int64_t)(split * p.batch + b) * p.heads + h) * p.seqlen + q_row;
        float* op = p.o_part + row * D;
        const bool seen = nb_begin < nb_end;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                v4f o;
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) o[b4] = seen ? o_acc[dt][4 * a4 + b4] * out_scale : 0.f;
                *(v4f*)(op + 32 * dt + 8 * a4 + 4 * lh) = o;
            }
        if (lh == 0) p.lse_part[row] = seen ? lse : -INFINITY;
        return;
    }
    char* orow = p.out + b * p.o_sb + h * p.o_sh + (int64_t)q_row * p.o_sn;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
            const int d0 = 32 * dt + 8 * a4 + 4 * lh;
            if (OUT_DT == 0) {
                v4h o;
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) o[b4] = (_Float16)(o_acc[dt][4 * a4 + b4] * out_scale);
                *(v4h*)(orow + d0 * 2) = o;
            } else {
                v4s o;
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) {
                    const float f = o_acc[dt][4 * a4 + b4] * out_scale;
                    uint32_t u = __builtin_bit_cast(uint32_t, f);
                    u += 0x7fffu + ((u >> 16) & 1u);                // round-to-nearest-even to bf16
                    o[b4] = (short)(u >> 16);
                }
                *(v4s*)(orow + d0 * 2) = o;
            }
        }
    if (p.lse != nullptr && lh == 0) p.lse[((int64_t)(b * p.heads) + h) * p.seqlen + q_row] = lse;
#endif  // __HIP_DEVICE_COMPILE__
}

}  // namespace intfa
