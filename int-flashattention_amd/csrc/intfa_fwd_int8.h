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

template <int D> struct SmemInt8 {
    char k[2][kBlockN * D];
    char v[2][kBlockN * D * 2];     // sized for 16-bit V; the int8 variant uses the first half of each
    float ks[2][kBlockN];
};

// One workgroup = one (batch, head, 128-query block[, split]).
template <int VARIANT, int D, bool CAUSAL, int OUT_DT /*0 f16, 1 bf16*/, int PROUND, bool DUMP_S, bool SPLIT>
__global__ void __launch_bounds__(kThreads, 2) fwd_int8_kernel(const KParams p) {
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

    const auto k_lane = tile_load_lane<D, false>((uint32_t)p.k_sn, wave, lane);
    const auto v_lane = tile_load_lane<VROW, true>((uint32_t)p.v_sn, wave, lane);
    auto issue_loads = [&](int nb, char* dK, char* dV) {
        issue_tile_load<D, false>(Kg + (int64_t)nb * kBlockN * p.k_sn, (uint32_t)p.k_sn, dK, wave, k_lane);
        if (!DUMP_S) issue_tile_load<VROW, true>(Vg + (int64_t)nb * kBlockN * p.v_sn, (uint32_t)p.v_sn, dV, wave, v_lane);
    };
    const uint32_t ks_lane = (uint32_t)tid * (uint32_t)p.ks_sn;
    auto load_ks = [&](int nb) -> float {
        if (DUMP_S || tid >= kBlockN) return 0.f;
        const int64_t base = ks_base + (int64_t)nb * kBlockN * p.ks_sn;     // wave-uniform
        if (p.scale_dtype == 0) return (float)((const _Float16*)Ksg + base)[ks_lane];
        if (p.scale_dtype == 1) return __builtin_bit_cast(float, ((uint32_t)((const uint16_t*)Ksg + base)[ks_lane]) << 16);
        return ((const float*)Ksg + base)[ks_lane];
    };

    auto compute = [&](int nb, const char* cK, const char* cV, const float* cKs) {
        const bool diag = CAUSAL && (nb == mb);
        // -------- pass 1: S^T sub-tiles, dequantise by k_scale, running row max
        float t[4][16];
        float mx = -INFINITY;
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            if (CAUSAL && diag && st > wave) {               // sub-tile entirely above the diagonal
#pragma unroll
                for (int r = 0; r < 16; ++r) t[st][r] = -INFINITY;
                continue;
            }
            v16i acc = {0};
            const char* krow = cK + (32 * st + lq) * D;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const v4i a = *(const v4i*)(krow + (((2 * ks + lh) ^ k_swz) << 4));
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
                    if (CAUSAL && diag && st == wave) {
                        const int key = 8 * a4 + 4 * lh + b4;       // position inside the 32x32 diagonal tile
                        if (key > lq) x = -INFINITY;
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
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                v16i acc = {0};
#pragma unroll
                for (int st = 0; st < 4; ++st) {
                    if (CAUSAL && diag && st > wave) continue;
                    const int c = 2 * dt + (g16 & 1);
                    const int r0 = 32 * st + v_row0, r1 = r0 + 16;
                    const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                        (__attribute__((address_space(3))) v2i*)INTFA_LDS(cV + r0 * VROW + ((c ^ swz_v<VROW>(r0)) << 4) + v_sub));
                    const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                        (__attribute__((address_space(3))) v2i*)INTFA_LDS(cV + r1 * VROW + ((c ^ swz_v<VROW>(r1)) << 4) + v_sub));
                    const v4i a = {lo[0], lo[1], hi[0], hi[1]};
                    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, p8[st], acc, 0, 0, 0);
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) o_acc[dt][r] = fmaf(o_acc[dt][r], alpha, (float)acc[r]);
            }
        }
        l_run = fmaf(l_run, alpha, lsum);
    };

    // ---- main loop: K/V tiles double-buffered in LDS, one barrier per key block
    if (nb_begin < nb_end) {
        issue_loads(nb_begin, sK0, sV0);
        {
            const float s0 = load_ks(nb_begin);
            if (tid < kBlockN) sKs0[tid] = s0;
        }
        for (int nb = nb_begin; nb < nb_end; nb += 2) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            float ks_next = 0.f;
            if (nb + 1 < nb_end) { issue_loads(nb + 1, sK1, sV1); ks_next = load_ks(nb + 1); }
            compute(nb, sK0, sV0, sKs0);
            if (nb + 1 < nb_end) {
                if (tid < kBlockN) sKs1[tid] = ks_next;
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                if (nb + 2 < nb_end) { issue_loads(nb + 2, sK0, sV0); ks_next = load_ks(nb + 2); }
                compute(nb + 1, sK1, sV1, sKs1);
                if (nb + 2 < nb_end && tid < kBlockN) sKs0[tid] = ks_next;
            }
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
}

}  // namespace intfa
