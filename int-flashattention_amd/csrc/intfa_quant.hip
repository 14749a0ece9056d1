// Symmetric int8 quantisers of the attention inputs (benchmark.py:96-107) as HBM-bound streaming kernels.
//
// Arithmetic follows the reference's torch expressions evaluated in the input's 16-bit type, operation by
// operation (each torch op on fp16/bf16 computes in fp32 and rounds the result to the 16-bit type):
//     scale = absmax / 127                      -> fp32 division, rounded to the 16-bit type
//     q     = round(x / scale).to(int8)         -> fp32 division rounded to the 16-bit type, round-half-even,
//                                                  integer conversion truncated to 8 bits
// Layout: x is [B, H, N, d] with arbitrary batch/head/row strides and contiguous d; q8 is written contiguous; a lane
// owns 8 consecutive elements (one 16-byte load, one 8-byte store) and d / 8 lanes share a row.
#include "../../include/intfa.h"
#include "intfa_device.h"
#include "intfa_launch.h"

using namespace intfa;

namespace {

template <int DT> __device__ __forceinline__ float to_f32(uint16_t bits) {
    if (DT == 0) return (float)__builtin_bit_cast(_Float16, bits);
    return __builtin_bit_cast(float, (uint32_t)bits << 16);
}
template <int DT> __device__ __forceinline__ uint16_t from_f32(float f) {      // round-to-nearest-even
    if (DT == 0) return __builtin_bit_cast(uint16_t, (_Float16)f);
    return (uint16_t)f32_to_bf16_bits(f);
}
// |x| of a 16-bit float as an unsigned integer: monotonic in |x| for finite values, so max works on the bits
__device__ __forceinline__ uint32_t abs_bits(uint16_t b) { return b & 0x7fffu; }

// A row's divisor is fixed, so the correctly rounded quotient x / scale is formed from the correctly rounded reciprocal
// (one IEEE division per lane and row) with one multiply and two fused multiply-adds per element:
//     q0 = RN(x * r),  e = x - q0 * scale (exact in one fma),  q = RN(q0 + e * r) = RN(x / scale)
// (Markstein's correction step; it needs r = RN(1 / scale), which the IEEE division delivers, and a divisor whose
// significand is not all ones, which a 16-bit scale cannot be).
struct RowDivisor { float scale, recip; };
__device__ __forceinline__ RowDivisor make_divisor(float scale) { return {scale, 1.0f / scale}; }

// Round-half-even of four quotients |q| < 128.5 to int8, packed into one word.  Adding 1.5 * 2^23 rounds to an integer
// in the adder (one unit in the last place of that binade is 1) and leaves the two's-complement byte in the low byte of
// the bit pattern; two byte permutes and an OR gather the four low bytes.  A NaN (0 / 0: a row or column of zeros has
// scale 0) keeps a zero low byte, so such elements quantise to 0 without a test per element.
constexpr float kRoundMagic = 12582912.0f;      // 1.5 * 2^23
__device__ __forceinline__ uint32_t pack4_rne(float q0, float q1, float q2, float q3) {
    const uint32_t b0 = __builtin_bit_cast(uint32_t, q0 + kRoundMagic), b1 = __builtin_bit_cast(uint32_t, q1 + kRoundMagic);
    const uint32_t b2 = __builtin_bit_cast(uint32_t, q2 + kRoundMagic), b3 = __builtin_bit_cast(uint32_t, q3 + kRoundMagic);
    // v_perm_b32: selector bytes 0-3 pick from the second operand, 4-7 from the first, 0x0c yields zero
    return __builtin_amdgcn_perm(b1, b0, 0x0c0c0400u) | __builtin_amdgcn_perm(b3, b2, 0x04000c0cu);
}

// x / scale rounded to the 16-bit type (both operands are values of that type), as a float
template <int DT> __device__ __forceinline__ float quotient16(uint16_t xb, RowDivisor d) {
    const float x = to_f32<DT>(xb);
    const float q0 = x * d.recip;
    const float e = __builtin_fmaf(-q0, d.scale, x);
    const float q = __builtin_fmaf(e, d.recip, q0);
    return to_f32<DT>(from_f32<DT>(q));
}

template <int DT> __device__ __forceinline__ void quant_store8(const v4i raw, RowDivisor scale, char* dst) {
    int out[2];
#pragma unroll
    for (int w = 0; w < 2; ++w) {
        float q[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t word = (uint32_t)raw[2 * w + j / 2];
            q[j] = quotient16<DT>((uint16_t)(j & 1 ? word >> 16 : word & 0xffffu), scale);
        }
        out[w] = (int)pack4_rne(q[0], q[1], q[2], q[3]);
    }
    *(v2i*)dst = (v2i){out[0], out[1]};
}

__device__ __forceinline__ uint32_t amax8(const v4i raw) {
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t w = (uint32_t)raw[i];
        const uint32_t a = abs_bits((uint16_t)(w & 0xffffu)), b = abs_bits((uint16_t)(w >> 16));
        m = m > a ? m : a;
        m = m > b ? m : b;
    }
    return m;
}

struct QuantParams {
    const char* x; char* q8; char* scale; uint32_t* amax;
    int64_t sb, sh, sn;             // bytes
    int32_t heads, seqlen, head_dim;
    int64_t rows;                   // batch * heads * seqlen
    FastDiv d_seqlen, d_heads;      // row index -> (batch, head, position) without a run-time division per row
};

// ---- per token: LPR = d / 8 lanes per row, reduction of the row maximum inside those lanes
constexpr int kRowsInFlight = 8;    // independent 16-byte loads a lane has in flight (HBM latency x bandwidth needs several)

// rows are numbered (batch, head, position) in that order; the count fits 31 bits (checked on the host), so the index
// arithmetic is 32-bit
__device__ __forceinline__ const char* row_ptr(const QuantParams& p, uint32_t row, int sub, uint32_t* bh_out) {
    const uint32_t bh = (uint32_t)fast_div((int)row, p.d_seqlen), n = row - bh * (uint32_t)p.seqlen;
    const uint32_t b = (uint32_t)fast_div((int)bh, p.d_heads), h = bh - b * (uint32_t)p.heads;
    *bh_out = bh;
    return p.x + b * p.sb + h * p.sh + n * p.sn + sub * 16;
}

template <int DT, int LPR> __global__ void __launch_bounds__(256) quant_pertoken_kernel(const QuantParams p) {
    constexpr int RPB = 256 / LPR;                       // rows per workgroup step
    const int sub = threadIdx.x % LPR, rl = threadIdx.x / LPR;
    const uint32_t step = gridDim.x * RPB, rows = (uint32_t)p.rows;
    for (uint32_t row0 = blockIdx.x * RPB + rl; row0 < rows; row0 += step * kRowsInFlight) {
        v4i raw[kRowsInFlight];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            const uint32_t row = row0 + u * step;
            uint32_t bh;
            raw[u] = row < rows ? *(const v4i*)row_ptr(p, row, sub, &bh) : (v4i){0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            const uint32_t row = row0 + u * step;
            uint32_t m = amax8(raw[u]);
#pragma unroll
            for (int off = LPR / 2; off > 0; off >>= 1) {
                const uint32_t o = (uint32_t)__shfl_xor((int)m, off, 64);
                m = m > o ? m : o;
            }
            if (row >= rows) continue;
            const uint16_t sbits = from_f32<DT>(to_f32<DT>((uint16_t)m) / 127.0f);
            if (sub == 0) ((uint16_t*)p.scale)[row] = sbits;
            quant_store8<DT>(raw[u], make_divisor(to_f32<DT>(sbits)), p.q8 + (int64_t)row * p.head_dim + sub * 8);
        }
    }
}

// ---- per (batch, head): maximum over the whole [N, d] slice in two launches
__global__ void quant_clear_kernel(uint32_t* amax, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) amax[i] = 0u;
}

template <int LPR> __global__ void __launch_bounds__(256) quant_slice_amax_kernel(const QuantParams p, int chunks) {
    constexpr int RPB = 256 / LPR;
    const int sub = threadIdx.x % LPR, rl = threadIdx.x / LPR;
    const int bh = blockIdx.x / chunks, chunk = blockIdx.x % chunks;
    const int64_t h = bh % p.heads, b = bh / p.heads;
    const char* base = p.x + b * p.sb + h * p.sh + sub * 16;
    uint32_t m = 0;
    const int nstep = chunks * RPB;
    for (int n0 = chunk * RPB + rl; n0 < p.seqlen; n0 += nstep * kRowsInFlight) {
        v4i raw[kRowsInFlight];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            const int n = n0 + u * nstep;
            raw[u] = n < p.seqlen ? *(const v4i*)(base + (int64_t)n * p.sn) : (v4i){0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            const uint32_t r = amax8(raw[u]);
            m = m > r ? m : r;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t o = (uint32_t)__shfl_xor((int)m, off, 64);
        m = m > o ? m : o;
    }
    if ((threadIdx.x & 63) == 0) atomicMax(p.amax + bh, m);
}

template <int DT, int LPR> __global__ void __launch_bounds__(256) quant_slice_apply_kernel(const QuantParams p) {
    constexpr int RPB = 256 / LPR;
    const int sub = threadIdx.x % LPR, rl = threadIdx.x / LPR;
    const uint32_t step = gridDim.x * RPB, rows = (uint32_t)p.rows;
    for (uint32_t row0 = blockIdx.x * RPB + rl; row0 < rows; row0 += step * kRowsInFlight) {
        v4i raw[kRowsInFlight];
        uint32_t bh[kRowsInFlight];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            const uint32_t row = row0 + u * step;
            bh[u] = 0;
            raw[u] = row < rows ? *(const v4i*)row_ptr(p, row, sub, &bh[u]) : (v4i){0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            const uint32_t row = row0 + u * step;
            if (row >= rows) continue;
            const uint16_t sbits = from_f32<DT>(to_f32<DT>((uint16_t)p.amax[bh[u]]) / 127.0f);
            if (row == bh[u] * (uint32_t)p.seqlen && sub == 0) ((uint16_t*)p.scale)[bh[u]] = sbits;
            quant_store8<DT>(raw[u], make_divisor(to_f32<DT>(sbits)), p.q8 + (int64_t)row * p.head_dim + sub * 8);
        }
    }
}

// ---- per (batch, head, block of rows, channel): fp32 scales, the layout of the V scales of the reference's CUDA
// kernel (csrc/flash_fwd_kernel_full_qi8.h:156-160).  One workgroup owns one block of rows: column maxima through LDS
// atomics, then a second sweep over the block (served by the cache) that divides and rounds in fp32.
template <int DT, int LPR> __global__ void __launch_bounds__(256) quant_blockchan_kernel(const QuantParams p, int block, int nblk,
                                                                                         float* scale_out) {
    constexpr int RPB = 256 / LPR;
    __shared__ uint32_t smax[LPR * 8];
    const int sub = threadIdx.x % LPR, rl = threadIdx.x / LPR;
    const int bh = blockIdx.x / nblk, blk = blockIdx.x % nblk;
    const int64_t h = bh % p.heads, b = bh / p.heads;
    const int n_lo = blk * block, n_hi = n_lo + block < p.seqlen ? n_lo + block : p.seqlen;
    const char* base = p.x + b * p.sb + h * p.sh + sub * 16;
    for (int i = threadIdx.x; i < LPR * 8; i += 256) smax[i] = 0u;
    __syncthreads();
    uint32_t m[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int n0 = n_lo + rl; n0 < n_hi; n0 += RPB * kRowsInFlight) {
        v4i raw[kRowsInFlight];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            const int n = n0 + u * RPB;
            raw[u] = n < n_hi ? *(const v4i*)(base + (int64_t)n * p.sn) : (v4i){0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t w = (uint32_t)raw[u][j / 2];
                const uint32_t a = abs_bits((uint16_t)(j & 1 ? w >> 16 : w & 0xffffu));
                m[j] = m[j] > a ? m[j] : a;
            }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) atomicMax(&smax[sub * 8 + j], m[j]);
    __syncthreads();
    float sc[8], rc[8];
    bool plain_division = false;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        sc[j] = to_f32<DT>((uint16_t)smax[sub * 8 + j]) / 127.0f;
        rc[j] = 1.0f / sc[j];
        // the reciprocal-based quotient below is correctly rounded unless the divisor's significand is all ones
        plain_division |= (__builtin_bit_cast(uint32_t, sc[j]) & 0x7fffffu) == 0x7fffffu;
    }
    if (rl == 0) {
        float* dst = scale_out + ((int64_t)bh * nblk + blk) * p.head_dim + sub * 8;
        *(v4f*)dst = (v4f){sc[0], sc[1], sc[2], sc[3]};
        *(v4f*)(dst + 4) = (v4f){sc[4], sc[5], sc[6], sc[7]};
    }
    char* qbase = p.q8 + (int64_t)bh * p.seqlen * p.head_dim + sub * 8;
    for (int n0 = n_lo + rl; n0 < n_hi; n0 += RPB * kRowsInFlight) {
        v4i raw[kRowsInFlight];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            const int n = n0 + u * RPB;
            raw[u] = n < n_hi ? *(const v4i*)(base + (int64_t)n * p.sn) : (v4i){0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            const int n = n0 + u * RPB;
            if (n >= n_hi) continue;
            int out[2];
#pragma unroll
            for (int w2 = 0; w2 < 2; ++w2) {
                float q[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t word = (uint32_t)raw[u][2 * w2 + j / 2];
                    const float x = to_f32<DT>((uint16_t)(j & 1 ? word >> 16 : word & 0xffffu));
                    const float s = sc[4 * w2 + j], r = rc[4 * w2 + j];
                    // RN(x / s) as in quotient16 (0 / 0 = NaN -> 0 below); IEEE division for the exceptional divisor
                    const float q0 = x * r;
                    const float e = __builtin_fmaf(-q0, s, x);
                    q[j] = plain_division ? x / s : __builtin_fmaf(e, r, q0);
                }
                out[w2] = (int)pack4_rne(q[0], q[1], q[2], q[3]);
            }
            *(v2i*)(qbase + (int64_t)n * p.head_dim) = (v2i){out[0], out[1]};
        }
    }
}

int check(const void* x, const void* q8, const void* scale, int64_t sb, int64_t sh, int64_t sn, int batch, int heads,
          int seqlen, int head_dim, int dtype, QuantParams* qp) {
    if (x == nullptr || q8 == nullptr || scale == nullptr) return INTFA_ERR_NULL;
    if (batch <= 0 || heads <= 0 || seqlen <= 0) return INTFA_ERR_SHAPE;
    if (head_dim != 16 && head_dim != 32 && head_dim != 64 && head_dim != 128 && head_dim != 256) return INTFA_ERR_HEAD_DIM;
    if (dtype != INTFA_F16 && dtype != INTFA_BF16) return INTFA_ERR_DTYPE;
    if ((reinterpret_cast<uintptr_t>(x) & 15u) || (reinterpret_cast<uintptr_t>(q8) & 7u) || (reinterpret_cast<uintptr_t>(scale) & 1u))
        return INTFA_ERR_ALIGN;
    if ((sb * 2) % 16 || (sh * 2) % 16 || (sn * 2) % 16) return INTFA_ERR_ALIGN;
    if (sn < head_dim) return INTFA_ERR_SHAPE;                       // rows must not overlap (as the forward entry points require)
    qp->x = (const char*)x; qp->q8 = (char*)q8; qp->scale = (char*)scale; qp->amax = nullptr;
    qp->sb = sb * 2; qp->sh = sh * 2; qp->sn = sn * 2;
    qp->heads = heads; qp->seqlen = seqlen; qp->head_dim = head_dim;
    qp->rows = (int64_t)batch * heads * seqlen;
    if (qp->rows >= (1ll << 31) - (1 << 24)) return INTFA_ERR_SHAPE;      // 32-bit row indices, with room for the strides
    qp->d_seqlen = make_fast_div(seqlen);
    qp->d_heads = make_fast_div(heads);
    return INTFA_OK;
}

int grid_for(int64_t rows, int rows_per_block) {
    const int64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
    const int64_t cap = 256 * 8;                         // every CU full (8 workgroups of 256 threads), grid-stride beyond
    return (int)(blocks < cap ? blocks : cap);
}

// ---- append to an int8 K/V cache: one row of new keys or values per LPR lanes, written at the row's position in the
// cache.  IS_V: the scale is the cache's (given), the quotient saturates; else the row's own scale, stored beside it.
struct AppendSide {
    const char* x; char* cache; char* scale;      // scale: k_scale_cache (written) or v_scale (read)
    int64_t xb, xh, xn;                           // bytes
    int64_t cb, ch, cn;                           // bytes (int8 elements)
    int64_t sb, sh, sn;                           // scale strides, elements (sn unused for V)
};
struct AppendParams {
    AppendSide k, v;
    const int32_t* seqlens_k;
    int32_t seqlen_filled, heads, seqlen_new, seqlen_cache, head_dim;
    int64_t rows;                                 // batch * heads * seqlen_new
    FastDiv d_seqlen_new, d_heads;
};

template <int DT, int LPR, bool IS_V> __global__ void __launch_bounds__(256) kv_append_kernel(const AppendParams p) {
    constexpr int RPB = 256 / LPR;
    constexpr int U = 4;                          // rows a lane has in flight
    const AppendSide& s = IS_V ? p.v : p.k;
    const int sub = threadIdx.x % LPR, rl = threadIdx.x / LPR;
    const uint32_t step = gridDim.x * RPB, rows = (uint32_t)p.rows;
    // (the lanes of a row share rl, so they enter and leave the loop together and the shuffles below see all of them)
    for (uint32_t row0 = blockIdx.x * RPB + rl; row0 < rows; row0 += step * U) {
        v4i raw[U];
        uint32_t bq[U], hq[U], iq[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t row = row0 + u * step;
            const uint32_t bh = (uint32_t)fast_div((int)row, p.d_seqlen_new);
            iq[u] = row - bh * (uint32_t)p.seqlen_new;
            bq[u] = (uint32_t)fast_div((int)bh, p.d_heads); hq[u] = bh - bq[u] * (uint32_t)p.heads;
            raw[u] = row < rows ? *(const v4i*)(s.x + bq[u] * s.xb + hq[u] * s.xh + iq[u] * s.xn + sub * 16) : (v4i){0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t row = row0 + u * step;
            const uint32_t b = bq[u], h = hq[u];
            uint16_t sbits = 0;
            if (IS_V) {
                if (row < rows) sbits = ((const uint16_t*)s.scale)[b * s.sb + h * s.sh];
            } else {
                uint32_t m = amax8(raw[u]);
#pragma unroll
                for (int off = LPR / 2; off > 0; off >>= 1) {
                    const uint32_t o = (uint32_t)__shfl_xor((int)m, off, 64);
                    m = m > o ? m : o;
                }
                sbits = from_f32<DT>(to_f32<DT>((uint16_t)m) / 127.0f);
            }
            if (row >= rows) continue;
            int len = p.seqlen_filled;
            if (p.seqlens_k != nullptr) {
                const int n = p.seqlens_k[b];
                len = n < 0 ? 0 : (n < p.seqlen_cache ? n : p.seqlen_cache);
            }
            const int64_t pos = (int64_t)len + iq[u];
            if (pos >= p.seqlen_cache) continue;                               // no room: the row is dropped
            char* dst = s.cache + b * s.cb + h * s.ch + pos * s.cn + sub * 8;
            const RowDivisor d = make_divisor(to_f32<DT>(sbits));
            if (IS_V) {
                int out[2];
#pragma unroll
                for (int w = 0; w < 2; ++w) {
                    float q[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t word = (uint32_t)raw[u][2 * w + j / 2];
                        const float t = quotient16<DT>((uint16_t)(j & 1 ? word >> 16 : word & 0xffffu), d);
                        q[j] = t != t ? t : __builtin_fminf(__builtin_fmaxf(t, -127.0f), 127.0f);  // (NaN from 0 / 0 stays NaN: byte 0)
                    }
                    out[w] = (int)pack4_rne(q[0], q[1], q[2], q[3]);
                }
                *(v2i*)dst = (v2i){out[0], out[1]};
            } else {
                if (sub == 0) ((uint16_t*)s.scale)[b * s.sb + h * s.sh + pos * s.sn] = sbits;
                quant_store8<DT>(raw[u], d, dst);
            }
        }
    }
}

}  // namespace

#define INTFA_LPR_SWITCH(d, CALL)            \
    switch (d) {                             \
        case 16: CALL(2); break;             \
        case 32: CALL(4); break;             \
        case 64: CALL(8); break;             \
        case 128: CALL(16); break;           \
        default: CALL(32); break;            \
    }

extern "C" {

int intfa_quant_pertoken(const void* x, int64_t stride_b, int64_t stride_h, int64_t stride_n, void* q8, void* scale,
                         int32_t batch, int32_t heads, int32_t seqlen, int32_t head_dim, int32_t dtype, void* stream) {
    QuantParams qp;
    const int rc = check(x, q8, scale, stride_b, stride_h, stride_n, batch, heads, seqlen, head_dim, dtype, &qp);
    if (rc != INTFA_OK) return rc;
    hipStream_t st = (hipStream_t)stream;
#define INTFA_CALL(LPR) do { const int g = grid_for(qp.rows, 256 / LPR); \
        if (dtype == INTFA_F16) hipLaunchKernelGGL((quant_pertoken_kernel<0, LPR>), dim3(g), dim3(256), 0, st, qp); \
        else hipLaunchKernelGGL((quant_pertoken_kernel<1, LPR>), dim3(g), dim3(256), 0, st, qp); } while (0)
    INTFA_LPR_SWITCH(head_dim, INTFA_CALL)
#undef INTFA_CALL
    return (int)hipGetLastError();
}

size_t intfa_quant_pertensor_workspace_bytes(int32_t batch, int32_t heads) {
    return (batch > 0 && heads > 0) ? (size_t)batch * heads * sizeof(uint32_t) : 0;
}

int intfa_quant_pertensor(const void* x, int64_t stride_b, int64_t stride_h, int64_t stride_n, void* q8, void* scale,
                          int32_t batch, int32_t heads, int32_t seqlen, int32_t head_dim, int32_t dtype,
                          void* workspace, size_t workspace_bytes, void* stream) {
    QuantParams qp;
    const int rc = check(x, q8, scale, stride_b, stride_h, stride_n, batch, heads, seqlen, head_dim, dtype, &qp);
    if (rc != INTFA_OK) return rc;
    if (workspace == nullptr || workspace_bytes < intfa_quant_pertensor_workspace_bytes(batch, heads) ||
        (reinterpret_cast<uintptr_t>(workspace) & 3u)) return INTFA_ERR_WORKSPACE;
    qp.amax = (uint32_t*)workspace;
    hipStream_t st = (hipStream_t)stream;
    const int slices = batch * heads;
    hipLaunchKernelGGL(quant_clear_kernel, dim3((slices + 255) / 256), dim3(256), 0, st, qp.amax, slices);
#define INTFA_CALL(LPR) do { \
        const int rpb = 256 / LPR; \
        int chunks = (seqlen + rpb - 1) / rpb; \
        const int want = (256 * 8 + slices - 1) / slices;          /* about 8 workgroups per CU over all slices */ \
        if (chunks > want) chunks = want; \
        hipLaunchKernelGGL((quant_slice_amax_kernel<LPR>), dim3(slices * chunks), dim3(256), 0, st, qp, chunks); \
        const int g = grid_for(qp.rows, rpb); \
        if (dtype == INTFA_F16) hipLaunchKernelGGL((quant_slice_apply_kernel<0, LPR>), dim3(g), dim3(256), 0, st, qp); \
        else hipLaunchKernelGGL((quant_slice_apply_kernel<1, LPR>), dim3(g), dim3(256), 0, st, qp); } while (0)
    INTFA_LPR_SWITCH(head_dim, INTFA_CALL)
#undef INTFA_CALL
    return (int)hipGetLastError();
}

int intfa_quant_perblock_channel(const void* x, int64_t stride_b, int64_t stride_h, int64_t stride_n, void* q8, float* scale,
                                 int32_t batch, int32_t heads, int32_t seqlen, int32_t head_dim, int32_t block,
                                 int32_t dtype, void* stream) {
    QuantParams qp;
    const int rc = check(x, q8, scale, stride_b, stride_h, stride_n, batch, heads, seqlen, head_dim, dtype, &qp);
    if (rc != INTFA_OK) return rc;
    if (block <= 0) return INTFA_ERR_VSCALE;
    if (reinterpret_cast<uintptr_t>(scale) & 15u) return INTFA_ERR_ALIGN;
    const int nblk = (seqlen + block - 1) / block;
    const int64_t grid = (int64_t)batch * heads * nblk;
    if (grid >= (1ll << 31)) return INTFA_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
#define INTFA_CALL(LPR) do { \
        if (dtype == INTFA_F16) hipLaunchKernelGGL((quant_blockchan_kernel<0, LPR>), dim3((int)grid), dim3(256), 0, st, qp, block, nblk, scale); \
        else hipLaunchKernelGGL((quant_blockchan_kernel<1, LPR>), dim3((int)grid), dim3(256), 0, st, qp, block, nblk, scale); } while (0)
    INTFA_LPR_SWITCH(head_dim, INTFA_CALL)
#undef INTFA_CALL
    return (int)hipGetLastError();
}

int intfa_kvcache_append_int8(const intfa_append_params* a, void* stream) {
    if (a == nullptr || a->k_new == nullptr || a->k_cache == nullptr || a->k_scale_cache == nullptr) return INTFA_ERR_NULL;
    const bool with_v = a->v_new != nullptr;
    if (with_v && (a->v_cache == nullptr || a->v_scale == nullptr)) return INTFA_ERR_NULL;
    if (a->batch <= 0 || a->heads_kv <= 0) return INTFA_ERR_SHAPE;
    if (a->seqlen_new <= 0 || a->seqlen_cache <= 0 ||
        (a->seqlens_k == nullptr && (a->seqlen_filled < 0 || a->seqlen_filled > a->seqlen_cache))) return INTFA_ERR_SEQLEN;
    const int d = a->head_dim;
    if (d != 16 && d != 32 && d != 64 && d != 128 && d != 256) return INTFA_ERR_HEAD_DIM;
    if (a->dtype != INTFA_F16 && a->dtype != INTFA_BF16) return INTFA_ERR_DTYPE;
    const int64_t rows = (int64_t)a->batch * a->heads_kv * a->seqlen_new;
    if (rows >= (1ll << 31) - (1 << 24)) return INTFA_ERR_SHAPE;
    // 16-byte loads of the 16-bit rows (strides in elements: multiples of 8), 8-byte stores of the int8 rows
    auto misaligned = [](const void* ptr, int64_t s0, int64_t s1, int64_t s2, unsigned bytes) {
        return (reinterpret_cast<uintptr_t>(ptr) & (bytes - 1u)) != 0 || s0 % 8 || s1 % 8 || s2 % 8;
    };
    if (misaligned(a->k_new, a->kn_stride_b, a->kn_stride_h, a->kn_stride_n, 16) ||
        misaligned(a->k_cache, a->kc_stride_b, a->kc_stride_h, a->kc_stride_n, 8)) return INTFA_ERR_ALIGN;
    if (with_v && (misaligned(a->v_new, a->vn_stride_b, a->vn_stride_h, a->vn_stride_n, 16) ||
                   misaligned(a->v_cache, a->vc_stride_b, a->vc_stride_h, a->vc_stride_n, 8))) return INTFA_ERR_ALIGN;
    if ((reinterpret_cast<uintptr_t>(a->k_scale_cache) & 1u) || (with_v && (reinterpret_cast<uintptr_t>(a->v_scale) & 1u)) ||
        (a->seqlens_k != nullptr && (reinterpret_cast<uintptr_t>(a->seqlens_k) & 3u))) return INTFA_ERR_ALIGN;
    if (a->kn_stride_n < d || a->kc_stride_n < d || (with_v && (a->vn_stride_n < d || a->vc_stride_n < d))) return INTFA_ERR_SHAPE;
    AppendParams ap;
    ap.k = {(const char*)a->k_new, (char*)a->k_cache, (char*)a->k_scale_cache, a->kn_stride_b * 2, a->kn_stride_h * 2,
            a->kn_stride_n * 2, a->kc_stride_b, a->kc_stride_h, a->kc_stride_n, a->ksc_stride_b, a->ksc_stride_h, a->ksc_stride_n};
    ap.v = {(const char*)a->v_new, (char*)a->v_cache, (char*)const_cast<void*>(a->v_scale), a->vn_stride_b * 2, a->vn_stride_h * 2,
            a->vn_stride_n * 2, a->vc_stride_b, a->vc_stride_h, a->vc_stride_n, a->vs_stride_b, a->vs_stride_h, 0};
    ap.seqlens_k = a->seqlens_k;
    ap.seqlen_filled = a->seqlen_filled;
    ap.heads = a->heads_kv; ap.seqlen_new = a->seqlen_new; ap.seqlen_cache = a->seqlen_cache; ap.head_dim = d;
    ap.d_seqlen_new = make_fast_div(a->seqlen_new);
    ap.d_heads = make_fast_div(a->heads_kv);
    ap.rows = rows;
    hipStream_t st = (hipStream_t)stream;
#define INTFA_CALL(LPR) do { const int g = grid_for(rows, 256 / LPR); \
        if (a->dtype == INTFA_F16) { \
            hipLaunchKernelGGL((kv_append_kernel<0, LPR, false>), dim3(g), dim3(256), 0, st, ap); \
            if (with_v) hipLaunchKernelGGL((kv_append_kernel<0, LPR, true>), dim3(g), dim3(256), 0, st, ap); \
        } else { \
            hipLaunchKernelGGL((kv_append_kernel<1, LPR, false>), dim3(g), dim3(256), 0, st, ap); \
            if (with_v) hipLaunchKernelGGL((kv_append_kernel<1, LPR, true>), dim3(g), dim3(256), 0, st, ap); \
        } } while (0)
    INTFA_LPR_SWITCH(d, INTFA_CALL)
#undef INTFA_CALL
    return (int)hipGetLastError();
}

}  // extern "C"
