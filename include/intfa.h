/*
 * intfa.h - C ABI of the MI355X (gfx950) INT8 FlashAttention forward library (libintfa.so).
 *
 * The reference ships no host API for this path: its Python entry points launch Triton kernels
 * directly (flash_atten_full_int8.py:186-221, flash_atten_int8.py:181-215, flash_atten_fp.py:155-187)
 * and its CUDA sources stop at the templates
 *     run_mha_fwd_full_qi8_<T,128>(Flash_fwd_params&, cudaStream_t)      (csrc/flash.h:205-208)
 * which take one parameter block plus a stream.  The entry points below keep that shape - one plain-C
 * parameter block (the counterpart of Qkv_params / Flash_fwd_params, csrc/flash.h:24-159) and a stream -
 * with the tensor conventions of the Python entry points ([Z,H,N,d] tensors, [Z,H,N] per-token scales,
 * [Z,H] value scale).
 *
 * Conventions of every entry point:
 *   - all pointers are DEVICE pointers borrowed for the duration of the enqueued work;
 *   - strides are in ELEMENTS of the tensor they describe; the head dimension is contiguous (stride 1);
 *   - work is enqueued on `stream` (a hipStream_t passed as void*, NULL = the null stream); the call does not
 *     synchronise, allocate or free;
 *   - return value: 0 on success, a negative INTFA_ERR_* for a rejected argument, a positive hipError_t when
 *     the launch itself failed;
 *   - re-entrant and thread-safe for distinct streams: no mutable global state, with ONE exception -
 *     intfa_fwd_full_int8_static keeps a per-device table of its scratch array's address and all its calls on one
 *     GPU share that array (see its declaration).
 */
#ifndef INTFA_H_
#define INTFA_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define INTFA_VERSION 8

/* forward variants (one entry point each, below) */
enum { INTFA_VARIANT_FULL_INT8 = 0, INTFA_VARIANT_HALF_INT8 = 1, INTFA_VARIANT_FP16 = 2 };

/* element types of scales / float tensors */
enum { INTFA_F16 = 0, INTFA_BF16 = 1, INTFA_F32 = 2 };

/* rounding used when P is requantised to int8 (full-int8 path) */
enum {
    /* the reference's fp16 sequence: fp16(p) * 127, + 0.5, truncating cast (flash_atten_full_int8.py:49-51); the
       default: what a zero-initialised parameter block selects */
    INTFA_PROUND_REFERENCE = 0,
    /* opt-in: 127*p evaluated in fp32 and rounded to nearest-even by one hardware convert */
    INTFA_PROUND_RNE = 1
};

enum {
    INTFA_OK = 0,
    INTFA_ERR_NULL = -1,          /* a required pointer is NULL */
    INTFA_ERR_HEAD_DIM = -2,      /* head_dim not supported by the kernels */
    INTFA_ERR_SEQLEN = -3,        /* seqlen not positive, seqlen_k negative, or causal_rows on a call it does not apply to */
    INTFA_ERR_ALIGN = -4,         /* pointer or row stride not 16-byte aligned */
    INTFA_ERR_DTYPE = -5,         /* unknown dtype enum */
    INTFA_ERR_WORKSPACE = -6,     /* workspace missing or too small for the requested split count */
    INTFA_ERR_SHAPE = -7,         /* batch/heads not positive, a row stride below head_dim, a (batch, head) slice of
                                     k or v spanning 4 GiB or more, or sizes that overflow 32-bit block indices */
    INTFA_ERR_SPLITS = -8,        /* num_splits out of range */
    INTFA_ERR_VSCALE = -9,        /* v_scale_block neither a multiple of the key-block length nor 64 at head_dim 128, or
                                     vs_stride_blk below head_dim */
    INTFA_ERR_SCRATCH = -10       /* intfa_fwd_full_int8_static: the call's split-KV partials exceed
                                     INTFA_STATIC_SCRATCH_BYTES, or the device index is beyond the table of 64 devices */
};

/*
 * Parameter block shared by the three forward variants.  Unused members of a variant are ignored
 * (q_scale/k_scale for the fp16 variant, v_scale for the half-int8 and fp16 variants).  k, v and their scales have
 * heads_kv heads when that member is set.
 *
 *   variant      q, k            v               out
 *   full-int8    int8            int8            out_dtype (fp16 as in the reference, or bf16)
 *   half-int8    int8            fp16 or bf16    out_dtype (= v's type)
 *   fp16         fp16 or bf16    same as q       same as q
 */
typedef struct intfa_fwd_params {
    const void* q;            /* [batch, heads, seqlen, head_dim] */
    const void* k;
    const void* v;
    void*       out;
    const void* q_scale;      /* [batch, heads, seqlen], scale_dtype */
    const void* k_scale;      /* [batch, heads, seqlen], scale_dtype */
    const void* v_scale;      /* [batch, heads], scale_dtype; with v_scale_block set:
                                 [batch, heads, ceil(seqlen_k / v_scale_block), head_dim], always fp32 */
    float*      lse;          /* optional [batch, heads, seqlen] contiguous: m + log2(l), base-2 as the
                                 reference's M (flash_atten_int8.py:172-175); NULL = not written */

    int64_t q_stride_b, q_stride_h, q_stride_n;
    int64_t k_stride_b, k_stride_h, k_stride_n;
    int64_t v_stride_b, v_stride_h, v_stride_n;
    int64_t o_stride_b, o_stride_h, o_stride_n;
    int64_t qs_stride_b, qs_stride_h, qs_stride_n;
    int64_t ks_stride_b, ks_stride_h, ks_stride_n;
    int64_t vs_stride_b, vs_stride_h;

    int32_t batch, heads, seqlen, head_dim;
    int32_t scale_dtype;      /* INTFA_F16 / INTFA_BF16 / INTFA_F32 */
    int32_t io_dtype;         /* type of out (and of fp q/k/v): INTFA_F16 or INTFA_BF16 */
    int32_t causal;           /* 0 / 1.  Query row i sees keys 0 .. i + (seqlen_k - seqlen): with equal lengths the reference's
                                 mask (flash_atten_full_int8.py:39-43); with more keys than queries (a chunk of new tokens
                                 against a cache) the mask is aligned to the bottom right corner as in the reference's CUDA
                                 tree (csrc/mask.h:53,172).  A row that sees no key (fewer keys than queries) gives zeros. */
    float   sm_scale;
    int32_t p_round;          /* INTFA_PROUND_* (full-int8 only) */

    int32_t num_splits;       /* <= 1: single pass; > 1: split-KV partials + combine (needs workspace).  The key blocks
                                 are dealt evenly to the splits (ceil(blocks / num_splits) consecutive blocks each).  With
                                 causal the general kernels deal, per query block of 128 rows, the blocks VISIBLE to that
                                 query block (ceil(visible / num_splits) each, so no split of a query block is empty);
                                 decode-shaped calls (seqlen <= 64; every variant and head_dim, except full-int8 at
                                 head_dim 128 with v_scale_block = 64, which runs the general kernel) keep the partition
                                 of the whole key sequence also with causal: split s takes blocks s * ceil(blocks /
                                 num_splits) onward, cut at the last visible block.  The requantisation frame of P depends
                                 on the ranges, so a bit-faithful CPU evaluation must use the same ones. */
    void*   workspace;        /* device scratch of at least intfa_fwd_workspace_bytes() bytes, or NULL */
    size_t  workspace_bytes;

    int32_t heads_kv;         /* grouped-query / multi-query attention: number of K/V heads; k, v, k_scale and v_scale
                                 then have heads_kv heads and query head h reads K/V head h / (heads / heads_kv).
                                 0 or heads = one K/V head per query head (the reference's Python API; its CUDA tree
                                 has the grouped form, csrc/flash_fwd_kernel_full_qi8.h:141).  Must divide heads. */
    int32_t seqlen_k;         /* number of keys when it differs from the number of queries (cross attention, decoding
                                 against a cache): k, v and k_scale then have seqlen_k rows.  0 = seqlen. */
    int32_t v_scale_block;    /* full-int8 only.  0: one V scale per (batch, head), the reference's Python API
                                 (flash_atten_full_int8.py:159-161).  > 0: V was quantised per block of v_scale_block keys
                                 and per channel, the layout its CUDA kernel reads (csrc/flash_fwd_kernel_full_qi8.h:
                                 156-160, applied per key block at csrc/mask.h:313-340); v_scale then has one row of
                                 head_dim fp32 scales per block of keys (channel stride 1, row stride vs_stride_blk, batch
                                 and head strides vs_stride_b / vs_stride_h over heads_kv heads; 4-byte aligned, fp32 as in
                                 that kernel whatever scale_dtype says).  Must be a multiple of
                                 intfa_fwd_block_n(INTFA_VARIANT_FULL_INT8, head_dim) (64, except 128 at head_dim 128),
                                 or 64 at head_dim 128: the granularity of the reference's kernel itself (kBlockN = 64 at
                                 head_dim 128, csrc/flash_fwd_launch_template.h:514-519).  At head_dim 128 the softmax
                                 then still advances per 128-key block (running maximum and P8 as intfa_fwd_block_n()
                                 says); P V is summed in int32 per 64-key half and each half is multiplied by its own
                                 scale row. */
    int32_t reserved0;        /* set to 0 */
    int64_t vs_stride_blk;    /* elements between consecutive scale rows of v_scale (>= head_dim) */
    const int32_t* seqlens_k; /* optional device array [batch]: number of keys of each batch entry, 0 <= n <= seqlen_k (a
                                 key/value cache filled to different lengths; the counterpart of the reference's
                                 seqused_k and of cu_seqlens_k used as lengths, csrc/flash.h:95-99,149-151,
                                 csrc/block_info.h:21-22).  k, v and k_scale keep their seqlen_k-row layout; rows past a
                                 batch entry's length are not read.  An entry with no key gives zeros (lse = -inf).
                                 NULL = every entry has seqlen_k keys.  With causal the mask of an entry is aligned to
                                 its own length. */
    int32_t causal_rows;      /* 0, or the number of query positions when the row axis holds several query heads of one
                                 K/V group one after the other (decoding with grouped heads described as heads = heads_kv,
                                 seqlen = group * positions, see heads_kv): row r is position r % causal_rows for the causal
                                 mask.  Only with causal and the shapes of the decode kernels: seqlen <= 64, any variant
                                 and head_dim (not with v_scale_block = 64 at head_dim 128).  seqlen must be a multiple
                                 of it. */
    int32_t reserved1;        /* set to 0 */
} intfa_fwd_params;

/* Library/ABI version (INTFA_VERSION of the build). */
int intfa_version(void);

/* Human-readable text for a negative return code; for a positive one returns "hip error". */
const char* intfa_error_string(int code);

/* Key-block length of a variant at a head_dim (the reference's BLOCK_N, an autotuned value there:
 * configs.py:13-19).  The running max and, on the full-int8 path, the requantisation of P advance per key block,
 * so a bit-faithful CPU evaluation must use the same value.  Full-int8: 128 at head_dim 128, 64 otherwise; half-int8 and
 * fp16: 64.  At head_dim >= 64 that is a length the reference's kernel admits (flash_atten_full_int8.py:88,
 * static_assert BLOCK_N <= HEAD_DIM); head_dim 16 and 32 are computed zero-padded to 64 and keep the 64-key block.  It holds for every shape: the kernel
 * that takes over decode-shaped calls (at most 64 query rows) walks the same blocks.
 * Negative INTFA_ERR_* for unknown arguments. */
int intfa_fwd_block_n(int variant, int head_dim);

/* A split count for the problem in *p (its num_splits and workspace members are ignored): 1 when the single-pass grid
 * already fills the GPU, otherwise enough splits to reach about two workgroups per compute unit while leaving every split
 * at least four key blocks; the counterpart of the heuristic that lives in the reference's absent flash_api.cpp
 * (csrc/flash_fwd_launch_template.h:193-253 only consumes it).  variant: INTFA_VARIANT_*; num_cus: compute units of
 * the device, 0 = 256 (MI355X).  Negative INTFA_ERR_* for a rejected block. */
int intfa_fwd_suggest_splits(const intfa_fwd_params* p, int variant, int num_cus);

/* Bytes of workspace the forward needs for p->num_splits (0 when num_splits <= 1). */
size_t intfa_fwd_workspace_bytes(const intfa_fwd_params* p);

/* attention_full_int8(q, k, v, q_scale, k_scale, v_scale, causal, sm_scale) -> o
 * replaces _attention_full_int8.forward + _attn_fwd_full_int8 (flash_atten_full_int8.py:73-221);
 * native counterpart run_mha_fwd_full_qi8_ (csrc/flash_fwd_launch_template.h:503-523). */
int intfa_fwd_full_int8(const intfa_fwd_params* p, void* stream);

/* intfa_fwd_full_int8 for callers that cannot allocate device memory - code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc - and so cannot provide the workspace of a split-KV call.  It has no
 * counterpart in the reference.  Same parameter block and results as intfa_fwd_full_int8 (bit for bit), but
 * p->workspace and p->workspace_bytes are ignored: the split-KV partials go to a scratch array that is part of the
 * library's device code (INTFA_STATIC_SCRATCH_BYTES bytes on each GPU the library runs on, held until the process
 * ends).  The call works on the CURRENT device (stream must belong to it) and allocates, frees and synchronises
 * nothing; the first call on a device looks the array's address up (make that call outside a graph capture).
 * A call whose partials need more than INTFA_STATIC_SCRATCH_BYTES (intfa_fwd_workspace_bytes says how much) is
 * rejected with INTFA_ERR_SCRATCH.  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU
 * (different streams, or threads) race on it; calls on one stream are ordered and safe.  With num_splits <= 1 it is
 * intfa_fwd_full_int8. */
#define INTFA_STATIC_SCRATCH_BYTES (32u << 20)
int intfa_fwd_full_int8_static(const intfa_fwd_params* p, void* stream);

/* attention_int8(q, k, v, q_scale, k_scale, causal, sm_scale) -> o
 * replaces _attention_int8.forward + _attn_fwd_int8 (flash_atten_int8.py:68-215);
 * native counterpart run_mha_fwd_half_qi8_ (csrc/flash_fwd_launch_template.h:469-501). */
int intfa_fwd_half_int8(const intfa_fwd_params* p, void* stream);

/* attention(q, k, v, causal, sm_scale) -> o
 * replaces _attention.forward + _attn_fwd (flash_atten_fp.py:62-187);
 * native counterpart run_mha_fwd_<T,128> (csrc/flash.h:205). */
int intfa_fwd_fp16(const intfa_fwd_params* p, void* stream);

/* Debug export of the int32 accumulators S = Q8 K8^T produced by the same MFMA tile code the forward
 * uses (flash_atten_full_int8.py:36).  s_out is [batch, heads, seqlen, seqlen_k] int32, contiguous.  Uses q, k and
 * their strides, batch, heads, heads_kv, seqlen, seqlen_k and head_dim of the block. */
int intfa_debug_qk_int32(const intfa_fwd_params* p, int32_t* s_out, void* stream);

/* quant_pertoken(X) -> (int8 X, scale) of the reference's harness (benchmark.py:96-100): per row of head_dim
 * elements, scale = absmax / 127 and q = round(x / scale), every step evaluated in x's 16-bit type as torch does.
 * x: [batch, heads, seqlen, head_dim] fp16 or bf16 (dtype = INTFA_F16 / INTFA_BF16), strides in elements, head_dim
 * contiguous and one of 16, 32, 64, 128, 256; q8: int8, written contiguous; scale: [batch, heads, seqlen] in x's
 * type, contiguous. */
int intfa_quant_pertoken(const void* x, int64_t stride_b, int64_t stride_h, int64_t stride_n, void* q8, void* scale,
                         int32_t batch, int32_t heads, int32_t seqlen, int32_t head_dim, int32_t dtype, void* stream);

/* quant_pertensor(X) -> (int8 X, scale) (benchmark.py:102-107): one scale per (batch, head) slice; scale is
 * [batch, heads] in x's type.  Needs intfa_quant_pertensor_workspace_bytes() bytes of device scratch (4-byte
 * aligned) for the per-slice maxima. */
size_t intfa_quant_pertensor_workspace_bytes(int32_t batch, int32_t heads);
int intfa_quant_pertensor(const void* x, int64_t stride_b, int64_t stride_h, int64_t stride_n, void* q8, void* scale,
                          int32_t batch, int32_t heads, int32_t seqlen, int32_t head_dim, int32_t dtype,
                          void* workspace, size_t workspace_bytes, void* stream);

/* Quantiser for the blocked V scales of intfa_fwd_params.v_scale_block: one fp32 scale per (batch, head, block of
 * `block` rows, channel), scale = absmax / 127 over the block's rows and q = round-half-even(x / scale), both in fp32
 * (the harness's formula, benchmark.py:102-107, at the granularity of the V scales its CUDA kernel reads,
 * csrc/flash_fwd_kernel_full_qi8.h:156-160; the reference itself holds no quantiser for that layout).  A channel that
 * is zero throughout a block gets scale 0 and zeros.  x as for intfa_quant_pertoken; q8 int8 contiguous; scale fp32
 * [batch, heads, ceil(seqlen / block), head_dim] contiguous, 16-byte aligned. */
int intfa_quant_perblock_channel(const void* x, int64_t stride_b, int64_t stride_h, int64_t stride_n, void* q8, float* scale,
                                 int32_t batch, int32_t heads, int32_t seqlen, int32_t head_dim, int32_t block,
                                 int32_t dtype, void* stream);

/* Appends new keys (and values) to an int8 K/V cache: the counterpart, for the quantised cache this library reads, of
 * the copy the reference's cache kernel makes of knew/vnew before it attends (csrc/flash_fwd_kernel.h:690-790,
 * Append_KV; csrc/flash.h:104-112; rotary embedding and paged caches are not part of this build).  For batch entry b the
 * rows go to positions len_b .. len_b + seqlen_new - 1 of the cache, len_b = seqlens_k[b] (device memory, clamped to
 * [0, seqlen_cache]) or seqlen_filled when seqlens_k is NULL; rows that would land at or past seqlen_cache are dropped.
 * The lengths themselves are the caller's to advance (a forward call with seqlens_k = len + seqlen_new then sees them).
 *   K: quantised per token exactly as intfa_quant_pertoken does (scale = absmax / 127 in k_new's type, stored into
 *      k_scale_cache at the row's position);
 *   V: quantised with the cache's existing scale v_scale[b, h] (V has one scale per (batch, head), which an append
 *      cannot change): q = round-half-even(v / scale) in v_new's type, saturated to [-127, 127].  v_new = NULL: K only.
 * k_new, v_new: [batch, heads_kv, seqlen_new, head_dim] fp16 or bf16 (dtype), head_dim contiguous, strides in elements;
 * k_cache, v_cache: int8 [batch, heads_kv, seqlen_cache, head_dim], head_dim contiguous, row strides multiples of 8;
 * k_scale_cache: [batch, heads_kv, seqlen_cache] and v_scale: [batch, heads_kv], both in k_new's type. */
typedef struct intfa_append_params {
    const void* k_new; const void* v_new;
    int64_t kn_stride_b, kn_stride_h, kn_stride_n;
    int64_t vn_stride_b, vn_stride_h, vn_stride_n;
    void* k_cache; void* v_cache;
    int64_t kc_stride_b, kc_stride_h, kc_stride_n;
    int64_t vc_stride_b, vc_stride_h, vc_stride_n;
    void* k_scale_cache;
    int64_t ksc_stride_b, ksc_stride_h, ksc_stride_n;
    const void* v_scale;
    int64_t vs_stride_b, vs_stride_h;
    const int32_t* seqlens_k;
    int32_t seqlen_filled;
    int32_t batch, heads_kv, seqlen_new, seqlen_cache, head_dim, dtype;
} intfa_append_params;
int intfa_kvcache_append_int8(const intfa_append_params* p, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* INTFA_H_ */
