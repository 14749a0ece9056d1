// C ABI of libintfa.so: argument validation, kernel selection and launch.  See include/intfa.h.
#include "../../include/intfa.h"
#include "intfa_device.h"
#include "intfa_launch.h"
#include "intfa_splitkv.h"

#include <atomic>

using namespace intfa;

// Scratch of intfa_fwd_full_int8_static (the split-KV partials of a call that may not allocate): part of the device
// code, so every GPU the library runs on holds its own copy at its own address until the process ends.  In host code
// the array's name is only a handle for hipGetSymbolAddress, never an address to hand to a kernel.
static __device__ __align__(256) unsigned char scratch[INTFA_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];          // device address of `scratch` per GPU, nullptr until looked up

// Address of the scratch array on the current device; looked up once per device (any thread may be the one).
int static_scratch_ptr(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return INTFA_ERR_SCRATCH;
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (ptr == nullptr) return (int)hipErrorInvalidSymbol;
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);     // every thread finds the same address
    }
    *out = ptr;
    return INTFA_OK;
}

constexpr int kMaxSplits = 64;

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Key-block length of a variant at a head_dim.  Full-int8: 128 keys at head_dim 128, 64 at head_dim 64 (the reference
// admits no key block longer than head_dim: tl.static_assert(BLOCK_N <= HEAD_DIM), flash_atten_full_int8.py:88) and at
// head_dim 256 (registers and LDS); the kernels with a 16-bit P V take 64.
int block_n_for(int variant, int head_dim) {
    if (variant == INTFA_VARIANT_FULL_INT8) return head_dim == 128 ? 128 : 64;
    return 64;
}

// Common validation; fills the kernel-side block.  elem sizes in bytes for q/k, v and out.
int make_kparams(const intfa_fwd_params* p, int qk_bytes, int v_bytes, bool need_scales, bool need_vscale, KParams* kp) {
    if (p == nullptr || p->q == nullptr || p->k == nullptr) return INTFA_ERR_NULL;
    if (p->batch <= 0 || p->heads <= 0) return INTFA_ERR_SHAPE;
    const int heads_kv = p->heads_kv > 0 ? p->heads_kv : p->heads;
    if (heads_kv > p->heads || p->heads % heads_kv != 0) return INTFA_ERR_SHAPE;
    if (p->seqlen <= 0 || p->seqlen_k < 0) return INTFA_ERR_SEQLEN;
    const int seqlen_k = p->seqlen_k > 0 ? p->seqlen_k : p->seqlen;
    if (p->head_dim != 64 && p->head_dim != 128 && p->head_dim != 256) return INTFA_ERR_HEAD_DIM;
    if (p->scale_dtype < 0 || p->scale_dtype > 2) return INTFA_ERR_DTYPE;
    if (p->io_dtype != INTFA_F16 && p->io_dtype != INTFA_BF16) return INTFA_ERR_DTYPE;
    const int64_t n_blocks = (int64_t)p->batch * p->heads * ((p->seqlen + kBlockM - 1) / kBlockM);
    if (n_blocks * kMaxSplits >= (1ll << 31)) return INTFA_ERR_SHAPE;
    // K and V slices are addressed through 32-bit buffer offsets: one (batch, head) slice must span less than 4 GiB
    if ((int64_t)(seqlen_k - 1) * p->k_stride_n * qk_bytes + (int64_t)p->head_dim * qk_bytes >= (1ll << 32)) return INTFA_ERR_SHAPE;
    if (v_bytes > 0 && (int64_t)(seqlen_k - 1) * p->v_stride_n * v_bytes + (int64_t)p->head_dim * v_bytes >= (1ll << 32)) return INTFA_ERR_SHAPE;
    if (!aligned16(p->q) || !aligned16(p->k)) return INTFA_ERR_ALIGN;
    if ((p->q_stride_n * qk_bytes) % 16 || (p->k_stride_n * qk_bytes) % 16) return INTFA_ERR_ALIGN;
    if ((p->q_stride_b * qk_bytes) % 16 || (p->q_stride_h * qk_bytes) % 16) return INTFA_ERR_ALIGN;
    if ((p->k_stride_b * qk_bytes) % 16 || (p->k_stride_h * qk_bytes) % 16) return INTFA_ERR_ALIGN;
    if (p->k_stride_n < p->head_dim || p->q_stride_n < p->head_dim) return INTFA_ERR_SHAPE;
    KParams k{};
    k.q = (const char*)p->q; k.k = (const char*)p->k;
    k.q_sb = p->q_stride_b * qk_bytes; k.q_sh = p->q_stride_h * qk_bytes; k.q_sn = p->q_stride_n * qk_bytes;
    k.k_sb = p->k_stride_b * qk_bytes; k.k_sh = p->k_stride_h * qk_bytes; k.k_sn = p->k_stride_n * qk_bytes;
    if (v_bytes > 0) {
        if (p->v == nullptr || p->out == nullptr) return INTFA_ERR_NULL;
        if (!aligned16(p->v) || !aligned16(p->out)) return INTFA_ERR_ALIGN;     // (the output rows are stored 16 bytes per lane)
        if ((p->v_stride_n * v_bytes) % 16 || (p->v_stride_b * v_bytes) % 16 || (p->v_stride_h * v_bytes) % 16) return INTFA_ERR_ALIGN;
        if ((p->o_stride_n * 2) % 16 || (p->o_stride_b * 2) % 16 || (p->o_stride_h * 2) % 16) return INTFA_ERR_ALIGN;
        if (p->v_stride_n < p->head_dim || p->o_stride_n < p->head_dim) return INTFA_ERR_SHAPE;
        k.v = (const char*)p->v; k.out = (char*)p->out;
        k.v_sb = p->v_stride_b * v_bytes; k.v_sh = p->v_stride_h * v_bytes; k.v_sn = p->v_stride_n * v_bytes;
        k.o_sb = p->o_stride_b * 2; k.o_sh = p->o_stride_h * 2; k.o_sn = p->o_stride_n * 2;
    }
    if (need_scales) {
        if (p->q_scale == nullptr || p->k_scale == nullptr) return INTFA_ERR_NULL;
        k.q_scale = (const char*)p->q_scale; k.k_scale = (const char*)p->k_scale;
        k.qs_sb = p->qs_stride_b; k.qs_sh = p->qs_stride_h; k.qs_sn = p->qs_stride_n;
        k.ks_sb = p->ks_stride_b; k.ks_sh = p->ks_stride_h; k.ks_sn = p->ks_stride_n;
    }
    if (need_vscale) {
        if (p->v_scale == nullptr) return INTFA_ERR_NULL;
        k.v_scale = (const char*)p->v_scale; k.vs_sb = p->vs_stride_b; k.vs_sh = p->vs_stride_h;
        if (p->v_scale_block < 0) return INTFA_ERR_VSCALE;
        if (p->v_scale_block > 0) {
            const int bn = block_n_for(INTFA_VARIANT_FULL_INT8, p->head_dim);
            // a multiple of the key block, or 64 where the key block is 128: the granularity of the reference's CUDA kernel
            // (kBlockN = 64, csrc/flash_fwd_launch_template.h:514-519), two scale rows per key block
            const bool half_block = bn == 128 && p->v_scale_block == 64;
            if ((p->v_scale_block % bn != 0 && !half_block) || p->vs_stride_blk < p->head_dim) return INTFA_ERR_VSCALE;
            if (reinterpret_cast<uintptr_t>(p->v_scale) & 3u) return INTFA_ERR_ALIGN;
            k.vs_g = half_block ? 1 : p->v_scale_block / bn;
            k.vs_sub = half_block ? 2 : 1;
            k.vs_sblk = p->vs_stride_blk;
        }
    }
    k.lse = p->lse;
    if (p->seqlens_k != nullptr) {
        if (reinterpret_cast<uintptr_t>(p->seqlens_k) & 3u) return INTFA_ERR_ALIGN;
        k.seqlens_k = p->seqlens_k;
    }
    k.batch = p->batch; k.heads = p->heads; k.seqlen = p->seqlen; k.seqlen_k = seqlen_k; k.head_dim = p->head_dim;
    k.scale_dtype = p->scale_dtype; k.causal = p->causal ? 1 : 0;
    k.kv_group = p->heads / heads_kv;
    k.num_splits = 1; k.blocks_per_split = p->seqlen;   // single pass: never the limit
    k.qk_scale_log2 = p->sm_scale * 1.44269504f;      // flash_atten_full_int8.py:156-157
    *kp = k;
    return INTFA_OK;
}

size_t workspace_bytes_for(const intfa_fwd_params* p) {
    if (p == nullptr || p->num_splits <= 1) return 0;
    const size_t rows = (size_t)p->num_splits * p->batch * p->heads * p->seqlen;
    return rows * (size_t)p->head_dim * sizeof(float) + rows * sizeof(float);
}

int setup_split(const intfa_fwd_params* p, int block_n, KParams* kp) {
    if (p->num_splits <= 1) return INTFA_OK;
    if (p->num_splits > kMaxSplits) return INTFA_ERR_SPLITS;
    const size_t need = workspace_bytes_for(p);
    if (p->workspace == nullptr || p->workspace_bytes < need || !aligned16(p->workspace)) return INTFA_ERR_WORKSPACE;
    const int n_blocks = ((p->seqlen_k > 0 ? p->seqlen_k : p->seqlen) + block_n - 1) / block_n;
    kp->num_splits = p->num_splits;
    kp->blocks_per_split = (n_blocks + p->num_splits - 1) / p->num_splits;     // csrc/flash_fwd_kernel.h:503
    const size_t rows = (size_t)p->num_splits * p->batch * p->heads * p->seqlen;
    kp->o_part = (float*)p->workspace;
    kp->lse_part = kp->o_part + rows * (size_t)p->head_dim;
    return INTFA_OK;
}

int launch_combine(const intfa_fwd_params* p, const KParams& kp, hipStream_t stream) {
    const int64_t rows = (int64_t)kp.batch * kp.heads * kp.seqlen;
    const int rpb = 256 / (kp.head_dim / 4);      // head_dim / 4 lanes per output row
    const int grid = (int)((rows + rpb - 1) / rpb);
#define INTFA_COMBINE(DD, ODT) hipLaunchKernelGGL((splitkv_combine_kernel<DD, ODT>), dim3(grid), dim3(256), 0, stream, kp)
    if (kp.head_dim == 64) { if (p->io_dtype == INTFA_F16) INTFA_COMBINE(64, 0); else INTFA_COMBINE(64, 1); }
    else if (kp.head_dim == 128) { if (p->io_dtype == INTFA_F16) INTFA_COMBINE(128, 0); else INTFA_COMBINE(128, 1); }
    else { if (p->io_dtype == INTFA_F16) INTFA_COMBINE(256, 0); else INTFA_COMBINE(256, 1); }
#undef INTFA_COMBINE
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? INTFA_OK : (int)e;
}

// Few query rows per head (decoding against a cache): the pass runs a kernel whose waves share the keys of a block
// instead of each taking 32 query rows (intfa_fwd_decode.h, intfa_fwd_decode_f16pv.h).
constexpr int kDecodeMaxRows = 2 * kDecodeRows;
bool decode_shaped(int seqlen) { return seqlen <= kDecodeMaxRows; }

int dispatch(int variant, const intfa_fwd_params* p, const KParams& kp, bool dump_s, hipStream_t stream) {
    const bool vblk = variant == INTFA_VARIANT_FULL_INT8 && !dump_s && kp.vs_g > 0;
    LaunchSel sel;
    sel.causal = kp.causal != 0;
    sel.io_dt = p->io_dtype == INTFA_BF16 ? 1 : 0;
    sel.p_round = p->p_round == INTFA_PROUND_REFERENCE ? 1 : 0;
    sel.split = kp.num_splits > 1;
    sel.dump_s = dump_s;
    const int d = kp.head_dim;
    if (vblk && kp.vs_sub == 2) {              // (also for few query rows: the decode kernel has one scale row per block)
        if (d == 128) return launch_full_int8_vblk64_d128(kp, sel, stream);
    } else if (!dump_s && decode_shaped(kp.seqlen)) {
        if (variant == INTFA_VARIANT_FULL_INT8) {
            if (d == 64) return launch_decode_full_int8_d64(kp, sel, stream);
            if (d == 128) return launch_decode_full_int8_d128(kp, sel, stream);
            if (d == 256) return launch_decode_full_int8_d256(kp, sel, stream);
        } else if (variant == INTFA_VARIANT_HALF_INT8) {
            if (d == 64) return launch_decode_half_int8_d64(kp, sel, stream);
            if (d == 128) return launch_decode_half_int8_d128(kp, sel, stream);
            if (d == 256) return launch_decode_half_int8_d256(kp, sel, stream);
        } else {
            if (d == 64) return launch_decode_fp16_d64(kp, sel, stream);
            if (d == 128) return launch_decode_fp16_d128(kp, sel, stream);
            if (d == 256) return launch_decode_fp16_d256(kp, sel, stream);
        }
    } else if (vblk) {
        if (d == 64) return launch_full_int8_vblk_d64(kp, sel, stream);
        if (d == 128) return launch_full_int8_vblk_d128(kp, sel, stream);
        if (d == 256) return launch_full_int8_vblk_d256(kp, sel, stream);
    } else if (variant == INTFA_VARIANT_FULL_INT8) {
        if (d == 64) return launch_full_int8_d64(kp, sel, stream);
        if (d == 128) return launch_full_int8_d128(kp, sel, stream);
        if (d == 256) return launch_full_int8_d256(kp, sel, stream);
    } else if (variant == INTFA_VARIANT_HALF_INT8) {
        if (d == 64) return launch_half_int8_d64(kp, sel, stream);
        if (d == 128) return launch_half_int8_d128(kp, sel, stream);
        if (d == 256) return launch_half_int8_d256(kp, sel, stream);
    } else {
        if (d == 64) return launch_fp16_d64(kp, sel, stream);
        if (d == 128) return launch_fp16_d128(kp, sel, stream);
        if (d == 256) return launch_fp16_d256(kp, sel, stream);
    }
    return INTFA_ERR_HEAD_DIM;
}

int run_forward(int variant, const intfa_fwd_params* p, int qk_bytes, int v_bytes, bool scales, bool vscale, hipStream_t stream) {
    KParams kp;
    int rc = make_kparams(p, qk_bytes, v_bytes, scales, vscale, &kp);
    if (rc != INTFA_OK) return rc;
    if (variant == INTFA_VARIANT_FULL_INT8 && p->p_round != INTFA_PROUND_RNE && p->p_round != INTFA_PROUND_REFERENCE) return INTFA_ERR_DTYPE;
    if (p->causal_rows != 0) {
        if (p->causal_rows < 0 || !p->causal || !decode_shaped(kp.seqlen) ||
            kp.seqlen % p->causal_rows != 0 || kp.vs_sub == 2) return INTFA_ERR_SEQLEN;
        kp.causal_rows = p->causal_rows;
    }
    rc = setup_split(p, block_n_for(variant, kp.head_dim), &kp);
    if (rc != INTFA_OK) return rc;
    kp.pair_mblocks = (kp.causal && kp.num_splits <= 1 && ((kp.seqlen + kBlockM - 1) / kBlockM) % 2 == 0) ? 1 : 0;
    rc = dispatch(variant, p, kp, false, stream);
    if (rc != INTFA_OK || kp.num_splits <= 1) return rc;
    return launch_combine(p, kp, stream);
}

}  // namespace

extern "C" {

int intfa_version(void) { return INTFA_VERSION; }

int intfa_fwd_block_n(int variant, int head_dim) {
    if (variant < INTFA_VARIANT_FULL_INT8 || variant > INTFA_VARIANT_FP16) return INTFA_ERR_DTYPE;
    if (head_dim != 64 && head_dim != 128 && head_dim != 256) return INTFA_ERR_HEAD_DIM;
    return block_n_for(variant, head_dim);
}

const char* intfa_error_string(int code) {
    switch (code) {
        case INTFA_OK: return "ok";
        case INTFA_ERR_NULL: return "a required pointer is NULL";
        case INTFA_ERR_HEAD_DIM: return "head_dim must be 64, 128 or 256";
        case INTFA_ERR_SEQLEN: return "seqlen must be positive, seqlen_k not negative, causal_rows only on causal decode-shaped calls";
        case INTFA_ERR_ALIGN: return "pointers and row/head/batch strides must be 16-byte aligned";
        case INTFA_ERR_DTYPE: return "unknown dtype enum";
        case INTFA_ERR_WORKSPACE: return "workspace missing, misaligned or too small for num_splits";
        case INTFA_ERR_SHAPE: return "batch and heads must be positive and the grid must fit 31 bits";
        case INTFA_ERR_SPLITS: return "num_splits must be at most 64";
        case INTFA_ERR_VSCALE: return "v_scale_block must be a multiple of the key-block length (or 64 at head_dim 128) and vs_stride_blk at least head_dim";
        case INTFA_ERR_SCRATCH: return "the split-KV partials of this call exceed INTFA_STATIC_SCRATCH_BYTES (or the device index exceeds 63)";
        default: return code > 0 ? "hip error" : "unknown error";
    }
}

size_t intfa_fwd_workspace_bytes(const intfa_fwd_params* p) { return workspace_bytes_for(p); }

int intfa_fwd_suggest_splits(const intfa_fwd_params* p, int variant, int num_cus) {
    if (p == nullptr) return INTFA_ERR_NULL;
    if (variant < INTFA_VARIANT_FULL_INT8 || variant > INTFA_VARIANT_FP16) return INTFA_ERR_DTYPE;
    if (p->batch <= 0 || p->heads <= 0) return INTFA_ERR_SHAPE;
    if (p->seqlen <= 0 || p->seqlen_k < 0) return INTFA_ERR_SEQLEN;
    if (p->head_dim != 64 && p->head_dim != 128 && p->head_dim != 256) return INTFA_ERR_HEAD_DIM;
    const int cus = num_cus > 0 ? num_cus : 256;
    int64_t slots = 2ll * cus;                                                 // two workgroups per compute unit
    int64_t wgs = (int64_t)p->batch * p->heads * ((p->seqlen + kBlockM - 1) / kBlockM);
    if (decode_shaped(p->seqlen)) {
        wgs = (int64_t)p->batch * p->heads * ((p->seqlen + kDecodeRows - 1) / kDecodeRows);
        // head_dim 256: 96 KiB and more of tiles, one workgroup per compute unit
        if (p->head_dim == 256) slots = cus;
    }
    else if (p->head_dim == 256) wgs *= 2;     // full-int8: eight-wave workgroups, one per compute unit; the others: column halves
    if (wgs * 5 >= slots * 4) return 1;                                        // at least 80 % of the slots are used anyway
    const int seqlen_k = p->seqlen_k > 0 ? p->seqlen_k : p->seqlen;
    const int bn = block_n_for(variant, p->head_dim);
    const int64_t blocks = (seqlen_k + bn - 1) / bn;
    int64_t splits = (slots + wgs - 1) / wgs;
    if (splits > blocks / 4) splits = blocks / 4;                              // keep four key blocks per split
    if (splits > kMaxSplits) splits = kMaxSplits;
    return splits < 1 ? 1 : (int)splits;
}

int intfa_fwd_full_int8(const intfa_fwd_params* p, void* stream) {
    return run_forward(INTFA_VARIANT_FULL_INT8, p, 1, 1, true, true, (hipStream_t)stream);
}

int intfa_fwd_full_int8_static(const intfa_fwd_params* p, void* stream) {
    if (p == nullptr) return INTFA_ERR_NULL;
    intfa_fwd_params q = *p;
    q.workspace = nullptr;
    q.workspace_bytes = 0;
    if (p->num_splits > 1) {
        if (p->num_splits > kMaxSplits) return INTFA_ERR_SPLITS;
        if (p->batch <= 0 || p->heads <= 0 || p->seqlen <= 0 || p->head_dim <= 0) return INTFA_ERR_SHAPE;
        if (workspace_bytes_for(p) > INTFA_STATIC_SCRATCH_BYTES) return INTFA_ERR_SCRATCH;
        void* ptr = nullptr;
        const int rc = static_scratch_ptr(&ptr);
        if (rc != INTFA_OK) return rc;
        // every (split, row) of the partials is written by the forward pass before the combine pass reads it, so
        // nothing of the previous call's contents has to be cleared
        q.workspace = ptr;
        q.workspace_bytes = INTFA_STATIC_SCRATCH_BYTES;
    }
    return run_forward(INTFA_VARIANT_FULL_INT8, &q, 1, 1, true, true, (hipStream_t)stream);
}

int intfa_fwd_half_int8(const intfa_fwd_params* p, void* stream) {
    return run_forward(INTFA_VARIANT_HALF_INT8, p, 1, 2, true, false, (hipStream_t)stream);
}

int intfa_fwd_fp16(const intfa_fwd_params* p, void* stream) {
    return run_forward(INTFA_VARIANT_FP16, p, 2, 2, false, false, (hipStream_t)stream);
}

int intfa_debug_qk_int32(const intfa_fwd_params* p, int32_t* s_out, void* stream) {
    KParams kp;
    if (s_out == nullptr) return INTFA_ERR_NULL;
    int rc = make_kparams(p, 1, 0, false, false, &kp);
    if (rc != INTFA_OK) return rc;
    kp.s_dump = s_out;
    kp.causal = 0;
    kp.scale_dtype = INTFA_F32;
    return dispatch(INTFA_VARIANT_FULL_INT8, p, kp, true, (hipStream_t)stream);
}

}  // extern "C"
