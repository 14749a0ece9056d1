// C ABI of libintfa.so: argument validation, kernel selection and launch.  See include/intfa.h.
#include "../../include/intfa.h"
#include "intfa_device.h"
#include "intfa_fwd_int8.h"
#include "intfa_fwd_fp16.h"
#include "intfa_splitkv.h"

using namespace intfa;

namespace {

constexpr int kMaxSplits = 64;

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int scale_size(int dt) { return dt == INTFA_F32 ? 4 : 2; }

// Common validation; fills the kernel-side block.  elem sizes in bytes for q/k, v and out.
int make_kparams(const intfa_fwd_params* p, int qk_bytes, int v_bytes, bool need_scales, bool need_vscale, KParams* kp) {
    if (p == nullptr || p->q == nullptr || p->k == nullptr) return INTFA_ERR_NULL;
    if (p->batch <= 0 || p->heads <= 0) return INTFA_ERR_SHAPE;
    if (p->seqlen <= 0 || p->seqlen % kBlockN != 0) return INTFA_ERR_SEQLEN;
    if (p->head_dim != 64 && p->head_dim != 128 && p->head_dim != 256) return INTFA_ERR_HEAD_DIM;
    if (p->scale_dtype < 0 || p->scale_dtype > 2) return INTFA_ERR_DTYPE;
    if (p->io_dtype != INTFA_F16 && p->io_dtype != INTFA_BF16) return INTFA_ERR_DTYPE;
    const int64_t n_blocks = (int64_t)p->batch * p->heads * (p->seqlen / kBlockM);
    if (n_blocks * kMaxSplits >= (1ll << 31)) return INTFA_ERR_SHAPE;
    if (!aligned16(p->q) || !aligned16(p->k)) return INTFA_ERR_ALIGN;
    if ((p->q_stride_n * qk_bytes) % 16 || (p->k_stride_n * qk_bytes) % 16) return INTFA_ERR_ALIGN;
    if ((p->q_stride_b * qk_bytes) % 16 || (p->q_stride_h * qk_bytes) % 16) return INTFA_ERR_ALIGN;
    if ((p->k_stride_b * qk_bytes) % 16 || (p->k_stride_h * qk_bytes) % 16) return INTFA_ERR_ALIGN;
    KParams k{};
    k.q = (const char*)p->q; k.k = (const char*)p->k;
    k.q_sb = p->q_stride_b * qk_bytes; k.q_sh = p->q_stride_h * qk_bytes; k.q_sn = p->q_stride_n * qk_bytes;
    k.k_sb = p->k_stride_b * qk_bytes; k.k_sh = p->k_stride_h * qk_bytes; k.k_sn = p->k_stride_n * qk_bytes;
    if (v_bytes > 0) {
        if (p->v == nullptr || p->out == nullptr) return INTFA_ERR_NULL;
        if (!aligned16(p->v) || (reinterpret_cast<uintptr_t>(p->out) & 7u)) return INTFA_ERR_ALIGN;
        if ((p->v_stride_n * v_bytes) % 16 || (p->v_stride_b * v_bytes) % 16 || (p->v_stride_h * v_bytes) % 16) return INTFA_ERR_ALIGN;
        if ((p->o_stride_n * 2) % 8 || (p->o_stride_b * 2) % 8 || (p->o_stride_h * 2) % 8) return INTFA_ERR_ALIGN;
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
    }
    k.lse = p->lse;
    k.batch = p->batch; k.heads = p->heads; k.seqlen = p->seqlen; k.head_dim = p->head_dim;
    k.scale_dtype = p->scale_dtype; k.causal = p->causal ? 1 : 0;
    k.num_splits = 1; k.blocks_per_split = p->seqlen / kBlockN;
    k.qk_scale_log2 = p->sm_scale * 1.44269504f;      // flash_atten_full_int8.py:156-157
    *kp = k;
    return INTFA_OK;
}

size_t workspace_bytes_for(const intfa_fwd_params* p) {
    if (p == nullptr || p->num_splits <= 1) return 0;
    const size_t rows = (size_t)p->num_splits * p->batch * p->heads * p->seqlen;
    return rows * (size_t)p->head_dim * sizeof(float) + rows * sizeof(float);
}

int setup_split(const intfa_fwd_params* p, KParams* kp) {
    if (p->num_splits <= 1) return INTFA_OK;
    if (p->num_splits > kMaxSplits) return INTFA_ERR_SPLITS;
    const size_t need = workspace_bytes_for(p);
    if (p->workspace == nullptr || p->workspace_bytes < need || !aligned16(p->workspace)) return INTFA_ERR_WORKSPACE;
    const int n_blocks = p->seqlen / kBlockN;
    kp->num_splits = p->num_splits;
    kp->blocks_per_split = (n_blocks + p->num_splits - 1) / p->num_splits;     // csrc/flash_fwd_kernel.h:503
    const size_t rows = (size_t)p->num_splits * p->batch * p->heads * p->seqlen;
    kp->o_part = (float*)p->workspace;
    kp->lse_part = kp->o_part + rows * (size_t)p->head_dim;
    return INTFA_OK;
}

template <typename K> int launch(K kernel, const KParams& kp, hipStream_t stream) {
    const int grid = kp.batch * kp.heads * (kp.seqlen / kBlockM) * kp.num_splits;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), 0, stream, kp);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? INTFA_OK : (int)e;
}

int launch_combine(const intfa_fwd_params* p, const KParams& kp, hipStream_t stream) {
    const int64_t rows = (int64_t)kp.batch * kp.heads * kp.seqlen;
    const int grid = (int)((rows + 3) / 4);       // one wave per output row, 4 rows per workgroup
#define INTFA_COMBINE(DD, ODT) hipLaunchKernelGGL((splitkv_combine_kernel<DD, ODT>), dim3(grid), dim3(256), 0, stream, kp)
    if (kp.head_dim == 64) { if (p->io_dtype == INTFA_F16) INTFA_COMBINE(64, 0); else INTFA_COMBINE(64, 1); }
    else if (kp.head_dim == 128) { if (p->io_dtype == INTFA_F16) INTFA_COMBINE(128, 0); else INTFA_COMBINE(128, 1); }
    else { if (p->io_dtype == INTFA_F16) INTFA_COMBINE(256, 0); else INTFA_COMBINE(256, 1); }
#undef INTFA_COMBINE
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? INTFA_OK : (int)e;
}

// Expands the runtime switches (head_dim, causal, out dtype, P rounding, split) into template arguments.
int dispatch_full_int8(const intfa_fwd_params* p, const KParams& kp, hipStream_t stream) {
    const bool causal = kp.causal != 0, bf = p->io_dtype == INTFA_BF16, split = kp.num_splits > 1;
    const int pr = (p->p_round == INTFA_PROUND_REFERENCE) ? 1 : 0;
#define INTFA_L(DD, C, O, PR, SP) return launch(fwd_full_int8_kernel<DD, C, O, PR, false, SP>, kp, stream)
#define INTFA_SW_SP(DD, C, O, PR) do { if (split) INTFA_L(DD, C, O, PR, true); else INTFA_L(DD, C, O, PR, false); } while (0)
#define INTFA_SW_PR(DD, C, O) do { if (pr) INTFA_SW_SP(DD, C, O, 1); else INTFA_SW_SP(DD, C, O, 0); } while (0)
#define INTFA_SW_O(DD, C) do { if (bf) INTFA_SW_PR(DD, C, 1); else INTFA_SW_PR(DD, C, 0); } while (0)
#define INTFA_SW_C(DD) do { if (causal) INTFA_SW_O(DD, true); else INTFA_SW_O(DD, false); } while (0)
    switch (kp.head_dim) {
        case 64: INTFA_SW_C(64);
        case 128: INTFA_SW_C(128);
    }
#undef INTFA_L
#undef INTFA_SW_SP
#undef INTFA_SW_PR
#undef INTFA_SW_O
#undef INTFA_SW_C
    return INTFA_ERR_HEAD_DIM;
}

}  // namespace

extern "C" {

int intfa_version(void) { return INTFA_VERSION; }

int intfa_block_n(void) { return kBlockN; }

const char* intfa_error_string(int code) {
    switch (code) {
        case INTFA_OK: return "ok";
        case INTFA_ERR_NULL: return "a required pointer is NULL";
        case INTFA_ERR_HEAD_DIM: return "head_dim must be 64, 128 or 256";
        case INTFA_ERR_SEQLEN: return "seqlen must be a positive multiple of 128";
        case INTFA_ERR_ALIGN: return "pointers and row/head/batch strides must be 16-byte aligned";
        case INTFA_ERR_DTYPE: return "unknown dtype enum";
        case INTFA_ERR_WORKSPACE: return "workspace missing, misaligned or too small for num_splits";
        case INTFA_ERR_SHAPE: return "batch and heads must be positive and the grid must fit 31 bits";
        case INTFA_ERR_SPLITS: return "num_splits must be at most 64";
        default: return code > 0 ? "hip error" : "unknown error";
    }
}

size_t intfa_fwd_workspace_bytes(const intfa_fwd_params* p) { return workspace_bytes_for(p); }

int intfa_fwd_full_int8(const intfa_fwd_params* p, void* stream) {
    KParams kp;
    int rc = make_kparams(p, 1, 1, true, true, &kp);
    if (rc != INTFA_OK) return rc;
    if (p->p_round != INTFA_PROUND_RNE && p->p_round != INTFA_PROUND_REFERENCE) return INTFA_ERR_DTYPE;
    rc = setup_split(p, &kp);
    if (rc != INTFA_OK) return rc;
    rc = dispatch_full_int8(p, kp, (hipStream_t)stream);
    if (rc != INTFA_OK || kp.num_splits <= 1) return rc;
    return launch_combine(p, kp, (hipStream_t)stream);
}

int intfa_fwd_half_int8(const intfa_fwd_params* p, void* stream) {
    KParams kp;
    int rc = make_kparams(p, 1, 2, true, false, &kp);
    if (rc != INTFA_OK) return rc;
    rc = setup_split(p, &kp);
    if (rc != INTFA_OK) return rc;
    return -100;
}

int intfa_fwd_fp16(const intfa_fwd_params* p, void* stream) {
    KParams kp;
    int rc = make_kparams(p, 2, 2, false, false, &kp);
    if (rc != INTFA_OK) return rc;
    rc = setup_split(p, &kp);
    if (rc != INTFA_OK) return rc;
    rc = dispatch_fp16(p, kp, (hipStream_t)stream);
    if (rc != INTFA_OK || kp.num_splits <= 1) return rc;
    return launch_combine(p, kp, (hipStream_t)stream);
}

int intfa_debug_qk_int32(const intfa_fwd_params* p, int32_t* s_out, void* stream) {
    KParams kp;
    if (s_out == nullptr) return INTFA_ERR_NULL;
    int rc = make_kparams(p, 1, 0, false, false, &kp);
    if (rc != INTFA_OK) return rc;
    kp.s_dump = s_out;
    kp.causal = 0;
    kp.scale_dtype = INTFA_F32;
    switch (kp.head_dim) {
        case 64: return launch(fwd_full_int8_kernel<64, false, 0, 0, true, false>, kp, (hipStream_t)stream);
        case 128: return launch(fwd_full_int8_kernel<128, false, 0, 0, true, false>, kp, (hipStream_t)stream);
    }
    return INTFA_ERR_HEAD_DIM;
}

}  // extern "C"
