// Host-side launch functions, one per (variant, head_dim), each defined in its own translation unit so that the
// kernel instances compile in parallel.
#pragma once
#include "intfa_device.h"

namespace intfa {

constexpr int kDecodeRows = 32;       // query rows per workgroup of the decode-shaped kernel (intfa_fwd_decode.h, intfa_fwd_decode_f16pv.h)

// Launch switches resolved to template arguments inside the instance files.
struct LaunchSel {
    bool causal;
    int io_dt;       // 0 fp16, 1 bf16 (type of out; also of V / fp Q,K where those are 16-bit)
    int p_round;     // full-int8 only
    bool split;      // write split-KV partials instead of the output
    bool dump_s;     // full-int8 only: export int32 S and stop
};

inline FastDiv make_fast_div(int d) {
    int l = 0;
    while ((1ll << l) < (long long)d) ++l;                   // ceil(log2 d), d >= 1
    const unsigned s = 31u + (unsigned)l;
    const unsigned long long m = ((1ull << s) + (unsigned long long)d - 1) / (unsigned long long)d;   // < 2^32
    return {(uint32_t)m, (uint32_t)s};
}
// Fills the workgroup -> work mapping of a launch of `grid` workgroups (grid = batch * heads * workgroups per head).
inline KParams finish_mapping(const KParams& kp, int grid) {
    KParams k = kp;
    const int n_split = kp.num_splits > 1 ? kp.num_splits : 1;
    k.per_head = grid / (kp.batch * kp.heads);
    k.heads_kv = kp.heads / kp.kv_group;
    const int per_kv = k.per_head * kp.kv_group, units = kp.batch * k.heads_kv;
    k.xcd_whole_wgs = (units / 8) * 8 * per_kv;
    k.xcd_rem_chunk = ((units % 8) * per_kv) % 8 == 0 ? (units % 8) * per_kv / 8 : 0;
    k.d_per_kv = make_fast_div(k.per_head * kp.kv_group);
    k.d_heads_kv = make_fast_div(k.heads_kv);
    k.d_per_head = make_fast_div(k.per_head);
    k.d_n_split = make_fast_div(n_split);
    k.d_heads = make_fast_div(kp.heads);
    k.d_kv_group = make_fast_div(kp.kv_group);
    return k;
}

// One workgroup per (batch, head, 128-row query block, split); causal single-pass launches pair the query blocks.
// `column_halves`: workgroups per query block (2 where a kernel splits the output columns over two workgroups).
template <typename K> inline int launch_kernel(K kernel, const KParams& kp, hipStream_t stream, int threads = kThreads,
                                               int column_halves = 1) {
    const int grid = kp.batch * kp.heads * ((kp.seqlen + kBlockM - 1) / kBlockM) * kp.num_splits / (kp.pair_mblocks ? 2 : 1) * column_halves;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), 0, stream, finish_mapping(kp, grid));
    return (int)hipGetLastError();
}

#define INTFA_DECL_LAUNCH(name) int name(const KParams& kp, const LaunchSel& sel, hipStream_t stream)
INTFA_DECL_LAUNCH(launch_full_int8_d64);
INTFA_DECL_LAUNCH(launch_full_int8_d128);
INTFA_DECL_LAUNCH(launch_full_int8_d256);
INTFA_DECL_LAUNCH(launch_full_int8_vblk_d64);     // per-block, per-channel V scales
INTFA_DECL_LAUNCH(launch_full_int8_vblk_d128);
INTFA_DECL_LAUNCH(launch_full_int8_vblk_d256);
INTFA_DECL_LAUNCH(launch_full_int8_vblk64_d128);  // V scale rows of 64 keys (two per 128-key block)
INTFA_DECL_LAUNCH(launch_decode_full_int8_d64);    // few query rows per head: the waves of a workgroup share the keys
INTFA_DECL_LAUNCH(launch_decode_full_int8_d128);
INTFA_DECL_LAUNCH(launch_decode_full_int8_d256);
INTFA_DECL_LAUNCH(launch_decode_half_int8_d64);     // (intfa_fwd_decode_f16pv.h)
INTFA_DECL_LAUNCH(launch_decode_half_int8_d128);
INTFA_DECL_LAUNCH(launch_decode_half_int8_d256);
INTFA_DECL_LAUNCH(launch_decode_fp16_d64);
INTFA_DECL_LAUNCH(launch_decode_fp16_d128);
INTFA_DECL_LAUNCH(launch_decode_fp16_d256);
INTFA_DECL_LAUNCH(launch_half_int8_d64);
INTFA_DECL_LAUNCH(launch_half_int8_d128);
INTFA_DECL_LAUNCH(launch_half_int8_d256);
INTFA_DECL_LAUNCH(launch_fp16_d64);
INTFA_DECL_LAUNCH(launch_fp16_d128);
INTFA_DECL_LAUNCH(launch_fp16_d256);

}  // namespace intfa
