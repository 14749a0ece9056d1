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

// One workgroup per (batch, head, 128-row query block, split); causal single-pass launches pair the query blocks.
// `column_halves`: workgroups per query block (2 where a kernel splits the output columns over two workgroups).
template <typename K> inline int launch_kernel(K kernel, const KParams& kp, hipStream_t stream, int threads = kThreads,
                                               int column_halves = 1) {
    const int grid = kp.batch * kp.heads * ((kp.seqlen + kBlockM - 1) / kBlockM) * kp.num_splits / (kp.pair_mblocks ? 2 : 1) * column_halves;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), 0, stream, kp);
    return (int)hipGetLastError();
}

#define INTFA_DECL_LAUNCH(name) int name(const KParams& kp, const LaunchSel& sel, hipStream_t stream)
INTFA_DECL_LAUNCH(launch_full_int8_d64);
INTFA_DECL_LAUNCH(launch_full_int8_d128);
INTFA_DECL_LAUNCH(launch_full_int8_d256);
INTFA_DECL_LAUNCH(launch_full_int8_vblk_d64);     // per-block, per-channel V scales
INTFA_DECL_LAUNCH(launch_full_int8_vblk_d128);
INTFA_DECL_LAUNCH(launch_full_int8_vblk_d256);
INTFA_DECL_LAUNCH(launch_full_int8_vblk64_d64);   // V scale rows of 64 keys (two per key block)
INTFA_DECL_LAUNCH(launch_full_int8_vblk64_d128);
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
