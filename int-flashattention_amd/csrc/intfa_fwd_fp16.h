// fp16 / bf16 forward (counterpart of flash_atten_fp.py:9-150).
#pragma once
#include "intfa_device.h"
#include "../../include/intfa.h"

namespace intfa {

inline int dispatch_fp16(const intfa_fwd_params*, const KParams&, hipStream_t) { return -100; }

}  // namespace intfa
