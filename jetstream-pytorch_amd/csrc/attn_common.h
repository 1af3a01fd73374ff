// Argument checks and addressing shared by the decode-attention kernels.
#pragma once

#include "common.h"

namespace jpt {

enum AttnMode { kRagged = 0, kDense = 1, kPaged = 2 };

int32_t check_attn_args(const jpt_attn_args& a, AttnMode mode);

// The MFMA kernel's own entry; returns JPT_OK after enqueueing, or
// JPT_E_BADARG (without setting the message) when the shape is outside what
// it handles and the generic kernel must run.
bool attn_fast_supported(const jpt_attn_args& a, AttnMode mode);
int32_t attn_fast_launch(const jpt_attn_args& a, AttnMode mode, hipStream_t stream);
int64_t attn_fast_workspace_bytes(const jpt_attn_args& a);
int32_t attn_plan_launch(const jpt_attn_args& a, bool paged, hipStream_t stream);

int32_t attn_generic_launch(const jpt_attn_args& a, AttnMode mode, hipStream_t stream);

}  // namespace jpt
