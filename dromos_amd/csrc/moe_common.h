// Shared by the decode experts (moe.hip) and the grouped experts (moe_grouped.hip).
#pragma once

#include "common.h"

namespace dro {

struct Stack {
  const uint8_t* data;
  const uint8_t* scale;
  const float* expert_global;
  float global;
};

struct DecodeArgs {
  const uint16_t* latent;  // bf16 [T, L]
  const int32_t* ids;      // [T, top_k]
  const float* weights;    // [T, top_k]
  Stack gu, dn;
  uint16_t* inter;  // bf16 [T * top_k, I], by pair
  float* out;       // f32 [T, L]
  int T, L, I, top_k;
};

// The row factor of row `row_in_stack` of expert e: its row scale (INT8 / FP8), the expert's NVFP4 global, or 1.
__device__ __forceinline__ float stack_factor(int type, const Stack& s, int e, int64_t row_in_stack) {
  if (type == LX_W_INT8 || type == LX_W_FP8) return reinterpret_cast<const float*>(s.scale)[row_in_stack];
  if (type == LX_W_NVFP4) return s.expert_global ? s.expert_global[e] : s.global;
  return 1.0f;
}

inline Stack as_stack(const lx_weight& w) {
  return Stack{static_cast<const uint8_t*>(w.data), static_cast<const uint8_t*>(w.scale), w.expert_global, w.global};
}

inline bool valid_stack(const lx_weight& w, int64_t K) {
  if (!w.data) return false;
  switch (w.type) {
    case LX_W_BF16: return true;
    case LX_W_INT8:
    case LX_W_FP8: return w.scale != nullptr;
    case LX_W_NVFP4: return w.scale != nullptr && K % 16 == 0;
    default: return false;
  }
}

// moe.hip: routing behind lx_moe_route, and the decode experts (T <= 8, top_k <= 8) on two stacks of any formats with
// the intermediate rows in `inter` (lx_moe_decode_workspace_bytes).
int route(const float* logits, const float* selection_bias, int32_t* ids, float* weights, float* entropy, float* confidence, int T,
          int E, int top_k, hipStream_t s);
int experts_decode(const void* latent, const int32_t* ids, const float* weights, const lx_weight& gate_up, const lx_weight& down,
                   float* out, void* inter, int T, int L, int I, int top_k, hipStream_t s);

// Element-wise experts for any T and any shape or alignment (one wavefront per output, pairs independent):
// gate/up into a.inter (by pair), then down and the ordered sum into a.out.
int experts_plain(const DecodeArgs& a, int gu_type, int dn_type, hipStream_t s);

}  // namespace dro
