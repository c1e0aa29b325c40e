// Shared pieces of the sequence-state kernels (recurrent mixers, short convolutions, head-mixing and latent
// attention, routed experts, fp32-residual norms).  Activations are bf16 or float (template parameter T); the
// residual stream, every norm, softmax, gate and recurrent state is float.
//
// A step's tokens are packed back to back, [Ttot, features].  Sequence b owns tokens seq_off[b] .. seq_off[b+1]-1,
// lives in state slot slots[b] and starts this step at position pos0[b] (0 = a fresh sequence: its state is taken
// as zero, whatever the slot held before).  live (optional) marks rows whose state may be touched.
#pragma once
#include "../common.h"

namespace lipa {

struct SeqDesc {
  const int* seq_off;   // [B + 1]
  const int* slots;     // [B]
  const int* pos0;      // [B]
  const int* tok_seq;   // [Ttot] sequence of a token
  const int* tok_pos;   // [Ttot] absolute position of a token
  const int* live;      // [B] or null
  int B, Ttot;
};

__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float softplusf_(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float logsigmoidf_(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// sum over a 256-thread block (4 waves); result in every thread
__device__ __forceinline__ float block_sum256(float v, float* scratch) { return block_sum<4>(v, scratch); }

}  // namespace lipa

#define SEQ_DISPATCH_T(code, ...)              \
  do {                                         \
    if ((code) == 0) {                         \
      using T = lipa::bf16;                    \
      __VA_ARGS__;                             \
    } else {                                   \
      using T = float;                         \
      __VA_ARGS__;                             \
    }                                          \
  } while (0)
