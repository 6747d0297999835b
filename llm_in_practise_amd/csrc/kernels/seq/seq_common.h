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
__device__ __forceinline__ float gelu_tanhf_(float v) {
  return 0.5f * v * (1.f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
}
__device__ __forceinline__ float logsigmoidf_(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// Entry c of a vector whose first `dims` entries are rotated by pos * inv_freq[pair]: neighbours (2i, 2i+1) form pair
// i, or with `half` entries (i, i + dims/2) do; the rest pass unchanged.  Sine and cosine are multiplied by mag.
// The pair (u, v) becomes (u cos - v sin, v cos + u sin); the angle is a float product.
template <typename T>
__device__ __forceinline__ float rotated_at(const T* __restrict__ v, int c, int dims, float pos,
                                            const float* __restrict__ inv_freq, int half, float mag) {
  const float a = (float)v[c];
  if (c >= dims) return a;
  const int hd = dims >> 1;
  const bool second = half ? c >= hd : (c & 1);
  const int pair = half ? (second ? c - hd : c) : (c >> 1);
  const float b = (float)v[half ? (second ? c - hd : c + hd) : (c ^ 1)];
  float sn, cs;
  sincosf(pos * inv_freq[pair], &sn, &cs);
  sn *= mag;
  cs *= mag;
  return second ? a * cs + b * sn : a * cs - b * sn;
}

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
