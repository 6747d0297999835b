// Token-wise kernels of models that keep their residual stream in float: scaled embedding with sinusoidal
// positions, RMS norms that read float and write the activation type, the gated + normed residual update
// (fused with the next sublayer's entry norm), the mean of two normed branches, PolyNorm, the per-head
// norm + output gate that follows a recurrent mixer, the token + hashed token-pair embedding, the post-norm residual
// update, RMS norm of activation rows and the gate-then-grouped-norm of a state-space mixer.  One 256-thread block per token (one wave per head for the
// head norm); rows are re-read for the second pass (they sit in L1/L2), so any width works.
#include "seq_common.h"

using namespace lipa;

// x[t, c] = table[tok[t], c] * scale + (c even ? sin : cos)(pos[t] * inv_freq[c / 2])
template <typename T>
__global__ __launch_bounds__(256) void k_embed_sincos(const long* __restrict__ tok, const int* __restrict__ pos,
                                                      const T* __restrict__ table, const float* __restrict__ inv_freq,
                                                      float* __restrict__ x, int W, float scale) {
  const int t = blockIdx.x;
  const long id = tok[t];
  const float p = (float)pos[t];
  for (int c = threadIdx.x; c < W; c += 256) {
    const float a = p * inv_freq[c >> 1];
    x[(size_t)t * W + c] = (float)table[(size_t)id * W + c] * scale + ((c & 1) ? cosf(a) : sinf(a));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void k_rms_f32(const float* __restrict__ x, const float* __restrict__ w,
                                                 T* __restrict__ out, int W, float eps) {
  __shared__ float sc[4];
  const size_t r = (size_t)blockIdx.x * W;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) { const float v = x[r + c]; s += v * v; }
  const float rs = rsqrtf(block_sum256(s, sc) / W + eps);
  for (int c = threadIdx.x; c < W; c += 256) out[r + c] = (T)(x[r + c] * rs * w[c]);
}

// z = y * sigmoid(r + b);  x += z / rms(z) * wb;  optionally h = x / rms(x) * wn
template <typename T>
__global__ __launch_bounds__(256) void k_gated_residual(float* __restrict__ x, const T* __restrict__ y, int ldy,
                                                        const T* __restrict__ r, int ldr, const float* __restrict__ b,
                                                        const float* __restrict__ wb, const float* __restrict__ wn,
                                                        T* __restrict__ h, int W, float eps) {
  __shared__ float sc[4];
  const size_t t = blockIdx.x;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float z = (float)y[t * ldy + c] * sigmoidf_((float)r[t * ldr + c] + b[c]);
    s += z * z;
  }
  const float rs = rsqrtf(block_sum256(s, sc) / W + eps);
  float s2 = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float z = (float)y[t * ldy + c] * sigmoidf_((float)r[t * ldr + c] + b[c]);
    const float v = x[t * W + c] + z * rs * wb[c];
    x[t * W + c] = v;
    s2 += v * v;
  }
  if (wn == nullptr) return;
  const float rs2 = rsqrtf(block_sum256(s2, sc) / W + eps);
  for (int c = threadIdx.x; c < W; c += 256) h[t * W + c] = (T)(x[t * W + c] * rs2 * wn[c]);
}

// out = 0.5 * (a / rms(a) * wa + b / rms(b) * wb)
template <typename T>
__global__ __launch_bounds__(256) void k_dual_norm_mean(const T* __restrict__ a, const T* __restrict__ b,
                                                        const float* __restrict__ wa, const float* __restrict__ wb,
                                                        T* __restrict__ out, int W, float eps) {
  __shared__ float sc[4];
  const size_t r = (size_t)blockIdx.x * W;
  float sa = 0.f, sb = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float u = (float)a[r + c], v = (float)b[r + c];
    sa += u * u;
    sb += v * v;
  }
  const float ra = rsqrtf(block_sum256(sa, sc) / W + eps);
  const float rb = rsqrtf(block_sum256(sb, sc) / W + eps);
  for (int c = threadIdx.x; c < W; c += 256)
    out[r + c] = (T)(0.5f * ((float)a[r + c] * ra * wa[c] + (float)b[r + c] * rb * wb[c]));
}

// PolyNorm: c0 z/rms(z) + c1 z^2/rms(z^2) + c2 z^3/rms(z^3) + c3 over a token's vector
template <typename T>
__global__ __launch_bounds__(256) void k_polynorm(const T* __restrict__ z, const float* __restrict__ coef,
                                                  T* __restrict__ out, int F, float eps) {
  __shared__ float sc[4];
  const size_t r = (size_t)blockIdx.x * F;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int c = threadIdx.x; c < F; c += 256) {
    const float v = (float)z[r + c], v2 = v * v;
    s1 += v2;
    s2 += v2 * v2;
    s3 += v2 * v2 * v2;
  }
  const float r1 = coef[0] * rsqrtf(block_sum256(s1, sc) / F + eps);
  const float r2 = coef[1] * rsqrtf(block_sum256(s2, sc) / F + eps);
  const float r3 = coef[2] * rsqrtf(block_sum256(s3, sc) / F + eps);
  const float c3 = coef[3];
  for (int c = threadIdx.x; c < F; c += 256) {
    const float v = (float)z[r + c], v2 = v * v;
    out[r + c] = (T)(v * r1 + v2 * r2 + v2 * v * r3 + c3);
  }
}

// out[t, h, c] = o[t, h, c] / rms_c(o[t, h, :]) * w[(per_head ? h * dv : 0) + c] * sigmoid(gate[t, h * dv + c]);
// with den / efl (per token and head) o is first divided by max(|den|, efl) + 1e-6 (the mLSTM read-out)
template <typename T>
__global__ __launch_bounds__(256) void k_head_norm_gate(const float* __restrict__ o, const float* __restrict__ w,
                                                        int per_head, const T* __restrict__ gate, int ldg,
                                                        const float* __restrict__ den, const float* __restrict__ efl,
                                                        T* __restrict__ out, int ldo, float scale, int nrows, int H,
                                                        int dv, float eps) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= nrows) return;
  const int t = row / H, hd = row % H;
  const float* src = o + (size_t)row * dv;
  const float dinv = den != nullptr ? 1.f / (fmaxf(fabsf(den[row]), efl[row]) + 1e-6f) : 1.f;
  float s = 0.f;
  for (int c = lane; c < dv; c += 64) {
    const float v = src[c] * dinv;
    s += v * v;
  }
  const float rs = rsqrtf(wave_sum(s) / dv + eps) * dinv;
  for (int c = lane; c < dv; c += 64) {
    const float g = sigmoidf_((float)gate[(size_t)t * ldg + hd * dv + c]) * scale;
    out[(size_t)t * ldo + hd * dv + c] = (T)(src[c] * rs * w[(per_head ? hd * dv : 0) + c] * g);
  }
}

// g = exp(-exp(A_log[h]) * softplus(pre + bias)), laid out [T, H * dk]
__global__ __launch_bounds__(256) void k_decay_gate(const float* __restrict__ pre, const float* __restrict__ bias,
                                                    const float* __restrict__ a_log, float* __restrict__ g, size_t n,
                                                    int HD, int dk) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int c = (int)(i % HD);
  g[i] = expf(-expf(a_log[c / dk]) * softplusf_(pre[i] + bias[c]));
}

// x[t] = table[tok[t]] * scale + pair[(prev * mul_prev + tok[t] * mul_cur) mod buckets]; a sequence's first token takes
// row `buckets`.  prev is the token before: the packed neighbour, or for a step's first token of a continued
// sequence the slot's carried token.  The block of a sequence's first token of the step also carries the step's last
// token into the slot (it alone reads the old one).  Writes the float stream and its copy in the activation type.
template <typename T>
__global__ __launch_bounds__(256) void k_embed_pair(const long* __restrict__ tok, const T* __restrict__ table,
                                                    const T* __restrict__ pair, int* __restrict__ prev_state,
                                                    float* __restrict__ x, T* __restrict__ h, int W, float scale,
                                                    long buckets, long mul_prev, long mul_cur, SeqDesc d) {
  const int t = blockIdx.x, s = d.tok_seq[t], j = t - d.seq_off[s], slot = d.slots[s];
  const long id = tok[t];
  long row = buckets;
  if (pair != nullptr) {
    if (j > 0)
      row = (tok[t - 1] * mul_prev + id * mul_cur) % buckets;
    else if (d.pos0[s] > 0)
      row = ((long)prev_state[slot] * mul_prev + id * mul_cur) % buckets;
  }
  __syncthreads();                                   // every thread has read the carried token
  if (j == 0 && threadIdx.x == 0 && prev_state != nullptr && !(d.live && !d.live[s]))
    prev_state[slot] = (int)tok[d.seq_off[s + 1] - 1];
  for (int c = threadIdx.x; c < W; c += 256) {
    float v = (float)table[(size_t)id * W + c] * scale;
    if (pair != nullptr) v += (float)pair[(size_t)row * W + c];
    x[(size_t)t * W + c] = v;
    h[(size_t)t * W + c] = (T)v;
  }
}

// post-norm residual: x <- rms(alpha x + y) * w in place (float), h = x in the activation type
template <typename T, typename YT>
__global__ __launch_bounds__(256) void k_scaled_postnorm(float* __restrict__ x, const YT* __restrict__ y, int ldy,
                                                         const float* __restrict__ w, T* __restrict__ h, int W,
                                                         float alpha, float eps) {
  __shared__ float sc[4];
  const size_t t = blockIdx.x;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = alpha * x[t * W + c] + (float)y[t * ldy + c];
    s += v * v;
  }
  const float rs = rsqrtf(block_sum256(s, sc) / W + eps);
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = (alpha * x[t * W + c] + (float)y[t * ldy + c]) * rs * w[c];
    x[t * W + c] = v;
    h[t * W + c] = (T)v;
  }
}

// RMS norm of activation rows (a column slice of a wider matrix is fine)
template <typename T>
__global__ __launch_bounds__(256) void k_rms_act(const T* __restrict__ u, int ldu, const float* __restrict__ w,
                                                 T* __restrict__ out, int n, float eps) {
  __shared__ float sc[4];
  const size_t t = blockIdx.x;
  float s = 0.f;
  for (int c = threadIdx.x; c < n; c += 256) {
    const float v = (float)u[t * ldu + c];
    s += v * v;
  }
  const float rs = rsqrtf(block_sum256(s, sc) / n + eps);
  for (int c = threadIdx.x; c < n; c += 256) out[t * n + c] = (T)((float)u[t * ldu + c] * rs * w[c]);
}

// gate first, then norm: v = y * silu(z); out = v / rms_part(v) * w, the row cut into equal parts of `gs` entries.
// VEC: four columns per thread and step (16-byte loads of y and w, 8- or 16-byte loads of z); the gated values of a
// thread's first two steps stay in registers for the second pass.
template <typename T>
__device__ __forceinline__ f32x4 load4_act(const T* p);
template <>
__device__ __forceinline__ f32x4 load4_act<float>(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
template <>
__device__ __forceinline__ f32x4 load4_act<bf16>(const bf16* p) {
  const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
  return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}
__device__ __forceinline__ void store4_act(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ __forceinline__ void store4_act(bf16* p, f32x4 v) {
  *reinterpret_cast<bf16x4*>(p) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void k_gate_group_norm(const float* __restrict__ y, const T* __restrict__ z, int ldz,
                                                         const float* __restrict__ w, T* __restrict__ out, int n, int gs,
                                                         float eps) {
  __shared__ float sc[4];
  const size_t t = blockIdx.x;
  const int c0 = blockIdx.y * gs;
  float s = 0.f;
  if (VEC) {
    constexpr int KEEP = 4;                       // steps whose gated values are kept: parts up to 4096 entries
    f32x4 kept[KEEP];
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
      const int c = c0 + 4 * threadIdx.x + 1024 * k;
      kept[k] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (c < c0 + gs) {
        const f32x4 g = load4_act<T>(z + t * ldz + c), yv = load4_act<float>(y + t * n + c);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          kept[k][j] = yv[j] * g[j] * sigmoidf_(g[j]);
          s += kept[k][j] * kept[k][j];
        }
      }
    }
    for (int c = c0 + 4 * threadIdx.x + 1024 * KEEP; c < c0 + gs; c += 1024) {
      const f32x4 g = load4_act<T>(z + t * ldz + c), yv = load4_act<float>(y + t * n + c);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float v = yv[j] * g[j] * sigmoidf_(g[j]);
        s += v * v;
      }
    }
    const float rs = rsqrtf(block_sum256(s, sc) / gs + eps);
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
      const int c = c0 + 4 * threadIdx.x + 1024 * k;
      if (c < c0 + gs) {
        const f32x4 wv = load4_act<float>(w + c);
        store4_act(out + t * n + c, f32x4{kept[k][0] * rs * wv[0], kept[k][1] * rs * wv[1], kept[k][2] * rs * wv[2],
                                          kept[k][3] * rs * wv[3]});
      }
    }
    for (int c = c0 + 4 * threadIdx.x + 1024 * KEEP; c < c0 + gs; c += 1024) {
      const f32x4 g = load4_act<T>(z + t * ldz + c), yv = load4_act<float>(y + t * n + c), wv = load4_act<float>(w + c);
      f32x4 o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = yv[j] * g[j] * sigmoidf_(g[j]) * rs * wv[j];
      store4_act(out + t * n + c, o);
    }
    return;
  }
  for (int c = c0 + threadIdx.x; c < c0 + gs; c += 256) {
    const float g = (float)z[t * ldz + c], v = y[t * n + c] * g * sigmoidf_(g);
    s += v * v;
  }
  const float rs = rsqrtf(block_sum256(s, sc) / gs + eps);
  for (int c = c0 + threadIdx.x; c < c0 + gs; c += 256) {
    const float g = (float)z[t * ldz + c];
    out[t * n + c] = (T)(y[t * n + c] * g * sigmoidf_(g) * rs * w[c]);
  }
}

// ---------------------------------------------------------------------------------------------- launchers
// x[t, s, c] = table[tok[t], c] + ptable[pos[t], c] for every stream s (learned positions, not scaled); a position past
// the table reads its last row (rows nobody reads may carry any position)
template <typename T>
__global__ __launch_bounds__(256) void k_embed_learned(const long* __restrict__ tok, const int* __restrict__ pos,
                                                       const T* __restrict__ table, const T* __restrict__ ptable,
                                                       float* __restrict__ x, int W, int S, int prow, int vocab) {
  const size_t t = blockIdx.x;
  const size_t id = (size_t)min(max(tok[t], 0l), (long)vocab - 1), p = (size_t)min(max(pos[t], 0), prow - 1);
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = (float)table[id * W + c] + (float)ptable[p * W + c];
    for (int s = 0; s < S; ++s) x[(t * S + s) * W + c] = v;
  }
}

// Several residual streams X [T, S, W] (float, in place).  With a sublayer output y: X_t <- sum_s mix[s, t] X_s +
// out[t] y for all t at once; then h = rmsnorm(sum_s read[s] X_s) * w, the next sublayer's input.  y == null: only h.
constexpr int MAXS = 8;
template <typename T, typename YT>
__global__ __launch_bounds__(256) void k_hyper_mix_norm(float* __restrict__ X, const YT* __restrict__ y, int ldy,
                                                        const float* __restrict__ mix, const float* __restrict__ outw,
                                                        const float* __restrict__ read, const float* __restrict__ w,
                                                        T* __restrict__ h, int W, int S, float eps) {
  __shared__ float sc[4];
  __shared__ float sm[MAXS * MAXS + 2 * MAXS];
  const size_t t = blockIdx.x;
  float* smix = sm;
  float* sout = sm + MAXS * MAXS;
  float* srd = sout + MAXS;
  if (threadIdx.x < S * S) smix[threadIdx.x] = y != nullptr ? mix[threadIdx.x] : 0.f;
  if (threadIdx.x < S) {
    sout[threadIdx.x] = y != nullptr ? outw[threadIdx.x] : 0.f;
    srd[threadIdx.x] = read[threadIdx.x];
  }
  __syncthreads();
  float* xr = X + t * S * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    float old[MAXS], u = 0.f;
#pragma unroll
    for (int s = 0; s < MAXS; ++s) old[s] = s < S ? xr[(size_t)s * W + c] : 0.f;
    if (y != nullptr) {
      const float yv = (float)y[t * ldy + c];
#pragma unroll
      for (int k = 0; k < MAXS; ++k)
        if (k < S) {
          float v = sout[k] * yv;
#pragma unroll
          for (int s = 0; s < MAXS; ++s)
            if (s < S) v += smix[s * S + k] * old[s];
          xr[(size_t)k * W + c] = v;
          u += srd[k] * v;
        }
    } else {
#pragma unroll
      for (int s = 0; s < MAXS; ++s)
        if (s < S) u += srd[s] * old[s];
    }
    ss += u * u;
  }
  const float rs = rsqrtf(block_sum256(ss, sc) / W + eps);
  for (int c = threadIdx.x; c < W; c += 256) {      // the thread re-reads the columns it wrote itself
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < MAXS; ++s)
      if (s < S) u += srd[s] * xr[(size_t)s * W + c];
    h[t * W + c] = (T)(u * rs * w[c]);
  }
}

// The same with four columns per thread and 16-byte accesses; the mixed columns a thread has read stay in its
// registers for the write after the reduction (widths up to 4 * 256 * HUC; wider rows re-read the rest).
constexpr int HUC = 4;
__device__ __forceinline__ f32x4 ld4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ f32x4 ld4(const bf16* p) {
  const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
  return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}
__device__ __forceinline__ void st4(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ __forceinline__ void st4(bf16* p, f32x4 v) {
  *reinterpret_cast<bf16x4*>(p) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
}

template <typename T, typename YT>
__global__ __launch_bounds__(256) void k_hyper_mix_norm4(float* __restrict__ X, const YT* __restrict__ y, int ldy,
                                                         const float* __restrict__ mix, const float* __restrict__ outw,
                                                         const float* __restrict__ read, const float* __restrict__ w,
                                                         T* __restrict__ h, int W, int S, float eps) {
  __shared__ float sc[4];
  __shared__ float sm[MAXS * MAXS + 2 * MAXS];
  const size_t t = blockIdx.x;
  float* smix = sm;
  float* sout = sm + MAXS * MAXS;
  float* srd = sout + MAXS;
  if (threadIdx.x < S * S) smix[threadIdx.x] = y != nullptr ? mix[threadIdx.x] : 0.f;
  if (threadIdx.x < S) {
    sout[threadIdx.x] = y != nullptr ? outw[threadIdx.x] : 0.f;
    srd[threadIdx.x] = read[threadIdx.x];
  }
  __syncthreads();
  float* xr = X + t * S * W;
  const int W4 = W >> 2;
  // four columns: streams mixed and written back (with y), their read-weighted sum returned
  auto columns = [&](int c4) -> f32x4 {
    f32x4 old[MAXS], u = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < MAXS; ++s)
      if (s < S) old[s] = ld4(xr + (size_t)s * W + 4 * c4);
    if (y != nullptr) {
      const f32x4 yv = ld4(y + t * ldy + 4 * c4);
#pragma unroll
      for (int k = 0; k < MAXS; ++k)
        if (k < S) {
          f32x4 v = yv * sout[k];
#pragma unroll
          for (int s = 0; s < MAXS; ++s)
            if (s < S) v += old[s] * smix[s * S + k];
          st4(xr + (size_t)k * W + 4 * c4, v);
          u += v * srd[k];
        }
    } else {
#pragma unroll
      for (int s = 0; s < MAXS; ++s)
        if (s < S) u += old[s] * srd[s];
    }
    return u;
  };
  f32x4 keep[HUC];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < HUC; ++i) {
    const int c4 = threadIdx.x + 256 * i;
    if (c4 < W4) {
      keep[i] = columns(c4);
      ss += keep[i][0] * keep[i][0] + keep[i][1] * keep[i][1] + keep[i][2] * keep[i][2] + keep[i][3] * keep[i][3];
    }
  }
  for (int c4 = threadIdx.x + 256 * HUC; c4 < W4; c4 += 256) {
    const f32x4 u = columns(c4);
    ss += u[0] * u[0] + u[1] * u[1] + u[2] * u[2] + u[3] * u[3];
  }
  const float rs = rsqrtf(block_sum256(ss, sc) / W + eps);
#pragma unroll
  for (int i = 0; i < HUC; ++i) {
    const int c4 = threadIdx.x + 256 * i;
    if (c4 < W4) st4(h + t * W + 4 * c4, keep[i] * ld4(w + 4 * c4) * rs);
  }
  for (int c4 = threadIdx.x + 256 * HUC; c4 < W4; c4 += 256) {      // the thread re-reads the columns it wrote itself
    f32x4 u = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < MAXS; ++s)
      if (s < S) u += ld4(xr + (size_t)s * W + 4 * c4) * srd[s];
    st4(h + t * W + 4 * c4, u * ld4(w + 4 * c4) * rs);
  }
}

// A step's [q | k | v] rows on their way into attention: q and k RMS-normed over their whole width, the normed k and
// the values (blended with another cache's values of the same slot and position when vfirst is given:
// (1 - lam) v + lam vfirst) written to the slot cache rows of each token's position.
template <typename T>
__global__ __launch_bounds__(256) void k_qk_norm_store(const T* __restrict__ u, int ldu, const float* __restrict__ qw,
                                                       const float* __restrict__ kw, T* __restrict__ qout,
                                                       T* __restrict__ kc, T* __restrict__ vc,
                                                       const T* __restrict__ vfirst, const float* __restrict__ lam,
                                                       int nq, int nk, int nv, int max_len, float eps, SeqDesc d) {
  __shared__ float sc[4];
  const size_t t = blockIdx.x;
  const T* r = u + t * ldu;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < nq; c += 256) { const float v = (float)r[c]; sq += v * v; }
  for (int c = threadIdx.x; c < nk; c += 256) { const float v = (float)r[nq + c]; sk += v * v; }
  const float rq = rsqrtf(block_sum256(sq, sc) / nq + eps);
  const float rk = rsqrtf(block_sum256(sk, sc) / nk + eps);
  for (int c = threadIdx.x; c < nq; c += 256) qout[t * nq + c] = (T)((float)r[c] * rq * qw[c]);
  const int pos = d.tok_pos[t], slot = d.slots[d.tok_seq[t]];
  if (pos < 0 || pos >= max_len) return;             // a row nobody reads may carry any position
  const size_t row = (size_t)slot * max_len + pos;
  for (int c = threadIdx.x; c < nk; c += 256) kc[row * nk + c] = (T)((float)r[nq + c] * rk * kw[c]);
  if (vfirst != nullptr) {
    const float l = lam[0];
    for (int c = threadIdx.x; c < nv; c += 256)
      vc[row * nv + c] = (T)((1.f - l) * (float)r[nq + nk + c] + l * (float)vfirst[row * nv + c]);
  } else {
    for (int c = threadIdx.x; c < nv; c += 256) vc[row * nv + c] = r[nq + nk + c];
  }
}

// A step's [q | k (| v)] rows on their way into rotary attention: the first `dims` entries of every q and k head are
// rotated at the token's position; the rotated k goes to the key cache; the value cache gets the v columns or, with
// vkeys, the k columns as they came (a design whose values are its unrotated keys).  One block per token.
template <typename T>
__global__ __launch_bounds__(256) void k_rope_kv_store(const T* __restrict__ u, int ldu, const float* __restrict__ inv_freq,
                                                       T* __restrict__ qout, T* __restrict__ kc, T* __restrict__ vc,
                                                       int nq, int nk, int nv, int dk, int dims, int half, float mag,
                                                       int vkeys, int max_len, SeqDesc d) {
  const size_t t = blockIdx.x;
  const T* r = u + t * ldu;
  const int pos = d.tok_pos[t], slot = d.slots[d.tok_seq[t]];
  const float p = (float)pos;
  for (int c = threadIdx.x; c < nq; c += 256) {
    const int cl = c % dk;
    qout[t * nq + c] = (T)rotated_at(r + (c - cl), cl, dims, p, inv_freq, half, mag);
  }
  if (pos < 0 || pos >= max_len) return;             // a row nobody reads may carry any position
  const size_t row = (size_t)slot * max_len + pos;
  for (int c = threadIdx.x; c < nk; c += 256) {
    const int cl = c % dk;
    kc[row * nk + c] = (T)rotated_at(r + nq + (c - cl), cl, dims, p, inv_freq, half, mag);
    if (vkeys) vc[row * nk + c] = r[nq + c];
  }
  if (!vkeys)
    for (int c = threadIdx.x; c < nv; c += 256) vc[row * nv + c] = r[nq + nk + c];
}

// out = y * sigmoid(gate), element by element; gate rows are ldg apart
template <typename T>
__global__ __launch_bounds__(256) void k_sigmoid_gate(const T* __restrict__ y, const T* __restrict__ gate, int ldg,
                                                      T* __restrict__ out, size_t n, int C) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const size_t t = i / C, c = i % C;
  out[i] = (T)((float)y[i] * sigmoidf_((float)gate[t * ldg + c]));
}

// What the generalised delta rule needs besides its projections, float [T, H * dk]: the decay
// w = exp(-dscale * sigmoid(pre + wb)) with pre = sum_j tanh(low[t, j]) up[c, j] (or pre = low[t, c] when up is null),
// the removal rate a = sigmoid(apre + ab), and per (token, head) kinv = 1 / (sum_head k^2 + 1e-6), the squared length
// that makes the key a unit vector.  One wave per (head, tpw consecutive tokens): a lane keeps the low-rank rows of
// its channels in registers (RK = 16: rank <= 16) and takes tanh of one low-rank input per token, handed round the
// wave; dk <= 256: 4 channels a lane.
template <typename T, typename LT, int RK>
__global__ __launch_bounds__(256) void k_delta_gates(const T* __restrict__ k, int ldk, const LT* __restrict__ low, int ldl,
                                                     const float* __restrict__ up, int rank,
                                                     const float* __restrict__ wb, const T* __restrict__ apre, int lda,
                                                     const float* __restrict__ ab, float* __restrict__ w,
                                                     float* __restrict__ ar, float* __restrict__ kinv, int T_, int tpw,
                                                     int nrows, int H, int dk, float dscale) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= nrows) return;
  const int hd = row % H, t0 = (row / H) * tpw, t1 = min(T_, t0 + tpw);
  float upr[4][RK > 0 ? RK : 1], bw[4], ba[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = lane + 64 * i, ch = hd * dk + c;
    bw[i] = (c < dk && wb != nullptr) ? wb[ch] : 0.f;
    ba[i] = (c < dk && ab != nullptr) ? ab[ch] : 0.f;
    if (RK > 0)
#pragma unroll
      for (int j = 0; j < RK; ++j) upr[i][j] = (c < dk && j < rank) ? up[(size_t)ch * rank + j] : 0.f;
  }
  for (int t = t0; t < t1; ++t) {
    const T* kr = k + (size_t)t * ldk + hd * dk;
    float ss = 0.f;
    for (int c = lane; c < dk; c += 64) {
      const float v = (float)kr[c];
      ss += v * v;
    }
    ss = wave_sum(ss);
    if (lane == 0) kinv[(size_t)t * H + hd] = 1.f / (ss + 1e-6f);
    float pre[4] = {0.f, 0.f, 0.f, 0.f};
    if (up != nullptr) {
      for (int j0 = 0; j0 < rank; j0 += 64) {
        const float tl = j0 + lane < rank ? tanhf((float)low[(size_t)t * ldl + j0 + lane]) : 0.f;
        if (RK > 0) {
#pragma unroll
          for (int jj = 0; jj < RK; ++jj) {
            const float tj = __shfl(tl, jj, 64);
#pragma unroll
            for (int i = 0; i < 4; ++i) pre[i] += tj * upr[i][jj];
          }
        } else {
          const int nj = min(64, rank - j0);
          for (int jj = 0; jj < nj; ++jj) {
            const float tj = __shfl(tl, jj, 64);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int c = lane + 64 * i;
              if (c < dk) pre[i] += tj * up[(size_t)(hd * dk + c) * rank + j0 + jj];
            }
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = lane + 64 * i;
      if (c >= dk) break;
      const int ch = hd * dk + c;
      const float pr = (up != nullptr ? pre[i] : (float)low[(size_t)t * ldl + ch]) + bw[i];
      const float a = (float)apre[(size_t)t * lda + ch] + ba[i];
      const size_t o = (size_t)t * ((size_t)H * dk) + ch;
      w[o] = expf(-dscale * sigmoidf_(pr));
      ar[o] = sigmoidf_(a);
    }
  }
}

void seq_rope_kv_store(int code, const void* u, int ldu, const float* inv_freq, void* qout, void* kc, void* vc, int nq,
                       int nk, int nv, int dk, int dims, int half, float mag, int vkeys, int max_len, SeqDesc d,
                       hipStream_t st) {
  if (d.Ttot == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_rope_kv_store<T>, dim3(d.Ttot), dim3(256), 0, st, (const T*)u, ldu, inv_freq,
                                          (T*)qout, (T*)kc, (T*)vc, nq, nk, nv, dk, dims, half, mag, vkeys, max_len, d));
  LIPA_CHECK_LAUNCH();
}

void seq_sigmoid_gate(int code, const void* y, const void* gate, int ldg, void* out, int T_, int C, hipStream_t st) {
  const size_t n = (size_t)T_ * C;
  if (n == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_sigmoid_gate<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                                          (const T*)y, (const T*)gate, ldg, (T*)out, n, C));
  LIPA_CHECK_LAUNCH();
}

// low_f32: the decay's pre-activation (or its low-rank input) is float whatever the activation type
void seq_delta_gates(int code, int low_f32, const void* k, int ldk, const void* low, int ldl, const float* up, int rank,
                     const float* wb, const void* apre, int lda, const float* ab, float* w, float* ar, float* kinv, int T_,
                     int H, int dk, float dscale, hipStream_t st) {
  if (T_ == 0) return;
  const int tpw = T_ >= 256 ? 8 : 1;                 // long steps: a wave keeps its low-rank rows for 8 tokens
  const int rows = ((T_ + tpw - 1) / tpw) * H;
  const bool reg = up != nullptr && rank <= 16;
#define SEQ_GATES_LAUNCH(LT, RK)                                                                                       \
  hipLaunchKernelGGL((k_delta_gates<T, LT, RK>), dim3((rows + 3) / 4), dim3(256), 0, st, (const T*)k, ldk, (const LT*)low, \
                     ldl, up, rank, wb, (const T*)apre, lda, ab, w, ar, kinv, T_, tpw, rows, H, dk, dscale)
  SEQ_DISPATCH_T(code, {
    if (low_f32) {
      if (reg) SEQ_GATES_LAUNCH(float, 16); else SEQ_GATES_LAUNCH(float, 0);
    } else {
      if (reg) SEQ_GATES_LAUNCH(T, 16); else SEQ_GATES_LAUNCH(T, 0);
    }
  });
#undef SEQ_GATES_LAUNCH
  LIPA_CHECK_LAUNCH();
}

void seq_embed_sincos(int code, const long* tok, const int* pos, const void* table, const float* inv_freq, float* x,
                      int T_, int W, float scale, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_embed_sincos<T>, dim3(T_), dim3(256), 0, st, tok, pos, (const T*)table,
                                          inv_freq, x, W, scale));
  LIPA_CHECK_LAUNCH();
}

void seq_rms_f32(int code, const float* x, const float* w, void* out, int T_, int W, float eps, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_rms_f32<T>, dim3(T_), dim3(256), 0, st, x, w, (T*)out, W, eps));
  LIPA_CHECK_LAUNCH();
}

void seq_gated_residual(int code, float* x, const void* y, int ldy, const void* r, int ldr, const float* b,
                        const float* wb, const float* wn, void* h, int T_, int W, float eps, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_gated_residual<T>, dim3(T_), dim3(256), 0, st, x, (const T*)y, ldy,
                                          (const T*)r, ldr, b, wb, wn, (T*)h, W, eps));
  LIPA_CHECK_LAUNCH();
}

void seq_dual_norm_mean(int code, const void* a, const void* b, const float* wa, const float* wb, void* out, int T_,
                        int W, float eps, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_dual_norm_mean<T>, dim3(T_), dim3(256), 0, st, (const T*)a, (const T*)b,
                                          wa, wb, (T*)out, W, eps));
  LIPA_CHECK_LAUNCH();
}

void seq_polynorm(int code, const void* z, const float* coef, void* out, int T_, int F, float eps, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code,
                 hipLaunchKernelGGL(k_polynorm<T>, dim3(T_), dim3(256), 0, st, (const T*)z, coef, (T*)out, F, eps));
  LIPA_CHECK_LAUNCH();
}

void seq_head_norm_gate(int code, const float* o, const float* w, int per_head, const void* gate, int ldg,
                        const float* den, const float* efl, void* out, int ldo, float scale, int T_, int H, int dv,
                        float eps, hipStream_t st) {
  const int rows = T_ * H;
  if (rows == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_head_norm_gate<T>, dim3((rows + 3) / 4), dim3(256), 0, st, o, w, per_head,
                                          (const T*)gate, ldg, den, efl, (T*)out, ldo, scale, rows, H, dv, eps));
  LIPA_CHECK_LAUNCH();
}

void seq_decay_gate(const float* pre, const float* bias, const float* a_log, float* g, int T_, int HD, int dk,
                    hipStream_t st) {
  const size_t n = (size_t)T_ * HD;
  if (n == 0) return;
  hipLaunchKernelGGL(k_decay_gate, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, pre, bias, a_log, g, n, HD, dk);
  LIPA_CHECK_LAUNCH();
}

void seq_embed_pair(int code, const long* tok, const void* table, const void* pair, int* prev_state, float* x, void* h,
                    int W, float scale, long buckets, long mul_prev, long mul_cur, SeqDesc d, hipStream_t st) {
  if (d.Ttot == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_embed_pair<T>, dim3(d.Ttot), dim3(256), 0, st, tok, (const T*)table,
                                          (const T*)pair, prev_state, x, (T*)h, W, scale, buckets, mul_prev, mul_cur, d));
  LIPA_CHECK_LAUNCH();
}

void seq_scaled_postnorm(int code, int y_f32, float* x, const void* y, int ldy, const float* w, void* h, int T_, int W,
                         float alpha, float eps, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, {
    if (y_f32)
      hipLaunchKernelGGL((k_scaled_postnorm<T, float>), dim3(T_), dim3(256), 0, st, x, (const float*)y, ldy, w, (T*)h, W,
                         alpha, eps);
    else
      hipLaunchKernelGGL((k_scaled_postnorm<T, T>), dim3(T_), dim3(256), 0, st, x, (const T*)y, ldy, w, (T*)h, W, alpha,
                         eps);
  });
  LIPA_CHECK_LAUNCH();
}

void seq_rms_act(int code, const void* u, int ldu, const float* w, void* out, int T_, int n, float eps, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code,
                 hipLaunchKernelGGL(k_rms_act<T>, dim3(T_), dim3(256), 0, st, (const T*)u, ldu, w, (T*)out, n, eps));
  LIPA_CHECK_LAUNCH();
}

void seq_gate_group_norm(int code, const float* y, const void* z, int ldz, const float* w, void* out, int T_, int n,
                         int parts, float eps, hipStream_t st) {
  if (T_ == 0) return;
  const int gs = n / parts;
  const bool vec = gs % 4 == 0 && n % 4 == 0 && ldz % 4 == 0 && ((uintptr_t)z & 15) == 0;   // 16-byte rows
  SEQ_DISPATCH_T(code, {
    if (vec)
      hipLaunchKernelGGL((k_gate_group_norm<T, true>), dim3(T_, parts), dim3(256), 0, st, y, (const T*)z, ldz, w,
                         (T*)out, n, gs, eps);
    else
      hipLaunchKernelGGL((k_gate_group_norm<T, false>), dim3(T_, parts), dim3(256), 0, st, y, (const T*)z, ldz, w,
                         (T*)out, n, gs, eps);
  });
  LIPA_CHECK_LAUNCH();
}

int seq_hyper_max_streams() { return MAXS; }

void seq_embed_learned(int code, const long* tok, const int* pos, const void* table, const void* ptable, float* x, int T_,
                       int W, int S, int prow, int vocab, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_embed_learned<T>, dim3(T_), dim3(256), 0, st, tok, pos, (const T*)table,
                                          (const T*)ptable, x, W, S, prow, vocab));
  LIPA_CHECK_LAUNCH();
}

void seq_hyper_mix_norm(int code, int y_f32, float* X, const void* y, int ldy, const float* mix, const float* outw,
                        const float* read, const float* w, void* h, int T_, int W, int S, float eps, hipStream_t st) {
  if (T_ == 0) return;
  const bool vec = W % 4 == 0 && ldy % 4 == 0 && ((uintptr_t)y & 15) == 0;      // 16-byte rows (X, w, h are whole tensors)
  SEQ_DISPATCH_T(code, {
    if (vec && y_f32)
      hipLaunchKernelGGL((k_hyper_mix_norm4<T, float>), dim3(T_), dim3(256), 0, st, X, (const float*)y, ldy, mix, outw,
                         read, w, (T*)h, W, S, eps);
    else if (vec)
      hipLaunchKernelGGL((k_hyper_mix_norm4<T, T>), dim3(T_), dim3(256), 0, st, X, (const T*)y, ldy, mix, outw, read, w,
                         (T*)h, W, S, eps);
    else if (y_f32)
      hipLaunchKernelGGL((k_hyper_mix_norm<T, float>), dim3(T_), dim3(256), 0, st, X, (const float*)y, ldy, mix, outw,
                         read, w, (T*)h, W, S, eps);
    else
      hipLaunchKernelGGL((k_hyper_mix_norm<T, T>), dim3(T_), dim3(256), 0, st, X, (const T*)y, ldy, mix, outw, read, w,
                         (T*)h, W, S, eps);
  });
  LIPA_CHECK_LAUNCH();
}

void seq_qk_norm_store(int code, const void* u, int ldu, const float* qw, const float* kw, void* qout, void* kc, void* vc,
                       const void* vfirst, const float* lam, int nq, int nk, int nv, int max_len, float eps, SeqDesc d,
                       hipStream_t st) {
  if (d.Ttot == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_qk_norm_store<T>, dim3(d.Ttot), dim3(256), 0, st, (const T*)u, ldu, qw, kw,
                                          (T*)qout, (T*)kc, (T*)vc, (const T*)vfirst, lam, nq, nk, nv, max_len, eps, d));
  LIPA_CHECK_LAUNCH();
}
