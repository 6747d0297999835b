// Mixture-of-experts feed-forward for serving: group-limited top-k routing over softmax scores with a selection-only
// correction and identity experts; a few-token path in which every (token, chosen expert) pair streams its expert's
// rows (no sort, no host round trip: decode steps and hipGraphs); and the weighted combine of expert outputs.
// Routing variants (`kind` bits): scores as each output's own sigmoid instead of the softmax (1), a group ranked by the
// sum of its two largest choices instead of its largest (2), weights divided by their sum over the chosen (4).
// Experts are clipped GLUs or SiLU GLUs; the shared expert may sit behind a per-token sigmoid gate.
// Router scores, weights and the combine are float; expert products read the activation type and accumulate in float.
#include "seq_common.h"

using namespace lipa;

constexpr int RPL = 4;   // router outputs per lane: experts + identity experts <= 64 * RPL

// (value, index) maximum over a wave; ties go to the lower index
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, 64);
    const int oi = __shfl_xor(i, o, 64);
    if (ov > v || (ov == v && oi < i)) {
      v = ov;
      i = oi;
    }
  }
}

// One wave routes one token from its n router logits z (global or LDS).  s = softmax(z) over all n outputs;
// choice = s + corr; the n outputs form `groups` equal runs of neighbours, a group's score is its largest choice and
// only the `keep` best groups stay eligible; the `top` largest eligible choices are taken and weighted by s * scale
// (s without the correction, not renormalised).
__device__ __forceinline__ void route_wave(const float* z, const float* __restrict__ corr, int* __restrict__ idx,
                                           float* __restrict__ wout, int lane, int n, int top, int groups, int keep,
                                           float scale, int kind) {
  float s[RPL], ch[RPL];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int e = lane + 64 * i;
    // a row nobody reads (an idle decode row) may carry anything, NaN included: it still gets ids inside [0, n)
    s[i] = e < n ? (isfinite(z[e]) ? z[e] : 0.f) : -INFINITY;
    mx = fmaxf(mx, s[i]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    if (kind & 1)
      s[i] = lane + 64 * i < n ? sigmoidf_(s[i]) : 0.f;
    else
      s[i] = lane + 64 * i < n ? expf(s[i] - mx) : 0.f;
    sum += s[i];
  }
  sum = (kind & 1) ? 1.f : wave_sum(sum);
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int e = lane + 64 * i;
    s[i] /= sum;
    ch[i] = e < n ? s[i] + (corr != nullptr ? corr[e] : 0.f) : -INFINITY;
  }
  if (groups > 1 && keep < groups && (kind & 2)) {
    // rank of group g = its largest choice + its second largest (a group of one: the one), held by lane g
    const int gs = n / groups;
    float rank = -INFINITY;
    for (int g = 0; g < groups; ++g) {
      float b1 = -INFINITY;
      int e1 = 1 << 30;
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        const int e = lane + 64 * i;
        if (e < n && e / gs == g && (ch[i] > b1 || (ch[i] == b1 && e < e1))) {
          b1 = ch[i];
          e1 = e;
        }
      }
      wave_argmax(b1, e1);
      float b2 = -INFINITY;
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        const int e = lane + 64 * i;
        if (e < n && e / gs == g && e != e1) b2 = fmaxf(b2, ch[i]);
      }
      b2 = wave_max(b2);
      if (lane == g) rank = b1 + (b2 == -INFINITY ? 0.f : b2);
    }
    unsigned long long kept = 0ull;               // groups <= 64
    for (int r = 0; r < keep; ++r) {
      float bv = rank;
      int bg = lane < groups ? lane : 1 << 30;
      wave_argmax(bv, bg);
      if (bg < groups) kept |= 1ull << bg;
      if (lane == bg) rank = -INFINITY;
    }
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      const int e = lane + 64 * i;
      if (e < n && !((kept >> (e / gs)) & 1ull)) ch[i] = -INFINITY;
    }
  } else if (groups > 1 && keep < groups) {
    const int gs = n / groups;
    // a lane's outputs may lie in different groups: the kept-group mask is built by `keep` rounds of
    // "best remaining group", each an argmax over (choice, group) pairs
    unsigned long long kept = 0ull;               // groups <= 64
    for (int r = 0; r < keep; ++r) {
      float bv = -INFINITY;
      int bg = 1 << 30;
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        const int e = lane + 64 * i, g = e / gs;
        if (e < n && !((kept >> g) & 1ull) && (ch[i] > bv || (ch[i] == bv && g < bg))) {
          bv = ch[i];
          bg = g;
        }
      }
      wave_argmax(bv, bg);
      if (bg < groups) kept |= 1ull << bg;
    }
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      const int e = lane + 64 * i;
      if (e < n && !((kept >> (e / gs)) & 1ull)) ch[i] = -INFINITY;
    }
  }
  unsigned taken = 0u;                            // bit i: this lane's output i is already chosen
  float tot = 0.f, myw = 0.f;                     // lane r keeps the r-th choice (top <= 64)
  int myid = 0;
  for (int r = 0; r < top; ++r) {
    float bv = -INFINITY;
    int be = 1 << 30;
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      const int e = lane + 64 * i;
      if (e < n && !((taken >> i) & 1u) && (ch[i] > bv || (ch[i] == bv && e < be))) {
        bv = ch[i];
        be = e;
      }
    }
    wave_argmax(bv, be);
    be = min(be, n - 1);                          // (only when fewer than `top` outputs are eligible)
    float cand = 0.f;
#pragma unroll
    for (int i = 0; i < RPL; ++i)
      if (i == (be >> 6)) cand = s[i];
    const float bs = __shfl(cand, be & 63, 64);
    if ((be & 63) == lane) taken |= 1u << (be >> 6);
    tot += bs;
    if (lane == r) {
      myw = bs;
      myid = be;
    }
  }
  if (lane < top) {
    idx[lane] = myid;
    wout[lane] = ((kind & 4) ? myw / (tot + 1e-20f) : myw) * scale;
  }
}

// routing from given logits: one wave per token
__global__ __launch_bounds__(256) void k_route_grouped(const float* __restrict__ z, const float* __restrict__ corr,
                                                       int* __restrict__ idx, float* __restrict__ wout, int T_, int n,
                                                       int top, int groups, int keep, float scale, int kind) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= T_) return;
  route_wave(z + (size_t)t * n, corr, idx + (size_t)t * top, wout + (size_t)t * top, lane, n, top, groups, keep, scale,
             kind);
}

// four entries of an activation row as floats (16-byte rows when the width allows)
__device__ __forceinline__ f32x4 load4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ f32x4 load4(const bf16* p) {
  const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
  return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}

// router product and routing in one kernel: one block of NW waves per token (16 for the few tokens of a decode step,
// so that its few blocks have many loads in flight; 4 for prompts).  A work item is (four router rows, one interleaved
// quarter of the columns): four independent accumulators over 16-byte loads; float weights, activations as they are,
// float accumulation.  Partial sums meet in LDS, then wave 0 routes.
template <typename T, int NW>
__global__ __launch_bounds__(64 * NW) void k_route_fused(const T* __restrict__ h, int ldh, const float* __restrict__ router,
                                                      const float* __restrict__ corr, int* __restrict__ idx,
                                                      float* __restrict__ wout, int n, int W, int top, int groups,
                                                      int keep, float scale, int kind, int extra,
                                                      float* __restrict__ xout) {
  // n counts all router rows; the last `extra` of them are not routed: their products go to xout [T, extra]
  __shared__ float part[64 * RPL][4];
  __shared__ float sz[64 * RPL];
  const int t = blockIdx.x, wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* x = h + (size_t)t * ldh;
  const bool vec = (W & 3) == 0 && (ldh & 3) == 0;
  const int items = ((n + 3) / 4) * 4;
  for (int it = wv; it < items; it += NW) {
    const int e0 = 4 * (it >> 2), qt = it & 3;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    const float* r[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = router + (size_t)min(e0 + i, n - 1) * W;
    if (vec) {
#pragma unroll 2
      for (int c = 4 * lane + 256 * qt; c < W; c += 1024) {
        const f32x4 xv = load4(x + c);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const f32x4 rv = load4(r[i] + c);
          acc[i] += rv[0] * xv[0] + rv[1] * xv[1] + rv[2] * xv[2] + rv[3] * xv[3];
        }
      }
    } else {
      for (int c = lane + 64 * qt; c < W; c += 256) {
        const float xv = (float)x[c];
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] += r[i][c] * xv;
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float v = wave_sum(acc[i]);
      if (lane == 0 && e0 + i < n) part[e0 + i][qt] = v;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n; e += 64 * NW) sz[e] = (part[e][0] + part[e][1]) + (part[e][2] + part[e][3]);
  __syncthreads();
  for (int e = threadIdx.x; e < extra; e += 64 * NW) xout[(size_t)t * extra + e] = sz[n - extra + e];
  if (wv == 0)
    route_wave(sz, corr, idx + (size_t)t * top, wout + (size_t)t * top, lane, n - extra, top, groups, keep, scale, kind);
}

// g = min(g, limit), u = clamp(u, -limit, limit): g * sigmoid(1.702 g) * (u + 1)
__device__ __forceinline__ float clipped_glu(float g, float u, float limit) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g * sigmoidf_(1.702f * g) * (u + 1.f);
}

// mode 1: the clipped GLU; mode 2: silu(g) * u; mode 3: gelu_tanh(g) * u
__device__ __forceinline__ float glu(float g, float u, float limit, int mode) {
  if (mode == 3) return gelu_tanhf_(g) * u;
  return mode == 2 ? g * sigmoidf_(g) * u : clipped_glu(g, u, limit);
}

template <typename T>
__device__ __forceinline__ float wave_dot(const T* __restrict__ a, const T* __restrict__ b, int n, int lane);

template <>
__device__ __forceinline__ float wave_dot<float>(const float* __restrict__ a, const float* __restrict__ b, int n,
                                                 int lane) {
  float acc = 0.f;
  if ((n & 3) == 0) {
    for (int c = 4 * lane; c < n; c += 256) {
      const f32x4 x = *reinterpret_cast<const f32x4*>(a + c), y = *reinterpret_cast<const f32x4*>(b + c);
      acc += x[0] * y[0] + x[1] * y[1] + x[2] * y[2] + x[3] * y[3];
    }
  } else {
    for (int c = lane; c < n; c += 64) acc += a[c] * b[c];
  }
  return wave_sum(acc);
}
template <>
__device__ __forceinline__ float wave_dot<bf16>(const bf16* __restrict__ a, const bf16* __restrict__ b, int n, int lane) {
  float acc = 0.f;
  if ((n & 7) == 0) {
    for (int c = 8 * lane; c < n; c += 512) {
      const bf16x8 x = *reinterpret_cast<const bf16x8*>(a + c), y = *reinterpret_cast<const bf16x8*>(b + c);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc += (float)x[j] * (float)y[j];
    }
  } else {
    for (int c = lane; c < n; c += 64) acc += (float)a[c] * (float)b[c];
  }
  return wave_sum(acc);
}

// pairs path, stage 1.  One wave per (pair, hidden unit r): a[pair, r] = glu(Wg_e[r] . h_t, Wu_e[r] . h_t).
// wgu: [E, 2, F, W] (gate rows then up rows of every expert).  Identity pairs (e >= E) have nothing to compute.
template <typename T>
__global__ __launch_bounds__(256) void k_moe_pair_up(const T* __restrict__ h, int ldh, const T* __restrict__ wgu,
                                                     const int* __restrict__ idx, T* __restrict__ a, int npairs, int top,
                                                     int E, int F, int W, float limit, int mode) {
  const int pair = blockIdx.x, r = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int e = idx[pair];
  if (r >= F || e < 0 || e >= E) return;
  const T* x = h + (size_t)(pair / top) * ldh;
  const T* wg = wgu + ((size_t)e * 2 * F + r) * W;
  const float g = wave_dot<T>(wg, x, W, lane), u = wave_dot<T>(wg + (size_t)F * W, x, W, lane);
  if (lane == 0) a[(size_t)pair * F + r] = (T)glu(g, u, limit, mode);
}

// pairs path, stage 2.  One wave per (token, output column c):
// out[t, c] = sum_j w[t, j] * (e_j < E ? Wd_e[c] . a[t, j] : h[t, c]) + shared[t, c]
template <typename T>
__global__ __launch_bounds__(256) void k_moe_pair_down(const T* __restrict__ a, const T* __restrict__ wd,
                                                       const int* __restrict__ idx, const float* __restrict__ wts,
                                                       const T* __restrict__ h, int ldh, const T* __restrict__ shared,
                                                       const float* __restrict__ sgate, float* __restrict__ out, int top,
                                                       int E, int F, int W) {
  const int t = blockIdx.x, c = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (c >= W) return;
  float acc = shared != nullptr ? (float)shared[(size_t)t * W + c] * (sgate != nullptr ? sigmoidf_(sgate[t]) : 1.f) : 0.f;
  for (int j = 0; j < top; ++j) {
    const int e = idx[(size_t)t * top + j];
    const float w = wts[(size_t)t * top + j];
    if (e >= E)
      acc += w * (float)h[(size_t)t * ldh + c];
    else if (e >= 0)
      acc += w * wave_dot<T>(wd + ((size_t)e * W + c) * F, a + ((size_t)t * top + j) * F, F, lane);
  }
  if (lane == 0) out[(size_t)t * W + c] = acc;
}

// sorted path: out[t, c] = sum_j w[t, j] * (e_j < E ? ys[pos[t, j], c] : h[t, c]) + shared[t, c]
template <typename T>
__global__ __launch_bounds__(256) void k_moe_combine(const T* __restrict__ ys, const long* __restrict__ pos,
                                                     const int* __restrict__ idx, const float* __restrict__ wts,
                                                     const T* __restrict__ h, int ldh, const T* __restrict__ shared,
                                                     const float* __restrict__ sgate, float* __restrict__ out, int top,
                                                     int E, int W) {
  const size_t t = blockIdx.x;
  const float sg = sgate != nullptr ? sigmoidf_(sgate[t]) : 1.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    float acc = shared != nullptr ? (float)shared[t * W + c] * sg : 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = idx[t * top + j];
      const float w = wts[t * top + j];
      if (e >= 0) acc += w * (e >= E ? (float)h[t * ldh + c] : (float)ys[(size_t)pos[t * top + j] * W + c]);
    }
    out[t * W + c] = acc;
  }
}

// feed-forward activations on a GEMM output: mode 0 tanh-form GELU of z [T, F]; mode 1 clipped GLU, mode 2 SiLU GLU,
// mode 3 tanh-form GELU GLU of the [gate | up] halves of z [T, 2F]
template <typename T>
__global__ __launch_bounds__(256) void k_ff_act(const T* __restrict__ z, T* __restrict__ out, size_t n, int F, int mode,
                                                float limit) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  if (mode == 0) {
    const float v = (float)z[i];
    out[i] = (T)gelu_tanhf_(v);
  } else {
    const size_t t = i / F, c = i % F;
    out[i] = (T)glu((float)z[t * 2 * F + c], (float)z[t * 2 * F + F + c], limit, mode);
  }
}

int seq_route_max_outputs() { return 64 * RPL; }

void seq_route_grouped(const float* z, const float* corr, int* idx, float* w, int T_, int n, int top, int groups,
                       int keep, float scale, int kind, hipStream_t st) {
  if (T_ == 0) return;
  hipLaunchKernelGGL(k_route_grouped, dim3((T_ + 3) / 4), dim3(256), 0, st, z, corr, idx, w, T_, n, top, groups, keep,
                     scale, kind);
  LIPA_CHECK_LAUNCH();
}

void seq_route_fused(int code, const void* h, int ldh, const float* router, const float* corr, int* idx, float* w,
                     int T_, int n, int W, int top, int groups, int keep, float scale, int kind, int extra, float* xout,
                     hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, {
    if (T_ < 256)
      hipLaunchKernelGGL((k_route_fused<T, 16>), dim3(T_), dim3(1024), 0, st, (const T*)h, ldh, router, corr, idx, w, n,
                         W, top, groups, keep, scale, kind, extra, xout);
    else
      hipLaunchKernelGGL((k_route_fused<T, 4>), dim3(T_), dim3(256), 0, st, (const T*)h, ldh, router, corr, idx, w, n, W,
                         top, groups, keep, scale, kind, extra, xout);
  });
  LIPA_CHECK_LAUNCH();
}

void seq_moe_pairs(int code, const void* h, int ldh, const void* wgu, const void* wd, const int* idx, const float* wts,
                   const void* shared, const float* sgate, void* a, float* out, int T_, int top, int E, int F, int W,
                   float limit, int mode, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, {
    hipLaunchKernelGGL(k_moe_pair_up<T>, dim3(T_ * top, (F + 3) / 4), dim3(256), 0, st, (const T*)h, ldh, (const T*)wgu,
                       idx, (T*)a, T_ * top, top, E, F, W, limit, mode);
    hipLaunchKernelGGL(k_moe_pair_down<T>, dim3(T_, (W + 3) / 4), dim3(256), 0, st, (const T*)a, (const T*)wd, idx, wts,
                       (const T*)h, ldh, (const T*)shared, sgate, out, top, E, F, W);
  });
  LIPA_CHECK_LAUNCH();
}

void seq_moe_combine(int code, const void* ys, const long* pos, const int* idx, const float* wts, const void* h, int ldh,
                     const void* shared, const float* sgate, float* out, int T_, int top, int E, int W, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_moe_combine<T>, dim3(T_), dim3(256), 0, st, (const T*)ys, pos, idx, wts,
                                          (const T*)h, ldh, (const T*)shared, sgate, out, top, E, W));
  LIPA_CHECK_LAUNCH();
}

void seq_ff_act(int code, const void* z, void* out, int T_, int F, int mode, float limit, hipStream_t st) {
  const size_t n = (size_t)T_ * F;
  if (n == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_ff_act<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, (const T*)z,
                                          (T*)out, n, F, mode, limit));
  LIPA_CHECK_LAUNCH();
}
