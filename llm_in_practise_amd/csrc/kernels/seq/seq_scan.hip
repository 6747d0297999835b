// Short causal convolutions with carried inputs, and the matrix-memory recurrences (mLSTM with a running maximum;
// gated delta rule with a per-channel decay; selective state space with a scalar decay per head), over packed
// variable-length sequences with per-slot state.
//
// Recurrences: every column of the state matrix S[dk, dv] evolves on its own given the step's k, q and gates, so a
// block owns one (sequence, head) and 256/R columns; a column's dk rows are spread over R adjacent lanes (R a power
// of two <= 16, a template parameter; 16 contiguous rows per lane) and live in registers for the whole scan.  Dot
// products over dk run as four independent partial sums per lane and are finished with constant-mask xor-shuffles
// inside the R-lane group: no barrier per token.  The step inputs of 16 tokens at a time are staged through LDS as
// float rows of 16*R entries, zero-padded past dk (a padded row never changes: k = 0), and read back as 16-byte
// vectors.  One token is the decode step: load state, one update, store.  State layout in HBM: S [slots, H, dv, dk],
// float.
#include "seq_common.h"

using namespace lipa;

constexpr int KR = 16;      // state rows per lane
constexpr int CT = 16;      // tokens staged per chunk
constexpr int MAXHW = 8;    // conv: head width <= 64 * MAXHW
constexpr int MAXTAPS = 8;

struct ConvSeg {
  int c0, nheads, hw, mode;   // mode 0: plain, 1: rms norm * w, 2: silu, 3: silu then unit vector * scale
  const float* w;
  float scale;
};
struct ConvArgs {
  ConvSeg seg[3];
  int nseg;
};

template <typename T>
__device__ __forceinline__ float conv_at(const T* __restrict__ u, int ldu, const T* __restrict__ state, int C, int taps,
                                         const float* __restrict__ w, int t, int j, int p0, int slot, int ch) {
  float acc = 0.f;
  for (int jj = 0; jj < taps; ++jj) {
    const int src = j - (taps - 1) + jj;
    float uv = 0.f;
    if (src >= 0)
      uv = (float)u[(size_t)(t - (taps - 1) + jj) * ldu + ch];
    else if (p0 > 0)
      uv = (float)state[((size_t)slot * (taps - 1) + (taps - 1 + src)) * C + ch];
    acc += w[(size_t)ch * taps + jj] * uv;
  }
  return acc;
}

// one wave per (token, head): convolution over time, then the head's activation / norm
template <typename T, typename OT>
__global__ __launch_bounds__(64) void k_short_conv(const T* __restrict__ u, int ldu, const float* __restrict__ w,
                                                   const float* __restrict__ bias, const T* __restrict__ state,
                                                   OT* __restrict__ out, int C, int taps, ConvArgs a, SeqDesc d,
                                                   float eps) {
  const int t = blockIdx.x, lane = threadIdx.x;
  int hl = blockIdx.y, si = 0;
  while (si < a.nseg - 1 && hl >= a.seg[si].nheads) hl -= a.seg[si++].nheads;
  const ConvSeg sg = a.seg[si];
  const int s = d.tok_seq[t], j = t - d.seq_off[s], p0 = d.pos0[s], slot = d.slots[s];
  const int cbase = sg.c0 + hl * sg.hw;
  float vals[MAXHW];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < MAXHW; ++i) {
    const int c = lane + 64 * i;
    vals[i] = 0.f;
    if (c < sg.hw) {
      float acc = conv_at(u, ldu, state, C, taps, w, t, j, p0, slot, cbase + c);
      if (bias != nullptr) acc += bias[cbase + c];
      if (sg.mode >= 2) acc = acc * sigmoidf_(acc);
      vals[i] = acc;
      ss += acc * acc;
    }
  }
  float mul = 1.f;
  if (sg.mode == 1) mul = rsqrtf(wave_sum(ss) / sg.hw + eps);
  if (sg.mode == 3) mul = rsqrtf(wave_sum(ss) + 1e-6f) * sg.scale;
#pragma unroll
  for (int i = 0; i < MAXHW; ++i) {
    const int c = lane + 64 * i;
    if (c < sg.hw) {
      float v = vals[i] * mul;
      if (sg.mode == 1) v *= sg.w[c];
      out[(size_t)t * C + cbase + c] = (OT)v;
    }
  }
}

// the last taps-1 inputs of every sequence become its carried state (older ones shift out)
template <typename T>
__global__ __launch_bounds__(256) void k_conv_state(const T* __restrict__ u, int ldu, T* __restrict__ state, int C,
                                                    int taps, SeqDesc d) {
  const int s = blockIdx.x, ch = blockIdx.y * 256 + threadIdx.x;
  if (ch >= C || (d.live && !d.live[s])) return;
  const int t0 = d.seq_off[s], len = d.seq_off[s + 1] - t0, p0 = d.pos0[s], slot = d.slots[s];
  float nv[MAXTAPS];
#pragma unroll
  for (int i = 0; i < MAXTAPS; ++i) {
    nv[i] = 0.f;
    if (i < taps - 1) {
      const int li = len - (taps - 1) + i;
      if (li >= 0)
        nv[i] = (float)u[(size_t)(t0 + li) * ldu + ch];
      else if (p0 > 0)
        nv[i] = (float)state[((size_t)slot * (taps - 1) + (taps - 1 + li)) * C + ch];
    }
  }
#pragma unroll
  for (int i = 0; i < MAXTAPS; ++i)
    if (i < taps - 1) state[((size_t)slot * (taps - 1) + i) * C + ch] = (T)nv[i];
}

// sum over the R adjacent lanes of a group (R <= 16, groups aligned inside a 16-lane row) with data-parallel
// primitives only: swap inside pairs, swap pairs inside quads, mirror the half row, mirror the row.  After each step
// every lane of the widened group holds the same partial sum, so a mirror pairs equal-valued halves.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int R>
__device__ __forceinline__ float group_sum(float v) {
  if (R >= 2) v = dpp_add<0xB1>(v);    // quad_perm [1, 0, 3, 2]
  if (R >= 4) v = dpp_add<0x4E>(v);    // quad_perm [2, 3, 0, 1]
  if (R >= 8) v = dpp_add<0x141>(v);   // row_half_mirror
  if (R >= 16) v = dpp_add<0x140>(v);  // row_mirror
  return v;
}

// a lane's 16 contiguous state rows: 16-byte accesses when the row length allows
__device__ __forceinline__ void load_rows(const float* p, int r0, int dk, bool on, float (&r)[KR]) {
  if (on && (dk & 3) == 0) {
#pragma unroll
    for (int i4 = 0; i4 < KR / 4; ++i4) {
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (r0 + 4 * i4 < dk) v = *reinterpret_cast<const f32x4*>(p + r0 + 4 * i4);
      r[4 * i4] = v[0]; r[4 * i4 + 1] = v[1]; r[4 * i4 + 2] = v[2]; r[4 * i4 + 3] = v[3];
    }
  } else {
#pragma unroll
    for (int i = 0; i < KR; ++i) r[i] = (on && r0 + i < dk) ? p[r0 + i] : 0.f;
  }
}
__device__ __forceinline__ void store_rows(float* p, int r0, int dk, const float (&r)[KR]) {
  if ((dk & 3) == 0) {
#pragma unroll
    for (int i4 = 0; i4 < KR / 4; ++i4)
      if (r0 + 4 * i4 < dk)
        *reinterpret_cast<f32x4*>(p + r0 + 4 * i4) = f32x4{r[4 * i4], r[4 * i4 + 1], r[4 * i4 + 2], r[4 * i4 + 3]};
  } else {
#pragma unroll
    for (int i = 0; i < KR; ++i)
      if (r0 + i < dk) p[r0 + i] = r[i];
  }
}

// Staging of a chunk of CT tokens goes through registers: fetch_rows issues all of a lane's loads back to back (one
// latency, and the next chunk's loads fly while the current chunk is computed), commit_rows writes them to LDS rows
// of DKP = 16 R floats (`pad` past dk).  CT * DKP / 256 = R elements per lane.
template <typename T, int R>
__device__ __forceinline__ void fetch_rows(float (&v)[R], const T* __restrict__ src, size_t ld, int col0, int dk, int n,
                                           float mul, float pad) {
  constexpr int DKP = KR * R;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int e = threadIdx.x + 256 * i, tt = e / DKP, r = e % DKP;
    v[i] = (tt < n && r < dk) ? (float)src[(size_t)tt * ld + col0 + r] * mul : pad;
  }
}
template <int R>
__device__ __forceinline__ void commit_rows(float* dst, const float (&v)[R]) {
#pragma unroll
  for (int i = 0; i < R; ++i) dst[threadIdx.x + 256 * i] = v[i];
}
// the chunk's value columns of this block: CT * NC / 256 = 16 / R elements per lane (at least one)
// (ones: column dv reads as 1 — the mLSTM's normaliser vector is the state column whose value is always 1)
template <typename T, int R>
__device__ __forceinline__ void fetch_cols(float (&v)[(16 + R - 1) / R], const T* __restrict__ src, size_t ld, int col0,
                                           int cb, int dv, int n, bool ones = false) {
  constexpr int NC = 256 / R, PER = (16 + R - 1) / R;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = threadIdx.x + 256 * i, tt = e / NC, cc = cb * NC + e % NC;
    v[i] = (e < CT * NC && tt < n && cc < dv) ? (float)src[(size_t)tt * ld + col0 + cc] : (ones && cc == dv ? 1.f : 0.f);
  }
}
template <int R>
__device__ __forceinline__ void commit_cols(float* dst, const float (&v)[(16 + R - 1) / R]) {
  constexpr int NC = 256 / R, PER = (16 + R - 1) / R;
#pragma unroll
  for (int i = 0; i < PER; ++i)
    if (threadIdx.x + 256 * i < CT * NC) dst[threadIdx.x + 256 * i] = v[i];
}

// mLSTM.  m_t = max(f + m, i); S = e^(f+m-m_t) S + e^(i-m_t) k v^T; n likewise; o = S^T q / (max(|n.q|, e^-m_t) + 1e-6)
// with i = cap tanh((ipre + ib) / cap), f = logsigmoid(cap tanh((fpre + fb) / cap)); m starts at 0.
// The normaliser n obeys S's recurrence with v = 1, so it runs as column dv of the same scan; the kernel writes the
// numerators S^T q, and per (token, head) the normaliser product n.q and the floor e^-m; the read-out kernel divides.
template <typename T, int R>
__global__ __launch_bounds__(256) void k_mlstm_scan(const T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk,
                                                    const T* __restrict__ v, int ldv, const float* __restrict__ ipre,
                                                    const float* __restrict__ fpre, const float* __restrict__ ib,
                                                    const float* __restrict__ fb, float cap, float qscale,
                                                    float* __restrict__ S, float* __restrict__ N, float* __restrict__ M,
                                                    float* __restrict__ out, float* __restrict__ den,
                                                    float* __restrict__ efl, int H, int dk, int dv, SeqDesc d) {
  constexpr int DKP = KR * R, NC = 256 / R;
  __shared__ __attribute__((aligned(16))) float sk[CT * DKP];
  __shared__ __attribute__((aligned(16))) float sq[CT * DKP];
  __shared__ float sv[CT * NC];
  __shared__ float sg[4 * CT];
  const int s = blockIdx.x / H, hd = blockIdx.x % H, cb = blockIdx.y, tid = threadIdx.x;
  if (d.live && !d.live[s]) return;
  const int rg = tid % R, cl = tid / R, col = cb * NC + cl, r0 = rg * KR;
  const bool colok = col <= dv, isn = col == dv;          // column dv is the normaliser
  const int t0 = d.seq_off[s], t1 = d.seq_off[s + 1], p0 = d.pos0[s], slot = d.slots[s];
  const size_t hbase = (size_t)slot * H + hd;
  float* Sp = isn ? N + hbase * dk : S + (hbase * dv + (colok ? col : 0)) * dk;
  float Sr[KR];
  float m = p0 > 0 ? M[hbase] : 0.f;
  load_rows(Sp, r0, dk, p0 > 0 && colok, Sr);
  float fk[R], fq[R], fv[(16 + R - 1) / R], fi = 0.f, ff = 0.f;
  auto fetch = [&](int c0) {
    const int n = min(CT, t1 - c0);
    fetch_rows<T, R>(fk, k + (size_t)c0 * ldk, ldk, hd * dk, dk, n, 1.f, 0.f);
    fetch_rows<T, R>(fq, q + (size_t)c0 * ldq, ldq, hd * dk, dk, n, qscale, 0.f);
    fetch_cols<T, R>(fv, v + (size_t)c0 * ldv, ldv, hd * dv, cb, dv, n, true);
    if (tid < n) {
      fi = ipre[(size_t)(c0 + tid) * H + hd];
      ff = fpre[(size_t)(c0 + tid) * H + hd];
    }
  };
  if (t0 < t1) fetch(t0);
  for (int c0 = t0; c0 < t1; c0 += CT) {
    const int n = min(CT, t1 - c0);
    __syncthreads();
    commit_rows<R>(sk, fk);
    commit_rows<R>(sq, fq);
    commit_cols<R>(sv, fv);
    if (tid < CT) {
      // the running maximum is a (max, +) recurrence of the gates alone: with F_t the prefix sum of the log forget
      // gates, m_t = F_t + max(m_0, max_{s<=t}(i_s - F_s)).  Lanes 0..15 solve the chunk's 16 steps with two
      // 4-step prefix scans and hand every token its decay e^(f+m'-m), input weight e^(i-m) and floor e^(-m).
      const bool on = tid < n;
      const float ig = on ? cap * tanhf((fi + ib[hd]) / cap) : -INFINITY;
      const float fg = on ? logsigmoidf_(cap * tanhf((ff + fb[hd]) / cap)) : 0.f;
      float F = fg;
#pragma unroll
      for (int o = 1; o < CT; o <<= 1) {
        const float t = __shfl_up(F, o, CT);
        if (tid >= o) F += t;
      }
      float pm = ig - F;
#pragma unroll
      for (int o = 1; o < CT; o <<= 1) {
        const float t = __shfl_up(pm, o, CT);
        if (tid >= o) pm = fmaxf(pm, t);
      }
      const float mt = F + fmaxf(m, pm);
      float mp = __shfl_up(mt, 1, CT);
      if (tid == 0) mp = m;
      sg[4 * tid] = expf(fg + mp - mt);
      sg[4 * tid + 1] = expf(ig - mt);
      sg[4 * tid + 2] = expf(-mt);
      sg[4 * tid + 3] = mt;
      if (on && cb == 0) efl[(size_t)(c0 + tid) * H + hd] = expf(-mt);
    }
    __syncthreads();
    if (c0 + CT < t1) fetch(c0 + CT);
    for (int tt = 0; tt < n; ++tt) {
      const float a = sg[4 * tt], b = sg[4 * tt + 1];
      const float bv = b * sv[tt * NC + cl];
      float num[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i4 = 0; i4 < KR / 4; ++i4) {
        const f32x4 kk = *reinterpret_cast<const f32x4*>(sk + tt * DKP + r0 + 4 * i4);
        const f32x4 qq = *reinterpret_cast<const f32x4*>(sq + tt * DKP + r0 + 4 * i4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int i = 4 * i4 + j;
          Sr[i] = a * Sr[i] + kk[j] * bv;
          num[j] += Sr[i] * qq[j];
        }
      }
      const float nm = group_sum<R>((num[0] + num[1]) + (num[2] + num[3]));
      if (rg == 0 && colok) {
        if (isn)
          den[(size_t)(c0 + tt) * H + hd] = nm;
        else
          out[((size_t)(c0 + tt) * H + hd) * dv + col] = nm;
      }
    }
    m = sg[4 * (n - 1) + 3];
  }
  if (colok) store_rows(Sp, r0, dk, Sr);
  if (cb == 0 && tid == 0) M[hbase] = m;
}

// Gated delta rule.  S <- g * S (g per key channel); u = beta (v - S^T k); S <- S + k u^T; o = S^T q.
// beta = sigmoid(bpre); head hd reads q/k head hd / (H / G).
template <typename T, int R>
__global__ __launch_bounds__(256) void k_delta_scan(const T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk,
                                                    const T* __restrict__ v, int ldv, const float* __restrict__ g,
                                                    const float* __restrict__ bpre, float* __restrict__ S,
                                                    float* __restrict__ out, int H, int G, int dk, int dv, SeqDesc d) {
  constexpr int DKP = KR * R, NC = 256 / R;
  __shared__ __attribute__((aligned(16))) float sk[CT * DKP];
  __shared__ __attribute__((aligned(16))) float sq[CT * DKP];
  __shared__ __attribute__((aligned(16))) float sd[CT * DKP];
  __shared__ float sv[CT * NC];
  __shared__ float sb[CT];
  const int s = blockIdx.x / H, hd = blockIdx.x % H, cb = blockIdx.y, tid = threadIdx.x;
  if (d.live && !d.live[s]) return;
  const int rg = tid % R, cl = tid / R, col = cb * NC + cl, kh = hd / (H / G), r0 = rg * KR;
  const bool colok = col < dv;
  const int t0 = d.seq_off[s], t1 = d.seq_off[s + 1], p0 = d.pos0[s], slot = d.slots[s];
  float* Sp = S + (((size_t)slot * H + hd) * dv + (colok ? col : 0)) * dk;
  float Sr[KR];
  load_rows(Sp, r0, dk, p0 > 0 && colok, Sr);
  float fk[R], fq[R], fd[R], fv[(16 + R - 1) / R], fb = 0.f;
  auto fetch = [&](int c0) {
    const int n = min(CT, t1 - c0);
    fetch_rows<T, R>(fk, k + (size_t)c0 * ldk, ldk, kh * dk, dk, n, 1.f, 0.f);
    fetch_rows<T, R>(fq, q + (size_t)c0 * ldq, ldq, kh * dk, dk, n, 1.f, 0.f);
    fetch_rows<float, R>(fd, g + (size_t)c0 * H * dk, (size_t)H * dk, hd * dk, dk, n, 1.f, 1.f);
    fetch_cols<T, R>(fv, v + (size_t)c0 * ldv, ldv, hd * dv, cb, dv, n);
    if (tid < n) fb = bpre[(size_t)(c0 + tid) * H + hd];
  };
  if (t0 < t1) fetch(t0);
  for (int c0 = t0; c0 < t1; c0 += CT) {
    const int n = min(CT, t1 - c0);
    __syncthreads();
    commit_rows<R>(sk, fk);
    commit_rows<R>(sq, fq);
    commit_rows<R>(sd, fd);
    commit_cols<R>(sv, fv);
    if (tid < n) sb[tid] = sigmoidf_(fb);
    __syncthreads();
    if (c0 + CT < t1) fetch(c0 + CT);
    for (int tt = 0; tt < n; ++tt) {
      f32x4 kk[KR / 4];
      float dot[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i4 = 0; i4 < KR / 4; ++i4) {
        kk[i4] = *reinterpret_cast<const f32x4*>(sk + tt * DKP + r0 + 4 * i4);
        const f32x4 gd = *reinterpret_cast<const f32x4*>(sd + tt * DKP + r0 + 4 * i4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          Sr[4 * i4 + j] *= gd[j];
          dot[j] += Sr[4 * i4 + j] * kk[i4][j];
        }
      }
      const float u = sb[tt] * (sv[tt * NC + cl] - group_sum<R>((dot[0] + dot[1]) + (dot[2] + dot[3])));
      float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i4 = 0; i4 < KR / 4; ++i4) {
        const f32x4 qq = *reinterpret_cast<const f32x4*>(sq + tt * DKP + r0 + 4 * i4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          Sr[4 * i4 + j] += kk[i4][j] * u;
          o[j] += Sr[4 * i4 + j] * qq[j];
        }
      }
      const float ov = group_sum<R>((o[0] + o[1]) + (o[2] + o[3]));
      if (rg == 0 && colok) out[((size_t)(c0 + tt) * H + hd) * dv + col] = ov;
    }
  }
  if (colok) store_rows(Sp, r0, dk, Sr);
}

// Generalised delta rule.  With the unit key u = k / |k|: S <- diag(w) S - (a * u)(u^T S) + k v^T, both the decay and
// the removal reading the old S; o = S^T r.  Per column of S that is  e = kinv (k . s);  s <- w * s + k (v - a e)
// with kinv = 1 / (|k|^2 + 1e-6) per (token, head): one dot product, one update, one dot product per token.
// w, a float [T, H * dk], kinv float [T, H].  The four staged row arrays live in dynamic shared memory (81 KB at
// dk > 128).
// commit_rows with 4 floats of padding after every lane's 16 rows: the 16-byte reads of lanes rg and rg + 4 then fall
// into different banks (unpadded, their rows are 256 bytes apart: the same banks)
constexpr int KRP = KR + 4;
template <int R>
__device__ __forceinline__ void commit_rows_padded(float* dst, const float (&v)[R]) {
  constexpr int DKP = KR * R;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int e = threadIdx.x + 256 * i, tt = e / DKP, r = e % DKP;
    dst[tt * (KRP * R) + (r / KR) * KRP + (r % KR)] = v[i];
  }
}

template <typename T, int R>
__global__ __launch_bounds__(256) void k_gdr_scan(const T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk,
                                                  const T* __restrict__ v, int ldv, const float* __restrict__ w,
                                                  const float* __restrict__ a, const float* __restrict__ kinv,
                                                  float* __restrict__ S, float* __restrict__ out, int H, int dk, int dv,
                                                  SeqDesc d) {
  constexpr int DKP = KR * R, NC = 256 / R, LDR = KRP * R;       // LDR: floats of a staged token row, padded
  extern __shared__ __attribute__((aligned(16))) float gdr_smem[];
  float* sk = gdr_smem;
  float* sq = sk + CT * LDR;
  float* sd = sq + CT * LDR;
  float* sa = sd + CT * LDR;
  float* sv = sa + CT * LDR;          // [CT * NC]
  float* sb = sv + CT * NC;           // [CT]
  const int s = blockIdx.x / H, hd = blockIdx.x % H, cb = blockIdx.y, tid = threadIdx.x;
  if (d.live && !d.live[s]) return;
  const int rg = tid % R, cl = tid / R, col = cb * NC + cl, r0 = rg * KR, l0 = rg * KRP;
  const bool colok = col < dv;
  const int t0 = d.seq_off[s], t1 = d.seq_off[s + 1], p0 = d.pos0[s], slot = d.slots[s];
  float* Sp = S + (((size_t)slot * H + hd) * dv + (colok ? col : 0)) * dk;
  float Sr[KR];
  load_rows(Sp, r0, dk, p0 > 0 && colok, Sr);
  float fk[R], fq[R], fd[R], fa[R], fv[(16 + R - 1) / R], fb = 0.f;
  auto fetch = [&](int c0) {
    const int n = min(CT, t1 - c0);
    fetch_rows<T, R>(fk, k + (size_t)c0 * ldk, ldk, hd * dk, dk, n, 1.f, 0.f);
    fetch_rows<T, R>(fq, q + (size_t)c0 * ldq, ldq, hd * dk, dk, n, 1.f, 0.f);
    fetch_rows<float, R>(fd, w + (size_t)c0 * H * dk, (size_t)H * dk, hd * dk, dk, n, 1.f, 1.f);
    fetch_rows<float, R>(fa, a + (size_t)c0 * H * dk, (size_t)H * dk, hd * dk, dk, n, 1.f, 0.f);
    fetch_cols<T, R>(fv, v + (size_t)c0 * ldv, ldv, hd * dv, cb, dv, n);
    if (tid < n) fb = kinv[(size_t)(c0 + tid) * H + hd];
  };
  if (t0 < t1) fetch(t0);
  for (int c0 = t0; c0 < t1; c0 += CT) {
    const int n = min(CT, t1 - c0);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < R; ++i) fa[i] *= fk[i];          // staged as k * a: the update is then two fused steps
    commit_rows_padded<R>(sk, fk);
    commit_rows_padded<R>(sq, fq);
    commit_rows_padded<R>(sd, fd);
    commit_rows_padded<R>(sa, fa);
    commit_cols<R>(sv, fv);
    if (tid < n) sb[tid] = fb;
    __syncthreads();
    if (c0 + CT < t1) fetch(c0 + CT);
    // the dot product k . s of a token runs in the same sweep as the read-out of the token before it (both read the
    // new s), so only the chunk's first token needs a sweep of its own.  The scan is bound by the bytes its LDS reads
    // move: a token's key is read once (as the next key of the token before it) and kept in registers; the loop runs
    // two tokens per turn so that the two register sets swap roles without copies.
    f32x4 ka_[KR / 4], kb_[KR / 4];
    float dot[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i4 = 0; i4 < KR / 4; ++i4) {
      ka_[i4] = *reinterpret_cast<const f32x4*>(sk + l0 + 4 * i4);
#pragma unroll
      for (int j = 0; j < 4; ++j) dot[j] += Sr[4 * i4 + j] * ka_[i4][j];
    }
    auto step = [&](int tt, const f32x4 (&kk)[KR / 4], f32x4 (&kn)[KR / 4]) {
      const int tn = min(tt + 1, n - 1);
      const float e = sb[tt] * group_sum<R>((dot[0] + dot[1]) + (dot[2] + dot[3]));
      const float vv = sv[tt * NC + cl];
      float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; ++j) dot[j] = 0.f;
#pragma unroll
      for (int i4 = 0; i4 < KR / 4; ++i4) {
        const f32x4 wd = *reinterpret_cast<const f32x4*>(sd + tt * LDR + l0 + 4 * i4);
        const f32x4 ka = *reinterpret_cast<const f32x4*>(sa + tt * LDR + l0 + 4 * i4);
        const f32x4 qq = *reinterpret_cast<const f32x4*>(sq + tt * LDR + l0 + 4 * i4);
        kn[i4] = *reinterpret_cast<const f32x4*>(sk + tn * LDR + l0 + 4 * i4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float sn = (wd[j] * Sr[4 * i4 + j] + kk[i4][j] * vv) - ka[j] * e;
          Sr[4 * i4 + j] = sn;
          o[j] += sn * qq[j];
          dot[j] += sn * kn[i4][j];
        }
      }
      const float ov = group_sum<R>((o[0] + o[1]) + (o[2] + o[3]));
      if (rg == 0 && colok) out[((size_t)(c0 + tt) * H + hd) * dv + col] = ov;
    };
    int tt = 0;
    for (; tt + 1 < n; tt += 2) {
      step(tt, ka_, kb_);
      step(tt + 1, kb_, ka_);
    }
    if (tt < n) step(tt, ka_, kb_);
  }
  if (colok) store_rows(Sp, r0, dk, Sr);
}

// State-space duality form of a selective state space (Mamba-2): per head a scalar decay and step size,
// dt = softplus(dtraw + dt_bias), S <- exp(-exp(A_log) dt) S + B (dt x)^T, y = S^T C + D x.  S is [N, P] per head, held
// as [P, N] rows like the other recurrences (key size N = dk, value size P = dv); head hd reads B and C of group
// hd / (H / G).  The step size and decay of a chunk's tokens are computed in float by the chunk's first lanes.
template <typename T, int R>
__global__ __launch_bounds__(256) void k_ssd_scan(const T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk,
                                                  const T* __restrict__ v, int ldv, const T* __restrict__ dtraw, int lddt,
                                                  const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                                                  const float* __restrict__ dskip, float* __restrict__ S,
                                                  float* __restrict__ out, int H, int G, int dk, int dv, SeqDesc d) {
  constexpr int DKP = KR * R, NC = 256 / R;
  __shared__ __attribute__((aligned(16))) float sk[CT * DKP];
  __shared__ __attribute__((aligned(16))) float sq[CT * DKP];
  __shared__ float sv[CT * NC];
  __shared__ float sg[2 * CT];
  const int s = blockIdx.x / H, hd = blockIdx.x % H, cb = blockIdx.y, tid = threadIdx.x;
  if (d.live && !d.live[s]) return;
  const int rg = tid % R, cl = tid / R, col = cb * NC + cl, kh = hd / (H / G), r0 = rg * KR;
  const bool colok = col < dv;
  const int t0 = d.seq_off[s], t1 = d.seq_off[s + 1], p0 = d.pos0[s], slot = d.slots[s];
  float* Sp = S + (((size_t)slot * H + hd) * dv + (colok ? col : 0)) * dk;
  float Sr[KR];
  load_rows(Sp, r0, dk, p0 > 0 && colok, Sr);
  const float rate = expf(a_log[hd]), bias = dt_bias[hd], skip = dskip[hd];
  float fk[R], fq[R], fv[(16 + R - 1) / R], fdt = 0.f;
  auto fetch = [&](int c0) {
    const int n = min(CT, t1 - c0);
    fetch_rows<T, R>(fk, k + (size_t)c0 * ldk, ldk, kh * dk, dk, n, 1.f, 0.f);
    fetch_rows<T, R>(fq, q + (size_t)c0 * ldq, ldq, kh * dk, dk, n, 1.f, 0.f);
    fetch_cols<T, R>(fv, v + (size_t)c0 * ldv, ldv, hd * dv, cb, dv, n);
    if (tid < n) fdt = (float)dtraw[(size_t)(c0 + tid) * lddt + hd];
  };
  if (t0 < t1) fetch(t0);
  for (int c0 = t0; c0 < t1; c0 += CT) {
    const int n = min(CT, t1 - c0);
    __syncthreads();
    commit_rows<R>(sk, fk);
    commit_rows<R>(sq, fq);
    commit_cols<R>(sv, fv);
    if (tid < n) {
      const float dt = softplusf_(fdt + bias);
      sg[2 * tid] = expf(-rate * dt);
      sg[2 * tid + 1] = dt;
    }
    __syncthreads();
    if (c0 + CT < t1) fetch(c0 + CT);
    for (int tt = 0; tt < n; ++tt) {
      const float a = sg[2 * tt], xv = sv[tt * NC + cl], bv = sg[2 * tt + 1] * xv;
      float num[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i4 = 0; i4 < KR / 4; ++i4) {
        const f32x4 kk = *reinterpret_cast<const f32x4*>(sk + tt * DKP + r0 + 4 * i4);
        const f32x4 qq = *reinterpret_cast<const f32x4*>(sq + tt * DKP + r0 + 4 * i4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int i = 4 * i4 + j;
          Sr[i] = a * Sr[i] + kk[j] * bv;
          num[j] += Sr[i] * qq[j];
        }
      }
      const float y = group_sum<R>((num[0] + num[1]) + (num[2] + num[3]));
      if (rg == 0 && colok) out[((size_t)(c0 + tt) * H + hd) * dv + col] = y + skip * xv;
    }
  }
  if (colok) store_rows(Sp, r0, dk, Sr);
}

// ---------------------------------------------------------------------------------------------- launchers
static int rows_split(int dk) {
  int R = 1;
  while (R * KR < dk) R <<= 1;
  return R;
}

int seq_scan_max_dk() { return KR * 16; }
int seq_conv_max_head() { return 64 * MAXHW; }
int seq_conv_max_taps() { return MAXTAPS; }

#define SEQ_DISPATCH_R(R_, ...)                          \
  switch (R_) {                                          \
    case 1: { constexpr int R = 1; __VA_ARGS__; } break; \
    case 2: { constexpr int R = 2; __VA_ARGS__; } break; \
    case 4: { constexpr int R = 4; __VA_ARGS__; } break; \
    case 8: { constexpr int R = 8; __VA_ARGS__; } break; \
    default: { constexpr int R = 16; __VA_ARGS__; } break; \
  }

// segs: nseg x {c0, nheads, hw, mode}; sw: nseg norm-weight pointers (or null); sscale: nseg scales
void seq_short_conv(int code, int out_f32, const void* u, int ldu, const float* w, const float* bias, void* state,
                    void* out, int C,
                    int taps, int nseg, const int* segs, const float* const* sw, const float* sscale, SeqDesc d,
                    float eps, hipStream_t st) {
  if (d.Ttot == 0) return;
  ConvArgs a;
  a.nseg = nseg;
  int heads = 0;
  for (int i = 0; i < nseg; ++i) {
    a.seg[i] = ConvSeg{segs[4 * i], segs[4 * i + 1], segs[4 * i + 2], segs[4 * i + 3], sw[i], sscale[i]};
    heads += segs[4 * i + 1];
  }
  SEQ_DISPATCH_T(code, {
    if (out_f32)
      hipLaunchKernelGGL((k_short_conv<T, float>), dim3(d.Ttot, heads), dim3(64), 0, st, (const T*)u, ldu, w, bias,
                         (const T*)state, (float*)out, C, taps, a, d, eps);
    else
      hipLaunchKernelGGL((k_short_conv<T, T>), dim3(d.Ttot, heads), dim3(64), 0, st, (const T*)u, ldu, w, bias,
                         (const T*)state, (T*)out, C, taps, a, d, eps);
    if (taps > 1)
      hipLaunchKernelGGL(k_conv_state<T>, dim3(d.B, (C + 255) / 256), dim3(256), 0, st, (const T*)u, ldu, (T*)state, C,
                         taps, d);
  });
  LIPA_CHECK_LAUNCH();
}

void seq_mlstm_scan(int code, const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, const float* ipre,
                    const float* fpre, const float* ib, const float* fb, float cap, float qscale, float* S, float* N,
                    float* M, float* out, float* den, float* efl, int H, int dk, int dv, SeqDesc d, hipStream_t st) {
  if (d.B == 0) return;
  const int Rr = rows_split(dk);
  SEQ_DISPATCH_T(code, SEQ_DISPATCH_R(Rr, {
    constexpr int NC = 256 / R;
    hipLaunchKernelGGL((k_mlstm_scan<T, R>), dim3(d.B * H, (dv + 1 + NC - 1) / NC), dim3(256), 0, st, (const T*)q, ldq,
                       (const T*)k, ldk, (const T*)v, ldv, ipre, fpre, ib, fb, cap, qscale, S, N, M, out, den, efl, H,
                       dk, dv, d);
  }));
  LIPA_CHECK_LAUNCH();
}

void seq_delta_scan(int code, const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, const float* g,
                    const float* bpre, float* S, float* out, int H, int G, int dk, int dv, SeqDesc d, hipStream_t st) {
  if (d.B == 0) return;
  const int Rr = rows_split(dk);
  SEQ_DISPATCH_T(code, SEQ_DISPATCH_R(Rr, {
    constexpr int NC = 256 / R;
    hipLaunchKernelGGL((k_delta_scan<T, R>), dim3(d.B * H, (dv + NC - 1) / NC), dim3(256), 0, st, (const T*)q, ldq,
                       (const T*)k, ldk, (const T*)v, ldv, g, bpre, S, out, H, G, dk, dv, d);
  }));
  LIPA_CHECK_LAUNCH();
}

void seq_gdr_scan(int code, const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, const float* w,
                  const float* a, const float* kinv, float* S, float* out, int H, int dk, int dv, SeqDesc d,
                  hipStream_t st) {
  if (d.B == 0) return;
  const int Rr = rows_split(dk);
  SEQ_DISPATCH_T(code, SEQ_DISPATCH_R(Rr, {
    constexpr int NC = 256 / R;
    constexpr size_t smem = sizeof(float) * (4 * CT * KRP * R + CT * NC + CT);
    if (smem > 64 * 1024) {                      // above the default limit of a block: ask for it (dk > 128 only)
      static bool asked = false;
      if (!asked) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gdr_scan<T, R>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) fprintf(stderr, "k_gdr_scan: %d bytes of LDS refused: %s\n", (int)smem, hipGetErrorString(e));
        asked = true;
      }
    }
    hipLaunchKernelGGL((k_gdr_scan<T, R>), dim3(d.B * H, (dv + NC - 1) / NC), dim3(256), smem, st, (const T*)q, ldq,
                       (const T*)k, ldk, (const T*)v, ldv, w, a, kinv, S, out, H, dk, dv, d);
  }));
  LIPA_CHECK_LAUNCH();
}

void seq_ssd_scan(int code, const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, const void* dtraw,
                  int lddt, const float* dt_bias, const float* a_log, const float* dskip, float* S, float* out, int H,
                  int G, int dk, int dv, SeqDesc d, hipStream_t st) {
  if (d.B == 0) return;
  const int Rr = rows_split(dk);
  SEQ_DISPATCH_T(code, SEQ_DISPATCH_R(Rr, {
    constexpr int NC = 256 / R;
    hipLaunchKernelGGL((k_ssd_scan<T, R>), dim3(d.B * H, (dv + NC - 1) / NC), dim3(256), 0, st, (const T*)q, ldq,
                       (const T*)k, ldk, (const T*)v, ldv, (const T*)dtraw, lddt, dt_bias, a_log, dskip, S, out, H, G,
                       dk, dv, d);
  }));
  LIPA_CHECK_LAUNCH();
}
