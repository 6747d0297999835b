// Latent attention: keys and values of every head are up-projections of one small per-token latent c, plus one
// rotated key part kr shared by all heads.  Only [c | kr] is cached (one row of R + dr entries per token), and the
// up-projections are moved to the query side:  score_h(i, j) = (W_uk_h^T q_h(i)) . c(j) + q_rot_h(i) . kr(j),
// out_h(i) = W_uv_h sum_j w_h(i, j) c(j).  Every head then reads the same cache rows (one "kv head" whose values are
// the first R columns of its keys), so the sweeps of seq_attn.hip serve it with ldk = ldv = R + dr.
//
// Here: the cache write (RMS norm of the latent, rotation of the shared key part), the query assembly (absorbed part
// copied beside the rotated part) and the merge of key splits with a per-head sigmoid gate.
#include "seq_common.h"

using namespace lipa;

// one block per token: row[0:R] = rms(u[0:R]) * w, row[R:R+dr] = rotate(u[R:R+dr]) at the token's position
template <typename T>
__global__ __launch_bounds__(256) void k_latent_kv_store(const T* __restrict__ u, int ldu, const float* __restrict__ w,
                                                         const float* __restrict__ inv_freq, T* __restrict__ cache,
                                                         int R, int dr, int dims, int max_len, float eps, int half,
                                                         float mag, SeqDesc d) {
  __shared__ float sc[4];
  const int t = blockIdx.x, s = d.tok_seq[t], p = d.tok_pos[t], slot = d.slots[s];
  const T* src = u + (size_t)t * ldu;
  T* row = cache + ((size_t)slot * max_len + p) * (R + dr);
  float ss = 0.f;
  for (int c = threadIdx.x; c < R; c += 256) {
    const float v = (float)src[c];
    ss += v * v;
  }
  const float rs = rsqrtf(block_sum256(ss, sc) / R + eps);
  for (int c = threadIdx.x; c < R; c += 256) row[c] = (T)((float)src[c] * rs * w[c]);
  for (int c = threadIdx.x; c < dr; c += 256) row[R + c] = (T)rotated_at(src + R, c, dims, (float)p, inv_freq, half, mag);
}

// one block per (token, head): Q[t, h, 0:R] = qa[h, t, 0:R] (the absorbed unrotated part),
// Q[t, h, R:R+dr] = rotate(q[t, h, dn:dn+dr])
template <typename T>
__global__ __launch_bounds__(128) void k_latent_q_assemble(const T* __restrict__ qa, size_t qa_sh, size_t qa_st,
                                                           const T* __restrict__ q, int ldq, int dn,
                                                           const float* __restrict__ inv_freq, T* __restrict__ out,
                                                           int H, int R, int dr, int dims, int half, float mag,
                                                           SeqDesc d) {
  const int t = blockIdx.x, h = blockIdx.y;
  const float p = (float)d.tok_pos[t];
  T* dst = out + ((size_t)t * H + h) * (R + dr);
  const T* a = qa + h * qa_sh + t * qa_st;
  for (int c = threadIdx.x; c < R; c += 128) dst[c] = a[c];
  const T* r = q + (size_t)t * ldq + (size_t)h * (dn + dr) + dn;
  for (int c = threadIdx.x; c < dr; c += 128) dst[R + c] = (T)rotated_at(r, c, dims, p, inv_freq, half, mag);
}

// one block per (token, head): merge the key splits, normalise, multiply by sigmoid(gate[t, h]).  The splits' weights
// e_z = exp(m_z - max m) go through LDS once; every thread then sums its columns over the splits.
constexpr int MERGE_Z = 128;     // splits whose weights are held in LDS (more are recomputed per column)
template <typename T>
__global__ __launch_bounds__(128) void k_latent_merge(const float* __restrict__ pm, const float* __restrict__ pl,
                                                      const float* __restrict__ pu, const T* __restrict__ gate, int ldg,
                                                      T* __restrict__ out, int H, int dv, int nsplit) {
  __shared__ float se[MERGE_Z];
  __shared__ float sred[4];
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const size_t b = ((size_t)t * H + h) * nsplit;
  float mx = -INFINITY;
  for (int z = tid; z < nsplit; z += 128) mx = fmaxf(mx, pm[b + z]);
  mx = wave_max(mx);
  if ((tid & 63) == 0) sred[tid >> 6] = mx;
  __syncthreads();
  mx = fmaxf(sred[0], sred[1]);
  float l = 0.f;
  for (int z = tid; z < nsplit; z += 128) {
    const float e = expf(pm[b + z] - mx);
    if (z < MERGE_Z) se[z] = e;
    l += e * pl[b + z];
  }
  l = wave_sum(l);
  if ((tid & 63) == 0) sred[2 + (tid >> 6)] = l;
  __syncthreads();
  l = sred[2] + sred[3];
  const float g = gate != nullptr ? sigmoidf_((float)gate[(size_t)t * ldg + h]) : 1.f;
  const float mul = g / l;
  for (int c = tid; c < dv; c += 128) {
    float u = 0.f;
#pragma unroll 4
    for (int z = 0; z < nsplit; ++z) u += (z < MERGE_Z ? se[z] : expf(pm[b + z] - mx)) * pu[(b + z) * dv + c];
    out[((size_t)t * H + h) * dv + c] = (T)(u * mul);
  }
}

void seq_latent_kv_store(int code, const void* u, int ldu, const float* w, const float* inv_freq, void* cache, int R,
                         int dr, int dims, int max_len, float eps, int half, float mag, SeqDesc d, hipStream_t st) {
  if (d.Ttot == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_latent_kv_store<T>, dim3(d.Ttot), dim3(256), 0, st, (const T*)u, ldu, w,
                                          inv_freq, (T*)cache, R, dr, dims, max_len, eps, half, mag, d));
  LIPA_CHECK_LAUNCH();
}

void seq_latent_q_assemble(int code, const void* qa, size_t qa_sh, size_t qa_st, const void* q, int ldq, int dn,
                           const float* inv_freq, void* out, int H, int R, int dr, int dims, int half, float mag,
                           SeqDesc d, hipStream_t st) {
  if (d.Ttot == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_latent_q_assemble<T>, dim3(d.Ttot, H), dim3(128), 0, st, (const T*)qa, qa_sh,
                                          qa_st, (const T*)q, ldq, dn, inv_freq, (T*)out, H, R, dr, dims, half, mag, d));
  LIPA_CHECK_LAUNCH();
}

void seq_latent_merge(int code, const float* pm, const float* pl, const float* pu, const void* gate, int ldg, void* out,
                      int T_, int H, int dv, int nsplit, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_latent_merge<T>, dim3(T_, H), dim3(128), 0, st, pm, pl, pu, (const T*)gate,
                                          ldg, (T*)out, H, dv, nsplit));
  LIPA_CHECK_LAUNCH();
}
