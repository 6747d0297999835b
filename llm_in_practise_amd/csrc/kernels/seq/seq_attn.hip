// Causal softmax attention over a slot-indexed K/V cache whose softmax weights are mixed across heads before they
// meet the values ("talking heads" after the softmax):  w'_h(i, j) = sum_g talk[h, g] w_g(i, j),
// o_h(i) = sum_j w'_h(i, j) v_kv(h)(j).
//
// Mixing is linear, so  o_h = sum_g talk[h, g] U[g, kv(h)]  with  U[g, c](i) = sum_j w_g(i, j) v_c(j): pass 1 is a
// flash-style single sweep per (query token, query head g) that accumulates its softmax weights against the values
// of ALL kv heads (G * dv columns) with a running maximum; keys may be cut into splits (decode: long caches, few
// rows).  Pass 2 merges the splits, normalises, mixes the heads with talk, applies the sigmoid output gate and writes
// the activation type.  Scores, weights and U are float.  One wave per (token, head, split): lanes own keys for
// q.k (each lane one key's full dot product, q broadcast from LDS), then own value columns for w.V.
//
// The same sweeps serve plain grouped-query attention (GQA = true): a query head meets only the values of its own kv
// head, and three optional parts change which keys count and how: a float bias per (head, distance) added to the
// scaled score, a block mask (a query sees only the keys of its own run of `block` positions, counted from the
// sequence's position 0), a sliding window (a query sees only the keys less than `window` positions back, itself
// included), and a sink (one more key of a fixed score, or of a learned score per head, without a value in every
// softmax).  With one key split the matrix-core sweep normalises and writes the activation type itself; otherwise
// k_gqa_merge does.  The output may be a column slice of a wider matrix (row stride ldo) and is multiplied by
// out_scale.
#include "seq_common.h"

using namespace lipa;

// what GQA = true adds to a sweep
struct GqaExtra {
  const float* bias;   // [H, nd] or null: bias[h][min(i - j, nd - 1)], in natural-log units
  int nd;
  int block;           // 0: every earlier key; > 0: keys of the query's own block
  int sink;            // 1: a key of score sink_logit (or sinks[h]) and no value
  float sink_logit;
  void* out;           // [T, H * dv] in the activation type, written when nsplit == 1 (matrix-core sweep)
  int window;          // 0: every earlier key; > 0: keys j with i - j < window
  const float* sinks;  // [H] or null: a sink score per head, in place of sink_logit
  int ldo;             // row stride of out
  float out_scale;
};

constexpr int MAXC = 16;   // value columns per lane: G * dv <= 64 * MAXC

template <typename T, bool GQA>
__global__ __launch_bounds__(64) void k_talk_attn_partial(const T* __restrict__ q, int ldq, const T* __restrict__ kc,
                                                          const T* __restrict__ vc, float* __restrict__ pm,
                                                          float* __restrict__ pl, float* __restrict__ pu, int H, int G,
                                                          int dk, int dv, int ldk, int ldv, int max_len, int nsplit,
                                                          float scale, SeqDesc d, GqaExtra x) {
  extern __shared__ float sq[];
  const int t = blockIdx.x, g = blockIdx.y, z = blockIdx.z, lane = threadIdx.x;
  const int s = d.tok_seq[t], p = d.tok_pos[t], slot = d.slots[s];
  const int kh = g / (H / G), GV = GQA ? dv : G * dv;
  for (int i = lane; i < dk; i += 64) sq[i] = (float)q[(size_t)t * ldq + g * dk + i];
  __syncthreads();
  int lo = (GQA && x.block > 0) ? (p / x.block) * x.block : 0;
  if (GQA && x.window > 0) lo = max(lo, p - x.window + 1);
  const int nkeys = p + 1 - lo, per = (nkeys + nsplit - 1) / nsplit;
  const int j0 = lo + z * per, j1 = min(p + 1, j0 + per);
  const T* kbase = kc + ((size_t)slot * max_len) * ldk + kh * dk;
  const T* vbase = vc + ((size_t)slot * max_len) * ldv + (GQA ? kh * dv : 0);
  float acc[MAXC];
#pragma unroll
  for (int c = 0; c < MAXC; ++c) acc[c] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int jb = j0; jb < j1; jb += 64) {
    const int j = jb + lane;
    float sc = -INFINITY;
    if (j < j1) {
      const T* kr = kbase + (size_t)j * ldk;
      float a = 0.f;
      for (int i = 0; i < dk; ++i) a += sq[i] * (float)kr[i];
      sc = a * scale;
      if (GQA && x.bias != nullptr) sc += x.bias[(size_t)g * x.nd + min(p - j, x.nd - 1)];
    }
    const float mn = fmaxf(m, wave_max(sc));
    if (mn == -INFINITY) continue;            // a split without keys (lanes agree: mn is wave-uniform)
    const float corr = expf(m - mn);          // m = -inf on the first chunk: exp(-inf) = 0
    const float w = j < j1 ? expf(sc - mn) : 0.f;
    l = l * corr + wave_sum(w);
    m = mn;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) acc[c] *= corr;
    const int cnt = min(64, j1 - jb);
    for (int jj = 0; jj < cnt; ++jj) {
      const float wj = __shfl(w, jj, 64);
      const T* vr = vbase + (size_t)(jb + jj) * ldv;
#pragma unroll
      for (int c = 0; c < MAXC; ++c) {
        const int col = c * 64 + lane;
        if (col < GV) acc[c] += wj * (float)vr[col];
      }
    }
  }
  const size_t o = ((size_t)t * H + g) * nsplit + z;
  if (lane == 0) {
    pm[o] = m;
    pl[o] = l;
  }
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int col = c * 64 + lane;
    if (col < GV) pu[o * GV + col] = acc[c];
  }
}


// ------------------------------------------------------------------------------------------------ MFMA pass 1 (bf16)
// One wave per (tile of up to 32 consecutive queries of one sequence, query head g, kv head c of the VALUES, key
// split).  Scores are computed transposed, S^T[key][query] = K Q^T with v_mfma_f32_32x32x16_bf16: a lane then owns one
// query (lane % 32) and 16 of the tile's 32 keys, so the softmax statistics are lane-local plus one exchange between
// the wave's halves, and the weights P^T are already laid out as the B operand of O^T[col][query] += V^T P^T.  The
// value tile goes through LDS row-major (16 B stores); a lane gets its column's 8 keys of a step with two transposing
// LDS reads (ds_read_tr16_b64).
// K and Q operands are 16 B global loads (Q stays in registers).  Rows past the cache end are clamped: their weights
// are 0.  Writes the same partial format as the scalar kernel: m, l per (token, g, split) and unnormalised U columns
// [c*dv, (c+1)*dv).
// HEADS = true is the decode form: a tile is ONE token and its "queries" are the H/G query heads that share kv head
// blockIdx.y, so a key tile is loaded once for the whole group instead of once per head.
typedef __attribute__((address_space(3))) bf16x4 lds_bf16x4;
__device__ __forceinline__ bf16x4 tr_read(const bf16* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(p));
}

// NW = 4 puts four query heads of one kv head (and one value head c) into a block: the key and value tiles are loaded
// once into LDS for the four waves instead of once per head.
template <int NDS, int NDT, bool HEADS, int NW, bool GQA>
__global__ __launch_bounds__(64 * NW) void k_talk_attn_mfma(const bf16* __restrict__ q, int ldq, const bf16* __restrict__ kc,
                                                       const bf16* __restrict__ vc, float* __restrict__ pm,
                                                       float* __restrict__ pl, float* __restrict__ pu,
                                                       const int* __restrict__ tile_seq, const int* __restrict__ tile_t0,
                                                       int H, int G, int dk, int dv, int ldk, int ldv, int max_len,
                                                       int nsplit, float scale, SeqDesc d, GqaExtra x) {
  constexpr int LDMAX = NDT * 32 + 8, LDKMAX = NDS * 16 + 8;
  __shared__ __attribute__((aligned(16))) bf16 sV[32 * LDMAX];
  __shared__ __attribute__((aligned(16))) bf16 sK[NW > 1 ? 32 * LDKMAX : 8];
  const int tile = blockIdx.x, z = GQA ? blockIdx.z : blockIdx.z / G;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, hi = lane >> 5, ql = lane & 31, rep = H / G;
  const int s = tile_seq[tile], t0 = tile_t0[tile], tend = d.seq_off[s + 1], slot = d.slots[s];
  const int tq = HEADS ? t0 : min(t0 + ql, tend - 1);
  const int g = HEADS ? blockIdx.y * rep + min(ql, rep - 1) : blockIdx.y * NW + wv;
  const bool valid_q = HEADS ? ql < rep : t0 + ql < tend;
  const int pos_q = d.tok_pos[tq], pmax = HEADS ? pos_q : d.tok_pos[min(t0 + 31, tend - 1)];
  const int nds = dk >> 4, ndt = dv >> 5, LD = dv + 8, LDK = dk + 8, kh = HEADS ? blockIdx.y : g / rep;
  const int c = GQA ? kh : blockIdx.z % G, GV = GQA ? dv : G * dv;
  // block mask: the tile's sweep starts at the block of its first query; every query keeps its own block's keys
  const int blk = GQA ? x.block : 0, win = GQA ? x.window : 0;
  int lo_t = blk > 0 ? ((HEADS ? pos_q : d.tok_pos[t0]) / blk) * blk : 0, lo_q = blk > 0 ? (pos_q / blk) * blk : 0;
  if (win > 0) {                                   // sliding window: nothing before the first query's oldest key
    lo_t = max(lo_t, (HEADS ? pos_q : d.tok_pos[t0]) - win + 1);
    lo_q = max(lo_q, pos_q - win + 1);
  }
  const float* brow = (GQA && x.bias != nullptr) ? x.bias + (size_t)g * x.nd : nullptr;
  // a tile's queries sit at consecutive positions p0 + ql, so a 32-key tile meets only the 63 distances
  // p0 - jb - 31 + i: lane i fetches that one bias and the 16 a lane needs come from its neighbours' registers
  const int p0 = HEADS ? pos_q : d.tok_pos[t0];
  const float sl2 = scale * 1.4426950408889634f;   // scores in units of log2: v_exp_f32 is 2^x
  const int trow = 4 * (lane >> 5) + ((lane & 15) >> 2), tcol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const int per = (pmax - lo_t + nsplit) / nsplit, j0 = lo_t + z * per, j1 = min(pmax + 1, j0 + per);
  const bf16* kbase = kc + ((size_t)slot * max_len) * ldk + kh * dk + 8 * hi;
  const bf16* vbase = vc + ((size_t)slot * max_len) * ldv + c * dv;
  bf16x8 qf[NDS];
#pragma unroll
  for (int ds = 0; ds < NDS; ++ds)
    if (ds < nds) qf[ds] = *reinterpret_cast<const bf16x8*>(q + (size_t)tq * ldq + g * dk + 16 * ds + 8 * hi);
  f32x16 acc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
  float m = -INFINITY, l = 0.f;
  const int vpr = dv >> 3, kpr = dk >> 3;        // 16 B vectors per value / key row
  // four waves: the next key / value tile is fetched into registers while the current one is computed on
  constexpr int VPT = NW > 1 ? (2 * NDT) / NW : 1, KPT = NW > 1 ? (2 * NDS) / NW : 1;
  bf16x8 pv[VPT], pk[KPT];
  auto fetch = [&](int jb) {
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int e = threadIdx.x + 64 * NW * i, row = e / vpr, cv = e % vpr;
      if (e < 32 * vpr)
        pv[i] = *reinterpret_cast<const bf16x8*>(vbase + (size_t)min(jb + row, max_len - 1) * ldv + cv * 8);
    }
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int e = threadIdx.x + 64 * NW * i, row = e / kpr, cv = e % kpr;
      if (e < 32 * kpr)
        pk[i] = *reinterpret_cast<const bf16x8*>(kbase - 8 * hi + (size_t)min(jb + row, max_len - 1) * ldk + cv * 8);
    }
  };
  if (NW > 1 && j0 < j1) fetch(j0);
  for (int jb = j0; jb < j1; jb += 32) {
    __syncthreads();
    if (NW > 1) {
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int e = threadIdx.x + 64 * NW * i;
        if (e < 32 * vpr) *reinterpret_cast<bf16x8*>(sV + (e / vpr) * LD + (e % vpr) * 8) = pv[i];
      }
#pragma unroll
      for (int i = 0; i < KPT; ++i) {
        const int e = threadIdx.x + 64 * NW * i;
        if (e < 32 * kpr) *reinterpret_cast<bf16x8*>(sK + (e / kpr) * LDK + (e % kpr) * 8) = pk[i];
      }
      __syncthreads();
      if (jb + 32 < j1) fetch(jb + 32);
    } else {
      for (int e = threadIdx.x; e < 32 * vpr; e += 64) {
        const int row = e / vpr, cv = e % vpr;
        *reinterpret_cast<bf16x8*>(sV + row * LD + cv * 8) =
            *reinterpret_cast<const bf16x8*>(vbase + (size_t)min(jb + row, max_len - 1) * ldv + cv * 8);
      }
    }
    f32x16 sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = 0.f;
    const bf16* kr = NW > 1 ? sK + ql * LDK + 8 * hi : kbase + (size_t)min(jb + ql, max_len - 1) * ldk;
#pragma unroll
    for (int ds = 0; ds < NDS; ++ds)
      if (ds < nds)
        sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(kr + 16 * ds), qf[ds], sc, 0, 0, 0);
    float mt = -INFINITY, bw = 0.f;
    if (GQA && !HEADS && brow != nullptr)
      bw = brow[min(max(p0 - jb - 31 + lane, 0), x.nd - 1)] * 1.4426950408889634f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int kk = (r & 3) + 8 * (r >> 2) + 4 * hi, key = jb + kk;
      const bool seen = key <= pos_q && key < j1 && (!GQA || key >= lo_q);
      float v = sc[r] * sl2;
      if (GQA && !HEADS && brow != nullptr) v += __shfl(bw, ql - kk + 31, 64);
      if (GQA && HEADS && brow != nullptr && seen) v += brow[min(pos_q - key, x.nd - 1)] * 1.4426950408889634f;
      sc[r] = seen ? v : -INFINITY;
      mt = fmaxf(mt, sc[r]);
    }
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float mn = fmaxf(m, mt), ms = mn == -INFINITY ? 0.f : mn;
    const float corr = __builtin_amdgcn_exp2f(m - ms);
    float rs = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      sc[r] = __builtin_amdgcn_exp2f(sc[r] - ms);
      rs += sc[r];
    }
    rs += __shfl_xor(rs, 32, 64);
    l = l * corr + rs;
    m = mn;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[dt][r] *= corr;
    if (NW == 1) __syncthreads();                  // (four waves: the barrier after the tile copies covers V too)
#pragma unroll
    for (int u2 = 0; u2 < 2; ++u2) {
      bf16x8 pb;
#pragma unroll
      for (int j = 0; j < 8; ++j) pb[j] = (bf16)sc[8 * u2 + j];
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
        if (dt < ndt) {
          // transposing LDS reads: the 16 lanes of a group address a 4-key x 16-column block (lane 4q'+p': key q',
          // columns 4p'..4p'+3) and lane i receives column i's four keys; keys 16u2 + 4hi + 0..3, then the same + 8
          const bf16* vp = sV + (16 * u2 + trow) * LD + dt * 32 + tcol;
          const bf16x4 v0 = tr_read(vp), v1 = tr_read(vp + 8 * LD);
          const bf16x8 vf = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
          acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pb, acc[dt], 0, 0, 0);
        }
    }
  }
  if (!valid_q) return;
  if (GQA && nsplit == 1) {                      // the whole softmax is here: add the sink, normalise, write
    const float sk = (x.sinks != nullptr ? x.sinks[g] : x.sink_logit) * 1.4426950408889634f, mf = x.sink ? fmaxf(m, sk) : m;
    const float e = mf == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - mf);
    const float den = l * e + (x.sink ? __builtin_amdgcn_exp2f(sk - mf) : 0.f);
    const float inv = den > 0.f ? e / den * x.out_scale : 0.f;
    bf16* orow = (bf16*)x.out + (size_t)tq * x.ldo + g * dv;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
      if (dt < ndt)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4)
          *reinterpret_cast<bf16x4*>(orow + dt * 32 + 8 * r4 + 4 * hi) =
              bf16x4{(bf16)(acc[dt][4 * r4] * inv), (bf16)(acc[dt][4 * r4 + 1] * inv), (bf16)(acc[dt][4 * r4 + 2] * inv),
                     (bf16)(acc[dt][4 * r4 + 3] * inv)};
    return;
  }
  const size_t o = ((size_t)tq * H + g) * nsplit + z;
  if ((GQA || c == 0) && hi == 0) {
    pm[o] = m * 0.6931471805599453f;             // back to natural units, as the scalar sweep writes them
    pl[o] = l;
  }
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
    if (dt < ndt)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4)
        *reinterpret_cast<f32x4*>(pu + o * GV + (GQA ? 0 : c * dv) + dt * 32 + 8 * r4 + 4 * hi) =
            f32x4{acc[dt][4 * r4], acc[dt][4 * r4 + 1], acc[dt][4 * r4 + 2], acc[dt][4 * r4 + 3]};
}

// Pass 2.  One block per (token, 64 value columns of one kv head c): first the splits of every query head g are
// merged and normalised into LDS, L[g][col] = sum_z e_z U_gz[col] / sum_z e_z l_gz with e_z = exp(m_gz - max_z m_gz);
// then every output head h of kv head c takes out[h][col] = sigmoid(gate) * sum_g talk[h][g] L[g][col].
constexpr int MH = 128;    // query heads held in LDS
template <typename T>
__global__ __launch_bounds__(256) void k_talk_attn_merge(const float* __restrict__ pm, const float* __restrict__ pl,
                                                         const float* __restrict__ pu, const float* __restrict__ talk,
                                                         const T* __restrict__ gate, int ldg, T* __restrict__ out, int H,
                                                         int G, int dv, int nsplit) {
  extern __shared__ float L[];                     // [H][64]
  const int t = blockIdx.x, nch = (dv + 63) / 64, c = blockIdx.y / nch, ch = blockIdx.y % nch;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, col = ch * 64 + lane, GV = G * dv, rep = H / G;
  for (int g = w; g < H; g += 4) {
    const size_t b = ((size_t)t * H + g) * nsplit;
    float mx = -INFINITY;
    for (int z = 0; z < nsplit; ++z) mx = fmaxf(mx, pm[b + z]);
    float l = 0.f, u = 0.f;
    for (int z = 0; z < nsplit; ++z) {
      const float e = expf(pm[b + z] - mx);
      l += e * pl[b + z];
      if (col < dv) u += e * pu[(b + z) * GV + c * dv + col];
    }
    L[g * 64 + lane] = u / l;
  }
  __syncthreads();
  if (col >= dv) return;
  for (int hl = w; hl < rep; hl += 4) {
    const int h = c * rep + hl;
    float o = 0.f;
    for (int g = 0; g < H; ++g) o += talk[h * H + g] * L[g * 64 + lane];
    out[(size_t)t * (H * dv) + h * dv + col] = (T)(o * sigmoidf_((float)gate[(size_t)t * ldg + h * dv + col]));
  }
}

template <typename T>
static void launch_merge(const float* pm, const float* pl, const float* pu, const float* talk, const T* gate, int ldg,
                         T* out, int Ttot, int H, int G, int dv, int nsplit, hipStream_t st) {
  hipLaunchKernelGGL(k_talk_attn_merge<T>, dim3(Ttot, G * ((dv + 63) / 64)), dim3(256), sizeof(float) * H * 64, st, pm,
                     pl, pu, talk, gate, ldg, out, H, G, dv, nsplit);
}

int seq_attn_max_heads() { return MH; }
int seq_attn_max_cols() { return 64 * MAXC; }

// the MFMA sweep needs bf16, 16-byte rows and whole operand tiles
bool seq_attn_mfma_ok(int code, int ldq, int dk, int dv) {
  return code == 0 && dk % 16 == 0 && dk <= 256 && dv % 32 == 0 && dv <= 256 && ldq % 8 == 0;
}

// Launches a sweep; returns true when it wrote the final output itself (GQA, matrix cores, one key split).
template <bool GQA>
static bool sweep(int code, const void* q, int ldq, const void* kc, int ldk, const void* vc, int ldv, float* pm, float* pl,
                  float* pu, int H, int G, int dk, int dv, int max_len, int nsplit, float scale, const int* tile_seq,
                  const int* tile_t0, int ntiles, SeqDesc d, GqaExtra x, hipStream_t st) {
  if (d.Ttot == 0) return false;
  if (tile_seq != nullptr && seq_attn_mfma_ok(code, ldq, dk, dv) && ldk % 8 == 0 && ldv % 8 == 0) {
    const bool heads = ntiles == d.Ttot && H / G <= 32 && H / G > 1;    // one token per tile: group the heads instead
    const int nw = (!heads && (H / G) % 4 == 0) ? 4 : 1;                 // four heads of a kv head share its tiles
    const dim3 grid(ntiles, heads ? G : H / nw, GQA ? nsplit : G * nsplit);
#define SEQ_ATTN_LAUNCH(NDS, NDT, HEADS, NW)                                                                        \
  hipLaunchKernelGGL((k_talk_attn_mfma<NDS, NDT, HEADS, NW, GQA>), grid, dim3(64 * NW), 0, st, (const bf16*)q, ldq,  \
                     (const bf16*)kc, (const bf16*)vc, pm, pl, pu, tile_seq, tile_t0, H, G, dk, dv, ldk, ldv, max_len, \
                     nsplit, scale, d, x)
    bool small = false;                            // small heads: half the accumulators, more waves per SIMD
    if constexpr (GQA) {
      small = dk <= 64 && dv <= 64;
      if (small) {
        if (heads) SEQ_ATTN_LAUNCH(4, 2, true, 1); else if (nw == 4) SEQ_ATTN_LAUNCH(4, 2, false, 4); else SEQ_ATTN_LAUNCH(4, 2, false, 1);
      }
    }
    if (small) {
    } else if (dk <= 128 && dv <= 128) {
      if (heads) SEQ_ATTN_LAUNCH(8, 4, true, 1); else if (nw == 4) SEQ_ATTN_LAUNCH(8, 4, false, 4); else SEQ_ATTN_LAUNCH(8, 4, false, 1);
    } else {
      if (heads) SEQ_ATTN_LAUNCH(16, 8, true, 1); else if (nw == 4) SEQ_ATTN_LAUNCH(16, 8, false, 4); else SEQ_ATTN_LAUNCH(16, 8, false, 1);
    }
#undef SEQ_ATTN_LAUNCH
    LIPA_CHECK_LAUNCH();
    return GQA && nsplit == 1;
  }
  SEQ_DISPATCH_T(code, {
    hipLaunchKernelGGL((k_talk_attn_partial<T, GQA>), dim3(d.Ttot, H, nsplit), dim3(64), sizeof(float) * dk, st,
                       (const T*)q, ldq, (const T*)kc, (const T*)vc, pm, pl, pu, H, G, dk, dv, ldk, ldv, max_len, nsplit,
                       scale, d, x);
  });
  LIPA_CHECK_LAUNCH();
  return false;
}

// Pass 1 for any caller: the partial sweeps over a slot-indexed cache whose key rows are ldk and value rows ldv
// elements apart (values may be columns of the key rows: a latent cache).  Writes pm, pl [T, H, nsplit] and
// pu [T, H, nsplit, G * dv].
void seq_attn_sweep(int code, const void* q, int ldq, const void* kc, int ldk, const void* vc, int ldv, float* pm,
                    float* pl, float* pu, int H, int G, int dk, int dv, int max_len, int nsplit, float scale,
                    const int* tile_seq, const int* tile_t0, int ntiles, SeqDesc d, hipStream_t st) {
  sweep<false>(code, q, ldq, kc, ldk, vc, ldv, pm, pl, pu, H, G, dk, dv, max_len, nsplit, scale, tile_seq, tile_t0,
               ntiles, d, GqaExtra{nullptr, 0, 0, 0, 0.f, nullptr, 0, nullptr, 0, 1.f}, st);
}

// Merge of a GQA sweep's key splits: one wave per (token, head); the sink joins the denominator here.
template <typename T>
__global__ __launch_bounds__(64) void k_gqa_merge(const float* __restrict__ pm, const float* __restrict__ pl,
                                                  const float* __restrict__ pu, T* __restrict__ out, int H, int dv,
                                                  int nsplit, int sink, float sink_logit,
                                                  const float* __restrict__ sinks, int ldo, float out_scale) {
  const int t = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
  const size_t b = ((size_t)t * H + g) * nsplit;
  if (sinks != nullptr) sink_logit = sinks[g];
  float mx = sink ? sink_logit : -INFINITY;
  for (int z = 0; z < nsplit; ++z) mx = fmaxf(mx, pm[b + z]);
  float l = sink ? expf(sink_logit - mx) : 0.f;
  for (int z = 0; z < nsplit; ++z) l += pm[b + z] == -INFINITY ? 0.f : expf(pm[b + z] - mx) * pl[b + z];
  const float inv = l > 0.f ? out_scale / l : 0.f;
  for (int col = lane; col < dv; col += 64) {
    float u = 0.f;
    for (int z = 0; z < nsplit; ++z)
      if (pm[b + z] != -INFINITY) u += expf(pm[b + z] - mx) * pu[(b + z) * dv + col];
    out[(size_t)t * ldo + g * dv + col] = (T)(u * inv);
  }
}

// Grouped-query attention over a slot-indexed cache with an optional distance bias, block mask, sliding window and
// sink.  Key rows are ldk and value rows ldv elements apart (values may be columns of the key rows: a latent cache
// with G = 1); the output rows are ldo elements apart.
void seq_gqa_attention(int code, const void* q, int ldq, const void* kc, int ldk, const void* vc, int ldv, float* pm,
                       float* pl, float* pu, const float* bias, int nd, int block, int window, int sink, float sink_logit,
                       const float* sinks, void* out, int ldo, float out_scale, int H, int G, int dk, int dv, int max_len,
                       int nsplit, float scale, const int* tile_seq, const int* tile_t0, int ntiles, SeqDesc d,
                       hipStream_t st) {
  if (d.Ttot == 0) return;
  const bool direct = sweep<true>(code, q, ldq, kc, ldk, vc, ldv, pm, pl, pu, H, G, dk, dv, max_len, nsplit, scale,
                                  tile_seq, tile_t0, ntiles, d,
                                  GqaExtra{bias, nd, block, sink, sink_logit, out, window, sinks, ldo, out_scale}, st);
  if (direct) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_gqa_merge<T>, dim3(d.Ttot, H), dim3(64), 0, st, pm, pl, pu, (T*)out, H, dv,
                                          nsplit, sink, sink_logit, sinks, ldo, out_scale));
  LIPA_CHECK_LAUNCH();
}

void seq_talk_attention(int code, const void* q, int ldq, const void* kc, const void* vc, float* pm, float* pl,
                        float* pu, const float* talk, const void* gate, int ldg, void* out, int H, int G, int dk, int dv,
                        int max_len, int nsplit, float scale, const int* tile_seq, const int* tile_t0, int ntiles,
                        SeqDesc d, hipStream_t st) {
  if (d.Ttot == 0) return;
  seq_attn_sweep(code, q, ldq, kc, G * dk, vc, G * dv, pm, pl, pu, H, G, dk, dv, max_len, nsplit, scale, tile_seq,
                 tile_t0, ntiles, d, st);
  SEQ_DISPATCH_T(code, launch_merge<T>(pm, pl, pu, talk, (const T*)gate, ldg, (T*)out, d.Ttot, H, G, dv, nsplit, st));
  LIPA_CHECK_LAUNCH();
}
