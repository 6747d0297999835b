// PyTorch bindings of the sequence-state kernels (csrc/kernels/seq/*.hip): raw pointers + the current HIP stream,
// so every op is ordered with PyTorch's own work and can be captured in a hipGraph.  Shapes and bounds that the
// kernels assume are checked here, on the host, before anything is launched.
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include <hip/hip_runtime.h>

#include <vector>

namespace lipa {
struct SeqDesc {
  const int* seq_off;
  const int* slots;
  const int* pos0;
  const int* tok_seq;
  const int* tok_pos;
  const int* live;
  int B, Ttot;
};
}  // namespace lipa
using lipa::SeqDesc;

void seq_embed_sincos(int, const long*, const int*, const void*, const float*, float*, int, int, float, hipStream_t);
void seq_rms_f32(int, const float*, const float*, void*, int, int, float, hipStream_t);
void seq_gated_residual(int, float*, const void*, int, const void*, int, const float*, const float*, const float*,
                        void*, int, int, float, hipStream_t);
void seq_dual_norm_mean(int, const void*, const void*, const float*, const float*, void*, int, int, float, hipStream_t);
void seq_polynorm(int, const void*, const float*, void*, int, int, float, hipStream_t);
void seq_head_norm_gate(int, const float*, const float*, int, const void*, int, const float*, const float*, void*, int,
                        float, int, int, int, float, hipStream_t);
void seq_decay_gate(const float*, const float*, const float*, float*, int, int, int, hipStream_t);
void seq_short_conv(int, int, const void*, int, const float*, const float*, void*, void*, int, int, int, const int*,
                    const float* const*, const float*, SeqDesc, float, hipStream_t);
void seq_ssd_scan(int, const void*, int, const void*, int, const void*, int, const void*, int, const float*, const float*,
                  const float*, float*, float*, int, int, int, int, SeqDesc, hipStream_t);
void seq_embed_pair(int, const long*, const void*, const void*, int*, float*, void*, int, float, long, long, long,
                    SeqDesc, hipStream_t);
void seq_scaled_postnorm(int, int, float*, const void*, int, const float*, void*, int, int, float, float, hipStream_t);
void seq_rms_act(int, const void*, int, const float*, void*, int, int, float, hipStream_t);
void seq_gate_group_norm(int, const float*, const void*, int, const float*, void*, int, int, int, float, hipStream_t);
void seq_attn_sweep(int, const void*, int, const void*, int, const void*, int, float*, float*, float*, int, int, int,
                    int, int, int, float, const int*, const int*, int, SeqDesc, hipStream_t);
void seq_latent_kv_store(int, const void*, int, const float*, const float*, void*, int, int, int, int, float, int, float,
                         SeqDesc, hipStream_t);
void seq_latent_q_assemble(int, const void*, size_t, size_t, const void*, int, int, const float*, void*, int, int, int,
                           int, int, float, SeqDesc, hipStream_t);
void seq_latent_merge(int, const float*, const float*, const float*, const void*, int, void*, int, int, int, int,
                      hipStream_t);
void seq_route_grouped(const float*, const float*, int*, float*, int, int, int, int, int, float, int, hipStream_t);
void seq_route_fused(int, const void*, int, const float*, const float*, int*, float*, int, int, int, int, int, int, float,
                     int, int, float*, hipStream_t);
void seq_moe_pairs(int, const void*, int, const void*, const void*, const int*, const float*, const void*, const float*,
                   void*, float*, int, int, int, int, int, float, int, hipStream_t);
void seq_moe_combine(int, const void*, const long*, const int*, const float*, const void*, int, const void*, const float*,
                     float*, int, int, int, int, hipStream_t);
void seq_embed_learned(int, const long*, const int*, const void*, const void*, float*, int, int, int, int, int,
                       hipStream_t);
void seq_hyper_mix_norm(int, int, float*, const void*, int, const float*, const float*, const float*, const float*, void*,
                        int, int, int, float, hipStream_t);
void seq_qk_norm_store(int, const void*, int, const float*, const float*, void*, void*, void*, const void*, const float*,
                       int, int, int, int, float, SeqDesc, hipStream_t);
void seq_gqa_attention(int, const void*, int, const void*, int, const void*, int, float*, float*, float*, const float*,
                       int, int, int, int, float, const float*, void*, int, float, int, int, int, int, int, int, float,
                       const int*, const int*, int, SeqDesc, hipStream_t);
void seq_rope_kv_store(int, const void*, int, const float*, void*, void*, void*, int, int, int, int, int, int, float, int,
                       int, SeqDesc, hipStream_t);
void seq_sigmoid_gate(int, const void*, const void*, int, void*, int, int, hipStream_t);
void seq_delta_gates(int, int, const void*, int, const void*, int, const float*, int, const float*, const void*, int,
                     const float*, float*, float*, float*, int, int, int, float, hipStream_t);
void seq_gdr_scan(int, const void*, int, const void*, int, const void*, int, const float*, const float*, const float*,
                  float*, float*, int, int, int, SeqDesc, hipStream_t);
int seq_hyper_max_streams();
bool seq_attn_mfma_ok(int, int, int, int);
void seq_ff_act(int, const void*, void*, int, int, int, float, hipStream_t);
int seq_route_max_outputs();
void seq_mlstm_scan(int, const void*, int, const void*, int, const void*, int, const float*, const float*, const float*,
                    const float*, float, float, float*, float*, float*, float*, float*, float*, int, int, int, SeqDesc,
                    hipStream_t);
void seq_delta_scan(int, const void*, int, const void*, int, const void*, int, const float*, const float*, float*,
                    float*, int, int, int, int, SeqDesc, hipStream_t);
void seq_talk_attention(int, const void*, int, const void*, const void*, float*, float*, float*, const float*,
                        const void*, int, void*, int, int, int, int, int, int, float, const int*, const int*, int,
                        SeqDesc, hipStream_t);
int seq_scan_max_dk();
int seq_conv_max_head();
int seq_conv_max_taps();
int seq_attn_max_cols();
int seq_attn_max_heads();

using at::Tensor;
using c10::optional;

static hipStream_t stream() { return at::hip::getCurrentHIPStream().stream(); }

static int code_of(const Tensor& t) {
  TORCH_CHECK(t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat, "activations must be bf16 or float");
  return t.scalar_type() == at::kBFloat16 ? 0 : 1;
}
static void f32c(const Tensor& t, const char* n) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), n, ": float, contiguous, on the GPU");
}
static void rows(const Tensor& t, int64_t T, int64_t C, int code, const char* n) {   // [T, C] view, unit inner stride
  TORCH_CHECK(t.is_cuda() && t.dim() == 2 && t.size(0) == T && t.size(1) == C && (T == 0 || t.stride(1) == 1) &&
                  code_of(t) == code, n, ": wrong shape, stride or dtype");
}
static int ld(const Tensor& t) { return (int)t.stride(0); }

// desc = [seq_off(B+1), slots(B), pos0(B), tok_seq(T), tok_pos(T)] int32 on the GPU, live optional [B]
static SeqDesc desc_of(const std::vector<Tensor>& d, const optional<Tensor>& live, int64_t T) {
  TORCH_CHECK(d.size() == 5, "sequence descriptor: 5 tensors");
  for (auto& t : d) TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), "descriptor: int32");
  const int B = (int)d[1].numel();
  TORCH_CHECK(d[0].numel() == B + 1 && d[2].numel() == B && d[3].numel() == T && d[4].numel() == T,
              "descriptor sizes do not fit the token count");
  SeqDesc s{d[0].data_ptr<int>(), d[1].data_ptr<int>(), d[2].data_ptr<int>(), d[3].data_ptr<int>(),
            d[4].data_ptr<int>(), nullptr, B, (int)T};
  if (live && live->defined()) {
    TORCH_CHECK(live->is_cuda() && live->scalar_type() == at::kInt && live->numel() >= B, "live: int32 [B]");
    s.live = live->data_ptr<int>();
  }
  return s;
}

Tensor embed_sincos(Tensor tok, Tensor pos, Tensor table, Tensor inv_freq, double scale) {
  TORCH_CHECK(tok.is_cuda() && tok.scalar_type() == at::kLong && tok.is_contiguous(), "tokens: int64");
  TORCH_CHECK(pos.is_cuda() && pos.scalar_type() == at::kInt && pos.is_contiguous() && pos.numel() == tok.numel(),
              "positions: int32, one per token");
  TORCH_CHECK(table.is_cuda() && table.is_contiguous() && table.dim() == 2, "table");
  const int T = (int)tok.numel(), W = (int)table.size(1);
  f32c(inv_freq, "inv_freq");
  TORCH_CHECK(inv_freq.numel() * 2 >= W, "inv_freq too short");
  auto x = at::empty({T, W}, table.options().dtype(at::kFloat));
  seq_embed_sincos(code_of(table), tok.data_ptr<long>(), pos.data_ptr<int>(), table.data_ptr(),
                   inv_freq.data_ptr<float>(), x.data_ptr<float>(), T, W, (float)scale, stream());
  return x;
}

Tensor rms_f32(Tensor x, Tensor w, double eps, bool out_bf16) {
  f32c(x, "x");
  f32c(w, "w");
  const int W = (int)x.size(-1), T = (int)(x.numel() / W);
  TORCH_CHECK(w.numel() == W, "norm weight size");
  auto out = at::empty_like(x, x.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  seq_rms_f32(out_bf16 ? 0 : 1, x.data_ptr<float>(), w.data_ptr<float>(), out.data_ptr(), T, W, (float)eps, stream());
  return out;
}

// x (float, in place) += norm(y * sigmoid(r + b)) * wb; returns norm(x) * wn in y's dtype when wn is given
optional<Tensor> gated_residual(Tensor x, Tensor y, Tensor r, Tensor b, Tensor wb, optional<Tensor> wn, double eps) {
  f32c(x, "x");
  const int W = (int)x.size(-1), T = (int)(x.numel() / W), code = code_of(y);
  rows(y, T, W, code, "y");
  rows(r, T, W, code, "r");
  f32c(b, "b");
  f32c(wb, "wb");
  TORCH_CHECK(b.numel() == W && wb.numel() == W, "gate bias / norm weight size");
  optional<Tensor> h;
  const float* wnp = nullptr;
  void* hp = nullptr;
  if (wn && wn->defined()) {
    f32c(*wn, "wn");
    TORCH_CHECK(wn->numel() == W, "next norm weight size");
    h = at::empty({T, W}, y.options());
    wnp = wn->data_ptr<float>();
    hp = h->data_ptr();
  }
  seq_gated_residual(code, x.data_ptr<float>(), y.data_ptr(), ld(y), r.data_ptr(), ld(r), b.data_ptr<float>(),
                     wb.data_ptr<float>(), wnp, hp, T, W, (float)eps, stream());
  return h;
}

Tensor dual_norm_mean(Tensor a, Tensor b, Tensor wa, Tensor wb, double eps) {
  const int code = code_of(a);
  TORCH_CHECK(a.is_cuda() && a.is_contiguous() && b.is_contiguous() && a.sizes() == b.sizes() && code_of(b) == code,
              "branches must match");
  const int W = (int)a.size(-1), T = (int)(a.numel() / W);
  f32c(wa, "wa");
  f32c(wb, "wb");
  TORCH_CHECK(wa.numel() == W && wb.numel() == W, "norm weight size");
  auto out = at::empty_like(a);
  seq_dual_norm_mean(code, a.data_ptr(), b.data_ptr(), wa.data_ptr<float>(), wb.data_ptr<float>(), out.data_ptr(), T, W,
                     (float)eps, stream());
  return out;
}

Tensor polynorm(Tensor z, Tensor coef, double eps) {
  TORCH_CHECK(z.is_cuda() && z.is_contiguous(), "z");
  f32c(coef, "coef");
  TORCH_CHECK(coef.numel() == 4, "PolyNorm has four coefficients");
  const int F = (int)z.size(-1), T = (int)(z.numel() / F);
  auto out = at::empty_like(z);
  seq_polynorm(code_of(z), z.data_ptr(), coef.data_ptr<float>(), out.data_ptr(), T, F, (float)eps, stream());
  return out;
}

// den / efl (optional, float [T, H]): o is divided by max(|den|, efl) + 1e-6 first
Tensor head_norm_gate(Tensor o, Tensor w, Tensor gate, double eps, optional<Tensor> den, optional<Tensor> efl,
                      optional<Tensor> out_, double scale) {
  f32c(o, "o");
  TORCH_CHECK(o.dim() == 3, "o: [T, H, dv]");
  const int T = (int)o.size(0), H = (int)o.size(1), dv = (int)o.size(2), code = code_of(gate);
  f32c(w, "w");
  TORCH_CHECK(w.numel() == dv || w.numel() == (int64_t)H * dv, "norm weight: [dv] or [H * dv]");
  rows(gate, T, (int64_t)H * dv, code, "gate");
  Tensor out;
  if (out_ && out_->defined()) {                     // a column slice of a wider matrix
    out = *out_;
    rows(out, T, (int64_t)H * dv, code, "out");
  } else {
    out = at::empty({T, (int64_t)H * dv}, gate.options());
  }
  const float* dp = nullptr;
  const float* ep = nullptr;
  if (den && den->defined()) {
    TORCH_CHECK(efl && efl->defined(), "den comes with efl");
    f32c(*den, "den");
    f32c(*efl, "efl");
    TORCH_CHECK(den->numel() == (int64_t)T * H && efl->numel() == (int64_t)T * H, "den / efl: [T, H]");
    dp = den->data_ptr<float>();
    ep = efl->data_ptr<float>();
  }
  seq_head_norm_gate(code, o.data_ptr<float>(), w.data_ptr<float>(), w.numel() != dv, gate.data_ptr(), ld(gate), dp, ep,
                     out.data_ptr(), T == 0 ? H * dv : ld(out), (float)scale, T, H, dv, (float)eps, stream());
  return out;
}

Tensor decay_gate(Tensor pre, Tensor bias, Tensor a_log, int64_t dk) {
  f32c(pre, "pre");
  f32c(bias, "bias");
  f32c(a_log, "A_log");
  const int HD = (int)pre.size(-1), T = (int)(pre.numel() / HD);
  TORCH_CHECK(bias.numel() == HD && HD % dk == 0 && a_log.numel() == HD / dk, "decay gate sizes");
  auto g = at::empty_like(pre);
  seq_decay_gate(pre.data_ptr<float>(), bias.data_ptr<float>(), a_log.data_ptr<float>(), g.data_ptr<float>(), T, HD,
                 (int)dk, stream());
  return g;
}

// u [T, C] (a column slice of a GEMM output is fine), w float [C, taps], state [slots, taps-1, C] in u's dtype
// (updated in place), segs = [[c0, heads, head width, mode]...], seg_w / seg_scale per segment.
Tensor short_conv(Tensor u, Tensor w, optional<Tensor> state, std::vector<std::vector<int64_t>> segs,
                  std::vector<optional<Tensor>> seg_w, std::vector<double> seg_scale, std::vector<Tensor> desc,
                  optional<Tensor> live, double eps, bool out_f32, optional<Tensor> bias) {
  const int code = code_of(u);
  TORCH_CHECK(u.dim() == 2, "u: [T, C]");
  const int64_t T = u.size(0), C = u.size(1);
  rows(u, T, C, code, "u");
  f32c(w, "conv weight");
  TORCH_CHECK(w.dim() == 2 && w.size(0) == C, "conv weight: [C, taps]");
  const int taps = (int)w.size(1);
  TORCH_CHECK(taps >= 1 && taps <= seq_conv_max_taps(), "conv taps out of range");
  const float* bp = nullptr;
  if (bias && bias->defined()) {
    f32c(*bias, "conv bias");
    TORCH_CHECK(bias->numel() == C, "conv bias: [C]");
    bp = bias->data_ptr<float>();
  }
  SeqDesc d = desc_of(desc, live, T);
  void* sp = nullptr;
  if (taps > 1) {
    TORCH_CHECK(state && state->defined() && state->is_cuda() && state->is_contiguous() && state->dim() == 3 &&
                    state->size(1) == taps - 1 && state->size(2) == C && code_of(*state) == code,
                "conv state: [slots, taps-1, C] in the input's dtype");
    sp = state->data_ptr();
  }
  const int nseg = (int)segs.size();
  TORCH_CHECK(nseg >= 1 && nseg <= 3 && (int)seg_w.size() == nseg && (int)seg_scale.size() == nseg, "1-3 segments");
  int flat[12];
  const float* wp[3];
  float sc[3];
  int64_t c = 0;
  for (int i = 0; i < nseg; ++i) {
    TORCH_CHECK(segs[i].size() == 4 && segs[i][0] == c && segs[i][2] >= 1 && segs[i][2] <= seq_conv_max_head(),
                "segments must tile the channels; head width <= ", seq_conv_max_head());
    for (int j = 0; j < 4; ++j) flat[4 * i + j] = (int)segs[i][j];
    c += segs[i][1] * segs[i][2];
    wp[i] = nullptr;
    if (segs[i][3] == 1) {
      TORCH_CHECK(seg_w[i] && seg_w[i]->defined(), "mode 1 needs a norm weight");
      f32c(*seg_w[i], "segment norm weight");
      TORCH_CHECK(seg_w[i]->numel() == segs[i][2], "segment norm weight size");
      wp[i] = seg_w[i]->data_ptr<float>();
    }
    sc[i] = (float)seg_scale[i];
  }
  TORCH_CHECK(c == C, "segments must cover all channels");
  auto out = at::empty({T, C}, u.options().dtype(out_f32 ? at::kFloat : u.scalar_type()));
  seq_short_conv(code, out_f32 ? 1 : 0, u.data_ptr(), ld(u), w.data_ptr<float>(), bp, sp, out.data_ptr(), (int)C, taps, nseg,
                 flat, wp, sc, d, (float)eps, stream());
  return out;
}

static void check_state(const Tensor& S, int64_t H, int64_t dv, int64_t dk) {
  f32c(S, "state");
  TORCH_CHECK(S.dim() == 4 && S.size(1) == H && S.size(2) == dv && S.size(3) == dk, "state: [slots, H, dv, dk]");
}

// returns {numerators S^T q [T, H, dv], n.q [T, H], e^-m [T, H]}: the read-out kernel divides
std::vector<Tensor> mlstm_scan(Tensor q, Tensor k, Tensor v, Tensor ipre, Tensor fpre, Tensor ib, Tensor fb, double cap,
                  double qscale, Tensor S, Tensor N, Tensor M, int64_t H, std::vector<Tensor> desc,
                  optional<Tensor> live) {
  const int code = code_of(q);
  const int64_t T = q.size(0);
  TORCH_CHECK(q.dim() == 2 && q.size(1) % H == 0 && v.dim() == 2 && v.size(1) % H == 0, "q/k/v: [T, H * d]");
  const int64_t dk = q.size(1) / H, dv = v.size(1) / H;
  rows(q, T, H * dk, code, "q");
  rows(k, T, H * dk, code, "k");
  rows(v, T, H * dv, code, "v");
  f32c(ipre, "ipre");
  f32c(fpre, "fpre");
  f32c(ib, "ib");
  f32c(fb, "fb");
  TORCH_CHECK(ipre.numel() == T * H && fpre.numel() == T * H && ib.numel() == H && fb.numel() == H, "gate sizes");
  TORCH_CHECK(dk <= seq_scan_max_dk(), "mlstm: key size above ", seq_scan_max_dk());
  TORCH_CHECK(cap > 0, "gate cap must be positive");
  check_state(S, H, dv, dk);
  f32c(N, "n");
  f32c(M, "m");
  TORCH_CHECK(N.numel() == S.size(0) * H * dk && M.numel() == S.size(0) * H, "n / m state sizes");
  SeqDesc d = desc_of(desc, live, T);
  auto out = at::empty({T, H, dv}, S.options());
  auto den = at::empty({T, H}, S.options()), efl = at::empty({T, H}, S.options());
  seq_mlstm_scan(code, q.data_ptr(), ld(q), k.data_ptr(), ld(k), v.data_ptr(), ld(v), ipre.data_ptr<float>(),
                 fpre.data_ptr<float>(), ib.data_ptr<float>(), fb.data_ptr<float>(), (float)cap, (float)qscale,
                 S.data_ptr<float>(), N.data_ptr<float>(), M.data_ptr<float>(), out.data_ptr<float>(),
                 den.data_ptr<float>(), efl.data_ptr<float>(), (int)H, (int)dk, (int)dv, d, stream());
  return {out, den, efl};
}

Tensor delta_scan(Tensor q, Tensor k, Tensor v, Tensor g, Tensor bpre, Tensor S, int64_t H, int64_t G,
                  std::vector<Tensor> desc, optional<Tensor> live) {
  const int code = code_of(q);
  const int64_t T = q.size(0);
  TORCH_CHECK(G >= 1 && H % G == 0 && q.dim() == 2 && q.size(1) % G == 0 && v.dim() == 2 && v.size(1) % H == 0,
              "q/k: [T, G * dk], v: [T, H * dv]");
  const int64_t dk = q.size(1) / G, dv = v.size(1) / H;
  rows(q, T, G * dk, code, "q");
  rows(k, T, G * dk, code, "k");
  rows(v, T, H * dv, code, "v");
  f32c(g, "g");
  f32c(bpre, "bpre");
  TORCH_CHECK(g.numel() == T * H * dk && bpre.numel() == T * H, "decay / beta sizes");
  TORCH_CHECK(dk <= seq_scan_max_dk(), "delta rule: key size above ", seq_scan_max_dk());
  check_state(S, H, dv, dk);
  SeqDesc d = desc_of(desc, live, T);
  auto out = at::empty({T, H, dv}, S.options());
  seq_delta_scan(code, q.data_ptr(), ld(q), k.data_ptr(), ld(k), v.data_ptr(), ld(v), g.data_ptr<float>(),
                 bpre.data_ptr<float>(), S.data_ptr<float>(), out.data_ptr<float>(), (int)H, (int)G, (int)dk, (int)dv, d,
                 stream());
  return out;
}

// q [T, H*dk]; kc [slots, max_len, G*dk], vc [slots, max_len, G*dv] already hold this step's keys and values
// tiles (optional): [tile_seq, tile_t0] int32 — runs of up to 32 consecutive tokens of one sequence that cover the step
Tensor talk_attention(Tensor q, Tensor kc, Tensor vc, Tensor talk, Tensor gate, int64_t H, int64_t G, double scale,
                      int64_t nsplit, std::vector<Tensor> desc, std::vector<Tensor> tiles) {
  const int code = code_of(q);
  const int64_t T = q.size(0);
  TORCH_CHECK(G >= 1 && H % G == 0 && q.dim() == 2 && q.size(1) % H == 0, "q: [T, H * dk]");
  const int64_t dk = q.size(1) / H;
  rows(q, T, H * dk, code, "q");
  TORCH_CHECK(kc.is_cuda() && kc.is_contiguous() && kc.dim() == 3 && kc.size(2) == G * dk && code_of(kc) == code,
              "key cache: [slots, max_len, G * dk]");
  TORCH_CHECK(vc.is_cuda() && vc.is_contiguous() && vc.dim() == 3 && vc.size(0) == kc.size(0) &&
                  vc.size(1) == kc.size(1) && vc.size(2) % G == 0 && code_of(vc) == code,
              "value cache: [slots, max_len, G * dv]");
  const int64_t dv = vc.size(2) / G, max_len = kc.size(1);
  TORCH_CHECK(G * dv <= seq_attn_max_cols(), "attention: G * dv above ", seq_attn_max_cols());
  TORCH_CHECK(H <= seq_attn_max_heads(), "attention: more than ", seq_attn_max_heads(), " heads");
  TORCH_CHECK(nsplit >= 1 && nsplit <= 1024, "nsplit");
  f32c(talk, "talk");
  TORCH_CHECK(talk.numel() == H * H, "talk: [H, H]");
  rows(gate, T, H * dv, code, "gate");
  SeqDesc d = desc_of(desc, optional<Tensor>(), T);
  const int* tseq = nullptr;
  const int* tt0 = nullptr;
  int ntiles = 0;
  if (tiles.size() == 2) {
    for (auto& t : tiles) TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), "tiles: int32");
    TORCH_CHECK(tiles[0].numel() == tiles[1].numel(), "tiles: two arrays of one length");
    tseq = tiles[0].data_ptr<int>();
    tt0 = tiles[1].data_ptr<int>();
    ntiles = (int)tiles[0].numel();
    TORCH_CHECK((int64_t)ntiles * 32 >= T && G * nsplit <= 65535, "tiles must cover the tokens");
  }
  auto fo = q.options().dtype(at::kFloat);
  auto pm = at::empty({T, H, nsplit}, fo), pl = at::empty({T, H, nsplit}, fo);
  auto pu = at::empty({T, H, nsplit, G * dv}, fo);
  auto out = at::empty({T, H * dv}, q.options());
  seq_talk_attention(code, q.data_ptr(), ld(q), kc.data_ptr(), vc.data_ptr(), pm.data_ptr<float>(),
                     pl.data_ptr<float>(), pu.data_ptr<float>(), talk.data_ptr<float>(), gate.data_ptr(), ld(gate),
                     out.data_ptr(), (int)H, (int)G, (int)dk, (int)dv, (int)max_len, (int)nsplit, (float)scale, tseq, tt0,
                     ntiles, d, stream());
  return out;
}

// ---- selective state space (state-space duality form): q = C, k = B [T, G * N], v = x [T, H * P], dtraw [T, H]
Tensor ssd_scan(Tensor q, Tensor k, Tensor v, Tensor dtraw, Tensor dt_bias, Tensor a_log, Tensor dskip, Tensor S,
                int64_t H, int64_t G, std::vector<Tensor> desc, optional<Tensor> live) {
  const int code = code_of(q);
  const int64_t T = q.size(0);
  TORCH_CHECK(G >= 1 && H % G == 0 && q.dim() == 2 && q.size(1) % G == 0 && v.dim() == 2 && v.size(1) % H == 0,
              "q/k: [T, G * N], v: [T, H * P]");
  const int64_t dk = q.size(1) / G, dv = v.size(1) / H;
  rows(q, T, G * dk, code, "C");
  rows(k, T, G * dk, code, "B");
  rows(v, T, H * dv, code, "x");
  rows(dtraw, T, H, code, "dt");
  f32c(dt_bias, "dt_bias");
  f32c(a_log, "A_log");
  f32c(dskip, "D");
  TORCH_CHECK(dt_bias.numel() == H && a_log.numel() == H && dskip.numel() == H, "per-head constants: [H]");
  TORCH_CHECK(dk <= seq_scan_max_dk(), "state size above ", seq_scan_max_dk());
  check_state(S, H, dv, dk);
  SeqDesc d = desc_of(desc, live, T);
  auto out = at::empty({T, H * dv}, S.options());
  seq_ssd_scan(code, q.data_ptr(), ld(q), k.data_ptr(), ld(k), v.data_ptr(), ld(v), dtraw.data_ptr(), ld(dtraw),
               dt_bias.data_ptr<float>(), a_log.data_ptr<float>(), dskip.data_ptr<float>(), S.data_ptr<float>(),
               out.data_ptr<float>(), (int)H, (int)G, (int)dk, (int)dv, d, stream());
  return out;
}

// returns {x float [T, W], h activation copy}; prev [slots] int32 (the token before a continued step), pair table
// [buckets + 1, W] or none
std::vector<Tensor> embed_pair(Tensor tok, Tensor table, optional<Tensor> pair, optional<Tensor> prev, double scale,
                               int64_t mul_prev, int64_t mul_cur, std::vector<Tensor> desc, optional<Tensor> live) {
  TORCH_CHECK(tok.is_cuda() && tok.scalar_type() == at::kLong && tok.is_contiguous(), "tokens: int64");
  TORCH_CHECK(table.is_cuda() && table.is_contiguous() && table.dim() == 2, "table");
  const int code = code_of(table);
  const int64_t T = tok.numel(), W = table.size(1);
  SeqDesc d = desc_of(desc, live, T);
  const void* pp = nullptr;
  int* sp = nullptr;
  long buckets = 0;
  if (pair && pair->defined()) {
    TORCH_CHECK(pair->is_cuda() && pair->is_contiguous() && pair->dim() == 2 && pair->size(1) == W &&
                    pair->size(0) >= 2 && code_of(*pair) == code, "pair table: [buckets + 1, W]");
    TORCH_CHECK(prev && prev->defined() && prev->is_cuda() && prev->scalar_type() == at::kInt && prev->is_contiguous(),
                "carried tokens: int32 [slots]");
    TORCH_CHECK(mul_prev >= 0 && mul_cur >= 0, "multipliers must not be negative");
    pp = pair->data_ptr();
    sp = prev->data_ptr<int>();
    buckets = pair->size(0) - 1;
  }
  auto x = at::empty({T, W}, table.options().dtype(at::kFloat));
  auto h = at::empty({T, W}, table.options());
  seq_embed_pair(code, tok.data_ptr<long>(), table.data_ptr(), pp, sp, x.data_ptr<float>(), h.data_ptr(), (int)W,
                 (float)scale, buckets, (long)mul_prev, (long)mul_cur, d, stream());
  return {x, h};
}

// x (float, in place) <- rms(alpha x + y) * w; returns its copy in the activation type (bf16 when out_bf16)
Tensor scaled_postnorm(Tensor x, Tensor y, Tensor w, double alpha, double eps, bool out_bf16) {
  f32c(x, "x");
  f32c(w, "w");
  const int W = (int)x.size(-1), T = (int)(x.numel() / W), code = out_bf16 ? 0 : 1;
  const bool yf = y.scalar_type() == at::kFloat;
  TORCH_CHECK(w.numel() == W, "norm weight size");
  TORCH_CHECK(y.is_cuda() && y.dim() == 2 && y.size(0) == T && y.size(1) == W && (T == 0 || y.stride(1) == 1) &&
                  (yf || code_of(y) == code), "y: [T, W], float or the activation type");
  auto h = at::empty({T, W}, x.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  seq_scaled_postnorm(code, yf ? 1 : 0, x.data_ptr<float>(), y.data_ptr(), ld(y), w.data_ptr<float>(), h.data_ptr(), T,
                      W, (float)alpha, (float)eps, stream());
  return h;
}

Tensor rms_act(Tensor u, Tensor w, double eps) {
  const int code = code_of(u);
  TORCH_CHECK(u.dim() == 2, "u: [T, n]");
  const int64_t T = u.size(0), n = u.size(1);
  rows(u, T, n, code, "u");
  f32c(w, "w");
  TORCH_CHECK(w.numel() == n, "norm weight size");
  auto out = at::empty({T, n}, u.options());
  seq_rms_act(code, u.data_ptr(), ld(u), w.data_ptr<float>(), out.data_ptr(), (int)T, (int)n, (float)eps, stream());
  return out;
}

Tensor gate_group_norm(Tensor y, Tensor z, Tensor w, int64_t parts, double eps) {
  f32c(y, "y");
  TORCH_CHECK(y.dim() == 2, "y: [T, n]");
  const int64_t T = y.size(0), n = y.size(1);
  const int code = code_of(z);
  rows(z, T, n, code, "z");
  f32c(w, "w");
  TORCH_CHECK(w.numel() == n && parts >= 1 && parts <= 65535 && n % parts == 0, "norm weight [n]; parts must divide n");
  auto out = at::empty({T, n}, z.options());
  seq_gate_group_norm(code, y.data_ptr<float>(), z.data_ptr(), ld(z), w.data_ptr<float>(), out.data_ptr(), (int)T, (int)n,
                      (int)parts, (float)eps, stream());
  return out;
}

// ---- latent attention over a cache of rows [c (R) | rotated shared key part (dr)]
static void check_latent_cache(const Tensor& cache, int64_t R, int64_t dr, int code) {
  TORCH_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 && cache.size(2) == R + dr &&
                  code_of(cache) == code, "latent cache: [slots, max_len, kv_rank + rot_dim]");
}
static void check_freq(const Tensor& f, int64_t dims, int64_t dr) {
  f32c(f, "inv_freq");
  TORCH_CHECK(dims >= 0 && dims % 2 == 0 && dims <= dr && f.numel() * 2 >= dims, "rotation: even dims <= rot_dim");
}

void latent_kv_store(Tensor u, Tensor w, Tensor inv_freq, Tensor cache, int64_t dims, double eps,
                     std::vector<Tensor> desc, bool half, double mag) {
  const int code = code_of(u);
  TORCH_CHECK(u.dim() == 2, "u: [T, kv_rank + rot_dim]");
  const int64_t T = u.size(0), R = w.numel(), dr = u.size(1) - R;
  TORCH_CHECK(dr >= 0, "down-projection narrower than the latent");
  rows(u, T, R + dr, code, "u");
  f32c(w, "w");
  check_freq(inv_freq, dims, dr);
  check_latent_cache(cache, R, dr, code);
  SeqDesc d = desc_of(desc, optional<Tensor>(), T);
  seq_latent_kv_store(code, u.data_ptr(), ld(u), w.data_ptr<float>(), inv_freq.data_ptr<float>(), cache.data_ptr(),
                      (int)R, (int)dr, (int)dims, (int)cache.size(1), (float)eps, half ? 1 : 0, (float)mag, d, stream());
}

// qa [H, T, R] (any strides with unit inner stride): the unrotated query parts already multiplied by W_uk;
// q [T, H * (dn + dr)]; gate [T, H] pre-activations or none.  Returns [T, H, R]: gate * softmax-weighted latents.
// half / mag: the rotation's layout and magnitude; window > 0 or sinks [H]: the grouped-query sweep (one kv head whose
// values are the first R columns of its key rows) with a sliding window and a sink score per head, no gate.
Tensor latent_attention(Tensor qa, Tensor q, Tensor cache, optional<Tensor> gate, Tensor inv_freq, int64_t H, int64_t dn,
                        int64_t dims, double scale, int64_t nsplit, std::vector<Tensor> desc, std::vector<Tensor> tiles,
                        bool half, double mag, int64_t window, optional<Tensor> sinks) {
  const int code = code_of(q);
  const int64_t T = q.size(0);
  TORCH_CHECK(qa.is_cuda() && qa.dim() == 3 && qa.size(0) == H && qa.size(1) == T && (qa.numel() == 0 || qa.stride(2) == 1) &&
                  code_of(qa) == code, "qa: [H, T, kv_rank]");
  const int64_t R = qa.size(2);
  TORCH_CHECK(q.dim() == 2 && q.size(1) % H == 0 && q.size(1) / H >= dn, "q: [T, H * (dim + rot_dim)]");
  const int64_t dr = q.size(1) / H - dn;
  rows(q, T, H * (dn + dr), code, "q");
  check_freq(inv_freq, dims, dr);
  check_latent_cache(cache, R, dr, code);
  TORCH_CHECK(R <= seq_attn_max_cols(), "attention: kv_rank above ", seq_attn_max_cols());
  TORCH_CHECK(nsplit >= 1 && nsplit <= 1024, "nsplit");
  const void* gp = nullptr;
  int ldg = 0;
  if (gate && gate->defined()) {
    rows(*gate, T, H, code, "gate");
    gp = gate->data_ptr();
    ldg = ld(*gate);
  }
  SeqDesc d = desc_of(desc, optional<Tensor>(), T);
  const int* tseq = nullptr;
  const int* tt0 = nullptr;
  int ntiles = 0;
  if (tiles.size() == 2) {
    for (auto& t : tiles) TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), "tiles: int32");
    TORCH_CHECK(tiles[0].numel() == tiles[1].numel(), "tiles: two arrays of one length");
    tseq = tiles[0].data_ptr<int>();
    tt0 = tiles[1].data_ptr<int>();
    ntiles = (int)tiles[0].numel();
    TORCH_CHECK((int64_t)ntiles * 32 >= T && nsplit <= 65535, "tiles must cover the tokens");
  }
  auto fo = q.options().dtype(at::kFloat);
  auto Q = at::empty({T, H * (R + dr)}, q.options());
  auto out = at::empty({T, H, R}, q.options());
  seq_latent_q_assemble(code, qa.data_ptr(), (size_t)qa.stride(0), (size_t)qa.stride(1), q.data_ptr(), ld(q), (int)dn,
                        inv_freq.data_ptr<float>(), Q.data_ptr(), (int)H, (int)R, (int)dr, (int)dims, half ? 1 : 0,
                        (float)mag, d, stream());
  const bool has_sinks = sinks && sinks->defined();
  if (window > 0 || has_sinks) {
    TORCH_CHECK(gp == nullptr && window >= 0, "latent attention: no per-head gate with a window or sinks");
    const float* sp = nullptr;
    if (has_sinks) {
      f32c(*sinks, "sinks");
      TORCH_CHECK(sinks->numel() == H, "sinks: [H]");
      sp = sinks->data_ptr<float>();
    }
    const bool direct = nsplit == 1 && tseq != nullptr && seq_attn_mfma_ok(code, (int)(H * (R + dr)), (int)(R + dr), (int)R) &&
                        (R + dr) % 8 == 0;
    const int64_t np = direct ? 0 : T;
    auto pm = at::empty({np, H, nsplit}, fo), pl = at::empty({np, H, nsplit}, fo), pu = at::empty({np, H, nsplit, R}, fo);
    seq_gqa_attention(code, Q.data_ptr(), (int)(H * (R + dr)), cache.data_ptr(), (int)(R + dr), cache.data_ptr(),
                      (int)(R + dr), pm.data_ptr<float>(), pl.data_ptr<float>(), pu.data_ptr<float>(), nullptr, 0, 0,
                      (int)window, has_sinks ? 1 : 0, 0.f, sp, out.data_ptr(), (int)(H * R), 1.f, (int)H, 1, (int)(R + dr),
                      (int)R, (int)cache.size(1), (int)nsplit, (float)scale, tseq, tt0, ntiles, d, stream());
    return out;
  }
  auto pm = at::empty({T, H, nsplit}, fo), pl = at::empty({T, H, nsplit}, fo), pu = at::empty({T, H, nsplit, R}, fo);
  seq_attn_sweep(code, Q.data_ptr(), (int)(H * (R + dr)), cache.data_ptr(), (int)(R + dr), cache.data_ptr(),
                 (int)(R + dr), pm.data_ptr<float>(), pl.data_ptr<float>(), pu.data_ptr<float>(), (int)H, 1,
                 (int)(R + dr), (int)R, (int)cache.size(1), (int)nsplit, (float)scale, tseq, tt0, ntiles, d, stream());
  seq_latent_merge(code, pm.data_ptr<float>(), pl.data_ptr<float>(), pu.data_ptr<float>(), gp, ldg, out.data_ptr(),
                   (int)T, (int)H, (int)R, (int)nsplit, stream());
  return out;
}

// ---- mixture of experts
static const float* check_routing(int64_t n, const optional<Tensor>& corr, int64_t top, int64_t groups, int64_t keep) {
  TORCH_CHECK(n >= 1 && n <= seq_route_max_outputs(), "router outputs above ", seq_route_max_outputs());
  TORCH_CHECK(top >= 1 && top <= n && top <= 64, "top");
  TORCH_CHECK(groups >= 1 && groups <= 64 && n % groups == 0 && keep >= 1 && keep <= groups, "groups must divide n");
  TORCH_CHECK(top <= keep * (n / groups), "fewer eligible outputs than `top`");
  if (corr && corr->defined()) {
    f32c(*corr, "correction");
    TORCH_CHECK(corr->numel() == n, "correction: [n]");
    return corr->data_ptr<float>();
  }
  return nullptr;
}

std::vector<Tensor> route_grouped(Tensor z, optional<Tensor> corr, int64_t top, int64_t groups, int64_t keep,
                                  double scale, int64_t kind) {
  TORCH_CHECK(kind >= 0 && kind < 8, "routing kind");
  f32c(z, "router logits");
  TORCH_CHECK(z.dim() == 2, "router logits: [T, n]");
  const int64_t T = z.size(0), n = z.size(1);
  const float* cp = check_routing(n, corr, top, groups, keep);
  auto idx = at::empty({T, top}, z.options().dtype(at::kInt));
  auto w = at::empty({T, top}, z.options());
  seq_route_grouped(z.data_ptr<float>(), cp, idx.data_ptr<int>(), w.data_ptr<float>(), (int)T, (int)n, (int)top,
                    (int)groups, (int)keep, (float)scale, (int)kind, stream());
  return {idx, w};
}

// the router product (float weights [n, W], activations h [T, W] as they are, float accumulation) and the routing
// the last `extra` router rows are not routed: their products come back as a third tensor, float [T, extra]
std::vector<Tensor> route_fused(Tensor h, Tensor router, optional<Tensor> corr, int64_t top, int64_t groups,
                                int64_t keep, double scale, int64_t kind, int64_t extra) {
  TORCH_CHECK(kind >= 0 && kind < 8, "routing kind");
  const int code = code_of(h);
  TORCH_CHECK(h.dim() == 2, "h: [T, W]");
  const int64_t T = h.size(0), W = h.size(1);
  rows(h, T, W, code, "h");
  f32c(router, "router");
  TORCH_CHECK(router.dim() == 2 && router.size(1) == W, "router: [n, W]");
  const int64_t n = router.size(0);
  TORCH_CHECK(extra >= 0 && extra < n && n <= seq_route_max_outputs(), "router rows");
  const float* cp = check_routing(n - extra, corr, top, groups, keep);
  auto idx = at::empty({T, top}, h.options().dtype(at::kInt));
  auto w = at::empty({T, top}, h.options().dtype(at::kFloat));
  auto ex = at::empty({T, extra}, h.options().dtype(at::kFloat));
  seq_route_fused(code, h.data_ptr(), ld(h), router.data_ptr<float>(), cp, idx.data_ptr<int>(), w.data_ptr<float>(),
                  (int)T, (int)n, (int)W, (int)top, (int)groups, (int)keep, (float)scale, (int)kind, (int)extra,
                  ex.data_ptr<float>(), stream());
  return {idx, w, ex};
}

static void check_route(const Tensor& idx, const Tensor& w, int64_t T) {
  TORCH_CHECK(idx.is_cuda() && idx.scalar_type() == at::kInt && idx.is_contiguous() && idx.dim() == 2 && idx.size(0) == T,
              "expert ids: int32 [T, top]");
  f32c(w, "weights");
  TORCH_CHECK(w.sizes() == idx.sizes(), "weights: [T, top]");
}

// few tokens: every (token, expert) pair streams its expert.  wgu [E, 2, F, W], wd [E, W, F]; returns float [T, W]
static const float* shared_gate_of(const optional<Tensor>& sg, int64_t T) {
  if (!(sg && sg->defined())) return nullptr;
  f32c(*sg, "shared gate");
  TORCH_CHECK(sg->numel() == T, "shared gate: float [T]");
  return sg->data_ptr<float>();
}

Tensor moe_pairs(Tensor h, Tensor wgu, Tensor wd, Tensor idx, Tensor w, optional<Tensor> shared, double limit,
                 int64_t mode, optional<Tensor> shared_gate) {
  TORCH_CHECK(mode == 1 || mode == 2, "expert activation: 1 clipped GLU, 2 SiLU GLU");
  const int code = code_of(h);
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.is_contiguous(), "h: [T, W] contiguous");
  const int64_t T = h.size(0), W = h.size(1);
  TORCH_CHECK(wgu.is_cuda() && wgu.is_contiguous() && wgu.dim() == 4 && wgu.size(1) == 2 && wgu.size(3) == W &&
                  code_of(wgu) == code, "wgu: [E, 2, F, W]");
  const int64_t E = wgu.size(0), F = wgu.size(2);
  TORCH_CHECK(wd.is_cuda() && wd.is_contiguous() && wd.dim() == 3 && wd.size(0) == E && wd.size(1) == W &&
                  wd.size(2) == F && code_of(wd) == code, "wd: [E, W, F]");
  check_route(idx, w, T);
  const int64_t top = idx.size(1);
  const void* sp = nullptr;
  if (shared && shared->defined()) {
    TORCH_CHECK(shared->is_cuda() && shared->is_contiguous() && shared->dim() == 2 && shared->size(0) == T &&
                    shared->size(1) == W && code_of(*shared) == code, "shared: [T, W]");
    sp = shared->data_ptr();
  }
  TORCH_CHECK(T * top <= 65535 && T <= 65535, "the pairs path is for few tokens");
  auto a = at::empty({T * top, F}, h.options());
  auto out = at::empty({T, W}, h.options().dtype(at::kFloat));
  seq_moe_pairs(code, h.data_ptr(), (int)W, wgu.data_ptr(), wd.data_ptr(), idx.data_ptr<int>(), w.data_ptr<float>(), sp,
                shared_gate_of(shared_gate, T), a.data_ptr(), out.data_ptr<float>(), (int)T, (int)top, (int)E, (int)F,
                (int)W, (float)limit, (int)mode, stream());
  return out;
}

// ys [rows, W]: expert outputs in expert-sorted order; pos [T, top] int64: the row of every pair
Tensor moe_combine_sorted(Tensor ys, Tensor pos, Tensor idx, Tensor w, Tensor h, optional<Tensor> shared, int64_t E,
                          optional<Tensor> shared_gate) {
  const int code = code_of(h);
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.is_contiguous(), "h: [T, W] contiguous");
  const int64_t T = h.size(0), W = h.size(1);
  check_route(idx, w, T);
  TORCH_CHECK(ys.is_cuda() && ys.is_contiguous() && ys.dim() == 2 && ys.size(1) == W && code_of(ys) == code, "ys: [rows, W]");
  TORCH_CHECK(pos.is_cuda() && pos.scalar_type() == at::kLong && pos.is_contiguous() && pos.numel() == idx.numel(),
              "pos: int64 [T, top]");
  const void* sp = nullptr;
  if (shared && shared->defined()) {
    TORCH_CHECK(shared->is_cuda() && shared->is_contiguous() && shared->dim() == 2 && shared->size(0) == T &&
                    shared->size(1) == W && code_of(*shared) == code, "shared: [T, W]");
    sp = shared->data_ptr();
  }
  auto out = at::empty({T, W}, h.options().dtype(at::kFloat));
  seq_moe_combine(code, ys.data_ptr(), pos.data_ptr<long>(), idx.data_ptr<int>(), w.data_ptr<float>(), h.data_ptr(),
                  (int)W, sp, shared_gate_of(shared_gate, T), out.data_ptr<float>(), (int)T, (int)idx.size(1), (int)E,
                  (int)W, stream());
  return out;
}

// mode 0: tanh-form GELU of z [T, F]; mode 1: clipped GLU, mode 2: SiLU GLU, mode 3: tanh-form GELU GLU of
// z [T, 2F] = [gate | up]
Tensor ff_act(Tensor z, int64_t mode, double limit) {
  TORCH_CHECK(z.is_cuda() && z.is_contiguous() && z.dim() == 2 &&
                  (mode == 0 || (mode >= 1 && mode <= 3 && z.size(1) % 2 == 0)), "z");
  const int64_t T = z.size(0), F = mode == 0 ? z.size(1) : z.size(1) / 2;
  auto out = at::empty({T, F}, z.options());
  seq_ff_act(code_of(z), z.data_ptr(), out.data_ptr(), (int)T, (int)F, (int)mode, (float)limit, stream());
  return out;
}

// ---- learned positions, several residual streams, q/k norm + cache write, biased block attention with a sink
Tensor embed_learned(Tensor tok, Tensor pos, Tensor table, Tensor ptable, int64_t streams) {
  TORCH_CHECK(tok.is_cuda() && tok.scalar_type() == at::kLong && tok.is_contiguous(), "tokens: int64");
  TORCH_CHECK(pos.is_cuda() && pos.scalar_type() == at::kInt && pos.is_contiguous() && pos.numel() == tok.numel(),
              "positions: int32, one per token");
  TORCH_CHECK(table.is_cuda() && table.is_contiguous() && table.dim() == 2 && ptable.is_cuda() && ptable.is_contiguous() &&
                  ptable.dim() == 2 && ptable.size(1) == table.size(1) && ptable.scalar_type() == table.scalar_type() &&
                  ptable.size(0) >= 1 && table.size(0) >= 1, "token and position tables: [rows, W], one dtype");
  TORCH_CHECK(streams >= 1 && streams <= seq_hyper_max_streams(), "streams: 1..", seq_hyper_max_streams());
  const int T = (int)tok.numel(), W = (int)table.size(1);
  auto x = at::empty({T, streams, W}, table.options().dtype(at::kFloat));
  seq_embed_learned(code_of(table), tok.data_ptr<long>(), pos.data_ptr<int>(), table.data_ptr(), ptable.data_ptr(),
                    x.data_ptr<float>(), T, W, (int)streams, (int)ptable.size(0), (int)table.size(0), stream());
  return x;
}

// X float [T, S, W] in place; y [T, W] (activation dtype or float) or none; returns the next sublayer's input [T, W]
Tensor hyper_mix_norm(Tensor X, optional<Tensor> y, optional<Tensor> mix, optional<Tensor> outw, Tensor read, Tensor w,
                      double eps, bool out_bf16) {
  f32c(X, "streams");
  TORCH_CHECK(X.dim() == 3, "streams: [T, S, W]");
  const int64_t T = X.size(0), S = X.size(1), W = X.size(2);
  TORCH_CHECK(S >= 1 && S <= seq_hyper_max_streams(), "streams: 1..", seq_hyper_max_streams());
  f32c(read, "read weights");
  f32c(w, "norm weight");
  TORCH_CHECK(read.numel() == S && w.numel() == W, "read weights [S], norm weight [W]");
  const void* yp = nullptr;
  const float* mp = nullptr;
  const float* op = nullptr;
  int ldy = 0, y_f32 = 0;
  if (y && y->defined()) {
    TORCH_CHECK(mix && mix->defined() && outw && outw->defined(), "a sublayer output needs mix and out weights");
    f32c(*mix, "mix");
    f32c(*outw, "out weights");
    TORCH_CHECK(mix->numel() == S * S && outw->numel() == S, "mix [S, S], out weights [S]");
    y_f32 = y->scalar_type() == at::kFloat;
    rows(*y, T, W, code_of(*y), "y");
    TORCH_CHECK(y_f32 || !out_bf16 || y->scalar_type() == at::kBFloat16, "y: float or the activation dtype");
    TORCH_CHECK(y_f32 || (code_of(*y) == (out_bf16 ? 0 : 1)), "y: float or the activation dtype");
    yp = y->data_ptr();
    ldy = ld(*y);
    mp = mix->data_ptr<float>();
    op = outw->data_ptr<float>();
  }
  auto h = at::empty({T, W}, X.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  seq_hyper_mix_norm(out_bf16 ? 0 : 1, y_f32, X.data_ptr<float>(), yp, ldy, mp, op, read.data_ptr<float>(),
                     w.data_ptr<float>(), h.data_ptr(), (int)T, (int)W, (int)S, (float)eps, stream());
  return h;
}

static void check_kv_cache(const Tensor& c, int64_t cols, int code, const char* n) {
  TORCH_CHECK(c.is_cuda() && c.is_contiguous() && c.dim() == 3 && c.size(2) == cols && code_of(c) == code, n,
              ": [slots, max_len, columns] in the activation dtype");
}

// u [T, nq + nk + nv]; returns the normed q [T, nq]; k and v rows go to the caches at each token's (slot, position).
// Slots are rows of the engine's pool (SeqBatch checks them on the host); the kernel skips positions outside the cache.
Tensor qk_norm_store(Tensor u, int64_t nq, int64_t nk, Tensor qw, Tensor kw, Tensor kc, Tensor vc,
                     optional<Tensor> vfirst, optional<Tensor> lam, double eps, std::vector<Tensor> desc) {
  const int code = code_of(u);
  TORCH_CHECK(u.dim() == 2 && nq >= 1 && nk >= 1 && u.size(1) > nq + nk, "u: [T, nq + nk + nv]");
  const int64_t T = u.size(0), nv = u.size(1) - nq - nk;
  rows(u, T, nq + nk + nv, code, "u");
  f32c(qw, "q norm weight");
  f32c(kw, "k norm weight");
  TORCH_CHECK(qw.numel() == nq && kw.numel() == nk, "norm weights: [nq], [nk]");
  check_kv_cache(kc, nk, code, "key cache");
  check_kv_cache(vc, nv, code, "value cache");
  TORCH_CHECK(vc.size(0) == kc.size(0) && vc.size(1) == kc.size(1), "caches: one pool of slots");
  const void* fp = nullptr;
  const float* lp = nullptr;
  if (vfirst && vfirst->defined()) {
    check_kv_cache(*vfirst, nv, code, "first value cache");
    TORCH_CHECK(vfirst->sizes() == vc.sizes() && lam && lam->defined(), "first value cache: the value cache's shape");
    f32c(*lam, "lambda");
    TORCH_CHECK(lam->numel() == 1, "lambda: one float");
    fp = vfirst->data_ptr();
    lp = lam->data_ptr<float>();
  }
  SeqDesc d = desc_of(desc, optional<Tensor>(), T);
  auto q = at::empty({T, nq}, u.options());
  seq_qk_norm_store(code, u.data_ptr(), ld(u), qw.data_ptr<float>(), kw.data_ptr<float>(), q.data_ptr(), kc.data_ptr(),
                    vc.data_ptr(), fp, lp, (int)nq, (int)nk, (int)nv, (int)kc.size(1), (float)eps, d, stream());
  return q;
}

Tensor biased_attention(Tensor q, Tensor kc, Tensor vc, optional<Tensor> bias, int64_t H, int64_t G, double scale,
                        int64_t block, bool sink, double sink_logit, int64_t nsplit, std::vector<Tensor> desc,
                        std::vector<Tensor> tiles, int64_t window, optional<Tensor> sinks, optional<Tensor> out_,
                        double out_scale) {
  const int code = code_of(q);
  TORCH_CHECK(q.dim() == 2 && H >= 1 && G >= 1 && H % G == 0 && q.size(1) % H == 0, "q: [T, H * dk]");
  const int64_t T = q.size(0), dk = q.size(1) / H;
  rows(q, T, H * dk, code, "q");
  check_kv_cache(kc, G * dk, code, "key cache");
  TORCH_CHECK(vc.is_cuda() && vc.is_contiguous() && vc.dim() == 3 && vc.size(0) == kc.size(0) && vc.size(1) == kc.size(1) &&
                  vc.size(2) % G == 0 && code_of(vc) == code, "value cache: [slots, max_len, G * dv]");
  const int64_t dv = vc.size(2) / G, max_len = kc.size(1);
  TORCH_CHECK(dv >= 1 && dv <= seq_attn_max_cols(), "attention: dv above ", seq_attn_max_cols());
  TORCH_CHECK(nsplit >= 1 && nsplit <= 1024 && block >= 0 && window >= 0, "nsplit, block, window");
  const float* sp = nullptr;
  if (sinks && sinks->defined()) {
    f32c(*sinks, "sinks");
    TORCH_CHECK(sink && sinks->numel() == H, "sinks: [H]");
    sp = sinks->data_ptr<float>();
  }
  const float* bp = nullptr;
  int nd = 0;
  if (bias && bias->defined()) {
    f32c(*bias, "distance bias");
    TORCH_CHECK(bias->dim() == 2 && bias->size(0) == H && bias->size(1) >= 1, "distance bias: [H, distances]");
    bp = bias->data_ptr<float>();
    nd = (int)bias->size(1);
  }
  SeqDesc d = desc_of(desc, optional<Tensor>(), T);
  const int* tseq = nullptr;
  const int* tt0 = nullptr;
  int ntiles = 0;
  if (tiles.size() == 2) {
    for (auto& t : tiles) TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), "tiles: int32");
    TORCH_CHECK(tiles[0].numel() == tiles[1].numel(), "tiles: two arrays of one length");
    tseq = tiles[0].data_ptr<int>();
    tt0 = tiles[1].data_ptr<int>();
    ntiles = (int)tiles[0].numel();
    TORCH_CHECK((int64_t)ntiles * 32 >= T && nsplit <= 65535 && H <= 65535, "tiles must cover the tokens");
  }
  auto fo = q.options().dtype(at::kFloat);
  Tensor out;
  if (out_ && out_->defined()) {                     // a column slice of a wider matrix
    out = *out_;
    rows(out, T, H * dv, code, "out");
  } else {
    out = at::empty({T, H * dv}, q.options());
  }
  const int ldo = T == 0 ? (int)(H * dv) : ld(out);
  if (ldo % 4 != 0 || ((uintptr_t)out.data_ptr() & 7) != 0) tseq = nullptr;    // the matrix-core sweep stores 8 bytes
  // one key split on the matrix-core sweep writes the output itself: no partial sums
  const bool direct = nsplit == 1 && tseq != nullptr && seq_attn_mfma_ok(code, ld(q), (int)dk, (int)dv) &&
                      (G * dk) % 8 == 0 && (G * dv) % 8 == 0;
  const int64_t np = direct ? 0 : T;
  auto pm = at::empty({np, H, nsplit}, fo), pl = at::empty({np, H, nsplit}, fo);
  auto pu = at::empty({np, H, nsplit, dv}, fo);
  seq_gqa_attention(code, q.data_ptr(), ld(q), kc.data_ptr(), (int)(G * dk), vc.data_ptr(), (int)(G * dv),
                    pm.data_ptr<float>(), pl.data_ptr<float>(), pu.data_ptr<float>(), bp, nd, (int)block, (int)window,
                    sink ? 1 : 0, (float)sink_logit, sp, out.data_ptr(), ldo, (float)out_scale, (int)H, (int)G, (int)dk,
                    (int)dv, (int)max_len, (int)nsplit, (float)scale, tseq, tt0, ntiles, d, stream());
  return out;
}

// u [T, nq + nk (+ nv)]: rotated q returned, rotated k and the values (u's v columns, or the k columns as they came) go
// to the caches at each token's (slot, position)
Tensor rope_kv_store(Tensor u, int64_t nq, int64_t nk, int64_t H, int64_t G, Tensor inv_freq, int64_t dims, Tensor kc,
                     Tensor vc, std::vector<Tensor> desc, bool half, double mag, bool values_are_keys) {
  const int code = code_of(u);
  TORCH_CHECK(u.dim() == 2 && H >= 1 && G >= 1 && nq % H == 0 && nk % G == 0 && nq / H == nk / G &&
                  u.size(1) >= nq + nk, "u: [T, H * dk + G * dk (+ nv)]");
  const int64_t T = u.size(0), nv = values_are_keys ? nk : u.size(1) - nq - nk, dk = nq / H;
  TORCH_CHECK(nv >= 1, "no value columns");
  rows(u, T, u.size(1), code, "u");
  check_freq(inv_freq, dims, dk);
  check_kv_cache(kc, nk, code, "key cache");
  check_kv_cache(vc, nv, code, "value cache");
  TORCH_CHECK(vc.size(0) == kc.size(0) && vc.size(1) == kc.size(1), "caches: one pool of slots");
  SeqDesc d = desc_of(desc, optional<Tensor>(), T);
  auto q = at::empty({T, nq}, u.options());
  seq_rope_kv_store(code, u.data_ptr(), ld(u), inv_freq.data_ptr<float>(), q.data_ptr(), kc.data_ptr(), vc.data_ptr(),
                    (int)nq, (int)nk, (int)nv, (int)dk, (int)dims, half ? 1 : 0, (float)mag, values_are_keys ? 1 : 0,
                    (int)kc.size(1), d, stream());
  return q;
}

Tensor sigmoid_gate(Tensor y, Tensor gate) {
  const int code = code_of(y);
  TORCH_CHECK(y.is_cuda() && y.is_contiguous() && y.dim() == 2, "y: [T, C], contiguous");
  const int64_t T = y.size(0), C = y.size(1);
  rows(gate, T, C, code, "gate");
  auto out = at::empty_like(y);
  seq_sigmoid_gate(code, y.data_ptr(), gate.data_ptr(), T == 0 ? (int)C : ld(gate), out.data_ptr(), (int)T, (int)C, stream());
  return out;
}

// returns {w, a} float [T, H * dk] and kinv float [T, H]
std::vector<Tensor> delta_rule_gates(Tensor k, Tensor low, optional<Tensor> up, optional<Tensor> wb, Tensor apre,
                                     optional<Tensor> ab, int64_t H, double dscale) {
  const int code = code_of(k);
  TORCH_CHECK(k.dim() == 2 && H >= 1 && k.size(1) % H == 0, "k: [T, H * dk]");
  const int64_t T = k.size(0), C = k.size(1), dk = C / H;
  TORCH_CHECK(dk <= seq_scan_max_dk(), "key size above ", seq_scan_max_dk());
  rows(k, T, C, code, "k");
  rows(apre, T, C, code, "a_pre");
  const float* upp = nullptr;
  int64_t rank = 0;
  const int low_f32 = low.scalar_type() == at::kFloat;
  if (up && up->defined()) {
    f32c(*up, "w_up");
    TORCH_CHECK(up->dim() == 2 && up->size(0) == C, "w_up: [H * dk, rank]");
    rank = up->size(1);
    upp = up->data_ptr<float>();
    rows(low, T, rank, low_f32 ? 1 : code, "w_low");
  } else {
    rows(low, T, C, low_f32 ? 1 : code, "w_pre");
  }
  const float* wbp = nullptr;
  const float* abp = nullptr;
  if (wb && wb->defined()) {
    f32c(*wb, "w_bias");
    TORCH_CHECK(wb->numel() == C, "w_bias: [H * dk]");
    wbp = wb->data_ptr<float>();
  }
  if (ab && ab->defined()) {
    f32c(*ab, "a_bias");
    TORCH_CHECK(ab->numel() == C, "a_bias: [H * dk]");
    abp = ab->data_ptr<float>();
  }
  auto fo = k.options().dtype(at::kFloat);
  auto w = at::empty({T, C}, fo), a = at::empty({T, C}, fo), kinv = at::empty({T, H}, fo);
  seq_delta_gates(code, low_f32, k.data_ptr(), T == 0 ? (int)C : ld(k), low.data_ptr(), T == 0 ? 1 : ld(low), upp,
                  (int)rank, wbp, apre.data_ptr(), T == 0 ? (int)C : ld(apre), abp, w.data_ptr<float>(),
                  a.data_ptr<float>(), kinv.data_ptr<float>(), (int)T, (int)H, (int)dk, (float)dscale, stream());
  return {w, a, kinv};
}

// r, k [T, H * dk], v [T, H * dv]; w, a float [T, H * dk], kinv float [T, H]; S float [slots, H, dv, dk] in place
Tensor general_delta_scan(Tensor r, Tensor k, Tensor v, Tensor w, Tensor a, Tensor kinv, Tensor S, int64_t H,
                          std::vector<Tensor> desc, optional<Tensor> live) {
  const int code = code_of(r);
  const int64_t T = r.size(0);
  TORCH_CHECK(H >= 1 && r.dim() == 2 && r.size(1) % H == 0 && v.dim() == 2 && v.size(1) % H == 0,
              "r/k: [T, H * dk], v: [T, H * dv]");
  const int64_t dk = r.size(1) / H, dv = v.size(1) / H;
  rows(r, T, H * dk, code, "r");
  rows(k, T, H * dk, code, "k");
  rows(v, T, H * dv, code, "v");
  f32c(w, "w");
  f32c(a, "a");
  f32c(kinv, "kinv");
  TORCH_CHECK(w.numel() == T * H * dk && a.numel() == T * H * dk && kinv.numel() == T * H, "w, a: [T, H * dk], kinv: [T, H]");
  TORCH_CHECK(dk <= seq_scan_max_dk(), "key size above ", seq_scan_max_dk());
  check_state(S, H, dv, dk);
  SeqDesc d = desc_of(desc, live, T);
  auto out = at::empty({T, H, dv}, S.options());
  seq_gdr_scan(code, r.data_ptr(), ld(r), k.data_ptr(), ld(k), v.data_ptr(), ld(v), w.data_ptr<float>(),
               a.data_ptr<float>(), kinv.data_ptr<float>(), S.data_ptr<float>(), out.data_ptr<float>(), (int)H, (int)dk,
               (int)dv, d, stream());
  return out;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_sincos", &embed_sincos);
  m.def("rms_f32", &rms_f32);
  m.def("gated_residual", &gated_residual);
  m.def("dual_norm_mean", &dual_norm_mean);
  m.def("polynorm", &polynorm);
  m.def("head_norm_gate", &head_norm_gate);
  m.def("decay_gate", &decay_gate);
  m.def("short_conv", &short_conv, py::arg("u"), py::arg("w"), py::arg("state"), py::arg("segs"), py::arg("seg_w"),
        py::arg("seg_scale"), py::arg("desc"), py::arg("live"), py::arg("eps"), py::arg("out_f32"),
        py::arg("bias") = py::none());
  m.def("mlstm_scan", &mlstm_scan);
  m.def("delta_scan", &delta_scan);
  m.def("talk_attention", &talk_attention);
  m.def("ssd_scan", &ssd_scan);
  m.def("embed_pair", &embed_pair);
  m.def("scaled_postnorm", &scaled_postnorm);
  m.def("rms_act", &rms_act);
  m.def("gate_group_norm", &gate_group_norm);
  m.def("latent_kv_store", &latent_kv_store);
  m.def("latent_attention", &latent_attention);
  m.def("route_grouped", &route_grouped);
  m.def("route_fused", &route_fused);
  m.def("moe_pairs", &moe_pairs);
  m.def("moe_combine_sorted", &moe_combine_sorted);
  m.def("ff_act", &ff_act);
  m.def("embed_learned", &embed_learned);
  m.def("hyper_mix_norm", &hyper_mix_norm);
  m.def("qk_norm_store", &qk_norm_store);
  m.def("biased_attention", &biased_attention);
  m.def("rope_kv_store", &rope_kv_store);
  m.def("sigmoid_gate", &sigmoid_gate);
  m.def("delta_rule_gates", &delta_rule_gates);
  m.def("general_delta_scan", &general_delta_scan);
}
