// tl_stack.hip — the layer-list engine: a decoder described layer by layer (tl_stack_config) instead of by the fixed Llama
// block of tl_model.hip. It owns the bf16 weights, the per-layer FP32 caches and recurrent states and the chunk workspaces,
// and runs T tokens through all layers: T = 1 is the decode step (GEMVs, position and token id read from the device, so the
// step can be captured into a hipGraph by tl_model.hip like the Llama step), T > 1 a chunk of a prompt (MFMA GEMMs).
//
// Blocks  TL_BLOCK_POST_NORM  x += norm1(mixer(x)); x += norm2(ff(x))   -- the sublayers read x itself, RMS norm on their OUTPUT
//         TL_BLOCK_PRE_NORM   x += mixer(norm1(x)); x += ff(norm2(x))   -- a layer norm in FRONT of each sublayer; the launch that
//                             finishes x also writes the norm of whatever reads x next (norm2, or the next layer's norm1)
//         TL_BLOCK_PARALLEL   h = norm1(x); x += mixer(h) + ff(h)       -- one Dynamic Tanh norm, both sublayers read its output;
//                             the norm of the NEXT block rides in the launch that finishes x (it is elementwise)
// Mixers  TL_MIXER_SWA    q | k (| v) = W h in one product; either the whole-projection q/k RMS norm with optional value mixing
//                         (tl_norm.hip), or rotary positions + per-head unit norm, values optionally the keys as projected
//                         (tl_rope.hip); k, v -> cache; windowed attention with softmax or sigmoid weights, optionally with
//                         the first keys kept visible (tl_swa.hip); W_o
//         TL_MIXER_DELTA  q | k | v | beta | a1 | g1 = W h in one product, a2 and g2 behind a1 and g1; convolution, unit norms
//                         and decay (delta_pre), the recurrence over a per-head state (delta_scan), gated head norm; W_o
//         TL_MIXER_LATENT query latent | key/value latent | rotated shared key part | head gates = W h in one product; norms,
//                         rotation and the cache row (tl_latent.hip); queries up-projected, their plain part absorbed through
//                         W_uk^T per head; attention over the cached latent rows themselves (tl_swa.hip, one "head" of keys whose
//                         values are the first kv_rank columns); W_uv per head, head gates, W_o. A layer may read an earlier
//                         latent layer's cache (kv_from) and then projects no latent of its own
//         TL_MIXER_GDELTA r | k | v | gate | a | w1 = W h in one product (tanh on the w1 rows in its epilogue), w2 behind w1;
//                         gdelta_pre, gdelta_scan over a per-head state, gated head norm with weights per head; W_o
//         TL_MIXER_LINEAR gated linear attention: q | f | v = W h in one product; silu, forget gate and what it writes (linear_pre);
//                         the delta rule's scan without its removal step; RMS norm per head; W_o
//         TL_MIXER_SWA with its options: two score maps per head over the same values (differential attention: one attention
//                         launch per map, then (a1 - lambda a2) / rms (1 - diff) sigmoid(gate)), a norm per head and map, biases
//                         and a causal convolution on q, k, v (tl_conv.hip), capped scores, a logarithmic distance bias, a learned
//                         sink per head; TL_MIXER_DELTA with one decay per head and direct projections for decay and gate
//         Two mixers side by side (tl_layer_spec::side): both read the same input, their first products are one product, the
//                         layer's mixer output is mix_scale * first + side_scale * second
//         Pre-norm blocks behind the plain RMS norm (TL_NORM_RMS) may add a causal convolution over time to what each sublayer
//                         reads (canon_taps); the embedding row may be scaled (embed_scale)
// Feed-forward  TL_MLP_UNIT  W_down act(W_up h), the activation in the first product's epilogue (pre-norm blocks)
//               TL_MLP_MOE  router (three kinds, tl_moe.hip) -> top experts (gated units) + optional shared expert, optionally
//                           gated per token;  TL_MLP_DENSE  one gated unit (it runs where a shared expert would)
// A layer may use an earlier layer's tensors (weights_of) with a cache or state of its own.
// The residual stream, norms, router, attention scores, caches and states are FP32; matrix operands of a prompt chunk are bf16
// (terms = 1) or the FP32-grade three-term split (terms = 3), see tl_dense.hip; the decode step's GEMVs are FP32 throughout.
//
// Cache and state: one allocation. Attention layers: K [max_positions][kv_heads * dim] and V [max_positions][kv_heads * vdim],
// flat by absolute position; a window only bounds what attention reads. Delta layers: S [heads][vdim][dim] and the
// convolution's last taps - 1 inputs (linear attention: S only; attention with a convolution on q, k, v: that history too;
// every layer: the histories of the convolutions on what its sublayers read); latent layers with a projection of their
// own: rows [max_positions][kv_rank + rot_dim]; generalized delta layers: S [heads][dim][dim]. tl_stack_reset gives everything back (one sequence at a time): zeros are the state of
// an empty sequence.
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <memory>
#include <set>
#include <string>
#include <vector>

#include "tl_stack.h"

namespace {

struct Layer {
  tl_layer_spec sp;
  int wsrc = 0;                        // layer whose tensors this one uses (itself unless weights_of)
  int qd = 0, kd = 0, vd = 0, od = 0;  // q / k / v projection sizes, mixer output size (heads * vdim)
  int pd = 0;                          // rows of the first product (q | k | v, plus beta | a1 | g1 for the delta rule)
  int vmix_mode = 0;                   // 0 none, 1 first mixing layer, 2 mixes with the first
  bool rotary_path = false;            // tl_rope.hip prepares q / k (otherwise tl_norm.hip's qkv_post)
  uint16_t *wqkv = nullptr, *wo = nullptr;
  float *q_norm = nullptr, *k_norm = nullptr, *lambda = nullptr, *norm1 = nullptr, *norm2 = nullptr;
  float *norm1_b = nullptr, *norm1_alpha = nullptr;  // Dynamic Tanh
  float* pb = nullptr;                               // sigmoid bias per head
  double* freq = nullptr;                            // rotary frequencies
  float mscale = 1.0f;
  uint16_t *wa2 = nullptr, *wg2 = nullptr, *conv = nullptr;  // delta rule
  float *a_log = nullptr, *dt_bias = nullptr, *onorm = nullptr;
  uint16_t *router = nullptr, *gu = nullptr, *down = nullptr, *sgu = nullptr, *sdown = nullptr, *sg = nullptr;
  float* router_b = nullptr;
  float *kc = nullptr, *vc = nullptr;        // attention: caches
  float *state = nullptr, *hist = nullptr;   // delta rule: S and the convolution's history
  float *norm2_b = nullptr;                  // layer norm
  // latent attention: wqkv = dq | dkv | g stacked; wuq [heads * (dim + rot_dim)][q_rank]; wukt [heads][kv_rank][dim] (the
  // TRANSPOSE of each head's block of mix.uk: the query of a decode step is absorbed through it); wuv [heads][vdim][kv_rank]
  // as stored
  uint16_t *wuq = nullptr, *wuk = nullptr, *wukt = nullptr, *wuv = nullptr;  // (wuk as stored: the expanded keys of a chunk)
  float *dq_norm = nullptr, *dkv_norm = nullptr;
  float* ckv = nullptr;                      // cache rows [max_pos][kv_rank + rot_dim] (an owner's; kv_src's otherwise)
  int kv_src = -1;                           // the latent layer whose cache this one reads (itself unless kv_from)
  int gate_off = 0;                          // column of the head gates in the first product
  // generalized delta rule: wqkv = r | k | v | g | a | w1 stacked, wa2 = w2
  float *w0 = nullptr, *a_bias = nullptr;
  float act_p = 0.0f, act_q = 0.0f;          // TL_MLP_UNIT: the activation's two numbers, transformed (tl_act_kind)
  // windowed attention with its options: biases of q | k | v, a convolution on them (conv, hist above), distance bias, sink
  // scores per head; two score maps: lambda from four vectors kept on the host until all have arrived
  float *qkv_b = nullptr, *r1 = nullptr, *r2 = nullptr, *sinkv = nullptr;
  std::vector<float> lvec[4];
  float lam = 0.0f;
  float *lower = nullptr, *f_bias = nullptr;  // gated linear attention: lower bound and bias of the forget gate
  uint16_t *canon1 = nullptr, *canon2 = nullptr;          // convolutions on what the sublayers read [width][taps]
  float *canon_hist1 = nullptr, *canon_hist2 = nullptr;   // ... and their last taps - 1 inputs (state)
  std::unique_ptr<Layer> side;               // the second mixer of a pair: its mixer fields, tensors and state only
  std::set<std::string> expect, optional;    // tensor names (without the "l<i>." prefix) still missing / accepted and ignored
};

}  // namespace

struct TlStack {
  tl_stack_config cfg;
  std::vector<Layer> layers;
  uint16_t *embed = nullptr, *head = nullptr;
  float *embed_norm = nullptr, *embed_norm_b = nullptr, *final_norm = nullptr, *final_b = nullptr, *final_alpha = nullptr;
  int got_globals = 0, need_globals = 0;
  std::vector<void*> allocs;
  bool finalized = false;
  int terms = 1;
  // tokens of a prompt that go through the layers together. Measured at width 4096 with 16 experts (top 4): 105.9 k tokens/s
  // at 512, 140.4 k at 1024, 171.6 k at 2048 -- the experts' grouped GEMMs see 4 x the tokens per expert, the dense ones
  // enough tiles for the 128 x 128 shape.
  int chunk = 2048;
  int lead = 1;             // tokens of tl_stack_lead_tokens (TL_STACK_LEAD; 0: none)
  int exact_below = 64;     // portions shorter than this always multiply with three terms (TL_STACK_EXACT_BELOW; at least 2)
  bool gemv_decode = true;
  bool fuse_router = true;  // TL_STACK_FUSE_ROUTER=0: the router as a launch of its own (A/B, tests)
  bool fuse_canon = true;   // TL_STACK_FUSE_CANON=0: the convolution on what a sublayer reads as a launch of its own also for one token
  // One token through a parallel block: mixer and feed-forward read the same h and meet only in the residual sum, so the
  // feed-forward's launches go to a second stream (forked and joined by events; under capture they become a parallel branch
  // of the graph) and the step's critical path per layer is the longer of the two chains, not their sum. TL_STACK_FORK=0: one stream.
  bool fork = true;
  hipStream_t side = nullptr;
  hipEvent_t ev_fork = nullptr, ev_join = nullptr;
  // workspaces for one chunk
  float *x = nullptr, *qkv = nullptr, *att = nullptr, *proj = nullptr, *v_first = nullptr, *xn = nullptr;
  float *att2 = nullptr, *proj2 = nullptr;  // the second score map of differential attention; the second mixer of a pair
  float* hn = nullptr;      // the norm of x before the convolution on what a sublayer reads
  bool any_pair = false, any_maps = false;
  float* h = nullptr;       // norm-first blocks: the normalised input both sublayers read
  float *dq = nullptr, *da = nullptr, *dg = nullptr, *dbeta = nullptr, *ddecay = nullptr;  // delta rule
  float *lq = nullptr, *lqa = nullptr;      // latent attention: up-projected queries, absorbed queries
  float *lk = nullptr, *lv = nullptr;       // ... and, for long chunks, keys / values per head of every row the chunk sees
  int max_lk = 0, max_lv = 0;
  int latent_expand = 64;                   // chunks of at least this many tokens expand (TL_STACK_LATENT_EXPAND; 0: never)
  float *gw = nullptr, *gu = nullptr, *gau = nullptr, *grau = nullptr, *grk = nullptr;  // generalized delta rule (gdelta_pre)
  int max_lq = 0, max_lqa = 0, max_gd = 0, gdelta_layers = 0;
  float *act_buf = nullptr, *eout = nullptr, *sact = nullptr, *sout = nullptr, *sgate = nullptr;
  float* wts = nullptr;
  float* swa_ws = nullptr;  // partial results of split attention launches (few tokens, long windows)
  unsigned* swa_cnt = nullptr;  // their arrival counters (zero between launches)
  int *ids = nullptr, *off = nullptr, *slot_of = nullptr;
  int max_qkv = 0, max_od = 0, max_vd = 0, max_top = 0, max_experts = 0, max_gu = 0, max_sff = 0;
  int max_dc = 0, max_da = 0, max_heads = 0;
  tl_stack_layer_hook hook = nullptr;
  void* hook_ctx = nullptr;
  size_t cache_bytes = 0;
  void* cache_base = nullptr;
};

namespace {

template <class T>
int dev_alloc(TlStack* st, T** p, size_t n) {
  void* q = nullptr;
  TL_HIP(hipMalloc(&q, sizeof(T) * (n ? n : 1)));
  st->allocs.push_back(q);
  *p = static_cast<T*>(q);
  return 0;
}

int upload_as_f32(float* dst, int type, const void* host, size_t n, hipStream_t s) {
  std::vector<float> wide(n);
  if (type == TL_BF16) {
    const uint16_t* b = static_cast<const uint16_t*>(host);
    for (size_t i = 0; i < n; ++i) {
      const uint32_t bits = (uint32_t)b[i] << 16;
      memcpy(&wide[i], &bits, 4);
    }
  } else {
    memcpy(wide.data(), host, n * 4);
  }
  TL_HIP(hipMemcpyAsync(dst, wide.data(), n * 4, hipMemcpyHostToDevice, s));
  TL_HIP(hipStreamSynchronize(s));
  return 0;
}

// rows of `cols` bf16 values to every second row of dst (gate rows to the even, up rows to the odd rows of a gate|up matrix)
int upload_bf16_alternate(uint16_t* dst, const void* host, size_t rows, size_t cols, hipStream_t s) {
  TL_HIP(hipMemcpy2DAsync(dst, 2 * cols * 2, host, cols * 2, cols * 2, rows, hipMemcpyHostToDevice, s));
  TL_HIP(hipStreamSynchronize(s));
  return 0;
}

int upload_bf16(uint16_t* dst, const void* host, size_t n, hipStream_t s) {
  TL_HIP(hipMemcpyAsync(dst, host, n * 2, hipMemcpyHostToDevice, s));
  TL_HIP(hipStreamSynchronize(s));
  return 0;
}

bool shape_is(const long long* shape, int ndim, long long a, long long b = -1) {
  if (b < 0) {
    long long n = 1;
    for (int i = 0; i < ndim; ++i) n *= shape[i];
    return n == a && ndim <= 1;
  }
  return ndim == 2 && shape[0] == a && shape[1] == b;
}

}  // namespace

namespace {

int upload_frequencies(TlStack* st, Layer& L, const std::vector<double>& f) {
  TL_TRY(dev_alloc(st, &L.freq, f.size()));
  TL_HIP(hipMemcpy(L.freq, f.data(), sizeof(double) * f.size(), hipMemcpyHostToDevice));
  return 0;
}

// The mixer of layer i (or the second mixer of its pair): checks, sizes, tensor names, device buffers of its tensors (own:
// the layer holds tensors of its own) and its share of the cache. first_mix: the first value-mixing layer so far.
int setup_mixer(TlStack* st, Layer& L, int i, bool own, int* first_mix) {
  const tl_stack_config* cfg = &st->cfg;
  const tl_layer_spec& sp = L.sp;
  const size_t W = cfg->width;
  TL_REQUIRE(sp.mixer >= TL_MIXER_SWA && sp.mixer <= TL_MIXER_LINEAR,
             "tl_stack_create: layer %d has mixer kind %d; this engine has windowed attention (%d), the gated delta rule (%d), "
             "latent attention (%d), the generalized delta rule (%d) and gated linear attention (%d)",
             i, sp.mixer, TL_MIXER_SWA, TL_MIXER_DELTA, TL_MIXER_LATENT, TL_MIXER_GDELTA, TL_MIXER_LINEAR);
  TL_REQUIRE(sp.heads > 0 && sp.kv_heads > 0 && sp.heads % sp.kv_heads == 0 && sp.dim > 0 && sp.vdim > 0,
             "tl_stack_create: layer %d: %d heads / %d key-value heads / sizes %d, %d", i, sp.heads, sp.kv_heads, sp.dim, sp.vdim);
  if (sp.mixer == TL_MIXER_SWA) {
    TL_REQUIRE(!sp.values_are_keys || sp.vdim == sp.dim, "tl_stack_create: layer %d: values that are keys need vdim == dim", i);
    TL_REQUIRE(sp.rot_dims >= 0 && sp.rot_dims <= sp.dim && (sp.rot_dims & 1) == 0 && (sp.rot_dims == 0 || sp.rot_base > 0.0f),
               "tl_stack_create: layer %d: %d rotating dimensions of %d, base %g", i, sp.rot_dims, sp.dim, sp.rot_base);
    TL_REQUIRE(sp.keep_first >= 0, "tl_stack_create: layer %d: %d kept first keys", i, sp.keep_first);
    TL_REQUIRE(sp.attn_weight >= TL_ATTN_SOFTMAX && sp.attn_weight <= TL_ATTN_SOFTMAX_LEARNED_SINK && sp.q_temp_every >= 0,
               "tl_stack_create: layer %d: attention weights of kind %d, query temperature every %d", i, sp.attn_weight,
               sp.q_temp_every);
    L.rotary_path = sp.rot_dims > 0 || sp.qk_norm == TL_QK_NORM_HEAD_UNIT || sp.values_are_keys;
    TL_REQUIRE(!L.rotary_path || (sp.qk_norm != TL_QK_NORM_WHOLE && sp.qk_norm != TL_QK_NORM_HEAD_RMS && !sp.v_mix &&
                                  sp.q_temp_every == 0 && sp.score_maps <= 1 && !sp.qkv_conv && !sp.qkv_bias),
               "tl_stack_create: layer %d: rotation / per-head unit norm / values-are-keys do not combine with the weighted q/k "
               "norms, value mixing, a query temperature, score maps or a convolution on q, k, v", i);
    TL_REQUIRE(sp.qk_norm >= TL_QK_NORM_NONE && sp.qk_norm <= TL_QK_NORM_HEAD_RMS, "tl_stack_create: layer %d: q/k norm %d", i, sp.qk_norm);
    TL_REQUIRE(sp.score_maps == 0 || sp.score_maps == 1 || sp.score_maps == 2, "tl_stack_create: layer %d: %d score maps", i, sp.score_maps);
    const int maps = sp.score_maps == 2 ? 2 : 1;
    TL_REQUIRE(maps == 1 || (sp.attn_weight == TL_ATTN_SOFTMAX && !sp.v_mix && sp.q_temp_every == 0 && sp.keep_first == 0),
               "tl_stack_create: layer %d: two score maps take the plain softmax", i);
    TL_REQUIRE(!sp.out_gate || maps == 2, "tl_stack_create: layer %d: the output gate rides in the combination of two score maps", i);
    TL_REQUIRE(sp.qk_norm != TL_QK_NORM_HEAD_RMS || (!sp.v_mix && sp.q_temp_every == 0),
               "tl_stack_create: layer %d: the per-head q/k norm does not combine with value mixing or a query temperature", i);
    TL_REQUIRE(sp.qkv_conv >= 0 && sp.qkv_conv <= 64 && (!sp.qkv_bias || sp.qkv_conv > 0) && (!sp.qkv_conv || !sp.v_mix),
               "tl_stack_create: layer %d: %d taps on q, k, v (biases ride in that convolution)", i, sp.qkv_conv);
    TL_REQUIRE(sp.score_softcap >= 0.0f, "tl_stack_create: layer %d: score cap %g", i, sp.score_softcap);
    L.qd = sp.heads * sp.dim * maps;
    L.kd = sp.kv_heads * sp.dim * maps;
    L.vd = sp.kv_heads * sp.vdim;
    L.od = sp.heads * sp.vdim;
    L.gate_off = L.qd + L.kd + (sp.values_are_keys ? 0 : L.vd);
    L.pd = L.gate_off + (sp.out_gate ? L.od : 0);
    if (maps == 2) st->any_maps = true;
    if (sp.v_mix) {
      if (*first_mix < 0) {
        *first_mix = i;
        L.vmix_mode = 1;
      } else {
        L.vmix_mode = 2;
        TL_REQUIRE(st->layers[*first_mix].vd == L.vd, "tl_stack_create: layer %d mixes %d values with the %d of layer %d", i,
                   L.vd, st->layers[*first_mix].vd, *first_mix);
      }
    }
    st->cache_bytes += sizeof(float) * (size_t)cfg->max_positions * (L.kd + L.vd);
    if (sp.qkv_conv > 0) {
      const int dc = L.qd + L.kd + L.vd;
      st->max_dc = dc > st->max_dc ? dc : st->max_dc;
      st->cache_bytes += sizeof(float) * (size_t)(sp.qkv_conv - 1) * dc;
    }
    if (own) {
      L.expect.insert({"mix.q", "mix.k", "mix.o"});
      if (!sp.values_are_keys) L.expect.insert("mix.v");
      if (sp.qk_norm == TL_QK_NORM_WHOLE || sp.qk_norm == TL_QK_NORM_HEAD_RMS) L.expect.insert({"mix.q.norm", "mix.k.norm"});
      else L.optional.insert({"mix.q.norm", "mix.k.norm"});
      if (L.vmix_mode == 2) L.expect.insert("mix.vmix");
      else L.optional.insert("mix.vmix");
      if (sp.attn_weight == TL_ATTN_SIGMOID) L.expect.insert("mix.pb");
      if (sp.attn_weight == TL_ATTN_SOFTMAX_LEARNED_SINK) L.expect.insert("mix.sink");
      if (maps == 2) L.expect.insert({"mix.lq1", "mix.lk1", "mix.lq2", "mix.lk2"});
      if (sp.out_gate) L.expect.insert("mix.g");
      if (sp.qkv_bias) L.expect.insert({"mix.q.b", "mix.k.b", "mix.v.b"});
      if (sp.qkv_conv > 0) L.expect.insert({"mix.q.conv", "mix.k.conv", "mix.v.conv"});
      if (sp.dist_bias) L.expect.insert({"mix.r1", "mix.r2"});
      TL_TRY(dev_alloc(st, &L.q_norm, L.qd));
      TL_TRY(dev_alloc(st, &L.k_norm, L.kd));
      TL_TRY(dev_alloc(st, &L.lambda, 1));
      TL_TRY(dev_alloc(st, &L.pb, sp.heads));
      TL_TRY(dev_alloc(st, &L.sinkv, sp.heads));
      TL_TRY(dev_alloc(st, &L.r1, sp.heads));
      TL_TRY(dev_alloc(st, &L.r2, sp.heads));
      if (sp.qkv_bias) TL_TRY(dev_alloc(st, &L.qkv_b, (size_t)L.qd + L.kd + L.vd));
      if (sp.qkv_conv > 0) TL_TRY(dev_alloc(st, &L.conv, (size_t)(L.qd + L.kd + L.vd) * sp.qkv_conv));
      if (sp.rot_dims > 0) {
        std::vector<double> f(sp.rot_dims / 2);
        tl_rotary_frequencies(sp.rot_dims, sp.rot_base, sp.rot_factor, sp.rot_original, sp.rot_fast, sp.rot_slow, f.data(), &L.mscale);
        TL_TRY(upload_frequencies(st, L, f));
      }
    }
  } else if (sp.mixer == TL_MIXER_LATENT) {
    TL_REQUIRE(sp.q_rank > 0 && sp.kv_rank > 0 && sp.rot_dim >= 0 && sp.rot_dims >= 0 && sp.rot_dims <= sp.rot_dim &&
                   (sp.rot_dims & 1) == 0 && (sp.rot_dims == 0 || sp.rot_base > 0.0f) && sp.kv_heads == sp.heads,
               "tl_stack_create: layer %d: latents of %d / %d, %d rotated dimensions of which %d turn (base %g), %d key heads",
               i, sp.q_rank, sp.kv_rank, sp.rot_dim, sp.rot_dims, sp.rot_base, sp.kv_heads);
    TL_REQUIRE(sp.kv_rank <= 512, "tl_stack_create: layer %d: a key/value latent of %d above 512", i, sp.kv_rank);
    TL_REQUIRE(sp.weights_of == 0 && own, "tl_stack_create: layer %d: a latent layer owns its tensors (it may share a cache: kv_from)", i);
    L.kv_src = i;
    if (sp.kv_from > 0) {
      const int j = sp.kv_from - 1;
      TL_REQUIRE(j < i && st->layers[j].sp.mixer == TL_MIXER_LATENT && st->layers[j].sp.kv_from == 0,
                 "tl_stack_create: layer %d reads the latent cache of layer %d, which is not an earlier latent layer "
                 "with a projection of its own", i, j);
      const tl_layer_spec& o = st->layers[j].sp;
      TL_REQUIRE(o.kv_rank == sp.kv_rank && o.rot_dim == sp.rot_dim && o.rot_dims == sp.rot_dims && o.rot_base == sp.rot_base,
                 "tl_stack_create: layer %d and layer %d, whose latent cache it reads, differ in latent size or rotation", i, j);
      L.kv_src = j;
    }
    const bool own_kv = L.kv_src == i;
    const int qh = sp.dim + sp.rot_dim, ah = sp.kv_rank + sp.rot_dim;
    L.qd = sp.heads * qh;
    L.kd = own_kv ? sp.kv_rank + sp.rot_dim : 0;
    L.vd = 0;
    L.od = sp.heads * sp.vdim;
    L.gate_off = sp.q_rank + L.kd;
    L.pd = L.gate_off + (sp.head_gate ? sp.heads : 0);
    if (own_kv) st->cache_bytes += sizeof(float) * (size_t)cfg->max_positions * L.kd;
    st->max_lq = L.qd > st->max_lq ? L.qd : st->max_lq;
    st->max_lqa = sp.heads * ah > st->max_lqa ? sp.heads * ah : st->max_lqa;
    st->max_lk = sp.heads * qh > st->max_lk ? sp.heads * qh : st->max_lk;
    st->max_lv = sp.heads * sp.vdim > st->max_lv ? sp.heads * sp.vdim : st->max_lv;
    st->max_od = sp.heads * sp.kv_rank > st->max_od ? sp.heads * sp.kv_rank : st->max_od;  // the weighted latents of all heads
    L.expect.insert({"mix.dq", "mix.dq.norm", "mix.uq", "mix.uk", "mix.uv", "mix.o"});
    if (own_kv) L.expect.insert({"mix.dkv", "mix.dkv.norm"});
    if (sp.head_gate) L.expect.insert("mix.g");
    TL_TRY(dev_alloc(st, &L.wuq, (size_t)L.qd * sp.q_rank));
    TL_TRY(dev_alloc(st, &L.wukt, (size_t)sp.heads * sp.kv_rank * sp.dim));
    TL_TRY(dev_alloc(st, &L.wuk, (size_t)sp.heads * sp.kv_rank * sp.dim));
    TL_TRY(dev_alloc(st, &L.wuv, (size_t)sp.heads * sp.vdim * sp.kv_rank));
    TL_TRY(dev_alloc(st, &L.dq_norm, sp.q_rank));
    TL_TRY(dev_alloc(st, &L.dkv_norm, sp.kv_rank));
    if (sp.rot_dims > 0) {
      std::vector<double> f(sp.rot_dims / 2);
      float unused = 1.0f;
      tl_rotary_frequencies(sp.rot_dims, sp.rot_base, 0.0, 0.0, 0.0, 0.0, f.data(), &unused);
      TL_TRY(upload_frequencies(st, L, f));
    }
  } else if (sp.mixer == TL_MIXER_GDELTA) {
    TL_REQUIRE(sp.decay_rank > 0 && sp.vdim == sp.dim && sp.kv_heads == sp.heads && sp.dim <= 256,
               "tl_stack_create: layer %d: generalized delta rule with inner size %d, head sizes %d / %d (equal, at most 256), "
               "%d key heads", i, sp.decay_rank, sp.dim, sp.vdim, sp.kv_heads);
    TL_REQUIRE(sp.weights_of == 0 && own, "tl_stack_create: layer %d: a generalized delta layer owns its tensors", i);
    const int hd = sp.heads * sp.dim;
    L.qd = L.kd = L.vd = L.od = hd;
    L.pd = 5 * hd + sp.decay_rank;
    st->max_gd = hd > st->max_gd ? hd : st->max_gd;
    ++st->gdelta_layers;
    st->cache_bytes += sizeof(float) * (size_t)sp.heads * sp.dim * sp.dim;
    L.expect.insert({"mix.r", "mix.k", "mix.v", "mix.g", "mix.a", "mix.a.b", "mix.w1", "mix.w2", "mix.w0", "mix.norm", "mix.o"});
    TL_TRY(dev_alloc(st, &L.wa2, (size_t)hd * sp.decay_rank));
    TL_TRY(dev_alloc(st, &L.w0, hd));
    TL_TRY(dev_alloc(st, &L.a_bias, hd));
    TL_TRY(dev_alloc(st, &L.onorm, hd));
  } else if (sp.mixer == TL_MIXER_LINEAR) {
    TL_REQUIRE(sp.kv_heads == sp.heads && sp.dim <= 256 && sp.vdim <= 512,
               "tl_stack_create: layer %d: gated linear attention with %d / %d heads, sizes %d (at most 256) / %d (at most 512)", i,
               sp.heads, sp.kv_heads, sp.dim, sp.vdim);
    const int hd = sp.heads * sp.dim;
    L.qd = L.kd = hd;  // q | forget gate
    L.vd = L.od = sp.heads * sp.vdim;
    L.pd = 2 * hd + L.vd;
    st->max_dc = 2 * hd > st->max_dc ? 2 * hd : st->max_dc;
    st->max_da = hd > st->max_da ? hd : st->max_da;
    st->cache_bytes += sizeof(float) * (size_t)sp.heads * sp.vdim * sp.dim;
    if (own) {
      L.expect.insert({"mix.q", "mix.f", "mix.f.b", "mix.lower", "mix.v", "mix.norm", "mix.o"});
      TL_TRY(dev_alloc(st, &L.lower, hd));
      TL_TRY(dev_alloc(st, &L.f_bias, hd));
      TL_TRY(dev_alloc(st, &L.onorm, sp.vdim));
    }
  } else {
    const bool ph = sp.decay_per_head != 0;
    TL_REQUIRE(sp.conv_taps >= 1 && sp.conv_taps <= 64 && (ph ? (sp.decay_rank == 0 && sp.gate_rank == 0) : (sp.decay_rank > 0 && sp.gate_rank > 0)),
               "tl_stack_create: layer %d: %d taps, inner sizes %d / %d (none with a decay per head)", i, sp.conv_taps,
               sp.decay_rank, sp.gate_rank);
    TL_REQUIRE(sp.dim <= 256 && sp.vdim <= 512, "tl_stack_create: layer %d: key size %d above 256 or value size %d above 512", i,
               sp.dim, sp.vdim);
    L.qd = sp.kv_heads * sp.dim;  // queries share the keys' heads
    L.kd = sp.kv_heads * sp.dim;
    L.vd = sp.heads * sp.vdim;
    L.od = sp.heads * sp.vdim;
    // q | k | v | beta, then (a1 | g1) for the two-step projections or (a | gate) when they are direct
    L.pd = L.qd + L.kd + L.vd + sp.heads + (ph ? sp.heads + L.vd : sp.decay_rank + sp.gate_rank);
    L.gate_off = L.qd + L.kd + L.vd + 2 * sp.heads;
    const int dc = L.qd + L.kd + L.vd, da = sp.heads * sp.dim;
    st->max_dc = dc > st->max_dc ? dc : st->max_dc;
    st->max_da = da > st->max_da ? da : st->max_da;
    st->cache_bytes += sizeof(float) * ((size_t)sp.heads * sp.vdim * sp.dim + (size_t)(sp.conv_taps - 1) * dc);
    if (own) {
      L.expect.insert({"mix.q", "mix.k", "mix.v", "mix.b", "mix.o", "mix.q.conv", "mix.k.conv", "mix.v.conv", "mix.A_log",
                       "mix.dt_bias", "mix.norm"});
      if (ph) {
        L.expect.insert({"mix.a", "mix.g"});
      } else {
        L.expect.insert({"mix.a1", "mix.g1", "mix.a2", "mix.g2"});
        TL_TRY(dev_alloc(st, &L.wa2, (size_t)da * sp.decay_rank));
        TL_TRY(dev_alloc(st, &L.wg2, (size_t)L.vd * sp.gate_rank));
      }
      TL_TRY(dev_alloc(st, &L.conv, (size_t)dc * sp.conv_taps));
      TL_TRY(dev_alloc(st, &L.a_log, sp.heads));
      TL_TRY(dev_alloc(st, &L.dt_bias, ph ? sp.heads : da));
      TL_TRY(dev_alloc(st, &L.onorm, sp.vdim));
    }
  }
  if (own) TL_TRY(dev_alloc(st, &L.wo, W * L.od));
  st->max_qkv = L.pd > st->max_qkv ? L.pd : st->max_qkv;
  st->max_od = L.od > st->max_od ? L.od : st->max_od;
  st->max_vd = L.vd > st->max_vd ? L.vd : st->max_vd;
  st->max_heads = sp.heads > st->max_heads ? sp.heads : st->max_heads;
  return 0;
}

// everything of layer i: block and feed-forward checks, the mixer (and the second mixer of a pair), norms, feed-forward tensors
int setup_layer(TlStack* st, int i, int* first_mix) {
  const tl_stack_config* cfg = &st->cfg;
  Layer& L = st->layers[i];
  const tl_layer_spec& sp = L.sp;
  const size_t W = cfg->width;
  const bool dyt = cfg->norm == TL_NORM_DYT, lnorm = cfg->norm == TL_NORM_LAYER, rms = cfg->norm == TL_NORM_RMS;
  TL_REQUIRE((sp.block == TL_BLOCK_POST_NORM && !dyt && !lnorm && !rms) || (sp.block == TL_BLOCK_PARALLEL && dyt) ||
                 (sp.block == TL_BLOCK_PRE_NORM && (lnorm || rms)),
             "tl_stack_create: layer %d: block kind %d with norm kind %d (post-norm blocks take the one-plus RMS norm, parallel "
             "blocks the Dynamic Tanh norm, pre-norm blocks the layer norm or the plain RMS norm)", i, sp.block, cfg->norm);
  TL_REQUIRE(sp.mlp >= TL_MLP_NONE && sp.mlp <= TL_MLP_UNIT, "tl_stack_create: layer %d has feed-forward kind %d", i, sp.mlp);
  TL_REQUIRE(sp.mlp != TL_MLP_DENSE || sp.block != TL_BLOCK_POST_NORM, "tl_stack_create: layer %d: a dense feed-forward "
             "runs in parallel and pre-norm blocks only", i);
  TL_REQUIRE(sp.mlp != TL_MLP_UNIT || sp.block == TL_BLOCK_PRE_NORM,
             "tl_stack_create: layer %d: the plain up / activation / down unit runs in pre-norm blocks only", i);
  TL_REQUIRE((sp.mixer != TL_MIXER_LATENT && sp.mixer != TL_MIXER_GDELTA && sp.mixer != TL_MIXER_LINEAR) || sp.block == TL_BLOCK_PRE_NORM,
             "tl_stack_create: layer %d: latent attention, the generalized delta rule and gated linear attention run in "
             "pre-norm blocks only", i);
  TL_REQUIRE(sp.mixer != TL_MIXER_DELTA || sp.block != TL_BLOCK_POST_NORM, "tl_stack_create: layer %d: the delta rule runs "
             "in parallel and pre-norm blocks only", i);
  TL_REQUIRE(sp.glu == TL_GLU_SWISH || sp.glu == TL_GLU_RELU, "tl_stack_create: layer %d: gated unit of kind %d", i, sp.glu);
  TL_REQUIRE(!L.side || sp.block == TL_BLOCK_PRE_NORM, "tl_stack_create: layer %d: two mixers side by side run in pre-norm blocks only", i);
  L.wsrc = i;
  if (sp.weights_of > 0) {
    TL_REQUIRE(sp.weights_of - 1 < i, "tl_stack_create: layer %d takes its tensors from layer %d, which is not an earlier "
               "layer", i, sp.weights_of - 1);
    L.wsrc = st->layers[sp.weights_of - 1].wsrc;  // (a layer that itself borrows hands on the owner)
    const Layer& O = st->layers[L.wsrc];
    tl_layer_spec a = sp, b = O.sp;
    a.weights_of = b.weights_of = 0;
    a.side = b.side = nullptr;
    bool same = memcmp(&a, &b, sizeof(a)) == 0 && !L.side == !O.side;
    if (same && L.side) same = memcmp(&L.side->sp, &O.side->sp, sizeof(a)) == 0;
    TL_REQUIRE(same, "tl_stack_create: layer %d differs from layer %d whose tensors it uses", i, L.wsrc);
  }
  const bool own = L.wsrc == i;
  TL_TRY(setup_mixer(st, L, i, own, first_mix));
  if (L.side) {
    TL_REQUIRE(L.side->sp.mixer == TL_MIXER_SWA || L.side->sp.mixer == TL_MIXER_DELTA || L.side->sp.mixer == TL_MIXER_LINEAR,
               "tl_stack_create: layer %d: a second mixer of kind %d", i, L.side->sp.mixer);
    TL_REQUIRE(!L.side->sp.v_mix && !sp.v_mix, "tl_stack_create: layer %d: value mixing inside a pair of mixers", i);
    L.side->wsrc = L.wsrc;
    TL_TRY(setup_mixer(st, *L.side, i, own, first_mix));
    st->any_pair = true;
  }
  {  // the first product's matrix; two mixers side by side share one, the second mixer's rows behind the first's: one product
    const int rows = L.pd + (L.side ? L.side->pd : 0);
    if (own) {
      TL_TRY(dev_alloc(st, &L.wqkv, (size_t)rows * W));
      if (L.side) L.side->wqkv = L.wqkv + (size_t)L.pd * W;
    }
    st->max_qkv = rows > st->max_qkv ? rows : st->max_qkv;
  }
  if (own) {
    TL_TRY(dev_alloc(st, &L.norm1, W));
    TL_TRY(dev_alloc(st, &L.norm2, W));
    L.expect.insert("norm1");
    if (lnorm) {
      TL_TRY(dev_alloc(st, &L.norm1_b, W));
      TL_TRY(dev_alloc(st, &L.norm2_b, W));
      L.expect.insert("norm1.b");
    }
    if (dyt) {
      TL_TRY(dev_alloc(st, &L.norm1_b, W));
      TL_TRY(dev_alloc(st, &L.norm1_alpha, 1));
      L.expect.insert({"norm1.b", "norm1.alpha"});
    }
    if (cfg->canon_taps > 0) {
      TL_TRY(dev_alloc(st, &L.canon1, W * cfg->canon_taps));
      L.expect.insert("canon1");
      if (sp.mlp != TL_MLP_NONE) {
        TL_TRY(dev_alloc(st, &L.canon2, W * cfg->canon_taps));
        L.expect.insert("canon2");
      } else {
        L.optional.insert("canon2");
      }
    }
  }
  if (cfg->canon_taps > 1) st->cache_bytes += sizeof(float) * (size_t)(cfg->canon_taps - 1) * W * (sp.mlp != TL_MLP_NONE ? 2 : 1);
  // ---- feed-forward ----
  const bool pre_rms = sp.block == TL_BLOCK_PRE_NORM && rms;
  if (sp.mlp == TL_MLP_MOE) {
    TL_REQUIRE(sp.block != TL_BLOCK_PRE_NORM || rms, "tl_stack_create: layer %d: routed experts behind a layer norm", i);
    TL_REQUIRE(sp.experts > 0 && sp.top > 0 && sp.top <= sp.experts && sp.expert_ff > 0 && sp.shared_ff >= 0,
               "tl_stack_create: layer %d: %d experts, top %d, sizes %d / %d", i, sp.experts, sp.top, sp.expert_ff, sp.shared_ff);
    TL_REQUIRE(sp.route == TL_ROUTE_TOP_LOGITS ||
                   ((sp.route == TL_ROUTE_SOFTMAX_GROUPS || sp.route == TL_ROUTE_SIGMOID_GROUPS) && sp.route_groups > 0 &&
                    sp.experts % sp.route_groups == 0 && sp.route_keep > 0 && sp.route_keep <= sp.route_groups &&
                    (long long)sp.route_keep * (sp.experts / sp.route_groups) >= sp.top),
               "tl_stack_create: layer %d: router kind %d, %d experts in %d groups, %d kept, top %d", i, sp.route, sp.experts,
               sp.route_groups, sp.route_keep, sp.top);
    TL_REQUIRE(!sp.shared_gate || sp.shared_ff > 0, "tl_stack_create: layer %d: a gate without a shared expert", i);
    TL_REQUIRE(!pre_rms || !sp.shared_gate, "tl_stack_create: layer %d: a gated shared expert runs in parallel blocks only", i);
    if (own) {
      if (sp.block == TL_BLOCK_POST_NORM || pre_rms) L.expect.insert("norm2");
      L.expect.insert("mlp.router");
      if (sp.route == TL_ROUTE_TOP_LOGITS) L.expect.insert("mlp.router.b");
      if (sp.route == TL_ROUTE_SIGMOID_GROUPS) L.expect.insert("mlp.correction");
      for (int e = 0; e < sp.experts; ++e)
        for (const char* k : {"gate", "up", "down"}) L.expect.insert("mlp.e" + std::to_string(e) + "." + k);
      TL_TRY(dev_alloc(st, &L.router, (size_t)sp.experts * W));
      TL_TRY(dev_alloc(st, &L.router_b, sp.experts));
      TL_TRY(dev_alloc(st, &L.gu, (size_t)sp.experts * 2 * sp.expert_ff * W));
      TL_TRY(dev_alloc(st, &L.down, (size_t)sp.experts * W * sp.expert_ff));
      if (sp.shared_ff) {
        L.expect.insert({"mlp.shared.gate", "mlp.shared.up", "mlp.shared.down"});
        TL_TRY(dev_alloc(st, &L.sgu, (size_t)2 * sp.shared_ff * W));
        TL_TRY(dev_alloc(st, &L.sdown, W * sp.shared_ff));
        if (sp.shared_gate) {
          L.expect.insert("mlp.shared.sg");
          TL_TRY(dev_alloc(st, &L.sg, W));
        }
      }
    }
    st->max_top = sp.top > st->max_top ? sp.top : st->max_top;
    st->max_experts = sp.experts > st->max_experts ? sp.experts : st->max_experts;
    st->max_gu = 2 * sp.expert_ff * sp.top > st->max_gu ? 2 * sp.expert_ff * sp.top : st->max_gu;
    st->max_sff = sp.shared_ff > st->max_sff ? sp.shared_ff : st->max_sff;
  } else if (sp.mlp == TL_MLP_DENSE) {
    TL_REQUIRE(sp.block != TL_BLOCK_PRE_NORM || rms, "tl_stack_create: layer %d: a gated unit behind a layer norm", i);
    TL_REQUIRE(sp.shared_ff > 0, "tl_stack_create: layer %d: a dense feed-forward of size %d", i, sp.shared_ff);
    if (own) {
      if (pre_rms) L.expect.insert("norm2");
      L.expect.insert({"mlp.gate", "mlp.up", "mlp.down"});
      TL_TRY(dev_alloc(st, &L.sgu, (size_t)2 * sp.shared_ff * W));
      TL_TRY(dev_alloc(st, &L.sdown, W * sp.shared_ff));
    }
    st->max_sff = sp.shared_ff > st->max_sff ? sp.shared_ff : st->max_sff;
  } else if (sp.mlp == TL_MLP_UNIT) {
    TL_REQUIRE(lnorm, "tl_stack_create: layer %d: the plain up / activation / down unit sits behind a layer norm", i);
    TL_REQUIRE(sp.shared_ff > 0 && sp.act >= TL_ACT_NONE && sp.act <= TL_ACT_TANH,
               "tl_stack_create: layer %d: a feed-forward of size %d with activation kind %d", i, sp.shared_ff, sp.act);
    if (own) {
      L.expect.insert({"norm2", "norm2.b", "mlp.up", "mlp.down"});
      if (sp.act == TL_ACT_XIELU) L.expect.insert("mlp.act");
      TL_TRY(dev_alloc(st, &L.sgu, (size_t)sp.shared_ff * W));
      TL_TRY(dev_alloc(st, &L.sdown, W * sp.shared_ff));
    }
    st->max_sff = sp.shared_ff > st->max_sff ? sp.shared_ff : st->max_sff;
  } else if (own) {
    L.optional.insert("norm2");
    if (lnorm) L.optional.insert("norm2.b");
  }
  return 0;
}

}  // namespace

int tl_stack_create(const tl_stack_config* cfg, TlStack** out) {
  TL_REQUIRE(cfg && out && cfg->layers, "tl_stack_create: null argument");
  TL_REQUIRE(cfg->width > 0 && cfg->vocab > 0 && cfg->n_layers > 0 && cfg->max_positions > 0,
             "tl_stack_create: non-positive size in the configuration");
  TL_REQUIRE(cfg->norm >= TL_NORM_RMS_ONE_PLUS && cfg->norm <= TL_NORM_RMS, "tl_stack_create: norm kind %d", cfg->norm);
  TL_REQUIRE(cfg->canon_taps >= 0 && cfg->canon_taps <= 64 && (cfg->canon_taps == 0 || cfg->norm == TL_NORM_RMS),
             "tl_stack_create: %d taps on what the sublayers read (a convolution there follows the plain RMS norm)", cfg->canon_taps);
  TL_REQUIRE(cfg->norm != TL_NORM_RMS || !cfg->embed_norm, "tl_stack_create: an embedding norm with the plain RMS norm");
  TlStack* st = new TlStack();
  st->cfg = *cfg;
  st->layers.resize(cfg->n_layers);
  const size_t W = cfg->width;
  int first_mix = -1;
  int rc = 0;
  auto fail = [&](int code) {
    tl_stack_free(st);
    return code;
  };
  for (int i = 0; i < cfg->n_layers && rc == 0; ++i) {
    Layer& L = st->layers[i];
    L.sp = cfg->layers[i];
    if (L.sp.side) {  // the second mixer's entry is copied: the caller's may not outlive this call
      L.side.reset(new Layer());
      L.side->sp = *L.sp.side;
      L.side->sp.side = nullptr;
      L.sp.side = &L.side->sp;
    }
    rc = setup_layer(st, i, &first_mix);
  }
  if (rc) return fail(rc);
  if ((rc = dev_alloc(st, &st->embed, (size_t)cfg->vocab * W)) || (rc = dev_alloc(st, &st->head, (size_t)cfg->vocab * W)) ||
      (rc = dev_alloc(st, &st->embed_norm, W)) || (rc = dev_alloc(st, &st->final_norm, W)) ||
      (rc = dev_alloc(st, &st->final_b, W)) || (rc = dev_alloc(st, &st->final_alpha, 1)) ||
      (rc = dev_alloc(st, &st->embed_norm_b, W)))
    return fail(rc);
  st->need_globals = 1 | 2 | 8 | (cfg->embed_norm ? 4 : 0) | (cfg->norm == TL_NORM_DYT ? 16 | 32 : 0) |
                     (cfg->norm == TL_NORM_LAYER ? 16 | (cfg->embed_norm ? 64 : 0) : 0);
  if (const char* e = getenv("TL_STACK_CHUNK")) st->chunk = atoi(e) > 0 ? atoi(e) : st->chunk;
  if (const char* e = getenv("TL_STACK_GEMV")) st->gemv_decode = atoi(e) != 0;
  if (const char* e = getenv("TL_STACK_FUSE_ROUTER")) st->fuse_router = atoi(e) != 0;
  if (const char* e = getenv("TL_STACK_FORK")) st->fork = atoi(e) != 0;
  if (const char* e = getenv("TL_STACK_FUSE_CANON")) st->fuse_canon = atoi(e) != 0;
  if (const char* e = getenv("TL_STACK_LEAD")) st->lead = atoi(e) > 0 ? atoi(e) : 0;
  if (const char* e = getenv("TL_STACK_EXACT_BELOW")) st->exact_below = atoi(e) > 2 ? atoi(e) : 2;
  if (const char* e = getenv("TL_STACK_LATENT_EXPAND")) st->latent_expand = atoi(e) > 0 ? atoi(e) : 0;
  *out = st;
  return 0;
}

void tl_stack_free(TlStack* st) {
  if (!st) return;
  for (void* p : st->allocs) hipFree(p);
  hipFree(st->cache_base);
  if (st->ev_fork) hipEventDestroy(st->ev_fork);
  if (st->ev_join) hipEventDestroy(st->ev_join);
  if (st->side) hipStreamDestroy(st->side);
  delete st;
}

int tl_stack_set_tensor(TlStack* st, const char* name, int type, const long long* shape, int ndim, const void* host,
                        hipStream_t s) {
  TL_REQUIRE(st && name && host && (shape || ndim == 0), "tl_stack_set_tensor: null argument");
  TL_REQUIRE(!st->finalized, "tl_stack_set_tensor: model already finalized");
  TL_REQUIRE(type == TL_BF16 || type == TL_F32, "tl_stack_set_tensor: %s has type %d; bf16 (matrices, vectors) or f32 (vectors)",
             name, type);
  const long long W = st->cfg.width, V = st->cfg.vocab;
  const std::string n(name);
#define MATRIX(dst, r, c)                                                                                                   \
  do {                                                                                                                      \
    TL_REQUIRE(type == TL_BF16, "tl_stack_set_tensor: matrix %s must be bf16", name);                                       \
    TL_REQUIRE(shape_is(shape, ndim, (r), (c)), "tl_stack_set_tensor: %s is not %lld x %lld", name, (long long)(r),         \
               (long long)(c));                                                                                             \
    return upload_bf16((dst), host, (size_t)(r) * (size_t)(c), s);                                                          \
  } while (0)
#define PAIRED(dst, r, c)                                                                                                   \
  do {                                                                                                                      \
    TL_REQUIRE(type == TL_BF16, "tl_stack_set_tensor: matrix %s must be bf16", name);                                       \
    TL_REQUIRE(shape_is(shape, ndim, (r), (c)), "tl_stack_set_tensor: %s is not %lld x %lld", name, (long long)(r),         \
               (long long)(c));                                                                                             \
    return upload_bf16_alternate((dst), host, (size_t)(r), (size_t)(c), s);                                                 \
  } while (0)
#define VECTOR(dst, len)                                                                                                    \
  do {                                                                                                                      \
    TL_REQUIRE(shape_is(shape, ndim, (len)), "tl_stack_set_tensor: %s does not have %lld elements", name, (long long)(len)); \
    return upload_as_f32((dst), type, host, (size_t)(len), s);                                                              \
  } while (0)
  if (n == "embed") { st->got_globals |= 1; MATRIX(st->embed, V, W); }
  if (n == "head") { st->got_globals |= 2; MATRIX(st->head, V, W); }
  if (n == "embed.norm") { st->got_globals |= 4; VECTOR(st->embed_norm, W); }
  if (n == "embed.norm.b") { st->got_globals |= 64; VECTOR(st->embed_norm_b, W); }
  if (n == "final.norm") { st->got_globals |= 8; VECTOR(st->final_norm, W); }
  if (n == "final.norm.b") { st->got_globals |= 16; VECTOR(st->final_b, W); }
  if (n == "final.norm.alpha") { st->got_globals |= 32; VECTOR(st->final_alpha, 1); }
  int li = -1, used = 0;
  TL_REQUIRE(sscanf(name, "l%d.%n", &li, &used) == 1 && used > 0 && li >= 0 && li < st->cfg.n_layers,
             "tl_stack_set_tensor: no place for a tensor named %s", name);
  Layer* target = &st->layers[li];
  std::string r = n.substr(used);
  if (target->side) {  // two mixers side by side: mix.left.* is the first mixer's mix.*, mix.right.* the second's
    if (r.compare(0, 9, "mix.left.") == 0) {
      r = "mix." + r.substr(9);
    } else if (r.compare(0, 10, "mix.right.") == 0) {
      r = "mix." + r.substr(10);
      target = target->side.get();
    } else {
      TL_REQUIRE(r.compare(0, 4, "mix.") != 0, "tl_stack_set_tensor: %s: the mixers of layer %d are mix.left and mix.right", name, li);
    }
  }
  Layer& L = *target;
  const tl_layer_spec& sp = L.sp;
  if (L.optional.count(r) && !L.expect.count(r)) {  // present in the checkpoint, not used by this configuration: checked, dropped
    return 0;
  }
  TL_REQUIRE(L.expect.erase(r) == 1, "tl_stack_set_tensor: no place for a tensor named %s in layer %d (unknown, given twice, or "
             "the layer uses another layer's tensors)", name, li);
  if (r == "norm1") VECTOR(L.norm1, W);
  if (r == "norm1.b") VECTOR(L.norm1_b, W);
  if (r == "norm1.alpha") VECTOR(L.norm1_alpha, 1);
  if (r == "norm2") VECTOR(L.norm2, W);
  if (r == "norm2.b") VECTOR(L.norm2_b, W);
  if (r == "canon1") MATRIX(L.canon1, W, st->cfg.canon_taps);
  if (r == "canon2") MATRIX(L.canon2, W, st->cfg.canon_taps);
  if (sp.mixer == TL_MIXER_LINEAR) {
    const long long hd = (long long)sp.heads * sp.dim;
    if (r == "mix.q") MATRIX(L.wqkv, hd, W);
    if (r == "mix.f") MATRIX(L.wqkv + (size_t)hd * W, hd, W);
    if (r == "mix.v") MATRIX(L.wqkv + (size_t)2 * hd * W, L.vd, W);
    if (r == "mix.f.b") VECTOR(L.f_bias, hd);
    if (r == "mix.lower") VECTOR(L.lower, hd);
    if (r == "mix.norm") VECTOR(L.onorm, sp.vdim);
    if (r == "mix.o") MATRIX(L.wo, W, L.od);
  }
  if (sp.mixer == TL_MIXER_SWA) {
    const long long hd = sp.dim, taps = sp.qkv_conv;
    if (sp.qk_norm == TL_QK_NORM_HEAD_RMS) {
      if (r == "mix.q.norm") VECTOR(L.q_norm, hd);
      if (r == "mix.k.norm") VECTOR(L.k_norm, hd);
    }
    if (r == "mix.g") MATRIX(L.wqkv + (size_t)L.gate_off * W, L.od, W);
    if (r == "mix.q.b") VECTOR(L.qkv_b, L.qd);
    if (r == "mix.k.b") VECTOR(L.qkv_b + L.qd, L.kd);
    if (r == "mix.v.b") VECTOR(L.qkv_b + L.qd + L.kd, L.vd);
    if (r == "mix.q.conv") MATRIX(L.conv, L.qd, taps);
    if (r == "mix.k.conv") MATRIX(L.conv + (size_t)L.qd * taps, L.kd, taps);
    if (r == "mix.v.conv") MATRIX(L.conv + (size_t)(L.qd + L.kd) * taps, L.vd, taps);
    if (r == "mix.r1") VECTOR(L.r1, sp.heads);
    if (r == "mix.r2") VECTOR(L.r2, sp.heads);
    if (r == "mix.sink") VECTOR(L.sinkv, sp.heads);
    for (int j = 0; j < 4; ++j) {
      static const char* const names[4] = {"mix.lq1", "mix.lk1", "mix.lq2", "mix.lk2"};
      if (r != names[j]) continue;
      TL_REQUIRE(shape_is(shape, ndim, hd), "tl_stack_set_tensor: %s does not have %lld elements", name, hd);
      L.lvec[j].resize((size_t)hd);
      for (long long d = 0; d < hd; ++d) {
        if (type == TL_BF16) {
          const uint32_t bits = (uint32_t) static_cast<const uint16_t*>(host)[d] << 16;
          memcpy(&L.lvec[j][d], &bits, 4);
        } else {
          L.lvec[j][d] = static_cast<const float*>(host)[d];
        }
      }
      if (L.expect.count("mix.lq1") + L.expect.count("mix.lk1") + L.expect.count("mix.lq2") + L.expect.count("mix.lk2") == 0) {
        double d1 = 0.0, d2 = 0.0;  // lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff_init: one number for the layer, formed once
        for (long long d = 0; d < hd; ++d) {
          d1 += (double)L.lvec[0][d] * L.lvec[1][d];
          d2 += (double)L.lvec[2][d] * L.lvec[3][d];
        }
        L.lam = (float)(exp(d1) - exp(d2) + (double)sp.diff_init);
      }
      return 0;
    }
  }
  if (sp.mixer == TL_MIXER_LATENT) {
    const long long qh = sp.dim + sp.rot_dim;
    if (r == "mix.dq") MATRIX(L.wqkv, sp.q_rank, W);
    if (r == "mix.dkv") MATRIX(L.wqkv + (size_t)sp.q_rank * W, L.kd, W);
    if (r == "mix.g") MATRIX(L.wqkv + (size_t)L.gate_off * W, sp.heads, W);
    if (r == "mix.dq.norm") VECTOR(L.dq_norm, sp.q_rank);
    if (r == "mix.dkv.norm") VECTOR(L.dkv_norm, sp.kv_rank);
    if (r == "mix.uq") MATRIX(L.wuq, sp.heads * qh, sp.q_rank);
    if (r == "mix.uv") MATRIX(L.wuv, (long long)sp.heads * sp.vdim, sp.kv_rank);
    if (r == "mix.o") MATRIX(L.wo, W, L.od);
    if (r == "mix.uk") {  // [heads * dim][kv_rank] -> per head its transpose [kv_rank][dim]
      TL_REQUIRE(type == TL_BF16 && shape_is(shape, ndim, (long long)sp.heads * sp.dim, sp.kv_rank),
                 "tl_stack_set_tensor: %s is not a bf16 matrix of %lld x %d", name, (long long)sp.heads * sp.dim, sp.kv_rank);
      const uint16_t* src = static_cast<const uint16_t*>(host);
      std::vector<uint16_t> tr((size_t)sp.heads * sp.kv_rank * sp.dim);
      for (int hh = 0; hh < sp.heads; ++hh)
        for (int d = 0; d < sp.dim; ++d)
          for (int c = 0; c < sp.kv_rank; ++c)
            tr[((size_t)hh * sp.kv_rank + c) * sp.dim + d] = src[((size_t)hh * sp.dim + d) * sp.kv_rank + c];
      TL_TRY(upload_bf16(L.wuk, host, tr.size(), s));
      return upload_bf16(L.wukt, tr.data(), tr.size(), s);
    }
  }
  if (sp.mixer == TL_MIXER_GDELTA) {
    const long long hd = (long long)sp.heads * sp.dim;
    if (r == "mix.r") MATRIX(L.wqkv, hd, W);
    if (r == "mix.k") MATRIX(L.wqkv + (size_t)hd * W, hd, W);
    if (r == "mix.v") MATRIX(L.wqkv + (size_t)2 * hd * W, hd, W);
    if (r == "mix.g") MATRIX(L.wqkv + (size_t)3 * hd * W, hd, W);
    if (r == "mix.a") MATRIX(L.wqkv + (size_t)4 * hd * W, hd, W);
    if (r == "mix.w1") MATRIX(L.wqkv + (size_t)5 * hd * W, sp.decay_rank, W);
    if (r == "mix.w2") MATRIX(L.wa2, hd, sp.decay_rank);
    if (r == "mix.w0") VECTOR(L.w0, hd);
    if (r == "mix.a.b") VECTOR(L.a_bias, hd);
    if (r == "mix.norm") VECTOR(L.onorm, hd);
    if (r == "mix.o") MATRIX(L.wo, W, L.od);
  }
  if (sp.mlp == TL_MLP_UNIT) {
    const long long ff = sp.shared_ff;
    if (r == "mlp.up") MATRIX(L.sgu, ff, W);
    if (r == "mlp.down") MATRIX(L.sdown, W, ff);
    if (r == "mlp.act") {  // two numbers (p, q): P = softplus(p), Q = 1/2 + softplus(q), formed once, in double
      TL_REQUIRE(shape_is(shape, ndim, 2), "tl_stack_set_tensor: %s does not have 2 elements", name);
      float pq[2];
      if (type == TL_BF16) {
        for (int j = 0; j < 2; ++j) {
          const uint32_t bits = (uint32_t) static_cast<const uint16_t*>(host)[j] << 16;
          memcpy(&pq[j], &bits, 4);
        }
      } else {
        memcpy(pq, host, 8);
      }
      auto softplus = [](double z) { return z > 30.0 ? z : log1p(exp(z)); };
      L.act_p = (float)softplus(pq[0]);
      L.act_q = (float)(0.5 + softplus(pq[1]));
      return 0;
    }
  }
  if (r == "mix.q") MATRIX(L.wqkv, L.qd, W);
  if (r == "mix.k") MATRIX(L.wqkv + (size_t)L.qd * W, L.kd, W);
  if (r == "mix.v") MATRIX(L.wqkv + (size_t)(L.qd + L.kd) * W, L.vd, W);
  if (r == "mix.o") MATRIX(L.wo, W, L.od);
  if (r == "mix.q.norm") VECTOR(L.q_norm, L.qd);
  if (r == "mix.k.norm") VECTOR(L.k_norm, L.kd);
  if (r == "mix.vmix") VECTOR(L.lambda, 1);
  if (r == "mix.pb") VECTOR(L.pb, sp.heads);
  if (sp.mixer == TL_MIXER_DELTA) {
    const long long c0 = L.qd + L.kd + L.vd, da = (long long)sp.heads * sp.dim, taps = sp.conv_taps;
    if (r == "mix.b") MATRIX(L.wqkv + (size_t)c0 * W, sp.heads, W);
    if (sp.decay_per_head) {
      if (r == "mix.a") MATRIX(L.wqkv + (size_t)(c0 + sp.heads) * W, sp.heads, W);
      if (r == "mix.g") MATRIX(L.wqkv + (size_t)L.gate_off * W, L.vd, W);
      if (r == "mix.dt_bias") VECTOR(L.dt_bias, sp.heads);
    }
    if (r == "mix.a1") MATRIX(L.wqkv + (size_t)(c0 + sp.heads) * W, sp.decay_rank, W);
    if (r == "mix.g1") MATRIX(L.wqkv + (size_t)(c0 + sp.heads + sp.decay_rank) * W, sp.gate_rank, W);
    if (r == "mix.a2") MATRIX(L.wa2, da, sp.decay_rank);
    if (r == "mix.g2") MATRIX(L.wg2, L.vd, sp.gate_rank);
    if (r == "mix.q.conv") MATRIX(L.conv, L.qd, taps);
    if (r == "mix.k.conv") MATRIX(L.conv + (size_t)L.qd * taps, L.kd, taps);
    if (r == "mix.v.conv") MATRIX(L.conv + (size_t)(L.qd + L.kd) * taps, L.vd, taps);
    if (r == "mix.A_log") VECTOR(L.a_log, sp.heads);
    if (r == "mix.dt_bias") VECTOR(L.dt_bias, da);
    if (r == "mix.norm") VECTOR(L.onorm, sp.vdim);
  }
  if (sp.mlp == TL_MLP_DENSE) {
    const long long ff = sp.shared_ff;
    if (r == "mlp.gate") PAIRED(L.sgu, ff, W);  // gate | up interleaved by unit (DenseArgs::glu)
    if (r == "mlp.up") PAIRED(L.sgu + W, ff, W);
    if (r == "mlp.down") MATRIX(L.sdown, W, ff);
  }
  if (sp.mlp == TL_MLP_MOE) {
    const long long ff = sp.expert_ff, sff = sp.shared_ff;
    if (r == "mlp.router") MATRIX(L.router, sp.experts, W);
    if (r == "mlp.router.b") VECTOR(L.router_b, sp.experts);
    if (r == "mlp.correction") VECTOR(L.router_b, sp.experts);
    if (sff) {
      if (r == "mlp.shared.gate") PAIRED(L.sgu, sff, W);  // gate | up interleaved by unit (DenseArgs::glu)
      if (r == "mlp.shared.up") PAIRED(L.sgu + W, sff, W);
      if (r == "mlp.shared.down") MATRIX(L.sdown, W, sff);
      if (r == "mlp.shared.sg") {
        TL_REQUIRE(type == TL_BF16 && ((ndim == 2 && shape[0] == 1 && shape[1] == W) || (ndim == 1 && shape[0] == W)),
                   "tl_stack_set_tensor: %s is not a bf16 row of %lld", name, W);
        return upload_bf16(L.sg, host, (size_t)W, s);
      }
    }
    int e = -1, u2 = 0;
    if (sscanf(r.c_str(), "mlp.e%d.%n", &e, &u2) == 1 && u2 > 0 && e >= 0 && e < sp.experts) {
      const std::string k = r.substr(u2);
      uint16_t* gu = L.gu + (size_t)e * 2 * ff * W;
      if (k == "gate") PAIRED(gu, ff, W);
      if (k == "up") PAIRED(gu + W, ff, W);
      if (k == "down") MATRIX(L.down + (size_t)e * W * ff, W, ff);
    }
  }
  TL_REQUIRE(false, "tl_stack_set_tensor: no place for a tensor named %s in layer %d", name, li);
#undef MATRIX
#undef PAIRED
#undef VECTOR
}

int tl_stack_finalize(TlStack* st, hipStream_t s) {
  TL_REQUIRE(st, "tl_stack_finalize: null handle");
  if (st->finalized) return 0;
  TL_REQUIRE((st->got_globals & st->need_globals) == st->need_globals,
             "tl_stack_finalize: embed / head / final.norm (and their parts) missing (have mask %d of %d)", st->got_globals,
             st->need_globals);
  for (size_t i = 0; i < st->layers.size(); ++i) {
    TL_REQUIRE(st->layers[i].expect.empty(), "tl_stack_finalize: layer %d lacks %zu tensors, the first is %s", (int)i,
               st->layers[i].expect.size(), st->layers[i].expect.begin()->c_str());
    const Layer* sd = st->layers[i].side.get();
    TL_REQUIRE(!sd || sd->expect.empty(), "tl_stack_finalize: the second mixer of layer %d lacks %zu tensors, the first is %s", (int)i,
               sd->expect.size(), sd->expect.begin()->c_str());
  }
  const size_t W = st->cfg.width, C = st->chunk;
  TL_HIP(hipMalloc(&st->cache_base, st->cache_bytes));
  float* p = static_cast<float*>(st->cache_base);
  for (Layer& L0 : st->layers) {
    if (st->cfg.canon_taps > 1) {
      L0.canon_hist1 = p;
      p += (size_t)(st->cfg.canon_taps - 1) * W;
      if (L0.sp.mlp != TL_MLP_NONE) {
        L0.canon_hist2 = p;
        p += (size_t)(st->cfg.canon_taps - 1) * W;
      }
    }
   for (Layer* Lp : {&L0, L0.side.get()}) {
    if (!Lp) continue;
    Layer& L = *Lp;
    if (L.sp.mixer == TL_MIXER_SWA) {
      L.kc = p;
      p += (size_t)st->cfg.max_positions * L.kd;
      L.vc = p;
      p += (size_t)st->cfg.max_positions * L.vd;
      if (L.sp.qkv_conv > 1) {
        L.hist = p;
        p += (size_t)(L.sp.qkv_conv - 1) * (L.qd + L.kd + L.vd);
      }
    } else if (L.sp.mixer == TL_MIXER_LINEAR) {
      L.state = p;
      p += (size_t)L.sp.heads * L.sp.vdim * L.sp.dim;
    } else if (L.sp.mixer == TL_MIXER_LATENT) {
      if (L.kd) {
        L.ckv = p;
        p += (size_t)st->cfg.max_positions * L.kd;
      } else {
        L.ckv = st->layers[L.kv_src].ckv;  // an earlier layer: already placed
      }
    } else if (L.sp.mixer == TL_MIXER_GDELTA) {
      L.state = p;
      p += (size_t)L.sp.heads * L.sp.dim * L.sp.dim;
    } else {
      L.state = p;
      p += (size_t)L.sp.heads * L.sp.vdim * L.sp.dim;
      L.hist = p;
      p += (size_t)(L.sp.conv_taps - 1) * (L.qd + L.kd + L.vd);
    }
   }
  }
  TL_REQUIRE((size_t)(p - static_cast<float*>(st->cache_base)) * sizeof(float) == st->cache_bytes,
             "tl_stack_finalize: the cache layout does not add up to its allocation");
  if (st->any_maps) TL_TRY(dev_alloc(st, &st->att2, C * st->max_od));
  if (st->any_pair) TL_TRY(dev_alloc(st, &st->proj2, C * W));
  if (st->cfg.canon_taps > 0) TL_TRY(dev_alloc(st, &st->hn, C * W));
  TL_TRY(dev_alloc(st, &st->x, C * W));
  TL_TRY(dev_alloc(st, &st->h, C * W));
  TL_TRY(dev_alloc(st, &st->qkv, C * st->max_qkv));
  TL_TRY(dev_alloc(st, &st->att, C * st->max_od));
  TL_TRY(dev_alloc(st, &st->proj, C * W));
  TL_TRY(dev_alloc(st, &st->v_first, C * st->max_vd));
  TL_TRY(dev_alloc(st, &st->xn, C * W));
  if (st->max_dc) {
    TL_TRY(dev_alloc(st, &st->dq, C * st->max_dc));
    if (st->max_da > st->max_gd) st->max_gd = st->max_da;  // one buffer serves both recurrences' decay pre-activations
    TL_TRY(dev_alloc(st, &st->ddecay, C * st->max_da));
    TL_TRY(dev_alloc(st, &st->dg, C * st->max_od));
    TL_TRY(dev_alloc(st, &st->dbeta, C * st->max_heads));
  }
  if (st->max_lq) {
    TL_TRY(dev_alloc(st, &st->lq, C * st->max_lq));
    TL_TRY(dev_alloc(st, &st->lqa, C * st->max_lqa));
    if (st->latent_expand > 0) {
      TL_TRY(dev_alloc(st, &st->lk, (size_t)st->cfg.max_positions * st->max_lk));
      TL_TRY(dev_alloc(st, &st->lv, (size_t)st->cfg.max_positions * st->max_lv));
    }
  }
  if (st->max_gd) {
    TL_TRY(dev_alloc(st, &st->da, C * st->max_gd));
  }
  if (st->gdelta_layers) {
    TL_TRY(dev_alloc(st, &st->gw, C * st->max_gd));
    TL_TRY(dev_alloc(st, &st->gu, C * st->max_gd));
    TL_TRY(dev_alloc(st, &st->gau, C * st->max_gd));
    TL_TRY(dev_alloc(st, &st->grau, C * st->max_heads));
    TL_TRY(dev_alloc(st, &st->grk, C * st->max_heads));
  }
  {
    size_t ws = 1;
    std::vector<const Layer*> mixers;
    for (const Layer& L : st->layers) {
      mixers.push_back(&L);
      if (L.side) mixers.push_back(L.side.get());
    }
    for (const Layer* Lp : mixers)
      for (int T = 1; T <= 4; ++T) {
        const Layer& L = *Lp;
        if (L.sp.mixer != TL_MIXER_SWA && L.sp.mixer != TL_MIXER_LATENT) continue;
        const bool lat = L.sp.mixer == TL_MIXER_LATENT;
        const size_t n = tl_swa_ws_floats(T, L.sp.heads, lat ? L.sp.kv_rank : L.sp.vdim,
                                          tl_swa_splits(T, lat ? 0 : L.sp.window, st->cfg.max_positions, lat ? 0 : L.sp.keep_first));
        ws = n > ws ? n : ws;
      }
    TL_TRY(dev_alloc(st, &st->swa_ws, ws));
    const size_t heads = st->max_heads > 0 ? st->max_heads : 1;
    TL_TRY(dev_alloc(st, &st->swa_cnt, 4 * heads));
    TL_HIP(hipMemsetAsync(st->swa_cnt, 0, sizeof(unsigned) * 4 * heads, s));
  }
  if (st->max_top) {
    const size_t S = C * st->max_top;
    TL_TRY(dev_alloc(st, &st->ids, S));
    TL_TRY(dev_alloc(st, &st->wts, S));
    TL_TRY(dev_alloc(st, &st->slot_of, S));
    TL_TRY(dev_alloc(st, &st->off, (size_t)st->max_experts + 1));
    TL_TRY(dev_alloc(st, &st->eout, S * W));
  }
  if (st->max_top || st->max_sff) {
    TL_TRY(dev_alloc(st, &st->act_buf, C * st->max_gu / 2 + st->max_sff));
    TL_TRY(dev_alloc(st, &st->sgate, C));
    TL_TRY(dev_alloc(st, &st->sout, C * W));
    if (st->max_sff) TL_TRY(dev_alloc(st, &st->sact, C * st->max_sff));
  }
  bool any_parallel = false;
  for (const Layer& L : st->layers) any_parallel |= L.sp.block == TL_BLOCK_PARALLEL && L.sp.mlp != TL_MLP_NONE;
  if (st->fork && any_parallel) {
    TL_HIP(hipStreamCreateWithFlags(&st->side, hipStreamNonBlocking));
    TL_HIP(hipEventCreateWithFlags(&st->ev_fork, hipEventDisableTiming));
    TL_HIP(hipEventCreateWithFlags(&st->ev_join, hipEventDisableTiming));
  } else {
    st->fork = false;
  }
  st->finalized = true;
  return tl_stack_reset(st, s);
}

int tl_stack_reset(TlStack* st, hipStream_t s) {
  TL_REQUIRE(st && st->finalized, "tl_stack_reset: model not finalized");
  TL_HIP(hipMemsetAsync(st->cache_base, 0, st->cache_bytes, s));
  TL_HIP(hipStreamSynchronize(s));
  return 0;
}

int tl_stack_set_terms(TlStack* st, int terms) {
  TL_REQUIRE(st, "tl_stack_set_terms: null handle");
  TL_REQUIRE(terms == 1 || terms == 3, "tl_stack_set_terms: a layer-list model multiplies with 1 (bf16 activations) or 3 "
             "(FP32-grade) terms, not %d", terms);
  st->terms = terms;
  return 0;
}

int tl_stack_chunk(const TlStack* st) { return st->chunk; }

// The generalized delta rule starts from S = 0: the first token leaves S = k v^T, its read-out is v (k . r), and the head norm
// behind it turns that into +-v / rms(v), softened only by eps. Where k . r happens to be small the SIGN hangs on the last
// bits of the layer's input, bf16 rounding of the activations in front moves the residual stream at position 0 by tens of
// percent (measured: 24 % of its size, against 0.3 % at later positions), and every early position attends to that token.
// So a sequence's first token goes through on its own, on the one-token path (FP32 GEMVs): one more pass over the weights per
// prompt, the cost of a decode step. (Sixteen tokens as a three-term chunk were measured first: such a chunk fills a third of
// the chip and cost a fifth of the prefill rate; the second token is five times less sensitive than the first, the third not
// at all.)
int tl_stack_lead_tokens(const TlStack* st, int num_tokens, int start_pos) {
  if (start_pos != 0 || st->lead <= 0 || st->gdelta_layers == 0 || st->terms == 3) return 0;
  return num_tokens >= st->exact_below && num_tokens > st->lead ? st->lead : 0;
}
const float* tl_stack_residual(const TlStack* st) { return st->x; }
void tl_stack_set_layer_hook(TlStack* st, tl_stack_layer_hook hook, void* ctx) {
  st->hook = hook;
  st->hook_ctx = ctx;
}

int tl_stack_cache_ptr(TlStack* st, int which, int layer, void** out) {
  TL_REQUIRE(st && st->finalized && out, "tl_stack_cache_ptr: model not finalized");
  TL_REQUIRE(layer >= 0 && layer < (int)st->layers.size(), "tl_stack_cache_ptr: layer %d out of range", layer);
  const Layer* Lp = &st->layers[layer];
  if (which >= 4) {  // 4, 5: what 0, 1 are for the second mixer of a pair
    TL_REQUIRE(Lp->side, "tl_stack_cache_ptr: layer %d has one mixer", layer);
    Lp = Lp->side.get();
    which -= 4;
  }
  if (which == 2 || which == 3) {  // the histories of the convolutions on what the two sublayers read
    *out = which == 2 ? st->layers[layer].canon_hist1 : st->layers[layer].canon_hist2;
    return 0;
  }
  const Layer& L = *Lp;
  // attention: 0 keys, 1 values; delta rule and linear attention: 0 the state S [heads][vdim][dim], 1 the convolution's history
  // latent attention: 0 the rows [max_pos][kv_rank + rot_dim] this layer reads; generalized delta rule: 0 the state
  if (L.sp.mixer == TL_MIXER_SWA) *out = which == 0 ? L.kc : L.vc;
  else if (L.sp.mixer == TL_MIXER_LATENT) *out = L.ckv;
  else *out = which == 0 ? L.state : L.hist;
  return 0;
}

void tl_stack_bytes_per_token(const TlStack* st, int pos, double* weight_bytes, double* kv_bytes) {
  const double W = st->cfg.width;
  double wb = 2.0 * W /*embedding row*/ + 2.0 * W * st->cfg.vocab, kb = 0.0;
  std::vector<const Layer*> mixers;
  for (const Layer& L : st->layers) {
    mixers.push_back(&L);
    if (L.side) mixers.push_back(L.side.get());
    if (st->cfg.canon_taps > 0) wb += 2.0 * W * st->cfg.canon_taps * (L.sp.mlp != TL_MLP_NONE ? 2 : 1);
  }
  for (const Layer* Lp : mixers) {
    const Layer& L = *Lp;
    const tl_layer_spec& sp = L.sp;
    wb += 2.0 * W * (L.pd + L.od);
    if (sp.mlp == TL_MLP_UNIT) wb += 2.0 * W * 2.0 * sp.shared_ff;
    if (sp.mixer == TL_MIXER_LATENT) {
      wb += 2.0 * ((double)L.qd * sp.q_rank + (double)sp.heads * sp.kv_rank * (sp.dim + sp.vdim));
      kb += 4.0 * (pos + 2.0) * (sp.kv_rank + sp.rot_dim);  // every head reads the same rows: counted once
      continue;
    }
    if (sp.mixer == TL_MIXER_GDELTA) {
      wb += 2.0 * (double)sp.heads * sp.dim * sp.decay_rank;
      kb += 2.0 * 4.0 * sp.heads * sp.dim * sp.dim;
      continue;
    }
    if (sp.mlp == TL_MLP_MOE)
      wb += 2.0 * W * (sp.experts + 3.0 * sp.expert_ff * sp.top + 3.0 * sp.shared_ff + (sp.shared_gate ? 1.0 : 0.0));
    if (sp.mlp == TL_MLP_DENSE) wb += 2.0 * W * 3.0 * sp.shared_ff;
    if (sp.mixer == TL_MIXER_DELTA || sp.mixer == TL_MIXER_LINEAR) {
      wb += 2.0 * ((double)sp.heads * sp.dim * sp.decay_rank + (double)L.vd * sp.gate_rank);
      kb += 2.0 * 4.0 * sp.heads * sp.vdim * sp.dim;  // the state is read and written
    } else {
      double seen = sp.window > 0 && pos + 1 > sp.window ? sp.window : pos + 1;
      if (sp.window > 0 && sp.keep_first > 0 && pos + 1 > sp.window)
        seen += sp.keep_first < pos + 1 - sp.window ? sp.keep_first : pos + 1 - sp.window;
      kb += 4.0 * (seen + 1.0) * (L.kd + L.vd);
    }
  }
  if (weight_bytes) *weight_bytes = wb;
  if (kv_bytes) *kv_bytes = kb;
}

namespace {

// One token is always FP32-grade: the decode step's GEMVs are, and where TL_STACK_GEMV=0 sends it through the chunk GEMMs
// instead (a test configuration) it takes three terms, whatever the chunks use; so the captured step never depends on a
// setting that may change after the capture.
// The same holds for every portion of fewer than exact_below tokens (one token tile of the small GEMM shape): such a product
// is bound by reading its weights, three terms cost it nothing, and a short portion then agrees with the same tokens decoded
// one by one to FP32 accuracy instead of bf16's.
inline int terms_for(const TlStack* st, int T) { return T < st->exact_below ? 3 : st->terms; }

// y[T][rows] = x[T][cols] W^T for a chunk, or the GEMV for the one token of a decode step
int project(TlStack* st, const uint16_t* w, int rows, int cols, const float* x, int ldx, float* y, int ldy, int T,
            hipStream_t s, float softcap = 0.0f) {
  if (T == 1 && st->gemv_decode) return tl_launch_dense_gemv(w, rows, cols, x, y, s, softcap);
  DenseArgs d = {};
  d.w = w;
  d.rows = rows;
  d.cols = cols;
  d.x = x;
  d.ldx = ldx;
  d.y = y;
  d.ldy = ldy;
  d.T = T;
  d.terms = terms_for(st, T);
  d.softcap = softcap;
  return tl_launch_dense_gemm(d, s);
}

// The routed experts (and the shared expert) of layer L on the rows of `in` (x itself for a post-norm block, the normalised
// h for a parallel one). Leaves: one token -> everything summed (router weights, the shared expert and its gate) in
// one_token_out [W]; a chunk -> st->eout [T * top][W] to be weighted by st->wts, and the shared expert's output in st->sout
// (its per-token gate, if any, in st->sgate).
int moe_experts(TlStack* st, const Layer& L, const Layer& Wt, const float* in, int T, float* one_token_out, hipStream_t s) {
  const tl_layer_spec& sp = L.sp;
  const int W = st->cfg.width, ff = sp.expert_ff, sff = sp.shared_ff, S = T * sp.top;
  if (T == 1 && st->gemv_decode) {
    MoeDecodeArgs d = {};
    d.x = in;
    d.width = W;
    d.top = sp.top;
    d.ids = st->ids;
    d.wts = st->wts;
    d.gu = Wt.gu;
    d.down = Wt.down;
    d.ff = ff;
    d.limit = sp.expert_limit;
    d.sgu = Wt.sgu;
    d.sdown = Wt.sdown;
    d.sff = sff;
    d.slimit = sp.shared_limit;
    d.alpha = sp.act_alpha;
    d.up_add = sp.glu_up_add;
    d.glu_kind = sp.glu;
    d.sgate = sp.shared_gate ? st->sgate : nullptr;
    d.act = st->act_buf;
    d.y = one_token_out;
    return tl_launch_moe_decode(d, s);
  }
  TL_TRY(tl_launch_moe_plan(st->ids, S, sp.experts, st->off, st->slot_of, s));
  DenseArgs g = {};  // gate | up of every slot, grouped by expert: item p reads token slot_of[p] / top
  g.w = Wt.gu;
  g.rows = 2 * ff;
  g.cols = W;
  g.x = in;
  g.ldx = W;
  g.y = st->act_buf;  // the gated unit is applied in the epilogue: [S][ff]
  g.ldy = ff;
  g.T = S;
  g.terms = terms_for(st, T);
  g.x_rows = st->slot_of;
  g.x_div = sp.top;
  g.groups = sp.experts;
  g.group_off = st->off;
  g.glu = 1;
  g.glu_limit = sp.expert_limit;
  g.glu_alpha = sp.act_alpha;
  g.glu_up_add = sp.glu_up_add;
  g.glu_kind = sp.glu;
  TL_TRY(tl_launch_dense_gemm(g, s));
  DenseArgs d = {};  // down: item p writes the row of its slot, so that a token's choices lie side by side
  d.w = Wt.down;
  d.rows = W;
  d.cols = ff;
  d.x = st->act_buf;
  d.ldx = ff;
  d.y = st->eout;
  d.ldy = W;
  d.T = S;
  d.terms = terms_for(st, T);
  d.y_rows = st->slot_of;
  d.groups = sp.experts;
  d.group_off = st->off;
  TL_TRY(tl_launch_dense_gemm(d, s));
  if (sff) {
    DenseArgs u = {};  // the shared expert's gate | up with the gated unit in the epilogue, then its down projection
    u.w = Wt.sgu;
    u.rows = 2 * sff;
    u.cols = W;
    u.x = in;
    u.ldx = W;
    u.y = st->sact;
    u.ldy = sff;
    u.T = T;
    u.terms = terms_for(st, T);
    u.glu = 1;
    u.glu_limit = sp.shared_limit;
    u.glu_alpha = sp.act_alpha;
    u.glu_up_add = sp.glu_up_add;
    u.glu_kind = sp.glu;
    TL_TRY(tl_launch_dense_gemm(u, s));
    TL_TRY(project(st, Wt.sdown, W, sff, st->sact, sff, st->sout, W, T, s));
  }
  return 0;
}

RouterArgs router_args(TlStack* st, const Layer& L, const Layer& Wt, const float* in, int T) {
  const tl_layer_spec& sp = L.sp;
  RouterArgs r = {};
  r.x = in;
  r.T = T;
  r.width = st->cfg.width;
  r.experts = sp.experts;
  r.top = sp.top;
  r.w = Wt.router;
  r.b = sp.route == TL_ROUTE_TOP_LOGITS ? Wt.router_b : nullptr;
  r.ids = st->ids;
  r.wts = st->wts;
  r.kind = sp.route;
  r.corr = sp.route == TL_ROUTE_SIGMOID_GROUPS ? Wt.router_b : nullptr;
  r.groups = sp.route_groups;
  r.keep = sp.route_keep;
  if (sp.shared_gate) {
    r.gate_w = Wt.sg;
    r.gate_out = st->sgate;
  }
  return r;
}

// x += norm2(ff(x)) of a post-norm block
int moe_layer(TlStack* st, Layer& L, int T, hipStream_t s) {
  const tl_layer_spec& sp = L.sp;
  const Layer& Wt = st->layers[L.wsrc];
  const int W = st->cfg.width;
  if (!st->fuse_router || sp.route != TL_ROUTE_TOP_LOGITS || sp.shared_gate)
    TL_TRY(tl_launch_router(router_args(st, L, Wt, st->x, T), s));  // (otherwise it rode in the x += N1 launch)
  ResidNormArgs n = {};
  n.x = st->x;
  n.T = T;
  n.width = W;
  n.w = Wt.norm2;
  n.eps = st->cfg.norm_eps;
  TL_REQUIRE(!sp.shared_gate, "layer-list engine: a gated shared expert runs in parallel blocks only");
  TL_TRY(moe_experts(st, L, Wt, st->x, T, st->proj, s));
  if (T == 1 && st->gemv_decode) {
    n.a = st->proj;
    return tl_launch_resid_norm(n, s);
  }
  if (sp.shared_ff) n.a = st->sout;
  n.slots = st->eout;
  n.slot_w = st->wts;
  n.top = sp.top;
  return tl_launch_resid_norm(n, s);
}

// ---- mixers: all read `in` [T][W] and leave their output in `out` [T][W] (st->proj unless the caller names another) ----
// pre != NULL: the first product has been done by the caller (rows pre_ld floats apart); `in` is then not read
int swa_mixer(TlStack* st, Layer& L, const Layer& Wt, const float* in, int T, int start_pos, const int* pos_dev, hipStream_t s,
              float* out = nullptr, float* pre = nullptr, int pre_ld = 0) {
  const tl_layer_spec& sp = L.sp;
  const tl_stack_config& c = st->cfg;
  const int W = c.width;
  int ld = pre ? pre_ld : L.pd;
  float* qkv = pre ? pre : st->qkv;
  float* const row0 = qkv;  // the product's rows (the gate columns stay there when q | k | v move on)
  const int ld0 = ld;
  if (!out) out = st->proj;
  if (!pre) TL_TRY(project(st, Wt.wqkv, ld, W, in, W, st->qkv, ld, T, s));
  if (sp.qkv_conv > 0) {  // q | k | v (+ their biases) through a convolution over time; the rest of the row is not touched
    ConvArgs cv = {};
    cv.in = qkv;
    cv.ldi = ld;
    cv.C = L.qd + L.kd + L.vd;
    cv.taps = sp.qkv_conv;
    cv.T = T;
    cv.bias = sp.qkv_bias ? Wt.qkv_b : nullptr;
    cv.w = Wt.conv;
    cv.hist = L.hist;
    cv.out = st->dq;
    cv.ldo = cv.C;
    TL_TRY(tl_launch_causal_conv(cv, s));
    qkv = st->dq;
    ld = cv.C;
  }
  if (L.rotary_path) {
    RotaryArgs r = {};
    r.qk = qkv;
    r.ld = ld;
    r.heads = sp.heads;
    r.kv_heads = sp.kv_heads;
    r.dim = sp.dim;
    r.rot_dims = sp.rot_dims;
    r.freq = Wt.freq;
    r.mscale = Wt.mscale;
    r.unit_norm = sp.qk_norm == TL_QK_NORM_HEAD_UNIT;
    r.eps = c.norm_eps;
    r.kc = L.kc;
    if (sp.values_are_keys) {
      r.vc = L.vc;
    } else {
      r.v_src = qkv + L.qd + L.kd;
      r.v_dst = L.vc;
      r.vd = L.vd;
    }
    r.T = T;
    r.start_pos = start_pos;
    r.pos_dev = pos_dev;
    TL_TRY(tl_launch_rotary(r, s));
  } else {
    QkvPostArgs q = {};
    q.qkv = qkv;
    q.ld = ld;
    q.qd = L.qd;
    q.kd = L.kd;
    q.vd = L.vd;
    const bool normed = sp.qk_norm == TL_QK_NORM_WHOLE || sp.qk_norm == TL_QK_NORM_HEAD_RMS;
    q.q_norm = normed ? Wt.q_norm : nullptr;
    q.k_norm = normed ? Wt.k_norm : nullptr;
    q.head_dim = sp.qk_norm == TL_QK_NORM_HEAD_RMS ? sp.dim : 0;
    q.eps = c.norm_eps;
    q.kc = L.kc;
    q.vc = L.vc;
    q.T = T;
    q.start_pos = start_pos;
    q.pos_dev = pos_dev;
    q.vmix = L.vmix_mode;
    q.v_first = st->v_first;
    q.lambda = Wt.lambda;
    q.q_temp_coef = sp.q_temp_coef;
    q.q_temp_every = sp.q_temp_every;
    TL_TRY(tl_launch_qkv_post(q, s));
  }
  SwaArgs a = {};
  a.q = qkv;
  a.ldq = ld;
  a.kc = L.kc;
  a.vc = L.vc;
  a.out = st->att;
  a.T = T;
  a.heads = sp.heads;
  a.kv_heads = sp.kv_heads;
  a.dim = sp.dim;
  a.vdim = sp.vdim;
  a.window = sp.window;
  a.scale = sp.scale;
  a.start_pos = start_pos;
  a.pos_dev = pos_dev;
  a.keep_first = sp.keep_first;
  a.sigmoid = sp.attn_weight == TL_ATTN_SIGMOID;
  a.sink = sp.attn_weight == TL_ATTN_SOFTMAX_SINK || sp.attn_weight == TL_ATTN_SOFTMAX_LEARNED_SINK;
  a.sink_val = sp.attn_weight == TL_ATTN_SOFTMAX_LEARNED_SINK ? Wt.sinkv : nullptr;
  a.head_bias = a.sigmoid ? Wt.pb : nullptr;
  a.softcap = sp.score_softcap;
  a.dist_r1 = sp.dist_bias ? Wt.r1 : nullptr;
  a.dist_r2 = sp.dist_bias ? Wt.r2 : nullptr;
  a.nsplit = tl_swa_splits(T, sp.window, c.max_positions, sp.keep_first);
  a.ws = st->swa_ws;
  a.done_cnt = st->swa_cnt;
  if (sp.score_maps == 2) {
    // two score maps per head over the same values: q and k rows hold [map 1 | map 2] per head, so each map is a launch over
    // every second block of dim; then o = (a1 - lambda a2) / rms (1 - diff_init) sigmoid(gate)
    a.q_hstride = a.k_hstride = 2 * sp.dim;
    TL_TRY(tl_launch_swa(a, s));
    a.q = qkv + sp.dim;
    a.kc = L.kc + sp.dim;
    a.kld = L.kd;
    a.out = st->att2;
    TL_TRY(tl_launch_swa(a, s));
    HeadNormArgs hn = {};
    hn.o = st->att;
    hn.sub = st->att2;
    hn.sub_coef = Wt.lam;
    hn.gate = sp.out_gate ? row0 + L.gate_off : nullptr;
    hn.gate_ld = ld0;
    hn.out_scale = 1.0f - sp.diff_init;
    hn.T = T;
    hn.heads = sp.heads;
    hn.vdim = sp.vdim;
    hn.eps = c.norm_eps;
    TL_TRY(tl_launch_head_norm(hn, s));
  } else {
    TL_TRY(tl_launch_swa(a, s));
  }
  return project(st, Wt.wo, W, L.od, st->att, L.od, out, W, T, s);
}

int delta_mixer(TlStack* st, Layer& L, const Layer& Wt, const float* in, int T, hipStream_t s, float* out = nullptr,
                float* pre = nullptr, int pre_ld = 0) {
  const tl_layer_spec& sp = L.sp;
  const int W = st->cfg.width, ld = pre ? pre_ld : L.pd, dc = L.qd + L.kd + L.vd, da = sp.heads * sp.dim;
  float* const P = pre ? pre : st->qkv;
  if (!out) out = st->proj;
  if (!pre) TL_TRY(project(st, Wt.wqkv, ld, W, in, W, st->qkv, ld, T, s));  // q | k | v | beta | a1 | g1  (or | a | gate)
  const float* a1 = P + dc + sp.heads;
  if (!sp.decay_per_head) {
    TL_TRY(project(st, Wt.wa2, da, sp.decay_rank, a1, ld, st->da, da, T, s));
    TL_TRY(project(st, Wt.wg2, L.vd, sp.gate_rank, a1 + sp.decay_rank, ld, st->dg, L.vd, T, s));
  }
  DeltaPreArgs p = {};
  p.p = P;
  p.ld = ld;
  p.a = sp.decay_per_head ? a1 : st->da;
  p.a_per_head = sp.decay_per_head;
  p.a_ld = ld;
  p.T = T;
  p.heads = sp.heads;
  p.kv_heads = sp.kv_heads;
  p.dim = sp.dim;
  p.vdim = sp.vdim;
  p.taps = sp.conv_taps;
  p.conv = Wt.conv;
  p.hist = L.hist;
  p.a_log = Wt.a_log;
  p.dt_bias = Wt.dt_bias;
  p.qkv = st->dq;
  p.beta = st->dbeta;
  p.g = st->ddecay;
  TL_TRY(tl_launch_delta_pre(p, s));
  DeltaScanArgs d = {};
  d.q = st->dq;
  d.k = st->dq + L.qd;
  d.ldq = dc;
  d.v = st->dq + L.qd + L.kd;
  d.ldv = dc;
  d.beta = st->dbeta;
  d.g = st->ddecay;
  d.state = L.state;
  d.o = st->att;
  d.T = T;
  d.heads = sp.heads;
  d.kv_heads = sp.kv_heads;
  d.dim = sp.dim;
  d.vdim = sp.vdim;
  TL_TRY(tl_launch_delta_scan(d, s));
  if (sp.decay_per_head) {  // the gate is a direct projection and passes silu
    HeadNormArgs hn = {};
    hn.o = st->att;
    hn.gate = P + L.gate_off;
    hn.gate_ld = ld;
    hn.gate_act = 1;
    hn.out_scale = 1.0f;
    hn.w = Wt.onorm;
    hn.T = T;
    hn.heads = sp.heads;
    hn.vdim = sp.vdim;
    hn.eps = st->cfg.norm_eps;
    TL_TRY(tl_launch_head_norm(hn, s));
  } else {
    TL_TRY(tl_launch_gated_head_norm(st->att, st->dg, Wt.onorm, T, sp.heads, sp.vdim, st->cfg.norm_eps, s));
  }
  return project(st, Wt.wo, W, L.od, st->att, L.od, out, W, T, s);
}

// gated linear attention: q | f | v = W h in one product; silu, the forget gate and what it writes (linear_pre); the delta
// rule's scan without its removal step, k = 1 - f, decay = f; RMS norm per head; W_o
int linear_mixer(TlStack* st, Layer& L, const Layer& Wt, const float* in, int T, hipStream_t s, float* out = nullptr,
                 float* pre = nullptr, int pre_ld = 0) {
  const tl_layer_spec& sp = L.sp;
  const int W = st->cfg.width, ld = pre ? pre_ld : L.pd, hd = sp.heads * sp.dim;
  float* const P = pre ? pre : st->qkv;
  if (!out) out = st->proj;
  if (!pre) TL_TRY(project(st, Wt.wqkv, ld, W, in, W, st->qkv, ld, T, s));
  LinearPreArgs p = {};
  p.p = P;
  p.ld = ld;
  p.T = T;
  p.heads = sp.heads;
  p.dim = sp.dim;
  p.lower = Wt.lower;
  p.f_bias = Wt.f_bias;
  p.qk = st->dq;
  p.g = st->ddecay;
  TL_TRY(tl_launch_linear_pre(p, s));
  DeltaScanArgs d = {};
  d.q = st->dq;
  d.k = st->dq + hd;
  d.ldq = 2 * hd;
  d.v = P + 2 * hd;
  d.ldv = ld;
  d.g = st->ddecay;
  d.state = L.state;
  d.o = st->att;
  d.T = T;
  d.heads = sp.heads;
  d.kv_heads = sp.heads;
  d.dim = sp.dim;
  d.vdim = sp.vdim;
  d.plain_write = 1;
  TL_TRY(tl_launch_delta_scan(d, s));
  HeadNormArgs hn = {};
  hn.o = st->att;
  hn.w = Wt.onorm;
  hn.out_scale = 1.0f;
  hn.T = T;
  hn.heads = sp.heads;
  hn.vdim = sp.vdim;
  hn.eps = st->cfg.norm_eps;
  TL_TRY(tl_launch_head_norm(hn, s));
  return project(st, Wt.wo, W, L.od, st->att, L.od, out, W, T, s);
}

// one product per head: y[t][n * y_stride ..] = W[n] x[t][n * x_stride ..]
int project_heads(TlStack* st, const uint16_t* w, int heads, int rows, int cols, const float* x, int ldx, int x_stride, float* y,
                  int ldy, int y_stride, int T, hipStream_t s) {
  if (T == 1 && st->gemv_decode) return tl_launch_dense_gemv_heads(w, heads, rows, cols, x, x_stride, y, y_stride, s);
  DenseArgs d = {};
  d.w = w;
  d.rows = rows;
  d.cols = cols;
  d.x = x;
  d.ldx = ldx;
  d.y = y;
  d.ldy = ldy;
  d.T = T;
  d.terms = terms_for(st, T);
  d.groups = heads;
  d.x_gstride = x_stride;
  d.y_gstride = y_stride;
  return tl_launch_dense_gemm(d, s);
}

// y = act(W x) on the rows from act_from on
int project_act(TlStack* st, const uint16_t* w, int rows, int cols, const float* x, int ldx, float* y, int ldy, int T, int act,
                int act_from, float act_p, float act_q, hipStream_t s) {
  if (T == 1 && st->gemv_decode) return tl_launch_dense_gemv_act(w, rows, cols, x, y, GemvActArgs{act, act_from, act_p, act_q}, s);
  DenseArgs d = {};
  d.w = w;
  d.rows = rows;
  d.cols = cols;
  d.x = x;
  d.ldx = ldx;
  d.y = y;
  d.ldy = ldy;
  d.T = T;
  d.terms = terms_for(st, T);
  d.act = act;
  d.act_from = act_from;
  d.act_p = act_p;
  d.act_q = act_q;
  return tl_launch_dense_gemm(d, s);
}

int latent_mixer(TlStack* st, Layer& L, const float* in, int T, int start_pos, const int* pos_dev, hipStream_t s) {
  const tl_layer_spec& sp = L.sp;
  const tl_stack_config& c = st->cfg;
  const int W = c.width, ld = L.pd, H = sp.heads, qh = sp.dim + sp.rot_dim, ah = sp.kv_rank + sp.rot_dim;
  TL_TRY(project(st, L.wqkv, ld, W, in, W, st->qkv, ld, T, s));  // query latent | (key/value latent | rotated part) | gates
  LatentPostArgs p = {};
  p.p = st->qkv;
  p.ld = ld;
  p.q_rank = sp.q_rank;
  p.kv_rank = sp.kv_rank;
  p.rot_dim = sp.rot_dim;
  p.q_norm = L.dq_norm;
  p.kv_norm = L.kd ? L.dkv_norm : nullptr;
  p.eps = c.norm_eps;
  p.rot_dims = sp.rot_dims;
  p.freq = L.freq;
  p.cache = L.kd ? L.ckv : nullptr;
  p.T = T;
  p.start_pos = start_pos;
  p.pos_dev = pos_dev;
  TL_TRY(tl_launch_latent_post(p, s));
  TL_TRY(project(st, L.wuq, L.qd, sp.q_rank, st->qkv, ld, st->lq, L.qd, T, s));
  LatentQueryArgs q = {};
  q.q = st->lq;
  q.q_stride = qh;
  q.q_off = sp.dim;
  q.heads = H;
  q.rot_dim = sp.rot_dim;
  q.rot_dims = sp.rot_dims;
  q.freq = L.freq;
  q.T = T;
  q.start_pos = start_pos;
  q.pos_dev = pos_dev;
  if (!pos_dev && st->latent_expand > 0 && T >= st->latent_expand) {
    // A long chunk: keys [W_uk,n c | rotated part] and values W_uv,n c per head for the rows [0, start_pos + T), then ordinary
    // attention with as many key heads as query heads (fewer products per query-key pair than over the latent rows).
    const int P = start_pos + T;
    q.out = st->lq;  // the rotated query part in place
    q.out_stride = qh;
    q.out_off = sp.dim;
    TL_TRY(tl_launch_latent_query(q, s));
    TL_TRY(project_heads(st, L.wuk, H, sp.dim, sp.kv_rank, L.ckv, ah, 0, st->lk, H * qh, qh, P, s));
    TL_TRY(tl_launch_latent_spread(L.ckv, sp.kv_rank, sp.rot_dim, st->lk, H, sp.dim, P, s));
    TL_TRY(project(st, L.wuv, H * sp.vdim, sp.kv_rank, L.ckv, ah, st->lv, H * sp.vdim, P, s));
    SwaArgs e = {};
    e.q = st->lq;
    e.ldq = H * qh;
    e.kc = st->lk;
    e.vc = st->lv;
    e.out = st->att;
    e.T = T;
    e.heads = H;
    e.kv_heads = H;
    e.dim = qh;
    e.vdim = sp.vdim;
    e.scale = sp.scale;
    e.start_pos = start_pos;
    e.nsplit = 1;
    TL_TRY(tl_launch_swa(e, s));
    if (sp.head_gate) TL_TRY(tl_launch_head_gate(st->att, st->qkv + L.gate_off, ld, T, H, sp.vdim, s));
    return project(st, L.wo, W, L.od, st->att, L.od, st->proj, W, T, s);
  }
  // the plain part of head n's query through W_uk,n^T: scores against the cached latent itself
  TL_TRY(project_heads(st, L.wukt, H, sp.kv_rank, sp.dim, st->lq, L.qd, qh, st->lqa, H * ah, ah, T, s));
  q.out = st->lqa;  // the rotated part behind each head's absorbed columns
  q.out_stride = ah;
  q.out_off = sp.kv_rank;
  TL_TRY(tl_launch_latent_query(q, s));
  SwaArgs a = {};
  a.q = st->lqa;
  a.ldq = H * ah;
  a.kc = L.ckv;  // keys: the whole row; values: its first kv_rank columns
  a.vc = L.ckv;
  a.kld = ah;
  a.vld = ah;
  a.out = st->att;
  a.T = T;
  a.heads = H;
  a.kv_heads = 1;
  a.dim = ah;
  a.vdim = sp.kv_rank;
  a.scale = sp.scale;
  a.start_pos = start_pos;
  a.pos_dev = pos_dev;
  a.nsplit = tl_swa_splits(T, 0, c.max_positions, 0);
  a.ws = st->swa_ws;
  a.done_cnt = st->swa_cnt;
  TL_TRY(tl_launch_swa(a, s));
  // head n's weighted latent through W_uv,n (lq is free again)
  TL_TRY(project_heads(st, L.wuv, H, sp.vdim, sp.kv_rank, st->att, H * sp.kv_rank, sp.kv_rank, st->lq, L.od, sp.vdim, T, s));
  if (sp.head_gate) TL_TRY(tl_launch_head_gate(st->lq, st->qkv + L.gate_off, ld, T, H, sp.vdim, s));
  return project(st, L.wo, W, L.od, st->lq, L.od, st->proj, W, T, s);
}

int gdelta_mixer(TlStack* st, Layer& L, const float* in, int T, hipStream_t s) {
  const tl_layer_spec& sp = L.sp;
  const int W = st->cfg.width, ld = L.pd, hd = sp.heads * sp.dim;
  // r | k | v | gate | a | tanh(w1 h)
  TL_TRY(project_act(st, L.wqkv, ld, W, in, W, st->qkv, ld, T, TL_ACT_TANH, 5 * hd, 0.0f, 0.0f, s));
  TL_TRY(project(st, L.wa2, hd, sp.decay_rank, st->qkv + 5 * hd, ld, st->da, hd, T, s));
  GDeltaPreArgs p = {};
  p.p = st->qkv;
  p.ld = ld;
  p.dw = st->da;
  p.w0 = L.w0;
  p.a_bias = L.a_bias;
  p.decay_scale = sp.decay_scale;
  p.T = T;
  p.heads = sp.heads;
  p.dim = sp.dim;
  p.w = st->gw;
  p.u = st->gu;
  p.au = st->gau;
  p.rau = st->grau;
  p.rk = st->grk;
  TL_TRY(tl_launch_gdelta_pre(p, s));
  GDeltaScanArgs d = {};
  d.r = st->qkv;
  d.k = st->qkv + hd;
  d.v = st->qkv + 2 * hd;
  d.ld = ld;
  d.w = st->gw;
  d.u = st->gu;
  d.au = st->gau;
  d.rau = st->grau;
  d.rk = st->grk;
  d.state = L.state;
  d.o = st->att;
  d.T = T;
  d.heads = sp.heads;
  d.dim = sp.dim;
  d.vdim = sp.dim;
  TL_TRY(tl_launch_gdelta_scan(d, s));
  TL_TRY(tl_launch_gated_head_norm_rows(st->att, st->qkv + 3 * hd, ld, L.onorm, 1, T, sp.heads, sp.dim, st->cfg.norm_eps, s));
  return project(st, L.wo, W, L.od, st->att, L.od, st->proj, W, T, s);
}

LnParams ln1_of_layer(const Layer& Wt) { return LnParams{Wt.norm1, Wt.norm1_b}; }

// The launch(es) that finish x in a pre-norm block: x += a_scale a + b_scale b + sum_j slot_w[j] slots[j], and the input of
// whatever reads x next -- sublayer `which` (1: the mixer, 2: the feed-forward) of layer `next`, or nothing (next == NULL) --
// into st->h: its norm and, where the model has one, the convolution over time on top of it (whose history is the reading
// layer's own state, also when it borrows its tensors).
struct Addends {
  const float* a = nullptr;
  float a_scale = 1.0f;
  const float* b = nullptr;
  float b_scale = 1.0f;
  const float* slots = nullptr;
  const float* slot_w = nullptr;
  int top = 0;
};
// *routed (optional): set when the router of `next`'s feed-forward rode in the launch (the caller then launches none)
int finish_x(TlStack* st, const Addends& add, Layer* next, int which, int T, hipStream_t s, bool* routed = nullptr) {
  const tl_stack_config& c = st->cfg;
  const int W = c.width;
  const Layer* Wn = next ? &st->layers[next->wsrc] : nullptr;
  if (c.norm == TL_NORM_LAYER) {
    TL_REQUIRE(add.a && !add.b && !add.slots && add.a_scale == 1.0f, "layer-list engine: a layer-norm block adds one sublayer output");
    LnParams n = {};
    if (Wn) n = which == 1 ? ln1_of_layer(*Wn) : LnParams{Wn->norm2, Wn->norm2_b};
    return tl_launch_resid_ln(st->x, add.a, T, W, n, c.norm_eps, st->h, s);
  }
  const bool canon = c.canon_taps > 0 && Wn;
  ResidRmsArgs r = {};
  r.x = st->x;
  r.T = T;
  r.width = W;
  r.a = add.a;
  r.a_scale = add.a_scale;
  r.b = add.b;
  r.b_scale = add.b_scale;
  r.slots = add.slots;
  r.slot_w = add.slot_w;
  r.top = add.top;
  r.w = Wn ? (which == 1 ? Wn->norm1 : Wn->norm2) : nullptr;
  r.eps = c.norm_eps;
  r.h = canon ? st->hn : st->h;
  const bool one_launch = !canon || (T == 1 && st->fuse_canon);  // h is finished by the norm's own launch
  if (routed) *routed = false;
  if (routed && one_launch && which == 2 && st->fuse_router && next->sp.mlp == TL_MLP_MOE && !next->sp.shared_gate) {
    r.route = router_args(st, *next, *Wn, nullptr, T);  // the router reads the row this launch has just finished
    *routed = true;
  }
  if (canon && T == 1 && st->fuse_canon) {  // one token: norm, convolution and the shift of its history in the same launch
    r.h = st->h;
    r.canon_w = which == 1 ? Wn->canon1 : Wn->canon2;
    r.canon_hist = which == 1 ? next->canon_hist1 : next->canon_hist2;
    r.canon_taps = c.canon_taps;
    return tl_launch_resid_rms(r, s);
  }
  if (r.w || r.a || r.b || r.slots) TL_TRY(tl_launch_resid_rms(r, s));
  if (!canon) return 0;
  ConvArgs cv = {};
  cv.in = st->hn;
  cv.ldi = W;
  cv.C = W;
  cv.taps = c.canon_taps;
  cv.T = T;
  cv.w = which == 1 ? Wn->canon1 : Wn->canon2;
  cv.hist = which == 1 ? next->canon_hist1 : next->canon_hist2;
  cv.add_input = 1;
  cv.out = st->h;
  cv.ldo = W;
  return tl_launch_causal_conv(cv, s);
}

int run_mixer(TlStack* st, Layer& L, const Layer& Wt, int T, int start_pos, const int* pos_dev, hipStream_t s, float* out,
              float* pre = nullptr, int pre_ld = 0) {
  switch (L.sp.mixer) {
    case TL_MIXER_SWA: return swa_mixer(st, L, Wt, st->h, T, start_pos, pos_dev, s, out, pre, pre_ld);
    case TL_MIXER_LATENT: return latent_mixer(st, L, st->h, T, start_pos, pos_dev, s);
    case TL_MIXER_GDELTA: return gdelta_mixer(st, L, st->h, T, s);
    case TL_MIXER_LINEAR: return linear_mixer(st, L, Wt, st->h, T, s, out, pre, pre_ld);
    default: return delta_mixer(st, L, Wt, st->h, T, s, out, pre, pre_ld);
  }
}

// one gated unit on the rows of `in`: W_down unit(W_gate in, W_up in) -> st->sout
int dense_unit(TlStack* st, const Layer& L, const Layer& Wt, const float* in, int T, hipStream_t s) {
  const tl_layer_spec& sp = L.sp;
  const int W = st->cfg.width, ff = sp.shared_ff;
  if (T == 1 && st->gemv_decode) {
    MoeDecodeArgs d = {};  // the one gated unit runs where a shared expert would
    d.x = in;
    d.width = W;
    d.sgu = Wt.sgu;
    d.sdown = Wt.sdown;
    d.sff = ff;
    d.slimit = sp.shared_limit;
    d.alpha = sp.act_alpha;
    d.up_add = sp.glu_up_add;
    d.glu_kind = sp.glu;
    d.act = st->act_buf;
    d.y = st->sout;
    return tl_launch_moe_decode(d, s);
  }
  DenseArgs u = {};
  u.w = Wt.sgu;
  u.rows = 2 * ff;
  u.cols = W;
  u.x = in;
  u.ldx = W;
  u.y = st->sact;
  u.ldy = ff;
  u.T = T;
  u.terms = terms_for(st, T);
  u.glu = 1;
  u.glu_limit = sp.shared_limit;
  u.glu_alpha = sp.act_alpha;
  u.glu_up_add = sp.glu_up_add;
  u.glu_kind = sp.glu;
  TL_TRY(tl_launch_dense_gemm(u, s));
  return project(st, Wt.sdown, W, ff, st->sact, ff, st->sout, W, T, s);
}

// h = the input of the mixer is already in st->h. x += mixer(h) (two mixers side by side: the weighted sum of both); then,
// with a feed-forward, h = its input from the new x, x += ff(h). The launch that finishes x prepares the input of whatever
// reads it next.
int pre_norm_layer(TlStack* st, size_t li, int T, int start_pos, const int* pos_dev, hipStream_t s) {
  Layer& L = st->layers[li];
  const Layer& Wt = st->layers[L.wsrc];
  const tl_layer_spec& sp = L.sp;
  const tl_stack_config& c = st->cfg;
  const int W = c.width;
  Layer* after = li + 1 < st->layers.size() ? &st->layers[li + 1] : nullptr;
  Addends mix;
  mix.a = st->proj;
  if (L.side) {
    // both mixers' first products as one (their matrices lie one behind the other); each then works on its columns
    const int ld = L.pd + L.side->pd;
    TL_TRY(project(st, Wt.wqkv, ld, W, st->h, W, st->qkv, ld, T, s));
    TL_TRY(run_mixer(st, L, Wt, T, start_pos, pos_dev, s, st->proj, st->qkv, ld));
    TL_TRY(run_mixer(st, *L.side, *Wt.side, T, start_pos, pos_dev, s, st->proj2, st->qkv + L.pd, ld));
  } else {
    TL_TRY(run_mixer(st, L, Wt, T, start_pos, pos_dev, s, st->proj, nullptr, 0));
  }
  if (L.side) {
    mix.a_scale = sp.mix_scale;
    mix.b = st->proj2;
    mix.b_scale = sp.side_scale;
  }
  if (sp.mlp == TL_MLP_NONE) return finish_x(st, mix, after, 1, T, s);
  bool routed = false;
  TL_TRY(finish_x(st, mix, &L, 2, T, s, &routed));
  Addends ffo;
  if (sp.mlp == TL_MLP_UNIT) {
    const int ff = sp.shared_ff;
    TL_TRY(project_act(st, Wt.sgu, ff, W, st->h, W, st->sact, ff, T, sp.act, 0, Wt.act_p, Wt.act_q, s));
    TL_TRY(project(st, Wt.sdown, W, ff, st->sact, ff, st->sout, W, T, s));
    ffo.a = st->sout;
  } else if (sp.mlp == TL_MLP_DENSE) {
    TL_TRY(dense_unit(st, L, Wt, st->h, T, s));
    ffo.a = st->sout;
  } else {
    if (!routed) TL_TRY(tl_launch_router(router_args(st, L, Wt, st->h, T), s));
    TL_TRY(moe_experts(st, L, Wt, st->h, T, st->sout, s));
    if (T == 1 && st->gemv_decode) {
      ffo.a = st->sout;  // experts (and a shared expert) already summed with the router weights
    } else {
      ffo.slots = st->eout;
      ffo.slot_w = st->wts;
      ffo.top = sp.top;
      if (sp.shared_ff) ffo.a = st->sout;
    }
  }
  return finish_x(st, ffo, after, 1, T, s);
}

DytParams dyt_of_layer(const Layer& Wt) { return DytParams{Wt.norm1_alpha, Wt.norm1, Wt.norm1_b}; }

// h = norm1(x) (already in st->h); x += mixer(h) + ff(h), and the next block's h in the same launch
int parallel_layer(TlStack* st, size_t li, int T, int start_pos, const int* pos_dev, hipStream_t s) {
  Layer& L = st->layers[li];
  const Layer& Wt = st->layers[L.wsrc];
  const tl_layer_spec& sp = L.sp;
  const int W = st->cfg.width;
  ResidSumArgs r = {};
  r.x = st->x;
  r.T = T;
  r.width = W;
  r.a = st->proj;
  const bool one = T == 1 && st->gemv_decode;
  const bool forked = st->fork && T == 1 && sp.mlp != TL_MLP_NONE;
  hipStream_t fs = forked ? st->side : s;  // the feed-forward's stream
  if (forked) {
    TL_HIP(hipEventRecord(st->ev_fork, s));
    TL_HIP(hipStreamWaitEvent(st->side, st->ev_fork, 0));
  }
  if (sp.mlp == TL_MLP_MOE) {
    TL_TRY(tl_launch_router(router_args(st, L, Wt, st->h, T), fs));
    TL_TRY(moe_experts(st, L, Wt, st->h, T, st->sout, fs));
    if (one) {
      r.b = st->sout;  // experts and shared expert already summed (the gate applied)
    } else {
      r.slots = st->eout;
      r.slot_w = st->wts;
      r.top = sp.top;
      if (sp.shared_ff) {
        r.b = st->sout;
        r.b_gate = sp.shared_gate ? st->sgate : nullptr;
      }
    }
  } else if (sp.mlp == TL_MLP_DENSE) {
    TL_TRY(dense_unit(st, L, Wt, st->h, T, fs));
    r.b = st->sout;
  }
  if (forked) TL_HIP(hipEventRecord(st->ev_join, st->side));
  if (sp.mixer == TL_MIXER_SWA) TL_TRY(swa_mixer(st, L, Wt, st->h, T, start_pos, pos_dev, s));
  else TL_TRY(delta_mixer(st, L, Wt, st->h, T, s));
  if (forked) TL_HIP(hipStreamWaitEvent(s, st->ev_join, 0));
  if (li + 1 < st->layers.size() && st->layers[li + 1].sp.block == TL_BLOCK_PARALLEL) {
    r.next = dyt_of_layer(st->layers[st->layers[li + 1].wsrc]);
    r.h = st->h;
  }
  return tl_launch_resid_sum(r, s);
}

}  // namespace

int tl_stack_forward(TlStack* st, const int* tokens_dev, int T, int start_pos, const int* pos_dev, const int* rows_dev,
                     int n_rows, float* logits_dev, hipStream_t s) {
  TL_REQUIRE(st && st->finalized && tokens_dev, "tl_stack_forward: model not finalized");
  TL_REQUIRE(T > 0 && T <= st->chunk, "tl_stack_forward: %d tokens outside (0, %d]", T, st->chunk);
  TL_REQUIRE(pos_dev || (start_pos >= 0 && start_pos + T <= st->cfg.max_positions),
             "tl_stack_forward: positions [%d, %d) outside the cache of %d", start_pos, start_pos + T, st->cfg.max_positions);
  TL_REQUIRE(n_rows >= 0 && n_rows <= T && (n_rows == 0 || logits_dev), "tl_stack_forward: bad logits request");
  const tl_stack_config& c = st->cfg;
  const int W = c.width;
  const bool dyt = c.norm == TL_NORM_DYT, lnorm = c.norm == TL_NORM_LAYER;
  if (c.norm == TL_NORM_RMS) {
    TL_TRY(tl_launch_embed_rows(st->embed, c.vocab, W, tokens_dev, T, st->x, DytParams{}, st->h, s,
                                c.embed_scale != 0.0f ? c.embed_scale : 1.0f));
    TL_TRY(finish_x(st, Addends{}, &st->layers[0], 1, T, s));
  } else if (lnorm) {
    const LnParams emb = c.embed_norm ? LnParams{st->embed_norm, st->embed_norm_b} : LnParams{};
    TL_TRY(tl_launch_embed_ln(st->embed, c.vocab, W, tokens_dev, T, emb, ln1_of_layer(st->layers[st->layers[0].wsrc]), c.norm_eps,
                              st->x, st->h, s));
  } else if (c.embed_norm) {
    TL_TRY(tl_launch_embed_norm(st->embed, c.vocab, W, tokens_dev, T, st->embed_norm, c.norm_eps, st->x, s));
    if (dyt) TL_TRY(tl_launch_dyt_rows(st->x, W, nullptr, T, dyt_of_layer(st->layers[st->layers[0].wsrc]), st->h, s));
  } else {
    const DytParams first = dyt ? dyt_of_layer(st->layers[st->layers[0].wsrc]) : DytParams{};
    TL_TRY(tl_launch_embed_rows(st->embed, c.vocab, W, tokens_dev, T, st->x, first, st->h, s));
  }
  for (size_t li = 0; li < st->layers.size(); ++li) {
    Layer& L = st->layers[li];
    const tl_layer_spec& sp = L.sp;
    if (sp.block == TL_BLOCK_PARALLEL) {
      TL_TRY(parallel_layer(st, li, T, start_pos, pos_dev, s));
    } else if (sp.block == TL_BLOCK_PRE_NORM) {
      TL_TRY(pre_norm_layer(st, li, T, start_pos, pos_dev, s));
    } else {
      const Layer& Wt = st->layers[L.wsrc];
      TL_TRY(swa_mixer(st, L, Wt, st->x, T, start_pos, pos_dev, s));
      ResidNormArgs n = {};
      n.x = st->x;
      n.T = T;
      n.width = W;
      n.a = st->proj;
      n.w = Wt.norm1;
      n.eps = c.norm_eps;
      if (sp.mlp == TL_MLP_MOE && st->fuse_router && sp.route == TL_ROUTE_TOP_LOGITS && !sp.shared_gate) {
        n.route.w = Wt.router;  // the router reads the row this launch has just finished
        n.route.b = Wt.router_b;
        n.route.experts = sp.experts;
        n.route.top = sp.top;
        n.route.ids = st->ids;
        n.route.wts = st->wts;
      }
      TL_TRY(tl_launch_resid_norm(n, s));
      if (sp.mlp == TL_MLP_MOE) TL_TRY(moe_layer(st, L, T, s));
    }
    if (st->hook) {
      TL_HIP(hipStreamSynchronize(s));
      st->hook(st->hook_ctx, (int)li, st->x, T, W);
    }
  }
  if (n_rows > 0) {
    const int last = T - 1;
    const float* src = st->x;
    if (!rows_dev && n_rows == 1) src = st->x + (size_t)last * W;
    TL_REQUIRE(rows_dev || n_rows == 1 || n_rows == T, "tl_stack_forward: %d rows without a list", n_rows);
    if (dyt) TL_TRY(tl_launch_dyt_rows(src, W, rows_dev, n_rows, DytParams{st->final_alpha, st->final_norm, st->final_b}, st->xn, s));
    else if (lnorm) TL_TRY(tl_launch_ln_rows(src, W, rows_dev, n_rows, LnParams{st->final_norm, st->final_b}, c.norm_eps, st->xn, s));
    else TL_TRY(tl_launch_norm_rows(src, W, rows_dev, n_rows, st->final_norm, c.norm_eps, st->xn, s, c.norm != TL_NORM_RMS));
    TL_TRY(project(st, st->head, c.vocab, W, st->xn, W, logits_dev, c.vocab, n_rows, s, c.logit_softcap));
  }
  return 0;
}
