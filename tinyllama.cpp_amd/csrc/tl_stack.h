// tl_stack.h — inside libtlhip.so: the layer-list engine (tl_stack.hip) and the operators it is built from. A "stack" model
// is described layer by layer (tl_stack_config, include/tlhip.h) instead of by the fixed Llama block of tl_model.hip; it
// lives behind the same tl_model handle and entry points (decode step, prefill, generation, cache reset).
//
// Operators (each with its sizes and constants as arguments, so that another design can use them):
//   tl_dense.hip  bf16 weight matrices [rows][cols]: GEMV (one token) and MFMA GEMM (a chunk of tokens, optionally grouped
//                 by expert with gathered input rows / scattered output rows); FP32 activations and accumulation
//   tl_swa.hip    sliding-window attention without rotation, key and value sizes independent, over a flat FP32 cache
//   tl_moe.hip    router (top-k, softmax over the chosen logits), grouping plan, clamped gated activation, decode GEMVs
//   tl_norm.hip   RMS norms with zero-centred weights: embedding gather + norm, whole-projection q/k norm + value mixing +
//                 cache write, residual += norm(sublayer output), row-gathering norm in front of the head; layer norms of
//                 pre-norm blocks (residual sum + the norm of the sublayer that follows)
//   tl_rope.hip   rotary positions, per-head unit norm;  tl_delta.hip  two delta-rule recurrences with their preparation
//   tl_conv.hip   a short causal convolution over time per channel with its history (sublayer inputs; projected q, k, v)
//   tl_latent.hip latent attention: norms of the latents, the rotated shared key part, cache rows, per-head output gate
#pragma once
#include "tl_internal.h"

// ---- tl_dense.hip ------------------------------------------------------------------------------------------------------
struct DenseArgs {
  const uint16_t* w;     // bf16 [groups][rows][cols], row-major (as the checkpoint stores it: y = W x)
  int rows, cols;        // output features, input features
  const float* x;        // activations, row r at x + r * ldx
  int ldx;
  float* y;              // outputs, row r at y + r * ldy
  int ldy;
  int T;                 // items (tokens); with group_off: upper bound of the items of one group
  int terms;             // bf16 MFMAs per product: 1 = activations rounded to bf16, 3 = FP32-grade (hi + mid + lo split)
  const int* x_rows;     // optional (device): item i reads activation row x_rows[i] / x_div
  int x_div;
  const int* y_rows;     // optional (device): item i writes output row y_rows[i]
  int groups;            // > 1 (or group_off set): group g uses matrix g and the items [group_off[g], group_off[g+1])
  const int* group_off;  // device, groups + 1 entries
  // glu = 1: the rows are (gate, up) pairs -- row 2 i the gate, row 2 i + 1 the up projection of unit i -- and the epilogue
  // stores the clamped gated unit of each pair instead of the pair: y[item][i] (ldy >= rows / 2), see tl_launch_glu_act
  int glu;
  float glu_limit, glu_alpha;
  float glu_up_add;      // 1 in the formula above; a design may add something else (0: the plain gated unit)
  int glu_kind;          // tl_glu_kind (0: the clamped swish unit above; TL_GLU_RELU: max(gate, 0) * up)
  float softcap;         // > 0 (not with glu): y <- softcap * tanh(y / softcap)
  // act != 0 (not with glu): a tl_act_kind on the output features from act_from on (TL_ACT_XIELU: act_p = softplus(p),
  // act_q = 1/2 + softplus(q))
  int act, act_from;
  float act_p, act_q;
  // groups > 1 without group_off: one product per head over ALL items -- group g multiplies matrix g with the columns
  // x[.][g * x_gstride ..] (0: every head reads the same columns) and writes y[.][g * y_gstride ..]
  int x_gstride, y_gstride;
};
int tl_launch_dense_gemm(const DenseArgs& a, hipStream_t s);
// y[rows] = W x for one token, FP32 throughout (weights widened exactly)
int tl_launch_dense_gemv(const uint16_t* w, int rows, int cols, const float* x, float* y, hipStream_t s, float softcap = 0.0f);
struct GemvActArgs {
  int act, act_from;     // as DenseArgs
  float act_p, act_q;
};
int tl_launch_dense_gemv_act(const uint16_t* w, int rows, int cols, const float* x, float* y, const GemvActArgs& act, hipStream_t s);
// one token, one product per head: y[g * y_stride + r] = W[g][r] . x[g * x_stride ..]
int tl_launch_dense_gemv_heads(const uint16_t* w, int groups, int rows, int cols, const float* x, int x_stride, float* y,
                               int y_stride, hipStream_t s);
// the activation of tl_act_kind, for kernels that apply it themselves
__host__ __device__ inline float tl_act_apply(int act, float z, float p, float q) {
  if (act == TL_ACT_XIELU) return z > 0.0f ? p * z * z + 0.5f * z : q * (expm1f(z) - z) + 0.5f * z;
  if (act == TL_ACT_TANH) return tanhf(z);
  return z;
}

// the gated unit of tl_glu_kind, for every kernel that applies it
__host__ __device__ inline float tl_glu_apply(int kind, float g, float u, float limit, float alpha, float up_add) {
  if (kind == TL_GLU_RELU) return fmaxf(g, 0.0f) * u;
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-alpha * g)) * (u + up_add);
}

// ---- tl_swa.hip --------------------------------------------------------------------------------------------------------
struct SwaArgs {
  const float* q;   // [T][ldq]: head h of token t at q + t * ldq + h * dim
  int ldq;
  const float* kc;  // keys   [max_pos][kv_heads * dim]
  const float* vc;  // values [max_pos][kv_heads * vdim]
  float* out;       // [T][heads * vdim]
  int T, heads, kv_heads, dim, vdim;
  int window;       // position i sees j with 0 <= i - j < window (<= 0: every j <= i)
  float scale;
  int start_pos;    // position of token 0 ...
  const int* pos_dev;  // ... or, when set, read from the device (graph replay)
  // nsplit > 1: the visible keys of a (token, head) are dealt to nsplit workgroups whose partial results meet in ws
  // (tl_swa_ws_floats floats) and are combined by a second small launch: the decode step's way to fill the chip
  int nsplit;
  float* ws;
  // optional: T * heads zeroed counters (left at zero by every launch): the last workgroup of a (token, head) to arrive merges
  // the records itself and the second launch falls away
  unsigned* done_cnt;
  // keys j < keep_first stay visible to every later position, beyond the window (at their true positions)
  int keep_first;
  // sigmoid != 0: the weight of a visible key is sigmoid(score + head_bias[head]) (head_bias may be NULL) and is not
  // normalised over the keys; 0: softmax
  int sigmoid;
  const float* head_bias;
  // sink != 0 (softmax only): the denominator has one more term, exp(0): a key of score 0 that carries no value
  int sink;
  // rows of the caches are kld / vld floats apart (0: kv_heads * dim, kv_heads * vdim): a cache of latent rows serves as
  // keys (the whole row) and values (its first vdim columns) at once
  int kld, vld;
  // heads of a query row / key row are q_hstride / k_hstride floats apart (0: dim): with two score maps per head laid out side
  // by side, one launch per map walks every second block of dim
  int q_hstride, k_hstride;
  float softcap;            // > 0: score <- softcap * tanh(score / softcap), after the scale
  const float* dist_r1;     // optional [heads] (with dist_r2): score <- score - r1 ln(1 + r2 (i - j)), after the cap
  const float* dist_r2;
  const float* sink_val;    // with sink: the sink's score per head (NULL: 0)
};
int tl_launch_swa(const SwaArgs& a, hipStream_t s);
int tl_swa_splits(int T, int window, int max_pos, int keep_first = 0);  // splits worth having for T tokens over a cache of max_pos rows
size_t tl_swa_ws_floats(int T, int heads, int vdim, int nsplit);

// ---- tl_norm.hip -------------------------------------------------------------------------------------------------------
// x[t] = embed[token[t]] / rms * (1 + w)   (bf16 table; an id outside the table embeds as zeros)
int tl_launch_embed_norm(const uint16_t* table, int vocab, int width, const int* tokens_dev, int T, const float* w, float eps,
                         float* x, hipStream_t s);
struct QkvPostArgs {
  float* qkv;            // [T][ld]: q (qd) | k (kd) | v (vd) of a token; q is normalised in place
  int ld, qd, kd, vd;
  const float* q_norm;   // plain weights over the whole projection (NULL: no norm)
  const float* k_norm;
  float eps;
  float* kc;             // [max_pos][kd], row pos
  float* vc;             // [max_pos][vd]
  int T, start_pos;
  const int* pos_dev;
  int vmix;              // 0: v as it is; 1: this layer's v is kept in v_first; 2: v = (1 - lambda) v + lambda v_first
  float* v_first;        // [T][vd]
  const float* lambda;   // device scalar (vmix == 2)
  // q_temp_every > 0: q at position p is multiplied by 1 + q_temp_coef * ln(floor((p + 1) / q_temp_every) + 1)
  float q_temp_coef;
  int q_temp_every;
  // head_dim > 0: q_norm / k_norm are ONE weight vector [head_dim] each and every block of head_dim of q and of k is
  // RMS-normed on its own (per head, and per score map where a head has several)
  int head_dim;
};
int tl_launch_qkv_post(const QkvPostArgs& a, hipStream_t s);
// (declared here because the residual norm may carry it; the launcher is tl_moe.hip's)
struct RouterArgs {
  const float* x;        // [T][width]
  int T, width, experts, top;
  const uint16_t* w;     // bf16 [experts][width]
  const float* b;        // [experts]
  int* ids;              // [T][top] chosen experts, largest logit first
  float* wts;            // [T][top] softmax over the chosen logits
  // kind = TL_ROUTE_SOFTMAX_GROUPS: scores = softmax over all experts; `groups` equal groups of neighbours ranked by their
  // best score, only the best `keep` can be chosen from; wts = the chosen scores divided by their sum (+ 1e-20)
  int kind, groups, keep;
  // optional: one more row of weights whose logit becomes a gate per token, gate_out[t] = sigmoid(gate_w . x[t])
  const uint16_t* gate_w;
  float* gate_out;
  // kind = TL_ROUTE_SIGMOID_GROUPS: scores = sigmoid(logits), choice = score + corr[expert]; a group ranks by the sum of its two
  // best choices; wts = the chosen experts' scores as they are
  const float* corr;
};
struct ResidNormArgs {
  float* x;              // [T][width] residual stream, updated in place: x += y / rms(y) * (1 + w)
  int T, width;
  const float* a;        // optional [T][width]
  const float* slots;    // optional [T * top][width] expert outputs, weighted by slot_w
  const float* slot_w;   // [T * top]
  int top;
  const float* w;
  float eps;
  // optional: the router of the feed-forward that reads the updated x rides in this launch (the row is in LDS already):
  // route.w != NULL -> route.ids / route.wts [T][top] as tl_launch_router writes them (route.x / T / width are ignored)
  RouterArgs route;
};
int tl_launch_resid_norm(const ResidNormArgs& a, hipStream_t s);
// pre-norm blocks with an RMS norm: x[t] += a_scale a[t] + b_scale b[t] + sum_j slot_w[j] slots[j]; then, when w is set,
// h[t] = x[t] / sqrt(mean(x[t]^2) + eps) * w (one_plus: * (1 + w)): the norm in front of the sublayer that reads x next
struct ResidRmsArgs {
  float* x;              // [T][width]
  int T, width;
  const float* a;        // optional [T][width]
  float a_scale;
  const float* b;        // optional [T][width]
  float b_scale;
  const float* slots;    // optional [T * top][width] expert outputs, weighted by slot_w
  const float* slot_w;   // [T * top]
  int top;
  const float* w;        // [width] (NULL: no norm asked for)
  int one_plus;
  float eps;
  float* h;              // [T][width]
  // one token (the decode step): the convolution over time on what the sublayer reads rides in this launch --
  // h <- h + conv(h) with canon_w bf16 [width][canon_taps] and its history [canon_taps - 1][width], which is shifted here
  // (a thread is the only reader of its channels' history). canon_w == NULL: none
  const uint16_t* canon_w;
  float* canon_hist;
  int canon_taps;
  // optional: the router of the feed-forward that reads h rides in this launch (the finished row is in LDS): route.w != NULL ->
  // route.ids / route.wts [T][top] as tl_launch_router writes them (route.x / T / width are ignored). Not with a convolution
  // that is a launch of its own (the router reads what the convolution leaves).
  RouterArgs route;
};
int tl_launch_resid_rms(const ResidRmsArgs& a, hipStream_t s);
// ---- norm-first blocks: Dynamic Tanh (elementwise, no statistics) and the plain residual sum ------------------------------
struct DytParams {
  const float* alpha;    // device scalar (NULL: no norm asked for)
  const float* w;        // [width]
  const float* b;        // [width]
};
// x[t] = embed[token[t]] (an id outside the table embeds as zeros); h[t] = tanh(alpha x[t]) * w + b when next.alpha is set
int tl_launch_embed_rows(const uint16_t* table, int vocab, int width, const int* tokens_dev, int T, float* x, const DytParams& next,
                         float* h, hipStream_t s, float scale = 1.0f);
struct ResidSumArgs {
  float* x;              // [T][width] residual stream: x += a + b * b_gate + sum_j slot_w[j] slots[j]
  int T, width;
  const float* a;        // optional [T][width]
  const float* b;        // optional [T][width]
  const float* b_gate;   // optional [T]: one factor per token on b
  const float* slots;    // optional [T * top][width] expert outputs, weighted by slot_w
  const float* slot_w;   // [T * top]
  int top;
  DytParams next;        // optional: h = norm of the updated x for the block that follows (saves that block a launch)
  float* h;
};
int tl_launch_resid_sum(const ResidSumArgs& a, hipStream_t s);
// out[i] = tanh(alpha x[rows[i]]) * w + b   (rows == NULL: row i)
int tl_launch_dyt_rows(const float* x, int width, const int* rows_dev, int n, const DytParams& p, float* out, hipStream_t s);
// out[i] = x[rows[i]] / rms * (1 + w)   (rows == NULL: row i)
int tl_launch_norm_rows(const float* x, int width, const int* rows_dev, int n, const float* w, float eps, float* out,
                        hipStream_t s, int one_plus = 1);

// ---- layer norm (pre-norm blocks): (x - mean) / sqrt(var + eps) * w + b, statistics in FP32 over the row staged in LDS -------
struct LnParams {
  const float* w;        // [width] (NULL: no norm asked for)
  const float* b;        // [width]
};
// x[t] = ln(embed[token[t]]; emb) (emb.w == NULL: the plain row); h[t] = ln(x[t]; next) when next.w is set
int tl_launch_embed_ln(const uint16_t* table, int vocab, int width, const int* tokens_dev, int T, const LnParams& emb,
                       const LnParams& next, float eps, float* x, float* h, hipStream_t s);
// x[t] += a[t]; h[t] = ln(x[t]; next) when next.w is set (the norm in front of the sublayer that follows)
int tl_launch_resid_ln(float* x, const float* a, int T, int width, const LnParams& next, float eps, float* h, hipStream_t s);
// out[i] = ln(x[rows[i]]; p)   (rows == NULL: row i)
int tl_launch_ln_rows(const float* x, int width, const int* rows_dev, int n, const LnParams& p, float eps, float* out,
                      hipStream_t s);

// ---- tl_conv.hip: a short causal convolution over time per channel, with its history as state ----------------------------
// out[t][c] = act(sum_j w[c][j] u[t - taps + 1 + j][c]) (+ u[t][c] with add_input), u[t][c] = in[t][c] (+ bias[c]); the inputs
// of the taps - 1 tokens before this call come from hist [taps - 1][C] (oldest first; zeros for an empty sequence), which
// afterwards holds the last taps - 1 inputs u. out must not overlap in when T > 1.
struct ConvArgs {
  const float* in;       // [T][ldi], channels [0, C)
  int ldi, C, taps, T;
  const float* bias;     // optional [C]
  const uint16_t* w;     // bf16 [C][taps], the last tap is the current token's
  float* hist;           // [taps - 1][C]
  int act;               // 0: none, 1: silu
  int add_input;
  float* out;            // [T][ldo]
  int ldo;
};
int tl_launch_causal_conv(const ConvArgs& a, hipStream_t s);

// ---- tl_latent.hip: what sits between the products of a latent-attention mixer ------------------------------------------
struct LatentPostArgs {
  float* p;              // [T][ld]: query latent (q_rank) | key/value latent (kv_rank) | rotated key part (rot_dim) | ...
  int ld, q_rank, kv_rank, rot_dim;
  const float* q_norm;   // plain weights [q_rank]: the query latent is RMS-normed in place
  const float* kv_norm;  // plain weights [kv_rank] (NULL: this layer projects no latent of its own; kv_rank columns absent)
  float eps;
  int rot_dims;          // the first rot_dims of the rot_dim part turn, (2i, 2i + 1) by position * freq[i]
  const double* freq;
  float* cache;          // [max_pos][kv_rank + rot_dim]: row pos = normalised latent | rotated key part
  int T, start_pos;
  const int* pos_dev;
};
int tl_launch_latent_post(const LatentPostArgs& a, hipStream_t s);
struct LatentQueryArgs {
  const float* q;        // [T][heads * q_stride]: head n's part to be rotated starts at column n * q_stride + q_off
  int q_stride, q_off;
  float* out;            // [T][heads * out_stride]: it goes to column n * out_stride + out_off (may be q itself: in place)
  int out_stride, out_off;
  int heads, rot_dim, rot_dims;
  const double* freq;
  int T, start_pos;
  const int* pos_dev;
};
int tl_launch_latent_query(const LatentQueryArgs& a, hipStream_t s);
// keys per head for a prompt chunk: k[p][n * (dim + rot_dim) + dim ..] = the rotated part of cache row p, for every head n and
// the rows p < P (the plain parts in front come from a product per head over the same rows)
int tl_launch_latent_spread(const float* cache, int kv_rank, int rot_dim, float* k, int heads, int dim, int P, hipStream_t s);
// o[t][n][:] *= sigmoid(gate[t * gate_ld + n]) for the heads n of a token; o [T][heads * vdim]
int tl_launch_head_gate(float* o, const float* gate, int gate_ld, int T, int heads, int vdim, hipStream_t s);

// ---- tl_moe.hip --------------------------------------------------------------------------------------------------------
int tl_launch_router(const RouterArgs& a, hipStream_t s);
// slots (t * top + j) grouped by expert: off[experts + 1], slot_of[T * top]
int tl_launch_moe_plan(const int* ids, int n_slots, int experts, int* off, int* slot_of, hipStream_t s);
// out[p][i] = g * sigmoid(alpha * g) * (u + 1), g = min(in[p][i], limit), u = clamp(in[p][ff + i], -limit, limit)
int tl_launch_glu_act(const float* in, int P, int ff, float limit, float alpha, float* out, hipStream_t s);
// one token: the chosen experts' (and the shared expert's) gate/up GEMVs + activation, then the down GEMVs summed with the
// router weights into y[width]. gu matrices are [2 * ff][width] with row 2 i the gate and row 2 i + 1 the up projection of
// unit i (the layout the chunk GEMM's fused activation wants); down [width][ff].
struct MoeDecodeArgs {
  const float* x;        // [width]
  int width, top;
  const int* ids;        // [top] (device)
  const float* wts;      // [top]
  const uint16_t* gu;    // [experts][2 * ff][width]
  const uint16_t* down;  // [experts][width][ff]
  int ff;
  float limit;
  const uint16_t* sgu;   // shared expert (NULL: none)
  const uint16_t* sdown;
  int sff;
  float slimit;
  float alpha;
  float* act;            // scratch [top * ff + sff]
  float* y;              // [width]
  float up_add;          // the gated unit's (u + up_add)
  const float* sgate;    // optional device scalar: factor on the shared expert's output
  int glu_kind;          // tl_glu_kind
};
int tl_launch_moe_decode(const MoeDecodeArgs& a, hipStream_t s);

// ---- tl_rope.hip -------------------------------------------------------------------------------------------------------
// f[i] (i < rot_dims / 2) and the factor on cos / sin of a layer's rotary positions (tl_layer_spec: rot_*), computed in double
void tl_rotary_frequencies(int rot_dims, double base, double factor, double original, double fast, double slow, double* f,
                           float* mscale);
struct RotaryArgs {
  float* qk;             // [T][ld]: q heads (heads * dim) | k heads (kv_heads * dim) of a token, updated in place
  int ld, heads, kv_heads, dim;
  int rot_dims;          // the first rot_dims dimensions of a head rotate: (2i, 2i + 1) by position * freq[i]
  const double* freq;    // device [rot_dims / 2], double: position * frequency is formed and reduced to [-pi, pi] in double
  float mscale;          // on cos and sin
  int unit_norm;         // 1: after the rotation a head is divided by its root mean square (eps inside the root)
  float eps;
  float* kc;             // optional cache [max_pos][kv_heads * dim]: row pos receives the finished keys
  float* vc;             // optional cache [max_pos][kv_heads * dim]: row pos receives the keys AS PROJECTED (values = keys)
  const float* v_src;    // optional: a projected value row of vd floats per token (v_src + t * ld) ...
  float* v_dst;          // ... copied to row pos of this cache [max_pos][vd]
  int vd;
  int T, start_pos;
  const int* pos_dev;
};
int tl_launch_rotary(const RotaryArgs& a, hipStream_t s);
// sin and cos of position * frequency: the product is formed and brought into [-pi, pi] in double, the functions are FP32
__device__ __forceinline__ void tl_rotary_sincos(int pos, double freq, float* sn, float* cs) {
  const double full = (double)pos * freq;
  const float ang = (float)(full - 6.283185307179586476925 * rint(full * 0.159154943091895335769));
  sincosf(ang, sn, cs);
}

// ---- tl_delta.hip ------------------------------------------------------------------------------------------------------
struct DeltaPreArgs {
  const float* p;        // [T][ld] projections of a token: q (kv_heads * dim) | k (kv_heads * dim) | v (heads * vdim) | beta (heads)
  int ld;
  const float* a;        // [T][heads * dim] decay pre-activation (before the bias)
  int T, heads, kv_heads, dim, vdim, taps;
  const uint16_t* conv;  // bf16 [channels][taps], channels = q | k | v in that order; the last tap is the current token's
  float* hist;           // [taps - 1][channels] inputs of the tokens before this call (oldest first); updated
  const float* a_log;    // [heads]
  const float* dt_bias;  // [heads * dim]
  float* qkv;            // out [T][channels]: silu(conv), q and k unit vectors per head (eps 1e-6), q times dim^-1/2
  float* beta;           // out [T][heads] = sigmoid
  float* g;              // out [T][heads * dim] = exp(-exp(a_log) softplus(a + dt_bias))
  // a_per_head != 0: one decay per head -- a holds one pre-activation per head (token t, head h at a + t * a_ld + h), dt_bias
  // is [heads], and g receives the head's decay in every key channel
  int a_per_head, a_ld;
};
int tl_launch_delta_pre(const DeltaPreArgs& a, hipStream_t s);
struct DeltaScanArgs {
  const float* q;        // token t, head j at q + t * ldq + j * dim (kv_heads heads)
  const float* k;
  int ldq;
  const float* v;        // token t, head h at v + t * ldv + h * vdim
  int ldv;
  const float* beta;     // [T][heads]
  const float* g;        // [T][heads * dim]
  float* state;          // [heads][vdim][dim]: column c of head h's S, contiguous over the key channels; updated
  float* o;              // [T][heads * vdim]
  int T, heads, kv_heads, dim, vdim;
  // plain_write != 0: nothing is removed before the write, u = beta v (a gated linear recurrence S <- diag(g) S + k v^T);
  // beta may then be NULL (1)
  int plain_write;
};
int tl_launch_delta_scan(const DeltaScanArgs& a, hipStream_t s);
// o[t][h] <- o / sqrt(mean(o^2) + eps) * w * sigmoid(gate[t][h]) per head (w [vdim] shared by the heads); in place
int tl_launch_gated_head_norm(float* o, const float* gate, const float* w, int T, int heads, int vdim, float eps, hipStream_t s);
// the same with gate rows gate_ld floats apart and, w_per_head != 0, weights [heads * vdim] of their own for every head
int tl_launch_gated_head_norm_rows(float* o, const float* gate, int gate_ld, const float* w, int w_per_head, int T, int heads,
                                   int vdim, float eps, hipStream_t s);
// the general form: o <- (o - sub_coef * sub) / sqrt(mean(.^2) + eps) * w * gate_fn(gate) * out_scale per head; sub, w and gate
// are optional; gate_act 0: sigmoid, 1: silu
struct HeadNormArgs {
  float* o;              // [T][heads * vdim], in place
  const float* sub;      // optional [T][heads * vdim]
  float sub_coef;
  const float* gate;     // optional, token t at gate + t * gate_ld
  int gate_ld, gate_act;
  const float* w;        // optional [vdim] (w_per_head: [heads * vdim])
  int w_per_head;
  float out_scale;       // (a factor of 1 has to be said: 0 gives zeros)
  int T, heads, vdim;
  float eps;
};
int tl_launch_head_norm(const HeadNormArgs& a, hipStream_t s);
// what precedes the gated linear recurrence of TL_MIXER_LINEAR: p [T][ld] = q | f (heads * dim each) | ...;
// qk [T][2 * heads * dim] = silu(q) | 1 - f, g [T][heads * dim] = f, f = lower + (1 - lower) sigmoid(p_f + f_bias)
struct LinearPreArgs {
  const float* p;
  int ld, T, heads, dim;
  const float* lower;    // [heads * dim]
  const float* f_bias;   // [heads * dim]
  float* qk;
  float* g;
};
int tl_launch_linear_pre(const LinearPreArgs& a, hipStream_t s);
// ---- generalized delta rule: S <- diag(w) S - (a u)(u^T S) + k v^T (both terms read the old S), o = S^T r ------------------
struct GDeltaPreArgs {
  const float* p;        // [T][ld]: r | k | v | gate | a, heads * dim each (the gate is not read here)
  int ld;
  const float* dw;       // [T][heads * dim] pre-activation of the decay
  const float* w0;       // [heads * dim]
  const float* a_bias;   // [heads * dim]
  float decay_scale;     // w = exp(-decay_scale * sigmoid(dw + w0))
  int T, heads, dim;
  float* w;              // out [T][heads * dim] decay
  float* u;              // out [T][heads * dim] unit key k / sqrt(sum k^2 + 1e-6)
  float* au;             // out [T][heads * dim] sigmoid(a + a_bias) * u
  float* rau;            // out [T][heads] r . (a u)
  float* rk;             // out [T][heads] r . k
};
int tl_launch_gdelta_pre(const GDeltaPreArgs& a, hipStream_t s);
struct GDeltaScanArgs {
  const float* r;        // token t, head h at r + t * ld + h * dim
  const float* k;
  const float* v;        // token t, head h at v + t * ld + h * vdim
  int ld;
  const float *w, *u, *au;  // [T][heads * dim]
  const float *rau, *rk;    // [T][heads]
  float* state;          // [heads][vdim][dim]: column c of head h's S, contiguous over the key channels; updated
  float* o;              // [T][heads * vdim]
  int T, heads, dim, vdim;
};
int tl_launch_gdelta_scan(const GDeltaScanArgs& a, hipStream_t s);

// ---- tl_stack.hip: the engine ------------------------------------------------------------------------------------------
struct TlStack;
int tl_stack_create(const tl_stack_config* cfg, TlStack** out);
void tl_stack_free(TlStack* st);
int tl_stack_set_tensor(TlStack* st, const char* name, int dtype, const long long* shape, int ndim, const void* host_data,
                        hipStream_t s);
int tl_stack_finalize(TlStack* st, hipStream_t s);
int tl_stack_reset(TlStack* st, hipStream_t s);
int tl_stack_set_terms(TlStack* st, int terms);
// T tokens (ids on the device) at positions start_pos.. (or *pos_dev..): updates the caches; logits of the n_rows token rows
// listed in rows_dev (NULL with n_rows == 1: the last token) go to logits_dev [n_rows][vocab]. T <= tl_stack_chunk().
int tl_stack_forward(TlStack* st, const int* tokens_dev, int T, int start_pos, const int* pos_dev, const int* rows_dev,
                     int n_rows, float* logits_dev, hipStream_t s);
int tl_stack_chunk(const TlStack* st);
// > 0: a prompt of num_tokens at start_pos should run its first so many tokens as a portion of their own (short portions
// multiply FP32-grade whatever the chunks use); 0: no such wish
int tl_stack_lead_tokens(const TlStack* st, int num_tokens, int start_pos);
int tl_stack_cache_ptr(TlStack* st, int which, int layer, void** out);
// residual stream of the last forward call, [T][width] (tests)
const float* tl_stack_residual(const TlStack* st);
void tl_stack_bytes_per_token(const TlStack* st, int pos, double* weight_bytes, double* kv_bytes);
// called after every layer of a forward call when set (tests: the residual stream layer by layer)
typedef void (*tl_stack_layer_hook)(void* ctx, int layer, const float* x_dev, int T, int width);
void tl_stack_set_layer_hook(TlStack* st, tl_stack_layer_hook hook, void* ctx);
