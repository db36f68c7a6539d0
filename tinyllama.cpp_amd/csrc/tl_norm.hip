// tl_norm.hip — the row-wise FP32 steps between the matrix products of a layer-list model. An RMS norm here is
// y = x / sqrt(mean(x^2) + eps) * weight, eps inside the root; "one-plus" weights are stored around zero and applied as
// (1 + w). Norm-first blocks with the Dynamic Tanh norm (tanh(alpha x) * w + b: elementwise, no statistics) need no staged
// row: embedding gather, residual sum and row gather carry the norm of the block that follows in the same pass. One workgroup per token row (256 threads for the rows of a prompt chunk, 1024 for the few rows of a decode step,
// whose launches are nothing but a chain of memory round trips); a row is staged in LDS, so that it is read from memory once.
#include <math.h>

#include "tl_bf16.h"
#include "tl_route.h"
#include "tl_stack.h"

namespace {

constexpr int kMaxWaves = 16;

__device__ __forceinline__ float block_sum(float v, float* red) {  // red: kMaxWaves floats of LDS; result in every thread
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.0f;
  for (int w = 0; w < (int)(blockDim.x >> 6); ++w) s += red[w];  // in wave order: the same sum in every thread
  return s;
}

inline int row_threads(int rows) { return rows <= 8 ? 1024 : 256; }

__global__ __launch_bounds__(1024) void embed_norm_kernel(const unsigned short* __restrict__ table, int vocab, int width,
                                                         const int* __restrict__ tokens, const float* __restrict__ w,
                                                         float eps, float* __restrict__ x) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  __shared__ float red[kMaxWaves];
  const int t = blockIdx.x, tok = tokens[t];
  const bool in = tok >= 0 && tok < vocab;
  const unsigned short* e = table + (size_t)(in ? tok : 0) * width;
  float ss = 0.0f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = in ? __uint_as_float((unsigned)e[c] << 16) : 0.0f;
    row[c] = v;
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int c = threadIdx.x; c < width; c += blockDim.x) x[(size_t)t * width + c] = row[c] * inv * (1.0f + w[c]);
}

__global__ __launch_bounds__(1024) void qkv_post_kernel(const QkvPostArgs a) {
  __shared__ float red[kMaxWaves];
  const int t = blockIdx.x;
  const int pos = (a.pos_dev ? *a.pos_dev : a.start_pos) + t;
  float* q = a.qkv + (size_t)t * a.ld;
  const float* k = q + a.qd;
  const float* v = k + a.kd;
  if (a.head_dim > 0) {  // every block of head_dim of q and of k on its own, one weight vector each: a wave per block in turn
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6, hd = a.head_dim;
    const int nq = a.qd / hd, nk = a.kd / hd;
    float* kr = a.kc + (size_t)pos * a.kd;
    for (int g = wave; g < nq + nk; g += nw) {
      const bool isq = g < nq;
      const float* src = isq ? q + (size_t)g * hd : k + (size_t)(g - nq) * hd;
      float* dst = isq ? q + (size_t)g * hd : kr + (size_t)(g - nq) * hd;
      const float* w = isq ? a.q_norm : a.k_norm;
      float ss = 0.0f;
      for (int d = lane; d < hd; d += 64) ss += src[d] * src[d];
      ss = tl_wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)hd + a.eps);
      for (int d = lane; d < hd; d += 64) dst[d] = src[d] * inv * w[d];
    }
    float* vr = a.vc + (size_t)pos * a.vd;
    for (int c = threadIdx.x; c < a.vd; c += blockDim.x) vr[c] = v[c];
    return;
  }
  float sq = 0.0f, sk = 0.0f;
  if (a.q_norm)
    for (int c = threadIdx.x; c < a.qd; c += blockDim.x) sq += q[c] * q[c];
  if (a.k_norm)
    for (int c = threadIdx.x; c < a.kd; c += blockDim.x) sk += k[c] * k[c];
  sq = block_sum(sq, red);
  sk = block_sum(sk, red);
  if (a.q_norm) {
    const float inv = 1.0f / sqrtf(sq / (float)a.qd + a.eps);
    for (int c = threadIdx.x; c < a.qd; c += blockDim.x) q[c] = q[c] * inv * a.q_norm[c];
  }
  if (a.q_temp_every > 0) {  // query temperature: grows by the logarithm of the position, in steps of q_temp_every positions
    const float f = 1.0f + a.q_temp_coef * logf((float)((pos + 1) / a.q_temp_every) + 1.0f);
    for (int c = threadIdx.x; c < a.qd; c += blockDim.x) q[c] *= f;
  }
  {
    const float inv = a.k_norm ? 1.0f / sqrtf(sk / (float)a.kd + a.eps) : 1.0f;
    float* kr = a.kc + (size_t)pos * a.kd;
    for (int c = threadIdx.x; c < a.kd; c += blockDim.x) kr[c] = a.k_norm ? k[c] * inv * a.k_norm[c] : k[c];
  }
  float* vr = a.vc + (size_t)pos * a.vd;
  if (a.vmix == 2) {
    const float lam = *a.lambda;
    const float* vf = a.v_first + (size_t)t * a.vd;
    for (int c = threadIdx.x; c < a.vd; c += blockDim.x) vr[c] = (1.0f - lam) * v[c] + lam * vf[c];
  } else {
    float* vf = a.vmix == 1 ? a.v_first + (size_t)t * a.vd : nullptr;
    for (int c = threadIdx.x; c < a.vd; c += blockDim.x) {
      vr[c] = v[c];
      if (vf) vf[c] = v[c];
    }
  }
}

__global__ __launch_bounds__(1024) void resid_norm_kernel(const ResidNormArgs a) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  __shared__ float red[kMaxWaves];
  const int t = blockIdx.x;
  float ss = 0.0f;
  for (int c = threadIdx.x; c < a.width; c += blockDim.x) {
    float y = a.a ? a.a[(size_t)t * a.width + c] : 0.0f;
    if (a.slots) {
      float e = 0.0f;
      for (int j = 0; j < a.top; ++j) e += a.slot_w[t * a.top + j] * a.slots[((size_t)t * a.top + j) * a.width + c];
      y += e;
    }
    row[c] = y;
    ss += y * y;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)a.width + a.eps);
  float* x = a.x + (size_t)t * a.width;
  for (int c = threadIdx.x; c < a.width; c += blockDim.x) {
    const float xn = x[c] + row[c] * inv * (1.0f + a.w[c]);
    x[c] = xn;
    row[c] = xn;  // the updated row stays in LDS for the router below
  }
  if (!a.route.w) return;
  // ---- the router of the feed-forward that follows: logits = W_r x + b over the row in LDS, a wave per expert in turn ----
  __syncthreads();
  float* z = row + ((a.width + 3) & ~3);  // [experts]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nwaves = blockDim.x >> 6;
  const bool vec = (a.width & 7) == 0 && ((size_t)a.route.w & 15) == 0;
  for (int e = wave; e < a.route.experts; e += nwaves) {
    float sdot;
    tl_wave_dot_rows<1>(a.route.w + (size_t)e * a.width, 0, 1, row, a.width, vec, lane, &sdot);
    if (lane == 0) z[e] = sdot + (a.route.b ? a.route.b[e] : 0.0f);
  }
  __syncthreads();
  if (wave == 0)
    tl_route_select(z, a.route.experts, a.route.top, a.route.ids + (size_t)t * a.route.top, a.route.wts + (size_t)t * a.route.top, lane);
}

__global__ __launch_bounds__(1024) void norm_rows_kernel(const float* __restrict__ x, int width, const int* __restrict__ rows,
                                                        const float* __restrict__ w, float eps, float* __restrict__ out,
                                                        float w_add) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  __shared__ float red[kMaxWaves];
  const int i = blockIdx.x;
  const float* xr = x + (size_t)(rows ? rows[i] : i) * width;
  float ss = 0.0f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = xr[c];
    row[c] = v;
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int c = threadIdx.x; c < width; c += blockDim.x) out[(size_t)i * width + c] = row[c] * inv * (w_add + w[c]);
}

// pre-norm blocks with an RMS norm: the residual sum and the norm of what reads x next
__global__ __launch_bounds__(1024) void resid_rms_kernel(const ResidRmsArgs a) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  __shared__ float red[kMaxWaves];
  const int t = blockIdx.x;
  float* xr = a.x + (size_t)t * a.width;
  const bool add = a.a || a.b || a.slots;
  float ss = 0.0f;
  for (int c = threadIdx.x; c < a.width; c += blockDim.x) {
    float v = xr[c];
    if (add) {
      float y = a.a ? a.a_scale * a.a[(size_t)t * a.width + c] : 0.0f;
      if (a.b) y += a.b_scale * a.b[(size_t)t * a.width + c];
      if (a.slots) {
        float e = 0.0f;
        for (int j = 0; j < a.top; ++j) e += a.slot_w[t * a.top + j] * a.slots[((size_t)t * a.top + j) * a.width + c];
        y += e;
      }
      v += y;
      xr[c] = v;
    }
    row[c] = v;
    ss += v * v;
  }
  if (!a.w) return;
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)a.width + a.eps), w_add = a.one_plus ? 1.0f : 0.0f;
  if (!a.canon_w) {
    for (int c = threadIdx.x; c < a.width; c += blockDim.x) {
      const float hv = row[c] * inv * (w_add + a.w[c]);
      a.h[(size_t)t * a.width + c] = hv;
      row[c] = hv;  // (own columns only) what the sublayer reads stays in LDS for the router below
    }
  } else {
    const int H = a.canon_taps - 1;  // (one token: the launcher checks)
    for (int c = threadIdx.x; c < a.width; c += blockDim.x) {
      const float cur = row[c] * inv * (w_add + a.w[c]);
      const unsigned short* w = a.canon_w + (size_t)c * a.canon_taps;
      float acc = tl_bf2f(w[H]) * cur;
      for (int j = 0; j < H; ++j) {
        const float u = a.canon_hist[(size_t)j * a.width + c];
        acc += tl_bf2f(w[j]) * u;
        if (j > 0) a.canon_hist[(size_t)(j - 1) * a.width + c] = u;
      }
      if (H > 0) a.canon_hist[(size_t)(H - 1) * a.width + c] = cur;
      a.h[c] = cur + acc;
      row[c] = cur + acc;
    }
  }
  if (!a.route.w) return;
  // ---- the router of the feed-forward that reads h: logits over the row in LDS, a wave per expert in turn ----
  __syncthreads();
  float* z = row + ((a.width + 3) & ~3);  // [experts] (+ [experts] keys + [groups] for the group-ranked kinds)
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nwaves = blockDim.x >> 6;
  const bool vec = (a.width & 7) == 0 && ((size_t)a.route.w & 15) == 0;
  for (int e = wave; e < a.route.experts; e += nwaves) {
    float sdot;
    tl_wave_dot_rows<1>(a.route.w + (size_t)e * a.width, 0, 1, row, a.width, vec, lane, &sdot);
    if (lane == 0) z[e] = sdot + (a.route.b ? a.route.b[e] : 0.0f);
  }
  __syncthreads();
  if (wave != 0) return;
  int* ids = a.route.ids + (size_t)t * a.route.top;
  float* wts = a.route.wts + (size_t)t * a.route.top;
  if (a.route.kind == TL_ROUTE_SIGMOID_GROUPS)
    tl_route_select_sigmoid_groups(z, z + a.route.experts, z + 2 * a.route.experts, a.route.corr, a.route.experts, a.route.top,
                                   a.route.groups, a.route.keep, ids, wts, lane);
  else if (a.route.kind == TL_ROUTE_SOFTMAX_GROUPS)
    tl_route_select_groups(z, z + a.route.experts, z + 2 * a.route.experts, a.route.experts, a.route.top, a.route.groups,
                           a.route.keep, ids, wts, lane);
  else
    tl_route_select(z, a.route.experts, a.route.top, ids, wts, lane);
}

constexpr int kMaxRowFloats = 16 * 1024;  // 64 KB of LDS for the staged row

// ---- layer norm: mean, then the mean of the squared deviations, both over the row staged in LDS (two passes, FP32) ----------
// row[] holds the input; every thread returns with (mean, 1 / sqrt(var + eps))
__device__ __forceinline__ void ln_stats(const float* row, int width, float eps, float* red, float* mean, float* inv) {
  float sm = 0.0f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) sm += row[c];
  const float mu = block_sum(sm, red) / (float)width;
  float sv = 0.0f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float d = row[c] - mu;
    sv += d * d;
  }
  const float var = block_sum(sv, red) / (float)width;
  *mean = mu;
  *inv = 1.0f / sqrtf(var + eps);
}

__global__ __launch_bounds__(1024) void embed_ln_kernel(const unsigned short* __restrict__ table, int vocab, int width,
                                                       const int* __restrict__ tokens, const LnParams emb, const LnParams next,
                                                       float eps, float* __restrict__ x, float* __restrict__ h) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  __shared__ float red[kMaxWaves];
  const int t = blockIdx.x, tok = tokens[t];
  const bool in = tok >= 0 && tok < vocab;
  const unsigned short* e = table + (size_t)(in ? tok : 0) * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) row[c] = in ? __uint_as_float((unsigned)e[c] << 16) : 0.0f;
  __syncthreads();
  float mu, inv;
  if (emb.w) {
    ln_stats(row, width, eps, red, &mu, &inv);
    for (int c = threadIdx.x; c < width; c += blockDim.x) row[c] = (row[c] - mu) * inv * emb.w[c] + emb.b[c];  // own columns only
    __syncthreads();
  }
  for (int c = threadIdx.x; c < width; c += blockDim.x) x[(size_t)t * width + c] = row[c];
  if (!next.w) return;
  ln_stats(row, width, eps, red, &mu, &inv);
  for (int c = threadIdx.x; c < width; c += blockDim.x) h[(size_t)t * width + c] = (row[c] - mu) * inv * next.w[c] + next.b[c];
}

__global__ __launch_bounds__(1024) void resid_ln_kernel(float* __restrict__ x, const float* __restrict__ a, int width,
                                                       const LnParams next, float eps, float* __restrict__ h) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  __shared__ float red[kMaxWaves];
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = xr[c] + a[(size_t)t * width + c];
    xr[c] = v;
    row[c] = v;
  }
  if (!next.w) return;
  __syncthreads();
  float mu, inv;
  ln_stats(row, width, eps, red, &mu, &inv);
  for (int c = threadIdx.x; c < width; c += blockDim.x) h[(size_t)t * width + c] = (row[c] - mu) * inv * next.w[c] + next.b[c];
}

__global__ __launch_bounds__(1024) void ln_rows_kernel(const float* __restrict__ x, int width, const int* __restrict__ rows,
                                                      const LnParams p, float eps, float* __restrict__ out) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  __shared__ float red[kMaxWaves];
  const int i = blockIdx.x;
  const float* xr = x + (size_t)(rows ? rows[i] : i) * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) row[c] = xr[c];
  __syncthreads();
  float mu, inv;
  ln_stats(row, width, eps, red, &mu, &inv);
  for (int c = threadIdx.x; c < width; c += blockDim.x) out[(size_t)i * width + c] = (row[c] - mu) * inv * p.w[c] + p.b[c];
}

__device__ __forceinline__ float dyt_of(float x, float alpha, float w, float b) { return tanhf(alpha * x) * w + b; }

// grid (column blocks of 256, T)
__global__ __launch_bounds__(256) void embed_rows_kernel(const unsigned short* __restrict__ table, int vocab, int width,
                                                        const int* __restrict__ tokens, float* __restrict__ x,
                                                        const DytParams next, float* __restrict__ h, float scale) {
  const int t = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  const int tok = tokens[t];
  const float v = (tok >= 0 && tok < vocab) ? __uint_as_float((unsigned)table[(size_t)tok * width + c] << 16) * scale : 0.0f;
  x[(size_t)t * width + c] = v;
  if (next.alpha) h[(size_t)t * width + c] = dyt_of(v, *next.alpha, next.w[c], next.b[c]);
}

__global__ __launch_bounds__(256) void resid_sum_kernel(const ResidSumArgs a) {
  const int t = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= a.width) return;
  const size_t i = (size_t)t * a.width + c;
  float y = a.a ? a.a[i] : 0.0f;
  if (a.slots) {
    float e = 0.0f;
    for (int j = 0; j < a.top; ++j) e += a.slot_w[t * a.top + j] * a.slots[((size_t)t * a.top + j) * a.width + c];
    y += e;
  }
  if (a.b) y += a.b_gate ? a.b_gate[t] * a.b[i] : a.b[i];
  const float xn = a.x[i] + y;
  a.x[i] = xn;
  if (a.next.alpha) a.h[i] = dyt_of(xn, *a.next.alpha, a.next.w[c], a.next.b[c]);
}

__global__ __launch_bounds__(256) void dyt_rows_kernel(const float* __restrict__ x, int width, const int* __restrict__ rows,
                                                      const DytParams p, float* __restrict__ out) {
  const int i = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  out[(size_t)i * width + c] = dyt_of(x[(size_t)(rows ? rows[i] : i) * width + c], *p.alpha, p.w[c], p.b[c]);
}

}  // namespace

int tl_launch_embed_rows(const uint16_t* table, int vocab, int width, const int* tokens_dev, int T, float* x, const DytParams& next,
                         float* h, hipStream_t s, float scale) {
  TL_REQUIRE(table && tokens_dev && x && T > 0 && T <= 65535 && vocab > 0 && width > 0, "embed_rows: bad arguments");
  TL_REQUIRE(!next.alpha || (next.w && next.b && h), "embed_rows: a norm without its weights or output");
  embed_rows_kernel<<<dim3((width + 255) / 256, T), 256, 0, s>>>(table, vocab, width, tokens_dev, x, next, h, scale);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_resid_sum(const ResidSumArgs& a, hipStream_t s) {
  TL_REQUIRE(a.x && a.T > 0 && a.T <= 65535 && a.width > 0 && (a.a || a.b || a.slots), "resid_sum: bad arguments");
  TL_REQUIRE(!a.slots || (a.slot_w && a.top > 0), "resid_sum: expert slots without weights");
  TL_REQUIRE(!a.next.alpha || (a.next.w && a.next.b && a.h), "resid_sum: a norm without its weights or output");
  resid_sum_kernel<<<dim3((a.width + 255) / 256, a.T), 256, 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_dyt_rows(const float* x, int width, const int* rows_dev, int n, const DytParams& p, float* out, hipStream_t s) {
  TL_REQUIRE(x && out && p.alpha && p.w && p.b && n > 0 && n <= 65535 && width > 0, "dyt_rows: bad arguments");
  dyt_rows_kernel<<<dim3((width + 255) / 256, n), 256, 0, s>>>(x, width, rows_dev, p, out);
  TL_HIP(hipGetLastError());
  return 0;
}

extern "C" int tl_dyt_norm(const float* x_dev, const float* alpha_dev, const float* weight_dev, const float* bias_dev,
                           float* out_dev, int num_tokens, int width, void* stream) {
  DytParams p = {alpha_dev, weight_dev, bias_dev};
  return tl_launch_dyt_rows(x_dev, width, nullptr, num_tokens, p, out_dev, static_cast<hipStream_t>(stream));
}

int tl_launch_embed_ln(const uint16_t* table, int vocab, int width, const int* tokens_dev, int T, const LnParams& emb,
                       const LnParams& next, float eps, float* x, float* h, hipStream_t s) {
  TL_REQUIRE(table && tokens_dev && x && T > 0 && vocab > 0, "embed_ln: bad arguments");
  TL_REQUIRE(width > 0 && width <= kMaxRowFloats, "embed_ln: width %d outside (0, %d]", width, kMaxRowFloats);
  TL_REQUIRE((!emb.w || emb.b) && (!next.w || (next.b && h)), "embed_ln: a norm without its bias or output");
  embed_ln_kernel<<<T, row_threads(T), sizeof(float) * width, s>>>(table, vocab, width, tokens_dev, emb, next, eps, x, h);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_resid_ln(float* x, const float* a, int T, int width, const LnParams& next, float eps, float* h, hipStream_t s) {
  TL_REQUIRE(x && a && T > 0, "resid_ln: bad arguments");
  TL_REQUIRE(width > 0 && width <= kMaxRowFloats, "resid_ln: width %d outside (0, %d]", width, kMaxRowFloats);
  TL_REQUIRE(!next.w || (next.b && h), "resid_ln: a norm without its bias or output");
  resid_ln_kernel<<<T, row_threads(T), sizeof(float) * width, s>>>(x, a, width, next, eps, h);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_ln_rows(const float* x, int width, const int* rows_dev, int n, const LnParams& p, float eps, float* out,
                      hipStream_t s) {
  TL_REQUIRE(x && out && p.w && p.b && n > 0, "ln_rows: bad arguments");
  TL_REQUIRE(width > 0 && width <= kMaxRowFloats, "ln_rows: width %d outside (0, %d]", width, kMaxRowFloats);
  ln_rows_kernel<<<n, row_threads(n), sizeof(float) * width, s>>>(x, width, rows_dev, p, eps, out);
  TL_HIP(hipGetLastError());
  return 0;
}

extern "C" int tl_layer_norm(const float* x_dev, const float* weight_dev, const float* bias_dev, float* out_dev, int num_tokens,
                             int width, float eps, void* stream) {
  return tl_launch_ln_rows(x_dev, width, nullptr, num_tokens, LnParams{weight_dev, bias_dev}, eps, out_dev,
                           static_cast<hipStream_t>(stream));
}

int tl_launch_embed_norm(const uint16_t* table, int vocab, int width, const int* tokens_dev, int T, const float* w, float eps,
                         float* x, hipStream_t s) {
  TL_REQUIRE(table && tokens_dev && w && x && T > 0 && vocab > 0, "embed_norm: bad arguments");
  TL_REQUIRE(width > 0 && width <= kMaxRowFloats, "embed_norm: width %d outside (0, %d]", width, kMaxRowFloats);
  embed_norm_kernel<<<T, row_threads(T), sizeof(float) * width, s>>>(table, vocab, width, tokens_dev, w, eps, x);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_qkv_post(const QkvPostArgs& a, hipStream_t s) {
  TL_REQUIRE(a.qkv && a.kc && a.vc && a.T > 0 && a.qd > 0 && a.kd > 0 && a.vd > 0 && a.ld >= a.qd + a.kd + a.vd,
             "qkv_post: bad arguments");
  TL_REQUIRE(a.vmix == 0 || a.v_first, "qkv_post: value mixing without a v_first buffer");
  TL_REQUIRE(a.vmix != 2 || a.lambda, "qkv_post: value mixing without its coefficient");
  TL_REQUIRE(a.head_dim == 0 || (a.head_dim > 0 && a.qd % a.head_dim == 0 && a.kd % a.head_dim == 0 && a.q_norm && a.k_norm &&
                                 a.vmix == 0 && a.q_temp_every == 0),
             "qkv_post: a norm per block of %d over %d / %d", a.head_dim, a.qd, a.kd);
  qkv_post_kernel<<<a.T, row_threads(a.T), 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_resid_norm(const ResidNormArgs& a, hipStream_t s) {
  TL_REQUIRE(a.x && a.w && a.T > 0 && (a.a || a.slots), "resid_norm: bad arguments");
  TL_REQUIRE(a.width > 0 && a.width <= kMaxRowFloats, "resid_norm: width %d outside (0, %d]", a.width, kMaxRowFloats);
  TL_REQUIRE(!a.slots || (a.slot_w && a.top > 0), "resid_norm: expert slots without weights");
  size_t lds = sizeof(float) * a.width;
  if (a.route.w) {
    TL_REQUIRE(a.route.ids && a.route.wts && a.route.experts > 0 && a.route.top > 0 && a.route.top <= a.route.experts,
               "resid_norm: bad router arguments");
    lds = sizeof(float) * (((a.width + 3) & ~3) + a.route.experts);
    TL_REQUIRE(lds <= 64 * 1024, "resid_norm: width %d + %d experts do not fit the staged row", a.width, a.route.experts);
  }
  resid_norm_kernel<<<a.T, row_threads(a.T), lds, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_resid_rms(const ResidRmsArgs& a, hipStream_t s) {
  TL_REQUIRE(a.x && a.T > 0 && (a.w || a.a || a.b || a.slots), "resid_rms: bad arguments");
  TL_REQUIRE(a.width > 0 && a.width <= kMaxRowFloats, "resid_rms: width %d outside (0, %d]", a.width, kMaxRowFloats);
  TL_REQUIRE(!a.slots || (a.slot_w && a.top > 0), "resid_rms: expert slots without weights");
  TL_REQUIRE(!a.w || a.h, "resid_rms: a norm without its output");
  TL_REQUIRE(!a.canon_w || (a.T == 1 && a.w && a.canon_taps >= 1 && (a.canon_taps == 1 || a.canon_hist)),
             "resid_rms: the convolution rides along for one token behind a norm (%d tokens, %d taps)", a.T, a.canon_taps);
  size_t lds = sizeof(float) * a.width;
  if (a.route.w) {
    const RouterArgs& r = a.route;
    TL_REQUIRE(a.w && r.ids && r.wts && r.experts > 0 && r.top > 0 && r.top <= r.experts && !r.gate_w,
               "resid_rms: bad router arguments");
    TL_REQUIRE(r.kind == TL_ROUTE_TOP_LOGITS || (r.groups > 0 && r.experts % r.groups == 0 && r.keep > 0 && r.keep <= r.groups &&
                                                  (long long)r.keep * (r.experts / r.groups) >= r.top),
               "resid_rms: %d experts in %d groups, %d kept, top %d", r.experts, r.groups, r.keep, r.top);
    lds = sizeof(float) * (((a.width + 3) & ~3) + 2 * (size_t)r.experts + (r.groups > 0 ? r.groups : 0));
    TL_REQUIRE(lds <= 64 * 1024, "resid_rms: width %d + %d experts do not fit the staged row", a.width, r.experts);
  }
  resid_rms_kernel<<<a.T, row_threads(a.T), lds, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_norm_rows(const float* x, int width, const int* rows_dev, int n, const float* w, float eps, float* out,
                        hipStream_t s, int one_plus) {
  TL_REQUIRE(x && w && out && n > 0, "norm_rows: bad arguments");
  TL_REQUIRE(width > 0 && width <= kMaxRowFloats, "norm_rows: width %d outside (0, %d]", width, kMaxRowFloats);
  norm_rows_kernel<<<n, row_threads(n), sizeof(float) * width, s>>>(x, width, rows_dev, w, eps, out, one_plus ? 1.0f : 0.0f);
  TL_HIP(hipGetLastError());
  return 0;
}

extern "C" int tl_resid_rmsnorm(float* x_dev, const float* y_dev, const float* weight_dev, int num_tokens, int width, float eps,
                                void* stream) {
  ResidNormArgs a = {};
  a.x = x_dev;
  a.T = num_tokens;
  a.width = width;
  a.a = y_dev;
  a.w = weight_dev;
  a.eps = eps;
  return tl_launch_resid_norm(a, static_cast<hipStream_t>(stream));
}
