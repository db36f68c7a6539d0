// tl_delta.hip — the gated delta rule with a decay per key channel, as a mixer of a layer-list model: a recurrent state
// S [dim][vdim] per head instead of a cache of keys. Per token and head (q / k head = head / (heads / kv_heads)):
//
//     S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q        (the read-out sees the token's own write)
//
// with q, k from a short causal convolution over time + silu, made unit vectors per head (q also times dim^-1/2),
// beta = sigmoid(.), g = exp(-exp(A_log[head]) * softplus(a + dt_bias)) per head and key channel. Everything that enters the
// recurrence is FP32, and so is the state.
//
//   delta_pre    one workgroup per token and head: convolution (its last taps - 1 inputs of earlier calls come from a history
//                that is part of the sequence's state), silu, the unit norms, beta and the decay.
//   delta_scan   the recurrence. The columns of S (one per value channel) never mix: o_c = s_c . q, u_c = beta (v_c - s_c . k),
//                s_c <- g * s_c + k u_c. Sixteen lanes share a column (each holds dim / 16 of its key channels in registers),
//                four columns a wave, sixteen a workgroup, heads * vdim / 16 workgroups; the tokens are walked in order with
//                the next token's operands in flight. The three dot products a token needs -- (g s) . k, (g s) . q and k . q,
//                since o = (g s) . q + u (k . q) -- are reduced together over the sixteen lanes with row-local lane swaps, so a
//                token costs one reduction latency, not two. A decode step is the same kernel with one token.
//   gated norm   o / rms(o) * w * sigmoid(gate) per head, in front of the output projection.
//
// A second recurrence lives here beside it, the generalized delta rule: a decay w and a removal rate a per head and key
// channel, the unit key u = k / sqrt(sum k^2 + 1e-6),
//
//     S <- diag(w) S - (a u)(u^T S) + k v^T      (both terms read the old S);   o = S^T r
//
//   gdelta_pre   per token and head: w = exp(-decay_scale sigmoid(dw + w0)), u, a u = sigmoid(a + b_a) u, and the two
//                products that do not touch the state, r . (a u) and r . k.
//   gdelta_scan  the same column-per-16-lanes layout as delta_scan. With x = u . s and y = (w r) . s over the OLD column s,
//                o_c = y - (r . a u) x + (r . k) v_c and s <- w s - (a u) x + k v_c: the two sums over the state are reduced
//                together, so a token again costs one reduction latency.
#include <math.h>

#include "tl_bf16.h"
#include "tl_stack.h"

namespace {

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// grid (T, 2 * kv_heads + heads): a workgroup of 128 threads owns one head of one token -- a q head, a k head (convolution,
// silu, unit norm), or a v head (convolution, silu) together with that head's decay channels and beta. One token (the decode
// step) is thereby spread over as many workgroups as the layer has heads.
__global__ __launch_bounds__(128) void delta_pre_kernel(const DeltaPreArgs a) {
  __shared__ float red[2];
  const int t = blockIdx.x, unit = blockIdx.y, tid = threadIdx.x;
  const int qd = a.kv_heads * a.dim, vd = a.heads * a.vdim, C = 2 * qd + vd, H = a.taps - 1;
  const bool is_v = unit >= 2 * a.kv_heads;
  const int n = is_v ? a.vdim : a.dim;                                            // channels of this head
  const int c0 = is_v ? 2 * qd + (unit - 2 * a.kv_heads) * a.vdim : unit * a.dim;  // its first channel
  float* out = a.qkv + (size_t)t * C + c0;
  float ss = 0.0f;
  float y[4];  // n <= 512: four channels a thread
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int d = tid + 128 * r;
    y[r] = 0.0f;
    if (d >= n) continue;
    const int c = c0 + d;
    const unsigned short* w = a.conv + (size_t)c * a.taps;
    float acc = 0.0f;
    for (int j = 0; j < a.taps; ++j) {
      const int tt = t - H + j;  // token of this tap, relative to the call
      const float in = tt >= 0 ? a.p[(size_t)tt * a.ld + c] : a.hist[(size_t)(H + tt) * C + c];
      acc += tl_bf2f(w[j]) * in;
    }
    y[r] = acc * sigmoidf_(acc);
    ss += y[r] * y[r];
    if (a.T == 1 && H > 0) {  // one token: this thread is the only reader of its channel's history, so it may shift it now
      for (int j = 0; j + 1 < H; ++j) a.hist[(size_t)j * C + c] = a.hist[(size_t)(j + 1) * C + c];
      a.hist[(size_t)(H - 1) * C + c] = a.p[c];
    }
  }
  float inv = 1.0f;
  if (!is_v) {
    ss = tl_wave_sum(ss);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    inv = 1.0f / sqrtf(red[0] + red[1] + 1e-6f);
    if (unit < a.kv_heads) inv *= 1.0f / sqrtf((float)a.dim);
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int d = tid + 128 * r;
    if (d < n) out[d] = y[r] * inv;
  }
  if (!is_v) return;
  const int h = unit - 2 * a.kv_heads, gd = a.heads * a.dim;
  if (tid == 0) a.beta[(size_t)t * a.heads + h] = sigmoidf_(a.p[(size_t)t * a.ld + C + h]);
  const float rate = expf(a.a_log[h]);
  if (a.a_per_head) {  // one decay for the whole head, spread over its key channels
    const float gh = expf(-rate * softplusf_(a.a[(size_t)t * a.a_ld + h] + a.dt_bias[h]));
    for (int d = tid; d < a.dim; d += 128) a.g[(size_t)t * gd + h * a.dim + d] = gh;
    return;
  }
  for (int d = tid; d < a.dim; d += 128) {
    const int c = h * a.dim + d;
    a.g[(size_t)t * gd + c] = expf(-rate * softplusf_(a.a[(size_t)t * gd + c] + a.dt_bias[c]));
  }
}

// after a call of several tokens: the history becomes the last taps - 1 inputs (a call shorter than that keeps the tail of
// the old history in front). A thread owns a channel and walks its rows in ascending order, so no row is read after it was
// overwritten.
__global__ __launch_bounds__(256) void conv_history_kernel(const DeltaPreArgs a) {
  const int qd = a.kv_heads * a.dim, C = 2 * qd + a.heads * a.vdim, H = a.taps - 1;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  for (int i = 0; i < H; ++i) {
    const int src = a.T - H + i;  // token whose input lands in row i
    a.hist[(size_t)i * C + c] = src >= 0 ? a.p[(size_t)src * a.ld + c] : a.hist[(size_t)(i + a.T) * C + c];
  }
}

// sum over the 16 lanes of a row, result in all of them: lane swaps inside quads, then mirrored halves (no LDS round trip)
__device__ __forceinline__ float row16_sum(float x) {
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x141, 0xf, 0xf, false));  // row_half_mirror
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x140, 0xf, 0xf, false));  // row_mirror
  return x;
}

// E key channels per lane: dim <= 16 E. grid (vdim / 16 rounded up, heads), 256 threads.
// The operands of 16 (8 for the largest key size) tokens at a time (k, q, g of the head; v of the workgroup's 16 columns; beta) are staged in LDS by
// all threads together, the next stage's global loads in flight while the tokens of the stage in hand are walked: a token
// then waits for an LDS read, not for a round trip to memory.
template <int E>
__global__ __launch_bounds__(256) void delta_scan_kernel(const DeltaScanArgs a) {
  constexpr int DELTA_TB = E == 16 ? 8 : 16;  // tokens per stage (48 KB of LDS at most)
  constexpr int DP = 16 * E;                 // padded key size
  constexpr int NL = (DELTA_TB * DP) / 256;  // k / q / g elements a thread stages = E
  __shared__ __attribute__((aligned(16))) float sk_[2][DELTA_TB][DP], sq_[2][DELTA_TB][DP], sg_[2][DELTA_TB][DP];
  __shared__ float sv_[2][DELTA_TB][16], sb_[2][DELTA_TB];
  const int tid = threadIdx.x, sub = tid & 15, cl = tid >> 4;
  const int col = blockIdx.x * 16 + cl, h = blockIdx.y;
  const int kvh = h / (a.heads / a.kv_heads);
  const bool live = col < a.vdim;           // lanes of a column beyond vdim compute on zeros and store nothing
  const int d0 = sub * E;
  float* sp = a.state + ((size_t)h * a.vdim + (live ? col : 0)) * a.dim;
  float s[E];
#pragma unroll
  for (int e = 0; e < E; ++e) s[e] = (live && d0 + e < a.dim) ? sp[d0 + e] : 0.0f;
  const float* qp = a.q + (size_t)kvh * a.dim;
  const float* kp = a.k + (size_t)kvh * a.dim;
  const float* gp = a.g + (size_t)h * a.dim;
  const int gd = a.heads * a.dim;
  // staging registers: element i of this thread is (token i * 256 + tid) / DP, channel (i * 256 + tid) % DP of the stage
  float rk[NL], rq[NL], rg[NL], rv, rb;
  auto fetch = [&](int t0) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int idx = i * 256 + tid, tt = idx / DP, d = idx % DP;
      const bool in = t0 + tt < a.T && d < a.dim;
      rk[i] = in ? kp[(size_t)(t0 + tt) * a.ldq + d] : 0.0f;
      rq[i] = in ? qp[(size_t)(t0 + tt) * a.ldq + d] : 0.0f;
      rg[i] = in ? gp[(size_t)(t0 + tt) * gd + d] : 0.0f;
    }
    const int tt = tid >> 4, c = blockIdx.x * 16 + (tid & 15);
    rv = (tt < DELTA_TB && t0 + tt < a.T && c < a.vdim) ? a.v[(size_t)(t0 + tt) * a.ldv + (size_t)h * a.vdim + c] : 0.0f;
    rb = (tid < DELTA_TB && t0 + tid < a.T) ? (a.beta ? a.beta[(size_t)(t0 + tid) * a.heads + h] : 1.0f) : 0.0f;
  };
  auto stash = [&](int b) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int idx = i * 256 + tid, tt = idx / DP, d = idx % DP;
      sk_[b][tt][d] = rk[i];
      sq_[b][tt][d] = rq[i];
      sg_[b][tt][d] = rg[i];
    }
    if ((tid >> 4) < DELTA_TB) sv_[b][tid >> 4][tid & 15] = rv;
    if (tid < DELTA_TB) sb_[b][tid] = rb;
  };
  fetch(0);
  stash(0);
  __syncthreads();
  int b = 0;
  for (int t0 = 0; t0 < a.T; t0 += DELTA_TB, b ^= 1) {
    const bool more = t0 + DELTA_TB < a.T;
    if (more) fetch(t0 + DELTA_TB);  // in flight under this stage's tokens
    const int nt = a.T - t0 < DELTA_TB ? a.T - t0 : DELTA_TB;
    for (int tt = 0; tt < nt; ++tt) {
      float kc[E], qc[E], gc[E];
#pragma unroll
      for (int e = 0; e < E; ++e) {
        kc[e] = sk_[b][tt][d0 + e];
        qc[e] = sq_[b][tt][d0 + e];
        gc[e] = sg_[b][tt][d0 + e];
      }
      const float vc = sv_[b][tt][cl], bc = sb_[b][tt];
      float sk = 0.0f, sq = 0.0f, kq = 0.0f;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        s[e] *= gc[e];
        sk += s[e] * kc[e];
        sq += s[e] * qc[e];
        kq += kc[e] * qc[e];
      }
      sk = row16_sum(sk);
      sq = row16_sum(sq);
      kq = row16_sum(kq);
      const float u = a.plain_write ? bc * vc : bc * (vc - sk);
#pragma unroll
      for (int e = 0; e < E; ++e) s[e] += kc[e] * u;
      if (live && sub == 0) a.o[(size_t)(t0 + tt) * a.heads * a.vdim + (size_t)h * a.vdim + col] = sq + u * kq;
    }
    if (more) stash(b ^ 1);  // the other buffer: its last readers passed the barrier at the end of the stage before
    __syncthreads();
  }
  if (live) {
#pragma unroll
    for (int e = 0; e < E; ++e)
      if (d0 + e < a.dim) sp[d0 + e] = s[e];
  }
}

// a wave per (token, head); gate rows gate_ld floats apart; weights of its own for every head or one vector for all
__global__ __launch_bounds__(256) void head_norm_kernel(const HeadNormArgs a) {
  const int i = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (i >= a.T * a.heads) return;
  const int t = i / a.heads, h = i - t * a.heads, vdim = a.vdim;
  float* x = a.o + (size_t)i * vdim;
  const float* sub = a.sub ? a.sub + (size_t)i * vdim : nullptr;
  const float* g = a.gate ? a.gate + (size_t)t * a.gate_ld + (size_t)h * vdim : nullptr;
  const float* wh = a.w ? a.w + (a.w_per_head ? (size_t)h * vdim : 0) : nullptr;
  const float scale = a.out_scale;
  float ss = 0.0f;
  for (int d = lane; d < vdim; d += 64) {
    const float v = sub ? x[d] - a.sub_coef * sub[d] : x[d];
    ss += v * v;
  }
  ss = tl_wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)vdim + a.eps);
  for (int d = lane; d < vdim; d += 64) {
    float v = (sub ? x[d] - a.sub_coef * sub[d] : x[d]) * inv * scale;
    if (wh) v *= wh[d];
    if (g) v *= a.gate_act == 1 ? g[d] * sigmoidf_(g[d]) : sigmoidf_(g[d]);
    x[d] = v;
  }
}

// grid (column blocks of 256 over heads * dim, T)
__global__ __launch_bounds__(256) void linear_pre_kernel(const LinearPreArgs a) {
  const int t = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x, hd = a.heads * a.dim;
  if (c >= hd) return;
  const float* row = a.p + (size_t)t * a.ld;
  const float q = row[c], z = row[hd + c] + a.f_bias[c], low = a.lower[c];
  a.qk[(size_t)t * 2 * hd + c] = q * sigmoidf_(q);
  a.qk[(size_t)t * 2 * hd + hd + c] = (1.0f - low) * sigmoidf_(-z);  // 1 - f
  a.g[(size_t)t * hd + c] = low + (1.0f - low) * sigmoidf_(z);
}

// grid (T, heads): a workgroup of 128 threads owns one head of one token (dim <= 512: four channels a thread)
__global__ __launch_bounds__(128) void gdelta_pre_kernel(const GDeltaPreArgs a) {
  __shared__ float red[3][2];
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int hd = a.heads * a.dim;
  const float* row = a.p + (size_t)t * a.ld;
  const float* rp = row + (size_t)h * a.dim;
  const float* kp = row + hd + (size_t)h * a.dim;
  const float* ap = row + 4 * (size_t)hd + (size_t)h * a.dim;
  const size_t o0 = (size_t)t * hd + (size_t)h * a.dim;
  float kv[4], rv[4], av[4];
  float ss = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int d = tid + 128 * j;
    kv[j] = rv[j] = av[j] = 0.0f;
    if (d >= a.dim) continue;
    kv[j] = kp[d];
    rv[j] = rp[d];
    av[j] = sigmoidf_(ap[d] + a.a_bias[h * a.dim + d]);
    ss += kv[j] * kv[j];
    a.w[o0 + d] = expf(-a.decay_scale * sigmoidf_(a.dw[o0 + d] + a.w0[h * a.dim + d]));
  }
  ss = tl_wave_sum(ss);
  if ((tid & 63) == 0) red[0][tid >> 6] = ss;
  __syncthreads();
  const float inv = 1.0f / sqrtf(red[0][0] + red[0][1] + 1e-6f);
  float s_rau = 0.0f, s_rk = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int d = tid + 128 * j;
    if (d >= a.dim) continue;
    const float u = kv[j] * inv, au = av[j] * u;
    a.u[o0 + d] = u;
    a.au[o0 + d] = au;
    s_rau += rv[j] * au;
    s_rk += rv[j] * kv[j];
  }
  s_rau = tl_wave_sum(s_rau);
  s_rk = tl_wave_sum(s_rk);
  if ((tid & 63) == 0) {
    red[1][tid >> 6] = s_rau;
    red[2][tid >> 6] = s_rk;
  }
  __syncthreads();
  if (tid == 0) {
    a.rau[(size_t)t * a.heads + h] = red[1][0] + red[1][1];
    a.rk[(size_t)t * a.heads + h] = red[2][0] + red[2][1];
  }
}

// E key channels per lane: dim <= 16 E. grid (vdim / 16 rounded up, heads), 256 threads; staging as in delta_scan_kernel
// (five key-channel vectors per token here: r, k, w, u, a u).
template <int E>
__global__ __launch_bounds__(256) void gdelta_scan_kernel(const GDeltaScanArgs a) {
  constexpr int TB = E == 16 ? 4 : E == 8 ? 8 : 16;  // tokens per stage (40 KB of LDS at most)
  constexpr int DP = 16 * E;                           // padded key size
  constexpr int NL = (TB * DP) / 256;                  // elements of each vector a thread stages
  __shared__ __attribute__((aligned(16))) float sr_[2][TB][DP], sk_[2][TB][DP], sw_[2][TB][DP], su_[2][TB][DP], sa_[2][TB][DP];
  __shared__ float sv_[2][TB][16], sc_[2][TB][2];
  const int tid = threadIdx.x, sub = tid & 15, cl = tid >> 4;
  const int col = blockIdx.x * 16 + cl, h = blockIdx.y;
  const bool live = col < a.vdim;  // lanes of a column beyond vdim compute on zeros and store nothing
  const int d0 = sub * E;
  float* sp = a.state + ((size_t)h * a.vdim + (live ? col : 0)) * a.dim;
  float s[E];
#pragma unroll
  for (int e = 0; e < E; ++e) s[e] = (live && d0 + e < a.dim) ? sp[d0 + e] : 0.0f;
  const int hd = a.heads * a.dim;
  const float* rp = a.r + (size_t)h * a.dim;
  const float* kp = a.k + (size_t)h * a.dim;
  const size_t c0 = (size_t)h * a.dim;
  float rr[NL], rk[NL], rw[NL], ru[NL], ra[NL], rv, rc;
  auto fetch = [&](int t0) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int idx = i * 256 + tid, tt = idx / DP, d = idx % DP;
      const bool in = t0 + tt < a.T && d < a.dim;
      const size_t g = (size_t)(t0 + tt) * hd + c0 + d;
      rr[i] = in ? rp[(size_t)(t0 + tt) * a.ld + d] : 0.0f;
      rk[i] = in ? kp[(size_t)(t0 + tt) * a.ld + d] : 0.0f;
      rw[i] = in ? a.w[g] : 0.0f;
      ru[i] = in ? a.u[g] : 0.0f;
      ra[i] = in ? a.au[g] : 0.0f;
    }
    const int tt = tid >> 4, c = blockIdx.x * 16 + (tid & 15);
    rv = (tt < TB && t0 + tt < a.T && c < a.vdim) ? a.v[(size_t)(t0 + tt) * a.ld + (size_t)h * a.vdim + c] : 0.0f;
    const int t2 = tid >> 1;  // threads 0 .. 2 TB - 1: (r . a u, r . k) of the stage's tokens
    rc = (t2 < TB && t0 + t2 < a.T) ? ((tid & 1) ? a.rk : a.rau)[(size_t)(t0 + t2) * a.heads + h] : 0.0f;
  };
  auto stash = [&](int b) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int idx = i * 256 + tid, tt = idx / DP, d = idx % DP;
      sr_[b][tt][d] = rr[i];
      sk_[b][tt][d] = rk[i];
      sw_[b][tt][d] = rw[i];
      su_[b][tt][d] = ru[i];
      sa_[b][tt][d] = ra[i];
    }
    if ((tid >> 4) < TB) sv_[b][tid >> 4][tid & 15] = rv;
    if ((tid >> 1) < TB) sc_[b][tid >> 1][tid & 1] = rc;
  };
  fetch(0);
  stash(0);
  __syncthreads();
  int b = 0;
  for (int t0 = 0; t0 < a.T; t0 += TB, b ^= 1) {
    const bool more = t0 + TB < a.T;
    if (more) fetch(t0 + TB);  // in flight under this stage's tokens
    const int nt = a.T - t0 < TB ? a.T - t0 : TB;
    for (int tt = 0; tt < nt; ++tt) {
      float rc_[E], kc[E], wc[E], uc[E], ac[E];
#pragma unroll
      for (int e = 0; e < E; ++e) {
        rc_[e] = sr_[b][tt][d0 + e];
        kc[e] = sk_[b][tt][d0 + e];
        wc[e] = sw_[b][tt][d0 + e];
        uc[e] = su_[b][tt][d0 + e];
        ac[e] = sa_[b][tt][d0 + e];
      }
      const float vc = sv_[b][tt][cl], rau = sc_[b][tt][0], rkk = sc_[b][tt][1];
      float x = 0.0f, y = 0.0f;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        x += uc[e] * s[e];
        s[e] *= wc[e];
        y += rc_[e] * s[e];
      }
      x = row16_sum(x);
      y = row16_sum(y);
#pragma unroll
      for (int e = 0; e < E; ++e) s[e] += kc[e] * vc - ac[e] * x;
      if (live && sub == 0) a.o[(size_t)(t0 + tt) * a.heads * a.vdim + (size_t)h * a.vdim + col] = y - rau * x + rkk * vc;
    }
    if (more) stash(b ^ 1);  // the other buffer: its last readers passed the barrier at the end of the stage before
    __syncthreads();
  }
  if (live) {
#pragma unroll
    for (int e = 0; e < E; ++e)
      if (d0 + e < a.dim) sp[d0 + e] = s[e];
  }
}

}  // namespace

int tl_launch_delta_pre(const DeltaPreArgs& a, hipStream_t s) {
  TL_REQUIRE(a.p && a.a && a.conv && a.a_log && a.dt_bias && a.qkv && a.beta && a.g && a.T > 0, "delta_pre: bad arguments");
  TL_REQUIRE(a.heads > 0 && a.kv_heads > 0 && a.heads % a.kv_heads == 0 && a.dim > 0 && a.vdim > 0,
             "delta_pre: %d heads over %d query/key heads, sizes %d / %d", a.heads, a.kv_heads, a.dim, a.vdim);
  TL_REQUIRE(a.taps >= 1 && (a.taps == 1 || a.hist), "delta_pre: %d taps", a.taps);
  const int C = 2 * a.kv_heads * a.dim + a.heads * a.vdim;
  TL_REQUIRE(a.ld >= C + a.heads, "delta_pre: row stride %d below %d", a.ld, C + a.heads);
  TL_REQUIRE(!a.a_per_head || a.a_ld >= a.heads, "delta_pre: a decay per head with row stride %d", a.a_ld);
  TL_REQUIRE(a.dim <= 512 && a.vdim <= 512, "delta_pre: head sizes %d / %d above 512", a.dim, a.vdim);
  TL_REQUIRE(2 * a.kv_heads + a.heads <= 65535, "delta_pre: too many heads");
  delta_pre_kernel<<<dim3(a.T, 2 * a.kv_heads + a.heads), 128, 0, s>>>(a);
  if (a.T > 1 && a.taps > 1) conv_history_kernel<<<(C + 255) / 256, 256, 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_delta_scan(const DeltaScanArgs& a, hipStream_t s) {
  TL_REQUIRE(a.q && a.k && a.v && (a.beta || a.plain_write) && a.g && a.state && a.o && a.T > 0, "delta_scan: bad arguments");
  TL_REQUIRE(a.heads > 0 && a.kv_heads > 0 && a.heads % a.kv_heads == 0 && a.dim > 0 && a.vdim > 0 && a.heads <= 65535,
             "delta_scan: %d heads over %d query/key heads, sizes %d / %d", a.heads, a.kv_heads, a.dim, a.vdim);
  TL_REQUIRE(a.dim <= 256, "delta_scan: key size %d above 256", a.dim);
  const dim3 grid((a.vdim + 15) / 16, a.heads);
  const int e = (a.dim + 15) / 16;
  if (e <= 1) delta_scan_kernel<1><<<grid, 256, 0, s>>>(a);
  else if (e <= 2) delta_scan_kernel<2><<<grid, 256, 0, s>>>(a);
  else if (e <= 4) delta_scan_kernel<4><<<grid, 256, 0, s>>>(a);
  else if (e <= 8) delta_scan_kernel<8><<<grid, 256, 0, s>>>(a);
  else delta_scan_kernel<16><<<grid, 256, 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_gated_head_norm_rows(float* o, const float* gate, int gate_ld, const float* w, int w_per_head, int T, int heads,
                                   int vdim, float eps, hipStream_t s) {
  TL_REQUIRE(o && gate && w, "gated_head_norm: bad arguments");
  HeadNormArgs a = {};
  a.o = o;
  a.gate = gate;
  a.gate_ld = gate_ld;
  a.w = w;
  a.w_per_head = w_per_head;
  a.out_scale = 1.0f;
  a.T = T;
  a.heads = heads;
  a.vdim = vdim;
  a.eps = eps;
  return tl_launch_head_norm(a, s);
}

int tl_launch_head_norm(const HeadNormArgs& a, hipStream_t s) {
  TL_REQUIRE(a.o && a.T > 0 && a.heads > 0 && a.vdim > 0 && (!a.gate || a.gate_ld >= a.heads * a.vdim), "head_norm: bad arguments");
  TL_REQUIRE(a.gate_act == 0 || a.gate_act == 1, "head_norm: gate activation %d", a.gate_act);
  const long long n = (long long)a.T * a.heads;
  TL_REQUIRE(n <= 0x7fffffffLL, "head_norm: too many heads");
  head_norm_kernel<<<(unsigned)((n + 3) / 4), 256, 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_linear_pre(const LinearPreArgs& a, hipStream_t s) {
  TL_REQUIRE(a.p && a.lower && a.f_bias && a.qk && a.g && a.T > 0 && a.T <= 65535 && a.heads > 0 && a.dim > 0,
             "linear_pre: bad arguments");
  TL_REQUIRE(a.ld >= 2 * a.heads * a.dim, "linear_pre: row stride %d below %d", a.ld, 2 * a.heads * a.dim);
  linear_pre_kernel<<<dim3((a.heads * a.dim + 255) / 256, a.T), 256, 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_gated_head_norm(float* o, const float* gate, const float* w, int T, int heads, int vdim, float eps, hipStream_t s) {
  return tl_launch_gated_head_norm_rows(o, gate, heads * vdim, w, 0, T, heads, vdim, eps, s);
}

int tl_launch_gdelta_pre(const GDeltaPreArgs& a, hipStream_t s) {
  TL_REQUIRE(a.p && a.dw && a.w0 && a.a_bias && a.w && a.u && a.au && a.rau && a.rk && a.T > 0, "gdelta_pre: bad arguments");
  TL_REQUIRE(a.heads > 0 && a.heads <= 65535 && a.dim > 0 && a.dim <= 512, "gdelta_pre: %d heads of size %d", a.heads, a.dim);
  TL_REQUIRE(a.ld >= 5 * a.heads * a.dim, "gdelta_pre: row stride %d below %d", a.ld, 5 * a.heads * a.dim);
  gdelta_pre_kernel<<<dim3(a.T, a.heads), 128, 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_gdelta_scan(const GDeltaScanArgs& a, hipStream_t s) {
  TL_REQUIRE(a.r && a.k && a.v && a.w && a.u && a.au && a.rau && a.rk && a.state && a.o && a.T > 0, "gdelta_scan: bad arguments");
  TL_REQUIRE(a.heads > 0 && a.heads <= 65535 && a.dim > 0 && a.vdim > 0, "gdelta_scan: %d heads, sizes %d / %d", a.heads, a.dim, a.vdim);
  TL_REQUIRE(a.dim <= 256, "gdelta_scan: key size %d above 256", a.dim);
  const dim3 grid((a.vdim + 15) / 16, a.heads);
  const int e = (a.dim + 15) / 16;
  if (e <= 1) gdelta_scan_kernel<1><<<grid, 256, 0, s>>>(a);
  else if (e <= 2) gdelta_scan_kernel<2><<<grid, 256, 0, s>>>(a);
  else if (e <= 4) gdelta_scan_kernel<4><<<grid, 256, 0, s>>>(a);
  else if (e <= 8) gdelta_scan_kernel<8><<<grid, 256, 0, s>>>(a);
  else gdelta_scan_kernel<16><<<grid, 256, 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

extern "C" int tl_general_delta(const float* p_dev, int ld, const float* dw_dev, const float* w0_dev, const float* a_bias_dev,
                                float decay_scale, float* state_dev, float* o_dev, float* scratch_dev, int num_tokens, int heads,
                                int dim, void* stream) {
  TL_REQUIRE(scratch_dev && num_tokens > 0 && heads > 0 && dim > 0, "tl_general_delta: bad arguments");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t n = (size_t)num_tokens * heads * dim, m = (size_t)num_tokens * heads;
  GDeltaPreArgs p = {};
  p.p = p_dev;
  p.ld = ld;
  p.dw = dw_dev;
  p.w0 = w0_dev;
  p.a_bias = a_bias_dev;
  p.decay_scale = decay_scale;
  p.T = num_tokens;
  p.heads = heads;
  p.dim = dim;
  p.w = scratch_dev;
  p.u = scratch_dev + n;
  p.au = scratch_dev + 2 * n;
  p.rau = scratch_dev + 3 * n;
  p.rk = scratch_dev + 3 * n + m;
  TL_TRY(tl_launch_gdelta_pre(p, s));
  GDeltaScanArgs d = {};
  d.r = p_dev;
  d.k = p_dev + (size_t)heads * dim;
  d.v = p_dev + 2 * (size_t)heads * dim;
  d.ld = ld;
  d.w = p.w;
  d.u = p.u;
  d.au = p.au;
  d.rau = p.rau;
  d.rk = p.rk;
  d.state = state_dev;
  d.o = o_dev;
  d.T = num_tokens;
  d.heads = heads;
  d.dim = dim;
  d.vdim = dim;
  return tl_launch_gdelta_scan(d, s);
}

extern "C" int tl_delta_prepare(const float* p_dev, int ld, const float* a_dev, int num_tokens, int heads, int kv_heads, int dim,
                                int vdim, int taps, const void* conv_bf16_dev, float* history_dev, const float* a_log_dev,
                                const float* dt_bias_dev, float* qkv_dev, float* beta_dev, float* g_dev, void* stream) {
  DeltaPreArgs a = {};
  a.p = p_dev;
  a.ld = ld;
  a.a = a_dev;
  a.T = num_tokens;
  a.heads = heads;
  a.kv_heads = kv_heads;
  a.dim = dim;
  a.vdim = vdim;
  a.taps = taps;
  a.conv = static_cast<const uint16_t*>(conv_bf16_dev);
  a.hist = history_dev;
  a.a_log = a_log_dev;
  a.dt_bias = dt_bias_dev;
  a.qkv = qkv_dev;
  a.beta = beta_dev;
  a.g = g_dev;
  return tl_launch_delta_pre(a, static_cast<hipStream_t>(stream));
}

extern "C" int tl_gated_head_norm(float* o_dev, const float* gate_dev, const float* weight_dev, int num_tokens, int heads, int vdim,
                                  float eps, void* stream) {
  return tl_launch_gated_head_norm(o_dev, gate_dev, weight_dev, num_tokens, heads, vdim, eps, static_cast<hipStream_t>(stream));
}

extern "C" int tl_delta_rule(const float* q_dev, const float* k_dev, const float* v_dev, const float* beta_dev, const float* g_dev,
                             float* state_dev, float* o_dev, int num_tokens, int heads, int kv_heads, int dim, int vdim,
                             void* stream) {
  DeltaScanArgs a = {};
  a.q = q_dev;
  a.k = k_dev;
  a.ldq = kv_heads * dim;
  a.v = v_dev;
  a.ldv = heads * vdim;
  a.beta = beta_dev;
  a.g = g_dev;
  a.state = state_dev;
  a.o = o_dev;
  a.T = num_tokens;
  a.heads = heads;
  a.kv_heads = kv_heads;
  a.dim = dim;
  a.vdim = vdim;
  return tl_launch_delta_scan(a, static_cast<hipStream_t>(stream));
}

extern "C" int tl_head_norm(float* o_dev, const float* sub_dev, float sub_coef, const float* gate_dev, int gate_ld, int gate_act,
                            const float* weight_dev, int weight_per_head, float out_scale, int num_tokens, int heads, int vdim,
                            float eps, void* stream) {
  HeadNormArgs a = {};
  a.o = o_dev;
  a.sub = sub_dev;
  a.sub_coef = sub_coef;
  a.gate = gate_dev;
  a.gate_ld = gate_ld;
  a.gate_act = gate_act;
  a.w = weight_dev;
  a.w_per_head = weight_per_head;
  a.out_scale = out_scale;
  a.T = num_tokens;
  a.heads = heads;
  a.vdim = vdim;
  a.eps = eps;
  return tl_launch_head_norm(a, static_cast<hipStream_t>(stream));
}

extern "C" int tl_gated_linear_attention(const float* p_dev, int ld, const float* lower_dev, const float* f_bias_dev,
                                         float* state_dev, float* o_dev, float* scratch_dev, int num_tokens, int heads, int dim,
                                         int vdim, void* stream) {
  TL_REQUIRE(scratch_dev && num_tokens > 0 && heads > 0 && dim > 0 && vdim > 0, "tl_gated_linear_attention: bad arguments");
  TL_REQUIRE(ld >= 2 * heads * dim + heads * vdim, "tl_gated_linear_attention: row stride %d below q | f | v", ld);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t hd = (size_t)heads * dim;
  LinearPreArgs p = {};
  p.p = p_dev;
  p.ld = ld;
  p.T = num_tokens;
  p.heads = heads;
  p.dim = dim;
  p.lower = lower_dev;
  p.f_bias = f_bias_dev;
  p.qk = scratch_dev;
  p.g = scratch_dev + 2 * hd * num_tokens;
  TL_TRY(tl_launch_linear_pre(p, s));
  DeltaScanArgs d = {};
  d.q = p.qk;
  d.k = p.qk + hd;
  d.ldq = (int)(2 * hd);
  d.v = p_dev + 2 * hd;
  d.ldv = ld;
  d.g = p.g;
  d.state = state_dev;
  d.o = o_dev;
  d.T = num_tokens;
  d.heads = heads;
  d.kv_heads = heads;
  d.dim = dim;
  d.vdim = vdim;
  d.plain_write = 1;
  return tl_launch_delta_scan(d, s);
}
