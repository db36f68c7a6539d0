// tl_latent.hip — what sits between the matrix products of a latent-attention mixer. Such a mixer caches, per token, one
// normalised latent c (kv_rank) and one rotated key part (rot_dim) that all heads share, instead of keys and values per head:
//
//   keys of head n   [W_uk,n c | rotated part],  values  W_uv,n c,  queries  [q_plain,n | q_rotated,n]
//   score            q_plain,n . (W_uk,n c) + q_rot,n . k_rot  =  (W_uk,n^T q_plain,n) . c + q_rot,n . k_rot
//   output           sum_j p_j W_uv,n c_j  =  W_uv,n (sum_j p_j c_j)
//
// so for one token, or a few, attention runs over the CACHE ROWS themselves (tl_swa.hip with one key/value "head": key = the whole row, value = its
// first kv_rank columns), with the query of head n absorbed through W_uk,n^T in front and W_uv,n applied to the weighted sum
// of latents behind (both are one product per head, tl_dense.hip): nothing per head is expanded over the context, and a
// decode step reads kv_rank + rot_dim floats per cached token instead of heads * (dim + rot_dim + vdim).
// A long prompt chunk is the other way round: its cost is the products per (query, key) pair, which the absorbed form makes
// (kv_rank + rot_dim + kv_rank) / (dim + rot_dim + vdim) times as many. There the engine expands keys and values per head for
// the rows the chunk can see (two matrix-core products over the cache rows, latent_spread for the shared rotated part) and
// runs ordinary attention with as many key heads as query heads.
//
//   latent_post    per token: the query latent is RMS-normed in place (plain weights); the key/value latent is RMS-normed and,
//                  with the rotated shared key part behind it, written to row `pos` of the cache.
//   latent_query   per token and head: the rotated query part goes behind the head's absorbed columns.
//   head_gate      head n's output times sigmoid(gate_n).
// Norms, angles and the cache are FP32; the angle is formed in double (tl_rotary_sincos).
#include <math.h>

#include "tl_stack.h"

namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// sum over a workgroup of up to 16 waves; result in every thread
__device__ __forceinline__ float group_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.0f;
  for (int w = 0; w < (int)(blockDim.x >> 6); ++w) s += red[w];
  return s;
}

// grid (T), 256 threads
__global__ __launch_bounds__(256) void latent_post_kernel(const LatentPostArgs a) {
  __shared__ float red[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int pos = (a.pos_dev ? *a.pos_dev : a.start_pos) + t;
  float* row = a.p + (size_t)t * a.ld;
  float ss = 0.0f;
  for (int c = tid; c < a.q_rank; c += 256) ss += row[c] * row[c];
  ss = group_sum(ss, red);
  const float qi = 1.0f / sqrtf(ss / (float)a.q_rank + a.eps);
  for (int c = tid; c < a.q_rank; c += 256) row[c] = row[c] * qi * a.q_norm[c];
  if (!a.kv_norm) return;
  const float* kv = row + a.q_rank;
  float sk = 0.0f;
  for (int c = tid; c < a.kv_rank; c += 256) sk += kv[c] * kv[c];
  sk = group_sum(sk, red);
  const float ki = 1.0f / sqrtf(sk / (float)a.kv_rank + a.eps);
  float* out = a.cache + (size_t)pos * (a.kv_rank + a.rot_dim);
  for (int c = tid; c < a.kv_rank; c += 256) out[c] = kv[c] * ki * a.kv_norm[c];
  const float* kr = kv + a.kv_rank;
  float* outr = out + a.kv_rank;
  for (int i = tid; 2 * i < a.rot_dim; i += 256) {  // pairs (2i, 2i + 1); a last odd dimension passes unchanged
    const int d0 = 2 * i, d1 = d0 + 1;
    float u = kr[d0], v = d1 < a.rot_dim ? kr[d1] : 0.0f;
    if (d1 < a.rot_dims) {
      float sn, cs;
      tl_rotary_sincos(pos, a.freq[i], &sn, &cs);
      const float nu = u * cs - v * sn, nv = v * cs + u * sn;
      u = nu;
      v = nv;
    }
    outr[d0] = u;
    if (d1 < a.rot_dim) outr[d1] = v;
  }
}

// grid (T, heads in fours), a wave per (token, head)
__global__ __launch_bounds__(256) void latent_query_kernel(const LatentQueryArgs a) {
  const int t = blockIdx.x, n = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (n >= a.heads) return;
  const int pos = (a.pos_dev ? *a.pos_dev : a.start_pos) + t;
  const float* src = a.q + ((size_t)t * a.heads + n) * a.q_stride + a.q_off;
  float* dst = a.out + ((size_t)t * a.heads + n) * a.out_stride + a.out_off;
  for (int i = lane; 2 * i < a.rot_dim; i += 64) {
    const int d0 = 2 * i, d1 = d0 + 1;
    float u = src[d0], v = d1 < a.rot_dim ? src[d1] : 0.0f;
    if (d1 < a.rot_dims) {
      float sn, cs;
      tl_rotary_sincos(pos, a.freq[i], &sn, &cs);
      const float nu = u * cs - v * sn, nv = v * cs + u * sn;
      u = nu;
      v = nv;
    }
    dst[d0] = u;
    if (d1 < a.rot_dim) dst[d1] = v;
  }
}

__global__ __launch_bounds__(256) void latent_spread_kernel(const float* __restrict__ cache, int kv_rank, int rot_dim,
                                                           float* __restrict__ k, int heads, int dim, long long total) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;  // (row, head, rotated dimension)
  if (i >= total) return;
  const int r = (int)(i % rot_dim);
  const long long ph = i / rot_dim;
  const long long p = ph / heads;
  k[ph * (dim + rot_dim) + dim + r] = cache[p * (kv_rank + rot_dim) + kv_rank + r];
}

__global__ __launch_bounds__(256) void head_gate_kernel(float* __restrict__ o, const float* __restrict__ gate, int gate_ld,
                                                       int heads, int vdim, long long total) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const long long th = i / vdim;  // token * heads + head
  const int t = (int)(th / heads), n = (int)(th % heads);
  o[i] *= 1.0f / (1.0f + expf(-gate[(size_t)t * gate_ld + n]));
}

}  // namespace

int tl_launch_latent_post(const LatentPostArgs& a, hipStream_t s) {
  TL_REQUIRE(a.p && a.q_norm && a.T > 0 && a.q_rank > 0, "latent_post: bad arguments");
  TL_REQUIRE(!a.kv_norm || (a.cache && a.kv_rank > 0 && a.rot_dim >= 0 && a.ld >= a.q_rank + a.kv_rank + a.rot_dim),
             "latent_post: a key/value latent without its cache, or a row of %d for %d + %d + %d", a.ld, a.q_rank, a.kv_rank, a.rot_dim);
  TL_REQUIRE(a.rot_dims >= 0 && a.rot_dims <= a.rot_dim && (a.rot_dims & 1) == 0 && (a.rot_dims == 0 || a.freq),
             "latent_post: %d turning dimensions of %d", a.rot_dims, a.rot_dim);
  TL_REQUIRE(a.pos_dev || a.start_pos >= 0, "latent_post: negative start position");
  latent_post_kernel<<<a.T, 256, 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_latent_query(const LatentQueryArgs& a, hipStream_t s) {
  TL_REQUIRE(a.q && a.out && a.T > 0 && a.heads > 0 && a.rot_dim >= 0 && a.q_off >= 0 && a.out_off >= 0 &&
                 a.q_stride >= a.q_off + a.rot_dim && a.out_stride >= a.out_off + a.rot_dim,
             "latent_query: bad arguments");
  TL_REQUIRE(a.rot_dims >= 0 && a.rot_dims <= a.rot_dim && (a.rot_dims & 1) == 0 && (a.rot_dims == 0 || a.freq),
             "latent_query: %d turning dimensions of %d", a.rot_dims, a.rot_dim);
  if (a.rot_dim == 0) return 0;
  const int per_token = (a.heads + 3) / 4;
  TL_REQUIRE(per_token <= 65535, "latent_query: too many heads");
  latent_query_kernel<<<dim3(a.T, per_token), 256, 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_latent_spread(const float* cache, int kv_rank, int rot_dim, float* k, int heads, int dim, int P, hipStream_t s) {
  TL_REQUIRE(cache && k && kv_rank > 0 && rot_dim >= 0 && heads > 0 && dim > 0 && P > 0, "latent_spread: bad arguments");
  if (rot_dim == 0) return 0;
  const long long total = (long long)P * heads * rot_dim;
  latent_spread_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(cache, kv_rank, rot_dim, k, heads, dim, total);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_head_gate(float* o, const float* gate, int gate_ld, int T, int heads, int vdim, hipStream_t s) {
  TL_REQUIRE(o && gate && T > 0 && heads > 0 && vdim > 0 && gate_ld >= heads, "head_gate: bad arguments");
  const long long total = (long long)T * heads * vdim;
  head_gate_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(o, gate, gate_ld, heads, vdim, total);
  TL_HIP(hipGetLastError());
  return 0;
}
