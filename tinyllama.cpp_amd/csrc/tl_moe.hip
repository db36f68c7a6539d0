// tl_moe.hip — mixture-of-experts feed-forward: router, grouping plan, the experts' clamped gated activation, and the
// one-token (decode) form of the experts.
//
//   router   logits z = W_r x + b in FP32 (bf16 weights widened exactly); the `top` largest are chosen (equal logits: the
//            lower index first) and weighted by the softmax over the chosen logits only.
//   plan     the T * top (token, choice) slots grouped by expert: off[e] .. off[e + 1] index slot_of[]. The order inside a
//            group is whatever the atomics give; no result depends on it (every slot's output is computed on its own and
//            summed per token in choice order).
//   act      y = g * sigmoid(alpha * g) * (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit).
//   decode   one token: gate/up GEMVs of the chosen experts (+ the shared expert) with the activation applied in the same
//            launch, then one launch in which a wave owns an output row and sums the chosen experts' down rows with the
//            router weights (and the shared expert's with weight 1).
#include <math.h>

#include "tl_bf16.h"
#include "tl_route.h"
#include "tl_stack.h"

namespace {

constexpr int kMaxExperts = 1024;

// dot of a bf16 row with an FP32 vector over the lanes of a wave; result in every lane
__device__ __forceinline__ float wave_dot(const unsigned short* __restrict__ wr, const float* __restrict__ x, int n, bool vec,
                                          int lane) {
  float s;
  tl_wave_dot_rows<1>(wr, 0, 1, x, n, vec, lane, &s);
  return s;
}

// 4 or 16 waves per token: a wave takes every (number of waves)-th expert
__global__ __launch_bounds__(1024) void router_kernel(const RouterArgs a, int vec) {
  extern __shared__ float z[];  // [experts] (+ [experts] keys + [groups] for the group-limited kind)
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float* x = a.x + (size_t)t * a.width;
  const int nwaves = blockDim.x >> 6;
  for (int e = wave; e < a.experts + (a.gate_w ? 1 : 0); e += nwaves) {
    if (e == a.experts) {  // the extra row: a gate per token
      const float s = wave_dot(a.gate_w, x, a.width, vec != 0 && ((size_t)a.gate_w & 15) == 0, lane);
      if (lane == 0) a.gate_out[t] = 1.0f / (1.0f + expf(-s));
      continue;
    }
    const float s = wave_dot(a.w + (size_t)e * a.width, x, a.width, vec != 0, lane);
    if (lane == 0) z[e] = s + (a.b ? a.b[e] : 0.0f);
  }
  __syncthreads();
  if (wave != 0) return;
  if (a.kind == TL_ROUTE_SIGMOID_GROUPS)
    tl_route_select_sigmoid_groups(z, z + a.experts, z + 2 * a.experts, a.corr, a.experts, a.top, a.groups, a.keep,
                                   a.ids + (size_t)t * a.top, a.wts + (size_t)t * a.top, lane);
  else if (a.kind == TL_ROUTE_SOFTMAX_GROUPS)
    tl_route_select_groups(z, z + a.experts, z + 2 * a.experts, a.experts, a.top, a.groups, a.keep, a.ids + (size_t)t * a.top,
                           a.wts + (size_t)t * a.top, lane);
  else
    tl_route_select(z, a.experts, a.top, a.ids + (size_t)t * a.top, a.wts + (size_t)t * a.top, lane);
}

__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ ids, int n_slots, int experts,
                                                        int* __restrict__ off, int* __restrict__ slot_of) {
  __shared__ int cnt[kMaxExperts + 1];
  for (int e = threadIdx.x; e <= experts; e += 1024) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n_slots; i += 1024) atomicAdd(&cnt[ids[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < experts; ++e) {
      const int c = cnt[e];
      off[e] = run;
      cnt[e] = run;  // becomes the group's cursor
      run += c;
    }
    off[experts] = run;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n_slots; i += 1024) slot_of[atomicAdd(&cnt[ids[i]], 1)] = i;
}

__device__ __forceinline__ float glu_act(float g, float u, float limit, float alpha, float up_add = 1.0f) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-alpha * g)) * (u + up_add);
}

__global__ __launch_bounds__(256) void glu_act_kernel(const float* __restrict__ in, size_t n, int ff, float limit, float alpha,
                                                      float* __restrict__ out) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const size_t p = i / ff;
  const int c = (int)(i - p * ff);
  out[i] = glu_act(in[p * 2 * ff + c], in[p * 2 * ff + ff + c], limit, alpha);
}

// grid: (rows of 4 waves over max(ff, sff), top + 1). Slot j < top: expert ids[j]; slot top: the shared expert.
__global__ __launch_bounds__(256) void moe_decode_gu_kernel(const MoeDecodeArgs a, int vec) {
  const int lane = threadIdx.x & 63, r = blockIdx.x * 4 + (threadIdx.x >> 6), j = blockIdx.y;
  const bool shared = j == a.top;
  const int ff = shared ? a.sff : a.ff;
  if (r >= ff) return;
  const unsigned short* gu = shared ? a.sgu : a.gu + (size_t)a.ids[j] * 2 * a.ff * a.width;
  float gu2[2];  // unit r's gate and up rows lie side by side; their loads are in flight together
  tl_wave_dot_rows<2>(gu + (size_t)2 * r * a.width, (size_t)a.width, 2, a.x, a.width, vec != 0, lane, gu2);
  if (lane == 0) a.act[(size_t)j * a.ff + r] = tl_glu_apply(a.glu_kind, gu2[0], gu2[1], shared ? a.slimit : a.limit, a.alpha, a.up_add);
}

__global__ __launch_bounds__(256) void moe_decode_down_kernel(const MoeDecodeArgs a, int vec_e, int vec_s) {
  const int lane = threadIdx.x & 63, r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= a.width) return;
  float y = 0.0f;
  for (int j = 0; j < a.top; ++j) {
    const unsigned short* d = a.down + ((size_t)a.ids[j] * a.width + r) * a.ff;
    y += a.wts[j] * wave_dot(d, a.act + (size_t)j * a.ff, a.ff, vec_e != 0, lane);
  }
  if (a.sdown) {
    const float sh = wave_dot(a.sdown + (size_t)r * a.sff, a.act + (size_t)a.top * a.ff, a.sff, vec_s != 0, lane);
    y += a.sgate ? *a.sgate * sh : sh;
  }
  if (lane == 0) a.y[r] = y;
}

}  // namespace

int tl_launch_router(const RouterArgs& a, hipStream_t s) {
  TL_REQUIRE(a.x && a.w && a.ids && a.wts && a.T > 0 && a.width > 0, "router: bad arguments");
  TL_REQUIRE(a.experts > 0 && a.experts <= kMaxExperts, "router: %d experts outside (0, %d]", a.experts, kMaxExperts);
  TL_REQUIRE(a.top > 0 && a.top <= a.experts, "router: top %d of %d experts", a.top, a.experts);
  TL_REQUIRE(!a.gate_w || a.gate_out, "router: a gate row without an output");
  size_t lds = sizeof(float) * a.experts;
  if (a.kind == TL_ROUTE_SOFTMAX_GROUPS || a.kind == TL_ROUTE_SIGMOID_GROUPS) {
    TL_REQUIRE(a.groups > 0 && a.experts % a.groups == 0 && a.keep > 0 && a.keep <= a.groups,
               "router: %d experts in %d groups, %d kept", a.experts, a.groups, a.keep);
    TL_REQUIRE((long long)a.keep * (a.experts / a.groups) >= a.top, "router: top %d of %d kept groups of %d", a.top, a.keep,
               a.experts / a.groups);
    lds = sizeof(float) * (2 * (size_t)a.experts + a.groups);
  } else {
    TL_REQUIRE(a.kind == TL_ROUTE_TOP_LOGITS, "router: kind %d", a.kind);
  }
  const int vec = (a.width & 7) == 0 && ((size_t)a.x & 15) == 0 && ((size_t)a.w & 15) == 0;
  // few tokens (the decode step): the experts' rows are latency-bound round trips, so spread them over 16 waves
  router_kernel<<<a.T, a.T <= 8 && a.experts > 4 ? 1024 : 256, lds, s>>>(a, vec);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_moe_plan(const int* ids, int n_slots, int experts, int* off, int* slot_of, hipStream_t s) {
  TL_REQUIRE(ids && off && slot_of && n_slots > 0, "moe_plan: bad arguments");
  TL_REQUIRE(experts > 0 && experts <= kMaxExperts, "moe_plan: %d experts outside (0, %d]", experts, kMaxExperts);
  moe_plan_kernel<<<1, 1024, 0, s>>>(ids, n_slots, experts, off, slot_of);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_glu_act(const float* in, int P, int ff, float limit, float alpha, float* out, hipStream_t s) {
  TL_REQUIRE(in && out && P > 0 && ff > 0, "glu_act: bad arguments");
  const size_t n = (size_t)P * ff;
  glu_act_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(in, n, ff, limit, alpha, out);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_moe_decode(const MoeDecodeArgs& a, hipStream_t s) {
  // top == 0: the shared unit alone (a dense feed-forward)
  TL_REQUIRE(a.x && a.act && a.y && a.width > 0 && a.top >= 0 && (a.top == 0 || (a.ids && a.wts && a.gu && a.down && a.ff > 0)),
             "moe_decode: bad arguments");
  TL_REQUIRE(a.top > 0 || a.sgu, "moe_decode: neither experts nor a shared unit");
  TL_REQUIRE(!a.sgu == !a.sdown && (!a.sgu || a.sff > 0), "moe_decode: shared expert half given");
  const bool al = ((size_t)a.x & 15) == 0 && ((size_t)a.act & 15) == 0 && ((size_t)a.gu & 15) == 0 && ((size_t)a.down & 15) == 0 &&
                  ((size_t)a.sgu & 15) == 0 && ((size_t)a.sdown & 15) == 0;
  const int vec_x = al && (a.width & 7) == 0;
  // the activations of slot j start at act + j * ff: 16-byte pieces need ff % 8 == 0 (which also aligns the rows of `down`)
  const int vec_e = al && (a.ff & 7) == 0;
  const int vec_s = vec_e && (a.sff & 7) == 0;
  const int ffmax = a.sgu && a.sff > a.ff ? a.sff : a.ff;
  moe_decode_gu_kernel<<<dim3((ffmax + 3) / 4, a.top + (a.sgu ? 1 : 0)), 256, 0, s>>>(a, vec_x);
  moe_decode_down_kernel<<<(a.width + 3) / 4, 256, 0, s>>>(a, vec_e, vec_s);
  TL_HIP(hipGetLastError());
  return 0;
}

extern "C" int tl_moe_route(const float* x_dev, int num_tokens, int width, const void* w_bf16_dev, const float* bias_dev,
                            int experts, int top, int* ids_dev, float* weights_dev, void* stream) {
  RouterArgs a = {};
  a.x = x_dev;
  a.T = num_tokens;
  a.width = width;
  a.experts = experts;
  a.top = top;
  a.w = static_cast<const uint16_t*>(w_bf16_dev);
  a.b = bias_dev;
  a.ids = ids_dev;
  a.wts = weights_dev;
  return tl_launch_router(a, static_cast<hipStream_t>(stream));
}

extern "C" int tl_glu_clamp(const float* gate_up_dev, int rows, int ff, float limit, float alpha, float* out_dev, void* stream) {
  return tl_launch_glu_act(gate_up_dev, rows, ff, limit, alpha, out_dev, static_cast<hipStream_t>(stream));
}

extern "C" int tl_moe_route_groups(const float* x_dev, int num_tokens, int width, const void* w_bf16_dev, int experts, int top,
                                   int groups, int keep, int* ids_dev, float* weights_dev, void* stream) {
  RouterArgs a = {};
  a.x = x_dev;
  a.T = num_tokens;
  a.width = width;
  a.experts = experts;
  a.top = top;
  a.w = static_cast<const uint16_t*>(w_bf16_dev);
  a.ids = ids_dev;
  a.wts = weights_dev;
  a.kind = TL_ROUTE_SOFTMAX_GROUPS;
  a.groups = groups;
  a.keep = keep;
  return tl_launch_router(a, static_cast<hipStream_t>(stream));
}

extern "C" int tl_moe_route_sigmoid_groups(const float* x_dev, int num_tokens, int width, const void* w_bf16_dev,
                                           const float* correction_dev, int experts, int top, int groups, int keep, int* ids_dev,
                                           float* weights_dev, void* stream) {
  RouterArgs a = {};
  a.x = x_dev;
  a.T = num_tokens;
  a.width = width;
  a.experts = experts;
  a.top = top;
  a.w = static_cast<const uint16_t*>(w_bf16_dev);
  a.corr = correction_dev;
  a.ids = ids_dev;
  a.wts = weights_dev;
  a.kind = TL_ROUTE_SIGMOID_GROUPS;
  a.groups = groups;
  a.keep = keep;
  return tl_launch_router(a, static_cast<hipStream_t>(stream));
}
