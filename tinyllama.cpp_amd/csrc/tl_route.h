// tl_route.h — the selection step of a mixture's router, shared by the stand-alone router launch (tl_moe.hip) and the
// residual-norm launch that carries the router of the feed-forward behind it (tl_norm.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>

// One wave (all 64 lanes) picks the `top` largest of z[experts] (LDS; overwritten), the lower index among equals, and writes
// ids[top] (largest first) and wts[top] = the softmax over the chosen logits.
__device__ __forceinline__ void tl_route_select(float* z, int experts, int top, int* ids, float* wts, int lane) {
    // `top` rounds: the lanes scan the experts not yet chosen for the largest logit (lower index wins among equals)
    float mx = 0.0f, denom = 0.0f, mine = 0.0f;
    int my_id = -1;
    for (int j = 0; j < top; ++j) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int e = lane; e < experts; e += 64) {
        const float v = z[e];
        if (v > bv || (v == bv && e < bi)) {
          bv = v;
          bi = e;
        }
      }
#pragma unroll
      for (int o = 32; o >= 1; o >>= 1) {
        const float ov = __shfl_xor(bv, o);
        const int oi = __shfl_xor(bi, o);
        if (ov > bv || (ov == bv && oi < bi)) {
          bv = ov;
          bi = oi;
        }
      }
      if (bi == 0x7fffffff) bi = 0;  // only when every logit is NaN
      if (j == 0) mx = bv;
      const float p = expf(bv - mx);
      denom += p;
      if (lane == j % 64 && j < 64) {
        mine = p;
        my_id = bi;
      }
      if (j >= 64 && lane == 0) {  // more than 64 choices: written unnormalised, fixed up below
        ids[j] = bi;
        wts[j] = p;
      }
      if (lane == 0) z[bi] = -INFINITY;  // chosen: out of the next rounds
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    if (lane < top && lane < 64) {
      ids[lane] = my_id;
      wts[lane] = mine / denom;
    }
    if (top > 64 && lane == 0)
      for (int j = 64; j < top; ++j) wts[j] /= denom;
}

// One wave: scores = softmax(z) over all experts (left in z[]); the experts form `groups` equal groups of neighbours, a
// group's score is its best expert's, and only experts of the best `keep` groups (lower index among equals) can be chosen;
// ids[top] = the chosen experts, largest score first (lower index among equals); wts = their scores divided by their sum
// (+ 1e-20). key[experts] and gs[groups] are LDS scratch.
__device__ __forceinline__ void tl_route_select_groups(float* z, float* key, float* gs, int experts, int top, int groups, int keep,
                                                       int* ids, float* wts, int lane) {
  auto wave_sync = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  float mx = -INFINITY;
  for (int e = lane; e < experts; e += 64) mx = fmaxf(mx, z[e]);
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
  float sum = 0.0f;
  for (int e = lane; e < experts; e += 64) {
    const float p = expf(z[e] - mx);
    z[e] = p;
    sum += p;
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o);
  const int per = experts / groups;
  for (int e = lane; e < experts; e += 64) {
    z[e] = z[e] / sum;
    key[e] = -1.0f;  // below every score: not choosable until its group is kept
  }
  wave_sync();
  for (int g = lane; g < groups; g += 64) {
    float b = -1.0f;
    for (int e = g * per; e < (g + 1) * per; ++e) b = fmaxf(b, z[e]);
    gs[g] = b;
  }
  wave_sync();
  for (int r = 0; r < keep; ++r) {  // the best group not yet kept
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int g = lane; g < groups; g += 64) {
      const float v = gs[g];
      if (v > bv || (v == bv && g < bi)) {
        bv = v;
        bi = g;
      }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      const float ov = __shfl_xor(bv, o);
      const int oi = __shfl_xor(bi, o);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    }
    if (bi == 0x7fffffff) bi = 0;
    for (int e = bi * per + lane; e < (bi + 1) * per; e += 64) key[e] = z[e];
    if (lane == 0) gs[bi] = -INFINITY;
    wave_sync();
  }
  float denom = 0.0f;
  for (int j = 0; j < top; ++j) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < experts; e += 64) {
      const float v = key[e];
      if (v > bv || (v == bv && e < bi)) {
        bv = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      const float ov = __shfl_xor(bv, o);
      const int oi = __shfl_xor(bi, o);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    }
    if (bi == 0x7fffffff) bi = 0;
    const float sc = z[bi];
    denom += sc;
    if (lane == 0) {
      ids[j] = bi;
      wts[j] = sc;
      key[bi] = -INFINITY;
    }
    wave_sync();
  }
  for (int j = lane; j < top; j += 64) wts[j] = wts[j] / (denom + 1e-20f);
}

// One wave: scores = sigmoid(z) (left in z[]); choice = score + corr[expert] (corr may be NULL); the experts form `groups` equal
// groups of neighbours, a group ranks by the sum of its two best choices (its one choice when a group is one expert), and only
// experts of the best `keep` groups (lower index among equals) can be chosen -- the others count as minus infinity, since a
// choice may be negative; ids[top] = the best choices first (lower index among equals); wts = the chosen experts' SCORES,
// without the correction and not normalised. key[experts] and gs[groups] are LDS scratch.
__device__ __forceinline__ void tl_route_select_sigmoid_groups(float* z, float* key, float* gs, const float* corr, int experts,
                                                               int top, int groups, int keep, int* ids, float* wts, int lane) {
  auto wave_sync = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  const int per = experts / groups;
  for (int e = lane; e < experts; e += 64) {
    const float sc = 1.0f / (1.0f + expf(-z[e]));
    z[e] = sc;
    key[e] = sc + (corr ? corr[e] : 0.0f);
  }
  wave_sync();
  for (int g = lane; g < groups; g += 64) {
    float b1 = -INFINITY, b2 = -INFINITY;
    for (int e = g * per; e < (g + 1) * per; ++e) {
      const float v = key[e];
      if (v > b1) {
        b2 = b1;
        b1 = v;
      } else if (v > b2) {
        b2 = v;
      }
    }
    gs[g] = per > 1 ? b1 + b2 : b1;
  }
  wave_sync();
  // groups are ranked `keep` times; a kept group is marked by +infinity in gs, the rest lose their choices afterwards
  for (int r = 0; r < keep; ++r) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int g = lane; g < groups; g += 64) {
      const float v = gs[g];
      if (v != INFINITY && (v > bv || (v == bv && g < bi) || bi == 0x7fffffff)) {
        bv = v;
        bi = g;
      }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      const float ov = __shfl_xor(bv, o);
      const int oi = __shfl_xor(bi, o);
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) {
        bv = ov;
        bi = oi;
      }
    }
    if (bi == 0x7fffffff) bi = 0;
    if (lane == 0) gs[bi] = INFINITY;
    wave_sync();
  }
  for (int e = lane; e < experts; e += 64)
    if (gs[e / per] != INFINITY) key[e] = -INFINITY;
  wave_sync();
  for (int j = 0; j < top; ++j) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < experts; e += 64) {
      const float v = key[e];
      if (v > bv || (v == bv && e < bi)) {
        bv = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      const float ov = __shfl_xor(bv, o);
      const int oi = __shfl_xor(bi, o);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    }
    if (bi == 0x7fffffff) bi = 0;
    if (lane == 0) {
      ids[j] = bi;
      wts[j] = z[bi];
      key[bi] = -INFINITY;
    }
    wave_sync();
  }
}
