// tl_dense.hip — products with bf16 weight matrices [rows][cols] (row-major, y = W x), FP32 activations and accumulation.
//
//   GEMV (one token): a wave per output row, 16 B of weights per lane per step, widened exactly to FP32: FP32 arithmetic
//   throughout, bound by the bytes of the matrix.
//   GEMM (a chunk of tokens) on the matrix cores: v_mfma_f32_32x32x8_bf16 with the WEIGHTS as the A operand (M = output
//   features) and the tokens as B (N = tokens), so that a lane ends up holding 4 x 4 consecutive features of ONE token and
//   stores them as 16-byte pieces of that token's output row. The FP32 activations are split while they are staged into
//   LDS: terms = 1 keeps their bf16 rounding, terms = 3 keeps hi + mid + lo (3 x 8 mantissa bits = all 24 of an FP32
//   value); the weights are bf16 to begin with, so three MFMAs per product reproduce the FP32 product exactly and only the
//   order of the FP32 accumulation differs from a scalar loop.
//   A workgroup of 4 waves owns a 64 x 64 or (enough rows and tokens) a 128 x 128 feature x token tile, BK = 32, with the
//   next k-block's global loads in flight under the products of the block in LDS. Items may be gathered (x_rows), scattered (y_rows) and
//   grouped (group_off: blockIdx.z = matrix of the group; tiles beyond a group's items leave at once), which is what the
//   experts of a mixture need: the plan lives on the device, the grid is sized for the worst case.
#include <math.h>
#include <stdlib.h>

#include "tl_bf16.h"
#include "tl_stack.h"

namespace {

typedef __attribute__((ext_vector_type(4))) short bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ __forceinline__ unsigned short f2bf(float f) {  // round to nearest even
  unsigned u = __float_as_uint(f);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (unsigned short)(u >> 16);
}
__device__ __forceinline__ float bf2f(unsigned short h) { return tl_bf2f(h); }

// y = g * sigmoid(alpha * g) * (u + 1), g = min(gate, limit), u = clamp(up, -limit, limit)  (tl_moe.hip has the operator)
__device__ __forceinline__ float dense_glu(float g, float u, float limit, float alpha, float up_add) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-alpha * g)) * (u + up_add);
}

constexpr int BK = 32, LDK = 40;  // LDK: padded row of a tile in LDS (80 B, keeps 16 B / 8 B alignment)

// A workgroup of 4 waves (2 x 2) owns a (64 WM)-feature x (64 WN)-token tile; a wave WM x WN products of 32 x 32. The next
// k-block's weights and activations are asked for (into registers) before the products of the block in LDS start.
template <int TERMS, int WM, int WN>
__global__ __launch_bounds__(256) void dense_gemm_kernel(const DenseArgs a) {
  constexpr int BM = 64 * WM, BN = 64 * WN;
  __shared__ __attribute__((aligned(16))) unsigned short Ws[BM][LDK];
  __shared__ __attribute__((aligned(16))) unsigned short Xs[TERMS][BN][LDK];
  __shared__ int xrow[BN];
  const int tid = threadIdx.x, g = blockIdx.z;
  int lo = 0, hi = a.T;
  if (a.group_off) {
    lo = a.group_off[g];
    hi = a.group_off[g + 1];
  }
  const int t0 = lo + blockIdx.y * BN;
  if (t0 >= hi) return;
  const int f0 = blockIdx.x * BM;
  const unsigned short* W = a.w + (size_t)g * a.rows * a.cols;
  const float* X = a.x + (size_t)g * a.x_gstride;  // (one product per head: the group picks its columns)
  float* Y = a.y + (size_t)g * a.y_gstride;
  for (int i = tid; i < BN; i += 256) {
    const int it = t0 + i;
    int r = -1;
    if (it < hi) r = a.x_rows ? a.x_rows[it] / a.x_div : it;
    xrow[i] = r;
  }
  __syncthreads();
  const int wave = tid >> 6, lane = tid & 63, wm = wave & 1, wn = wave >> 1;
  const int lr = tid >> 2, lk = (tid & 3) * 8;  // this thread stages 8 consecutive k of rows lr + 64 i of both tiles
  const int K = a.cols;
  const bool vec = (K & 7) == 0 && (a.ldx & 3) == 0 && ((size_t)X & 15) == 0 && ((size_t)W & 15) == 0;
  const unsigned short* wp[WM];
  const float* xp[WN];
  bool wok[WM], xok[WN];
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int frow = f0 + lr + 64 * i;
    wok[i] = frow < a.rows;
    wp[i] = W + (size_t)(wok[i] ? frow : 0) * K;
  }
#pragma unroll
  for (int j = 0; j < WN; ++j) {
    const int xr = xrow[lr + 64 * j];
    xok[j] = xr >= 0;
    xp[j] = X + (size_t)(xok[j] ? xr : 0) * a.ldx;
  }
  uint4 wreg[WM];
  float xreg[WN][8];
  auto fetch = [&](int k0) __attribute__((always_inline)) {
    const int k = k0 + lk;
    if (vec && k + 8 <= K) {
#pragma unroll
      for (int i = 0; i < WM; ++i) wreg[i] = wok[i] ? *reinterpret_cast<const uint4*>(wp[i] + k) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        float4 x0 = make_float4(0, 0, 0, 0), x1 = x0;
        if (xok[j]) {
          x0 = *reinterpret_cast<const float4*>(xp[j] + k);
          x1 = *reinterpret_cast<const float4*>(xp[j] + k + 4);
        }
        xreg[j][0] = x0.x; xreg[j][1] = x0.y; xreg[j][2] = x0.z; xreg[j][3] = x0.w;
        xreg[j][4] = x1.x; xreg[j][5] = x1.y; xreg[j][6] = x1.z; xreg[j][7] = x1.w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < WM; ++i) {
        unsigned short wv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) wv[e] = (k + e < K && wok[i]) ? wp[i][k + e] : (unsigned short)0;
        wreg[i].x = wv[0] | ((unsigned)wv[1] << 16); wreg[i].y = wv[2] | ((unsigned)wv[3] << 16);
        wreg[i].z = wv[4] | ((unsigned)wv[5] << 16); wreg[i].w = wv[6] | ((unsigned)wv[7] << 16);
      }
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) xreg[j][e] = (k + e < K && xok[j]) ? xp[j][k + e] : 0.0f;
    }
  };
  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int i = 0; i < WM; ++i) *reinterpret_cast<uint4*>(&Ws[lr + 64 * i][lk]) = wreg[i];
#pragma unroll
    for (int j = 0; j < WN; ++j) {
#pragma unroll
      for (int t = 0; t < TERMS; ++t) {
        unsigned short h[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          h[e] = f2bf(xreg[j][e]);
          xreg[j][e] -= bf2f(h[e]);  // exact: the remainder of an FP32 value after its leading 8 bits
        }
        uint4 p;
        p.x = h[0] | ((unsigned)h[1] << 16); p.y = h[2] | ((unsigned)h[3] << 16);
        p.z = h[4] | ((unsigned)h[5] << 16); p.w = h[6] | ((unsigned)h[7] << 16);
        *reinterpret_cast<uint4*>(&Xs[t][lr + 64 * j][lk]) = p;
      }
    }
    __syncthreads();
    if (k0 + BK < K) fetch(k0 + BK);  // in flight while the products below run
#pragma unroll
    for (int ks = 0; ks < BK / 8; ++ks) {
      const int kk = ks * 8 + (lane >> 5) * 4;
      bf16x4 af[WM];
#pragma unroll
      for (int i = 0; i < WM; ++i) af[i] = *reinterpret_cast<const bf16x4*>(&Ws[(wm * WM + i) * 32 + (lane & 31)][kk]);
#pragma unroll
      for (int t = TERMS - 1; t >= 0; --t) {  // small terms first
#pragma unroll
        for (int j = 0; j < WN; ++j) {
          const bf16x4 bfr = *reinterpret_cast<const bf16x4*>(&Xs[t][(wn * WN + j) * 32 + (lane & 31)][kk]);
#pragma unroll
          for (int i = 0; i < WM; ++i) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(af[i], bfr, acc[i][j], 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }
  // C layout: lane holds token (lane & 31) of a 32 x 32 product, features (e / 4) * 8 + (lane >> 5) * 4 + (e & 3)
  const bool v4 = (a.ldy & 3) == 0 && ((size_t)Y & 15) == 0;
#pragma unroll
  for (int j = 0; j < WN; ++j) {
    const int it = t0 + (wn * WN + j) * 32 + (lane & 31);
    if (it >= hi) continue;
    const int orow = a.y_rows ? a.y_rows[it] : it;
    float* yr = Y + (size_t)orow * a.ldy;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        const int f = f0 + (wm * WM + i) * 32 + gq * 8 + (lane >> 5) * 4;
        if (a.glu) {  // (gate, up) pairs: features f, f + 1 -> unit f / 2; f + 2, f + 3 -> the next one
#pragma unroll
          for (int e = 0; e < 2; ++e)
            if (f + 2 * e + 1 < a.rows)
              yr[(f >> 1) + e] = tl_glu_apply(a.glu_kind, acc[i][j][gq * 4 + 2 * e], acc[i][j][gq * 4 + 2 * e + 1], a.glu_limit, a.glu_alpha, a.glu_up_add);
          continue;
        }
        if (a.softcap > 0.0f) {
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[i][j][gq * 4 + e] = a.softcap * tanhf(acc[i][j][gq * 4 + e] / a.softcap);
        }
        if (a.act) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (f + e >= a.act_from) acc[i][j][gq * 4 + e] = tl_act_apply(a.act, acc[i][j][gq * 4 + e], a.act_p, a.act_q);
        }
        if (v4 && f + 4 <= a.rows) {
          *reinterpret_cast<float4*>(yr + f) =
              make_float4(acc[i][j][gq * 4], acc[i][j][gq * 4 + 1], acc[i][j][gq * 4 + 2], acc[i][j][gq * 4 + 3]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (f + e < a.rows) yr[f + e] = acc[i][j][gq * 4 + e];
        }
      }
    }
  }
}

// RW rows per wave, 4 waves per workgroup: 2 x RW sixteen-byte weight loads in flight per lane (tl_bf16.h)
template <int RW>
__global__ __launch_bounds__(256) void dense_gemv_kernel(const unsigned short* __restrict__ W, int rows, int cols,
                                                         const float* __restrict__ x, float* __restrict__ y, int vec,
                                                         float softcap, const GemvActArgs act, int x_stride, int y_stride) {
  const int lane = threadIdx.x & 63;
  const int row0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * RW;
  if (row0 >= rows) return;
  // blockIdx.y: the head of a one-product-per-head launch (its matrix, its columns of x, its piece of y)
  W += (size_t)blockIdx.y * rows * cols;
  x += (size_t)blockIdx.y * x_stride;
  y += (size_t)blockIdx.y * y_stride;
  float out[RW];
  tl_wave_dot_rows<RW>(W + (size_t)row0 * cols, (size_t)cols, rows - row0, x, cols, vec != 0, lane, out);
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < RW; ++r)
      if (row0 + r < rows) {
        float v = softcap > 0.0f ? softcap * tanhf(out[r] / softcap) : out[r];
        if (act.act && row0 + r >= act.act_from) v = tl_act_apply(act.act, v, act.act_p, act.act_q);
        y[row0 + r] = v;
      }
  }
}

}  // namespace

int tl_launch_dense_gemm(const DenseArgs& a, hipStream_t s) {
  TL_REQUIRE(a.w && a.x && a.y && a.rows > 0 && a.cols > 0 && a.T > 0, "dense gemm: bad arguments");
  TL_REQUIRE(a.terms == 1 || a.terms == 3, "dense gemm: terms must be 1 or 3 (got %d)", a.terms);
  TL_REQUIRE(!a.x_rows || a.x_div >= 1, "dense gemm: x_div must be >= 1");
  TL_REQUIRE(!a.glu || (a.rows & 1) == 0, "dense gemm: gated pairs need an even number of rows (got %d)", a.rows);
  const int groups = a.groups > 0 ? a.groups : 1;
  TL_REQUIRE(groups == 1 || a.group_off || (a.x_gstride >= 0 && a.y_gstride > 0 && !a.x_rows && !a.y_rows),
             "dense gemm: groups without group_off or per-head column strides");
  TL_REQUIRE(!a.act || !a.glu, "dense gemm: an activation and a gated unit in one epilogue");
  // 128 x 128 tiles when there is enough of both sides to fill them (grouped launches: tokens per group on average)
  const long long per_group = a.group_off ? (long long)a.T / groups : a.T;
  // Measured at width 4096, chunks of 512 tokens: a dense launch has too few 128 x 128 tiles to fill 256 CUs (6144 x 512:
  // 192 tiles, 117 us against 109 us in 768 small ones); the experts' grouped launches, whose small tiles are mostly
  // half-empty, gain from them with one term (221 -> 193 us) and lose with three (356 -> 413 us).
  const long long big_tiles = ((a.rows + 127) / 128) * ((per_group + 127) / 128) * groups;
  const char* force = getenv("TL_DENSE_TILE");  // 64 / 128: tests and A/B runs pick the tile themselves
  const bool big = force ? atoi(force) == 128
                         : a.rows >= 256 && (a.group_off ? a.terms == 1 && per_group >= 96 : big_tiles >= 2 * tl_num_cus());
  const int BM = big ? 128 : 64, BN = big ? 128 : 64;
  dim3 grid((a.rows + BM - 1) / BM, (a.T + BN - 1) / BN, groups);
  TL_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "dense gemm: launch too large");
  if (big) {
    if (a.terms == 1) dense_gemm_kernel<1, 2, 2><<<grid, 256, 0, s>>>(a);
    else dense_gemm_kernel<3, 2, 2><<<grid, 256, 0, s>>>(a);
  } else {
    if (a.terms == 1) dense_gemm_kernel<1, 1, 1><<<grid, 256, 0, s>>>(a);
    else dense_gemm_kernel<3, 1, 1><<<grid, 256, 0, s>>>(a);
  }
  TL_HIP(hipGetLastError());
  return 0;
}

static int launch_gemv(const uint16_t* w, int groups, int rows, int cols, const float* x, int x_stride, float* y, int y_stride,
                       float softcap, const GemvActArgs& act, hipStream_t s) {
  TL_REQUIRE(w && x && y && rows > 0 && cols > 0 && groups > 0 && groups <= 65535, "dense gemv: bad arguments");
  // 16-byte loads need every head's matrix and columns aligned as the first one's
  const int vec = (cols & 7) == 0 && ((size_t)x & 15) == 0 && ((size_t)w & 15) == 0 &&
                  (groups == 1 || ((x_stride & 3) == 0 && (((size_t)rows * cols) & 7) == 0));
  // rows per wave: as many as still leave every CU a few workgroups
  const int cus = tl_num_cus();
  const long long all = (long long)rows * groups;
  if (all >= 16 * 4 * cus) dense_gemv_kernel<4><<<dim3((rows + 15) / 16, groups), 256, 0, s>>>(w, rows, cols, x, y, vec, softcap, act, x_stride, y_stride);
  else if (all >= 8 * 4 * cus) dense_gemv_kernel<2><<<dim3((rows + 7) / 8, groups), 256, 0, s>>>(w, rows, cols, x, y, vec, softcap, act, x_stride, y_stride);
  else dense_gemv_kernel<1><<<dim3((rows + 3) / 4, groups), 256, 0, s>>>(w, rows, cols, x, y, vec, softcap, act, x_stride, y_stride);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_dense_gemv(const uint16_t* w, int rows, int cols, const float* x, float* y, hipStream_t s, float softcap) {
  return launch_gemv(w, 1, rows, cols, x, 0, y, 0, softcap, GemvActArgs{}, s);
}

int tl_launch_dense_gemv_act(const uint16_t* w, int rows, int cols, const float* x, float* y, const GemvActArgs& act, hipStream_t s) {
  return launch_gemv(w, 1, rows, cols, x, 0, y, 0, 0.0f, act, s);
}

int tl_launch_dense_gemv_heads(const uint16_t* w, int groups, int rows, int cols, const float* x, int x_stride, float* y,
                               int y_stride, hipStream_t s) {
  return launch_gemv(w, groups, rows, cols, x, x_stride, y, y_stride, 0.0f, GemvActArgs{}, s);
}

extern "C" int tl_dense_matmul(const void* w_bf16_dev, int rows, int cols, const float* x_dev, float* y_dev, int num_tokens,
                               int terms, void* stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (terms == 0) {
    TL_REQUIRE(num_tokens == 1, "tl_dense_matmul: terms 0 (FP32 GEMV) takes one token, not %d", num_tokens);
    return tl_launch_dense_gemv(static_cast<const uint16_t*>(w_bf16_dev), rows, cols, x_dev, y_dev, s);
  }
  DenseArgs a = {};
  a.w = static_cast<const uint16_t*>(w_bf16_dev);
  a.rows = rows;
  a.cols = cols;
  a.x = x_dev;
  a.ldx = cols;
  a.y = y_dev;
  a.ldy = rows;
  a.T = num_tokens;
  a.terms = terms;
  return tl_launch_dense_gemm(a, s);
}

extern "C" int tl_dense_matmul_act(const void* w_bf16_dev, int rows, int cols, const float* x_dev, float* y_dev, int num_tokens,
                                   int terms, int act, float act_p, float act_q, int act_from, void* stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  TL_REQUIRE(act >= TL_ACT_NONE && act <= TL_ACT_TANH, "tl_dense_matmul_act: activation kind %d", act);
  if (terms == 0) {
    TL_REQUIRE(num_tokens == 1, "tl_dense_matmul_act: terms 0 (FP32 GEMV) takes one token, not %d", num_tokens);
    return tl_launch_dense_gemv_act(static_cast<const uint16_t*>(w_bf16_dev), rows, cols, x_dev, y_dev,
                                    GemvActArgs{act, act_from, act_p, act_q}, s);
  }
  DenseArgs a = {};
  a.w = static_cast<const uint16_t*>(w_bf16_dev);
  a.rows = rows;
  a.cols = cols;
  a.x = x_dev;
  a.ldx = cols;
  a.y = y_dev;
  a.ldy = rows;
  a.T = num_tokens;
  a.terms = terms;
  a.act = act;
  a.act_from = act_from;
  a.act_p = act_p;
  a.act_q = act_q;
  return tl_launch_dense_gemm(a, s);
}

extern "C" int tl_dense_matmul_heads(const void* w_bf16_dev, int groups, int rows, int cols, const float* x_dev, int ldx,
                                     int x_stride, float* y_dev, int ldy, int y_stride, int num_tokens, int terms, void* stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (terms == 0) {
    TL_REQUIRE(num_tokens == 1, "tl_dense_matmul_heads: terms 0 (FP32 GEMV) takes one token, not %d", num_tokens);
    return tl_launch_dense_gemv_heads(static_cast<const uint16_t*>(w_bf16_dev), groups, rows, cols, x_dev, x_stride, y_dev,
                                      y_stride, s);
  }
  DenseArgs a = {};
  a.w = static_cast<const uint16_t*>(w_bf16_dev);
  a.rows = rows;
  a.cols = cols;
  a.x = x_dev;
  a.ldx = ldx;
  a.y = y_dev;
  a.ldy = ldy;
  a.T = num_tokens;
  a.terms = terms;
  a.groups = groups;
  a.x_gstride = x_stride;
  a.y_gstride = y_stride;
  return tl_launch_dense_gemm(a, s);
}
