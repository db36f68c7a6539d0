// tl_conv.hip — a short causal convolution over time on every channel of a row, as layer-list models use it in two places:
// on what a sublayer reads (out = in + conv(in): add_input) and on projected queries, keys and values right behind their
// product (with the projection's bias added first, optionally followed by silu). Token t of a call needs the inputs of the
// taps - 1 tokens before it; those that precede the call are part of the sequence's state (hist, zeros for an empty sequence),
// so a prompt may be cut anywhere. Everything is FP32; the weights are the checkpoint's bf16 values widened exactly.
//
//   conv_kernel     grid (column blocks of 256, T): one thread per (token, channel). With one token (the decode step) the
//                   thread is the only reader of its channel's history and shifts it in the same launch.
//   conv4_kernel    the same for several tokens of densely packed rows when sizes allow 16-byte accesses: a thread owns four
//                   neighbouring channels of a token (width 4096, 2048 tokens, 67 MB: 21 us against 63 us with one channel per
//                   thread; on the q | k | v columns of a much wider product's rows it measured slower, 105 us against 63 us,
//                   so rows that are further apart than they are wide keep the one-channel kernel).
//   history_kernel  after a call of several tokens: the history becomes the last taps - 1 inputs (a call shorter than that
//                   keeps the tail of the old history in front). A thread owns a channel and walks its rows in ascending order.
#include <math.h>

#include "tl_bf16.h"
#include "tl_stack.h"

namespace {

__global__ __launch_bounds__(256) void conv_kernel(const ConvArgs a) {
  const int t = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= a.C) return;
  const int H = a.taps - 1;
  const float b = a.bias ? a.bias[c] : 0.0f;
  const unsigned short* w = a.w + (size_t)c * a.taps;
  float acc = 0.0f, cur = 0.0f;
  for (int j = 0; j < a.taps; ++j) {
    const int tt = t - H + j;  // token of this tap, relative to the call
    const float u = tt >= 0 ? a.in[(size_t)tt * a.ldi + c] + b : a.hist[(size_t)(H + tt) * a.C + c];
    acc += tl_bf2f(w[j]) * u;
    cur = u;
  }
  if (a.act == 1) acc = acc / (1.0f + expf(-acc));
  if (a.add_input) acc += cur;
  a.out[(size_t)t * a.ldo + c] = acc;
  if (a.T == 1 && H > 0) {
    for (int j = 0; j + 1 < H; ++j) a.hist[(size_t)j * a.C + c] = a.hist[(size_t)(j + 1) * a.C + c];
    a.hist[(size_t)(H - 1) * a.C + c] = cur;
  }
}

__global__ __launch_bounds__(256) void conv4_kernel(const ConvArgs a) {
  const int t = blockIdx.y, c = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (c >= a.C) return;
  const int H = a.taps - 1;
  const float4 b = a.bias ? *reinterpret_cast<const float4*>(a.bias + c) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  const unsigned short* w = a.w + (size_t)c * a.taps;  // four rows of taps weights, one behind the other
  float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f), cur = acc;
  for (int j = 0; j < a.taps; ++j) {
    const int tt = t - H + j;
    float4 u;
    if (tt >= 0) {
      u = *reinterpret_cast<const float4*>(a.in + (size_t)tt * a.ldi + c);
      u.x += b.x, u.y += b.y, u.z += b.z, u.w += b.w;
    } else {
      u = *reinterpret_cast<const float4*>(a.hist + (size_t)(H + tt) * a.C + c);
    }
    acc.x += tl_bf2f(w[j]) * u.x;
    acc.y += tl_bf2f(w[a.taps + j]) * u.y;
    acc.z += tl_bf2f(w[2 * a.taps + j]) * u.z;
    acc.w += tl_bf2f(w[3 * a.taps + j]) * u.w;
    cur = u;
  }
  if (a.act == 1) {
    acc.x = acc.x / (1.0f + expf(-acc.x)), acc.y = acc.y / (1.0f + expf(-acc.y));
    acc.z = acc.z / (1.0f + expf(-acc.z)), acc.w = acc.w / (1.0f + expf(-acc.w));
  }
  if (a.add_input) acc.x += cur.x, acc.y += cur.y, acc.z += cur.z, acc.w += cur.w;
  *reinterpret_cast<float4*>(a.out + (size_t)t * a.ldo + c) = acc;
}

__global__ __launch_bounds__(256) void conv_history_rows_kernel(const ConvArgs a) {
  const int c = blockIdx.x * 256 + threadIdx.x, H = a.taps - 1;
  if (c >= a.C) return;
  const float b = a.bias ? a.bias[c] : 0.0f;
  for (int i = 0; i < H; ++i) {
    const int src = a.T - H + i;  // token whose input lands in row i
    a.hist[(size_t)i * a.C + c] = src >= 0 ? a.in[(size_t)src * a.ldi + c] + b : a.hist[(size_t)(i + a.T) * a.C + c];
  }
}

}  // namespace

int tl_launch_causal_conv(const ConvArgs& a, hipStream_t s) {
  TL_REQUIRE(a.in && a.w && a.out && a.T > 0 && a.T <= 65535 && a.C > 0, "causal_conv: bad arguments");
  TL_REQUIRE(a.taps >= 1 && (a.taps == 1 || a.hist), "causal_conv: %d taps", a.taps);
  TL_REQUIRE(a.ldi >= a.C && a.ldo >= a.C, "causal_conv: row strides %d / %d below %d channels", a.ldi, a.ldo, a.C);
  TL_REQUIRE(a.T == 1 || a.out + (size_t)a.T * a.ldo <= a.in || a.in + (size_t)a.T * a.ldi <= a.out,
             "causal_conv: output over input with more than one token");
  TL_REQUIRE(a.act == 0 || a.act == 1, "causal_conv: activation %d", a.act);
  const bool vec = a.T > 1 && (a.C & 3) == 0 && a.ldi == a.C && (a.ldo & 3) == 0 && ((size_t)a.in & 15) == 0 &&
                   ((size_t)a.out & 15) == 0 && ((size_t)a.hist & 15) == 0 && ((size_t)a.bias & 15) == 0;
  if (vec) conv4_kernel<<<dim3((a.C / 4 + 255) / 256, a.T), 256, 0, s>>>(a);
  else conv_kernel<<<dim3((a.C + 255) / 256, a.T), 256, 0, s>>>(a);
  if (a.T > 1 && a.taps > 1) conv_history_rows_kernel<<<(a.C + 255) / 256, 256, 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

extern "C" int tl_causal_conv(const float* in_dev, int ld_in, int channels, int taps, int num_tokens, const float* bias_dev,
                              const void* w_bf16_dev, float* history_dev, int act, int add_input, float* out_dev, int ld_out,
                              void* stream) {
  ConvArgs a = {};
  a.in = in_dev;
  a.ldi = ld_in;
  a.C = channels;
  a.taps = taps;
  a.T = num_tokens;
  a.bias = bias_dev;
  a.w = static_cast<const uint16_t*>(w_bf16_dev);
  a.hist = history_dev;
  a.act = act;
  a.add_input = add_input;
  a.out = out_dev;
  a.ldo = ld_out;
  return tl_launch_causal_conv(a, static_cast<hipStream_t>(stream));
}
