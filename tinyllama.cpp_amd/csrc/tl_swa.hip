// tl_swa.hip — sliding-window attention over a flat FP32 cache (rotation, if any, was applied before the keys were cached):
// scores are (q . k) * scale, position i sees the keys j with 0 <= i - j < window and, when keep_first > 0, the keys
// j < keep_first as well (the first tokens of the sequence stay visible at their true positions); the weights are an ordinary
// softmax or, in sigmoid mode, sigmoid(score + bias[head]) without normalisation over the keys. Everything in FP32. Key size
// (dim) and value size (vdim) are independent; query head h reads key/value head h / (heads / kv_heads).
// With a sink the softmax's denominator has one more term exp(0): where partial (max, sum) pairs are merged, the maximum is
// taken together with 0 and exp(-max) joins the sum once. The rows of the caches may be further apart than a row is wide
// (kld, vld): a cache of latent rows is read as keys over its whole row and as values over its first vdim columns.
// Sigmoid mode runs through the softmax machinery with the running maximum pinned to 0: every correction factor is exp(0) = 1,
// the partial sums of waves and splits are simply added, and the final division falls away.
//
// One workgroup of 4 waves per (token, head), for the tokens of a prompt chunk and for the single token of a decode step
// alike. The visible keys are cut into pieces of 64; piece c belongs to wave c % 4. Within a piece a lane owns one key
// (score = its dot product with the query held in LDS), the wave keeps a running maximum and sum, and the weighted values
// are accumulated with the lanes spread over the value columns (coalesced rows of V; a key's weight is read from its lane). The four waves' partial
// (max, sum, output) are merged through LDS at the end.
#include <math.h>
#include <stdlib.h>

#include "tl_stack.h"

namespace {

constexpr int SWA_WAVES = 4;
constexpr int SWA_MAX_VR = 8;  // value columns per lane: vdim <= 512

// cap * tanh(sc / cap) and r1 * ln(1 + r2 * d) for every score of a capped / distance-biased layer. Both are formed from the
// hardware's exp2 / log2 / reciprocal instead of the library's tanhf / log1pf: the absolute error of a score stays near 1e-6
// for caps of a few tens (a short series takes over below 0.1, where 1 - e^-2x would cancel), the same order as the rounding
// of the dot product itself, and the matrix-core kernel, which pays for them on the vector unit, runs 1.3 x as fast.
__device__ __forceinline__ float swa_cap(float sc, float cap, float inv_cap) {
  const float x = sc * inv_cap, ax = fabsf(x), x2 = x * x;
  const float e = __expf(-2.0f * ax);
  const float big = copysignf(__fdividef(1.0f - e, 1.0f + e), x);
  const float small = x * (1.0f + x2 * (-0.33333333f + x2 * (0.13333333f - 0.053968254f * x2)));
  return cap * (ax < 0.1f ? small : big);
}
__device__ __forceinline__ float swa_dist(float r1, float r2, int d) { return r1 * __logf(1.0f + r2 * (float)d); }

__device__ __forceinline__ void swa_st_agent(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float swa_ld_agent(const float* p) {  // past this CU's L1: the records come from other workgroups
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// out = sum_z o_z e^(m_z - M) / sum_z l_z e^(m_z - M) over the nsplit records of a (token, head), in split order; one wave
__device__ __forceinline__ void swa_merge_records(const SwaArgs& a, int t, int h, int lane) {
  const int rs = a.vdim + 2;
  const float* rec = a.ws + ((size_t)t * a.heads + h) * a.nsplit * rs;
  // lane z holds record z's max and sum (nsplit <= 64): one round trip, then everything is in registers
  const float mz = lane < a.nsplit ? swa_ld_agent(rec + (size_t)lane * rs) : -INFINITY;
  const float lz = lane < a.nsplit ? swa_ld_agent(rec + (size_t)lane * rs + 1) : 0.0f;
  float M = mz;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) M = fmaxf(M, __shfl_xor(M, o));
  const float sv = a.sink && a.sink_val ? a.sink_val[h] : 0.0f;
  if (a.sink) M = fmaxf(M, sv);
  const float fz = mz == -INFINITY ? 0.0f : expf(mz - M);
  float L = a.sink ? expf(sv - M) : 0.0f;
  for (int z = 0; z < a.nsplit; ++z) L += __shfl(lz * fz, z);  // in split order
  float* op = a.out + (size_t)t * a.heads * a.vdim + (size_t)h * a.vdim;
  for (int d0 = 0; d0 < a.vdim; d0 += 64) {  // every lane stays in the loop: a shuffle reads nothing from a lane that has left
    const int d = d0 + lane;
    float acc = 0.0f;
    for (int z0 = 0; z0 < a.nsplit; z0 += 8) {  // eight records' values in flight together (clamped index, weight 0 beyond)
      float v[8], f[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int z = z0 + u < a.nsplit ? z0 + u : a.nsplit - 1;
        v[u] = d < a.vdim ? swa_ld_agent(rec + (size_t)z * rs + 2 + d) : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float fu = __shfl(fz, z0 + u < a.nsplit ? z0 + u : 0);
        f[u] = z0 + u < a.nsplit ? fu : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) acc += v[u] * f[u];  // in split order
    }
    if (d < a.vdim) op[d] = a.sigmoid ? acc : acc / L;
  }
}

__global__ __launch_bounds__(256) void swa_kernel(const SwaArgs a) {
  extern __shared__ float lds[];
  float* qs = lds;                                  // [dim]
  float* ow = qs + ((a.dim + 3) & ~3);              // [waves][vdim]
  float* ml = ow + SWA_WAVES * a.vdim;              // [waves][2]
  const int t = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int i = (a.pos_dev ? *a.pos_dev : a.start_pos) + t;
  const int g = h / (a.heads / a.kv_heads);
  const int jlo = (a.window > 0 && i - a.window + 1 > 0) ? i - a.window + 1 : 0;
  const int n = i - jlo + 1;
  // kept first keys that lie before the window: pieces [0, pf) walk them, pieces [pf, pieces) the window
  const int nf = a.keep_first > 0 ? (a.keep_first < jlo ? a.keep_first : jlo) : 0;
  const int pf = (nf + 63) >> 6;
  const float hb = a.sigmoid && a.head_bias ? a.head_bias[h] : 0.0f;
  const int kld = a.kld > 0 ? a.kld : a.kv_heads * (a.k_hstride > 0 ? a.k_hstride : a.dim), vld = a.vld > 0 ? a.vld : a.kv_heads * a.vdim;
  const int qhs = a.q_hstride > 0 ? a.q_hstride : a.dim, khs = a.k_hstride > 0 ? a.k_hstride : a.dim;
  const float* qp = a.q + (size_t)t * a.ldq + (size_t)h * qhs;
  const float r1 = a.dist_r1 ? a.dist_r1[h] : 0.0f, r2 = a.dist_r1 ? a.dist_r2[h] : 0.0f;
  for (int d = tid; d < a.dim; d += 256) qs[d] = qp[d];
  __syncthreads();
  const bool v4 = (a.dim & 3) == 0 && (kld & 3) == 0 && (khs & 3) == 0 && ((size_t)a.kc & 15) == 0;
  float m = -INFINITY, l = 0.0f;
  float o[SWA_MAX_VR];
#pragma unroll
  for (int r = 0; r < SWA_MAX_VR; ++r) o[r] = 0.0f;
  const int pieces = pf + ((n + 63) >> 6);
  // nsplit > 1 (few tokens, long windows): workgroup z of (token, head) takes pieces [z * per, (z + 1) * per) and leaves its
  // (max, sum, unnormalised output) in ws for swa_combine_kernel
  const int nsplit = a.nsplit > 1 ? a.nsplit : 1;
  const int per = (pieces + nsplit - 1) / nsplit;
  const int c_lo = blockIdx.z * per, c_hi = c_lo + per < pieces ? c_lo + per : pieces;
  for (int c = c_lo + wave; c < c_hi; c += SWA_WAVES) {
    const int j0 = c < pf ? c * 64 : jlo + (c - pf) * 64;
    const int jend = c < pf ? nf - 1 : i;  // last visible key of this piece's region
    const int j = j0 + lane;
    const bool valid = j <= jend;
    float sc = -INFINITY;
    if (valid) {
      const float* kp = a.kc + (size_t)j * kld + (size_t)g * khs;
      float acc = 0.0f;
      if (v4) {
        int d = 0;
        for (; d + 32 <= a.dim; d += 32) {  // eight 16-byte pieces of the key row in flight before the first product
          float4 kv[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) kv[u] = *reinterpret_cast<const float4*>(kp + d + 4 * u);
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const float4 qv = *reinterpret_cast<const float4*>(qs + d + 4 * u);
            acc += qv.x * kv[u].x + qv.y * kv[u].y + qv.z * kv[u].z + qv.w * kv[u].w;
          }
        }
        for (; d < a.dim; d += 4) {
          const float4 kv = *reinterpret_cast<const float4*>(kp + d);
          const float4 qv = *reinterpret_cast<const float4*>(qs + d);
          acc += qv.x * kv.x + qv.y * kv.y + qv.z * kv.z + qv.w * kv.w;
        }
      } else {
        for (int d = 0; d < a.dim; ++d) acc += qs[d] * kp[d];
      }
      sc = acc * a.scale;
      if (a.softcap > 0.0f) sc = swa_cap(sc, a.softcap, 1.0f / a.softcap);
      if (a.dist_r1) sc -= swa_dist(r1, r2, i - j);
    }
    float cm = sc;
#pragma unroll
    for (int w = 32; w >= 1; w >>= 1) cm = fmaxf(cm, __shfl_xor(cm, w));
    const float mn = a.sigmoid ? 0.0f : fmaxf(m, cm);  // finite: lane 0 of a piece is always a visible key
    const float p = !valid ? 0.0f : a.sigmoid ? 1.0f / (1.0f + expf(-(sc + hb))) : expf(sc - mn);
    const float corr = expf(m - mn);  // m = -inf at the first piece: 0
    float ps = p;
#pragma unroll
    for (int w = 32; w >= 1; w >>= 1) ps += __shfl_xor(ps, w);
    l = l * corr + ps;
    m = mn;
    const int cnt = (jend - j0 + 1) < 64 ? (jend - j0 + 1) : 64;
#pragma unroll
    for (int r = 0; r < SWA_MAX_VR; ++r) o[r] *= corr;
    const float* vp = a.vc + (size_t)j0 * vld + (size_t)g * a.vdim;
    // jj is wave-uniform: the weight of key jj comes straight from its lane's register; eight rows of V per step, so that
    // their loads are in flight together
    int jj = 0;
    for (; jj + 8 <= cnt; jj += 8) {
      float pj[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) pj[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), jj + u));
      const float* vr = vp + (size_t)jj * vld;
#pragma unroll
      for (int r = 0; r < SWA_MAX_VR; ++r) {
        const int d = lane + 64 * r;
        if (d < a.vdim) {
          float vv[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) vv[u] = vr[(size_t)u * vld + d];
          o[r] += ((pj[0] * vv[0] + pj[1] * vv[1]) + (pj[2] * vv[2] + pj[3] * vv[3])) +
                  ((pj[4] * vv[4] + pj[5] * vv[5]) + (pj[6] * vv[6] + pj[7] * vv[7]));
        }
      }
    }
    for (; jj < cnt; ++jj) {
      const float pj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), jj));
      const float* vr = vp + (size_t)jj * vld;
#pragma unroll
      for (int r = 0; r < SWA_MAX_VR; ++r) {
        const int d = lane + 64 * r;
        if (d < a.vdim) o[r] += pj * vr[d];
      }
    }
  }
  if (lane == 0) {
    ml[wave * 2] = m;
    ml[wave * 2 + 1] = l;
  }
#pragma unroll
  for (int r = 0; r < SWA_MAX_VR; ++r) {
    const int d = lane + 64 * r;
    if (d < a.vdim) ow[wave * a.vdim + d] = o[r];
  }
  __syncthreads();
  float M = -INFINITY;
#pragma unroll
  for (int w = 0; w < SWA_WAVES; ++w) M = fmaxf(M, ml[w * 2]);
  // the sink joins where the LAST merge happens: here without splits, in swa_merge_records with them
  const bool sink_here = a.sink && nsplit == 1;
  const float sv = a.sink && a.sink_val ? a.sink_val[h] : 0.0f;
  if (sink_here) M = fmaxf(M, sv);
  float f[SWA_WAVES], L = sink_here ? expf(sv - M) : 0.0f;
#pragma unroll
  for (int w = 0; w < SWA_WAVES; ++w) {
    f[w] = ml[w * 2] == -INFINITY ? 0.0f : expf(ml[w * 2] - M);  // a wave without a piece counts nothing
    L += ml[w * 2 + 1] * f[w];
  }
  if (nsplit > 1) {
    float* rec = a.ws + (((size_t)t * a.heads + h) * nsplit + blockIdx.z) * (a.vdim + 2);
    // (agent-scope stores: with the merge in this launch the reader may sit on another XCD, behind another L2)
    if (tid == 0) {
      swa_st_agent(rec, M);  // -inf and sum 0 when this split had no piece
      swa_st_agent(rec + 1, M == -INFINITY ? 0.0f : L);
    }
    for (int d = tid; d < a.vdim; d += 256) {
      float acc = 0.0f;
#pragma unroll
      for (int w = 0; w < SWA_WAVES; ++w) acc += f[w] == 0.0f ? 0.0f : ow[w * a.vdim + d] * f[w];
      swa_st_agent(rec + 2 + d, M == -INFINITY ? 0.0f : acc);
    }
    if (!a.done_cnt) return;  // swa_combine_kernel follows
    // The last workgroup of this (token, head) to arrive merges the records itself (no second launch): the record stores
    // are acknowledged, then one arrival per workgroup is counted; the counter goes back to zero for the next launch.
    __shared__ int is_last;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
      unsigned* c = a.done_cnt + (size_t)t * a.heads + h;
      const unsigned before = __hip_atomic_fetch_add(c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      is_last = before + 1u == (unsigned)nsplit;
      if (is_last) __hip_atomic_store(c, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!is_last || wave != 0) return;
    swa_merge_records(a, t, h, lane);
    return;
  }
  float* op = a.out + (size_t)t * a.heads * a.vdim + (size_t)h * a.vdim;
  for (int d = tid; d < a.vdim; d += 256) {
    float acc = 0.0f;
#pragma unroll
    for (int w = 0; w < SWA_WAVES; ++w) acc += f[w] == 0.0f ? 0.0f : ow[w * a.vdim + d] * f[w];
    op[d] = a.sigmoid ? acc : acc / L;
  }
}

__global__ __launch_bounds__(64) void swa_combine_kernel(const SwaArgs a) { swa_merge_records(a, blockIdx.x, blockIdx.y, threadIdx.x); }

// ---- prompt chunks on the FP32 matrix instruction (v_mfma_f32_32x32x2_f32: exact FP32 products, FP32 accumulation) --------
// One workgroup of 4 waves per (32-query tile, head). The key tiles of 32 positions that any query of the tile can see
// (from the first query's window start to the last query's position) are dealt round-robin to the waves; each wave walks its
// tiles with an online softmax of its own and the four (max, sum, O) are merged through LDS in wave order.
//   S^T[key][query] = K Q^T: A = a lane's own cache row (16 bytes per load: lane half h owns d = 8 i + 4 h + 0..3 -- the
//     order of a sum does not matter to the instruction), B = the query tile in LDS, zero-padded to a multiple of 8.
//   The result has the query on the lane and 16 keys in registers; those registers are the A operand of O += P V as they
//     stand (the result layout puts the key index where the next product's k index lives); V rows are read 128 B per half wave.
typedef float swa_f32x4 __attribute__((ext_vector_type(4)));
typedef float swa_f32x16 __attribute__((ext_vector_type(16)));

// key (row of the 32x32 result) held in accumulator register e of lane half h
__device__ __forceinline__ int swa_acc_row(int e, int h) { return (e & 3) + 8 * (e >> 2) + 4 * h; }

__host__ __device__ inline int swa_dim_padded(int dim) { return (dim + 7) & ~7; }
constexpr int SWA_SLOTS = 2;     // output slots in LDS: waves w and w + 2 share slot w (added in wave order)
constexpr int SWA_KREG4 = 16;    // 16-byte pieces of a key row a lane half can hold in registers: dim <= 128
__host__ __device__ inline size_t swa_mfma_lds_floats(int dim, int db) {
  return (size_t)32 * (swa_dim_padded(dim) + 4) + 3 * SWA_WAVES * 32 + 32 + (size_t)SWA_SLOTS * 32 * 32 * db;
}

// DB: value columns per lane (vdim <= 32 * DB; lane r owns columns DB * r .. DB * r + DB - 1, one wide load per V row).
// PRE: the lane's key row lives in registers (dim <= 128) and the NEXT tile's row is asked for as soon as the products have
// read this one, so that its round trip runs under the softmax and P V of the tile in hand.
template <int DB, bool PRE>
__global__ __launch_bounds__(256, 2) void swa_mfma_kernel(const SwaArgs a) {  // two workgroups per CU: 256 registers a lane
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int dp = swa_dim_padded(a.dim), qs = dp + 4, dk = dp / 8;
  float* sm_q = lds;                        // [32][dp + 4]
  float* sm_m = sm_q + 32 * qs;             // [waves][32] running max per query
  float* sm_l = sm_m + SWA_WAVES * 32;      // [waves][32] sum
  float* sm_f = sm_l + SWA_WAVES * 32;      // [waves][32] the wave's factor exp(m_w - M)
  float* sm_inv = sm_f + SWA_WAVES * 32;    // [32] 1 / L
  float* sm_o = sm_inv + 32;                // [slots][32][32 * DB]
  const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, h = lane >> 5, wave = tid >> 6;
  const int head = blockIdx.y, q0 = blockIdx.x * 32;
  const int g = head / (a.heads / a.kv_heads);
  const int start = a.pos_dev ? *a.pos_dev : a.start_pos;
  const int kld = a.kld > 0 ? a.kld : a.kv_heads * (a.k_hstride > 0 ? a.k_hstride : a.dim), vld = a.vld > 0 ? a.vld : a.kv_heads * a.vdim;
  const int last_i = q0 + 31 < a.T ? q0 + 31 : a.T - 1;
  const int qpos = start + (q0 + r < a.T ? q0 + r : a.T - 1);  // rows beyond the chunk repeat its last query; never stored
  const int last_q = start + last_i;
  const int klo = a.window > 0 && start + q0 - a.window + 1 > 0 ? start + q0 - a.window + 1 : 0;
  const int t_lo = klo >> 5, t_hi = last_q >> 5;
  // kept first keys: their tiles of 32 positions below the window's first tile are walked before the window's tiles
  // (virtual tile vt < tf is tile vt, vt >= tf is tile t_lo + vt - tf)
  const int tf = a.keep_first > 0 ? (((a.keep_first + 31) >> 5) < t_lo ? ((a.keep_first + 31) >> 5) : t_lo) : 0;
  const int nvt = tf + t_hi - t_lo + 1;
  auto tile_of = [&](int vt) { return vt < tf ? vt : t_lo + vt - tf; };
  const float hb = a.sigmoid && a.head_bias ? a.head_bias[head] : 0.0f;
  // a row that no query of the tile can see (it carries weight 0) is read from a row that one of them can
  auto clamp_row = [&](int pr) { return pr > last_q ? last_q : (pr < klo && pr >= a.keep_first) ? klo : pr; };
  const int qhs = a.q_hstride > 0 ? a.q_hstride : a.dim, khs = a.k_hstride > 0 ? a.k_hstride : a.dim;
  const float r1 = a.dist_r1 ? a.dist_r1[head] : 0.0f, r2 = a.dist_r1 ? a.dist_r2[head] : 0.0f;
  const float inv_cap = a.softcap > 0.0f ? 1.0f / a.softcap : 0.0f;
  const bool kvec = (a.dim & 3) == 0 && (kld & 3) == 0 && (khs & 3) == 0 && ((size_t)a.kc & 15) == 0;
  const bool vvec = (a.vdim % DB) == 0 && (DB == 1 || (((size_t)a.vc & 15) == 0 && (DB != 3) && (vld % DB) == 0));
  // piece i (d = 8 i + 4 h + 0..3) of the lane's key row of a tile; rows outside [klo, last_q] are seen by no query of the
  // tile (masked below): their loads stay inside that range, so that nothing is read that the tile could not read
  auto load_k4 = [&](int tile, int i) -> swa_f32x4 {
    const int krow = clamp_row(tile * 32 + r);
    const float* kp = a.kc + (size_t)krow * kld + (size_t)g * khs + 4 * h + 8 * i;
    const int d = 8 * i + 4 * h;
    swa_f32x4 kv;
    if (kvec) {
      kv = d + 4 <= a.dim ? *reinterpret_cast<const swa_f32x4*>(kp) : swa_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) kv[c] = d + c < a.dim ? kp[c] : 0.0f;
    }
    return kv;
  };
  // the lane's DB value columns of the keys held in accumulator registers e0 .. e0 + 7 (masked keys carry weight 0; their
  // rows are clamped like the key rows)
  auto load_v = [&](int p0, int e0, float (*vv)[DB]) __attribute__((always_inline)) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int vrow = clamp_row(p0 + swa_acc_row(e0 + e, h));
      const float* vp = a.vc + (size_t)vrow * vld + (size_t)g * a.vdim + DB * r;
      if (vvec && DB * r < a.vdim) {
        if (DB == 4) {
          const swa_f32x4 t4 = *reinterpret_cast<const swa_f32x4*>(vp);
#pragma unroll
          for (int b = 0; b < DB; ++b) vv[e][b] = t4[b];
        } else if (DB == 2) {
          const float2 t2 = *reinterpret_cast<const float2*>(vp);
          vv[e][0] = t2.x;
          vv[e][DB - 1] = t2.y;
        } else {
#pragma unroll
          for (int b = 0; b < DB; ++b) vv[e][b] = vp[b];
        }
      } else {
#pragma unroll
        for (int b = 0; b < DB; ++b) vv[e][b] = DB * r + b < a.vdim ? vp[b] : 0.0f;
      }
    }
  };
  swa_f32x4 kreg[PRE ? SWA_KREG4 : 1];
  if (PRE && wave < nvt) {
#pragma unroll
    for (int i = 0; i < SWA_KREG4; ++i)
      if (i < dk) kreg[i] = load_k4(tile_of(wave), i);
  }
  for (int i = tid; i < 32 * dp; i += 256) {
    const int row = i / dp, d = i - row * dp;
    sm_q[row * qs + d] = (q0 + row < a.T && d < a.dim) ? a.q[(size_t)(q0 + row) * a.ldq + (size_t)head * qhs + d] : 0.0f;
  }
  __syncthreads();
  swa_f32x16 o[DB];
#pragma unroll
  for (int b = 0; b < DB; ++b)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[b][e] = 0.0f;
  float mrun = -INFINITY, lrun = 0.0f;
  const float* qrow = sm_q + r * qs + 4 * h;
  for (int vt = wave; vt < nvt; vt += SWA_WAVES) {
    const int tile = tile_of(vt);
    const int p0 = tile * 32;
    swa_f32x16 s;
#pragma unroll
    for (int e = 0; e < 16; ++e) s[e] = 0.0f;
    if (PRE) {
#pragma unroll
      for (int i = 0; i < SWA_KREG4; ++i)
        if (i < dk) {
          const swa_f32x4 qv = *reinterpret_cast<const swa_f32x4*>(qrow + 8 * i);
#pragma unroll
          for (int c = 0; c < 4; ++c) s = __builtin_amdgcn_mfma_f32_32x32x2f32(kreg[i][c], qv[c], s, 0, 0, 0);
        }
      if (vt + SWA_WAVES < nvt) {
#pragma unroll
        for (int i = 0; i < SWA_KREG4; ++i)
          if (i < dk) kreg[i] = load_k4(tile_of(vt + SWA_WAVES), i);
      }
    } else {
      for (int i = 0; i < dk; ++i) {
        const swa_f32x4 kv = load_k4(tile, i);
        const swa_f32x4 qv = *reinterpret_cast<const swa_f32x4*>(qrow + 8 * i);
#pragma unroll
        for (int c = 0; c < 4; ++c) s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[c], qv[c], s, 0, 0, 0);
      }
    }
    float va[8][DB];
    load_v(p0, 0, va);  // the V rows of the first 8 registers' keys: asked for now, needed after the softmax
    float tmax = -INFINITY;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int p = p0 + swa_acc_row(e, h);
      const bool seen = p <= qpos && (a.window <= 0 || qpos - p < a.window || p < a.keep_first);
      float sc = s[e] * a.scale;
      if (a.softcap > 0.0f) sc = swa_cap(sc, a.softcap, inv_cap);
      if (a.dist_r1) sc -= swa_dist(r1, r2, seen ? qpos - p : 0);
      s[e] = seen ? sc : -INFINITY;
      tmax = fmaxf(tmax, s[e]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
    // sigmoid mode: the maximum is pinned to 0 once the query has seen a key, so that no factor ever differs from 1
    const float mnew = a.sigmoid ? (tmax == -INFINITY ? mrun : 0.0f) : fmaxf(mrun, tmax);  // may still be -inf: a tile can lie wholly outside one query's window
    const float corr = mrun == -INFINITY ? 0.0f : expf(mrun - mnew);
    mrun = mnew;
    float psum = 0.0f;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      s[e] = s[e] == -INFINITY ? 0.0f : a.sigmoid ? 1.0f / (1.0f + expf(-(s[e] + hb))) : expf(s[e] - mnew);
      psum += s[e];
    }
    lrun = lrun * corr + psum;
    if (__any(corr != 1.0f)) {  // O's rows are queries: each row's factor comes from the lane that owns the query
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float c = __shfl(corr, swa_acc_row(e, h));
#pragma unroll
        for (int b = 0; b < DB; ++b) o[b][e] *= c;
      }
    }
    float vb[8][DB];
    load_v(p0, 8, vb);  // the second half's round trip runs under the first half's products
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
      for (int b = 0; b < DB; ++b) o[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(s[e], va[e][b], o[b], 0, 0, 0);
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
      for (int b = 0; b < DB; ++b) o[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(s[8 + e], vb[e][b], o[b], 0, 0, 0);
  }
  const float ltot = lrun + __shfl_xor(lrun, 32);
  if (h == 0) {
    sm_m[wave * 32 + r] = mrun;
    sm_l[wave * 32 + r] = ltot;
  }
  __syncthreads();
  if (h == 0) {
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < SWA_WAVES; ++w) M = fmaxf(M, sm_m[w * 32 + r]);  // finite: every query sees itself
    const float sv = a.sink && a.sink_val ? a.sink_val[head] : 0.0f;
    if (a.sink) M = fmaxf(M, sv);
    const float mw = sm_m[wave * 32 + r];
    sm_f[wave * 32 + r] = mw == -INFINITY ? 0.0f : expf(mw - M);
    if (wave == 0) {
      float L = a.sink ? expf(sv - M) : 0.0f;
#pragma unroll
      for (int w = 0; w < SWA_WAVES; ++w) {
        const float m2 = sm_m[w * 32 + r];
        L += m2 == -INFINITY ? 0.0f : sm_l[w * 32 + r] * expf(m2 - M);
      }
      sm_inv[r] = a.sigmoid ? 1.0f : 1.0f / L;
    }
  }
  __syncthreads();
  // merge in wave order through SWA_SLOTS slots: waves 0, 1 store, then waves 2, 3 add to the slot of wave - 2
  constexpr int OW = 32 * DB;
  float* slot = sm_o + (size_t)(wave % SWA_SLOTS) * 32 * OW;
#pragma unroll
  for (int round = 0; round < SWA_WAVES / SWA_SLOTS; ++round) {
    if (wave / SWA_SLOTS == round) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = swa_acc_row(e, h);
        const float f = sm_f[wave * 32 + row];
#pragma unroll
        for (int b = 0; b < DB; ++b) {
          float* p = slot + row * OW + DB * r + b;
          *p = round == 0 ? o[b][e] * f : *p + o[b][e] * f;
        }
      }
    }
    __syncthreads();
  }
  for (int i = tid; i < 32 * OW; i += 256) {
    const int row = i / OW, col = i - row * OW;
    if (q0 + row >= a.T || col >= a.vdim) continue;
    float acc = 0.0f;
#pragma unroll
    for (int w = 0; w < SWA_SLOTS; ++w) acc += sm_o[(size_t)w * 32 * OW + i];
    a.out[(size_t)(q0 + row) * a.heads * a.vdim + (size_t)head * a.vdim + col] = acc * sm_inv[row];
  }
}

template <int DB, bool PRE>
int launch_swa_mfma_as(const SwaArgs& a, hipStream_t s) {
  static TlDeviceOnce lds_raised;  // per instantiation, per device
  const size_t lds = sizeof(float) * swa_mfma_lds_floats(a.dim, DB);
  TL_TRY(tl_raise_lds_limit(swa_mfma_kernel<DB, PRE>, 160 * 1024, lds_raised));
  swa_mfma_kernel<DB, PRE><<<dim3((a.T + 31) / 32, a.heads), 256, lds, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}
template <int DB>
int launch_swa_mfma(const SwaArgs& a, hipStream_t s) {
  return swa_dim_padded(a.dim) <= 8 * SWA_KREG4 ? launch_swa_mfma_as<DB, true>(a, s) : launch_swa_mfma_as<DB, false>(a, s);
}

}  // namespace

// prompt chunks whose shapes fit go to the matrix cores (TL_SWA_MFMA=0: never)
static bool swa_mfma_wanted(const SwaArgs& a) {
  static const bool on = [] {
    const char* e = getenv("TL_SWA_MFMA");
    return !e || atoi(e) != 0;
  }();
  const int db = (a.vdim + 31) / 32;
  return on && a.T >= 16 && db <= 4 && sizeof(float) * swa_mfma_lds_floats(a.dim, db) <= 160 * 1024;
}

int tl_launch_swa(const SwaArgs& a, hipStream_t s) {
  TL_REQUIRE(a.q && a.kc && a.vc && a.out && a.T > 0, "swa: bad arguments");
  TL_REQUIRE(a.heads > 0 && a.kv_heads > 0 && a.heads % a.kv_heads == 0, "swa: %d heads over %d key/value heads", a.heads,
             a.kv_heads);
  TL_REQUIRE(a.dim > 0 && a.vdim > 0 && a.vdim <= 64 * SWA_MAX_VR, "swa: value size %d outside (0, %d]", a.vdim,
             64 * SWA_MAX_VR);
  TL_REQUIRE(a.pos_dev || a.start_pos >= 0, "swa: negative start position");
  TL_REQUIRE(a.heads <= 65535, "swa: too many heads");
  TL_REQUIRE(a.keep_first >= 0, "swa: negative number of kept first keys");
  TL_REQUIRE(!a.sink || !a.sigmoid, "swa: a sink belongs to a softmax");
  TL_REQUIRE(!a.sink_val || a.sink, "swa: sink scores without a sink");
  TL_REQUIRE(!a.dist_r1 == !a.dist_r2, "swa: the distance bias needs both of its vectors");
  TL_REQUIRE(a.q_hstride >= 0 && a.k_hstride >= 0 && (a.q_hstride == 0 || a.q_hstride >= a.dim) &&
                 (a.k_hstride == 0 || a.k_hstride >= a.dim),
             "swa: head strides %d / %d below the key size %d", a.q_hstride, a.k_hstride, a.dim);
  TL_REQUIRE((a.kld == 0 || a.kld >= (a.kv_heads - 1) * (a.k_hstride > 0 ? a.k_hstride : a.dim) + a.dim) && (a.vld == 0 || a.vld >= a.kv_heads * a.vdim),
             "swa: cache rows %d / %d shorter than the heads they hold", a.kld, a.vld);
  if (swa_mfma_wanted(a)) {
    switch ((a.vdim + 31) / 32) {
      case 1: return launch_swa_mfma<1>(a, s);
      case 2: return launch_swa_mfma<2>(a, s);
      case 3: return launch_swa_mfma<3>(a, s);
      default: return launch_swa_mfma<4>(a, s);
    }
  }
  const size_t lds = sizeof(float) * (((a.dim + 3) & ~3) + SWA_WAVES * a.vdim + SWA_WAVES * 2);
  TL_REQUIRE(lds <= 64 * 1024, "swa: key size %d too large", a.dim);
  TL_REQUIRE(a.heads <= 65535, "swa: too many heads");
  const int nsplit = a.nsplit > 1 ? a.nsplit : 1;
  TL_REQUIRE(nsplit == 1 || a.ws, "swa: split launch without a workspace");
  TL_REQUIRE(nsplit <= 64, "swa: %d splits", nsplit);
  swa_kernel<<<dim3(a.T, a.heads, nsplit), 256, lds, s>>>(a);
  if (nsplit > 1 && !a.done_cnt) swa_combine_kernel<<<dim3(a.T, a.heads), 64, 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_swa_splits(int T, int window, int max_pos, int keep_first) {
  if (T > 4) return 1;  // a chunk of a prompt has workgroups enough
  int keys = window > 0 && window < max_pos ? window : max_pos;
  if (window > 0 && keep_first > 0) keys = keys + keep_first + 63 < max_pos ? keys + keep_first + 63 : max_pos;
  const int pieces = (keys + 63) / 64;
  int n = (pieces + SWA_WAVES - 1) / SWA_WAVES;  // a piece per wave and split
  return n < 1 ? 1 : n > 32 ? 32 : n;
}

size_t tl_swa_ws_floats(int T, int heads, int vdim, int nsplit) { return (size_t)T * heads * nsplit * (vdim + 2); }

extern "C" int tl_swa_attention(const float* q_dev, const float* k_cache_dev, const float* v_cache_dev, float* out_dev,
                                int num_tokens, int start_pos, int heads, int kv_heads, int dim, int vdim, int window,
                                float scale, void* stream) {
  SwaArgs a = {};
  a.q = q_dev;
  a.ldq = heads * dim;
  a.kc = k_cache_dev;
  a.vc = v_cache_dev;
  a.out = out_dev;
  a.T = num_tokens;
  a.heads = heads;
  a.kv_heads = kv_heads;
  a.dim = dim;
  a.vdim = vdim;
  a.window = window;
  a.scale = scale;
  a.start_pos = start_pos;
  a.nsplit = tl_swa_splits(num_tokens, window, start_pos + num_tokens);
  if (a.nsplit > 1) {
    void* ws = nullptr;
    TL_TRY(tl_scratch(TL_SCRATCH_ATTN, sizeof(float) * tl_swa_ws_floats(num_tokens, heads, vdim, a.nsplit), &ws));
    a.ws = static_cast<float*>(ws);
  }
  return tl_launch_swa(a, static_cast<hipStream_t>(stream));
}

extern "C" int tl_window_attention(const float* q_dev, const float* k_cache_dev, const float* v_cache_dev, float* out_dev,
                                   int num_tokens, int start_pos, int heads, int kv_heads, int dim, int vdim, int window,
                                   int keep_first, float scale, int sigmoid, const float* head_bias_dev, void* stream) {
  SwaArgs a = {};
  a.q = q_dev;
  a.ldq = heads * dim;
  a.kc = k_cache_dev;
  a.vc = v_cache_dev;
  a.out = out_dev;
  a.T = num_tokens;
  a.heads = heads;
  a.kv_heads = kv_heads;
  a.dim = dim;
  a.vdim = vdim;
  a.window = window;
  a.scale = scale;
  a.start_pos = start_pos;
  a.keep_first = keep_first;
  a.sigmoid = sigmoid;
  a.head_bias = head_bias_dev;
  a.nsplit = tl_swa_splits(num_tokens, window, start_pos + num_tokens, keep_first);
  if (a.nsplit > 1) {
    void* ws = nullptr;
    TL_TRY(tl_scratch(TL_SCRATCH_ATTN, sizeof(float) * tl_swa_ws_floats(num_tokens, heads, vdim, a.nsplit), &ws));
    a.ws = static_cast<float*>(ws);
  }
  return tl_launch_swa(a, static_cast<hipStream_t>(stream));
}

extern "C" int tl_window_attention_rows(const float* q_dev, const float* k_cache_dev, const float* v_cache_dev, float* out_dev,
                                        int num_tokens, int start_pos, int heads, int kv_heads, int dim, int vdim, int k_ld,
                                        int v_ld, int window, int keep_first, float scale, int mode, const float* head_bias_dev,
                                        void* stream) {
  TL_REQUIRE(mode >= TL_ATTN_SOFTMAX && mode <= TL_ATTN_SOFTMAX_SINK, "tl_window_attention_rows: weight kind %d", mode);
  SwaArgs a = {};
  a.q = q_dev;
  a.ldq = heads * dim;
  a.kc = k_cache_dev;
  a.vc = v_cache_dev;
  a.out = out_dev;
  a.T = num_tokens;
  a.heads = heads;
  a.kv_heads = kv_heads;
  a.dim = dim;
  a.vdim = vdim;
  a.kld = k_ld;
  a.vld = v_ld;
  a.window = window;
  a.scale = scale;
  a.start_pos = start_pos;
  a.keep_first = keep_first;
  a.sigmoid = mode == TL_ATTN_SIGMOID;
  a.sink = mode == TL_ATTN_SOFTMAX_SINK;
  a.head_bias = head_bias_dev;
  a.nsplit = tl_swa_splits(num_tokens, window, start_pos + num_tokens, keep_first);
  if (a.nsplit > 1) {
    void* ws = nullptr;
    TL_TRY(tl_scratch(TL_SCRATCH_ATTN, sizeof(float) * tl_swa_ws_floats(num_tokens, heads, vdim, a.nsplit), &ws));
    a.ws = static_cast<float*>(ws);
  }
  return tl_launch_swa(a, static_cast<hipStream_t>(stream));
}

extern "C" int tl_window_attention_opts(const float* q_dev, int ldq, int q_hstride, const float* k_cache_dev, int k_ld,
                                        int k_hstride, const float* v_cache_dev, int v_ld, float* out_dev, int num_tokens,
                                        int start_pos, int heads, int kv_heads, int dim, int vdim, int window, float scale,
                                        float softcap, const float* r1_dev, const float* r2_dev, int sink,
                                        const float* sink_dev, void* stream) {
  SwaArgs a = {};
  a.q = q_dev;
  a.ldq = ldq > 0 ? ldq : heads * (q_hstride > 0 ? q_hstride : dim);
  a.q_hstride = q_hstride;
  a.kc = k_cache_dev;
  a.kld = k_ld;
  a.k_hstride = k_hstride;
  a.vc = v_cache_dev;
  a.vld = v_ld;
  a.out = out_dev;
  a.T = num_tokens;
  a.heads = heads;
  a.kv_heads = kv_heads;
  a.dim = dim;
  a.vdim = vdim;
  a.window = window;
  a.scale = scale;
  a.softcap = softcap;
  a.dist_r1 = r1_dev;
  a.dist_r2 = r2_dev;
  a.sink = sink;
  a.sink_val = sink_dev;
  a.start_pos = start_pos;
  a.nsplit = tl_swa_splits(num_tokens, window, start_pos + num_tokens, 0);
  if (a.nsplit > 1) {
    void* ws = nullptr;
    TL_TRY(tl_scratch(TL_SCRATCH_ATTN, sizeof(float) * tl_swa_ws_floats(num_tokens, heads, vdim, a.nsplit), &ws));
    a.ws = static_cast<float*>(ws);
  }
  return tl_launch_swa(a, static_cast<hipStream_t>(stream));
}
