// Per-head RMSNorm of q and k, rotary embedding of both, and the KV-store, in one pass.
// Replaces the chain in front of the attention call of the reference's Qwen3 attention layer
// (mini_sglang_mlx/models/qwen3.py:60-68: q_norm, k_norm, rope(q), rope(k), then the store
// inside AttnBackend.forward, attention/backend.py:139), which materialises normalised q and k,
// rotated q and k, and then reads k and v again to scatter them into the pools.
//
//   y   = w * bf16(x * rsqrt(mean(x^2) + eps))                       (per head, fp32 inside)
//   o_i = y_i cos(t_i) - y_{i+d/2} sin(t_i),  o_{i+d/2} = y_i sin(t_i) + y_{i+d/2} cos(t_i)
//   t_i = float(position) * exp2(-(i / (d/2)) * log2(base))          (rotate-half form, rotary_dim = d)
//   q_out[t, h] = o(q[t, h]);  k_cache[out_loc[t], h] = o(k[t, h]);  v_cache[out_loc[t], h] = v[t, h]
//
// HBM-bound: every element of q, k, v is read once and written once
// (2 * (n_q + 2 n_kv) * d * 2 bytes per token, + 8 for position and slot).
// Sixteen lanes own one token's head: lane j holds elements E j .. E j + E - 1 of both halves
// (E = d / 32), so the rotation pairs are lane-local and the mean is a 16-lane xor reduction.
// A group walks a chunk of the token's heads, so sines and cosines (accurate range reduction:
// positions reach 10^5 radians) are computed once per chunk, not once per head.
#include "msgl_device.h"
#include "msgl_internal.h"

namespace msgl {
namespace {

constexpr int kHeadsPerGroup = 8;
constexpr int kGroupLanes = 16;
constexpr int kThreads = 256;

struct NormRopeParams {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  const uint16_t* q_weight;
  const uint16_t* k_weight;
  const int32_t* positions;
  const int32_t* out_loc;
  uint16_t* q_out;
  uint16_t* k_cache;
  uint16_t* v_cache;
  int64_t q_stride0, k_stride0, v_stride0, kc_stride0, vc_stride0, num_slots;
  int32_t n_tokens, n_q, n_kv, chunks;  // chunks of kHeadsPerGroup heads per token
  float eps, log2_base;
};

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}

template <int E>
struct Vec;  // E bf16 values as one load
template <>
struct Vec<4> { typedef u32x2_t type; };
template <>
struct Vec<8> { typedef u32x4_t type; };

template <int D>
__global__ __launch_bounds__(kThreads) void qk_norm_rope_store_kernel(NormRopeParams p) {
  constexpr int E = D / 32;  // elements per lane and half
  using V = typename Vec<E>::type;
  const int j = threadIdx.x & (kGroupLanes - 1);
  const int64_t item = (int64_t)blockIdx.x * (kThreads / kGroupLanes) + (threadIdx.x / kGroupLanes);
  if (item >= (int64_t)p.n_tokens * p.chunks) return;  // whole groups leave together
  const int t = (int)(item / p.chunks);
  const int chunk = (int)(item - (int64_t)t * p.chunks);
  const int n_heads = p.n_q + 2 * p.n_kv;
  const int h_begin = chunk * kHeadsPerGroup;
  const int h_end = min(h_begin + kHeadsPerGroup, n_heads);

  // sines and cosines of this lane's pairs (only if the chunk holds a q or k head)
  float cs[E], sn[E];
  if (h_begin < p.n_q + p.n_kv) {
    const float pos = (float)p.positions[t];
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const float d = (float)(j * E + e) / (float)(D / 2);
      const float inv_freq = exp2f(-d * p.log2_base);
      sincosf(pos * inv_freq, &sn[e], &cs[e]);
    }
  }
  const int64_t slot = p.out_loc[t];
  // a slot id outside the pools stores no k / v row (q_out is still produced): a wild store
  // would be a GPU memory fault
  const bool slot_ok = (uint64_t)slot < (uint64_t)p.num_slots;
  const int off = j * E;

  for (int h = h_begin; h < h_end; ++h) {
    const uint16_t* src;
    uint16_t* dst;
    const uint16_t* w = nullptr;
    if (h < p.n_q) {
      src = p.q + (int64_t)t * p.q_stride0 + (int64_t)h * D;
      dst = p.q_out + ((int64_t)t * p.n_q + h) * D;
      w = p.q_weight;
    } else if (h < p.n_q + p.n_kv) {
      src = p.k + (int64_t)t * p.k_stride0 + (int64_t)(h - p.n_q) * D;
      dst = p.k_cache + slot * p.kc_stride0 + (int64_t)(h - p.n_q) * D;
      w = p.k_weight;
    } else {
      src = p.v + (int64_t)t * p.v_stride0 + (int64_t)(h - p.n_q - p.n_kv) * D;
      dst = p.v_cache + slot * p.vc_stride0 + (int64_t)(h - p.n_q - p.n_kv) * D;
    }
    V lo = *reinterpret_cast<const V*>(src + off);
    V hi = *reinterpret_cast<const V*>(src + D / 2 + off);
    if (w != nullptr) {
      const V wl = *reinterpret_cast<const V*>(w + off);
      const V wh = *reinterpret_cast<const V*>(w + D / 2 + off);
      float xl[E], xh[E];
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        const uint32_t a = lo[e >> 1], b = hi[e >> 1];
        xl[e] = bf16_to_f32((uint16_t)((e & 1) ? a >> 16 : a & 0xffffu));
        xh[e] = bf16_to_f32((uint16_t)((e & 1) ? b >> 16 : b & 0xffffu));
        ss += xl[e] * xl[e] + xh[e] * xh[e];
      }
#pragma unroll
      for (int m = 1; m < kGroupLanes; m <<= 1) ss += __shfl_xor(ss, m, kWave);
      const float norm = rsqrtf(ss * (1.0f / D) + p.eps);
      uint16_t ol[E], oh[E];
#pragma unroll
      for (int e = 0; e < E; ++e) {
        const uint32_t a = wl[e >> 1], b = wh[e >> 1];
        const float wlo = bf16_to_f32((uint16_t)((e & 1) ? a >> 16 : a & 0xffffu));
        const float whi = bf16_to_f32((uint16_t)((e & 1) ? b >> 16 : b & 0xffffu));
        // normalised value and weighted value each pass through bf16, as they do when the
        // norm is a kernel of its own with a bf16 result
        const float yl = bf16_to_f32(f32_to_bf16(wlo * bf16_to_f32(f32_to_bf16(xl[e] * norm))));
        const float yh = bf16_to_f32(f32_to_bf16(whi * bf16_to_f32(f32_to_bf16(xh[e] * norm))));
        ol[e] = f32_to_bf16(yl * cs[e] - yh * sn[e]);
        oh[e] = f32_to_bf16(yl * sn[e] + yh * cs[e]);
      }
#pragma unroll
      for (int e = 0; e < E; e += 2) {
        lo[e >> 1] = (uint32_t)ol[e] | ((uint32_t)ol[e + 1] << 16);
        hi[e >> 1] = (uint32_t)oh[e] | ((uint32_t)oh[e + 1] << 16);
      }
    }
    if (h >= p.n_q && !slot_ok) continue;
    *reinterpret_cast<V*>(dst + off) = lo;
    *reinterpret_cast<V*>(dst + D / 2 + off) = hi;
  }
}

}  // namespace

int launch_qk_norm_rope_store(const NormRopeArgs& a, hipStream_t stream) {
  NormRopeParams p;
  p.q = static_cast<const uint16_t*>(a.q);
  p.k = static_cast<const uint16_t*>(a.k);
  p.v = static_cast<const uint16_t*>(a.v);
  p.q_weight = static_cast<const uint16_t*>(a.q_weight);
  p.k_weight = static_cast<const uint16_t*>(a.k_weight);
  p.positions = a.positions;
  p.out_loc = a.out_loc;
  p.q_out = static_cast<uint16_t*>(a.q_out);
  p.k_cache = static_cast<uint16_t*>(a.k_cache);
  p.v_cache = static_cast<uint16_t*>(a.v_cache);
  p.q_stride0 = a.q_stride0;
  p.k_stride0 = a.k_stride0;
  p.v_stride0 = a.v_stride0;
  p.kc_stride0 = a.kc_stride0;
  p.vc_stride0 = a.vc_stride0;
  p.num_slots = a.num_slots;
  p.n_tokens = (int32_t)a.n_tokens;
  p.n_q = (int32_t)a.n_q;
  p.n_kv = (int32_t)a.n_kv;
  const int64_t n_heads = a.n_q + 2 * a.n_kv;
  p.chunks = (int32_t)((n_heads + kHeadsPerGroup - 1) / kHeadsPerGroup);
  p.eps = a.eps;
  p.log2_base = log2f(a.rope_base);
  const int64_t items = a.n_tokens * p.chunks;
  const int64_t per_block = kThreads / kGroupLanes;
  const int64_t blocks = (items + per_block - 1) / per_block;
  if (blocks <= 0) return MSGL_OK;
  if (blocks > 0x7fffffffLL) return MSGL_ERR_SHAPE;
  if (a.head_dim == 128)
    hipLaunchKernelGGL(qk_norm_rope_store_kernel<128>, dim3((unsigned)blocks), dim3(kThreads), 0, stream, p);
  else if (a.head_dim == 256)
    hipLaunchKernelGGL(qk_norm_rope_store_kernel<256>, dim3((unsigned)blocks), dim3(kThreads), 0, stream, p);
  else
    return MSGL_ERR_HEAD_DIM;
  return check_launch();
}

}  // namespace msgl
