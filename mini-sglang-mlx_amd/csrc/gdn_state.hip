// Gated delta-rule recurrence with a slot-indexed fp32 state that is updated in place.
// Replaces gdn_state_inplace (mini-sglang-mlx-kernel/csrc/gdn_state.metal:14-99, host side
// gdn_state.cpp:87-183).  For request b with state rows S[hv][dv][dk] at slot slot_ids[b] and
// every token t of the request, in order:
//     S *= g[t, hv]
//     delta = (v[t, hv, dv] - <S[hv][dv][:], k[t, hk]>) * beta[t, hv]
//     S[hv][dv][:] += k[t, hk] * delta
//     y[t, hv, dv] = <S[hv][dv][:], q[t, hk]>                    hk = hv / (HV / HK)
// q, k, v, g, beta, y are bf16; the state and all arithmetic are fp32.
//
// One state row (dk = 128 floats) lives in the registers of 16 lanes, 8 values each, for the
// whole token loop: the two inner products are 8 lane-local FMAs and a 4-step rotate-and-add
// inside the 16-lane DPP row (no LDS, no cross-row traffic).  A lane group carries R rows, so
// one load of k and q serves R independent recurrences whose latencies overlap; the inputs of
// the next kDepth tokens are always in flight.  Decode (one token) is
// HBM-bound: 2 * dv * dk * 4 bytes of state per (request, hv head) read and written once.
// Prefill is a serial chain per row (as in the reference); parallelism is batch * hv * dv rows.
#include <atomic>

#include "msgl_device.h"
#include "msgl_internal.h"

namespace msgl {
namespace {

constexpr int kDK = 128, kDV = 128;
constexpr int kLanesPerRow = 16;
constexpr int kPerLane = kDK / kLanesPerRow;  // 8 state values per lane and row

struct GdnParams {
  float* state;
  uint16_t* y;
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  const uint16_t* g;
  const uint16_t* beta;
  const int32_t* slot_ids;
  const int32_t* qo_indptr;
  int64_t state_stride0, q_stride0, k_stride0, v_stride0;
  int32_t batch, hv, hv_per_hk, tokens, single_token;
};

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __builtin_bit_cast(float, b << 16); }

template <int N>
__device__ __forceinline__ float row_rotate(float x) {  // lane i of a 16-lane row reads lane (i + N) % 16
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x),
                                                               0x120 + N, 0xf, 0xf, true));
}
__device__ __forceinline__ float row_sum(float x) {  // every lane of the row gets the sum
  x += row_rotate<8>(x);
  x += row_rotate<4>(x);
  x += row_rotate<2>(x);
  x += row_rotate<1>(x);
  return x;
}

__device__ __forceinline__ void unpack8(const u32x4_t raw, float (&f)[kPerLane]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    f[2 * e] = __builtin_bit_cast(float, raw[e] << 16);
    f[2 * e + 1] = __builtin_bit_cast(float, raw[e] & 0xffff0000u);
  }
}

// R = dv rows per 16-lane group.  Workgroup = 256 threads = 16 groups = 16 R consecutive rows
// of one (request, hv head).
template <int R, int kDepth>
__global__ __launch_bounds__(256) void gdn_state_kernel(GdnParams p) {
  constexpr int kRowsPerBlock = 16 * R;
  constexpr int kBlocksPerHead = kDV / kRowsPerBlock;
  const int lane16 = threadIdx.x & 15;
  const int group = threadIdx.x >> 4;
  const int head_item = blockIdx.x / kBlocksPerHead;      // (request, hv head)
  const int row0 = (blockIdx.x - head_item * kBlocksPerHead) * kRowsPerBlock + group * R;
  const int b = head_item / p.hv;
  const int hv = head_item - b * p.hv;
  const int hk = hv / p.hv_per_hk;
  const int start = p.single_token ? b : p.qo_indptr[b];
  const int end = min(p.single_token ? b + 1 : p.qo_indptr[b + 1], p.tokens);
  if (end <= start) return;  // nothing to do: the state stays as it is

  float* srow = p.state + (int64_t)p.slot_ids[b] * p.state_stride0 +
                ((int64_t)hv * kDV + row0) * kDK + lane16 * kPerLane;
  float s[R][kPerLane];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const f32x4_t a = *reinterpret_cast<const f32x4_t*>(srow + r * kDK);
    const f32x4_t c = *reinterpret_cast<const f32x4_t*>(srow + r * kDK + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      s[r][e] = a[e];
      s[r][4 + e] = c[e];
    }
  }

  auto load_token = [&](int t, u32x4_t& kraw, u32x4_t& qraw, uint32_t& graw, uint32_t& braw,
                        uint32_t (&vraw)[R]) {
    kraw = ld_global_b128(p.k + (int64_t)t * p.k_stride0 + hk * kDK + lane16 * kPerLane);
    qraw = ld_global_b128(p.q + (int64_t)t * p.q_stride0 + hk * kDK + lane16 * kPerLane);
    graw = p.g[(int64_t)t * p.hv + hv];
    braw = p.beta[(int64_t)t * p.hv + hv];
#pragma unroll
    for (int r = 0; r < R; ++r) vraw[r] = p.v[(int64_t)t * p.v_stride0 + hv * kDV + row0 + r];
  };

  // The inputs of the next kDepth tokens are always in flight: one iteration is far shorter
  // than a memory round trip, so a single token of lookahead would leave every iteration
  // waiting for its loads.  Loads are unconditional (clamped to the request's last token).
  struct TokenIn {
    u32x4_t kraw, qraw;
    uint32_t graw, braw, vraw[R];
  };
  TokenIn ring[kDepth];
#pragma unroll
  for (int j = 0; j < kDepth; ++j)
    load_token(min(start + j, end - 1), ring[j].kraw, ring[j].qraw, ring[j].graw, ring[j].braw, ring[j].vraw);
  for (int t0 = start; t0 < end; t0 += kDepth) {
#pragma unroll
    for (int j = 0; j < kDepth; ++j) {
      const int t = t0 + j;
      const TokenIn in = ring[j];
      load_token(min(t + kDepth, end - 1), ring[j].kraw, ring[j].qraw, ring[j].graw, ring[j].braw, ring[j].vraw);
      if (t >= end) break;  // the same for every lane of the workgroup
      float kf[kPerLane], qf[kPerLane];
      unpack8(in.kraw, kf);
      unpack8(in.qraw, qf);
      const float gs = bf16_bits_to_f32(in.graw), bs = bf16_bits_to_f32(in.braw);
      float out[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        // two partial sums per inner product: half the length of the dependent FMA chain
        float dot0 = 0.f, dot1 = 0.f;
#pragma unroll
        for (int e = 0; e < kPerLane; e += 2) {
          s[r][e] *= gs;
          s[r][e + 1] *= gs;
          dot0 = __builtin_fmaf(s[r][e], kf[e], dot0);
          dot1 = __builtin_fmaf(s[r][e + 1], kf[e + 1], dot1);
        }
        const float delta = (bf16_bits_to_f32(in.vraw[r]) - row_sum(dot0 + dot1)) * bs;
        float o0 = 0.f, o1 = 0.f;
#pragma unroll
        for (int e = 0; e < kPerLane; e += 2) {
          s[r][e] = __builtin_fmaf(kf[e], delta, s[r][e]);
          s[r][e + 1] = __builtin_fmaf(kf[e + 1], delta, s[r][e + 1]);
          o0 = __builtin_fmaf(s[r][e], qf[e], o0);
          o1 = __builtin_fmaf(s[r][e + 1], qf[e + 1], o1);
        }
        out[r] = row_sum(o0 + o1);
      }
      // lane r of the group writes row r
      float mine = out[0];
#pragma unroll
      for (int r = 1; r < R; ++r) mine = (lane16 == r) ? out[r] : mine;
      if (lane16 < R)
        p.y[((int64_t)t * p.hv + hv) * kDV + row0 + lane16] = __builtin_bit_cast(uint16_t, (__bf16)mine);
    }
  }

#pragma unroll
  for (int r = 0; r < R; ++r) {
    f32x4_t a, c;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      a[e] = s[r][e];
      c[e] = s[r][4 + e];
    }
    *reinterpret_cast<f32x4_t*>(srow + r * kDK) = a;
    *reinterpret_cast<f32x4_t*>(srow + r * kDK + 4) = c;
  }
}

}  // namespace

static thread_local int t_force_rows = 0;  // benchmarking switch, one value per host thread
void gdn_set_rows(int v) { t_force_rows = (v == 1 || v == 2 || v == 4) ? v : 0; }

int launch_gdn_state(const GdnArgs& a, hipStream_t stream) {
  GdnParams p;
  p.state = static_cast<float*>(a.state);
  p.y = static_cast<uint16_t*>(a.y);
  p.q = static_cast<const uint16_t*>(a.q);
  p.k = static_cast<const uint16_t*>(a.k);
  p.v = static_cast<const uint16_t*>(a.v);
  p.g = static_cast<const uint16_t*>(a.g);
  p.beta = static_cast<const uint16_t*>(a.beta);
  p.slot_ids = a.slot_ids;
  p.qo_indptr = a.qo_indptr;
  p.state_stride0 = a.state_stride0;
  p.q_stride0 = a.q_stride0;
  p.k_stride0 = a.k_stride0;
  p.v_stride0 = a.v_stride0;
  p.batch = (int32_t)a.batch;
  p.hv = (int32_t)a.hv;
  p.hv_per_hk = (int32_t)(a.hv / a.hk);
  p.tokens = (int32_t)a.tokens;
  p.single_token = a.single_token_mode ? 1 : 0;
  const int64_t heads = a.batch * a.hv;
  if (heads <= 0) return MSGL_OK;
  // more rows per lane group (more overlap inside a wave) once there are enough workgroups
  // to fill the chip without it
  const int64_t blocks_r1 = heads * (kDV / 16);
  int r = 1;
  if (blocks_r1 >= 8 * 1024) r = 4;
  else if (blocks_r1 >= 4 * 1024) r = 2;
  if (t_force_rows > 0) r = t_force_rows;
  const int64_t blocks = heads * (kDV / (16 * r));
  if (blocks > 0x7fffffffLL) return MSGL_ERR_SHAPE;
  const dim3 grid((unsigned)blocks), block(256);
  // decode has one token per request: nothing to look ahead to
  if (p.single_token) {
    if (r == 4) hipLaunchKernelGGL((gdn_state_kernel<4, 1>), grid, block, 0, stream, p);
    else if (r == 2) hipLaunchKernelGGL((gdn_state_kernel<2, 1>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((gdn_state_kernel<1, 1>), grid, block, 0, stream, p);
  } else {
    if (r == 4) hipLaunchKernelGGL((gdn_state_kernel<4, 8>), grid, block, 0, stream, p);
    else if (r == 2) hipLaunchKernelGGL((gdn_state_kernel<2, 8>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((gdn_state_kernel<1, 8>), grid, block, 0, stream, p);
  }
  return check_launch();
}

}  // namespace msgl
