// Device-side building blocks shared by the gfx950 paged-attention kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace msgl {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegInf = -__builtin_inff();

// 16-byte global load / store of 8 bf16 (one lane's MFMA operand slice).
__device__ __forceinline__ u32x4_t ld_global_b128(const void* p) {
  return *reinterpret_cast<const u32x4_t*>(p);
}
__device__ __forceinline__ void st_global_b128(void* p, u32x4_t v) {
  *reinterpret_cast<u32x4_t*>(p) = v;
}

__device__ __forceinline__ bf16x8_t as_bf16x8(u32x4_t v) {
  return __builtin_bit_cast(bf16x8_t, v);
}

// Two fp32 -> packed bf16x2 (round to nearest even); lowers to v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2_t p;
  p[0] = (__bf16)lo;
  p[1] = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, p);
}

// Optimisation barrier on one register value: it must be computed before this point and
// is treated as modified after it.
__device__ __forceinline__ void pin(float& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void pin(uint32_t& x) { asm volatile("" : "+v"(x)); }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// v_perm_b32: result byte i = byte sel[i] of the 8-byte value {hi:lo} (lo = bytes 0..3).
__device__ __forceinline__ uint32_t perm_b32(uint32_t hi, uint32_t lo, uint32_t sel) {
  return __builtin_amdgcn_perm(hi, lo, sel);
}
// {a.lo16, b.lo16} and {a.hi16, b.hi16}: the two halves of a 2x2 transpose of 16-bit lanes.
__device__ __forceinline__ uint32_t pack_lo16(uint32_t a, uint32_t b) {
  return perm_b32(b, a, 0x05040100u);
}
__device__ __forceinline__ uint32_t pack_hi16(uint32_t a, uint32_t b) {
  return perm_b32(b, a, 0x07060302u);
}

// D(16x16 f32) += A(16x32 bf16) * B(32x16 bf16).
//   A: lane l holds A[l%16][8*(l/16) .. +8]      B: lane l holds B[8*(l/16) .. +8][l%16]
//   D: lane l holds D[4*(l/16) + i][l%16], i = 0..3
__device__ __forceinline__ f32x4_t mfma_16x16x32(bf16x8_t a, bf16x8_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
// D(32x32 f32) += A(32x16 bf16) * B(16x32 bf16).
//   A: lane l holds A[l%32][8*(l/32) .. +8]      B: lane l holds B[8*(l/32) .. +8][l%32]
//   D: lane l holds D[8*(i/4) + 4*(l/32) + i%4][l%32], i = 0..15
__device__ __forceinline__ f32x16_t mfma_32x32x16(bf16x8_t a, bf16x8_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// The same product on raw 16-bit operands: bf16 or, with F16, IEEE half.
template <bool F16>
__device__ __forceinline__ f32x4_t mfma_16x16x32_raw(u32x4_t a, u32x4_t b, f32x4_t c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  else
    return mfma_16x16x32(as_bf16x8(a), as_bf16x8(b), c);
}
// Two fp32 -> packed 16-bit pair, round to nearest even.
template <bool F16>
__device__ __forceinline__ uint32_t pack_16x2(float lo, float hi) {
  if constexpr (F16) {
    f16x2_t p;
    p[0] = (_Float16)lo;
    p[1] = (_Float16)hi;
    return __builtin_bit_cast(uint32_t, p);
  } else {
    return pack_bf16x2(lo, hi);
  }
}

__device__ __forceinline__ float wave_max_xor(float v, int mask) {
  return fmaxf(v, __shfl_xor(v, mask, kWave));
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Measurement aid: when `dst` is given, thread 0 of workgroup 0 leaves the shader cycles and the
// 100 MHz wall ticks between its construction and its destruction (every way out of the kernel) in
// dst[0], dst[1]: cycles / ticks x 0.1 is the shader clock in GHz while the kernel ran.  (Both
// counters are read by the same wave: the cycle counters of different compute units are unrelated.)
struct ClockProbe {
  long long* dst;
  long long c0, w0;
  __device__ __forceinline__ explicit ClockProbe(long long* d)
      : dst((d != nullptr && blockIdx.x == 0 && threadIdx.x == 0) ? d : nullptr), c0(0), w0(0) {
    if (dst != nullptr) {
      c0 = clock64();
      w0 = wall_clock64();
    }
  }
  __device__ __forceinline__ ~ClockProbe() {
    if (dst != nullptr) {
      dst[0] = clock64() - c0;
      dst[1] = wall_clock64() - w0;
    }
  }
};

// Inclusive prefix sum over the 64 lanes of a wave.
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  const int lane = lane_id();
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int n = __shfl_up(v, off, kWave);
    if (lane >= off) v += n;
  }
  return v;
}

}  // namespace msgl
