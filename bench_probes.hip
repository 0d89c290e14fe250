// Measurements that bench.py reports beside the attention figures; benchmarking aids, built
// into bench_probes.so beside bench.py, not part of the paged-attention library.
//
// (1) What the matrix pipe sustains on this board when nothing else runs: back-to-back
// v_mfma_f32_32x32x16_bf16 on register-resident operands, one workgroup of four waves per CU.
// The board holds a power limit by lowering the shader clock, and MFMA power depends on how
// many operand bits toggle, so the rate is measured for all-zero operands and for operands
// drawn from N(0,1) that change with every instruction.  The second figure is the ceiling a
// bf16 attention kernel on random data is measured against; the datasheet peak assumes the
// boost clock.  A third run feeds the A operand of every instruction from LDS.
//
// (2) What a plain streaming read sustains: every lane reads 16 bytes per load, consecutive
// lanes consecutive addresses, a grid-stride loop over a buffer far larger than the 256 MB
// Infinity Cache, eight loads in flight per lane.  The HBM-bound attention kernels are read
// beside this figure as well as beside the datasheet's 8 TB/s.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

__device__ uint32_t mix(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}
// roughly N(0,1): centred sum of four uniforms
__device__ float draw(uint32_t seed) {
  float s = 0.f;
  for (int i = 0; i < 4; ++i) {
    seed = mix(seed + i * 0x9e3779b9U);
    s += (seed >> 8) * (1.0f / 16777216.0f);
  }
  return (s - 2.0f) * 1.7320508f;
}

__global__ __launch_bounds__(256) void mfma_rate_kernel(int random_operands, int iters, float* sink,
                                                        long long* clocks) {
  f32x16_t acc[4];
  for (int a = 0; a < 4; ++a)
    for (int i = 0; i < 16; ++i) acc[a][i] = 0.f;
  bf16x8_t av[8], bv[8];
  const uint32_t tid = blockIdx.x * 256 + threadIdx.x;
  for (int r = 0; r < 8; ++r)
    for (int i = 0; i < 8; ++i) {
      av[r][i] = (__bf16)(random_operands ? draw(tid * 131 + r * 17 + i) : 0.f);
      bv[r][i] = (__bf16)(random_operands ? draw(tid * 257 + r * 29 + i + 1000) : 0.f);
    }
  const long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 8; ++r)
      acc[r & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[r], bv[r], acc[r & 3], 0, 0, 0);
    if ((it & 255) == 255)  // keep the sums finite
      for (int a = 0; a < 4; ++a)
        for (int i = 0; i < 16; ++i) acc[a][i] *= 1e-3f;
  }
  const long long c1 = clock64(), w1 = wall_clock64();
  float s = 0.f;
  for (int a = 0; a < 4; ++a)
    for (int i = 0; i < 16; ++i) s += acc[a][i];
  sink[tid] = s;
  if (threadIdx.x == 0) {
    clocks[blockIdx.x * 2] = c1 - c0;
    clocks[blockIdx.x * 2 + 1] = w1 - w0;
  }
}

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// The same stream with the A operand of every MFMA read from LDS (16 bytes per lane, 1 KB per
// instruction, conflict-free), the way an attention kernel receives its K and V tiles: what the
// matrix pipe sustains when operand delivery draws from the same power budget.  Eight waves per CU
// (two per SIMD, as in the extend kernel): one wave's LDS latency hides behind the other's MFMAs.
__global__ __launch_bounds__(512) void mfma_lds_rate_kernel(int iters, float* sink, long long* clocks) {
  __shared__ __attribute__((aligned(16))) u32x4_t tiles[8 * 16 * 64];  // 128 KB: 16 operands per wave
  f32x16_t acc[4];
  for (int a = 0; a < 4; ++a)
    for (int i = 0; i < 16; ++i) acc[a][i] = 0.f;
  bf16x8_t bv[8];
  const uint32_t tid = blockIdx.x * 512 + threadIdx.x;
  for (int r = 0; r < 8; ++r)
    for (int i = 0; i < 8; ++i) bv[r][i] = (__bf16)draw(tid * 257 + r * 29 + i + 1000);
  for (int t = threadIdx.x; t < 8 * 16 * 64; t += 512) {
    bf16x8_t v;
    for (int i = 0; i < 8; ++i) v[i] = (__bf16)draw((blockIdx.x * 8192 + t) * 131 + i);
    tiles[t] = __builtin_bit_cast(u32x4_t, v);
  }
  __syncthreads();
  const u32x4_t* mine = tiles + (threadIdx.x >> 6) * (16 * 64) + (threadIdx.x & 63);
  const long long c0 = clock64(), w0 = wall_clock64();
  // the operands of one iteration are requested while the MFMAs of the one before run
  bf16x8_t av[2][8];
#pragma unroll
  for (int r = 0; r < 8; ++r) av[0][r] = __builtin_bit_cast(bf16x8_t, mine[r * 64]);
  for (int it = 0; it < iters; it += 2) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int r = 0; r < 8; ++r) av[half ^ 1][r] = __builtin_bit_cast(bf16x8_t, mine[((half ^ 1) * 8 + r) * 64]);
#pragma unroll
      for (int r = 0; r < 8; ++r)
        acc[r & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[half][r], bv[r], acc[r & 3], 0, 0, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);  // the 8 LDS reads first
      __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);  // then the 8 MFMAs
      __builtin_amdgcn_sched_barrier(0);
    }
    if ((it & 255) == 254)  // keep the sums finite
      for (int a = 0; a < 4; ++a)
        for (int i = 0; i < 16; ++i) acc[a][i] *= 1e-3f;
  }
  const long long c1 = clock64(), w1 = wall_clock64();
  float s = 0.f;
  for (int a = 0; a < 4; ++a)
    for (int i = 0; i < 16; ++i) s += acc[a][i];
  sink[tid] = s;
  if (threadIdx.x == 0) {
    clocks[blockIdx.x * 2] = c1 - c0;
    clocks[blockIdx.x * 2 + 1] = w1 - w0;
  }
}

__global__ __launch_bounds__(256) void hbm_read_kernel(const u32x4_t* __restrict__ src, size_t n_vec,
                                                       uint32_t* sink) {
  const size_t stride = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  u32x4_t acc = {0u, 0u, 0u, 0u};
  for (; i + 7 * stride < n_vec; i += 8 * stride) {
    u32x4_t v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u];
  }
  for (; i < n_vec; i += stride) acc ^= __builtin_nontemporal_load(src + i);
  const uint32_t x = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  if (x == 0x9e3779b9u) sink[0] = x;  // never true for the fill pattern; keeps the loads alive
}

// (3) Rates behind the kernels' schedules, in shader cycles counted by one workgroup per launch:
// what LDS delivers per CU and clock to eight waves that do nothing but read (16-byte reads, and
// the transposing 8-byte reads that feed V to the matrix pipe, in the extend kernels' address
// pattern), and how a wave's VALU work shares the issue port with its MFMAs (one MFMA followed by
// K independent v_fma_f32, one or two waves per SIMD).
typedef short s16x4_t __attribute__((ext_vector_type(4)));
#define PROBE_LDS(T, a) ((__attribute__((address_space(3))) T*)(uintptr_t)(a))
template <int MODE>  // 0: ds_read_b128, consecutive lanes consecutive; 1: ds_read_b64_tr_b16
__global__ __launch_bounds__(512) void lds_rate_kernel(long long* out, uint32_t* sink, int iters) {
  __shared__ __attribute__((aligned(16))) unsigned char tile[65536];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < 65536 / 4; i += 512) reinterpret_cast<uint32_t*>(tile)[i] = mix(i);
  __syncthreads();
  uint32_t addr = (uint32_t)(uintptr_t)PROBE_LDS(unsigned char, tile);
  if (MODE == 0) addr += lane * 16 + w * 1024;
  else addr += ((lane & 15) >> 2) * 1088 + ((lane >> 4) & 1) * 32 + (lane & 3) * 8 + (lane >> 5) * 4 * 1088 + w * 64;
  u32x4_t acc = {0u, 0u, 0u, 0u};
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (MODE == 1) {
        const s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(PROBE_LDS(s16x4_t, addr + u * 64));
        acc[0] ^= (uint32_t)v[0];
        acc[1] ^= (uint32_t)v[2];
      } else {
        u32x4_t v;  // (through asm: a plain read of a loop-invariant address would be hoisted)
        asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr + u * 32) : "memory");
        asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(v));
        acc ^= v;
      }
    }
  }
  const long long t1 = clock64();
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) sink[0] = acc[0];
  if ((threadIdx.x & 63) == 0 && blockIdx.x == 0) {  // per wave: see issue_rate_kernel
    out[2 * w] = t0;
    out[2 * w + 1] = t1;
  }
}

template <int K, int WAVES, int E = 0>  // E: v_exp_f32 per MFMA beside the K v_fma_f32
__global__ __launch_bounds__(WAVES * 64) void issue_rate_kernel(long long* out, float* sink, int iters) {
  f32x16_t acc[4];
  for (int a = 0; a < 4; ++a)
    for (int i = 0; i < 16; ++i) acc[a][i] = 0.f;
  bf16x8_t av, bv;
  for (int i = 0; i < 8; ++i) {
    av[i] = (__bf16)(threadIdx.x * 0.001f + i);
    bv[i] = (__bf16)(i * 0.5f - threadIdx.x * 0.002f);
  }
  float f[8];
  for (int i = 0; i < 8; ++i) f[i] = threadIdx.x + i;
  const float m = 1.0001f, c = 0.5f;
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc[a], 0, 0, 0);
#pragma unroll
      for (int j = 0; j < K; ++j) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(f[j & 7]) : "v"(m), "v"(c));
#pragma unroll
      for (int j = 0; j < E; ++j) asm volatile("v_exp_f32 %0, %0" : "+v"(f[(j + 5) & 7]));
    }
  }
  const long long t1 = clock64();
  float s = 0.f;
  for (int a = 0; a < 4; ++a)
    for (int i = 0; i < 16; ++i) s += acc[a][i];
  for (int i = 0; i < 8; ++i) s += f[i];
  sink[blockIdx.x * WAVES * 64 + threadIdx.x] = s;
  // every wave of workgroup 0 leaves its own start and end: with two waves on a SIMD the older
  // one wins the arbitration and runs at the rate of a lone wave, so one wave's time says nothing
  if ((threadIdx.x & 63) == 0 && blockIdx.x == 0) {
    out[2 * (threadIdx.x >> 6)] = t0;
    out[2 * (threadIdx.x >> 6) + 1] = t1;
  }
}

}  // namespace

// Runs the probes of (3) on the current device (blocking).  out[0], out[1]: LDS bytes per clock and
// CU for ds_read_b128 and ds_read_b64_tr_b16; out[2..5]: cycles per MFMA and SIMD with K = 0, 4, 8,
// 16 v_fma_f32 behind each MFMA, one wave per SIMD; out[6..8]: the same with K = 0, 8, 16, two
// waves per SIMD (from the first start to the last end of the workgroup's waves, per MFMA of one
// SIMD); out[9]: two waves per SIMD, four v_fma_f32 and one v_exp_f32 per MFMA, the extend kernel's
// mix.  n_out must be at least 10.  Returns 0 or a hipError_t value.
extern "C" __attribute__((visibility("default"))) int msgl_probe_issue_rates(double* out, int n_out) {
  if (!out || n_out < 10) return (int)hipErrorInvalidValue;
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return (int)e;
  long long* clk = nullptr;
  float* sink = nullptr;
  e = hipMalloc(&clk, 16 * sizeof(long long));
  if (e != hipSuccess) return (int)e;
  e = hipMalloc(&sink, (size_t)cus * 512 * sizeof(float));
  if (e != hipSuccess) {
    (void)hipFree(clk);
    return (int)e;
  }
  auto span = [&](int waves) {  // first start to last end over the waves of workgroup 0
    long long h[16] = {0};
    if (hipDeviceSynchronize() != hipSuccess) return 0.0;
    (void)hipMemcpy(h, clk, sizeof(h), hipMemcpyDeviceToHost);
    long long lo = h[0], hi = h[1];
    for (int w = 1; w < waves; ++w) {
      lo = h[2 * w] < lo ? h[2 * w] : lo;
      hi = h[2 * w + 1] > hi ? h[2 * w + 1] : hi;
    }
    return (double)(hi - lo);
  };
  const int lds_iters = 2000, mfma_iters = 20000;
  const dim3 grid((unsigned)cus);
  for (int rep = 0; rep < 2; ++rep)  // the second launch is the one read
    hipLaunchKernelGGL((lds_rate_kernel<0>), grid, dim3(512), 0, 0, clk, (uint32_t*)sink, lds_iters);
  out[0] = 8.0 * lds_iters * 8 * 1024 / span(8);
  for (int rep = 0; rep < 2; ++rep)
    hipLaunchKernelGGL((lds_rate_kernel<1>), grid, dim3(512), 0, 0, clk, (uint32_t*)sink, lds_iters);
  out[1] = 8.0 * lds_iters * 8 * 512 / span(8);
#define MSGL_ISSUE_PROBE(slot, K, WAVES)                                                            \
  for (int rep = 0; rep < 2; ++rep)                                                                 \
    hipLaunchKernelGGL((issue_rate_kernel<K, WAVES>), grid, dim3(WAVES * 64), 0, 0, clk, sink, mfma_iters); \
  out[slot] = span(WAVES) / (mfma_iters * 4.0 * (WAVES / 4));
  MSGL_ISSUE_PROBE(2, 0, 4)
  MSGL_ISSUE_PROBE(3, 4, 4)
  MSGL_ISSUE_PROBE(4, 8, 4)
  MSGL_ISSUE_PROBE(5, 16, 4)
  MSGL_ISSUE_PROBE(6, 0, 8)
  MSGL_ISSUE_PROBE(7, 8, 8)
  MSGL_ISSUE_PROBE(8, 16, 8)
#undef MSGL_ISSUE_PROBE
  for (int rep = 0; rep < 2; ++rep)
    hipLaunchKernelGGL((issue_rate_kernel<4, 8, 1>), grid, dim3(512), 0, 0, clk, sink, mfma_iters);
  out[9] = span(8) / (mfma_iters * 4.0 * 2);
  e = hipGetLastError();
  (void)hipFree(clk);
  (void)hipFree(sink);
  return (int)e;
}

// Reads `bytes` (a multiple of 16; at least 1 GiB is sensible) `reps` times and reports the best
// and the mean rate in TB/s.  Blocking; allocates and frees its own buffer.  Returns 0 or a
// hipError_t value.
extern "C" __attribute__((visibility("default"))) int msgl_probe_hbm_read(size_t bytes, int reps,
                                                                        double* best_tbps,
                                                                        double* mean_tbps) {
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return (int)e;
  if (reps < 1 || bytes < 16) return (int)hipErrorInvalidValue;
  void* buf = nullptr;
  uint32_t* sink = nullptr;
  e = hipMalloc(&buf, bytes);
  if (e != hipSuccess) return (int)e;
  e = hipMalloc(&sink, 4);
  if (e != hipSuccess) {
    (void)hipFree(buf);
    return (int)e;
  }
  (void)hipMemset(buf, 0x5a, bytes);
  const size_t n_vec = bytes / 16;
  const dim3 grid((unsigned)(cus * 8)), block(256);
  hipEvent_t t0, t1;
  (void)hipEventCreate(&t0);
  (void)hipEventCreate(&t1);
  hipLaunchKernelGGL(hbm_read_kernel, grid, block, 0, 0, (const u32x4_t*)buf, n_vec, sink);
  double best = 0.0, total_ms = 0.0;
  for (int r = 0; r < reps; ++r) {
    (void)hipEventRecord(t0, 0);
    hipLaunchKernelGGL(hbm_read_kernel, grid, block, 0, 0, (const u32x4_t*)buf, n_vec, sink);
    (void)hipEventRecord(t1, 0);
    e = hipEventSynchronize(t1);
    if (e != hipSuccess) break;
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, t0, t1);
    total_ms += ms;
    const double rate = (double)bytes / (ms * 1e-3) / 1e12;
    if (rate > best) best = rate;
  }
  *best_tbps = best;
  *mean_tbps = total_ms > 0.0 ? (double)bytes * reps / (total_ms * 1e-3) / 1e12 : 0.0;
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  (void)hipFree(buf);
  (void)hipFree(sink);
  return (int)e;
}

// Runs the probe on the current device (blocking).  random_operands: 0 all-zero operands in
// registers, 1 random operands in registers, 2 random operands with A read from LDS for every
// instruction.  tflops: achieved MFMA rate; shader_ghz:
// shader clock during the run (cycle counter against the 100 MHz wall counter).
// Returns 0, or a hipError_t value.
extern "C" __attribute__((visibility("default"))) int msgl_probe_mfma_rate(int random_operands,
                                                                         int iters, double* tflops,
                                                                         double* shader_ghz) {
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return (int)e;
  float* sink = nullptr;
  long long* clocks = nullptr;
  e = hipMalloc(&sink, (size_t)cus * 512 * sizeof(float));
  if (e != hipSuccess) return (int)e;
  e = hipMalloc(&clocks, (size_t)cus * 2 * sizeof(long long));
  if (e != hipSuccess) {
    (void)hipFree(sink);
    return (int)e;
  }
  hipEvent_t t0, t1;
  (void)hipEventCreate(&t0);
  (void)hipEventCreate(&t1);
  if (random_operands == 2) {  // random operands, A through LDS
    iters /= 2;  // eight waves per CU share the pipe
    hipLaunchKernelGGL(mfma_lds_rate_kernel, dim3(cus), dim3(512), 0, 0, iters / 10 + 1, sink, clocks);
    (void)hipEventRecord(t0, 0);
    hipLaunchKernelGGL(mfma_lds_rate_kernel, dim3(cus), dim3(512), 0, 0, iters, sink, clocks);
    (void)hipEventRecord(t1, 0);
  } else {
    hipLaunchKernelGGL(mfma_rate_kernel, dim3(cus), dim3(256), 0, 0, random_operands, iters / 10 + 1, sink, clocks);
    (void)hipEventRecord(t0, 0);
    hipLaunchKernelGGL(mfma_rate_kernel, dim3(cus), dim3(256), 0, 0, random_operands, iters, sink, clocks);
    (void)hipEventRecord(t1, 0);
  }
  e = hipEventSynchronize(t1);
  float ms = 0.f;
  (void)hipEventElapsedTime(&ms, t0, t1);
  long long c[2] = {0, 1};
  (void)hipMemcpy(c, clocks, sizeof(c), hipMemcpyDeviceToHost);
  const double waves = random_operands == 2 ? 8.0 : 4.0;
  *tflops = (double)cus * waves * iters * 8.0 * 32768.0 / (ms * 1e-3) / 1e12;
  *shader_ghz = (double)c[0] / (double)c[1] * 0.1;
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  (void)hipFree(sink);
  (void)hipFree(clocks);
  return (int)e;
}
