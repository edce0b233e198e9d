// Bench-only probe, not part of the product library: what the matrix cores of the
// current device sustain on back-to-back MFMAs (the clock, and with it the rate,
// depends on how much the operands toggle), for bench.py to print beside the
// published peak.  Built into bench_probe/libmfma_probe.so (bench_probe/build.py).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../mmcv_amd/csrc/mdcn_fused.h"

namespace mdcn {

// Back-to-back MFMAs on eight accumulator blocks per wave (the consumers' block
// shape), operands from `in` (4096 32-bit words) or zeros: what the matrix cores
// sustain, for the bench to put beside the published peak.
template <typename E>
__global__ __launch_bounds__(256) void mfma_probe_kernel(const uint4 *__restrict__ in, float *out, int iters, int zero) {
  using TR = ElemTraits<E>;
  const int tid = threadIdx.x;
  uint4 a[2], b[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) a[i] = zero ? make_uint4(0u, 0u, 0u, 0u) : in[(tid * 7 + i * 13) & 1023];
#pragma unroll
  for (int i = 0; i < 4; ++i) b[i] = zero ? make_uint4(0u, 0u, 0u, 0u) : in[(tid * 5 + i * 29 + 100) & 1023];
  f32x16 acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) TR::mma(acc[i][j], a[i], b[j]);
    if (!zero) {  // keep the operands changing
      a[0].x ^= (uint32_t)it;
      b[1].y += 0x00010001u;
    }
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += acc[i][j][r];
  if (s == 1.2345f) out[tid] = s;  // (never: keeps the loop alive)
}

}  // namespace mdcn

using namespace mdcn;

// Every CU runs `waves_per_simd` (1 or 2) wavefronts of back-to-back 32x32x16 MFMAs
// (dtype 2 = bf16, 1 = fp16) on pseudo-random operands, or on zeros with
// `zero_data` != 0.  Launches on `hip_stream`, waits for it and stores TFLOP/s in
// *tflops.  Uses `scratch`, at least 16 KiB of device memory.  Returns 0 or a
// negative status.
extern "C" int mdcn_mfma_probe(int dtype, int waves_per_simd, int zero_data, void *scratch, void *hip_stream, float *tflops) {
  if (!scratch || !tflops) return -1;
  if (dtype != 2 && dtype != 1) return -3;
  if (waves_per_simd < 1 || waves_per_simd > 2) return -2;
  hipStream_t st = (hipStream_t)hip_stream;
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
  // operands: 4096 words of two 16-bit values of magnitude 0.5 .. 2 with random signs and
  // mantissas (finite in both formats)
  uint32_t host[4096];
  uint32_t rng = 12345u;
  auto next = [&]() { rng = rng * 1664525u + 1013904223u; return rng >> 8; };
  const uint32_t base = dtype == 2 ? 0x3f00u : 0x3800u;
  for (int i = 0; i < 4096; ++i) {
    const uint32_t lo = base + (next() & 0xffu) + ((next() & 1u) << 15);
    const uint32_t hi = base + (next() & 0xffu) + ((next() & 1u) << 15);
    host[i] = lo | (hi << 16);
  }
  if (hipMemcpyAsync(scratch, host, sizeof(host), hipMemcpyHostToDevice, st) != hipSuccess) return -7;
  if (hipStreamSynchronize(st) != hipSuccess) return -7;
  const int blocks = cus * waves_per_simd, iters = 20000;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return -7;
  auto launch = [&](int n) {
    if (dtype == 2)
      hipLaunchKernelGGL(mfma_probe_kernel<bf16_t>, dim3(blocks), dim3(256), 0, st, (const uint4 *)scratch,
                         (float *)scratch, n, zero_data);
    else
      hipLaunchKernelGGL(mfma_probe_kernel<f16_t>, dim3(blocks), dim3(256), 0, st, (const uint4 *)scratch,
                         (float *)scratch, n, zero_data);
  };
  launch(2000);  // warm up (clocks)
  int rc = 0;
  if (hipEventRecord(e0, st) != hipSuccess) rc = -7;
  launch(iters);
  if (hipEventRecord(e1, st) != hipSuccess) rc = -7;
  float ms = 0.0f;
  if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess ||
      hipGetLastError() != hipSuccess || ms <= 0.0f)
    rc = -7;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc == 0) *tflops = (float)((double)blocks * 4 * iters * 8 * 32768.0 / ms / 1e9);
  return rc;
}

