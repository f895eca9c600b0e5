// Measurement aid: what rate of v_mfma_f32_32x32x16_bf16 the chip sustains when nothing else runs.
//
// The published dense bf16 peak (32 768 flop per instruction, one instruction per 32 cycles and SIMD
// at the top clock) is a ceiling for smooth operands only: with operands whose bits toggle the way
// random data does, the chip lowers its clock under the load.  The benchmark reports both rates
// beside the attention kernel's, so that its fraction of the published peak can be read against
// what a pure MFMA stream reaches on the same box.
#include "mvpa_common.h"

namespace mvpa {

typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8;
typedef __attribute__((ext_vector_type(16))) float probe_f32x16;

constexpr int PROBE_THREADS = 256, PROBE_MFMA_PER_ITER = 8;

template <bool RANDOM>
__global__ __launch_bounds__(PROBE_THREADS, 2) void mvpa_probe_mfma_kernel(float* sink, int iters) {
  const int lane = threadIdx.x & 63;
  probe_bf16x8 A[8], B[4];
  for (int q = 0; q < 8; ++q)
    for (int i = 0; i < 8; ++i) {
      // RANDOM: a hash of (lane, fragment, element) mapped to [-1, 1); else the same small value in every lane
      uint32_t h = (lane * 2654435761u) ^ (q * 40503u + i * 9973u);
      h ^= h >> 13;
      h *= 0x5bd1e995u;
      h ^= h >> 15;
      const float ra = ((int)(h & 0xffff) - 32768) * (1.f / 32768.f);
      const float rb = ((int)((h >> 8) & 0xffff) - 32768) * (1.f / 32768.f);
      A[q][i] = (__bf16)(RANDOM ? ra : 0.01f * (q + 1));
      if (q < 4) B[q][i] = (__bf16)(RANDOM ? rb : 0.02f * (q + 1));
    }
  probe_f32x16 c[4];
  for (int j = 0; j < 4; ++j)
    for (int i = 0; i < 16; ++i) c[j][i] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int q = 0; q < PROBE_MFMA_PER_ITER; ++q)
      c[q & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A[q], B[q >> 1], c[q & 3], 0, 0, 0);
  }
  float s = 0.f;
  for (int j = 0; j < 4; ++j)
    for (int i = 0; i < 16; ++i) s += c[j][i];
  sink[blockIdx.x * PROBE_THREADS + threadIdx.x] = s;
}

}  // namespace mvpa

extern "C" int64_t mvpa_probe_mfma_flops(int32_t iters) {
  // 512 workgroups of 4 waves (two waves per SIMD on 256 CUs), 8 MFMAs of 32x32x16 per iteration
  return iters <= 0 ? 0 : (int64_t)512 * 4 * mvpa::PROBE_MFMA_PER_ITER * 2 * 32 * 32 * 16 * (int64_t)iters;
}

extern "C" int mvpa_probe_mfma(int32_t random_operands, int32_t iters, float* sink, void* stream) {
  if (!sink) return MVPA_ERR_NULL;
  if (iters <= 0) return MVPA_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (random_operands)
    hipLaunchKernelGGL(mvpa::mvpa_probe_mfma_kernel<true>, dim3(512), dim3(mvpa::PROBE_THREADS), 0, s, sink, iters);
  else
    hipLaunchKernelGGL(mvpa::mvpa_probe_mfma_kernel<false>, dim3(512), dim3(mvpa::PROBE_THREADS), 0, s, sink, iters);
  return hipGetLastError() == hipSuccess ? MVPA_OK : MVPA_ERR_LAUNCH;
}
