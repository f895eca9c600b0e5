// Preparation of the fp8 content term (MVPA_FLAG_FP8_QK): per-head amax scales of (q + u) and of
// k, and the keys rounded to e4m3 once, so that the attention kernel's window steps stream
// one-byte keys and convert nothing.  HBM bound: one pass over q and k for the maxima, one more
// over k for the rounding.
#include "mvpa_mfma_tools.h"

namespace mvpa {

constexpr int FP8_THREADS = 256;

__global__ void fp8_amax_clear_kernel(uint32_t* q_amax, uint32_t* k_amax, int H, int Hkv) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < H) q_amax[i] = 0u;
  if (i < Hkv) k_amax[i] = 0u;
}

// grid (chunks of rows, B * (H + Hkv)): row y of the grid is one (sample, query head) or one
// (sample, kv head).  Magnitudes are non-negative floats, whose order is that of their bit
// patterns, so the per-head maximum is an integer atomic maximum.
__global__ __launch_bounds__(FP8_THREADS) void fp8_amax_kernel(mvpa_fwd_args a, uint32_t* q_amax, uint32_t* k_amax) {
  const int per_b = a.H + a.Hkv;
  const int b = blockIdx.y / per_b, r = blockIdx.y % per_b;
  const bool is_q = r < a.H;
  const int64_t n_all = (int64_t)a.T * a.C;
  const int64_t rows = is_q ? ((a.flags & MVPA_FLAG_LAST_STEP) ? a.C : n_all) : n_all;
  const int cpr = a.Dh / 8;                                   // 16-byte chunks per row
  const int g = is_q ? r / (a.H / a.Hkv) : r - a.H;
  const bf16_t* base = is_q ? (const bf16_t*)a.q + b * a.q_stride_b + r * a.q_stride_h
                            : (const bf16_t*)a.k + b * a.k_stride_b + g * a.k_stride_h;
  const int64_t stride = is_q ? a.q_stride_n : a.k_stride_n;
  const bf16_t* bias = (const bf16_t*)a.bias_u + g * a.Dh;
  float mx = 0.f;
  // a thread keeps one column chunk (and its bias) and walks rows, four loads in flight at a time
  const int tpr = FP8_THREADS / cpr * cpr;                    // threads in use (a whole number of rows)
  const int col = (int)(threadIdx.x % cpr) * 8;
  const int64_t rstep = (int64_t)gridDim.x * (tpr / cpr);
  u32x4 braw = {0u, 0u, 0u, 0u};
  if (is_q) braw = *(const u32x4*)(bias + col);
  auto fold = [&](const u32x4& raw) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float lo = __uint_as_float(raw[i] << 16) + __uint_as_float(braw[i] << 16);
      const float hi = __uint_as_float(raw[i] & 0xffff0000u) + __uint_as_float(braw[i] & 0xffff0000u);
      mx = fmaxf(mx, fmaxf(fabsf(lo), fabsf(hi)));
    }
  };
  if ((int)threadIdx.x < tpr) {
    int64_t row = (int64_t)blockIdx.x * (tpr / cpr) + threadIdx.x / cpr;
    for (; row + 3 * rstep < rows; row += 4 * rstep) {
      const u32x4 r0 = *(const u32x4*)(base + row * stride + col);
      const u32x4 r1 = *(const u32x4*)(base + (row + rstep) * stride + col);
      const u32x4 r2 = *(const u32x4*)(base + (row + 2 * rstep) * stride + col);
      const u32x4 r3 = *(const u32x4*)(base + (row + 3 * rstep) * stride + col);
      fold(r0);
      fold(r1);
      fold(r2);
      fold(r3);
    }
    for (; row < rows; row += rstep) fold(*(const u32x4*)(base + row * stride + col));
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
  if ((threadIdx.x & 63) == 0 && mx > 0.f) atomicMax(is_q ? q_amax + r : k_amax + g, __float_as_uint(mx));
}

__global__ void fp8_scale_kernel(float* q_scale, float* k_scale, int H, int Hkv, float q_mul) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < H) q_scale[i] = fmaxf(q_scale[i] * q_mul, 1e-20f);
  if (i < Hkv) k_scale[i] = fmaxf(k_scale[i] / 224.0f, 1e-20f);
}

// k8[b][g][n][d] = e4m3(k[b][g][n][d] / k_scale[g]); a lane takes 8 elements.
__global__ __launch_bounds__(FP8_THREADS) void fp8_round_keys_kernel(mvpa_fwd_args a, const float* k_scale, uint8_t* k8) {
  const int b = blockIdx.y / a.Hkv, g = blockIdx.y % a.Hkv;
  const int64_t rows = (int64_t)a.T * a.C;
  const int cpr = a.Dh / 8;
  const bf16_t* base = (const bf16_t*)a.k + b * a.k_stride_b + g * a.k_stride_h;
  uint8_t* out = k8 + ((int64_t)b * a.Hkv + g) * rows * a.Dh;
  const float inv = 1.f / k_scale[g];
  for (int64_t c = (int64_t)blockIdx.x * FP8_THREADS + threadIdx.x; c < rows * cpr;
       c += (int64_t)gridDim.x * FP8_THREADS) {
    const int64_t row = c / cpr;
    const int col = (int)(c % cpr) * 8;
    const u32x4 raw = *(const u32x4*)(base + row * a.k_stride_n + col);
    *(long*)(out + row * a.Dh + col) = kfrag_fp8(raw, inv);
  }
}

}  // namespace mvpa

extern "C" int mvpa_fp8_prepare(const mvpa_fwd_args* a, float* q_scale, float* k_scale, void* k_fp8, void* stream) {
  using namespace mvpa;
  if (!a || !q_scale || !k_scale) return MVPA_ERR_NULL;
  if (a->struct_size != sizeof(mvpa_fwd_args)) return MVPA_ERR_STRUCT;
  if (a->dtype != MVPA_BF16) return MVPA_ERR_UNSUPPORTED;
  if (a->Dh != 16 && a->Dh != 32 && a->Dh != 64 && a->Dh != 128) return MVPA_ERR_HEAD_DIM;
  if (a->B <= 0 || a->H <= 0 || a->Hkv <= 0) return MVPA_ERR_SHAPE;
  if (a->H % a->Hkv != 0) return MVPA_ERR_HEAD_RATIO;
  if (a->T <= 0 || a->C <= 0) return MVPA_ERR_CTX;
  if (!a->q || !a->k || !a->bias_u) return MVPA_ERR_NULL;
  const uintptr_t p = (uintptr_t)a->q | (uintptr_t)a->k | (uintptr_t)a->bias_u | (uintptr_t)k_fp8;
  const int64_t s = a->q_stride_b | a->q_stride_h | a->q_stride_n | a->k_stride_b | a->k_stride_h | a->k_stride_n;
  if ((p & 15) || (s & 7)) return MVPA_ERR_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const int64_t rows = (int64_t)a->T * a->C;
  const int heads = a->H > a->Hkv ? a->H : a->Hkv;
  uint32_t* qa = (uint32_t*)q_scale;
  uint32_t* ka = (uint32_t*)k_scale;
  MVPA_LAUNCH(fp8_amax_clear_kernel, dim3((unsigned)((heads + 255) / 256)), dim3(256), 0, st, qa, ka, a->H, a->Hkv);
  // enough workgroups per head to fill the chip, at least 2048 chunks each
  const int64_t chunks = rows * (a->Dh / 8);
  int64_t gx = (chunks + 2047) / 2048;
  const int64_t want = 2048 / ((int64_t)a->B * (a->H + a->Hkv)) + 1;
  if (gx > want) gx = want;
  if (gx < 1) gx = 1;
  MVPA_LAUNCH(fp8_amax_kernel, dim3((unsigned)gx, (unsigned)(a->B * (a->H + a->Hkv))), dim3(FP8_THREADS), 0, st, *a, qa, ka);
  const float q_mul = (float)((double)a->sm_scale * 1.4426950408889634 / 224.0);
  MVPA_LAUNCH(fp8_scale_kernel, dim3((unsigned)((heads + 255) / 256)), dim3(256), 0, st, q_scale, k_scale, a->H, a->Hkv, q_mul);
  if (k_fp8) {
    int64_t gk = (chunks + 1023) / 1024;
    const int64_t want_k = 4096 / ((int64_t)a->B * a->Hkv) + 1;
    if (gk > want_k) gk = want_k;
    MVPA_LAUNCH(fp8_round_keys_kernel, dim3((unsigned)gk, (unsigned)(a->B * a->Hkv)), dim3(FP8_THREADS), 0, st, *a,
                (const float*)k_scale, (uint8_t*)k_fp8);
  }
  return mvpa::take_launch_status();
}
