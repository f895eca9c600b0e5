// Dense ops around the attention kernel: bf16 MFMA linear (y = x w^T), RMSNorm, the
// three-way residual add and the db4 wavelet analysis of the segment encoder.
#include "mvpa_common.h"

namespace mvpa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// -----------------------------------------------------------------------------------------
// y[M,N] = x[M,K] w[N,K]^T.  Both operands are K-contiguous, which is the layout the
// 32x32x16 bf16 MFMA wants for its A and B fragments (8 consecutive k per lane), so tiles go
// global -> registers -> LDS -> fragments without any transposition.
//   workgroup tile 128 x 128 x 64, 4 waves in a 2x2 grid, 64x64 per wave (2x2 MFMA tiles),
//   LDS double buffered, rows padded by 16 B so the b128 fragment reads spread over banks.
// EPI == 1 fuses the gated MLP: w holds gate rows [0,N) and up rows [N,2N); every wave computes
// 32 gate and the matching 32 up columns in the same lanes and writes silu(gate)*up.
// -----------------------------------------------------------------------------------------
constexpr int GBM = 128, GBN = 128, GBK = 64, GPITCH = GBK + 8;

__device__ inline u32x4 load_chunk(const bf16_t* row, int64_t k, int64_t K, bool row_ok) {
  u32x4 r = {0u, 0u, 0u, 0u};
  if (!row_ok || k >= K) return r;
  if (k + 8 <= K) return *(const u32x4*)(row + k);
  bf16_t tmp[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) tmp[i] = (k + i < K) ? row[k + i] : (bf16_t)0;
  r.x = tmp[0] | ((uint32_t)tmp[1] << 16);
  r.y = tmp[2] | ((uint32_t)tmp[3] << 16);
  r.z = tmp[4] | ((uint32_t)tmp[5] << 16);
  r.w = tmp[6] | ((uint32_t)tmp[7] << 16);
  return r;
}

template <int EPI>
__global__ __launch_bounds__(256) void linear_bf16_kernel(const bf16_t* __restrict__ X,
                                                          const bf16_t* __restrict__ W,
                                                          bf16_t* __restrict__ Y, int64_t M,
                                                          int64_t N, int64_t K, int64_t ldx,
                                                          int64_t ldw, int64_t ldy) {
  __shared__ __attribute__((aligned(16))) bf16_t As[2][GBM * GPITCH];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[2][GBN * GPITCH];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave >> 1, wc = wave & 1;
  const int64_t m0 = (int64_t)blockIdx.y * GBM;
  // output columns owned by this workgroup: 128 plain, 64 when gate/up are fused
  const int64_t n0 = (int64_t)blockIdx.x * (EPI == 1 ? GBN / 2 : GBN);

  // per-thread global chunk assignment: 4 chunks of A and 4 of B per k-tile
  const bf16_t* arow[4];
  const bf16_t* brow[4];
  bool aok[4], bok[4];
  int lds_off[4], kc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = tid + 256 * i;
    const int r = c >> 3;
    kc[i] = (c & 7) * 8;
    lds_off[i] = r * GPITCH + kc[i];
    const int64_t am = m0 + r;
    aok[i] = am < M;
    arow[i] = X + (aok[i] ? am : 0) * ldx;
    int64_t wn;
    if (EPI == 1) {
      const int wcol = r >> 6, nb = (r >> 5) & 1, j = r & 31;
      const int64_t col = n0 + wcol * 32 + j;
      bok[i] = col < N;
      wn = (nb ? N : 0) + col;
    } else {
      wn = n0 + r;
      bok[i] = wn < N;
    }
    brow[i] = W + (bok[i] ? wn : 0) * ldw;
  }

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  u32x4 ra[4], rb[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    ra[i] = load_chunk(arow[i], kc[i], K, aok[i]);
    rb[i] = load_chunk(brow[i], kc[i], K, bok[i]);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    *(u32x4*)(&As[0][lds_off[i]]) = ra[i];
    *(u32x4*)(&Bs[0][lds_off[i]]) = rb[i];
  }
  __syncthreads();

  const int nkt = (int)((K + GBK - 1) / GBK);
  const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;
  for (int kt = 0; kt < nkt; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nkt) {
      const int64_t k0 = (int64_t)(kt + 1) * GBK;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        ra[i] = load_chunk(arow[i], k0 + kc[i], K, aok[i]);
        rb[i] = load_chunk(brow[i], k0 + kc[i], K, bok[i]);
      }
    }
#pragma unroll
    for (int ks = 0; ks < GBK / 16; ++ks) {
      bf16x8 af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        af[i] = *(const bf16x8*)(&As[cur][(wr * 64 + i * 32 + frag_row) * GPITCH + ks * 16 + frag_k]);
        bf[i] = *(const bf16x8*)(&Bs[cur][(wc * 64 + i * 32 + frag_row) * GPITCH + ks * 16 + frag_k]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nkt) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        *(u32x4*)(&As[cur ^ 1][lds_off[i]]) = ra[i];
        *(u32x4*)(&Bs[cur ^ 1][lds_off[i]]) = rb[i];
      }
    }
    __syncthreads();
  }

  // epilogue: lane holds column (lane%32) and rows 8*(r/4) + 4*(lane/32) + r%4 of each tile
  const int col_in = lane & 31, row_half = (lane >> 5) * 4;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int64_t m = m0 + wr * 64 + i * 32 + (r >> 2) * 8 + row_half + (r & 3);
      if (m >= M) continue;
      if (EPI == 1) {
        const int64_t n = n0 + wc * 32 + col_in;
        if (n < N) {
          const float gte = acc[i][0][r], up = acc[i][1][r];
          Y[m * ldy + n] = f32_to_bf16(gte / (1.f + __expf(-gte)) * up);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int64_t n = n0 + wc * 64 + j * 32 + col_in;
          if (n < N) Y[m * ldy + n] = f32_to_bf16(acc[i][j][r]);
        }
      }
    }
  }
}

// -----------------------------------------------------------------------------------------
// RMSNorm: one workgroup per row, fp32 statistics.
// -----------------------------------------------------------------------------------------
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const TI* __restrict__ x,
                                                      const float* __restrict__ w,
                                                      TO* __restrict__ y, int cols, int64_t ldx,
                                                      int64_t ldy, float eps) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const TI* xr = x + row * ldx;
  TO* yr = y + row * ldy;
  float ss = 0.f;
  for (int c = threadIdx.x; c < cols; c += 256) {
    const float v = io<TI>::load(xr + c);
    ss += v * v;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float tot = red[0] + red[1] + red[2] + red[3];
  const float inv = rsqrtf(tot / (float)cols + eps);
  for (int c = threadIdx.x; c < cols; c += 256)
    io<TO>::store(yr + c, io<TI>::load(xr + c) * inv * w[c]);
}

__global__ __launch_bounds__(256) void add3_bf16_kernel(const bf16_t* __restrict__ a,
                                                        const bf16_t* __restrict__ b,
                                                        const bf16_t* __restrict__ c,
                                                        bf16_t* __restrict__ o, int64_t n) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x);
  if (i < n) o[i] = f32_to_bf16(bf16_to_f32(a[i]) + bf16_to_f32(b[i]) + bf16_to_f32(c[i]));
}

// -----------------------------------------------------------------------------------------
// Multilevel db4 analysis with periodic extension: per level
//   lo[k] = sum_j dec_lo[j] * a[(2k+1-j) mod n],  hi[k] likewise,  k < floor((n+7)/2).
// One workgroup per row; the running approximation ping-pongs between two LDS buffers.
// -----------------------------------------------------------------------------------------
__constant__ float kDb4Lo[8] = {-0.010597401784997278f, 0.032883011666982945f,
                                0.030841381835986965f,  -0.18703481171888114f,
                                -0.02798376941698385f,  0.6308807679295904f,
                                0.7148465705525415f,    0.23037781330885523f};

__global__ __launch_bounds__(256) void wavedec_db4_kernel(const float* __restrict__ x,
                                                          float* __restrict__ out, int L,
                                                          int levels, int dwt_size, int64_t ldc) {
  extern __shared__ float buf[];   // 2 * L floats
  float* cur = buf;
  float* nxt = buf + L;
  const int64_t row = blockIdx.x;
  for (int i = threadIdx.x; i < L; i += 256) cur[i] = x[row * L + i];
  __syncthreads();
  // offset of the detail block of level lv (1-based): after cA_L and the deeper details
  int n = L;
  int tail = dwt_size;   // details of level 1 sit at the very end
  for (int lv = 1; lv <= levels; ++lv) {
    const int m = (n + 7) >> 1;
    tail -= m;
    float* det = out + row * ldc + tail;
    for (int k = threadIdx.x; k < m; k += 256) {
      float lo = 0.f, hi = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        int idx = (2 * k + 1 - j) % n;
        if (idx < 0) idx += n;
        const float v = cur[idx];
        lo += kDb4Lo[j] * v;
        // dec_hi[j] = (-1)^(j+1) * dec_lo[7-j]
        hi += ((j & 1) ? kDb4Lo[7 - j] : -kDb4Lo[7 - j]) * v;
      }
      nxt[k] = lo;
      det[k] = hi;
    }
    __syncthreads();
    float* t = cur; cur = nxt; nxt = t;
    n = m;
  }
  for (int k = threadIdx.x; k < n; k += 256) out[row * ldc + k] = cur[k];
}

}  // namespace mvpa

using namespace mvpa;

extern "C" int mvpa_linear_bf16(const void* x, const void* w, void* y, int64_t M, int64_t N,
                                int64_t K, int64_t ldx, int64_t ldw, int64_t ldy,
                                int32_t epilogue, void* stream) {
  if (!x || !w || !y) return MVPA_ERR_NULL;
  if (M <= 0 || N <= 0 || K <= 0 || ldx < K || ldw < K || ldy < N) return MVPA_ERR_SHAPE;
  if (((uintptr_t)x & 15) || ((uintptr_t)w & 15) || (ldx & 7) || (ldw & 7)) return MVPA_ERR_ALIGN;
  if (epilogue != 0 && epilogue != 1) return MVPA_ERR_UNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  if (epilogue == 1) {
    dim3 grid((unsigned)((N + GBN / 2 - 1) / (GBN / 2)), (unsigned)((M + GBM - 1) / GBM));
    hipLaunchKernelGGL(linear_bf16_kernel<1>, grid, dim3(256), 0, s, (const bf16_t*)x,
                       (const bf16_t*)w, (bf16_t*)y, M, N, K, ldx, ldw, ldy);
  } else {
    dim3 grid((unsigned)((N + GBN - 1) / GBN), (unsigned)((M + GBM - 1) / GBM));
    hipLaunchKernelGGL(linear_bf16_kernel<0>, grid, dim3(256), 0, s, (const bf16_t*)x,
                       (const bf16_t*)w, (bf16_t*)y, M, N, K, ldx, ldw, ldy);
  }
  return hipGetLastError() == hipSuccess ? MVPA_OK : MVPA_ERR_LAUNCH;
}

extern "C" int mvpa_rmsnorm(const void* x, const float* weight, void* y, int64_t rows,
                            int32_t cols, int64_t ldx, int64_t ldy, float eps, int32_t in_dtype,
                            int32_t out_dtype, void* stream) {
  if (!x || !weight || !y) return MVPA_ERR_NULL;
  if (rows <= 0 || cols <= 0 || ldx < cols || ldy < cols) return MVPA_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((unsigned)rows), block(256);
  if (in_dtype == MVPA_F32 && out_dtype == MVPA_F32)
    hipLaunchKernelGGL((rmsnorm_kernel<float, float>), grid, block, 0, s, (const float*)x, weight, (float*)y, cols, ldx, ldy, eps);
  else if (in_dtype == MVPA_F32 && out_dtype == MVPA_BF16)
    hipLaunchKernelGGL((rmsnorm_kernel<float, bf16_t>), grid, block, 0, s, (const float*)x, weight, (bf16_t*)y, cols, ldx, ldy, eps);
  else if (in_dtype == MVPA_BF16 && out_dtype == MVPA_BF16)
    hipLaunchKernelGGL((rmsnorm_kernel<bf16_t, bf16_t>), grid, block, 0, s, (const bf16_t*)x, weight, (bf16_t*)y, cols, ldx, ldy, eps);
  else if (in_dtype == MVPA_BF16 && out_dtype == MVPA_F32)
    hipLaunchKernelGGL((rmsnorm_kernel<bf16_t, float>), grid, block, 0, s, (const bf16_t*)x, weight, (float*)y, cols, ldx, ldy, eps);
  else
    return MVPA_ERR_DTYPE;
  return hipGetLastError() == hipSuccess ? MVPA_OK : MVPA_ERR_LAUNCH;
}

extern "C" int mvpa_add3_bf16(const void* a, const void* b, const void* c, void* out, int64_t n,
                              void* stream) {
  if (!a || !b || !c || !out) return MVPA_ERR_NULL;
  if (n <= 0) return MVPA_ERR_SHAPE;
  hipLaunchKernelGGL(add3_bf16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, (const bf16_t*)a, (const bf16_t*)b, (const bf16_t*)c,
                     (bf16_t*)out, n);
  return hipGetLastError() == hipSuccess ? MVPA_OK : MVPA_ERR_LAUNCH;
}

extern "C" int mvpa_wavedec_db4(const float* x, float* coeffs, int64_t M, int32_t L,
                                int32_t levels, int32_t dwt_size, int64_t ldc, void* stream) {
  if (!x || !coeffs) return MVPA_ERR_NULL;
  if (M <= 0 || L < 8 || levels < 1 || L > 16384 || ldc < dwt_size) return MVPA_ERR_SHAPE;
  int n = L, total = 0;
  for (int lv = 0; lv < levels; ++lv) { n = (n + 7) >> 1; total += n; }
  total += n;
  if (total != dwt_size) return MVPA_ERR_SHAPE;
  hipLaunchKernelGGL(wavedec_db4_kernel, dim3((unsigned)M), dim3(256), 2 * L * sizeof(float),
                     (hipStream_t)stream, x, coeffs, L, levels, dwt_size, ldc);
  return hipGetLastError() == hipSuccess ? MVPA_OK : MVPA_ERR_LAUNCH;
}
