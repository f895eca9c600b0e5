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
// Skinny variant for at most 128 rows of x (one decoding step: a time step of C <= 128 channels):
// the work is reading w once, so it is spread over as many workgroups as there are 32-column
// slices of the output, and inside a workgroup over 8 waves that split K (wave v takes the
// 16-wide k-steps v, v+8, ...).  Fragments go from global memory straight into the MFMA operands
// (A = 32 rows of w, B = 32 rows of x, so a lane owns one x row and 4 consecutive output columns
// per accumulator quad), several k-steps are requested before the first is used, and the 8
// partial tiles are summed through LDS.  XT = 32-row tiles of x (2 or 4).  EPI == 1: gate rows n
// and up rows N + n of w side by side.
// -----------------------------------------------------------------------------------------
constexpr int SK_WAVES = 8;

__device__ inline bf16x8 chunk_as_bf16x8(u32x4 v) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = v;
  return c.b;
}

template <int EPI, int XT>
__global__ __launch_bounds__(SK_WAVES * 64) void linear_bf16_skinny_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, bf16_t* __restrict__ Y, int64_t M,
    int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldy) {
  constexpr int NA = EPI == 1 ? 2 : 1;            // w tiles per workgroup (gate, up)
  constexpr int UNROLL = XT == 2 ? 8 : 4;         // k-steps in flight per wave
  extern __shared__ __attribute__((aligned(16))) float sk_red[];   // [SK_WAVES][XT][16][64]
  const int tid = threadIdx.x, lane = tid & 63, ln = lane & 31, hh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t n0 = (int64_t)blockIdx.x * 32;
  const int xt_live = (int)((M + 31) / 32);       // tiles of x rows in use

  const bf16_t* wrow[NA];
  bool wok[NA];
#pragma unroll
  for (int a = 0; a < NA; ++a) {
    const int64_t n = n0 + ln;
    wok[a] = n < N;
    wrow[a] = W + ((wok[a] ? n : 0) + (a ? N : 0)) * ldw;
  }
  const bf16_t* xrow[XT];
  bool xok[XT];
#pragma unroll
  for (int t = 0; t < XT; ++t) {
    const int64_t m = t * 32 + ln;
    xok[t] = m < M;
    xrow[t] = X + (xok[t] ? m : 0) * ldx;
  }

  f32x16 acc[NA][XT];
#pragma unroll
  for (int a = 0; a < NA; ++a)
#pragma unroll
    for (int t = 0; t < XT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][t][r] = 0.f;

  const int nks = (int)((K + 15) / 16);
  for (int s0 = wave; s0 < nks; s0 += SK_WAVES * UNROLL) {
    u32x4 wf[UNROLL][NA], xf[UNROLL][XT];
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
      const int64_t k = (int64_t)(s0 + j * SK_WAVES) * 16 + hh * 8;     // past K: zeros
#pragma unroll
      for (int a = 0; a < NA; ++a) wf[j][a] = load_chunk(wrow[a], k, K, wok[a]);
#pragma unroll
      for (int t = 0; t < XT; ++t)
        if (t < xt_live) xf[j][t] = load_chunk(xrow[t], k, K, xok[t]);
    }
#pragma unroll
    for (int j = 0; j < UNROLL; ++j)
#pragma unroll
      for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int t = 0; t < XT; ++t)
          if (t < xt_live)
            acc[a][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(chunk_as_bf16x8(wf[j][a]), chunk_as_bf16x8(xf[j][t]), acc[a][t], 0, 0, 0);
  }

  // reduction over the waves, one w tile at a time through the same buffer.  Item -> (x tile t,
  // accumulator quad q, lane l): x row t*32 + l%32, columns 8q + 4(l/32) + 0..3
  constexpr int ITEMS = XT * 256 / (SK_WAVES * 64);
  float sum[NA][ITEMS][4];
#pragma unroll
  for (int a = 0; a < NA; ++a) {
    if (a) __syncthreads();
#pragma unroll
    for (int t = 0; t < XT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) sk_red[((wave * XT + t) * 16 + r) * 64 + lane] = acc[a][t][r];
    __syncthreads();
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int item = tid + it * SK_WAVES * 64;
      const int t = item >> 8, q = (item >> 6) & 3, l = item & 63;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < SK_WAVES; ++w) v += sk_red[((w * XT + t) * 16 + 4 * q + r) * 64 + l];
        sum[a][it][r] = v;
      }
    }
  }
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) {
    const int item = tid + it * SK_WAVES * 64;
    const int t = item >> 8, q = (item >> 6) & 3, l = item & 63;
    const int64_t m = t * 32 + (l & 31);
    const int64_t n = n0 + 8 * q + 4 * (l >> 5);
    if (m >= M || n >= N) continue;
    bf16_t out[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float g = sum[0][it][r];
      out[r] = f32_to_bf16(EPI == 1 ? g / (1.f + __expf(-g)) * sum[NA - 1][it][r] : g);
    }
    bf16_t* yp = Y + m * ldy + n;
    if (n + 3 < N && (((uintptr_t)yp) & 7) == 0) {
      uint2 pk;
      pk.x = out[0] | ((uint32_t)out[1] << 16);
      pk.y = out[2] | ((uint32_t)out[3] << 16);
      *(uint2*)yp = pk;
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n + r < N) yp[r] = out[r];
    }
  }
}

// -----------------------------------------------------------------------------------------
// K-split variant for at most 128 rows of x against a large weight (the projections of one decoding
// step of a wide model): workgroup (c, s) multiplies the 64 rows of w from 64c on with all rows of
// x over the K slice [256 s, 256 s + 256).  Both slices are fetched once, coalesced, into LDS (row
// pitch 528 bytes, so the 16-byte fragment reads of 32 rows spread over the banks), each of the
// 4 waves takes 32 rows of x, and the fp32 partial tile goes to a workspace [slices][M][rows of w];
// linear_splitk_reduce_kernel sums the slices and applies the epilogue.  Against the kernel above
// this reads x once per 64 columns instead of once per 32 with one access per 128-byte line
// instead of four, and has enough workgroups for every CU whatever N is.
// -----------------------------------------------------------------------------------------
constexpr int SPK_KS = 256, SPK_COLS = 64, SPK_PITCH = SPK_KS + 8, SPK_XROWS = 128;
constexpr int SPK_LDS_BYTES = (SPK_XROWS + SPK_COLS) * SPK_PITCH * 2;

__global__ __launch_bounds__(256) void linear_splitk_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, float* __restrict__ P, int64_t M,
    int64_t NW, int64_t K, int64_t ldx, int64_t ldw, int per_group) {
  extern __shared__ __attribute__((aligned(16))) bf16_t spk_lds[];
  bf16_t* Xs = spk_lds;                               // [128][SPK_PITCH]
  bf16_t* Ws = spk_lds + SPK_XROWS * SPK_PITCH;       // [64][SPK_PITCH]
  const int tid = threadIdx.x, lane = tid & 63, ln = lane & 31, hh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t n0 = (int64_t)blockIdx.x * SPK_COLS;
  const int xrows = (int)((M + 31) / 32) * 32;        // rows of x staged (whole 32-row tiles)
  f32x16 acc[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;

  // a workgroup takes per_group consecutive K slices, one after the other through the same buffer
  for (int sl = 0; sl < per_group; ++sl) {
  const int64_t k0 = ((int64_t)blockIdx.y * per_group + sl) * SPK_KS;
  if (k0 >= K) break;
  if (sl) __syncthreads();

  // stage both slices: 32 chunks of 16 bytes per row, consecutive lanes on consecutive chunks
  u32x4 xr[SPK_XROWS * 32 / 256], wr[SPK_COLS * 32 / 256];
#pragma unroll
  for (int i = 0; i < SPK_XROWS * 32 / 256; ++i) {
    const int c = tid + 256 * i, r = c >> 5, kc = (c & 31) * 8;
    if (r < xrows) xr[i] = load_chunk(X + (r < M ? r : 0) * ldx, k0 + kc, K, r < M);
  }
#pragma unroll
  for (int i = 0; i < SPK_COLS * 32 / 256; ++i) {
    const int c = tid + 256 * i, r = c >> 5, kc = (c & 31) * 8;
    const int64_t n = n0 + r;
    wr[i] = load_chunk(W + (n < NW ? n : 0) * ldw, k0 + kc, K, n < NW);
  }
#pragma unroll
  for (int i = 0; i < SPK_XROWS * 32 / 256; ++i) {
    const int c = tid + 256 * i, r = c >> 5, kc = (c & 31) * 8;
    if (r < xrows) *(u32x4*)(Xs + r * SPK_PITCH + kc) = xr[i];
  }
#pragma unroll
  for (int i = 0; i < SPK_COLS * 32 / 256; ++i) {
    const int c = tid + 256 * i, r = c >> 5, kc = (c & 31) * 8;
    *(u32x4*)(Ws + r * SPK_PITCH + kc) = wr[i];
  }
  __syncthreads();
  if (wave * 32 < M) {                                // else this wave's rows of x do not exist
#pragma unroll 4
  for (int ks = 0; ks < SPK_KS / 16; ++ks) {
    const bf16x8 xf = *(const bf16x8*)(Xs + (wave * 32 + ln) * SPK_PITCH + ks * 16 + hh * 8);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const bf16x8 wf = *(const bf16x8*)(Ws + (j * 32 + ln) * SPK_PITCH + ks * 16 + hh * 8);
      acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf, acc[j], 0, 0, 0);   // [w row][x row]
    }
  }
  }
  }   // K slices of this workgroup
  // lane: x row wave*32 + ln, rows of w n0 + 32j + 8q + 4hh + 0..3 -> 16-byte stores
  const int64_t m = wave * 32 + ln;
  if (m >= M) return;
  float* prow = P + ((int64_t)blockIdx.y * M + m) * NW;
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int64_t n = n0 + j * 32 + q * 8 + hh * 4;
      if (n + 3 < NW && (NW & 3) == 0) {
        *(float4*)(prow + n) = make_float4(acc[j][4 * q], acc[j][4 * q + 1], acc[j][4 * q + 2], acc[j][4 * q + 3]);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < NW) prow[n + r] = acc[j][4 * q + r];
      }
    }
}

// Sums the K slices of linear_splitk_kernel and writes bf16: one thread per 4 output columns.
template <int EPI>
__global__ __launch_bounds__(256) void linear_splitk_reduce_kernel(
    const float* __restrict__ P, bf16_t* __restrict__ Y, int64_t M, int64_t N, int64_t NW,
    int slices, int64_t ldy) {
  const int64_t n4 = (N + 3) / 4;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= M * n4) return;
  const int64_t m = i / n4, n = (i % n4) * 4;
  float g[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
  const bool vec = n + 3 < N && (NW & 3) == 0 && (N & 3) == 0;
  for (int s = 0; s < slices; ++s) {
    const float* row = P + ((int64_t)s * M + m) * NW;
    if (vec) {
      const float4 a = *(const float4*)(row + n);
      g[0] += a.x; g[1] += a.y; g[2] += a.z; g[3] += a.w;
      if (EPI == 1) {
        const float4 b = *(const float4*)(row + N + n);
        u[0] += b.x; u[1] += b.y; u[2] += b.z; u[3] += b.w;
      }
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n + r < N) {
          g[r] += row[n + r];
          if (EPI == 1) u[r] += row[N + n + r];
        }
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (n + r < N) Y[m * ldy + n + r] = f32_to_bf16(EPI == 1 ? g[r] / (1.f + __expf(-g[r])) * u[r] : g[r]);
}

// -----------------------------------------------------------------------------------------
// Large-tile variant for the big projections (M >= 256, K a multiple of 8):
//   workgroup tile 256 (rows of x) x BN (rows of w) x 64, 8 waves as 4 (x) x 2 (w), 2 waves/SIMD;
//   tiles go HBM/L2 -> LDS with direct-to-LDS loads (no staging registers) into two buffers,
//   rows are 128 bytes with the 16-byte chunks XOR-swizzled so the b128 fragment reads of 16
//   consecutive rows hit distinct banks.
// The product is formed transposed (A operand = w rows, B operand = x rows), so a lane owns one
// x row and 4 consecutive output columns per accumulator quad: 8-byte stores.
// EPI == 1: sub-blocks of the w tile alternate gate / up rows, see row mapping below.
// -----------------------------------------------------------------------------------------
__device__ inline void dma_to_lds_16(const void* gptr, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :: "v"(gptr), "s"(lds_base) : "memory", "m0");
}

// Linear workgroup id L -> tile coordinates.  Ids that are equal mod 8 run on one XCD (each has an
// L2 of its own).  Where the tile rows divide evenly (a multiple of 8 * GM), an XCD is given an
// eighth of the tile rows and walks it in groups of GM tile rows, column by column: the 32
// workgroups that an XCD runs side by side then cover GM rows x 32/GM columns of tiles and read
// GM + 32/GM operand panels between them instead of one panel per workgroup and more.  Otherwise
// row-major.
__device__ inline void tile_of_workgroup(int64_t L, int64_t mt, int64_t nt, int64_t* tm, int64_t* tn) {
  constexpr int GM = 4;
  int64_t m, n;
  if (mt % (8 * GM) == 0) {
    const int64_t xcd = L & 7, s = L >> 3, per = mt / 8;
    const int64_t g = s / (GM * nt), r = s % (GM * nt);
    n = r / GM;
    m = xcd * per + g * GM + r % GM;
  } else {
    m = L / nt;
    n = L % nt;
  }
  // (wave-uniform by construction; said so to the compiler, which keeps them in scalar registers)
  *tm = __builtin_amdgcn_readfirstlane((int)m);
  *tn = __builtin_amdgcn_readfirstlane((int)n);
}

// ---- epilogue of the large-tile kernels, through LDS (LDS_BYTES of it, idle by now).
// In the accumulators a lane holds 4 consecutive output columns of one x row (quad a4 = w rows
// 8*a4 + 4*hh + 0..3 of sub-block i, x row ln of block j): stored from there, an instruction writes
// 16 bytes to each of 32 rows.  Staged through LDS, a wave's 32 x WC outputs of a block j leave as
// whole rows: 16 bytes per lane, a row's lanes side by side.  EPI 1: SiLU gate; EPI 2: the residual
// rows R are added where the staged rows are read back.
// Row statistics that ride an epilogue, so that an RMSNorm between two products costs no pass of
// its own (models/mvpformer.py:133: the norm in front of the block's projections):
//   STATS 1  the product's x rows are RAW rows whose norm is still due: every output row is
//            scaled by r = rsqrt(sum of the row's partial sums of squares / cols + eps) while it
//            is converted (the norm's weight is folded into w's columns by the caller);
//   STATS 2  the partial sums of squares of the rows this product writes (final bf16 values, this
//            wave's columns) go to ss_out[m][2 * column tile + column half].
struct row_stats {
  const float* ss_in;      // [M][parts_in]
  int32_t parts_in;
  float inv_cols, eps;
  float* ss_out;           // [M][parts_out]
  int32_t parts_out;
};

template <int BN, int EPI, int LDS_BYTES, int STATS = 0>
__device__ inline void staged_epilogue(const f32x16 (&acc)[BN / 64][2], unsigned char* gsm, int wave, int lane,
                                       int64_t m0, int64_t n0, int64_t M, int64_t N,
                                       bf16_t* __restrict__ Y, int64_t ldy,
                                       const bf16_t* __restrict__ R, int64_t ldr,
                                       const row_stats* rs = nullptr, int64_t tile_n = 0) {
  typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
  constexpr int WN = BN / 2, NB = WN / 32;
  const int ln = lane & 31, hh = lane >> 5;
  const int wm = wave >> 1, wc = wave & 1;
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");   // requests past the end; last reads
  constexpr int WC = EPI == 1 ? WN / 2 : WN;          // output columns of a wave
  constexpr int PITCH = WC * 2 + 16;                  // bytes per staged row (+16: rows spread over the banks)
  constexpr int CPR = WC * 2 / 16;                    // 16-byte chunks per row
  constexpr int RPI = 64 / CPR;                       // rows per store instruction
  static_assert(8 * 32 * PITCH <= LDS_BYTES, "the staging area fits the ring");
  unsigned char* stg = gsm + wave * (32 * PITCH);
  const bool vec16 = (ldy & 7) == 0 && ((uintptr_t)Y & 15) == 0 &&
                     (EPI != 2 || ((ldr & 7) == 0 && ((uintptr_t)R & 15) == 0));
  const int64_t ncol0 = n0 + wc * WC;
  float rnorm[2] = {1.f, 1.f};
  if (STATS == 1) {        // the tile's 256 factors were put behind the ring when the tile began
    const float* rstat = (const float*)(gsm + LDS_BYTES);
#pragma unroll
    for (int j = 0; j < 2; ++j) rnorm[j] = rstat[wm * 64 + j * 32 + ln];
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    if (EPI == 1) {
#pragma unroll
      for (int p2 = 0; p2 < NB / 2; ++p2)
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
          bf16x4 o;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float gte = acc[2 * p2][j][a4 * 4 + r] * rnorm[j], up = acc[2 * p2 + 1][j][a4 * 4 + r] * rnorm[j];
            o[r] = (__bf16)(gte / (1.f + __expf(-gte)) * up);
          }
          *(bf16x4*)(stg + ln * PITCH + (p2 * 32 + a4 * 8 + hh * 4) * 2) = o;
        }
    } else {
#pragma unroll
      for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
          bf16x4 o;
#pragma unroll
          for (int r = 0; r < 4; ++r) o[r] = (__bf16)(STATS == 1 ? acc[i][j][a4 * 4 + r] * rnorm[j] : acc[i][j][a4 * 4 + r]);
          *(bf16x4*)(stg + ln * PITCH + (i * 32 + a4 * 8 + hh * 4) * 2) = o;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int rr = lane / CPR, cc = lane % CPR;
#pragma unroll
    for (int it = 0; it < (32 + RPI - 1) / RPI; ++it) {
      const int row = it * RPI + rr;
      if (rr >= RPI || row >= 32) continue;         // (CPR = 12: 60 lanes carry 5 rows)
      u32x4 v = *(const u32x4*)(stg + row * PITCH + cc * 16);
      const int64_t m = m0 + wm * 64 + j * 32 + row;
      const int64_t n = ncol0 + cc * 8;
      float sq = 0.f;
      if (m < M) {
        bf16_t* dst = Y + m * ldy + n;
        if (n + 7 < N && vec16) {
          if (EPI == 2) {
            const u32x4 r = *(const u32x4*)(R + m * ldr + n);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float lo = __uint_as_float(v[e] << 16) + __uint_as_float(r[e] << 16);
              const float hi = __uint_as_float(v[e] & 0xffff0000u) + __uint_as_float(r[e] & 0xffff0000u);
              v[e] = (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
            }
          }
          if (STATS == 2) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float lo = __uint_as_float(v[e] << 16), hi = __uint_as_float(v[e] & 0xffff0000u);
              sq += lo * lo + hi * hi;
            }
          }
          __builtin_nontemporal_store(v, (u32x4*)dst);   // (streamed out: the operand panels keep the L2)
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (n + e < N) {
              bf16_t o = (bf16_t)((v[e >> 1] >> ((e & 1) * 16)) & 0xffffu);
              if (EPI == 2) o = f32_to_bf16(bf16_to_f32(o) + bf16_to_f32(R[m * ldr + n + e]));
              dst[e] = o;
            }
        }
      }
      if (STATS == 2) {
        // the row's CPR lanes sit side by side: lane cc = 0 collects their sums (host side: this
        // product only runs on shapes that take the 16-byte path above for every chunk)
#pragma unroll
        for (int off = 1; off < CPR; off <<= 1) {
          const float o = __shfl_down(sq, off);
          if (cc + off < CPR) sq += o;
        }
        if (cc == 0 && m < M) rs->ss_out[m * rs->parts_out + tile_n * 2 + wc] = sq;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

template <int BN, int EPI>
__global__ __launch_bounds__(512) void linear_bf16_big_kernel(const bf16_t* __restrict__ X,
                                                              const bf16_t* __restrict__ W,
                                                              bf16_t* __restrict__ Y, int64_t M,
                                                              int64_t N, int64_t K, int64_t ldx,
                                                              int64_t ldw, int64_t ldy) {
  constexpr int BM = 256, BK = 64, ROWB = BK * 2;
  constexpr int WN = BN / 2, NB = WN / 32;            // per-wave extent over w rows
  constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE = A_BYTES + B_BYTES;
  constexpr int A_LOADS = A_BYTES / 1024 / 8, B_LOADS = B_BYTES / 1024 / 8;   // per wave
  static_assert(EPI != 1 || NB % 2 == 0, "gate/up pairs need an even number of sub-blocks");
  extern __shared__ __attribute__((aligned(1024))) unsigned char gsm[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, hh = lane >> 5;
  const int wm = wave >> 1, wc = wave & 1;
  constexpr int OUT_COLS = EPI == 1 ? BN / 2 : BN;    // output columns per workgroup
  const int64_t mt = (M + BM - 1) / BM, nt = (N + OUT_COLS - 1) / OUT_COLS;

  int64_t m0 = 0, n0 = 0;                             // first x row / output column of the tile
  const bf16_t* asrc[A_LOADS];
  const bf16_t* bsrc[B_LOADS];
  auto w_row = [&](int r) -> int64_t {                // which w row feeds tile row r
    if (EPI == 1) {
      const int wcol = r / WN, nb = (r % WN) / 32, i = r & 31;
      const int64_t col = n0 + wcol * (WN / 2) + (nb >> 1) * 32 + i;
      return ((nb & 1) ? N : 0) + (col < N ? col : N - 1);
    }
    const int64_t n = n0 + r;
    return n < N ? n : N - 1;
  };
  // per-lane source rows of this wave's loads (row clamped into range: such rows are never stored)
  auto set_tile = [&](int64_t L) {
    int64_t tile_m, tile_n;
    tile_of_workgroup(L, mt, nt, &tile_m, &tile_n);
    m0 = tile_m * BM;
    n0 = tile_n * OUT_COLS;
    const int rsub = lane >> 3, phys = lane & 7;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int row = (wave * A_LOADS + i) * 8 + rsub;
      const int64_t m = m0 + row;
      asrc[i] = X + (m < M ? m : M - 1) * ldx + ((phys ^ ((row >> 1) & 7)) << 3);
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const int row = (wave * B_LOADS + i) * 8 + rsub;
      bsrc[i] = W + w_row(row) * ldw + ((phys ^ ((row >> 1) & 7)) << 3);
    }
  };
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)gsm;
  auto issue = [&](int kt, int stage) {
    const int64_t k0 = (int64_t)kt * BK;
    const uint32_t base = lds0 + stage * STAGE;
    if (k0 + BK <= K) {                               // (uniform) a whole k-block: nothing but the loads
#pragma unroll
      for (int i = 0; i < A_LOADS; ++i) dma_to_lds_16(asrc[i] + k0, base + (wave * A_LOADS + i) * 1024);
#pragma unroll
      for (int i = 0; i < B_LOADS; ++i) dma_to_lds_16(bsrc[i] + k0, base + A_BYTES + (wave * B_LOADS + i) * 1024);
      return;
    }
    // the tail block of K: chunks past the end are zero-filled
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const uint32_t dst = base + (wave * A_LOADS + i) * 1024;
      const int row = (wave * A_LOADS + i) * 8 + (lane >> 3);
      const int64_t kk = k0 + (((lane & 7) ^ ((row >> 1) & 7)) << 3);
      if (kk < K) dma_to_lds_16(asrc[i] + k0, dst);
      else *(u32x4*)(gsm + (dst - lds0) + lane * 16) = u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const uint32_t dst = base + A_BYTES + (wave * B_LOADS + i) * 1024;
      const int row = (wave * B_LOADS + i) * 8 + (lane >> 3);
      const int64_t kk = k0 + (((lane & 7) ^ ((row >> 1) & 7)) << 3);
      if (kk < K) dma_to_lds_16(bsrc[i] + k0, dst);
      else *(u32x4*)(gsm + (dst - lds0) + lane * 16) = u32x4{0u, 0u, 0u, 0u};
    }
  };

  // loop-invariant fragment offsets: row ln of a 32-row block, chunk (2ks+hh) ^ swizzle(ln)
  int frag_off[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) frag_off[ks] = ln * ROWB + (((2 * ks + hh) ^ ((ln >> 1) & 7)) << 4);

  const int nkt = (int)((K + BK - 1) / BK);
  int stage = 0;                                      // ring stage of the k-block to multiply next
  set_tile(blockIdx.x);
  issue(0, 0);
  {
    const int64_t cm0 = m0, cn0 = n0;
    f32x16 acc[NB][2];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    for (int kt = 0; kt < nkt; ++kt) {
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      const unsigned char* sa = gsm + stage * STAGE + (wm * 64) * ROWB;
      const unsigned char* sb = gsm + stage * STAGE + A_BYTES + (wc * WN) * ROWB;
      // the first fragments are requested before the next block's loads, whose issue covers their
      // latency; inside the block the fragments of k-step s+1 are requested before the products of s
      bf16x8 xf[2][2], wf[2][NB];
#pragma unroll
      for (int j = 0; j < 2; ++j) xf[0][j] = *(const bf16x8*)(sa + j * 32 * ROWB + frag_off[0]);
#pragma unroll
      for (int i = 0; i < NB; ++i) wf[0][i] = *(const bf16x8*)(sb + i * 32 * ROWB + frag_off[0]);
      __builtin_amdgcn_sched_barrier(0);
      if (kt + 1 < nkt) issue(kt + 1, stage ^ 1);
      stage ^= 1;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const int cur = ks & 1, nxt = cur ^ 1;
        if (ks + 1 < 4) {
#pragma unroll
          for (int j = 0; j < 2; ++j) xf[nxt][j] = *(const bf16x8*)(sa + j * 32 * ROWB + frag_off[ks + 1]);
#pragma unroll
          for (int i = 0; i < NB; ++i) wf[nxt][i] = *(const bf16x8*)(sb + i * 32 * ROWB + frag_off[ks + 1]);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < NB; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[cur][i], xf[cur][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    staged_epilogue<BN, EPI, 2 * STAGE>(acc, gsm, wave, lane, cm0, cn0, M, N, Y, ldy, nullptr, 0);
  }
}

template <int BN, int EPI>
static int launch_big(const bf16_t* x, const bf16_t* w, bf16_t* y, int64_t M, int64_t N, int64_t K,
                      int64_t ldx, int64_t ldw, int64_t ldy, hipStream_t s) {
  constexpr int LDS = 2 * (256 + BN) * 128;
  auto kern = linear_bf16_big_kernel<BN, EPI>;
  mvpa::want_dynamic_lds((const void*)kern, (int)LDS);
  constexpr int OUT_COLS = EPI == 1 ? BN / 2 : BN;
  dim3 grid((unsigned)(((N + OUT_COLS - 1) / OUT_COLS) * ((M + 255) / 256)));
  MVPA_LAUNCH(kern, grid, dim3(512), LDS, s, x, w, y, M, N, K, ldx, ldw, ldy);
  return mvpa::take_launch_status();
}

// -----------------------------------------------------------------------------------------
// The large-tile kernel on a ring of four k-blocks of 32 (K a multiple of 32).
// With one workgroup per CU and two k-blocks of 64 in LDS, the loads of block k+1 are requested
// when block k is published and must have landed when it is consumed: every k-block waits out
// whatever of the L2 / HBM latency its own 2048 matrix cycles do not cover (1.3-1.6 us per
// k-block measured against 0.85 us of matrix time).  Here a k-block is 32 wide and four are in
// LDS: the barrier of block k publishes block k+1 (block k was published by the one before),
// blocks k+2 is in flight and k+3 is requested right after the barrier, so a load has two to
// three blocks' time to arrive; the first fragments of block k+1 are read before its barrier
// (the bare s_barrier leaves them in flight), so that a wave leaves the barrier with products to
// issue.  One block is requested per step without a branch (past the end the last block once
// more, into a stage nobody reads) so that the waits are fixed vmcnt immediates.
// Same tile order, roles, row mapping and epilogues as linear_bf16_big_kernel.
// -----------------------------------------------------------------------------------------
// EPI 2: Y = X W^T + R, the residual rows R (bf16, row pitch ldr) added where the staged rows
// are read back, 16 bytes per lane like the stores.
template <int BN, int EPI>
__global__ __launch_bounds__(512) void linear_bf16_ring_kernel(const bf16_t* __restrict__ X,
                                                               const bf16_t* __restrict__ W,
                                                               bf16_t* __restrict__ Y, int64_t M,
                                                               int64_t N, int64_t K, int64_t ldx,
                                                               int64_t ldw, int64_t ldy,
                                                               const bf16_t* __restrict__ R, int64_t ldr) {
  constexpr int BM = 256, BK = 32, ROWB = BK * 2, STAGES = 4;
  constexpr int WN = BN / 2, NB = WN / 32;            // per-wave extent over w rows
  constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE = A_BYTES + B_BYTES;
  constexpr int A_LOADS = A_BYTES / 1024 / 8;         // 1 KiB wave loads per wave and block (x rows)
  constexpr int B_TOT = B_BYTES / 1024, B_LOADS = (B_TOT + 7) / 8;   // w rows: B_TOT loads over 8 waves
  constexpr bool RAGGED = B_TOT % 8 != 0;             // (BN = 192: waves 0..3 have one load more)
  static_assert(EPI != 1 || NB % 2 == 0, "gate/up pairs need an even number of sub-blocks");
  extern __shared__ __attribute__((aligned(1024))) unsigned char gsm[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, hh = lane >> 5;
  const int wm = wave >> 1, wc = wave & 1;
  constexpr int OUT_COLS = EPI == 1 ? BN / 2 : BN;    // output columns per workgroup
  int64_t tile_m, tile_n;
  tile_of_workgroup(blockIdx.x, (M + BM - 1) / BM, (N + OUT_COLS - 1) / OUT_COLS, &tile_m, &tile_n);
  const int64_t m0 = tile_m * BM, n0 = tile_n * OUT_COLS;
  const int nkb = (int)(K / BK);

  auto w_row = [&](int r) -> int64_t {                // which w row feeds tile row r
    if (EPI == 1) {
      const int wcol = r / WN, nb = (r % WN) / 32, i = r & 31;
      const int64_t col = n0 + wcol * (WN / 2) + (nb >> 1) * 32 + i;
      return ((nb & 1) ? N : 0) + (col < N ? col : N - 1);
    }
    const int64_t n = n0 + r;
    return n < N ? n : N - 1;
  };

  // ---- the request side: the stream of k-blocks, three blocks ahead of the products.  A wave
  // load covers 16 tile rows x 64 bytes: lane L is row L/4, physical chunk L%4; per-lane byte
  // offsets from wave-uniform bases (rows clamped into range: such rows are never stored).
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)gsm;
  int iss_kb = 0;
  uint32_t iss_lds = lds0;
  const int64_t wrow0 = w_row(0);
  const bf16_t* xs = X + m0 * ldx;
  const bf16_t* ws = W + wrow0 * ldw;
  uint32_t aoff[A_LOADS], boff[B_LOADS];
  {
    const int rsub = lane >> 2, phys = lane & 3;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int row = (wave + 8 * i) * 16 + rsub;
      const int64_t m = m0 + row;
      aoff[i] = (uint32_t)((((m < M ? m : M - 1) - m0) * ldx + ((phys ^ ((row >> 2) & 3)) << 3)) * 2);
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const int row = min((wave + 8 * i) * 16 + rsub, BN - 1);
      boff[i] = (uint32_t)(((w_row(row) - wrow0) * ldw + ((phys ^ ((row >> 2) & 3)) << 3)) * 2);
    }
  }
  auto issue_block = [&]() {
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i)
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(aoff[i]), "s"(xs), "s"(iss_lds + (wave + 8 * i) * 1024) : "memory", "m0");
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      if (RAGGED && i == B_LOADS - 1 && wave + 8 * i >= B_TOT) continue;   // (uniform per wave)
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(boff[i]), "s"(ws), "s"(iss_lds + A_BYTES + (wave + 8 * i) * 1024) : "memory", "m0");
    }
    iss_lds = iss_lds + STAGE == lds0 + STAGES * STAGE ? lds0 : iss_lds + STAGE;
    // on to the next block of the stream; past its end the last block is requested again, into
    // a stage nobody reads, so that the count of loads in flight stays what the waits assume
    if (iss_kb + 1 < nkb) {
      ++iss_kb;
      xs += BK;
      ws += BK;
    }
  };
  // at most 1 / 2 blocks' worth of this wave's loads outstanding
  const bool short_wave = RAGGED && wave + 8 * (B_LOADS - 1) >= B_TOT;
  auto wait_blocks1 = [&]() {
    if (short_wave) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(A_LOADS + B_LOADS - 1) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(A_LOADS + B_LOADS) : "memory");
  };
  auto wait_blocks2 = [&]() {
    if (short_wave) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (A_LOADS + B_LOADS - 1)) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (A_LOADS + B_LOADS)) : "memory");
  };

  // fragment offsets: row ln of a 32-row block, chunk (2ks+hh) ^ swizzle(ln)
  int frag_off[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) frag_off[ks] = ln * ROWB + (((2 * ks + hh) ^ ((ln >> 2) & 3)) << 4);
  const int a_lane = (wm * 64) * ROWB, b_lane = A_BYTES + (wc * WN) * ROWB;

  issue_block();
  issue_block();
  issue_block();
  wait_blocks2();
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  bf16x8 xf0[2], wf0[NB];
#pragma unroll
  for (int j = 0; j < 2; ++j) xf0[j] = *(const bf16x8*)(gsm + a_lane + j * 32 * ROWB + frag_off[0]);
#pragma unroll
  for (int i = 0; i < NB; ++i) wf0[i] = *(const bf16x8*)(gsm + b_lane + i * 32 * ROWB + frag_off[0]);
  int cur = 0;                                        // stage of the block being multiplied
  typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;

  {
    f32x16 acc[NB][2];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    for (int kb = 0; kb < nkb; ++kb) {
      wait_blocks1();
      asm volatile("s_barrier" ::: "memory");         // (fragments read ahead stay in flight across it)
      const unsigned char* st = gsm + cur * STAGE;
      cur = (cur + 1) & (STAGES - 1);
      const unsigned char* sn = gsm + cur * STAGE;
      bf16x8 xf1[2], wf1[NB];
#pragma unroll
      for (int j = 0; j < 2; ++j) xf1[j] = *(const bf16x8*)(st + a_lane + j * 32 * ROWB + frag_off[1]);
#pragma unroll
      for (int i = 0; i < NB; ++i) wf1[i] = *(const bf16x8*)(st + b_lane + i * 32 * ROWB + frag_off[1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf0[i], xf0[j], acc[i][j], 0, 0, 0);
          if (i == 0 && j == 0) {
            __builtin_amdgcn_sched_barrier(0);
            issue_block();
          }
        }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 2; ++j) xf0[j] = *(const bf16x8*)(sn + a_lane + j * 32 * ROWB + frag_off[0]);
#pragma unroll
      for (int i = 0; i < NB; ++i) wf0[i] = *(const bf16x8*)(sn + b_lane + i * 32 * ROWB + frag_off[0]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf1[i], xf1[j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }

    staged_epilogue<BN, EPI, STAGES * STAGE>(acc, gsm, wave, lane, m0, n0, M, N, Y, ldy, R, ldr);
  }
}

template <int BN, int EPI>
static int launch_ring(const bf16_t* x, const bf16_t* w, bf16_t* y, int64_t M, int64_t N, int64_t K,
                       int64_t ldx, int64_t ldw, int64_t ldy, hipStream_t s,
                       const bf16_t* r = nullptr, int64_t ldr = 0) {
  constexpr int LDS = 4 * (256 + BN) * 64;
  auto kern = linear_bf16_ring_kernel<BN, EPI>;
  mvpa::want_dynamic_lds((const void*)kern, (int)LDS);
  constexpr int OUT_COLS = EPI == 1 ? BN / 2 : BN;
  dim3 grid((unsigned)(((N + OUT_COLS - 1) / OUT_COLS) * ((M + 255) / 256)));
  MVPA_LAUNCH(kern, grid, dim3(512), LDS, s, x, w, y, M, N, K, ldx, ldw, ldy, r, ldr);
  return mvpa::take_launch_status();
}

// -----------------------------------------------------------------------------------------
// The large-tile kernel on two stages of 64-wide k-blocks (K a multiple of 64).
// A request of the 32-wide ring covers 64 bytes of a row - half a cache line, whose other half
// the next k-block asks for again, one k-block's worth of other lines (32 KiB per CU) later.  Here
// a wave load covers 8 rows x 128 bytes, whole lines, and LDS holds two blocks of 64.  The order of a
// block keeps what the ring gained: the barrier sits in front of the block's LAST quarter, whose
// fragments are in registers by then (lgkmcnt 0 before it: nobody still reads the block); it
// publishes the next block, whose first fragments are read under that last quarter's products, and
// frees this block's stage, into which the block after next is requested at once - a full block's
// time ahead of the barrier that will wait for it.  One request per block without a branch (past
// the end the last block again, into a stage nobody reads), so the wait is a fixed vmcnt(0).
// Same tile order, roles, row mapping and epilogues as the other large-tile kernels.
// -----------------------------------------------------------------------------------------
template <int BN, int EPI, int STATS = 0>
__device__ __forceinline__ void linear_pair_tile(int64_t tile, unsigned char* gsm,
                                                 const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                 bf16_t* __restrict__ Y, int64_t M, int64_t N, int64_t K,
                                                 int64_t ldx, int64_t ldw, int64_t ldy,
                                                 const bf16_t* __restrict__ R, int64_t ldr,
                                                 const row_stats* rs = nullptr) {
  constexpr int BM = 256, BK = 64, ROWB = BK * 2, STAGES = 2;
  constexpr int WN = BN / 2, NB = WN / 32;            // per-wave extent over w rows
  constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE = A_BYTES + B_BYTES;
  constexpr int A_LOADS = A_BYTES / 1024 / 8, B_LOADS = B_BYTES / 1024 / 8;   // 1 KiB wave loads per wave and block
  static_assert(B_BYTES % (8 * 1024) == 0, "every wave issues the same number of loads");
  static_assert(EPI != 1 || NB % 2 == 0, "gate/up pairs need an even number of sub-blocks");

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, hh = lane >> 5;
  const int wm = wave >> 1, wc = wave & 1;
  constexpr int OUT_COLS = EPI == 1 ? BN / 2 : BN;    // output columns per workgroup
  int64_t tile_m, tile_n;
  tile_of_workgroup(tile, (M + BM - 1) / BM, (N + OUT_COLS - 1) / OUT_COLS, &tile_m, &tile_n);
  const int64_t m0 = tile_m * BM, n0 = tile_n * OUT_COLS;
  const int nkb = (int)(K / BK);

  auto w_row = [&](int r) -> int64_t {                // which w row feeds tile row r
    if (EPI == 1) {
      const int wcol = r / WN, nb = (r % WN) / 32, i = r & 31;
      const int64_t col = n0 + wcol * (WN / 2) + (nb >> 1) * 32 + i;
      return ((nb & 1) ? N : 0) + (col < N ? col : N - 1);
    }
    const int64_t n = n0 + r;
    return n < N ? n : N - 1;
  };

  // ---- the request side.  A wave load covers 8 tile rows x 128 bytes: lane L is row L/8, physical
  // chunk L%8; per-lane byte offsets from wave-uniform bases (rows clamped into range: such rows
  // are never stored).
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)gsm;
  int iss_kb = 0;
  uint32_t iss_lds = lds0;
  const int64_t wrow0 = w_row(0);
  const bf16_t* xs = X + m0 * ldx;
  const bf16_t* ws = W + wrow0 * ldw;
  uint32_t aoff[A_LOADS], boff[B_LOADS];
  {
    const int rsub = lane >> 3, phys = lane & 7;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int row = (wave + 8 * i) * 8 + rsub;
      const int64_t m = m0 + row;
      aoff[i] = (uint32_t)((((m < M ? m : M - 1) - m0) * ldx + ((phys ^ ((row >> 1) & 7)) << 3)) * 2);
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const int row = (wave + 8 * i) * 8 + rsub;
      boff[i] = (uint32_t)(((w_row(row) - wrow0) * ldw + ((phys ^ ((row >> 1) & 7)) << 3)) * 2);
    }
  }
  auto issue_block = [&]() {
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i)
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(aoff[i]), "s"(xs), "s"(iss_lds + (wave + 8 * i) * 1024) : "memory", "m0");
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i)
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(boff[i]), "s"(ws), "s"(iss_lds + A_BYTES + (wave + 8 * i) * 1024) : "memory", "m0");
    iss_lds = iss_lds == lds0 ? lds0 + STAGE : lds0;
    if (iss_kb + 1 < nkb) {
      ++iss_kb;
      xs += BK;
      ws += BK;
    }
  };

  // fragment offsets: row ln of a 32-row block, chunk (2s+hh) ^ swizzle(ln) for the four 16-wide slices
  int frag_off[4];
#pragma unroll
  for (int sl = 0; sl < 4; ++sl) frag_off[sl] = ln * ROWB + (((2 * sl + hh) ^ ((ln >> 1) & 7)) << 4);
  const int a_lane = (wm * 64) * ROWB, b_lane = A_BYTES + (wc * WN) * ROWB;

  // STATS 1: the norm factors of the tile's 256 rows, r = rsqrt(sum of the row's partial sums of
  // squares / K + eps).  Two threads share a row and half of its partial sums each; the loads go
  // out in front of the first blocks and are long back when those have landed.  The factors wait
  // in LDS behind the ring for the epilogue.
  float rpart = 0.f;
  if (STATS == 1) {
    const int row = tid >> 1, half = tid & 1;
    const int64_t m = m0 + row;
    const int parts = rs->parts_in;
    if (m < M) {
      const float* pp = rs->ss_in + m * parts;
      if ((parts & 7) == 0 && parts <= 16) {
        typedef __attribute__((ext_vector_type(4))) float f32x4;
        const f32x4* q4 = (const f32x4*)(pp + half * (parts >> 1));
        const f32x4 a = q4[0];
        rpart = (a.x + a.y) + (a.z + a.w);
        if (parts == 16) {
          const f32x4 b4 = q4[1];
          rpart += (b4.x + b4.y) + (b4.z + b4.w);
        }
      } else if (half == 0) {
        for (int p2 = 0; p2 < parts; ++p2) rpart += pp[p2];
      }
    }
  }
  issue_block();
  issue_block();
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(A_LOADS + B_LOADS) : "memory");
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  bf16x8 xf0[2], wf0[NB];
#pragma unroll
  for (int j = 0; j < 2; ++j) xf0[j] = *(const bf16x8*)(gsm + a_lane + j * 32 * ROWB + frag_off[0]);
#pragma unroll
  for (int i = 0; i < NB; ++i) wf0[i] = *(const bf16x8*)(gsm + b_lane + i * 32 * ROWB + frag_off[0]);
  int cur = 0;                                        // stage of the block being multiplied

  f32x16 acc[NB][2];
#pragma unroll
  for (int i = 0; i < NB; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  for (int kb = 0; kb < nkb; ++kb) {
    const unsigned char* st = gsm + cur * STAGE;
    cur ^= 1;
    const unsigned char* sn = gsm + cur * STAGE;
    bf16x8 xf1[2], wf1[NB];
    // slices 0 .. 2: the fragments of slice s+1 are requested before the products of slice s
#pragma unroll
    for (int j = 0; j < 2; ++j) xf1[j] = *(const bf16x8*)(st + a_lane + j * 32 * ROWB + frag_off[1]);
#pragma unroll
    for (int i = 0; i < NB; ++i) wf1[i] = *(const bf16x8*)(st + b_lane + i * 32 * ROWB + frag_off[1]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf0[i], xf0[j], acc[i][j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 2; ++j) xf0[j] = *(const bf16x8*)(st + a_lane + j * 32 * ROWB + frag_off[2]);
#pragma unroll
    for (int i = 0; i < NB; ++i) wf0[i] = *(const bf16x8*)(st + b_lane + i * 32 * ROWB + frag_off[2]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf1[i], xf1[j], acc[i][j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 2; ++j) xf1[j] = *(const bf16x8*)(st + a_lane + j * 32 * ROWB + frag_off[3]);
#pragma unroll
    for (int i = 0; i < NB; ++i) wf1[i] = *(const bf16x8*)(st + b_lane + i * 32 * ROWB + frag_off[3]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf0[i], xf0[j], acc[i][j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    // the next block has landed, and every fragment of this one is in registers: publish / free
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (STATS == 1 && kb == 0) {
      // (every load of this wave is back here, the partial sums among them: no wait of their own;
      // the factors are published by the barriers of the blocks that follow)
      rpart += __shfl_xor(rpart, 1);
      if ((tid & 1) == 0) ((float*)(gsm + STAGES * STAGE))[tid >> 1] = rsqrtf(rpart * rs->inv_cols + rs->eps);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) xf0[j] = *(const bf16x8*)(sn + a_lane + j * 32 * ROWB + frag_off[0]);
#pragma unroll
    for (int i = 0; i < NB; ++i) wf0[i] = *(const bf16x8*)(sn + b_lane + i * 32 * ROWB + frag_off[0]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf1[i], xf1[j], acc[i][j], 0, 0, 0);
        if (i == 0 && j == 0) {
          __builtin_amdgcn_sched_barrier(0);
          issue_block();                              // the block after next, into the stage just freed
        }
      }
    __builtin_amdgcn_sched_barrier(0);
  }
  staged_epilogue<BN, EPI, STAGES * STAGE, STATS>(acc, gsm, wave, lane, m0, n0, M, N, Y, ldy, R, ldr, rs, tile_n);
}

template <int BN, int EPI>
__global__ __launch_bounds__(512) void linear_bf16_pair_kernel(const bf16_t* __restrict__ X,
                                                               const bf16_t* __restrict__ W,
                                                               bf16_t* __restrict__ Y, int64_t M,
                                                               int64_t N, int64_t K, int64_t ldx,
                                                               int64_t ldw, int64_t ldy,
                                                               const bf16_t* __restrict__ R, int64_t ldr) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char gsm[];
  linear_pair_tile<BN, EPI>(blockIdx.x, gsm, X, W, Y, M, N, K, ldx, ldw, ldy, R, ldr);
}

// Two products of one launch: y0 = x w0^T (tiles 256 x BN0) and y1 = silu(x wg^T) * (x wu^T)
// (tiles 256 x 256), both on the same x.  Launched one after the other, each product ends on a
// round of tiles that fills part of the chip; in one grid - the gated product's tiles first, they
// are the longer ones - only the sum does.
struct linear_pair_problem {
  const bf16_t* w;
  bf16_t* y;
  int64_t N, ldw, ldy;
};

template <int BN0>
__global__ __launch_bounds__(512) void linear_bf16_pair_dual_kernel(const bf16_t* __restrict__ X, int64_t M,
                                                                    int64_t K, int64_t ldx,
                                                                    linear_pair_problem plain,
                                                                    linear_pair_problem gated,
                                                                    int64_t gated_tiles) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char gsm[];
  const int64_t L = blockIdx.x;
  if (L < gated_tiles)
    linear_pair_tile<256, 1>(L, gsm, X, gated.w, gated.y, M, gated.N, K, ldx, gated.ldw, gated.ldy, nullptr, 0);
  else
    linear_pair_tile<BN0, 0>(L - gated_tiles, gsm, X, plain.w, plain.y, M, plain.N, K, ldx, plain.ldw, plain.ldy,
                             nullptr, 0);
}

// the residual product that also writes the partial sums of squares of its output rows
template <int BN>
__global__ __launch_bounds__(512) void linear_bf16_pair_sumsq_kernel(const bf16_t* __restrict__ X,
                                                                     const bf16_t* __restrict__ W,
                                                                     bf16_t* __restrict__ Y, int64_t M,
                                                                     int64_t N, int64_t K, int64_t ldx,
                                                                     int64_t ldw, int64_t ldy,
                                                                     const bf16_t* __restrict__ R, int64_t ldr,
                                                                     row_stats rs) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char gsm[];
  linear_pair_tile<BN, 2, 2>(blockIdx.x, gsm, X, W, Y, M, N, K, ldx, ldw, ldy, R, ldr, &rs);
}

// the two products on raw rows whose RMSNorm is applied in the epilogue
template <int BN0>
__global__ __launch_bounds__(512) void linear_bf16_pair_dual_normed_kernel(const bf16_t* __restrict__ X, int64_t M,
                                                                           int64_t K, int64_t ldx,
                                                                           linear_pair_problem plain,
                                                                           linear_pair_problem gated,
                                                                           int64_t gated_tiles, row_stats rs) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char gsm[];
  const int64_t L = blockIdx.x;
  if (L < gated_tiles)
    linear_pair_tile<256, 1, 1>(L, gsm, X, gated.w, gated.y, M, gated.N, K, ldx, gated.ldw, gated.ldy, nullptr, 0, &rs);
  else
    linear_pair_tile<BN0, 0, 1>(L - gated_tiles, gsm, X, plain.w, plain.y, M, plain.N, K, ldx, plain.ldw, plain.ldy,
                                nullptr, 0, &rs);
}

// sums of squares of bf16 rows (one part per row): the statistics of the first block's input
__global__ __launch_bounds__(256) void row_sumsq_bf16_kernel(const bf16_t* __restrict__ x, float* __restrict__ ss,
                                                             int64_t rows, int32_t cols, int64_t ldx) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  float sq = 0.f;
  for (int c = lane * 8; c < cols; c += 512) {
    const u32x4 v = *(const u32x4*)(x + row * ldx + c);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float lo = __uint_as_float(v[e] << 16), hi = __uint_as_float(v[e] & 0xffff0000u);
      sq += lo * lo + hi * hi;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sq += __shfl_xor(sq, off);
  if (lane == 0) ss[row] = sq;
}

template <int BN>
static int launch_pair_sumsq(const bf16_t* x, const bf16_t* w, bf16_t* y, int64_t M, int64_t N, int64_t K,
                             int64_t ldx, int64_t ldw, int64_t ldy, hipStream_t s, const bf16_t* r, int64_t ldr,
                             float* ss_out, int32_t parts) {
  constexpr int LDS = 2 * (256 + BN) * 128;
  auto kern = linear_bf16_pair_sumsq_kernel<BN>;
  mvpa::want_dynamic_lds((const void*)kern, (int)LDS);
  dim3 grid((unsigned)(((N + BN - 1) / BN) * ((M + 255) / 256)));
  const mvpa::row_stats rs{nullptr, 0, 0.f, 0.f, ss_out, parts};
  MVPA_LAUNCH(kern, grid, dim3(512), LDS, s, x, w, y, M, N, K, ldx, ldw, ldy, r, ldr, rs);
  return mvpa::take_launch_status();
}

template <int BN0>
static int launch_pair_dual_normed(const bf16_t* x, int64_t M, int64_t K, int64_t ldx,
                                   const mvpa::linear_pair_problem& plain, const mvpa::linear_pair_problem& gated,
                                   const mvpa::row_stats& rs, hipStream_t s) {
  constexpr int LDS = 2 * (256 + 256) * 128 + 1024;     // ring + the tile's 256 norm factors
  auto kern = linear_bf16_pair_dual_normed_kernel<BN0>;
  mvpa::want_dynamic_lds((const void*)kern, (int)LDS);
  const int64_t mt = (M + 255) / 256;
  const int64_t gated_tiles = mt * ((gated.N + 127) / 128), plain_tiles = mt * ((plain.N + BN0 - 1) / BN0);
  MVPA_LAUNCH(kern, dim3((unsigned)(gated_tiles + plain_tiles)), dim3(512), LDS, s, x, M, K, ldx, plain, gated,
              gated_tiles, rs);
  return mvpa::take_launch_status();
}

template <int BN, int EPI>
static int launch_pair(const bf16_t* x, const bf16_t* w, bf16_t* y, int64_t M, int64_t N, int64_t K,
                       int64_t ldx, int64_t ldw, int64_t ldy, hipStream_t s,
                       const bf16_t* r = nullptr, int64_t ldr = 0) {
  constexpr int LDS = 2 * (256 + BN) * 128;
  auto kern = linear_bf16_pair_kernel<BN, EPI>;
  mvpa::want_dynamic_lds((const void*)kern, (int)LDS);
  constexpr int OUT_COLS = EPI == 1 ? BN / 2 : BN;
  dim3 grid((unsigned)(((N + OUT_COLS - 1) / OUT_COLS) * ((M + 255) / 256)));
  MVPA_LAUNCH(kern, grid, dim3(512), LDS, s, x, w, y, M, N, K, ldx, ldw, ldy, r, ldr);
  return mvpa::take_launch_status();
}

template <int BN0>
static int launch_pair_dual(const bf16_t* x, int64_t M, int64_t K, int64_t ldx, const mvpa::linear_pair_problem& plain,
                            const mvpa::linear_pair_problem& gated, hipStream_t s) {
  constexpr int LDS = 2 * (256 + 256) * 128;
  auto kern = linear_bf16_pair_dual_kernel<BN0>;
  mvpa::want_dynamic_lds((const void*)kern, (int)LDS);
  const int64_t mt = (M + 255) / 256;
  const int64_t gated_tiles = mt * ((gated.N + 127) / 128), plain_tiles = mt * ((plain.N + BN0 - 1) / BN0);
  MVPA_LAUNCH(kern, dim3((unsigned)(gated_tiles + plain_tiles)), dim3(512), LDS, s, x, M, K, ldx, plain, gated,
              gated_tiles);
  return mvpa::take_launch_status();
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

// ---- 8 elements per lane and access (16 bytes of bf16, 32 bytes of fp32) --------------------
template <typename T> struct vec8;
template <> struct vec8<float> {
  __device__ static inline void load(const float* p, float (&v)[8]) {
    const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  __device__ static inline void store(float* p, const float (&v)[8]) {
    *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
    *(float4*)(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
};
template <> struct vec8<bf16_t> {
  __device__ static inline void load(const bf16_t* p, float (&v)[8]) {
    const uint4 r = *(const uint4*)p;
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  __device__ static inline void store(bf16_t* p, const float (&v)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = (uint32_t)f32_to_bf16(v[2 * i]) | ((uint32_t)f32_to_bf16(v[2 * i + 1]) << 16);
    *(uint4*)p = make_uint4(w[0], w[1], w[2], w[3]);
  }
};

__device__ inline float wave_sum(float x) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off);
  return x;
}

// One wave per row, 8 elements per lane and access; needs cols % 8 == 0 and 16-byte aligned rows.
// The second pass re-reads the row, which is still in the CU's cache.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const TI* __restrict__ x,
                                                           const float* __restrict__ w,
                                                           TO* __restrict__ y, int64_t rows, int cols,
                                                           int64_t ldx, int64_t ldy, float eps) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const TI* xr = x + row * ldx;
  TO* yr = y + row * ldy;
  float ss = 0.f;
  for (int c = lane * 8; c < cols; c += 512) {
    float v[8];
    vec8<TI>::load(xr + c, v);
#pragma unroll
    for (int i = 0; i < 8; ++i) ss += v[i] * v[i];
  }
  const float inv = rsqrtf(wave_sum(ss) / (float)cols + eps);
  for (int c = lane * 8; c < cols; c += 512) {
    float v[8], g[8];
    vec8<TI>::load(xr + c, v);
    vec8<float>::load(w + c, g);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = v[i] * inv * g[i];
    vec8<TO>::store(yr + c, v);
  }
}

// Cosine similarity of row pairs: out[r] = a_r . b_r / (max(|a_r|, eps) * max(|b_r|, eps)), fp32
// arithmetic, one wave per row pair.  Rows come in groups (a batch entry each) of rows_per_group
// consecutive rows, group g starting at a + g * group_stride_a (elements), so that "all time steps
// but the first" of one tensor can be paired with "all but the last" of another without copies.
__global__ __launch_bounds__(256) void cosine_rows_bf16_kernel(const bf16_t* __restrict__ a,
                                                               const bf16_t* __restrict__ b,
                                                               float* __restrict__ out, int64_t rows,
                                                               int64_t rows_per_group, int cols,
                                                               int64_t lda, int64_t ldb,
                                                               int64_t group_stride_a,
                                                               int64_t group_stride_b, float eps) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const int64_t g = row / rows_per_group, r = row % rows_per_group;
  const bf16_t* ar = a + g * group_stride_a + r * lda;
  const bf16_t* br = b + g * group_stride_b + r * ldb;
  float dot = 0.f, na = 0.f, nb = 0.f;
  for (int c = lane * 8; c < cols; c += 512) {
    float x[8], y[8];
    vec8<bf16_t>::load(ar + c, x);
    vec8<bf16_t>::load(br + c, y);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      dot += x[i] * y[i];
      na += x[i] * x[i];
      nb += y[i] * y[i];
    }
  }
  dot = wave_sum(dot);
  na = wave_sum(na);
  nb = wave_sum(nb);
  if (lane == 0) out[row] = dot / (fmaxf(sqrtf(na), eps) * fmaxf(sqrtf(nb), eps));
}

// sum = bf16(a + b + c) and norm = RMSNorm(sum) * w in one pass over the three inputs: the
// residual update of one block fused with the input norm of the next.  The norm is taken over
// the ROUNDED sum, so the result equals the two separate kernels bit for bit.
template <int CHUNKS>     // 16-byte chunks per lane kept in registers (cols <= 512 * CHUNKS); 0 = re-read the sum
__global__ __launch_bounds__(256) void add3_rmsnorm_bf16_kernel(
    const bf16_t* __restrict__ a, const bf16_t* __restrict__ b, const bf16_t* __restrict__ c,
    const float* __restrict__ w, bf16_t* __restrict__ sum, bf16_t* __restrict__ norm, int64_t rows,
    int cols, float eps) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const int64_t base = row * cols;
  float ss = 0.f;
  if constexpr (CHUNKS > 0) {
    float keep[CHUNKS][8];
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      const int col = lane * 8 + 512 * j;
      if (col < cols) {
        float vb[8], vc[8];
        vec8<bf16_t>::load(a + base + col, keep[j]);
        vec8<bf16_t>::load(b + base + col, vb);
        vec8<bf16_t>::load(c + base + col, vc);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          keep[j][i] = bf16_to_f32(f32_to_bf16(keep[j][i] + vb[i] + vc[i]));
          ss += keep[j][i] * keep[j][i];
        }
        vec8<bf16_t>::store(sum + base + col, keep[j]);
      }
    }
    const float inv = rsqrtf(wave_sum(ss) / (float)cols + eps);
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      const int col = lane * 8 + 512 * j;
      if (col < cols) {
        float g[8];
        vec8<float>::load(w + col, g);
#pragma unroll
        for (int i = 0; i < 8; ++i) keep[j][i] = keep[j][i] * inv * g[i];
        vec8<bf16_t>::store(norm + base + col, keep[j]);
      }
    }
    return;
  }
  for (int col = lane * 8; col < cols; col += 512) {
    float va[8], vb[8], vc[8];
    vec8<bf16_t>::load(a + base + col, va);
    vec8<bf16_t>::load(b + base + col, vb);
    vec8<bf16_t>::load(c + base + col, vc);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      va[i] = bf16_to_f32(f32_to_bf16(va[i] + vb[i] + vc[i]));
      ss += va[i] * va[i];
    }
    vec8<bf16_t>::store(sum + base + col, va);
  }
  const float inv = rsqrtf(wave_sum(ss) / (float)cols + eps);
  for (int col = lane * 8; col < cols; col += 512) {
    float v[8], g[8];
    vec8<bf16_t>::load(sum + base + col, v);      // this lane's own stores, read back
    vec8<float>::load(w + col, g);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = v[i] * inv * g[i];
    vec8<bf16_t>::store(norm + base + col, v);
  }
}

__global__ __launch_bounds__(256) void add3_bf16_vec_kernel(const bf16_t* __restrict__ a,
                                                            const bf16_t* __restrict__ b,
                                                            const bf16_t* __restrict__ c,
                                                            bf16_t* __restrict__ o, int64_t n8) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  float va[8], vb[8], vc[8];
  vec8<bf16_t>::load(a + i * 8, va);
  vec8<bf16_t>::load(b + i * 8, vb);
  vec8<bf16_t>::load(c + i * 8, vc);
#pragma unroll
  for (int k = 0; k < 8; ++k) va[k] += vb[k] + vc[k];
  vec8<bf16_t>::store(o + i * 8, va);
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

// One new time step of keys and values into the slot *head of two ring buffers
// [B,Hkv,steps,C,Dh]: k_new / v_new are [B,Hkv,C,Dh] views (element strides sb, sh, sc, unit
// last stride) of the projection output.  One thread per 16 bytes.
__global__ __launch_bounds__(256) void ring_append_bf16_kernel(
    const bf16_t* __restrict__ k_new, const bf16_t* __restrict__ v_new, bf16_t* __restrict__ k_ring,
    bf16_t* __restrict__ v_ring, const int32_t* __restrict__ head, int Hkv, int C, int Dh, int steps,
    int64_t sb, int64_t sh, int64_t sc, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int d8 = Dh / 8;
  const int d = (int)(i % d8) * 8;
  const int c = (int)((i / d8) % C);
  const int h = (int)((i / ((int64_t)d8 * C)) % Hkv);
  const int64_t b = i / ((int64_t)d8 * C * Hkv);
  const int slot = *head;
  const int64_t src = b * sb + h * sh + c * sc + d;
  const int64_t dst = (((b * Hkv + h) * steps + slot) * C + c) * Dh + d;
  *(u32x4*)(k_ring + dst) = *(const u32x4*)(k_new + src);
  *(u32x4*)(v_ring + dst) = *(const u32x4*)(v_new + src);
}

// -----------------------------------------------------------------------------------------
// y[M,N] = x[M,K] w[N,K]^T in fp32 (v_mfma_f32_32x32x2_f32): the projections of the fp32 layer
// path (the small fp32 configuration: plumbing and golden outputs), so that they too run in this
// library.  64 x 64 tile, 4 waves of one 32 x 32 block each, 32-wide k-blocks staged in LDS
// (rows padded by one float against bank conflicts).  Any M, N, K.
// -----------------------------------------------------------------------------------------
constexpr int F32_BK = 32, F32_PITCH = F32_BK + 1;

__global__ __launch_bounds__(256) void linear_f32_kernel(const float* __restrict__ X, const float* __restrict__ W,
                                                         float* __restrict__ Y, int64_t M, int64_t N, int64_t K,
                                                         int64_t ldx, int64_t ldw, int64_t ldy) {
  __shared__ float xs[64 * F32_PITCH], ws[64 * F32_PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, hh = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t m0 = (int64_t)blockIdx.y * 64, n0 = (int64_t)blockIdx.x * 64;
  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  for (int64_t k0 = 0; k0 < K; k0 += F32_BK) {
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int e = it * 256 + tid, r = e / F32_BK, c = e % F32_BK;
      const int64_t k = k0 + c;
      xs[r * F32_PITCH + c] = (m0 + r < M && k < K) ? X[(m0 + r) * ldx + k] : 0.f;
      ws[r * F32_PITCH + c] = (n0 + r < N && k < K) ? W[(n0 + r) * ldw + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int s2 = 0; s2 < F32_BK / 2; ++s2) {
      const float av = xs[(wm * 32 + ln) * F32_PITCH + 2 * s2 + hh];
      const float bv = ws[(wn * 32 + ln) * F32_PITCH + 2 * s2 + hh];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
    }
  }
  const int64_t n = n0 + wn * 32 + ln;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t m = m0 + wm * 32 + (i >> 2) * 8 + hh * 4 + (i & 3);
    if (m < M && n < N) Y[m * ldy + n] = acc[i];
  }
}

}  // namespace mvpa

using namespace mvpa;

template <int EPI, int XT>
static int launch_skinny(const bf16_t* x, const bf16_t* w, bf16_t* y, int64_t M, int64_t N, int64_t K,
                         int64_t ldx, int64_t ldw, int64_t ldy, hipStream_t s) {
  constexpr int lds = SK_WAVES * XT * 16 * 64 * (int)sizeof(float);
  auto kern = linear_bf16_skinny_kernel<EPI, XT>;
  if (lds > 64 * 1024)
    mvpa::want_dynamic_lds((const void*)kern, (int)lds);
  MVPA_LAUNCH(kern, dim3((unsigned)((N + 31) / 32)), dim3(SK_WAVES * 64), lds, s, x, w, y, M, N, K, ldx, ldw, ldy);
  return mvpa::take_launch_status();
}

// K slices per workgroup and the number of workgroup rows that follows: as few partial tiles as
// still give every CU a workgroup (about 256 in all)
static void splitk_groups(int64_t nw, int64_t K, int* per_group, int* groups) {
  const int64_t slices = (K + SPK_KS - 1) / SPK_KS, col_tiles = (nw + SPK_COLS - 1) / SPK_COLS;
  int64_t g = (256 + col_tiles - 1) / col_tiles;          // workgroup rows wanted
  if (g > slices) g = slices;
  if (g < 1) g = 1;
  *per_group = (int)((slices + g - 1) / g);
  *groups = (int)((slices + *per_group - 1) / *per_group);
}

extern "C" size_t mvpa_linear_splitk_ws_bytes(int64_t M, int64_t N, int64_t K, int32_t epilogue) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const int64_t nw = epilogue == 1 ? 2 * N : N;
  int per_group, groups;
  splitk_groups(nw, K, &per_group, &groups);
  return (size_t)((int64_t)groups * M * nw) * sizeof(float);
}

extern "C" int mvpa_linear_bf16_splitk(const void* x, const void* w, void* y, int64_t M, int64_t N,
                                       int64_t K, int64_t ldx, int64_t ldw, int64_t ldy,
                                       int32_t epilogue, void* ws, size_t ws_bytes, void* stream) {
  if (!x || !w || !y || !ws) return MVPA_ERR_NULL;
  if (M <= 0 || M > SPK_XROWS || N <= 0 || K <= 0 || ldx < K || ldw < K || ldy < N) return MVPA_ERR_SHAPE;
  if (((uintptr_t)x & 15) || ((uintptr_t)w & 15) || ((uintptr_t)ws & 15) || (ldx & 7) || (ldw & 7))
    return MVPA_ERR_ALIGN;
  if (epilogue != 0 && epilogue != 1) return MVPA_ERR_UNSUPPORTED;
  if (ws_bytes < mvpa_linear_splitk_ws_bytes(M, N, K, epilogue)) return MVPA_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const int64_t nw = epilogue == 1 ? 2 * N : N;
  int per_group, slices;          // slices: partial tiles per output tile = workgroup rows
  splitk_groups(nw, K, &per_group, &slices);
  mvpa::want_dynamic_lds((const void*)linear_splitk_kernel, (int)SPK_LDS_BYTES);
  MVPA_LAUNCH(linear_splitk_kernel, dim3((unsigned)((nw + SPK_COLS - 1) / SPK_COLS), (unsigned)slices), dim3(256),
                     SPK_LDS_BYTES, s, (const bf16_t*)x, (const bf16_t*)w, (float*)ws, M, nw, K, ldx, ldw, per_group);
  const int64_t items = M * ((N + 3) / 4);
  if (epilogue == 1)
    MVPA_LAUNCH(linear_splitk_reduce_kernel<1>, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s,
                       (const float*)ws, (bf16_t*)y, M, N, nw, slices, ldy);
  else
    MVPA_LAUNCH(linear_splitk_reduce_kernel<0>, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s,
                       (const float*)ws, (bf16_t*)y, M, N, nw, slices, ldy);
  return mvpa::take_launch_status();
}

extern "C" int mvpa_linear_bf16(const void* x, const void* w, void* y, int64_t M, int64_t N,
                                int64_t K, int64_t ldx, int64_t ldw, int64_t ldy,
                                int32_t epilogue, void* stream) {
  if (!x || !w || !y) return MVPA_ERR_NULL;
  if (M <= 0 || N <= 0 || K <= 0 || ldx < K || ldw < K || ldy < N) return MVPA_ERR_SHAPE;
  if (((uintptr_t)x & 15) || ((uintptr_t)w & 15) || (ldx & 7) || (ldw & 7)) return MVPA_ERR_ALIGN;
  if (epilogue != 0 && epilogue != 1) return MVPA_ERR_UNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  const bf16_t *xp = (const bf16_t*)x, *wp = (const bf16_t*)w;
  bf16_t* yp = (bf16_t*)y;
  // large tiles when there is enough work and rows can be fetched in whole 16-byte chunks;
  // the tile width is the one that needs the fewest (workgroup rounds x width) on 256 CUs
  if (M >= 512 && (K & 7) == 0 && (ldy & 3) == 0 && ((uintptr_t)y & 7) == 0) {
    const int64_t mt = (M + 255) / 256;
    auto cost = [&](int bn, int out_cols) -> int64_t {
      const int64_t wgs = mt * ((N + out_cols - 1) / out_cols);
      return ((wgs + 255) / 256) * bn;
    };
    // the four-stage ring needs whole k-blocks of 32 and 32-bit byte offsets from a tile's first rows
    const bool ring = (K & 31) == 0 && K >= 96 && 256 * ldx < ((int64_t)1 << 30) &&
                      (epilogue == 1 ? 2 * N : (int64_t)256) * ldw < ((int64_t)1 << 30);
    // whole cache lines per request where K is a multiple of 64
    const bool pair = ring && (K & 63) == 0 && K >= 128;
    if (epilogue == 1) {
      // (the wider tile unless it costs a fifth more: [16384 x 768] x [768 x 3456] 114 -> 103 us)
      if (cost(256, 128) * 5 <= cost(128, 64) * 6)
        return pair ? launch_pair<256, 1>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s)
           : ring ? launch_ring<256, 1>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s)
                    : launch_big<256, 1>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s);
      return pair ? launch_pair<128, 1>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s)
           : ring ? launch_ring<128, 1>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s)
                  : launch_big<128, 1>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s);
    }
    const int64_t c256 = cost(256, 256), c192 = cost(192, 192), c128 = cost(128, 128);
    if (c256 <= c192 && c256 <= c128)
      return pair ? launch_pair<256, 0>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s)
           : ring ? launch_ring<256, 0>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s)
                  : launch_big<256, 0>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s);
    if (c192 <= c128)
      return pair ? launch_pair<192, 0>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s)
           : ring ? launch_ring<192, 0>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s)
                  : launch_big<192, 0>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s);
    return pair ? launch_pair<128, 0>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s)
           : ring ? launch_ring<128, 0>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s)
                : launch_big<128, 0>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s);
  }
  if (M <= 128) {
    // one decoding step's worth of rows: weight-read bound, spread over N/32 workgroups
    return M <= 64 ? (epilogue == 1 ? launch_skinny<1, 2>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s)
                                    : launch_skinny<0, 2>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s))
                   : (epilogue == 1 ? launch_skinny<1, 4>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s)
                                    : launch_skinny<0, 4>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s));
  }
  if (epilogue == 1) {
    dim3 grid((unsigned)((N + GBN / 2 - 1) / (GBN / 2)), (unsigned)((M + GBM - 1) / GBM));
    MVPA_LAUNCH(linear_bf16_kernel<1>, grid, dim3(256), 0, s, xp, wp, yp, M, N, K, ldx, ldw, ldy);
  } else {
    dim3 grid((unsigned)((N + GBN - 1) / GBN), (unsigned)((M + GBM - 1) / GBM));
    MVPA_LAUNCH(linear_bf16_kernel<0>, grid, dim3(256), 0, s, xp, wp, yp, M, N, K, ldx, ldw, ldy);
  }
  return mvpa::take_launch_status();
}

extern "C" int mvpa_linear_f32(const float* x, const float* w, float* y, int64_t M, int64_t N, int64_t K,
                               int64_t ldx, int64_t ldw, int64_t ldy, void* stream) {
  if (!x || !w || !y) return MVPA_ERR_NULL;
  if (M <= 0 || N <= 0 || K <= 0 || ldx < K || ldw < K || ldy < N) return MVPA_ERR_SHAPE;
  MVPA_LAUNCH(mvpa::linear_f32_kernel, dim3((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64)), dim3(256), 0,
              (hipStream_t)stream, x, w, y, M, N, K, ldx, ldw, ldy);
  return mvpa::take_launch_status();
}

// y0 = x w0^T and y1 = silu(x wg^T) * (x wu^T) in one launch (w1 holds the gate rows [0, N1) and
// the up rows [N1, 2 N1)): the two products that read ln_1(x) in the parallel block.  Large
// shapes only: at least 512 rows, K a multiple of 64; MVPA_ERR_UNSUPPORTED otherwise.
// With sumsq given, x holds the RAW rows and their RMSNorm happens in the epilogue
// (mvpa_linear_bf16_dual_normed).
static int linear_dual_impl(const void* x, const void* w0, void* y0, const void* w1, void* y1,
                            int64_t M, int64_t N0, int64_t N1, int64_t K, int64_t ldx,
                            int64_t ldw0, int64_t ldy0, int64_t ldw1, int64_t ldy1,
                            const float* sumsq, int32_t parts, float eps, void* stream) {
  if (!x || !w0 || !y0 || !w1 || !y1) return MVPA_ERR_NULL;
  if (M <= 0 || N0 <= 0 || N1 <= 0 || K <= 0 || ldx < K || ldw0 < K || ldw1 < K || ldy0 < N0 || ldy1 < N1)
    return MVPA_ERR_SHAPE;
  if ((((uintptr_t)x | (uintptr_t)w0 | (uintptr_t)w1) & 15) || (ldx & 7) || (ldw0 & 7) || (ldw1 & 7))
    return MVPA_ERR_ALIGN;
  if (((uintptr_t)y0 | (uintptr_t)y1) & 1) return MVPA_ERR_ALIGN;
  const bool ok = M >= 512 && (K & 63) == 0 && K >= 128 && 256 * ldx < ((int64_t)1 << 30) &&
                  256 * ldw0 < ((int64_t)1 << 30) && 2 * N1 * ldw1 < ((int64_t)1 << 30);
  if (!ok) return MVPA_ERR_UNSUPPORTED;
  const mvpa::linear_pair_problem plain{(const bf16_t*)w0, (bf16_t*)y0, N0, ldw0, ldy0};
  const mvpa::linear_pair_problem gated{(const bf16_t*)w1, (bf16_t*)y1, N1, ldw1, ldy1};
  // the plain product's tile width: the one that wastes the fewest padded columns
  const int64_t pad256 = (N0 + 255) / 256 * 256, pad192 = (N0 + 191) / 192 * 192, pad128 = (N0 + 127) / 128 * 128;
  hipStream_t s = (hipStream_t)stream;
  if (sumsq) {
    const mvpa::row_stats rs{sumsq, parts, 1.f / (float)K, eps, nullptr, 0};
    if (pad256 <= pad192 && pad256 <= pad128)
      return mvpa::launch_pair_dual_normed<256>((const bf16_t*)x, M, K, ldx, plain, gated, rs, s);
    if (pad192 <= pad128) return mvpa::launch_pair_dual_normed<192>((const bf16_t*)x, M, K, ldx, plain, gated, rs, s);
    return mvpa::launch_pair_dual_normed<128>((const bf16_t*)x, M, K, ldx, plain, gated, rs, s);
  }
  if (pad256 <= pad192 && pad256 <= pad128) return launch_pair_dual<256>((const bf16_t*)x, M, K, ldx, plain, gated, s);
  if (pad192 <= pad128) return launch_pair_dual<192>((const bf16_t*)x, M, K, ldx, plain, gated, s);
  return launch_pair_dual<128>((const bf16_t*)x, M, K, ldx, plain, gated, s);
}

extern "C" int mvpa_linear_bf16_dual(const void* x, const void* w0, void* y0, const void* w1, void* y1,
                                     int64_t M, int64_t N0, int64_t N1, int64_t K, int64_t ldx,
                                     int64_t ldw0, int64_t ldy0, int64_t ldw1, int64_t ldy1, void* stream) {
  return linear_dual_impl(x, w0, y0, w1, y1, M, N0, N1, K, ldx, ldw0, ldy0, ldw1, ldy1, nullptr, 0, 0.f, stream);
}

extern "C" int mvpa_linear_bf16_dual_normed(const void* x, const void* w0, void* y0, const void* w1, void* y1,
                                            int64_t M, int64_t N0, int64_t N1, int64_t K, int64_t ldx,
                                            int64_t ldw0, int64_t ldy0, int64_t ldw1, int64_t ldy1,
                                            const float* sumsq, int32_t parts, float eps, void* stream) {
  if (!sumsq) return MVPA_ERR_NULL;
  if (parts <= 0 || parts > 64) return MVPA_ERR_SHAPE;
  return linear_dual_impl(x, w0, y0, w1, y1, M, N0, N1, K, ldx, ldw0, ldy0, ldw1, ldy1, sumsq, parts, eps, stream);
}

// tile width of the residual product for a shape (the one that needs the fewest workgroup rounds x
// width on 256 CUs), and with it the number of partial sums a row gets
static int residual_tile_width(int64_t M, int64_t N) {
  const int64_t mt = (M + 255) / 256;
  auto cost = [&](int bn) -> int64_t { return ((mt * ((N + bn - 1) / bn) + 255) / 256) * bn; };
  const int64_t c256 = cost(256), c192 = cost(192), c128 = cost(128);
  return (c256 <= c192 && c256 <= c128) ? 256 : c192 <= c128 ? 192 : 128;
}

extern "C" int32_t mvpa_linear_sumsq_parts(int64_t M, int64_t N) {
  if (M <= 0 || N <= 0) return 0;
  const int bn = residual_tile_width(M, N);
  return (int32_t)(2 * ((N + bn - 1) / bn));
}

extern "C" int mvpa_linear_bf16_residual_sumsq(const void* x, const void* w, const void* r, void* y, float* sumsq,
                                               int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw,
                                               int64_t ldr, int64_t ldy, void* stream) {
  if (!x || !w || !y || !r || !sumsq) return MVPA_ERR_NULL;
  if (M <= 0 || N <= 0 || K <= 0 || ldx < K || ldw < K || ldy < N || ldr < N) return MVPA_ERR_SHAPE;
  if (((uintptr_t)x & 15) || ((uintptr_t)w & 15) || (ldx & 7) || (ldw & 7)) return MVPA_ERR_ALIGN;
  // whole 16-byte chunks of every output row, so that each takes the vector path of the epilogue
  if (((uintptr_t)y & 15) || ((uintptr_t)r & 15) || (ldy & 7) || (ldr & 7) || (N & 7)) return MVPA_ERR_ALIGN;
  const bool pair = M >= 512 && (K & 63) == 0 && K >= 128 && 256 * ldx < ((int64_t)1 << 30) &&
                    256 * ldw < ((int64_t)1 << 30);
  if (!pair) return MVPA_ERR_UNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  const bf16_t *xp = (const bf16_t*)x, *wp = (const bf16_t*)w, *rp = (const bf16_t*)r;
  const int bn = residual_tile_width(M, N);
  const int32_t parts = (int32_t)(2 * ((N + bn - 1) / bn));
  if (bn == 256) return mvpa::launch_pair_sumsq<256>(xp, wp, (bf16_t*)y, M, N, K, ldx, ldw, ldy, s, rp, ldr, sumsq, parts);
  if (bn == 192) return mvpa::launch_pair_sumsq<192>(xp, wp, (bf16_t*)y, M, N, K, ldx, ldw, ldy, s, rp, ldr, sumsq, parts);
  return mvpa::launch_pair_sumsq<128>(xp, wp, (bf16_t*)y, M, N, K, ldx, ldw, ldy, s, rp, ldr, sumsq, parts);
}

extern "C" int mvpa_row_sumsq_bf16(const void* x, float* sumsq, int64_t rows, int32_t cols, int64_t ldx, void* stream) {
  if (!x || !sumsq) return MVPA_ERR_NULL;
  if (rows <= 0 || cols <= 0 || ldx < cols) return MVPA_ERR_SHAPE;
  if (((uintptr_t)x & 15) || (ldx & 7) || (cols & 7)) return MVPA_ERR_ALIGN;
  MVPA_LAUNCH(mvpa::row_sumsq_bf16_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
              (const bf16_t*)x, sumsq, rows, cols, ldx);
  return mvpa::take_launch_status();
}

// Y = X W^T + R in one kernel (the large-tile ring kernel only): at least 512 rows, K a multiple
// of 32 and at least 96.  Other shapes: MVPA_ERR_UNSUPPORTED (the caller adds R itself).
extern "C" int mvpa_linear_bf16_residual(const void* x, const void* w, const void* r, void* y,
                                         int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw,
                                         int64_t ldr, int64_t ldy, void* stream) {
  if (!x || !w || !y || !r) return MVPA_ERR_NULL;
  if (M <= 0 || N <= 0 || K <= 0 || ldx < K || ldw < K || ldy < N || ldr < N) return MVPA_ERR_SHAPE;
  if (((uintptr_t)x & 15) || ((uintptr_t)w & 15) || (ldx & 7) || (ldw & 7)) return MVPA_ERR_ALIGN;
  if (((uintptr_t)y & 1) || ((uintptr_t)r & 1)) return MVPA_ERR_ALIGN;
  const bool ring = M >= 512 && (K & 31) == 0 && K >= 96 && 256 * ldx < ((int64_t)1 << 30) &&
                    256 * ldw < ((int64_t)1 << 30);
  if (!ring) return MVPA_ERR_UNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  const bf16_t *xp = (const bf16_t*)x, *wp = (const bf16_t*)w, *rp = (const bf16_t*)r;
  bf16_t* yp = (bf16_t*)y;
  const int64_t mt = (M + 255) / 256;
  auto cost = [&](int bn) -> int64_t { return ((mt * ((N + bn - 1) / bn) + 255) / 256) * bn; };
  const int64_t c256 = cost(256), c192 = cost(192), c128 = cost(128);
  const bool pair = (K & 63) == 0 && K >= 128;
  if (c256 <= c192 && c256 <= c128)
    return pair ? launch_pair<256, 2>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s, rp, ldr)
                : launch_ring<256, 2>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s, rp, ldr);
  if (c192 <= c128)
    return pair ? launch_pair<192, 2>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s, rp, ldr)
                : launch_ring<192, 2>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s, rp, ldr);
  return pair ? launch_pair<128, 2>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s, rp, ldr)
              : launch_ring<128, 2>(xp, wp, yp, M, N, K, ldx, ldw, ldy, s, rp, ldr);
}

extern "C" int mvpa_rmsnorm(const void* x, const float* weight, void* y, int64_t rows,
                            int32_t cols, int64_t ldx, int64_t ldy, float eps, int32_t in_dtype,
                            int32_t out_dtype, void* stream) {
  if (!x || !weight || !y) return MVPA_ERR_NULL;
  if (rows <= 0 || cols <= 0 || ldx < cols || ldy < cols) return MVPA_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((unsigned)rows), block(256);
  const int in_b = in_dtype == MVPA_F32 ? 4 : 2, out_b = out_dtype == MVPA_F32 ? 4 : 2;
  const bool vec_ok = (in_dtype == MVPA_F32 || in_dtype == MVPA_BF16) &&
                      (out_dtype == MVPA_F32 || out_dtype == MVPA_BF16) && cols % 8 == 0 &&
                      (((uintptr_t)x | (uintptr_t)y | (uintptr_t)weight) & 15) == 0 &&
                      (ldx * in_b) % 16 == 0 && (ldy * out_b) % 16 == 0;
  if (vec_ok) {
    dim3 vgrid((unsigned)((rows + 3) / 4));
    if (in_dtype == MVPA_F32 && out_dtype == MVPA_F32)
      MVPA_LAUNCH((rmsnorm_rows_kernel<float, float>), vgrid, block, 0, s, (const float*)x, weight, (float*)y, rows, cols, ldx, ldy, eps);
    else if (in_dtype == MVPA_F32)
      MVPA_LAUNCH((rmsnorm_rows_kernel<float, bf16_t>), vgrid, block, 0, s, (const float*)x, weight, (bf16_t*)y, rows, cols, ldx, ldy, eps);
    else if (out_dtype == MVPA_BF16)
      MVPA_LAUNCH((rmsnorm_rows_kernel<bf16_t, bf16_t>), vgrid, block, 0, s, (const bf16_t*)x, weight, (bf16_t*)y, rows, cols, ldx, ldy, eps);
    else
      MVPA_LAUNCH((rmsnorm_rows_kernel<bf16_t, float>), vgrid, block, 0, s, (const bf16_t*)x, weight, (float*)y, rows, cols, ldx, ldy, eps);
    return mvpa::take_launch_status();
  }
  if (in_dtype == MVPA_F32 && out_dtype == MVPA_F32)
    MVPA_LAUNCH((rmsnorm_kernel<float, float>), grid, block, 0, s, (const float*)x, weight, (float*)y, cols, ldx, ldy, eps);
  else if (in_dtype == MVPA_F32 && out_dtype == MVPA_BF16)
    MVPA_LAUNCH((rmsnorm_kernel<float, bf16_t>), grid, block, 0, s, (const float*)x, weight, (bf16_t*)y, cols, ldx, ldy, eps);
  else if (in_dtype == MVPA_BF16 && out_dtype == MVPA_BF16)
    MVPA_LAUNCH((rmsnorm_kernel<bf16_t, bf16_t>), grid, block, 0, s, (const bf16_t*)x, weight, (bf16_t*)y, cols, ldx, ldy, eps);
  else if (in_dtype == MVPA_BF16 && out_dtype == MVPA_F32)
    MVPA_LAUNCH((rmsnorm_kernel<bf16_t, float>), grid, block, 0, s, (const bf16_t*)x, weight, (float*)y, cols, ldx, ldy, eps);
  else
    return MVPA_ERR_DTYPE;
  return mvpa::take_launch_status();
}

extern "C" int mvpa_cosine_rows_bf16(const void* a, const void* b, float* out, int64_t groups,
                                     int64_t rows_per_group, int32_t cols, int64_t lda, int64_t ldb,
                                     int64_t group_stride_a, int64_t group_stride_b, float eps,
                                     void* stream) {
  if (!a || !b || !out) return MVPA_ERR_NULL;
  if (groups <= 0 || rows_per_group <= 0 || cols <= 0 || lda < cols || ldb < cols) return MVPA_ERR_SHAPE;
  if ((cols & 7) || (lda & 7) || (ldb & 7) || (group_stride_a & 7) || (group_stride_b & 7) ||
      (((uintptr_t)a | (uintptr_t)b) & 15))
    return MVPA_ERR_ALIGN;
  const int64_t rows = groups * rows_per_group;
  MVPA_LAUNCH(cosine_rows_bf16_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
              (const bf16_t*)a, (const bf16_t*)b, out, rows, rows_per_group, cols, lda, ldb,
              group_stride_a, group_stride_b, eps);
  return mvpa::take_launch_status();
}

extern "C" int mvpa_add3_bf16(const void* a, const void* b, const void* c, void* out, int64_t n,
                              void* stream) {
  if (!a || !b || !c || !out) return MVPA_ERR_NULL;
  if (n <= 0) return MVPA_ERR_SHAPE;
  if (n % 8 == 0 && (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c | (uintptr_t)out) & 15) == 0) {
    const int64_t n8 = n / 8;
    MVPA_LAUNCH(add3_bf16_vec_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (const bf16_t*)a, (const bf16_t*)b, (const bf16_t*)c,
                       (bf16_t*)out, n8);
    return mvpa::take_launch_status();
  }
  MVPA_LAUNCH(add3_bf16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, (const bf16_t*)a, (const bf16_t*)b, (const bf16_t*)c,
                     (bf16_t*)out, n);
  return mvpa::take_launch_status();
}

extern "C" int mvpa_ring_append_bf16(const void* k_new, const void* v_new, void* k_ring, void* v_ring,
                                     const int32_t* head, int32_t B, int32_t Hkv, int32_t C, int32_t Dh,
                                     int32_t steps, int64_t stride_b, int64_t stride_h, int64_t stride_c,
                                     void* stream) {
  if (!k_new || !v_new || !k_ring || !v_ring || !head) return MVPA_ERR_NULL;
  if (B <= 0 || Hkv <= 0 || C <= 0 || Dh <= 0 || steps <= 0) return MVPA_ERR_SHAPE;
  if (Dh % 8 != 0 || ((stride_b | stride_h | stride_c) & 7) ||
      (((uintptr_t)k_new | (uintptr_t)v_new | (uintptr_t)k_ring | (uintptr_t)v_ring) & 15))
    return MVPA_ERR_ALIGN;
  const int64_t total = (int64_t)B * Hkv * C * (Dh / 8);
  MVPA_LAUNCH(ring_append_bf16_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, (const bf16_t*)k_new, (const bf16_t*)v_new, (bf16_t*)k_ring,
                     (bf16_t*)v_ring, head, Hkv, C, Dh, steps, stride_b, stride_h, stride_c, total);
  return mvpa::take_launch_status();
}

extern "C" int mvpa_add3_rmsnorm_bf16(const void* a, const void* b, const void* c,
                                      const float* weight, void* sum, void* norm, int64_t rows,
                                      int32_t cols, float eps, void* stream) {
  if (!a || !b || !c || !weight || !sum || !norm) return MVPA_ERR_NULL;
  if (rows <= 0 || cols <= 0) return MVPA_ERR_SHAPE;
  if (cols % 8 != 0 || (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c | (uintptr_t)sum |
                         (uintptr_t)norm | (uintptr_t)weight) & 15) != 0)
    return MVPA_ERR_ALIGN;
  auto kern = cols <= 1024 ? add3_rmsnorm_bf16_kernel<2> : cols <= 2048 ? add3_rmsnorm_bf16_kernel<4>
                                                                        : add3_rmsnorm_bf16_kernel<0>;
  MVPA_LAUNCH(kern, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0,
                     (hipStream_t)stream, (const bf16_t*)a, (const bf16_t*)b, (const bf16_t*)c,
                     weight, (bf16_t*)sum, (bf16_t*)norm, rows, cols, eps);
  return mvpa::take_launch_status();
}

extern "C" int mvpa_wavedec_db4(const float* x, float* coeffs, int64_t M, int32_t L,
                                int32_t levels, int32_t dwt_size, int64_t ldc, void* stream) {
  if (!x || !coeffs) return MVPA_ERR_NULL;
  if (M <= 0 || L < 8 || levels < 1 || L > 16384 || ldc < dwt_size) return MVPA_ERR_SHAPE;
  int n = L, total = 0;
  for (int lv = 0; lv < levels; ++lv) { n = (n + 7) >> 1; total += n; }
  total += n;
  if (total != dwt_size) return MVPA_ERR_SHAPE;
  // two ping-pong rows of L floats: past 64 KiB of dynamic LDS the kernel has to be told
  if (2 * L * sizeof(float) > 64 * 1024)
    mvpa::want_dynamic_lds((const void*)wavedec_db4_kernel, (int)(2 * L * sizeof(float)));
  MVPA_LAUNCH(wavedec_db4_kernel, dim3((unsigned)M), dim3(256), 2 * L * sizeof(float),
                     (hipStream_t)stream, x, coeffs, L, levels, dwt_size, ldc);
  return mvpa::take_launch_status();
}
