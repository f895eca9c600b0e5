// MVPA backward on MFMA (bf16, Dh = 64, C <= 64): the QUERY pass (the KEY pass follows below).
//
// Same tiling as the forward kernel: queries and keys are tiled by time step, a wave owns 32
// query channels of one time step, products are formed transposed (a lane owns one query), the
// channel-bias tile is built once per wave and used as the C operand of K Q^T, the time bias is
// one scalar per (query, key step) taken from 32-step slabs.  With the forward's base-2
// log-sum-exp L nothing is "online" here: per key step
//     S^T  = K (q+u)^T + Bc + st          (content product only inside the window)
//     P^T  = exp2(S^T - L)
//     dP^T = V dO^T
//     dS^T = P^T o (dP^T - delta) * scale,          delta = dO . O
//     dq^T += K^T dS^T                     (inside the window)
//     dbias_time[q, tk] = sum_ck dS,       dbias_chan[q, |cq-ck|] += dS.
// Outputs and workspace are those of mvpa_backward (include/mvpa_hip.h): the content share of dq,
// the two bias-table gradients, delta, and the forward bias tables in natural units for the key
// pass.  K and V tiles are staged through LDS once per key step for the whole workgroup, K in two
// copies (row fragments for K Q^T, transposed fragments for K^T dS^T).
#include "mvpa_common.h"

namespace mvpa {
namespace bwdq {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

#define BWD_LDS_PTR(T) __attribute__((address_space(3))) T*

constexpr int DH = 64, KS = 4, MT = 2, ROWB = 128, NW = 4;

__device__ inline void wave_sync_lds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ inline bf16x8 as_frag(u32x4 v) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = v;
  return c.b;
}

// 8 bf16 of a q row + bias, scaled, as an MFMA fragment
__device__ inline bf16x8 qfrag(u32x4 raw, const bf16_t* __restrict__ bias, float scale) {
  const u32x4 braw = *(const u32x4*)bias;
  bf16x8 out;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t w = raw[i], bw = braw[i];
    out[2 * i] = (__bf16)((__uint_as_float(w << 16) + __uint_as_float(bw << 16)) * scale);
    out[2 * i + 1] = (__bf16)((__uint_as_float(w & 0xffff0000u) + __uint_as_float(bw & 0xffff0000u)) * scale);
  }
  return out;
}

__device__ inline bf16x8 pack8(const f32x16& v, int base) {
  bf16x8 out;
#pragma unroll
  for (int i = 0; i < 8; ++i) out[i] = (__bf16)v[base + i];
  return out;
}

__device__ inline float xhalf_sum(float x) { return x + __shfl_xor(x, 32); }

// chunk swizzles of a 128-byte row: row fragments / transposing reads (as in the forward)
__device__ inline int swz_row(int row) { return (row >> 1) & 7; }
__device__ inline int swz_tr(int row) { return ((row >> 1) & 1) << 2; }

template <int NCT>
__global__ __launch_bounds__(NW * 64) void mvpa_bwd_query_mfma_kernel(mvpa_bwd_args a) {
  constexpr int CP = NCT * 32, TQW = NW / NCT, TILE = CP * ROWB;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char* Krow = smem;                     // K tile, row-fragment swizzle
  unsigned char* Ktr = smem + TILE;               // K tile, transposing-read swizzle
  unsigned char* Vrow = smem + 2 * TILE;          // V tile, row-fragment swizzle
  float* wave_base = (float*)(smem + 3 * TILE);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, hh = lane >> 5;
  float* Stb = wave_base + wave * (2 * 1024 + CP * 32);   // [32][32] time-bias scores of a slab
  float* Gtb = Stb + 1024;                                // [32][32] their gradients
  float* scr = Gtb + 1024;                                // [CP][32] channel table, later [32][CP]

  const int T_ = a.T, C_ = a.C, W = a.window, N = a.T * a.C;
  const bool has_content = a.flags & MVPA_FLAG_CONTENT;
  const bool has_time = a.flags & MVPA_FLAG_TIME_BIAS;
  const bool has_chan = a.flags & MVPA_FLAG_CHAN_BIAS;
  const int nt = (T_ + TQW - 1) / TQW;
  const int tile = nt - 1 - (int)blockIdx.x;      // long tiles first
  const int bh = blockIdx.y;
  const int b = bh / a.H, h = bh % a.H;
  const int g = h / (a.H / a.Hkv);
  const int tq0 = tile * TQW;
  const int tq_hi = min(T_ - 1, tq0 + TQW - 1);
  const int tq = tq0 + wave / NCT;
  const bool active = tq < T_;
  const int cq = (wave % NCT) * 32 + ln;
  const bool qok = active && cq < C_;
  const int nq = active ? tq * C_ + min(cq, C_ - 1) : 0;
  const int64_t row = ((int64_t)b * a.H + h) * N + nq;

  const bf16_t* qrow = (const bf16_t*)a.q + b * a.q_stride_b + h * a.q_stride_h + (int64_t)nq * a.q_stride_n;
  const bf16_t* orow = (const bf16_t*)a.o + b * a.o_stride_b + h * a.o_stride_h + (int64_t)nq * a.o_stride_n;
  const bf16_t* drow = (const bf16_t*)a.d_o + b * a.do_stride_b + h * a.do_stride_h + (int64_t)nq * a.do_stride_n;
  const bf16_t* kbase = (const bf16_t*)a.k + b * a.k_stride_b + g * a.k_stride_h;
  const bf16_t* vbase = (const bf16_t*)a.v + b * a.v_stride_b + g * a.v_stride_h;
  const bf16_t* ktime = (const bf16_t*)a.k_time + (int64_t)g * T_ * DH;
  const bf16_t* kchan = (const bf16_t*)a.k_chan + (int64_t)g * C_ * DH;
  const bf16_t* bu = (const bf16_t*)a.bias_u + g * DH;
  const bf16_t* bv = (const bf16_t*)a.bias_v + g * DH;
  const bf16_t* bz = (const bf16_t*)a.bias_z + g * DH;
  const uint8_t* valid = a.chan_valid ? a.chan_valid + (int64_t)b * C_ : nullptr;
  const float sc2 = a.sm_scale * kLog2e;          // scores live in the base-2 domain
  const float inv_sc2 = 1.f / sc2;

  // ---- set-up: operand fragments, delta, channel-bias tile
  bf16x8 Qu[KS], Qv[KS], dOf[KS];
  f32x16 Bc[NCT];
  float delta = 0.f;
  uint32_t kbits[NCT];
  {
    f32x16 sct[NCT];
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) sct[t][i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 16 + hh * 8;
      const u32x4 raw = *(const u32x4*)(qrow + d0);
      const u32x4 draw = *(const u32x4*)(drow + d0);
      const u32x4 oraw = *(const u32x4*)(orow + d0);
      Qu[ks] = qfrag(raw, bu + d0, sc2);
      Qv[ks] = qfrag(raw, bv + d0, sc2);
      const bf16x8 qz = qfrag(raw, bz + d0, sc2);
      dOf[ks] = as_frag(draw);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        delta += __uint_as_float(draw[i] << 16) * __uint_as_float(oraw[i] << 16);
        delta += __uint_as_float(draw[i] & 0xffff0000u) * __uint_as_float(oraw[i] & 0xffff0000u);
      }
#pragma unroll
      for (int t = 0; t < NCT; ++t) {
        const int j = min(t * 32 + ln, C_ - 1);
        const u32x4 er = *(const u32x4*)(kchan + (int64_t)j * DH + d0);
        sct[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(er), qz, sct[t], 0, 0, 0);
      }
    }
    delta = xhalf_sum(delta);
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int j = t * 32 + (i >> 2) * 8 + hh * 4 + (i & 3);
        scr[j * 32 + ln] = has_chan ? sct[t][i] : 0.f;
      }
    uint64_t kmask[2];
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      const int ck = w * 64 + lane;
      bool ok = ck < C_;
      if (valid) ok = ok && valid[min(ck, C_ - 1)] != 0;
      kmask[w] = __ballot(ok);
    }
#pragma unroll
    for (int t = 0; t < NCT; ++t) kbits[t] = (uint32_t)(kmask[t >> 1] >> ((t & 1) * 32 + 4 * hh));
    wave_sync_lds();
    const uint32_t cq4 = (uint32_t)(cq - 4 * hh + 4);
    const int gbase = ((C_ - 1) * 32 + ln) * 4;
    const unsigned char* scr_b = (const unsigned char*)scr;
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint32_t ci4 = (uint32_t)(t * 32 + (i >> 2) * 8 + (i & 3) + 4);
        const uint32_t dist = min(max(cq4, ci4) - min(cq4, ci4), (uint32_t)(C_ - 1));
        const float val = *(const float*)(scr_b + (gbase - (int)(dist * 128u)));
        const bool kv = (kbits[t] >> ((i >> 2) * 8 + (i & 3))) & 1u;
        Bc[t][i] = kv ? val : -INFINITY;
      }
    // forward tables for the key pass, natural units; rows of dbias_time that no key step reaches
    if (qok && hh == 0) {
      a.ws_delta[row] = delta;
      for (int i = 0; i < C_; ++i) a.ws_chan[row * C_ + i] = scr[i * 32 + ln] * inv_sc2;
      for (int j = 0; j < T_ - 1 - tq; ++j) a.dbias_time[row * T_ + j] = 0.f;
    }
    wave_sync_lds();
  }
  const float lse = a.lse[row];

  f32x16 dq[MT], dSc[NCT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) dq[mt][i] = 0.f;
#pragma unroll
  for (int t = 0; t < NCT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) dSc[t][i] = 0.f;

  // ---- loop-invariant fragment offsets
  int r_lane[KS], t_lane[MT];
  {
    const int e = (ln & 15) >> 2, aa = ln & 3, grp = ln >> 4;
    const int row0 = 4 * hh + e;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) r_lane[ks] = ln * ROWB + (((2 * ks + hh) ^ swz_row(ln)) << 4);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      t_lane[mt] = row0 * ROWB + (((4 * mt + 2 * grp + (aa >> 1)) ^ swz_tr(row0)) << 4) + ((aa & 1) << 3);
  }
  auto tr_frag = [&](const unsigned char* tile_p, int t, int s, int mt) -> bf16x8 {
    const unsigned char* p = tile_p + t_lane[mt] + (32 * t + 16 * s) * ROWB;
    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((BWD_LDS_PTR(bf16x4))p);
    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((BWD_LDS_PTR(bf16x4))(p + 8 * ROWB));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };

  // writes the gradients of the slab that started at key step tk0 (and its forward scores)
  auto flush_slab = [&](int tk0) {
    if (hh == 0 && qok) {
      for (int jj = 0; jj < 32; ++jj) {
        const int tkk = tk0 + jj;
        if (tkk > tq) break;
        const int j = time_row(tq, tkk, T_);
        a.dbias_time[row * T_ + j] = Gtb[jj * 32 + ln];
        a.ws_time[row * T_ + j] = Stb[jj * 32 + ln] * inv_sc2;
      }
    }
  };

  // per-thread shares of the cooperative tile load: 16-byte chunk c of row r, twice per tile
  constexpr int CHUNKS = CP * 8;                  // 16-byte chunks per tile
  for (int tk = 0; tk <= tq_hi; ++tk) {
    __syncthreads();                              // everyone is done with the previous tiles
    for (int c = tid; c < CHUNKS; c += NW * 64) {
      const int r = c >> 3, ch = c & 7;
      const int rc = min(r, C_ - 1);
      const int64_t n = (int64_t)tk * C_ + rc;
      const u32x4 kk = *(const u32x4*)(kbase + n * a.k_stride_n + ch * 8);
      const u32x4 vv = *(const u32x4*)(vbase + n * a.v_stride_n + ch * 8);
      *(u32x4*)(Krow + r * ROWB + ((ch ^ swz_row(r)) << 4)) = kk;
      *(u32x4*)(Ktr + r * ROWB + ((ch ^ swz_tr(r)) << 4)) = kk;
      *(u32x4*)(Vrow + r * ROWB + ((ch ^ swz_row(r)) << 4)) = vv;
    }
    __syncthreads();
    if (!active || tk > tq) continue;             // the workgroup's other time step runs longer

    if ((tk & 31) == 0) {
      if (tk > 0) {
        wave_sync_lds();
        flush_slab(tk - 32);
        wave_sync_lds();
      }
      f32x16 stc;
#pragma unroll
      for (int i = 0; i < 16; ++i) stc[i] = 0.f;
      if (has_time) {
        const int j = min(time_row(tq, tk, T_) + ln, T_ - 1);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const u32x4 rr = *(const u32x4*)(ktime + (int64_t)j * DH + ks * 16 + hh * 8);
          stc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(rr), Qv[ks], stc, 0, 0, 0);
        }
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) Stb[((i >> 2) * 8 + hh * 4 + (i & 3)) * 32 + ln] = stc[i];
      wave_sync_lds();
    }

    const float st = Stb[(tk & 31) * 32 + ln];
    const bool near = has_content && (W <= 0 || tq - tk <= W || tq == T_ - 1);
    f32x16 S[NCT], dP[NCT];
#pragma unroll
    for (int t = 0; t < NCT; ++t) {
      S[t] = Bc[t];
#pragma unroll
      for (int i = 0; i < 16; ++i) dP[t][i] = 0.f;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int t = 0; t < NCT; ++t) {
        const int off = r_lane[ks] + t * 32 * ROWB;
        if (near) S[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)(Krow + off), Qu[ks], S[t], 0, 0, 0);
        dP[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)(Vrow + off), dOf[ks], dP[t], 0, 0, 0);
      }
    const float off2 = st - lse;
    float gt = 0.f;
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float p = __builtin_amdgcn_exp2f(S[t][i] + off2);     // masked keys: exp2(-inf) = 0
        const float ds = p * (dP[t][i] - delta) * a.sm_scale;
        S[t][i] = ds;
        dSc[t][i] += ds;
        gt += ds;
      }
    gt = xhalf_sum(gt);
    if (hh == 0) Gtb[(tk & 31) * 32 + ln] = gt;
    if (near) {
#pragma unroll
      for (int t = 0; t < NCT; ++t)
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const bf16x8 dsf = pack8(S[t], 8 * s);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            dq[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(Ktr, t, s, mt), dsf, dq[mt], 0, 0, 0);
        }
    }
  }

  if (!active) return;
  wave_sync_lds();
  flush_slab(tq & ~31);

  // dq^T[d][q]: this lane's query, d = 32mt + 8a4 + 4hh + 0..3
  if (qok) {
    float* dqo = a.dq + row * DH;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4)
        *(float4*)(dqo + mt * 32 + a4 * 8 + hh * 4) =
            make_float4(dq[mt][a4 * 4], dq[mt][a4 * 4 + 1], dq[mt][a4 * 4 + 2], dq[mt][a4 * 4 + 3]);
  }

  // channel-table gradient: element (ck) of query cq goes to column C-1-|cq-ck|; the two key
  // channels at the same distance add up.  Per-wave table [32 queries][CP] in the scratch.
  wave_sync_lds();
  for (int i = lane; i < 32 * CP; i += 64) scr[i] = 0.f;
  wave_sync_lds();
  {
    const uint32_t cq4 = (uint32_t)(cq - 4 * hh + 4);
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint32_t ci4 = (uint32_t)(t * 32 + (i >> 2) * 8 + (i & 3) + 4);
        const uint32_t dist = max(cq4, ci4) - min(cq4, ci4);
        const bool kv = (kbits[t] >> ((i >> 2) * 8 + (i & 3))) & 1u;
        if (kv && dist < (uint32_t)C_ && qok) atomicAdd(&scr[ln * CP + (C_ - 1 - (int)dist)], dSc[t][i]);
      }
  }
  wave_sync_lds();
  if (qok && hh == 0) {
    float* gc = a.dbias_chan + row * C_;
    for (int i = 0; i < C_; ++i) gc[i] = scr[ln * CP + i];
  }
}

}  // namespace bwdq
}  // namespace mvpa

// 1 if the MFMA query pass can serve these (already validated) arguments
int mvpa_bwd_query_mfma_supported(const mvpa_bwd_args* a) {
  if (a->dtype != MVPA_BF16 || a->Dh != 64 || a->C > 64) return 0;
  if (!(a->flags & MVPA_FLAG_CAUSAL) || a->key_bias) return 0;
  const uintptr_t p = (uintptr_t)a->q | (uintptr_t)a->k | (uintptr_t)a->v | (uintptr_t)a->o |
                      (uintptr_t)a->d_o | (uintptr_t)a->bias_u | (uintptr_t)a->bias_v |
                      (uintptr_t)a->bias_z | (uintptr_t)a->k_time | (uintptr_t)a->k_chan |
                      (uintptr_t)a->dq;
  const int64_t s = a->q_stride_b | a->q_stride_h | a->q_stride_n | a->k_stride_b | a->k_stride_h |
                    a->k_stride_n | a->v_stride_b | a->v_stride_h | a->v_stride_n |
                    a->o_stride_b | a->o_stride_h | a->o_stride_n | a->do_stride_b |
                    a->do_stride_h | a->do_stride_n;
  if ((p & 15) || (s & 7)) return 0;
  return 1;
}

int mvpa_launch_bwd_query_mfma(const mvpa_bwd_args* a, hipStream_t stream) {
  using namespace mvpa::bwdq;
  const int nct = a->C <= 32 ? 1 : 2;
  const int tqw = NW / nct;
  const int nt = (a->T + tqw - 1) / tqw;
  const int cp = nct * 32;
  const size_t lds = (size_t)3 * cp * ROWB + (size_t)NW * (2 * 1024 + cp * 32) * sizeof(float);
  dim3 grid((unsigned)nt, (unsigned)(a->B * a->H));
  if (nct == 1) {
    auto kern = mvpa_bwd_query_mfma_kernel<1>;
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(kern, grid, dim3(NW * 64), lds, stream, *a);
  } else {
    auto kern = mvpa_bwd_query_mfma_kernel<2>;
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(kern, grid, dim3(NW * 64), lds, stream, *a);
  }
  return hipGetLastError() == hipSuccess ? MVPA_OK : MVPA_ERR_LAUNCH;
}

// ==========================================================================================
// The KEY pass: dk, dv.  One workgroup per key time step tk and kv head; a wave owns 32 key
// channels (its K and V rows stay in registers as MFMA B operands) and one of the NCT query-channel
// tiles; it walks the query time steps tq >= tk of every query head of the group.  Products are
// formed NON-transposed here, S[q][key] = (q+u) K^T, so that a lane owns one key and the
// contraction index of dv^T = dO^T P and dk^T = (q+u)^T dS is the register index:
//     S   = (q+u) K^T (inside the window) + chan[q][C-1-|cq-ck|] + time[q][tk]
//     P   = exp2(S - L[q]),  dP = dO V^T,  dS = P o (dP - delta[q])
//     dv^T[d][key] += dO^T[d][q] P[q][key],   dk^T[d][key] += (q+u)^T[d][q] dS[q][key]
// The per-query bias tables, L and delta come from the query pass (workspace, natural units).
// Per (head, tq) the workgroup stages (q+u) * scale and dO (each in the two swizzles), the
// channel-table rows and the per-query scalars in LDS.
// ==========================================================================================
namespace mvpa {
namespace bwdq {

template <int NCT>
__global__ __launch_bounds__(NCT * NCT * 64) void mvpa_bwd_key_mfma_kernel(mvpa_bwd_args a) {
  constexpr int CP = NCT * 32, TILE = CP * ROWB, NWK = NCT * NCT, NTHR = NWK * 64;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char* Qrow = smem;                     // (q+u)*scale, row-fragment swizzle
  unsigned char* Qtr = smem + TILE;               // same, transposing-read swizzle
  unsigned char* Drow = smem + 2 * TILE;          // dO, row-fragment swizzle
  unsigned char* Dtr = smem + 3 * TILE;           // dO, transposing-read swizzle
  float* Cs = (float*)(smem + 4 * TILE);          // [CP][CP] channel-table rows * scale
  float* Ls = Cs + CP * CP;                       // [CP] log-sum-exp (+inf for padded queries)
  float* Es = Ls + CP;                            // [CP] delta
  float* Ts = Es + CP;                            // [CP] time-table entry for this tk * scale

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, hh = lane >> 5;
  const int kt = wave % NCT, qt = wave / NCT;     // this wave's key tile and query tile
  const int T_ = a.T, C_ = a.C, W = a.window, N = a.T * a.C;
  const bool has_content = a.flags & MVPA_FLAG_CONTENT;
  const bool has_time = a.flags & MVPA_FLAG_TIME_BIAS;
  const bool has_chan = a.flags & MVPA_FLAG_CHAN_BIAS;
  const int tk = blockIdx.x;                      // early key steps (most queries) first
  const int b = blockIdx.y / a.Hkv, g = blockIdx.y % a.Hkv;
  const int grp = a.H / a.Hkv;
  const float sc2 = a.sm_scale * kLog2e;

  const int ck = kt * 32 + ln;
  bool key_ok = ck < C_;
  if (key_ok && a.chan_valid) key_ok = a.chan_valid[(int64_t)b * C_ + ck] != 0;
  const int64_t nk = (int64_t)tk * C_ + min(ck, C_ - 1);
  const bf16_t* krow = (const bf16_t*)a.k + b * a.k_stride_b + g * a.k_stride_h + nk * a.k_stride_n;
  const bf16_t* vrow = (const bf16_t*)a.v + b * a.v_stride_b + g * a.v_stride_h + nk * a.v_stride_n;
  const bf16_t* bu = (const bf16_t*)a.bias_u + g * DH;
  bf16x8 Kf[KS], Vf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    Kf[ks] = as_frag(*(const u32x4*)(krow + ks * 16 + hh * 8));
    Vf[ks] = as_frag(*(const u32x4*)(vrow + ks * 16 + hh * 8));
  }

  f32x16 dK[MT], dV[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) { dK[mt][i] = 0.f; dV[mt][i] = 0.f; }

  int r_lane[KS], t_lane[MT];
  {
    const int e = (ln & 15) >> 2, aa = ln & 3, grp16 = ln >> 4;
    const int row0 = 4 * hh + e;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      r_lane[ks] = (qt * 32 + ln) * ROWB + (((2 * ks + hh) ^ swz_row(ln)) << 4);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      t_lane[mt] = (qt * 32 + row0) * ROWB + (((4 * mt + 2 * grp16 + (aa >> 1)) ^ swz_tr(row0)) << 4) + ((aa & 1) << 3);
  }
  auto tr_frag = [&](const unsigned char* tile_p, int s, int mt) -> bf16x8 {
    const unsigned char* p = tile_p + t_lane[mt] + 16 * s * ROWB;
    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((BWD_LDS_PTR(bf16x4))p);
    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((BWD_LDS_PTR(bf16x4))(p + 8 * ROWB));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };

  constexpr int CHUNKS = CP * 8;
  for (int hq = 0; hq < grp; ++hq) {
    const int h = g * grp + hq;
    const bf16_t* qbase = (const bf16_t*)a.q + b * a.q_stride_b + h * a.q_stride_h;
    const bf16_t* dbase = (const bf16_t*)a.d_o + b * a.do_stride_b + h * a.do_stride_h;
    const int64_t rbase = ((int64_t)b * a.H + h) * N;
    for (int tq = tk; tq < T_; ++tq) {
      const bool near = has_content && (W <= 0 || tq - tk <= W || tq == T_ - 1);
      const int jt = time_row(tq, tk, T_);
      __syncthreads();                            // everyone is done with the previous stage
      for (int c = tid; c < CHUNKS; c += NTHR) {
        const int r = c >> 3, ch = c & 7;
        const int64_t n = (int64_t)tq * C_ + min(r, C_ - 1);
        const u32x4 qq = *(const u32x4*)(qbase + n * a.q_stride_n + ch * 8);
        const u32x4 dd = *(const u32x4*)(dbase + n * a.do_stride_n + ch * 8);
        const bf16x8 qu = qfrag(qq, bu + ch * 8, sc2);
        union { bf16x8 f; u32x4 u; } cv;
        cv.f = qu;
        *(u32x4*)(Qrow + r * ROWB + ((ch ^ swz_row(r)) << 4)) = cv.u;
        *(u32x4*)(Qtr + r * ROWB + ((ch ^ swz_tr(r)) << 4)) = cv.u;
        *(u32x4*)(Drow + r * ROWB + ((ch ^ swz_row(r)) << 4)) = dd;
        *(u32x4*)(Dtr + r * ROWB + ((ch ^ swz_tr(r)) << 4)) = dd;
      }
      for (int idx = tid; idx < C_ * C_; idx += NTHR) {
        const int r = idx / C_, i = idx - r * C_;
        Cs[r * CP + i] = has_chan ? a.ws_chan[(rbase + (int64_t)tq * C_ + r) * C_ + i] * sc2 : 0.f;
      }
      for (int r = tid; r < CP; r += NTHR) {
        const bool ok = r < C_;
        const int64_t rw = rbase + (int64_t)tq * C_ + min(r, C_ - 1);
        Ls[r] = ok ? a.lse[rw] : INFINITY;        // padded queries: exp2(-inf) = 0
        Es[r] = ok ? a.ws_delta[rw] : 0.f;
        Ts[r] = (ok && has_time) ? a.ws_time[rw * T_ + jt] * sc2 : 0.f;
      }
      __syncthreads();

      // ---- S[q][key] and dP[q][key] for this wave's (query tile, key tile)
      f32x16 S, dP;
#pragma unroll
      for (int i = 0; i < 16; ++i) { S[i] = 0.f; dP[i] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (near) S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)(Qrow + r_lane[ks]), Kf[ks], S, 0, 0, 0);
        dP = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)(Drow + r_lane[ks]), Vf[ks], dP, 0, 0, 0);
      }
      f32x16 dS;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int r = qt * 32 + (i >> 2) * 8 + hh * 4 + (i & 3);     // query channel of this row
        const int dist = r > ck ? r - ck : ck - r;
        const int col = min(max(C_ - 1 - dist, 0), CP - 1);
        const float s = S[i] + Cs[r * CP + col] + Ts[r] - Ls[r];
        const float p = (key_ok && r < C_) ? __builtin_amdgcn_exp2f(s) : 0.f;   // padded rows/keys
        S[i] = p;
        dS[i] = p * (dP[i] - Es[r]) * (1.f / kLog2e);
      }
      // ---- dv^T[d][key] += dO^T[d][q] P[q][key];  dk^T[d][key] += (q+u)^T[d][q] dS[q][key]
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const bf16x8 pf = pack8(S, 8 * s);
        const bf16x8 sf = pack8(dS, 8 * s);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          dV[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(Dtr, s, mt), pf, dV[mt], 0, 0, 0);
          if (near) dK[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(Qtr, s, mt), sf, dK[mt], 0, 0, 0);
        }
      }
    }
  }

  // ---- reduce the query tiles' partial sums (waves with the same key tile) and store
  __syncthreads();
  float* red = (float*)smem;                      // [NCT key tiles][2][64 d][32 keys] fp32
  if (NCT > 1) {
    for (int round = 1; round < NCT; ++round) {
      if (qt == round) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int d = mt * 32 + (i >> 2) * 8 + hh * 4 + (i & 3);
            red[((kt * 2 + 0) * 64 + d) * 32 + ln] = dK[mt][i];
            red[((kt * 2 + 1) * 64 + d) * 32 + ln] = dV[mt][i];
          }
      }
      __syncthreads();
      if (qt == 0) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int d = mt * 32 + (i >> 2) * 8 + hh * 4 + (i & 3);
            dK[mt][i] += red[((kt * 2 + 0) * 64 + d) * 32 + ln];
            dV[mt][i] += red[((kt * 2 + 1) * 64 + d) * 32 + ln];
          }
      }
      __syncthreads();
    }
  }
  if (qt == 0 && ck < C_) {
    const int64_t o = ((((int64_t)b * a.Hkv + g) * N) + (int64_t)tk * C_ + ck) * DH;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4) {
        const int d = mt * 32 + a4 * 8 + hh * 4;
        *(float4*)(a.dk + o + d) = make_float4(dK[mt][a4 * 4], dK[mt][a4 * 4 + 1], dK[mt][a4 * 4 + 2], dK[mt][a4 * 4 + 3]);
        *(float4*)(a.dv + o + d) = make_float4(dV[mt][a4 * 4], dV[mt][a4 * 4 + 1], dV[mt][a4 * 4 + 2], dV[mt][a4 * 4 + 3]);
      }
  }
}

}  // namespace bwdq
}  // namespace mvpa

int mvpa_launch_bwd_key_mfma(const mvpa_bwd_args* a, hipStream_t stream) {
  using namespace mvpa::bwdq;
  const int nct = a->C <= 32 ? 1 : 2;
  const int cp = nct * 32;
  size_t lds = (size_t)4 * cp * ROWB + (size_t)(cp * cp + 3 * cp) * sizeof(float);
  const size_t red = (size_t)nct * 2 * 64 * 32 * sizeof(float);
  if (red > lds) lds = red;
  dim3 grid((unsigned)a->T, (unsigned)(a->B * a->Hkv));
  if (nct == 1) {
    auto kern = mvpa_bwd_key_mfma_kernel<1>;
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(kern, grid, dim3(64), lds, stream, *a);
  } else {
    auto kern = mvpa_bwd_key_mfma_kernel<2>;
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, *a);
  }
  return hipGetLastError() == hipSuccess ? MVPA_OK : MVPA_ERR_LAUNCH;
}
