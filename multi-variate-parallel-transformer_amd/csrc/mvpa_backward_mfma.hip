// MVPA backward on MFMA (bf16, Dh = 64 or 128, up to 64 channels per launch, 128 in parts): the QUERY pass (the KEY pass follows below).
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
// Outputs are those of mvpa_backward (include/mvpa_hip.h): the content share of dq and the two
// bias-table gradients.  For the key pass the workspace receives, in base-2 score units, delta,
// the channel-table rows, (time bias - L) laid out [b,h,tq,tk,cq] and (q+u) * scale in bf16.
// K and V tiles come through a ring of LDS stages filled by direct-to-LDS loads two key steps
// ahead, K in two copies (row fragments for K Q^T, transposed fragments for K^T dS^T); far key
// steps fetch V only.
#include "mvpa_common.h"

#include <type_traits>

namespace mvpa {
namespace bwdq {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

#define BWD_LDS_PTR(T) __attribute__((address_space(3))) T*

// Head dim DH is 64 or 128: KS = DH / 16 contraction blocks per product, MT = DH / 32 output tiles
// of the gradients, rows of ROWB = 2 DH bytes (CPR = DH / 8 chunks of 16 bytes) in the LDS tiles.
constexpr int KSTAGES = 3;                        // ring depth of the key pass
// ring depth of the query pass: three stages, two where three would not fit the LDS
template <int DH, int NCT> constexpr int QSTAGES = (DH == 128 && NCT == 2) ? 2 : 3;
// waves per workgroup of the query pass: with two channel tiles of Dh 64 8 waves (4 query time
// steps) share the K/V ring and each SIMD holds two waves
template <int DH, int NCT> constexpr int QUERY_WAVES = (NCT == 2 && DH == 64) ? 8 : 4;
// floats of per-wave scratch in the query pass: the two time-bias slabs [32][32] + [32][33]; the
// channel tables of the set-up ([32 NCT][32]) and of the epilogue ([32][32 NCT + 1]) overlay them
constexpr int WAVE_SCRATCH = 1024 + 32 * 33;

__device__ inline void wave_sync_lds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// workgroup barrier that orders LDS traffic only (global loads of the ring stay in flight)
__device__ inline void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// direct-to-LDS loads: lane L's 16 (4) bytes land at lds_base + 16 L (4 L).  Inline assembly so
// that the compiler does not drain the ring in front of later LDS reads; completion is awaited
// with wait_vmcnt() before the barrier that publishes a stage.
__device__ inline void dma16(const void* gptr, uint32_t lds_base) {
  lds_base = __builtin_amdgcn_readfirstlane(lds_base);    // uniform by construction; pins it to an SGPR
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :: "v"(gptr), "s"(lds_base) : "memory", "m0");
}
__device__ inline void dma4(const void* gptr, uint32_t lds_base) {
  lds_base = __builtin_amdgcn_readfirstlane(lds_base);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
               :: "v"(gptr), "s"(lds_base) : "memory", "m0");
}

template <int N>
__device__ inline void wait_vmcnt_imm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// wait until at most n (0..6) of this wave's vector-memory operations are outstanding
__device__ inline void wait_vmcnt(int n) {
  switch (n) {
    case 0: wait_vmcnt_imm<0>(); break;
    case 1: wait_vmcnt_imm<1>(); break;
    case 2: wait_vmcnt_imm<2>(); break;
    case 3: wait_vmcnt_imm<3>(); break;
    case 4: wait_vmcnt_imm<4>(); break;
    case 5: wait_vmcnt_imm<5>(); break;
    default: wait_vmcnt_imm<6>(); break;
  }
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

// 8 floats to a bf16 fragment, two per conversion instruction
__device__ inline bf16x8 pack8(const f32x16& v, int base) {
  union { bf16x8 f; bf16x2 q[4]; } out;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    out.q[i] = __builtin_convertvector(f32x2{v[base + 2 * i], v[base + 2 * i + 1]}, bf16x2);
  return out.f;
}

__device__ inline float xhalf_sum(float x) { return x + __shfl_xor(x, 32); }

// chunk swizzles of a row of 2 DH bytes: row fragments / transposing reads (as in the forward)
template <int DH> __device__ inline int swz_row(int row) { return DH == 64 ? ((row >> 1) & 7) : (row & 15); }
template <int DH> __device__ inline int swz_tr(int row) { return DH == 64 ? (((row >> 1) & 1) << 2) : ((row & 3) << 2); }

template <int DH, int NCT>
__global__ __launch_bounds__((QUERY_WAVES<DH, NCT> * 64)) void mvpa_bwd_query_mfma_kernel(mvpa_bwd_args a, int q0, int k0, int accum) {
  constexpr int KS = DH / 16, MT = DH / 32, ROWB = 2 * DH, CPR = DH / 8;
  constexpr int NW = QUERY_WAVES<DH, NCT>;
  constexpr int CP = NCT * 32, TQW = NW / NCT, TILE = CP * ROWB;
  static_assert(64 * 32 <= WAVE_SCRATCH && 32 * (CP + 1) <= WAVE_SCRATCH, "channel tables overlay the slabs");
  constexpr int STAGES = QSTAGES<DH, NCT>, STAGE_BYTES = 3 * TILE;   // stage: V | K | K (transposing)
  constexpr int LPW = TILE / 1024 / NW;           // 1 KiB wave loads per wave and tile copy
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  float* wave_base = (float*)(smem + STAGES * STAGE_BYTES);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, hh = lane >> 5;
  constexpr int GP = 33, PC = CP + 1;             // padded pitches: the transposed reads spread over the banks
  float* Stb = wave_base + wave * WAVE_SCRATCH;           // [32][32] time-bias scores of a slab
  float* Gtb = Stb + 1024;                                // [32][GP] their gradients
  float* scr = Stb;       // before the first slab [CP][32] channel table, after the last one [32][PC]

  const int T_ = a.T, C_ = a.C, W = a.window, N = a.T * a.C;
  const int CW = (C_ + 3) & ~3;                   // row pitch of the Ec tiles in the workspace
  const bool has_content = a.flags & MVPA_FLAG_CONTENT;
  const bool has_time = a.flags & MVPA_FLAG_TIME_BIAS;
  const bool has_chan = a.flags & MVPA_FLAG_CHAN_BIAS;
  const int nt = (T_ + TQW - 1) / TQW;
  // blocks go round-robin over the 8 XCDs: keep the tiles of one (b,h) on one XCD (they walk the
  // same K and V in step, so its L2 serves all but the first), long tiles first.  The tile with
  // the last time step keeps the content term at every key step and runs about twice as long as
  // the next one: all of those go first, or the last of them would end the launch alone.
  const int nbh = a.B * a.H;
  int bh, tile;
  {
    const int L = blockIdx.x;
    if (nt == 1) {
      bh = L;
      tile = 0;
    } else if (L < nbh) {
      bh = L;
      tile = nt - 1;
    } else if ((nbh & 7) == 0) {
      const int s = (L - nbh) >> 3;
      bh = ((L - nbh) & 7) + 8 * (s / (nt - 1));
      tile = nt - 2 - s % (nt - 1);
    } else {
      bh = (L - nbh) / (nt - 1);
      tile = nt - 2 - (L - nbh) % (nt - 1);
    }
  }
  const int b = bh / a.H, h = bh % a.H;
  const int g = h / (a.H / a.Hkv);
  const int tq0 = tile * TQW;
  const int tq_hi = min(T_ - 1, tq0 + TQW - 1);
  const int tq = tq0 + wave / NCT;
  const bool active = tq < T_;
  const int cqw0 = q0 + (wave % NCT) * 32;        // first query channel of this wave
  const int cq = cqw0 + ln;
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

  // ---- the ring: per-wave source offsets (the swizzle is applied on the source side), prologue
  int k_off_r[LPW], k_off_t[LPW], v_off[LPW];
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int pc = (wave + NW * i) * 64 + lane;
    const int r = pc / CPR, phys = pc % CPR;
    const int rc = min(k0 + r, C_ - 1);           // key channels k0 .. of this launch
    k_off_r[i] = rc * (int)a.k_stride_n + ((phys ^ swz_row<DH>(r)) << 3);
    k_off_t[i] = rc * (int)a.k_stride_n + ((phys ^ swz_tr<DH>(r)) << 3);
    v_off[i] = rc * (int)a.v_stride_n + ((phys ^ swz_row<DH>(r)) << 3);
  }
  // first key step whose K is needed: the band of the earliest query step of the workgroup
  const int tk_near = !has_content ? tq_hi + 1 : (W <= 0 || tq_hi == T_ - 1) ? 0 : max(0, tq0 - W);
  const uint32_t ring_lds = (uint32_t)(uintptr_t)(BWD_LDS_PTR(unsigned char))smem;
  auto issue_tile = [&](int tk, int stage_idx, bool with_k) {
    const uint32_t st = ring_lds + stage_idx * STAGE_BYTES;
    const bf16_t* vsrc = vbase + (int64_t)tk * C_ * a.v_stride_n;
#pragma unroll
    for (int i = 0; i < LPW; ++i) dma16(vsrc + v_off[i], st + (wave + NW * i) * 1024);
    if (with_k) {
      const bf16_t* ksrc = kbase + (int64_t)tk * C_ * a.k_stride_n;
#pragma unroll
      for (int i = 0; i < LPW; ++i) {
        dma16(ksrc + k_off_r[i], st + TILE + (wave + NW * i) * 1024);
        dma16(ksrc + k_off_t[i], st + 2 * TILE + (wave + NW * i) * 1024);
      }
    }
  };
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s <= tq_hi) issue_tile(s, s, s >= tk_near);

  // ---- set-up: operand fragments, delta, channel-bias tile
  bf16x8 dOf[KS];            // (q+u), (q+v) fragments are re-formed where needed, not kept
  f32x16 Ec[NCT];            // exp2(channel bias - mc): the far steps' probabilities up to a scalar
  float delta = 0.f, mc = -INFINITY, sumEc = 0.f;
  uint32_t kbits[NCT];
  // every global load of the set-up goes out before the first use: one round trip, not one per
  // fragment.  The log-sum-exp is among them so that its wait does not fall into the loops, where
  // it would drain the whole ring (vmcnt 0) at every key step.
  u32x4 raw_[KS], draw_[KS], oraw_[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d0 = ks * 16 + hh * 8;
    raw_[ks] = *(const u32x4*)(qrow + d0);
    draw_[ks] = *(const u32x4*)(drow + d0);
    oraw_[ks] = *(const u32x4*)(orow + d0);
  }
  const float lse = a.lse[row];
  uint64_t kmask;                                 // the (up to 64) key channels of this launch
  {
    const int ck = k0 + lane;
    bool ok = ck < C_ && lane < CP;
    if (valid) ok = ok && valid[min(ck, C_ - 1)] != 0;
    kmask = __ballot(ok);
  }
  asm volatile("" :: "v"(lse));
  {
    bf16x8 qz[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 16 + hh * 8;
      const u32x4 raw = raw_[ks], draw = draw_[ks], oraw = oraw_[ks];
      if (qok) *(bf16x8*)((bf16_t*)a.ws_qu + row * DH + d0) = qfrag(raw, bu + d0, sc2);   // for the key pass
      qz[ks] = qfrag(raw, bz + d0, sc2);
      dOf[ks] = as_frag(draw);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        delta += __uint_as_float(draw[i] << 16) * __uint_as_float(oraw[i] << 16);
        delta += __uint_as_float(draw[i] & 0xffff0000u) * __uint_as_float(oraw[i] & 0xffff0000u);
      }
    }
    delta = xhalf_sum(delta);
#pragma unroll
    for (int t = 0; t < NCT; ++t) kbits[t] = (uint32_t)(kmask >> (t * 32 + 4 * hh));
    // Channel-bias tile, one key tile at a time: the 32 queries of this wave and the 32 keys of
    // tile t are at most 63 channels apart in either direction, so the rows C-1-d of the table
    // (q+z).k_chan^T they need lie in a window of 64 rows starting at jlo.  That window goes
    // through the per-wave scratch ([64][32]), and Bc[key][q] = table[C-1-|cq-ck|][q] is
    // gathered from it; -inf where the key channel is padding or absent.
#pragma unroll
    for (int t = 0; t < NCT; ++t) {
      const int ck0 = k0 + t * 32;
      const int dmax = max(cqw0 + 31 - ck0, ck0 + 31 - cqw0);       // > 0
      const int jlo = max(C_ - 1 - dmax, 0);
      f32x16 sct[2];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int i = 0; i < 16; ++i) sct[tt][i] = 0.f;
      u32x4 er[KS][2];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
          er[ks][tt] = *(const u32x4*)(kchan + (int64_t)min(jlo + tt * 32 + ln, C_ - 1) * DH + ks * 16 + hh * 8);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
          sct[tt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(er[ks][tt]), qz[ks], sct[tt], 0, 0, 0);
      wave_sync_lds();                            // the previous tile's gather is done with the scratch
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int j = tt * 32 + (i >> 2) * 8 + hh * 4 + (i & 3);
          scr[j * 32 + ln] = has_chan ? sct[tt][i] : 0.f;
        }
      wave_sync_lds();
      // row of the window for key ck = c_i + 4hh: (C-1-jlo) - |cq - ck|, clamped into the window
      // for padded queries / keys (their values are never used)
      const uint32_t cq4 = (uint32_t)(cq - 4 * hh + 4);
      const int top = C_ - 1 - jlo;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint32_t ci4 = (uint32_t)(ck0 + (i >> 2) * 8 + (i & 3) + 4);
        const int dist = (int)(max(cq4, ci4) - min(cq4, ci4));
        const int jr = min(max(top - dist, 0), 63);
        const float val = scr[jr * 32 + ln];
        const bool kv = (kbits[t] >> ((i >> 2) * 8 + (i & 3))) & 1u;
        Ec[t][i] = kv ? val : -INFINITY;
      }
    }
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) mc = fmaxf(mc, Ec[t][i]);
    mc = fmaxf(mc, __shfl_xor(mc, 32));
    if (mc == -INFINITY) mc = 0.f;                // no valid key channel at all
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        Ec[t][i] = __builtin_amdgcn_exp2f(Ec[t][i] - mc);
        sumEc += Ec[t][i];
      }
    sumEc = xhalf_sum(sumEc);
    // for the key pass: (q+u) * scale, delta, and the tile exp2(channel bias - mc) by
    // [query][key channel]; and the rows of dbias_time that no key step reaches
    if (qok) {
      float* wc = a.ws_chan + row * CW + k0;      // rows of CW floats: 16-byte aligned for any C
#pragma unroll
      for (int t = 0; t < NCT; ++t)
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
          const int ci = t * 32 + a4 * 8 + hh * 4;
          if (k0 + ci < CW)
            *(float4*)(wc + ci) = make_float4(Ec[t][a4 * 4], Ec[t][a4 * 4 + 1], Ec[t][a4 * 4 + 2], Ec[t][a4 * 4 + 3]);
        }
    }
    if (qok && hh == 0) a.ws_delta[row] = delta;
  }

  f32x16 dq[MT], dSc[NCT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) dq[mt][i] = 0.f;
#pragma unroll
  for (int t = 0; t < NCT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) dSc[t][i] = 0.f;

  // this wave's query rows are consecutive in memory; outputs are written a row at a time (the
  // two half-waves take alternate rows) so that each store covers one contiguous run
  const int cq0 = cqw0;
  const int nq_live = active ? max(0, min(32, C_ - cq0)) : 0;
  const int64_t wrow0 = ((int64_t)b * a.H + h) * N + (int64_t)(active ? tq : 0) * C_ + cq0;

  // the columns of dbias_time that no key step reaches (once: by the launch that does not add)
  if (!accum)
    for (int q = hh; q < nq_live; q += 2)
      for (int j = ln; j < T_ - 1 - tq; j += 32) a.dbias_time[(wrow0 + q) * T_ + j] = 0.f;

  // ---- loop-invariant fragment offsets
  int r_lane[KS], t_lane[MT];
  {
    const int e = (ln & 15) >> 2, aa = ln & 3, grp = ln >> 4;
    const int row0 = 4 * hh + e;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) r_lane[ks] = ln * ROWB + (((2 * ks + hh) ^ swz_row<DH>(ln)) << 4);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      t_lane[mt] = row0 * ROWB + (((4 * mt + 2 * grp + (aa >> 1)) ^ swz_tr<DH>(row0)) << 4) + ((aa & 1) << 3);
  }
  auto tr_frag = [&](const unsigned char* tile_p, int t, int s, int mt) -> bf16x8 {
    const unsigned char* p = tile_p + t_lane[mt] + (32 * t + 16 * s) * ROWB;
    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((BWD_LDS_PTR(bf16x4))p);
    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((BWD_LDS_PTR(bf16x4))(p + 8 * ROWB));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };

  // writes the gradients of the slab that started at key step tks, and its per-pair scalars for
  // the key pass (the exponent e = time bias - L + mc for pairs inside the window, else exp2(e))
  auto flush_slab = [&](int tks) {
    const int nj = min(32, tq - tks + 1);
    // fixed trip counts with predicates: the LDS reads of several iterations go out together
#pragma unroll 8
    for (int it = 0; it < 16; ++it) {
      const int jj = 2 * it + hh, tkk = tks + jj;
      const float e = Stb[jj * 32 + ln] - lse + mc;
      const bool near_pair = has_content && (W <= 0 || tq - tkk <= W || tq == T_ - 1);
      const float val = near_pair ? e : __builtin_amdgcn_exp2f(e);
      if (qok && jj < nj) a.ws_time[(((int64_t)bh * T_ + tq) * T_ + tkk) * C_ + cq] = val;
    }
    const int j0 = time_row(tq, tks, T_);
#pragma unroll 8
    for (int it = 0; it < 16; ++it) {
      const int q = 2 * it + hh;
      const float g = Gtb[ln * GP + q];
      if (q < nq_live && ln < nj) {
        float* dst = a.dbias_time + (wrow0 + q) * T_ + j0 + ln;
        // launches of one stream: the key parts add up.  An atomic add without a return value,
        // not a load and a store: nothing waits for the old value (every address has one writer)
        if (accum) atomicAdd(dst, g);
        else *dst = g;
      }
    }
  };

  int stage = 0;
  // advances the ring to key step tk and returns the stage that holds its tiles
  auto ring_step = [&](int tk) -> const unsigned char* {
    // tile tk has landed once at most the loads of the younger tiles are in flight (a count that
    // is too small only waits longer)
    if (tk + 1 >= tk_near && tk + STAGES - 2 <= tq_hi) {
      wait_vmcnt_imm<(STAGES - 2) * 3 * LPW>();
    } else {
      int younger = 0;
#pragma unroll
      for (int d = 1; d <= STAGES - 2; ++d)
        if (tk + d <= tq_hi) younger += LPW * (tk + d >= tk_near ? 3 : 1);
      wait_vmcnt(younger);
    }
    lds_barrier();            // tile tk visible to all; everyone is done with tile tk-1's stage
    if (tk + STAGES - 1 <= tq_hi)
      issue_tile(tk + STAGES - 1, stage == 0 ? STAGES - 1 : stage - 1, tk + STAGES - 1 >= tk_near);
    const unsigned char* Vrow = smem + stage * STAGE_BYTES;
    stage = stage + 1 == STAGES ? 0 : stage + 1;
    return Vrow;
  };

  // every 32 key steps: write the finished slab, form the next slab of time-bias scores
  auto time_slab = [&](int tk) {
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
        u32x4 rr[KS], qr[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {         // every load before the first use
          rr[ks] = *(const u32x4*)(ktime + (int64_t)j * DH + ks * 16 + hh * 8);
          qr[ks] = *(const u32x4*)(qrow + ks * 16 + hh * 8);
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          stc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(rr[ks]), qfrag(qr[ks], bv + ks * 16 + hh * 8, sc2), stc, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) Stb[((i >> 2) * 8 + hh * 4 + (i & 3)) * 32 + ln] = stc[i];
      wave_sync_lds();
    }
  };

  // A far key step (content term dropped): P^T = Ec et with et = exp2(time bias - L + mc) one
  // scalar per query, so with dP^T = V dO^T
  //     dbias_time[q, tk]  = scale et (sum_keys Ec dP - delta sumEc)
  //     dbias_chan share   = Ec (sum_tk scale et dP - delta sum_tk scale et)   (formed after the loop)
  // costs two FMAs per element and no exponential per element.
  // The loop is software-pipelined: the products of step tk are issued to the matrix cores, and
  // the vector work on the products of step tk-1 runs meanwhile.
  float esum = 0.f;
  // reduces the products of far step tkp (none if tkp < 0)
  auto far_reduce = [&](const f32x16 (&dP)[NCT], int tkp) {
    if (tkp < 0) return;
    const float et = __builtin_amdgcn_exp2f(Stb[(tkp & 31) * 32 + ln] - lse + mc) * a.sm_scale;
    float dot[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        dot[i & 3] += Ec[t][i] * dP[t][i];
        dSc[t][i] += et * dP[t][i];
      }
    esum += et;
    const float gt = et * (xhalf_sum((dot[0] + dot[1]) + (dot[2] + dot[3])) - delta * sumEc);
    if (hh == 0) Gtb[(tkp & 31) * GP + ln] = gt;
  };
  // one far step: products of tile tk into cur, reduction of step tk-1 (in prev) alongside
  auto far_step = [&](int tk, int& tkp, f32x16 (&cur)[NCT], const f32x16 (&prev)[NCT]) {
    const unsigned char* Vrow = ring_step(tk);
    if ((tk & 31) == 0) {                         // the slab about to be written must be complete
      far_reduce(prev, tkp);
      tkp = -1;
      time_slab(tk);
    }
    bf16x8 vf[KS][NCT];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int t = 0; t < NCT; ++t) vf[ks][t] = *(const bf16x8*)(Vrow + r_lane[ks] + t * 32 * ROWB);
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) cur[t][i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int t = 0; t < NCT; ++t)
        cur[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[ks][t], dOf[ks], cur[t], 0, 0, 0);
    far_reduce(prev, tkp);
    tkp = tk;
  };

  // A key step inside the content window
  f32x16 Bc[NCT];
  bf16x8 Qu[KS];
  auto near_step = [&](const unsigned char* Vrow, int tk) {
    const unsigned char* Krow = Vrow + TILE;
    const unsigned char* Ktr = Vrow + 2 * TILE;
    const float off2 = Stb[(tk & 31) * 32 + ln] - lse;
    float gt = 0.f;
#pragma unroll
    for (int t = 0; t < NCT; ++t) {               // one key-channel tile at a time: fewer live tiles
      f32x16 S = Bc[t], dP;
#pragma unroll
      for (int i = 0; i < 16; ++i) dP[i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int off = r_lane[ks] + t * 32 * ROWB;
        S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)(Krow + off), Qu[ks], S, 0, 0, 0);
        dP = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)(Vrow + off), dOf[ks], dP, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float p = __builtin_amdgcn_exp2f(S[i] + off2);        // masked keys: exp2(-inf) = 0
        const float ds = p * (dP[i] - delta) * a.sm_scale;
        S[i] = ds;
        dSc[t][i] += ds;
        gt += ds;
      }
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const bf16x8 dsf = pack8(S, 8 * s);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          dq[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(Ktr, t, s, mt), dsf, dq[mt], 0, 0, 0);
      }
    }
    gt = xhalf_sum(gt);
    if (hh == 0) Gtb[(tk & 31) * GP + ln] = gt;
  };

  // far steps first (none for the last time step, whose queries keep the content term everywhere),
  // then the steps inside the window; waves that are done keep the ring and the barriers going
  const int far_end = !active ? 0 : !has_content ? tq + 1 : (W <= 0 || tq == T_ - 1) ? 0 : max(0, tq - W);
  int tk = 0;
  {
    f32x16 dPa[NCT], dPb[NCT];
    int tkp = -1;
    for (; tk + 1 < far_end; tk += 2) {
      far_step(tk, tkp, dPa, dPb);
      far_step(tk + 1, tkp, dPb, dPa);
    }
    if (tk < far_end) {
      far_step(tk, tkp, dPa, dPb);
      ++tk;
      far_reduce(dPa, tkp);
    } else {
      far_reduce(dPb, tkp);
    }
  }
  // the far steps' share of the channel-table gradient; from here on the tile holds the bias
#pragma unroll
  for (int t = 0; t < NCT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) dSc[t][i] = Ec[t][i] * (dSc[t][i] - delta * esum);
  // Bc = mc + log2(Ec): the table it was gathered from lies under the slabs by now (-inf where
  // Ec = 0: masked keys, and biases more than 126 octaves below the row's largest)
#pragma unroll
  for (int t = 0; t < NCT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) Bc[t][i] = mc + __builtin_amdgcn_logf(Ec[t][i]);
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    Qu[ks] = qfrag(*(const u32x4*)(qrow + ks * 16 + hh * 8), bu + ks * 16 + hh * 8, sc2);
  for (; tk <= tq_hi; ++tk) {
    const unsigned char* Vrow = ring_step(tk);
    if (active && tk <= tq) {
      time_slab(tk);
      near_step(Vrow, tk);
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
      {
        float4* dst = (float4*)(dqo + mt * 32 + a4 * 8 + hh * 4);
        float4 val = make_float4(dq[mt][a4 * 4], dq[mt][a4 * 4 + 1], dq[mt][a4 * 4 + 2], dq[mt][a4 * 4 + 3]);
        if (accum) {
          const float4 old = *dst;
          val = make_float4(val.x + old.x, val.y + old.y, val.z + old.z, val.w + old.w);
        }
        *dst = val;
      }
  }

  // channel-table gradient: element (ck) of query cq goes to column C-1-|cq-ck|, so column
  // C-1-d collects the two key channels cq-d and cq+d (those of them that this launch holds).
  // The tile goes to a per-wave table [32 queries][PC] by local key channel, and each output row
  // is gathered from it (LDS float atomics for the scatter form were measured at ~0.3 us apiece).
  wave_sync_lds();
#pragma unroll
  for (int t = 0; t < NCT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) scr[ln * PC + t * 32 + (i >> 2) * 8 + hh * 4 + (i & 3)] = dSc[t][i];
  wave_sync_lds();
  for (int c0 = 0; c0 < C_; c0 += 64) {
    const int col = c0 + lane;
    const int d = C_ - 1 - col;                   // this lane's column holds distance d
#pragma unroll 8
    for (int q = 0; q < 32; ++q) {
      const int lo = cq0 + q - d - k0, hi = cq0 + q + d - k0;      // local key channels
      float g = scr[q * PC + max(0, min(lo, CP - 1))];
      const float g2 = scr[q * PC + max(0, min(hi, CP - 1))];
      if (lo < 0 || lo >= CP || d < 0) g = 0.f;
      if (d > 0 && hi >= 0 && hi < CP) g += g2;
      if (q < nq_live && col < C_) {
        float* dst = a.dbias_chan + (wrow0 + q) * C_ + col;
        if (accum) atomicAdd(dst, g);
        else *dst = g;
      }
    }
  }
}

}  // namespace bwdq
}  // namespace mvpa

// 1 if the MFMA query pass can serve these (already validated) arguments
int mvpa_bwd_query_mfma_supported(const mvpa_bwd_args* a) {
  if (a->dtype != MVPA_BF16 || (a->Dh != 64 && a->Dh != 128) || a->C > 128) return 0;
  if (!(a->flags & MVPA_FLAG_CAUSAL) || a->key_bias || !a->ws_qu) return 0;
  const uintptr_t p = (uintptr_t)a->q | (uintptr_t)a->k | (uintptr_t)a->v | (uintptr_t)a->o |
                      (uintptr_t)a->d_o | (uintptr_t)a->bias_u | (uintptr_t)a->bias_v |
                      (uintptr_t)a->bias_z | (uintptr_t)a->k_time | (uintptr_t)a->k_chan |
                      (uintptr_t)a->dq | (uintptr_t)a->ws_qu | (uintptr_t)a->ws_chan |
                      (uintptr_t)a->dk | (uintptr_t)a->dv;
  const int64_t s = a->q_stride_b | a->q_stride_h | a->q_stride_n | a->k_stride_b | a->k_stride_h |
                    a->k_stride_n | a->v_stride_b | a->v_stride_h | a->v_stride_n |
                    a->o_stride_b | a->o_stride_h | a->o_stride_n | a->do_stride_b |
                    a->do_stride_h | a->do_stride_n;
  if ((p & 15) || (s & 7)) return 0;
  // row offsets within one time step are kept in 32 bits inside the kernels
  const int64_t big = (int64_t)1 << 31;
  if (a->C * a->q_stride_n >= big || a->C * a->k_stride_n >= big || a->C * a->v_stride_n >= big ||
      a->C * a->do_stride_n >= big || a->q_stride_n < 0 || a->k_stride_n < 0 || a->v_stride_n < 0 ||
      a->do_stride_n < 0)
    return 0;
  return 1;
}

template <int DH, int NCT>
static void launch_query(const mvpa_bwd_args* a, hipStream_t stream, int q0, int k0, int accum) {
  using namespace mvpa::bwdq;
  constexpr int nw = QUERY_WAVES<DH, NCT>, tqw = nw / NCT, cp = NCT * 32, ROWB = 2 * DH;
  const int nt = (a->T + tqw - 1) / tqw;
  const size_t lds = (size_t)QSTAGES<DH, NCT> * 3 * cp * ROWB + (size_t)nw * WAVE_SCRATCH * sizeof(float);
  dim3 grid((unsigned)(nt * a->B * a->H));
  auto kern = mvpa_bwd_query_mfma_kernel<DH, NCT>;
  mvpa::want_dynamic_lds((const void*)kern, (int)lds);
  MVPA_LAUNCH(kern, grid, dim3(nw * 64), lds, stream, *a, q0, k0, accum);
}

// ==========================================================================================
// The KEY pass: dk, dv.  A workgroup owns 4 consecutive key time steps of one kv head; a
// wave owns 32 key channels of one of them (its K and V rows stay in registers as MFMA B
// operands) and walks every query time step tq >= tk of every query head of the group, both
// query-channel tiles in turn.  Products are formed NON-transposed here, S[q][key] = (q+u) K^T,
// so that a lane owns one key and the contraction index of dv^T = dO^T P and dk^T = (q+u)^T dS
// is the register index.  With Ec[q][key] = exp2(channel bias - mc[q]) and, per (query, tk), one
// scalar from the query pass (the exponent e = time bias - L + mc inside the content window,
// exp2(e) outside it):
//     inside :  P = exp2((q+u) K^T + e) o Ec,  dP = dO V^T,  dS = P o (dP - delta[q])
//               dv^T[d][key] += dO^T[d][q] P[q][key],   dk^T[d][key] += (q+u)^T[d][q] dS[q][key]
//     outside:  P = exp2(e) Ec,                dv^T += dO^T P           (dk gets nothing)
// Per (head, tq) one ring stage holds dO in the transposing-read swizzle, the Ec tile and the
// scalars, and for steps that are inside the window for some wave also dO in the row-fragment
// swizzle, (q+u) * scale in both swizzles and delta; direct-to-LDS loads fetch it two steps
// ahead.  The query steps are walked from the last one down and the workgroups of one
// (b, kv head) sit on one XCD: they then read the same stage data at about the same time and
// share it in L2.  MASKED: the query part holds fewer channels than its tiles, padded query rows are cut.
// ==========================================================================================
namespace mvpa {
namespace bwdq {

// waves per workgroup of the key pass: every wave of a workgroup reads the same stage (only the
// per-key-step scalars differ), so with two channel tiles 8 waves (4 key steps) share it and each
// SIMD holds two waves
template <int NCT> constexpr int KEY_WAVES = NCT == 2 ? 8 : 4;

template <int DH, int NCT, bool MASKED>
__global__ __launch_bounds__(KEY_WAVES<NCT> * 64) void mvpa_bwd_key_mfma_kernel(mvpa_bwd_args a, int k0, int q0, int accum) {
  constexpr int KS = DH / 16, MT = DH / 32, ROWB = 2 * DH, CPR = DH / 8;
  constexpr int NW = KEY_WAVES<NCT>;
  constexpr int CP = NCT * 32, KT = NW / NCT, TILE = CP * ROWB;
  constexpr int CS_BYTES = CP * CP * 4, SC_BYTES = (KT + 1) * 256;
  constexpr int STAGES = KSTAGES, STAGE_BYTES = 4 * TILE + CS_BYTES + SC_BYTES;
  static_assert(STAGES == 3, "the wait below counts the loads of exactly one younger step");
  constexpr int LPW = TILE / 1024 / NW, CS_LPW = CS_BYTES / 1024 / NW;
  // direct-to-LDS loads per wave and step
  constexpr int LPS_FAR = LPW + CS_LPW + 1, LPS_NEAR = 4 * LPW + CS_LPW + 2;
  // stage layout: dO (transposing) | Ec | scalars | dO (rows) | (q+u) (rows) | (q+u) (transposing)
  constexpr int OFF_DTR = 0, OFF_EC = TILE, OFF_SC = TILE + CS_BYTES, OFF_DROW = OFF_SC + SC_BYTES,
                OFF_QROW = OFF_DROW + TILE, OFF_QTR = OFF_QROW + TILE;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, hh = lane >> 5;
  const int ktw = wave / NCT, kt = wave % NCT;    // this wave's key step and key-channel tile
  const int T_ = a.T, C_ = a.C, W = a.window, N = a.T * a.C;
  const int CW = (C_ + 3) & ~3;                   // row pitch of the Ec tiles in the workspace
  const bool has_content = a.flags & MVPA_FLAG_CONTENT;
  const int nbg = a.B * a.Hkv, ntk = (T_ + KT - 1) / KT;
  int bg, tile;
  {
    const int L = blockIdx.x;
    if ((nbg & 7) == 0) {
      const int s = L >> 3;
      bg = (L & 7) + 8 * (s / ntk);
      tile = s % ntk;                             // early key steps (most queries) first
    } else {
      bg = L / ntk;
      tile = L % ntk;
    }
  }
  const int b = bg / a.Hkv, g = bg % a.Hkv;
  const int grp = a.H / a.Hkv;
  const int tk0 = tile * KT;
  const int tk = tk0 + ktw;
  const bool wave_on = tk < T_;
  const int tkc = min(tk, T_ - 1);

  const int ck = k0 + kt * 32 + ln;               // key channels k0 .., query channels q0 .. in this launch
  const int ckl = kt * 32 + ln;                   // ... local to the launch
  // Lanes of key channels beyond C own columns of dk / dv that are never stored, and a product's
  // column depends on no other lane's operand: they need no masking.  Padded QUERY rows are the
  // contraction index of both gradient products; their probabilities are cut after packing, with
  // one mask per fragment dword (two queries) kept in registers (per-element predicates were
  // hoisted out of the loop as 32 lane masks and spilled the scalar registers).
  uint32_t qmask[NCT][8];
#pragma unroll
  for (int qt = 0; qt < NCT; ++qt)
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      const int i = 2 * w;                        // elements i, i + 1 of the tile: queries qa, qa + 1
      const int qa = q0 + qt * 32 + (i >> 2) * 8 + hh * 4 + (i & 3);
      qmask[qt][w] = MASKED ? ((qa < C_ ? 0x0000ffffu : 0u) | (qa + 1 < C_ ? 0xffff0000u : 0u)) : 0xffffffffu;
    }
  auto cut = [&](bf16x8 f, int qt, int s) -> bf16x8 {
    if (!MASKED) return f;
    union { bf16x8 b; u32x4 u; } c;
    c.b = f;
#pragma unroll
    for (int w = 0; w < 4; ++w) c.u[w] &= qmask[qt][4 * s + w];
    return c.b;
  };
  const int64_t nk = (int64_t)tkc * C_ + min(ck, C_ - 1);
  const bf16_t* krow = (const bf16_t*)a.k + b * a.k_stride_b + g * a.k_stride_h + nk * a.k_stride_n;
  const bf16_t* vrow = (const bf16_t*)a.v + b * a.v_stride_b + g * a.v_stride_h + nk * a.v_stride_n;
  bf16x8 Kf[KS], Vf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    Kf[ks] = as_frag(*(const u32x4*)(krow + ks * 16 + hh * 8));
    Vf[ks] = as_frag(*(const u32x4*)(vrow + ks * 16 + hh * 8));
  }

  // ---- the ring: per-wave source offsets (swizzles applied on the source side)
  int q_off_r[LPW], q_off_t[LPW], d_off_r[LPW], d_off_t[LPW], cs_off[CS_LPW];
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int pc = (wave + NW * i) * 64 + lane;
    const int r = pc / CPR, phys = pc % CPR;
    const int rc = min(q0 + r, C_ - 1);
    q_off_r[i] = rc * DH + ((phys ^ swz_row<DH>(r)) << 3);
    q_off_t[i] = rc * DH + ((phys ^ swz_tr<DH>(r)) << 3);
    d_off_r[i] = rc * (int)a.do_stride_n + ((phys ^ swz_row<DH>(r)) << 3);
    d_off_t[i] = rc * (int)a.do_stride_n + ((phys ^ swz_tr<DH>(r)) << 3);
  }
  // the Ec tile [C][C] lands with a row pitch of CP floats
#pragma unroll
  for (int i = 0; i < CS_LPW; ++i) {
    const int pc = (wave + NW * i) * 64 + lane;   // 16-byte chunk: row pc / (CP/4), 4 columns
    const int r = min(q0 + pc / (CP / 4), C_ - 1), c4 = min((pc % (CP / 4)) * 4, max(CW - k0 - 4, 0));
    cs_off[i] = r * CW + k0 + c4;
  }
  const int sc_lane = min(q0 + lane, C_ - 1);
  const uint32_t ring_lds = (uint32_t)(uintptr_t)(BWD_LDS_PTR(unsigned char))smem;
  // a step is fetched in full when it lies inside the content window of one of the waves
  auto wg_near = [&](int tq) -> bool {
    return has_content && (W <= 0 || tq == T_ - 1 || tq - tk0 <= W + KT - 1);
  };
  // source pointers of the step the ring fetches next: re-based at each head, stepped down by
  // one query time step otherwise (the full address arithmetic per step cost as many scalar
  // instructions as a far step has vector ones)
  const bf16_t* p_do = nullptr;
  const bf16_t* p_qu = nullptr;
  const float* p_ec = nullptr;
  const float* p_sc = nullptr;
  const float* p_de = nullptr;
  const int64_t d_do = (int64_t)C_ * a.do_stride_n, d_sc = (int64_t)T_ * C_;
  const int d_ec = C_ * CW, d_qu = C_ * DH;
  auto rebase = [&](int hq) {
    const int h = g * grp + hq;
    const int64_t bhq = (int64_t)b * a.H + h;
    const int64_t r0 = bhq * N + (int64_t)(T_ - 1) * C_;    // first query row of step T-1
    p_do = (const bf16_t*)a.d_o + b * a.do_stride_b + h * a.do_stride_h + (int64_t)(T_ - 1) * d_do;
    p_qu = (const bf16_t*)a.ws_qu + r0 * DH;
    p_ec = a.ws_chan + r0 * CW;
    p_sc = a.ws_time + ((bhq * T_ + (T_ - 1)) * T_ + tkc) * C_;
    p_de = a.ws_delta + r0;
  };
  auto issue_step = [&](int tq, int stage_idx) {
    const uint32_t st = ring_lds + stage_idx * STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < LPW; ++i) dma16(p_do + d_off_t[i], st + OFF_DTR + (wave + NW * i) * 1024);
#pragma unroll
    for (int i = 0; i < CS_LPW; ++i) dma16(p_ec + cs_off[i], st + OFF_EC + (wave + NW * i) * 1024);
    // per-query scalar of this wave's key step
    dma4(p_sc + sc_lane, st + OFF_SC + ktw * 256);
    if (wg_near(tq)) {
#pragma unroll
      for (int i = 0; i < LPW; ++i) {
        const uint32_t dst = st + (wave + NW * i) * 1024;
        dma16(p_do + d_off_r[i], dst + OFF_DROW);
        dma16(p_qu + q_off_r[i], dst + OFF_QROW);
        dma16(p_qu + q_off_t[i], dst + OFF_QTR);
      }
      dma4(p_de + sc_lane, st + OFF_SC + KT * 256);
    }
  };

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
    for (int ks = 0; ks < KS; ++ks) r_lane[ks] = ln * ROWB + (((2 * ks + hh) ^ swz_row<DH>(ln)) << 4);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      t_lane[mt] = row0 * ROWB + (((4 * mt + 2 * grp16 + (aa >> 1)) ^ swz_tr<DH>(row0)) << 4) + ((aa & 1) << 3);
  }
  auto tr_frag = [&](const unsigned char* tile_p, int qt, int s, int mt) -> bf16x8 {
    const unsigned char* p = tile_p + t_lane[mt] + (32 * qt + 16 * s) * ROWB;
    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((BWD_LDS_PTR(bf16x4))p);
    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((BWD_LDS_PTR(bf16x4))(p + 8 * ROWB));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };

  // steps: query heads of the group, and for each the query steps T-1 .. tk0
  const int span = T_ - tk0, nsteps = grp * span;
  int ihq = 0, itq = T_ - 1;                      // the step the ring fetches next
  rebase(0);
  auto next_issue = [&]() {
    if (--itq < tk0) {
      itq = T_ - 1;
      if (++ihq < grp) rebase(ihq);
    } else {
      p_do -= d_do;
      p_qu -= d_qu;
      p_ec -= d_ec;
      p_sc -= d_sc;
      p_de -= C_;
    }
  };
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s < nsteps) { issue_step(itq, s); next_issue(); }

  int stage = 0, it = 0, ring_tq = T_ - 1;        // ring_tq: query step of the stage handed out next
  // advances the ring by one step and returns the stage that holds its data
  auto ring_step = [&]() -> const unsigned char* {
    // the step has landed once only the loads of the one younger step are in flight
    const int next_tq = ring_tq - 1 < tk0 ? T_ - 1 : ring_tq - 1;
    if (it + 1 >= nsteps) wait_vmcnt_imm<0>();
    else if (wg_near(next_tq)) wait_vmcnt_imm<LPS_NEAR>();
    else wait_vmcnt_imm<LPS_FAR>();
    lds_barrier();            // this step's stage visible to all; the previous one is free
    if (it + STAGES - 1 < nsteps) { issue_step(itq, stage == 0 ? STAGES - 1 : stage - 1); next_issue(); }
    const unsigned char* base = smem + stage * STAGE_BYTES;
    stage = stage + 1 == STAGES ? 0 : stage + 1;
    ring_tq = next_tq;
    ++it;
    return base;
  };

  // ---- a query step outside the content window: P = Ec * exp2(e), dv only
  auto far_step = [&](const unsigned char* base) {
    const unsigned char* Dtr = base + OFF_DTR;
    const float* Ecs = (const float*)(base + OFF_EC) + ckl;
    const float* ET = (const float*)(base + OFF_SC) + ktw * 64;
#pragma unroll
    for (int qt = 0; qt < NCT; ++qt) {
      f32x16 P;
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4) {
        const int rb = qt * 32 + a4 * 8 + hh * 4;              // query channels rb .. rb+3
        const float4 e4 = *(const float4*)(ET + rb);
        const float es[4] = {e4.x, e4.y, e4.z, e4.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          P[a4 * 4 + j] = Ecs[(rb + j) * CP] * es[j];
        }
      }
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const bf16x8 pf = cut(pack8(P, 8 * s), qt, s);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          dV[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(Dtr, qt, s, mt), pf, dV[mt], 0, 0, 0);
      }
    }
  };

  // ---- a query step inside the content window
  auto near_step = [&](const unsigned char* base) {
    const unsigned char* Dtr = base + OFF_DTR;
    const unsigned char* Drow = base + OFF_DROW;
    const unsigned char* Qrow = base + OFF_QROW;
    const unsigned char* Qtr = base + OFF_QTR;
    const float* Ecs = (const float*)(base + OFF_EC) + ckl;
    const float* TL = (const float*)(base + OFF_SC) + ktw * 64;
    const float* De = (const float*)(base + OFF_SC) + KT * 64;
#pragma unroll
    for (int qt = 0; qt < NCT; ++qt) {
      f32x16 S, dP, dS;
#pragma unroll
      for (int i = 0; i < 16; ++i) { S[i] = 0.f; dP[i] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int off = r_lane[ks] + qt * 32 * ROWB;
        S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)(Qrow + off), Kf[ks], S, 0, 0, 0);
        dP = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)(Drow + off), Vf[ks], dP, 0, 0, 0);
      }
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4) {
        const int rb = qt * 32 + a4 * 8 + hh * 4;
        const float4 tl = *(const float4*)(TL + rb);
        const float4 de = *(const float4*)(De + rb);
        const float tls[4] = {tl.x, tl.y, tl.z, tl.w}, des[4] = {de.x, de.y, de.z, de.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int i = a4 * 4 + j;
          const float p = __builtin_amdgcn_exp2f(S[i] + tls[j]) * Ecs[(rb + j) * CP];
          S[i] = p;
          dS[i] = p * (dP[i] - des[j]) * (1.f / kLog2e);
        }
      }
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const bf16x8 pf = cut(pack8(S, 8 * s), qt, s);
        const bf16x8 sf = cut(pack8(dS, 8 * s), qt, s);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          dV[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(Dtr, qt, s, mt), pf, dV[mt], 0, 0, 0);
          dK[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(Qtr, qt, s, mt), sf, dK[mt], 0, 0, 0);
        }
      }
    }
  };

  // this wave's steps of one head, walking down from tq = T-1: the last query step keeps the
  // content term, then the steps beyond the window, then the window, then the steps before tk
  int n_last = 0, n_far = 0, n_win = 0;
  if (wave_on) {
    const int live = T_ - tk;
    if (!has_content) n_far = live;
    else if (W <= 0) n_win = live;
    else {
      n_last = 1;
      n_far = max(0, live - 2 - W);
      n_win = live - 1 - n_far;
    }
  }
  const int n_idle = span - n_last - n_far - n_win;
  for (int hq = 0; hq < grp; ++hq) {
    for (int n = n_last; n > 0; --n) near_step(ring_step());
    for (int n = n_far; n > 0; --n) far_step(ring_step());
    for (int n = n_win; n > 0; --n) near_step(ring_step());
    for (int n = n_idle; n > 0; --n) (void)ring_step();
  }

  if (wave_on && ck < C_) {
    const int64_t o = ((((int64_t)b * a.Hkv + g) * N) + (int64_t)tk * C_ + ck) * DH;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4) {
        const int d = mt * 32 + a4 * 8 + hh * 4;
        float4 vk = make_float4(dK[mt][a4 * 4], dK[mt][a4 * 4 + 1], dK[mt][a4 * 4 + 2], dK[mt][a4 * 4 + 3]);
        float4 vv = make_float4(dV[mt][a4 * 4], dV[mt][a4 * 4 + 1], dV[mt][a4 * 4 + 2], dV[mt][a4 * 4 + 3]);
        if (accum) {                              // launches of one stream: the query parts add up
          const float4 ok = *(const float4*)(a.dk + o + d), ov = *(const float4*)(a.dv + o + d);
          vk = make_float4(vk.x + ok.x, vk.y + ok.y, vk.z + ok.z, vk.w + ok.w);
          vv = make_float4(vv.x + ov.x, vv.y + ov.y, vv.z + ov.z, vv.w + ov.w);
        }
        *(float4*)(a.dk + o + d) = vk;
        *(float4*)(a.dv + o + d) = vv;
      }
  }
}

}  // namespace bwdq
}  // namespace mvpa

template <int DH, int NCT, bool MASKED>
static void launch_key(const mvpa_bwd_args* a, hipStream_t stream, int k0, int q0, int accum) {
  using namespace mvpa::bwdq;
  constexpr int nw = KEY_WAVES<NCT>, cp = NCT * 32, kt = nw / NCT, ROWB = 2 * DH;
  static_assert((size_t)KSTAGES * (4 * cp * ROWB + cp * cp * 4 + (kt + 1) * 256) <= 160 * 1024, "key-pass ring exceeds the LDS");
  const size_t lds = (size_t)KSTAGES * (4 * cp * ROWB + cp * cp * 4 + (kt + 1) * 256);
  dim3 grid((unsigned)(((a->T + kt - 1) / kt) * a->B * a->Hkv));
  auto kern = mvpa_bwd_key_mfma_kernel<DH, NCT, MASKED>;
  mvpa::want_dynamic_lds((const void*)kern, (int)lds);
  MVPA_LAUNCH(kern, grid, dim3(nw * 64), lds, stream, *a, k0, q0, accum);
}

// Both passes.  Up to 32 channels: one launch each with one channel tile per wave; up to 64: one
// launch each with two.  Beyond that the channels are taken in parts of 64: with the forward's
// log-sum-exp known, the contributions of disjoint key channels (to dq and the bias-table
// gradients) and of disjoint query channels (to dk, dv) simply add up, so every (query part, key
// part) pair is one query-pass launch followed by the key-pass launch that consumes its
// workspace; later launches add to what earlier ones wrote (one stream, hence ordered).
// At Dh 128 a key-pass stage of 64 channels does not fit the LDS three times: the key pass then
// takes the (query part, key part) pair of a query-pass launch in quarters of 32 x 32 channels
// (the workspace is indexed by absolute channel, and its per-row maximum covers the whole key part).
template <int DH>
static void launch_bwd_parts(const mvpa_bwd_args* a, hipStream_t stream) {
  const int C = a->C;
  constexpr int KEY_CP = DH == 64 ? 64 : 32;      // channels per key-pass launch
  auto key_launches = [&](int q0, int k0, int span, bool first_q) {
    for (int kk = k0; kk < min(k0 + span, C); kk += KEY_CP)
      for (int qq = q0; qq < min(q0 + span, C); qq += KEY_CP) {
        const int accum = !(first_q && qq == q0);
        const bool full = C - qq >= KEY_CP && C - kk >= KEY_CP;
        if (full) launch_key<DH, KEY_CP / 32, false>(a, stream, kk, qq, accum);
        else launch_key<DH, KEY_CP / 32, true>(a, stream, kk, qq, accum);
      }
  };
  if (C <= 32) {
    launch_query<DH, 1>(a, stream, 0, 0, 0);
    if (C == 32) launch_key<DH, 1, false>(a, stream, 0, 0, 0);
    else launch_key<DH, 1, true>(a, stream, 0, 0, 0);
  } else {
    const int parts = (C + 63) / 64;
    for (int kp = 0; kp < parts; ++kp)
      for (int qp = 0; qp < parts; ++qp) {
        launch_query<DH, 2>(a, stream, qp * 64, kp * 64, kp > 0);
        key_launches(qp * 64, kp * 64, 64, qp == 0);
      }
  }
}

int mvpa_launch_bwd_mfma(const mvpa_bwd_args* a, hipStream_t stream) {
  if (a->Dh == 64) launch_bwd_parts<64>(a, stream);
  else launch_bwd_parts<128>(a, stream);
  return mvpa::take_launch_status();
}
