// bf16 MFMA forward for 33..128 channels at head size 128 or 64 (gfx950, wave64): a wave owns one
// tile of 32 queries and 64 output columns.
//
// Head size 128: the general tiled kernel (mvpa_mfma.hip) gives a wave one tile of 32 queries and
// all 128 output columns: 64 accumulator registers, 64 more for the product of a far step, the
// channel-bias tile and the (q+u) fragments - it only fits at one wave per SIMD, and there every
// wait (an LDS read, the barrier, a dependent matrix instruction) idles the matrix pipe.  Here the
// output columns of a query tile are split over two waves: a workgroup is one time step, 8 waves
// = (up to) 4 query tiles x 2 column halves, two waves per SIMD.  The two waves of a query tile
// compute the same scores and the same soft-max state (nothing is exchanged between them) and
// differ only in the V^T fragments they read and the columns they write.
//
// Head size 64: a wave owns every output column of its tile, and the 8 waves of a workgroup are
// the 4 query tiles of TWO consecutive time steps on one K/V ring (the general kernel instead
// splits the keys of a step over two waves, each with half the products per key step and a merge
// at the end).  The keys are padded to 64 or 128 channels (two or four key tiles; with two, a time
// step has two query tiles and a workgroup takes twice as many time steps).
//
// The key steps are taken window steps first, far steps after (the online soft-max does not care
// about the order): the channel-bias tile Bc and the (q+u) fragments are live only in the window
// steps, the operands Ec = exp2(Bc - mc) of the far products (layers/mvpa.py:231-245:
// p = et[q,tk] * Ec[q,ck] wherever the content term is zeroed) only afterwards.
//
// K/V tiles travel through a ring of four slots of one tile each: a window step takes two slots
// (K, V), a far step one (V), so that three far tiles are in flight while one is consumed.
#include "mvpa_mfma_tools.h"

namespace mvpa {
namespace d128 {

constexpr int MT = 2, NW = 8, SLOTS = 4;                // a wave owns 64 output columns
constexpr int STB_WAVE = 32 * 32 * 4;                  // time-bias slab of a wave's query tile

template <int DH, int NCT>
struct Geo {
  static constexpr int KS = DH / 16, ROWB = DH * 2, CHUNKS = DH / 8;
  static constexpr int HALVES = DH / 64;               // waves per query tile (column halves)
  static constexpr int QT = NCT <= 2 ? 2 : 4;          // query-tile slots per time step
  static constexpr int TQW = NW / (HALVES * QT);       // time steps per workgroup
  static constexpr int CP = 32 * NCT;                  // channels, padded
  static constexpr int TILE_BYTES = CP * ROWB;         // one K or V tile
  static constexpr int LPW = TILE_BYTES / 1024 / NW;   // 64-lane x 16-byte loads per tile and wave
  static constexpr int RING_BYTES = SLOTS * TILE_BYTES;
  static constexpr int SCRATCH_WAVE = CP * 32 * 4;     // set-up scratch [CP][32] of a wave
  // the scratch lies over the ring and the slabs (both are idle during the set-up)
  static constexpr int LDS_BYTES = RING_BYTES + NW * STB_WAVE > NW * SCRATCH_WAVE ? RING_BYTES + NW * STB_WAVE
                                                                                   : NW * SCRATCH_WAVE;
  static_assert(DH == 64 || DH == 128, "head size 64 or 128");
  static_assert(LPW * 1024 * NW == TILE_BYTES, "a tile is a whole number of loads per wave");
};

template <int U>
__device__ inline void wait_units(int n) {            // at most n * U loads of this wave outstanding
  if (n <= 0) wait_vmcnt_imm<0>();
  else if (n == 1) wait_vmcnt_imm<U>();
  else if (n == 2) wait_vmcnt_imm<2 * U>();
  else wait_vmcnt_imm<3 * U>();
}

template <int DH, int NCT, bool FP8>
__global__ __launch_bounds__(NW * 64) void mvpa_mfma128_kernel(mvpa_fwd_args a) {
  using G = Geo<DH, NCT>;
  constexpr int TILE_BYTES = G::TILE_BYTES, LPW = G::LPW, RING_BYTES = G::RING_BYTES;
  constexpr int KS = G::KS, ROWB = G::ROWB, CHUNKS = G::CHUNKS, HALVES = G::HALVES, TQW = G::TQW, QT = G::QT;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, hh = lane >> 5;
  // query tile, column half and time step (within the workgroup) of this wave
  const int half = wave % HALVES, qi = (wave / HALVES) % QT, ts = wave / (HALVES * QT);
  const int C_ = a.C, W = a.window, T_ = a.T;
  const bool has_content = a.flags & MVPA_FLAG_CONTENT;
  const bool has_time = a.flags & MVPA_FLAG_TIME_BIAS;
  const bool has_chan = a.flags & MVPA_FLAG_CHAN_BIAS;

  // ---- block -> (b*H + h, time step): ids that are equal mod 8 run on one XCD and get the same
  // (b, h), so that its K/V stay in that XCD's L2.  The last time step of every (b, h) goes out
  // first (with the content term on it keeps that term for every key step, layers/mvpa.py:244,
  // and takes longest), then one (b, h) after the other, late (= long) steps first; the last two
  // (b, h) of an XCD are interleaved so that the grid does not end on the long steps of one.
  const int nt = (T_ + TQW - 1) / TQW;
  const int nbh = a.B * a.H;
  int bh, tile;
  map_block(blockIdx.x, nbh, nt, a.H / a.Hkv, bh, tile);
  const int b = bh / a.H, h = bh % a.H;
  const int g = h / (a.H / a.Hkv);
  const int tq0 = tile * TQW, tq_hi = min(T_ - 1, tq0 + TQW - 1);
  const int tq = min(tq0 + ts, T_ - 1);              // (a wave past the end repeats the last step and stores nothing)
  const int cb = 32 * qi;                            // first channel of this wave's queries
  const bool live = cb < C_ && tq0 + ts < T_;        // (a wave without queries still moves tiles)

  // ---- for this wave's queries key steps 0 .. far_max are far (content term absent or zeroed),
  // far_max+1 .. tq window steps.  The workgroup walks window tiles NLO .. tq_hi (a wave skips
  // what lies outside its own window) and far tiles 0 .. FM (a wave stops at its own far_max).
  const int far_max = !has_content ? tq : (W > 0 && tq != T_ - 1) ? max(-1, tq - W - 1) : -1;
  int FM = -1;
  if (!has_content) {
    FM = tq_hi;
  } else if (W > 0) {
    const int tql = tq_hi == T_ - 1 ? tq_hi - 1 : tq_hi;       // the last step has no far steps
    if (tql >= tq0) FM = max(-1, tql - W - 1);
  }
  const int NLO = (W <= 0 || tq_hi == T_ - 1) ? 0 : max(0, tq0 - W);
  const int n_near = has_content ? tq_hi - NLO + 1 : 0;
  const int n_far = FM + 1;

  // Loads below are unconditional: rows of padded channels are redirected to an existing row and
  // their results are never used.
  const unsigned char* qbase = (const unsigned char*)((const bf16_t*)a.q + b * a.q_stride_b + h * a.q_stride_h);
  const uint32_t qoff = (uint32_t)((tq * C_ + min(cb + ln, C_ - 1)) * a.q_stride_n) * 2u + hh * 16;
  auto q_chunk = [&](int ks) -> u32x4 { return *(const u32x4*)(qbase + qoff + ks * 32); };
  const bf16_t* kbase = (const bf16_t*)a.k + b * a.k_stride_b + g * a.k_stride_h;
  const bf16_t* vbase = (const bf16_t*)a.v + b * a.v_stride_b + g * a.v_stride_h;
  const bf16_t* ktime = (const bf16_t*)a.k_time + (int64_t)g * T_ * DH;
  const bf16_t* kchan = (const bf16_t*)a.k_chan + (int64_t)g * C_ * DH;
  const bf16_t* bu = (const bf16_t*)a.bias_u + g * DH;
  const bf16_t* bv = (const bf16_t*)a.bias_v + g * DH;
  const bf16_t* bz = (const bf16_t*)a.bias_z + g * DH;
  const uint8_t* valid = a.chan_valid ? a.chan_valid + (int64_t)b * C_ : nullptr;
  const float sc2 = a.sm_scale * kLog2e;           // scores live in the base-2 domain

  // =========================== tile ring ===========================
  // rows in natural [key][dh] order, 16-byte chunks XOR-swizzled on the global side; rows of padded
  // channels fetch the last real channel and are neutralised by Ec = 0 / Bc = -inf
  uint32_t k_off[LPW], v_off[LPW];         // byte offsets of this lane's chunks within a tile
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int pc = (wave + NW * i) * 64 + lane;
    const int row = pc / CHUNKS, phys = pc % CHUNKS;
    const int rowc = min(row, C_ - 1);
    k_off[i] = (uint32_t)(rowc * a.k_stride_n) * 2u + ((phys ^ swz_k<DH>(row)) << 4);
    v_off[i] = (uint32_t)(rowc * a.v_stride_n) * 2u + ((phys ^ swz_v<DH>(row)) << 4);
  }
  // fp8 content term: the window steps stream the e4m3 copy of the keys (a.k_fp8, one byte per
  // element, contiguous [B,Hkv,N,DH]) into the K slot instead of the bf16 rows: rows of DH bytes
  // in natural [key][dh] order, 16-byte chunks XOR-swizzled so that 8 lanes reading the same
  // logical chunk of 8 consecutive rows cover all banks.  A key tile is K8_LOADS loads of 64 x 16
  // bytes; with fewer of them than waves some waves fetch a chunk a second time (same bytes to
  // the same place), so that every wave issues the same number of loads.
  constexpr int K8_CHUNKS = DH / 16, K8_LOADS = G::CP * DH / 1024, LPW8 = (K8_LOADS + NW - 1) / NW;
  auto swz8 = [](int row) -> int { return DH == 128 ? (row & 7) : ((row >> 1) & 3); };
  uint32_t k8_off[LPW8], k8_dst[LPW8];
  if (FP8) {
#pragma unroll
    for (int i = 0; i < LPW8; ++i) {
      const int ld = (wave + NW * i) % K8_LOADS;
      const int pc = ld * 64 + lane;
      const int row = pc / K8_CHUNKS, phys = pc % K8_CHUNKS;
      k8_off[i] = (uint32_t)(min(row, C_ - 1) * DH) + ((phys ^ swz8(row)) << 4);
      k8_dst[i] = ld * 1024;
    }
  }
  const unsigned char* k8base = FP8 ? (const unsigned char*)a.k_fp8 + ((int64_t)b * a.Hkv + g) * ((int64_t)T_ * C_ * DH) : nullptr;
  const int64_t k8step = (int64_t)C_ * DH;
  const uint32_t ring_lds = (uint32_t)(uintptr_t)(LDS_PTR(unsigned char))smem_raw;
  // Tiles are requested in stream order - window steps NLO .. tq (K and V), then far steps
  // 0 .. far_max (V only) - whenever the slots they need are free.  `used` counts the slots of
  // tiles requested and not yet consumed; `issued` the requests in units of LPW loads.
  const int64_t kstep = (int64_t)C_ * a.k_stride_n, vstep = (int64_t)C_ * a.v_stride_n;
  int iss_pos = 0, iss_slot = 0, used = 0, issued = 0;
  const bf16_t* iss_k = kbase + (n_near > 0 ? NLO : 0) * kstep;
  const bf16_t* iss_v = vbase + (n_near > 0 ? NLO : 0) * vstep;
  const unsigned char* iss_k8 = FP8 ? k8base + (n_near > 0 ? NLO : 0) * k8step : nullptr;
  auto issue_avail = [&]() {
    while (iss_pos < n_near) {
      const bool is_near = true;
      if (used + (is_near ? 2 : 1) > SLOTS) break;
      uint32_t slot = ring_lds + iss_slot * TILE_BYTES;
      if (is_near) {
        if (FP8) {
#pragma unroll
          for (int i = 0; i < LPW8; ++i) load_to_lds_16(iss_k8, k8_off[i], slot + k8_dst[i]);
          iss_k8 += k8step;
        } else {
#pragma unroll
          for (int i = 0; i < LPW; ++i) load_to_lds_16(iss_k, k_off[i], slot + (wave + NW * i) * 1024);
          iss_k += kstep;
        }
        slot += TILE_BYTES;
      }
#pragma unroll
      for (int i = 0; i < LPW; ++i) load_to_lds_16(iss_v, v_off[i], slot + (wave + NW * i) * 1024);
      iss_v += vstep;
      const int ns = is_near ? 2 : 1;
      used += ns;
      issued += ns;
      iss_slot = (iss_slot + ns) & (SLOTS - 1);
      ++iss_pos;
      if (iss_pos == n_near) iss_v = vbase;       // the far phase starts at key step 0
    }
  };

  float* stb_wave = (float*)(smem_raw + RING_BYTES + wave * STB_WAVE);

  // ---- per-lane pieces of the LDS fragment addresses (see the general kernel)
  int v_lane[MT], k_lane[KS];
  {
    const int e = (ln & 15) >> 2, aa = ln & 3, grp = ln >> 4;
    const int row0 = 4 * hh + e;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const int mt = (HALVES == 2 ? 2 * half : 0) + m;     // output tile (32 columns) within the row
      v_lane[m] = row0 * ROWB + (((4 * mt + 2 * grp + (aa >> 1)) ^ swz_v<DH>(row0)) << 4) + ((aa & 1) << 3);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_lane[ks] = ln * ROWB + (((2 * ks + hh) ^ swz_k<DH>(ln)) << 4);
    // fp8 keys: one 16-byte read serves two products.  Read p of a lane covers the head
    // dimensions [(2p + hh) * 16, +16) of its key row: the low 8 bytes go to product 2p, the high
    // 8 to product 2p + 1 (the query fragments are laid out to match).
    if (FP8) {
#pragma unroll
      for (int p2 = 0; p2 < KS / 2; ++p2) k_lane[p2] = ln * DH + (((2 * p2 + hh) ^ swz8(ln)) << 4);
    }
  }
  // Fragment addresses of a step: one register per output tile (V^T) / k-step (K) = lane part +
  // slot, formed once per step and made opaque to the compiler, so that everything else of an
  // address stays an immediate offset of the LDS instruction.
  struct VAddr { uint32_t v[MT]; };
  struct KAddr { uint32_t k[KS]; };
  auto v_addr = [&](int slot) {
    VAddr sa;
    const uint32_t base = ring_lds + slot * TILE_BYTES;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      sa.v[m] = base + v_lane[m];
      asm volatile("" : "+v"(sa.v[m]));
    }
    return sa;
  };
  auto k_addr = [&](int slot) {
    KAddr sa;
    const uint32_t base = ring_lds + slot * TILE_BYTES;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      sa.k[ks] = base + k_lane[ks];
      asm volatile("" : "+v"(sa.k[ks]));
    }
    return sa;
  };
  auto v_frag = [&](const VAddr& sa, int t, int s, int m) -> bf16x8 {
    const uint32_t p = sa.v[m] + (32 * t + 16 * s) * ROWB;
    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((LDS_PTR(bf16x4))(uintptr_t)p);
    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((LDS_PTR(bf16x4))(uintptr_t)(p + 8 * ROWB));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  auto k_frag = [&](const KAddr& sa, int t, int ks) -> bf16x8 {
    return *(LDS_PTR(const bf16x8))(uintptr_t)(sa.k[ks] + t * 32 * ROWB);
  };

  // running soft-max state (a lane owns one query): reference point, per-half-wave partial sum
  f32x16 acc[MT];
  float m_run = kMFloor, l_run = 0.f;
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[m][i] = 0.f;

  // in-place rescale of the accumulators.  Inline assembly: the products before it are matrix
  // instructions whose results the assembler's hazard logic cannot see into, hence the waits.
  auto rescale_acc = [&](float alpha) {
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      f32x16 x = acc[m];
      asm volatile(
          "s_nop 7\n\ts_nop 3\n\t"
          "v_mul_f32 %0, %16, %0\n\tv_mul_f32 %1, %16, %1\n\tv_mul_f32 %2, %16, %2\n\tv_mul_f32 %3, %16, %3\n\t"
          "v_mul_f32 %4, %16, %4\n\tv_mul_f32 %5, %16, %5\n\tv_mul_f32 %6, %16, %6\n\tv_mul_f32 %7, %16, %7\n\t"
          "v_mul_f32 %8, %16, %8\n\tv_mul_f32 %9, %16, %9\n\tv_mul_f32 %10, %16, %10\n\tv_mul_f32 %11, %16, %11\n\t"
          "v_mul_f32 %12, %16, %12\n\tv_mul_f32 %13, %16, %13\n\tv_mul_f32 %14, %16, %14\n\tv_mul_f32 %15, %16, %15\n\t"
          "s_nop 1"
          : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7]),
            "+v"(x[8]), "+v"(x[9]), "+v"(x[10]), "+v"(x[11]), "+v"(x[12]), "+v"(x[13]), "+v"(x[14]), "+v"(x[15])
          : "v"(alpha));
      acc[m] = x;
    }
  };

  // =========================== set-up ===========================
  // Bc[ck][q] = (q+z).e[C-1-|cq-ck|] * scale in accumulator layout (-inf = masked key) and the
  // (q+u) fragments.  The whole channel table (every distance) goes through the wave's scratch,
  // which is its eighth of the ring: no tile is requested before every wave is through.
  // fp8 content term (FP8): q' = (q+u)*scale/sq and k' = k/sk are rounded to e4m3 with the
  // per-head amax scales sq, sk chosen by the caller; the MFMA accumulates in units of 1/(sq*sk),
  // the channel-bias tile is pre-divided accordingly for the window steps and the product sq*sk
  // returns inside the exp2 fma.  K arrives rounded (a.k_fp8).
  f32x16 Bc[NCT];
  bf16x8 Qu[KS];
  long Qu8[KS];
  float fp8_d = 1.f;
  if (FP8) {
    const float sq = a.fp8_q_scale[h], sk = a.fp8_k_scale[g];
    fp8_d = sq * sk;
    // product s = 2p + j contracts, in lane half hh, the head dimensions [(2p + hh) * 16 + 8j, +8)
#pragma unroll
    for (int s8 = 0; s8 < KS; ++s8) {
      const int d0 = ((s8 >> 1) * 2 + hh) * 16 + (s8 & 1) * 8;
      const u32x4 raw = *(const u32x4*)(qbase + (qoff - hh * 16) + d0 * 2);
      Qu8[s8] = make_qfrag_fp8(raw, bu + d0, sc2 / sq);
    }
  }
  {
    f32x16 sct[NCT];
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) sct[t][i] = 0.f;
#pragma unroll
    for (int kh = 0; kh < KS; kh += 4) {
      u32x4 raw[4];
#pragma unroll
      for (int k4 = 0; k4 < 4; ++k4) raw[k4] = q_chunk(kh + k4);
#pragma unroll
      for (int k4 = 0; k4 < 4; ++k4) {
        const int ks = kh + k4;
        const int d0 = ks * 16 + hh * 8;
        if (!FP8) Qu[ks] = make_qfrag(raw[k4], bu + d0, sc2);
        const bf16x8 qz = make_qfrag(raw[k4], bz + d0, sc2);
#pragma unroll
        for (int t = 0; t < NCT; ++t) {
          const int j = min(t * 32 + ln, C_ - 1);
          const u32x4 er = *(const u32x4*)(kchan + (int64_t)j * DH + d0);
          sct[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(er), qz, sct[t], 0, 0, 0);
        }
      }
    }
    float* scr = (float*)(smem_raw + wave * G::SCRATCH_WAVE);
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int j = t * 32 + (i >> 2) * 8 + hh * 4 + (i & 3);
        scr[j * 32 + ln] = has_chan ? sct[t][i] : 0.f;
      }
    // key-channel mask: bit ck set = channel exists and is present; a lane keeps the bits of its
    // own keys shifted down by 4hh, so that the bit of element i sits at 8(i/4) + i%4
    uint32_t kbits[NCT];
#pragma unroll
    for (int t2 = 0; t2 < NCT; t2 += 2) {
      const int ck = t2 * 32 + lane;
      bool ok = ck < C_;
      if (valid) ok = ok && valid[min(ck, C_ - 1)] != 0;
      const uint64_t kmask = __ballot(ok);
      kbits[t2] = (uint32_t)(kmask >> (4 * hh));
      if (t2 + 1 < NCT) kbits[t2 + 1] = (uint32_t)(kmask >> (32 + 4 * hh));
    }
    wave_lds_sync();
    const int cq = cb + ln;
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
        Bc[t][i] = kv ? (FP8 ? val * (1.f / fp8_d) : val) : -INFINITY;
      }
  }
  lds_barrier();               // the scratch is ring memory from here on
  issue_avail();

  // ---- time-bias slab: St[j][q] for key steps [tk, tk+32) -> the wave's slab memory.  The
  // operands come in two trips of four k-steps (registers).  In the far phase (for_far) the
  // soft-max rescale that covers every far step of the slab is done here, once.
  float mc = 0.f;              // max of the channel bias over the keys (set when the window is done)
  auto time_slab = [&](int tk, bool for_far) {
    const int j0 = time_row(tq, tk, T_);
    const int j = min(max(j0 + ln, 0), T_ - 1);       // rows outside the table belong to tk > tq
    f32x16 stc;
#pragma unroll
    for (int i = 0; i < 16; ++i) stc[i] = 0.f;
    if (has_time) {
#pragma unroll
      for (int kh = 0; kh < KS; kh += 4) {
        u32x4 rr[4], br[4], qr[4];
#pragma unroll
        for (int k4 = 0; k4 < 4; ++k4) {
          const int ks = kh + k4;
          rr[k4] = *(const u32x4*)((const unsigned char*)ktime + ((uint32_t)j * (DH * 2) + hh * 16) + ks * 32);
          br[k4] = *(const u32x4*)((const unsigned char*)bv + (uint32_t)(hh * 16) + ks * 32);
          qr[k4] = q_chunk(ks);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k4 = 0; k4 < 4; ++k4) {
          bf16x8 qv;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t w = qr[k4][i], bw = br[k4][i];
            qv[2 * i] = (__bf16)((__uint_as_float(w << 16) + __uint_as_float(bw << 16)) * sc2);
            qv[2 * i + 1] = (__bf16)((__uint_as_float(w & 0xffff0000u) + __uint_as_float(bw & 0xffff0000u)) * sc2);
          }
          stc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(rr[k4]), qv, stc, 0, 0, 0);
        }
      }
    }
    float cm = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int jj = (i >> 2) * 8 + hh * 4 + (i & 3);
      stb_wave[jj * 32 + ln] = stc[i];
      cm = fmaxf(cm, tk + jj <= far_max ? stc[i] : -INFINITY);
    }
    cm = xhalf_max(cm);
    if (for_far) {                                 // (the slab holds at least one far step)
      const float m_new = fmaxf(m_run, cm + mc);
      const float alpha = fast_exp2(m_run - m_new);
      m_run = m_new;
      l_run *= alpha;
      rescale_acc(alpha);
    }
    wave_lds_sync();
  };

  // ---- window step: per key tile S^T = K Q^T + Bc, online soft-max, acc += V^T P^T (this wave's
  // output columns).  Lazy running max: the reference point only moves when some row max outgrew
  // it by 2^8.
  auto near_step = [&](const KAddr& ka_, const VAddr& va_, int tk) {
    const float st = stb_wave[(tk & 31) * 32 + ln];
    float ls = 0.f;
#pragma unroll
    for (int t = 0; t < NCT; ++t) {
      f32x16 S = Bc[t];
      if (FP8) {
        u32x4 kr[KS / 2];
#pragma unroll
        for (int p2 = 0; p2 < KS / 2; ++p2) kr[p2] = *(LDS_PTR(const u32x4))(uintptr_t)(ka_.k[p2] + t * 32 * DH);
#pragma unroll
        for (int p2 = 0; p2 < KS / 2; ++p2) {
          const long lo = (long)(((unsigned long)kr[p2][1] << 32) | kr[p2][0]);
          const long hi = (long)(((unsigned long)kr[p2][3] << 32) | kr[p2][2]);
          S = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(lo, Qu8[2 * p2], S, 0, 0, 0);
          S = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(hi, Qu8[2 * p2 + 1], S, 0, 0, 0);
        }
      } else {
        bf16x8 ka[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) ka[ks] = k_frag(ka_, t, ks);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[ks], Qu[ks], S, 0, 0, 0);
      }
      bf16x8 vf[2][MT];
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int m = 0; m < MT; ++m) vf[s][m] = v_frag(va_, t, s, m);
      float rmax = -INFINITY;
#pragma unroll
      for (int i = 0; i < 16; ++i) rmax = fmaxf(rmax, S[i]);
      rmax = xhalf_max(rmax);
      if (FP8) rmax *= fp8_d;
      const float cand = rmax + st;
      if (__ballot(cand > m_run + 8.f) != 0ull) {
        const float m_new = fmaxf(m_run, cand);
        const float alpha = fast_exp2(m_run - m_new);
        m_run = m_new;
        l_run *= alpha;
        ls *= alpha;
        rescale_acc(alpha);
      }
      const float off = st - m_run;
#pragma unroll
      for (int i = 0; i < 16; ++i) S[i] = FP8 ? fast_exp2(__builtin_fmaf(S[i], fp8_d, off)) : fast_exp2(S[i] + off);
      bf16x8 P[2];
      P[0] = pack8(S, 0);
      P[1] = pack8(S, 8);
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        union { bf16x8 v; bf16x2 q[4]; } u;
        u.v = P[s];
#pragma unroll
        for (int j = 0; j < 4; ++j) ls = __builtin_amdgcn_fdot2_f32_bf16(u.q[j], kOnes2, ls, false);
      }
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int m = 0; m < MT; ++m)
          acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[s][m], P[s], acc[m], 0, 0, 0);
    }
    l_run += ls;
  };

  // =========================== window steps ===========================
  int need = 0;                  // requests (units of LPW loads) up to and including the current tile
  int cur_slot = 0, prev_slots = 0;
  for (int p = 0; p < n_near; ++p) {
    const int tk = NLO + p;
    need += 2;
    if (FP8) wait_units<LPW + LPW8>((issued - need) / 2);     // (a window tile is LPW8 + LPW loads)
    else wait_units<LPW>(issued - need);
    lds_barrier();
    used -= prev_slots;          // the previous tile is consumed by every wave
    prev_slots = 2;
    // (a slab waits for its own operands from global memory and the load counter is in order: the
    // next tiles are requested after it, not before, or the slab would wait for them too)
    if (live && (p == 0 || (tk & 31) == 0)) time_slab(tk & ~31, false);
    issue_avail();
    if (live && tk > far_max && tk <= tq) near_step(k_addr(cur_slot), v_addr(cur_slot + 1), tk);
    cur_slot = (cur_slot + 2) & (SLOTS - 1);
  }

  // ---- Bc -> mc, Ec, sumEc: the far steps' side of the channel bias
  bf16x8 Ec[NCT][2];
  float sumEc = 0.f;
  {
    if (FP8) {                                 // back to the units of the scores
#pragma unroll
      for (int k = 0; k < NCT; ++k)
#pragma unroll
        for (int i = 0; i < 16; ++i) Bc[k][i] *= fp8_d;
    }
    float mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < NCT; ++k)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, Bc[k][i]);
    mc = xhalf_max(mx);
    if (mc == -INFINITY) mc = 0.f;            // no valid key at all: Ec = 0
#pragma unroll
    for (int k = 0; k < NCT; ++k) {
      f32x16 e;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        e[i] = fast_exp2(Bc[k][i] - mc);
        sumEc += e[i];
      }
      Ec[k][0] = pack8(e, 0);
      Ec[k][1] = pack8(e, 8);
    }
  }

  // =========================== far phase ===========================
  // acc += et * (V^T Ec^T).  Far tile f lives in slot f mod 4.  Everything in a step is laid out
  // so that a wave leaves the barrier with matrix work in hand and nothing but straight-line code
  // up to the next barrier:
  //  - the barrier of step f publishes tile f+1 (tile f was published by the one before), and the
  //    fragments of output tile 0 are read a step ahead;
  //  - the accumulate of a step's product runs in the next step;
  //  - one tile is requested per step, without a branch: past the end it is the last tile once
  //    more, into a slot nobody reads any longer, so that the count of loads in flight is fixed.
  // The phase goes slab by slab (32 key steps).
  if (n_far > 0) {
    wait_vmcnt_imm<0>();
    lds_barrier();                       // every wave is through with the window tiles
    const bf16_t* fv = vbase;
    int f_iss = 0;
    uint32_t iss_lds = ring_lds, cur_lds = ring_lds;
    auto issue_far = [&]() {
#pragma unroll
      for (int i = 0; i < LPW; ++i) load_to_lds_16(fv, v_off[i], iss_lds + (wave + NW * i) * 1024);
      ++f_iss;
      fv = f_iss < n_far ? fv + vstep : fv;
      iss_lds = iss_lds + TILE_BYTES == ring_lds + RING_BYTES ? ring_lds : iss_lds + TILE_BYTES;
    };
    auto v_addr_at = [&](uint32_t base) {
      VAddr sa;
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        sa.v[m] = base + v_lane[m];
        asm volatile("" : "+v"(sa.v[m]));
      }
      return sa;
    };
    issue_far();
    issue_far();
    issue_far();
    wait_vmcnt_imm<2 * LPW>();
    lds_barrier();
    bf16x8 vf0[NCT * 2];
    {
      const VAddr va_ = v_addr_at(cur_lds);
#pragma unroll
      for (int t = 0; t < NCT; ++t)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) vf0[t * 2 + s2] = v_frag(va_, t, s2, 0);
    }
    for (int tk0 = 0; tk0 < n_far; tk0 += 32) {
      if (live && tk0 <= far_max) time_slab(tk0, true);
      f32x16 ptmp[MT];
      float pet1 = 0.f;                  // weight of the product waiting in ptmp[1]
#pragma unroll
      for (int i = 0; i < 16; ++i) ptmp[1][i] = 0.f;
      const int tk1 = min(tk0 + 32, n_far);
      for (int tk = tk0; tk < tk1; ++tk) {
        wait_vmcnt_imm<LPW>();
        bare_barrier();                  // (the fragments read ahead stay in flight across it)
        const uint32_t now_lds = cur_lds;
        cur_lds = cur_lds + TILE_BYTES == ring_lds + RING_BYTES ? ring_lds : cur_lds + TILE_BYTES;
        if (live && tk <= far_max) {
          const VAddr va_ = v_addr_at(now_lds), vn_ = v_addr_at(cur_lds);
          // Order of a step, fenced for the scheduler product by product.  First the products of
          // output tile 0 (fragments in registers since the last step); with each of them a
          // fragment of tile 1 is read and a share of the accumulate of the PREVIOUS step's
          // product for tile 1 runs; the next tile is requested after the first.  Then the
          // products of tile 1; with each of them one of the next step's fragments of tile 0 is
          // read and a share of the accumulate for tile 0 runs.
          float st;
          bf16x8 vf1[NCT * 2];
          constexpr int NC = NCT * 2;
#pragma unroll
          for (int c = 0; c < NC; ++c) {
            if (c == 0) {
#pragma unroll
              for (int i = 0; i < 16; ++i) ptmp[0][i] = 0.f;
            }
            ptmp[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf0[c], Ec[c >> 1][c & 1], ptmp[0], 0, 0, 0);
            if (c == 0) {
              __builtin_amdgcn_sched_barrier(0);
              issue_far();
            }
            if (c == 1) st = stb_wave[(tk & 31) * 32 + ln];
            vf1[c] = v_frag(va_, c >> 1, c & 1, 1);
#pragma unroll
            for (int i = (16 * c) / NC; i < (16 * (c + 1)) / NC; ++i) acc[1][i] += pet1 * ptmp[1][i];
            __builtin_amdgcn_sched_barrier(0);
          }
          const float pet = fast_exp2(st + mc - m_run);
          l_run += pet * sumEc;
#pragma unroll
          for (int c = 0; c < NC; ++c) {
            if (c == 0) {
#pragma unroll
              for (int i = 0; i < 16; ++i) ptmp[1][i] = 0.f;
            }
            ptmp[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf1[c], Ec[c >> 1][c & 1], ptmp[1], 0, 0, 0);
            vf0[c] = v_frag(vn_, c >> 1, c & 1, 0);
            // (the accumulate starts two products late: the last product of tile 0 has to land)
            if (c >= 2) {
#pragma unroll
              for (int i = (16 * (c - 2)) / (NC - 2); i < (16 * (c - 1)) / (NC - 2); ++i) acc[0][i] += pet * ptmp[0][i];
            }
            __builtin_amdgcn_sched_barrier(0);
          }
          pet1 = pet;
        } else {
          issue_far();
        }
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[1][i] += pet1 * ptmp[1][i];
    }
    wait_vmcnt_imm<0>();                 // (the requests past the end)
  }

  // =========================== epilogue ===========================
  const int cq = cb + ln;
  const float ltot = l_run + __shfl_xor(l_run, 32);
  if (live && cq < C_) {
    const float inv = 1.f / ltot;
    const int64_t n = (int64_t)tq * C_ + cq;
    bf16_t* orow = (bf16_t*)a.o + b * a.o_stride_b + h * a.o_stride_h + n * a.o_stride_n;
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4) {
        const int d0 = ((HALVES == 2 ? 2 * half : 0) + m) * 32 + a4 * 8 + hh * 4;
        bf16x4 w;
#pragma unroll
        for (int r = 0; r < 4; ++r) w[r] = (__bf16)(acc[m][a4 * 4 + r] * inv);
        *(bf16x4*)(orow + d0) = w;
      }
    if (a.lse && hh == 0 && half == 0) a.lse[((int64_t)b * a.H + h) * ((int64_t)T_ * C_) + n] = m_run + log2f(ltot);
  }
}

}  // namespace d128
}  // namespace mvpa

// Shapes this build serves: bf16, 33..128 channels at head size 128 (output columns split over two
// waves) or 64 (a wave owns every column; the keys are padded to 64 or 128 there), a plain
// forward (no decoding step), bf16 or fp8 content term; everything else about the arguments is as
// for the general kernel (mvpa_mfma_supported).
int mvpa_mfma128_supported(const mvpa_fwd_args* a) {
  if (a->dtype != MVPA_BF16 || (a->Dh != 128 && a->Dh != 64) || a->C <= 32 || a->C > 128) return 0;
  if (a->flags & (MVPA_FLAG_LAST_STEP | MVPA_FLAG_RING)) return 0;
  // the fp8 content term streams the keys' e4m3 copy (the general kernel rounds bf16 keys itself)
  if ((a->flags & MVPA_FLAG_FP8_QK) && (!a->k_fp8 || ((uintptr_t)a->k_fp8 & 15))) return 0;
  return 1;
}

template <int DH, int NCT, bool FP8>
static int launch128(const mvpa_fwd_args* a, hipStream_t stream) {
  using namespace mvpa::d128;
  using G = Geo<DH, NCT>;
  auto kern = mvpa_mfma128_kernel<DH, NCT, FP8>;
  mvpa::want_dynamic_lds((const void*)kern, (int)G::LDS_BYTES);
  const int nt = (a->T + G::TQW - 1) / G::TQW;
  MVPA_LAUNCH(kern, dim3((unsigned)(nt * a->B * a->H)), dim3(NW * 64), G::LDS_BYTES, stream, *a);
  return mvpa::take_launch_status();
}

int mvpa_launch_mfma128(const mvpa_fwd_args* a, hipStream_t stream) {
  const bool fp8 = a->flags & MVPA_FLAG_FP8_QK;
  if (a->C <= 64) {
    if (a->Dh == 64) return fp8 ? launch128<64, 2, true>(a, stream) : launch128<64, 2, false>(a, stream);
    return fp8 ? launch128<128, 2, true>(a, stream) : launch128<128, 2, false>(a, stream);
  }
  if (a->Dh == 64) return fp8 ? launch128<64, 4, true>(a, stream) : launch128<64, 4, false>(a, stream);
  if (fp8) return a->C <= 96 ? launch128<128, 3, true>(a, stream) : launch128<128, 4, true>(a, stream);
  return a->C <= 96 ? launch128<128, 3, false>(a, stream) : launch128<128, 4, false>(a, stream);
}
