// bf16 MFMA forward for head size 64 and 33..64 channels (gfx950, wave64): a wave owns a WHOLE
// time step, i.e. two tiles of 32 queries.
//
// The general tiled kernel (mvpa_mfma.hip) gives a wave one tile of 32 queries.  In its far steps
// (content term zeroed, p = et[q,tk] * Ec[q,ck], layers/mvpa.py:231-245) every V^T fragment that a
// wave reads from LDS feeds exactly one matrix instruction, and the costs that come per key step
// and per workgroup - fragment reads, the tile ring, the barrier, the set-up, the time-bias slabs,
// the dispatch of a workgroup - are paid per 8 matrix instructions.  Here a fragment feeds two
// instructions (one per query tile of the wave) and all of those costs are paid per 16.
//
// Two query tiles do not fit the registers next to the operands of the window steps (the channel
// bias tile Bc and the (q+u) fragments, 48 registers per tile), so the key steps are taken in an
// order that never needs both at once - the online soft-max does not care about the order:
//   pass A   window steps of query tile 0   (needs Bc, (q+u) of tile 0; 32 queries per wave)
//   pass B   window steps of query tile 1   (the same key tiles once more)
//   far      every far step, both tiles     (needs only Ec of both tiles; 64 queries per wave)
// Bc of a tile is turned into Ec = exp2(Bc - mc) when its pass ends.  A workgroup is 4 waves =
// 4 consecutive time steps on one K/V ring; two workgroups share a CU.
#include "mvpa_mfma_tools.h"

namespace mvpa {
namespace q64 {

constexpr int DH = 64, KS = 4, MT = 2, NCT = 2, CP = 64, NW = 4, TQW = 4, STAGES = 3;
constexpr int ROWB = DH * 2, CHUNKS = DH / 8;
constexpr int TILE_BYTES = CP * ROWB;                  // one K or V tile: 8 KiB
constexpr int STAGE_BYTES = 2 * TILE_BYTES;            // K tile then V tile
constexpr int RING_BYTES = STAGES * STAGE_BYTES;
constexpr int LPW = TILE_BYTES / 1024 / NW;            // 64-lane x 16-byte loads per tile and wave
constexpr int STB_TILE = 32 * 32 * 4;                  // time-bias slab of one query tile
constexpr int STB_WAVE = 2 * STB_TILE;                 // also the set-up scratch [CP][32] of a wave
constexpr int LDS_BYTES = RING_BYTES + NW * STB_WAVE;  // 80 KiB
static_assert(STB_WAVE == CP * 32 * 4, "the set-up scratch of a wave is its two slabs");

// running soft-max state of one tile of 32 queries (a lane owns one query of each tile)
struct Tile {
  f32x16 acc[MT];
  float m, l;              // reference point and (per half-wave partial) sum
  float mc, sumEc;         // max of the channel bias over the keys; sum of Ec (per half-wave)
  bf16x8 Ec[NCT][2];       // exp2(Bc - mc) as B operands of the far products
};

__global__ __launch_bounds__(NW * 64, 2) void mvpa_mfma64_kernel(mvpa_fwd_args a) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, hh = lane >> 5;
  const int C_ = a.C, W = a.window, T_ = a.T;
  const bool has_content = a.flags & MVPA_FLAG_CONTENT;
  const bool has_time = a.flags & MVPA_FLAG_TIME_BIAS;
  const bool has_chan = a.flags & MVPA_FLAG_CHAN_BIAS;

  // ---- block -> (b*H + h, time tile): ids that are equal mod 8 run on one XCD and get the same
  // (b, h), so that its K/V stay in that XCD's L2.  The last time tile of every (b, h) goes out
  // first (its last row keeps the content term for every key step and takes longest), then one
  // (b, h) after the other, late (= long) tiles first; the last two (b, h) of an XCD are
  // interleaved tile by tile so that the grid does not end on the long tiles of a single (b, h).
  // With the content term on, the queries of the LAST time step keep it for every key step
  // (layers/mvpa.py:244): no far steps at all, T window steps.  That step gets a workgroup of its
  // own ("last-step workgroup"): wave w takes query tile w & 1 and the key steps of parity w >> 1,
  // and the two partial soft-max states of a tile are merged through LDS at the end.  The other
  // T-1 time steps are tiled four to a workgroup.
  const bool own_last = has_content && T_ > 1;
  const int t_main = own_last ? T_ - 1 : T_;
  const int nt = (t_main + TQW - 1) / TQW + (own_last ? 1 : 0);
  const int nbh = a.B * a.H;
  int bh, tile;
  map_block(blockIdx.x, nbh, nt, a.H / a.Hkv, bh, tile);
  const int b = bh / a.H, h = bh % a.H;
  const int g = h / (a.H / a.Hkv);
  const bool last_wg = own_last && tile == nt - 1;
  const int par = wave >> 1;                       // last-step workgroup: parity of this wave's key steps
  const int tq0 = last_wg ? T_ - 1 : tile * TQW, tq_hi = last_wg ? T_ - 1 : min(t_main - 1, tq0 + TQW - 1);
  const int tq = last_wg ? T_ - 1 : tq0 + wave;
  const bool active = tq <= tq_hi;
  // channel base of the wave's two query-tile slots (the last-step workgroup uses slot 0 only)
  const int cb0 = last_wg ? 32 * (wave & 1) : 0, cb1 = 32;

  // ---- which key steps are what.  For this wave's queries steps 0 .. far_max are far (content
  // term absent or zeroed), far_max+1 .. tq are window steps.  For the workgroup: the passes walk
  // key steps NLO .. tq_hi (a wave skips what lies outside its own window), the far phase walks
  // 0 .. FM (a wave stops at its own far_max).
  const int far_max = !active ? -1 : !has_content ? tq : (W > 0 && tq != T_ - 1) ? tq - W - 1 : -1;
  int FM = -1;
  if (!has_content) {
    FM = tq_hi;
  } else if (W > 0) {
    const int tql = tq_hi == T_ - 1 ? tq_hi - 1 : tq_hi;       // the last step has no far steps
    if (tql >= tq0) FM = max(-1, tql - W - 1);
  }
  const int NLO = (W <= 0 || tq_hi == T_ - 1) ? 0 : max(0, tq0 - W);
  const int n_pass = has_content ? tq_hi - NLO + 1 : 0;        // key steps of a pass
  const int n_near = last_wg ? n_pass : 2 * n_pass;             // ... of all passes: the tiles with K
  const int n_far = FM + 1;
  const int n_total = n_near + n_far;

  // Loads below are unconditional: rows that do not exist (padded channels, time steps past the
  // end) are redirected to an existing row and their results are never used.
  // (a q row is addressed as a wave-uniform base plus a 32-bit byte offset per lane: one register
  // per tile instead of a 64-bit pointer)
  const unsigned char* qbase = (const unsigned char*)((const bf16_t*)a.q + b * a.q_stride_b + h * a.q_stride_h);
  uint32_t qoff[2];
#pragma unroll
  for (int x = 0; x < 2; ++x)
    qoff[x] = (uint32_t)((active ? tq * C_ + min((x == 0 ? cb0 : cb1) + ln, C_ - 1) : 0) * a.q_stride_n) * 2u + hh * 16;
  auto q_chunk = [&](int x, int ks) -> u32x4 { return *(const u32x4*)(qbase + qoff[x] + ks * 32); };
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
  // as in the general kernel: rows in natural [key][dh] order, 16-byte chunks XOR-swizzled on the
  // global side; rows of padded channels fetch the last real channel and are neutralised by
  // Ec = 0 / Bc = -inf
  uint32_t k_off[LPW], v_off[LPW];         // byte offsets of this lane's chunks within a tile
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int pc = (wave + NW * i) * 64 + lane;
    const int row = pc / CHUNKS, phys = pc % CHUNKS;
    const int rowc = min(row, C_ - 1);
    k_off[i] = (uint32_t)(rowc * a.k_stride_n) * 2u + ((phys ^ swz_k<DH>(row)) << 4);
    v_off[i] = (uint32_t)(rowc * a.v_stride_n) * 2u + ((phys ^ swz_v<DH>(row)) << 4);
  }
  const uint32_t ring_lds = (uint32_t)(uintptr_t)(LDS_PTR(unsigned char))smem_raw;
  // The window tiles are requested in stream order - pass A (key steps NLO .. tq_hi, K and V),
  // pass B (the same again) - by a little scalar state machine
  // that moves two pointers along, so that a request costs a handful of scalar instructions.
  const int64_t kstep = (int64_t)C_ * a.k_stride_n, vstep = (int64_t)C_ * a.v_stride_n;
  int iss_pos = 0, iss_stage = 0;
  const bf16_t* iss_k = kbase + (n_pass > 0 ? NLO : 0) * kstep;
  const bf16_t* iss_v = vbase + (n_pass > 0 ? NLO : 0) * vstep;
  auto issue_next = [&]() {
    if (iss_pos >= n_near) return;
    const uint32_t stage = ring_lds + iss_stage * STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < LPW; ++i) load_to_lds_16(iss_v, v_off[i], stage + TILE_BYTES + (wave + NW * i) * 1024);
#pragma unroll
    for (int i = 0; i < LPW; ++i) load_to_lds_16(iss_k, k_off[i], stage + (wave + NW * i) * 1024);
    ++iss_pos;
    iss_stage = iss_stage + 1 == STAGES ? 0 : iss_stage + 1;
    if (iss_pos == n_pass) {                 // pass B walks the window once more
      iss_k = kbase + NLO * kstep;
      iss_v = vbase + NLO * vstep;
    } else {
      iss_k += kstep;
      iss_v += vstep;
    }
  };
  // the set-up scratch is the wave's own slab memory, not the ring: the first tiles go out now
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s) issue_next();

  float* stb_wave = (float*)(smem_raw + RING_BYTES + wave * STB_WAVE);

  // ---- per-lane pieces of the LDS fragment addresses (see the general kernel)
  int v_lane[MT], k_lane[KS];
  {
    const int e = (ln & 15) >> 2, aa = ln & 3, grp = ln >> 4;
    const int row0 = 4 * hh + e;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      v_lane[mt] = TILE_BYTES + row0 * ROWB + (((4 * mt + 2 * grp + (aa >> 1)) ^ swz_v<DH>(row0)) << 4) + ((aa & 1) << 3);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_lane[ks] = ln * ROWB + (((2 * ks + hh) ^ swz_k<DH>(ln)) << 4);
  }
  // Fragment addresses of a step: one register per output tile (V^T) / k-step (K) = lane part +
  // stage, formed once per step and made opaque to the compiler, so that everything else of an
  // address stays an immediate offset of the LDS instruction instead of being hoisted into
  // registers of its own and added up again at every read.
  struct StageAddr { uint32_t v[MT], k[KS]; };
  auto stage_addr = [&](int stage_idx) {
    StageAddr sa;
    const uint32_t base = ring_lds + stage_idx * STAGE_BYTES;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      sa.v[mt] = base + v_lane[mt];
      asm volatile("" : "+v"(sa.v[mt]));
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      sa.k[ks] = base + k_lane[ks];
      asm volatile("" : "+v"(sa.k[ks]));
    }
    return sa;
  };
  auto v_frag = [&](const StageAddr& sa, int t, int s, int mt) -> bf16x8 {
    const uint32_t p = sa.v[mt] + (32 * t + 16 * s) * ROWB;
    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((LDS_PTR(bf16x4))(uintptr_t)p);
    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((LDS_PTR(bf16x4))(uintptr_t)(p + 8 * ROWB));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  auto k_frag = [&](const StageAddr& sa, int t, int ks) -> bf16x8 {
    return *(LDS_PTR(const bf16x8))(uintptr_t)(sa.k[ks] + t * 32 * ROWB);
  };

  Tile qt[2];
#pragma unroll
  for (int x = 0; x < 2; ++x) {
    qt[x].m = kMFloor;
    qt[x].l = 0.f;
    qt[x].mc = 0.f;
    qt[x].sumEc = 0.f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) qt[x].acc[mt][i] = 0.f;
  }

  // =========================== set-up of one query tile ===========================
  // Bc[ck][q] = (q+z).e[C-1-|cq-ck|] * scale in accumulator layout (-inf = masked key) and the
  // (q+u) fragments.  The whole channel table (every distance) goes through the wave's scratch.
  auto setup_tile = [&](int x, f32x16 (&Bc)[NCT], bf16x8 (&Qu)[KS]) {
    u32x4 raw[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) raw[ks] = q_chunk(x, ks);
    f32x16 sct[NCT];
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) sct[t][i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 16 + hh * 8;
      Qu[ks] = make_qfrag(raw[ks], bu + d0, sc2);
      const bf16x8 qz = make_qfrag(raw[ks], bz + d0, sc2);
#pragma unroll
      for (int t = 0; t < NCT; ++t) {
        const int j = min(t * 32 + ln, C_ - 1);
        const u32x4 er = *(const u32x4*)(kchan + (int64_t)j * DH + d0);
        sct[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(er), qz, sct[t], 0, 0, 0);
      }
    }
    float* scr = stb_wave;
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
    {
      bool ok = lane < C_;
      if (valid) ok = ok && valid[min(lane, C_ - 1)] != 0;
      const uint64_t kmask = __ballot(ok);
#pragma unroll
      for (int t = 0; t < NCT; ++t) kbits[t] = (uint32_t)(kmask >> (t * 32 + 4 * hh));
    }
    wave_lds_sync();
    const int cq = (x == 0 ? cb0 : cb1) + ln;
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
    wave_lds_sync();          // the scratch is slab memory again from here on
  };

  // Bc -> mc, Ec, sumEc of the tile (the far steps' side of the channel bias)
  auto finish_tile = [&](Tile& t, const f32x16 (&Bc)[NCT]) {
    float mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < NCT; ++k)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, Bc[k][i]);
    float mc = xhalf_max(mx);
    if (mc == -INFINITY) mc = 0.f;            // no valid key at all: Ec = 0
    float se = 0.f;
#pragma unroll
    for (int k = 0; k < NCT; ++k) {
      f32x16 e;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        e[i] = fast_exp2(Bc[k][i] - mc);
        se += e[i];
      }
      t.Ec[k][0] = pack8(e, 0);
      t.Ec[k][1] = pack8(e, 8);
    }
    t.mc = mc;
    t.sumEc = se;
  };

  // in-place rescale of a tile's accumulators (inline assembly: see the general kernel)
  auto rescale_acc = [&](Tile& t, float alpha) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      f32x16 x = t.acc[mt];
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
      t.acc[mt] = x;
    }
  };

  // ---- time-bias slabs: St[j][q] for key steps [tk, tk+32) -> LDS, for the query tiles x0 .. x1.
  // Every operand (the 32 table rows, the time bias vector, the q rows) is requested from global
  // memory before the first one is used.
  // In the far phase (for_far) the soft-max rescale that covers every far step of the slab is
  // done here, once.
  auto time_slab = [&](int x0, int x1, int tk, bool for_far) {
    const int j0 = time_row(tq, tk, T_);
    const int j = min(max(j0 + ln, 0), T_ - 1);       // rows outside the table belong to tk > tq
    u32x4 rr[KS], br[KS], qr[2][KS];
    if (has_time) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        rr[ks] = *(const u32x4*)((const unsigned char*)ktime + ((uint32_t)j * (DH * 2) + hh * 16) + ks * 32);
        br[ks] = *(const u32x4*)((const unsigned char*)bv + (uint32_t)(hh * 16) + ks * 32);
        qr[0][ks] = q_chunk(x0, ks);
      }
      if (x1 > x0) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qr[1][ks] = q_chunk(x1, ks);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      if (x < x0 || x > x1) continue;
      Tile& t = qt[x];
      float* Stb = stb_wave + x * (32 * 32);
      f32x16 stc;
#pragma unroll
      for (int i = 0; i < 16; ++i) stc[i] = 0.f;
      if (has_time) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          bf16x8 qv;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t w = qr[x > x0 ? 1 : 0][ks][i], bw = br[ks][i];
            qv[2 * i] = (__bf16)((__uint_as_float(w << 16) + __uint_as_float(bw << 16)) * sc2);
            qv[2 * i + 1] = (__bf16)((__uint_as_float(w & 0xffff0000u) + __uint_as_float(bw & 0xffff0000u)) * sc2);
          }
          stc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(rr[ks]), qv, stc, 0, 0, 0);
        }
      }
      float cm = -INFINITY;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int jj = (i >> 2) * 8 + hh * 4 + (i & 3);
        Stb[jj * 32 + ln] = stc[i];
        cm = fmaxf(cm, tk + jj <= far_max ? stc[i] : -INFINITY);
      }
      cm = xhalf_max(cm);
      if (for_far && tk <= far_max && __ballot(cm + t.mc > t.m) != 0ull) {   // a far step of the slab outgrows the reference
        const float m_new = fmaxf(t.m, cm + t.mc);
        const float alpha = fast_exp2(t.m - m_new);
        t.m = m_new;
        t.l *= alpha;
        rescale_acc(t, alpha);
      }
    }
    wave_lds_sync();
  };

  // ---- window step of one query tile: S^T = K Q^T + Bc, online soft-max, acc += V^T P^T.
  // One row maximum and at most one rescale per step (over both key tiles), so that everything
  // after it - exponentials, packing, row sums, PV products of the two key tiles - is one
  // straight-line block in which the matrix products of one tile run beside the vector work of
  // the other.  V^T fragments are requested ahead of their use.
  auto near_step = [&](Tile& tl, const f32x16 (&Bc)[NCT], const bf16x8 (&Qu)[KS], const float* st_at,
                       const StageAddr& stage) {
    const float st = *st_at;
    f32x16 S[NCT];
#pragma unroll
    for (int t = 0; t < NCT; ++t) {
      bf16x8 ka[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ka[ks] = k_frag(stage, t, ks);
      S[t] = Bc[t];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        S[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[ks], Qu[ks], S[t], 0, 0, 0);
    }
    bf16x8 vf[2][MT];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) vf[s][mt] = v_frag(stage, 0, s, mt);
    __builtin_amdgcn_sched_barrier(0);
    float rmax = -INFINITY;
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) rmax = fmaxf(rmax, S[t][i]);
    rmax = xhalf_max(rmax);
    // lazy running max: the reference point only moves when some row max outgrew it by 2^8
    const float cand = rmax + st;
    if (__ballot(cand > tl.m + 8.f) != 0ull) {
      const float m_new = fmaxf(tl.m, cand);
      const float alpha = fast_exp2(tl.m - m_new);
      tl.m = m_new;
      tl.l *= alpha;
      rescale_acc(tl, alpha);
    }
    const float off = st - tl.m;
    float ls = 0.f;
#pragma unroll
    for (int t = 0; t < NCT; ++t) {
#pragma unroll
      for (int i = 0; i < 16; ++i) S[t][i] = fast_exp2(S[t][i] + off);
      bf16x8 P[2];
      P[0] = pack8(S[t], 0);
      P[1] = pack8(S[t], 8);
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
        for (int mt = 0; mt < MT; ++mt)
          tl.acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[s][mt], P[s], tl.acc[mt], 0, 0, 0);
      if (t + 1 < NCT) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) vf[s][mt] = v_frag(stage, t + 1, s, mt);
      }
    }
    tl.l += ls;
  };

  // wait until the window tile of stream position s has landed: at most the loads of the one
  // younger tile in flight (STAGES = 3) may still be outstanding
  auto wait_tile = [&](int s) {
    if (s + 1 < n_near) wait_vmcnt_imm<2 * LPW>();
    else wait_vmcnt_imm<0>();
  };

  // Tile requests of the far phase.  The ring is cut anew into slots of one V tile; far tile f
  // lives in slot (f0 + f) mod FSLOTS, and the barrier of step f publishes it.  One tile is
  // requested per step, without a branch: past the end it is the last tile once more, into a slot
  // nobody reads any longer, so that the count of loads in flight is fixed.
  constexpr int FSLOTS = RING_BYTES / TILE_BYTES;
  const bf16_t* fv = vbase;
  int f_iss = 0;
  uint32_t iss_lds = ring_lds, cur_lds = ring_lds;       // (f0 = 0 unless the passes say otherwise)
  auto issue_far = [&]() {
#pragma unroll
    for (int i = 0; i < LPW; ++i) load_to_lds_16(fv, v_off[i], iss_lds + (wave + NW * i) * 1024);
    ++f_iss;
    fv = f_iss < n_far ? fv + vstep : fv;
    iss_lds = iss_lds + TILE_BYTES == ring_lds + RING_BYTES ? ring_lds : iss_lds + TILE_BYTES;
  };
  auto v_addr_at = [&](uint32_t base) {
    StageAddr sa;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      sa.v[mt] = base + (v_lane[mt] - TILE_BYTES);
      asm volatile("" : "+v"(sa.v[mt]));
    }
    return sa;
  };

  // =========================== passes: window steps, one query tile each ===========================
  int s = 0, stg = 0;                                // stream position and its ring stage
#pragma unroll
  for (int x = 0; x < 2; ++x) {
    if (x == 1 && last_wg) break;                    // (uniform over the workgroup)
    f32x16 Bc[NCT];
    bf16x8 Qu[KS];
    setup_tile(x, Bc, Qu);
    const float* Stb = stb_wave + x * (32 * 32);
    const int nlo = far_max + 1;                     // this wave's first window step
    // the time-bias slab of the pass starts at the wave's own first window step: a window of up
    // to 32 steps never needs a second one
    int sb = max(nlo, NLO);
    if (n_pass > 0 && active) time_slab(x, x, sb, false);
    for (int p = 0; p < n_pass; ++p, ++s) {
      const int tk = NLO + p;
      wait_tile(s);
      lds_barrier();
      // (a slab waits for its own operands from global memory, and the load counter is in order:
      // the next tile is requested after it, not before, or the slab would wait for that tile too)
      if (active && tk == sb + 32 && tk <= tq) {
        sb += 32;
        time_slab(x, x, sb, false);
      }
      issue_next();
      if (s + 1 == n_near && n_far > 0) {
        // the last window tile: the other two stages are free, the first four far tiles go there
        iss_lds = cur_lds = ring_lds + (stg + 1 == STAGES ? 0 : stg + 1) * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < FSLOTS - 2; ++i) issue_far();
      }
      if (active && tk >= nlo && tk <= tq && (!last_wg || (tk & 1) == par))
        near_step(qt[x], Bc, Qu, Stb + (tk - sb) * 32 + ln, stage_addr(stg));
      stg = stg + 1 == STAGES ? 0 : stg + 1;
    }
    finish_tile(qt[x], Bc);
  }

  // last-step workgroup: the state of the odd key steps goes through LDS into that of the even ones
  if (last_wg) {
    lds_barrier();                                 // every wave is done with the ring
    float* mb = (float*)smem_raw + (wave & 1) * ((2 + MT * 16) * 64) + lane;
    Tile& t = qt[0];
    if (par == 1) {
      mb[0] = t.m;
      mb[64] = t.l;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mb[(2 + mt * 16 + i) * 64] = t.acc[mt][i];
    }
    lds_barrier();
    if (par == 1) return;
    const float m1 = mb[0], l1 = mb[64];
    const float m = fmaxf(t.m, m1);
    const float a0 = fast_exp2(t.m - m), a1 = fast_exp2(m1 - m);   // (an empty state holds the floor: weight 0)
    t.m = m;
    t.l = a0 * t.l + a1 * l1;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) t.acc[mt][i] = a0 * t.acc[mt][i] + a1 * mb[(2 + mt * 16 + i) * 64];
  }

  // =========================== far phase: both query tiles ===========================
  // acc += et * (V^T Ec^T) with one set of fragment reads for the two tiles.  The accumulate of a
  // step is deferred to the next one, where it fills the wait for that step's first fragments.
  // The phase goes slab by slab (32 key steps): the slabs of both tiles are computed between two
  // segments, where the products of the far steps are not live, so their registers are free for
  // the slab's operands.
  if (n_far > 0) {
    if (n_near > 0) {
      lds_barrier();                     // every wave is through with the last window tile
      issue_far();
    } else {
#pragma unroll
      for (int i = 0; i < FSLOTS - 1; ++i) issue_far();
    }
  }
  for (int tk0 = 0; tk0 < n_far; tk0 += 32) {
    if (tk0 <= far_max) time_slab(0, 1, tk0, true);   // (never for inactive waves)
    f32x16 ptmp[2][MT];
    float pet[2] = {0.f, 0.f};
#pragma unroll
    for (int x = 0; x < 2; ++x)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) ptmp[x][mt][i] = 0.f;
    const int tk1 = min(tk0 + 32, n_far);
    for (int tk = tk0; tk < tk1; ++tk) {
      wait_vmcnt_imm<(FSLOTS - 2) * LPW>();
      lds_barrier();
      issue_far();
      const uint32_t now_lds = cur_lds;
      cur_lds = cur_lds + TILE_BYTES == ring_lds + RING_BYTES ? ring_lds : cur_lds + TILE_BYTES;
      if (tk <= far_max) {
        const StageAddr stage = v_addr_at(now_lds);
        const float st0 = stb_wave[(tk & 31) * 32 + ln];
        const float st1 = stb_wave[32 * 32 + (tk & 31) * 32 + ln];
        // Order of a step, pinned for the scheduler: the fragments of output tile 0 are requested
        // first and arrive under the previous step's accumulate for that tile; the fragments of
        // output tile 1 are requested next and arrive under the products of tile 0, between which
        // the accumulate for tile 1 is spread; the products of tile 1 close the step.
        bf16x8 vf[MT][NCT * 2];
#pragma unroll
        for (int t = 0; t < NCT; ++t)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) vf[0][t * 2 + s2] = v_frag(stage, t, s2, 0);
#pragma unroll
        for (int x = 0; x < 2; ++x)
#pragma unroll
          for (int i = 0; i < 16; ++i) qt[x].acc[0][i] += pet[x] * ptmp[x][0][i];
#pragma unroll
        for (int t = 0; t < NCT; ++t)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) vf[1][t * 2 + s2] = v_frag(stage, t, s2, 1);
#pragma unroll
        for (int x = 0; x < 2; ++x)
#pragma unroll
          for (int i = 0; i < 16; ++i) ptmp[x][0][i] = 0.f;
#pragma unroll
        for (int t = 0; t < NCT; ++t)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
            for (int x = 0; x < 2; ++x)
              ptmp[x][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[0][t * 2 + s2], qt[x].Ec[t][s2], ptmp[x][0], 0, 0, 0);
#pragma unroll
        for (int x = 0; x < 2; ++x)
#pragma unroll
          for (int i = 0; i < 16; ++i) qt[x].acc[1][i] += pet[x] * ptmp[x][1][i];
#pragma unroll
        for (int x = 0; x < 2; ++x)
#pragma unroll
          for (int i = 0; i < 16; ++i) ptmp[x][1][i] = 0.f;
#pragma unroll
        for (int t = 0; t < NCT; ++t)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
            for (int x = 0; x < 2; ++x)
              ptmp[x][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[1][t * 2 + s2], qt[x].Ec[t][s2], ptmp[x][1], 0, 0, 0);
        // 8 LDS reads, 32 FMAs, 8 LDS reads, then 8 x (1 MFMA + 4 FMAs), then 8 MFMAs
        __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 32, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
        pet[0] = fast_exp2(st0 + qt[0].mc - qt[0].m);
        qt[0].l += pet[0] * qt[0].sumEc;
        pet[1] = fast_exp2(st1 + qt[1].mc - qt[1].m);
        qt[1].l += pet[1] * qt[1].sumEc;
      }
    }
#pragma unroll
    for (int x = 0; x < 2; ++x)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) qt[x].acc[mt][i] += pet[x] * ptmp[x][mt][i];
  }

  wait_vmcnt_imm<0>();                   // (the far requests past the end)

  // =========================== epilogue ===========================
  // In the accumulators a lane holds 4 consecutive output columns of its query (8 bytes) for each
  // of 8 column groups: stored from there, an instruction writes 16 bytes to each of 32 rows.
  // Staged through the wave's slab memory (idle by now), a tile leaves as whole 128-byte rows, 16
  // bytes per lane, 8 lanes side by side on a row; the stores are streamed (non-temporal).
  constexpr int OPITCH = DH * 2 + 16;                    // staged row pitch in bytes (+16: rows spread over the banks)
  static_assert(32 * OPITCH <= STB_WAVE, "a staged tile fits the wave's slab memory");
  unsigned char* ostage = (unsigned char*)stb_wave;
  const bool ovec = (a.o_stride_n & 7) == 0 && (a.o_stride_b & 7) == 0 && (a.o_stride_h & 7) == 0 &&
                    ((uintptr_t)a.o & 15) == 0;
#pragma unroll
  for (int x = 0; x < 2; ++x) {
    if (x == 1 && last_wg) break;
    const int cq0 = x == 0 ? cb0 : cb1, cq = cq0 + ln;
    const float ltot = qt[x].l + __shfl_xor(qt[x].l, 32);
    const float inv = 1.f / ltot;
    bf16_t* obase = (bf16_t*)a.o + b * a.o_stride_b + h * a.o_stride_h;
    if (a.lse && active && cq < C_ && hh == 0)
      a.lse[((int64_t)b * a.H + h) * ((int64_t)T_ * C_) + (int64_t)tq * C_ + cq] = qt[x].m + log2f(ltot);
    if (ovec) {
      wave_lds_sync();                                 // (the slab memory's last readers / the tile before)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
          bf16x4 w;
#pragma unroll
          for (int r = 0; r < 4; ++r) w[r] = (__bf16)(qt[x].acc[mt][a4 * 4 + r] * inv);
          *(bf16x4*)(ostage + ln * OPITCH + (mt * 32 + a4 * 8 + hh * 4) * 2) = w;
        }
      wave_lds_sync();
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        const int row = it * 8 + (lane >> 3), ch = lane & 7;
        const u32x4 v = *(const u32x4*)(ostage + row * OPITCH + ch * 16);
        if (active && cq0 + row < C_) {
          const int64_t n = (int64_t)tq * C_ + cq0 + row;
          __builtin_nontemporal_store(v, (u32x4*)(obase + n * a.o_stride_n + ch * 8));
        }
      }
    } else if (active && cq < C_) {
      bf16_t* orow = obase + ((int64_t)tq * C_ + cq) * a.o_stride_n;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
          const int d0 = mt * 32 + a4 * 8 + hh * 4;
          bf16x4 w;
#pragma unroll
          for (int r = 0; r < 4; ++r) w[r] = (__bf16)(qt[x].acc[mt][a4 * 4 + r] * inv);
          *(bf16x4*)(orow + d0) = w;
        }
    }
  }
}

}  // namespace q64
}  // namespace mvpa

// Shapes the whole-time-step kernel serves: bf16, head size 64, 33..64 channels, a plain forward
// (no decoding step, no fp8 content term); everything else about the arguments is as for the
// general kernel (mvpa_mfma_supported).
int mvpa_mfma64_supported(const mvpa_fwd_args* a) {
  if (a->dtype != MVPA_BF16 || a->Dh != 64 || a->C <= 32 || a->C > 64) return 0;
  if (a->flags & (MVPA_FLAG_LAST_STEP | MVPA_FLAG_RING | MVPA_FLAG_FP8_QK)) return 0;
  return 1;
}

int mvpa_launch_mfma64(const mvpa_fwd_args* a, hipStream_t stream) {
  using namespace mvpa::q64;
  mvpa::want_dynamic_lds((const void*)mvpa_mfma64_kernel, (int)LDS_BYTES);
  const bool own_last = (a->flags & MVPA_FLAG_CONTENT) && a->T > 1;       // as in the kernel
  const int nt = ((own_last ? a->T - 1 : a->T) + TQW - 1) / TQW + (own_last ? 1 : 0);
  MVPA_LAUNCH(mvpa_mfma64_kernel, dim3((unsigned)(nt * a->B * a->H)), dim3(NW * 64), LDS_BYTES, stream, *a);
  return mvpa::take_launch_status();
}
