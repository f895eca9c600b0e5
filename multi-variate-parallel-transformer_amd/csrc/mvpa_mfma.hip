// Tiled MFMA kernel (bf16, or fp16 through the element-type parameter E) for the MVPA forward on gfx950 (CDNA4, wave64).
//
// Tokens are a T x C grid (n = t*C + c).  Both queries and keys are tiled BY TIME STEP: a key
// tile is the C keys of one time step tk (channels padded to CP = 32/64/128), a query block is
// 32 channels of one time step tq and belongs to one wave.  With that tiling
//   * the time-causal mask is uniform per (query block, key tile): tile tk is either fully
//     visible (tk <= tq) or skipped - there is no diagonal tile to mask element-wise;
//   * the relative-time term (q+v).r[T-1-(tq-tk)] is ONE scalar per query row per key tile;
//   * the relative-channel term (q+z).e[C-1-|cq-ck|] is a [CP x 32] tile per query block that
//     is IDENTICAL for every key tile: it is built once, kept in registers in MFMA accumulator
//     layout and fed to the QK^T MFMA as its C operand, so adding it costs nothing;
//   * the content window (layers/mvpa.py:231-245) is uniform per (query block, key tile) too.
//     Outside the window the content term is zeroed, so the score is a SUM of a per-tile scalar
//     and a per-channel value and its exponential FACTORISES:
//         p(q, tk, ck) = et[q,tk] * Ec[q,ck].
//     Such "far" tiles need no QK^T, no per-element exp and no K load:
//         acc[q,:] += et[q,tk] * (Ec[q,:] @ V[tk]),   l[q] += et[q,tk] * sum_ck Ec[q,ck],
//     with Ec resident in registers as the MFMA B operand for the whole kernel.
//
// Everything is computed transposed, S^T = K Q^T and O^T = V^T P^T, so that a lane owns ONE
// query (MFMA column): the soft-max statistics are per-lane scalars, the row max is an in-lane
// reduction plus one exchange between the two half-waves, and P^T leaves the QK^T MFMA already
// in the layout the PV MFMA wants for its B operand (the contraction index is permuted
// consistently on the V side instead).
//
// Data movement: K/V tiles go HBM/L2 -> LDS with direct-to-LDS loads (no staging registers)
// into a ring of STAGES buffers, several tiles ahead of the compute; rows keep their natural
// [key][dh] layout with an XOR swizzle of the 16-byte chunks (chosen per lane on the global
// side, since the LDS side of such a load is lane-linear).  K fragments are plain 16-byte LDS
// reads; V^T fragments come from the transposing LDS read (ds_read_b64_tr_b16), which turns four
// keys x 16 dh of row-major V into "4 keys per lane, one dh per lane".
// One workgroup = NW waves = NW query blocks = NW/NCT consecutive time steps; one barrier per
// key tile.  Where registers allow, two 4-wave workgroups share a CU so that one computes while
// the other sits at its barrier.
#include "mvpa_mfma_tools.h"

namespace mvpa {

// NCT = key-channel tiles a WAVE handles per key step; KH = parts the keys of a step are split
// into (each part has its own waves, which keep a partial soft-max state over their keys and merge
// at the end).  Queries and keys cover the same QT = NCT * KH tiles of 32 channels.
template <int DH, int NCT, int NW, int STAGES, int KH = 1>
struct Cfg {
  static constexpr int QT = NCT * KH;          // 32-channel tiles per time step
  static constexpr int CP = QT * 32;           // padded channels per time step (rows of a K/V tile)
  static constexpr int WPT = QT * KH;          // waves per time step: query tiles x key parts
  static constexpr int KS = DH / 16;           // k-steps of the QK^T contraction
  static constexpr int MT = DH / 32;           // 32-row tiles of O^T
  static constexpr int TQW = NW / WPT;         // time steps per workgroup
  static constexpr int THREADS = NW * 64;
  static constexpr int ROWB = DH * 2;          // bytes per K/V row
  static constexpr int CHUNKS = DH / 8;        // 16-byte chunks per row
  static constexpr int TILE_BYTES = CP * ROWB;
  static constexpr int WLOADS = TILE_BYTES / 1024;           // 64-lane x 16-byte loads per tile
  static constexpr int LPW = (WLOADS + NW - 1) / NW;         // ... per wave
  static constexpr int STAGE_BYTES = 2 * TILE_BYTES;         // K tile then V tile
  static constexpr int RING_BYTES = STAGES * STAGE_BYTES;
  static constexpr int STB_BYTES = NW * 32 * 32 * 4;
  static constexpr int MAIN_BYTES = RING_BYTES + STB_BYTES;
  static constexpr int SETUP_BYTES = NW * CP * 32 * 4;
  static constexpr int LDS_BYTES = MAIN_BYTES > SETUP_BYTES ? MAIN_BYTES : SETUP_BYTES;
  // the set-up scratch fits behind the stages of the prologue tiles
  static constexpr bool EARLY = STAGES >= 2 && SETUP_BYTES <= STAGE_BYTES + STB_BYTES;
  static_assert(NW % WPT == 0, "waves must cover whole time steps");
  static_assert(TILE_BYTES % 1024 == 0, "tile must be a whole number of wave loads");
  static_assert(WLOADS % NW == 0 || WLOADS < NW, "every loading wave issues the same number of loads");
};

template <int DH, int NCT, int NW, int STAGES, int MINB, bool FP8, int KH, bool RUNS, typename E>
__global__ __launch_bounds__(NW * 64, MINB) void mvpa_mfma_kernel(mvpa_fwd_args a) {
  using x8 = typename E::x8;                     // fragments of the element type (bf16 or fp16)
  using x4 = typename E::x4;
  using x2 = typename E::x2;
  using G = Cfg<DH, NCT, NW, STAGES, KH>;
  constexpr int CP = G::CP, KS = G::KS, MT = G::MT, ROWB = G::ROWB, CHUNKS = G::CHUNKS;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  float* Stb_all = (float*)(smem_raw + G::RING_BYTES);          // [NW][32][32]
  // [NW][CP][32] set-up scratch; aliases the ring (and the slabs), see EARLY
  float* setup_all = (float*)(smem_raw + (G::EARLY ? (STAGES - 1) * G::STAGE_BYTES : 0));

  const int tid = threadIdx.x, lane = tid & 63;
  // the wave index is uniform by construction; reading it through a scalar register lets the
  // compiler branch on everything derived from it (tq, far/near, ...) without exec masking
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, hh = lane >> 5;
  const int C_ = a.C, W = a.window;
  // MVPA_FLAG_LAST_STEP with a split workspace: block L works on run L / (B*H) of the key steps,
  // steps [t_lo, t_lo + T_).  Seen from the queries of the last step a run is a problem of its
  // own (content term everywhere, every key visible, table row of key step tk is tk), so the rest
  // of the kernel just takes T_ steps from pointers moved on by t_lo; its normalised output and
  // log-sum-exp go to the workspace, from where mvpa_split_merge_kernel combines the runs.
  // (RUNS: a build of the kernel of its own, so that the usual launch carries none of this.)
  const int n_split = RUNS ? max(a.n_split, 1) : 1;
  const int split_len = (a.T + n_split - 1) / n_split;
  const int run = n_split > 1 ? (int)blockIdx.x / (a.B * a.H) : 0;
  const int t_lo = run * split_len;
  const int T_ = n_split > 1 ? min(split_len, a.T - t_lo) : a.T;
  const bool has_content = a.flags & MVPA_FLAG_CONTENT;
  const bool has_time = a.flags & MVPA_FLAG_TIME_BIAS;
  const bool has_chan = a.flags & MVPA_FLAG_CHAN_BIAS;

  // ---- block -> (b*H + h, time tile).  Workgroups are dealt round-robin to the 8 XCDs, so
  // ids that are equal mod 8 share an L2: give them the same (b, h) so its K/V stay in that L2.
  // The LAST time tile of every (b, h) goes out first: its final row keeps the content term for
  // every key step (no far steps at all), which makes it several times longer than any other
  // workgroup, and it must not be what the rest of the grid ends up waiting for.  After those,
  // within a (b, h) the latest (= longest) time tiles are issued first.
  // SPLIT (two query time steps per workgroup, ring of 4): the last time step gets a workgroup
  // of its own, both pairs of waves on tq = T-1; the ring then advances two key steps per
  // barrier, one pair of waves takes the even and the other the odd one at the same time, and the
  // two partial soft-max states are merged through LDS at the end.  That workgroup is the critical
  // path of a launch (content term at every key step), and this halves it.
  constexpr bool SPLIT = G::TQW == 2 && STAGES == 4 && KH == 1;
  const int nt = SPLIT ? 1 + T_ / 2 : (T_ + G::TQW - 1) / G::TQW;
  const int nbh = a.B * a.H;
  // MVPA_FLAG_LAST_STEP: only the workgroup of the last time step runs, one per (b, h); q, o and
  // lse are indexed by channel alone
  const bool last_only = a.flags & MVPA_FLAG_LAST_STEP;
  int bh, tile;
  {
    const int L = blockIdx.x;
    if (last_only) {
      bh = n_split > 1 ? L % nbh : L;
      tile = nt - 1;
    } else {
      map_block(L, nbh, nt, a.H / a.Hkv, bh, tile);
    }
  }
  const int b = bh / a.H, h = bh % a.H;
  const int g = h / (a.H / a.Hkv);
  const bool split_last = SPLIT && tile == nt - 1;
  const int par = wave / G::WPT;                   // split_last: parity of this wave's key steps
  const int kh = KH > 1 ? (wave / G::QT) % KH : 0; // the part of the keys this wave works on
  const int key0 = kh * (NCT * 32);                // its first key channel
  const int key_off = key0 * G::ROWB;              // ... as a byte offset into a K or V tile
  const int tq0 = split_last ? T_ - 1 : tile * G::TQW;
  const int tq_hi = split_last ? T_ - 1 : min(T_ - 1 - (SPLIT ? 1 : 0), tq0 + G::TQW - 1);
  const int tq = split_last ? T_ - 1 : tq0 + wave / G::WPT;
  const bool active = tq <= tq_hi && (!last_only || tq == T_ - 1);
  const int cq = (wave % G::QT) * 32 + ln;         // this lane's query channel
  const bool qok = active && cq < C_;

  // Loads below are unconditional: rows that do not exist (padded channels, time steps past the
  // end) are redirected to an existing row and their results are never used.
  const bf16_t* qrow = (const bf16_t*)a.q + b * a.q_stride_b + h * a.q_stride_h +
                       (int64_t)(active ? (last_only ? 0 : tq * C_) + min(cq, C_ - 1) : 0) * a.q_stride_n;
  const bf16_t* kbase = (const bf16_t*)a.k + b * a.k_stride_b + g * a.k_stride_h + (int64_t)t_lo * C_ * a.k_stride_n;
  const bf16_t* vbase = (const bf16_t*)a.v + b * a.v_stride_b + g * a.v_stride_h + (int64_t)t_lo * C_ * a.v_stride_n;
  // MVPA_FLAG_RING: slot s holds the step whose table row is (s + ring_rot) mod T
  const bool ring = RUNS && (a.flags & MVPA_FLAG_RING);
  const int ring_rot = ring ? a.T - 1 - __builtin_amdgcn_readfirstlane(*a.ring_head) : 0;
  const bf16_t* ktime = (const bf16_t*)a.k_time + ((int64_t)g * a.T + (ring ? 0 : t_lo)) * DH;
  const bf16_t* kchan = (const bf16_t*)a.k_chan + (int64_t)g * C_ * DH;
  const bf16_t* bu = (const bf16_t*)a.bias_u + g * DH;
  const bf16_t* bv = (const bf16_t*)a.bias_v + g * DH;
  const bf16_t* bz = (const bf16_t*)a.bias_z + g * DH;
  const uint8_t* valid = a.chan_valid ? a.chan_valid + (int64_t)b * C_ : nullptr;
  const float sc2 = a.sm_scale * kLog2e;           // scores live in the base-2 domain

  // =========================== tile ring ===========================
  // Wave-load li of a tile covers bytes [li*1024, li*1024+1024): lane L delivers physical chunk
  // li*64+L, i.e. row (li*64+L)/CHUNKS; the logical chunk it fetches is un-swizzled here.  Rows of
  // padded channels fetch the last real channel instead; whatever lands in rows of padded or
  // absent channels is neutralised by Ec = 0 / Bc = -inf.
  int k_off[G::LPW], v_off[G::LPW];
#pragma unroll
  for (int i = 0; i < G::LPW; ++i) {
    const int pc = (wave + NW * i) * 64 + lane;
    const int row = pc / CHUNKS, phys = pc % CHUNKS;
    const int rowc = min(row, C_ - 1);
    k_off[i] = (int)(rowc * a.k_stride_n) + ((phys ^ swz_k<DH>(row)) << 3);
    v_off[i] = (int)(rowc * a.v_stride_n) + ((phys ^ swz_v<DH>(row)) << 3);
  }
  // first key step that needs K: the band of the earliest query step of this workgroup
  const int tk_near = !has_content ? tq_hi + 1 : (W <= 0 || tq_hi == T_ - 1) ? 0 : max(0, tq0 - W);
  const uint32_t ring_lds = (uint32_t)(uintptr_t)(LDS_PTR(unsigned char))smem_raw;
  auto issue_tile = [&](int tk, int stage_idx, bool with_k) {
    const uint32_t stage = ring_lds + stage_idx * G::STAGE_BYTES;
    const bf16_t* vsrc = vbase + (int64_t)tk * C_ * a.v_stride_n;
#pragma unroll
    for (int i = 0; i < G::LPW; ++i) {
      const int li = wave + NW * i;
      if (li < G::WLOADS) load_to_lds_16(vsrc + v_off[i], stage + G::TILE_BYTES + li * 1024);
    }
    if (with_k) {
      const bf16_t* ksrc = kbase + (int64_t)tk * C_ * a.k_stride_n;
#pragma unroll
      for (int i = 0; i < G::LPW; ++i) {
        const int li = wave + NW * i;
        if (li < G::WLOADS) load_to_lds_16(ksrc + k_off[i], stage + li * 1024);
      }
    }
  };
  // wave loads this wave issues per (V or K) tile: a compile-time count unless the tile is
  // smaller than one load per wave
  const int n_issue = G::WLOADS >= NW ? G::LPW : (wave < G::WLOADS ? 1 : 0);

  // Phase A (further down) walks the key steps that are far for every query of the workgroup in
  // groups of STAGES; only V tiles are in flight there, so the K halves of the ring stages lie
  // idle.  They are used to take the latency of the time-bias slabs off the critical path:
  //   * the K half of stage 0 receives the 32 + TQW - 1 rows of the time table that the
  //     workgroup's next slab needs ("row tile": row r = table row base + r, K-tile swizzle),
  //     requested like a K tile four key steps before the slab is due;
  //   * the K halves of stages 1 .. hold each wave's (q+v) fragments, written once at set-up.
  // A slab inside phase A then takes both MFMA operands from LDS instead of waiting for global
  // memory.  Slabs outside phase A (the window steps at the end) use the global path.
  const int fast_end = RUNS ? 0 : min(tk_near - (STAGES - 1), tq0 + 1);
  const int n_groups = fast_end > 0 ? fast_end / STAGES : 0;
  // (with EARLY the set-up scratch lies over the last stage while the fragments are stored)
  constexpr bool SLAB_LDS = !RUNS && STAGES >= 3 && G::WLOADS % NW == 0 && CP >= 31 + G::TQW &&
                            (STAGES - (G::EARLY ? 2 : 1)) * G::TILE_BYTES >= NW * KS * 1024;
  const bool slab_lds = SLAB_LDS && n_groups > 0 && has_time;
  auto issue_rows = [&](int tk) {            // row tile of the slab that starts at key step tk
    const int base = time_row(tq_hi, tk, T_);
#pragma unroll
    for (int i = 0; i < G::LPW; ++i) {
      const int pc = (wave + NW * i) * 64 + lane;
      const int row = pc / CHUNKS, phys = pc % CHUNKS;
      const bf16_t* src = ktime + (int64_t)min(base + row, T_ - 1) * DH + ((phys ^ swz_k<DH>(row)) << 3);
      load_to_lds_16(src, ring_lds + (wave + NW * i) * 1024);
    }
  };

  // prologue: tiles 0 .. STAGES-2 in flight.  Where the set-up scratch fits into what the
  // prologue leaves alone (the last stage and the time-bias slabs, both first written after the
  // first barrier of the key loop) the tiles are requested right away, so that their round trip
  // overlaps the set-up instead of following it.
  if (G::EARLY) {
    if (SLAB_LDS && slab_lds) issue_rows(0);
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
      if (s <= tq_hi) issue_tile(s, s, s >= tk_near);
  }

  // =========================== setup: Qu, Qv, channel bias tile, Ec ===========================
  // big configurations (Dh 128, or 4 key tiles per wave) are register bound: there the K
  // fragments of a near step are requested tile by tile instead of all at once.  The (q+v)
  // fragments are needed once per 32-step slab only and are re-formed there from q (an L2 hit)
  // instead of kept in registers.
  constexpr bool LEAN = KS * NCT > 8;
  x8 Qu[KS];                        // (q+u) * scale as QK^T B operand
  // fp8 content term: q' = (q+u)*scale/sq and k' = k/sk are rounded to e4m3 with the per-head
  // amax scales sq, sk chosen by the caller; the MFMA accumulates in units of 1/(sq*sk), the
  // channel-bias tile is pre-divided accordingly and the product sq*sk returns inside the exp2 fma
  long Qu8[KS];
  float fp8_d = 1.f, fp8_inv_sk = 1.f;
  if (FP8) {
    const float sq = a.fp8_q_scale[h], sk = a.fp8_k_scale[g];
    fp8_d = sq * sk;
    fp8_inv_sk = 1.f / sk;
  }
  // this wave's (q+v) fragments for the slabs of phase A, in the K halves of stages 1 ..
  unsigned char* qv_lds = smem_raw + G::STAGE_BYTES + ((wave * KS * 1024) / G::TILE_BYTES) * G::STAGE_BYTES +
                          (wave * KS * 1024) % G::TILE_BYTES + lane * 16;
  f32x16 Bc[NCT];            // channel-bias tile, [ck][q] in accumulator layout; -inf = masked key
  {
    u32x4 raw[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) raw[ks] = *(const u32x4*)(qrow + ks * 16 + hh * 8);
    f32x16 sct[G::QT];       // the whole channel table (every distance), whatever the key part
#pragma unroll
    for (int t = 0; t < G::QT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) sct[t][i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 16 + hh * 8;
      Qu[ks] = E::qfrag(raw[ks], bu + d0, sc2);
      if (FP8) Qu8[ks] = make_qfrag_fp8(raw[ks], bu + d0, sc2 / a.fp8_q_scale[h]);
      if (SLAB_LDS && G::EARLY && slab_lds) *(x8*)(qv_lds + ks * 1024) = E::qfrag(raw[ks], bv + d0, sc2);
      const x8 qz = E::qfrag(raw[ks], bz + d0, sc2);
#pragma unroll
      for (int t = 0; t < G::QT; ++t) {
        const int j = min(t * 32 + ln, C_ - 1);
        const u32x4 er = *(const u32x4*)(kchan + (int64_t)j * DH + d0);
        sct[t] = E::mfma(E::as8(er), qz, sct[t], 0, 0, 0);
      }
    }
    float* scr = setup_all + wave * (CP * 32);
#pragma unroll
    for (int t = 0; t < G::QT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int j = t * 32 + (i >> 2) * 8 + hh * 4 + (i & 3);
        scr[j * 32 + ln] = has_chan ? sct[t][i] : 0.f;
      }
    // key-channel mask: bit ck set = channel exists and is present.  Each lane keeps the bits of
    // its own 32 keys (8(i/4) + 4hh + i%4 within key tile t) shifted down by 4hh, so that the bit
    // of element i sits at the compile-time position 8(i/4) + i%4.
    uint32_t kbits[NCT];
    {
      uint64_t kmask[2];
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const int ck = w * 64 + lane;
        bool ok = ck < C_;
        if (valid) ok = ok && valid[min(ck, C_ - 1)] != 0;
        kmask[w] = __ballot(ok);
      }
#pragma unroll
      for (int t = 0; t < NCT; ++t) {
        const int gt = kh * NCT + t;           // key tile within the time step
        kbits[t] = (uint32_t)(kmask[gt >> 1] >> ((gt & 1) * 32 + 4 * hh));
      }
    }
    wave_lds_sync();
    // Bc[ck][q] = scr[C-1-|cq-ck|][q].  With ck = c_i + 4hh (c_i a compile-time constant) the
    // distance is |(cq - 4hh + 4) - (c_i + 4)| on unsigned operands; distances past C-1 only occur
    // for padded queries or keys, whose values are never used, and are clamped into the scratch.
    const uint32_t cq4 = (uint32_t)(cq - 4 * hh + 4);
    const int gbase = ((C_ - 1) * 32 + ln) * 4;
    const unsigned char* scr_b = (const unsigned char*)scr;
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint32_t ci4 = (uint32_t)(key0 + t * 32 + (i >> 2) * 8 + (i & 3) + 4);
        const uint32_t dist = min(max(cq4, ci4) - min(cq4, ci4), (uint32_t)(C_ - 1));
        const float val = *(const float*)(scr_b + (gbase - (int)(dist * 128u)));
        const bool kv = (kbits[t] >> ((i >> 2) * 8 + (i & 3))) & 1u;
        Bc[t][i] = kv ? val : -INFINITY;
      }
  }

  float mc, sumEc;
  x8 Ec[NCT][2];         // exp2(Bc - mc) as PV B-operand fragments
  {
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, Bc[t][i]);
    mc = xhalf_max(mx);
    // every key channel of this wave's part absent (a KH = 2 wave whose channels 64.. are all
    // masked): Ec = 0 and sumEc = 0 with a finite reference, so the part contributes exactly nothing
    if (mc == -INFINITY) mc = 0.f;
    float se = 0.f;
#pragma unroll
    for (int t = 0; t < NCT; ++t) {
      f32x16 e;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        e[i] = fast_exp2(Bc[t][i] - mc);
        se += e[i];
      }
      Ec[t][0] = E::pack(e, 0);
      Ec[t][1] = E::pack(e, 8);
    }
    sumEc = se;               // partial: this half-wave's keys only
  }
  if (FP8) {
    const float inv_d = 1.f / fp8_d;
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) Bc[t][i] *= inv_d;
  }

  // running soft-max state of this lane's query; l is a per-half-wave partial sum.  The reference
  // point starts at a finite floor instead of -inf: exp2(floor - m) is 0 all the same, and a step
  // whose scores are all -inf (every key of the part masked) gives exp2(-inf + (st - floor)) = 0
  // instead of exp2(-inf + inf) = NaN
  float m_run = kMFloor, l_run = 0.f;
  f32x16 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[mt][i] = 0.f;

  if (!G::EARLY) {
    lds_barrier();           // the set-up scratch aliases the stages the prologue fills
    if (SLAB_LDS && slab_lds) issue_rows(0);
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
      if (s <= tq_hi) issue_tile(s, s, s >= tk_near);
  }
  if (SLAB_LDS && slab_lds && !G::EARLY) {        // (with EARLY the set-up stored them already)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 16 + hh * 8;
      *(x8*)(qv_lds + ks * 1024) = E::qfrag(*(const u32x4*)(qrow + d0), bv + d0, sc2);
    }
  }

  float* Stb = Stb_all + wave * (32 * 32);
  // key steps 0 .. far_max are "far" for this wave's queries (content term absent or zeroed)
  // (RUNS launches are last-step launches with the content term on: no far steps at all, and the
  // far path is compiled out of that build of the kernel)
  const int far_max = RUNS ? -1 : !has_content ? tq : (W > 0 && tq != T_ - 1) ? tq - W - 1 : -1;
  auto is_far = [&](int tk) -> bool { return tk <= far_max; };

  // ---- per-lane pieces of the LDS fragment addresses (loop invariant)
  //   V^T fragment (t, s, mt), read rd: row 32t+16s+8rd+4hh+e, dh 32mt+16grp+4a (transposing read);
  //   the row's swizzle depends only on e, so (t, s, rd) become immediate offsets
  //   K fragment (t, ks): row 32t+ln, logical chunk 2ks+hh; the swizzle depends only on ln
  int v_lane[MT], k_lane[KS];
  {
    const int e = (ln & 15) >> 2, aa = ln & 3, grp = ln >> 4;
    const int row0 = 4 * hh + e;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      v_lane[mt] = G::TILE_BYTES + row0 * ROWB +
                   (((4 * mt + 2 * grp + (aa >> 1)) ^ swz_v<DH>(row0)) << 4) + ((aa & 1) << 3);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_lane[ks] = ln * ROWB + (((2 * ks + hh) ^ swz_k<DH>(ln)) << 4);
  }
  auto v_frag = [&](const unsigned char* stage, int t, int s, int mt) -> x8 {
    const unsigned char* p = stage + v_lane[mt] + (32 * t + 16 * s) * ROWB;
    const x4 lo = E::read_tr(p);
    const x4 hi = E::read_tr(p + 8 * ROWB);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };

  // ---- time-bias slab: St[j][q] for key steps [tk, tk+32) -> LDS, plus one soft-max rescale that
  //      covers every far step of the slab
  auto time_slab = [&](int tk, bool from_lds) {
    const int j0 = time_row(tq, tk, T_);
    f32x16 stc;
#pragma unroll
    for (int i = 0; i < 16; ++i) stc[i] = 0.f;
    if (SLAB_LDS && from_lds) {
      // row tile in the K half of stage 0: this wave's rows start tq_hi - tq rows into it
      const int row = tq_hi - tq + ln;
      const unsigned char* rp = smem_raw + row * ROWB;
      const int sw = swz_k<DH>(row);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const x8 rr = *(const x8*)(rp + (((2 * ks + hh) ^ sw) << 4));
        const x8 qv = *(const x8*)(qv_lds + ks * 1024);
        stc = E::mfma(rr, qv, stc, 0, 0, 0);
      }
    } else if (has_time) {
      int j = min(j0 + ln, T_ - 1);                // rows past T-1 belong to tk > tq: never used
      if (ring) j = (t_lo + tk + ln + ring_rot) % a.T;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const u32x4 rr = *(const u32x4*)(ktime + (int64_t)j * DH + ks * 16 + hh * 8);
        const x8 qv = E::qfrag(*(const u32x4*)(qrow + ks * 16 + hh * 8), bv + ks * 16 + hh * 8, sc2);
        stc = E::mfma(E::as8(rr), qv, stc, 0, 0, 0);
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
    if (tk <= far_max) {                       // the slab holds at least one far step
      const float m_new = fmaxf(m_run, cm + mc);
      const float alpha = fast_exp2(m_run - m_new);     // exp2(floor - m) = 0 on the first slab
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][i] *= alpha;
    }
    wave_lds_sync();
  };

  // ---- far tile: acc += et * (V^T Ec^T), no K, no per-element exp
  auto far_step = [&](const unsigned char* stage, int tk) {
    const float st = Stb[(tk & 31) * 32 + ln];
    f32x16 tmp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) tmp[mt][i] = 0.f;
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          tmp[mt] = E::mfma(v_frag(stage, t, s, mt), Ec[t][s], tmp[mt], 0, 0, 0);
    const float et = fast_exp2(st + mc - m_run);
    l_run += et * sumEc;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][i] += et * tmp[mt][i];
  };

  // Soft-max rescale of the running state.  The multiplies are inline assembly on purpose: they
  // keep the accumulator tiles in their registers on both sides of the (rarely taken) branch
  // around the rescale; left to the compiler, the branch that skips it copies all the tiles.
  // The compiler does not see into the assembly, so the wait states that a vector instruction
  // needs after a matrix instruction wrote its operand (and before one reads its result) are
  // spelled out: 12 before, 2 after.  The branch is taken a few times per workgroup.
  auto rescale_acc = [&](float alpha) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      f32x16 x = acc[mt];
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
      acc[mt] = x;
    }
  };

  // ---- near tile: S^T = K Q^T + Bc, online soft-max, acc += V^T P^T.  The key-channel tiles are
  // taken one after the other (QK^T chains issued tile by tile, then per tile: row max, lazy
  // rescale, exp2, PV), so that the matrix cores work on the next tile's QK^T / the previous
  // tile's PV while this wave does the vector work of a tile.  The V^T fragments of a tile are
  // requested from LDS BEFORE the vector work of that tile (the first tile's right after the QK^T
  // chains are issued, the next tile's before the PV products of the current one), so that their
  // round trip is over when the PV products need them.
  auto near_step = [&](const unsigned char* stage, int tk) {
    const float st = Stb[(tk & 31) * 32 + ln];
    f32x16 S[NCT];
#pragma unroll
    for (int t = 0; t < NCT; ++t) S[t] = Bc[t];
    if (FP8) {
#pragma unroll
      for (int t = 0; t < NCT; ++t)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const u32x4 kr = *(const u32x4*)(stage + k_lane[ks] + t * 32 * ROWB);
          S[t] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(kfrag_fp8(kr, fp8_inv_sk), Qu8[ks], S[t], 0, 0, 0);
        }
    } else {
      if (!LEAN) {
        // every K fragment of the step is requested before the first MFMA waits for one
        x8 ka[KS][NCT];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
          for (int t = 0; t < NCT; ++t) ka[ks][t] = *(const x8*)(stage + k_lane[ks] + t * 32 * ROWB);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < NCT; ++t)
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            S[t] = E::mfma(ka[ks][t], Qu[ks], S[t], 0, 0, 0);
      } else {
#pragma unroll
        for (int t = 0; t < NCT; ++t) {
          x8 ka[KS];
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) ka[ks] = *(const x8*)(stage + k_lane[ks] + t * 32 * ROWB);
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            S[t] = E::mfma(ka[ks], Qu[ks], S[t], 0, 0, 0);
        }
      }
    }
    // V^T fragments of one key tile, [s][mt]; PREFETCH: requested a tile ahead of their use
    constexpr bool PREFETCH = !LEAN;
    x8 vf[2][MT];
    if (PREFETCH) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) vf[s][mt] = v_frag(stage, 0, s, mt);
      __builtin_amdgcn_sched_barrier(0);
    }
    float ls = 0.f;
#pragma unroll
    for (int t = 0; t < NCT; ++t) {
      float rmax = -INFINITY;
#pragma unroll
      for (int i = 0; i < 16; ++i) rmax = fmaxf(rmax, S[t][i]);
      rmax = xhalf_max(rmax);
      if (FP8) rmax *= fp8_d;
      // Lazy running max: the reference point only moves when some query's row max outgrew it by
      // more than 2^8; until then probabilities are formed against the old reference (at most
      // 256 times larger, harmless in fp32/bf16) and the accumulator rescale is skipped.
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
      for (int i = 0; i < 16; ++i)
        S[t][i] = FP8 ? fast_exp2(__builtin_fmaf(S[t][i], fp8_d, off)) : fast_exp2(S[t][i] + off);
      x8 P[2];
      P[0] = E::pack(S[t], 0);
      P[1] = E::pack(S[t], 8);
      // the row sum is taken over the bf16 probabilities the PV product uses, two per
      // instruction (v_dot2c_f32_bf16 against a pair of ones), accumulated in fp32
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        union { x8 v; x2 q[4]; } u;
        u.v = P[s];
#pragma unroll
        for (int j = 0; j < 4; ++j) ls = E::add_pair(u.q[j], ls);
      }
      if (PREFETCH) {
        x8 vn[2][MT];
        if (t + 1 < NCT) {
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) vn[s][mt] = v_frag(stage, t + 1, s, mt);
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[mt] = E::mfma(vf[s][mt], P[s], acc[mt], 0, 0, 0);
        if (t + 1 < NCT) {
#pragma unroll
          for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) vf[s][mt] = vn[s][mt];
        }
      } else {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[mt] = E::mfma(v_frag(stage, t, s, mt), P[s], acc[mt], 0, 0, 0);
      }
    }
    l_run += ls;
  };

  // =========================== split last time step: two key steps per barrier ===============
  // Tile t lives in stage t % 4.  The prologue has tiles 0..2 in flight; at the barrier of pair k
  // the stages of pair k-1 are free and receive pair k+1 (tile 3 alone at k = 0), which then has
  // the whole pair k to arrive: one wait for everything outstanding in front of each barrier.
  if (split_last) {
    for (int k2 = 0; k2 <= T_ - 1; k2 += 4) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int t0 = k2 + 2 * u;                 // first tile of this pair, stage 2u
        if (t0 > T_ - 1) break;                    // uniform over the workgroup
        wait_vmcnt_imm<0>();
        lds_barrier();
        if (t0 == 0) {
          if (3 <= T_ - 1) issue_tile(3, 3, 3 >= tk_near);
        } else {
          if (t0 + 2 <= T_ - 1) issue_tile(t0 + 2, 2 - 2 * u, t0 + 2 >= tk_near);
          if (t0 + 3 <= T_ - 1) issue_tile(t0 + 3, 3 - 2 * u, t0 + 3 >= tk_near);
        }
        if ((t0 & 31) == 0) time_slab(t0, false);
        const int tkw = t0 + par;
        if (tkw <= T_ - 1) {
          const unsigned char* stage = smem_raw + (2 * u) * G::STAGE_BYTES + par * G::STAGE_BYTES;
          if (!RUNS && is_far(tkw)) far_step(stage, tkw);
          else near_step(stage, tkw);
        }
      }
    }
  } else {
  // =========================== phase A: far tiles for every wave ===========================
  // Key steps below tk_near are far for all queries of the workgroup and only V is in flight, so
  // the number of younger loads is a compile-time constant.  The loop is unrolled over the ring so
  // that stage addresses are immediates.  It stops early enough that every tile it issues is
  // still V-only; the generic loop below takes over from there.
  // Within a step the accumulate acc += et * tmp of the PREVIOUS step is deferred to here, so that
  // it fills the LDS latency of this step's first fragments instead of trailing the MFMAs.
  int tk = 0;
  {
    // uniform over the workgroup (every wave must reach the same barriers): all of these steps
    // are at or before tq0, hence visible to every query of the workgroup
    f32x16 ptmp[MT];                       // V^T Ec^T of the previous step, not yet accumulated
    float pet = 0.f;                       // its weight
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) ptmp[mt][i] = 0.f;
    auto flush = [&]() {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][i] += pet * ptmp[mt][i];
      pet = 0.f;
    };
    for (int grp = 0; grp < n_groups; ++grp) {
#pragma unroll
      for (int s = 0; s < STAGES; ++s, ++tk) {
        wait_vmcnt_imm<(STAGES - 2) * G::LPW>();
        lds_barrier();
        // the row tile of a slab that phase A will still reach goes out four steps ahead of it
        // (everybody is past the previous slab's reads of that buffer by now)
        if (SLAB_LDS && slab_lds && ((tk + 4) & 31) == 0 && tk + 4 < n_groups * STAGES) issue_rows(tk + 4);
        issue_tile(tk + STAGES - 1, (s + STAGES - 1) % STAGES, false);
        if ((tk & 31) == 0 && active) {
          flush();
          time_slab(tk, slab_lds);
        }
        if (active) {
          const unsigned char* stage = smem_raw + s * G::STAGE_BYTES + key_off;
          const float st = Stb[(tk & 31) * 32 + ln];
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            x8 vf[NCT * 2];
#pragma unroll
            for (int t = 0; t < NCT; ++t)
#pragma unroll
              for (int s2 = 0; s2 < 2; ++s2) vf[t * 2 + s2] = v_frag(stage, t, s2, mt);
            // previous step's contribution to this output tile, while the fragments arrive
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mt][i] += pet * ptmp[mt][i];
#pragma unroll
            for (int i = 0; i < 16; ++i) ptmp[mt][i] = 0.f;
#pragma unroll
            for (int t = 0; t < NCT; ++t)
#pragma unroll
              for (int s2 = 0; s2 < 2; ++s2)
                ptmp[mt] = E::mfma(vf[t * 2 + s2], Ec[t][s2], ptmp[mt], 0, 0, 0);
          }
          pet = fast_exp2(st + mc - m_run);
          l_run += pet * sumEc;
        }
      }
    }
    flush();
  }

  // =========================== generic loop: remaining key steps ===========================
  // tk is a multiple of STAGES here, so the ring position of each unrolled step is static.
  for (; tk <= tq_hi; ) {
#pragma unroll
    for (int s = 0; s < STAGES; ++s, ++tk) {
      if (tk > tq_hi) break;                       // uniform over the workgroup
      // tile tk has landed once at most the loads of the younger tiles are still in flight
      if (tk + 1 >= tk_near && tk + STAGES - 2 <= tq_hi) {
        wait_vmcnt_imm<2 * (STAGES - 2) * G::LPW>();   // steady state: K and V of STAGES-2 tiles
      } else {
        int younger = 0;
#pragma unroll
        for (int d = 1; d <= STAGES - 2; ++d)
          if (tk + d <= tq_hi) younger += n_issue * (tk + d >= tk_near ? 2 : 1);
        wait_vmcnt(younger);
      }
      lds_barrier();          // tile tk visible to all; everyone is done with tile tk-1's buffer
      if (tk + STAGES - 1 <= tq_hi)
        issue_tile(tk + STAGES - 1, (s + STAGES - 1) % STAGES, tk + STAGES - 1 >= tk_near);
      if ((tk & 31) == 0 && active) time_slab(tk, false);
      if (active && tk <= tq) {
        const unsigned char* stage = smem_raw + s * G::STAGE_BYTES + key_off;
        if (!RUNS && is_far(tk)) far_step(stage, tk);
        else near_step(stage, tk);
      }
    }
  }
  }   // !split_last

  // =========================== epilogue ===========================
  if (split_last || KH > 1) {
    // two waves hold partial soft-max states of the same queries (split last time step: even and
    // odd key steps; KH = 2: the two parts of the key channels): the second one's m, l and
    // accumulator tiles go through LDS into the first one's
    lds_barrier();                                 // every wave is done with the ring
    const int mpar = KH > 1 ? kh : par;
    const int slot = KH > 1 ? (wave / G::WPT) * G::QT + wave % G::QT : wave % NCT;
    float* mb = (float*)smem_raw + slot * ((2 + MT * 16) * 64) + lane;
    if (mpar == 1) {
      mb[0] = m_run;
      mb[64] = l_run;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mb[(2 + mt * 16 + i) * 64] = acc[mt][i];
    }
    lds_barrier();
    if (mpar == 1) return;
    const float m1 = mb[0], l1 = mb[64];
    const float m = fmaxf(m_run, m1);
    // a state that never saw a key still holds the floor: its weight is exp2(floor - m) = 0 and
    // its l and accumulators are 0, unless both are empty (no valid key at all: 0/0 as before)
    const float a0 = fast_exp2(m_run - m);
    const float a1 = fast_exp2(m1 - m);
    m_run = m;
    l_run = a0 * l_run + a1 * l1;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][i] = a0 * acc[mt][i] + a1 * mb[(2 + mt * 16 + i) * 64];
  }
  {
    const float ltot = l_run + __shfl_xor(l_run, 32);
    if (qok) {
      const float inv = 1.f / ltot;
      const int64_t n = (last_only ? 0 : (int64_t)tq * C_) + cq;
      const int64_t prow = ((int64_t)run * nbh + bh) * C_ + cq;      // row of the split workspace
      bf16_t* orow = n_split > 1 ? (bf16_t*)a.split_ws + prow * DH
                                 : (bf16_t*)a.o + b * a.o_stride_b + h * a.o_stride_h + n * a.o_stride_n;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
          const int d0 = mt * 32 + a4 * 8 + hh * 4;
          x4 w;
#pragma unroll
          for (int r = 0; r < 4; ++r) w[r] = E::cvt(acc[mt][a4 * 4 + r] * inv);
          *(x4*)(orow + d0) = w;
        }
      if (n_split > 1) {
        float* plse = (float*)((bf16_t*)a.split_ws + (int64_t)n_split * nbh * C_ * DH);
        if (hh == 0) plse[prow] = m_run + log2f(ltot);
      } else if (a.lse && hh == 0) {
        a.lse[((int64_t)b * a.H + h) * (last_only ? (int64_t)C_ : (int64_t)T_ * C_) + n] = m_run + log2f(ltot);
      }
    }
  }
}

// Combines the runs of a split last-step launch: out = sum_r 2^(lse_r - lse) o_r with
// lse = log2 sum_r 2^lse_r.  DH/8 lanes per output row, 16 bytes each.
template <int DH, typename E>
__global__ __launch_bounds__(256) void mvpa_split_merge_kernel(mvpa_fwd_args a) {
  using x8 = typename E::x8;
  constexpr int LPR = DH / 8, RPB = 256 / LPR;         // lanes per row (8 elements each), rows per block
  const int sub = threadIdx.x % LPR;
  const int nbh = a.B * a.H, C_ = a.C, rows = nbh * C_;
  const int row = blockIdx.x * RPB + threadIdx.x / LPR;
  if (row >= rows) return;
  const bf16_t* po = (const bf16_t*)a.split_ws;
  const float* plse = (const float*)(po + (int64_t)a.n_split * rows * DH);
  float m = -INFINITY;
  for (int r = 0; r < a.n_split; ++r) m = fmaxf(m, plse[(int64_t)r * rows + row]);
  float l = 0.f, acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  for (int r = 0; r < a.n_split; ++r) {
    const float w = fast_exp2(plse[(int64_t)r * rows + row] - m);
    l += w;
    const x8 v = *(const x8*)(po + ((int64_t)r * rows + row) * DH + 8 * sub);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += w * (float)v[i];
  }
  const int bh = row / C_, cq = row % C_, b = bh / a.H, h = bh % a.H;
  const float inv = 1.f / l;
  x8 w8;
#pragma unroll
  for (int i = 0; i < 8; ++i) w8[i] = E::cvt(acc[i] * inv);
  *(x8*)((bf16_t*)a.o + b * a.o_stride_b + h * a.o_stride_h + (int64_t)cq * a.o_stride_n + 8 * sub) = w8;
  if (a.lse && sub == 0) a.lse[row] = m + log2f(l);
}

template <int DH, int NCT, int NW, int STAGES, int MINB, bool FP8, int KH, typename E>
static int launch_one(const mvpa_fwd_args* a, hipStream_t stream) {
  using G = Cfg<DH, NCT, NW, STAGES, KH>;
  static_assert(KH <= 2 && (KH == 1 || G::TQW * G::QT * (2 + G::MT * 16) * 256 <= G::RING_BYTES), "merge buffer");
  static_assert(G::LDS_BYTES <= 160 * 1024, "LDS budget");
  const bool last = a->flags & MVPA_FLAG_LAST_STEP;
  int n_split = (last && a->split_ws && a->n_split > 1) ? a->n_split : 1;
  const bool ring = last && (a->flags & MVPA_FLAG_RING);
  const bool content = a->flags & MVPA_FLAG_CONTENT;
  if (ring && !content) return MVPA_ERR_UNSUPPORTED;      // the run build has no far path
  if (!content) n_split = 1;
  auto kern = (n_split > 1 || ring) ? mvpa_mfma_kernel<DH, NCT, NW, STAGES, MINB, FP8, KH, true, E>
                          : mvpa_mfma_kernel<DH, NCT, NW, STAGES, MINB, FP8, KH, false, E>;
  mvpa::want_dynamic_lds((const void*)kern, (int)G::LDS_BYTES);
  const int nt = (G::TQW == 2 && STAGES == 4 && KH == 1) ? 1 + a->T / 2 : (a->T + G::TQW - 1) / G::TQW;   // as in the kernel
  dim3 grid((unsigned)((last ? n_split : nt) * a->B * a->H));
  MVPA_LAUNCH(kern, grid, dim3(G::THREADS), G::LDS_BYTES, stream, *a);
  if (n_split > 1) {
    const int rows = a->B * a->H * a->C;
    MVPA_LAUNCH((mvpa_split_merge_kernel<DH, E>), dim3((unsigned)((rows + 2048 / DH - 1) / (2048 / DH))), dim3(256), 0, stream, *a);
  }
  return mvpa::take_launch_status();
}

template <int DH, int NCT, int NW, int STAGES, int MINB = 1, int KH = 1>
static int launch_cfg(const mvpa_fwd_args* a, hipStream_t stream) {
  if (a->dtype == MVPA_F16) return launch_one<DH, NCT, NW, STAGES, MINB, false, KH, el_f16>(a, stream);
  if (a->flags & MVPA_FLAG_FP8_QK) return launch_one<DH, NCT, NW, STAGES, MINB, true, KH, el_bf16>(a, stream);
  return launch_one<DH, NCT, NW, STAGES, MINB, false, KH, el_bf16>(a, stream);
}

}  // namespace mvpa

int mvpa_mfma_supported(const mvpa_fwd_args* a) {
  if (a->dtype != MVPA_BF16 && a->dtype != MVPA_F16) return 0;
  if (a->dtype == MVPA_F16 && (a->flags & MVPA_FLAG_FP8_QK)) return 0;
  if (!(a->flags & MVPA_FLAG_CAUSAL)) return 0;
  if (a->key_bias) return 0;
  if (a->C > 128) return 0;
  if (a->Dh != 32 && a->Dh != 64 && a->Dh != 128) return 0;
  const uintptr_t p = (uintptr_t)a->q | (uintptr_t)a->k | (uintptr_t)a->v | (uintptr_t)a->o |
                      (uintptr_t)a->bias_u | (uintptr_t)a->bias_v | (uintptr_t)a->bias_z |
                      (uintptr_t)a->k_time | (uintptr_t)a->k_chan;
  const int64_t s = a->q_stride_b | a->q_stride_h | a->q_stride_n | a->k_stride_b | a->k_stride_h |
                    a->k_stride_n | a->v_stride_b | a->v_stride_h | a->v_stride_n |
                    a->o_stride_b | a->o_stride_h | a->o_stride_n;
  if ((p & 15) || (s & 7)) return 0;
  // per-sample element offsets are kept in 32 bits inside the kernel
  const int64_t n = (int64_t)a->T * a->C;
  if (n * a->k_stride_n >= ((int64_t)1 << 31) || n * a->v_stride_n >= ((int64_t)1 << 31)) return 0;
  // so are the byte offsets of q and o rows (2 bytes per element)
  const int64_t nq = (a->flags & MVPA_FLAG_LAST_STEP) ? a->C : n;
  if (nq * a->q_stride_n >= ((int64_t)1 << 30) || nq * a->o_stride_n >= ((int64_t)1 << 30)) return 0;
  return 1;
}

int mvpa_launch_mfma(const mvpa_fwd_args* a, hipStream_t stream) {
  using namespace mvpa;
  const int nct = a->C <= 32 ? 1 : a->C <= 64 ? 2 : 4;
  switch (a->Dh) {
    case 32:
      if (nct == 1) return launch_cfg<32, 1, 8, 4>(a, stream);
      if (nct == 2) return launch_cfg<32, 2, 8, 4>(a, stream);
      return launch_cfg<32, 4, 4, 4>(a, stream);
    case 64:
      if (nct == 1) return launch_cfg<64, 1, 8, 4>(a, stream);
      if (nct == 2) return launch_cfg<64, 2, 4, 4, 2>(a, stream);   // two workgroups per CU (2 x 80 KiB)
      // 65..128 channels: the keys of a step in two parts of two tiles, 8 waves for one time step
      // (4 query tiles x 2 key parts), two waves per SIMD
      return launch_cfg<64, 2, 8, 3, 1, 2>(a, stream);
    case 128:
      if (nct == 1) return launch_cfg<128, 1, 4, 4>(a, stream);
      if (nct == 2) return launch_cfg<128, 2, 4, 3>(a, stream);
      // key-run (decoding) launches of 97..128 channels: the keys of a step in two parts, 8 waves,
      // two per SIMD (that build has no far path and fits the registers)
      if ((a->flags & MVPA_FLAG_LAST_STEP) && (a->flags & MVPA_FLAG_CONTENT) &&
          ((a->split_ws && a->n_split > 1) || (a->flags & MVPA_FLAG_RING)))
        return launch_cfg<128, 2, 8, 2, 1, 2>(a, stream);
      return launch_cfg<128, 4, 4, 2>(a, stream);
  }
  return MVPA_ERR_UNSUPPORTED;
}
