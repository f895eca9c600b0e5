// Tiled bf16 MFMA kernel for the MVPA forward on gfx950 (CDNA4, wave64).
//
// Tokens are a T x C grid (n = t*C + c).  Both queries and keys are tiled BY TIME STEP: a key
// tile is the C keys of one time step tk (channels padded to CP = 32/64/128), a query block is
// 32 channels of one time step tq.  With that tiling
//   * the time-causal mask is uniform per (query block, key tile): tile tk is either fully
//     visible (tk <= tq) or skipped - there is no diagonal tile to mask element-wise;
//   * the relative-time term (q+v).r[T-1-(tq-tk)] is ONE scalar per query row per key tile;
//   * the relative-channel term (q+z).e[C-1-|cq-ck|] is a [CP x 32] tile per query block that
//     is IDENTICAL for every key tile: it is built once, kept in registers in MFMA accumulator
//     layout and fed to the QK^T MFMA as its C operand, so adding it costs nothing;
//   * the content window (layers/mvpa.py:231-245) is uniform per (query block, key tile) too.
//     Outside the window the content term is zeroed, so the score is a SUM of a per-tile scalar
//     and a per-channel value and its exponential FACTORISES:
//         p(q, tk, ck) = 2^(st[q,tk] - ..) * 2^(bc[q,ck] - ..)  =  et[q,tk] * Ec[q,ck].
//     Such "far" tiles need no QK^T, no per-element exp and no K load:
//         acc[q,:] += et[q,tk] * (Ec[q,:] @ V[tk]),   l[q] += et[q,tk] * sum_ck Ec[q,ck],
//     with Ec resident in registers as the MFMA B operand for the whole kernel.
//
// Everything is computed transposed, S^T = K Q^T and O^T = V^T P^T, so that a lane owns ONE
// query (MFMA column): the soft-max statistics are per-lane scalars, the row max is an in-lane
// reduction plus one exchange between the two half-waves, and P^T leaves the QK^T MFMA already
// in the layout the PV MFMA wants for its B operand (the contraction index is permuted
// consistently on the V side instead).  V is stored in LDS in "octet" order: the 8 keys that one
// lane contracts in one MFMA are adjacent, so the V^T fragment is a single 16-byte LDS read.
//
// One workgroup = 4 waves = 4*QB query blocks; K/V tiles are staged global -> registers -> LDS,
// double buffered, one barrier per key tile.
#include "mvpa_common.h"

namespace mvpa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// order LDS traffic between the lanes of ONE wave (no workgroup barrier needed)
__device__ inline void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ inline float xhalf_max(float x) { return fmaxf(x, __shfl_xor(x, 32)); }

// 8 bf16 (one 16-byte chunk of a q row) + bias, scaled, back to a bf16 MFMA fragment
__device__ inline bf16x8 make_qfrag(u32x4 raw, const bf16_t* __restrict__ bias, float scale) {
  const u32x4 braw = *(const u32x4*)bias;
  bf16x8 out;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t w = raw[i], bw = braw[i];
    const float lo = (__uint_as_float(w << 16) + __uint_as_float(bw << 16)) * scale;
    const float hi = (__uint_as_float(w & 0xffff0000u) + __uint_as_float(bw & 0xffff0000u)) * scale;
    out[2 * i] = (__bf16)lo;
    out[2 * i + 1] = (__bf16)hi;
  }
  return out;
}

__device__ inline bf16x8 as_bf16x8(u32x4 v) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = v;
  return c.b;
}

__device__ inline bf16x8 pack8(const f32x16& v, int base) {
  bf16x8 out;
#pragma unroll
  for (int i = 0; i < 8; ++i) out[i] = (__bf16)v[base + i];
  return out;
}

template <int DH, int NCT, int QB>
struct Cfg {
  static constexpr int CP = NCT * 32;          // padded channels per time step
  static constexpr int KS = DH / 16;           // k-steps of the QK^T contraction
  static constexpr int MT = DH / 32;           // 32-row tiles of O^T
  static constexpr int WPT = NCT / QB;         // waves per time step
  static constexpr int TQW = 4 / WPT;          // time steps per workgroup
  static constexpr int QW = QB * 32;           // queries per wave
  static constexpr int KPITCH = DH + 8;        // K row pitch (elements): 16 B pad
  static constexpr int K_ELEMS = CP * KPITCH;
  static constexpr int V_ELEMS = CP * DH;
  static constexpr int NV = (CP / 4) * (DH / 8);     // V staging tasks per tile
  static constexpr int NKC = CP * (DH / 8);          // K staging chunks per tile
  static constexpr int VPT = (NV + 255) / 256;       // per thread
  static constexpr int KPT = (NKC + 255) / 256;
  static constexpr size_t KV_BYTES = 2 * (size_t)(K_ELEMS + V_ELEMS) * 2;
  static constexpr size_t STB_BYTES = 4 * 32 * (size_t)QW * 4;
  static constexpr size_t MAIN_BYTES = KV_BYTES + STB_BYTES;
  static constexpr size_t SETUP_BYTES = 4 * (size_t)CP * QW * 4;
  static constexpr size_t LDS_BYTES = MAIN_BYTES > SETUP_BYTES ? MAIN_BYTES : SETUP_BYTES;
};

template <int DH, int NCT, int QB>
__global__ __launch_bounds__(256, 1) void mvpa_mfma_kernel(mvpa_fwd_args a) {
  using G = Cfg<DH, NCT, QB>;
  constexpr int CP = G::CP, KS = G::KS, MT = G::MT, QW = G::QW, KPITCH = G::KPITCH;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t* Ks = (bf16_t*)smem_raw;                               // [2][CP][KPITCH]
  bf16_t* Vt = Ks + 2 * G::K_ELEMS;                             // [2][CP/8][DH][8]
  float* Stb_all = (float*)(smem_raw + G::KV_BYTES);            // [4][32][QW]
  float* setup_all = (float*)smem_raw;                          // [4][CP][QW], aliases the above

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, hh = lane >> 5;
  const int T_ = a.T, C_ = a.C, W = a.window;
  const bool has_content = a.flags & MVPA_FLAG_CONTENT;
  const bool has_time = a.flags & MVPA_FLAG_TIME_BIAS;
  const bool has_chan = a.flags & MVPA_FLAG_CHAN_BIAS;

  // ---- block -> (b*H + h, time tile).  Workgroups are dealt round-robin to the 8 XCDs, so
  // ids that are equal mod 8 share an L2: give them the same (b, h) so its K/V stay in that L2.
  // Within a (b, h) the latest (= longest) time tiles are issued first.
  const int nt = (T_ + G::TQW - 1) / G::TQW;
  const int nbh = a.B * a.H;
  int bh, tile;
  {
    const int L = blockIdx.x;
    if ((nbh & 7) == 0) {
      const int xcd = L & 7, s = L >> 3;
      bh = xcd + 8 * (s / nt);
      tile = s % nt;
    } else {
      bh = L / nt;
      tile = L % nt;
    }
    tile = nt - 1 - tile;
  }
  const int b = bh / a.H, h = bh % a.H;
  const int g = h / (a.H / a.Hkv);
  const int tq0 = tile * G::TQW;
  const int tq_hi = min(T_ - 1, tq0 + G::TQW - 1);
  const int tq = tq0 + wave / G::WPT;
  const bool active = tq < T_;
  const int cb0 = (wave % G::WPT) * QB;            // first 32-channel block of this wave

  const bf16_t* qbase = (const bf16_t*)a.q + b * a.q_stride_b + h * a.q_stride_h;
  const bf16_t* kbase = (const bf16_t*)a.k + b * a.k_stride_b + g * a.k_stride_h;
  const bf16_t* vbase = (const bf16_t*)a.v + b * a.v_stride_b + g * a.v_stride_h;
  const bf16_t* ktime = (const bf16_t*)a.k_time + (int64_t)g * T_ * DH;
  const bf16_t* kchan = (const bf16_t*)a.k_chan + (int64_t)g * C_ * DH;
  const bf16_t* bu = (const bf16_t*)a.bias_u + g * DH;
  const bf16_t* bv = (const bf16_t*)a.bias_v + g * DH;
  const bf16_t* bz = (const bf16_t*)a.bias_z + g * DH;
  const uint8_t* valid = a.chan_valid ? a.chan_valid + (int64_t)b * C_ : nullptr;
  const float sc2 = a.sm_scale * kLog2e;           // scores live in the base-2 domain

  // this lane's query rows
  int cq[QB];
  bool qok[QB];
  const bf16_t* qrow[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    cq[qb] = (cb0 + qb) * 32 + ln;
    qok[qb] = active && cq[qb] < C_;
    qrow[qb] = qbase + (int64_t)(qok[qb] ? tq * C_ + cq[qb] : 0) * a.q_stride_n;
  }

  // =========================== setup: Qu, channel bias tile, Ec ===========================
  bf16x8 Qu[QB][KS];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 16 + hh * 8;
      u32x4 raw = {0u, 0u, 0u, 0u};
      if (qok[qb]) raw = *(const u32x4*)(qrow[qb] + d0);
      Qu[qb][ks] = make_qfrag(raw, bu + d0, sc2);
    }

  f32x16 Bc[QB][NCT];        // channel-bias tile, [ck][q] in accumulator layout; -inf = masked key
  {
    float* scr = setup_all + wave * (CP * QW);
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      f32x16 sct[NCT];
#pragma unroll
      for (int t = 0; t < NCT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) sct[t][i] = 0.f;
      if (has_chan) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const int d0 = ks * 16 + hh * 8;
          u32x4 raw = {0u, 0u, 0u, 0u};
          if (qok[qb]) raw = *(const u32x4*)(qrow[qb] + d0);
          const bf16x8 qz = make_qfrag(raw, bz + d0, sc2);
#pragma unroll
          for (int t = 0; t < NCT; ++t) {
            const int j = t * 32 + ln;
            u32x4 er = {0u, 0u, 0u, 0u};
            if (j < C_) er = *(const u32x4*)(kchan + (int64_t)j * DH + d0);
            sct[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(er), qz, sct[t], 0, 0, 0);
          }
        }
      }
#pragma unroll
      for (int t = 0; t < NCT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int j = t * 32 + (i >> 2) * 8 + hh * 4 + (i & 3);
          scr[j * QW + qb * 32 + ln] = sct[t][i];
        }
    }
    wave_lds_sync();
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int t = 0; t < NCT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int ck = t * 32 + (i >> 2) * 8 + hh * 4 + (i & 3);
          const bool kv = ck < C_ && (!valid || valid[ck] != 0);
          int j = chan_row(cq[qb], ck, C_);
          j = j < 0 ? 0 : j;                   // padded query rows: any in-range row will do
          const float val = scr[j * QW + qb * 32 + ln];
          Bc[qb][t][i] = kv ? val : -INFINITY;
        }
  }

  float mc[QB], sumEc[QB];
  bf16x8 Ec[QB][NCT][2];     // exp2(Bc - mc) as PV B-operand fragments
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < NCT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, Bc[qb][t][i]);
    mx = xhalf_max(mx);
    mc[qb] = mx;
    float se = 0.f;
#pragma unroll
    for (int t = 0; t < NCT; ++t) {
      f32x16 e;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        e[i] = fast_exp2(Bc[qb][t][i] - mx);
        se += e[i];
      }
      Ec[qb][t][0] = pack8(e, 0);
      Ec[qb][t][1] = pack8(e, 8);
    }
    sumEc[qb] = se;           // partial: this half-wave's keys only
  }

  // running soft-max state, per query (lane); l is a per-half-wave partial sum
  float m_run[QB], l_run[QB];
  f32x16 acc[QB][MT];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m_run[qb] = -INFINITY;
    l_run[qb] = 0.f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[qb][mt][i] = 0.f;
  }

  __syncthreads();           // setup scratch aliases the K/V buffers

  // =========================== K/V staging ===========================
  u32x4 vreg[G::VPT][4];
  u32x4 kreg[G::KPT];
  auto need_k = [&](int tk) -> bool {
    return has_content && (W <= 0 || tk >= tq0 - W || tq_hi == T_ - 1);
  };
  auto load_tile = [&](int tk, bool with_k) {
#pragma unroll
    for (int i = 0; i < G::VPT; ++i) {
      const int task = tid + 256 * i;
      if (task < G::NV) {
        const int quad = task / (DH / 8), seg = task % (DH / 8);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int ck = quad * 4 + r;
          u32x4 x = {0u, 0u, 0u, 0u};
          if (ck < C_ && (!valid || valid[ck] != 0))
            x = *(const u32x4*)(vbase + (int64_t)(tk * C_ + ck) * a.v_stride_n + seg * 8);
          vreg[i][r] = x;
        }
      }
    }
    if (with_k) {
#pragma unroll
      for (int i = 0; i < G::KPT; ++i) {
        const int c = tid + 256 * i;
        if (c < G::NKC) {
          const int ck = c / (DH / 8), seg = c % (DH / 8);
          u32x4 x = {0u, 0u, 0u, 0u};
          if (ck < C_ && (!valid || valid[ck] != 0))
            x = *(const u32x4*)(kbase + (int64_t)(tk * C_ + ck) * a.k_stride_n + seg * 8);
          kreg[i] = x;
        }
      }
    }
  };
  auto store_tile = [&](int buf, bool with_k) {
    bf16_t* vdst = Vt + buf * G::V_ELEMS;
#pragma unroll
    for (int i = 0; i < G::VPT; ++i) {
      const int task = tid + 256 * i;
      if (task < G::NV) {
        const int quad = task / (DH / 8), seg = task % (DH / 8);
        const int key0 = quad * 4;
        const int oct = (key0 >> 4) * 2 + ((key0 >> 2) & 1);   // 16-key group, half-wave
        const int jhalf = (key0 >> 3) & 1;
        bf16_t* dst = vdst + ((int64_t)oct * DH + seg * 8) * 8 + jhalf * 4;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const uint32_t x0 = vreg[i][0][w], x1 = vreg[i][1][w], x2 = vreg[i][2][w], x3 = vreg[i][3][w];
          u32x2 lo, hi;
          lo.x = __builtin_amdgcn_perm(x1, x0, 0x05040100u);
          lo.y = __builtin_amdgcn_perm(x3, x2, 0x05040100u);
          hi.x = __builtin_amdgcn_perm(x1, x0, 0x07060302u);
          hi.y = __builtin_amdgcn_perm(x3, x2, 0x07060302u);
          *(u32x2*)(dst + (2 * w) * 8) = lo;
          *(u32x2*)(dst + (2 * w + 1) * 8) = hi;
        }
      }
    }
    if (with_k) {
      bf16_t* kdst = Ks + buf * G::K_ELEMS;
#pragma unroll
      for (int i = 0; i < G::KPT; ++i) {
        const int c = tid + 256 * i;
        if (c < G::NKC) {
          const int ck = c / (DH / 8), seg = c % (DH / 8);
          *(u32x4*)(kdst + ck * KPITCH + seg * 8) = kreg[i];
        }
      }
    }
  };

  load_tile(0, need_k(0));
  store_tile(0, need_k(0));
  __syncthreads();

  float* Stb = Stb_all + wave * (32 * QW);
  const bool last_row = tq == T_ - 1;
  auto is_far = [&](int tk) -> bool {
    return !has_content || (W > 0 && !last_row && tq - tk > W);
  };

  // =========================== main loop over key time steps ===========================
  for (int tk = 0; tk <= tq_hi; ++tk) {
    const int cur = tk & 1;
    const bool more = tk + 1 <= tq_hi;
    const bool nk = more && need_k(tk + 1);
    if (more) load_tile(tk + 1, nk);

    // ---- every 32 key steps: time-bias slab St[j][q] for the next 32 steps -> LDS, and one
    //      soft-max rescale that covers all far steps of the slab
    if ((tk & 31) == 0 && active) {
      const int j0 = time_row(tq, tk, T_);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        f32x16 stc;
#pragma unroll
        for (int i = 0; i < 16; ++i) stc[i] = 0.f;
        if (has_time) {
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const int d0 = ks * 16 + hh * 8;
            u32x4 raw = {0u, 0u, 0u, 0u};
            if (qok[qb]) raw = *(const u32x4*)(qrow[qb] + d0);
            const bf16x8 qv = make_qfrag(raw, bv + d0, sc2);
            const int j = j0 + ln;
            u32x4 rr = {0u, 0u, 0u, 0u};
            if (j >= 0 && j < T_) rr = *(const u32x4*)(ktime + (int64_t)j * DH + d0);
            stc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(rr), qv, stc, 0, 0, 0);
          }
        }
        float cm = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int jj = (i >> 2) * 8 + hh * 4 + (i & 3);
          Stb[jj * QW + qb * 32 + ln] = stc[i];
          const int tkk = tk + jj;
          if (tkk <= tq && is_far(tkk)) cm = fmaxf(cm, stc[i]);
        }
        cm = xhalf_max(cm);
        if (cm > -INFINITY) {
          const float m_new = fmaxf(m_run[qb], cm + mc[qb]);
          const float alpha = fast_exp2(m_run[qb] - m_new);
          m_run[qb] = m_new;
          l_run[qb] *= alpha;
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[qb][mt][i] *= alpha;
        }
      }
      wave_lds_sync();
    }

    if (active && tk <= tq) {
      const bf16_t* vt = Vt + cur * G::V_ELEMS;
      float st[QB];
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) st[qb] = Stb[(tk & 31) * QW + qb * 32 + ln];

      if (is_far(tk)) {
        // ------------------------------ far tile ------------------------------
        f32x16 tmp[QB][MT];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) tmp[qb][mt][i] = 0.f;
#pragma unroll
        for (int t = 0; t < NCT; ++t)
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const int oct = (t * 2 + s) * 2 + hh;
            bf16x8 va[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              va[mt] = *(const bf16x8*)(vt + ((int64_t)oct * DH + mt * 32 + ln) * 8);
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
#pragma unroll
              for (int mt = 0; mt < MT; ++mt)
                tmp[qb][mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[mt], Ec[qb][t][s], tmp[qb][mt], 0, 0, 0);
          }
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          const float et = fast_exp2(st[qb] + mc[qb] - m_run[qb]);
          l_run[qb] += et * sumEc[qb];
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[qb][mt][i] += et * tmp[qb][mt][i];
        }
      } else {
        // ------------------------------ near tile ------------------------------
        const bf16_t* ks_ = Ks + cur * G::K_ELEMS;
        f32x16 S[QB][NCT];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
#pragma unroll
          for (int t = 0; t < NCT; ++t) S[qb][t] = Bc[qb][t];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
          for (int t = 0; t < NCT; ++t) {
            const bf16x8 ka = *(const bf16x8*)(ks_ + (t * 32 + ln) * KPITCH + ks * 16 + hh * 8);
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
              S[qb][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, Qu[qb][ks], S[qb][t], 0, 0, 0);
          }
        bf16x8 P[QB][NCT][2];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          float rmax = -INFINITY;
#pragma unroll
          for (int t = 0; t < NCT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) rmax = fmaxf(rmax, S[qb][t][i]);
          rmax = xhalf_max(rmax);
          const float m_new = fmaxf(m_run[qb], rmax + st[qb]);
          const float alpha = fast_exp2(m_run[qb] - m_new);
          const float off = st[qb] - m_new;
          float ls = 0.f;
#pragma unroll
          for (int t = 0; t < NCT; ++t) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const float p = fast_exp2(S[qb][t][i] + off);
              S[qb][t][i] = p;
              ls += p;
            }
            P[qb][t][0] = pack8(S[qb][t], 0);
            P[qb][t][1] = pack8(S[qb][t], 8);
          }
          m_run[qb] = m_new;
          l_run[qb] = l_run[qb] * alpha + ls;
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[qb][mt][i] *= alpha;
        }
#pragma unroll
        for (int t = 0; t < NCT; ++t)
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const int oct = (t * 2 + s) * 2 + hh;
            bf16x8 va[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              va[mt] = *(const bf16x8*)(vt + ((int64_t)oct * DH + mt * 32 + ln) * 8);
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
#pragma unroll
              for (int mt = 0; mt < MT; ++mt)
                acc[qb][mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[mt], P[qb][t][s], acc[qb][mt], 0, 0, 0);
          }
      }
    }

    if (more) store_tile(cur ^ 1, nk);
    __syncthreads();
  }

  // =========================== epilogue ===========================
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const float ltot = l_run[qb] + __shfl_xor(l_run[qb], 32);
    if (!qok[qb]) continue;
    const float inv = 1.f / ltot;
    const int64_t n = (int64_t)tq * C_ + cq[qb];
    bf16_t* orow = (bf16_t*)a.o + b * a.o_stride_b + h * a.o_stride_h + n * a.o_stride_n;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4) {
        const int d0 = mt * 32 + a4 * 8 + hh * 4;
        u32x2 w;
        const float x0 = acc[qb][mt][a4 * 4 + 0] * inv, x1 = acc[qb][mt][a4 * 4 + 1] * inv;
        const float x2 = acc[qb][mt][a4 * 4 + 2] * inv, x3 = acc[qb][mt][a4 * 4 + 3] * inv;
        w.x = (uint32_t)f32_to_bf16(x0) | ((uint32_t)f32_to_bf16(x1) << 16);
        w.y = (uint32_t)f32_to_bf16(x2) | ((uint32_t)f32_to_bf16(x3) << 16);
        *(u32x2*)(orow + d0) = w;
      }
    if (a.lse && hh == 0) a.lse[((int64_t)b * a.H + h) * ((int64_t)T_ * C_) + n] = m_run[qb] + log2f(ltot);
  }
}

template <int DH, int NCT, int QB>
static int launch_cfg(const mvpa_fwd_args* a, hipStream_t stream) {
  using G = Cfg<DH, NCT, QB>;
  auto kern = mvpa_mfma_kernel<DH, NCT, QB>;
  (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)G::LDS_BYTES);
  const int nt = (a->T + G::TQW - 1) / G::TQW;
  dim3 grid((unsigned)(nt * a->B * a->H));
  hipLaunchKernelGGL(kern, grid, dim3(256), G::LDS_BYTES, stream, *a);
  return hipGetLastError() == hipSuccess ? MVPA_OK : MVPA_ERR_LAUNCH;
}

template <int DH>
static int launch_dh(const mvpa_fwd_args* a, hipStream_t stream) {
  constexpr int QB2 = DH <= 64 ? 2 : 1;
  if (a->C <= 32) return launch_cfg<DH, 1, 1>(a, stream);
  if (a->C <= 64) return launch_cfg<DH, 2, QB2>(a, stream);
  return launch_cfg<DH, 4, 1>(a, stream);
}

}  // namespace mvpa

int mvpa_mfma_supported(const mvpa_fwd_args* a) {
  if (a->dtype != MVPA_BF16) return 0;
  if (!(a->flags & MVPA_FLAG_CAUSAL)) return 0;
  if (a->flags & MVPA_FLAG_FP8_QK) return 0;
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
  return 1;
}

int mvpa_launch_mfma(const mvpa_fwd_args* a, hipStream_t stream) {
  switch (a->Dh) {
    case 32: return mvpa::launch_dh<32>(a, stream);
    case 64: return mvpa::launch_dh<64>(a, stream);
    case 128: return mvpa::launch_dh<128>(a, stream);
  }
  return MVPA_ERR_UNSUPPORTED;
}
