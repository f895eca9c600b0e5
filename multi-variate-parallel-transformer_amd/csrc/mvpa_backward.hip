// MVPA backward, first version: fp32 arithmetic, one lane per row, any shape the forward takes.
//
// Boundary (attentions/attn.py:1140-1302, FlashMVPA.backward): given do and the forward's
// base-2 log-sum-exp, produce
//   dq          [B,H,N,Dh]   gradient through the CONTENT term only (the reference's dq),
//   dk, dv      [B,Hkv,N,Dh] (summed over the query heads of a GQA group),
//   dbias_time  [B,H,N,T]    gradient of the [B,H,N,T] time-bias table (q+v).r[j], column j,
//   dbias_chan  [B,H,N,C]    gradient of the [B,H,N,C] channel-bias table (q+z).e[i], column i.
// The gradients of q_btime / q_bchan / k_time / k_chan and the bias-term share of dq are plain
// matrix products of those two tables (attentions/attn.py:1305-1314 under autograd) and are
// formed by the caller; dq_bias (the gradient of u) is the sum of dq over batch, group and rows.
//
// With ds = p * (do.v - delta) * scale, delta = do.o :
//   dq[n]           = sum_m ds[n,m] * W(tq,tk) * k[m]
//   dk[m]           = sum_n ds[n,m] * W(tq,tk) * (q[n] + u)
//   dv[m]           = sum_n p[n,m] * do[n]
//   dbias_time[n,j] = sum_{m: T-1-(tq-tk) = j} ds[n,m]
//   dbias_chan[n,i] = sum_{m: C-1-|cq-ck| = i} ds[n,m]
//
// Two passes.  The QUERY pass (one lane per query row, keys staged through LDS like the generic
// forward) writes dq, both table gradients, delta, and the two forward bias tables it has to form
// anyway.  The KEY pass (one lane per key row, queries staged through LDS) reads those tables
// back, recomputes p, and accumulates dk and dv without atomics.
#include "mvpa_common.h"

namespace mvpa {

constexpr int BWD_THREADS = 128;
constexpr int BWD_TILE = 32;

template <typename T, int DH>
__global__ __launch_bounds__(BWD_THREADS) void mvpa_bwd_query_kernel(mvpa_bwd_args a) {
  extern __shared__ float smem[];
  float* Ks = smem;                               // [TILE][DH]
  float* Vs = Ks + BWD_TILE * DH;                 // [TILE][DH]
  float* Gc = Vs + BWD_TILE * DH;                 // [128][C+1] per-lane channel-table gradient

  const int tid = threadIdx.x;
  const int T_ = a.T, C_ = a.C, N = a.T * a.C;
  const int b = blockIdx.y / a.H, h = blockIdx.y % a.H;
  const int g = h / (a.H / a.Hkv);
  const bool causal = a.flags & MVPA_FLAG_CAUSAL;
  const bool has_content = a.flags & MVPA_FLAG_CONTENT;
  const bool has_time = a.flags & MVPA_FLAG_TIME_BIAS;
  const bool has_chan = a.flags & MVPA_FLAG_CHAN_BIAS;

  const int nq_raw = blockIdx.x * BWD_THREADS + tid;
  const bool live = nq_raw < N;
  const int nq = live ? nq_raw : N - 1;
  const int tq = nq / C_, cq = nq % C_;
  const int64_t row = ((int64_t)b * a.H + h) * N + nq;

  const T* qrow = (const T*)a.q + b * a.q_stride_b + h * a.q_stride_h + (int64_t)nq * a.q_stride_n;
  const T* orow = (const T*)a.o + b * a.o_stride_b + h * a.o_stride_h + (int64_t)nq * a.o_stride_n;
  const T* drow = (const T*)a.d_o + b * a.do_stride_b + h * a.do_stride_h + (int64_t)nq * a.do_stride_n;
  const T* kbase = (const T*)a.k + b * a.k_stride_b + g * a.k_stride_h;
  const T* vbase = (const T*)a.v + b * a.v_stride_b + g * a.v_stride_h;
  const T* bu = (const T*)a.bias_u + g * DH;
  const T* bv = (const T*)a.bias_v + g * DH;
  const T* bz = (const T*)a.bias_z + g * DH;
  const T* ktime = (const T*)a.k_time + (int64_t)g * T_ * DH;
  const T* kchan = (const T*)a.k_chan + (int64_t)g * C_ * DH;
  const uint8_t* valid = a.chan_valid ? a.chan_valid + (int64_t)b * C_ : nullptr;
  const float* kbias = a.key_bias ? a.key_bias + (int64_t)b * N : nullptr;

  float qu[DH], dov[DH], dq[DH];
  float delta = 0.f;
#pragma unroll
  for (int d = 0; d < DH; ++d) {
    qu[d] = io<T>::load(qrow + d) + io<T>::load(bu + d);
    dov[d] = io<T>::load(drow + d);
    delta += dov[d] * io<T>::load(orow + d);
    dq[d] = 0.f;
  }
  const float lse = a.lse[row];
  if (live) a.ws_delta[row] = delta;

  // forward channel table (q+z).e[i] -> workspace; its gradient accumulates in LDS
  const int gp = C_ + 1;
  float* wchan = a.ws_chan + row * C_;
  float* wtime = a.ws_time + row * T_;
  for (int i = 0; i < C_; ++i) {
    float s = 0.f;
    if (has_chan) {
      const T* e = kchan + (int64_t)i * DH;
#pragma unroll 8
      for (int d = 0; d < DH; ++d) s += (io<T>::load(qrow + d) + io<T>::load(bz + d)) * io<T>::load(e + d);
    }
    if (live) wchan[i] = s;
    Gc[tid * gp + i] = 0.f;
  }
  if (live)
    for (int j = 0; j < T_; ++j) a.dbias_time[row * T_ + j] = 0.f;

  const int q_last = min(N - 1, (int)blockIdx.x * BWD_THREADS + BWD_THREADS - 1);
  const int hi = causal ? (q_last / C_ + 1) * C_ : N;
  int cur_tk = -1;
  float st = 0.f, gt = 0.f;        // time-bias score of the current key step and its gradient

  auto flush_time = [&]() {
    if (cur_tk >= 0 && cur_tk <= tq && live) {
      const int j = time_row(tq, cur_tk, T_);
      wtime[j] = st;
      a.dbias_time[row * T_ + j] = gt;
    }
  };

  for (int k0 = 0; k0 < hi; k0 += BWD_TILE) {
    __syncthreads();
    for (int i = tid; i < BWD_TILE * DH; i += BWD_THREADS) {
      const int kk = i / DH, d = i % DH;
      const int nk = k0 + kk;
      float kv = 0.f, vv = 0.f;
      if (nk < hi) {
        kv = io<T>::load(kbase + (int64_t)nk * a.k_stride_n + d);
        vv = io<T>::load(vbase + (int64_t)nk * a.v_stride_n + d);
      }
      Ks[i] = kv;
      Vs[i] = vv;
    }
    __syncthreads();
    for (int kk = 0; kk < BWD_TILE; ++kk) {
      const int nk = k0 + kk;
      if (nk >= hi) break;
      const int tk = nk / C_, ck = nk - tk * C_;
      if (tk != cur_tk) {          // uniform across the workgroup
        flush_time();
        cur_tk = tk;
        st = 0.f;
        gt = 0.f;
        if (has_time && tk <= tq) {
          const T* r = ktime + (int64_t)time_row(tq, tk, T_) * DH;
#pragma unroll 8
          for (int d = 0; d < DH; ++d)
            st += (io<T>::load(qrow + d) + io<T>::load(bv + d)) * io<T>::load(r + d);
        }
      }
      const bool vis = causal_visible(tq, tk, causal) && (!valid || valid[ck] != 0);
      if (!vis) continue;
      const int ci = chan_row(cq, ck, C_);
      const bool kept = has_content && content_kept(tq, tk, T_, a.window);
      const float* kr = Ks + kk * DH;
      const float* vr = Vs + kk * DH;
      float s = st + (has_chan ? wchan[ci] : 0.f);   // this lane's own store, read back
      float dot = 0.f, dp = 0.f;
#pragma unroll
      for (int d = 0; d < DH; ++d) {
        dot += qu[d] * kr[d];
        dp += dov[d] * vr[d];
      }
      if (kept) s += dot;
      s *= a.sm_scale;
      if (kbias) s += kbias[nk];
      const float p = exp2f(s * kLog2e - lse);
      const float ds = p * (dp - delta) * a.sm_scale;
      if (kept) {
#pragma unroll
        for (int d = 0; d < DH; ++d) dq[d] += ds * kr[d];
      }
      gt += ds;
      Gc[tid * gp + ci] += ds;
    }
  }
  flush_time();

  if (live) {
    float* dqo = a.dq + row * DH;
#pragma unroll
    for (int d = 0; d < DH; ++d) dqo[d] = dq[d];
    float* gc = a.dbias_chan + row * C_;
    for (int i = 0; i < C_; ++i) gc[i] = Gc[tid * gp + i];
  }
}

template <typename T, int DH>
__global__ __launch_bounds__(BWD_THREADS) void mvpa_bwd_key_kernel(mvpa_bwd_args a) {
  extern __shared__ float smem[];
  float* Qs = smem;                               // [TILE][DH]  q + u
  float* Ds = Qs + BWD_TILE * DH;                 // [TILE][DH]  do
  float* Ls = Ds + BWD_TILE * DH;                 // [TILE] lse
  float* Es = Ls + BWD_TILE;                      // [TILE] delta

  const int tid = threadIdx.x;
  const int T_ = a.T, C_ = a.C, N = a.T * a.C;
  const int b = blockIdx.y / a.Hkv, g = blockIdx.y % a.Hkv;
  const int grp = a.H / a.Hkv;
  const bool causal = a.flags & MVPA_FLAG_CAUSAL;
  const bool has_content = a.flags & MVPA_FLAG_CONTENT;
  const bool has_time = a.flags & MVPA_FLAG_TIME_BIAS;
  const bool has_chan = a.flags & MVPA_FLAG_CHAN_BIAS;

  const int nk_raw = blockIdx.x * BWD_THREADS + tid;
  const bool live = nk_raw < N;
  const int nk = live ? nk_raw : N - 1;
  const int tk = nk / C_, ck = nk % C_;
  const bool key_ok = !a.chan_valid || a.chan_valid[(int64_t)b * C_ + ck] != 0;
  const float kb = a.key_bias ? a.key_bias[(int64_t)b * N + nk] : 0.f;

  const T* krow = (const T*)a.k + b * a.k_stride_b + g * a.k_stride_h + (int64_t)nk * a.k_stride_n;
  const T* vrow = (const T*)a.v + b * a.v_stride_b + g * a.v_stride_h + (int64_t)nk * a.v_stride_n;
  const T* bu = (const T*)a.bias_u + g * DH;
  float kv[DH], vv[DH], dk[DH], dv[DH];
#pragma unroll
  for (int d = 0; d < DH; ++d) {
    kv[d] = io<T>::load(krow + d);
    vv[d] = io<T>::load(vrow + d);
    dk[d] = 0.f;
    dv[d] = 0.f;
  }

  // first query row that can see any key of this workgroup
  const int k_first = blockIdx.x * BWD_THREADS;
  const int lo = causal ? (k_first / C_) * C_ : 0;

  for (int hh = 0; hh < grp; ++hh) {
    const int h = g * grp + hh;
    const T* qbase = (const T*)a.q + b * a.q_stride_b + h * a.q_stride_h;
    const T* dbase = (const T*)a.d_o + b * a.do_stride_b + h * a.do_stride_h;
    const int64_t rbase = ((int64_t)b * a.H + h) * N;
    for (int q0 = lo; q0 < N; q0 += BWD_TILE) {
      __syncthreads();
      for (int i = tid; i < BWD_TILE * DH; i += BWD_THREADS) {
        const int qq = i / DH, d = i % DH;
        const int n = q0 + qq;
        float x = 0.f, y = 0.f;
        if (n < N) {
          x = io<T>::load(qbase + (int64_t)n * a.q_stride_n + d) + io<T>::load(bu + d);
          y = io<T>::load(dbase + (int64_t)n * a.do_stride_n + d);
        }
        Qs[i] = x;
        Ds[i] = y;
      }
      if (tid < BWD_TILE) {
        const int n = q0 + tid;
        Ls[tid] = n < N ? a.lse[rbase + n] : 0.f;
        Es[tid] = n < N ? a.ws_delta[rbase + n] : 0.f;
      }
      __syncthreads();
      for (int qq = 0; qq < BWD_TILE; ++qq) {
        const int n = q0 + qq;
        if (n >= N) break;
        const int tq = n / C_, cq = n - tq * C_;
        if (!(causal_visible(tq, tk, causal) && key_ok)) continue;
        const bool kept = has_content && content_kept(tq, tk, T_, a.window);
        const float* qr = Qs + qq * DH;
        const float* dr = Ds + qq * DH;
        float s = 0.f;
        if (has_time) s += a.ws_time[(rbase + n) * T_ + time_row(tq, tk, T_)];
        if (has_chan) s += a.ws_chan[(rbase + n) * C_ + chan_row(cq, ck, C_)];
        float dot = 0.f, dp = 0.f;
#pragma unroll
        for (int d = 0; d < DH; ++d) {
          dot += qr[d] * kv[d];
          dp += dr[d] * vv[d];
        }
        if (kept) s += dot;
        s = s * a.sm_scale + kb;
        const float p = exp2f(s * kLog2e - Ls[qq]);
        const float ds = p * (dp - Es[qq]) * a.sm_scale;
#pragma unroll
        for (int d = 0; d < DH; ++d) dv[d] += p * dr[d];
        if (kept) {
#pragma unroll
          for (int d = 0; d < DH; ++d) dk[d] += ds * qr[d];
        }
      }
    }
  }

  if (live) {
    const int64_t krow_o = (((int64_t)b * a.Hkv + g) * N + nk) * DH;
#pragma unroll
    for (int d = 0; d < DH; ++d) {
      a.dk[krow_o + d] = dk[d];
      a.dv[krow_o + d] = dv[d];
    }
  }
}

template <typename T, int DH>
static int launch_bwd_t(const mvpa_bwd_args* a, hipStream_t stream, bool query_pass) {
  const int N = a->T * a->C;
  const size_t lds_q = (size_t)(2 * BWD_TILE * DH + BWD_THREADS * (a->C + 1)) * sizeof(float);
  const size_t lds_k = (size_t)(2 * BWD_TILE * DH + 2 * BWD_TILE) * sizeof(float);
  if (lds_q > 160 * 1024) return MVPA_ERR_UNSUPPORTED;
  auto kq = mvpa_bwd_query_kernel<T, DH>;
  auto kk = mvpa_bwd_key_kernel<T, DH>;
  mvpa::want_dynamic_lds((const void*)kq, (int)lds_q);
  const unsigned nb = (unsigned)((N + BWD_THREADS - 1) / BWD_THREADS);
  if (query_pass) {
    MVPA_LAUNCH(kq, dim3(nb, a->B * a->H), dim3(BWD_THREADS), lds_q, stream, *a);
    if (mvpa::take_launch_status() != MVPA_OK) return MVPA_ERR_LAUNCH;
  }
  MVPA_LAUNCH(kk, dim3(nb, a->B * a->Hkv), dim3(BWD_THREADS), lds_k, stream, *a);
  return mvpa::take_launch_status();
}

template <typename T>
static int launch_bwd_dh(const mvpa_bwd_args* a, hipStream_t stream, bool query_pass) {
  switch (a->Dh) {
    case 16: return launch_bwd_t<T, 16>(a, stream, query_pass);
    case 32: return launch_bwd_t<T, 32>(a, stream, query_pass);
    case 64: return launch_bwd_t<T, 64>(a, stream, query_pass);
    case 128: return launch_bwd_t<T, 128>(a, stream, query_pass);
  }
  return MVPA_ERR_HEAD_DIM;
}

}  // namespace mvpa

extern "C" int mvpa_backward(const mvpa_bwd_args* a, void* stream) {
  if (!a) return MVPA_ERR_NULL;
  if (a->struct_size != sizeof(mvpa_bwd_args)) return MVPA_ERR_STRUCT;
  if (!a->q || !a->k || !a->v || !a->o || !a->d_o || !a->lse || !a->dq || !a->dk || !a->dv ||
      !a->dbias_time || !a->dbias_chan || !a->ws_delta || !a->ws_time || !a->ws_chan ||
      !a->bias_u || !a->bias_v || !a->bias_z || !a->k_time || !a->k_chan)
    return MVPA_ERR_NULL;
  if (a->Dh != 16 && a->Dh != 32 && a->Dh != 64 && a->Dh != 128) return MVPA_ERR_HEAD_DIM;
  if (a->H <= 0 || a->Hkv <= 0 || a->H % a->Hkv != 0) return MVPA_ERR_HEAD_RATIO;
  if (a->T <= 0 || a->C <= 0) return MVPA_ERR_CTX;
  if (a->B <= 0) return MVPA_ERR_SHAPE;
  if ((a->flags & (MVPA_FLAG_TIME_BIAS | MVPA_FLAG_CHAN_BIAS)) && !(a->flags & MVPA_FLAG_CAUSAL))
    return MVPA_ERR_NONCAUSAL_BIAS;
  if (a->dtype == MVPA_F32) return mvpa::launch_bwd_dh<float>(a, (hipStream_t)stream, true);
  if (a->dtype == MVPA_BF16) {
    // bf16, Dh = 64 or 128, C <= 128: both passes run on MFMA
    if (mvpa_bwd_query_mfma_supported(a)) return mvpa_launch_bwd_mfma(a, (hipStream_t)stream);
    return mvpa::launch_bwd_dh<mvpa::bf16_t>(a, (hipStream_t)stream, true);
  }
  return MVPA_ERR_DTYPE;
}
