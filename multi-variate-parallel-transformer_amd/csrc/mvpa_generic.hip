// Generic MVPA forward: one lane per query row, fp32 arithmetic throughout, any shape.
//
// This is the kernel behind the fp32 path (max-abs parity with the fp32 PyTorch MVPA,
// layers/mvpa.py:173-278) and behind every request the tiled bf16 MFMA kernel does not take
// (additive key bias, C > 128, content term without causal mask, ...).  It keeps the three
// score terms separate exactly as the reference sums them and uses expf, not a base-2
// shortcut, so that its rounding stays within a few ulp of torch.softmax.
//
// Work split: grid = (ceil(N/128), B*H); a workgroup owns 128 consecutive query tokens of one
// (b, h).  Key/value rows are staged through LDS 32 at a time as fp32 and broadcast to all
// lanes; the per-row channel table (q+z).e[j], j < C, is computed once into LDS.
#include "mvpa_common.h"

namespace mvpa {

constexpr int GEN_THREADS = 128;
constexpr int GEN_KT = 32;

template <typename T, int DH>
__global__ __launch_bounds__(GEN_THREADS) void mvpa_generic_kernel(mvpa_fwd_args a,
                                                                   int chan_table) {
  extern __shared__ float smem[];
  float* Ks = smem;                               // [KT][DH]
  float* Vs = Ks + GEN_KT * DH;                   // [KT][DH]
  float* Ss = Vs + GEN_KT * DH;                   // [KT][128] scores of the current tile
  float* Sc = Ss + GEN_KT * GEN_THREADS;          // [128][C+1] channel table (if chan_table)

  const int tid = threadIdx.x;
  const int T_ = a.T, C_ = a.C, N = a.T * a.C;
  const int b = blockIdx.y / a.H, h = blockIdx.y % a.H;
  const int g = h / (a.H / a.Hkv);
  const bool causal = a.flags & MVPA_FLAG_CAUSAL;
  const bool has_content = a.flags & MVPA_FLAG_CONTENT;
  const bool has_time = a.flags & MVPA_FLAG_TIME_BIAS;
  const bool has_chan = a.flags & MVPA_FLAG_CHAN_BIAS;

  // MVPA_FLAG_LAST_STEP: only the C queries of the last time step exist; rq is the row of q / o,
  // nq the query's place in the full sequence
  const bool last_only = a.flags & MVPA_FLAG_LAST_STEP;
  const int Nq = last_only ? C_ : N;
  const int nq_raw = blockIdx.x * GEN_THREADS + tid;
  const bool live = nq_raw < Nq;
  const int rq = live ? nq_raw : Nq - 1;          // clamp: dead lanes still take part in barriers
  const int nq = last_only ? (T_ - 1) * C_ + rq : rq;
  const int tq = nq / C_, cq = nq % C_;

  const T* qrow = (const T*)a.q + b * a.q_stride_b + h * a.q_stride_h + (int64_t)rq * a.q_stride_n;
  const T* kbase = (const T*)a.k + b * a.k_stride_b + g * a.k_stride_h;
  const T* vbase = (const T*)a.v + b * a.v_stride_b + g * a.v_stride_h;
  const T* bu = (const T*)a.bias_u + g * DH;
  const T* bv = (const T*)a.bias_v + g * DH;
  const T* bz = (const T*)a.bias_z + g * DH;
  const T* ktime = (const T*)a.k_time + (int64_t)g * T_ * DH;
  const T* kchan = (const T*)a.k_chan + (int64_t)g * C_ * DH;
  const uint8_t* valid = a.chan_valid ? a.chan_valid + (int64_t)b * C_ : nullptr;
  const float* kbias = a.key_bias ? a.key_bias + (int64_t)b * N : nullptr;

  float qu[DH];
#pragma unroll
  for (int d = 0; d < DH; ++d) qu[d] = io<T>::load(qrow + d) + io<T>::load(bu + d);

  // channel table: Sc[tid][j] = (q+z).e[j]
  const int sc_pitch = C_ + 1;
  if (has_chan && chan_table) {
    for (int j = 0; j < C_; ++j) {
      const T* e = kchan + (int64_t)j * DH;
      float s = 0.f;
#pragma unroll 8
      for (int d = 0; d < DH; ++d) s += (io<T>::load(qrow + d) + io<T>::load(bz + d)) * io<T>::load(e + d);
      Sc[tid * sc_pitch + j] = s;
    }
  }

  const int q_last = min(N - 1, (int)blockIdx.x * GEN_THREADS + GEN_THREADS - 1);
  const int hi = (causal && !last_only) ? (q_last / C_ + 1) * C_ : N;   // last step: every key

  float m = -INFINITY, l = 0.f;
  float acc[DH];
#pragma unroll
  for (int d = 0; d < DH; ++d) acc[d] = 0.f;
  int cur_tk = -1;
  float st = 0.f;

  for (int k0 = 0; k0 < hi; k0 += GEN_KT) {
    __syncthreads();
    for (int i = tid; i < GEN_KT * DH; i += GEN_THREADS) {
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

    float tmax = -INFINITY;
    for (int kk = 0; kk < GEN_KT; ++kk) {
      const int nk = k0 + kk;
      float x = -INFINITY;
      if (nk < hi) {
        const int tk = nk / C_, ck = nk - tk * C_;
        if (tk != cur_tk) {   // uniform across the workgroup: keys advance in lock step
          cur_tk = tk;
          st = 0.f;
          if (has_time && tk <= tq) {
            const T* r = ktime + (int64_t)time_row(tq, tk, T_) * DH;
#pragma unroll 8
            for (int d = 0; d < DH; ++d)
              st += (io<T>::load(qrow + d) + io<T>::load(bv + d)) * io<T>::load(r + d);
          }
        }
        const bool vis = causal_visible(tq, tk, causal) && (!valid || valid[ck] != 0);
        float sc = 0.f;
        if (has_chan) {
          const int j = chan_row(cq, ck, C_);
          if (chan_table) {
            sc = Sc[tid * sc_pitch + j];
          } else {
            const T* e = kchan + (int64_t)j * DH;
#pragma unroll 8
            for (int d = 0; d < DH; ++d)
              sc += (io<T>::load(qrow + d) + io<T>::load(bz + d)) * io<T>::load(e + d);
          }
        }
        float s = st + sc;
        const bool kept = has_content && content_kept(tq, tk, T_, a.window);
        if (__ballot(kept && vis) != 0ull) {   // wave-uniform skip of the content dot product
          float dot = 0.f;
          const float* kr = Ks + kk * DH;
#pragma unroll
          for (int d = 0; d < DH; ++d) dot += qu[d] * kr[d];
          if (kept) s += dot;
        }
        s *= a.sm_scale;
        if (kbias) s += kbias[nk];
        x = vis ? s : -INFINITY;
      }
      Ss[kk * GEN_THREADS + tid] = x;
      tmax = fmaxf(tmax, x);
    }

    const float m_new = fmaxf(m, tmax);
    if (m_new > -INFINITY) {
      const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
      l *= alpha;
#pragma unroll
      for (int d = 0; d < DH; ++d) acc[d] *= alpha;
      for (int kk = 0; kk < GEN_KT; ++kk) {
        const float x = Ss[kk * GEN_THREADS + tid];
        const float p = (x == -INFINITY) ? 0.f : expf(x - m_new);
        l += p;
        const float* vr = Vs + kk * DH;
#pragma unroll
        for (int d = 0; d < DH; ++d) acc[d] += p * vr[d];
      }
      m = m_new;
    }
  }

  if (live) {
    T* orow = (T*)a.o + b * a.o_stride_b + h * a.o_stride_h + (int64_t)rq * a.o_stride_n;
    const float inv = 1.f / l;
#pragma unroll
    for (int d = 0; d < DH; ++d) io<T>::store(orow + d, acc[d] * inv);
    if (a.lse) a.lse[((int64_t)b * a.H + h) * Nq + rq] = (m + logf(l)) * kLog2e;
  }
}

__global__ void mvpa_debug_maps_kernel(int T_, int C_, int window, unsigned flags,
                                       const uint8_t* valid, int32_t* time_idx,
                                       int32_t* chan_idx, uint8_t* mask_bits) {
  const int N = T_ * C_;
  const int nk = blockIdx.x * blockDim.x + threadIdx.x;
  const int nq = blockIdx.y;
  if (nk >= N) return;
  const int tq = nq / C_, cq = nq % C_, tk = nk / C_, ck = nk % C_;
  const bool causal = flags & MVPA_FLAG_CAUSAL;
  const bool vis = causal_visible(tq, tk, causal) && (!valid || valid[ck] != 0);
  const bool kept = (flags & MVPA_FLAG_CONTENT) && content_kept(tq, tk, T_, window);
  const int64_t i = (int64_t)nq * N + nk;
  time_idx[i] = tk <= tq ? time_row(tq, tk, T_) : -1;
  chan_idx[i] = chan_row(cq, ck, C_);
  mask_bits[i] = (uint8_t)((vis ? 1 : 0) | (kept ? 2 : 0));
}

template <typename T, int DH>
static int launch_generic_t(const mvpa_fwd_args* a, hipStream_t stream) {
  const int N = a->T * a->C;
  const size_t base = (size_t)(2 * GEN_KT * DH + GEN_KT * GEN_THREADS) * sizeof(float);
  const size_t table = (size_t)GEN_THREADS * (a->C + 1) * sizeof(float);
  const int chan_table = (base + table <= 150 * 1024) ? 1 : 0;
  const size_t lds = base + (chan_table ? table : 0);
  auto kern = mvpa_generic_kernel<T, DH>;
  mvpa::want_dynamic_lds((const void*)kern, (int)lds);
  const int n_rows = (a->flags & MVPA_FLAG_LAST_STEP) ? a->C : N;
  dim3 grid((n_rows + GEN_THREADS - 1) / GEN_THREADS, a->B * a->H);
  MVPA_LAUNCH(kern, grid, dim3(GEN_THREADS), lds, stream, *a, chan_table);
  return mvpa::take_launch_status();
}

template <typename T>
static int launch_generic_dh(const mvpa_fwd_args* a, hipStream_t stream) {
  switch (a->Dh) {
    case 16: return launch_generic_t<T, 16>(a, stream);
    case 32: return launch_generic_t<T, 32>(a, stream);
    case 64: return launch_generic_t<T, 64>(a, stream);
    case 128: return launch_generic_t<T, 128>(a, stream);
  }
  return MVPA_ERR_HEAD_DIM;
}

}  // namespace mvpa

int mvpa_launch_generic(const mvpa_fwd_args* a, hipStream_t stream) {
  if (a->dtype == MVPA_F32) return mvpa::launch_generic_dh<float>(a, stream);
  if (a->dtype == MVPA_BF16) return mvpa::launch_generic_dh<mvpa::bf16_t>(a, stream);
  if (a->dtype == MVPA_F16) return mvpa::launch_generic_dh<mvpa::f16_t>(a, stream);
  return MVPA_ERR_DTYPE;
}

extern "C" int mvpa_debug_maps(int32_t T, int32_t C, int32_t window, uint32_t flags,
                               const uint8_t* chan_valid, int32_t* time_idx, int32_t* chan_idx,
                               uint8_t* mask_bits, void* stream) {
  if (!time_idx || !chan_idx || !mask_bits) return MVPA_ERR_NULL;
  if (T <= 0 || C <= 0) return MVPA_ERR_CTX;
  const int N = T * C;
  dim3 grid((N + 255) / 256, N);
  MVPA_LAUNCH(mvpa::mvpa_debug_maps_kernel, grid, dim3(256), 0, (hipStream_t)stream, T, C,
                     window, flags, chan_valid, time_idx, chan_idx, mask_bits);
  return mvpa::take_launch_status();
}
