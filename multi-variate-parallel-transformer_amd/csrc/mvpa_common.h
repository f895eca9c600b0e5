// Shared device/host helpers for the MVPA kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <tuple>
#include <unordered_map>
#include <utility>

#include "mvpa_hip.h"

namespace mvpa {

// ---- token index maps -------------------------------------------------------------------
// Token n of a sample is (t, c) = (n / C, n % C).  The reference obtains the two relative
// gathers with a pad-and-reshape shift (layers/mvpa.py:127-138) and an index matrix
// (layers/mvpa.py:140-159); both reduce to the closed forms below, which its fused kernel
// also uses (attentions/attn.py:279-308).

// Row of the time table [T, Dh] used by a query at time tq for a key at time tk <= tq.
__host__ __device__ inline int time_row(int tq, int tk, int T) { return T - 1 - (tq - tk); }

// Row of the channel table [C, Dh] used by query channel cq for key channel ck.
__host__ __device__ inline int chan_row(int cq, int ck, int C) {
  int d = cq - ck;
  return C - 1 - (d < 0 ? -d : d);
}

// Content term kept?  layers/mvpa.py:231-245: band |tq-tk| <= window, plus every key for the
// queries of the last time step.  window == 0 keeps the term everywhere.
__host__ __device__ inline bool content_kept(int tq, int tk, int T, int window) {
  int d = tq - tk;
  if (d < 0) d = -d;
  return window <= 0 || d <= window || tq == T - 1;
}

// Key visible under the time-causal mask (layers/mvpa.py:255-264)?
__host__ __device__ inline bool causal_visible(int tq, int tk, bool causal) {
  return !causal || tk <= tq;
}

// ---- bf16 <-> fp32 ----------------------------------------------------------------------
typedef uint16_t bf16_t;

__host__ __device__ inline float bf16_to_f32(bf16_t x) {
  union { uint32_t u; float f; } c;
  c.u = ((uint32_t)x) << 16;
  return c.f;
}

// round-to-nearest-even, NaN kept quiet
__host__ __device__ inline bf16_t f32_to_bf16(float f) {
  union { uint32_t u; float f; } c;
  c.f = f;
  uint32_t u = c.u;
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}

template <typename T> struct io;
template <> struct io<float> {
  __device__ static inline float load(const float* p) { return *p; }
  __device__ static inline void store(float* p, float v) { *p = v; }
};
template <> struct io<bf16_t> {
  __device__ static inline float load(const bf16_t* p) { return bf16_to_f32(*p); }
  __device__ static inline void store(bf16_t* p, float v) { *p = f32_to_bf16(v); }
};
typedef _Float16 f16_t;            // IEEE half as a storage type
template <> struct io<f16_t> {
  __device__ static inline float load(const f16_t* p) { return (float)*p; }
  __device__ static inline void store(f16_t* p, float v) { *p = (f16_t)v; }
};

constexpr float kLog2e = 1.4426950408889634f;

}  // namespace mvpa

// ---- launches ------------------------------------------------------------------------------
// A launch reports its OWN status: hipLaunchKernel's return value.  The runtime's global
// last-error slot is neither read nor cleared, so an error that unrelated earlier work of the
// host application left pending stays where that application will look for it.
namespace mvpa {

template <typename... KArgs, size_t... I>
inline hipError_t launch_impl(void (*kern)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t s,
                              std::tuple<KArgs...>& vals, std::index_sequence<I...>) {
  void* ptrs[] = {(void*)&std::get<I>(vals)..., nullptr};
  return hipLaunchKernel((const void*)kern, grid, block, ptrs, lds, s);
}

template <typename... KArgs, typename... Args>
inline hipError_t launch(void (*kern)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t s,
                         Args&&... args) {
  static_assert(sizeof...(KArgs) == sizeof...(Args), "kernel argument count");
  std::tuple<KArgs...> vals{static_cast<KArgs>(args)...};    // converted to the parameter types
  return launch_impl(kern, grid, block, lds, s, vals, std::index_sequence_for<KArgs...>{});
}

// Status of the launches this thread made since the last take_launch_status().
inline int& pending_launch_status() {
  static thread_local int st = MVPA_OK;
  return st;
}
inline void note_launch(hipError_t e) {
  if (e != hipSuccess) pending_launch_status() = MVPA_ERR_LAUNCH;
}
inline int take_launch_status() {
  const int st = pending_launch_status();
  pending_launch_status() = MVPA_OK;
  return st;
}

// hipFuncAttributeMaxDynamicSharedMemorySize, set once per (kernel, device) instead of on every
// launch: the call costs about as much as the launch itself on the decoding path.
inline void want_dynamic_lds(const void* kern, int bytes) {
  static std::mutex mu;
  static std::unordered_map<uint64_t, int> seen;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  const uint64_t key = (uint64_t)(uintptr_t)kern * 64u + (uint64_t)(dev & 63);
  {
    std::lock_guard<std::mutex> g(mu);
    auto it = seen.find(key);
    if (it != seen.end() && it->second >= bytes) return;
    seen[key] = bytes;
  }
  (void)hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

}  // namespace mvpa

#define MVPA_LAUNCH(...) mvpa::note_launch(mvpa::launch(__VA_ARGS__))

// ---- launchers implemented by the kernel translation units ----------------------------------
int mvpa_launch_generic(const mvpa_fwd_args* a, hipStream_t stream);
int mvpa_launch_mfma(const mvpa_fwd_args* a, hipStream_t stream);
// 1 if the tiled MFMA kernel can serve these (already validated) arguments
int mvpa_mfma_supported(const mvpa_fwd_args* a);
// the build of it in which a wave owns a whole time step (head size 64, 33..64 channels)
int mvpa_mfma64_supported(const mvpa_fwd_args* a);
int mvpa_launch_mfma64(const mvpa_fwd_args* a, hipStream_t stream);
int mvpa_mfma128_supported(const mvpa_fwd_args* a);
int mvpa_launch_mfma128(const mvpa_fwd_args* a, hipStream_t stream);
// backward, query pass on MFMA (bf16, Dh = 64, C <= 64)
int mvpa_bwd_query_mfma_supported(const mvpa_bwd_args* a);
int mvpa_launch_bwd_mfma(const mvpa_bwd_args* a, hipStream_t stream);
