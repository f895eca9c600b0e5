// Device helpers shared by the tiled MFMA forward kernels (gfx950, wave64): vector types,
// LDS-direct tile loads, wait counters, fragment packing, the XOR swizzles of the K / V rows.
#pragma once

#include "mvpa_common.h"

namespace mvpa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define LDS_PTR(T) __attribute__((address_space(3))) T*
#define GLOBAL_PTR(T) __attribute__((address_space(1))) T*

__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

#define kOnes2 (bf16x2{(__bf16)1.0f, (__bf16)1.0f})
constexpr float kMFloor = -1.0e30f;     // "nothing seen yet" value of a running maximum

// order LDS traffic between the lanes of ONE wave (no workgroup barrier needed)
__device__ inline void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() would also drain every
// outstanding global load (vmcnt 0), which would serialise the tile prefetch ring.
__device__ inline void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// One 64-lane x 16-byte direct-to-LDS load: lane L's 16 bytes land at lds_base + 16*L.  Issued as
// inline assembly on purpose: the compiler then keeps no record of an LDS write in flight and
// does not drain the whole prefetch ring (vmcnt 0) in front of every later LDS read; completion
// is awaited explicitly with wait_vmcnt() before the barrier that publishes the tile.
__device__ inline void load_to_lds_16(const void* gptr, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :: "v"(gptr), "s"(lds_base) : "memory", "m0");
}

// The same load with the address split into a wave-uniform base (scalar registers) and a 32-bit
// byte offset per lane: one vector register per load instead of a 64-bit pair, and no 64-bit
// vector add per tile.
__device__ inline void load_to_lds_16(const void* sbase, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(sbase), "s"(lds_base) : "memory", "m0");
}

// The bare workgroup barrier: LDS reads of this wave may stay in flight across it.  For places
// where the barrier publishes tiles that arrived by direct-to-LDS loads (awaited with
// wait_vmcnt) and no wave's outstanding reads touch memory that is rewritten before they return.
__device__ inline void bare_barrier() {
  asm volatile("s_barrier" ::: "memory");
}

template <int N>
__device__ inline void wait_vmcnt_imm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// wait until at most n of this wave's vector-memory operations are outstanding
__device__ inline void wait_vmcnt(int n) {
  switch (n) {
    case 0: wait_vmcnt_imm<0>(); break;
    case 1: wait_vmcnt_imm<1>(); break;
    case 2: wait_vmcnt_imm<2>(); break;
    case 3: wait_vmcnt_imm<3>(); break;
    case 4: wait_vmcnt_imm<4>(); break;
    case 5: wait_vmcnt_imm<5>(); break;
    case 6: wait_vmcnt_imm<6>(); break;
    case 7: wait_vmcnt_imm<7>(); break;
    default: wait_vmcnt_imm<8>(); break;      // n >= 8: waiting for <= 8 is only stricter
  }
}

// max over a lane and its partner in the other half-wave (lane ^ 32): one register swap between
// the halves instead of a round trip through the LDS crossbar
__device__ inline float xhalf_max(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

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

// 8 floats -> 8 fp8 (e4m3) packed in 64 bits, the operand of the 32x32x16 fp8 MFMA
__device__ inline long pack_fp8(const float (&f)[8]) {
  int lo = 0, hi = 0;
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], lo, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], hi, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
  return (long)(((unsigned long)(unsigned)hi << 32) | (unsigned)lo);
}

// (q + bias) * scale as an fp8 fragment
__device__ inline long make_qfrag_fp8(u32x4 raw, const bf16_t* __restrict__ bias, float scale) {
  const u32x4 braw = *(const u32x4*)bias;
  float f[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t w = raw[i], bw = braw[i];
    f[2 * i] = (__uint_as_float(w << 16) + __uint_as_float(bw << 16)) * scale;
    f[2 * i + 1] = (__uint_as_float(w & 0xffff0000u) + __uint_as_float(bw & 0xffff0000u)) * scale;
  }
  return pack_fp8(f);
}

// a bf16 K fragment, scaled, as an fp8 fragment
__device__ inline long kfrag_fp8(u32x4 raw, float scale) {
  float f[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(raw[i] << 16) * scale;
    f[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u) * scale;
  }
  return pack_fp8(f);
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

// ---- element types of the general tiled kernel --------------------------------------------
// The 16-bit storage type of q, k, v, the tables and the output: what differs between bf16 and
// fp16 is the MFMA instruction, the conversions from and to fp32, and the pair-sum instruction.
// Pointers stay 2-byte element pointers (bf16_t) in either case.
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;

struct el_bf16 {
  using x8 = bf16x8;
  using x4 = bf16x4;
  using x2 = bf16x2;
  static __device__ inline f32x16 mfma(x8 a, x8 b, f32x16 c, int, int, int) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ inline x8 qfrag(u32x4 raw, const bf16_t* __restrict__ bias, float scale) { return make_qfrag(raw, bias, scale); }
  static __device__ inline x8 as8(u32x4 v) { return as_bf16x8(v); }
  static __device__ inline x8 pack(const f32x16& v, int base) { return pack8(v, base); }
  static __device__ inline float add_pair(x2 p, float acc) { return __builtin_amdgcn_fdot2_f32_bf16(p, kOnes2, acc, false); }
  static __device__ inline x4 read_tr(const unsigned char* p) { return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((LDS_PTR(bf16x4))p); }
  static __device__ inline __bf16 cvt(float f) { return (__bf16)f; }
};

struct el_f16 {
  using x8 = f16x8;
  using x4 = f16x4;
  using x2 = f16x2;
  static __device__ inline f32x16 mfma(x8 a, x8 b, f32x16 c, int, int, int) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  // 8 fp16 of a q row + bias, scaled, back to an fp16 fragment
  static __device__ inline x8 qfrag(u32x4 raw, const bf16_t* __restrict__ bias, float scale) {
    union { u32x4 u; x8 h; } r, b;
    r.u = raw;
    b.u = *(const u32x4*)bias;
    x8 out;
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = (_Float16)(((float)r.h[i] + (float)b.h[i]) * scale);
    return out;
  }
  static __device__ inline x8 as8(u32x4 v) {
    union { u32x4 u; x8 h; } c;
    c.u = v;
    return c.h;
  }
  static __device__ inline x8 pack(const f32x16& v, int base) {
    x8 out;
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = (_Float16)v[base + i];
    return out;
  }
  static __device__ inline float add_pair(x2 p, float acc) {
    return __builtin_amdgcn_fdot2(p, f16x2{(_Float16)1.0f, (_Float16)1.0f}, acc, false);
  }
  // the transposing read moves 16-bit units whatever they hold
  static __device__ inline x4 read_tr(const unsigned char* p) {
    union { bf16x4 b; x4 h; } c;
    c.b = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((LDS_PTR(bf16x4))p);
    return c.h;
  }
  static __device__ inline _Float16 cvt(float f) { return (_Float16)f; }
};

// XOR swizzles of the 16-byte chunk index within a K / V row, chosen so that the lanes that
// read LDS together (16 consecutive rows at one chunk for K; 4 consecutive rows x 4 chunks for
// the transposing V read) spread over all banks.
template <int DH> __device__ inline int swz_k(int row) {
  return DH == 64 ? ((row >> 1) & 7) : DH == 128 ? (row & 15) : ((row >> 2) & 3);
}
template <int DH> __device__ inline int swz_v(int row) {
  return DH == 64 ? (((row >> 1) & 1) << 2) : DH == 128 ? ((row & 3) << 2) : 0;
}

// ---- workgroup id -> ((b, h), time tile) ---------------------------------------------------
// Workgroup ids that are equal mod 8 run on one XCD and share its L2.  An XCD is given a
// contiguous range of (b, h) - with grouped-query attention the heads of one kv group are
// neighbours there, so the K/V of a kv head fill ONE L2, once - and walks it in this order:
//   * first the LAST time tile of every (b, h) it owns (the last time step keeps the content
//     term for every key step, layers/mvpa.py:244, and takes several times longer than any other
//     tile: it must not be what the grid ends on);
//   * then unit by unit, a unit being the heads of one kv group (one head without grouping),
//     late (= long) tiles first, the heads of the unit side by side on a tile so that they
//     stream the same K/V tiles at the same time;
//   * the last two units are interleaved tile by tile, so that the grid does not end on the long
//     tiles of a single unit.
// Without XCD affinity to keep (the (b, h) do not divide over 8 XCDs): last tiles first, then
// (b, h) by (b, h).
__host__ __device__ inline void map_block(int L, int nbh, int nt, int grp, int& bh, int& tile) {
  constexpr int TAIL_MERGE = 2;
  if (nt <= 1) {
    bh = L;
    tile = 0;
    return;
  }
  if ((nbh & 7) != 0) {
    if (L < nbh) {
      bh = L;
      tile = nt - 1;
    } else {
      bh = (L - nbh) / (nt - 1);
      tile = nt - 2 - (L - nbh) % (nt - 1);
    }
    return;
  }
  const int per_xcd = nbh >> 3;
  if (L < nbh) {
    bh = (L & 7) * per_xcd + (L >> 3);
    tile = nt - 1;
    return;
  }
  const int L2 = L - nbh;
  const int xcd = L2 & 7, s = L2 >> 3;
  const int u = (grp > 1 && per_xcd % grp == 0) ? grp : 1;      // heads per unit
  const int n_units = per_xcd / u, items = u * (nt - 1);
  const int merged = n_units < TAIL_MERGE ? n_units : TAIL_MERGE;
  const int plain = (n_units - merged) * items;
  int unit, i;
  if (s < plain) {
    unit = s / items;
    i = s % items;
  } else {
    const int r = s - plain;
    unit = n_units - merged + r % merged;
    i = r / merged;
  }
  bh = xcd * per_xcd + unit * u + i % u;
  tile = nt - 2 - i / u;
}

}  // namespace mvpa
