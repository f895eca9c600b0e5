// Host side of the C ABI: argument validation, kernel selection, status strings.
// Nothing here touches device memory, so mvpa_validate / mvpa_select_kernel work on a machine
// without a GPU.
#include "mvpa_common.h"
#include "mvpa_mfma_tools.h"

extern "C" int mvpa_version(void) { return MVPA_ABI_VERSION; }

extern "C" const char* mvpa_error_string(int status) {
  switch (status) {
    case MVPA_OK: return "ok";
    case MVPA_ERR_NULL: return "required pointer is null";
    case MVPA_ERR_HEAD_DIM: return "head dim must be one of 16, 32, 64, 128";
    case MVPA_ERR_HEAD_RATIO: return "Q heads must be divisible by KV heads";
    case MVPA_ERR_CTX: return "time and channel context must be positive";
    case MVPA_ERR_SHAPE: return "bad shape (B, H must be positive; N must equal T*C)";
    case MVPA_ERR_DTYPE: return "unknown dtype or kernel selector";
    case MVPA_ERR_ALIGN: return "pointer or stride not aligned to 16 bytes";
    case MVPA_ERR_UNSUPPORTED: return "request not supported by the selected kernel";
    case MVPA_ERR_STRUCT: return "argument struct size does not match the library";
    case MVPA_ERR_LAUNCH: return "kernel launch failed";
    case MVPA_ERR_NONCAUSAL_BIAS: return "relative biases require the time-causal mask";
    case MVPA_ERR_WS_SIZE: return "request needs more workspace than the library's built-in array holds";
  }
  return "unknown status";
}

extern "C" int mvpa_validate(const mvpa_fwd_args* a) {
  if (!a) return MVPA_ERR_NULL;
  if (a->struct_size != sizeof(mvpa_fwd_args)) return MVPA_ERR_STRUCT;
  if (a->dtype != MVPA_F32 && a->dtype != MVPA_BF16 && a->dtype != MVPA_F16) return MVPA_ERR_DTYPE;
  if (a->kernel < MVPA_KERNEL_AUTO || a->kernel > MVPA_KERNEL_MFMA_SPLIT) return MVPA_ERR_DTYPE;
  if (a->Dh != 16 && a->Dh != 32 && a->Dh != 64 && a->Dh != 128) return MVPA_ERR_HEAD_DIM;
  if (a->B <= 0 || a->H <= 0 || a->Hkv <= 0) return MVPA_ERR_SHAPE;
  if (a->H % a->Hkv != 0) return MVPA_ERR_HEAD_RATIO;
  if (a->T <= 0 || a->C <= 0) return MVPA_ERR_CTX;
  if ((int64_t)a->T * a->C > (int64_t)1 << 24) return MVPA_ERR_SHAPE;
  if (a->window < 0) return MVPA_ERR_SHAPE;
  if (!a->q || !a->k || !a->v || !a->o) return MVPA_ERR_NULL;
  if (!a->bias_u || !a->bias_v || !a->bias_z || !a->k_time || !a->k_chan) return MVPA_ERR_NULL;
  if ((a->flags & (MVPA_FLAG_TIME_BIAS | MVPA_FLAG_CHAN_BIAS)) && !(a->flags & MVPA_FLAG_CAUSAL))
    return MVPA_ERR_NONCAUSAL_BIAS;
  if ((a->flags & MVPA_FLAG_LAST_STEP) && !(a->flags & MVPA_FLAG_CAUSAL)) return MVPA_ERR_UNSUPPORTED;
  const int64_t n = (int64_t)a->T * a->C;
  // a token stride smaller than Dh (or a head/batch stride of 0 with more than one head)
  // means the caller's N does not match T*C or the view is wrong
  if (a->q_stride_n < a->Dh || a->k_stride_n < a->Dh || a->v_stride_n < a->Dh ||
      a->o_stride_n < a->Dh)
    return MVPA_ERR_SHAPE;
  (void)n;
  if (a->flags & MVPA_FLAG_FP8_QK) {
    if (a->dtype != MVPA_BF16) return MVPA_ERR_UNSUPPORTED;
    if (!a->fp8_q_scale || !a->fp8_k_scale) return MVPA_ERR_NULL;
  }
  if (a->flags & MVPA_FLAG_RING) {
    if (!(a->flags & MVPA_FLAG_LAST_STEP)) return MVPA_ERR_UNSUPPORTED;
    if (!a->ring_head) return MVPA_ERR_NULL;
  }
  if (a->n_split < 0 || a->n_split > a->T) return MVPA_ERR_SHAPE;
  if (a->n_split > 1) {
    if (!(a->flags & MVPA_FLAG_LAST_STEP)) return MVPA_ERR_UNSUPPORTED;
    if (!a->split_ws) return MVPA_ERR_NULL;
    if ((uintptr_t)a->split_ws & 15) return MVPA_ERR_ALIGN;
    const int len = (a->T + a->n_split - 1) / a->n_split;
    if ((int64_t)(a->n_split - 1) * len >= a->T) return MVPA_ERR_SHAPE;   // an empty run
  }
  if (a->kernel == MVPA_KERNEL_MFMA_STEP && mvpa_mfma_supported(a) && !mvpa_mfma64_supported(a))
    return MVPA_ERR_UNSUPPORTED;
  if (a->kernel == MVPA_KERNEL_MFMA_SPLIT && mvpa_mfma_supported(a) && !mvpa_mfma128_supported(a))
    return MVPA_ERR_UNSUPPORTED;
  if (a->kernel >= MVPA_KERNEL_MFMA && !mvpa_mfma_supported(a)) {
    if (a->dtype == MVPA_BF16) {
      const uintptr_t p = (uintptr_t)a->q | (uintptr_t)a->k | (uintptr_t)a->v | (uintptr_t)a->o;
      const int64_t s = a->q_stride_b | a->q_stride_h | a->q_stride_n | a->k_stride_b |
                        a->k_stride_h | a->k_stride_n | a->v_stride_b | a->v_stride_h |
                        a->v_stride_n | a->o_stride_b | a->o_stride_h | a->o_stride_n;
      if ((p & 15) || (s & 7)) return MVPA_ERR_ALIGN;
    }
    return MVPA_ERR_UNSUPPORTED;
  }
  return MVPA_OK;
}

extern "C" size_t mvpa_split_ws_bytes(const mvpa_fwd_args* a) {
  if (!a || a->n_split <= 1) return 0;
  return (size_t)a->n_split * a->B * a->H * a->C * ((size_t)a->Dh * 2 + sizeof(float));
}

extern "C" int mvpa_debug_block_order(int32_t n_bh, int32_t n_tiles, int32_t heads_per_kv, int32_t* bh,
                                      int32_t* tile) {
  if (!bh || !tile) return MVPA_ERR_NULL;
  if (n_bh <= 0 || n_tiles <= 0 || heads_per_kv <= 0) return MVPA_ERR_SHAPE;
  for (int L = 0; L < n_bh * n_tiles; ++L) {
    int x, y;
    mvpa::map_block(L, n_bh, n_tiles, heads_per_kv, x, y);
    bh[L] = x;
    tile[L] = y;
  }
  return MVPA_OK;
}

extern "C" int mvpa_select_kernel(const mvpa_fwd_args* a) {
  const int st = mvpa_validate(a);
  if (st != MVPA_OK) return st;
  if (a->kernel == MVPA_KERNEL_GENERIC) return MVPA_KERNEL_GENERIC;
  if (a->kernel >= MVPA_KERNEL_MFMA) return MVPA_KERNEL_MFMA;
  return mvpa_mfma_supported(a) ? MVPA_KERNEL_MFMA : MVPA_KERNEL_GENERIC;
}

extern "C" int mvpa_forward(const mvpa_fwd_args* a, void* stream) {
  const int sel = mvpa_select_kernel(a);
  if (sel < 0) return sel;
  if (sel == MVPA_KERNEL_MFMA) {
    hipStream_t st = (hipStream_t)stream;
    if (a->kernel == MVPA_KERNEL_MFMA_STEP) return mvpa_launch_mfma64(a, st);
    if (a->kernel == MVPA_KERNEL_MFMA_SPLIT) return mvpa_launch_mfma128(a, st);
    if (a->kernel == MVPA_KERNEL_MFMA) return mvpa_launch_mfma(a, st);
    // AUTO: the specialised builds where they are the faster ones.
    // 65..128 channels at head size 64 or 128: the build of csrc/mvpa_mfma128.hip wins at every
    // length and channel count measured (Dh 128, B1 H16: C128 T 16 .. 1024 13 .. 20 % less time than
    // the general kernel, C 80 .. 100 21 .. 40 %; Dh 64, H16: B8 C117 T256 11.14 -> 8.58 ms,
    // B4 C128 T128 1.86 -> 1.34, B4 C80 T128 1.78 -> 1.21, B8 C128 T32 0.53 -> 0.38, B2 C128 T512
    // 9.99 -> 7.66 ms).
    if (mvpa_mfma128_supported(a) && a->C > 64) return mvpa_launch_mfma128(a, st);
    // The same build with two key tiles serves 33..64 channels: at head size 128 it wins too
    // (B1 H16 C64 T512 3.71 -> 2.87 ms, B4 C64 T64 0.42 -> 0.39); at head size 64 it loses to both
    // other builds (c2 0.49 against 0.40 and 0.38 ms: 8 products per wave and far step, one
    // workgroup per CU).
    if (mvpa_mfma128_supported(a) && a->Dh == 128) return mvpa_launch_mfma128(a, st);
    // Head size 64, 33..64 channels: the whole-time-step build pays for its window passes with a
    // cheaper far phase; against the general kernel it loses at 64 time steps (B4 H12 C64: 0.131
    // against 0.109 ms), is level at 128 and wins from there on (T 256: 6 %, T 512: 10 %), and
    // wins by 15 % when there are no window steps at all (content term off).
    if (mvpa_mfma64_supported(a) && (a->T >= 128 || !(a->flags & MVPA_FLAG_CONTENT))) return mvpa_launch_mfma64(a, st);
    return mvpa_launch_mfma(a, st);
  }
  if (a->flags & (MVPA_FLAG_FP8_QK | MVPA_FLAG_RING)) return MVPA_ERR_UNSUPPORTED;
  return mvpa_launch_generic(a, (hipStream_t)stream);
}
