/*
 * C ABI of libmvpa_hip.so - MI355X (gfx950) kernels for MVPFormer's multi-variate
 * parallel attention (MVPA) forward and the dense ops around it.
 *
 * Every entry point takes plain pointers and sizes, returns an int status
 * (0 = MVPA_OK, negative = error, never throws or aborts), allocates nothing and keeps
 * no state between calls.  Device pointers are owned by the caller; kernels are
 * enqueued on the hipStream_t passed in (as an opaque void*) and the call returns
 * without synchronising.
 */
#ifndef MVPA_HIP_H
#define MVPA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MVPA_ABI_VERSION 3

/* ---- status codes ---------------------------------------------------------------- */
enum {
  MVPA_OK = 0,
  MVPA_ERR_NULL = -1,          /* a required pointer is null                             */
  MVPA_ERR_HEAD_DIM = -2,      /* Dh not in {16,32,64,128}   (attentions/attn.py:1041-1043) */
  MVPA_ERR_HEAD_RATIO = -3,    /* H % Hkv != 0               (attentions/attn.py:1044, 1339) */
  MVPA_ERR_CTX = -4,           /* T <= 0 or C <= 0           (attentions/attn.py:1045)      */
  MVPA_ERR_SHAPE = -5,         /* B/H <= 0, or N != T*C      (attentions/attn.py:1344)      */
  MVPA_ERR_DTYPE = -6,         /* unknown dtype / kernel selector                        */
  MVPA_ERR_ALIGN = -7,         /* pointer or stride not aligned for vector loads         */
  MVPA_ERR_UNSUPPORTED = -8,   /* valid request that the selected kernel cannot serve    */
  MVPA_ERR_STRUCT = -9,        /* struct_size does not match this library                */
  MVPA_ERR_LAUNCH = -10,       /* hipLaunchKernel reported an error                      */
  MVPA_ERR_NONCAUSAL_BIAS = -11, /* relative biases need the time-causal mask
                                   (attentions/attn.py:1335-1336)                        */
  MVPA_ERR_WS_SIZE = -12        /* the request needs more workspace than the library's
                                   built-in array holds (MVPA_STATIC_WS_BYTES)           */
};

/* ---- element types ----------------------------------------------------------------- */
enum {
  MVPA_F32 = 0,   /* fp32 in, fp32 math, fp32 out                                   */
  MVPA_BF16 = 1,  /* bf16 in/out, bf16 MFMA with fp32 accumulation                  */
  MVPA_F16 = 2    /* fp16 in/out, forward only: fp16 MFMA with fp32 accumulation on the general
                     tiled kernel (the shapes and alignment the bf16 MFMA kernel takes), fp32 math
                     on the row-per-lane kernel otherwise (the reference's kernel takes fp16 or
                     bf16, attentions/attn.py:1064-1066) */
};

/* ---- kernel selector --------------------------------------------------------------- */
enum {
  MVPA_KERNEL_AUTO = 0,     /* bf16: the fastest MFMA build that supports the shape (the general
                               tiled kernel or one of the two specialised builds below), the
                               fp32 kernel otherwise                                       */
  MVPA_KERNEL_GENERIC = 1,  /* fp32-math row-per-lane kernel, any shape                 */
  MVPA_KERNEL_MFMA = 2,     /* the general tiled bf16 MFMA kernel (a wave owns one tile of 32
                               queries and every output column), error if the shape is
                               unsupported                                                 */
  MVPA_KERNEL_MFMA_STEP = 3, /* the build in which a wave owns a whole time step (two tiles of
                               32 queries; head size 64, 33..64 channels, plain forward),
                               whatever the length; error if the shape is unsupported.  AUTO
                               picks it for 128 time steps and more or when the content term
                               is off, where it is the faster one.                         */
  MVPA_KERNEL_MFMA_SPLIT = 4 /* the build in which a wave owns 32 queries x 64 output columns
                               (33..128 channels, head size 64 or 128, plain forward, bf16 or
                               fp8 content term): at head size 128 the output columns of a
                               query tile are split over two waves, at head size 64 a
                               workgroup takes several time steps; error if the shape is
                               unsupported.  AUTO picks it for 65..128 channels, and for
                               33..64 channels at head size 128.                           */
};

/* ---- flags ------------------------------------------------------------------------- */
#define MVPA_FLAG_CAUSAL 1u     /* key time > query time is masked (layers/mvpa.py:255-264) */
#define MVPA_FLAG_CONTENT 2u    /* (q+u).k term present ("global_att", layers/mvpa.py:188)  */
#define MVPA_FLAG_TIME_BIAS 4u  /* (q+v).r[T-1-(tq-tk)]      (layers/mvpa.py:223,225)      */
#define MVPA_FLAG_CHAN_BIAS 8u  /* (q+z).e[C-1-|cq-ck|]      (layers/mvpa.py:224,226)      */
#define MVPA_FLAG_FP8_QK 16u    /* content term QK^T in fp8 e4m3 with per-head scales      */
#define MVPA_FLAG_LAST_STEP 32u /* q, o (and lse) hold only the C rows of the LAST time step,
                                   tq = T-1; k and v hold all T*C rows.  One step of incremental
                                   decoding against cached keys and values (the use the
                                   layer_past / use_cache arguments of layers/mvpa.py:314-321
                                   are for).  Needs MVPA_FLAG_CAUSAL.                        */
#define MVPA_FLAG_RING 64u      /* with MVPA_FLAG_LAST_STEP on the bf16 MFMA kernel: the T time
                                   steps of k and v are the slots of a ring; *ring_head (device
                                   memory, read by the kernel) is the slot of the newest step and
                                   slot s holds the step (ring_head - s) mod T steps older.  Lets
                                   a caller keep a sliding window of keys and values in place and
                                   replay one decoding step as a fixed sequence of launches.  */

/*
 * Arguments of the fused MVPA forward.  Replaces the pair
 *   attentions/attn.py:1305-1314 (_rel_bias: two matmuls into HBM tables) and
 *   attentions/attn.py:1064-1123 (the _fwd_kernel launch)
 * behind flash_mvpa (attentions/attn.py:1317-1366), and the whole of
 *   layers/mvpa.py:173-278 (_rel_attn) for the non-flash layer.
 *
 * Token n of a sample is (time t, channel c) with n = t*C + c.  q/o are indexed
 * [b][h][n][d], k/v [b][g][n][d] with g = h / (H/Hkv); strides are in ELEMENTS and the
 * d-stride is 1, so both the reference's contiguous [B,H,N,Dh] and a head-interleaved
 * [B,T,C,H,Dh] view can be passed without a copy.
 *
 *   score(nq,nk) = sm_scale * ( W(tq,tk) * (q+u).k  +  (q+v).r[T-1-(tq-tk)]
 *                               + (q+z).e[C-1-|cq-ck|] )  + key_bias[b][nk]
 *   W = 1 if window == 0, or |tq-tk| <= window, or tq == T-1; else 0 (term zeroed, not
 *   masked - layers/mvpa.py:231-245).  Keys with tk > tq and keys whose channel has
 *   chan_valid[b][ck] == 0 get probability exactly 0.
 */
typedef struct mvpa_fwd_args {
  uint32_t struct_size;   /* sizeof(mvpa_fwd_args)                                     */
  int32_t dtype;          /* MVPA_F32 | MVPA_BF16 | MVPA_F16                           */
  int32_t kernel;         /* MVPA_KERNEL_*                                             */
  uint32_t flags;         /* MVPA_FLAG_*                                               */
  int32_t B, H, Hkv, T, C, Dh;
  int32_t window;         /* 0 = content term everywhere                               */
  float sm_scale;         /* multiplies the sum of the three terms                     */
  const void* q;          /* [B,H,N,Dh]   */
  const void* k;          /* [B,Hkv,N,Dh] */
  const void* v;          /* [B,Hkv,N,Dh] */
  void* o;                /* [B,H,N,Dh]   */
  int64_t q_stride_b, q_stride_h, q_stride_n;
  int64_t k_stride_b, k_stride_h, k_stride_n;
  int64_t v_stride_b, v_stride_h, v_stride_n;
  int64_t o_stride_b, o_stride_h, o_stride_n;
  const void* bias_u;     /* [Hkv,Dh] content bias  (attn_bias[0:kvE])                 */
  const void* bias_v;     /* [Hkv,Dh] time bias     (attn_bias[kvE:2kvE])              */
  const void* bias_z;     /* [Hkv,Dh] channel bias  (attn_bias[2kvE:3kvE])             */
  const void* k_time;     /* [Hkv,T,Dh] position_net(positional_embedding)             */
  const void* k_chan;     /* [Hkv,C,Dh] channel_net(channel_embedding)                 */
  const uint8_t* chan_valid; /* nullable [B,C]; 0 = channel absent in this sample       */
  const float* key_bias;     /* nullable [B,N] additive, in score units (generic kernel) */
  float* lse;                /* nullable [B*H,N] base-2 log-sum-exp of the scores
                                (the reference's L, attentions/attn.py:327-333)         */
  const float* fp8_q_scale;  /* nullable [H]   per-head amax scales for MVPA_FLAG_FP8_QK */
  const float* fp8_k_scale;  /* nullable [Hkv]                                          */
  void* split_ws;            /* nullable; MVPA_FLAG_LAST_STEP on the bf16 MFMA kernel only: with
                                n_split > 1 the T key steps are cut into n_split runs, each run
                                goes to a workgroup of its own per (b, h) and the partial results
                                (soft-max over the run, its log-sum-exp) are merged by a second
                                small kernel.  Without it one workgroup per (b, h) walks the whole
                                cache.  Holds mvpa_split_ws_bytes(args) bytes, 16-byte aligned.
                                No counterpart in the reference (its cache path,
                                layers/mvpa.py:314-321, re-enters the full kernel).           */
  int32_t n_split;           /* 0 or 1 = no split; at most T                              */
  int32_t reserved0;
  const int32_t* ring_head;  /* MVPA_FLAG_RING: device pointer to the newest slot, in [0, T)  */
  const void* k_fp8;         /* nullable, MVPA_FLAG_FP8_QK: the keys already rounded to e4m3,
                                k / fp8_k_scale[g], contiguous [B,Hkv,N,Dh] bytes, 16-byte aligned
                                (mvpa_fp8_prepare writes it).  The column-split build
                                (MVPA_KERNEL_MFMA_SPLIT) streams these rows for its window steps
                                and needs them for the fp8 content term; the general kernel rounds
                                the bf16 keys itself and ignores the field.                      */
} mvpa_fwd_args;

/* ABI version of the loaded library. */
int mvpa_version(void);

/* Human-readable text for a status code (static storage). */
const char* mvpa_error_string(int status);

/* Host-only check of an argument block; touches no device memory and needs no GPU.
 * Mirrors the asserts of attentions/attn.py:1041-1045, 1339, 1344. */
int mvpa_validate(const mvpa_fwd_args* args);

/* What MVPA_FLAG_FP8_QK needs besides the tensors themselves, from q, k, bias_u, sm_scale, the
 * shapes and the strides of an argument block (its fp8_* and k_fp8 fields are not read):
 *   q_scale[h] = max |q + u| over the head's rows * sm_scale * log2(e) / 224   (>= 1e-20)
 *   k_scale[g] = max |k| over the kv head's rows / 224                          (>= 1e-20)
 *   k_fp8      = e4m3(k / k_scale[g]), contiguous [B,Hkv,N,Dh] bytes (nullable: scales only)
 * 224 keeps the largest magnitude inside the range of either e4m3 flavour.  With
 * MVPA_FLAG_LAST_STEP q holds C rows per head.  bf16 tensors; a handful of small launches on
 * `stream`, no allocation.  The reference has no fp8 path (attentions/attn.py:1064-1066 takes
 * fp16 or bf16). */
int mvpa_fp8_prepare(const mvpa_fwd_args* args, float* q_scale, float* k_scale, void* k_fp8, void* stream);

/* Bytes of mvpa_fwd_args.split_ws for args->n_split runs: n_split * B * H * C partial output
 * rows of Dh bf16 values followed by as many float log-sum-exps.  0 if n_split <= 1. */
size_t mvpa_split_ws_bytes(const mvpa_fwd_args* args);

/* Fused forward; replaces attentions/attn.py:1064-1123 + 1305-1314 and
 * layers/mvpa.py:173-278.  Validates, then enqueues on `stream`. */
int mvpa_forward(const mvpa_fwd_args* args, void* stream);

/*
 * The split decoding step of mvpa_forward (MVPA_FLAG_LAST_STEP, n_split > 1, bf16 matrix-core
 * kernel) on a workspace inside the library instead of args->split_ws, which is ignored.  No
 * counterpart in the reference: it is for callers that cannot allocate device memory - code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The entry point
 * allocates nothing and frees nothing; q, k, v, o (and lse) are still the caller's.  Same kernels,
 * same results as mvpa_forward with a caller workspace, bit for bit.
 *
 * The workspace is a device array of MVPA_STATIC_WS_BYTES that every GPU the library runs on
 * holds until the process ends.  Requests with mvpa_split_ws_bytes(args) above that return
 * MVPA_ERR_WS_SIZE (take fewer runs, or use mvpa_forward with a workspace of your own).  All calls
 * on one GPU share the array: calls that overlap in time on one GPU (different streams, different
 * threads) race on it and must be ordered by the caller; calls on different GPUs do not interact.
 */
#define MVPA_STATIC_WS_BYTES (16u << 20)
int mvpa_forward_last_step_static(const mvpa_fwd_args* args, void* stream);
size_t mvpa_static_ws_bytes(void);
/* Set-up for the entry point above, once per GPU with that GPU current and outside any stream
 * capture: resolves and keeps the array's address on that GPU, so that the first
 * mvpa_forward_last_step_static call may itself be recorded into a graph.  (A first call that
 * finds the address unresolved resolves it itself, which is a runtime query mid-capture.)
 * Returns MVPA_OK or MVPA_ERR_LAUNCH.  No counterpart in the reference. */
int mvpa_static_ws_init(void);

/* ---- backward ------------------------------------------------------------------------------
 * Argument block of mvpa_backward: the boundary of FlashMVPA.backward
 * (attentions/attn.py:1140-1302).  Inputs as in mvpa_fwd_args plus the forward output o, the
 * incoming gradient d_o and the forward's base-2 log-sum-exp.  Every gradient buffer and every
 * workspace but ws_qu is fp32; all are contiguous and caller-allocated; none needs to be cleared. */
typedef struct mvpa_bwd_args {
  uint32_t struct_size;      /* = sizeof(mvpa_bwd_args)                                       */
  int32_t dtype;             /* dtype of q, k, v, o, d_o, biases and tables                   */
  uint32_t flags;            /* MVPA_FLAG_CAUSAL | CONTENT | TIME_BIAS | CHAN_BIAS            */
  int32_t B, H, Hkv, T, C, Dh;
  int32_t window;
  float sm_scale;
  const void* q;             /* [B,H,N,Dh]-indexable, element strides below                   */
  const void* k;             /* [B,Hkv,N,Dh]                                                  */
  const void* v;
  const void* o;             /* forward output                                                */
  const void* d_o;           /* gradient of the loss with respect to o                        */
  int64_t q_stride_b, q_stride_h, q_stride_n;
  int64_t k_stride_b, k_stride_h, k_stride_n;
  int64_t v_stride_b, v_stride_h, v_stride_n;
  int64_t o_stride_b, o_stride_h, o_stride_n;
  int64_t do_stride_b, do_stride_h, do_stride_n;
  const void* bias_u;        /* [Hkv,Dh]                                                      */
  const void* bias_v;
  const void* bias_z;
  const void* k_time;        /* [Hkv,T,Dh]                                                    */
  const void* k_chan;        /* [Hkv,C,Dh]                                                    */
  const uint8_t* chan_valid; /* nullable [B,C]                                                */
  const float* key_bias;     /* nullable [B,N]                                                */
  const float* lse;          /* [B*H,N] from the forward                                      */
  float* dq;                 /* [B,H,N,Dh]   content-term share of dq (the reference's dq);
                                its sum over batch, group and rows is dq_bias               */
  float* dk;                 /* [B,Hkv,N,Dh] summed over the query heads of a group           */
  float* dv;                 /* [B,Hkv,N,Dh]                                                  */
  float* dbias_time;         /* [B,H,N,T] gradient of the table (q+v).k_time^T, by table column */
  float* dbias_chan;         /* [B,H,N,C] gradient of the table (q+z).k_chan^T, by table column */
  float* ws_delta;           /* workspace [B*H,N]      (contents after the call unspecified)  */
  float* ws_time;            /* workspace [B,H,N,T]                                           */
  float* ws_chan;            /* workspace [B,H,N,C rounded up to a multiple of 4]             */
  void* ws_qu;               /* nullable workspace [B,H,N,Dh] of `dtype`, 16-byte aligned; the
                                matrix-core kernels (bf16, Dh = 64 or 128, C <= 128, no key_bias)
                                run only when it is given                                     */
} mvpa_bwd_args;

/* Backward of the fused forward; replaces FlashMVPA.backward and its _bwd_kernel
 * (attentions/attn.py:350-1010, 1140-1302).  The gradients of q_btime, q_bchan, k_time and
 * k_chan, and the bias-term share of dq, follow from dbias_time / dbias_chan by the matrix
 * products that autograd applies to attentions/attn.py:1305-1314. */
int mvpa_backward(const mvpa_bwd_args* args, void* stream);

/* Which kernel mvpa_forward would run for these arguments: MVPA_KERNEL_GENERIC or
 * MVPA_KERNEL_MFMA (or a negative status). */
int mvpa_select_kernel(const mvpa_fwd_args* args);

/* Host-only: the order in which the matrix-core forward kernels hand their work out.  Workgroup L
 * of a launch with n_bh (batch, head) pairs and n_tiles time tiles each takes time tile tile[L] of
 * pair bh[L]; workgroups whose ids are equal mod 8 run on one XCD (one L2), and the map keeps the
 * heads of a kv group (heads_per_kv = H / Hkv neighbours in bh) on one XCD and side by side in
 * time.  The reference's grid is (query tiles, B*H) in plain order (attentions/attn.py:1048).
 * bh and tile hold n_bh * n_tiles entries.  Launches nothing. */
int mvpa_debug_block_order(int32_t n_bh, int32_t n_tiles, int32_t heads_per_kv, int32_t* bh, int32_t* tile);

/*
 * Index/mask maps exactly as the kernels compute them, for bit-exact tests against
 * layers/mvpa.py:127-159 (shifts) and :230-264 (window and causal masks).
 * For every (nq, nk) of one sample writes
 *   time_idx[nq*N+nk] = T-1-(tq-tk)  (or -1 when tk > tq),
 *   chan_idx[nq*N+nk] = C-1-|cq-ck|,
 *   mask_bits[nq*N+nk] = bit0 visible (causal & channel valid), bit1 content term kept.
 * chan_valid is nullable [C].
 */
int mvpa_debug_maps(int32_t T, int32_t C, int32_t window, uint32_t flags,
                    const uint8_t* chan_valid, int32_t* time_idx, int32_t* chan_idx,
                    uint8_t* mask_bits, void* stream);

/*
 * y[M,N] = x[M,K] @ w[N,K]^T  (torch.nn.functional.linear without bias), bf16 in/out,
 * fp32 accumulate on MFMA.  Replaces the Linear calls on the forward path:
 * models/fftencoder.py:95 (encoder proj), layers/mvpa.py:354-359, 400 (q_attn, c_attn,
 * position_net, channel_net, c_proj) and the MLP projections (models/mvpformer.py:146).
 * Row strides are in elements; K may be any positive value (tail is zero-padded
 * in-kernel).  epilogue: 0 none, 1 = y = silu(x@w_gate^T) * (x@w_up^T) where w holds
 * gate rows [0,N) and up rows [N,2N).
 */
int mvpa_linear_bf16(const void* x, const void* w, void* y, int64_t M, int64_t N, int64_t K,
                     int64_t ldx, int64_t ldw, int64_t ldy, int32_t epilogue, void* stream);

/* y[M,N] = x[M,K] @ w[N,K]^T + r[M,N]: the product with the residual rows added in its epilogue
 * (the sum is rounded to bf16 once more after the add).  With x = [attention output | MLP
 * activations] side by side and w = [c_proj | down_proj] it is the whole tail of the parallel
 * block, hidden + attn + mlp (layers/mvpa.py:400, models/mvpformer.py:146-147), in one kernel.
 * Large shapes only: M >= 512, K a multiple of 32 and >= 96; MVPA_ERR_UNSUPPORTED otherwise.
 * y may be r (in place).  ldr is r's row pitch in elements. */
int mvpa_linear_bf16_residual(const void* x, const void* w, const void* r, void* y, int64_t M,
                              int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldr,
                              int64_t ldy, void* stream);

/* The same product in fp32 (fp32 in and out, fp32 MFMA): the projections of the fp32 layer path
 * (layers/mvpa.py:303-313, 336 on fp32 tensors - the small plumbing configuration).  Any positive
 * M, N, K; row strides in elements. */
int mvpa_linear_f32(const float* x, const float* w, float* y, int64_t M, int64_t N, int64_t K,
                    int64_t ldx, int64_t ldw, int64_t ldy, void* stream);

/* Two products on one x in one launch: y0[M,N0] = x @ w0^T and y1[M,N1] = silu(x @ wg^T) * (x @ wu^T)
 * with w1 holding the gate rows [0,N1) and the up rows [N1,2*N1) - the fused q/kv projection
 * (layers/mvpa.py:354-356) and the MLP's gate/up product (models/mvpformer.py:146), which both read
 * ln_1(x) in the parallel block.  Launched separately each product ends on a partly filled round
 * of tiles; in one grid only their sum does.  Large shapes only: M >= 512, K a multiple of 64 and
 * at least 128 (two k-blocks: the kernel's two-stage pipeline); MVPA_ERR_UNSUPPORTED otherwise. */
int mvpa_linear_bf16_dual(const void* x, const void* w0, void* y0, const void* w1, void* y1, int64_t M,
                          int64_t N0, int64_t N1, int64_t K, int64_t ldx, int64_t ldw0, int64_t ldy0,
                          int64_t ldw1, int64_t ldy1, void* stream);

/* RMSNorm between two products without a pass of its own (models/mvpformer.py:133: ln_1 in front
 * of the block's projections; :146-147: its input is the sum the previous block's tail product
 * wrote).  The producer writes, beside its rows, their partial sums of squares; the consumer reads
 * the RAW rows, multiplies them with weights whose columns already carry the norm's weight
 * (w[n][k] * ln[k], folded by the caller), and scales every output row by
 * rsqrt(sum of the row's partial sums / K + eps) while it converts it - before the SiLU gate.
 *   mvpa_linear_sumsq_parts(M, N)      host-only: partial sums per row that the residual product
 *                                      writes for an [M, N] output (two per column tile)
 *   mvpa_linear_bf16_residual_sumsq    mvpa_linear_bf16_residual that also writes
 *                                      sumsq[M][parts] (fp32; sums over the final bf16 values);
 *                                      pair-kernel shapes: M >= 512, K a multiple of 64 and >= 128,
 *                                      N a multiple of 8, y and r 16-byte aligned with row strides
 *                                      that are multiples of 8
 *   mvpa_row_sumsq_bf16                sumsq[rows] of plain bf16 rows (parts = 1): the statistics
 *                                      of the first block's input
 *   mvpa_linear_bf16_dual_normed       mvpa_linear_bf16_dual on raw rows x with sumsq[M][parts] */
int32_t mvpa_linear_sumsq_parts(int64_t M, int64_t N);
int mvpa_linear_bf16_residual_sumsq(const void* x, const void* w, const void* r, void* y, float* sumsq, int64_t M,
                                    int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldr, int64_t ldy,
                                    void* stream);
int mvpa_row_sumsq_bf16(const void* x, float* sumsq, int64_t rows, int32_t cols, int64_t ldx, void* stream);
int mvpa_linear_bf16_dual_normed(const void* x, const void* w0, void* y0, const void* w1, void* y1, int64_t M,
                                 int64_t N0, int64_t N1, int64_t K, int64_t ldx, int64_t ldw0, int64_t ldy0,
                                 int64_t ldw1, int64_t ldy1, const float* sumsq, int32_t parts, float eps,
                                 void* stream);

/* The same product for at most 128 rows of x against a large weight (the projections of one
 * decoding step of a wide model), with K split over workgroups: fp32 partial tiles go through the
 * caller's workspace ws (mvpa_linear_splitk_ws_bytes(M, N, K, epilogue) bytes, 16-byte aligned)
 * and a second kernel sums them and applies the epilogue.  Same arguments and results (to fp32
 * summation order) as mvpa_linear_bf16. */
int mvpa_linear_bf16_splitk(const void* x, const void* w, void* y, int64_t M, int64_t N, int64_t K,
                            int64_t ldx, int64_t ldw, int64_t ldy, int32_t epilogue, void* ws,
                            size_t ws_bytes, void* stream);
size_t mvpa_linear_splitk_ws_bytes(int64_t M, int64_t N, int64_t K, int32_t epilogue);

/* RMSNorm over the last dim: y = x * rsqrt(mean(x^2)+eps) * weight
 * (models/mvpformer.py:108,133,167,380; models/fftencoder.py:67,93).
 * in_dtype/out_dtype: MVPA_F32 | MVPA_BF16; weight is fp32; ldx/ldy are row pitches in
 * elements (>= cols). */
int mvpa_rmsnorm(const void* x, const float* weight, void* y, int64_t rows, int32_t cols,
                 int64_t ldx, int64_t ldy, float eps, int32_t in_dtype, int32_t out_dtype,
                 void* stream);

/* Cosine similarity of row pairs in fp32: out[g * rows_per_group + r] = a_gr . b_gr /
 * (max(|a_gr|, eps) * max(|b_gr|, eps)) with a_gr = a + g * group_stride_a + r * lda (elements;
 * cols a multiple of 8, 16-byte aligned rows).  The generative score of the reference,
 * torch.cosine_similarity(next segment's encoding, head's prediction, dim=-1)
 * (models/mvpformer.py:749-764), in one pass over both tensors: a group is one batch entry, its
 * rows "all time steps but the first" of one tensor against "all but the last" of the other. */
int mvpa_cosine_rows_bf16(const void* a, const void* b, float* out, int64_t groups,
                          int64_t rows_per_group, int32_t cols, int64_t lda, int64_t ldb,
                          int64_t group_stride_a, int64_t group_stride_b, float eps, void* stream);

/* out = a + b + c elementwise, bf16 (models/mvpformer.py:147 residual + mlp + attn). */
int mvpa_add3_bf16(const void* a, const void* b, const void* c, void* out, int64_t n,
                   void* stream);

/* sum = a + b + c (bf16, one rounding) and norm = RMSNorm(sum) * weight in one pass: the residual
 * update of a block (models/mvpformer.py:147) fused with the input norm of the next block
 * (models/mvpformer.py:133) or with ln_f (models/mvpformer.py:380).  Rows are contiguous
 * ([rows, cols]); cols % 8 == 0 and 16-byte aligned pointers, else MVPA_ERR_ALIGN.  The norm is
 * taken over the rounded sum: identical to mvpa_add3_bf16 followed by mvpa_rmsnorm. */
int mvpa_add3_rmsnorm_bf16(const void* a, const void* b, const void* c, const float* weight,
                           void* sum, void* norm, int64_t rows, int32_t cols, float eps,
                           void* stream);

/* Multilevel db4 analysis with periodic extension of fp32 rows x[M,L] into
 * coeffs[M,dwt_size] (row pitch ldc >= dwt_size) ordered [cA_L, cD_L, ..., cD_1]
 * (models/fftencoder.py:80-88). */
int mvpa_wavedec_db4(const float* x, float* coeffs, int64_t M, int32_t L, int32_t levels,
                     int32_t dwt_size, int64_t ldc, void* stream);

/* One new time step of keys and values ([B,Hkv,C,Dh] views with element strides
 * stride_b/h/c and unit last stride, e.g. slices of the fused projection output) into slot *head
 * (device memory) of the ring buffers [B,Hkv,steps,C,Dh] that MVPA_FLAG_RING reads: the in-place
 * form of the cache concatenation of layers/mvpa.py:314-317, both tensors in one launch. */
int mvpa_ring_append_bf16(const void* k_new, const void* v_new, void* k_ring, void* v_ring,
                          const int32_t* head, int32_t B, int32_t Hkv, int32_t C, int32_t Dh,
                          int32_t steps, int64_t stride_b, int64_t stride_h, int64_t stride_c,
                          void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MVPA_HIP_H */
