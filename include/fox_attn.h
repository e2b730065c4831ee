/*
 * fox_attn.h -- flat C ABI of libfox_attn.so: Forgetting Attention for AMD gfx950.
 *
 * Every function takes raw device pointers, element strides and a HIP stream
 * (passed as void*), launches on that stream without synchronising, allocates
 * nothing and returns 0 on success or a negative FOX_E_* code; fox_last_error()
 * gives the message of the calling thread's last failure.  The caller owns all
 * buffers.  Citations name the interface of the reference implementation
 * (src/forgetting_transformer/ops/forgetting_attention.py) that each entry point
 * replaces.
 *
 * Tensors q, k, v, o, do, dq, dk, dv are 16-bit (bf16 or fp16) with logical shape
 * (B, H, T, D), arbitrary element strides for B, H, T, unit stride for D; base
 * pointers must be 16-byte aligned and strides multiples of 8 elements.
 * D is one of 16, 32, 64, 128.  M = query length, N = key length, M <= N; query
 * row i sits at key position i + (N - M).
 */
#ifndef FOX_ATTN_H
#define FOX_ATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FOX_OK 0
#define FOX_E_ARG (-1)     /* null pointer, bad size, unsupported head dim / dtype */
#define FOX_E_ALIGN (-2)   /* pointer or stride alignment */
#define FOX_E_LAUNCH (-3)  /* HIP reported a launch failure */

#define FOX_DTYPE_BF16 0
#define FOX_DTYPE_FP16 1
#define FOX_DTYPE_FP32 2   /* gate logits only */

/* A (B, H, T, D) tensor view: element strides of the first three axes. */
typedef struct fox_view {
  void* ptr;
  int64_t stride_b, stride_h, stride_t;
} fox_view;

typedef struct fox_dims {
  int32_t B, H, M, N, D;
  int32_t dtype; /* FOX_DTYPE_* */
} fox_dims;

/* Library version (major*10000 + minor*100 + patch). */
int fox_version(void);
const char* fox_last_error(void);

/*
 * Tile sizes the kernels use for a head dim: block_m/block_n of the forward and
 * dQ kernels (pruning bounds are multiples of block_n per block_m query rows),
 * and kv_block_n/kv_block_m of the dK/dV kernel.
 * Replaces get_fwd_config / get_bwd_kv_config / get_bwd_q_config (:460-493, :838-890).
 */
int fox_tile_config(int32_t D, int32_t* block_m, int32_t* block_n, int32_t* kv_block_n, int32_t* kv_block_m);

/*
 * No counterpart in the reference; a measuring stick for benchmarks.  Launches `workgroups` workgroups of four
 * waves that do nothing but 32x32x16 bf16 MFMAs on operands held in registers (32 per iteration and wave, `iters`
 * iterations: workgroups * 4 * iters * 32 * 32768 flop).  `operands` is 16 KiB of device memory holding any 16-bit
 * values (what the matrix pipe is fed with: on N(0,1) data the power limit of the socket, not the instruction
 * stream, sets the rate); `sink` is one float of device memory that is never written in practice.  workgroups in [1, 65536], iters in
 * [1, 2^20] (about half a second per launch at most).
 */
int fox_probe_mfma(const void* operands, float* sink, int32_t workgroups, int32_t iters, void* stream);

/*
 * Under pruning the dK/dV pass is served by two kernels: 128-key tiles whose pruning bound lies within `keys`
 * positions of their diagonal (a few query steps: a short chain of loads and stores) go to a variant that
 * splits the head dim over two waves and runs two workgroups per CU, the others to the kernel built for long
 * loops.  This sets `keys` (256 by default, the measured crossover) for all later calls of the process and returns the previous value: 0 = the long-loop
 * kernel only, negative = the split variant for every tile of every call it supports (head dim 128), with or
 * without a threshold.  The results obey the same contract either way.  Like the reference's tile pickers,
 * which "can be overwritten at runtime" (get_bwd_kv_config, :838).
 */
int32_t fox_set_acp_light_limit(int32_t keys);

/*
 * No counterpart in the reference.  A forward whose (batch, head) pairs have a single query tile (chunked prefill,
 * short query blocks against a long cache) reads every K and V tile exactly once; from `bytes` of K and V together
 * on (512 MiB by default) it loads them with the non-temporal hint, which is worth 8-12 % on a stream from HBM and
 * costs 5-14 % on tensors small enough to stay in the last-level cache between calls.  Sets the limit for all
 * later calls of the process and returns the previous value; 0 = always, INT64_MAX = never.  Results are bit for
 * bit the same either way.
 */
int64_t fox_set_stream_min_kv_bytes(int64_t bytes);

/*
 * c[b,h,n] = sum_{l<=n} g[b,h,l] with g[b,h,l] taken as 0 for l < seq_start[b].
 * g is fp32 with element strides (g_sb, g_sh, g_sn); c is (B,H,N) contiguous fp32.
 * seq_start may be NULL.  Replaces the prologue at :117-127 (clone, masked zero
 * fill, torch.cumsum).
 */
int fox_cumsum_fwd(const float* g, int64_t g_sb, int64_t g_sh, int64_t g_sn, const int64_t* seq_start, float* c,
                   int32_t B, int32_t H, int32_t N, void* stream);

/*
 * dg[b,h,l] = sum_{n>=l} dc[b,h,n]; dc is (B,H,N) contiguous fp32, dg is fp32 with element strides
 * (dg_sb, dg_sh, dg_sn) -- the layout of the caller's log_fgate, so that autograd can take the gradient as it
 * is -- or (B,H,N) contiguous when all three strides are 0.  Replaces the reverse cumulative sum at :390-392.
 * Positions l <= seq_start[b] (l = 0 when seq_start is NULL) get an exact 0: their gradient is the sum of all dc,
 * which vanishes in exact arithmetic (the reference returns the rounding noise of that sum).
 */
int fox_cumsum_bwd(const float* dc, float* dg, int64_t dg_sb, int64_t dg_sh, int64_t dg_sn, const int64_t* seq_start,
                   int32_t B, int32_t H, int32_t N, void* stream);

/*
 * The prologue of the FoX layer fused with the scan: c[b,h,n] = sum_{seq_start[b] <= l <= n} logsigmoid(x[b,h,l])
 * from the gate logits x (dtype FOX_DTYPE_BF16 / FP16 / FP32, element strides (sb, sh, sn)), evaluated in fp32.
 * Replaces logsigmoid(fgate_logit.float()) of the layer (model/forgetting_transformer/
 * modeling_forgetting_transformer.py:343-346) followed by the operator's prologue (:117-127).  log_fgate, if
 * not NULL, receives logsigmoid(x) as (B,H,N) contiguous fp32 (the layer's decode cache stores it,
 * modeling_forgetting_transformer.py:356-357).
 */
int fox_gate_cumsum_fwd(const void* logits, int32_t logits_dtype, int64_t sb, int64_t sh, int64_t sn,
                        const int64_t* seq_start, float* log_fgate, float* c, int32_t B, int32_t H, int32_t N, void* stream);

/*
 * dlogits[b,h,l] = (sum_{n>=l} dc[b,h,n]) * (1 - sigmoid(x[b,h,l])): the reverse cumulative sum (:390-392)
 * fused with the derivative of logsigmoid; dlogits has the dtype of the logits and its own element strides.
 * Positions l <= seq_start[b] (l = 0 when seq_start is NULL) get an exact 0, as in fox_cumsum_bwd.
 */
int fox_gate_cumsum_bwd(const float* dc, const void* logits, int32_t logits_dtype, int64_t sb, int64_t sh, int64_t sn,
                        const int64_t* seq_start, void* dlogits, int64_t db, int64_t dh, int64_t dn, int32_t B, int32_t H,
                        int32_t N, void* stream);

/*
 * thr[b,h] = -(2 * max_m|q| * max_n|k| * sm_scale + log N) - 10, with the row norms
 * and every intermediate rounded to the input dtype as the reference's tensor
 * arithmetic does (:95-102).  thr is (B,H) contiguous fp32; scratch is 3*B*H
 * uint32 that this call overwrites (it needs no initialisation).
 */
int fox_auto_threshold(const fox_dims* dims, const fox_view* q, const fox_view* k, float sm_scale, float* thr,
                       uint32_t* scratch, void* stream);

typedef struct fox_fwd_args {
  fox_dims dims;
  fox_view q, k, v, o;        /* o is written */
  const float* log_lambda;    /* (B,H,N) contiguous, from fox_cumsum_fwd */
  float* lse;                 /* (B,H,M) contiguous, written: log of the softmax normaliser, -inf for empty rows */
  const int64_t* seq_start;   /* (B,) or NULL */
  const float* threshold;     /* (B,H) contiguous or NULL (no pruning) */
  float sm_scale;
  int32_t* first_block;       /* optional (B,H,ceil(M/block_m)): first key block each query block visits */
  void* workspace;            /* optional scratch of fox_attn_fwd_workspace_bytes() bytes, 16-byte aligned; NULL = never split keys */
  int64_t workspace_bytes;    /* size of workspace; too small a workspace is an error */
} fox_fwd_args;

/*
 * Forward: o = softmax(q k^T sm_scale + c_i - c_j over seq_start <= j <= i+N-M) v.
 * Replaces _find_start_index_kernel (:695-745) + _fwd_kernel (:505-693) as launched
 * by ForgettingAttention.forward (:159-204).  M == 1 (one new token against the cache) takes a
 * dot-free streaming kernel, like the reference's BLOCK_M = 1 case (:148-153, :637-641, :665-668).
 */
int fox_attn_fwd(const fox_fwd_args* args, void* stream);

/*
 * Scratch the forward can use to split the key loop of each query tile over several
 * workgroups (flash-decoding style partial (max, sum, accumulator) + combine).  Shapes with
 * few query tiles and long key sequences -- chunked prefill, decode (the reference's
 * M == 1 path, :148-153) -- otherwise leave most of the chip idle.  *bytes is 0 when the
 * shape is not split.  No counterpart in the reference, which always runs one program per
 * query tile (:186).
 */
int fox_attn_fwd_workspace_bytes(const fox_dims* dims, int64_t* bytes);

/*
 * fox_attn_fwd for callers that cannot allocate device memory or bring a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same
 * arguments and results as fox_attn_fwd (bit for bit), except that args->workspace / workspace_bytes are
 * ignored: the partial results of a key-split forward go to a 64 MiB array that lives inside the library
 * (one copy per GPU, held until the process ends).  The call allocates nothing.  A shape whose splits need
 * more than 64 MiB (fox_attn_fwd_workspace_bytes) is rejected with FOX_E_ARG; shapes that are not split
 * never touch the array.  The device that owns `stream` must be the current device.  All calls on one GPU
 * share that GPU's array: calls that may overlap in time on one GPU (different streams, or graphs replayed
 * concurrently) race on it; calls ordered on one stream do not.  Every element a call reads it has written
 * before, so nothing needs clearing between calls.
 */
int fox_attn_fwd_noalloc(const fox_fwd_args* args, void* stream);

typedef struct fox_bwd_args {
  fox_dims dims;
  fox_view q, k, v, o, d_o;   /* inputs */
  fox_view dq, dk, dv;        /* written */
  const float* log_lambda;    /* (B,H,N) */
  const float* lse;           /* (B,H,M) from the forward */
  const int64_t* seq_start;   /* (B,) or NULL */
  const float* threshold;     /* (B,H) or NULL */
  float sm_scale;
  float* delta;               /* (B,H,M) workspace, written by the dQ stage: rowsum(o * do) */
  float* drow;                /* (B,H,M) workspace, written by the dQ stage, read by the dK/dV stage: row sums of dS */
  float* dlog_lambda;         /* (B,H,N) workspace, written: gradient w.r.t. c */
  float* dlog_fgate;          /* (B,H,N) written: gradient w.r.t. log_fgate */
  int64_t dlog_fgate_stride_b, dlog_fgate_stride_h, dlog_fgate_stride_n;  /* its element strides; all 0 = contiguous */
  /* Optional outputs (NULL = not wanted): the pruning bounds the two kernels worked with, the counterparts of
   * fox_fwd_args.first_block for the results of _find_start_index_kernel (:695-745, as the dQ kernel uses them,
   * :1239-1261) and _find_end_index_kernel (:747-795, as the dK/dV kernel uses them, :1038-1049). */
  int32_t* q_first_block;     /* (B,H,ceil(M/block_m)), written by fox_attn_bwd_dq: first key block (of block_n keys) each
                                 query block visits, left padding included */
  int32_t* kv_end_row;        /* (B,H,ceil(N/64)), written by fox_attn_bwd_dkdv: for every 64 keys, the query row at which
                                 the walk over the query blocks below them stops (M = nothing pruned; the first row of the
                                 walk = nothing visited).  A key tile is kv_block_n keys walked in steps of kv_block_m rows,
                                 or, for the tiles fox_set_acp_light_limit hands to the split variant, 64 keys in steps of 64 */
} fox_bwd_args;

/*
 * The stages of the backward pass, in the order they must run on a stream:
 *   fox_attn_bwd_dq    : dq; delta = rowsum(o * do) and drow[i] = sum_j dS[i,j]
 *                        (_bwd_preprocess :902-943 + _find_start_index_kernel + _bwd_q_kernel :1156-1344)
 *   fox_attn_bwd_dkdv  : dk, dv, dlog_lambda[n] = drow[n-(N-M)] - sum_i dS[i,n]; reads delta and drow
 *                        (_find_end_index_kernel :747-795 + _bwd_kv_kernel :956-1143)
 *   fox_cumsum_bwd     : dlog_fgate from dlog_lambda                (:390-392)
 * fox_attn_bwd runs all three (ForgettingAttention.backward :232-400).  The reference launches the key/value
 * kernel first and lets the query kernel add its row sums into the same buffer (:1334-1344); here every stage
 * only stores, so repeating a stage (or timing it alone) leaves the result unchanged, and only the order
 * dq before dkdv matters.  fox_attn_bwd_delta writes `delta` alone (_bwd_preprocess as a stage of its own; only
 * dims, o, d_o and delta are read from the argument block); the backward does not need it.
 */
int fox_attn_bwd_delta(const fox_bwd_args* args, void* stream);
int fox_attn_bwd_dkdv(const fox_bwd_args* args, void* stream);
int fox_attn_bwd_dq(const fox_bwd_args* args, void* stream);
int fox_attn_bwd(const fox_bwd_args* args, void* stream);

/*
 * Token shift, the data-dependent mix of every key / value row with its predecessor that the FoX
 * layer applies in front of the attention (ShiftLinear, model/forgetting_transformer/
 * modeling_forgetting_transformer.py:68-95).  x, out, dout, dx are 16-bit (B, T, H, D) tensors that
 * share one set of element strides (unit stride for D, 16-byte aligned, strides multiples of 8);
 * prev_weight, curr_weight and their gradients are fp32 (B, T, H) tensors that share one set of
 * element strides.  D is one of 16, 32, 64, 128.  No buffer may alias another.
 */
typedef struct fox_shift_args {
  int32_t B, T, H, D;
  int32_t dtype;                      /* FOX_DTYPE_* of x, out, dout, dx */
  const void* x;
  int64_t x_stride_b, x_stride_t, x_stride_h;
  const float* prev_weight;
  const float* curr_weight;
  int64_t w_stride_b, w_stride_t, w_stride_h;
  void* out;                          /* written by fox_token_shift_fwd */
  const void* dout;                   /* backward only */
  void* dx;                           /* written by fox_token_shift_bwd */
  float* dprev_weight;                /* written by fox_token_shift_bwd */
  float* dcurr_weight;                /* written by fox_token_shift_bwd */
} fox_shift_args;

/*
 * out[b,t,h,:] = x[b,t,h,:] * curr_weight[b,t,h] + x[b,t-1,h,:] * prev_weight[b,t,h], with x[b,-1] = 0,
 * evaluated in fp32 and rounded once.  Replaces shift_fwd_kernel as launched by TokenShift.forward
 * (model/forgetting_transformer/token_shift.py:21-71, :160-191).
 */
int fox_token_shift_fwd(const fox_shift_args* args, void* stream);

/*
 * dx[b,t,h,:] = dout[b,t,h,:] * curr_weight[b,t,h] + dout[b,t+1,h,:] * prev_weight[b,t+1,h],
 * dcurr_weight[b,t,h] = sum_d dout[b,t,h,d] * x[b,t,h,d], dprev_weight[b,t,h] = sum_d dout[b,t,h,d] * x[b,t-1,h,d].
 * Replaces shift_bwd_kernel as launched by TokenShift.backward (token_shift.py:83-156, :193-233).
 */
int fox_token_shift_bwd(const fox_shift_args* args, void* stream);

/*
 * Per-head RMS normalisation, gated or plain.  Gated: the epilogue the FoX layer applies to the attention
 * output before the output projection (FusedGroupNormGated(num_groups=heads, is_rms_norm=True,
 * activation="sigmoid"), model/forgetting_transformer/modeling_forgetting_transformer.py:243, :417-420).
 * Plain (FOX_ACT_NONE; g and dg are ignored and may be NULL): the normalisation of queries and keys in
 * front of the attention, GroupNorm(num_groups=heads, is_rms_norm=True) or RMSNorm(head_dim) (:258-265,
 * :314-325; the latter is G = 1 with one row per (token, head)), and the ungated output norm (:245).
 *   y[r,h,:] = x[r,h,:] * rstd[r,h] * weight[h,:] * act(g[r,h,:]),  rstd = 1/sqrt(mean_d x[r,h,:]^2 + eps),
 * act = sigmoid (FOX_ACT_SIGMOID), g*sigmoid(g) (FOX_ACT_SWISH) or 1 (FOX_ACT_NONE).  x, g, y, dy, dx, dg are 16-bit tensors of
 * `rows` rows of G*D contiguous elements, each with its own row stride in elements (a multiple of 8, base
 * pointers 16-byte aligned); weight and dweight are G*D fp32; rstd is (rows, G) fp32, written by the
 * forward and read by the backward.  No bias, no residual.  D is one of 16, 32, 64, 128.
 */
#define FOX_ACT_SIGMOID 0
#define FOX_ACT_SWISH 1
#define FOX_ACT_NONE 2

typedef struct fox_norm_gate_args {
  int64_t rows;
  int32_t G, D;
  int32_t dtype;        /* FOX_DTYPE_BF16 / FP16 of the 16-bit tensors */
  int32_t activation;   /* FOX_ACT_* */
  float eps;
  const void* x;  int64_t x_stride_row;
  const void* g;  int64_t g_stride_row;
  const float* weight;
  void* y;        int64_t y_stride_row;    /* written by fox_norm_gate_fwd */
  float* rstd;
  const void* dy; int64_t dy_stride_row;   /* backward only from here on */
  void* dx;       int64_t dx_stride_row;
  void* dg;       int64_t dg_stride_row;
  float* dweight;
  float* workspace;     /* fox_norm_gate_workspace_bytes() bytes, 16-byte aligned */
} fox_norm_gate_args;

/* Replaces layer_norm_gated_fwd_kernel as launched by LayerNormGatedFunction.forward (fuse_norm_gate.py:132-206, :539-618)
 * and, with FOX_ACT_NONE, layer_norm_fwd_kernel as launched by LayerNormFunction.forward (layernorm.py:183-254, :520-600). */
int fox_norm_gate_fwd(const fox_norm_gate_args* args, void* stream);

/*
 * dx, dg and dweight = sum over rows of dy*act(g)*xhat.  Replaces layer_norm_gated_bwd_kernel and the sum over
 * its partial weight gradients (fuse_norm_gate.py:309-417, :620-724; with FOX_ACT_NONE layer_norm_bwd_kernel,
 * layernorm.py:328-435, :603-703; dg is then not written).  The partial sums live in `workspace`
 * and are added in a fixed order, so the result is reproducible bit for bit.
 */
int fox_norm_gate_bwd(const fox_norm_gate_args* args, void* stream);

/* Size of the backward's workspace for `rows` rows of G heads of D elements. */
int fox_norm_gate_workspace_bytes(int64_t rows, int32_t G, int32_t D, int64_t* bytes);

/*
 * The forward with the layer's output norm and gate applied in its epilogue: while a query tile's output rows
 * are on their way from the accumulators to memory, the kernel also writes
 *   y[b,h,m,:] = o[b,h,m,:] * rstd[b,m,h] * weight[h,:] * act(gate[b,h,m,:]),  rstd = 1/sqrt(mean_d o^2 + eps),
 * computed from the rounded 16-bit o, i.e. what fox_attn_fwd followed by fox_norm_gate_fwd over o gives, without
 * the second pass over o.  Fuses forgetting_attention (ops/forgetting_attention.py:505-693) with the call of
 * FusedGroupNormGated / GroupNorm on its output (modeling_forgetting_transformer.py:243-245, :417-422;
 * fuse_norm_gate.py:132-206).  gate and y are (B,H,M,D) views like o (gate may be NULL with FOX_ACT_NONE);
 * weight is (H*D) fp32; rstd is (B,M,H) fp32 contiguous: the layout fox_norm_gate_bwd reads with rows = (b,m)
 * and G = H.  args->o may have a NULL ptr when the caller needs only y (inference), except for the shapes below.
 * Shapes whose forward splits the key loop (fox_attn_fwd_workspace_bytes() > 0 with a workspace given) and
 * M == 1 run fox_attn_fwd and then the standalone norm kernel; that needs o, and o, gate and y with adjacent
 * heads (stride_h == D, stride_b == M * stride_t), otherwise FOX_E_ARG.
 */
typedef struct fox_fwd_epilogue {
  fox_view gate;        /* read; 16-bit, same dtype as q */
  fox_view y;           /* written */
  const float* weight;
  float* rstd;          /* written */
  float eps;
  int32_t activation;   /* FOX_ACT_* */
} fox_fwd_epilogue;

int fox_attn_fwd_norm_gate(const fox_fwd_args* args, const fox_fwd_epilogue* epilogue, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FOX_ATTN_H */
