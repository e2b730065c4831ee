// Flat C ABI of libfox_attn.so: argument validation and kernel dispatch.
// Declarations and their reference citations live in include/fox_attn.h.
#include "../../include/fox_attn.h"

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>

#include <atomic>
#include <mutex>

#include "fox_common.hpp"
#include "fox_kernels.hpp"

// Library-owned scratch of fox_attn_fwd_noalloc: the partial (max, sum, accumulator) results of a key-split
// forward.  Every GPU the library runs on holds its own copy of this array, at its own address, until the
// process ends.  In host code the name is only a handle for hipGetSymbolAddress; kernels and copies get the
// per-device address that call returns.
#define FOX_NOALLOC_SCRATCH_BYTES (64ll << 20)
static __device__ __align__(256) unsigned char scratch[FOX_NOALLOC_SCRATCH_BYTES];

namespace {

thread_local char g_err[256] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return FOX_OK;
  return fail(FOX_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

int check_dims(const fox_dims* d) {
  if (!d) return fail(FOX_E_ARG, "dims is NULL");
  if (d->B <= 0 || d->H <= 0 || d->M <= 0 || d->N <= 0) return fail(FOX_E_ARG, "B, H, M, N must be positive (got %d, %d, %d, %d)", d->B, d->H, d->M, d->N);
  if (d->M > d->N) return fail(FOX_E_ARG, "the key/value tensors must be at least as long as the query tensor (M=%d > N=%d)", d->M, d->N);
  if (d->D != 16 && d->D != 32 && d->D != 64 && d->D != 128) return fail(FOX_E_ARG, "head dim must be one of 16, 32, 64, 128 (got %d)", d->D);
  if (d->dtype != FOX_DTYPE_BF16 && d->dtype != FOX_DTYPE_FP16) return fail(FOX_E_ARG, "dtype must be FOX_DTYPE_BF16 or FOX_DTYPE_FP16 (got %d)", d->dtype);
  // B*H is the y extent of some grids (at most 65535), and every grid that folds (batch, head) into x
  // must stay below 2^31 workgroups: tiles of at least 64 rows over the longer sequence.
  if ((int64_t)d->B * d->H > 65535) return fail(FOX_E_ARG, "B*H must not exceed 65535 (got %lld)", (long long)d->B * d->H);
  if ((int64_t)d->B * d->H * ((d->N + 63) / 64) * 64 > 0x7fffffffLL)
    return fail(FOX_E_ARG, "B*H*ceil(N/64) must stay below 2^25 workgroups (got B*H = %lld, N = %d)", (long long)d->B * d->H, d->N);
  return FOX_OK;
}

int check_view(const fox_view* v, const char* name) {
  if (!v || !v->ptr) return fail(FOX_E_ARG, "%s is NULL", name);
  if (((uintptr_t)v->ptr & 15) != 0) return fail(FOX_E_ALIGN, "%s must be 16-byte aligned", name);
  if ((v->stride_b & 7) || (v->stride_h & 7) || (v->stride_t & 7)) return fail(FOX_E_ALIGN, "strides of %s must be multiples of 8 elements", name);
  return FOX_OK;
}

// The tile loaders address one (batch, head) slice with 32-bit byte offsets.
int check_extent(const fox_view* v, int rows, int D, const char* name) {
  const int64_t bytes = ((int64_t)(rows - 1) * v->stride_t + D) * 2;
  if (v->stride_t <= 0 || bytes >= (int64_t)1 << 31) return fail(FOX_E_ARG, "%s: one (batch, head) slice must span less than 2 GiB with a positive row stride", name);
  return FOX_OK;
}

// Distance from the diagonal, in keys, within which the pruning bound of a 128-key tile must lie for the tile to go
// to the split variant of the dK/dV kernel (fox_set_acp_light_limit): 0 = never, negative = every tile of every
// call that the variant supports.
std::atomic<int> g_light_limit{256};   // measured crossover of the two kernels at head dim 128

// Bytes of K and V together from which on a forward with one query tile per (batch, head) loads its K and V tiles
// with the non-temporal hint (fox_set_stream_min_kv_bytes).  Such a call reads every tile once; the hint pays
// (chunked prefill at 4 GiB: 12 %) unless the tensors are small enough to still sit in the 256 MiB last-level cache
// when the next call on them comes (32-270 MB, called in a loop: 5-14 % faster with cached loads).
std::atomic<int64_t> g_stream_min_kv_bytes{(int64_t)512 << 20};

// The tile classes of a call: *first and *second are the classes of the launches to make (kClassAll alone,
// kClassLight alone, or kClassLight then kClassHeavy), *limit the distance handed to the kernels.
void tile_classes(bool pruned, bool light_ok, int* first, int* second, int* limit) {
  const int lim = g_light_limit.load(std::memory_order_relaxed);
  *first = fox::kClassAll;
  *second = -1;
  *limit = lim;
  if (!light_ok || lim == 0) return;
  if (lim < 0) { *first = fox::kClassLight; return; }
  if (!pruned) return;
  *first = fox::kClassLight;
  *second = fox::kClassHeavy;
}

// Device address of `scratch` on the current device, looked up once per device.
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

int scratch_of_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(FOX_E_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(FOX_E_ARG, "device index %d is outside the scratch table (0..%d)", dev, kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return fail(FOX_E_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return FOX_OK;
}

fox::View to_view(const fox_view& v) { return fox::View{(const uint16_t*)v.ptr, v.stride_b, v.stride_h, v.stride_t}; }

#define FOX_TRY(x)            \
  do {                        \
    const int rc_ = (x);      \
    if (rc_ != FOX_OK) return rc_; \
  } while (0)

int make_bwd(const fox_bwd_args* args, fox::BwdK& k, bool need_grads) {
  if (!args) return fail(FOX_E_ARG, "args is NULL");
  FOX_TRY(check_dims(&args->dims));
  FOX_TRY(check_view(&args->o, "o"));
  FOX_TRY(check_view(&args->d_o, "do"));
  if (!args->delta) return fail(FOX_E_ARG, "delta is NULL");
  k = fox::BwdK{};
  k.o = to_view(args->o);
  k.d_o = to_view(args->d_o);
  k.delta = args->delta;
  k.drow = args->drow;
  k.B = args->dims.B; k.H = args->dims.H; k.M = args->dims.M; k.N = args->dims.N;
  k.sm_scale = args->sm_scale;
  k.n_tiles = 0;
  if (!need_grads) return FOX_OK;
  FOX_TRY(check_view(&args->q, "q"));
  FOX_TRY(check_view(&args->k, "k"));
  FOX_TRY(check_view(&args->v, "v"));
  FOX_TRY(check_extent(&args->q, args->dims.M, args->dims.D, "q"));
  FOX_TRY(check_extent(&args->d_o, args->dims.M, args->dims.D, "do"));
  FOX_TRY(check_extent(&args->k, args->dims.N, args->dims.D, "k"));
  FOX_TRY(check_extent(&args->v, args->dims.N, args->dims.D, "v"));
  if (!args->log_lambda || !args->lse || !args->dlog_lambda) return fail(FOX_E_ARG, "log_lambda, lse and dlog_lambda must not be NULL");
  if (!args->drow) return fail(FOX_E_ARG, "drow is NULL");
  if (args->drow == args->delta) return fail(FOX_E_ARG, "delta and drow must not alias");
  k.q = to_view(args->q);
  k.k = to_view(args->k);
  k.v = to_view(args->v);
  k.c = args->log_lambda;
  k.lse = args->lse;
  k.seq_start = args->seq_start;
  k.thr = args->threshold;
  k.dc = args->dlog_lambda;
  k.q_first_block = args->q_first_block;
  k.kv_end_row = args->kv_end_row;
  return FOX_OK;
}

int make_shift(const fox_shift_args* a, fox::ShiftK& k, bool bwd) {
  if (!a) return fail(FOX_E_ARG, "args is NULL");
  if (a->B <= 0 || a->T <= 0 || a->H <= 0) return fail(FOX_E_ARG, "B, T, H must be positive (got %d, %d, %d)", a->B, a->T, a->H);
  if (a->D != 16 && a->D != 32 && a->D != 64 && a->D != 128) return fail(FOX_E_ARG, "head dim must be one of 16, 32, 64, 128 (got %d)", a->D);
  if (a->dtype != FOX_DTYPE_BF16 && a->dtype != FOX_DTYPE_FP16) return fail(FOX_E_ARG, "dtype must be FOX_DTYPE_BF16 or FOX_DTYPE_FP16 (got %d)", a->dtype);
  if (a->B > 65535) return fail(FOX_E_ARG, "B must not exceed 65535");
  if (!a->x || !a->prev_weight || !a->curr_weight) return fail(FOX_E_ARG, "x, prev_weight and curr_weight must not be NULL");
  if ((a->x_stride_b & 7) || (a->x_stride_t & 7) || (a->x_stride_h & 7)) return fail(FOX_E_ALIGN, "strides of x must be multiples of 8 elements");
  const void* vec[4] = {a->x, bwd ? a->dout : a->out, bwd ? a->dx : a->out, a->x};
  for (const void* p : vec) {
    if (!p) return fail(FOX_E_ARG, bwd ? "dout and dx must not be NULL" : "out must not be NULL");
    if (((uintptr_t)p & 15) != 0) return fail(FOX_E_ALIGN, "x, out, dout and dx must be 16-byte aligned");
  }
  if (bwd && (!a->dprev_weight || !a->dcurr_weight)) return fail(FOX_E_ARG, "dprev_weight and dcurr_weight must not be NULL");
  if (!bwd && a->out == a->x) return fail(FOX_E_ARG, "out must not alias x");
  if (bwd && (a->dx == a->dout || a->dx == a->x)) return fail(FOX_E_ARG, "dx must not alias dout or x");
  k = fox::ShiftK{};
  k.x = (const uint16_t*)a->x;
  k.out = (uint16_t*)a->out;
  k.dout = (const uint16_t*)a->dout;
  k.dx = (uint16_t*)a->dx;
  k.prev_w = a->prev_weight;
  k.curr_w = a->curr_weight;
  k.dprev_w = a->dprev_weight;
  k.dcurr_w = a->dcurr_weight;
  k.x_sb = a->x_stride_b; k.x_st = a->x_stride_t; k.x_sh = a->x_stride_h;
  k.w_sb = a->w_stride_b; k.w_st = a->w_stride_t; k.w_sh = a->w_stride_h;
  k.B = a->B; k.T = a->T; k.H = a->H;
  return FOX_OK;
}

int make_norm_gate(const fox_norm_gate_args* a, fox::NormGateK& k, bool bwd) {
  if (!a) return fail(FOX_E_ARG, "args is NULL");
  if (a->rows <= 0 || a->G <= 0) return fail(FOX_E_ARG, "rows and G must be positive");
  if (a->D != 16 && a->D != 32 && a->D != 64 && a->D != 128) return fail(FOX_E_ARG, "head dim must be one of 16, 32, 64, 128 (got %d)", a->D);
  if (a->dtype != FOX_DTYPE_BF16 && a->dtype != FOX_DTYPE_FP16) return fail(FOX_E_ARG, "dtype must be FOX_DTYPE_BF16 or FOX_DTYPE_FP16 (got %d)", a->dtype);
  if (a->activation != FOX_ACT_SIGMOID && a->activation != FOX_ACT_SWISH && a->activation != FOX_ACT_NONE) return fail(FOX_E_ARG, "activation must be FOX_ACT_SIGMOID, FOX_ACT_SWISH or FOX_ACT_NONE (got %d)", a->activation);
  const bool gated = a->activation != FOX_ACT_NONE;
  if (a->rows * a->G * (a->D / 8) > ((int64_t)1 << 39)) return fail(FOX_E_ARG, "tensor too large");
  if (!a->x || !a->weight || !a->rstd) return fail(FOX_E_ARG, "x, weight and rstd must not be NULL");
  if (gated && !a->g) return fail(FOX_E_ARG, "g must not be NULL for a gated activation");
  // the ungated form neither reads g nor writes dg: both are ignored and may be NULL
  const void* ptrs[6] = {a->x, gated ? a->g : a->x, bwd ? a->dy : a->y, bwd ? a->dx : a->y,
                         bwd ? (gated ? a->dg : a->dx) : a->y, a->weight};
  const int64_t strides[6] = {a->x_stride_row, gated ? a->g_stride_row : 8, bwd ? a->dy_stride_row : a->y_stride_row,
                              bwd ? a->dx_stride_row : a->y_stride_row,
                              bwd ? (gated ? a->dg_stride_row : 8) : a->y_stride_row, 8};
  for (int i = 0; i < 6; ++i) {
    if (!ptrs[i]) return fail(FOX_E_ARG, bwd ? "dy, dx and (for a gated activation) dg must not be NULL" : "y must not be NULL");
    if (((uintptr_t)ptrs[i] & 15) != 0) return fail(FOX_E_ALIGN, "tensors must be 16-byte aligned");
    if (strides[i] & 7) return fail(FOX_E_ALIGN, "row strides must be multiples of 8 elements");
  }
  if (bwd && (!a->dweight || !a->workspace)) return fail(FOX_E_ARG, "dweight and workspace must not be NULL");
  if (bwd && ((uintptr_t)a->workspace & 15) != 0) return fail(FOX_E_ALIGN, "workspace must be 16-byte aligned");
  k = fox::NormGateK{};
  k.x = (const uint16_t*)a->x; k.g = gated ? (const uint16_t*)a->g : nullptr; k.y = (uint16_t*)a->y;
  k.dy = (const uint16_t*)a->dy; k.dx = (uint16_t*)a->dx; k.dg = gated ? (uint16_t*)a->dg : nullptr;
  k.w = a->weight; k.rstd = a->rstd; k.dw = a->dweight; k.dw_partial = a->workspace;
  k.x_sr = a->x_stride_row; k.g_sr = a->g_stride_row; k.y_sr = a->y_stride_row;
  k.dy_sr = a->dy_stride_row; k.dx_sr = a->dx_stride_row; k.dg_sr = a->dg_stride_row;
  k.R = a->rows; k.G = a->G; k.eps = a->eps;
  return FOX_OK;
}

// The forward with its key-split scratch passed separately: the caller's workspace (fox_attn_fwd) or the
// library's own array (fox_attn_fwd_noalloc).  workspace == NULL never splits keys.
// epi: the norm-and-gate epilogue (already validated), or NULL.  With an epilogue, shapes the unsplit kernel does
// not handle run the plain forward followed by the standalone norm kernel.
int fwd_impl(const fox_fwd_args* args, void* workspace, int64_t workspace_bytes, void* stream, const char* what,
             const fox_fwd_epilogue* epi = nullptr) {
  FOX_TRY(check_dims(&args->dims));
  FOX_TRY(check_view(&args->q, "q"));
  FOX_TRY(check_view(&args->k, "k"));
  FOX_TRY(check_view(&args->v, "v"));
  if (!(epi && !args->o.ptr)) FOX_TRY(check_view(&args->o, "o"));
  FOX_TRY(check_extent(&args->k, args->dims.N, args->dims.D, "k"));
  FOX_TRY(check_extent(&args->v, args->dims.N, args->dims.D, "v"));
  if (!args->log_lambda || !args->lse) return fail(FOX_E_ARG, "log_lambda and lse must not be NULL");
  fox::FwdK k{};
  k.q = to_view(args->q);
  k.k = to_view(args->k);
  k.v = to_view(args->v);
  k.o = to_view(args->o);
  k.c = args->log_lambda;
  k.lse = args->lse;
  k.seq_start = args->seq_start;
  k.thr = args->threshold;
  k.first_block = args->first_block;
  k.B = args->dims.B; k.H = args->dims.H; k.M = args->dims.M; k.N = args->dims.N;
  k.sm_scale = args->sm_scale;
  k.n_mtiles = (args->dims.M + fox::kFwdBM - 1) / fox::kFwdBM;
  k.splits = 1;
  k.stream = k.n_mtiles == 1 && (int64_t)k.B * k.H * k.N * args->dims.D * 4 >= g_stream_min_kv_bytes.load(std::memory_order_relaxed);
  if (workspace) {
    const int splits = fox::fwd_key_splits(k.B, k.H, k.M, k.N);
    const int64_t need = splits <= 1 ? 0 : (int64_t)splits * k.B * k.H * k.M * (args->dims.D + 2) * (int64_t)sizeof(float);
    if (need > 0) {
      if (workspace_bytes < need) return fail(FOX_E_ARG, "workspace too small: %lld < %lld bytes", (long long)workspace_bytes, (long long)need);
      if (((uintptr_t)workspace & 15) != 0) return fail(FOX_E_ALIGN, "workspace must be 16-byte aligned");
      k.splits = splits;
      k.ws_o = (float*)workspace;
      k.ws_ml = k.ws_o + (int64_t)k.splits * k.B * k.H * k.M * args->dims.D;
    }
  }
  if (epi) {
    const int D = args->dims.D;
    if (k.M == 1 || k.splits > 1) {
      // two passes: the plain forward, then the norm over o as (B*M rows, H heads)
      const fox_view* vs[3] = {&args->o, &epi->y, &epi->gate};
      for (int i = 0; i < 3; ++i) {
        if (i == 2 && epi->activation == FOX_ACT_NONE) break;
        if (!vs[i]->ptr || vs[i]->stride_h != D || vs[i]->stride_b != (int64_t)k.M * vs[i]->stride_t)
          return fail(FOX_E_ARG, "%s: a key-split or single-query shape needs o, gate and y with adjacent heads "
                                 "(stride_h == D, stride_b == M * stride_t)", what);
      }
      FOX_TRY(check_hip(fox::launch_fwd(k, D, args->dims.dtype, (hipStream_t)stream), what));
      fox::NormGateK n{};
      n.x = (const uint16_t*)args->o.ptr; n.x_sr = args->o.stride_t;
      n.g = epi->activation == FOX_ACT_NONE ? nullptr : (const uint16_t*)epi->gate.ptr; n.g_sr = epi->gate.stride_t;
      n.y = (uint16_t*)epi->y.ptr; n.y_sr = epi->y.stride_t;
      n.w = epi->weight; n.rstd = epi->rstd; n.R = (int64_t)k.B * k.M; n.G = k.H; n.eps = epi->eps;
      return check_hip(fox::launch_norm_gate(n, D, args->dims.dtype, false, epi->activation, (hipStream_t)stream), what);
    }
    k.epi.gate = epi->activation == FOX_ACT_NONE ? fox::View{} : to_view(epi->gate);
    k.epi.y = to_view(epi->y);
    k.epi.w = epi->weight;
    k.epi.rstd = epi->rstd;
    k.epi.eps = epi->eps;
    k.epi.act = epi->activation;
  }
  return check_hip(fox::launch_fwd(k, args->dims.D, args->dims.dtype, (hipStream_t)stream), what);
}

}  // namespace

extern "C" {

int fox_version(void) { return 201; }  // 0.2.x: fox_bwd_args and the scan entry points differ from 0.1.0; 0.2.1 adds fox_set_stream_min_kv_bytes and fox_probe_mfma

const char* fox_last_error(void) { return g_err; }

int32_t fox_set_acp_light_limit(int32_t keys) { return g_light_limit.exchange(keys, std::memory_order_relaxed); }

int64_t fox_set_stream_min_kv_bytes(int64_t bytes) { return g_stream_min_kv_bytes.exchange(bytes, std::memory_order_relaxed); }

int fox_probe_mfma(const void* operands, float* sink, int32_t workgroups, int32_t iters, void* stream) {
  if (!operands || !sink) return fail(FOX_E_ARG, "fox_probe_mfma: operands and sink must not be NULL");
  if (workgroups < 1 || workgroups > 65536 || iters < 1 || iters > (1 << 20))   // at most about half a second per launch
    return fail(FOX_E_ARG, "fox_probe_mfma: workgroups in [1, 65536] and iters in [1, 2^20]");
  return check_hip(fox::launch_mfma_probe(operands, sink, workgroups, iters, (hipStream_t)stream), "fox_probe_mfma");
}

int fox_tile_config(int32_t D, int32_t* block_m, int32_t* block_n, int32_t* kv_block_n, int32_t* kv_block_m) {
  if (D != 16 && D != 32 && D != 64 && D != 128) return fail(FOX_E_ARG, "head dim must be one of 16, 32, 64, 128 (got %d)", D);
  if (block_m) *block_m = fox::kFwdBM;
  if (block_n) *block_n = fox::kFwdBN;
  if (kv_block_n) *kv_block_n = fox::kKvBN;
  if (kv_block_m) *kv_block_m = fox::kKvBM;
  return FOX_OK;
}

int fox_attn_fwd_norm_gate(const fox_fwd_args* args, const fox_fwd_epilogue* epi, void* stream) {
  if (!args || !epi) return fail(FOX_E_ARG, "args and epilogue must not be NULL");
  if (epi->activation != FOX_ACT_SIGMOID && epi->activation != FOX_ACT_SWISH && epi->activation != FOX_ACT_NONE)
    return fail(FOX_E_ARG, "activation must be FOX_ACT_SIGMOID, FOX_ACT_SWISH or FOX_ACT_NONE (got %d)", epi->activation);
  FOX_TRY(check_view(&epi->y, "y"));
  if (epi->activation != FOX_ACT_NONE) FOX_TRY(check_view(&epi->gate, "gate"));
  if (!epi->weight || !epi->rstd) return fail(FOX_E_ARG, "weight and rstd must not be NULL");
  if (((uintptr_t)epi->weight & 15) != 0) return fail(FOX_E_ALIGN, "weight must be 16-byte aligned");
  if (epi->y.ptr == args->o.ptr) return fail(FOX_E_ARG, "y must not alias o");
  return fwd_impl(args, args->workspace, args->workspace_bytes, stream, "fox_attn_fwd_norm_gate", epi);
}

int fox_norm_gate_fwd(const fox_norm_gate_args* args, void* stream) {
  fox::NormGateK k;
  FOX_TRY(make_norm_gate(args, k, false));
  return check_hip(fox::launch_norm_gate(k, args->D, args->dtype, false, args->activation, (hipStream_t)stream),
                   "fox_norm_gate_fwd");
}

int fox_norm_gate_bwd(const fox_norm_gate_args* args, void* stream) {
  fox::NormGateK k;
  FOX_TRY(make_norm_gate(args, k, true));
  return check_hip(fox::launch_norm_gate(k, args->D, args->dtype, true, args->activation, (hipStream_t)stream),
                   "fox_norm_gate_bwd");
}

int fox_norm_gate_workspace_bytes(int64_t rows, int32_t G, int32_t D, int64_t* bytes) {
  if (!bytes) return fail(FOX_E_ARG, "bytes is NULL");
  if (rows <= 0 || G <= 0 || (D != 16 && D != 32 && D != 64 && D != 128)) return fail(FOX_E_ARG, "rows and G must be positive and D one of 16, 32, 64, 128");
  *bytes = fox::norm_gate_workspace_rows(rows) * G * D * (int64_t)sizeof(float);
  return FOX_OK;
}

int fox_token_shift_fwd(const fox_shift_args* args, void* stream) {
  fox::ShiftK k;
  FOX_TRY(make_shift(args, k, false));
  return check_hip(fox::launch_shift_fwd(k, args->D, args->dtype, (hipStream_t)stream), "fox_token_shift_fwd");
}

int fox_token_shift_bwd(const fox_shift_args* args, void* stream) {
  fox::ShiftK k;
  FOX_TRY(make_shift(args, k, true));
  return check_hip(fox::launch_shift_bwd(k, args->D, args->dtype, (hipStream_t)stream), "fox_token_shift_bwd");
}

int fox_cumsum_fwd(const float* g, int64_t g_sb, int64_t g_sh, int64_t g_sn, const int64_t* seq_start, float* c, int32_t B,
                   int32_t H, int32_t N, void* stream) {
  if (!g || !c) return fail(FOX_E_ARG, "g and c must not be NULL");
  if (B <= 0 || H <= 0 || N <= 0) return fail(FOX_E_ARG, "B, H, N must be positive");
  return check_hip(fox::launch_cumsum_fwd(g, g_sb, g_sh, g_sn, seq_start, c, B, H, N, (hipStream_t)stream), "fox_cumsum_fwd");
}

int fox_gate_cumsum_fwd(const void* logits, int32_t logits_dtype, int64_t sb, int64_t sh, int64_t sn, const int64_t* seq_start,
                        float* log_fgate, float* c, int32_t B, int32_t H, int32_t N, void* stream) {
  if (!logits || !c) return fail(FOX_E_ARG, "logits and c must not be NULL");
  if (B <= 0 || H <= 0 || N <= 0) return fail(FOX_E_ARG, "B, H, N must be positive");
  if (logits_dtype < FOX_DTYPE_BF16 || logits_dtype > FOX_DTYPE_FP32) return fail(FOX_E_ARG, "logits_dtype must be FOX_DTYPE_BF16, FP16 or FP32 (got %d)", logits_dtype);
  return check_hip(fox::launch_gate_cumsum_fwd(logits, logits_dtype, sb, sh, sn, seq_start, log_fgate, c, B, H, N, (hipStream_t)stream),
                   "fox_gate_cumsum_fwd");
}

int fox_gate_cumsum_bwd(const float* dc, const void* logits, int32_t logits_dtype, int64_t sb, int64_t sh, int64_t sn,
                        const int64_t* seq_start, void* dlogits, int64_t db, int64_t dh, int64_t dn, int32_t B, int32_t H,
                        int32_t N, void* stream) {
  if (!dc || !logits || !dlogits) return fail(FOX_E_ARG, "dc, logits and dlogits must not be NULL");
  if (B <= 0 || H <= 0 || N <= 0) return fail(FOX_E_ARG, "B, H, N must be positive");
  if (logits_dtype < FOX_DTYPE_BF16 || logits_dtype > FOX_DTYPE_FP32) return fail(FOX_E_ARG, "logits_dtype must be FOX_DTYPE_BF16, FP16 or FP32 (got %d)", logits_dtype);
  if ((const void*)dc == dlogits || logits == dlogits) return fail(FOX_E_ARG, "dlogits must not alias dc or logits");
  return check_hip(fox::launch_gate_cumsum_bwd(dc, logits, logits_dtype, sb, sh, sn, seq_start, dlogits, db, dh, dn, B, H, N,
                                               (hipStream_t)stream),
                   "fox_gate_cumsum_bwd");
}

int fox_cumsum_bwd(const float* dc, float* dg, int64_t dg_sb, int64_t dg_sh, int64_t dg_sn, const int64_t* seq_start, int32_t B,
                   int32_t H, int32_t N, void* stream) {
  if (!dc || !dg) return fail(FOX_E_ARG, "dc and dg must not be NULL");
  if (B <= 0 || H <= 0 || N <= 0) return fail(FOX_E_ARG, "B, H, N must be positive");
  if (dc == dg) return fail(FOX_E_ARG, "dc and dg must not alias");
  if (dg_sb == 0 && dg_sh == 0 && dg_sn == 0) { dg_sb = (int64_t)H * N; dg_sh = N; dg_sn = 1; }   // contiguous (B,H,N)
  return check_hip(fox::launch_cumsum_bwd(dc, dg, dg_sb, dg_sh, dg_sn, seq_start, B, H, N, (hipStream_t)stream), "fox_cumsum_bwd");
}

int fox_auto_threshold(const fox_dims* dims, const fox_view* q, const fox_view* k, float sm_scale, float* thr,
                       uint32_t* norm_scratch, void* stream) {
  FOX_TRY(check_dims(dims));
  FOX_TRY(check_view(q, "q"));
  FOX_TRY(check_view(k, "k"));
  if (!thr || !norm_scratch) return fail(FOX_E_ARG, "thr and norm_scratch must not be NULL");
  return check_hip(fox::launch_auto_threshold(to_view(*q), to_view(*k), dims->B, dims->H, dims->M, dims->N, dims->D,
                                              dims->dtype, sm_scale, thr, norm_scratch, (hipStream_t)stream),
                   "fox_auto_threshold");
}

int fox_attn_fwd_workspace_bytes(const fox_dims* dims, int64_t* bytes) {
  FOX_TRY(check_dims(dims));
  if (!bytes) return fail(FOX_E_ARG, "bytes is NULL");
  const int splits = fox::fwd_key_splits(dims->B, dims->H, dims->M, dims->N);
  *bytes = splits <= 1 ? 0 : (int64_t)splits * dims->B * dims->H * dims->M * (dims->D + 2) * (int64_t)sizeof(float);
  return FOX_OK;
}

int fox_attn_fwd(const fox_fwd_args* args, void* stream) {
  if (!args) return fail(FOX_E_ARG, "args is NULL");
  return fwd_impl(args, args->workspace, args->workspace_bytes, stream, "fox_attn_fwd");
}

int fox_attn_fwd_noalloc(const fox_fwd_args* args, void* stream) {
  if (!args) return fail(FOX_E_ARG, "args is NULL");
  FOX_TRY(check_dims(&args->dims));
  int64_t need = 0;
  FOX_TRY(fox_attn_fwd_workspace_bytes(&args->dims, &need));
  if (need > FOX_NOALLOC_SCRATCH_BYTES)
    return fail(FOX_E_ARG, "fox_attn_fwd_noalloc: this shape needs %lld bytes of key-split scratch, the library holds %lld; "
                "use fox_attn_fwd with a caller-provided workspace", (long long)need, (long long)FOX_NOALLOC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (need > 0) FOX_TRY(scratch_of_current_device(&ws));
  return fwd_impl(args, ws, need, stream, "fox_attn_fwd_noalloc");
}

int fox_attn_bwd_delta(const fox_bwd_args* args, void* stream) {
  fox::BwdK k;
  FOX_TRY(make_bwd(args, k, false));
  return check_hip(fox::launch_bwd_delta(k, args->dims.D, args->dims.dtype, (hipStream_t)stream), "fox_attn_bwd_delta");
}

int fox_attn_bwd_dkdv(const fox_bwd_args* args, void* stream) {
  fox::BwdK k;
  FOX_TRY(make_bwd(args, k, true));
  FOX_TRY(check_view(&args->dk, "dk"));
  FOX_TRY(check_view(&args->dv, "dv"));
  k.dk = to_view(args->dk);
  k.dv = to_view(args->dv);
  int first, second;
  tile_classes(k.thr != nullptr, fox::dkdv_split_supports(args->dims.D), &first, &second, &k.light_limit);
  k.cls = first;
  FOX_TRY(check_hip(fox::launch_bwd_dkdv(k, args->dims.D, args->dims.dtype, (hipStream_t)stream), "fox_attn_bwd_dkdv"));
  if (second < 0) return FOX_OK;
  k.cls = second;
  return check_hip(fox::launch_bwd_dkdv(k, args->dims.D, args->dims.dtype, (hipStream_t)stream), "fox_attn_bwd_dkdv");
}

int fox_attn_bwd_dq(const fox_bwd_args* args, void* stream) {
  fox::BwdK k;
  FOX_TRY(make_bwd(args, k, true));
  FOX_TRY(check_view(&args->dq, "dq"));
  k.dq = to_view(args->dq);
  return check_hip(fox::launch_bwd_dq(k, args->dims.D, args->dims.dtype, (hipStream_t)stream), "fox_attn_bwd_dq");
}

int fox_attn_bwd(const fox_bwd_args* args, void* stream) {
  if (!args) return fail(FOX_E_ARG, "args is NULL");
  if (!args->dlog_fgate) return fail(FOX_E_ARG, "dlog_fgate is NULL");
  FOX_TRY(fox_attn_bwd_dq(args, stream));
  FOX_TRY(fox_attn_bwd_dkdv(args, stream));
  return fox_cumsum_bwd(args->dlog_lambda, args->dlog_fgate, args->dlog_fgate_stride_b, args->dlog_fgate_stride_h,
                        args->dlog_fgate_stride_n, args->seq_start, args->dims.B, args->dims.H, args->dims.N, stream);
}

}  // extern "C"
