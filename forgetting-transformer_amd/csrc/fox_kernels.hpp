// Kernel argument blocks and launcher declarations shared by the C ABI layer and
// the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fox {

struct View {
  const uint16_t* ptr;
  int64_t sb, sh, st;
};

// Optional epilogue of the forward: the gated per-head RMS norm of the output rows (see store_rows_norm_gate).
// Off when y.ptr is null.  gate and y are (B, H, M, D) views like o; w is (H*D) fp32; rstd is (B, M, H) fp32.
struct FwdEpilogue {
  View gate, y;
  const float* w;
  float* rstd;
  float eps;
  int act;
};

struct FwdK {
  View q, k, v, o;
  const float* c;
  float* lse;
  const int64_t* seq_start;
  const float* thr;
  int32_t* first_block;
  int B, H, M, N;
  float sm_scale;
  int n_mtiles;
  int splits;      // key splits of the forward (1 = none)
  float* ws_o;     // (splits, B, H, M, D) partial accumulators
  float* ws_ml;    // (splits, B, H, M, 2) partial row maximum and row sum
  FwdEpilogue epi; // only for splits == 1 and M > 1 (the launcher rejects it otherwise)
  bool stream;     // K and V tiles are read once and not again soon: load them with the non-temporal hint
};

struct BwdK {
  View q, k, v, o, d_o, dq, dk, dv;
  const float* c;
  const float* lse;
  const int64_t* seq_start;
  const float* thr;
  float* delta;   // (B,H,M): rowsum(o * do), written by the dQ kernel
  float* drow;    // (B,H,M): row sums of dS, written by the dQ kernel, read by the dK/dV kernel
  float* dc;
  int B, H, M, N;
  float sm_scale;
  int n_tiles;
  int cls;         // kClassAll, or the class of key tiles this dK/dV launch handles (fox_common.hpp)
  int light_limit; // distance from the diagonal, in keys, that separates the two classes
  int32_t* q_first_block;  // optional (B,H,ceil(M/kFwdBM)): first key block (of kFwdBN keys) each query tile of the dQ kernel visits
  int32_t* kv_end_row;     // optional (B,H,ceil(N/kKvUnit)): per unit of kKvUnit keys, the query row at which the dK/dV kernel stops
};

constexpr int kKvUnit = 64;  // granularity of kv_end_row: the smallest key tile any dK/dV variant uses

// Token shift: x, out, dout, dx are (B, T, H, D) 16-bit with shared element strides; the weights and
// their gradients are (B, T, H) fp32 with shared element strides.
struct ShiftK {
  const uint16_t* x;
  uint16_t* out;
  const uint16_t* dout;
  uint16_t* dx;
  const float* prev_w;
  const float* curr_w;
  float* dprev_w;
  float* dcurr_w;
  int64_t x_sb, x_st, x_sh, w_sb, w_st, w_sh;
  int B, T, H;
};

// Gated per-head RMS norm: x, g, y, dy, dx, dg are (R rows, G heads, D) 16-bit, heads and head dim
// contiguous, each with its own row stride; w, dw are (G*D) fp32; rstd is (R, G) fp32.
struct NormGateK {
  const uint16_t* x;
  const uint16_t* g;
  uint16_t* y;
  const uint16_t* dy;
  uint16_t* dx;
  uint16_t* dg;
  const float* w;
  float* rstd;
  float* dw;
  float* dw_partial;
  int64_t x_sr, g_sr, y_sr, dy_sr, dx_sr, dg_sr;
  int64_t R;
  int G;
  float eps;
};

// Tile sizes (see fox_tile_config in the public header)
constexpr int kFwdBM = 128;
constexpr int kFwdBN = 64;
constexpr int kKvBN = 128;   // key rows per workgroup in the dK/dV kernel
constexpr int kKvBM = 128;   // query rows per step in the dK/dV kernel

hipError_t launch_fwd(const FwdK& a, int D, int dtype, hipStream_t s);
int fwd_key_splits(int B, int H, int M, int N);
hipError_t launch_bwd_delta(const BwdK& a, int D, int dtype, hipStream_t s);
hipError_t launch_bwd_dkdv(const BwdK& a, int D, int dtype, hipStream_t s);   // a.cls selects the variant and its tiles
bool dkdv_split_supports(int D);   // head dims the split (kClassLight) variant of the dK/dV kernel exists for
hipError_t launch_bwd_dq(const BwdK& a, int D, int dtype, hipStream_t s);
hipError_t launch_fwd_decode(const FwdK& a, int D, int dtype, hipStream_t s);  // M == 1, without the merge of the splits
hipError_t launch_norm_gate(const NormGateK& a, int D, int dtype, bool bwd, int act, hipStream_t s);  // act: FOX_ACT_*
int64_t norm_gate_strips(int64_t rows);
int64_t norm_gate_workspace_rows(int64_t rows);
hipError_t launch_shift_fwd(const ShiftK& a, int D, int dtype, hipStream_t s);
hipError_t launch_shift_bwd(const ShiftK& a, int D, int dtype, hipStream_t s);
hipError_t launch_cumsum_fwd(const float* g, int64_t sb, int64_t sh, int64_t sn, const int64_t* seq_start, float* c, int B,
                             int H, int N, hipStream_t s);
hipError_t launch_gate_cumsum_fwd(const void* logits, int dtype, int64_t sb, int64_t sh, int64_t sn, const int64_t* seq_start,
                                  float* log_fgate, float* c, int B, int H, int N, hipStream_t s);
hipError_t launch_gate_cumsum_bwd(const float* dc, const void* logits, int dtype, int64_t sb, int64_t sh, int64_t sn,
                                  const int64_t* seq_start, void* dlogits, int64_t db, int64_t dh, int64_t dn, int B, int H, int N,
                                  hipStream_t s);
hipError_t launch_cumsum_bwd(const float* dc, float* dg, int64_t db, int64_t dh, int64_t dn, const int64_t* seq_start, int B, int H,
                             int N, hipStream_t s);
hipError_t launch_mfma_probe(const void* operands, float* sink, int workgroups, int iters, hipStream_t s);  // fox_probe.hip
hipError_t launch_auto_threshold(const View& q, const View& k, int B, int H, int M, int N, int D, int dtype, float sm_scale,
                                 float* thr, uint32_t* scratch, hipStream_t s);

}  // namespace fox
