// Backward kernels of Forgetting Attention for gfx950.
//
//   dq_kernel    : one workgroup keeps 128 query rows (Q, dO in registers) and
//                  walks the key tiles like the forward; computes delta_i =
//                  sum_d o_id * do_id for its rows on the way in, writes dq,
//                  delta and the row sums drow[i] = sum_j dS[i,j].
//   dkdv_kernel  : runs after it.  One workgroup keeps 128 key rows (K, V in
//                  registers as MFMA B operands; dK^T, dV^T accumulators) and
//                  walks the query tiles below its diagonal; writes dk, dv and
//                  dc[n] = drow[n - (N - M)] - sum_i dS[i,n].
//   delta_kernel : delta alone (a stage of its own for callers that want it;
//                  the backward does not launch it).
// Every kernel only stores: no read-modify-write of anything another kernel wrote,
// so a stage may be repeated or timed alone without changing the result.
//
// Probabilities are rebuilt from the stored log-normaliser:
//   P = exp2( (q.k)*sm_scale*log2e + rowc_i - colc_j ),
//   rowc_i = (c_i - c_ref - lse_i)*log2e   (-inf for rows past M or empty rows),
//   colc_j = (c_j - c_ref)*log2e           (+inf left of seq_start or past N),
// so row/column validity costs nothing in the loop; only tiles that cross the
// diagonal run the causal compare.  In every kernel the first MFMA leaves each
// lane with one index of the dimension that stays free in the second MFMA, so the
// recomputed P / dS feed the second MFMA straight from registers.
#include "fox_common.hpp"
#include "fox_kernels.hpp"

namespace fox {

// ---------------------------------------------------------------------------
template <typename Tr, int D>
__global__ __launch_bounds__(256) void delta_kernel(const BwdK a) {
  constexpr int LPR = D / 8;          // lanes per row
  constexpr int RPP = 256 / LPR;      // rows per pass
  constexpr int ROWS = 128;           // rows per workgroup
  const int tid = threadIdx.x;
  const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
  const uint16_t* op = a.o.ptr + b * a.o.sb + h * a.o.sh;
  const uint16_t* dop = a.d_o.ptr + b * a.d_o.sb + h * a.d_o.sh;
  const int ch = tid % LPR;
  // every load of the workgroup's rows is requested before the first one is used (rows past the end repeat the last row)
  constexpr int NP = ROWS / RPP;
  u32x4 x[NP], y[NP];
#pragma unroll
  for (int pass = 0; pass < NP; ++pass) {
    const int m = min(blockIdx.x * ROWS + pass * RPP + tid / LPR, a.M - 1);
    x[pass] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(op + (int64_t)m * a.o.st + ch * 8));
    y[pass] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(dop + (int64_t)m * a.d_o.st + ch * 8));
  }
#pragma unroll
  for (int pass = 0; pass < NP; ++pass) {
    const int m = blockIdx.x * ROWS + pass * RPP + tid / LPR;
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) acc += Tr::lo(x[pass][e]) * Tr::lo(y[pass][e]) + Tr::hi(x[pass][e]) * Tr::hi(y[pass][e]);
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    if (m < a.M && ch == 0) a.delta[(int64_t)bh * a.M + m] = acc;
  }
}

// ---------------------------------------------------------------------------
// One step (BMQ query rows) of the dK/dV kernel for one wave (32 key rows).
// rc_s holds rowc_i / (sm_scale*log2e) and dl_s holds -delta_i.  The wave accumulates the NDB 32-column
// blocks of dK and dV that start at block db0 (all of them, or one half of the head dim when two waves
// share a block of keys).
template <typename Tr, int D, int BMQ = kKvBM, int NDB = (D + 31) / 32>
__device__ __forceinline__ void dkdv_step(const char* q_tile, const char* do_tile, const float* rc_s, const float* dl_s,
                                 const u32x4 (&kreg)[D / 16], const u32x4 (&vreg)[D / 16], f32x16 (&dkacc)[NDB],
                                 f32x16 (&dvacc)[NDB], float& csum, int a_s0, int n, int n_w0, float qk_scale,
                                 float colc, int lane, int db0 = 0) {
  constexpr int KK = D / 16, MB = BMQ / 32;
  const int g = lane >> 5, i = lane & 31;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int a_b0 = a_s0 + 32 * mb;   // key position of the block's first query row
    if (a_b0 + 31 < n_w0) continue;    // block entirely above the diagonal for this wave
    f32x16 s = acc_init(rc_s, 32 * mb, g), dp = acc_init(dl_s, 32 * mb, g);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) s = Tr::mfma32(lds_row_operand<D>(q_tile, 32 * mb + i, 2 * kk + g), kreg[kk], s);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) dp = Tr::mfma32(lds_row_operand<D>(do_tile, 32 * mb + i, 2 * kk + g), vreg[kk], dp);
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = __builtin_amdgcn_exp2f(fmaf(s[r], qk_scale, -colc));
    if (a_b0 < n_w0 + 31) {  // causal compare, only on blocks that cross the diagonal
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = (n > a_b0 + c_row(r, g)) ? 0.f : s[r];
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float ds = s[r] * dp[r];
      dp[r] = ds;
      csum += ds;
    }
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const u32x4 pb = pack8<Tr>(s, 8 * hh);
      const u32x4 dsb = pack8<Tr>(dp, 8 * hh);
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        dvacc[db] = Tr::mfma32(lds_col_operand<D>(do_tile, 32 * mb + 16 * hh, db0 + db, lane), pb, dvacc[db]);
        dkacc[db] = Tr::mfma32(lds_col_operand<D>(q_tile, 32 * mb + 16 * hh, db0 + db, lane), dsb, dkacc[db]);
      }
    }
  }
}

// Interior step (every query row of the step sits at or below every key of the
// tile: no causal compare, nothing to skip): branch-free and software-pipelined by
// hand, because the kernel holds one wave per SIMD and nobody else can fill the
// matrix pipe while this wave does its exp/scale arithmetic.  The step is cut
// into slots; slot b issues, interleaved in chunks of 4 MFMAs + 2 scores,
//   * the score MFMAs        S, dP   of block b+1,
//   * the vector arithmetic  P, dS   of block b,
//   * the accumulation MFMAs dV, dK  of block b-1,
// which are mutually independent (one MFMA, then a few vector instructions, four times per chunk, in source order
// between scheduling fences).  The global loads of the next tile are spread over
// the step as well (dma(k) issues the k-th of NDMA instructions): issued back to back
// after the barrier by all four waves they would hold every wave's issue slot, and
// with one wave per SIMD the matrix pipe, for over a thousand cycles per step.
// The LDS operands of a chunk are requested three
// chunks (about twelve MFMAs) ahead, across slot boundaries, so their latency hides
// behind the chunks in between.
template <typename Tr, int D, int NDMA, typename Dma>
__device__ __forceinline__ void dkdv_step_interior(const char* q_tile, const char* do_tile, const float* rc_s, const float* dl_s,
                                          const u32x4 (&kreg)[D / 16], const u32x4 (&vreg)[D / 16],
                                          f32x16 (&dkacc)[(D + 31) / 32], f32x16 (&dvacc)[(D + 31) / 32], float& csum,
                                          float qk_scale, float colc, int lane, Dma dma) {
  constexpr int BMQ = kKvBM, KK = D / 16, DB = (D + 31) / 32, MB = BMQ / 32;
  // chunks per slot: as many as the larger of the two MFMA groups needs (one k-step of S and dP, one accumulation
  // pair of dV and dK per chunk), so that every chunk carries matrix work; the 16 scores per lane of a block are
  // dealt out evenly over them
  constexpr int NCH = KK > 2 * DB ? KK : 2 * DB, SPC = 16 / NCH;
  static_assert(16 % NCH == 0 && (SPC == 2 || SPC == 4 || SPC == 8), "whole scores per chunk, whole operands per 8 scores");
  constexpr int NC = (MB + 2) * NCH;  // chunks of the step: slots -1 .. MB
  constexpr int PF = 3;               // LDS operands are requested this many chunks before their MFMAs
  constexpr int kDmaEvery = (NC - NCH) / (NDMA > 0 ? NDMA : 1) > 0 ? (NC - NCH) / (NDMA > 0 ? NDMA : 1) : 1;
  static_assert(NDMA * kDmaEvery <= NC - NCH, "every load instruction of the next tile finds a chunk");
  static_assert(KK <= NCH && 2 * DB <= NCH, "one k-step and one accumulation pair per chunk");
  const int g = lane >> 5, i = lane & 31;
  f32x16 s[MB], dp[MB];
  u32x4 pb[MB][2], dsb[MB][2];
  u32x4 aq[NC + PF], ado[NC + PF], cq[NC + PF], cdo[NC + PF];  // indexed by chunk; only a few are live at a time
  auto fetch = [&](auto ic) {
    constexpr int c = decltype(ic)::value;
    constexpr int slot = c / NCH - 1, u = c % NCH, bs = slot + 1, bc = slot - 1;
    if constexpr (c < NC && bs < MB && u < KK) {
      aq[c] = lds_row_operand<D>(q_tile, 32 * bs + i, 2 * u + g);
      ado[c] = lds_row_operand<D>(do_tile, 32 * bs + i, 2 * u + g);
    }
    if constexpr (c < NC && slot >= 1 && u < 2 * DB) {
      cdo[c] = lds_col_operand<D>(do_tile, 32 * bc + 16 * (u / DB), u % DB, lane);
      cq[c] = lds_col_operand<D>(q_tile, 32 * bc + 16 * (u / DB), u % DB, lane);
    }
  };
  // the accumulators of block b start from the row terms instead of zero; requested PF chunks early too
  auto init_block = [&](int b) {  // b is a constant at every call site
    if (b < MB) {
      s[b] = acc_init(rc_s, 32 * b, g);
      dp[b] = acc_init(dl_s, 32 * b, g);
    }
  };
  init_block(0);
  static_for<0, PF>([&](auto ic) { fetch(ic); });
  static_for<0, NC>([&](auto ic) {
    constexpr int c = decltype(ic)::value;
    constexpr int slot = c / NCH - 1, u = c % NCH;
    constexpr bool do_s = slot + 1 < MB, do_v = slot >= 0 && slot < MB, do_c = slot >= 1;
    constexpr int bs = slot + 1, bv = slot, bc = slot - 1;
    fetch(std::integral_constant<int, c + PF>{});
    if constexpr (u == (NCH > PF ? NCH - PF : 0)) init_block(bs + 1);
    // the next tile's load instructions, one every kDmaEvery chunks from the second slot on
    if constexpr (c >= NCH && (c - NCH) % kDmaEvery == 0 && (c - NCH) / kDmaEvery < NDMA)
      dma(std::integral_constant<int, (c - NCH) / kDmaEvery>{});
    // The chunk in issue order, every group fenced so that matrix and vector instructions alternate: S MFMA, exp2 of
    // SPC scores, dP MFMA, dS and the column sum of those scores, dV MFMA, pack P (when eight scores are complete),
    // dK MFMA, pack dS.  S and dP accumulate in VGPRs (mfma32_vgpr_acc), so this code keeps the distance between an
    // MFMA that writes s[b] / dp[b] and the first vector instruction that reads them (12 issued instructions).  Block
    // b's last S MFMA opens chunk NCH-1 of slot b-1 and its first score is read in chunk 0 of slot b, after that
    // chunk's S MFMA.  For b >= 1 the instructions in between are the 2*SPC exp2 / fma, the dP MFMA, the 2*SPC multiply
    // / add and the 8 packs of chunk NCH-1 (it completes eight scores), then the next chunk's operand requests and
    // S MFMA: >= 20.  dP's last MFMA is followed by 2*SPC + 8 of those, the requests, the S MFMA and 2*SPC exp2 / fma
    // before dS reads it: >= 18.  Block 0 is computed in a slot without vector work, so its first chunk of vector
    // work starts with explicit wait states.
    constexpr bool mf_s = do_s && u < KK, mf_c = do_c && u < 2 * DB;
    constexpr bool pack_due = do_v && (SPC * (u + 1)) % 8 == 0;   // eight scores complete: one MFMA operand each of P and dS
    constexpr int hh = pack_due ? SPC * (u + 1) / 8 - 1 : 0;
    static_assert(SPC >= 2 && NCH * SPC == 16, "the distances above count on at least two scores per chunk, eight per pack");
    if constexpr (mf_s) Tr::mfma32_vgpr_acc(s[bs], aq[c], kreg[u]);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (do_v && bv == 0 && u == 0) {
      asm volatile("s_nop 11");
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (do_v) {
#pragma unroll
      for (int e = 0; e < SPC; ++e) s[bv][SPC * u + e] = __builtin_amdgcn_exp2f(fmaf(s[bv][SPC * u + e], qk_scale, -colc));
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (mf_s) Tr::mfma32_vgpr_acc(dp[bs], ado[c], vreg[u]);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (do_v) {
#pragma unroll
      for (int e = 0; e < SPC; ++e) {
        const float ds = s[bv][SPC * u + e] * dp[bv][SPC * u + e];
        dp[bv][SPC * u + e] = ds;
        csum += ds;
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (mf_c) dvacc[u % DB] = Tr::mfma32(cdo[c], pb[bc][u / DB], dvacc[u % DB]);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (pack_due) pb[bv][hh] = pack8<Tr>(s[bv], 8 * hh);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (mf_c) dkacc[u % DB] = Tr::mfma32(cq[c], dsb[bc][u / DB], dkacc[u % DB]);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (pack_due) dsb[bv][hh] = pack8<Tr>(dp[bv], 8 * hh);
    __builtin_amdgcn_sched_barrier(0);
  });
}

// DSPLIT: the variant for key tiles that pruning leaves a few query steps (class kClassLight).  Such a workgroup
// is a short chain of loads, a few steps and stores; at one workgroup per CU nothing overlaps with it.  Here two
// waves share 32 keys, each recomputing S and dP and accumulating one half of the head dim of dK and dV, so that
// the kernel fits in 256 registers; a workgroup is 64 keys x 2 halves with query steps of 64 rows, and two
// workgroups (two waves per SIMD) share a CU.
template <typename Tr, int D, bool DSPLIT>
__global__ __launch_bounds__(256, (D <= 64 || DSPLIT) ? 2 : 1) void dkdv_kernel(const BwdK a) {
  constexpr int BN = DSPLIT ? 64 : kKvBN, BMQ = DSPLIT ? 64 : kKvBM;
  constexpr int KK = D / 16, DB = (D + 31) / 32, NDB = DSPLIT ? DB / 2 : DB, DW = DSPLIT ? D / 2 : D;
  static_assert(!DSPLIT || DB % 2 == 0, "the head dim splits into two halves of whole 32-column blocks");
  __shared__ __align__(16) char q_tile0[Tile<D>::bytes(BMQ)];
  __shared__ __align__(16) char q_tile1[Tile<D>::bytes(BMQ)];
  __shared__ __align__(16) char do_tile0[Tile<D>::bytes(BMQ)];
  __shared__ __align__(16) char do_tile1[Tile<D>::bytes(BMQ)];
  __shared__ __align__(16) float rc_s0[BMQ];
  __shared__ __align__(16) float rc_s1[BMQ];
  __shared__ __align__(16) float dl_s0[BMQ];
  __shared__ __align__(16) float dl_s1[BMQ];

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), g = lane >> 5, i = lane & 31;
  const int kb = DSPLIT ? wave >> 1 : wave;   // block of 32 keys this wave owns
  const int dh = DSPLIT ? wave & 1 : 0;       // half of the head dim it accumulates
  int bh, nt;
  decode_block(blockIdx.x, a.n_tiles, a.B * a.H, bh, nt);
  nt = a.n_tiles - 1 - nt;  // the first key tiles see the most query rows: start them first
  const int b = bh / a.H, h = bh % a.H;
  const int M = a.M, N = a.N, p_seq = N - M;
  const int n0 = nt * BN;
  const float* c_row = a.c + (int64_t)bh * N;
  if (a.cls != kClassAll) {  // the class of the 128-key tile this workgroup's keys belong to decides who handles them
    const int n_last = min(N - 1, (n0 / kKvBN) * kKvBN + kKvBN - 1);
    const bool light = acp_light_k(c_row, c_row[n_last], a.thr ? a.thr[bh] : 0.f, n_last, N, a.light_limit);
    if (light != (a.cls == kClassLight)) return;
  }
  const float* lse_row = a.lse + (int64_t)bh * M;
  const float* delta_row = a.delta + (int64_t)bh * M;
  const uint16_t* qp = a.q.ptr + b * a.q.sb + h * a.q.sh;
  const uint16_t* kp = a.k.ptr + b * a.k.sb + h * a.k.sh;
  const uint16_t* vp = a.v.ptr + b * a.v.sb + h * a.v.sh;
  const uint16_t* dop = a.d_o.ptr + b * a.d_o.sb + h * a.d_o.sh;
  uint16_t* dkp = const_cast<uint16_t*>(a.dk.ptr) + b * a.dk.sb + h * a.dk.sh;
  uint16_t* dvp = const_cast<uint16_t*>(a.dv.ptr) + b * a.dv.sb + h * a.dv.sh;

  int seq = 0;
  if (a.seq_start) {
    const int64_t s64 = a.seq_start[b];
    seq = (int)(s64 < 0 ? 0 : (s64 > N ? N : s64));
  }
  // query range: rows whose key position reaches this tile, up to the pruning bound
  int m_lo = max(n0 - p_seq, 0);
  m_lo = (m_lo / BMQ) * BMQ;
  const int n_w0 = n0 + 32 * kb;
  const int n = n_w0 + i;  // this lane's key row
  // Everything the workgroup needs first is requested before anything is waited for: the tile of the
  // first diagonal step (it does not depend on the pruning bound), K and V, then the per-row terms.
  const DirectTileLoader<D, BMQ> qld(a.q.st, wave, lane), dold(a.d_o.st, wave, lane);
  const bool early = m_lo < M && p_seq + m_lo < n0 + BN - 1 && !(n0 + BN <= seq);
  if (early) {
    qld.issue(qp, a.q.st, m_lo, M, q_tile1);
    dold.issue(dop, a.d_o.st, m_lo, M, do_tile1);
  }
  u32x4 kreg[KK], vreg[KK];
  // The split variant lives for two or three steps, so the way its K and V rows arrive counts: as register loads
  // every instruction touches 32 rows for 32 bytes each; as tile loads they come in whole rows, through buffer set 0
  // (free until the second step), and go from LDS to the registers like any row operand.
  constexpr bool kStageKV = DSPLIT;
  if constexpr (kStageKV) {
    static_assert(BN == BMQ, "the key rows of a workgroup fill one step tile");
    const DirectTileLoader<D, BN> kld(a.k.st, wave, lane), vld(a.v.st, wave, lane);
    kld.issue(kp, a.k.st, n0, N, q_tile0);
    vld.issue(vp, a.v.st, n0, N, do_tile0);
  } else {
    load_row_operand_regs<D>(kreg, kp, a.k.st, n, N, g);
    load_row_operand_regs<D>(vreg, vp, a.v.st, n, N, g);
  }
  const float c_ref = c_row[n0];
  const float c_key = c_row[min(n, N - 1)];
  const float c_last = c_row[min(N - 1, n0 + BN - 1)];  // for the pruning bound below
  const float qk_scale = nonzero_scale(a.sm_scale * kLog2e), inv_scale = 1.0f / qk_scale;

  // Per-row terms of a step: the loads are requested here, the arithmetic on them is done where the values
  // go to LDS (a step later), so that nothing waits for the loads in between.  Rows past M and empty rows
  // (lse = -inf) get -inf through the subtraction.
  // The BMQ rows of a step are dealt out evenly over the four waves (their first BMQ/4 lanes each), so that
  // no wave arrives late at the barrier because of them.
  const bool row_lane = lane < BMQ / 4;
  const int row_slot = wave * (BMQ / 4) + lane;
  float l_raw = 0.f, c_raw = 0.f, d_raw = 0.f;
  bool row_ok = false;
  auto issue_rows = [&](int ms) {
    if (row_lane) {
      const int mm = ms + row_slot, mc = min(mm, M - 1);
      row_ok = mm < M;
      l_raw = lse_row[mc];
      c_raw = c_row[p_seq + mc];
      d_raw = delta_row[mc];
    }
  };
  auto rc_term = [&]() {
    const float l_eff = (row_ok & (l_raw > -INFINITY)) ? l_raw : INFINITY;
    return (c_raw - c_ref - l_eff) * kLog2e * inv_scale;
  };
  auto dl_term = [&]() { return row_ok ? -d_raw : 0.f; };
  auto issue = [&](int ms, char* qt, char* dot) {
    issue_rows(ms);  // small loads first: vmcnt retires in order, so they must not queue behind the tile
    qld.issue(qp, a.q.st, ms, M, qt);
    dold.issue(dop, a.d_o.st, ms, M, dot);
  };
  if (early) issue_rows(m_lo);
  const float colc = (n < N && n >= seq) ? (c_key - c_ref) * kLog2e : INFINITY;

  f32x16 dkacc[NDB], dvacc[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dkacc[db][r] = 0.f; dvacc[db][r] = 0.f; }
  float csum = 0.f;


  int m_hi = M;
  if (a.thr) {
    const int U = (M + BMQ - 1) / BMQ;
    const int u = acp_first_pruned_qblock(c_row, c_last, a.thr[bh], p_seq, BMQ, m_lo / BMQ, U, lane);
    m_hi = min(M, u * BMQ);
  }
  if (n0 + BN <= seq) m_hi = m_lo;  // every key of the tile is left padding
  if (a.kv_end_row && tid < BN / kKvUnit && n0 + tid * kKvUnit < N)  // the bound this workgroup works with, for callers that check it
    a.kv_end_row[(int64_t)bh * ((N + kKvUnit - 1) / kKvUnit) + n0 / kKvUnit + tid] = m_hi;
  const int n_steps = m_hi > m_lo ? (m_hi - m_lo + BMQ - 1) / BMQ : 0;
  if constexpr (kStageKV) {
    wait_vmem_all();
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      kreg[kk] = lds_row_operand<D>(q_tile0, 32 * kb + i, 2 * kk + g);
      vreg[kk] = lds_row_operand<D>(do_tile0, 32 * kb + i, 2 * kk + g);
    }
    __syncthreads();   // buffer set 0 is free for the second step's tiles
  }

  // The long-loop kernel (head dim 128, one workgroup per CU).  Phase 1: the steps that touch the tile's
  // diagonal (at most BN/BMQ + 1 of them) run one at a
  // time through buffer 1 with the masking code; the first interior tile is requested into
  // buffer 0 before the last of them is computed.  Phase 2: interior steps, double-buffered,
  // from the end of the sequence down: the workgroups of one (batch, head) that run together on
  // an XCD then request the same Q / dO tile at about the same time, and all but the first
  // request hit that XCD's L2.
  int n_diag = 0;
  while (n_diag < n_steps && p_seq + m_lo + n_diag * BMQ < n0 + BN - 1) ++n_diag;
  const int n_int = n_steps - n_diag, m_top = m_lo + (n_steps - 1) * BMQ;
  if constexpr (D <= 64 || DSPLIT) {
    // Small head dims (and the split variant) leave room for two workgroups per CU: the second wave on each SIMD
    // fills the matrix pipe while the first does its vector work, so every step takes the plain code path.  The
    // steps, diagonal ones first (upwards from m_lo), then the interior ones (downwards from m_top), alternate
    // between the two buffer sets, starting with set 1 (which the early request above has filled): the next step's
    // tiles are requested before the current one is computed.
    auto step_rows = [&](int idx) { return idx < n_diag ? m_lo + idx * BMQ : m_top - (idx - n_diag) * BMQ; };
    if (n_steps > 0) {
      if (!early) issue(step_rows(0), q_tile1, do_tile1);
      if (row_lane) { rc_s1[row_slot] = rc_term(); dl_s1[row_slot] = dl_term(); }
    }
    for (int idx = 0; idx < n_steps; ++idx) {
      const bool odd = idx & 1;
      wait_vmem_all();
      __syncthreads();
      if (idx + 1 < n_steps) issue(step_rows(idx + 1), odd ? q_tile1 : q_tile0, odd ? do_tile1 : do_tile0);
      dkdv_step<Tr, D, BMQ, NDB>(odd ? q_tile0 : q_tile1, odd ? do_tile0 : do_tile1, odd ? rc_s0 : rc_s1, odd ? dl_s0 : dl_s1, kreg,
                                 vreg, dkacc, dvacc, csum, p_seq + step_rows(idx), n, n_w0, qk_scale, colc, lane, dh * NDB);
      if (idx + 1 < n_steps && row_lane) {
        (odd ? rc_s1 : rc_s0)[row_slot] = rc_term();
        (odd ? dl_s1 : dl_s0)[row_slot] = dl_term();
      }
    }
  } else {
  for (int t = 0; t < n_diag; ++t) {
    const int ms = m_lo + t * BMQ;
    if (!(early && t == 0)) {
      __syncthreads();  // buffer 1 is free again
      issue(ms, q_tile1, do_tile1);
    }
    if (row_lane) { rc_s1[row_slot] = rc_term(); dl_s1[row_slot] = dl_term(); }
    wait_vmem_all();
    __syncthreads();
    if (t == n_diag - 1 && n_int > 0) issue(m_top, q_tile0, do_tile0);
    dkdv_step<Tr, D, BMQ, NDB>(q_tile1, do_tile1, rc_s1, dl_s1, kreg, vreg, dkacc, dvacc, csum, p_seq + ms, n, n_w0, qk_scale, colc,
                               lane, dh * NDB);
  }
  if (n_int > 0) {
    if (n_diag == 0) issue(m_top, q_tile0, do_tile0);
    if (row_lane) { rc_s0[row_slot] = rc_term(); dl_s0[row_slot] = dl_term(); }
  }
  constexpr int PER = DirectTileLoader<D, BMQ>::PER;
  // Every tile below the first interior one is a whole tile, so the source of the loads a step spreads over its chunks
  // is a pointer that moves back by one tile per step and an extent that is either a whole tile's or, when there is no
  // next tile, zero (the loads then write zeros into the free buffer): no address arithmetic per step beyond that.
  const int64_t q_back = (int64_t)BMQ * a.q.st, do_back = (int64_t)BMQ * a.d_o.st;
  const int q_whole = qld.extent(a.q.st, 0, BMQ), do_whole = dold.extent(a.d_o.st, 0, BMQ);
  const uint16_t *q_next = qp + (int64_t)(m_top - BMQ) * a.q.st, *do_next = dop + (int64_t)(m_top - BMQ) * a.d_o.st;
  for (int t = 0; t < n_int; t += 2) {
    wait_vmem_all();
    __syncthreads();
    {  // tile t from buffers 0; tile t+1 (if any) into buffers 1
      const bool more = t + 1 < n_int;
      if (more) issue_rows(m_top - (t + 1) * BMQ);
      const int q_bytes = more ? q_whole : 0, do_bytes = more ? do_whole : 0;
      dkdv_step_interior<Tr, D, 2 * PER>(q_tile0, do_tile0, rc_s0, dl_s0, kreg, vreg, dkacc, dvacc, csum, qk_scale, colc, lane, [&](auto k) {
        constexpr int K = decltype(k)::value;
        if constexpr (K < PER) qld.issue_one(K, q_next, q_bytes, q_tile1);
        else dold.issue_one(K - PER, do_next, do_bytes, do_tile1);
      });
      q_next -= q_back;
      do_next -= do_back;
    }
    if (t + 1 >= n_int) break;
    if (row_lane) { rc_s1[row_slot] = rc_term(); dl_s1[row_slot] = dl_term(); }
    wait_vmem_all();
    __syncthreads();
    {
      const bool more = t + 2 < n_int;
      if (more) issue_rows(m_top - (t + 2) * BMQ);
      const int q_bytes = more ? q_whole : 0, do_bytes = more ? do_whole : 0;
      dkdv_step_interior<Tr, D, 2 * PER>(q_tile1, do_tile1, rc_s1, dl_s1, kreg, vreg, dkacc, dvacc, csum, qk_scale, colc, lane, [&](auto k) {
        constexpr int K = decltype(k)::value;
        if constexpr (K < PER) qld.issue_one(K, q_next, q_bytes, q_tile0);
        else dold.issue_one(K - PER, do_next, do_bytes, do_tile0);
      });
      q_next -= q_back;
      do_next -= do_back;
      if (more && row_lane) { rc_s0[row_slot] = rc_term(); dl_s0[row_slot] = dl_term(); }
    }
  }

  }
  wait_vmem_all();  // whatever was requested last (possibly an empty tile) has landed before the buffers are reused
  const float ctot = half_sum(csum);
  // gradient w.r.t. the cumulative sum: the row sum the dQ kernel left for the query row that sits at this key
  // position (none left of the first query row) minus this key's column sum
  if (n < N && g == 0 && dh == 0) {  // (the two waves of a split pair hold the same column sums)
    const float rtot = n >= p_seq ? a.drow[(int64_t)bh * M + (n - p_seq)] : 0.f;
    a.dc[(int64_t)bh * N + n] = rtot - ctot;
  }
  // dK and dV leave through LDS (the tile buffers are free now) so that the global stores are whole rows (of the
  // wave's DW columns)
  static_assert(2 * kStoreStageBytes<DW> <= Tile<D>::bytes(BMQ), "two waves stage in one tile buffer");
  __syncthreads();  // every wave is done with the tiles of the last step
  char* stage = (wave < 2 ? q_tile0 : do_tile0) + (wave & 1) * kStoreStageBytes<DW>;
  store_rows_via_lds<Tr, DW>(stage, dkacc, a.sm_scale, dkp + dh * DW, a.dk.st, n_w0, N, lane);
  store_rows_via_lds<Tr, DW>(stage, dvacc, 1.0f, dvp + dh * DW, a.dv.st, n_w0, N, lane);
}

// ---------------------------------------------------------------------------
// One 64-key tile of the dQ kernel for one wave (32 query rows).
// cn_s holds -colc_j / (sm_scale*log2e), the start value of the score accumulators.
template <typename Tr, int D>
__device__ __forceinline__ void dq_tile(const char* k_tile, const char* v_tile, const float* cn_s, const u32x4 (&qreg)[D / 16],
                               const u32x4 (&doreg)[D / 16], f32x16 (&dqacc)[(D + 31) / 32], float& rsum, int n0, int a_m,
                               int a_w0, float qk_scale, float rowc, float delta, int lane) {
  constexpr int BN = kFwdBN, KK = D / 16, DB = (D + 31) / 32, NB = BN / 32;
  const int g = lane >> 5, i = lane & 31;
  // dP starts from -delta (constant along a query row, i.e. per lane) instead of zero: the matrix pipe does the
  // subtraction.  The sixteen equal registers are loop-invariant for the caller.
  f32x16 neg_delta;
#pragma unroll
  for (int r = 0; r < 16; ++r) neg_delta[r] = -delta;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int nb0 = n0 + 32 * nb;
    if (nb0 > a_w0 + 31) continue;  // block entirely above this wave's rows
    f32x16 s = acc_init(cn_s, 32 * nb, g);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) s = Tr::mfma32(lds_row_operand<D>(k_tile, 32 * nb + i, 2 * kk + g), qreg[kk], s);
    f32x16 dp = Tr::mfma32(lds_row_operand<D>(v_tile, 32 * nb + i, g), doreg[0], neg_delta);
#pragma unroll
    for (int kk = 1; kk < KK; ++kk) dp = Tr::mfma32(lds_row_operand<D>(v_tile, 32 * nb + i, 2 * kk + g), doreg[kk], dp);
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = __builtin_amdgcn_exp2f(fmaf(s[r], qk_scale, rowc));
    if (nb0 + 31 > a_w0) {  // causal compare, only on blocks that cross the diagonal
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = (nb0 + c_row(r, g) > a_m) ? 0.f : s[r];
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float ds = s[r] * dp[r];
      dp[r] = ds;
      rsum += ds;
    }
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const u32x4 dsb = pack8<Tr>(dp, 8 * hh);
#pragma unroll
      for (int db = 0; db < DB; ++db)
        dqacc[db] = Tr::mfma32(lds_col_operand<D>(k_tile, 32 * nb + 16 * hh, db, lane), dsb, dqacc[db]);
    }
  }
}

template <typename Tr, int D>
__global__ __launch_bounds__(256, 2) void dq_kernel(const BwdK a) {
  constexpr int BM = kFwdBM, BN = kFwdBN;
  constexpr int KK = D / 16, DB = (D + 31) / 32;
  __shared__ __align__(16) char k_tile0[Tile<D>::bytes(BN)];
  __shared__ __align__(16) char k_tile1[Tile<D>::bytes(BN)];
  __shared__ __align__(16) char v_tile0[Tile<D>::bytes(BN)];
  __shared__ __align__(16) char v_tile1[Tile<D>::bytes(BN)];
  __shared__ __align__(16) float cn_s0[BN];
  __shared__ __align__(16) float cn_s1[BN];

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), g = lane >> 5, i = lane & 31;
  int bh, mt;
  decode_block(blockIdx.x, a.n_tiles, a.B * a.H, bh, mt);
  const int b = bh / a.H, h = bh % a.H;
  const int M = a.M, N = a.N, p_seq = N - M;
  const int m0 = mt * BM;
  const float* c_row = a.c + (int64_t)bh * N;
  const uint16_t* qp = a.q.ptr + b * a.q.sb + h * a.q.sh;
  const uint16_t* kp = a.k.ptr + b * a.k.sb + h * a.k.sh;
  const uint16_t* vp = a.v.ptr + b * a.v.sb + h * a.v.sh;
  const uint16_t* dop = a.d_o.ptr + b * a.d_o.sb + h * a.d_o.sh;
  const uint16_t* op = a.o.ptr + b * a.o.sb + h * a.o.sh;
  uint16_t* dqp = const_cast<uint16_t*>(a.dq.ptr) + b * a.dq.sb + h * a.dq.sh;

  const int a0 = p_seq + m0;
  const int hi = min(N, a0 + BM);
  int seq = 0;
  if (a.seq_start) {
    const int64_t s64 = a.seq_start[b];
    seq = (int)(s64 < 0 ? 0 : (s64 > N ? N : s64));
  }
  const int m = m0 + 32 * wave + i;
  const int a_m = p_seq + m;
  const int a_w0 = a0 + 32 * wave;
  const float qk_scale = nonzero_scale(a.sm_scale * kLog2e), inv_scale = 1.0f / qk_scale;
  // Everything the workgroup needs first is requested before anything is waited for: the first tile to
  // visit (it does not depend on the pruning bound), Q and dO, then the per-row and per-key terms.
  const DirectTileLoader<D, BN> kld(a.k.st, wave, lane), vld(a.v.st, wave, lane);
  const int n0_first = hi > 0 ? ((hi - 1) / BN) * BN : 0;
  const bool early = hi > (min(seq, hi) / BN) * BN;
  // The tile before it as well, when neither the pruning bound (it never cuts right of the first row's own
  // position) nor seq_start can exclude it: under pruning a workgroup visits two or three tiles, and every round
  // trip taken out of that chain counts.
  const int n0_second = n0_first - BN;
  const bool early2 = early && n0_second >= (a0 / BN) * BN && n0_second >= (min(seq, hi) / BN) * BN;
  if (early) {
    kld.issue(kp, a.k.st, n0_first, N, k_tile0);
    vld.issue(vp, a.v.st, n0_first, N, v_tile0);
  }
  if (early2) {
    kld.issue(kp, a.k.st, n0_second, N, k_tile1);
    vld.issue(vp, a.v.st, n0_second, N, v_tile1);
  }
  u32x4 qreg[KK], doreg[KK], oreg[KK];
  load_row_operand_regs<D>(qreg, qp, a.q.st, m, M, g);
  load_row_operand_regs<D>(doreg, dop, a.d_o.st, m, M, g);
  load_row_operand_regs<D>(oreg, op, a.o.st, m, M, g);
  const float c_ref = c_row[a0];
  const int mc = min(m, M - 1);
  const float l = a.lse[(int64_t)bh * M + mc], c_m = c_row[min(p_seq + mc, N - 1)];

  // Key terms of a tile: the load is requested here, the arithmetic on it is done where the value goes to
  // LDS (a tile later), so that nothing waits for the load in between.  Masked keys get -inf through the
  // subtraction.
  float cn_raw = 0.f;
  bool cn_ok = false;
  auto issue_cn = [&](int n0) {
    if (tid < BN) {
      const int nn = n0 + tid;
      cn_ok = (nn < N) & (nn >= seq);
      cn_raw = c_row[min(nn, N - 1)];
    }
  };
  auto cn_term = [&]() { return (c_ref - (cn_ok ? cn_raw : INFINITY)) * kLog2e * inv_scale; };
  auto issue = [&](int n0, char* kt, char* vt) {
    issue_cn(n0);  // small load first: vmcnt retires in order, so it must not queue behind the tile loads
    kld.issue(kp, a.k.st, n0, N, kt);
    vld.issue(vp, a.v.st, n0, N, vt);
  };
  if (early) issue_cn(n0_first);
  float cn_raw2 = 0.f;   // key terms of the second early tile: handed to cn_raw once the first tile's are in LDS
  bool cn_ok2 = false;
  if (early2 && tid < BN) {
    const int nn = n0_second + tid;
    cn_ok2 = (nn < N) & (nn >= seq);
    cn_raw2 = c_row[min(nn, N - 1)];
  }

  // The pruning bound: its loads are the last to join the ones above, and the search's first wait is the wait for
  // all of them.  Nothing before this point waits for a load: one round trip covers the whole prologue.
  int lo = min(seq, hi);
  if (a.thr) {
    const int t = acp_first_kept_block(c_row, c_ref, a.thr[bh], N, BN, a0 / BN, lane);
    lo = max(lo, t * BN);
  }
  lo = (lo / BN) * BN;
  if (a.q_first_block && tid == 0) a.q_first_block[(int64_t)bh * a.n_tiles + mt] = lo / BN;
  const int n_tiles = (hi - lo + BN - 1) / BN;

  // rows past M and empty rows (lse = -inf) get rowc = -inf through the subtraction: no load behind a branch
  const float l_eff = ((m < M) & (l > -INFINITY)) ? l : INFINITY;
  const float rowc = (c_m - c_ref - l_eff) * kLog2e;
  // delta_i = sum_d o_id * do_id (_bwd_preprocess of the reference, :902-943) for this lane's row: each half of
  // the wave holds half of the row's elements.  Rows past M were loaded as zeros.  Stored for the dK/dV kernel.
  float delta;
  {
    float part = 0.f;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        part += Tr::lo(oreg[kk][e]) * Tr::lo(doreg[kk][e]) + Tr::hi(oreg[kk][e]) * Tr::hi(doreg[kk][e]);
    delta = half_sum(part);
    if (m < M && g == 0) a.delta[(int64_t)bh * M + m] = delta;
  }

  f32x16 dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) dqacc[db][r] = 0.f;
  float rsum = 0.f;

  const bool wave_has_rows = m0 + 32 * wave < M;  // a wave without query rows only moves tiles
  auto compute = [&](int n0, const char* kt, const char* vt, const float* cn) {
    if (!wave_has_rows) return;
    dq_tile<Tr, D>(kt, vt, cn, qreg, doreg, dqacc, rsum, n0, a_m, a_w0, qk_scale, rowc, delta, lane);
  };

  auto tile_n0 = [&](int t) { return lo + t * BN; };   // start of the tile at loop position t
  if (n_tiles > 0) {
    if (!early) issue(tile_n0(n_tiles - 1), k_tile0, v_tile0);
    if (tid < BN) cn_s0[tid] = cn_term();
    if (early2) { cn_raw = cn_raw2; cn_ok = cn_ok2; }
  }
  bool requested = early2;  // buffers 1 already hold (or await) the next tile
  for (int t = n_tiles - 1; t >= 0; t -= 2) {
    wait_vmem_all();
    __syncthreads();
    if (t >= 1 && !requested) issue(tile_n0(t - 1), k_tile1, v_tile1);
    requested = false;
    compute(tile_n0(t), k_tile0, v_tile0, cn_s0);
    if (t < 1) break;
    if (tid < BN) cn_s1[tid] = cn_term();
    wait_vmem_all();
    __syncthreads();
    if (t >= 2) issue(tile_n0(t - 2), k_tile0, v_tile0);
    compute(tile_n0(t - 1), k_tile1, v_tile1, cn_s1);
    if (t >= 2 && tid < BN) cn_s0[tid] = cn_term();
  }

  const float rtot = half_sum(rsum);
  if (m < M && g == 0) a.drow[(int64_t)bh * M + m] = rtot;  // the dK/dV kernel, next on this stream, folds it into dc
  // dQ leaves through LDS (the tile buffers are free now, one per wave) so that the global stores are whole rows
  static_assert(kStoreStageBytes<D> <= Tile<D>::bytes(BN), "one wave stages in one tile buffer");
  __syncthreads();  // every wave is done with the last tile
  char* stage = wave == 0 ? k_tile0 : wave == 1 ? k_tile1 : wave == 2 ? v_tile0 : v_tile1;
  store_rows_via_lds<Tr, D>(stage, dqacc, a.sm_scale, dqp, a.dq.st, m0 + 32 * wave, M, lane);
}

// explicit instantiations: every (dtype, head dim) pair the dispatchers can reach
#define FOX_INSTANTIATE_BWD(KERNEL, TR)                      \
  template __global__ void KERNEL<TR, 16>(const BwdK);       \
  template __global__ void KERNEL<TR, 32>(const BwdK);       \
  template __global__ void KERNEL<TR, 64>(const BwdK);       \
  template __global__ void KERNEL<TR, 128>(const BwdK);
FOX_INSTANTIATE_BWD(delta_kernel, Bf16)
FOX_INSTANTIATE_BWD(delta_kernel, Fp16)
#define FOX_INSTANTIATE_DKDV(TR)                                     \
  template __global__ void dkdv_kernel<TR, 16, false>(const BwdK);   \
  template __global__ void dkdv_kernel<TR, 32, false>(const BwdK);   \
  template __global__ void dkdv_kernel<TR, 64, false>(const BwdK);   \
  template __global__ void dkdv_kernel<TR, 128, false>(const BwdK);  \
  template __global__ void dkdv_kernel<TR, 128, true>(const BwdK);
FOX_INSTANTIATE_DKDV(Bf16)
FOX_INSTANTIATE_DKDV(Fp16)
FOX_INSTANTIATE_BWD(dq_kernel, Bf16)
FOX_INSTANTIATE_BWD(dq_kernel, Fp16)

// ---------------------------------------------------------------------------
#define FOX_DISPATCH_D(KERNEL, GRID, SMEM)                                                        \
  switch (D) {                                                                                    \
    case 16: hipLaunchKernelGGL((KERNEL<Tr, 16>), GRID, dim3(256), SMEM, s, a); break;            \
    case 32: hipLaunchKernelGGL((KERNEL<Tr, 32>), GRID, dim3(256), SMEM, s, a); break;            \
    case 64: hipLaunchKernelGGL((KERNEL<Tr, 64>), GRID, dim3(256), SMEM, s, a); break;            \
    case 128: hipLaunchKernelGGL((KERNEL<Tr, 128>), GRID, dim3(256), SMEM, s, a); break;          \
    default: return hipErrorInvalidValue;                                                         \
  }

template <typename Tr>
static hipError_t delta_t(const BwdK& a, int D, hipStream_t s) {
  const dim3 grid((unsigned)((a.M + 127) / 128), (unsigned)(a.B * a.H));
  FOX_DISPATCH_D(delta_kernel, grid, 0)
  return hipGetLastError();
}
template <typename Tr>
static hipError_t dkdv_t(const BwdK& a0, int D, hipStream_t s) {
  BwdK a = a0;
  if (a.cls == kClassLight) {  // the split variant: 64 keys per workgroup
    if (!dkdv_split_supports(D)) return hipErrorInvalidValue;
    a.n_tiles = (a.N + 63) / 64;
    hipLaunchKernelGGL((dkdv_kernel<Tr, 128, true>), dim3((unsigned)(a.n_tiles * a.B * a.H)), dim3(256), 0, s, a);
    return hipGetLastError();
  }
  a.n_tiles = (a.N + kKvBN - 1) / kKvBN;
  const dim3 grid((unsigned)(a.n_tiles * a.B * a.H));
  switch (D) {
    case 16: hipLaunchKernelGGL((dkdv_kernel<Tr, 16, false>), grid, dim3(256), 0, s, a); break;
    case 32: hipLaunchKernelGGL((dkdv_kernel<Tr, 32, false>), grid, dim3(256), 0, s, a); break;
    case 64: hipLaunchKernelGGL((dkdv_kernel<Tr, 64, false>), grid, dim3(256), 0, s, a); break;
    case 128: hipLaunchKernelGGL((dkdv_kernel<Tr, 128, false>), grid, dim3(256), 0, s, a); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}
template <typename Tr>
static hipError_t dq_t(const BwdK& a0, int D, hipStream_t s) {
  BwdK a = a0;
  a.n_tiles = (a.M + kFwdBM - 1) / kFwdBM;
  const dim3 grid((unsigned)(a.n_tiles * a.B * a.H));
  FOX_DISPATCH_D(dq_kernel, grid, 0)
  return hipGetLastError();
}

bool dkdv_split_supports(int D) { return D == 128; }

hipError_t launch_bwd_delta(const BwdK& a, int D, int dtype, hipStream_t s) {
  return dtype == 0 ? delta_t<Bf16>(a, D, s) : delta_t<Fp16>(a, D, s);
}
hipError_t launch_bwd_dkdv(const BwdK& a, int D, int dtype, hipStream_t s) {
  return dtype == 0 ? dkdv_t<Bf16>(a, D, s) : dkdv_t<Fp16>(a, D, s);
}
hipError_t launch_bwd_dq(const BwdK& a, int D, int dtype, hipStream_t s) {
  return dtype == 0 ? dq_t<Bf16>(a, D, s) : dq_t<Fp16>(a, D, s);
}

}  // namespace fox
