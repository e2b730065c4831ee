// Forward kernel of Forgetting Attention for gfx950.
//
// One workgroup (4 waves) owns 128 query rows of one (batch, head); wave w owns
// rows 32w..32w+31 and keeps them in registers as the B operand of
// S^T = K Q^T (32x32x16 MFMA).  With the scores transposed, lane (g, i) holds one
// query row i and 16 key columns per 32-column block, so the online-softmax row
// statistics are lane-local plus one exchange between the two 32-lane halves, and
// the probabilities are already laid out as the B operand of O^T = V^T P^T.
//
// K and V tiles of 64 keys go from HBM straight into LDS (buffer loads with the
// LDS bit: no registers, no ds_write; out-of-range rows read as zero), into two
// alternating buffers, so the loads of the next tile fly while the current one is
// consumed and there is one barrier per tile.  V^T is read with the transposing
// LDS load.
// When a (batch, head) has a single query tile nobody reads a K or V tile twice, and the
// loads carry the non-temporal hint (the STREAM instantiation).
//
// Key tiles are walked from the diagonal backwards.  Under a forget gate the
// scores shrink with distance, so the running row maximum is set by the first
// tiles; it is only raised when a tile exceeds it by more than 2^8, which keeps
// every exponent <= 8 (exact in fp32/bf16 terms, the factor cancels in o = acc/l)
// and makes the rescale of the accumulator a rare, wave-uniform branch.
//
// The decay bias enters relative to c_ref = c[first query row of the tile]:
//   x = (q.k) * sm_scale*log2e - (c_n - c_ref)*log2e          (per score)
// and the row term (c_m - c_ref)*log2e, constant along a row, is only added to the
// stored log-normaliser.  Columns left of seq_start (and beyond N) get
// (c_n - c_ref) = +inf, which makes x = -inf without a compare in the loop; only
// tiles crossing the diagonal run the causal compare (separate code path).
#include <stddef.h>

#include "fox_common.hpp"
#include "fox_kernels.hpp"

namespace fox {

constexpr float kLazyMaxLog2 = 8.0f;
constexpr int kMinPipelinedTiles = 4;   // interior tiles below which the software-pipelined path is not entered

template <typename Tr, int D>
__device__ __forceinline__ void fwd_tile(const char* k_tile, const char* v_tile, const float* cn_s, const u32x4 (&qreg)[D / 16],
                                f32x16 (&oacc)[(D + 31) / 32], float& m_i, float& l_i, int n0, int a_m, float qk_scale,
                                int lane, bool diag) {
  constexpr int BN = kFwdBN, KK = D / 16, DB = (D + 31) / 32, NB = BN / 32;
  const int g = lane >> 5, i = lane & 31;

  // S^T = K Q^T + key term
  f32x16 s[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    u32x4 ka[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) ka[kk] = lds_row_operand<D>(k_tile, 32 * nb + i, 2 * kk + g);
    s[nb] = acc_init(cn_s, 32 * nb, g);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) s[nb] = Tr::mfma32(ka[kk], qreg[kk], s[nb]);
  }

  // scores in the log2 domain and their maximum
  float mloc = -INFINITY;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int r = 0; r < 16; ++r) s[nb][r] *= qk_scale;
  if (diag) {  // causal compare, only on tiles that cross the diagonal
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int n = n0 + 32 * nb + c_row(r, g);
        s[nb][r] = (n > a_m) ? -INFINITY : s[nb][r];
      }
  }
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int r = 0; r < 16; ++r) mloc = fmaxf(mloc, s[nb][r]);
  mloc = half_max(mloc);
  const bool raise = mloc > m_i + kLazyMaxLog2;
  if (__any(raise)) {  // rare: rescale what has been accumulated so far
    const float m_new = raise ? mloc : m_i;
    const float alpha = __builtin_amdgcn_exp2f(m_i - m_new);
    m_i = m_new;
    l_i *= alpha;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
  }
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int r = 0; r < 16; ++r) s[nb][r] = __builtin_amdgcn_exp2f(s[nb][r] - m_i);

  // O^T += V^T P^T.  The row sum is taken over the probabilities as rounded for the MFMA (the weights that
  // multiply V then add up to exactly l), two at a time: per-lane partial sum, the two halves are added in the epilogue.
  float rsum = 0.f;
#pragma unroll
  for (int sl = 0; sl < BN / 16; ++sl) {
    const u32x4 pb = pack8<Tr>(s[sl >> 1], 8 * (sl & 1));
#pragma unroll
    for (int e = 0; e < 4; ++e) rsum = Tr::add_pair(pb[e], rsum);
    u32x4 va[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) va[db] = lds_col_operand<D>(v_tile, 16 * sl, db, lane);
#pragma unroll
    for (int db = 0; db < DB; ++db) oacc[db] = Tr::mfma32(va[db], pb, oacc[db]);
  }
  l_i += rsum;
}

// Interior tile (no key of the tile is right of any query row of the workgroup): branch-free and
// software-pipelined across tiles.  While the vector ALU turns the scores of the current tile into
// probabilities, the matrix pipe already computes the scores of the next tile (from k_next) and then
// accumulates the current tile's P V (from v_cur).  s_cur holds the raw scores of the current tile
// on entry; s_next holds those of the next tile on exit.  Work is issued in small chunks separated
// by scheduling fences so that MFMA and vector instructions alternate in the instruction stream.
// dma(u) issues chunk u's share of the global loads of the tiles after next: spread over the tile they
// do not hold the wave's issue slot back to back right after the barrier.
template <typename Tr, int D, typename Dma>
__device__ __forceinline__ void fwd_tile_pipelined(const char* k_next, const char* v_cur, const float* cn_next,
                                                  const u32x4 (&qreg)[D / 16], f32x16 (&oacc)[(D + 31) / 32], float& m_i,
                                                  float& l_i, float qk_scale, int lane, f32x16 (&s_cur)[kFwdBN / 32],
                                                  f32x16 (&s_next)[kFwdBN / 32], Dma dma) {
  constexpr int BN = kFwdBN, KK = D / 16, DB = (D + 31) / 32, NB = BN / 32, NSL = BN / 16;
  constexpr int SPC = 16 * NB / KK;  // scores handled per chunk of phase A
  static_assert(16 * NB % KK == 0 && SPC % 4 == 0, "whole float4 groups of scores per chunk");
  const int g = lane >> 5, i = lane & 31;

  // Phase A: scores of the next tile  ||  maximum of the current tile's raw scores (sm_scale > 0 here)
  float mloc = -INFINITY;
  u32x4 ka[NB][KK + 1];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    ka[nb][0] = lds_row_operand<D>(k_next, 32 * nb + i, g);
    s_next[nb] = acc_init(cn_next, 32 * nb, g);
  }
  static_for<0, KK>([&](auto uc) {
    constexpr int u = decltype(uc)::value;
    dma(u);  // this chunk's share of the global loads of the tiles after next
    if constexpr (u + 1 < KK) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) ka[nb][u + 1] = lds_row_operand<D>(k_next, 32 * nb + i, 2 * (u + 1) + g);
    }
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) s_next[nb] = Tr::mfma32(ka[nb][u], qreg[u], s_next[nb]);
#pragma unroll
    for (int e = 0; e < SPC; ++e) {
      const int idx = u * SPC + e;
      mloc = fmaxf(mloc, s_cur[idx >> 4][idx & 15]);
    }
#pragma unroll
    for (int k = 0; k < NB; ++k) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, (SPC / 2 + NB - 1) / NB, 0);  // the chunk's v_max3 dealt out over its MFMAs
    }
    __builtin_amdgcn_sched_barrier(0);
  });
  mloc = half_max(mloc) * qk_scale;
  const bool raise = mloc > m_i + kLazyMaxLog2;
  if (__any(raise)) {  // rare: rescale what has been accumulated so far
    const float m_new = raise ? mloc : m_i;
    const float alpha = __builtin_amdgcn_exp2f(m_i - m_new);
    m_i = m_new;
    l_i *= alpha;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
  }

  // Phase B: p = exp2(s*scale - m), row sums, pack  ||  O^T += V^T P^T, one 16-key slice behind
  const float neg_m = -m_i;
  float rsum = 0.f;
  u32x4 pb[NSL];
  u32x4 va[NSL][DB];
#pragma unroll
  for (int c = 0; c <= NSL; ++c) {
    if (c < NSL) {
#pragma unroll
      for (int db = 0; db < DB; ++db) va[c][db] = lds_col_operand<D>(v_cur, 16 * c, db, lane);
    }
    if (c >= 1) {
#pragma unroll
      for (int db = 0; db < DB; ++db) oacc[db] = Tr::mfma32(va[c - 1][db], pb[c - 1], oacc[db]);
    }
    if (c < NSL) {
      const int nb = c >> 1, r0 = 8 * (c & 1);
#pragma unroll
      for (int e = 0; e < 8; ++e) s_cur[nb][r0 + e] = __builtin_amdgcn_exp2f(fmaf(s_cur[nb][r0 + e], qk_scale, neg_m));
      pb[c] = pack8<Tr>(s_cur[nb], r0);
#pragma unroll
      for (int e = 0; e < 4; ++e) rsum = Tr::add_pair(pb[c][e], rsum);  // row sum of the rounded probabilities
    }
    if (c >= 1 && c < NSL) {
#pragma unroll
      for (int k = 0; k < DB; ++k) {  // a slice has 16 vector and 8 exp instructions: dealt out over its DB MFMAs
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 16 / DB, 0);
        __builtin_amdgcn_sched_group_barrier(0x400, 8 / DB, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  l_i += rsum;
}

// The global loads of a K tile and a V tile, dealt out over the D/16 chunks of a pipelined tile:
// dma(u) issues chunk u's share.
template <int D, int AUX>
struct TileDma {
  static constexpr int KK = D / 16, PER = DirectTileLoader<D, kFwdBN, 4, AUX>::PER, PER_CHUNK = (2 * PER + KK - 1) / KK;
  const DirectTileLoader<D, kFwdBN, 4, AUX>& kld;
  const DirectTileLoader<D, kFwdBN, 4, AUX>& vld;
  const uint16_t* k_src;
  const uint16_t* v_src;
  int k_bytes, v_bytes;
  char* k_fill;
  char* v_fill;
  __device__ __forceinline__ void all() const {
#pragma unroll
    for (int j = 0; j < PER; ++j) kld.issue_one(j, k_src, k_bytes, k_fill);
#pragma unroll
    for (int j = 0; j < PER; ++j) vld.issue_one(j, v_src, v_bytes, v_fill);
  }
  __device__ __forceinline__ void operator()(int u) const {  // u is a constant at every call site
#pragma unroll
    for (int r = 0; r < PER_CHUNK; ++r) {
      const int idx = u * PER_CHUNK + r;
      if (idx < PER) kld.issue_one(idx, k_src, k_bytes, k_fill);
      else if (idx < 2 * PER) vld.issue_one(idx - PER, v_src, v_bytes, v_fill);
    }
  }
};

// EPI: the variant whose epilogue also applies the layer's output norm and gate (a.epi); a variant of its own so
// that the plain kernel's register allocation is not touched by it.
// Waves per SIMD the forward is compiled for: the register budget that goes with it (512 / waves) holds the
// kernel to the occupancy its head dim allows.
template <int D>
constexpr int kFwdWaves = D <= 64 ? 3 : 2;

// STREAM: the variant for shapes with a single query tile per (batch, head): every K and V tile is read by exactly one
// workgroup, so the tile loads carry the non-temporal hint (with it the chunked-prefill shape B16 M128 N32768 H16 D128
// takes 0.62 ms instead of 0.71).  Where tiles are shared by the workgroups of several query tiles the hint costs 16-28 %.
template <typename Tr, int D, bool SPLIT, bool EPI = false, bool STREAM = false>
__global__ __launch_bounds__(256, kFwdWaves<D>) void fwd_kernel(const FwdK a) {
  static_assert(!(SPLIT && EPI), "partial results of a key split are not normalised");
  static_assert(!(STREAM && EPI), "no streaming variant with the epilogue");
  constexpr int AUX = STREAM ? kLoadNonTemporal : 0;
  constexpr int BM = kFwdBM, BN = kFwdBN;
  constexpr int KK = D / 16, DB = (D + 31) / 32, NB = BN / 32;
  static_assert(BM == 128, "four waves of 32 rows");
  __shared__ __align__(16) char k_tile0[Tile<D>::bytes(BN)];
  __shared__ __align__(16) char k_tile1[Tile<D>::bytes(BN)];
  __shared__ __align__(16) char v_tile0[Tile<D>::bytes(BN)];
  __shared__ __align__(16) char v_tile1[Tile<D>::bytes(BN)];
  __shared__ __align__(16) float cn_s0[BN];
  __shared__ __align__(16) float cn_s1[BN];

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), g = lane >> 5, i = lane & 31;
  int bh, mt, sp = 0;
  if constexpr (SPLIT) {  // (query tile, key split) pairs take the place of query tiles
    int mts;
    decode_block(blockIdx.x, a.n_mtiles * a.splits, a.B * a.H, bh, mts);
    mt = mts / a.splits;
    sp = mts % a.splits;
  } else {
    decode_block(blockIdx.x, a.n_mtiles, a.B * a.H, bh, mt);
  }
  const int b = bh / a.H, h = bh % a.H;
  const int M = a.M, N = a.N, p_seq = N - M;
  const int m0 = mt * BM;
  const float* c_row = a.c + (int64_t)bh * N;
  const uint16_t* qp = a.q.ptr + b * a.q.sb + h * a.q.sh;
  const uint16_t* kp = a.k.ptr + b * a.k.sb + h * a.k.sh;
  const uint16_t* vp = a.v.ptr + b * a.v.sb + h * a.v.sh;
  uint16_t* op = const_cast<uint16_t*>(a.o.ptr) + b * a.o.sb + h * a.o.sh;

  const int a0 = p_seq + m0;  // key position of the tile's first query row
  const int hi = min(N, a0 + BM);
  int seq = 0;
  if (a.seq_start) {
    const int64_t s64 = a.seq_start[b];
    seq = (int)(s64 < 0 ? 0 : (s64 > N ? N : s64));
  }
  const int m = m0 + 32 * wave + i;  // this lane's query row
  const int a_m = p_seq + m;
  const int a_w0 = a0 + 32 * wave;   // key position of the wave's first row
  const float qk_scale = nonzero_scale(a.sm_scale * kLog2e), inv_scale = 1.0f / qk_scale;
  // Everything the workgroup needs first is requested before anything is waited for.  The first tile to
  // visit (the one under the end of the diagonal) does not depend on the pruning bound, so it goes
  // first; then Q, then the per-row and per-key terms; the bound search's loads queue behind them.
  const DirectTileLoader<D, BN, 4, AUX> kld(a.k.st, wave, lane), vld(a.v.st, wave, lane);
  const int n0_first = hi > 0 ? ((hi - 1) / BN) * BN : 0;
  const bool early = !SPLIT && hi > (min(seq, hi) / BN) * BN && (n0_first + BN - 1 > a0 || !(qk_scale > 0.f));
  // The tile before it is requested as well when nothing can exclude it: it still reaches the workgroup's first row
  // (the pruning bound never cuts there) and lies right of seq_start.  Under pruning a workgroup visits two or
  // three tiles, and every round trip taken out of that chain counts.
  const int n0_second = n0_first - BN;
  const bool early2 = early && n0_second >= (a0 / BN) * BN && n0_second >= (min(seq, hi) / BN) * BN &&
                      (n0_second + BN - 1 > a0 || !(qk_scale > 0.f));
  if (early) {
    kld.issue(kp, a.k.st, n0_first, N, k_tile0);
    vld.issue(vp, a.v.st, n0_first, N, v_tile0);
  }
  if (early2) {
    kld.issue(kp, a.k.st, n0_second, N, k_tile1);
    vld.issue(vp, a.v.st, n0_second, N, v_tile1);
  }
  u32x4 qreg[KK];
  load_row_operand_regs<D>(qreg, qp, a.q.st, m, M, g);
  const float c_ref = c_row[a0];
  const float c_m = c_row[min(a_m, N - 1)];
  // Under pruning the third tile of the walk (the look-back tile, which is also the next query tile's upper diagonal
  // tile) is wanted more often than not, but its LDS buffer is busy until the first tile is done.  One dword per cache
  // line brings it into L2 now, while the neighbour fetches it as well (pruned forward 0.253 -> 0.246 ms at B4 T16384
  // H16 D128; the same in the dQ and dK/dV kernels costs 2-4 %, so only here).
  int l2_touch = 0;
  if (a.thr && early2) {
    const int n0_third = n0_second - BN;
    if (n0_third >= 0 && n0_third + BN > seq) {
      constexpr int LPR = (2 * D + 127) / 128;   // cache lines per row
      const int idx = tid & 127, row = idx / LPR, part = idx % LPR;
      if (row < BN) {
        const uint16_t* src = (tid < 128 ? kp + (int64_t)(n0_third + row) * a.k.st : vp + (int64_t)(n0_third + row) * a.v.st) + part * 64;
        l2_touch = *reinterpret_cast<const int*>(src);
      }
    }
  }

  // Key terms of a tile: the load is requested here, the arithmetic on it is done where the value goes to
  // LDS (a tile later), so that nothing waits for the load in between.  Masked keys get -inf through the
  // subtraction.
  float cn_raw = 0.f;
  bool cn_ok = false;
  auto issue_cn = [&](int n0) {
    if (tid < BN) {
      const int n = n0 + tid;
      cn_ok = (n < N) & (n >= seq);
      cn_raw = c_row[min(n, N - 1)];
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
    const int n = n0_second + tid;
    cn_ok2 = (n < N) & (n >= seq);
    cn_raw2 = c_row[min(n, N - 1)];
  }
  const float cm2 = (m < M) ? (c_m - c_ref) * kLog2e : 0.f;

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
  float m_i = -3.0e38f, l_i = 0.f;  // finite floor: a row that has seen no valid key yet yields exp2(-inf) = 0

  int lo = min(seq, hi);
  if (a.thr) {
    const int t = acp_first_kept_block(c_row, c_ref, a.thr[bh], N, BN, a0 / BN, lane);
    lo = max(lo, t * BN);
  }
  lo = (lo / BN) * BN;
  if (a.first_block && tid == 0 && sp == 0) a.first_block[(int64_t)bh * a.n_mtiles + mt] = lo / BN;
  int n_tiles = (hi - lo + BN - 1) / BN;  // walked from the last (diagonal) tile down to lo
  if constexpr (SPLIT) {  // this workgroup's contiguous share of the key tiles
    const int per = (n_tiles + a.splits - 1) / a.splits;
    const int t0 = min(n_tiles, sp * per), t1 = min(n_tiles, t0 + per);
    lo += t0 * BN;
    n_tiles = t1 - t0;
  }

  // A wave whose 32 rows all lie beyond M (decode and other short query blocks) still moves its share
  // of every tile but computes nothing.
  const bool wave_has_rows = m0 + 32 * wave < M;
  auto compute = [&](int n0, const char* kt, const char* vt, const float* cn) {
    if (n0 > a_w0 + 31 || !wave_has_rows) return;  // tile entirely above this wave's rows
    fwd_tile<Tr, D>(kt, vt, cn, qreg, oacc, m_i, l_i, n0, a_m, qk_scale, lane, n0 + BN - 1 > a_w0);
  };

  // Phase 1: the tiles that reach the workgroup's diagonal (the last ceil(BM/BN) + 1 at most), with
  // the masking code, double-buffered.  Phase 2: interior tiles, software-pipelined across tiles.
  // The pipelined code takes the row maximum on the raw accumulators, which needs sm_scale > 0;
  // otherwise every tile goes through phase 1.
  int n_diag = 0;
  while (n_diag < n_tiles && lo + (n_tiles - 1 - n_diag) * BN + BN - 1 > a0) ++n_diag;
  if (!(qk_scale > 0.f)) n_diag = n_tiles;
  // The pipelined path starts with two round trips of its own (K of its first tile, then V): worth it for a long
  // walk only.  With a few interior tiles (the usual case under pruning) they go through phase 1 as well.
  if (n_tiles - n_diag < kMinPipelinedTiles) n_diag = n_tiles;
  const int t_stop = n_tiles - n_diag;
  auto tile_n0 = [&](int t) { return lo + t * BN; };   // start of the tile at loop position t
  if (n_diag > 0) {
    if (!early) issue(tile_n0(n_tiles - 1), k_tile0, v_tile0);
    if (tid < BN) cn_s0[tid] = cn_term();
    if (early2) { cn_raw = cn_raw2; cn_ok = cn_ok2; }
  }
  bool requested = early2;  // buffers 1 already hold (or await) the next tile
  for (int t = n_tiles - 1; t >= t_stop; t -= 2) {
    // even step: consume buffers 0, fill buffers 1
    wait_vmem_all();
    __syncthreads();
    if (t - 1 >= t_stop && !requested) issue(tile_n0(t - 1), k_tile1, v_tile1);
    requested = false;
    compute(tile_n0(t), k_tile0, v_tile0, cn_s0);
    if (t - 1 < t_stop) break;
    if (tid < BN) cn_s1[tid] = cn_term();
    // odd step: consume buffers 1, fill buffers 0
    wait_vmem_all();
    __syncthreads();
    if (t - 2 >= t_stop) issue(tile_n0(t - 2), k_tile0, v_tile0);
    compute(tile_n0(t - 1), k_tile1, v_tile1, cn_s1);
    if (t - 2 >= t_stop && tid < BN) cn_s0[tid] = cn_term();
  }

  const int n_int = t_stop;  // interior tile j (0 = nearest to the diagonal) starts at key lo + (n_int-1-j)*BN
  if (n_int > 0) {
    auto issue_k = [&](int j, char* kt) {
      const int n0 = lo + (n_int - 1 - j) * BN;
      issue_cn(n0);
      kld.issue(kp, a.k.st, n0, N, kt);
    };
    auto issue_v = [&](int j, char* vt) { vld.issue(vp, a.v.st, lo + (n_int - 1 - j) * BN, N, vt); };
    // K runs one tile ahead of V: iteration j computes S(j+1) and P(j) V(j).
    __syncthreads();  // phase 1 is done with every buffer
    issue_k(0, k_tile0);
    if (tid < BN) cn_s0[tid] = cn_term();
    wait_vmem_all();
    __syncthreads();
    if (n_int > 1) issue_k(1, k_tile1);
    issue_v(0, v_tile0);
    f32x16 s_a[NB], s_b[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      if (!wave_has_rows) break;
      s_a[nb] = acc_init(cn_s0, 32 * nb, g);
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) s_a[nb] = Tr::mfma32(lds_row_operand<D>(k_tile0, 32 * nb + i, 2 * kk + g), qreg[kk], s_a[nb]);
    }
    // Iteration j: S(j+1) from k_nx, P(j) V(j) from v_cur; meanwhile K(j+2) is requested into k_fill and
    // V(j+1) into v_fill, one load instruction per chunk of the tile (an empty extent when there is no such
    // tile: the loads then write zeros into the free buffer).
    auto pipelined_tile = [&](int j, const char* k_nx, const char* v_cur, const float* cn_nx, char* k_fill, char* v_fill,
                              f32x16 (&s_cur)[NB], f32x16 (&s_nx)[NB]) {
      const bool more_k = j + 2 < n_int, more_v = j + 1 < n_int;
      const int nk = more_k ? lo + (n_int - 3 - j) * BN : lo, nv = more_v ? lo + (n_int - 2 - j) * BN : lo;
      if (more_k) issue_cn(nk);
      const uint16_t *k_src = kp + (int64_t)nk * a.k.st, *v_src = vp + (int64_t)nv * a.v.st;
      const int k_bytes = kld.extent(a.k.st, nk, more_k ? N : nk), v_bytes = vld.extent(a.v.st, nv, more_v ? N : nv);
      const TileDma<D, AUX> dma{kld, vld, k_src, v_src, k_bytes, v_bytes, k_fill, v_fill};
      if (wave_has_rows) fwd_tile_pipelined<Tr, D>(k_nx, v_cur, cn_nx, qreg, oacc, m_i, l_i, qk_scale, lane, s_cur, s_nx, dma);
      else dma.all();  // a wave without query rows only moves its share of the tiles
    };
    for (int j = 0; j < n_int; j += 2) {
      // even iteration: K(j+1) in k_tile1 with its key terms in cn_s1, V(j) in v_tile0.  The key
      // terms of tile j+1 go to LDS before the barrier: their buffer was last read two iterations ago.
      wait_vmem_all();
      if (j + 1 < n_int && tid < BN) cn_s1[tid] = cn_term();
      __syncthreads();
      pipelined_tile(j, k_tile1, v_tile0, cn_s1, k_tile0, v_tile1, s_a, s_b);
      if (j + 1 >= n_int) break;
      // odd iteration: K(j+2) in k_tile0 with its key terms in cn_s0, V(j+1) in v_tile1
      wait_vmem_all();
      if (j + 2 < n_int && tid < BN) cn_s0[tid] = cn_term();
      __syncthreads();
      pipelined_tile(j + 1, k_tile0, v_tile1, cn_s0, k_tile1, v_tile0, s_b, s_a);
    }
  }

  // epilogue
  const float l_tot = half_sum(l_i);
  if constexpr (SPLIT) {
    // partial result of this key split: unnormalised accumulator, row maximum (log2 domain,
    // including the row term) and row sum; fox::combine_kernel merges the splits
    if (m < M) {
      const int64_t row = ((int64_t)sp * a.B * a.H + bh) * M + m;
      float* wo = a.ws_o + row * D;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int d = 32 * db + 8 * q4 + 4 * g;
          if (d < D) {
            f32x4 w = {oacc[db][4 * q4 + 0], oacc[db][4 * q4 + 1], oacc[db][4 * q4 + 2], oacc[db][4 * q4 + 3]};
            *reinterpret_cast<f32x4*>(wo + d) = w;
          }
        }
      if (g == 0) {
        a.ws_ml[2 * row] = m_i + cm2;
        a.ws_ml[2 * row + 1] = l_tot;
      }
    }
    return;
  }
  const bool empty = a_m < seq;
  const float inv = empty ? 0.f : 1.0f / l_tot;
  if (m < M && g == 0) a.lse[(int64_t)bh * M + m] = empty ? -INFINITY : (m_i + cm2) * kLn2 + __logf(l_tot);
  // o leaves through LDS (the tile buffers are free now, one per wave) so that the global stores are whole rows
  static_assert(kStoreStageBytes<D> <= Tile<D>::bytes(BN), "one wave stages in one tile buffer");
  wait_vmem_all();  // whatever was requested last (possibly an empty tile) has landed
  __syncthreads();  // every wave is done with the last tile
  char* stage = wave == 0 ? k_tile0 : wave == 1 ? k_tile1 : wave == 2 ? v_tile0 : v_tile1;
  if constexpr (EPI) {  // the layer's output norm and gate, applied while the rows are on their way out
    // The epilogue's arguments are fetched from the kernel argument block only here, through a pointer the
    // compiler cannot see through: loaded at kernel entry they would occupy scalar registers across the key loop.
    typedef const char __attribute__((address_space(4)))* kernarg_bytes;
    typedef const FwdEpilogue __attribute__((address_space(4)))* kernarg_epilogue;
    kernarg_epilogue ep = (kernarg_epilogue)((kernarg_bytes)__builtin_amdgcn_kernarg_segment_ptr() + offsetof(FwdK, epi));
    asm volatile("" : "+s"(ep));
    const uint16_t* gp = ep->gate.ptr ? ep->gate.ptr + b * ep->gate.sb + h * ep->gate.sh : nullptr;
    uint16_t* yp = const_cast<uint16_t*>(ep->y.ptr) + b * ep->y.sb + h * ep->y.sh;
    store_rows_norm_gate<Tr, D>(stage, oacc, inv, a.o.ptr ? op : nullptr, a.o.st, gp, ep->gate.st, yp, ep->y.st,
                                ep->w + h * D, ep->rstd + (int64_t)b * M * a.H + h, a.H, ep->eps, ep->act, m0 + 32 * wave,
                                M, lane);
  } else {
    store_rows_via_lds<Tr, D>(stage, oacc, inv, op, a.o.st, m0 + 32 * wave, M, lane);
  }
  asm volatile("" ::"v"(l2_touch));   // the value is never used; this keeps the load
}

// Merge the partial results of the key splits of one query row:
//   m = max_s m_s,  l = sum_s l_s 2^(m_s - m),  o = sum_s acc_s 2^(m_s - m) / l,  lse = m ln2 + ln l.
// One thread per (row, 4 head-dim elements).
template <typename Tr, int D>
__global__ __launch_bounds__(256) void combine_kernel(const FwdK a) {
  constexpr int TPR = D / 4;  // threads per row
  const int64_t n_rows = (int64_t)a.B * a.H * a.M;
  const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) / TPR;
  const int d = (threadIdx.x % TPR) * 4;
  if (row >= n_rows) return;
  const int bh = (int)(row / a.M), m = (int)(row % a.M), b = bh / a.H, h = bh % a.H;
  float mx = -INFINITY;
  for (int sp = 0; sp < a.splits; ++sp) mx = fmaxf(mx, a.ws_ml[2 * (sp * n_rows + row)]);
  float l = 0.f;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int sp = 0; sp < a.splits; ++sp) {
    const int64_t r = sp * n_rows + row;
    const float w = __builtin_amdgcn_exp2f(a.ws_ml[2 * r] - mx);
    l += a.ws_ml[2 * r + 1] * w;
    const f32x4 o = *reinterpret_cast<const f32x4*>(a.ws_o + r * D + d);
    acc += o * w;
  }
  int seq = 0;
  if (a.seq_start) {
    const int64_t s64 = a.seq_start[b];
    seq = (int)(s64 < 0 ? 0 : (s64 > a.N ? a.N : s64));
  }
  const bool empty = (a.N - a.M + m) < seq;
  const float inv = empty ? 0.f : 1.0f / l;
  uint16_t* op = const_cast<uint16_t*>(a.o.ptr) + b * a.o.sb + h * a.o.sh + (int64_t)m * a.o.st + d;
  u32x2 w;
  w[0] = Tr::pack2(acc[0] * inv, acc[1] * inv);
  w[1] = Tr::pack2(acc[2] * inv, acc[3] * inv);
  *reinterpret_cast<u32x2*>(op) = w;
  if (d == 0) a.lse[row] = empty ? -INFINITY : mx * kLn2 + __logf(l);
}

// Query tiles per (batch, head) up to which the forward's K and V tile loads may carry the non-temporal hint
// (FwdK::stream asks for it).
constexpr int kStreamMaxQueryTiles = 1;

// explicit instantiations: every (dtype, head dim) pair the dispatcher can reach
#define FOX_INSTANTIATE_FWD(TR)                                          \
  template __global__ void fwd_kernel<TR, 16, false>(const FwdK);        \
  template __global__ void fwd_kernel<TR, 32, false>(const FwdK);        \
  template __global__ void fwd_kernel<TR, 64, false>(const FwdK);        \
  template __global__ void fwd_kernel<TR, 128, false>(const FwdK);       \
  template __global__ void fwd_kernel<TR, 16, false, true>(const FwdK);  \
  template __global__ void fwd_kernel<TR, 32, false, true>(const FwdK);  \
  template __global__ void fwd_kernel<TR, 64, false, true>(const FwdK);  \
  template __global__ void fwd_kernel<TR, 128, false, true>(const FwdK); \
  template __global__ void fwd_kernel<TR, 16, true>(const FwdK);         \
  template __global__ void fwd_kernel<TR, 32, true>(const FwdK);         \
  template __global__ void fwd_kernel<TR, 64, true>(const FwdK);         \
  template __global__ void fwd_kernel<TR, 128, true>(const FwdK);        \
  template __global__ void fwd_kernel<TR, 16, false, false, true>(const FwdK);  \
  template __global__ void fwd_kernel<TR, 32, false, false, true>(const FwdK);  \
  template __global__ void fwd_kernel<TR, 64, false, false, true>(const FwdK);  \
  template __global__ void fwd_kernel<TR, 128, false, false, true>(const FwdK); \
  template __global__ void fwd_kernel<TR, 16, true, false, true>(const FwdK);   \
  template __global__ void fwd_kernel<TR, 32, true, false, true>(const FwdK);   \
  template __global__ void fwd_kernel<TR, 64, true, false, true>(const FwdK);   \
  template __global__ void fwd_kernel<TR, 128, true, false, true>(const FwdK);  \
  template __global__ void combine_kernel<TR, 16>(const FwdK);           \
  template __global__ void combine_kernel<TR, 32>(const FwdK);           \
  template __global__ void combine_kernel<TR, 64>(const FwdK);           \
  template __global__ void combine_kernel<TR, 128>(const FwdK);
FOX_INSTANTIATE_FWD(Bf16)
FOX_INSTANTIATE_FWD(Fp16)

template <typename Tr, int D>
static hipError_t launch_fwd_d(const FwdK& a, int dtype, hipStream_t s) {
  if (a.epi.y.ptr && (a.M == 1 || a.splits > 1)) return hipErrorInvalidValue;  // the epilogue lives in the unsplit kernel only
  const bool stream = a.stream && a.n_mtiles <= kStreamMaxQueryTiles;
  if (a.M == 1) {  // decode step: the streaming kernel, one workgroup per (batch, head, key split)
    const hipError_t e = launch_fwd_decode(a, D, dtype, s);
    if (e != hipSuccess || a.splits <= 1) return e;
  } else if (a.splits <= 1) {
    const dim3 grid((unsigned)(a.n_mtiles * a.B * a.H));
    if (a.epi.y.ptr) hipLaunchKernelGGL((fwd_kernel<Tr, D, false, true>), grid, dim3(256), 0, s, a);
    else if (stream) hipLaunchKernelGGL((fwd_kernel<Tr, D, false, false, true>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((fwd_kernel<Tr, D, false>), grid, dim3(256), 0, s, a);
    return hipGetLastError();
  } else {
    const dim3 grid((unsigned)(a.n_mtiles * a.splits * a.B * a.H));
    if (stream) hipLaunchKernelGGL((fwd_kernel<Tr, D, true, false, true>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((fwd_kernel<Tr, D, true>), grid, dim3(256), 0, s, a);
  }
  const int64_t threads = (int64_t)a.B * a.H * a.M * (D / 4);
  hipLaunchKernelGGL((combine_kernel<Tr, D>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, a);
  return hipGetLastError();
}

template <typename Tr>
static hipError_t launch_fwd_t(const FwdK& a, int D, int dtype, hipStream_t s) {
  switch (D) {
    case 16: return launch_fwd_d<Tr, 16>(a, dtype, s);
    case 32: return launch_fwd_d<Tr, 32>(a, dtype, s);
    case 64: return launch_fwd_d<Tr, 64>(a, dtype, s);
    case 128: return launch_fwd_d<Tr, 128>(a, dtype, s);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_fwd(const FwdK& a, int D, int dtype, hipStream_t s) {
  return dtype == 0 ? launch_fwd_t<Bf16>(a, D, dtype, s) : launch_fwd_t<Fp16>(a, D, dtype, s);
}

// Number of key splits the forward uses for a shape: 1 unless the grid of query tiles
// alone leaves most of the chip idle while each workgroup has a long key loop (chunked
// prefill, decode).  Splits are sized to give every CU about two workgroups; the streaming
// kernel of the single-query case keeps no tile in LDS and takes about eight per CU, at
// least 512 keys each.
int fwd_key_splits(int B, int H, int M, int N) {
  if (M == 1) {
    const int64_t bh = (int64_t)B * H;
    int64_t splits = (2048 + bh - 1) / bh;
    splits = splits > N / 512 ? N / 512 : splits;
    splits = splits > 64 ? 64 : splits;
    return splits < 1 ? 1 : (int)splits;
  }
  const int64_t wgs = (int64_t)((M + kFwdBM - 1) / kFwdBM) * B * H;
  const int key_tiles = (N + kFwdBN - 1) / kFwdBN;
  if (wgs >= 512 || key_tiles < 16) return 1;
  int splits = (int)((512 + wgs - 1) / wgs);
  splits = splits > key_tiles / 8 ? key_tiles / 8 : splits;
  splits = splits > 32 ? 32 : splits;
  return splits < 1 ? 1 : splits;
}

}  // namespace fox
