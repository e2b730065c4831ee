// Row scans and the "auto" pruning threshold for gfx950.
//
//   scan_kernel<false> : c[n]  = sum_{l<=n} g[l], with g[l] := 0 for l < seq_start
//   scan_kernel<true>  : dg[l] = sum_{n>=l} dc[n]
//   gate_scan_fwd/bwd  : the same two scans fused with logsigmoid of the gate logits and its derivative
//   norm_max_kernel    : the "auto" threshold from the largest row L2 norms of q and k.
//
// One workgroup scans one (batch, head) row.  Partial sums are carried in fp64 and
// rounded once on store, so c is exactly non-increasing whenever g <= 0 (the
// pruning bounds rely on that) and long rows lose no precision to the scan order.
#include "fox_common.hpp"
#include "fox_kernels.hpp"

namespace fox {

constexpr int kScanThreads = 1024;  // one workgroup per row: few rows, long rows, so the workgroup is as wide as it gets

// Scan of one row: element idx is produced by load(idx) and the running sum up to and including
// it is handed to store(idx, sum).  REVERSE walks the row from its last element to its first.
// A span of 8 x 1024 elements moves between memory and LDS with consecutive lanes on consecutive
// elements (whole cache lines per wave instruction, whatever the caller's stride), and between LDS and
// registers with eight consecutive elements per thread, the order the scan wants.
template <bool REVERSE, typename Load, typename Store>
__device__ __forceinline__ void scan_row(int N, Load load, Store store) {
  constexpr int PER = 8, NT = kScanThreads, SPAN = PER * NT;
  __shared__ double wave_tot[NT / kWave];
  __shared__ __align__(16) float stage[SPAN];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  double carry = 0.0;
  float x[PER], x_next[PER];
  auto fetch = [&](int base, float (&dst)[PER]) {  // element e of a thread sits at position base + e*NT + tid of the scan order
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int pos = base + e * NT + tid;
      const int idx = REVERSE ? N - 1 - pos : pos;
      dst[e] = pos < N ? load(idx) : 0.f;
    }
  };
  fetch(0, x);
  for (int base = 0; base < N; base += SPAN) {
#pragma unroll
    for (int e = 0; e < PER; ++e) stage[e * NT + tid] = x[e];
    if (base + SPAN < N) fetch(base + SPAN, x_next);   // in flight while this span is scanned
    __syncthreads();
    const f32x4 lo4 = *reinterpret_cast<const f32x4*>(stage + tid * PER), hi4 = *reinterpret_cast<const f32x4*>(stage + tid * PER + 4);
    double v[PER];
    double run = 0.0;
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      run += (double)(e < 4 ? lo4[e & 3] : hi4[e & 3]);
      v[e] = run;
    }
    // inclusive scan of the per-thread totals across the wave, then across waves
    double incl = run;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const double up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    if (lane == kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    double before = carry, total = 0.0;
#pragma unroll
    for (int w = 0; w < NT / kWave; ++w) {
      const double t = wave_tot[w];
      if (w < wave) before += t;
      total += t;
    }
    before += incl - run;
    f32x4 o_lo, o_hi;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      o_lo[e] = (float)(before + v[e]);
      o_hi[e] = (float)(before + v[4 + e]);
    }
    *reinterpret_cast<f32x4*>(stage + tid * PER) = o_lo;   // each thread overwrites the eight values it read
    *reinterpret_cast<f32x4*>(stage + tid * PER + 4) = o_hi;
    carry += total;
    __syncthreads();
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int pos = base + e * NT + tid;
      const int idx = REVERSE ? N - 1 - pos : pos;
      if (pos < N) store(idx, stage[e * NT + tid]);
    }
#pragma unroll
    for (int e = 0; e < PER; ++e) x[e] = x_next[e];
    __syncthreads();  // the span has left LDS before the next one is written
  }
}

template <bool REVERSE>
__global__ __launch_bounds__(kScanThreads) void scan_kernel(const float* __restrict__ in, int64_t sb, int64_t sh, int64_t sn,
                                                   const int64_t* __restrict__ seq_start, float* __restrict__ out, int64_t ob,
                                                   int64_t oh, int64_t on, int H, int N) {
  const int bh = blockIdx.x, b = bh / H, h = bh % H;
  const float* src = in + b * sb + h * sh;
  float* dst = out + b * ob + h * oh;
  int seq = 0;
  if (seq_start) {
    const int64_t s64 = seq_start[b];
    seq = (int)(s64 < 0 ? 0 : (s64 > N ? N : s64));
  }
  // Reverse: the gradient of every gate up to and including position seq is the sum of all dc, zero in exact
  // arithmetic (those gates shift every cumulative sum the kernels see by the same amount, or are zeroed by the
  // forward); it is stored as an exact zero instead of the rounding noise of that sum.
  scan_row<REVERSE>(
      N, [&](int idx) { return (REVERSE || idx >= seq) ? src[(int64_t)idx * sn] : 0.f; },
      [&](int idx, float sum) { dst[(int64_t)idx * on] = (REVERSE && idx <= seq) ? 0.f : sum; });
}

// Forget-gate logits in fp32, bf16 or fp16 (the output of the gate projection of the FoX layer).
template <int DT>
__device__ __forceinline__ float load_logit(const void* p, int64_t i) {
  if constexpr (DT == 2) return reinterpret_cast<const float*>(p)[i];
  const uint32_t w = reinterpret_cast<const uint16_t*>(p)[i];
  if constexpr (DT == 0) return Bf16::lo(w);
  return Fp16::lo(w);
}
template <int DT>
__device__ __forceinline__ void store_logit(void* p, int64_t i, float x) {
  if constexpr (DT == 2) reinterpret_cast<float*>(p)[i] = x;
  else if constexpr (DT == 0) reinterpret_cast<uint16_t*>(p)[i] = (uint16_t)(Bf16::pack2(x, 0.f) & 0xffffu);
  else reinterpret_cast<uint16_t*>(p)[i] = (uint16_t)(Fp16::pack2(x, 0.f) & 0xffffu);
}

// logsigmoid(x) = min(x, 0) - log1p(exp(-|x|)), stable on both sides, from the hardware exp / log:
// log1p(z) for z in (0, 1] is log(u) + (z - (u - 1)) / u with u = fl(1 + z), which repairs the rounding
// of 1 + z (absolute error ~1e-8, and log1p(z) -> z for tiny z as it must).  The result is clamped to <= 0:
// a log gate is never positive, and the pruning bounds rely on the cumulative sums not increasing, whatever
// the last bit of the hardware logarithm does near u = 1.
__device__ __forceinline__ float log_sigmoid(float x) {
  const float z = __expf(-fabsf(x));
  const float u = 1.0f + z;
  const float l = fmaxf(__logf(u) + __fdividef(z - (u - 1.0f), u), 0.f);
  return fminf(fminf(x, 0.f) - l, 0.f);
}

// c[n] = sum_{seq_start <= l <= n} logsigmoid(x[l]) in one pass over the logits; optionally also
// stores log_fgate[n] = logsigmoid(x[n]) (the decode cache of the FoX layer keeps it).
template <int DT>
__global__ __launch_bounds__(kScanThreads) void gate_scan_fwd_kernel(const void* __restrict__ logits, int64_t sb, int64_t sh, int64_t sn,
                                                            const int64_t* __restrict__ seq_start,
                                                            float* __restrict__ log_fgate, float* __restrict__ out, int H,
                                                            int N) {
  const int bh = blockIdx.x, b = bh / H, h = bh % H;
  const int64_t base = b * sb + h * sh;
  float* dst = out + (int64_t)bh * N;
  float* lg = log_fgate ? log_fgate + (int64_t)bh * N : nullptr;
  int seq = 0;
  if (seq_start) {
    const int64_t s64 = seq_start[b];
    seq = (int)(s64 < 0 ? 0 : (s64 > N ? N : s64));
  }
  scan_row<false>(
      N,
      [&](int idx) {
        const float x = load_logit<DT>(logits, base + (int64_t)idx * sn);
        const float g = log_sigmoid(x);
        if (lg) lg[idx] = g;
        return idx >= seq ? g : 0.f;
      },
      [&](int idx, float sum) { dst[idx] = sum; });
}

// dlogit[l] = (sum_{n>=l} dc[n]) * d logsigmoid(x_l)/dx = dg[l] * (1 - sigmoid(x_l)), stored in the
// dtype and layout of the logits.
template <int DT>
__global__ __launch_bounds__(kScanThreads) void gate_scan_bwd_kernel(const float* __restrict__ dc, const void* __restrict__ logits,
                                                            int64_t sb, int64_t sh, int64_t sn, const int64_t* __restrict__ seq_start,
                                                            void* __restrict__ dlogits, int64_t db, int64_t dh, int64_t dn, int H,
                                                            int N) {
  const int bh = blockIdx.x, b = bh / H, h = bh % H;
  const float* src = dc + (int64_t)bh * N;
  const int64_t lbase = b * sb + h * sh, dbase = b * db + h * dh;
  int seq = 0;
  if (seq_start) {
    const int64_t s64 = seq_start[b];
    seq = (int)(s64 < 0 ? 0 : (s64 > N ? N : s64));
  }
  scan_row<true>(
      N, [&](int idx) { return src[idx]; },
      [&](int idx, float sum) {
        const float x = load_logit<DT>(logits, lbase + (int64_t)idx * sn);
        const float z = __expf(-fabsf(x));
        const float r = __fdividef(z, 1.f + z);              // sigmoid(-|x|)
        // positions up to and including seq: an exact zero, as in scan_kernel<true>
        store_logit<DT>(dlogits, dbase + (int64_t)idx * dn, idx <= seq ? 0.f : sum * (x < 0.f ? 1.f - r : r));
      });
}

hipError_t launch_gate_cumsum_fwd(const void* logits, int dtype, int64_t sb, int64_t sh, int64_t sn, const int64_t* seq_start,
                                  float* log_fgate, float* c, int B, int H, int N, hipStream_t s) {
  const dim3 grid((unsigned)(B * H));
  switch (dtype) {
    case 0: hipLaunchKernelGGL(gate_scan_fwd_kernel<0>, grid, dim3(kScanThreads), 0, s, logits, sb, sh, sn, seq_start, log_fgate, c, H, N); break;
    case 1: hipLaunchKernelGGL(gate_scan_fwd_kernel<1>, grid, dim3(kScanThreads), 0, s, logits, sb, sh, sn, seq_start, log_fgate, c, H, N); break;
    case 2: hipLaunchKernelGGL(gate_scan_fwd_kernel<2>, grid, dim3(kScanThreads), 0, s, logits, sb, sh, sn, seq_start, log_fgate, c, H, N); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_gate_cumsum_bwd(const float* dc, const void* logits, int dtype, int64_t sb, int64_t sh, int64_t sn,
                                  const int64_t* seq_start, void* dlogits, int64_t db, int64_t dh, int64_t dn, int B, int H, int N,
                                  hipStream_t s) {
  const dim3 grid((unsigned)(B * H));
  switch (dtype) {
    case 0: hipLaunchKernelGGL(gate_scan_bwd_kernel<0>, grid, dim3(kScanThreads), 0, s, dc, logits, sb, sh, sn, seq_start, dlogits, db, dh, dn, H, N); break;
    case 1: hipLaunchKernelGGL(gate_scan_bwd_kernel<1>, grid, dim3(kScanThreads), 0, s, dc, logits, sb, sh, sn, seq_start, dlogits, db, dh, dn, H, N); break;
    case 2: hipLaunchKernelGGL(gate_scan_bwd_kernel<2>, grid, dim3(kScanThreads), 0, s, dc, logits, sb, sh, sn, seq_start, dlogits, db, dh, dn, H, N); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_cumsum_fwd(const float* g, int64_t sb, int64_t sh, int64_t sn, const int64_t* seq_start, float* c, int B,
                             int H, int N, hipStream_t s) {
  hipLaunchKernelGGL(scan_kernel<false>, dim3((unsigned)(B * H)), dim3(kScanThreads), 0, s, g, sb, sh, sn, seq_start, c,
                     (int64_t)H * N, (int64_t)N, (int64_t)1, H, N);
  return hipGetLastError();
}

hipError_t launch_cumsum_bwd(const float* dc, float* dg, int64_t db, int64_t dh, int64_t dn, const int64_t* seq_start, int B, int H,
                             int N, hipStream_t s) {
  hipLaunchKernelGGL(scan_kernel<true>, dim3((unsigned)(B * H)), dim3(kScanThreads), 0, s, dc, (int64_t)H * N, (int64_t)N, (int64_t)1,
                     seq_start, dg, db, dh, dn, H, N);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// "auto" threshold
// ---------------------------------------------------------------------------
template <typename Tr>
__device__ __forceinline__ float round16(float x) {  // round to the 16-bit dtype and back
  return Tr::lo(Tr::pack2(x, 0.f));
}

__global__ void zero_u32_kernel(uint32_t* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

// grid (row blocks, B*H, 2): z = 0 scans q (T = M), z = 1 scans k (T = N).  scratch holds, per (batch, head), the two
// running maxima (float bits) and the number of workgroups that have added theirs; the workgroup that arrives last
// turns the maxima into the threshold, so no kernel of its own is needed for that.
template <typename Tr, int D>
__global__ __launch_bounds__(256) void norm_max_kernel(View q, View k, int H, int M, int N, uint32_t* scratch, float* thr,
                                                       float sm_scale, float log_n) {
  constexpr int LPR = D / 8, RPP = 256 / LPR, ROWS = 512;
  const int tid = threadIdx.x;
  const int bh = blockIdx.y, b = bh / H, h = bh % H;
  const View& t = blockIdx.z == 0 ? q : k;
  const int T = blockIdx.z == 0 ? M : N;
  const uint16_t* p = t.ptr + b * t.sb + h * t.sh;
  const int ch = tid % LPR;
  float best = 0.f;
  constexpr int U = (ROWS / RPP) < 8 ? (ROWS / RPP) : 8;  // rows in flight per thread
  for (int pass = 0; pass < ROWS / RPP; pass += U) {
    u32x4 x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int row = min(blockIdx.x * ROWS + (pass + u) * RPP + tid / LPR, T - 1);  // rows past the end repeat the last one
      x[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p + (int64_t)row * t.st + ch * 8));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float acc = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) acc += Tr::lo(x[u][e]) * Tr::lo(x[u][e]) + Tr::hi(x[u][e]) * Tr::hi(x[u][e]);
#pragma unroll
      for (int off = LPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
      best = fmaxf(best, round16<Tr>(sqrtf(acc)));
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) best = fmaxf(best, __shfl_xor(best, off));
  __shared__ float wave_best[4];
  if ((tid & 63) == 0) wave_best[tid >> 6] = best;
  __syncthreads();
  if (tid != 0) return;
  best = fmaxf(fmaxf(wave_best[0], wave_best[1]), fmaxf(wave_best[2], wave_best[3]));
  uint32_t* mine = scratch + bh * 3;
  // Non-negative floats order like uints.  The arrival is counted only after the maximum has been applied: the count's
  // operand depends on the value the first atomic returns, and a returning atomic has been carried out where all
  // workgroups' atomics meet.  (No fence: a device-wide release would write back the whole L2 once per workgroup.)
  const uint32_t before = atomicMax(&mine[blockIdx.z], __float_as_uint(best));
  uint32_t one = 1u;
  asm volatile("" : "+v"(one) : "v"(before));
  if (atomicAdd(&mine[2], one) != gridDim.x * 2u - 1u) return;
  // the last workgroup of this (batch, head): every maximum has been added (read through the atomic unit as well)
  const float qn = __uint_as_float(atomicMax(&mine[0], 0u)), kn = __uint_as_float(atomicMax(&mine[1], 0u));
  // every tensor op of the reference rounds to the input dtype
  float ub = round16<Tr>(qn * kn);
  ub = round16<Tr>(ub * sm_scale);
  float th = round16<Tr>(2.f * ub);
  th = round16<Tr>(th + log_n);
  th = -th;
  th = round16<Tr>(th - 10.f);
  thr[bh] = th;
}

template <typename Tr>
static hipError_t auto_threshold_t(const View& q, const View& k, int B, int H, int M, int N, int D, float sm_scale, float* thr,
                                   uint32_t* scratch, hipStream_t s) {
  const int n_bh = B * H;
  hipLaunchKernelGGL(zero_u32_kernel, dim3((unsigned)((3 * n_bh + 255) / 256)), dim3(256), 0, s, scratch, 3 * n_bh);
  const dim3 grid((unsigned)((N + 511) / 512), (unsigned)n_bh, 2u);
  const float log_n = (float)log((double)N);
  switch (D) {
    case 16: hipLaunchKernelGGL((norm_max_kernel<Tr, 16>), grid, dim3(256), 0, s, q, k, H, M, N, scratch, thr, sm_scale, log_n); break;
    case 32: hipLaunchKernelGGL((norm_max_kernel<Tr, 32>), grid, dim3(256), 0, s, q, k, H, M, N, scratch, thr, sm_scale, log_n); break;
    case 64: hipLaunchKernelGGL((norm_max_kernel<Tr, 64>), grid, dim3(256), 0, s, q, k, H, M, N, scratch, thr, sm_scale, log_n); break;
    case 128: hipLaunchKernelGGL((norm_max_kernel<Tr, 128>), grid, dim3(256), 0, s, q, k, H, M, N, scratch, thr, sm_scale, log_n); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_auto_threshold(const View& q, const View& k, int B, int H, int M, int N, int D, int dtype, float sm_scale,
                                 float* thr, uint32_t* scratch, hipStream_t s) {
  return dtype == 0 ? auto_threshold_t<Bf16>(q, k, B, H, M, N, D, sm_scale, thr, scratch, s)
                    : auto_threshold_t<Fp16>(q, k, B, H, M, N, D, sm_scale, thr, scratch, s);
}

}  // namespace fox
