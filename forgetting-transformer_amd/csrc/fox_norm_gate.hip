// Per-head RMS normalisation for gfx950, gated or plain: the epilogue the FoX layer applies to the
// attention output before the output projection, and the normalisation of queries and keys in front
// of the attention (QK-norm),
//   y[r,h,:] = x[r,h,:] * rstd[r,h] * w[h,:] * act(g[r,h,:]),   rstd = 1 / sqrt(mean_d x^2 + eps),
// act(g) = sigmoid(g), g*sigmoid(g) (swish) or 1 (no gate tensor), and its backward
//   yn = xhat * w (xhat = x * rstd),  dg = dy * yn * act'(g),  dyn = dy * act(g),
//   dw[h,:] = sum_r dyn * xhat,  dx = (dyn*w - xhat * mean_d(dyn*w*xhat)) * rstd.
// (reference: model/forgetting_transformer/fuse_norm_gate.py:132-206 forward, :309-417 backward, the
// configuration FusedGroupNormGated(num_groups=heads, is_rms_norm=True, activation="sigmoid") of
// modeling_forgetting_transformer.py:243, no bias, no residual; the plain form is layer_norm_fwd_kernel /
// layer_norm_bwd_kernel of layernorm.py:183-254, :328-435 as used by GroupNorm(num_groups=heads,
// is_rms_norm=True) and RMSNorm(head_dim), modeling_forgetting_transformer.py:258-265, :314-325)
//
// Both are pure streams over HBM.  A (row, head) group of D elements is spread over D/8 lanes, 16
// bytes each; the two row reductions are shuffles inside that lane group.  In the backward every
// thread keeps one (head, 8 elements) column and walks a strip of rows, so the weight gradient is
// accumulated in registers and leaves as one partial per strip; a second kernel adds the partials in
// a fixed order (no atomics: the result does not depend on scheduling).
#include "fox_common.hpp"
#include "fox_kernels.hpp"

namespace fox {

template <typename Tr>
__device__ __forceinline__ void unpack8v(const u32x4& v, float (&f)[8]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    f[2 * e] = Tr::lo(v[e]);
    f[2 * e + 1] = Tr::hi(v[e]);
  }
}
template <typename Tr>
__device__ __forceinline__ u32x4 pack8v(const float (&f)[8]) {
  u32x4 r;
#pragma unroll
  for (int e = 0; e < 4; ++e) r[e] = Tr::pack2(f[2 * e], f[2 * e + 1]);
  return r;
}
template <typename Tr, int D, int ACT>
__global__ __launch_bounds__(256) void norm_gate_fwd_kernel(const NormGateK a) {
  constexpr int CH = D / 8;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int chunk = (int)(gid % CH);
  const int64_t grp = gid / CH;             // (row, head) index
  const bool live = grp < (int64_t)a.R * a.G;
  const int64_t row = live ? grp / a.G : 0;
  const int h = live ? (int)(grp % a.G) : 0;
  const int64_t off = h * (int64_t)D + chunk * 8;
  float x[8], g[8], w[8], y[8];
  unpack8v<Tr>(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a.x + row * a.x_sr + off)), x);
  if (ACT != kActNone) unpack8v<Tr>(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a.g + row * a.g_sr + off)), g);
  {
    const f32x4 w0 = *reinterpret_cast<const f32x4*>(a.w + off), w1 = *reinterpret_cast<const f32x4*>(a.w + off + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { w[e] = w0[e]; w[4 + e] = w1[e]; }
  }
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
#pragma unroll
  for (int o = CH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
  const float rstd = 1.0f / sqrtf(ss / D + a.eps);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    y[e] = x[e] * rstd * w[e];
    if (ACT != kActNone) {
      const float s = sigmoidf(g[e]);
      y[e] *= ACT == kActSwish ? g[e] * s : s;
    }
  }
  if (live) {
    *reinterpret_cast<u32x4*>(a.y + row * a.y_sr + off) = pack8v<Tr>(y);
    if (chunk == 0) a.rstd[grp] = rstd;
  }
}

constexpr int kNormStrip = 32;  // rows per thread in the backward

template <typename Tr, int D, int ACT>
__global__ __launch_bounds__(256) void norm_gate_bwd_kernel(const NormGateK a) {
  constexpr int CH = D / 8;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int chunk = (int)(gid % CH);
  const int64_t col = gid / CH;
  const int h = (int)(col % a.G);
  const int64_t strip = col / a.G;
  const int64_t r0 = strip * kNormStrip;
  const bool live = r0 < a.R;
  const int64_t r1 = live ? min((int64_t)a.R, r0 + kNormStrip) : r0;
  const int hh = live ? h : 0;
  const int64_t off = hh * (int64_t)D + chunk * 8;
  float w[8], dw[8];
  {
    const f32x4 w0 = *reinterpret_cast<const f32x4*>(a.w + off), w1 = *reinterpret_cast<const f32x4*>(a.w + off + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { w[e] = w0[e]; w[4 + e] = w1[e]; }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) dw[e] = 0.f;

  constexpr int U = 4;  // rows in flight
  for (int64_t rb = r0; rb < r1; rb += U) {
    u32x4 xv[U], gv[U], dyv[U];
    float rs[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t r = min(rb + u, r1 - 1);
      xv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a.x + r * a.x_sr + off));
      if (ACT != kActNone) gv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a.g + r * a.g_sr + off));
      dyv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a.dy + r * a.dy_sr + off));
      rs[u] = a.rstd[r * a.G + hh];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t r = rb + u;
      if (r < r1) {  // uniform over the lanes of a (head, strip) group
        float x[8], g[8], dy[8], dx[8], dg[8], wdy[8];
        unpack8v<Tr>(xv[u], x);
        if (ACT != kActNone) unpack8v<Tr>(gv[u], g);
        unpack8v<Tr>(dyv[u], dy);
        float c1 = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float xhat = x[e] * rs[u];
          const float yn = xhat * w[e];
          float dyn = dy[e];
          if (ACT != kActNone) {
            const float s = sigmoidf(g[e]);
            if (ACT == kActSwish) {
              dg[e] = dy[e] * yn * (s + g[e] * s * (1.f - s));
              dyn = dy[e] * g[e] * s;
            } else {
              dg[e] = dy[e] * yn * s * (1.f - s);
              dyn = dy[e] * s;
            }
          }
          dw[e] += dyn * xhat;
          wdy[e] = dyn * w[e];
          c1 += xhat * wdy[e];
          x[e] = xhat;
        }
#pragma unroll
        for (int o = CH / 2; o > 0; o >>= 1) c1 += __shfl_xor(c1, o);
        c1 *= 1.0f / D;
#pragma unroll
        for (int e = 0; e < 8; ++e) dx[e] = (wdy[e] - x[e] * c1) * rs[u];
        // Every input is read once (non-temporal loads above).  With a gate the kernel writes two streams and the
        // non-temporal hint on the stores pays as well (0.277 -> 0.262 ms at B4 T16384 H16 D128); with dx alone it costs.
        if (ACT != kActNone) {
          __builtin_nontemporal_store(pack8v<Tr>(dx), reinterpret_cast<u32x4*>(a.dx + r * a.dx_sr + off));
          __builtin_nontemporal_store(pack8v<Tr>(dg), reinterpret_cast<u32x4*>(a.dg + r * a.dg_sr + off));
        } else {
          *reinterpret_cast<u32x4*>(a.dx + r * a.dx_sr + off) = pack8v<Tr>(dx);
        }
      }
    }
  }
  if (live) {
    float* p = a.dw_partial + strip * (int64_t)a.G * D + off;
    const f32x4 lo = {dw[0], dw[1], dw[2], dw[3]}, hi = {dw[4], dw[5], dw[6], dw[7]};
    *reinterpret_cast<f32x4*>(p) = lo;
    *reinterpret_cast<f32x4*>(p + 4) = hi;
  }
}

// dst[group][j] = sum of src[s][j] over the rows s of the group (per_group consecutive rows), added in
// index order.  Two passes (strips -> groups of kReduceGroup strips -> total) turn the partial weight
// gradients into dw with enough parallelism and a summation order that does not depend on scheduling.
constexpr int kReduceGroup = 32;
__global__ __launch_bounds__(256) void reduce_rows_kernel(const float* __restrict__ src, float* __restrict__ dst, int64_t n_rows,
                                                          int width, int per_group) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= width) return;
  const int64_t s0 = (int64_t)blockIdx.y * per_group;
  const int64_t s1 = min(n_rows, s0 + per_group);
  float acc = 0.f;
  int64_t s = s0;
  for (; s + 8 <= s1; s += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = src[(s + u) * width + j];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u];
  }
  for (; s < s1; ++s) acc += src[s * width + j];
  dst[(int64_t)blockIdx.y * width + j] = acc;
}

#define FOX_NG_INST(TR, DD)                                                   \
  template __global__ void norm_gate_fwd_kernel<TR, DD, kActSigmoid>(const NormGateK); \
  template __global__ void norm_gate_fwd_kernel<TR, DD, kActSwish>(const NormGateK);   \
  template __global__ void norm_gate_fwd_kernel<TR, DD, kActNone>(const NormGateK);    \
  template __global__ void norm_gate_bwd_kernel<TR, DD, kActSigmoid>(const NormGateK); \
  template __global__ void norm_gate_bwd_kernel<TR, DD, kActSwish>(const NormGateK);   \
  template __global__ void norm_gate_bwd_kernel<TR, DD, kActNone>(const NormGateK);
#define FOX_NG_INST_ALL(TR) FOX_NG_INST(TR, 16) FOX_NG_INST(TR, 32) FOX_NG_INST(TR, 64) FOX_NG_INST(TR, 128)
FOX_NG_INST_ALL(Bf16)
FOX_NG_INST_ALL(Fp16)

int64_t norm_gate_strips(int64_t rows) { return (rows + kNormStrip - 1) / kNormStrip; }
// rows of G*D floats the backward needs as workspace: one per strip plus one per group of strips
int64_t norm_gate_workspace_rows(int64_t rows) {
  const int64_t strips = norm_gate_strips(rows);
  return strips + (strips + kReduceGroup - 1) / kReduceGroup;
}

template <typename Tr, int D>
static hipError_t norm_gate_d(const NormGateK& a, bool bwd, int act, hipStream_t s) {
  constexpr int CH = D / 8;
  if (!bwd) {
    const int64_t threads = (int64_t)a.R * a.G * CH;
    const dim3 grid((unsigned)((threads + 255) / 256));
    if (act == kActSwish) hipLaunchKernelGGL((norm_gate_fwd_kernel<Tr, D, kActSwish>), grid, dim3(256), 0, s, a);
    else if (act == kActNone) hipLaunchKernelGGL((norm_gate_fwd_kernel<Tr, D, kActNone>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((norm_gate_fwd_kernel<Tr, D, kActSigmoid>), grid, dim3(256), 0, s, a);
    return hipGetLastError();
  }
  const int64_t strips = norm_gate_strips(a.R);
  const int64_t threads = strips * a.G * CH;
  const dim3 grid((unsigned)((threads + 255) / 256));
  if (act == kActSwish) hipLaunchKernelGGL((norm_gate_bwd_kernel<Tr, D, kActSwish>), grid, dim3(256), 0, s, a);
  else if (act == kActNone) hipLaunchKernelGGL((norm_gate_bwd_kernel<Tr, D, kActNone>), grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL((norm_gate_bwd_kernel<Tr, D, kActSigmoid>), grid, dim3(256), 0, s, a);
  const int width = a.G * D;
  const int64_t groups = (strips + kReduceGroup - 1) / kReduceGroup;
  float* stage = a.dw_partial + strips * width;  // second part of the workspace
  hipLaunchKernelGGL(reduce_rows_kernel, dim3((unsigned)((width + 255) / 256), (unsigned)groups), dim3(256), 0, s, a.dw_partial,
                     stage, strips, width, kReduceGroup);
  hipLaunchKernelGGL(reduce_rows_kernel, dim3((unsigned)((width + 255) / 256), 1u), dim3(256), 0, s, stage, a.dw, groups, width,
                     (int)groups);
  return hipGetLastError();
}

template <typename Tr>
static hipError_t norm_gate_t(const NormGateK& a, int D, bool bwd, int act, hipStream_t s) {
  switch (D) {
    case 16: return norm_gate_d<Tr, 16>(a, bwd, act, s);
    case 32: return norm_gate_d<Tr, 32>(a, bwd, act, s);
    case 64: return norm_gate_d<Tr, 64>(a, bwd, act, s);
    case 128: return norm_gate_d<Tr, 128>(a, bwd, act, s);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_norm_gate(const NormGateK& a, int D, int dtype, bool bwd, int act, hipStream_t s) {
  return dtype == 0 ? norm_gate_t<Bf16>(a, D, bwd, act, s) : norm_gate_t<Fp16>(a, D, bwd, act, s);
}

}  // namespace fox
