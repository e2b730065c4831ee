// Shared device-side building blocks for the gfx950 Forgetting Attention kernels:
// vector types, MFMA wrappers, the swizzled LDS tile layout with its two read
// patterns (row operand via ds_read_b128, transposed operand via
// ds_read_b64_tr_b16), the global->LDS tile loader and small wave helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>
#include <utility>

namespace fox {

// Compile-time loop: f(std::integral_constant<int, I>{}) for I = BEGIN .. END-1, so that everything
// derived from the index is a constant expression inside f.
template <int BEGIN, typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, BEGIN + I>{}), ...);
}
template <int BEGIN, int END, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl<BEGIN>(f, std::make_integer_sequence<int, END - BEGIN>{});
}

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr int kWave = 64;

// ---------------------------------------------------------------------------
// Element traits: bf16 and fp16 share every kernel; only the MFMA opcode and the
// fp32 <-> 16-bit conversions differ.
// ---------------------------------------------------------------------------
struct Bf16 {
  static __device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  // c += a b with the accumulator in architectural VGPRs and the B operand in accumulation registers, whatever
  // register form the compiler picks for the kernel's other MFMAs (see mfma32_vgpr_acc below).
  static __device__ __forceinline__ void mfma32_vgpr_acc(f32x16& c, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  static __device__ __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
  static __device__ __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
  // acc + lo(w) + hi(w) in one instruction (v_dot2c_f32_bf16 against a pair of ones)
  static __device__ __forceinline__ float add_pair(uint32_t w, float acc) {
    const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), ones, acc, false);
  }
};

struct Fp16 {
  static __device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ void mfma32_vgpr_acc(f32x16& c, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    f16x2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  static __device__ __forceinline__ float lo(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[0]; }
  static __device__ __forceinline__ float hi(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[1]; }
  static __device__ __forceinline__ float add_pair(uint32_t w, float acc) {
    const f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, w), ones, acc, false);
  }
};

// mfma32_vgpr_acc: why an MFMA is written in assembly.  A kernel compiled for one wave per SIMD (512 registers) gets
// every MFMA builtin in the form whose accumulator lives in the accumulation registers (AGPRs); a vector
// instruction cannot read those, so each score that goes from an MFMA into exp2 / multiply costs a v_accvgpr_read
// first (two per score in the dK/dV kernel, 13 % of its instruction stream, and that kernel's time follows its
// instruction count).  The assembly form keeps such an accumulator in VGPRs and takes the loop-invariant B operand
// (the K or V rows a wave holds) from AGPRs, where it costs nothing.  The compiler inserts the memory waits for the
// operands of an asm statement, but not the wait states this target needs between an MFMA's write and a vector
// instruction's read of the same registers (12 issued instructions for this 8-pass MFMA): the caller must keep
// that distance by construction.  Back-to-back MFMAs that accumulate into the same registers need none.
//
// Pack eight consecutive accumulator values into one 16-byte MFMA operand.
template <typename Tr>
__device__ __forceinline__ u32x4 pack8(const f32x16& c, int first) {
  u32x4 r;
  r[0] = Tr::pack2(c[first + 0], c[first + 1]);
  r[1] = Tr::pack2(c[first + 2], c[first + 3]);
  r[2] = Tr::pack2(c[first + 4], c[first + 5]);
  r[3] = Tr::pack2(c[first + 6], c[first + 7]);
  return r;
}

// ---------------------------------------------------------------------------
// MFMA 32x32x16 register layouts (lane = 32*g + i):
//   A operand: row i,  k = 8*g .. 8*g+7          B operand: col i, same k
//   C/D:       col i,  row(r) = 8*(r/4) + 4*g + r%4   for r = 0..15
// A C tile can feed the next MFMA as its B operand with the C rows as the
// contraction index: operand element e = 4*u + t of k-slice h (16 rows) is
// accumulator register r = 8*h + e, i.e. C row 16*h + 8*u + 4*g + t.
// ---------------------------------------------------------------------------
__device__ __forceinline__ int c_row(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }

// ---------------------------------------------------------------------------
// LDS tile of ROWS x D 16-bit elements, organised in blocks of 64 sixteen-byte
// slots (1 KiB of data = 4 lines of 256 bytes; for D = 128 a line is a row), the
// unit one LDS-direct load instruction fills.  Blocks are 1040 bytes apart and
// within a block the slot index inside line l is XORed with 4*l.  With that
//   * 16 lanes reading the same chunk of 16 consecutive rows (MFMA row operand,
//     ds_read_b128) hit 16 different bank groups: 4 from the XOR, 4 from the pad;
//   * 32 lanes reading 4 rows x 64 bytes (transposed operand, ds_read_b64_tr_b16)
//     cover all 64 banks exactly once;
//   * the address is  lane term(chunk bits 2-3) + immediate(other chunk bits, row
//     block), so a kernel keeps 4 address registers per read pattern.
// ---------------------------------------------------------------------------
template <int D>
struct Tile {
  static constexpr int CH = D / 8;             // 16-byte chunks per row
  static constexpr int RPB = 64 / CH;          // rows per block
  static constexpr int BLOCK_BYTES = 1040;
  static constexpr int bytes(int rows) { return rows / RPB * BLOCK_BYTES; }
  static __device__ __forceinline__ int off(int row, int chunk) {
    const int p = (row % RPB) * CH + chunk;    // slot within the block
    const int line = p >> 4, q = p & 15;
    return (row / RPB) * BLOCK_BYTES + line * 256 + ((q ^ (line << 2)) << 4);
  }
};

// Row operand: eight consecutive elements (one chunk) of one row.
template <int D>
__device__ __forceinline__ u32x4 lds_row_operand(const char* tile, int row, int chunk) {
  return *reinterpret_cast<const u32x4*>(tile + Tile<D>::off(row, chunk));
}

__device__ __forceinline__ u32x2 lds_tr_read(const char* p) {
  typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
  return __builtin_bit_cast(u32x2, v);
}

// Transposed operand for k-slice rows [row16, row16+16) and the 32 columns
// [32*db, 32*db+32): lane (g, i) receives column 32*db + i at rows
// row16 + 8*u + 4*g + t (element 4*u + t).  ds_read_b64_tr_b16 works on blocks of
// 16 lanes: lane x of a block supplies the address of 4 consecutive columns
// 4*(x%4).. of row (x/4), and receives column x of those four rows.
template <int D>
__device__ __forceinline__ u32x4 lds_col_operand(const char* tile, int row16, int db, int lane) {
  const int g = lane >> 5, blk = (lane >> 4) & 1, x = lane & 15;
  int col = 32 * db + 16 * blk + 4 * (x & 3);
  if constexpr (D < 32) col &= (D - 1);  // columns >= D feed output rows nobody stores
  const int row = row16 + 4 * g + (x >> 2);
  const int inner = (col & 7) * 2;
  u32x2 lo = lds_tr_read(tile + Tile<D>::off(row, col >> 3) + inner);
  u32x2 hi = lds_tr_read(tile + Tile<D>::off(row + 8, col >> 3) + inner);
  u32x4 r = {lo[0], lo[1], hi[0], hi[1]};
  return r;
}

// ---------------------------------------------------------------------------
// Global -> register -> LDS loader for a ROWS x D tile of 16-bit elements.
// Rows at or beyond row_limit read as zero.  Split into load() and store() so the
// global loads of the next tile fly while the current one is consumed.
// ---------------------------------------------------------------------------
template <int D, int ROWS, int NT>
struct TileLoader {
  static constexpr int CH = D / 8;
  static constexpr int CHUNKS = ROWS * CH;
  static constexpr int PER = (CHUNKS + NT - 1) / NT;
  u32x4 reg[PER];

  __device__ __forceinline__ void load(const uint16_t* base, int64_t row_stride, int row0, int row_limit, int tid) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = tid + j * NT;
      const int row = idx / CH, ch = idx % CH;
      u32x4 z = {0u, 0u, 0u, 0u};
      reg[j] = z;
      if ((CHUNKS % NT == 0 || idx < CHUNKS) && row0 + row < row_limit)
        reg[j] = *reinterpret_cast<const u32x4*>(base + (int64_t)(row0 + row) * row_stride + ch * 8);
    }
  }
  __device__ __forceinline__ void store(char* tile, int tid) const {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = tid + j * NT;
      const int row = idx / CH, ch = idx % CH;
      if (CHUNKS % NT == 0 || idx < CHUNKS) *reinterpret_cast<u32x4*>(tile + Tile<D>::off(row, ch)) = reg[j];
    }
  }
};

// ---------------------------------------------------------------------------
// HBM -> LDS tile loader without registers: buffer loads with the LDS bit.  Each
// wave instruction moves 64 x 16 bytes into a contiguous 1 KiB block of LDS (slot
// of lane l = block base + 16*l, whatever address the lane reads from), so the
// swizzle is applied on the global side: each lane fetches the (row, chunk) that
// the tile layout assigns to its slot.  Rows at or beyond row_limit lie
// outside the buffer resource and read as zero.  The caller waits for vmcnt(0) and
// a barrier before the tile is read.
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void* lds_void_ptr;

__device__ __forceinline__ void wait_vmem_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }  // vmcnt(0), other counters untouched

// AUX is the cache-policy field of the load instruction: 0 for tiles that other workgroups read again out of L2 (the
// usual case), kLoadNonTemporal for a stream that nobody reads twice.
constexpr int kLoadNonTemporal = 2;
template <int D, int ROWS, int NW = 4, int AUX = 0>
struct DirectTileLoader {
  static constexpr int CH = D / 8;
  static constexpr int NBLK = ROWS * CH / 64;        // 1 KiB blocks per tile
  static constexpr int PER = (NBLK + NW - 1) / NW;   // blocks per wave (NW waves)
  static_assert(ROWS * CH % 64 == 0, "tile must be a whole number of 1 KiB blocks");
  int voff[PER];
  int wave;

  __device__ __forceinline__ DirectTileLoader(int64_t row_stride, int wave_, int lane) : wave(wave_) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      // physical slot of this lane inside block (wave + NW*j) -> the (row, chunk) stored there
      const int line = lane >> 4, q = (lane & 15) ^ (line << 2);
      const int p = line * 16 + q;
      const int row = (wave + NW * j) * Tile<D>::RPB + p / CH, c = p % CH;
      voff[j] = (int)(row * row_stride * 2) + (c << 4);
    }
  }
  // Byte extent of the tile whose first row is row0, for its buffer resource: rows at or beyond row_limit
  // are out of range, and an extent of 0 (row_limit <= row0) makes every load return zero.
  // Only the tile's own ROWS rows count, so the extent stays far below the 32-bit limit of a buffer resource
  // however long the sequence and however large the row stride.
  __device__ __forceinline__ int extent(int64_t row_stride, int row0, int row_limit) const {
    const int rows = row_limit - row0 < ROWS ? row_limit - row0 : ROWS;
    return rows > 0 ? (int)(((int64_t)(rows - 1) * row_stride + D) * 2) : 0;
  }
  // The j-th (a constant at every call site) of this wave's PER load instructions of the tile that
  // starts at p, so that a kernel can spread them over its compute instead of issuing them back to back
  // (each one occupies the wave's issue slot, and the CU's memory pipeline, for tens of cycles).
  __device__ __forceinline__ void issue_one(int j, const uint16_t* p, int bytes, char* tile) const {
    const int blk = wave + NW * j;
    if (NBLK % NW == 0 || blk < NBLK) {
      const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p), 0, bytes, 0x00020000);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_ptr)(tile + blk * Tile<D>::BLOCK_BYTES), 16, voff[j], 0, 0, AUX);
    }
  }
  __device__ __forceinline__ void issue(const uint16_t* base, int64_t row_stride, int row0, int row_limit, char* tile) const {
    const uint16_t* p = base + (int64_t)row0 * row_stride;
    const int bytes = extent(row_stride, row0, row_limit);
#pragma unroll
    for (int j = 0; j < PER; ++j) issue_one(j, p, bytes, tile);
  }
};

// Operand held in registers for a whole kernel: lane (g, i) keeps row (row0 + i),
// elements 16*kk + 8*g .. +7 for every k-step kk.  Rows >= row_limit are zero.
template <int D>
__device__ __forceinline__ void load_row_operand_regs(u32x4 (&dst)[D / 16], const uint16_t* base, int64_t row_stride, int row,
                                             int row_limit, int g) {
  // branch-free: every load is issued before any of them is waited for (rows past the limit read the
  // last valid row and are zeroed afterwards; row_limit >= 1)
  const bool valid = row < row_limit;
  const uint16_t* p = base + (int64_t)(valid ? row : row_limit - 1) * row_stride + 8 * g;
#pragma unroll
  for (int kk = 0; kk < D / 16; ++kk) dst[kk] = *reinterpret_cast<const u32x4*>(p + 16 * kk);
  const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int kk = 0; kk < D / 16; ++kk) dst[kk] = valid ? dst[kk] : z;
}

// ---------------------------------------------------------------------------
// Wave helpers
// ---------------------------------------------------------------------------
// Value held by the partner lane in the other 32-lane half.
__device__ __forceinline__ float half_max(float x) {
  unsigned v = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_sum(float x) {
  unsigned v = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Store a wave's transposed accumulator block as rows of 16-bit values.  Lane (g, i) holds row i of
// 32 rows; register r of acc[db] is column 32*db + 8*(r/4) + 4*g + r%4.  Written straight to global
// memory that is 8 bytes per lane scattered over 32 rows; staged through a wave-private LDS area of
// kStoreStageBytes<D> the global stores are 16 bytes per lane and each instruction covers whole rows.
// Rows at or beyond row_limit are not stored.  The caller makes sure nobody else uses the staging area.
template <int D>
constexpr int kStoreStageBytes = 32 * (2 * D + 16);

template <typename Tr, int D>
__device__ __forceinline__ void store_rows_via_lds(char* stage, const f32x16 (&acc)[(D + 31) / 32], float mul, uint16_t* dst,
                                                   int64_t row_stride, int row0, int row_limit, int lane) {
  constexpr int DB = (D + 31) / 32, CH = D / 8, RS = 2 * D + 16;
  const int g = lane >> 5, i = lane & 31;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const int d = 32 * db + 8 * q4 + 4 * g;
      if (d < D) {
        u32x2 w;
        w[0] = Tr::pack2(acc[db][4 * q4 + 0] * mul, acc[db][4 * q4 + 1] * mul);
        w[1] = Tr::pack2(acc[db][4 * q4 + 2] * mul, acc[db][4 * q4 + 3] * mul);
        *reinterpret_cast<u32x2*>(stage + i * RS + 2 * d) = w;
      }
    }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int idx0 = 0; idx0 < 32 * CH; idx0 += kWave) {
    const int idx = idx0 + lane, row = idx / CH, ch = idx % CH;
    if ((32 * CH % kWave == 0 || idx < 32 * CH) && row0 + row < row_limit) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(stage + row * RS + 16 * ch);
      // written once, read by a later kernel at the earliest: the non-temporal hint keeps the rows from pushing K, V and
      // Q tiles that other workgroups still want out of L2 (2-3 % of a heavily pruned step and of small shapes, nothing where the kernels are matrix-bound)
      __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst + (int64_t)(row0 + row) * row_stride + 8 * ch));
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();   // the staging area may be rewritten after this
}

// Gate activations of the per-head RMS norm (FOX_ACT_* of the public header).
enum : int { kActSigmoid = 0, kActSwish = 1, kActNone = 2 };
__device__ __forceinline__ float sigmoidf(float x) { return 1.0f / (1.0f + __expf(-x)); }

// store_rows_via_lds with the gated per-head RMS norm applied on the way out: besides the rows themselves
// (x = acc * mul rounded to 16 bits, to x_dst unless that is null) it writes
//   y[row, :] = x * rstd[row] * w[:] * act(gate[row, :]),   rstd = 1 / sqrt(mean_d x^2 + eps),
// computed from the rounded x, as a separate normalisation pass over the stored rows would, and rstd itself
// (one float per row, rstd_stride apart).  gate is not read when act is kActNone.  The 16 spare bytes that
// pad every staged row carry its rstd from the lanes that own the row to the lanes that store it.  Nothing of
// the epilogue is prefetched while the accumulators are live: the kernels that end with it run at the register
// limit of their occupancy.
template <typename Tr, int D>
__device__ __forceinline__ void store_rows_norm_gate(char* stage, const f32x16 (&acc)[(D + 31) / 32], float mul, uint16_t* x_dst,
                                                     int64_t x_stride, const uint16_t* gate, int64_t gate_stride, uint16_t* y_dst,
                                                     int64_t y_stride, const float* w, float* rstd_dst, int64_t rstd_stride,
                                                     float eps, int act, int row0, int row_limit, int lane) {
  constexpr int DB = (D + 31) / 32, CH = D / 8, RS = 2 * D + 16, NIT = (32 * CH + kWave - 1) / kWave;
  const int g = lane >> 5, i = lane & 31;
  float ss = 0.f;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const int d = 32 * db + 8 * q4 + 4 * g;
      if (d < D) {
        u32x2 v;
        v[0] = Tr::pack2(acc[db][4 * q4 + 0] * mul, acc[db][4 * q4 + 1] * mul);
        v[1] = Tr::pack2(acc[db][4 * q4 + 2] * mul, acc[db][4 * q4 + 3] * mul);
#pragma unroll
        for (int e = 0; e < 2; ++e) ss += Tr::lo(v[e]) * Tr::lo(v[e]) + Tr::hi(v[e]) * Tr::hi(v[e]);
        *reinterpret_cast<u32x2*>(stage + i * RS + 2 * d) = v;
      }
    }
  ss = half_sum(ss);  // the two halves of the wave hold the two halves of every row
  const float rs_own = 1.0f / sqrtf(ss / D + eps);
  if (g == 0) *reinterpret_cast<float*>(stage + i * RS + 2 * D) = rs_own;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int idx = it * kWave + lane, row = idx / CH, ch = idx % CH;
    if ((32 * CH % kWave == 0 || idx < 32 * CH) && row0 + row < row_limit) {
      u32x4 gv = {0u, 0u, 0u, 0u};
      if (act != kActNone) gv = *reinterpret_cast<const u32x4*>(gate + (int64_t)(row0 + row) * gate_stride + 8 * ch);
      const u32x4 xv = *reinterpret_cast<const u32x4*>(stage + row * RS + 16 * ch);
      const float rs = *reinterpret_cast<const float*>(stage + row * RS + 2 * D);
      if (x_dst) __builtin_nontemporal_store(xv, reinterpret_cast<u32x4*>(x_dst + (int64_t)(row0 + row) * x_stride + 8 * ch));
      const f32x4 w0 = *reinterpret_cast<const f32x4*>(w + 8 * ch), w1 = *reinterpret_cast<const f32x4*>(w + 8 * ch + 4);
      u32x4 yv;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float y0 = Tr::lo(xv[e]) * rs * (e < 2 ? w0[2 * e] : w1[2 * e - 4]);
        float y1 = Tr::hi(xv[e]) * rs * (e < 2 ? w0[2 * e + 1] : w1[2 * e - 3]);
        if (act != kActNone) {
          const float g0 = Tr::lo(gv[e]), g1 = Tr::hi(gv[e]);
          // (hardware reciprocal, one unit in the last place: this loop sits at the tail of a workgroup's critical path)
          const float s0 = __builtin_amdgcn_rcpf(1.0f + __expf(-g0)), s1 = __builtin_amdgcn_rcpf(1.0f + __expf(-g1));
          y0 *= act == kActSwish ? g0 * s0 : s0;
          y1 *= act == kActSwish ? g1 * s1 : s1;
        }
        yv[e] = Tr::pack2(y0, y1);
      }
      __builtin_nontemporal_store(yv, reinterpret_cast<u32x4*>(y_dst + (int64_t)(row0 + row) * y_stride + 8 * ch));
      if (ch == 0) rstd_dst[(int64_t)(row0 + row) * rstd_stride] = rs;
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();   // the staging area may be rewritten after this
}

// Start value of a 32x32 MFMA accumulator whose row r carries the per-row term
// t[row0 + r] (read from LDS): the matrix pipe then adds the dot products to it for
// free, which saves one vector instruction per score.
__device__ __forceinline__ f32x16 acc_init(const float* t, int row0, int g) {
  f32x16 v;
#pragma unroll
  for (int q4 = 0; q4 < 4; ++q4) {
    const f32x4 x = *reinterpret_cast<const f32x4*>(&t[row0 + 8 * q4 + 4 * g]);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[4 * q4 + e] = x[e];
  }
  return v;
}

// The kernels fold per-row bias terms into the MFMA accumulators as bias / scale and multiply
// the finished dot product by scale, so scale must not be zero: a scale below 1e-30 in
// magnitude is replaced by 1e-30, for which scale * (q.k) still rounds to nothing against
// the bias.
__device__ __forceinline__ float nonzero_scale(float s) { return fabsf(s) < 1e-30f ? 1e-30f : s; }

// Workgroup id -> (bh, tile) with every tile of one (batch, head) on one XCD (the
// hardware deals consecutive workgroup ids round-robin over 8 XCDs, each with its
// own L2), heaviest tiles (largest index under a causal mask) first.
__device__ __forceinline__ void decode_block(int wid, int n_tiles, int n_bh, int& bh, int& tile) {
  if ((n_bh & 7) == 0) {
    const int xcd = wid & 7, seq = wid >> 3;
    bh = (seq / n_tiles) * 8 + xcd;
    tile = n_tiles - 1 - (seq % n_tiles);
  } else {
    bh = wid / n_tiles;
    tile = n_tiles - 1 - (wid % n_tiles);
  }
}

// Adaptive Computation Pruning, query-side bound: the first key block of width BN
// in [0, t_max] whose largest decay  c_out - c[last column of the block]  is not
// below thr.  c is non-increasing, so the blocks before it are exactly the
// prunable ones and the kept blocks form one run that ends at t_max.  The search
// walks back from t_max, 64 candidate blocks per round (one per lane, one memory
// round trip): where pruning bites, the run is short and the first round finds its
// start; where nothing is pruned the rounds are few against the work that follows.
// Evaluated by all 64 lanes at once; the result is wave-uniform.  Returns t_max when
// no block qualifies (the diagonal block is always visited).
__device__ __forceinline__ int acp_first_kept_block(const float* c_row, float c_out, float thr, int N, int BN, int t_max, int lane) {
  int first = t_max;
  for (int top = t_max; top >= 0; top -= kWave) {
    const int t = top - lane;
    bool keep = false;
    if (t >= 0) {
      int col = t * BN + BN - 1;
      col = col < N - 1 ? col : N - 1;
      keep = !((c_out - c_row[col]) < thr);
    }
    const unsigned long long m = __ballot(keep);
    if (m == 0) break;                                  // the run ended exactly at the previous round
    first = top - (63 - __clzll((long long)m));          // lowest kept block of this round
    const int valid = top + 1 < kWave ? top + 1 : kWave;
    if (__popcll(m) < valid) break;                     // a pruned block inside this round: the run starts here
  }
  return first;
}

// Classes of key tiles in the dK/dV pass under pruning.  A launch of class kClassLight handles only the 128-key
// tiles whose pruning bound lies within `limit` positions of their diagonal, a launch of class kClassHeavy only
// the others; both evaluate the same predicate, so every tile is handled exactly once.  limit < 0 names every
// tile light.
constexpr int kClassAll = 0, kClassLight = 1, kClassHeavy = 2;

// Key tile whose last key is at position n_last (c_last = c[n_last]): light when the query row that sits
// `limit` positions after n_last is already below the threshold against that key (c is non-increasing, so
// every later row is too), or when there is no such row.
__device__ __forceinline__ bool acp_light_k(const float* c_row, float c_last, float thr, int n_last, int N, int limit) {
  if (limit < 0 || n_last + limit >= N) return true;
  return (c_row[n_last + limit] - c_last) < thr;
}

// Key-side bound: the first query block (BMQ rows, first row u*BMQ) in [u_lo, U)
// whose largest decay against the key tile,  c[P_SEQ + u*BMQ] - c_last,  is below
// thr; every later block is prunable too.  Returns U when none is.
__device__ __forceinline__ int acp_first_pruned_qblock(const float* c_row, float c_last, float thr, int p_seq, int BMQ, int u_lo,
                                              int U, int lane) {
  for (int base = u_lo; base < U; base += kWave) {
    const int u = base + lane;
    bool pruned = false;
    if (u < U) pruned = (c_row[p_seq + u * BMQ] - c_last) < thr;
    const unsigned long long m = __ballot(pruned);
    if (m) return base + __ffsll((long long)m) - 1;
  }
  return U;
}

}  // namespace fox
