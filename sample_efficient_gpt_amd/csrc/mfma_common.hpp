// Building blocks shared by the bf16 MFMA kernels (gfx950, wave64).
//
// MFMA used everywhere: v_mfma_f32_32x32x16_bf16, D(32x32) += A(32x16) * B(16x32).
//   A operand, lane l: row  = l % 32, k = 8*(l/32) + t, t = 0..7   (8 bf16 = 4 VGPRs)
//   B operand, lane l: col  = l % 32, k = 8*(l/32) + t
//   C/D,       lane l: col  = l % 32, row(r) = 8*(r/4) + 4*(l/32) + r%4, r = 0..15
// A C tile whose rows are the contraction index of the next product is reused directly as that
// product's B (or A) operand: registers 8s..8s+7 of a lane hold rows {4hh..4hh+3, 8+4hh..8+4hh+3} + 16s
// (hh = l/32).  The contraction order inside an MFMA is free as long as both operands agree, so the
// other operand is fetched in exactly that row order ("CPERM order") with two transposing LDS reads.
#pragma once

#include <type_traits>

#include "common.hpp"

namespace segpt {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kBK = 64;        // streamed rows per LDS tile
constexpr int kThreadsM = 256; // 4 waves

__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// value held by lane l^32 combined with the own value
__device__ __forceinline__ float half_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// acc + lo + hi of one packed bf16 pair (v_dot2c_f32_bf16 with a (1,1) operand): sums the ROUNDED values,
// i.e. exactly what the MFMA consuming the packed operand sees.
__device__ __forceinline__ float add_bf16_pair(uint32_t w, float acc) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  const bf2 one = {(__bf16)1.0f, (__bf16)1.0f};
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf2, w), one, acc, false);
}

__device__ __forceinline__ u32x4 scale8(u32x4 v, float f) {
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = pack_bf16x2(bf16lo(v[i]) * f, bf16hi(v[i]) * f);
  return r;
}
// ---------------------------------------------------------------------------------------------------
// Swizzled, unpadded LDS tiles filled by direct global->LDS loads (global_load_lds_dwordx4: every lane
// names its own 16 global bytes, the wave's 64 x 16 B land contiguously at a wave-uniform LDS address).
// Tile = 64 rows of kRB = 2*D bytes; the 16-byte chunk c of row r is stored at chunk position c ^ f(r).
// LDS has 64 banks of 4 bytes; a ds_read_b128 is served 16 lanes at a time, and the 16 lanes of a row-major
// fragment read sit in 16 consecutive rows at one logical chunk, so f must spread rows that share banks
// (every second row at D=64, every row at D=128) over distinct chunk positions; the transposing b64 reads
// touch 4 rows x 32 bytes per 16 lanes and want the rows of a pair two apart in different chunk pairs.
//   D = 64  (8 chunks / row):   f(r) = (r >> 1) & 7
//   D = 128 (16 chunks / row):  f(r) = ((r & 3) << 2) | ((r >> 2) & 3)
// Both depend on r mod 16 only and satisfy f(r + 8) = f(r) ^ kHiXorChunks for r < 8.
template <int D, int ROWS = kBK>
struct Swz {
  static constexpr int kRows = ROWS;                    // rows per tile (64; the head_dim-128 forward streams 32-row tiles)
  static constexpr int kRB = 2 * D;                     // bytes per row
  static constexpr int kTileBytes = ROWS * kRB;         // 8 KB (D=64, or D=128 with 32 rows) / 16 KB (D=128)
  static constexpr int kChunks = kRB / 16;              // chunks per row
  static constexpr int kRowsPerInst = 1024 / kRB;       // rows one wave-wide load covers
  static constexpr int kPasses = kTileBytes / 1024 / 4; // wave-wide loads per wave per tile (4 waves)
  static constexpr int kHiXor = (D == 64 ? 4 : 2) << 4; // byte XOR between the swizzle terms of rows r and r+8
  static __device__ __forceinline__ int f(int row) {
    return D == 64 ? ((row >> 1) & 7) : (((row & 3) << 2) | ((row >> 2) & 3));
  }
  static_assert(D == 64 || D == 128, "swizzle is defined for 128- and 256-byte rows");
  static_assert(kPasses >= 1 && kPasses * 4 * kRowsPerInst == ROWS, "four waves fill a tile in whole passes");
};

// s_waitcnt vmcnt(n) only (gfx9 encoding: vmcnt = {imm[15:14], imm[3:0]}, expcnt / lgkmcnt left at max)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0F70);
}

// LDS is addressed by 32-bit byte addresses below (integers, so that the XOR swizzle is plain arithmetic)
typedef __attribute__((address_space(3))) char* lds_char_ptr;
__device__ __forceinline__ uint32_t lds_addr_of(const void* shared_obj) {
  return (uint32_t)(uintptr_t)(lds_char_ptr)shared_obj;
}
// The two direct loads are written as inline assembly on purpose: the compiler treats the builtin form
// as an LDS write of unknown extent and drains every outstanding vector load (s_waitcnt vmcnt(0)) before
// each barrier and before issuing further ones, which would serialise the whole prefetch pipeline.
// Completion is tracked by hand instead: wait_vmcnt<N>() followed by __syncthreads() publishes a stage.
// (Hidden loads only make the compiler's own vmcnt waits conservative, never too weak: the counter
// retires in order.)
// On this architecture family an LDS-DMA instruction may not read M0 in the instruction slot right after a scalar
// write to it (one wait state is required; the compiler inserts it for its own code but cannot see inside an
// asm string), hence the s_nop: without it the load can, rarely, land at the previous destination.
__device__ __forceinline__ void gload_lds16(const void* gsrc, uint32_t lds_dst_wave_uniform) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(gsrc), "s"(lds_dst_wave_uniform)
               : "memory", "m0");
}
// the same load addressed as a wave-uniform base pointer plus a 32-bit byte offset per lane (no 64-bit vector
// arithmetic per load; the offset can be loop-invariant while the base walks over the tensor)
__device__ __forceinline__ void gload_lds16_so(const void* base_wave_uniform, uint32_t lane_off, uint32_t lds_dst_wave_uniform) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(lane_off), "s"(base_wave_uniform), "s"(lds_dst_wave_uniform)
               : "memory", "m0");
}
__device__ __forceinline__ void gload_lds4_so(const void* base_wave_uniform, uint32_t lane_off, uint32_t lds_dst_wave_uniform) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
               :
               : "v"(lane_off), "s"(base_wave_uniform), "s"(lds_dst_wave_uniform)
               : "memory", "m0");
}
__device__ __forceinline__ void gload_lds4(const void* gsrc, uint32_t lds_dst_wave_uniform) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
               :
               : "v"(gsrc), "s"(lds_dst_wave_uniform)
               : "memory", "m0");
}
__device__ __forceinline__ u32x4 lds_read16(uint32_t addr) {
  return *(const __attribute__((address_space(3))) u32x4*)addr;
}
typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4 lds_read_f4(uint32_t addr) {
  return *(const __attribute__((address_space(3))) f32x4*)addr;
}

// Which (row, global chunk) a lane fetches for the wave-wide load number `wave` of a tile (later passes add
// 4*kRowsPerInst rows, a multiple of 16, so the swizzle term does not change): returns row in .x, byte column in .y
template <int D>
__device__ __forceinline__ int2 swz_src(int lane, int wave) {
  const int row = wave * Swz<D>::kRowsPerInst + lane / Swz<D>::kChunks;
  const int c = (lane % Swz<D>::kChunks) ^ Swz<D>::f(row);
  return make_int2(row, c * 16);
}
// Per-lane byte offset (within a tile) of the row-major fragment of k-step 0, row block 0; k-step ks is
// this offset XOR (ks << 5), row block rb adds 32*kRB.
template <int D>
__device__ __forceinline__ int swz_off_rm(int lane) {
  const int ln = lane & 31, hh = lane >> 5;
  return ln * Swz<D>::kRB + ((hh ^ Swz<D>::f(ln)) << 4);
}
// Transposed fragment of a row-major tile [row][col]: the lane's MFMA row is a COLUMN of the tile
// (col = 32*cb + l%32) and its 8 contraction entries are tile rows in CPERM order 16*s + {4hh..4hh+3, 8+4hh..8+4hh+3}.
// ds_read_b64_tr_b16 semantics (per 16-lane group, source lane r gives the address of 4 elements):
//   result[lane i][e] = LDS[addr(4e + i/4) + i%4]
// so source lane r points at row base + r/4, column cbase + 4*(r%4) and lane i receives column cbase + i,
// rows base..base+3.
// Per-lane byte offset of the transposed fragment of column block 0, row step 0 (first of its two
// 8-byte reads; the second is 8 rows further, which also flips kHiXor in the swizzle term): column block
// cb is this offset XOR (cb << 6), row step s adds 16*s*kRB.
template <int D>
__device__ __forceinline__ int swz_off_tr(int lane) {
  const int r = lane & 15, g1 = (lane >> 4) & 1, hh = lane >> 5;
  const int row = 4 * hh + (r >> 2);          // 0..7
  const int c = 2 * g1 + ((r & 3) >> 1);      // chunk within the 64-byte column block
  return row * Swz<D>::kRB + ((c ^ Swz<D>::f(row)) << 4) + ((r & 1) << 3);
}
template <int D>
__device__ __forceinline__ bf16x8 swz_frag_rm(uint32_t tile_plus_lane_off, int rb, int ks) {
  return as_bf16x8(lds_read16((tile_plus_lane_off ^ (uint32_t)(ks << 5)) + rb * 32 * Swz<D>::kRB));
}
template <int D>
__device__ __forceinline__ bf16x8 swz_frag_tr(uint32_t tile_plus_lane_off, int cb, int s) {
  const uint32_t p = (tile_plus_lane_off ^ (uint32_t)(cb << 6)) + 16 * s * Swz<D>::kRB;
  const uint32_t q = (tile_plus_lane_off ^ (uint32_t)((cb << 6) ^ Swz<D>::kHiXor)) + (16 * s + 8) * Swz<D>::kRB;
  typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(q));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, v);
}

template <int N>
using IC = std::integral_constant<int, N>;

// pack registers 8s..8s+7 of a C tile into a bf16 operand (CPERM order)
__device__ __forceinline__ bf16x8 pack_c_half(const f32x16& c, int s) {
  u32x4 w;
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = pack_bf16x2(c[8 * s + 2 * i], c[8 * s + 2 * i + 1]);
  return as_bf16x8(w);
}

// same, and adds the eight packed values to `sum` (the scalar words are summed before the vector is
// assembled: summing elements extracted back out of the assembled vector was miscompiled by hipcc 7.2)
// Two running sums (the caller adds them at the end): ONE accumulator makes every block a chain of eight dependent
// dot instructions whose latency, not their count, is what costs (measured on a register-only skeleton of the
// forward block: 51 % of the MFMA rate with one chain, 62 % with two or four, 63 % with no row sum at all; in
// the forward kernel itself the scheduler already parks the sums behind the tile wait, so its time is unchanged).
__device__ __forceinline__ bf16x8 pack_c_half_sum(const f32x16& c, int s, float (&sum)[2]) {
  const uint32_t w0 = pack_bf16x2(c[8 * s + 0], c[8 * s + 1]);
  const uint32_t w1 = pack_bf16x2(c[8 * s + 2], c[8 * s + 3]);
  const uint32_t w2 = pack_bf16x2(c[8 * s + 4], c[8 * s + 5]);
  const uint32_t w3 = pack_bf16x2(c[8 * s + 6], c[8 * s + 7]);
  sum[0] = add_bf16_pair(w1, add_bf16_pair(w0, sum[0]));
  sum[1] = add_bf16_pair(w3, add_bf16_pair(w2, sum[1]));
  const u32x4 w = {w0, w1, w2, w3};
  return as_bf16x8(w);
}

// ---- rotary embedding in the two register layouts of a tensor row.  The table entries of the row's position
// (cosr / sinr: D/2 floats each) are LOADED into registers by one function and APPLIED by another, so that a kernel
// can request them together with its other start-up loads (one memory round trip) and use them later.
// B-operand layout: x[ks][t] = element 16 ks + 8 hh + t; the partner of ks is ks + KS/2 in the same lane
template <int KS>
struct RopeB {
  float c[KS / 2][8], s[KS / 2][8];
};
template <int KS>
__device__ __forceinline__ RopeB<KS> rope_b_load(const float* cosr, const float* sinr, int hh) {
  RopeB<KS> r;
#pragma unroll
  for (int ks = 0; ks < KS / 2; ++ks) {
    const float4 c0 = *reinterpret_cast<const float4*>(cosr + 16 * ks + 8 * hh);
    const float4 c1 = *reinterpret_cast<const float4*>(cosr + 16 * ks + 8 * hh + 4);
    const float4 s0 = *reinterpret_cast<const float4*>(sinr + 16 * ks + 8 * hh);
    const float4 s1 = *reinterpret_cast<const float4*>(sinr + 16 * ks + 8 * hh + 4);
    r.c[ks][0] = c0.x; r.c[ks][1] = c0.y; r.c[ks][2] = c0.z; r.c[ks][3] = c0.w;
    r.c[ks][4] = c1.x; r.c[ks][5] = c1.y; r.c[ks][6] = c1.z; r.c[ks][7] = c1.w;
    r.s[ks][0] = s0.x; r.s[ks][1] = s0.y; r.s[ks][2] = s0.z; r.s[ks][3] = s0.w;
    r.s[ks][4] = s1.x; r.s[ks][5] = s1.y; r.s[ks][6] = s1.z; r.s[ks][7] = s1.w;
  }
  return r;
}
template <int KS>
__device__ __forceinline__ void rope_b_apply(float (&x)[KS][8], const RopeB<KS>& r) {
#pragma unroll
  for (int ks = 0; ks < KS / 2; ++ks)
#pragma unroll
    for (int t = 0; t < 8; ++t) rope_pair(x[ks][t], x[ks + KS / 2][t], r.c[ks][t], r.s[ks][t]);
}
template <int KS>
__device__ __forceinline__ void rope_b_layout(float (&x)[KS][8], const float* cosr, const float* sinr, int hh) {
  rope_b_apply<KS>(x, rope_b_load<KS>(cosr, sinr, hh));
}
// C-tile layout of load_ct_block / store_ct_block: x[mb][4c + i] = element 32 mb + 8 c + 4 hh + i; the
// partner of mb is mb + MB/2 in the same lane and register
template <int MB>
struct RopeCt {
  float c[MB / 2][16], s[MB / 2][16];
};
template <int MB>
__device__ __forceinline__ RopeCt<MB> rope_ct_load(const float* cosr, const float* sinr, int hh) {
  RopeCt<MB> r;
#pragma unroll
  for (int mb = 0; mb < MB / 2; ++mb)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const float4 c4 = *reinterpret_cast<const float4*>(cosr + 32 * mb + 8 * c + 4 * hh);
      const float4 s4 = *reinterpret_cast<const float4*>(sinr + 32 * mb + 8 * c + 4 * hh);
      r.c[mb][4 * c] = c4.x; r.c[mb][4 * c + 1] = c4.y; r.c[mb][4 * c + 2] = c4.z; r.c[mb][4 * c + 3] = c4.w;
      r.s[mb][4 * c] = s4.x; r.s[mb][4 * c + 1] = s4.y; r.s[mb][4 * c + 2] = s4.z; r.s[mb][4 * c + 3] = s4.w;
    }
  return r;
}
template <int MB, bool INVERSE>
__device__ __forceinline__ void rope_ct_apply(float (&x)[MB][16], const RopeCt<MB>& r) {
#pragma unroll
  for (int mb = 0; mb < MB / 2; ++mb)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if (INVERSE) rope_pair_inv(x[mb][i], x[mb + MB / 2][i], r.c[mb][i], r.s[mb][i]);
      else rope_pair(x[mb][i], x[mb + MB / 2][i], r.c[mb][i], r.s[mb][i]);
    }
}
// raw bf16 words of a B-operand row -> floats
template <int KS>
__device__ __forceinline__ void unpack_b_layout(const u32x4 (&raw)[KS], float (&x)[KS][8]) {
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
#pragma unroll
    for (int i = 0; i < 4; ++i) { x[ks][2 * i] = bf16lo(raw[ks][i]); x[ks][2 * i + 1] = bf16hi(raw[ks][i]); }
}

// ---- helpers shared by the ring kernels (forward, dQ, dK/dV)
__device__ __forceinline__ float gprod_at(const segpt_attn_params& p, int d) {
  float g = p.gq_numel == 1 ? p.g_q[0] : p.g_q[d];
  if (p.gk_numel == 1) g *= p.g_k[0];
  else if (p.gk_numel > 1) g *= p.g_k[d];
  return g;
}

// store a C tile column block: lane = row of the output tensor, registers = 32 consecutive columns
// starting at 32*mb, values already scaled.  Lanes l and l^32 exchange halves so that each lane
// writes 16 contiguous bytes.
__device__ __forceinline__ void store_ct_block(uint16_t* rowp, int mb, int hh, bool live, const float (&val)[16]) {
#pragma unroll
  for (int cc = 0; cc < 2; ++cc) {
    const uint32_t x0 = pack_bf16x2(val[8 * cc + 0], val[8 * cc + 1]);
    const uint32_t x1 = pack_bf16x2(val[8 * cc + 2], val[8 * cc + 3]);
    const uint32_t y0 = pack_bf16x2(val[8 * cc + 4], val[8 * cc + 5]);
    const uint32_t y1 = pack_bf16x2(val[8 * cc + 6], val[8 * cc + 7]);
    auto s0 = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
    auto s1 = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
    const u32x4 w = {s0[0], s1[0], s0[1], s1[1]};
    if (live) *reinterpret_cast<u32x4*>(rowp + 32 * mb + 16 * cc + 8 * hh) = w;
  }
}

// raw bf16 values of a tensor row at the 16 columns a lane's C registers of block mb map to
__device__ __forceinline__ void load_ct_block(const uint16_t* rowp, int mb, int hh, float (&out)[16]) {
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const u32x2 w = *reinterpret_cast<const u32x2*>(rowp + 32 * mb + 8 * c + 4 * hh);
    out[4 * c + 0] = bf16lo(w[0]); out[4 * c + 1] = bf16hi(w[0]);
    out[4 * c + 2] = bf16lo(w[1]); out[4 * c + 3] = bf16hi(w[1]);
  }
}

// the same 16 columns kept as packed bf16 pairs (8 registers), for a row that is read early and used late
__device__ __forceinline__ void load_ct_block_raw(const uint16_t* rowp, int mb, int hh, u32x2 (&out)[4]) {
#pragma unroll
  for (int c = 0; c < 4; ++c) out[c] = *reinterpret_cast<const u32x2*>(rowp + 32 * mb + 8 * c + 4 * hh);
}
__device__ __forceinline__ void unpack_ct_block(const u32x2 (&w)[4], float (&out)[16]) {
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    out[4 * c + 0] = bf16lo(w[c][0]); out[4 * c + 1] = bf16hi(w[c][0]);
    out[4 * c + 2] = bf16lo(w[c][1]); out[4 * c + 3] = bf16hi(w[c][1]);
  }
}

__device__ __forceinline__ f32x16 splat16(float x) {
  f32x16 v;
#pragma unroll
  for (int r = 0; r < 16; ++r) v[r] = x;
  return v;
}

// Direct global->LDS loads of two [64, D] bf16 tiles (rows row0..row0+63 of two row-major tensors) into one
// stage.  The lane's byte offsets from row `row0` do not depend on the tile as long as it is full, so they are
// computed once (rows_left = 64) and a tile then costs no vector arithmetic; a last, partial tile gets its own
// set, in which rows past rows_left re-read the last valid row (callers mask them).
//   step_*: bytes between rows; lane_row / lane_col: from swz_src()
template <int D, int ROWS = kBK>
struct TileLaneOff {
  uint32_t a[Swz<D, ROWS>::kPasses], b[Swz<D, ROWS>::kPasses];
};
template <int D, int ROWS = kBK>
__device__ __forceinline__ TileLaneOff<D, ROWS> tile_lane_offsets(uint32_t step_a, uint32_t step_b, int rows_left, int lane_row, int lane_col) {
  using Z = Swz<D, ROWS>;
  TileLaneOff<D, ROWS> o;
#pragma unroll
  for (int ps = 0; ps < Z::kPasses; ++ps) {
    const int row = min(lane_row + ps * 4 * Z::kRowsPerInst, rows_left - 1);
    o.a[ps] = (uint32_t)row * step_a + lane_col;
    o.b[ps] = (uint32_t)row * step_b + lane_col;
  }
  return o;
}
// The same for 2*ROWS rows of ONE tensor, staged as the two tiles of a stage: a = rows row_first .. +ROWS-1, b = the
// ROWS rows after them, both as offsets from the tensor block's first row (row 0, of which rows_left >= 1 exist;
// later rows re-read the last one), so the rows are issued as issue_tile_pair(base, base, offsets, stage).
template <int D, int ROWS = kBK>
__device__ __forceinline__ TileLaneOff<D, ROWS> rowblock_lane_offsets(uint32_t step, int row_first, int rows_left, int lane_row, int lane_col) {
  using Z = Swz<D, ROWS>;
  TileLaneOff<D, ROWS> o;
#pragma unroll
  for (int ps = 0; ps < Z::kPasses; ++ps) {
    const int r = row_first + lane_row + ps * 4 * Z::kRowsPerInst;
    o.a[ps] = (uint32_t)min(r, rows_left - 1) * step + lane_col;
    o.b[ps] = (uint32_t)min(r + ROWS, rows_left - 1) * step + lane_col;
  }
  return o;
}
// Per-lane byte offset (within a tile) of the lane's 8 bytes of chunk 0 in the C-tile layout of load_ct_block
// (lane = row l%32, bytes 8*hh.. of the chunk): chunk c is this offset XOR (c << 4), row block rb adds 32*kRB.
template <int D>
__device__ __forceinline__ int swz_off_ct(int lane) {
  const int ln = lane & 31, hh = lane >> 5;
  return ln * Swz<D>::kRB + (Swz<D>::f(ln) << 4) + 8 * hh;
}
__device__ __forceinline__ u32x2 lds_read8(uint32_t addr) {
  return *(const __attribute__((address_space(3))) u32x2*)addr;
}
// Per-lane byte offset (within a tile) of chunk 0 of the lane's row (row l%32 of a 32-row block): the 16-byte chunk
// c of that row is at this offset XOR (c << 4); row block rb adds 32*kRB.
template <int D>
__device__ __forceinline__ int swz_off_row16(int lane) {
  const int ln = lane & 31;
  return ln * Swz<D>::kRB + (Swz<D>::f(ln) << 4);
}
// Rotary table rows staged in LDS as row blocks: a table row (D/2 floats) is as long as a bf16 tensor row (kRB bytes),
// so the 128 positions of a workgroup travel and are laid out exactly like 128 tensor rows.  cos16 / sin16: LDS
// address of chunk 0 of the lane's row in either block.  Same register contents as rope_b_load / rope_ct_load.
template <int KS>
__device__ __forceinline__ RopeB<KS> rope_b_from_lds(uint32_t cos16, uint32_t sin16, int hh) {
  RopeB<KS> r;
#pragma unroll
  for (int ks = 0; ks < KS / 2; ++ks)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint32_t off = (uint32_t)((4 * ks + 2 * hh + j) << 4);  // floats 16 ks + 8 hh + 4 j ..
      const f32x4 c = lds_read_f4(cos16 ^ off), sn = lds_read_f4(sin16 ^ off);
#pragma unroll
      for (int i = 0; i < 4; ++i) { r.c[ks][4 * j + i] = c[i]; r.s[ks][4 * j + i] = sn[i]; }
    }
  return r;
}
template <int MB>
__device__ __forceinline__ RopeCt<MB> rope_ct_from_lds(uint32_t cos16, uint32_t sin16, int hh) {
  RopeCt<MB> r;
#pragma unroll
  for (int mb = 0; mb < MB / 2; ++mb)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint32_t off = (uint32_t)((8 * mb + 2 * c + hh) << 4);  // floats 32 mb + 8 c + 4 hh ..
      const f32x4 cs = lds_read_f4(cos16 ^ off), sn = lds_read_f4(sin16 ^ off);
#pragma unroll
      for (int i = 0; i < 4; ++i) { r.c[mb][4 * c + i] = cs[i]; r.s[mb][4 * c + i] = sn[i]; }
    }
  return r;
}
//   src_a/src_b: wave-uniform pointers to row `row0` of each tensor; dst: LDS byte address of the stage + wave*1024
template <int D, int ROWS = kBK>
__device__ __forceinline__ void issue_tile_pair(const char* src_a, const char* src_b, const TileLaneOff<D, ROWS>& o, uint32_t dst) {
  using Z = Swz<D, ROWS>;
#pragma unroll
  for (int ps = 0; ps < Z::kPasses; ++ps) {
    gload_lds16_so(src_a, o.a[ps], dst + ps * 4096);
    gload_lds16_so(src_b, o.b[ps], dst + Z::kTileBytes + ps * 4096);
  }
}

// Decode a 1-D workgroup id into (tile, head, batch).  Heavy (late) tiles are issued first, and (batch, kv head)
// pairs can be pinned to one XCD each (workgroups are dealt round-robin over the 8 XCDs, so workgroup id mod 8 is the
// XCD) so that all query heads of a GQA group and all their tiles read K/V through the same L2: measured at B*Hkv = 84
// without pinning, the forward fetched 389 MB from HBM for 60 MB of operands.  `pinned` (a multiple of 8, at most
// B*Hkv) pairs are pinned; the others are spread over all XCDs (pinning a remainder would leave some XCDs a whole
// pair short) and go FIRST in the grid, heaviest tile first, padded with up to 7 idle workgroups so that the pinned part
// starts at a multiple of 8.
struct WgCoord {
  int tile, b, g, hh;
  bool valid;  // false: one of the idle padding workgroups
};
// how many pairs a launch pins: all full groups of 8, or (only_if_all) all pairs or none
__host__ __device__ inline int wg_pinned_pairs(int B, int Hkv, bool only_if_all) {
  const int pairs = B * Hkv;
  return only_if_all ? ((pairs & 7) == 0 ? pairs : 0) : (pairs & ~7);
}
__host__ __device__ inline int wg_grid(int n_tiles, int B, int Hkv, int rep, int pinned) {
  const int per_pair = n_tiles * rep;
  const int rem_wgs = (B * Hkv - pinned) * per_pair;
  return (pinned ? ((rem_wgs + 7) & ~7) : rem_wgs) + pinned * per_pair;
}
__device__ __forceinline__ WgCoord decode_wg(int bid, int n_tiles, int B, int Hkv, int rep, int pinned) {
  const int rem = B * Hkv - pinned, pp = pinned >> 3;
  const int rem_wgs = rem * n_tiles * rep;
  const int rem_pad = pinned ? ((rem_wgs + 7) & ~7) : rem_wgs;
  WgCoord c;
  c.valid = true;
  int trev, pair;
  if (bid < rem_pad) {
    if (bid >= rem_wgs) {
      c.valid = false;
      c.tile = c.b = c.g = c.hh = 0;
      return c;
    }
    const int per_tile = rem * rep;
    trev = bid / per_tile;
    const int r = bid - trev * per_tile;
    const int pl = r / rep;
    c.hh = r - pl * rep;
    pair = pinned + pl;
  } else {
    const int b2 = bid - rem_pad;  // rem_pad is a multiple of 8: b2 mod 8 is the workgroup's XCD
    const int xcd = b2 & 7, slot = b2 >> 3;
    const int per_tile = pp * rep;
    trev = slot / per_tile;
    const int r = slot - trev * per_tile;
    const int pl = r / rep;
    c.hh = r - pl * rep;
    pair = pl * 8 + xcd;
  }
  c.b = pair / Hkv;
  c.g = pair - c.b * Hkv;
  c.tile = n_tiles - 1 - trev;
  return c;
}

}  // namespace segpt
