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

template <int D>
struct Tile {
  static constexpr int kRS = D + 8;                 // LDS row stride in bf16 elements (16 B pad)
  static constexpr int kElems = kBK * kRS;          // elements of one staged tile
  static constexpr int kTPR = D / 8;                // threads per row when staging (16 B each)
  static constexpr int kRowsPerPass = kThreadsM / kTPR;
  static constexpr int kPasses = kBK / kRowsPerPass;  // 16-byte loads per thread per tile
};

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
__device__ __forceinline__ float fast_rsq(float x) { return __builtin_amdgcn_rsqf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// Wait for every outstanding vector-memory load of this wave and keep the compiler from moving memory
// operations across this point.  Used once before a pipelined loop: loads that stay in flight ACROSS loop
// iterations must be the youngest ones, or every in-loop wait for an older load drains them as well.
__device__ __forceinline__ void drain_vector_loads() {
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), expcnt/lgkmcnt untouched
  __builtin_amdgcn_sched_barrier(0);
}

// x + (x of another lane) through a DPP lane pattern (no LDS traffic, fuses into v_add_f32_dpp)
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  return x + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}

// sum over the kTPR (8 or 16) adjacent lanes that stage one row; every lane of the group gets the total
template <int TPR>
__device__ __forceinline__ float row_group_sum(float x) {
  static_assert(TPR == 8 || TPR == 16, "row groups are 8 or 16 lanes");
  x = dpp_add<0xB1>(x);   // quad_perm [1,0,3,2]
  x = dpp_add<0x4E>(x);   // quad_perm [2,3,0,1]
  x = dpp_add<0x141>(x);  // row_half_mirror: the other quad of the 8-lane half row
  if (TPR == 16) x = dpp_add<0x140>(x);  // row_mirror: the other half of the 16-lane row
  return x;
}

// acc + lo + hi of one packed bf16 pair (v_dot2c_f32_bf16 with a (1,1) operand): sums the ROUNDED values,
// i.e. exactly what the MFMA consuming the packed operand sees.
__device__ __forceinline__ float add_bf16_pair(uint32_t w, float acc) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  const bf2 one = {(__bf16)1.0f, (__bf16)1.0f};
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf2, w), one, acc, false);
}

__device__ __forceinline__ float sumsq8(u32x4 v) {
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float lo = bf16lo(v[i]), hi = bf16hi(v[i]);
    s += lo * lo + hi * hi;
  }
  return s;
}
__device__ __forceinline__ u32x4 scale8(u32x4 v, float f) {
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = pack_bf16x2(bf16lo(v[i]) * f, bf16hi(v[i]) * f);
  return r;
}
__device__ __forceinline__ u32x4 mix8(u32x4 a, u32x4 b, float ca, float cb) {
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    r[i] = pack_bf16x2(ca * bf16lo(a[i]) + cb * bf16lo(b[i]), ca * bf16hi(a[i]) + cb * bf16hi(b[i]));
  return r;
}

// A/B fragment of a row-major LDS tile for the 32-row block `rb`, contraction step `ks` (16 columns):
// lane reads 16 contiguous bytes at row 32*rb + l%32, column 16*ks + 8*(l/32).
template <int D>
__device__ __forceinline__ bf16x8 frag_rowmajor(const uint16_t* tile, int rb, int ks, int lane) {
  const uint16_t* p = tile + (32 * rb + (lane & 31)) * Tile<D>::kRS + 16 * ks + 8 * (lane >> 5);
  return as_bf16x8(*reinterpret_cast<const u32x4*>(p));
}

// Transposed fragment of a row-major LDS tile [row][col]: the lane's MFMA row is a COLUMN of the tile
// (col = 32*cb + l%32) and its 8 contraction entries are tile rows in CPERM order
//   16*s + {4hh..4hh+3, 8+4hh..8+4hh+3}.
// ds_read_b64_tr_b16 semantics (per 16-lane group, source lane r gives the address of 4 elements):
//   result[lane i][e] = LDS[addr(4e + i/4) + i%4]
// so source lane r points at row base + r/4, column cbase + 4*(r%4) and lane i receives column cbase + i,
// rows base..base+3.
template <int D>
__device__ __forceinline__ bf16x8 frag_transposed(const uint16_t* tile, int cb, int s, int lane) {
  const int r = lane & 15;
  const int hh = lane >> 5;
  const int col = 32 * cb + 16 * ((lane >> 4) & 1) + 4 * (r & 3);
  const int row = 16 * s + 4 * hh + (r >> 2);
  const uint16_t* p = tile + row * Tile<D>::kRS + col;
  typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 8 * Tile<D>::kRS));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, v);
}

// ---- the same two fragment readers with every term but one per-lane base folded into the instruction's
// immediate offset: `base` = LDS byte address of the tile + lane_off_rm / lane_off_tr, block indices constant.
template <int D>
__device__ __forceinline__ int lane_off_rm(int lane) {
  return ((lane & 31) * Tile<D>::kRS + 8 * (lane >> 5)) * 2;
}
template <int D>
__device__ __forceinline__ int lane_off_tr(int lane) {
  const int r = lane & 15;
  return ((4 * (lane >> 5) + (r >> 2)) * Tile<D>::kRS + 16 * ((lane >> 4) & 1) + 4 * (r & 3)) * 2;
}
template <int D>
__device__ __forceinline__ bf16x8 frag_rm_at(const char* base, int rb, int ks) {
  return as_bf16x8(*reinterpret_cast<const u32x4*>(base + (32 * rb * Tile<D>::kRS + 16 * ks) * 2));
}
template <int D>
__device__ __forceinline__ bf16x8 frag_tr_at(const char* base, int cb, int s) {
  const char* p = base + (16 * s * Tile<D>::kRS + 32 * cb) * 2;
  typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 8 * Tile<D>::kRS * 2));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, v);
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
template <int D>
struct Swz {
  static constexpr int kRB = 2 * D;                     // bytes per row
  static constexpr int kTileBytes = kBK * kRB;          // 8 KB (D=64) / 16 KB (D=128)
  static constexpr int kChunks = kRB / 16;              // chunks per row
  static constexpr int kRowsPerInst = 1024 / kRB;       // rows one wave-wide load covers
  static constexpr int kPasses = kTileBytes / 1024 / 4; // wave-wide loads per wave per tile (4 waves)
  static constexpr int kHiXor = (D == 64 ? 4 : 2) << 4; // byte XOR between the swizzle terms of rows r and r+8
  static __device__ __forceinline__ int f(int row) {
    return D == 64 ? ((row >> 1) & 7) : (((row & 3) << 2) | ((row >> 2) & 3));
  }
  static_assert(D == 64 || D == 128, "swizzle is defined for 128- and 256-byte rows");
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
__device__ __forceinline__ void gload_lds16(const void* gsrc, uint32_t lds_dst_wave_uniform) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(gsrc), "s"(lds_dst_wave_uniform)
               : "memory", "m0");
}
__device__ __forceinline__ void gload_lds4(const void* gsrc, uint32_t lds_dst_wave_uniform) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dword %0, off"
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
__device__ __forceinline__ bf16x8 pack_c_half_sum(const f32x16& c, int s, float& sum) {
  const uint32_t w0 = pack_bf16x2(c[8 * s + 0], c[8 * s + 1]);
  const uint32_t w1 = pack_bf16x2(c[8 * s + 2], c[8 * s + 3]);
  const uint32_t w2 = pack_bf16x2(c[8 * s + 4], c[8 * s + 5]);
  const uint32_t w3 = pack_bf16x2(c[8 * s + 6], c[8 * s + 7]);
  sum = add_bf16_pair(w3, add_bf16_pair(w2, add_bf16_pair(w1, add_bf16_pair(w0, sum))));
  const u32x4 w = {w0, w1, w2, w3};
  return as_bf16x8(w);
}

// ---- K/V tile staging: global -> registers (16 B per thread per pass) -> normalise / mix -> LDS (row-major)
template <int D>
struct StageRegs {
  u32x4 k[Tile<D>::kPasses], v[Tile<D>::kPasses], vf[Tile<D>::kPasses];
};

template <int D, bool VR>
__device__ __forceinline__ void stage_load(const segpt_attn_params& p, int b, int g, int j0, StageRegs<D>& r) {
  using T = Tile<D>;
  const int tid = threadIdx.x;
  const int chunk = tid % T::kTPR, r0 = tid / T::kTPR;
#pragma unroll
  for (int ps = 0; ps < T::kPasses; ++ps) {
    const int j = j0 + r0 + ps * T::kRowsPerPass;
    if (j < p.Sk) {
      r.k[ps] = *reinterpret_cast<const u32x4*>(row_ptr<uint16_t>(p.k, b, g, j) + chunk * 8);
      r.v[ps] = *reinterpret_cast<const u32x4*>(row_ptr<uint16_t>(p.v, b, g, j) + chunk * 8);
      if (VR) r.vf[ps] = *reinterpret_cast<const u32x4*>(row_ptr<uint16_t>(p.v_first, b, g, j) + chunk * 8);
    } else {
      r.k[ps] = u32x4{0, 0, 0, 0};
      r.v[ps] = u32x4{0, 0, 0, 0};
      if (VR) r.vf[ps] = u32x4{0, 0, 0, 0};
    }
  }
}

template <int D, bool VR>
__device__ __forceinline__ void stage_store(const StageRegs<D>& r, uint16_t* kt, uint16_t* vt, float eps, float c1, float c2) {
  using T = Tile<D>;
  const int tid = threadIdx.x;
  const int chunk = tid % T::kTPR, r0 = tid / T::kTPR;
#pragma unroll
  for (int ps = 0; ps < T::kPasses; ++ps) {
    const int row = r0 + ps * T::kRowsPerPass;
    const float ss = row_group_sum<T::kTPR>(sumsq8(r.k[ps]));
    const float beta = fast_rsq(ss * (1.0f / D) + eps);
    *reinterpret_cast<u32x4*>(kt + row * T::kRS + chunk * 8) = scale8(r.k[ps], beta);
    *reinterpret_cast<u32x4*>(vt + row * T::kRS + chunk * 8) = VR ? mix8(r.v[ps], r.vf[ps], c1, c2) : r.v[ps];
  }
}

// Decode a 1-D workgroup id into (tile, head, batch).  Heavy (late) tiles are issued first and,
// when the number of (batch, kv head) pairs is a multiple of 8, every pair is pinned to one XCD
// (workgroups are dealt round-robin over the 8 XCDs) so that all query heads of a GQA group and all
// their tiles read K/V through the same L2.
struct WgCoord {
  int tile, b, g, hh;
};
__device__ __forceinline__ WgCoord decode_wg(int bid, int n_tiles, int B, int Hkv, int rep) {
  const int pairs = B * Hkv;
  int xcd = 0, slot = bid, pp = pairs;
  if ((pairs & 7) == 0) {
    xcd = bid & 7;
    slot = bid >> 3;
    pp = pairs >> 3;
  }
  const int per_tile = pp * rep;
  const int trev = slot / per_tile;
  const int rem = slot - trev * per_tile;
  const int pl = rem / rep;
  WgCoord c;
  c.hh = rem - pl * rep;
  const int pair = ((pairs & 7) == 0) ? pl * 8 + xcd : pl;
  c.b = pair / Hkv;
  c.g = pair - c.b * Hkv;
  c.tile = n_tiles - 1 - trev;
  return c;
}

}  // namespace segpt
