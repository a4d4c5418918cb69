// Shared device/host definitions for libsegpt_attn.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "segpt_attn.h"

namespace segpt {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Everything a kernel needs: the caller's params by value plus the carved-up workspace.
struct KArgs {
  segpt_attn_params p;
  float* delta;       // [B,H,Sq] fp32: rowsum(dO_eff * o)  (fp32 path) / its NEGATIVE (bf16 path: MFMA C operand)
  float* nlse2;       // [B,H,Sq] fp32: -lse*log2(e)                 (bf16 path only: MFMA C operand)
  void* do_eff;       // [B,H,Sq,D] dtype, contiguous: gate-scaled dO (fp32 path; bf16 path only for a gate scale <= 0), else null
  uint16_t* qhat;     // [B,H,Sq,D]   bf16: sm_scale*log2e * a_i q_i * g_q*g_k   (bf16 path only)
  uint16_t* khat;     // [B,Hkv,Sk,D] bf16: b_j k_j                               (bf16 path only; kv_workspace)
  uint16_t* vmix;     // [B,Hkv,Sk,D] bf16: c1 v + c2 v_first (only with a value residual, else NULL; kv_workspace)
  float* dg_part;     // [n_dq_blocks, D] fp32 partial sums of the combined scale gradient
  float* dcoef_part;  // [n_dkdv_blocks, 2] fp32 partial sums of (dc1, dc2)
  int32_t n_dq_blocks;
  int32_t n_dkdv_blocks;
  // decode path (split keys): partial O [B*Hkv, splits, 32, D] and (max, sum) [B*Hkv, splits, 32, 2], both fp32,
  // carved from kv_workspace
  float* dec_part;
  float* dec_stat;
  int32_t dec_splits, dec_chunk, dec_kend;
};

// Row normaliser 1/sqrt(mean x^2 + eps) from the row's sum of squares ss (inv_d = 1/D); exactly 1 for plain
// attention (SEGPT_FLAG_NO_NORM).
__device__ __forceinline__ float row_normaliser(const segpt_attn_params& p, float ss, float inv_d) {
  return (p.flags & SEGPT_FLAG_NO_NORM) ? 1.0f : 1.0f / sqrtf(ss * inv_d + p.eps);
}
__device__ __forceinline__ float row_normaliser_fast(const segpt_attn_params& p, float ss, float inv_d) {
  return (p.flags & SEGPT_FLAG_NO_NORM) ? 1.0f : __builtin_amdgcn_rsqf(ss * inv_d + p.eps);
}
// n^3/D, the factor of the normaliser's own term in dx = n u - (n^3/D)(u.x) x; 0 when there is no normaliser
__device__ __forceinline__ float norm_grad_coef(const segpt_attn_params& p, float n, float inv_d) {
  return (p.flags & SEGPT_FLAG_NO_NORM) ? 0.0f : n * n * n * inv_d;
}

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

// round-to-nearest-even fp32 -> bf16 (inputs are finite in every use below)
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  f2 v = {lo, hi};
  bf2 r = __builtin_convertvector(v, bf2);  // v_cvt_pk_bf16_f32 on gfx950 (RNE)
  return __builtin_bit_cast(uint32_t, r);
}

__device__ __forceinline__ float bf16lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

template <typename T>
struct Elem;
template <>
struct Elem<float> {
  static constexpr int kVec = 4;  // elements per 16-byte access
  static __device__ __forceinline__ void load(const float* p, float (&out)[4]) {
    float4 v = *reinterpret_cast<const float4*>(p);
    out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&in)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(in[0], in[1], in[2], in[3]);
  }
  static __device__ __forceinline__ float load1(const float* p) { return *p; }
  static __device__ __forceinline__ void store1(float* p, float v) { *p = v; }
};
template <>
struct Elem<uint16_t> {  // bf16 bits
  static constexpr int kVec = 8;
  static __device__ __forceinline__ void load(const uint16_t* p, float (&out)[8]) {
    uint4 v = *reinterpret_cast<const uint4*>(p);
    out[0] = bf16lo(v.x); out[1] = bf16hi(v.x); out[2] = bf16lo(v.y); out[3] = bf16hi(v.y);
    out[4] = bf16lo(v.z); out[5] = bf16hi(v.z); out[6] = bf16lo(v.w); out[7] = bf16hi(v.w);
  }
  static __device__ __forceinline__ void store(uint16_t* p, const float (&in)[8]) {
    uint4 v;
    v.x = pack_bf16x2(in[0], in[1]); v.y = pack_bf16x2(in[2], in[3]);
    v.z = pack_bf16x2(in[4], in[5]); v.w = pack_bf16x2(in[6], in[7]);
    *reinterpret_cast<uint4*>(p) = v;
  }
  static __device__ __forceinline__ float load1(const uint16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void store1(uint16_t* p, float v) { *p = f32_to_bf16(v); }
};

template <typename T>
__device__ __forceinline__ const T* row_ptr(const segpt_tensor4& t, int b, int h, int s) {
  return reinterpret_cast<const T*>(t.ptr) + (int64_t)b * t.stride_b + (int64_t)h * t.stride_h + (int64_t)s * t.stride_s;
}
template <typename T>
__device__ __forceinline__ T* row_ptr_mut(const segpt_tensor4& t, int b, int h, int s) {
  return reinterpret_cast<T*>(t.ptr) + (int64_t)b * t.stride_b + (int64_t)h * t.stride_h + (int64_t)s * t.stride_s;
}

// Rotary embedding of one split-half pair (x1 = element j, x2 = element j + D/2), rope.py:50-55, and its
// transpose (the gradient with respect to the unrotated pair).
__device__ __forceinline__ void rope_pair(float& x1, float& x2, float c, float s) {
  const float a = x1, b = x2;
  x1 = a * c - b * s;
  x2 = a * s + b * c;
}
__device__ __forceinline__ void rope_pair_inv(float& x1, float& x2, float c, float s) {
  const float a = x1, b = x2;
  x1 = a * c + b * s;
  x2 = b * c - a * s;
}

__device__ __forceinline__ float sigmoidf_acc(float z) { return 1.0f / (1.0f + expf(-z)); }

// Final reduction of the scale-vector gradient by ONE workgroup of THREADS threads:
//   tot[d] = sum over the n_dq_blocks partial rows of dg_part[., d]   (fixed order: deterministic)
//   dg_q = g_k * tot, dg_k = g_q * tot  (summed over d for a scalar parameter)
// `red` (THREADS floats) and `tot` (D floats) are workgroup-shared scratch.
template <int THREADS>
__device__ __forceinline__ void reduce_scale_grad(const KArgs& a, int tid, float* red, float* tot) {
  const segpt_attn_params& p = a.p;
  const int D = p.D;
  const int lanes = THREADS / D;  // threads cooperating on one d
  const int d = tid % D, sl = tid / D;
  // eight independent chains hide the load latency
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const float* src = a.dg_part + d;
  const int n = a.n_dq_blocks;
  int blk = sl;
  for (; blk + 7 * lanes < n; blk += 8 * lanes) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = src[(int64_t)(blk + u * lanes) * D];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc[u] += v[u];
  }
  for (; blk < n; blk += lanes) acc[0] += src[(int64_t)blk * D];
  red[tid] = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
  __syncthreads();
  if (tid < D) {
    float t = 0.f;
    for (int x = 0; x < lanes; ++x) t += red[x * D + tid];
    tot[tid] = t;
  }
  __syncthreads();
  if (tid < D) {
    if (p.gq_numel == D) {
      const float gk = p.gk_numel == 0 ? 1.f : (p.gk_numel == 1 ? p.g_k[0] : p.g_k[tid]);
      p.dg_q[tid] = gk * tot[tid];
    }
    if (p.gk_numel == D) {
      const float gq = p.gq_numel == 1 ? p.g_q[0] : p.g_q[tid];
      p.dg_k[tid] = gq * tot[tid];
    }
  }
  if (tid == 0) {
    if (p.gq_numel == 1) {
      float t = 0.f;
      for (int x = 0; x < D; ++x) {
        const float gk = p.gk_numel == 0 ? 1.f : (p.gk_numel == 1 ? p.g_k[0] : p.g_k[x]);
        t += gk * tot[x];
      }
      p.dg_q[0] = t;
    }
    if (p.gk_numel == 1) {
      float t = 0.f;
      for (int x = 0; x < D; ++x) {
        const float gq = p.gq_numel == 1 ? p.g_q[0] : p.g_q[x];
        t += gq * tot[x];
      }
      p.dg_k[0] = t;
    }
  }
}

// host-side launchers (one per translation unit); each returns a hipError_t as int
int launch_fwd_f32(const KArgs& a, hipStream_t st);
int launch_bwd_dkdv_f32(const KArgs& a, hipStream_t st);
int launch_bwd_dq_f32(const KArgs& a, hipStream_t st);
int launch_fwd_bf16(const KArgs& a, hipStream_t st);
int launch_bwd_dkdv_bf16(const KArgs& a, hipStream_t st);
int launch_bwd_dq_bf16(const KArgs& a, hipStream_t st);
int launch_bwd_pre(const KArgs& a, hipStream_t st);     // fp32 path: delta, dgate, do_eff
int launch_fwd_decode_bf16(KArgs a, hipStream_t st);    // split-key forward for a few query rows against a long cache
size_t decode_plan(const segpt_attn_params& p, int* kend, int* splits, int* chunk);  // returns its scratch bytes
int launch_kv_prep(const KArgs& a, hipStream_t st);     // bf16 path: Khat (and V') into kv_workspace
int launch_bwd_reduce(const KArgs& a, hipStream_t st);  // fp32: dg_q, dg_k, dvr_coef from the partials; bf16: dvr_coef only

// block counts shared by the workspace carve-up and the launchers
int dq_blocks(const segpt_attn_params& p);
int dkdv_blocks(const segpt_attn_params& p);

}  // namespace segpt
