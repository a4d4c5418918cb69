// fp32 path: plain-FMA flash attention with fused QK-norm, forward and backward.
// It exists for the 1e-5 parity case (fp32 tensors, as in the reference's self-check
// triton_flash_attn_qknorm.py:346-352); the bf16 MFMA kernels are the performance path.
//
// Layout of a workgroup: 256 threads = 64 rows x 4 lanes; lane `sub` of a row owns the
// contiguous slice [sub*D/4, (sub+1)*D/4) of the head dimension.  Tiles of the other
// operand (32 rows) are normalised / mixed while being staged into LDS.
#include "common.hpp"

namespace segpt {
namespace {

constexpr int kRows = 64;   // rows owned by a workgroup
constexpr int kTile = 32;   // rows of the streamed operand per LDS tile
constexpr int kThreads = 256;

__device__ __forceinline__ float quad_sum(float x) {
  x += __shfl_xor(x, 1, 64);
  x += __shfl_xor(x, 2, 64);
  return x;
}
__device__ __forceinline__ float oct_sum(float x) {
  x += __shfl_xor(x, 1, 64);
  x += __shfl_xor(x, 2, 64);
  x += __shfl_xor(x, 4, 64);
  return x;
}

// Split-half rotary embedding (rope.py:50-55) of a row spread over TPR consecutive lanes, N = D/TPR contiguous
// elements per lane starting at d0 = (lane % TPR) * N: the partner element d +- D/2 sits TPR/2 lanes away at
// the same index.  `pos` is the row's table row.  Every lane of the wave must get here (the lanes shuffle).
// INVERSE applies the transpose, i.e. takes a gradient in the rotated frame back to the unrotated row.
template <int D, int N, int TPR, bool INVERSE>
__device__ __forceinline__ void rope_lanes(const segpt_attn_params& p, float (&x)[N], int pos, int d0) {
  static_assert(N * TPR == D, "row split");
  const bool hi = d0 >= D / 2;
  const float* cosr = p.rope_cos + (int64_t)pos * (D / 2) + (hi ? d0 - D / 2 : d0);
  const float* sinr = p.rope_sin + (int64_t)pos * (D / 2) + (hi ? d0 - D / 2 : d0);
#pragma unroll
  for (int e = 0; e < N; ++e) {
    const float o = __shfl_xor(x[e], TPR / 2, 64);
    const float c = cosr[e];
    const float sn = INVERSE ? -sinr[e] : sinr[e];
    x[e] = hi ? o * sn + x[e] * c : x[e] * c - o * sn;
  }
}

template <int D>
__device__ __forceinline__ float gprod(const segpt_attn_params& p, int d) {
  float gq = p.gq_numel == 1 ? p.g_q[0] : p.g_q[d];
  float gk = p.gk_numel == 0 ? 1.0f : (p.gk_numel == 1 ? p.g_k[0] : p.g_k[d]);
  return gq * gk;
}

// Stage `kTile` kv rows starting at j0 into LDS: khat = k * rsqrt(mean k^2 + eps), vmix = c1 v + c2 v_first.
// 8 threads per row.
template <int D>
__device__ __forceinline__ void stage_kv(const segpt_attn_params& p, int b, int g, int j0, float c1, float c2,
                                         float* kh, float* vm) {
  constexpr int PT = D / 8;  // elements per thread
  const int tid = threadIdx.x;
  const int r = tid >> 3, part = tid & 7;
  const int j = j0 + r;
  float kreg[PT], vreg[PT];
  if (j < p.Sk) {
    const float* kp = row_ptr<float>(p.k, b, g, j) + part * PT;
    const float* vp = row_ptr<float>(p.v, b, g, j) + part * PT;
#pragma unroll
    for (int e = 0; e < PT; e += 4) {
      float t[4];
      Elem<float>::load(kp + e, t);
      kreg[e] = t[0]; kreg[e + 1] = t[1]; kreg[e + 2] = t[2]; kreg[e + 3] = t[3];
      Elem<float>::load(vp + e, t);
      vreg[e] = t[0]; vreg[e + 1] = t[1]; vreg[e + 2] = t[2]; vreg[e + 3] = t[3];
    }
    if (p.v_first.ptr) {
      const float* fp = row_ptr<float>(p.v_first, b, g, j) + part * PT;
#pragma unroll
      for (int e = 0; e < PT; e += 4) {
        float t[4];
        Elem<float>::load(fp + e, t);
#pragma unroll
        for (int x = 0; x < 4; ++x) vreg[e + x] = c1 * vreg[e + x] + c2 * t[x];
      }
    }
  } else {
#pragma unroll
    for (int e = 0; e < PT; ++e) { kreg[e] = 0.f; vreg[e] = 0.f; }
  }
  if (p.rope_cos) rope_lanes<D, PT, 8, false>(p, kreg, p.rope_k_pos0 + min(j, p.Sk - 1), part * PT);
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < PT; ++e) ss += kreg[e] * kreg[e];
  ss = oct_sum(ss);
  const float beta = row_normaliser(p, ss, 1.0f / D);
#pragma unroll
  for (int e = 0; e < PT; ++e) {
    kh[r * D + part * PT + e] = kreg[e] * beta;
    vm[r * D + part * PT + e] = vreg[e];
  }
}

template <int D>
__global__ __launch_bounds__(kThreads) void fwd_f32_kernel(KArgs a) {
  const segpt_attn_params& p = a.p;
  constexpr int DP = D / 4;
  __shared__ float kh[kTile * D];
  __shared__ float vm[kTile * D];
  const int tid = threadIdx.x, sub = tid & 3, lr = tid >> 2;
  const int q0 = blockIdx.x * kRows, h = blockIdx.y, b = blockIdx.z;
  const int g = h / (p.H / p.Hkv);
  const int row = q0 + lr;
  const bool live = row < p.Sq;
  const int rowc = live ? row : p.Sq - 1;
  float c1 = 1.f, c2 = 0.f;
  if (p.vr_coef) { c1 = p.vr_coef[0]; c2 = p.vr_coef[1]; }

  float qh[DP], acc[DP];
  {
    const float* qp = row_ptr<float>(p.q, b, h, rowc) + sub * DP;
#pragma unroll
    for (int e = 0; e < DP; e += 4) {
      float t[4];
      Elem<float>::load(qp + e, t);
#pragma unroll
      for (int x = 0; x < 4; ++x) qh[e + x] = t[x];
    }
    if (p.rope_cos) rope_lanes<D, DP, 4, false>(p, qh, p.rope_q_pos0 + rowc, sub * DP);
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < DP; ++e) ss += qh[e] * qh[e];
    ss = quad_sum(ss);
    const float alpha = row_normaliser(p, ss, 1.0f / D);
#pragma unroll
    for (int e = 0; e < DP; ++e) {
      qh[e] = qh[e] * alpha * gprod<D>(p, sub * DP + e) * p.sm_scale;
      acc[e] = 0.f;
    }
  }
  float m = -INFINITY, l = 0.f;
  int kend = p.Sk;
  if (p.causal) kend = min(p.Sk, q0 + kRows + p.q_start);
  for (int j0 = 0; j0 < kend; j0 += kTile) {
    __syncthreads();
    stage_kv<D>(p, b, g, j0, c1, c2, kh, vm);
    __syncthreads();
#pragma unroll 1
    for (int c = 0; c < kTile; c += 8) {
      float s[8];
      float mx = m;
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const float* kr = kh + (c + x) * D + sub * DP;
        float d = 0.f;
#pragma unroll
        for (int e = 0; e < DP; ++e) d += qh[e] * kr[e];
        d = quad_sum(d);
        const int j = j0 + c + x;
        const bool vis = j < p.Sk && (!p.causal || j <= row + p.q_start);
        s[x] = vis ? d : -INFINITY;
        mx = fmaxf(mx, s[x]);
      }
      const float mu = (mx == -INFINITY) ? 0.f : mx;
      const float sc = expf(m - mu);
      l *= sc;
#pragma unroll
      for (int e = 0; e < DP; ++e) acc[e] *= sc;
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const float pj = expf(s[x] - mu);
        l += pj;
        const float* vr = vm + (c + x) * D + sub * DP;
#pragma unroll
        for (int e = 0; e < DP; ++e) acc[e] += pj * vr[e];
      }
      m = mx;
    }
  }
  if (live) {
    float gate = 1.f;
    if (p.gate.ptr) {
      const float z = reinterpret_cast<const float*>(p.gate.ptr)[(int64_t)b * p.gate.stride_b + (int64_t)row * p.gate.stride_s + (int64_t)h * p.gate.stride_h];
      gate = p.gate_scale * sigmoidf_acc(z);
    }
    const float inv = gate / l;
    float* op = row_ptr_mut<float>(p.o, b, h, row) + sub * DP;
#pragma unroll
    for (int e = 0; e < DP; e += 4) {
      float t[4] = {acc[e] * inv, acc[e + 1] * inv, acc[e + 2] * inv, acc[e + 3] * inv};
      Elem<float>::store(op + e, t);
    }
    if (sub == 0) p.lse[((int64_t)b * p.H + h) * p.Sq + row] = m + logf(l);
  }
}

// dQ: one workgroup per 64 query rows; streams kv tiles.  Also emits this block's partial of the
// combined scale gradient  dg[d] = sum_i sm_scale * (a_i q_id) * T_id,  T = dS Khat.
template <int D>
__global__ __launch_bounds__(kThreads) void bwd_dq_f32_kernel(KArgs a) {
  const segpt_attn_params& p = a.p;
  constexpr int DP = D / 4;
  __shared__ float kh[kTile * D];
  __shared__ float vm[kTile * D];
  __shared__ float red[4 * D];
  const int tid = threadIdx.x, sub = tid & 3, lr = tid >> 2;
  const int q0 = blockIdx.x * kRows, h = blockIdx.y, b = blockIdx.z;
  const int g = h / (p.H / p.Hkv);
  const int row = q0 + lr;
  const bool live = row < p.Sq;
  const int rowc = live ? row : p.Sq - 1;
  float c1 = 1.f, c2 = 0.f;
  if (p.vr_coef) { c1 = p.vr_coef[0]; c2 = p.vr_coef[1]; }

  float qraw[DP], qh[DP], dout[DP], T[DP];
  float alpha;
  {
    const float* qp = row_ptr<float>(p.q, b, h, rowc) + sub * DP;
    const float* dp = a.do_eff ? reinterpret_cast<const float*>(a.do_eff) + (((int64_t)b * p.H + h) * p.Sq + rowc) * D + sub * DP
                               : row_ptr<float>(p.d_o, b, h, rowc) + sub * DP;
#pragma unroll
    for (int e = 0; e < DP; e += 4) {
      float t[4];
      Elem<float>::load(qp + e, t);
#pragma unroll
      for (int x = 0; x < 4; ++x) qraw[e + x] = t[x];
      Elem<float>::load(dp + e, t);
#pragma unroll
      for (int x = 0; x < 4; ++x) dout[e + x] = t[x];
    }
    // with a rotary embedding qraw is the ROTATED row from here on: the normaliser and the scale act on it
    if (p.rope_cos) rope_lanes<D, DP, 4, false>(p, qraw, p.rope_q_pos0 + rowc, sub * DP);
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < DP; ++e) ss += qraw[e] * qraw[e];
    ss = quad_sum(ss);
    alpha = row_normaliser(p, ss, 1.0f / D);
#pragma unroll
    for (int e = 0; e < DP; ++e) {
      qh[e] = qraw[e] * alpha * gprod<D>(p, sub * DP + e) * p.sm_scale;
      T[e] = 0.f;
    }
  }
  const int64_t ridx = ((int64_t)b * p.H + h) * p.Sq + rowc;
  const float lse = p.lse[ridx];
  const float delta = a.delta[ridx];
  int kend = p.Sk;
  if (p.causal) kend = min(p.Sk, q0 + kRows + p.q_start);
  for (int j0 = 0; j0 < kend; j0 += kTile) {
    __syncthreads();
    stage_kv<D>(p, b, g, j0, c1, c2, kh, vm);
    __syncthreads();
#pragma unroll 2
    for (int x = 0; x < kTile; ++x) {
      const float* kr = kh + x * D + sub * DP;
      const float* vr = vm + x * D + sub * DP;
      float s = 0.f, dpv = 0.f;
#pragma unroll
      for (int e = 0; e < DP; ++e) { s += qh[e] * kr[e]; dpv += dout[e] * vr[e]; }
      s = quad_sum(s);
      dpv = quad_sum(dpv);
      const int j = j0 + x;
      const bool vis = j < p.Sk && (!p.causal || j <= row + p.q_start);
      const float pj = vis ? expf(s - lse) : 0.f;
      const float ds = pj * (dpv - delta);
#pragma unroll
      for (int e = 0; e < DP; ++e) T[e] += ds * kr[e];
    }
  }
  // through the q normaliser; u = dL/d(a q) = sm_scale * g * T
  float dot = 0.f;
  float u[DP], dgl[DP];
#pragma unroll
  for (int e = 0; e < DP; ++e) {
    u[e] = p.sm_scale * gprod<D>(p, sub * DP + e) * T[e];
    dot += u[e] * qraw[e];
    dgl[e] = live ? p.sm_scale * alpha * qraw[e] * T[e] : 0.f;
  }
  dot = quad_sum(dot);
  {
    const float a3 = norm_grad_coef(p, alpha, 1.0f / D) * dot;
#pragma unroll
    for (int e = 0; e < DP; ++e) u[e] = alpha * u[e] - a3 * qraw[e];  // gradient of the (rotated) row
    if (p.rope_cos) rope_lanes<D, DP, 4, true>(p, u, p.rope_q_pos0 + rowc, sub * DP);
    if (live) {
      float* op = row_ptr_mut<float>(p.dq, b, h, row) + sub * DP;
#pragma unroll
      for (int e = 0; e < DP; e += 4) {
        float t[4] = {u[e], u[e + 1], u[e + 2], u[e + 3]};
        Elem<float>::store(op + e, t);
      }
    }
  }
  // block partial of dg: sum over the 16 rows of a wave (lanes with equal sub), then over 4 waves
#pragma unroll
  for (int e = 0; e < DP; ++e) {
    float x = dgl[e];
    x += __shfl_xor(x, 4, 64);
    x += __shfl_xor(x, 8, 64);
    x += __shfl_xor(x, 16, 64);
    x += __shfl_xor(x, 32, 64);
    dgl[e] = x;
  }
  const int wave = tid >> 6, lane = tid & 63;
  if (lane < 4) {
#pragma unroll
    for (int e = 0; e < DP; ++e) red[wave * D + lane * DP + e] = dgl[e];
  }
  __syncthreads();
  const int blk = (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
  for (int d = tid; d < D; d += kThreads) a.dg_part[(int64_t)blk * D + d] = red[d] + red[D + d] + red[2 * D + d] + red[3 * D + d];
}

// dK, dV: one workgroup per 64 key rows of one kv head; streams the query tiles of every query head
// of the group.  The staged query tile is already normalised and scaled (qhat).
template <int D>
__global__ __launch_bounds__(kThreads) void bwd_dkdv_f32_kernel(KArgs a) {
  const segpt_attn_params& p = a.p;
  constexpr int DP = D / 4;
  constexpr int PT = D / 8;
  __shared__ float qs[kTile * D];
  __shared__ float dos[kTile * D];
  __shared__ float ls[kTile], des[kTile];
  __shared__ float red[8];
  const int tid = threadIdx.x, sub = tid & 3, lr = tid >> 2;
  const int j0 = blockIdx.x * kRows, g = blockIdx.y, b = blockIdx.z;
  const int rep = p.H / p.Hkv;
  const int j = j0 + lr;
  const bool live = j < p.Sk;
  const int jc = live ? j : p.Sk - 1;
  float c1 = 1.f, c2 = 0.f;
  if (p.vr_coef) { c1 = p.vr_coef[0]; c2 = p.vr_coef[1]; }

  float kh[DP], vmix[DP], W[DP], dV[DP];
  float beta;
  {
    const float* kp = row_ptr<float>(p.k, b, g, jc) + sub * DP;
    const float* vp = row_ptr<float>(p.v, b, g, jc) + sub * DP;
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < DP; e += 4) {
      float t[4];
      Elem<float>::load(kp + e, t);
#pragma unroll
      for (int x = 0; x < 4; ++x) kh[e + x] = t[x];
      Elem<float>::load(vp + e, t);
#pragma unroll
      for (int x = 0; x < 4; ++x) vmix[e + x] = t[x];
    }
    if (p.v_first.ptr) {
      const float* fp = row_ptr<float>(p.v_first, b, g, jc) + sub * DP;
#pragma unroll
      for (int e = 0; e < DP; e += 4) {
        float t[4];
        Elem<float>::load(fp + e, t);
#pragma unroll
        for (int x = 0; x < 4; ++x) vmix[e + x] = c1 * vmix[e + x] + c2 * t[x];
      }
    }
    if (p.rope_cos) rope_lanes<D, DP, 4, false>(p, kh, p.rope_k_pos0 + jc, sub * DP);
#pragma unroll
    for (int e = 0; e < DP; ++e) ss += kh[e] * kh[e];
    ss = quad_sum(ss);
    beta = row_normaliser(p, ss, 1.0f / D);
#pragma unroll
    for (int e = 0; e < DP; ++e) {
      kh[e] *= beta;
      W[e] = 0.f;
      dV[e] = 0.f;
    }
  }
  int istart = 0;
  if (p.causal) istart = max(0, j0 - p.q_start) / kTile * kTile;
  for (int hh = 0; hh < rep; ++hh) {
    const int h = g * rep + hh;
    for (int i0 = istart; i0 < p.Sq; i0 += kTile) {
      __syncthreads();
      {  // stage qhat, dO_eff, lse, delta for rows i0..i0+31 (8 threads per row)
        const int r = tid >> 3, part = tid & 7;
        const int i = i0 + r;
        float qreg[PT], dreg[PT];
        if (i < p.Sq) {
          const float* qp = row_ptr<float>(p.q, b, h, i) + part * PT;
          const float* dp = a.do_eff ? reinterpret_cast<const float*>(a.do_eff) + (((int64_t)b * p.H + h) * p.Sq + i) * D + part * PT
                                     : row_ptr<float>(p.d_o, b, h, i) + part * PT;
#pragma unroll
          for (int e = 0; e < PT; e += 4) {
            float t[4];
            Elem<float>::load(qp + e, t);
            qreg[e] = t[0]; qreg[e + 1] = t[1]; qreg[e + 2] = t[2]; qreg[e + 3] = t[3];
            Elem<float>::load(dp + e, t);
            dreg[e] = t[0]; dreg[e + 1] = t[1]; dreg[e + 2] = t[2]; dreg[e + 3] = t[3];
          }
        } else {
#pragma unroll
          for (int e = 0; e < PT; ++e) { qreg[e] = 0.f; dreg[e] = 0.f; }
        }
        if (p.rope_cos) rope_lanes<D, PT, 8, false>(p, qreg, p.rope_q_pos0 + min(i, p.Sq - 1), part * PT);
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < PT; ++e) ss += qreg[e] * qreg[e];
        ss = oct_sum(ss);
        const float alpha = row_normaliser(p, ss, 1.0f / D);
#pragma unroll
        for (int e = 0; e < PT; ++e) {
          qs[r * D + part * PT + e] = qreg[e] * alpha * gprod<D>(p, part * PT + e) * p.sm_scale;
          dos[r * D + part * PT + e] = dreg[e];
        }
        if (part == 0) {
          const int64_t ridx = ((int64_t)b * p.H + h) * p.Sq + min(i, p.Sq - 1);
          ls[r] = p.lse[ridx];
          des[r] = a.delta[ridx];
        }
      }
      __syncthreads();
#pragma unroll 2
      for (int x = 0; x < kTile; ++x) {
        const float* qr = qs + x * D + sub * DP;
        const float* dr = dos + x * D + sub * DP;
        float s = 0.f, dpv = 0.f;
#pragma unroll
        for (int e = 0; e < DP; ++e) { s += kh[e] * qr[e]; dpv += vmix[e] * dr[e]; }
        s = quad_sum(s);
        dpv = quad_sum(dpv);
        const int i = i0 + x;
        const bool vis = live && i < p.Sq && (!p.causal || j <= i + p.q_start);
        const float pj = vis ? expf(s - ls[x]) : 0.f;
        const float ds = pj * (dpv - des[x]);
#pragma unroll
        for (int e = 0; e < DP; ++e) { dV[e] += pj * dr[e]; W[e] += ds * qr[e]; }
      }
    }
  }
  // through the k normaliser (khat = b k; the k scale vector lives in qhat); raw rows are re-read
  float dot = 0.f, s1 = 0.f, s2 = 0.f;
  float kraw[DP];
  {
    const float* kp = row_ptr<float>(p.k, b, g, jc) + sub * DP;
#pragma unroll
    for (int e = 0; e < DP; e += 4) {
      float t[4];
      Elem<float>::load(kp + e, t);
#pragma unroll
      for (int x = 0; x < 4; ++x) kraw[e + x] = t[x];
    }
  }
  if (p.rope_cos) rope_lanes<D, DP, 4, false>(p, kraw, p.rope_k_pos0 + jc, sub * DP);  // the normaliser saw the rotated row
#pragma unroll
  for (int e = 0; e < DP; ++e) dot += W[e] * kraw[e];
  dot = quad_sum(dot);
  {
    const float b3 = norm_grad_coef(p, beta, 1.0f / D) * dot;
#pragma unroll
    for (int e = 0; e < DP; ++e) W[e] = beta * W[e] - b3 * kraw[e];
    if (p.rope_cos) rope_lanes<D, DP, 4, true>(p, W, p.rope_k_pos0 + jc, sub * DP);
  }
  if (live) {
    float* okp = row_ptr_mut<float>(p.dk, b, g, j) + sub * DP;
    float* ovp = row_ptr_mut<float>(p.dv, b, g, j) + sub * DP;
#pragma unroll
    for (int e = 0; e < DP; e += 4) {
      float t[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) t[x] = W[e + x];
      Elem<float>::store(okp + e, t);
#pragma unroll
      for (int x = 0; x < 4; ++x) t[x] = c1 * dV[e + x];
      Elem<float>::store(ovp + e, t);
    }
    if (p.v_first.ptr) {
      float* ofp = row_ptr_mut<float>(p.dv_first, b, g, j) + sub * DP;
      const float* vp = row_ptr<float>(p.v, b, g, j) + sub * DP;
      const float* fp = row_ptr<float>(p.v_first, b, g, j) + sub * DP;
#pragma unroll
      for (int e = 0; e < DP; e += 4) {
        float t[4], tv[4], tf[4];
        Elem<float>::load(vp + e, tv);
        Elem<float>::load(fp + e, tf);
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          t[x] = c2 * dV[e + x];
          s1 += dV[e + x] * tv[x];
          s2 += dV[e + x] * tf[x];
        }
        Elem<float>::store(ofp + e, t);
      }
    }
  }
  if (p.vr_coef) {
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) { s1 += __shfl_xor(s1, o, 64); s2 += __shfl_xor(s2, o, 64); }
    const int wave = tid >> 6, lane = tid & 63;
    __syncthreads();
    if (lane == 0) { red[wave * 2] = s1; red[wave * 2 + 1] = s2; }
    __syncthreads();
    if (tid < 2) {
      const int blk = (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
      a.dcoef_part[(int64_t)blk * 2 + tid] = red[tid] + red[2 + tid] + red[4 + tid] + red[6 + tid];
    }
  }
}

}  // namespace

int f32_rows_per_block() { return kRows; }

int launch_fwd_f32(const KArgs& a, hipStream_t st) {
  const segpt_attn_params& p = a.p;
  dim3 grid((p.Sq + kRows - 1) / kRows, p.H, p.B), block(kThreads);
  switch (p.D) {
    case 32: hipLaunchKernelGGL(fwd_f32_kernel<32>, grid, block, 0, st, a); break;
    case 64: hipLaunchKernelGGL(fwd_f32_kernel<64>, grid, block, 0, st, a); break;
    case 128: hipLaunchKernelGGL(fwd_f32_kernel<128>, grid, block, 0, st, a); break;
    default: return (int)hipErrorInvalidValue;
  }
  return (int)hipGetLastError();
}

int launch_bwd_dq_f32(const KArgs& a, hipStream_t st) {
  const segpt_attn_params& p = a.p;
  dim3 gq((p.Sq + kRows - 1) / kRows, p.H, p.B), block(kThreads);
  switch (p.D) {
    case 32: hipLaunchKernelGGL(bwd_dq_f32_kernel<32>, gq, block, 0, st, a); break;
    case 64: hipLaunchKernelGGL(bwd_dq_f32_kernel<64>, gq, block, 0, st, a); break;
    case 128: hipLaunchKernelGGL(bwd_dq_f32_kernel<128>, gq, block, 0, st, a); break;
    default: return (int)hipErrorInvalidValue;
  }
  return (int)hipGetLastError();
}

int launch_bwd_dkdv_f32(const KArgs& a, hipStream_t st) {
  const segpt_attn_params& p = a.p;
  dim3 gk((p.Sk + kRows - 1) / kRows, p.Hkv, p.B), block(kThreads);
  switch (p.D) {
    case 32: hipLaunchKernelGGL(bwd_dkdv_f32_kernel<32>, gk, block, 0, st, a); break;
    case 64: hipLaunchKernelGGL(bwd_dkdv_f32_kernel<64>, gk, block, 0, st, a); break;
    case 128: hipLaunchKernelGGL(bwd_dkdv_f32_kernel<128>, gk, block, 0, st, a); break;
    default: return (int)hipErrorInvalidValue;
  }
  return (int)hipGetLastError();
}

}  // namespace segpt
