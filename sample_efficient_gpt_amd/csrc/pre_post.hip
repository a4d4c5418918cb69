// HBM-bound helper kernels:
//   bwd_pre     (fp32 path) delta_i = rowsum(dY_i * Y_i); with a gate also dgate = (1 - sigmoid(z)) * delta
//               and dO_eff = gate_scale * sigmoid(z) * dY  (Y is the saved, already gated output, so
//               rowsum(dO_eff * O) == rowsum(dY * Y) and no division by the gate is needed).  On the bf16 path
//               the dQ kernel's prologue does this.
//   kv_prep     (bf16 path, forward and backward) the normalised keys Khat and mixed values V' that the MFMA
//               kernels stream, so that their inner loops carry no norm arithmetic.
//   bwd_reduce  second stage of the scale-gradient reduction: sums the per-workgroup partial
//               vectors and applies dg_q = g_k * dg, dg_k = g_q * dg (the logits depend on the two
//               scale vectors only through their product); also sums the (dc1, dc2) partials.
#include "common.hpp"

namespace segpt {
namespace {

template <typename T, int D>
__global__ __launch_bounds__(256) void bwd_pre_kernel(KArgs a) {
  const segpt_attn_params& p = a.p;
  constexpr int V = Elem<T>::kVec;
  constexpr int TPR = D / V;          // threads per row
  constexpr int RPB = 256 / TPR;      // rows per pass of a block
  const int tid = threadIdx.x;
  const int part = tid % TPR;
  const int64_t nrows = (int64_t)p.B * p.H * p.Sq;
  for (int64_t row0 = (int64_t)blockIdx.x * RPB; row0 < nrows; row0 += (int64_t)gridDim.x * RPB) {
    const int64_t rid = row0 + tid / TPR;  // flat (b, h, s)
    const bool live = rid < nrows;
    const int64_t r = live ? rid : nrows - 1;
    const int s = (int)(r % p.Sq);
    const int h = (int)((r / p.Sq) % p.H);
    const int b = (int)(r / ((int64_t)p.Sq * p.H));
    float y[V], dy[V];
    Elem<T>::load(row_ptr<T>(p.o, b, h, s) + part * V, y);
    Elem<T>::load(row_ptr<T>(p.d_o, b, h, s) + part * V, dy);
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < V; ++e) acc += y[e] * dy[e];
#pragma unroll
    for (int o = 1; o < TPR; o <<= 1) acc += __shfl_xor(acc, o, 64);
    if (!live) continue;
    if (part == 0) a.delta[r] = acc;
    if (p.gate.ptr) {
      const int64_t gi = (int64_t)b * p.gate.stride_b + (int64_t)s * p.gate.stride_s + (int64_t)h * p.gate.stride_h;
      const float z = Elem<T>::load1(reinterpret_cast<const T*>(p.gate.ptr) + gi);
      const float sg = sigmoidf_acc(z);
      if (part == 0) {
        const int64_t di = (int64_t)b * p.dgate.stride_b + (int64_t)s * p.dgate.stride_s + (int64_t)h * p.dgate.stride_h;
        Elem<T>::store1(reinterpret_cast<T*>(p.dgate.ptr) + di, (1.0f - sg) * acc);
      }
      const float f = p.gate_scale * sg;
#pragma unroll
      for (int e = 0; e < V; ++e) dy[e] *= f;
      Elem<T>::store(reinterpret_cast<T*>(a.do_eff) + r * D + part * V, dy);
    }
  }
}

// bf16 path: Khat = b_j k_j and (with a value residual) V' = c1 v + c2 v_first, one row per 8/16 lanes
template <int D>
__global__ __launch_bounds__(256) void kv_prep_kernel(KArgs a) {
  const segpt_attn_params& p = a.p;
  constexpr int TPR = D / 8;
  constexpr int RPB = 256 / TPR;
  const int tid = threadIdx.x;
  const int part = tid % TPR;
  const int64_t rid = (int64_t)blockIdx.x * RPB + tid / TPR;  // flat (b, g, s)
  const int64_t nrows = (int64_t)p.B * p.Hkv * p.Sk;
  const bool live = rid < nrows;
  const int64_t r = live ? rid : nrows - 1;
  const int s = (int)(r % p.Sk);
  const int g = (int)((r / p.Sk) % p.Hkv);
  const int b = (int)(r / ((int64_t)p.Sk * p.Hkv));
  float k[8];
  Elem<uint16_t>::load(row_ptr<uint16_t>(p.k, b, g, s) + part * 8, k);
  if (p.rope_cos) {
    // split-half pairs (j, j + D/2): the partner element sits TPR/2 lanes away, same slot.  The lane's eight table
    // entries come in as four 16-byte loads (table rows are 16-byte aligned and jp is a multiple of 8 floats) and the
    // two halves share one expression, x' = x c + sign * partner * s, so that no lane-dependent branch splits the loads.
    const int jp = (part % (TPR / 2)) * 8;
    const float* cr = p.rope_cos + (int64_t)(p.rope_k_pos0 + s) * (D / 2) + jp;
    const float* sr = p.rope_sin + (int64_t)(p.rope_k_pos0 + s) * (D / 2) + jp;
    const float4 c0 = *reinterpret_cast<const float4*>(cr), c1 = *reinterpret_cast<const float4*>(cr + 4);
    const float4 s0 = *reinterpret_cast<const float4*>(sr), s1 = *reinterpret_cast<const float4*>(sr + 4);
    const float cv[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
    const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
    const float sign = part < TPR / 2 ? -1.f : 1.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float other = __shfl_xor(k[e], TPR / 2, 64);
      k[e] = k[e] * cv[e] + sign * other * sv[e];
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) ss += k[e] * k[e];
#pragma unroll
  for (int o = 1; o < TPR; o <<= 1) ss += __shfl_xor(ss, o, 64);
  const float beta = row_normaliser(p, ss, 1.0f / D);
#pragma unroll
  for (int e = 0; e < 8; ++e) k[e] *= beta;
  if (live) Elem<uint16_t>::store(a.khat + r * D + part * 8, k);
  if (a.vmix) {
    const float c1 = p.vr_coef[0], c2 = p.vr_coef[1];
    float v[8], f[8];
    Elem<uint16_t>::load(row_ptr<uint16_t>(p.v, b, g, s) + part * 8, v);
    Elem<uint16_t>::load(row_ptr<uint16_t>(p.v_first, b, g, s) + part * 8, f);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = c1 * v[e] + c2 * f[e];
    if (live) Elem<uint16_t>::store(a.vmix + r * D + part * 8, v);
  }
}

constexpr int kReduceThreads = 1024;

__global__ __launch_bounds__(kReduceThreads) void bwd_reduce_kernel(KArgs a) {
  const segpt_attn_params& p = a.p;
  __shared__ float red[kReduceThreads];
  __shared__ float tot[128];
  const int tid = threadIdx.x;
  // bf16: the scale-vector gradient is reduced inside the dK/dV kernel (by its lightest workgroup)
  if (p.dtype == SEGPT_DTYPE_FP32) reduce_scale_grad<kReduceThreads>(a, tid, red, tot);
  if (p.vr_coef) {
    __syncthreads();
    float s1 = 0.f, s2 = 0.f;
    for (int b2 = tid; b2 < a.n_dkdv_blocks; b2 += kReduceThreads) {
      s1 += a.dcoef_part[(int64_t)b2 * 2];
      s2 += a.dcoef_part[(int64_t)b2 * 2 + 1];
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) { s1 += __shfl_xor(s1, o, 64); s2 += __shfl_xor(s2, o, 64); }
    if ((tid & 63) == 0) { red[(tid >> 6) * 2] = s1; red[(tid >> 6) * 2 + 1] = s2; }
    __syncthreads();
    if (tid < 2) {
      float t = 0.f;
      for (int w = 0; w < kReduceThreads / 64; ++w) t += red[w * 2 + tid];
      p.dvr_coef[tid] = t;
    }
  }
}

template <typename T>
int launch_pre_t(const KArgs& a, hipStream_t st) {
  const segpt_attn_params& p = a.p;
  const int64_t nrows = (int64_t)p.B * p.H * p.Sq;
  constexpr int V = Elem<T>::kVec;
  const int rpb = 256 / (p.D / V);
  const int64_t groups = (nrows + rpb - 1) / rpb;
  dim3 grid((unsigned)(groups < 8192 ? groups : 8192)), block(256);  // grid-stride: <= 32 blocks per CU
  switch (p.D) {
    case 32:
      if constexpr (sizeof(T) == 4) { hipLaunchKernelGGL((bwd_pre_kernel<T, 32>), grid, block, 0, st, a); break; }
      return (int)hipErrorInvalidValue;
    case 64: hipLaunchKernelGGL((bwd_pre_kernel<T, 64>), grid, block, 0, st, a); break;
    case 128: hipLaunchKernelGGL((bwd_pre_kernel<T, 128>), grid, block, 0, st, a); break;
    default: return (int)hipErrorInvalidValue;
  }
  return (int)hipGetLastError();
}

}  // namespace

int launch_bwd_pre(const KArgs& a, hipStream_t st) {
  if (a.p.dtype != SEGPT_DTYPE_FP32) return (int)hipErrorInvalidValue;
  return launch_pre_t<float>(a, st);
}

// bf16: the per-key-row pre-pass shared by forward and backward (the per-query-row quantities of the backward,
// delta / Qhat / gate terms, come from the dQ kernel's prologue)
int launch_kv_prep(const KArgs& a, hipStream_t st) {
  const segpt_attn_params& p = a.p;
  const int64_t nrows = (int64_t)p.B * p.Hkv * p.Sk;
  const int rpb = 256 / (p.D / 8);
  dim3 grid((unsigned)((nrows + rpb - 1) / rpb)), block(256);
  if (p.D == 64) hipLaunchKernelGGL(kv_prep_kernel<64>, grid, block, 0, st, a);
  else hipLaunchKernelGGL(kv_prep_kernel<128>, grid, block, 0, st, a);
  return (int)hipGetLastError();
}

int launch_bwd_reduce(const KArgs& a, hipStream_t st) {
  if (a.p.dtype == SEGPT_DTYPE_BF16 && !a.p.vr_coef) return 0;  // nothing left to reduce
  hipLaunchKernelGGL(bwd_reduce_kernel, dim3(1), dim3(kReduceThreads), 0, st, a);
  return (int)hipGetLastError();
}

}  // namespace segpt
