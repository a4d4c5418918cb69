// bf16 forward: causal GQA flash attention with the QK RMS-norm fused into the tile loads.
//
// Workgroup = 4 waves (two workgroups share a CU so that one's softmax overlaps the other's MFMAs);
// wave w owns NQB blocks of 32 queries.  Scores are produced TRANSPOSED,
//   S^T[key][query] = Khat[key][:] . Qhat[query][:]          (A = Khat tile from LDS, B = Qhat registers)
// so every lane owns one query column: the online-softmax state (m, l) and the rescale factor are
// per-lane scalars, row reductions are in-register plus one exchange with lane^32, and the bf16
// probabilities are already laid out as the B operand of
//   O^T[d][query] += V'^T[d][key] . P^T[key][query]          (A = transposing LDS read of the V' tile).
// Qhat = sm_scale*log2(e) * a_i * q_i * g_q * g_k  (both scale vectors live on the query side),
// Khat = b_j * k_j, V' = c1 v + c2 v_first; all three are formed in fp32 and rounded to bf16 once.
// K/V tiles (64 keys) are double-buffered in LDS against the global loads of the next tile.
#include "mfma_common.hpp"

namespace segpt {
namespace {

template <int D, int NQB>
struct FwdCfg {
  static constexpr int kBQ = 4 * 32 * NQB;  // queries per workgroup
};

// Largest |log2-unit logit| the normalised operands can produce: |Qhat.Khat| <= |Qhat| |Khat| with
// |Khat| <= sqrt(D) and |Qhat| <= sm_scale*log2e*sqrt(D)*max|g_q g_k|.  When it is small the softmax needs
// no running maximum at all (softmax is shift invariant and exp2 cannot overflow): P = exp2(S2) directly.
__device__ __forceinline__ float logit_bound(const segpt_attn_params& p, int lane) {
  float gm = 0.f;
  for (int d = lane; d < p.D; d += 64) {
    float g = p.gq_numel == 1 ? p.g_q[0] : p.g_q[d];
    if (p.gk_numel == 1) g *= p.g_k[0];
    else if (p.gk_numel > 1) g *= p.g_k[d];
    gm = fmaxf(gm, fabsf(g));
  }
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) gm = fmaxf(gm, __shfl_xor(gm, o, 64));
  return p.sm_scale * kLog2e * (float)p.D * gm * 1.02f;
}

constexpr float kNoMaxBound = 64.f;   // |S2| below this: P in [2^-64, 2^64], sums stay far inside fp32 range
constexpr float kLazyThresh = 16.f;   // general path: the subtracted reference is raised only when exceeded by 2^16

template <int D, int NQB, bool VR>
#ifndef SEGPT_FWD_OCC
#define SEGPT_FWD_OCC 2
#endif
#ifndef SEGPT_FWD_NQB
#define SEGPT_FWD_NQB 2
#endif
__global__ __launch_bounds__(kThreadsM, SEGPT_FWD_OCC) void fwd_bf16_kernel(KArgs a) {
  using T = Tile<D>;
  constexpr int BQ = FwdCfg<D, NQB>::kBQ;
  constexpr int KS = D / 16;  // contraction steps of QK^T
  constexpr int MB = D / 32;  // 32-row blocks of O^T
  const segpt_attn_params& p = a.p;
  __shared__ __attribute__((aligned(16))) uint16_t lds[2 * 2 * T::kElems];
  __shared__ __attribute__((aligned(16))) float gsm[D];  // sm_scale*log2e * g_q * g_k, read as float4 slices

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, hh = lane >> 5;
  const int rep = p.H / p.Hkv;
  const int n_qt = (p.Sq + BQ - 1) / BQ;
  const WgCoord wg = decode_wg(blockIdx.x, n_qt, p.B, p.Hkv, rep);
  const int b = wg.b, g = wg.g, h = wg.g * rep + wg.hh;
  const int q0 = wg.tile * BQ;
  const int qw0 = q0 + wave * 32 * NQB;  // first query of this wave

  float c1 = 1.f, c2 = 0.f;
  if (VR) { c1 = p.vr_coef[0]; c2 = p.vr_coef[1]; }
  const bool bounded = logit_bound(p, lane) <= kNoMaxBound;  // wave-uniform

  // ---- Qhat registers: B operands of S^T, [nb][ks]
  if (tid < D) {
    float gp = p.gq_numel == 1 ? p.g_q[0] : p.g_q[tid];
    if (p.gk_numel == 1) gp *= p.g_k[0];
    else if (p.gk_numel > 1) gp *= p.g_k[tid];
    gsm[tid] = gp * p.sm_scale * kLog2e;
  }
  __syncthreads();
  bf16x8 qreg[NQB][KS];
#pragma unroll
  for (int nb = 0; nb < NQB; ++nb) {
    const int row = min(qw0 + 32 * nb + ln, p.Sq - 1);
    const uint16_t* qp = row_ptr<uint16_t>(p.q, b, h, row) + 8 * hh;
    u32x4 raw[KS];
    float ss = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      raw[ks] = *reinterpret_cast<const u32x4*>(qp + 16 * ks);
      ss += sumsq8(raw[ks]);
    }
    ss = half_sum(ss);
    const float alpha = fast_rsq(ss * (1.0f / D) + p.eps);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const float4 ga = *reinterpret_cast<const float4*>(gsm + 16 * ks + 8 * hh);
      const float4 gb = *reinterpret_cast<const float4*>(gsm + 16 * ks + 8 * hh + 4);
      u32x4 w;
      w[0] = pack_bf16x2(bf16lo(raw[ks][0]) * alpha * ga.x, bf16hi(raw[ks][0]) * alpha * ga.y);
      w[1] = pack_bf16x2(bf16lo(raw[ks][1]) * alpha * ga.z, bf16hi(raw[ks][1]) * alpha * ga.w);
      w[2] = pack_bf16x2(bf16lo(raw[ks][2]) * alpha * gb.x, bf16hi(raw[ks][2]) * alpha * gb.y);
      w[3] = pack_bf16x2(bf16lo(raw[ks][3]) * alpha * gb.z, bf16hi(raw[ks][3]) * alpha * gb.w);
      qreg[nb][ks] = as_bf16x8(w);
    }
  }

  f32x16 oacc[MB][NQB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[mb][nb][r] = 0.f;
  // m_ref: the value subtracted from the logits before exp2 (0 on the bounded path); l_run: this lane's
  // share of the row sum (its half of the keys; halves are added in the epilogue)
  float m_ref[NQB], l_run[NQB];
#pragma unroll
  for (int nb = 0; nb < NQB; ++nb) { m_ref[nb] = bounded ? 0.f : -INFINITY; l_run[nb] = 0.f; }

  int kend = p.Sk;
  if (p.causal) kend = min(p.Sk, q0 + BQ + p.q_start);
  const int n_kt = (kend + kBK - 1) / kBK;

  StageRegs<D> sr;
  stage_load<D, VR>(p, b, g, 0, sr);
  stage_store<D, VR>(sr, lds, lds + T::kElems, p.eps, c1, c2);
  __syncthreads();

  for (int jt = 0; jt < n_kt; ++jt) {
    const int j0 = jt * kBK;
    const uint16_t* kt = lds + (jt & 1) * 2 * T::kElems;
    const uint16_t* vt = kt + T::kElems;
    const bool more = jt + 1 < n_kt;
    if (more) stage_load<D, VR>(p, b, g, j0 + kBK, sr);

#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int jb = j0 + 32 * kb;  // first key of this 32-key block
      // wave-uniform: does this wave see any key of the block?
      const bool active = jb < p.Sk && (!p.causal || jb <= qw0 + 32 * NQB - 1 + p.q_start);
      if (active) {
        f32x16 s[NQB];
#pragma unroll
        for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
          for (int r = 0; r < 16; ++r) s[nb][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8 af = frag_rowmajor<D>(kt, kb, ks, lane);
#pragma unroll
          for (int nb = 0; nb < NQB; ++nb) s[nb] = mfma32(af, qreg[nb][ks], s[nb]);
        }
        const bool need_mask = (p.causal && jb + 31 > qw0 + p.q_start) || jb + 32 > p.Sk;
        if (need_mask) {
#pragma unroll
          for (int nb = 0; nb < NQB; ++nb) {
            const int qlim = p.causal ? min(qw0 + 32 * nb + ln + p.q_start, p.Sk - 1) : p.Sk - 1;
            // register r holds key jb + 4hh + c_r, c_r = 8(r/4) + r%4: masked iff c_r > qlim - jb - 4hh
            const int t = qlim - jb - 4 * hh;
#pragma unroll
            for (int r = 0; r < 16; ++r)
              if (8 * (r >> 2) + (r & 3) > t) s[nb][r] = -INFINITY;
          }
        }
        if (!bounded) {
          // general path: lazily maintained reference, raised only when a row exceeds it by 2^kLazyThresh
#pragma unroll
          for (int nb = 0; nb < NQB; ++nb) {
            float mx = s[nb][0];
#pragma unroll
            for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[nb][r]);
            mx = half_max(mx);
            const bool need = mx > m_ref[nb] + kLazyThresh;
            if (__builtin_amdgcn_ballot_w64(need) != 0) {
              const float m_new = need ? mx : m_ref[nb];
              const float corr = fast_exp2(m_ref[nb] - m_new);
              m_ref[nb] = m_new;
              l_run[nb] *= corr;
#pragma unroll
              for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[mb][nb][r] *= corr;
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) s[nb][r] -= m_ref[nb];
          }
        }
        bf16x8 pb[2][NQB];
#pragma unroll
        for (int nb = 0; nb < NQB; ++nb) {
#pragma unroll
          for (int r = 0; r < 16; ++r) s[nb][r] = fast_exp2(s[nb][r]);
          pb[0][nb] = pack_c_half_sum(s[nb], 0, l_run[nb]);
          pb[1][nb] = pack_c_half_sum(s[nb], 1, l_run[nb]);
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            const bf16x8 vf = frag_transposed<D>(vt, mb, 2 * kb + s2, lane);
#pragma unroll
            for (int nb = 0; nb < NQB; ++nb) oacc[mb][nb] = mfma32(vf, pb[s2][nb], oacc[mb][nb]);
          }
      }
    }
    if (more) {
      uint16_t* nk = lds + ((jt + 1) & 1) * 2 * T::kElems;
      stage_store<D, VR>(sr, nk, nk + T::kElems, p.eps, c1, c2);
    }
    __syncthreads();
  }

  // ---- epilogue: normalise, gate, store y (bf16) and lse (fp32, natural log)
#pragma unroll
  for (int nb = 0; nb < NQB; ++nb) {
    const int row = qw0 + 32 * nb + ln;
    const bool live = row < p.Sq;
    const float l = half_sum(l_run[nb]);
    float f = fast_rcp(l);
    if (p.gate.ptr) {
      const int rc = live ? row : p.Sq - 1;
      const float z = bf16_to_f32(reinterpret_cast<const uint16_t*>(p.gate.ptr)[(int64_t)b * p.gate.stride_b + (int64_t)rc * p.gate.stride_s + (int64_t)h * p.gate.stride_h]);
      f *= p.gate_scale / (1.0f + __expf(-z));
    }
    if (live && hh == 0) p.lse[((int64_t)b * p.H + h) * p.Sq + row] = (m_ref[nb] + __log2f(l)) * kLn2;
    uint16_t* op = live ? row_ptr_mut<uint16_t>(p.o, b, h, row) : nullptr;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        // registers 8cc..8cc+3 hold d = 32mb+16cc+4hh+{0..3}; 8cc+4..8cc+7 hold d = 32mb+16cc+8+4hh+{0..3}
        const f32x16& o = oacc[mb][nb];
        const uint32_t x0 = pack_bf16x2(o[8 * cc + 0] * f, o[8 * cc + 1] * f);
        const uint32_t x1 = pack_bf16x2(o[8 * cc + 2] * f, o[8 * cc + 3] * f);
        const uint32_t y0 = pack_bf16x2(o[8 * cc + 4] * f, o[8 * cc + 5] * f);
        const uint32_t y1 = pack_bf16x2(o[8 * cc + 6] * f, o[8 * cc + 7] * f);
        // lanes < 32 end up with d = 32mb+16cc+0..7, lanes >= 32 with d = 32mb+16cc+8..15
        auto s0 = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
        auto s1 = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
        const u32x4 w = {s0[0], s1[0], s0[1], s1[1]};
        if (live) *reinterpret_cast<u32x4*>(op + 32 * mb + 16 * cc + 8 * hh) = w;
      }
    }
  }
}

template <int D, int NQB>
int launch_fwd_t(const KArgs& a, hipStream_t st) {
  const segpt_attn_params& p = a.p;
  constexpr int BQ = FwdCfg<D, NQB>::kBQ;
  const int n_qt = (p.Sq + BQ - 1) / BQ;
  dim3 grid((unsigned)(n_qt * p.H * p.B)), block(kThreadsM);
  if (p.v_first.ptr) hipLaunchKernelGGL((fwd_bf16_kernel<D, NQB, true>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((fwd_bf16_kernel<D, NQB, false>), grid, block, 0, st, a);
  return (int)hipGetLastError();
}

}  // namespace

int launch_fwd_bf16(const KArgs& a, hipStream_t st) {
  if (a.p.D == 64) return launch_fwd_t<64, SEGPT_FWD_NQB>(a, st);
  if (a.p.D == 128) return launch_fwd_t<128, 1>(a, st);
  return (int)hipErrorInvalidValue;
}

}  // namespace segpt
