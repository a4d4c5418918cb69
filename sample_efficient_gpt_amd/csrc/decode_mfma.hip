// bf16 forward for decode-shaped calls: a handful of query rows (H/Hkv * Sq <= 32 per kv head) against a long
// key/value cache (the reference's generation path: attention.py:191-198 builds q_start = past length,
// KVCache :15-27 grows K/V, the module masks with k_idx <= q_start + q_idx, :72-78).
//
// The training kernel would run B*H workgroups that each walk the whole cache; here the KEYS are split
// ("flash decoding"): workgroup (b, kv head g, split s) handles one contiguous chunk of the cache for ALL query
// rows of the group (n = hq * Sq + i, at most 32 = one MFMA column block), writes an unnormalised partial
// (running maximum M, sum L, O) and a second tiny kernel merges the splits.  Memory-bound by design: every
// K / V row is read exactly once from HBM, so the key normalisation, the rotary embedding and the value
// residual mix are done on the fly in registers (no pre-pass, no normalised copy).
//
// Per wave and 32-key block (orientation as in the training forward: lane = query column):
//   K rows -> registers in the MFMA A layout (row = key, 16-byte chunks), rotate, b_j = rsqrt(mean k^2 + eps)
//   across the lane pair that holds a row, scale, pack            S^T = Khat . Qhat^T          (4 or 8 MFMAs)
//   online softmax per lane, P^T packed to bf16 = B operand
//   V rows -> wave-private LDS tile (row-major, padded) -> transposing reads    O^T += V'^T . P^T
#include "mfma_common.hpp"

namespace segpt {
namespace {

constexpr int kDecThreads = 256;  // 4 waves, 32 keys each per step
constexpr int kDecKeysPerStep = 4 * 32;

template <int D>
struct DecTile {
  static constexpr int kRS = D + 8;  // padded row stride (elements) of the wave-private V tile
};

// Transposed fragment of a padded row-major tile (see swz_off_tr for the ds_read_b64_tr_b16 semantics):
// lane's MFMA row = tile column 32*cb + l%32, contraction entries = tile rows 16*s + {4hh.., 8+4hh..}
template <int D>
__device__ __forceinline__ bf16x8 dec_frag_tr(const uint16_t* tile, int cb, int s, int lane) {
  const int r = lane & 15, hh = lane >> 5;
  const int col = 32 * cb + 16 * ((lane >> 4) & 1) + 4 * (r & 3);
  const int row = 16 * s + 4 * hh + (r >> 2);
  const uint16_t* p = tile + row * DecTile<D>::kRS + col;
  typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 8 * DecTile<D>::kRS));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, v);
}

template <int D>
__global__ __launch_bounds__(kDecThreads) void decode_split_kernel(KArgs a) {
  constexpr int KS = D / 16;
  constexpr int MB = D / 32;
  constexpr int RS = DecTile<D>::kRS;
  const segpt_attn_params& p = a.p;
  // wave-private V' tiles during the key loop; afterwards the same memory holds the per-wave O^T partials
  constexpr int kVtBytes = 4 * 32 * RS * 2, kOsmBytes = 4 * D * 32 * 4;
  __shared__ __attribute__((aligned(16))) char tile_mem[kVtBytes > kOsmBytes ? kVtBytes : kOsmBytes];
  uint16_t (*vt)[32 * RS] = reinterpret_cast<uint16_t (*)[32 * RS]>(tile_mem);
  float (*osm)[D][32] = reinterpret_cast<float (*)[D][32]>(tile_mem);
  __shared__ __attribute__((aligned(16))) float gsm[D];
  __shared__ float msm[4][32], lsm[4][32];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, hh = lane >> 5;
  const int rep = p.H / p.Hkv;
  const int n_rows = rep * p.Sq;  // query rows of this kv head, <= 32
  const int split = blockIdx.x % a.dec_splits;
  const int bg = blockIdx.x / a.dec_splits;
  const int g = bg % p.Hkv, b = bg / p.Hkv;

  // ---- this lane's query (B operand column n): Qhat = sm_scale*log2e * a q g_q g_k, zero for padding columns
  if (tid < D) gsm[tid] = gprod_at(p, tid) * p.sm_scale * kLog2e;
  __syncthreads();
  const bool qlive = ln < n_rows;
  const int hq = qlive ? ln / p.Sq : 0, qi = qlive ? ln % p.Sq : 0;
  bf16x8 qreg[KS];
  {
    const uint16_t* qp = row_ptr<uint16_t>(p.q, b, g * rep + hq, qi) + 8 * hh;
    u32x4 raw[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) raw[ks] = *reinterpret_cast<const u32x4*>(qp + 16 * ks);
    float x[KS][8];
    unpack_b_layout<KS>(raw, x);
    if (p.rope_cos) {
      const int64_t pos = (int64_t)(p.rope_q_pos0 + qi) * (D / 2);
      rope_b_layout<KS>(x, p.rope_cos + pos, p.rope_sin + pos, hh);
    }
    float ss = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int t = 0; t < 8; ++t) ss += x[ks][t] * x[ks][t];
    ss = half_sum(ss);
    const float alpha = qlive ? row_normaliser_fast(p, ss, 1.0f / D) : 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const float4 ga = *reinterpret_cast<const float4*>(gsm + 16 * ks + 8 * hh);
      const float4 gb = *reinterpret_cast<const float4*>(gsm + 16 * ks + 8 * hh + 4);
      u32x4 w;
      w[0] = pack_bf16x2(x[ks][0] * alpha * ga.x, x[ks][1] * alpha * ga.y);
      w[1] = pack_bf16x2(x[ks][2] * alpha * ga.z, x[ks][3] * alpha * ga.w);
      w[2] = pack_bf16x2(x[ks][4] * alpha * gb.x, x[ks][5] * alpha * gb.y);
      w[3] = pack_bf16x2(x[ks][6] * alpha * gb.z, x[ks][7] * alpha * gb.w);
      qreg[ks] = as_bf16x8(w);
    }
  }
  // last visible key of this lane's query
  const int qlim = p.causal ? min(qi + p.q_start, p.Sk - 1) : p.Sk - 1;

  float c1 = 1.f, c2 = 0.f;
  if (p.vr_coef) { c1 = p.vr_coef[0]; c2 = p.vr_coef[1]; }

  f32x16 oacc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) oacc[mb] = splat16(0.f);
  float m_run = -INFINITY, l_run[2] = {0.f, 0.f};  // l_run: this lane's half of the keys, as two partial sums

  // keys [k_lo, k_hi) of this split; wave w takes the 32-key blocks w, w+4, ...
  const int k_lo = split * a.dec_chunk;
  const int k_hi = min(k_lo + a.dec_chunk, a.dec_kend);
  uint16_t* my_vt = vt[wave];
  for (int jb = k_lo + 32 * wave; jb < k_hi; jb += kDecKeysPerStep) {
    // ---- K rows of the block in the A layout: lane (row ln, chunk hh)
    const int krow = min(jb + ln, p.Sk - 1);
    const uint16_t* kp = row_ptr<uint16_t>(p.k, b, g, krow) + 8 * hh;
    const uint16_t* vp = row_ptr<uint16_t>(p.v, b, g, krow) + 8 * hh;
    u32x4 kraw[KS], vraw[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kraw[ks] = *reinterpret_cast<const u32x4*>(kp + 16 * ks);
      vraw[ks] = *reinterpret_cast<const u32x4*>(vp + 16 * ks);
    }
    if (p.v_first.ptr) {
      const uint16_t* fp = row_ptr<uint16_t>(p.v_first, b, g, krow) + 8 * hh;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const u32x4 f = *reinterpret_cast<const u32x4*>(fp + 16 * ks);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          vraw[ks][i] = pack_bf16x2(c1 * bf16lo(vraw[ks][i]) + c2 * bf16lo(f[i]), c1 * bf16hi(vraw[ks][i]) + c2 * bf16hi(f[i]));
      }
    }
    float kx[KS][8];
    unpack_b_layout<KS>(kraw, kx);
    if (p.rope_cos) {
      const int64_t pos = (int64_t)(p.rope_k_pos0 + krow) * (D / 2);
      rope_b_layout<KS>(kx, p.rope_cos + pos, p.rope_sin + pos, hh);
    }
    float ss = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int t = 0; t < 8; ++t) ss += kx[ks][t] * kx[ks][t];
    ss = half_sum(ss);
    const float beta = row_normaliser_fast(p, ss, 1.0f / D);
    f32x16 s = splat16(0.f);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 w;
#pragma unroll
      for (int i = 0; i < 4; ++i) w[i] = pack_bf16x2(kx[ks][2 * i] * beta, kx[ks][2 * i + 1] * beta);
      s = mfma32(as_bf16x8(w), qreg[ks], s);
    }
    // ---- V' rows into the wave's LDS tile (row-major); read back transposed after the softmax
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) *reinterpret_cast<u32x4*>(my_vt + ln * RS + 16 * ks + 8 * hh) = vraw[ks];

    // ---- mask: register r holds key jb + 4hh + c_r, c_r = 8(r/4) + r%4; visible iff <= qlim and < k_hi
    {
      const int t = min(qlim, k_hi - 1) - jb - 4 * hh;
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if (8 * (r >> 2) + (r & 3) > t) s[r] = -INFINITY;
    }
    // ---- online softmax (per lane = per query; the two lane halves hold different keys)
    float mx = s[0];
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[r]);
    mx = half_max(mx);
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // nothing visible yet: keep exp2 away from inf - inf
    const float corr = fast_exp2(m_run - m_use);           // m_run = -inf gives 0
    m_run = m_new;
    l_run[0] *= corr;
    l_run[1] *= corr;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[mb][r] *= corr;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = fast_exp2(s[r] - m_use);
    bf16x8 pb[2];
    pb[0] = pack_c_half_sum(s, 0, l_run);
    pb[1] = pack_c_half_sum(s, 1, l_run);
    __builtin_amdgcn_wave_barrier();  // the tile was written by this wave only; keep the reads below the writes
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) oacc[mb] = mfma32(dec_frag_tr<D>(my_vt, mb, s2, lane), pb[s2], oacc[mb]);
    __builtin_amdgcn_wave_barrier();  // next iteration overwrites the tile
  }

  // ---- merge the four waves (different keys, same queries) and write this split's partial
  __syncthreads();  // every wave is done with its V' tile: the memory is reused for the partials
  const float l_tot = half_sum(l_run[0] + l_run[1]);
  if (hh == 0) { msm[wave][ln] = m_run; lsm[wave][ln] = l_tot; }
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) osm[wave][32 * mb + 8 * (r >> 2) + 4 * hh + (r & 3)][ln] = oacc[mb][r];
  __syncthreads();
  float* part_o = a.dec_part + ((int64_t)bg * a.dec_splits + split) * 32 * D;
  float* part_s = a.dec_stat + ((int64_t)bg * a.dec_splits + split) * 32 * 2;
  for (int e = tid; e < 32 * D; e += kDecThreads) {
    const int n = e % 32, d = e / 32;
    const float m0 = msm[0][n], m1 = msm[1][n], m2 = msm[2][n], m3 = msm[3][n];
    const float M = fmaxf(fmaxf(m0, m1), fmaxf(m2, m3));
    const float Mu = M == -INFINITY ? 0.f : M;
    const float w0 = fast_exp2(m0 - Mu), w1 = fast_exp2(m1 - Mu), w2 = fast_exp2(m2 - Mu), w3 = fast_exp2(m3 - Mu);
    part_o[n * D + d] = (osm[0][d][n] * w0 + osm[1][d][n] * w1) + (osm[2][d][n] * w2 + osm[3][d][n] * w3);
    if (d == 0) {
      part_s[n * 2] = M;
      part_s[n * 2 + 1] = (lsm[0][n] * w0 + lsm[1][n] * w1) + (lsm[2][n] * w2 + lsm[3][n] * w3);
    }
  }
}

// One workgroup per (batch, kv head, query row): merges the splits, normalises, gates, writes y (bf16) and lse
// (natural log).  Thread (group gi, column d) sums the splits gi, gi + G, ... of output column d (G = threads / D);
// its first partial values are requested before the split statistics are reduced, so that the kernel is about
// two memory round trips long whatever the number of splits.  Every sum has a fixed order: deterministic.
constexpr int kMergeThreads = 256;
constexpr int kMaxSplits = 512;
constexpr int kMergeEarly = 16;  // partial values per thread requested up front

__global__ __launch_bounds__(kMergeThreads) void decode_merge_kernel(KArgs a) {
  const segpt_attn_params& p = a.p;
  __shared__ float wsm[kMaxSplits];
  __shared__ float redm[4], redl[4];
  __shared__ float part[kMergeThreads];
  const int D = p.D, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rep = p.H / p.Hkv;
  const int n_rows = rep * p.Sq;
  const int n = blockIdx.x % n_rows, bg = blockIdx.x / n_rows;
  const int g = bg % p.Hkv, b = bg / p.Hkv;
  const int S = a.dec_splits;
  const int G = kMergeThreads / D, gi = tid / D, d = tid - gi * D;
  const float* col = a.dec_part + (int64_t)bg * S * 32 * D + (int64_t)n * D + d;
  const float* ss = a.dec_stat + (int64_t)bg * S * 32 * 2;
  float pv[kMergeEarly];
#pragma unroll
  for (int u = 0; u < kMergeEarly; ++u) {
    const int sp = gi + G * u;
    pv[u] = sp < S ? col[(int64_t)sp * 32 * D] : 0.f;
  }
  float m = -INFINITY;
  for (int sp = tid; sp < S; sp += kMergeThreads) m = fmaxf(m, ss[(sp * 32 + n) * 2]);
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if (lane == 0) redm[wave] = m;
  __syncthreads();
  const float M = fmaxf(fmaxf(redm[0], redm[1]), fmaxf(redm[2], redm[3]));
  float l = 0.f;
  for (int sp = tid; sp < S; sp += kMergeThreads) {
    const float w = exp2f(ss[(sp * 32 + n) * 2] - M);  // a split with nothing visible has (-inf, 0): weight 0
    wsm[sp] = w;
    l += ss[(sp * 32 + n) * 2 + 1] * w;
  }
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) l += __shfl_xor(l, o, 64);
  if (lane == 0) redl[wave] = l;
  __syncthreads();  // also publishes wsm
  const float L = (redl[0] + redl[1]) + (redl[2] + redl[3]);
  float acc = 0.f;
#pragma unroll
  for (int u = 0; u < kMergeEarly; ++u) {
    const int sp = gi + G * u;
    if (sp < S) acc += pv[u] * wsm[sp];
  }
  for (int sp = gi + G * kMergeEarly; sp < S; sp += G) acc += col[(int64_t)sp * 32 * D] * wsm[sp];
  part[tid] = acc;
  __syncthreads();
  const int hq = n / p.Sq, qi = n % p.Sq;
  const int h = g * rep + hq;
  if (tid == 0) p.lse[((int64_t)b * p.H + h) * p.Sq + qi] = (M + log2f(L)) * kLn2;
  if (tid < D) {
    float f = 1.0f / L;
    if (p.gate.ptr) {
      const float z = bf16_to_f32(reinterpret_cast<const uint16_t*>(p.gate.ptr)[(int64_t)b * p.gate.stride_b + (int64_t)qi * p.gate.stride_s + (int64_t)h * p.gate.stride_h]);
      f *= p.gate_scale / (1.0f + __expf(-z));
    }
    float tot = part[tid];
    for (int x = 1; x < G; ++x) tot += part[x * D + tid];
    row_ptr_mut<uint16_t>(p.o, b, h, qi)[tid] = f32_to_bf16(tot * f);
  }
}

}  // namespace

// Split plan of a decode-shaped call: keys [0, kend) in `splits` chunks of `chunk` keys (a multiple of 128):
// enough workgroups for one resident round, no empty split: three per CU at head_dim 64 (what the kernel's
// registers allow; measured 17 % faster than two per CU, four is slower again), one per CU at head_dim 128
// (15 % faster than two).  Returns the scratch bytes the partials need.
size_t decode_plan(const segpt_attn_params& p, int* kend_out, int* splits_out, int* chunk_out) {
  int kend = p.Sk;
  if (p.causal && p.Sq + p.q_start < kend) kend = p.Sq + p.q_start;
  const int groups = p.B * p.Hkv;
  const int target = p.D == 64 ? 768 : 256;
  int s = (target + groups - 1) / groups;
  const int max_s = (kend + kDecKeysPerStep - 1) / kDecKeysPerStep;
  if (s > max_s) s = max_s;
  if (s > kMaxSplits) s = kMaxSplits;
  if (s < 1) s = 1;
  const int per = (kend + s - 1) / s;
  const int chunk = (per + kDecKeysPerStep - 1) / kDecKeysPerStep * kDecKeysPerStep;
  s = (kend + chunk - 1) / chunk;
  *kend_out = kend; *splits_out = s; *chunk_out = chunk;
  return (size_t)p.B * p.Hkv * s * 32 * ((size_t)p.D + 2) * sizeof(float);
}

int launch_fwd_decode_bf16(KArgs a, hipStream_t st) {
  const segpt_attn_params& p = a.p;
  decode_plan(p, &a.dec_kend, &a.dec_splits, &a.dec_chunk);
  char* ws = reinterpret_cast<char*>(p.kv_workspace);
  a.dec_part = reinterpret_cast<float*>(ws);
  a.dec_stat = a.dec_part + (size_t)p.B * p.Hkv * a.dec_splits * 32 * p.D;
  const dim3 grid((unsigned)(p.B * p.Hkv * a.dec_splits));
  if (p.D == 64) hipLaunchKernelGGL(decode_split_kernel<64>, grid, dim3(kDecThreads), 0, st, a);
  else if (p.D == 128) hipLaunchKernelGGL(decode_split_kernel<128>, grid, dim3(kDecThreads), 0, st, a);
  else return (int)hipErrorInvalidValue;
  int rc = (int)hipGetLastError();
  if (rc) return rc;
  hipLaunchKernelGGL(decode_merge_kernel, dim3((unsigned)(p.B * p.Hkv * (p.H / p.Hkv) * p.Sq)), dim3(kMergeThreads), 0, st, a);
  return (int)hipGetLastError();
}

}  // namespace segpt
