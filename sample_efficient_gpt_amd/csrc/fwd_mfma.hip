// bf16 forward: causal GQA flash attention on the normalised keys of the key/value pre-pass.
//
// Workgroup = 4 waves (two or three workgroups share a CU at head_dim 64 so that one's softmax overlaps the
// others' MFMAs); wave w owns NQB blocks of 32 queries (see FwdShape).  Scores are produced TRANSPOSED,
//   S^T[key][query] = Khat[key][:] . Qhat[query][:]          (A = Khat tile from LDS, B = Qhat registers)
// so every lane owns one query column: the softmax state (reference point, row sum) is a per-lane scalar,
// row reductions are in-register plus one exchange with lane^32, and the bf16 probabilities are already
// laid out as the B operand of
//   O^T[d][query] += V'^T[d][key] . P^T[key][query]          (A = transposing LDS read of the V' tile).
// Qhat = sm_scale*log2(e) * a_i * q_i * g_q * g_k  (both scale vectors live on the query side) is formed in
// the prologue; Khat = b_j * k_j and V' = c1 v + c2 v_first are read as written by the pre-pass.
#include "mfma_common.hpp"
#include "ring_protocol.hpp"

namespace segpt {
namespace {

// Largest |log2-unit logit| the normalised operands can produce: |Qhat.Khat| <= |Qhat| |Khat| with
// |Khat| <= sqrt(D) and |Qhat| <= sm_scale*log2e*sqrt(D)*max|g_q g_k|.  When it is small the softmax needs
// no running maximum at all (softmax is shift invariant and exp2 cannot overflow): P = exp2(S2) directly.
// Read from the scale vector already in LDS (gsm[d] = sm_scale * log2e * g_q[d] * g_k[d]); 2 % of slack for the
// bf16 rounding of the operands.
template <int D>
__device__ __forceinline__ float logit_bound(const float* gsm, int lane) {
  float gm = 0.f;
#pragma unroll
  for (int d = lane; d < D; d += 64) gm = fmaxf(gm, fabsf(gsm[d]));
  // wave-wide maximum by six DPP steps (shifts by 1, 2, 4, 8 inside the rows of 16 lanes, then the row maxima
  // passed on to the next row and the next half): lane 63 ends up with it.  A lane whose source does not exist
  // keeps its own value.
  auto step = [](float v, auto ctrl, auto rows) {
    const int t = __builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), decltype(ctrl)::value, decltype(rows)::value, 0xf, false);
    return fmaxf(v, __int_as_float(t));
  };
  gm = step(gm, IC<0x111>{}, IC<0xf>{});
  gm = step(gm, IC<0x112>{}, IC<0xf>{});
  gm = step(gm, IC<0x114>{}, IC<0xf>{});
  gm = step(gm, IC<0x118>{}, IC<0xf>{});
  gm = step(gm, IC<0x142>{}, IC<0xa>{});
  gm = step(gm, IC<0x143>{}, IC<0xc>{});
  gm = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(gm), 63));
  return (float)D * gm * 1.02f;
}

constexpr float kNoMaxBound = 64.f;   // |S2| below this: P in [2^-64, 2^64], sums stay far inside fp32 range
constexpr float kLazyThresh = 16.f;   // general path: the subtracted reference is raised only when exceeded by 2^16

// Khat / V' come from the key/value pre-pass (bf16, contiguous [B,Hkv,Sk,D]) and travel global->LDS
// directly into a swizzled ring of stages, so the loop holds no staging registers and no normalisation
// work.  Software pipeline over 32-key blocks n (two per staged tile), one barrier per tile:
//   B(n)   S^T MFMAs from the row-major Khat fragments requested one block earlier
//   C(n)   request the transposed V' fragments of block n
//   D(n)   mask (diagonal blocks only), exp2, bf16 pack, row sums
//   A(n+1) request the row-major Khat fragments of block n+1 (possibly of the next tile, already landed)
//   E(n)   O^T += V'^T P^T MFMAs
// Two shapes at head_dim 64.  WIDE: 64 query rows per wave (K fragments shared by two query blocks), four LDS
// stages, two workgroups per CU: best when a workgroup streams many key tiles (S = 8192: 7 % faster than
// NARROW).  NARROW: 32 rows per wave, three stages (48 KB), three workgroups per CU: twice as many, lighter
// workgroups whose start-up / write-out latencies hide behind two neighbours instead of one (S = 2048: 1 %
// faster, S = 1152: 10 %, S = 768: 13 %, S = 384: 27 %).  The launcher picks by the number of keys.
// head_dim 128: 32 rows per wave and 32-KEY tiles (a tile pair is then the same 16 KB as at head_dim 64, a block of a
// tile carries twice the MFMAs, so one block per tile keeps the ratio of barriers and tile loads to MFMAs), four stages
// = 64 KB, two workgroups per CU.  With 64-key tiles the ring alone is 96 KB and a CU holds one workgroup, i.e. one
// wave per SIMD with nothing to overlap its softmax phase with.
template <int D, bool WIDE>
struct FwdShape {
  static constexpr int kNQB = (D == 64 && WIDE) ? 2 : 1;  // 32-query blocks per wave
  static constexpr int kBK = D == 64 ? 64 : 32;           // keys per streamed tile
  static constexpr int kStages = D == 64 ? (WIDE ? 4 : 3) : 4;
  static constexpr int kOcc = D == 64 ? (WIDE ? 2 : 3) : 2;
  static constexpr int kBQ = 4 * 32 * kNQB;
};

// ROPE (rope tables given) is a compile-time switch so that the table rows are ordinary, unconditional loads that
// travel with the start-up tiles instead of costing a memory round trip of their own behind a branch.
template <int D, bool WIDE, bool ROPE>
__global__ __launch_bounds__(kThreadsM, (FwdShape<D, WIDE>::kOcc)) void fwd_bf16_kernel(KArgs a) {
  using F = FwdShape<D, WIDE>;
  constexpr int NQB = F::kNQB, BQ = F::kBQ, NS = F::kStages, BK = F::kBK;
  constexpr int kBlocksPerTile = BK / 32;
  using Z = Swz<D, BK>;
  constexpr int KS = D / 16;
  constexpr int MB = D / 32;
  constexpr int kStageBytes = 2 * Z::kTileBytes;
  constexpr int kLoadsPerTile = 2 * Z::kPasses;  // per wave
  const segpt_attn_params& p = a.p;
  __shared__ __attribute__((aligned(1024))) char lds[NS * kStageBytes];
  __shared__ __attribute__((aligned(16))) float gsm[D];  // sm_scale*log2e * g_q * g_k, read as float4 slices

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: everything derived from it stays scalar
  const int ln = lane & 31, hh = lane >> 5;
  const int rep = p.H / p.Hkv;
  const int n_qt = (p.Sq + BQ - 1) / BQ;
  const WgCoord wg = decode_wg(blockIdx.x, n_qt, p.B, p.Hkv, rep, wg_pinned_pairs(p.B, p.Hkv, false));
  if (!wg.valid) return;  // idle padding workgroup (whole workgroup, before any barrier)
  const int b = wg.b, g = wg.g, h = wg.g * rep + wg.hh;
  const int q0 = wg.tile * BQ;
  const int qw0 = q0 + wave * 32 * NQB;  // first query of this wave

  int kend = p.Sk;
  if (p.causal) kend = min(p.Sk, q0 + BQ + p.q_start);
  const int n_kt = (kend + BK - 1) / BK;
  const char* kbase = reinterpret_cast<const char*>(a.khat + ((int64_t)b * p.Hkv + g) * p.Sk * D);
  const char* vbase = a.vmix ? reinterpret_cast<const char*>(a.vmix + ((int64_t)b * p.Hkv + g) * p.Sk * D)
                             : reinterpret_cast<const char*>(row_ptr<uint16_t>(p.v, b, g, 0));
  const uint32_t kstep = D * 2, vstep = a.vmix ? (uint32_t)D * 2 : (uint32_t)p.v.stride_s * 2;

  const uint32_t lds0 = lds_addr_of(lds);
  const int2 src = swz_src<D>(lane, wave);
  const uint32_t wave_dst = lds0 + wave * 1024;
  const TileLaneOff<D, BK> full_tile = tile_lane_offsets<D, BK>(kstep, vstep, BK, src.x, src.y);
  auto issue_tile = [&](int jt) {  // tile jt -> stage jt % NS
    const char* ksrc = kbase + (int64_t)jt * BK * kstep;
    const char* vsrc = vbase + (int64_t)jt * BK * vstep;
    const uint32_t dst = wave_dst + (jt % NS) * kStageBytes;
    const int left = p.Sk - jt * BK;
    if (left >= BK) issue_tile_pair<D, BK>(ksrc, vsrc, full_tile, dst);
    else issue_tile_pair<D, BK>(ksrc, vsrc, tile_lane_offsets<D, BK>(kstep, vstep, left, src.x, src.y), dst);
  };

  // ---- start-up.  The workgroup's query rows come in as tiles too (read row-per-lane from global memory, every
  // wave-wide load would touch 32 cache lines for 32 bytes each; staged through LDS by direct loads they are
  // whole lines, and the row-major fragment read of a tile is exactly the B-operand layout): they take the last
  // kQStages stages of the ring, the first kEarlyTiles key tiles (those that fit before them) are requested at the
  // same time, the scale vector behind them: one memory round trip.  The remaining start-up tiles follow once the
  // query rows sit in registers (run() below).
  constexpr int kQStages = BQ / (2 * BK);       // a stage holds two tiles of BK rows
  constexpr ring::Protocol R = ring::forward(NS, kQStages, Z::kPasses);  // the pipeline's numbers: ring_protocol.hpp
  static_assert(ring::well_formed(R) && R.loads_per_tile == kLoadsPerTile && !R.wait_before_loop && R.issue_at_top, "tile pipeline");
  static_assert(R.early_tiles >= ring::kTilesNeededAtLoopStart, "the loop is entered without a further wait");
#pragma unroll
  for (int t = 0; t < R.early_tiles; ++t)
    if (t < n_kt) issue_tile(t);
  {
    const char* qb = reinterpret_cast<const char*>(row_ptr<uint16_t>(p.q, b, h, q0));
#pragma unroll
    for (int i = 0; i < kQStages; ++i)
      issue_tile_pair<D, BK>(qb, qb, rowblock_lane_offsets<D, BK>((uint32_t)p.q.stride_s * 2, 2 * BK * i, p.Sq - q0, src.x, src.y),
                         wave_dst + (R.row_stage_first + i) * kStageBytes);
  }

  // ---- Qhat registers: B operands of S^T, [nb][ks]
  RopeB<KS> rope_b[NQB];
  if (ROPE) {
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) {
      const int64_t pos = (int64_t)(p.rope_q_pos0 + min(qw0 + 32 * nb + ln, p.Sq - 1)) * (D / 2);
      rope_b[nb] = rope_b_load<KS>(p.rope_cos + pos, p.rope_sin + pos, hh);
    }
  }
  float gval = 0.f;
  if (tid < D) gval = gprod_at(p, tid) * p.sm_scale * kLog2e;
  if (tid < D) gsm[tid] = gval;
  wait_vmcnt<0>();
  __syncthreads();
  const bool bounded = !(p.flags & (SEGPT_FLAG_RUNNING_MAX | SEGPT_FLAG_NO_NORM)) && logit_bound<D>(gsm, lane) <= kNoMaxBound;  // wave-uniform
  bf16x8 qreg[NQB][KS];
#pragma unroll
  for (int nb = 0; nb < NQB; ++nb) {
    const int row = min(qw0 + 32 * nb + ln, p.Sq - 1);
    // rows 32*(NQB*wave + nb) .. +31 of the block: which BK-row tile of the staged block, and which 32-row block of it
    const int blk = NQB * wave + nb, tile = blk / kBlocksPerTile, rb = blk % kBlocksPerTile;
    const uint32_t rm = lds0 + (R.row_stage_first + (tile >> 1)) * kStageBytes + (tile & 1) * Z::kTileBytes + swz_off_rm<D>(lane);
    u32x4 raw[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) raw[ks] = __builtin_bit_cast(u32x4, swz_frag_rm<D>(rm, rb, ks));
    float x[KS][8];
    unpack_b_layout<KS>(raw, x);
    if (ROPE) rope_b_apply<KS>(x, rope_b[nb]);
    float ss = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int t = 0; t < 8; ++t) ss += x[ks][t] * x[ks][t];
    ss = half_sum(ss);
    const float alpha = row_normaliser_fast(p, ss, 1.0f / D);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const float4 ga = *reinterpret_cast<const float4*>(gsm + 16 * ks + 8 * hh);
      const float4 gb = *reinterpret_cast<const float4*>(gsm + 16 * ks + 8 * hh + 4);
      u32x4 w;
      w[0] = pack_bf16x2(x[ks][0] * alpha * ga.x, x[ks][1] * alpha * ga.y);
      w[1] = pack_bf16x2(x[ks][2] * alpha * ga.z, x[ks][3] * alpha * ga.w);
      w[2] = pack_bf16x2(x[ks][4] * alpha * gb.x, x[ks][5] * alpha * gb.y);
      w[3] = pack_bf16x2(x[ks][6] * alpha * gb.z, x[ks][7] * alpha * gb.w);
      qreg[nb][ks] = as_bf16x8(w);
    }
  }

  f32x16 oacc[MB][NQB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) oacc[mb][nb] = splat16(0.f);
  // m_ref: the value subtracted from the logits before exp2 (0 on the bounded path); l_run: this lane's
  // share of the row sum (its half of the keys; halves are added in the epilogue)
  float m_ref[NQB], l_run[NQB][2];
  int qlim[NQB];  // last visible key of this lane's query in block nb
#pragma unroll
  for (int nb = 0; nb < NQB; ++nb) {
    m_ref[nb] = bounded ? 0.f : -INFINITY;
    l_run[nb][0] = l_run[nb][1] = 0.f;
    qlim[nb] = p.causal ? min(qw0 + 32 * nb + ln + p.q_start, p.Sk - 1) : p.Sk - 1;
  }

  // 32-key blocks this wave has to visit (causal: up to the block holding its last query's diagonal)
  int n_act = (kend + 31) / 32;
  if (p.causal) n_act = min(n_act, (qw0 + 32 * NQB - 1 + p.q_start) / 32 + 1);

  const uint32_t rm_lane = lds0 + swz_off_rm<D>(lane);
  const uint32_t tr_lane = lds0 + swz_off_tr<D>(lane) + Z::kTileBytes;  // V' tile of a stage
  bf16x8 kf[KS];
  auto request_rowmajor = [&](uint32_t rm, int kb) {  // kb compile-time at every call site
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kf[ks] = swz_frag_rm<D>(rm, kb, ks);
  };
  // One 32-key block.  MASKED / BOUNDED are compile-time so that a whole block is one straight-line
  // scheduling region (a branch in the middle would keep the compiler from interleaving the exp2 work with
  // the neighbouring MFMAs and LDS reads).
  auto step = [&](auto masked_c, auto bounded_c, uint32_t tr, int kb, int jb, uint32_t next_rm, int next_kb) {
    constexpr bool MASKED = decltype(masked_c)::value != 0, BOUNDED = decltype(bounded_c)::value != 0;
    f32x16 s[NQB];
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) s[nb] = splat16(0.f);
    // one query block's chain after the other (not interleaved): the first block's scores are complete while
    // the second block's MFMAs still run, so its exp2 work has something to hide behind
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) s[nb] = mfma32(kf[ks], qreg[nb][ks], s[nb]);
    bf16x8 vT[MB][2];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      vT[mb][0] = swz_frag_tr<D>(tr, mb, 2 * kb);
      vT[mb][1] = swz_frag_tr<D>(tr, mb, 2 * kb + 1);
    }
    if (MASKED) {  // block touches the diagonal or the end of the keys
#pragma unroll
      for (int nb = 0; nb < NQB; ++nb) {
        // register r holds key jb + 4hh + c_r, c_r = 8(r/4) + r%4: masked iff c_r > qlim - jb - 4hh
        const int t = qlim[nb] - jb - 4 * hh;
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (8 * (r >> 2) + (r & 3) > t) s[nb][r] = -INFINITY;
      }
    }
    if (!BOUNDED) {
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
          l_run[nb][0] *= corr;
          l_run[nb][1] *= corr;
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
    request_rowmajor(next_rm, next_kb);  // unconditional: past the last block the fragments are simply unused
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) oacc[mb][nb] = mfma32(vT[mb][s2], pb[s2][nb], oacc[mb][nb]);
  };

  // leading blocks of this wave that need no mask: every key of the block is visible to every query of the
  // wave and lies inside the key range
  int n_full = p.Sk / 32;
  if (p.causal) n_full = min(n_full, (qw0 + p.q_start + 1) / 32);

  // ---- pipeline.  The tile loads that stay in flight across iterations must be the youngest vector-memory
  // operations of the wave (waits are in-order): the prologue's wait left nothing else behind.
  // Protocol: at the top of iteration jt tiles jt and jt+1 have landed and tiles jt+2 .. jt+NS-2 are in
  // flight; the stage of tile jt-1 is free (everyone passed the barrier that ended iteration jt-1), so tile
  // jt+NS-1 is requested right away and has a whole iteration to land; the wait at the bottom leaves the
  // youngest NS-3 tiles in flight, i.e. tile jt+2 is complete before the barrier.
  auto run = [&](auto bounded_c) {
    __syncthreads();  // every wave has its query rows in registers: their stages are free
#pragma unroll
    for (int t = R.early_tiles; t < R.startup_tiles; ++t)
      if (t < n_kt) issue_tile(t);
    if (n_act > 0) request_rowmajor(rm_lane, 0);
    int stage = 0;
    // Two loops instead of a per-block choice inside one: each body is then a single straight-line region
    // with one variant of the block (a join of the two variants costs a copy of every accumulator).
    // Loop A: tiles whose two blocks need no mask.  Loop B: the rest (masking a fully visible block is a no-op).
    const int n_a = n_full / kBlocksPerTile;  // n_full <= n_act, so these tiles are all active
    int jt = 0;
    for (; jt < n_a; ++jt) {
      const int nstage = stage == NS - 1 ? 0 : stage + 1;
      const bool issued = jt + R.issue_ahead < n_kt;
      if (issued) issue_tile(jt + R.issue_ahead);
      const uint32_t rm = rm_lane + stage * kStageBytes, tr = tr_lane + stage * kStageBytes;
      if constexpr (kBlocksPerTile == 2) {
        step(IC<0>{}, bounded_c, tr, 0, BK * jt, rm, 1);
        step(IC<0>{}, bounded_c, tr, 1, BK * jt + 32, rm_lane + nstage * kStageBytes, 0);
      } else {
        step(IC<0>{}, bounded_c, tr, 0, BK * jt, rm_lane + nstage * kStageBytes, 0);
      }
      if (issued) wait_vmcnt<ring::loads_kept_after_iteration(R, true)>(); else wait_vmcnt<ring::loads_kept_after_iteration(R, false)>();
      __syncthreads();
      stage = nstage;
    }
    for (; jt < n_kt; ++jt) {
      const int nstage = stage == NS - 1 ? 0 : stage + 1;
      const bool issued = jt + R.issue_ahead < n_kt;
      if (issued) issue_tile(jt + R.issue_ahead);
      const uint32_t rm = rm_lane + stage * kStageBytes, tr = tr_lane + stage * kStageBytes;
      if constexpr (kBlocksPerTile == 2) {
        if (2 * jt < n_act) step(IC<1>{}, bounded_c, tr, 0, BK * jt, rm, 1);
        if (2 * jt + 1 < n_act) step(IC<1>{}, bounded_c, tr, 1, BK * jt + 32, rm_lane + nstage * kStageBytes, 0);
      } else {
        if (jt < n_act) step(IC<1>{}, bounded_c, tr, 0, BK * jt, rm_lane + nstage * kStageBytes, 0);
      }
      if (issued) wait_vmcnt<ring::loads_kept_after_iteration(R, true)>(); else wait_vmcnt<ring::loads_kept_after_iteration(R, false)>();
      __syncthreads();
      stage = nstage;
    }
  };
  if (bounded) run(IC<1>{}); else run(IC<0>{});

  // ---- epilogue: normalise, gate, store y (bf16) and lse (fp32, natural log)
#pragma unroll
  for (int nb = 0; nb < NQB; ++nb) {
    const int row = qw0 + 32 * nb + ln;
    const bool live = row < p.Sq;
    const float l = half_sum(l_run[nb][0] + l_run[nb][1]);
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
      float val[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) val[r] = oacc[mb][nb][r] * f;
      store_ct_block(op, mb, hh, live, val);
    }
  }
}

template <int D, bool WIDE>
int launch_fwd_t(const KArgs& a, hipStream_t st) {
  const segpt_attn_params& p = a.p;
  const int n_qt = (p.Sq + FwdShape<D, WIDE>::kBQ - 1) / FwdShape<D, WIDE>::kBQ;
  const dim3 grid((unsigned)wg_grid(n_qt, p.B, p.Hkv, p.H / p.Hkv, wg_pinned_pairs(p.B, p.Hkv, false)));
  if (p.rope_cos) hipLaunchKernelGGL((fwd_bf16_kernel<D, WIDE, true>), grid, dim3(kThreadsM), 0, st, a);
  else hipLaunchKernelGGL((fwd_bf16_kernel<D, WIDE, false>), grid, dim3(kThreadsM), 0, st, a);
  return (int)hipGetLastError();
}

}  // namespace

int launch_fwd_bf16(const KArgs& a, hipStream_t st) {
  if (a.p.D == 64) return a.p.Sk > 2048 ? launch_fwd_t<64, true>(a, st) : launch_fwd_t<64, false>(a, st);
  if (a.p.D == 128) return launch_fwd_t<128, true>(a, st);
  return (int)hipErrorInvalidValue;
}

}  // namespace segpt
