// bf16 backward: two deterministic MFMA kernels (no floating-point atomics).
//
// Operands are normalised tensors held in the workspace (bf16):
//   Khat = b_j k_j and V' = c1 v + c2 v_first, written by the key/value pre-pass (pre_post.hip);
//   Qhat = sm_scale*log2e * a_i q_i * g_q*g_k and the two row statistics -lse2, -delta (which also carry a positive
//   gate factor), written by the dQ kernel for the dK/dV kernel that runs after it.
//
//  bwd_dq    query-stationary, same orientation as the forward (a lane owns one query column):
//              S^T  = Khat . Qhat^T - lse2        dP^T = V' . dO^T - delta     (A from LDS row-major,
//              dS^T = exp2(S^T) * dP^T            T^T += Khat^T . dS^T          B = registers; the row
//            statistics enter as the MFMA's C operand, so no subtraction is spent on them)
//            epilogue: through the q normaliser, dq (bf16), and this workgroup's partial of the
//            combined scale gradient dg[d] = sum_i sm_scale * (a_i q_id) * T_id.
//  bwd_dkdv  key-stationary (a lane owns one key column); a wave owns 32 keys of one kv head and walks
//            the query tiles of every query head of the group (dK/dV of a GQA group are summed in
//            registers):
//              S  = Qhat . Khat^T - lse2          dP = dO . V'^T - delta
//              dV'^T += dO^T . P                  dKhat^T += Qhat^T . dS        (A = transposing LDS read)
//            epilogue: through the k normaliser, dk, dv (= c1 dV'), dv_first (= c2 dV'), (dc1, dc2) partials.
//
// One workgroup = 4 waves (one per SIMD); several workgroups share a CU so that the softmax-like VALU
// phase of one overlaps the MFMA phase of another.  Streamed tiles (64 rows) are double-buffered in LDS.
#include "mfma_common.hpp"
#include "ring_protocol.hpp"

namespace segpt {
namespace {

constexpr int kBwdRows = 4 * 32;  // rows (queries for dQ, keys for dK/dV) owned by a workgroup

// The dK/dV launch pins (batch, kv head) pairs to XCDs only when ALL of them can be pinned: with a spread remainder it
// was measured 13 % slower at B*Hkv = 12, S = 8192 (where forward and dQ gain 2-4 % from pinning 8 of the 12).
__host__ __device__ inline int dkdv_pinned(const segpt_attn_params& p) { return wg_pinned_pairs(p.B, p.Hkv, true); }

constexpr float kGateFactorFloor = 1e-30f;  // a smaller gate factor switches its row off in the dK/dV kernel

constexpr int kStages = 4;  // LDS ring of streamed stages (two tiles each): tile t lives in stage t % 4

// ============================================================================================ dQ
// Also the producer of the per-query-row quantities the dK/dV kernel streams afterwards: Qhat, -delta,
// -lse*log2e and (with a gate) dgate; the gate-scaled copy of dO only when the gate scale is not positive.
//
// Software pipeline over 32-key blocks n (two per staged tile), one barrier per tile:
//   B(n)  S^T, dP^T MFMAs from the row-major fragments requested one block earlier
//   C(n)  request the transposed Khat fragments of block n
//   D(n)  dS^T = exp2(S^T) * dP^T, pack to bf16
//   A(n+1) request the row-major fragments of block n+1 (possibly the next tile, already in LDS)
//   E(n)  T^T += Khat^T dS^T MFMAs
// Tiles travel global->LDS directly (no registers), three tiles ahead of their use.
// ROPE (rope tables given) is a compile-time switch so that the table rows are ordinary, unconditional loads which
// travel with the start-up tiles (prologue) and with the first stores (epilogue) instead of costing a memory round
// trip of their own behind a branch.
template <int D, bool ROPE>
__global__ __launch_bounds__(kThreadsM, D == 64 ? 2 : 1) void bwd_dq_bf16_kernel(KArgs a) {
  using Z = Swz<D>;
  constexpr int BQ = kBwdRows;
  constexpr int KS = D / 16;
  constexpr int MB = D / 32;
  constexpr int kStageBytes = 2 * Z::kTileBytes;
  // the pipeline's numbers: ring_protocol.hpp
  constexpr ring::Protocol R = ROPE ? ring::dq_rope(Z::kPasses) : ring::dq(Z::kPasses);
  static_assert(ring::well_formed(R) && R.stages == kStages && !R.issue_at_top, "tile pipeline");
  static_assert(ROPE ? (R.pre_row_stages == 4 && R.row_stages == 1 && R.early_tiles == R.startup_tiles && !R.wait_before_loop && R.epilogue_row_stages == 2)
                     : (R.pre_row_stages == 0 && R.row_stages == 3 && R.wait_before_loop && R.epilogue_row_stages == 0), "tile pipeline");
  const segpt_attn_params& p = a.p;
  __shared__ __attribute__((aligned(1024))) char lds[kStages * kStageBytes];
  __shared__ __attribute__((aligned(16))) float gsm[D];       // g_q * g_k, read as float4 slices
  constexpr int kRedStride = D + 4;                 // floats per row of the dg staging area (16-byte aligned rows)
  constexpr int kColGroups = D / 4;                 // a thread sums 4 adjacent columns ...
  constexpr int kRowGroups = kThreadsM / kColGroups;  // ... over one of these groups of rows
  constexpr int kRowsPerGroup = BQ / kRowGroups;
  __shared__ __attribute__((aligned(16))) float red4[kRowGroups * D];  // per-row-group column sums of the dg partial
  static_assert(kStages * kStageBytes >= BQ * kRedStride * 4, "LDS reuse for the dg partial");

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: everything derived from it stays scalar
  const int ln = lane & 31, hh = lane >> 5;
  const int rep = p.H / p.Hkv;
  const int n_qt = (p.Sq + BQ - 1) / BQ;
  const WgCoord wg = decode_wg(blockIdx.x, n_qt, p.B, p.Hkv, rep, wg_pinned_pairs(p.B, p.Hkv, false));
  if (!wg.valid) {  // idle padding workgroup: its row of the scale-gradient partials must still read as zero
    if (tid < D) a.dg_part[(int64_t)blockIdx.x * D + tid] = 0.f;
    return;
  }
  const int b = wg.b, g = wg.g, h = wg.g * rep + wg.hh;
  const int q0 = wg.tile * BQ;
  const int qw0 = q0 + wave * 32;
  const int row = qw0 + ln;
  const bool live = row < p.Sq;
  const int row_c = live ? row : p.Sq - 1;  // padding lanes recompute the last row and store nothing
  const int64_t ridx = ((int64_t)b * p.H + h) * p.Sq + row_c;

  int kend = p.Sk;
  if (p.causal) kend = min(p.Sk, q0 + BQ + p.q_start);
  const int n_kt = (kend + kBK - 1) / kBK;
  const char* kbase = reinterpret_cast<const char*>(a.khat + ((int64_t)b * p.Hkv + g) * p.Sk * D);
  const char* vbase = a.vmix ? reinterpret_cast<const char*>(a.vmix + ((int64_t)b * p.Hkv + g) * p.Sk * D)
                             : reinterpret_cast<const char*>(row_ptr<uint16_t>(p.v, b, g, 0));
  const uint32_t kstep = D * 2, vstep = a.vmix ? (uint32_t)D * 2 : (uint32_t)p.v.stride_s * 2;

  const uint32_t lds0 = lds_addr_of(lds);
  const int2 src = swz_src<D>(lane, wave);
  const uint32_t wave_dst = lds0 + wave * 1024;
  const TileLaneOff<D> full_tile = tile_lane_offsets<D>(kstep, vstep, kBK, src.x, src.y);
  auto issue_tile = [&](int jt) {  // tile jt -> stage jt % kStages
    const char* ksrc = kbase + (int64_t)jt * kBK * kstep;
    const char* vsrc = vbase + (int64_t)jt * kBK * vstep;
    const uint32_t dst = wave_dst + (jt % kStages) * kStageBytes;
    const int left = p.Sk - jt * kBK;
    if (left >= kBK) issue_tile_pair<D>(ksrc, vsrc, full_tile, dst);
    else issue_tile_pair<D>(ksrc, vsrc, tile_lane_offsets<D>(kstep, vstep, left, src.x, src.y), dst);
  };

  // ---- The workgroup's 128 query / dO / output rows come in as tiles too: read row-per-lane from global memory
  // every wave-wide load would touch 32 cache lines for 32 bytes each and the prologue would spend its time in
  // the address path of the vector memory unit; staged through LDS by direct loads they are whole lines, and the
  // row-major fragment read of a tile is exactly the B-operand layout (lane = row, 8 entries of k-step ks).
  // Without a rotary embedding: stage 0 takes key tile 0; stages 1..3 hold the q, dO and o blocks until the rows sit
  // in registers, then key tiles 1 and 2 are requested into stages 1 and 2 and the ring turns as usual.  All of it
  // is in flight at once, with the row's lse, the gate logit and the scale vector behind it: one memory round trip
  // (vector-memory waits are in order, and the compiler's own count does not see the direct loads, so its first
  // wait covers them).
  // With a rotary embedding the table rows of the 128 positions (D/2 floats: as long as a tensor row) are two more
  // blocks, for the same reason, and the start-up has two phases: q, cos, sin, dO in stages 0..3; once they are in
  // registers, the o block in stage 3 and key tiles 0..2 in stages 0..2, which arrive while Qhat is computed.
  // The prologue's results (Qhat, gated dO, -delta, -lse2, dgate) are stored from the epilogue, so no store is in
  // flight while the loop counts its tile loads.
  constexpr int kRowStage = R.row_stage_first;
  constexpr int kQStage = ROPE ? 0 : kRowStage, kCosStage = 1, kSinStage = 2;
  constexpr int kDoStage = ROPE ? 3 : kRowStage + 1, kOStage = ROPE ? kRowStage : kRowStage + 2;
  static_assert(!ROPE || kOStage == 3, "first phase: q, cos, sin, dO; second phase: tiles 0..2, o");
  const int rows_left = p.Sq - q0;
  const char* qb = reinterpret_cast<const char*>(row_ptr<uint16_t>(p.q, b, h, q0));
  const char* db = reinterpret_cast<const char*>(row_ptr<uint16_t>(p.d_o, b, h, q0));
  const char* yb = reinterpret_cast<const char*>(row_ptr<uint16_t>(p.o, b, h, q0));
  const int64_t rope_row0 = ROPE ? (int64_t)(p.rope_q_pos0 + q0) * (D / 2) : 0;  // the tables' row of query q0
  auto issue_rope_rows = [&](int cos_stage, int sin_stage) {  // 128 table rows each, laid out like tensor rows
    const TileLaneOff<D> o = rowblock_lane_offsets<D>(D * 2, 0, rows_left, src.x, src.y);
    const char* cb = reinterpret_cast<const char*>(p.rope_cos + rope_row0);
    const char* sb = reinterpret_cast<const char*>(p.rope_sin + rope_row0);
    issue_tile_pair<D>(cb, cb, o, wave_dst + cos_stage * kStageBytes);
    issue_tile_pair<D>(sb, sb, o, wave_dst + sin_stage * kStageBytes);
  };
  if constexpr (ROPE) {
    issue_tile_pair<D>(qb, qb, rowblock_lane_offsets<D>((uint32_t)p.q.stride_s * 2, 0, rows_left, src.x, src.y), wave_dst + kQStage * kStageBytes);
    issue_rope_rows(kCosStage, kSinStage);
    issue_tile_pair<D>(db, db, rowblock_lane_offsets<D>((uint32_t)p.d_o.stride_s * 2, 0, rows_left, src.x, src.y), wave_dst + kDoStage * kStageBytes);
  } else {
#pragma unroll
    for (int t = 0; t < R.early_tiles; ++t)
      if (t < n_kt) issue_tile(t);
    issue_tile_pair<D>(qb, qb, rowblock_lane_offsets<D>((uint32_t)p.q.stride_s * 2, 0, rows_left, src.x, src.y), wave_dst + kQStage * kStageBytes);
    issue_tile_pair<D>(db, db, rowblock_lane_offsets<D>((uint32_t)p.d_o.stride_s * 2, 0, rows_left, src.x, src.y), wave_dst + kDoStage * kStageBytes);
    issue_tile_pair<D>(yb, yb, rowblock_lane_offsets<D>((uint32_t)p.o.stride_s * 2, 0, rows_left, src.x, src.y), wave_dst + kOStage * kStageBytes);
  }
  const float lse_row = p.lse[ridx];
  // the conditional reads last: the compiler waits for every outstanding load where their branches join
  float gate_z = 0.f;
  if (p.gate.ptr)
    gate_z = bf16_to_f32(reinterpret_cast<const uint16_t*>(p.gate.ptr)[(int64_t)b * p.gate.stride_b + (int64_t)row_c * p.gate.stride_s + (int64_t)h * p.gate.stride_h]);
  float gval = 0.f;
  if (tid < D) gval = gprod_at(p, tid);
  if (tid < D) gsm[tid] = gval;
  wait_vmcnt<0>();
  __syncthreads();
  // rows 32*wave .. 32*wave+31 of the block: half (wave >> 1) of each stage, row block (wave & 1) of that tile
  u32x4 qraw[KS], dyraw[KS], yraw[KS];
  u32x2 qct[MB][4];  // the query row once more, in the layout of the epilogue's C tiles (packed pairs)
  RopeB<KS> rope_b;
  const uint32_t row_half = (wave >> 1) * Z::kTileBytes, row_rb = wave & 1;
  const uint32_t row_rm = lds0 + row_half + swz_off_rm<D>(lane);
  const uint32_t row16 = lds0 + row_half + swz_off_row16<D>(lane) + row_rb * 32 * Z::kRB;  // chunk 0 of the lane's row
  {
    const uint32_t ct = lds0 + kQStage * kStageBytes + row_half + swz_off_ct<D>(lane) + row_rb * 32 * Z::kRB;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qraw[ks] = __builtin_bit_cast(u32x4, swz_frag_rm<D>(row_rm + kQStage * kStageBytes, row_rb, ks));
      dyraw[ks] = __builtin_bit_cast(u32x4, swz_frag_rm<D>(row_rm + kDoStage * kStageBytes, row_rb, ks));
      if constexpr (!ROPE) yraw[ks] = __builtin_bit_cast(u32x4, swz_frag_rm<D>(row_rm + kOStage * kStageBytes, row_rb, ks));
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int c = 0; c < 4; ++c) qct[mb][c] = lds_read8(ct ^ (uint32_t)((4 * mb + c) << 4));
    if constexpr (ROPE) rope_b = rope_b_from_lds<KS>(row16 + kCosStage * kStageBytes, row16 + kSinStage * kStageBytes, hh);
  }
  __syncthreads();  // the borrowed stages are free again
  if constexpr (ROPE) {
    issue_tile_pair<D>(yb, yb, rowblock_lane_offsets<D>((uint32_t)p.o.stride_s * 2, 0, rows_left, src.x, src.y), wave_dst + kOStage * kStageBytes);
#pragma unroll
    for (int t = 0; t < R.early_tiles; ++t)
      if (t < n_kt) issue_tile(t);
  } else {
#pragma unroll
    for (int t = R.early_tiles; t < R.startup_tiles; ++t)
      if (t < n_kt) issue_tile(t);
  }

  // ---- query-row prologue: alpha, Qhat, delta, gate; B operands stay in registers
  bf16x8 qreg[KS], doreg[KS];
  float alpha, delta, dgate_row = 0.f, gfac = 1.f, gate_sg = 0.f;
  auto row_dot = [&]() {  // delta = rowsum(dY * Y): the o block is the last thing the second phase waits for
    float dl = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int i = 0; i < 4; ++i) dl += bf16lo(yraw[ks][i]) * bf16lo(dyraw[ks][i]) + bf16hi(yraw[ks][i]) * bf16hi(dyraw[ks][i]);
    delta = half_sum(dl);
    if (p.gate.ptr) dgate_row = (1.0f - gate_sg) * delta;
  };
  if (p.gate.ptr) {
    gate_sg = 1.0f / (1.0f + __expf(-gate_z));
    gfac = p.gate_scale * gate_sg;
  }
  if constexpr (!ROPE) row_dot();
  {
    float qx[KS][8];
    unpack_b_layout<KS>(qraw, qx);
    if (ROPE) rope_b_apply<KS>(qx, rope_b);
    float ss = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int t = 0; t < 8; ++t) ss += qx[ks][t] * qx[ks][t];
    ss = half_sum(ss);
    alpha = row_normaliser_fast(p, ss, 1.0f / D);
    const float f = alpha * p.sm_scale * kLog2e;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const float4 ga = *reinterpret_cast<const float4*>(gsm + 16 * ks + 8 * hh);
      const float4 gb = *reinterpret_cast<const float4*>(gsm + 16 * ks + 8 * hh + 4);
      u32x4 w;
      w[0] = pack_bf16x2(qx[ks][0] * f * ga.x, qx[ks][1] * f * ga.y);
      w[1] = pack_bf16x2(qx[ks][2] * f * ga.z, qx[ks][3] * f * ga.w);
      w[2] = pack_bf16x2(qx[ks][4] * f * gb.x, qx[ks][5] * f * gb.y);
      w[3] = pack_bf16x2(qx[ks][6] * f * gb.z, qx[ks][7] * f * gb.w);
      qreg[ks] = as_bf16x8(w);
      doreg[ks] = as_bf16x8(p.gate.ptr ? scale8(dyraw[ks], gfac) : dyraw[ks]);
    }
  }
  if constexpr (ROPE) {
    // second phase landed (tile 2 with it: no late tile, no further wait before the loop); the o rows go to registers
    // and one more barrier frees their stage, which iteration 0 refills
    wait_vmcnt<0>();
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) yraw[ks] = __builtin_bit_cast(u32x4, swz_frag_rm<D>(row_rm + kOStage * kStageBytes, row_rb, ks));
    row_dot();
    __syncthreads();
  }
  // row statistics as MFMA C operands (every register of a lane belongs to the lane's query); the dK/dV
  // kernel reads the same two numbers per row from the workspace
  const float nlse2 = -lse_row * kLog2e;
  const f32x16 c_lse = splat16(nlse2);
  const f32x16 c_del = splat16(-delta);

  f32x16 acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) acc[mb] = splat16(0.f);

  // blocks this wave has to visit (causal: up to the block holding its last query's diagonal)
  int n_act = (kend + 31) / 32;
  if (p.causal) n_act = min(n_act, (qw0 + 31 + p.q_start) / 32 + 1);
  const int qlim = p.causal ? min(row + p.q_start, p.Sk - 1) : p.Sk - 1;  // last visible key of this lane's query

  const uint32_t rm_lane = lds0 + swz_off_rm<D>(lane);
  const uint32_t tr_lane = lds0 + swz_off_tr<D>(lane);
  bf16x8 kf[KS], vf[KS];
  auto request_rowmajor = [&](uint32_t rm, int kb) {  // kb compile-time at every call site
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kf[ks] = swz_frag_rm<D>(rm, kb, ks);
      vf[ks] = swz_frag_rm<D>(rm + Z::kTileBytes, kb, ks);
    }
  };
  // one 32-key block: tr = lane address inside the block's stage; `more`: a block follows, its row-major
  // fragments start at next_rm
  // MASKED is compile-time so that a whole block is one straight-line scheduling region
  auto step = [&](auto masked_c, uint32_t tr, int kb, int jb, uint32_t next_rm, int next_kb) {
    constexpr bool MASKED = decltype(masked_c)::value != 0;
    // head_dim 128 runs one wave per SIMD with all 256 ordinary registers in use: left to itself the compiler requests
    // each LDS fragment one MFMA ahead of its use and the wave stalls on LDS latency before most MFMAs.  Asking for
    // the block as 24 groups of (1 MFMA, 2 LDS reads, 2 vector instructions) keeps two requests ahead: -6 % on this
    // kernel (neighbouring group shapes are 2-10 % slower; at head_dim 64, two waves per SIMD, none changes anything).
    if constexpr (D == 128) {
#pragma unroll
      for (int i = 0; i < 3 * KS; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // LDS read
        __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);  // VALU
      }
    }
    f32x16 s = c_lse, dpv = c_del;
    // the S chain first, then the dP chain: exp2 of the finished scores runs behind the dP MFMAs
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) s = mfma32(kf[ks], qreg[ks], s);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) dpv = mfma32(vf[ks], doreg[ks], dpv);
    bf16x8 kT[MB][2];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      kT[mb][0] = swz_frag_tr<D>(tr, mb, 2 * kb);
      kT[mb][1] = swz_frag_tr<D>(tr, mb, 2 * kb + 1);
    }
    if (MASKED) {  // block touches the diagonal or the end of the keys
      // register r holds key jb + 4hh + c_r, c_r = 8(r/4) + r%4: masked iff c_r > qlim - jb - 4hh
      const int t = qlim - jb - 4 * hh;
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if (8 * (r >> 2) + (r & 3) > t) s[r] = -INFINITY;
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = fast_exp2(s[r]) * dpv[r];
    const bf16x8 ds0 = pack_c_half(s, 0), ds1 = pack_c_half(s, 1);
    request_rowmajor(next_rm, next_kb);  // unconditional: past the last block the fragments are simply unused
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      acc[mb] = mfma32(kT[mb][0], ds0, acc[mb]);
      acc[mb] = mfma32(kT[mb][1], ds1, acc[mb]);
    }
  };

  // ---- pipeline start-up.  Every iteration of the loop starts with its own tile AND the next one landed (the
  // second block of a tile already requests the next tile's fragments) and at most one more in flight, so tile 1,
  // requested after the row blocks had left its stage, must be complete here; the row prologue above ran in
  // between, so this wait is short.  Tile 2 stays in flight.
  if constexpr (R.wait_before_loop) {
    if (n_kt >= R.startup_tiles) wait_vmcnt<ring::loads_kept_before_loop(R, R.startup_tiles)>(); else wait_vmcnt<0>();
    __syncthreads();
  }
  if (n_act > 0) request_rowmajor(rm_lane, 0);
  // leading blocks of this wave that need no mask (every key visible to every query of the wave, inside Sk)
  int n_full = p.Sk / 32;
  if (p.causal) n_full = min(n_full, (qw0 + p.q_start + 1) / 32);
  // Loop A: tiles whose two blocks need no mask; loop B: the rest (masking a fully visible block is a no-op).
  // Two loops, so that each body holds one variant of the block and the accumulators never meet at a join.
  const int n_a = n_full / 2;  // n_full <= n_act
  int stage = 0, jt = 0;
  for (; jt < n_a; ++jt) {
    const int nstage = stage == kStages - 1 ? 0 : stage + 1;
    const uint32_t rm = rm_lane + stage * kStageBytes, tr = tr_lane + stage * kStageBytes;
    step(IC<0>{}, tr, 0, 64 * jt, rm, 1);
    step(IC<0>{}, tr, 1, 64 * jt + 32, rm_lane + nstage * kStageBytes, 0);
    // stage (jt+3) % 4 == (jt-1) % 4 was last read in the previous iteration: refill it, then make sure
    // this wave's part of tile jt+2 (needed from the next iteration's prefetch on) has landed
    if (jt + R.issue_ahead < n_kt) { issue_tile(jt + R.issue_ahead); wait_vmcnt<ring::loads_kept_after_iteration(R, true)>(); } else wait_vmcnt<ring::loads_kept_after_iteration(R, false)>();
    __syncthreads();
    stage = nstage;
  }
  for (; jt < n_kt; ++jt) {
    const int nstage = stage == kStages - 1 ? 0 : stage + 1;
    const uint32_t rm = rm_lane + stage * kStageBytes, tr = tr_lane + stage * kStageBytes;
    if (2 * jt < n_act) step(IC<1>{}, tr, 0, 64 * jt, rm, 1);
    if (2 * jt + 1 < n_act) step(IC<1>{}, tr, 1, 64 * jt + 32, rm_lane + nstage * kStageBytes, 0);
    if (jt + R.issue_ahead < n_kt) { issue_tile(jt + R.issue_ahead); wait_vmcnt<ring::loads_kept_after_iteration(R, true)>(); } else wait_vmcnt<ring::loads_kept_after_iteration(R, false)>();
    __syncthreads();
    stage = nstage;
  }

  // ---- epilogue.  First what the dK/dV kernel reads of this row: Qhat, -delta, -lse2 (and dgate).  A gate factor
  // f > 0 reaches that kernel through the two statistics and it streams the caller's dO as it is: with
  // P' = f P = exp2(S - lse2 + log2 f) it holds dV' = P'^T dO and dS = P (f dP - delta) = P' (dP - delta / f).  A
  // factor that underflowed switches the row off (P' = 0).  Only a gate scale <= 0 needs the gated copy of dO.
  // With a rotary embedding the table rows come in once more, into the idle ring (every wave has passed the last
  // iteration's barrier), now for the accumulators' layout; the second barrier keeps the scale-gradient staging
  // below, which reuses the ring, behind every wave's reads.
  RopeCt<MB> rope_ct;
  if constexpr (ROPE) {
    issue_rope_rows(0, 1);
    wait_vmcnt<0>();
    __syncthreads();
    rope_ct = rope_ct_from_lds<MB>(row16, row16 + kStageBytes, hh);
    __syncthreads();
  }
  if (live) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      *reinterpret_cast<bf16x8*>(a.qhat + ridx * D + 16 * ks + 8 * hh) = qreg[ks];
      if (a.do_eff) *reinterpret_cast<bf16x8*>(reinterpret_cast<uint16_t*>(a.do_eff) + ridx * D + 16 * ks + 8 * hh) = doreg[ks];
    }
    if (hh == 0) {
      float stat_d = -delta, stat_l = nlse2;
      if (p.gate.ptr && !a.do_eff) {
        const bool on = gfac > kGateFactorFloor;
        stat_l = on ? nlse2 + __log2f(gfac) : -INFINITY;
        stat_d = on ? -delta / gfac : 0.f;
      }
      a.delta[ridx] = stat_d;
      a.nlse2[ridx] = stat_l;
      if (p.gate.ptr)
        reinterpret_cast<uint16_t*>(p.dgate.ptr)[(int64_t)b * p.dgate.stride_b + (int64_t)row * p.dgate.stride_s + (int64_t)h * p.dgate.stride_h] = f32_to_bf16(dgate_row);
    }
  }
  // acc = T^T: lane = query, registers = head-dim entries.
  float dot = 0.f;
  float* red = reinterpret_cast<float*>(lds);
  // q in the C-tile layout (rotated like the operand was), then dq = a (u - (a^2/D)(u.q) q) in the rotated frame
  // and back through the transpose of the rotation
  float qv[MB][16];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) unpack_ct_block(qct[mb], qv[mb]);
  const float aq = live ? alpha : 0.f;  // padding rows add nothing to the scale gradient
  if (ROPE) rope_ct_apply<MB, false>(qv, rope_ct);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int d0 = 32 * mb + 8 * c + 4 * hh;
      const float4 g4 = *reinterpret_cast<const float4*>(gsm + d0);
      const float gv[4] = {g4.x, g4.y, g4.z, g4.w};
      float dgc[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 4 * c + i;
        const float t = acc[mb][r] * p.sm_scale;                 // sm_scale * T
        dgc[i] = t * aq * qv[mb][r];                             // dg contribution of this row
        acc[mb][r] = t * gv[i];                                  // u = dL/d(a q)
        dot += acc[mb][r] * qv[mb][r];
      }
      *reinterpret_cast<float4*>(red + (wave * 32 + ln) * kRedStride + d0) = make_float4(dgc[0], dgc[1], dgc[2], dgc[3]);
    }
  }
  dot = half_sum(dot);
  const float a3 = norm_grad_coef(p, alpha, 1.0f / D) * dot;
  uint16_t* op = row_ptr_mut<uint16_t>(p.dq, b, h, row_c);
  float val[MB][16];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) val[mb][r] = alpha * acc[mb][r] - a3 * qv[mb][r];
  if (ROPE) rope_ct_apply<MB, true>(val, rope_ct);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) store_ct_block(op, mb, hh, live, val[mb]);
  // workgroup partial of dg: column sums over the 128 (wave, lane%32) rows, in two levels so that all
  // 256 threads share the LDS reads (fixed order: deterministic)
  __syncthreads();
  {
    const int cg = tid % kColGroups, rg = tid / kColGroups;
    float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int x = 0; x < kRowsPerGroup; ++x) {
      const float4 v = *reinterpret_cast<const float4*>(red + (rg * kRowsPerGroup + x) * kRedStride + 4 * cg);
      t.x += v.x; t.y += v.y; t.z += v.z; t.w += v.w;
    }
    *reinterpret_cast<float4*>(red4 + rg * D + 4 * cg) = t;
  }
  __syncthreads();
  if (tid < D) {
    float t = 0.f;
#pragma unroll
    for (int x = 0; x < kRowGroups; ++x) t += red4[x * D + tid];
    a.dg_part[(int64_t)blockIdx.x * D + tid] = t;
  }
}

// ============================================================================================ dK, dV
// Same pipeline with the roles swapped: the streamed tiles are Qhat / dO (64 queries of one head), the
// blocks are 32 queries, and B(n) starts from the two row statistics of the block, read from LDS
// straight into the accumulators of S and dP.
template <int D, bool ROPE>
__global__ __launch_bounds__(kThreadsM, D == 64 ? 2 : 1) void bwd_dkdv_bf16_kernel(KArgs a) {
  using Z = Swz<D>;
  constexpr int BKV = kBwdRows;
  constexpr int KS = D / 16;
  constexpr int MB = D / 32;
  constexpr int kStageBytes = 2 * Z::kTileBytes;
  constexpr ring::Protocol R = ring::dkdv(Z::kPasses);  // the pipeline's numbers: ring_protocol.hpp
  static_assert(ring::well_formed(R) && R.stages == kStages && R.row_stages == 2 && !R.wait_before_loop && !R.issue_at_top, "tile pipeline");
  static_assert(R.early_tiles >= ring::kTilesNeededAtLoopStart, "the loop is entered without a further wait");
  static_assert(R.loads_per_tile == 2 * Z::kPasses + 1, "per wave: the two tiles plus one row-statistics load");
  const segpt_attn_params& p = a.p;
  __shared__ __attribute__((aligned(1024))) char lds[kStages * kStageBytes];
  __shared__ __attribute__((aligned(256))) float ldl[kStages * 128];  // per stage: [0,64) -lse2, [64,128) -delta
  __shared__ float red[8];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: everything derived from it stays scalar
  const int ln = lane & 31, hh = lane >> 5;
  const int rep = p.H / p.Hkv;
  const int n_kvt = (p.Sk + BKV - 1) / BKV;
  // Workgroup 0 is an extra one: dispatched first, it only folds the dQ kernel's per-workgroup partials of the
  // scale-vector gradient (complete: that kernel ran before this one on the stream) while the others compute.
  if (blockIdx.x == 0) {
    float* red = reinterpret_cast<float*>(lds);
    reduce_scale_grad<kThreadsM>(a, tid, red, red + kThreadsM);
    return;
  }
  const int bid = blockIdx.x - 1;  // still a fixed rotation of the hardware's round-robin over the XCDs
  WgCoord wg = decode_wg(bid, n_kvt, p.B, p.Hkv, 1, dkdv_pinned(p));
  if (!wg.valid) {  // idle padding workgroup: its (dc1, dc2) partial must still read as zero
    if (tid < 2) a.dcoef_part[(int64_t)bid * 2 + tid] = 0.f;
    return;
  }
  wg.tile = n_kvt - 1 - wg.tile;  // early key tiles see the most queries: issue them first
  const int b = wg.b, g = wg.g;
  const int k0 = wg.tile * BKV;
  const int kw0 = k0 + wave * 32;
  const int key = kw0 + ln;
  const int key_c = min(key, p.Sk - 1);

  const int n_qt = (p.Sq + kBK - 1) / kBK;
  int qt_start = 0;
  if (p.causal) qt_start = min(max(0, k0 - p.q_start) / kBK, n_qt);
  const int n_vis = n_qt - qt_start;  // visible query tiles per head
  const int n_it = n_vis * rep;       // streamed tiles in total

  // ---- staging of one (head, query tile): Qhat and dO tiles plus the two row statistics, all by direct
  // global->LDS loads.  Every wave issues the same number of loads (waves 2/3 repeat the statistics load
  // of waves 0/1) so that one immediate vmcnt fits all.
  const uint32_t lds0 = lds_addr_of(lds), ldl0 = lds_addr_of(ldl);
  const int2 src = swz_src<D>(lane, wave);
  const bool do_contig = a.do_eff != nullptr;
  const float* const stat_arr = (wave & 1) ? a.delta : a.nlse2;
  const uint32_t dstep = do_contig ? (uint32_t)D * 2 : (uint32_t)p.d_o.stride_s * 2;
  const TileLaneOff<D> full_tile = tile_lane_offsets<D>(D * 2, dstep, kBK, src.x, src.y);
  // The stream of (head, query tile) pairs is walked by running pointers kept beside the compute loop's own
  // counters (three tiles ahead of it): per tile a few scalar additions, per head one address computation.
  const char* q_it = nullptr;
  const char* d_it = nullptr;
  const float* s_it = nullptr;
  int left_it = 0, iss_h = 0, iss_t = 0, iss_stage = 0;
  auto set_head = [&](int hq) {
    const int h = g * rep + hq, i0 = qt_start * kBK;
    const int64_t row = ((int64_t)b * p.H + h) * p.Sq + i0;
    q_it = reinterpret_cast<const char*>(a.qhat + row * D);
    d_it = do_contig ? reinterpret_cast<const char*>(reinterpret_cast<const uint16_t*>(a.do_eff) + row * D)
                     : reinterpret_cast<const char*>(row_ptr<uint16_t>(p.d_o, b, h, i0));
    s_it = stat_arr + row;
    left_it = p.Sq - i0;
  };
  if (n_it > 0) set_head(0);
  const uint32_t lane4 = lane * 4;
  auto issue_next = [&]() {
    const uint32_t dst = lds0 + iss_stage * kStageBytes + wave * 1024;
    const uint32_t sdst = ldl0 + (iss_stage * 128 + (wave & 1) * 64) * 4;
    if (left_it >= kBK) {
      issue_tile_pair<D>(q_it, d_it, full_tile, dst);
      gload_lds4_so(s_it, lane4, sdst);
    } else {
      issue_tile_pair<D>(q_it, d_it, tile_lane_offsets<D>(D * 2, dstep, left_it, src.x, src.y), dst);
      gload_lds4_so(s_it, (uint32_t)min(lane, left_it - 1) * 4, sdst);
    }
    iss_stage = iss_stage == kStages - 1 ? 0 : iss_stage + 1;
    if (++iss_t == n_vis) {
      iss_t = 0;
      if (++iss_h < rep) set_head(iss_h);
    } else {
      q_it += kBK * D * 2;
      d_it += (int64_t)kBK * dstep;
      s_it += kBK;
      left_it -= kBK;
    }
  };

  // ---- start-up: streamed tiles 0 and 1 into stages 0 and 1, and with them the workgroup's 128 Khat and V' rows
  // as tiles into stages 2 and 3 (whole cache lines by direct loads instead of 16 bytes per lane and row; the
  // row-major fragment read of a tile is the B-operand layout): one memory round trip.  Once the rows sit in
  // registers, tile 2 is requested into stage 2 and the ring turns as usual (every iteration needs its own tile and
  // the next one landed, and leaves one more in flight).
#pragma unroll
  for (int t = 0; t < R.early_tiles; ++t)
    if (t < n_it) issue_next();
  constexpr int kRowStage = R.row_stage_first;  // Khat block in stage kRowStage, V' block in the next
  {
    const int rows_left = p.Sk - k0;
    const int64_t krow = ((int64_t)b * p.Hkv + g) * p.Sk + k0;
    const char* kb = reinterpret_cast<const char*>(a.khat + krow * D);
    const char* vb = a.vmix ? reinterpret_cast<const char*>(a.vmix + krow * D) : reinterpret_cast<const char*>(row_ptr<uint16_t>(p.v, b, g, k0));
    const uint32_t vstep = a.vmix ? (uint32_t)D * 2 : (uint32_t)p.v.stride_s * 2;
    const uint32_t wave_dst = lds0 + wave * 1024;
    issue_tile_pair<D>(kb, kb, rowblock_lane_offsets<D>(D * 2, 0, rows_left, src.x, src.y), wave_dst + kRowStage * kStageBytes);
    issue_tile_pair<D>(vb, vb, rowblock_lane_offsets<D>(vstep, 0, rows_left, src.x, src.y), wave_dst + (kRowStage + 1) * kStageBytes);
  }
  wait_vmcnt<0>();
  __syncthreads();
  // stationary B operands: Khat and V' rows of this lane's key (rows 32*wave .. +31 of the block)
  bf16x8 kreg[KS], vreg[KS];
  {
    const uint32_t rm = lds0 + (wave >> 1) * Z::kTileBytes + swz_off_rm<D>(lane);
    const int rb = wave & 1;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kreg[ks] = swz_frag_rm<D>(rm + kRowStage * kStageBytes, rb, ks);
      vreg[ks] = swz_frag_rm<D>(rm + (kRowStage + 1) * kStageBytes, rb, ks);
    }
  }
  __syncthreads();  // the borrowed stages are free again
#pragma unroll
  for (int t = R.early_tiles; t < R.startup_tiles; ++t)
    if (t < n_it) issue_next();
  f32x16 dvacc[MB], dkacc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) { dvacc[mb] = splat16(0.f); dkacc[mb] = splat16(0.f); }

  const uint32_t rm_lane = lds0 + swz_off_rm<D>(lane);
  const uint32_t tr_lane = lds0 + swz_off_tr<D>(lane);
  const uint32_t st_lane = ldl0 + 16 * hh;

  bf16x8 qf[KS], df[KS];
  auto request_rowmajor = [&](uint32_t rm, int qb) {  // qb is a compile-time constant at every call site
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = swz_frag_rm<D>(rm, qb, ks);
      df[ks] = swz_frag_rm<D>(rm + Z::kTileBytes, qb, ks);
    }
  };
  // one 32-query block (qb = 0/1, compile-time) of the tile whose stage the pointers address;
  // ib = first query of the block; the row-major fragments of the block after it start at next_rm.
  // The mask variant is compile-time so that a whole block is one straight-line scheduling region:
  // 0 none, 1 causal diagonal only (every query of the block exists), 2 diagonal and / or end of the queries.
  auto step = [&](auto masked_c, uint32_t tr, uint32_t st, int qb, int ib, uint32_t next_rm, int next_qb) {
    constexpr int MASK = decltype(masked_c)::value;
    // head_dim 128 (one wave per SIMD, nothing else to hide the exp2 phase behind): the compiler's interleaving
    // strategy for exp2 work between MFMA chains, measured -3 % on this kernel; at head_dim 64 it changes nothing
    if constexpr (D == 128) __builtin_amdgcn_iglp_opt(3);
    // accumulators of S and dP start from -lse2 / -delta of the 16 query rows their registers map to
    f32x16 s, dpv;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const f32x4 l4 = lds_read_f4(st + (32 * qb + 8 * c) * 4);
      const f32x4 d4 = lds_read_f4(st + (64 + 32 * qb + 8 * c) * 4);
      s[4 * c] = l4[0]; s[4 * c + 1] = l4[1]; s[4 * c + 2] = l4[2]; s[4 * c + 3] = l4[3];
      dpv[4 * c] = d4[0]; dpv[4 * c + 1] = d4[1]; dpv[4 * c + 2] = d4[2]; dpv[4 * c + 3] = d4[3];
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) s = mfma32(qf[ks], kreg[ks], s);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) dpv = mfma32(df[ks], vreg[ks], dpv);
    bf16x8 dT[MB][2], qT[MB][2];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      dT[mb][0] = swz_frag_tr<D>(tr + Z::kTileBytes, mb, 2 * qb);
      qT[mb][0] = swz_frag_tr<D>(tr, mb, 2 * qb);
      dT[mb][1] = swz_frag_tr<D>(tr + Z::kTileBytes, mb, 2 * qb + 1);
      qT[mb][1] = swz_frag_tr<D>(tr, mb, 2 * qb + 1);
    }
    if (MASK != 0) {  // block touches the diagonal or the end of the queries
      // register r holds query ib + 4hh + c_r with c_r = 8(r/4) + r%4 a compile-time constant.
      // masked iff key > query + q_start  <=>  c_r < key - q_start - ib - 4hh,   or query >= Sq
      const int t = p.causal ? key - p.q_start - ib - 4 * hh : -1;
      const int u = p.Sq - ib - 4 * hh;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = 8 * (r >> 2) + (r & 3);
        if (MASK == 1 ? c < t : (c < t || c >= u)) s[r] = -INFINITY;
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      s[r] = fast_exp2(s[r]);
      dpv[r] *= s[r];
    }
    const bf16x8 p0 = pack_c_half(s, 0), p1 = pack_c_half(s, 1);
    const bf16x8 ds0 = pack_c_half(dpv, 0), ds1 = pack_c_half(dpv, 1);
    request_rowmajor(next_rm, next_qb);  // unconditional: past the last block the fragments are simply unused
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      dvacc[mb] = mfma32(dT[mb][0], p0, dvacc[mb]);
      dkacc[mb] = mfma32(qT[mb][0], ds0, dkacc[mb]);
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      dvacc[mb] = mfma32(dT[mb][1], p1, dvacc[mb]);
      dkacc[mb] = mfma32(qT[mb][1], ds1, dkacc[mb]);
    }
  };

  // ---- pipeline start-up: tiles 0 and 1 have landed (first wait above), tile 2 is in flight
  if (n_it > 0) request_rowmajor(rm_lane, 0);
  // Per head the visible query tiles t = 0 .. n_vis-1 (first query (qt_start + t) * 64) fall into runs for this
  // wave: [0, t_diag) touch the causal diagonal (those before t_full lie inside Sq and need the diagonal test only),
  // [t_diag, t_end) need no mask, [t_end, n_vis) run past Sq.  Each run is its own loop so that a loop body holds
  // one variant of the block (whole-block scheduling regions, no accumulator copies at joins).
  int t_diag = 0;
  if (p.causal) t_diag = min(max((max(kw0 + 31 - p.q_start, 0) + kBK - 1) / kBK - qt_start, 0), n_vis);
  const int t_full = min(max(p.Sq / kBK - qt_start, 0), n_vis);  // tiles whose 64 queries all exist
  const int t_end = max(t_full, t_diag);
  int stage = 0, it = 0;
  auto run_tiles = [&](auto masked_c, int t_lo, int t_hi) {
    constexpr int MASK = decltype(masked_c)::value;
    for (int t = t_lo; t < t_hi; ++t, ++it) {
      const int nstage = stage == kStages - 1 ? 0 : stage + 1;
      const int i0 = (qt_start + t) * kBK;
      const uint32_t rm = rm_lane + stage * kStageBytes, tr = tr_lane + stage * kStageBytes;
      const uint32_t st = st_lane + stage * 512;
      // on the diagonal a block whose last query still lies before this wave's first key is masked entirely:
      // it only passes the fragment request on (wave-uniform, so the barrier below is reached all the same)
      if (MASK == 1 && kw0 > i0 + 31 + p.q_start) request_rowmajor(rm, 1); else step(masked_c, tr, st, 0, i0, rm, 1);
      if (MASK == 1 && kw0 > i0 + 63 + p.q_start) request_rowmajor(rm_lane + nstage * kStageBytes, 0);
      else step(masked_c, tr, st, 1, i0 + 32, rm_lane + nstage * kStageBytes, 0);
      if (it + R.issue_ahead < n_it) { issue_next(); wait_vmcnt<ring::loads_kept_after_iteration(R, true)>(); } else wait_vmcnt<ring::loads_kept_after_iteration(R, false)>();
      __syncthreads();
      stage = nstage;
    }
  };
  for (int hq = 0; hq < rep; ++hq) {
    run_tiles(IC<1>{}, 0, min(t_diag, t_full));
    run_tiles(IC<2>{}, min(t_diag, t_full), t_diag);
    run_tiles(IC<0>{}, t_diag, t_end);
    run_tiles(IC<2>{}, t_end, n_vis);
  }

  // ---- epilogue: lane = key row, registers = head-dim entries.  The rows it reads (the raw key for the normaliser's
  // gradient, with a value residual the raw v and v_first rows for the coefficient gradients) come in like the
  // prologue's rows: as 128-row blocks by direct loads into the ring's stages, which are idle now (every wave has
  // passed the last iteration's barrier), and from there in the accumulators' layout.  Read row-per-lane from global
  // memory, 8 bytes per lane, every wave-wide load would touch 32 cache lines and the three tensors would keep the
  // address path of the vector memory unit busy for 4-12 us of the launch.
  static_assert(R.epilogue_row_stages == 3, "k, v, v_first blocks in stages 0, 1, 2");
  const bool live = key < p.Sk;
  float c1 = 1.f, c2 = 0.f;
  if (p.vr_coef) { c1 = p.vr_coef[0]; c2 = p.vr_coef[1]; }
  u32x2 kraw[MB][4], vraw[MB][4], fraw[MB][4];
  {
    const int rows_left = p.Sk - k0;
    const uint32_t wave_dst = lds0 + wave * 1024;
    const char* kb = reinterpret_cast<const char*>(row_ptr<uint16_t>(p.k, b, g, k0));
    issue_tile_pair<D>(kb, kb, rowblock_lane_offsets<D>((uint32_t)p.k.stride_s * 2, 0, rows_left, src.x, src.y), wave_dst);
    if (p.vr_coef) {
      const char* vb = reinterpret_cast<const char*>(row_ptr<uint16_t>(p.v, b, g, k0));
      const char* fb = reinterpret_cast<const char*>(row_ptr<uint16_t>(p.v_first, b, g, k0));
      issue_tile_pair<D>(vb, vb, rowblock_lane_offsets<D>((uint32_t)p.v.stride_s * 2, 0, rows_left, src.x, src.y), wave_dst + kStageBytes);
      issue_tile_pair<D>(fb, fb, rowblock_lane_offsets<D>((uint32_t)p.v_first.stride_s * 2, 0, rows_left, src.x, src.y), wave_dst + 2 * kStageBytes);
    }
    wait_vmcnt<0>();
    __syncthreads();
    // rows 32*wave .. +31 of a block: half (wave >> 1) of its stage, row block (wave & 1) of that tile
    const uint32_t ct = lds0 + (wave >> 1) * Z::kTileBytes + swz_off_ct<D>(lane) + (wave & 1) * 32 * Z::kRB;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const uint32_t off = (uint32_t)((4 * mb + c) << 4);
        kraw[mb][c] = lds_read8(ct ^ off);
        if (p.vr_coef) {
          vraw[mb][c] = lds_read8((ct + kStageBytes) ^ off);
          fraw[mb][c] = lds_read8((ct + 2 * kStageBytes) ^ off);
        }
      }
  }
  RopeCt<MB> rope_ct;
  if (ROPE) {
    const int64_t pos = (int64_t)(p.rope_k_pos0 + key_c) * (D / 2);
    rope_ct = rope_ct_load<MB>(p.rope_cos + pos, p.rope_sin + pos, hh);
  }
  {
    uint16_t* ovp = row_ptr_mut<uint16_t>(p.dv, b, g, key_c);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      float val[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) val[r] = c1 * dvacc[mb][r];
      store_ct_block(ovp, mb, hh, live, val);
    }
  }
  if (p.vr_coef) {
    float s1 = 0.f, s2 = 0.f;
    uint16_t* ofp = row_ptr_mut<uint16_t>(p.dv_first, b, g, key_c);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      float val[16], vv[16], ff[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) val[r] = c2 * dvacc[mb][r];
      store_ct_block(ofp, mb, hh, live, val);
      unpack_ct_block(vraw[mb], vv);
      unpack_ct_block(fraw[mb], ff);
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if (live) { s1 += dvacc[mb][r] * vv[r]; s2 += dvacc[mb][r] * ff[r]; }
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) { s1 += __shfl_xor(s1, o, 64); s2 += __shfl_xor(s2, o, 64); }
    if (lane == 0) { red[wave * 2] = s1; red[wave * 2 + 1] = s2; }
    __syncthreads();
    if (tid < 2) a.dcoef_part[(int64_t)bid * 2 + tid] = red[tid] + red[2 + tid] + red[4 + tid] + red[6 + tid];
  }
  // dk through the normaliser: W = ln2 * dkacc = dL/dKhat (natural units), dk = b W - (b^3/D)(W.k) k
  {
    float kv[MB][16];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) unpack_ct_block(kraw[mb], kv[mb]);
    // the normaliser acted on the rotated key: work in that frame, rotate the gradient back
    if (ROPE) rope_ct_apply<MB, false>(kv, rope_ct);
    float dot = 0.f, ss = 0.f;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) { dot += dkacc[mb][r] * kv[mb][r]; ss += kv[mb][r] * kv[mb][r]; }
    dot = half_sum(dot) * kLn2;
    ss = half_sum(ss);
    const float beta = row_normaliser_fast(p, ss, 1.0f / D);
    const float b3 = norm_grad_coef(p, beta, 1.0f / D) * dot;
    uint16_t* okp = row_ptr_mut<uint16_t>(p.dk, b, g, key_c);
    float val[MB][16];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) val[mb][r] = beta * kLn2 * dkacc[mb][r] - b3 * kv[mb][r];
    if (ROPE) rope_ct_apply<MB, true>(val, rope_ct);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) store_ct_block(okp, mb, hh, live, val[mb]);
  }
}

template <int D>
int launch_dkdv_t(const KArgs& a, hipStream_t st) {
  const segpt_attn_params& p = a.p;
  const int n_kvt = (p.Sk + kBwdRows - 1) / kBwdRows;
  const dim3 grid((unsigned)(wg_grid(n_kvt, p.B, p.Hkv, 1, dkdv_pinned(p)) + 1));
  if (p.rope_cos) hipLaunchKernelGGL((bwd_dkdv_bf16_kernel<D, true>), grid, dim3(kThreadsM), 0, st, a);
  else hipLaunchKernelGGL((bwd_dkdv_bf16_kernel<D, false>), grid, dim3(kThreadsM), 0, st, a);
  return (int)hipGetLastError();
}

template <int D>
int launch_dq_t(const KArgs& a, hipStream_t st) {
  const segpt_attn_params& p = a.p;
  const int n_qt = (p.Sq + kBwdRows - 1) / kBwdRows;
  const dim3 grid((unsigned)wg_grid(n_qt, p.B, p.Hkv, p.H / p.Hkv, wg_pinned_pairs(p.B, p.Hkv, false)));
  if (p.rope_cos) hipLaunchKernelGGL((bwd_dq_bf16_kernel<D, true>), grid, dim3(kThreadsM), 0, st, a);
  else hipLaunchKernelGGL((bwd_dq_bf16_kernel<D, false>), grid, dim3(kThreadsM), 0, st, a);
  return (int)hipGetLastError();
}

}  // namespace

// workgroups of the two launches (the dK/dV launch has one more, its extra reducing workgroup): the workspace holds one
// row of partial sums per workgroup, idle padding workgroups included
int bf16_dq_grid(const segpt_attn_params& p) { return wg_grid((p.Sq + kBwdRows - 1) / kBwdRows, p.B, p.Hkv, p.H / p.Hkv, wg_pinned_pairs(p.B, p.Hkv, false)); }
int bf16_dkdv_grid(const segpt_attn_params& p) { return wg_grid((p.Sk + kBwdRows - 1) / kBwdRows, p.B, p.Hkv, 1, dkdv_pinned(p)); }

int launch_bwd_dkdv_bf16(const KArgs& a, hipStream_t st) {
  if (a.p.D == 64) return launch_dkdv_t<64>(a, st);
  if (a.p.D == 128) return launch_dkdv_t<128>(a, st);
  return (int)hipErrorInvalidValue;
}

int launch_bwd_dq_bf16(const KArgs& a, hipStream_t st) {
  if (a.p.D == 64) return launch_dq_t<64>(a, st);
  if (a.p.D == 128) return launch_dq_t<128>(a, st);
  return (int)hipErrorInvalidValue;
}

}  // namespace segpt
