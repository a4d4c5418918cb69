// The tile pipeline of the three ring kernels (forward, dQ, dK/dV), written once as data.
//
// Streamed 64-row tile pairs travel global -> LDS by direct loads that the compiler cannot see, into a ring of
// `stages` LDS stages (tile t lives in stage t % stages); completion is tracked by hand with s_waitcnt vmcnt(N)
// (vector-memory operations retire in order, so "all but the youngest N" is what a wait guarantees) followed by a
// workgroup barrier that publishes the stage to the other waves.  At start-up some stages are borrowed for the
// workgroup's stationary rows until those sit in registers.  Every number the kernels use for this (which tiles are
// requested when, into which stage, how many loads a wait may leave in flight) is a field below, and
// tests/ring_protocol_check.cpp replays the resulting order of requests, waits, barriers and fragment reads on the
// host for every kernel shape and tile count, asserting that each read hits a tile that has landed and been
// published and that no stage is refilled while another wave may still read it.
//
// Plain C++ (no HIP types): included by the kernels and by the host-side checker.
#pragma once

namespace segpt {
namespace ring {

struct Protocol {
  int stages;            // ring depth
  int loads_per_tile;    // vector-memory instructions ONE wave issues per streamed tile (the unit of vmcnt)
  int early_tiles;       // streamed tiles requested at the very start, together with the stationary rows
  int row_stage_first;   // the rows borrow stages [row_stage_first, row_stage_first + row_stages) ...
  int row_stages;        // ... until every wave has them in registers (one barrier later the stages are free)
  int startup_tiles;     // tiles requested before the loop in all: the early ones, then tiles early_tiles ..
                         // startup_tiles-1 once the borrowed stages are free
  bool wait_before_loop; // a wait + barrier between those late requests and the loop: required iff a late tile is
                         // tile 0 or 1 (iteration 0 reads its own tile and the row-major fragments of the next)
  bool issue_at_top;     // iteration jt requests its new tile before (forward) or after (backward) its two blocks
  int issue_ahead;       // ... namely tile jt + issue_ahead, into the stage that tile jt-1 has just left
  int keep_tiles;        // the wait that ends an iteration which requested a tile leaves this many of the youngest
                         // tiles in flight (an iteration that requested none waits for everything)
  int pre_row_stages = 0;   // a start-up phase of its own BEFORE all of the above: row blocks in stages
                            // [0, pre_row_stages), awaited, read into registers, one barrier; then the stages are free
  int epilogue_row_stages = 0;  // behind the loop (the ring is idle: every wave has passed the last iteration's
                            // barrier) up to this many row blocks for the epilogue are requested into stages
                            // [0, epilogue_row_stages), awaited, published by one barrier and read into registers
  bool epilogue_reuses_ring = false;  // the epilogue afterwards writes scratch data over the ring's stages
};

// An iteration needs its own tile and the next one landed.
constexpr int kTilesNeededAtLoopStart = 2;

// vmcnt immediate of the wait before the loop: the late tiles beyond the first two may stay in flight
constexpr int loads_kept_before_loop(const Protocol& p, int n_tiles) {
  const int requested = n_tiles < p.startup_tiles ? n_tiles : p.startup_tiles;
  const int kept = requested - kTilesNeededAtLoopStart;
  return (kept > 0 ? kept : 0) * p.loads_per_tile;
}
// vmcnt immediate of the wait that ends an iteration
constexpr int loads_kept_after_iteration(const Protocol& p, bool requested_a_tile) {
  return requested_a_tile ? p.keep_tiles * p.loads_per_tile : 0;
}

// ---- the kernels' protocols.  passes = wave-wide 16-byte loads per wave and [64, D] tile (2 at both head dims).
// Forward: `stages` and the rows of the query block (q_stages stages of 128 rows, the LAST stages of the ring) depend
// on the shape; the tile of iteration jt + stages - 1 is requested at the top of iteration jt.
constexpr Protocol forward(int stages, int q_stages, int passes) {
  return Protocol{stages, 2 * passes, stages - (q_stages > 1 ? q_stages : 1), stages - q_stages, q_stages, stages - 1,
                  false, true, stages - 1, stages - 3};
}
// dQ: key tile 0 in stage 0, the q / dO / o row blocks in stages 1..3, then key tiles 1 and 2; tile 1 is a late
// request, hence the wait before the loop.
constexpr Protocol dq(int passes) { return Protocol{4, 2 * passes, 1, 1, 3, 3, true, false, 3, 1, 0, 0, true}; }
// dQ with a rotary embedding: the table rows of the workgroup's 128 positions are row blocks too.  First phase: q,
// cos, sin, dO in stages 0..3; second phase: key tiles 0..2 in stages 0..2 and the o block in stage 3 (everything
// awaited: no late tiles).  The cos and sin blocks come once more behind the loop, for the epilogue.
constexpr Protocol dq_rope(int passes) { return Protocol{4, 2 * passes, 3, 3, 1, 3, false, false, 3, 1, 4, 2, true}; }
// dK/dV: (Qhat, dO) tiles 0 and 1 in stages 0 and 1 with the Khat / V' row blocks in stages 2 and 3, then tile 2;
// a tile is the two [64, D] tiles plus one row-statistics load.
// Behind the loop: the raw k block (and, with a value residual, the raw v and v_first blocks) for the epilogue.
constexpr Protocol dkdv(int passes) { return Protocol{4, 2 * passes + 1, 2, 2, 2, 3, false, false, 3, 1, 0, 3, false}; }

constexpr bool well_formed(const Protocol& p) {
  return p.stages >= 3 && p.early_tiles >= 1 && p.early_tiles <= p.startup_tiles && p.startup_tiles <= p.stages - 1 &&
         p.row_stage_first >= p.early_tiles && p.row_stage_first + p.row_stages <= p.stages && p.keep_tiles >= 0 &&
         p.issue_ahead >= kTilesNeededAtLoopStart && p.pre_row_stages >= 0 && p.pre_row_stages <= p.stages &&
         p.epilogue_row_stages >= 0 && p.epilogue_row_stages <= p.stages;
}

}  // namespace ring
}  // namespace segpt
