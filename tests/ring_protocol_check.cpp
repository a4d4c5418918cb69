// Host-side replay of the ring kernels' tile pipeline (no GPU): built and run by tests/test_ring_protocol.py.
//
// For a protocol (sample_efficient_gpt_amd/csrc/ring_protocol.hpp: the numbers the kernels themselves compile in) and
// a tile count, the order of operations ONE wave executes is generated in the kernels' control flow:
//   requests of tiles / row blocks (direct global->LDS loads, `loads` vector-memory operations each),
//   s_waitcnt vmcnt(N), workgroup barriers, fragment reads of a stage.
// All waves of a workgroup run the same order and each loads its quarter of every tile, so the replay keeps one
// symbolic wave plus the count of barriers passed ("epoch"):
//   - vector memory retires in order: a wait with immediate N retires everything but the youngest N operations;
//   - a read of a stage in epoch e is safe iff the stage holds the expected content and ALL of that content's loads
//     were retired by a wait in an epoch < e (every wave waited for its own quarter before a barrier that the reader
//     has passed);
//   - a request that refills a stage in epoch e is safe iff the last read of the stage's previous content happened
//     in an epoch < e (a barrier separates the slowest reader from the first new byte) and that content had landed.
// Exit code 0 and "ok" per line when everything holds; the deliberately broken protocols at the end must each be
// reported as a violation, or the program fails: a checker that cannot see the known bug proves nothing.
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "ring_protocol.hpp"

using segpt::ring::Protocol;

namespace {

enum Kind { REQUEST, WAIT, BARRIER, READ };
struct Op {
  Kind kind;
  int stage;    // REQUEST / READ
  int content;  // REQUEST / READ: tile index >= 0, kRows, kPreRows, kEpilogueRows or kScratch
  int n;        // REQUEST: loads issued by the wave (0: plain LDS stores, e.g. the epilogue's scratch); WAIT: the vmcnt immediate
};
constexpr int kRows = -1, kPreRows = -3, kEpilogueRows = -5, kScratch = -4;

// The order of operations of one wave, following fwd_mfma.hip / bwd_mfma.hip:
//   [first start-up phase: row blocks in stages 0 .., wait for everything, barrier, rows -> registers, barrier;]
//   start-up: early tiles, row blocks, wait for everything, barrier, rows -> registers, barrier, late tiles,
//             [wait + barrier], fragment request of tile 0;
//   iteration jt: [request at top], blocks of tile jt (its stage; the second block also requests the row-major
//             fragments of tile jt+1 from the NEXT stage), [request at bottom], wait, barrier;
//   [behind the loop: `epilogue_rows` row blocks (at most p.epilogue_row_stages) requested into stages 0 .., wait for
//    everything, barrier, rows -> registers, barrier, scratch stores over the ring].
std::vector<Op> wave_program(const Protocol& p, int n_tiles, int row_loads_per_stage, int epilogue_rows = 0) {
  std::vector<Op> ops;
  auto request_tile = [&](int t) { ops.push_back({REQUEST, t % p.stages, t, p.loads_per_tile}); };
  if (p.pre_row_stages > 0) {
    for (int i = 0; i < p.pre_row_stages; ++i) ops.push_back({REQUEST, i, kPreRows, row_loads_per_stage});
    ops.push_back({WAIT, 0, 0, 0});
    ops.push_back({BARRIER, 0, 0, 0});
    for (int i = 0; i < p.pre_row_stages; ++i) ops.push_back({READ, i, kPreRows, 0});
    ops.push_back({BARRIER, 0, 0, 0});
  }
  for (int t = 0; t < p.early_tiles; ++t)
    if (t < n_tiles) request_tile(t);
  for (int i = 0; i < p.row_stages; ++i) ops.push_back({REQUEST, p.row_stage_first + i, kRows, row_loads_per_stage});
  ops.push_back({WAIT, 0, 0, 0});
  ops.push_back({BARRIER, 0, 0, 0});
  for (int i = 0; i < p.row_stages; ++i) ops.push_back({READ, p.row_stage_first + i, kRows, 0});
  ops.push_back({BARRIER, 0, 0, 0});
  for (int t = p.early_tiles; t < p.startup_tiles; ++t)
    if (t < n_tiles) request_tile(t);
  if (p.wait_before_loop) {
    const int keep = n_tiles >= p.startup_tiles ? segpt::ring::loads_kept_before_loop(p, p.startup_tiles) : 0;
    ops.push_back({WAIT, 0, 0, keep});
    ops.push_back({BARRIER, 0, 0, 0});
  }
  if (n_tiles > 0) ops.push_back({READ, 0, 0, 0});  // row-major fragments of the first block
  for (int jt = 0; jt < n_tiles; ++jt) {
    const bool requested = jt + p.issue_ahead < n_tiles;
    if (p.issue_at_top && requested) request_tile(jt + p.issue_ahead);
    ops.push_back({READ, jt % p.stages, jt, 0});                                      // both blocks, both orientations
    if (jt + 1 < n_tiles) ops.push_back({READ, (jt + 1) % p.stages, jt + 1, 0});      // next tile's first fragments
    if (!p.issue_at_top && requested) request_tile(jt + p.issue_ahead);
    ops.push_back({WAIT, 0, 0, segpt::ring::loads_kept_after_iteration(p, requested)});
    ops.push_back({BARRIER, 0, 0, 0});
  }
  if (epilogue_rows > 0) {
    for (int i = 0; i < epilogue_rows; ++i) ops.push_back({REQUEST, i, kEpilogueRows, row_loads_per_stage});
    ops.push_back({WAIT, 0, 0, 0});
    ops.push_back({BARRIER, 0, 0, 0});
    for (int i = 0; i < epilogue_rows; ++i) ops.push_back({READ, i, kEpilogueRows, 0});
    if (p.epilogue_reuses_ring) ops.push_back({BARRIER, 0, 0, 0});
  }
  if (p.epilogue_reuses_ring)
    for (int i = 0; i < p.stages; ++i) ops.push_back({REQUEST, i, kScratch, 0});
  return ops;
}

// returns "" or the first violation
std::string replay(const Protocol& p, const std::vector<Op>& ops) {
  struct Load { int stage, content; };
  struct StageState { int content = -2; int loads_pending = 0; int retired_epoch = -1; int last_read_epoch = -1; bool ever = false; };
  std::vector<StageState> st(p.stages);
  std::vector<Load> queue;  // this wave's vector-memory operations still in flight, oldest first
  int epoch = 0;
  char buf[256];
  for (size_t i = 0; i < ops.size(); ++i) {
    const Op& o = ops[i];
    switch (o.kind) {
      case REQUEST: {
        if (o.stage < 0 || o.stage >= p.stages) return "request outside the ring";
        StageState& s = st[o.stage];
        if (s.ever) {
          if (s.loads_pending > 0) {
            snprintf(buf, sizeof buf, "op %zu: stage %d refilled with content %d while content %d is still in flight", i, o.stage, o.content, s.content);
            return buf;
          }
          if (s.last_read_epoch >= epoch) {
            snprintf(buf, sizeof buf, "op %zu: stage %d refilled with content %d in the epoch of the last read of content %d (no barrier in between)", i, o.stage, o.content, s.content);
            return buf;
          }
        }
        s.content = o.content; s.loads_pending = o.n; s.retired_epoch = o.n == 0 ? epoch : -1; s.last_read_epoch = -1; s.ever = true;
        for (int k = 0; k < o.n; ++k) queue.push_back({o.stage, o.content});
        break;
      }
      case WAIT: {
        while ((int)queue.size() > o.n) {
          const Load l = queue.front();
          queue.erase(queue.begin());
          StageState& s = st[l.stage];
          if (s.content == l.content && s.loads_pending > 0 && --s.loads_pending == 0) s.retired_epoch = epoch;
        }
        break;
      }
      case BARRIER: ++epoch; break;
      case READ: {
        StageState& s = st[o.stage];
        if (!s.ever || s.content != o.content) {
          snprintf(buf, sizeof buf, "op %zu: read of content %d from stage %d, which holds content %d", i, o.content, o.stage, s.content);
          return buf;
        }
        if (s.loads_pending > 0 || s.retired_epoch < 0 || s.retired_epoch >= epoch) {
          snprintf(buf, sizeof buf, "op %zu: read of content %d (stage %d) before it has landed and been published (pending loads %d, waited in epoch %d, read in epoch %d)",
                   i, o.content, o.stage, s.loads_pending, s.retired_epoch, epoch);
          return buf;
        }
        s.last_read_epoch = epoch;
        break;
      }
    }
  }
  return "";
}

// every streamed-tile count from min_tiles on, with every count of epilogue row blocks the protocol allows
std::string check(const Protocol& p, int max_tiles, int min_tiles = 1) {
  if (!segpt::ring::well_formed(p)) return "not well formed";
  for (int rows = 0; rows <= p.epilogue_row_stages; ++rows)
    for (int n = min_tiles; n <= max_tiles; ++n) {
      const std::string v = replay(p, wave_program(p, n, 2 * p.loads_per_tile, rows));
      if (!v.empty()) return "n_tiles " + std::to_string(n) + " + " + std::to_string(rows) + " epilogue row blocks: " + v;
    }
  return "";
}

}  // namespace

int main() {
  using namespace segpt::ring;
  struct Named { const char* name; Protocol p; };
  int failures = 0;
  // wave-wide 16-byte loads per wave and [64, D] tile: 2 at head_dim 64, 4 at head_dim 128
  for (const int passes : {2, 4}) {
    const Named shipped[] = {
        {"forward, 32 rows per wave (3 stages; head_dim 64 up to 2048 keys, head_dim 128)", forward(3, 1, passes)},
        {"forward, 64 rows per wave (4 stages; head_dim 64 beyond 2048 keys)", forward(4, 2, passes)},
        {"dQ", dq(passes)},
        {"dQ with a rotary embedding (two start-up phases, table rows once more behind the loop)", dq_rope(passes)},
        {"dK/dV (k, v, v_first rows behind the loop; a key tile may see no query at all)", dkdv(passes)},
    };
    for (const Named& k : shipped) {
      const bool can_be_empty = k.p.loads_per_tile == 2 * passes + 1;  // dK/dV: key tiles beyond every query
      const std::string v = check(k.p, 70, can_be_empty ? 0 : 1);
      printf("passes %d  %-82s %s\n", passes, k.name, v.empty() ? "ok" : ("VIOLATION: " + v).c_str());
      failures += !v.empty();
    }
  }
  const int passes = 2;
  // Other ring depths and borrowed-stage layouts the formulas claim to cover (not shipped): must hold as well.
  for (int stages = 3; stages <= 6; ++stages)
    for (int q_stages = 1; q_stages <= stages - 2; ++q_stages) {
      const std::string v = check(forward(stages, q_stages, passes), 40);
      if (!v.empty()) { printf("forward(%d stages, %d row stages): VIOLATION: %s\n", stages, q_stages, v.c_str()); ++failures; }
    }

  // ---- protocols that are wrong on purpose: each must be caught
  struct Broken { const char* name; Protocol p; };
  Protocol dq_no_wait = dq(passes);
  dq_no_wait.wait_before_loop = false;  // the start-up that shipped once: tile 1, a late request, not awaited before iteration 0
  Protocol dq_keep2 = dq(passes);
  dq_keep2.keep_tiles = 2;              // the iteration's wait leaves the tile in flight that the next iteration prefetches from
  Protocol dkdv_ahead4 = dkdv(passes);
  dkdv_ahead4.issue_ahead = 4;          // refills the stage the iteration has just read, before the barrier
  Protocol fwd_early_into_rows = forward(4, 2, passes);
  fwd_early_into_rows.early_tiles = 3;  // an early tile lands in a stage the query rows borrow
  const Broken broken[] = {
      {"dQ without the wait before the loop", dq_no_wait},
      {"dQ leaving two tiles in flight per iteration", dq_keep2},
      {"dK/dV requesting four tiles ahead in a ring of four", dkdv_ahead4},
      {"forward with an early tile in a borrowed stage", fwd_early_into_rows},
  };
  for (const Broken& k : broken) {
    const std::string v = replay(k.p, wave_program(k.p, 12, 2 * k.p.loads_per_tile));
    printf("%-93s %s\n", k.name, v.empty() ? "NOT CAUGHT" : ("caught: " + v).c_str());
    failures += v.empty();
  }
  {  // a vmcnt unit larger than what a wave really issues per tile (say the statistics load was dropped from the
     // kernel but not from the count): the iteration's wait then leaves part of the next tile in flight
    const Protocol p = dkdv(passes);
    std::vector<Op> ops = wave_program(p, 12, 2 * p.loads_per_tile);
    for (Op& o : ops)
      if (o.kind == REQUEST && o.content >= 0) o.n = p.loads_per_tile - 1;
    const std::string v = replay(p, ops);
    printf("%-82s %s\n", "dK/dV counting five loads per tile while issuing four", v.empty() ? "NOT CAUGHT" : ("caught: " + v).c_str());
    failures += v.empty();
  }
  // ---- the row blocks around the loop, broken by leaving out one barrier or wait of the generated order
  auto drop = [](std::vector<Op> ops, Kind kind, int which_from_end) {  // removes the which-th last op of a kind
    for (int i = (int)ops.size() - 1; i >= 0; --i)
      if (ops[i].kind == kind && which_from_end-- == 0) { ops.erase(ops.begin() + i); break; }
    return ops;
  };
  auto drop_nth = [](std::vector<Op> ops, Kind kind, int which) {        // removes the which-th op of a kind
    for (size_t i = 0; i < ops.size(); ++i)
      if (ops[i].kind == kind && which-- == 0) { ops.erase(ops.begin() + i); break; }
    return ops;
  };
  struct BrokenOps { const char* name; Protocol p; std::vector<Op> ops; };
  const Protocol dr = dq_rope(passes), dk = dkdv(passes);
  const BrokenOps broken_ops[] = {
      {"dK/dV reading its epilogue row blocks without the wait behind their requests", dk,
       drop(wave_program(dk, 12, 2 * dk.loads_per_tile, 3), WAIT, 0)},
      {"dK/dV reading its epilogue row blocks without the barrier behind the wait", dk,
       drop(wave_program(dk, 12, 2 * dk.loads_per_tile, 3), BARRIER, 0)},
      {"dQ (rotary) requesting the second start-up phase without the barrier behind the first phase's reads", dr,
       drop_nth(wave_program(dr, 12, 2 * dr.loads_per_tile, 2), BARRIER, 1)},
      {"dQ (rotary) writing the epilogue's scratch over the ring without a barrier behind the table-row reads", dr,
       drop(wave_program(dr, 12, 2 * dr.loads_per_tile, 2), BARRIER, 0)},
  };
  for (const BrokenOps& k : broken_ops) {
    const std::string v = replay(k.p, k.ops);
    printf("%-104s %s\n", k.name, v.empty() ? "NOT CAUGHT" : ("caught: " + v).c_str());
    failures += v.empty();
  }
  return failures ? 1 : 0;
}
