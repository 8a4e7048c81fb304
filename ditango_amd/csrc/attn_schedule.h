// The tile-load schedule of attn_fwd_kernel as a table of constants.
//
// K/V tiles travel from global memory straight into the LDS through loads the compiler does not see, so
// nothing but the hand-placed waits below keeps a wavefront from reading a buffer before every wavefront's
// share of the tile has landed, or from overwriting a buffer somebody still reads.  The kernel takes its wait
// counts, buffer count and call order FROM this table (no literal appears in attn_fwd.hip), and a host-side
// model (tests/test_attn_schedule_model.py) parses the same `#define DT_SCHED_...` lines and replays the
// schedule of both wavefront groups to check those two properties for every tile count.  One line per
// constant, integer values only, so that a plain text scan can read them.
//
// Units: a "share" is what one wavefront loads of one operand of one tile (kLoads instructions: 2 at
// D = 128, 1 at D = 64).  A call of load_tile issues two shares: V of the tile before the load cursor, then K
// of the tile under it.  The vmcnt immediates are the in-flight shares below times kLoads.
#pragma once

#define DT_SCHED_NUM_BUF 4                     // LDS buffers per operand; tile X uses buffer X % 4
#define DT_SCHED_LOADS_D128 2                  // load instructions per share at D = 128
#define DT_SCHED_LOADS_D64 1                   // ... at D = 64
#define DT_SCHED_LOAD_AFTER_MATRIX_D128 0      // D = 128: a phase's load_tile call opens the vector phase
#define DT_SCHED_LOAD_AFTER_MATRIX_D64 1       // D = 64: it follows the MFMAs of the matrix phase
#define DT_SCHED_PROLOGUE_CALLS_LEADING 3      // load_tile calls in front of the loop, leading group (tiles 0..2)
#define DT_SCHED_PROLOGUE_CALLS_TRAILING 4     // ... trailing group (tiles 0..3)
#define DT_SCHED_CALL_AHEAD 3                  // in the phase pair of tile t, group g calls load_tile for tile t + 3 + g
#define DT_SCHED_PROLOGUE_INFLIGHT_LEADING 3   // shares still in flight behind the prologue's wait: K1, V1, K2
#define DT_SCHED_PROLOGUE_INFLIGHT_TRAILING 5  // ... trailing group: K1, V1, K2, V2, K3
#define DT_SCHED_TRAILING_K1_INFLIGHT 4        // trailing group, in front of the barrier behind the first scores:
                                               // K1 must have landed (the leading group reads it next)
#define DT_SCHED_VECTOR_BARRIER_INFLIGHT_D128 3  // at the barrier that ends a vector phase: the newest call and the K
                                               // share of the one before stay in flight
#define DT_SCHED_VECTOR_BARRIER_INFLIGHT_D64 1   // D = 64 (calls behind the matrix phase): the newest K share only
