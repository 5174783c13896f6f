// Device-side control block of one closest_vectors loop (ann.py:38-93).
// Batch-wide facts that the reference obtains with host round trips live here
// so that the per-iteration kernels can be enqueued back to back:
//   stop        - set once a checking iteration saw no row change (ann.py:90-91)
//   first[3]    - largest visited-list fill over all rows, one slot per iteration
//                 modulo 3 (iteration t reads t-1 and t, raises t+1, and rows of
//                 one launch may be in different phases); it is the first column
//                 that is empty in every row (utils.py:63-66) because rows are
//                 kept sorted
//   changed[64] - ring of "some row changed" flags, one per checking iteration
//   sketch_rows - how many rows currently use the 8-bit sketch (they opt in once and may opt out once)
//   error       - a row found its own state impossible (see beam_row_state_ok)
#pragma once
#include "vl_common.h"

constexpr int kBeamStripes = 1024;

struct BeamCtrl {
    int stop;
    int ended_after;  // iterations run when stop was set (for callers that enqueue a fixed number of launches)
    int first[3];
    int changed[64];
    int sketch_rows;    // rows that currently look at their candidates through the 8-bit sketch first
    int error;          // set by a row whose visited-list fill is beyond what the iteration count allows: the
                        // workspace was overwritten while the loop ran (VL_ERR_STATE on the host)
    // profiling only, striped by workgroup so that the atomic adds do not queue up on one address:
    unsigned long long evals[kBeamStripes];   // candidate rows actually fetched
    unsigned long long wanted[kBeamStripes];  // candidate distances asked for (fetched or served by the cache)
    unsigned long long sketched[kBeamStripes];  // candidate rows looked at through the 8-bit sketch only
};

// A row's visited list holds at most Vt ids per earlier iteration and never more than its E slots.  A
// count beyond that was not written by this loop (its workspace is shared with another call): the row
// must not run - its copy loops would run to that count - and the loop ends with an error.
__device__ inline bool beam_row_state_ok(BeamCtrl *c, int cnt, int bound, bool writer) {
    if (cnt >= 0 && cnt <= bound) return true;
    if (writer) {
        c->error = 1;
        c->stop = 1;
    }
    return false;
}

// State of iteration t as seen by a kernel launched for it:
//   2  the loop has ended, do nothing
//   1  the visited list filled up earlier (add_new_to_seen_ returned None,
//      utils.py:68-69): the visit queue is no longer fed and pops yield empty ids
//   0  normal
// `writer` is true for exactly one thread of the launch, which records stop
// and clears the ring slot of the next checking iteration.
// look_at_fill = false (a launch that takes rows through several iterations, none of which can find a
// visited list full): state 1 is not looked for - rows of such a launch that finish early raise the slot of
// `first` that the launch after it reads, which for some lengths is the slot of iteration t - 1 modulo 3.
__device__ inline int beam_gate(BeamCtrl *c, int t, int R, int E, bool writer, bool look_at_fill = true) {
    int stop = c->stop;
    const bool after_check = t > 1 && ((t - 1) % R) == 0;
    if (!stop && after_check && c->changed[((t - 1) / R) & 63] == 0) {
        stop = 1;
        if (writer) c->ended_after = t - 1;  // the loop ran t - 1 iterations
    }
    if (stop) {
        if (writer) c->stop = 1;
        return 2;
    }
    // the slot of the check after next: this iteration itself may be a checking one (R == 1)
    // and rows of one launch set their flag while others are still here
    if (writer && ((t - 1) % R) == 0) c->changed[((t - 1) / R + 2) & 63] = 0;
    if (look_at_fill && t >= 2 && c->first[(t - 1) % 3] >= E) return 1;
    return 0;
}
