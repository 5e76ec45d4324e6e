// The lowered program: device buffers, generated kernels and a tree of launch / loop / branch steps.
#pragma once
#include <map>
#include <string>
#include <vector>

#include "common.hpp"

namespace adhip {

struct PlanBuffer {
    enum Kind { HOME, TEMP, CONSTPOOL } kind = TEMP;
    int64_t elems = 0;
    std::string name;
    const float* host = nullptr;  // upload source (borrowed until upload)
    int64_t host_elems = 0;
    int slot = -1;                // TEMP: physical slot shared with other temporaries
    bool zero_init = false;       // HOME: may be read before any kernel has written it; cleared at upload
};

struct KernelDef {
    std::string entry;   // symbol name
    std::string source;  // complete HIP C++ translation unit
    std::string kind;    // "elw", "reduce_row", "reduce_col", "dot", ...
    std::vector<int> regions;  // the straight-line regions (in lowering order) whose launches use it
};

struct Arg {
    enum Kind { BUF, I32, I64, F32, FLAG } kind = I32;
    int buf = -1;
    int64_t off = 0;  // BUF: element offset
    int64_t iv = 0;   // FLAG: the flag slot whose address is passed
    float fv = 0.f;
};

struct Launch {
    int kernel = -1;  // index into Plan::kernels
    unsigned grid[3] = {1, 1, 1};
    unsigned block[3] = {1, 1, 1};
    unsigned lds_bytes = 0;
    std::vector<Arg> args;  // after the leading guard pointer
    int guard = -1;         // flag slot or -1
    std::string label;
    double bytes = 0, flops = 0;  // algorithmic work of one launch
    int stat = -1;                // index into Plan::stats
};

struct Step {
    enum Kind { LAUNCH, LOOP, BRANCH, EXIT } kind = LAUNCH;
    Launch launch;
    // LOOP: while (cond[0] != 0) body; trip_count >= 0 when it is known on the host
    int cond_buf = -1;
    int64_t trip_count = -1;
    // counted loop: the body's only effect on the predicate is `x += inc; cond = (x + add) < 0` on a
    // one-element buffer x, so the trip count follows from x and cond at loop entry
    int counter_buf = -1;
    float counter_inc = 0.f, counter_add = 0.f;
    std::vector<Step> body;
    // BRANCH: first arm whose cond[0] == 1 runs, else else_body
    std::vector<std::pair<int, std::vector<Step>>> arms;
    std::vector<Step> else_body;
    // Device-predicated execution.  A data-dependent LOOP with flag_slot >= 0 is enqueued several
    // iterations ahead: a one-thread kernel latches `parent && cond != 0` into flags[flag_slot] at the
    // top of every iteration and every kernel of the body returns at once when its flag is 0, so
    // iterations enqueued past the end of the loop change nothing.  A BRANCH inside such a loop cannot
    // be decided on the host either: each arm gets a flag (arm_slots / else_slot, `taken_slot` records
    // that an earlier arm ran).  parent_guard is the flag of the enclosing predicated block or -1.
    int flag_slot = -1, parent_guard = -1, taken_slot = -1, else_slot = -1;
    std::vector<int> arm_slots;
    // LOOP with flag_slot >= 0: the last kernel of the body, which produces the predicate, latches the flag for the
    // next iteration itself; the one-thread kernel runs only once, before the first iteration.
    bool latch_in_body = false;
};

struct KernelStat {
    std::string label;
    std::string kind;
    int kernel = -1;
    double bytes = 0, flops = 0;
    uint64_t launches = 0;
    double total_ms = 0;
};

struct ResultDesc {
    int buf = -1;
    Shape shape;
};

struct Plan {
    std::vector<PlanBuffer> buffers;
    std::vector<KernelDef> kernels;
    std::vector<Step> steps;
    std::vector<KernelStat> stats;
    std::map<std::string, ResultDesc> results;  // kept id -> where its value lives at exit
    std::vector<int64_t> slot_elems;            // physical temp slots
    int n_flags = 0;
    std::string describe() const;
};

}  // namespace adhip
