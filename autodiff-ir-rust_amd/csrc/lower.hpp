// IR -> Plan.  Replaces the reference's `to_kernel` pipeline (reference
// src/kernel/to_kernel.rs:34-106: per-command kernels, buffer renaming, proximity reordering,
// alloc insertion, three fusion passes) with a value-graph lowering per straight-line region.
#pragma once
#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "ir.hpp"
#include "plan.hpp"

namespace adhip {

struct LowerOptions {
    bool fuse = true;  // false: one kernel per compute command (diagnostic mode)
    bool group_dots = true;  // same-shape independent matrix products share a launch
    bool layer_kernels = true;  // groups that run the same generated kernels on other buffers share their launches
    bool merge_small = true;    // consecutive single-block launches of a region run as phases of one launch
    bool fuse_attention = true;  // dot(softmax(scale * dot(Q, K^T)), V) runs as one kernel
    bool row_chains = true;      // row reductions and the element-wise values between them run as one kernel per row
    // Bounds on the size of one generated kernel, in what drives its register pressure: the places it loads from
    // (a tensor reference with several concat pieces loads once per piece, under a predicate) and the buffers it
    // names.  Beyond them values are cut out into kernels of their own.
    int max_pieces = 24;            // pieces of one tensor reference; wider ones are copied part by part first
    int max_inline_sites = 48;      // load sites of one folded expression
    int max_inline_loads = 32;      // distinct in-memory operands of one folded expression
    int max_kernel_sites = 96;      // load sites of all members of one kernel together
    int max_kernel_pointers = 40;   // buffers a kernel names: operands, outputs, sums
    int max_carrier_sites = 24;     // a pass that carries sums along (1024 threads a block: 128 vector registers a lane)
    int max_carrier_pointers = 20;
    // Per straight-line region (numbered in the order they are lowered): how many times the bounds above are halved
    // there.  A region at shift >= 1 also takes no fused epilogues and no sums riding along.  The runtime raises the
    // shift of a region whose kernel the compiler could only build by spilling vector registers, and lowers again.
    std::map<int, int> region_shift;
    int min_shift = 0;              // diagnostic (ADHIP_TIGHTEN): every region is lowered at this shift at least
};

std::unique_ptr<Plan> lower_program(const Proc& prog, const std::vector<std::string>& dep_ids,
                                    const LowerOptions& opt = LowerOptions());

// The current values of the environment switches that change what lower_program makes of a program, as one string:
// part of the key under which a context remembers a lowered program.
std::string lowering_switches();

// Fixed (not generated) kernels
const char* fixed_kernels_source();

}  // namespace adhip
