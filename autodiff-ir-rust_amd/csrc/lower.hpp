// IR -> Plan.  Replaces the reference's `to_kernel` pipeline (reference
// src/kernel/to_kernel.rs:34-106: per-command kernels, buffer renaming, proximity reordering,
// alloc insertion, three fusion passes) with a value-graph lowering per straight-line region.
#pragma once
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
};

std::unique_ptr<Plan> lower_program(const Proc& prog, const std::vector<std::string>& dep_ids,
                                    const LowerOptions& opt = LowerOptions());

// Fixed (not generated) kernels
const char* fixed_kernels_source();

}  // namespace adhip
