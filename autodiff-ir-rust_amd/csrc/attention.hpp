// Source generator for the fused attention kernel (see attention.cpp).
#pragma once
#include <string>

namespace adhip {

struct AttentionConfig {
    int d = 128;   // features of a query / key row (multiple of 4, at most 256)
    int dv = 128;  // features of a value / result row (multiple of 16, at most 256)
    int bn = 64;   // keys per iteration (64 or 32)
};

// Problem slots of one launch (blockIdx.y picks the problem: the heads of multi-head attention); a launch may use
// fewer and fills the rest with any valid pointers.
constexpr int kAttentionSlots = 16;

std::string attention_kernel_source(const AttentionConfig& cfg, const std::string& entry);

}  // namespace adhip
