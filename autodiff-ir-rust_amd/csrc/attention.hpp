// Source generator for the fused attention kernel (see attention.cpp).
#pragma once
#include <cstddef>
#include <string>

namespace adhip {

struct AttentionConfig {
    int d = 128;   // features of a query / key row (multiple of 4, at most 256)
    int dv = 128;  // features of a value / result row (multiple of 16, at most 256)
    int bn = 64;   // keys per tile (64 or 32)
    int wg = 2;    // key groups: 1 (a block is 4 wavefronts) or 2 (8 wavefronts, each group takes half of every tile)
    bool mask = false;  // the scaled scores are multiplied by a [Sq, Sk] mask before the softmax
};

// bytes of LDS a block of this configuration needs (two stages of K and V tiles and a patch per wavefront)
size_t attention_lds_bytes(const AttentionConfig& cfg);

// Problem slots of one launch (the heads of multi-head attention; a block's number picks problem and row block); a launch may use
// fewer and fills the rest with any valid pointers.
constexpr int kAttentionSlots = 16;

std::string attention_kernel_source(const AttentionConfig& cfg, const std::string& entry);

}  // namespace adhip
