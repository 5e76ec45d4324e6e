// Source generator for the FP32 MFMA matrix-product kernel (see gemm.cpp).
#pragma once
#include <string>

namespace adhip {

struct GemmConfig {
    bool a_kcontig = true;  // A[m,k]: k has unit stride (else m has)
    bool b_kcontig = false; // B[k,n]: k has unit stride (else n has)
    bool edge = false;      // bounds-checked scalar accesses (odd sizes or unaligned operands)
    int bm = 128;           // block tile rows: 128 (4 waves) or 256 (8 waves); the tile is bm x 128 x 16
};

std::string gemm_kernel_source(const GemmConfig& cfg, const std::string& entry);

}  // namespace adhip
