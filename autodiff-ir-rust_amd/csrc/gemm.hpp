// Source generator for the FP32 MFMA matrix-product kernel (see gemm.cpp).
#pragma once
#include <string>

namespace adhip {

struct GemmConfig {
    bool a_kcontig = true;  // A[m,k]: k has unit stride (else m has)
    bool b_kcontig = false; // B[k,n]: k has unit stride (else n has)
    bool edge = false;      // bounds-checked scalar accesses (odd sizes or unaligned operands)
};

std::string gemm_kernel_source(const GemmConfig& cfg, const std::string& entry);

}  // namespace adhip
