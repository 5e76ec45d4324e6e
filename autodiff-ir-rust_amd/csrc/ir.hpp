// Program representation received over the C ABI: the reference's nested IRProcedure with its
// 26 command variants (reference src/core/ir.rs:8-112), parsed from the wire format.
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "common.hpp"

namespace adhip {

enum Tag : uint8_t {
    T_CREATE_MAT = 0, T_CREATE_CONSTANT, T_ELW_MULTIPLY, T_ELW_ADD, T_ELW_MULTIPLY_EQ, T_ELW_ADD_EQ,
    T_EQUAL_ZERO, T_MORE_ZERO, T_LESS_ZERO, T_SUM, T_DOT_PRODUCT, T_VIEW, T_INDEX, T_CONCAT, T_PERMUTE,
    T_BROADCAST, T_CONTIGIOUS, T_EXP2, T_LOG2, T_SIN, T_RECIP, T_SQRT, T_WHILE, T_IF, T_EX, T_HEADING,
    // Not a variant of the reference's enum: the reduction it declares but never emits (ReduceOp::Max, reference
    // src/kernel/kernel_decl.rs:75-78; "add max, min" in src/core/ir.rs:49).  Same operand rules as Sum.
    T_MAX,
    T_COUNT
};

struct Proc;

struct Cmd {
    Tag tag = T_EX;
    std::string a, b, res;   // operand / result ids (s,o of the *Eq forms are a,b; `id` is res)
    Shape dims;              // dim / target_dim / permutation
    int64_t i0 = 0, i1 = 0;  // Index{index,dim}, Concat{dim}, Broadcast{dim,r}
    float f = 0.f;           // CreateConstant contents
    const float* host = nullptr;  // CreateMat contents (borrowed)
    uint64_t count = 0;
    std::string text;        // Heading
    std::unique_ptr<Proc> block;                                     // While body
    std::vector<std::pair<std::string, std::unique_ptr<Proc>>> conds;  // If
    std::unique_ptr<Proc> else_block;
};

struct Proc {
    std::string id;
    std::vector<Cmd> cmds;
};

// Parses the byte stream produced by the host-side serialiser.  Throws Error on malformed input.
// `payload_offsets`, when given, receives the byte offset of every CreateMat host-pointer field in stream order.
std::unique_ptr<Proc> parse_program(const uint8_t* data, size_t len, std::vector<size_t>* payload_offsets = nullptr);

const char* tag_name(Tag t);

}  // namespace adhip
