// Value graph of one straight-line region of the program.
//
// Every compute command of the IR becomes a Node whose operands are tensor references (views,
// possibly piecewise) onto other nodes.  Nothing is computed or stored when a node is created:
// the lowering later decides which nodes are written to memory ("roots", one kernel output each)
// and which are folded into the kernels that consume them.  This replaces the reference's
// one-kernel-per-command lowering followed by three peephole fusion passes
// (reference src/kernel/to_kernel.rs:13-106, src/kernel/fusion/*.rs).
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "view.hpp"

namespace adhip {

enum class Op : uint8_t {
    // leaves
    LIVEIN,   // contents of an id's home buffer at region entry
    UPLOAD,   // contents of a CreateMat payload kept in a read-only device buffer
    // element-wise
    ADD, MUL, EXP2, LOG2, SIN, RECIP, SQRT, EQ0, GT0, LT0, COPY, FILL,
    // kernels of their own
    SUM,  // [V,R] -> [V]
    MAX,  // [V,R] -> [V], the largest element of every row (NaN only where a whole row is NaN)
    DOT,  // [M,K] x [K,N] -> [M,N]
    // softmax over the rows of (cval * Q K^T), times V: operands Q [Sq,D], K^T [D,Sk] (a transposed view of K), V [Sk,DV].
    // Never built from a command: the lowering puts it in the place of a DOT whose first operand it recognises as
    // that softmax (the attention of reference src/nn/transformer.rs:10-18).
    ATTN,
};

inline bool op_is_leaf(Op o) { return o == Op::LIVEIN || o == Op::UPLOAD; }
inline bool op_is_elw(Op o) { return o >= Op::ADD && o <= Op::FILL; }
inline bool op_is_reduce(Op o) { return o == Op::SUM || o == Op::MAX; }
inline bool op_is_transcendental(Op o) { return o == Op::EXP2 || o == Op::LOG2 || o == Op::SIN; }
const char* op_name(Op o);

struct Node {
    int id = -1;
    Op op = Op::COPY;
    Shape shape;
    std::vector<TRef> in;  // operands (resolved: no SYM/NESTED sources)
    float cval = 0.f;      // FILL
    std::string name;      // IR id this node was bound to when created (for diagnostics / home buffers)
    double order = 0;      // program order (creation order; helper copies sit just before their consumer)

    // filled in by the lowering
    bool root = false;        // gets a buffer
    bool force_root = false;  // Contigious, live-out, dot operand ...
    bool transpose = false;   // dense copy of a strided view, produced by the LDS-tiled transposing kernel
    int transpose_u = -1;     // the dim of `shape` that is contiguous in the source
    int buffer = -1;          // plan buffer id holding this node's dense row-major value
    int kernel = -1;          // index of the kernel (group) that produces it
    int last_use_kernel = -1;
    std::string key;          // structural key for common-subexpression merging
};

}  // namespace adhip
