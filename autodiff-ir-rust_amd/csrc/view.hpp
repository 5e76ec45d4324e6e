// View algebra: how a tensor id refers to the values of other ids without moving data.
//
// The reference keeps, per id, a chain of data commands back to a source buffer and pushes the
// sink coordinate backwards through it when it prints an index expression
// (reference src/kernel/trackers/kernel.rs:76-232, src/kernel/helper/shape.rs:13-76).  Here the
// same information is held as strided stages (a permute, broadcast, index or slice only edits
// strides/offset; a reshape that cannot be expressed in strides adds a stage) and, for Concat,
// as a list of boxes ("pieces") of the logical shape, each with its own source and view.
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "common.hpp"

namespace adhip {

struct Node;
struct TRef;

// Maps coordinates in `shape` to offset + sum(coord[i] * stride[i]).
struct Stage {
    Shape shape, stride;
    int64_t offset = 0;
};

// Stages are applied front to back; between two stages the linear index produced by one is split
// row-major over the next stage's shape.  The last stage yields the flat index into the source.
struct View {
    std::vector<Stage> st;
};

struct Src {
    enum Kind { NODE, SYM, CONST, NESTED } kind = CONST;
    Node* node = nullptr;           // NODE: a value of the current region's graph
    std::string sym;                // SYM: "whatever id `sym` holds when this is consumed"
    float c = 0.f;                  // CONST
    std::shared_ptr<TRef> nested;   // NESTED: the dense row-major image of another reference
    bool same(const Src& o) const;
};

struct Piece {
    Shape lo, hi;  // box of the logical shape this piece covers
    View view;     // over local coordinates (coord - lo)
    Src src;
};

struct TRef {
    Shape shape;
    std::vector<Piece> pieces;
    bool single_full() const;  // exactly one piece covering the whole shape
};

Stage contiguous_stage(const Shape& shape);
bool stage_is_identity(const Stage& s);
// Reshape a stage in place (no new stage) when strides allow it.
bool stage_try_reshape(const Stage& in, const Shape& new_shape, Stage& out);
void view_reshape(View& v, const Shape& new_shape);

TRef tr_sym(const std::string& id, const Shape& shape);
TRef tr_node(Node* n, const Shape& shape);
TRef tr_const(float c, const Shape& shape);
TRef tr_permute(const TRef& t, const Shape& p);
TRef tr_broadcast(const TRef& t, int64_t dim, int64_t r);
TRef tr_index(const TRef& t, int64_t index, int64_t dim);
TRef tr_concat(const TRef& a, const TRef& b, int64_t dim);
TRef tr_reshape(const TRef& t, const Shape& new_shape);

std::string stage_str(const Stage& s);
std::string tref_str(const TRef& t);

}  // namespace adhip
