// HIP C++ source generation for fused kernels.
//
// A kernel is described by its iteration space, the graph nodes it must produce and the set of
// nodes that are available in memory.  Everything between is folded into one expression per
// lane: view, permute, broadcast, index/slice and concat arithmetic becomes integer index math
// on the loads (the reference prints the same information as div/mod chains per operand,
// src/kernel/indexing/matrix.rs:83-132, src/kernel/helper/shape.rs:13-76), element-wise
// operations become register arithmetic (the reference stores every intermediate,
// src/devices/opencl/kernels/fuse_elw.rs:3-21).
#pragma once
#include <map>
#include <set>
#include <string>
#include <vector>

#include "graph.hpp"

namespace adhip {

struct GenBuffer {
    Node* node;         // value held densely in memory
    std::string param;  // parameter name in the kernel signature
    bool written = false;
    int64_t max_index = 0;
};

struct ElwKernelSpec {
    std::vector<Node*> outputs;  // all with the same element count; written densely (may be empty with colsums)
    std::string name;
    // Column sums produced by the same pass: the iteration space is viewed as [rows, cols]; for every
    // entry the kernel also writes partial sums over a tile of rows of `value` (an element-wise node
    // with rows*cols elements) to a [tiles][cols] buffer (`partial`).  The caller adds the partials.
    struct ColSum { Node* value; Node* partial; };
    std::vector<ColSum> colsums;
    // Row sums produced by the same pass: a wavefront adds up `value` over its run of a row (256 columns) and writes the
    // result to `partial`, a [rows][ceil(cols / 256)] buffer.  The caller adds the runs of a row.
    struct RowSum { Node* value; Node* partial; };
    std::vector<RowSum> rowsums;
    int64_t rows = 0, cols = 0;
    // with column or row sums: how many full-size streams the pass moves (results stored + full-size operands read);
    // decides how many rows a wavefront walks, so it must be what elw_colsum_tiles is asked with
    int streams = 8;
    // A one-element output that is the predicate of the device-predicated loop the kernel runs in: the thread that
    // stores it also latches `value != 0` into the loop's flag (a trailing `int* latch` parameter), which saves the
    // one-thread kernel that would do so at the top of the next iteration.  Honoured by the plain kernel form only;
    // `GeneratedKernel::latch_done` tells.
    const Node* latch = nullptr;
};

// number of 256-column runs a row of the column-/row-sum layout is cut into
int64_t elw_rowsum_runs(int64_t cols);

struct ReduceKernelSpec {
    Node* node = nullptr;  // Op::SUM, operand [V,R]
    std::string name;
    // Element-wise values with V*R elements that this kernel also stores (row layout only): the
    // reduction's own operand chain is evaluated once, stored and summed in the same pass.
    std::vector<Node*> side_outputs;
    // Element-wise values with V elements that follow the reduction (they read its result element for element):
    // the lane that holds a finished sum also evaluates and stores them, so no further kernel is needed.  Done only
    // in the row layout when one pass finishes the sum; `GeneratedKernel::epilogue_done` tells.
    std::vector<Node*> epilogue_outputs;
    // as ElwKernelSpec::latch, for a one-element epilogue output
    const Node* latch = nullptr;
};

struct GeneratedKernel {
    std::string source;
    std::string entry;
    std::string kind;
    std::vector<Node*> buffer_args;  // in signature order (after guard); outputs included
    std::vector<int64_t> int_args;   // trailing integer arguments
    unsigned grid[3] = {1, 1, 1}, block[3] = {1, 1, 1};
    unsigned lds_bytes = 0;
    double bytes = 0, flops = 0;
    // reductions that need a second pass: partial sums [chunks][V] written to `out`, then summed
    // (for element-wise kernels with column sums: the number of row tiles)
    int64_t chunks = 1;
    bool side_done = false;  // the reduction stored its side outputs
    bool epilogue_done = false;  // the reduction evaluated and stored its epilogue outputs
    bool latch_done = false;     // the kernel takes a trailing `int* latch` and stores the loop flag
};

GeneratedKernel gen_elw_kernel(const ElwKernelSpec& spec, const std::set<const Node*>& members);
// Reduce over the last dim of a [V,R] operand.  If the result needs `chunks > 1`, the kernel writes
// partial sums laid out [chunks][V]; the caller reduces those with a second (column) reduction over the partials.
GeneratedKernel gen_reduce_kernel(const ReduceKernelSpec& spec, int64_t force_chunks = 0);
// A chain of row reductions and element-wise values over one [V, R] space that depend on one another row by row (max ->
// exp(x - max) -> sum -> divide; mean -> x - mean -> variance -> normalise): one kernel in which a wavefront (rows of
// up to 2048 elements) or a block owns a row.  Every reduction is a sweep over the row; what a sweep loads that a later
// sweep needs again stays in registers, so the row is read from memory once and each stored value written once.
struct RowChainSpec {
    int64_t V = 0, R = 0;
    std::string name;
    // every member, producers first: reductions of a [V, R] operand, element-wise values of V elements (one per row)
    // and element-wise values of V * R elements
    std::vector<Node*> order;
    std::set<const Node*> stored;  // the members that are written to memory; the others only exist inside the kernel
};
// How a tensor reference, evaluated at the element (x, y) of a [V, R] space (or, with `row_level`, at row x alone),
// addresses its source: FULL -- element x * R + y of it (the same element); ROW -- element x (one value per row);
// OTHER -- anything else.
enum class RowAccess { FULL, ROW, OTHER };
RowAccess row_access(const TRef& t, int64_t V, int64_t R, bool row_level);
// whether rows of R elements fit the kernel (a thread holds at most 8 x 4 elements of each operand)
bool rowchain_fits(int64_t V, int64_t R);
// buffer_args: the stored members in the order of `order`, then the operands
GeneratedKernel gen_rowchain_kernel(const RowChainSpec& spec);

// Number of row tiles an element-wise kernel with column sums over [rows, cols] that moves `streams` full-size
// streams (ElwKernelSpec::streams) will use.
int64_t elw_colsum_tiles(int64_t rows, int64_t cols, int streams);

// 2-D strided access description of a matmul operand, if the reference can be expressed that way.
struct Affine2D {
    Node* base = nullptr;
    int64_t offset = 0, s0 = 0, s1 = 0;
};
bool tref_affine2d(const TRef& t, Affine2D& out);

// Element-wise values with M*N elements that follow a matrix product `dot` ([M,N]) and read it element for element:
// statements for the product kernel's store loop (they use `row`, `col`, `sum_value`), the extra parameters, and the
// buffers behind them in parameter order (outputs first).
struct DotEpilogueCode {
    std::string params, code;
    std::vector<Node*> buffer_args;
    double flops = 0;  // per output element
};
DotEpilogueCode gen_dot_epilogue(const Node* dot, const std::vector<Node*>& outputs);

const char* kernel_prelude();

}  // namespace adhip
