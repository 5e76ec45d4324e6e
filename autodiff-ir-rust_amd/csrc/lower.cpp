#include "lower.hpp"

#include <algorithm>
#include <array>
#include <cctype>
#include <cmath>
#include <cstring>
#include <functional>
#include <map>
#include <unordered_map>

#include "attention.hpp"
#include "codegen.hpp"
#include "gemm.hpp"
#include "graph.hpp"

namespace adhip {

const char* fixed_kernels_source() {
    return R"(
extern "C" __global__ __launch_bounds__(256) void adhip_copy(const int* __restrict__ guard, float* __restrict__ dst,
                                                             const float* __restrict__ src, unsigned long long n) {
    if (guard && *guard == 0) return;
    unsigned long long i = (unsigned long long)blockIdx.x * 256u + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

// Dense copy of a strided view whose contiguous source dim (u) is not the innermost dim of the result (v):
// a 64x64 tile goes through LDS so that both the reads (along u) and the writes (along v) are coalesced.
// Up to three further dims are batch dims, given by extent and by source / result strides.  All tiles of all batches
// are numbered along grid dimension x (the only one that is 2^31 wide).
extern "C" __global__ __launch_bounds__(256) void adhip_transpose_copy(
    const int* __restrict__ guard, float* __restrict__ out, const float* __restrict__ in, long long in_off,
    long long nb0, long long nb1, long long nb2, long long ib0, long long ib1, long long ib2, long long ob0, long long ob1,
    long long ob2, long long U, long long V, long long in_sv, long long out_su, long long ut, long long vt) {
    if (guard && *guard == 0) return;
    __shared__ float tile[64][65];
    long long b = blockIdx.x;   // tile along u fastest, then tile along v, then the batch dims
    const long long tu = b % ut; b /= ut;
    const long long tv = b % vt; b /= vt;
    const long long b2 = b % nb2; b /= nb2;
    const long long b1 = b % nb1; b /= nb1;
    const long long b0 = b;
    const float* src = in + in_off + b0 * ib0 + b1 * ib1 + b2 * ib2;
    float* dst = out + b0 * ob0 + b1 * ob1 + b2 * ob2;
    const unsigned tx = threadIdx.x & 63u, ty = threadIdx.x >> 6;
    const long long u0 = tu * 64, v0 = tv * 64;
    // all 16 loads are issued before the first value is parked (an element beyond the edge reads the view's first
    // element instead: a load under a condition would be a branch with a wait behind it)
    float q[16];
#pragma unroll
    for (unsigned i = 0; i < 16u; ++i) {
        const long long u = u0 + tx, v = v0 + ty + 4u * i;
        q[i] = src[(u < U && v < V) ? v * in_sv + u : 0];
    }
#pragma unroll
    for (unsigned i = 0; i < 16u; ++i) tile[ty + 4u * i][tx] = q[i];
    __syncthreads();
#pragma unroll 4
    for (unsigned r = ty; r < 64u; r += 4u) {
        const long long u = u0 + r, v = v0 + tx;
        if (u < U && v < V) dst[u * out_su + v] = tile[tx][r];
    }
}

// Same, 128-bit accesses: U, V, all strides and offsets are multiples of 4 elements.
extern "C" __global__ __launch_bounds__(256) void adhip_transpose_copy4(
    const int* __restrict__ guard, float* __restrict__ out, const float* __restrict__ in, long long in_off,
    long long nb0, long long nb1, long long nb2, long long ib0, long long ib1, long long ib2, long long ob0, long long ob1,
    long long ob2, long long U, long long V, long long in_sv, long long out_su, long long ut, long long vt) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    if (guard && *guard == 0) return;
    __shared__ float tile[64][65];
    long long b = blockIdx.x;   // tile along u fastest, then tile along v, then the batch dims
    const long long tu = b % ut; b /= ut;
    const long long tv = b % vt; b /= vt;
    const long long b2 = b % nb2; b /= nb2;
    const long long b1 = b % nb1; b /= nb1;
    const long long b0 = b;
    const float* src = in + in_off + b0 * ib0 + b1 * ib1 + b2 * ib2;
    float* dst = out + b0 * ob0 + b1 * ob1 + b2 * ob2;
    const unsigned c4 = threadIdx.x & 15u, rr = threadIdx.x >> 4;
    const long long u0 = tu * 64, v0 = tv * 64;
    f4 q[4];
#pragma unroll
    for (unsigned i = 0; i < 4u; ++i) {
        const long long u = u0 + 4 * c4, v = v0 + rr + 16u * i;
        q[i] = *(const f4*)(src + ((u < U && v < V) ? v * in_sv + u : 0));
    }
#pragma unroll
    for (unsigned i = 0; i < 4u; ++i) {
        const unsigned r = rr + 16u * i;
        tile[r][4 * c4 + 0] = q[i].x; tile[r][4 * c4 + 1] = q[i].y; tile[r][4 * c4 + 2] = q[i].z; tile[r][4 * c4 + 3] = q[i].w;
    }
    __syncthreads();
#pragma unroll
    for (unsigned r = rr; r < 64u; r += 16u) {
        const long long u = u0 + r, v = v0 + 4 * c4;
        if (u < U && v < V) {
            f4 q = {tile[4 * c4 + 0][r], tile[4 * c4 + 1][r], tile[4 * c4 + 2][r], tile[4 * c4 + 3][r]};
            *(f4*)(dst + u * out_su + v) = q;
        }
    }
}

// Control-flow flags for device-predicated blocks (one thread).
//   mode 0 (loop):  flags[slot] = parent && cond[0] != 0
//   mode 1 (arm):   flags[slot] = parent && !flags[taken] && cond[0] == 1; sets flags[taken] when it fires
//   mode 2 (else):  flags[slot] = parent && !flags[taken]
//   mode 3 (clear): flags[slot] = 0
extern "C" __global__ void adhip_flag(int* __restrict__ flags, int slot, int parent, const float* __restrict__ cond,
                                      int mode, int taken) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const int p = parent < 0 ? 1 : flags[parent];
    int v = 0;
    if (mode == 0) v = p && (cond[0] != 0.0f);
    else if (mode == 1) {
        v = p && !flags[taken] && (cond[0] == 1.0f);
        if (v) flags[taken] = 1;
    } else if (mode == 2) v = p && !flags[taken];
    flags[slot] = v;
}

// Second pass of column sums that rode along with an element-wise kernel: up to four sums, each the sum over
// `tiles` rows of its dense partial buffer [tiles][cols] (cols a multiple of 4), in one launch (blockIdx.y picks the
// sum).  A block is 16 four-column groups x 64 row groups; the row groups are combined through LDS by a tree of fixed
// shape, so the result does not depend on scheduling.
static __device__ __forceinline__ void adhip_colsum_finalize_body(float* o, const float* p, long long tiles, long long cols) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    __shared__ f4 part[64][16];
    const unsigned lx = threadIdx.x & 15u, ly = threadIdx.x >> 4;
    const long long x = ((long long)blockIdx.x * 16 + lx) * 4;
    const bool ok = x < cols;
    f4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    if (ok) {
#pragma unroll 4
        for (long long y = ly; y < tiles; y += 64) acc += *(const f4*)(p + y * cols + x);
    }
    part[ly][lx] = acc;
    __syncthreads();
    if (ly < 16) part[ly][lx] = (part[ly][lx] + part[ly + 16][lx]) + (part[ly + 32][lx] + part[ly + 48][lx]);
    __syncthreads();
    if (ly < 4) part[ly][lx] = (part[ly][lx] + part[ly + 4][lx]) + (part[ly + 8][lx] + part[ly + 12][lx]);
    __syncthreads();
    if (ly == 0 && ok) *(f4*)(o + x) = (part[0][lx] + part[1][lx]) + (part[2][lx] + part[3][lx]);
}

extern "C" __global__ __launch_bounds__(1024) void adhip_colsum_finalize(
    const int* __restrict__ guard, float* o0, float* o1, float* o2, float* o3, const float* p0, const float* p1,
    const float* p2, const float* p3, long long tiles, long long cols) {
    if (guard && *guard == 0) return;
    const unsigned which = blockIdx.y;
    const float* p = which == 0 ? p0 : (which == 1 ? p1 : (which == 2 ? p2 : p3));
    float* o = which == 0 ? o0 : (which == 1 ? o1 : (which == 2 ? o2 : o3));
    adhip_colsum_finalize_body(o, p, tiles, cols);
}

// Second pass of both kinds of sums that rode along with one element-wise kernel, in one launch.  Blocks
// [0, col_blocks) along x add column partials as adhip_colsum_finalize does (blockIdx.y picks one of up to four sums);
// the blocks beyond add the run sums of rows: a thread per row, out[row] = the row's `runs` consecutive partial sums
// added in ascending order (blockIdx.y picks one of up to two sums).
extern "C" __global__ __launch_bounds__(1024) void adhip_sums_finalize(
    const int* __restrict__ guard, float* o0, float* o1, float* o2, float* o3, const float* p0, const float* p1,
    const float* p2, const float* p3, long long tiles, long long cols, long long n_cols, float* r0, float* r1,
    const float* q0, const float* q1, long long rows, long long runs, long long n_rows, long long col_blocks) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    if (guard && *guard == 0) return;
    const unsigned which = blockIdx.y;
    if ((long long)blockIdx.x >= col_blocks) {
        if (which >= n_rows) return;
        const long long row = ((long long)blockIdx.x - col_blocks) * 1024 + threadIdx.x;
        if (row >= rows) return;
        const float* src = (which ? q1 : q0) + row * runs;
        float sum = 0.0f;
        if ((runs & 3) == 0) {
#pragma unroll 4
            for (long long j = 0; j < runs; j += 4) {
                const f4 v = *(const f4*)(src + j);
                sum = (((sum + v.x) + v.y) + v.z) + v.w;
            }
        } else {
            for (long long j = 0; j < runs; ++j) sum += src[j];
        }
        (which ? r1 : r0)[row] = sum;
        return;
    }
    if (which >= n_cols) return;
    const float* p = which == 0 ? p0 : (which == 1 ? p1 : (which == 2 ? p2 : p3));
    float* o = which == 0 ? o0 : (which == 1 ? o1 : (which == 2 ? o2 : o3));
    adhip_colsum_finalize_body(o, p, tiles, cols);
}

// out[i] = slices[0][i] + slices[1][i] + ... in that order, i < n; four elements per thread when n allows.
// Adds the partial products of a matrix product whose k range was cut into `count` pieces.
extern "C" __global__ __launch_bounds__(256) void adhip_sum_slices(const int* __restrict__ guard, float* __restrict__ out,
                                                                   const float* __restrict__ slices, long long count,
                                                                   long long n) {
    if (guard && *guard == 0) return;
    const long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n) return;
    if ((n & 3) == 0) {
        float4 acc = *(const float4*)(slices + i);
#pragma unroll 4
        for (long long s = 1; s < count; ++s) {
            const float4 v = *(const float4*)(slices + s * n + i);
            acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
        }
        *(float4*)(out + i) = acc;
    } else {
        for (long long j = i; j < n && j < i + 4; ++j) {
            float acc = slices[j];
            for (long long s = 1; s < count; ++s) acc += slices[s * n + j];
            out[j] = acc;
        }
    }
}

// The same for up to 16 products that shared one launch: blockIdx.y picks the product, whose slices are
// slices[y][count][n] and whose result goes to o<y>.
#define ADHIP_O16 float* o0, float* o1, float* o2, float* o3, float* o4, float* o5, float* o6, float* o7, float* o8, float* o9, \
                  float* o10, float* o11, float* o12, float* o13, float* o14, float* o15
extern "C" __global__ __launch_bounds__(256) void adhip_sum_slices_grouped(const int* __restrict__ guard, ADHIP_O16,
                                                                           const float* __restrict__ slices, long long count,
                                                                           long long n) {
    if (guard && *guard == 0) return;
    float* __restrict__ out;
    switch (blockIdx.y) {
    case 0: out = o0; break; case 1: out = o1; break; case 2: out = o2; break; case 3: out = o3; break;
    case 4: out = o4; break; case 5: out = o5; break; case 6: out = o6; break; case 7: out = o7; break;
    case 8: out = o8; break; case 9: out = o9; break; case 10: out = o10; break; case 11: out = o11; break;
    case 12: out = o12; break; case 13: out = o13; break; case 14: out = o14; break; case 15: out = o15; break;
    default: return;
    }
    slices += (long long)blockIdx.y * count * n;
    const long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n) return;
    if ((n & 3) == 0) {
        float4 acc = *(const float4*)(slices + i);
#pragma unroll 4
        for (long long s = 1; s < count; ++s) {
            const float4 v = *(const float4*)(slices + s * n + i);
            acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
        }
        *(float4*)(out + i) = acc;
    } else {
        for (long long j = i; j < n && j < i + 4; ++j) {
            float acc = slices[j];
            for (long long s = 1; s < count; ++s) acc += slices[s * n + j];
            out[j] = acc;
        }
    }
}

// One thread per output element, k ascending, one accumulator: the reference's dot kernel
// (src/devices/opencl/kernels/dotprod.rs:23-53).  Used for small products.
extern "C" __global__ __launch_bounds__(256) void adhip_dot_naive(const int* __restrict__ guard, float* __restrict__ c,
                                                                  const float* __restrict__ a, const float* __restrict__ b,
                                                                  long long m, long long n, long long k,
                                                                  long long a_off, long long a_sm, long long a_sk,
                                                                  long long b_off, long long b_sk, long long b_sn) {
    if (guard && *guard == 0) return;
    long long g = (long long)blockIdx.x * 256 + threadIdx.x;
    if (g >= m * n) return;
    long long row = g / n, col = g % n;
    float acc = 0.0f;
    const float* pa = a + a_off + row * a_sm;
    const float* pb = b + b_off + col * b_sn;
    for (long long kk = 0; kk < k; ++kk) acc = __builtin_fmaf(pa[kk * a_sk], pb[kk * b_sk], acc);
    c[g] = acc;
}
)";
}

namespace {

bool is_control(Tag t) { return t == T_WHILE || t == T_IF || t == T_EX; }
bool is_view_op(Tag t) { return t == T_VIEW || t == T_INDEX || t == T_CONCAT || t == T_PERMUTE || t == T_BROADCAST; }

struct Binding {
    enum Kind { NONE, HOME, VAL, CONST, ALIAS } kind = NONE;
    Node* node = nullptr;
    float c = 0.f;
    TRef alias;
    Shape shape;
};

using IdSet = std::set<std::string>;
using RegionKey = std::pair<const Proc*, size_t>;

struct Group {
    std::vector<Node*> members;
    int64_t n = 0;
    enum Kind { ELW, SUM, DOT, TRANSPOSE, ATTN, ROWCHAIN } kind = ELW;
    // column sums computed by this element-wise kernel: (value node, SUM node that wanted it)
    std::vector<std::pair<Node*, Node*>> colsums;
    // row sums computed by this element-wise kernel, likewise: every wavefront adds up its run of a row, the runs of a
    // row are added by a second pass
    std::vector<std::pair<Node*, Node*>> rowsums;
    int64_t cs_rows = 0, cs_cols = 0;  // the [rows, cols] view of the iteration space both kinds of sums refer to
    int cs_streams = 8;                // full-size streams of a pass with sums (ElwKernelSpec::streams)
    bool rides() const { return !colsums.empty() || !rowsums.empty(); }
    std::vector<std::pair<Node*, Node*>> riders() const {
        std::vector<std::pair<Node*, Node*>> r = colsums;
        r.insert(r.end(), rowsums.begin(), rowsums.end());
        return r;
    }
    // element-wise values a row reduction stores while it sums them
    std::vector<Node*> side;
    // element-wise values of the result's size that the reduction evaluates and stores right after summing
    std::vector<Node*> epi;
    // ROWCHAIN: members that only exist inside the kernel (nobody outside the chain reads them, no id holds them)
    std::set<Node*> unstored;
    bool dead = false;  // its only member was absorbed by another group
    bool tiled = false; // fetches an operand read against the grain through LDS tiles (takes no sums along)
    int lead = -1;      // >= 0: runs inside the launches of that group (same kernels on other buffers), which it follows directly
};

struct Lowerer {
    const Proc& prog;
    LowerOptions opt;
    IdSet deps;
    IdSet cond_ids;
    std::unique_ptr<Plan> plan{new Plan()};
    std::unordered_map<std::string, Binding> env;
    std::map<std::string, int> home_buf;
    std::map<std::string, IdSet> alias_srcs;
    std::map<RegionKey, IdSet> region_live;
    std::vector<std::unique_ptr<Node>> arena;
    std::map<std::string, int> kernel_by_source;
    int kernel_counter = 0;
    std::map<std::pair<int, int>, int> layered_kernels;
    int fixed_copy = -1, fixed_dot = -1, fixed_transpose = -1, fixed_transpose4 = -1, fixed_finalize = -1, fixed_sums_finalize = -1, fixed_sum_slices = -1, fixed_sum_slices_grouped = -1;
    int dot_epilogue_counter = 0;
    int cur_guard = -1;  // flag slot guarding the block being lowered, or -1
    // The device-predicated loop whose body is being lowered: its block, predicate id and flag.  The last region of the
    // block may hand the flag's upkeep to its last kernel (`latch_attached`).
    const Proc* latch_block = nullptr;
    std::string latch_id;
    int latch_slot = -1;
    bool latch_region = false, latch_attached = false;
    // Straight-line regions are numbered in the order they are lowered; the caller may ask for tighter kernel-size
    // bounds in some of them (LowerOptions::region_shift).
    int region_counter = 0, cur_region = -1;
    int region_shift() const {
        auto it = opt.region_shift.find(cur_region);
        return std::min(std::max(it == opt.region_shift.end() ? 0 : it->second, opt.min_shift), 8);
    }
    int64_t bound(int v) const { return std::max<int64_t>(2, (int64_t)v >> region_shift()); }
    bool tight() const { return region_shift() > 0; }

    // per region
    std::vector<Node*> rnodes;
    std::map<std::string, Node*> cse;
    std::map<std::string, Node*> livein;

    Lowerer(const Proc& p, const std::vector<std::string>& d, const LowerOptions& o) : prog(p), opt(o) {
        for (auto& s : d) deps.insert(s);
    }

    // -----------------------------------------------------------------------------------
    // liveness over the structured program
    // -----------------------------------------------------------------------------------
    void collect_alias_srcs(const Proc& p) {
        for (const Cmd& c : p.cmds) {
            if (is_view_op(c.tag)) {
                alias_srcs[c.res].insert(c.a);
                if (c.tag == T_CONCAT) alias_srcs[c.res].insert(c.b);
            }
            if (c.tag == T_WHILE) { cond_ids.insert(c.a); collect_alias_srcs(*c.block); }
            if (c.tag == T_IF) {
                for (auto& arm : c.conds) { cond_ids.insert(arm.first); collect_alias_srcs(*arm.second); }
                if (c.else_block) collect_alias_srcs(*c.else_block);
            }
        }
    }

    void add_use(IdSet& live, const std::string& id) {
        if (id.empty()) return;
        if (!live.insert(id).second) return;
        auto it = alias_srcs.find(id);
        if (it != alias_srcs.end())
            for (auto& s : it->second) add_use(live, s);
    }

    void transfer_cmd(const Cmd& c, IdSet& live) {
        auto ru = reuse.find(&c);
        if (ru != reuse.end()) {
            if (ru->second != c.res) { live.erase(c.res); add_use(live, ru->second); }
            return;
        }
        switch (c.tag) {
        case T_CREATE_MAT: case T_CREATE_CONSTANT: live.erase(c.res); break;
        case T_ELW_MULTIPLY: case T_ELW_ADD: case T_DOT_PRODUCT:
            live.erase(c.res); add_use(live, c.a); add_use(live, c.b); break;
        case T_ELW_MULTIPLY_EQ: case T_ELW_ADD_EQ:
            add_use(live, c.a); add_use(live, c.b); break;
        case T_CONCAT:
            live.erase(c.res); add_use(live, c.a); add_use(live, c.b); break;
        case T_HEADING: break;
        default:
            if (!is_control(c.tag)) { live.erase(c.res); add_use(live, c.a); }
        }
    }

    // -----------------------------------------------------------------------------------
    // available reductions and products
    //
    // A forward analysis over the structured program: after `s = Sum(v)` (or a DotProduct) the fact "s holds
    // Sum(<v written out down to the ids it views>)" stays true until s or one of those ids is redefined.  Facts are
    // intersected where paths join and iterated to a fixed point around loops.  A later Sum / DotProduct whose
    // operands spell the same expression does not run again: its result id is bound to s.  This is what removes the
    // second pass over the data from a loop whose predicate and body both reduce the same tensor (the predicate's sum
    // at the end of one iteration is the body's sum at the start of the next).
    // -----------------------------------------------------------------------------------
    struct AvEntry {
        std::string text;             // views: expression over root ids; facts: id that holds the value
        std::set<std::string> roots;  // ids the expression reads
        bool operator==(const AvEntry& o) const { return text == o.text && roots == o.roots; }
    };
    struct AvState {
        std::map<std::string, AvEntry> views;  // view id -> what it spells (expanded when the view is made, as aliases are)
        std::map<std::string, AvEntry> facts;  // expression -> holder
        bool operator==(const AvState& o) const { return views == o.views && facts == o.facts; }
    };
    std::map<const Cmd*, std::string> reuse;  // Sum / DotProduct commands whose value an id already holds
    bool av_poison = false;

    static AvEntry av_canon(const AvState& st, const std::string& id) {
        auto it = st.views.find(id);
        if (it != st.views.end()) return it->second;
        return AvEntry{"#" + id, {id}};
    }
    static void av_define(AvState& st, const std::string& id) {
        st.views.erase(id);
        for (auto it = st.facts.begin(); it != st.facts.end();) {
            if (it->second.text == id || it->second.roots.count(id)) it = st.facts.erase(it);
            else ++it;
        }
    }
    static AvState av_join(const AvState& a, const AvState& b) {
        AvState o;
        for (auto& kv : a.views) { auto it = b.views.find(kv.first); if (it != b.views.end() && it->second == kv.second) o.views.insert(kv); }
        for (auto& kv : a.facts) { auto it = b.facts.find(kv.first); if (it != b.facts.end() && it->second == kv.second) o.facts.insert(kv); }
        return o;
    }
    void av_cmd(AvState& st, const Cmd& c, bool record) {
        switch (c.tag) {
        case T_HEADING: case T_EX: return;
        case T_CREATE_MAT: case T_CREATE_CONSTANT: av_define(st, c.res); return;
        case T_VIEW: case T_INDEX: case T_PERMUTE: case T_BROADCAST: case T_CONCAT: {
            AvEntry a = av_canon(st, c.a);
            AvEntry e;
            e.roots = a.roots;
            e.text = std::string(tag_name(c.tag)) + shape_str(c.dims) + strf("[%lld,%lld](", (long long)c.i0, (long long)c.i1) + a.text;
            if (c.tag == T_CONCAT) {
                AvEntry b = av_canon(st, c.b);
                e.text += "," + b.text;
                e.roots.insert(b.roots.begin(), b.roots.end());
            }
            e.text += ")";
            if (e.roots.count(c.res)) av_poison = true;  // a view of itself: nothing here reasons about that
            av_define(st, c.res);
            st.views[c.res] = e;
            return;
        }
        case T_SUM: case T_MAX: case T_DOT_PRODUCT: {
            AvEntry a = av_canon(st, c.a);
            std::string key = std::string(tag_name(c.tag)) + "(" + a.text;
            std::set<std::string> roots = a.roots;
            if (c.tag == T_DOT_PRODUCT) {
                AvEntry b = av_canon(st, c.b);
                key += "|" + b.text;
                roots.insert(b.roots.begin(), b.roots.end());
            }
            key += ")";
            auto hit = st.facts.find(key);
            const bool have = hit != st.facts.end();
            const std::string holder = have ? hit->second.text : std::string();
            if (record && have) reuse[&c] = holder;
            if (have && holder == c.res) return;  // the id already holds exactly this
            av_define(st, c.res);
            if (have) return;                     // the older holder stays the one later commands are pointed to
            if (!roots.count(c.res)) st.facts[key] = AvEntry{c.res, roots};
            return;
        }
        case T_WHILE: {
            AvState head = st;
            for (int it = 0; it < 64; ++it) {
                AvState out = head;
                av_block(out, *c.block, false);
                AvState next = av_join(head, out);
                if (next == head) break;
                head = next;
                if (it == 63) { head = AvState(); }
            }
            AvState out = head;
            av_block(out, *c.block, record);
            st = head;
            return;
        }
        case T_IF: {
            AvState in = st;
            bool first = true;
            AvState acc;
            auto fold = [&](const AvState& o) { acc = first ? o : av_join(acc, o); first = false; };
            for (auto& arm : c.conds) {
                AvState a = in;
                av_block(a, *arm.second, record);
                fold(a);
            }
            if (c.else_block) {
                AvState a = in;
                av_block(a, *c.else_block, record);
                fold(a);
            } else {
                fold(in);
            }
            st = acc;
            return;
        }
        default:
            // every other command defines c.res (the in-place forms have res == their first operand)
            av_define(st, c.res);
            return;
        }
    }
    void av_block(AvState& st, const Proc& p, bool record) {
        for (const Cmd& c : p.cmds) av_cmd(st, c, record);
    }

    // Returns the live-in set of the block; records the live-out set of every region.
    IdSet live_block(const Proc& p, const IdSet& live_out) {
        // segment boundaries
        std::vector<size_t> ctrl;
        for (size_t i = 0; i < p.cmds.size(); ++i)
            if (is_control(p.cmds[i].tag)) ctrl.push_back(i);
        IdSet live = live_out;
        size_t end = p.cmds.size();
        for (size_t ci = ctrl.size() + 1; ci-- > 0;) {
            size_t start = ci == 0 ? 0 : ctrl[ci - 1] + 1;
            // region [start, end)
            IdSet& rec = region_live[{&p, start}];
            rec.insert(live.begin(), live.end());
            for (size_t i = end; i-- > start;) transfer_cmd(p.cmds[i], live);
            if (ci == 0) break;
            const Cmd& c = p.cmds[ctrl[ci - 1]];
            if (c.tag == T_EX) {
                // kept views are materialised by the region that ends here; their sources need not
                // outlive it, so no alias closure
                live.clear();
                for (auto& d : deps) live.insert(d);
            } else if (c.tag == T_WHILE) {
                IdSet L = live;
                add_use(L, c.a);
                for (int it = 0; it < 8; ++it) {
                    IdSet in = live_block(*c.block, L);
                    size_t before = L.size();
                    for (auto& s : in) add_use(L, s);
                    if (L.size() == before) break;
                }
                live_block(*c.block, L);
                live = L;
            } else {  // If
                IdSet L = live;
                for (auto& arm : c.conds) {
                    add_use(L, arm.first);
                    IdSet in = live_block(*arm.second, live);
                    for (auto& s : in) add_use(L, s);
                }
                if (c.else_block) {
                    IdSet in = live_block(*c.else_block, live);
                    for (auto& s : in) add_use(L, s);
                }
                live = L;
            }
            end = ctrl[ci - 1];
        }
        return live;
    }

    // -----------------------------------------------------------------------------------
    // buffers
    // -----------------------------------------------------------------------------------
    int home(const std::string& id, int64_t elems) {
        auto it = home_buf.find(id);
        if (it == home_buf.end()) {
            PlanBuffer b;
            b.kind = PlanBuffer::HOME;
            b.name = id;
            b.elems = std::max<int64_t>(elems, 1);
            plan->buffers.push_back(b);
            home_buf[id] = (int)plan->buffers.size() - 1;
            return home_buf[id];
        }
        PlanBuffer& b = plan->buffers[it->second];
        b.elems = std::max<int64_t>(b.elems, elems);
        return it->second;
    }

    std::vector<std::pair<int64_t, bool>> slots;  // (elems, in use)
    int alloc_temp(int64_t elems, const std::string& name) {
        elems = std::max<int64_t>(elems, 1);
        int best = -1;
        for (size_t i = 0; i < slots.size(); ++i) {
            if (slots[i].second) continue;
            if (best < 0) { best = (int)i; continue; }
            const int64_t cur = slots[best].first, cand = slots[i].first;
            const bool cur_fits = cur >= elems, cand_fits = cand >= elems;
            if (cand_fits && (!cur_fits || cand < cur)) best = (int)i;
            else if (!cand_fits && !cur_fits && cand > cur) best = (int)i;
        }
        if (best < 0) { slots.push_back({elems, true}); best = (int)slots.size() - 1; }
        slots[best].first = std::max(slots[best].first, elems);
        slots[best].second = true;
        PlanBuffer b;
        b.kind = PlanBuffer::TEMP;
        b.name = name;
        b.elems = elems;
        b.slot = best;
        plan->buffers.push_back(b);
        return (int)plan->buffers.size() - 1;
    }
    void free_temp(int buf) {
        const PlanBuffer& b = plan->buffers[buf];
        if (b.kind == PlanBuffer::TEMP) slots[b.slot].second = false;
    }

    // -----------------------------------------------------------------------------------
    // graph building
    // -----------------------------------------------------------------------------------
    Node* new_node(Op op, const Shape& shape, std::vector<TRef> in, const std::string& name, float cval = 0.f,
                   bool allow_cse = true) {
        std::string key = std::string(op_name(op)) + shape_str(shape) + "(";
        for (auto& t : in) key += tref_str(t) + ";";
        key += ")";
        if (op == Op::FILL) key += strf("%a", cval);
        if (allow_cse && op != Op::LIVEIN && op != Op::UPLOAD) {
            auto it = cse.find(key);
            if (it != cse.end()) return it->second;
        }
        arena.emplace_back(new Node());
        Node* n = arena.back().get();
        n->id = (int)arena.size() - 1;
        n->order = (double)n->id;
        n->op = op;
        n->shape = shape;
        n->in = std::move(in);
        n->cval = cval;
        n->name = name;
        n->key = key;
        rnodes.push_back(n);
        if (allow_cse && op != Op::LIVEIN && op != Op::UPLOAD) cse[key] = n;
        return n;
    }

    Node* get_livein(const std::string& id) {
        auto it = livein.find(id);
        if (it != livein.end()) return it->second;
        Binding& b = env[id];
        Node* n = new_node(Op::LIVEIN, b.shape, {}, id);
        n->buffer = home(id, numel(b.shape));
        livein[id] = n;
        return n;
    }

    Binding& lookup(const std::string& id) {
        auto it = env.find(id);
        ADHIP_CHECK(it != env.end() && it->second.kind != Binding::NONE, "id '%s' is used before it is defined", id.c_str());
        return it->second;
    }

    TRef resolve(const TRef& t) {
        TRef o;
        o.shape = t.shape;
        for (const Piece& p : t.pieces) {
            Piece q = p;
            if (p.src.kind == Src::SYM) {
                Binding& b = lookup(p.src.sym);
                if (b.kind == Binding::CONST) { q.src = Src(); q.src.kind = Src::CONST; q.src.c = b.c; }
                else if (b.kind == Binding::VAL) { q.src = Src(); q.src.kind = Src::NODE; q.src.node = b.node; }
                else if (b.kind == Binding::HOME) { q.src = Src(); q.src.kind = Src::NODE; q.src.node = get_livein(p.src.sym); }
                else {  // an alias that was (re)defined after this reference was made
                    TRef inner = resolve(b.alias);
                    Node* c = new_node(Op::COPY, inner.shape, {inner}, p.src.sym);
                    q.src = Src(); q.src.kind = Src::NODE; q.src.node = c;
                }
            } else if (p.src.kind == Src::NESTED) {
                TRef inner = resolve(*p.src.nested);
                Node* c = new_node(Op::COPY, inner.shape, {inner}, "");
                q.src = Src(); q.src.kind = Src::NODE; q.src.node = c;
            }
            o.pieces.push_back(std::move(q));
        }
        return o;
    }

    // symbolic reference to id (for building aliases)
    TRef sym_ref(const std::string& id) {
        Binding& b = lookup(id);
        if (b.kind == Binding::ALIAS) return b.alias;
        return tr_sym(id, b.shape);
    }

    // resolved operand of a compute command
    TRef operand(const std::string& id, const Shape* want_shape = nullptr) {
        Binding& b = lookup(id);
        TRef t;
        switch (b.kind) {
        case Binding::CONST: t = tr_const(b.c, want_shape ? *want_shape : b.shape); break;
        case Binding::VAL: t = tr_node(b.node, b.shape); break;
        case Binding::HOME: t = tr_node(get_livein(id), b.shape); break;
        case Binding::ALIAS: t = resolve(b.alias); break;
        default: throw Error("unreachable");
        }
        if (want_shape && t.shape != *want_shape) {
            ADHIP_CHECK(numel(t.shape) == numel(*want_shape), "operand '%s' of shape %s used where %s is expected", id.c_str(),
                        shape_str(t.shape).c_str(), shape_str(*want_shape).c_str());
            t = tr_reshape(t, *want_shape);
            t = resolve(t);
        }
        return t;
    }

    void bind_val(const std::string& id, Node* n, const Shape& shape) {
        Binding& b = env[id];
        b.kind = Binding::VAL;
        b.node = n;
        b.shape = shape;
        b.alias = TRef();
    }

    void build_cmd(const Cmd& c, bool once) {
        auto ru = reuse.find(&c);
        if (ru != reuse.end()) {
            // the value is already held by another id (see "available reductions and products")
            if (ru->second == c.res) return;
            Binding& bf = lookup(ru->second);
            ADHIP_CHECK(bf.kind == Binding::VAL || bf.kind == Binding::HOME, "internal: holder of a reused value is not a tensor");
            const Shape sh = bf.shape;
            Node* n = bf.kind == Binding::VAL ? bf.node : get_livein(ru->second);
            bind_val(c.res, n, sh);
            return;
        }
        switch (c.tag) {
        case T_HEADING: return;
        case T_CREATE_MAT: {
            const int64_t ne = numel(c.dims);
            if (once && !home_buf.count(c.res)) {
                // executed exactly once: the payload is uploaded straight into the id's own buffer
                int hb = home(c.res, ne);
                plan->buffers[hb].host = c.host;
                plan->buffers[hb].host_elems = ne;
                Binding& b = env[c.res];
                b = Binding();
                b.kind = Binding::HOME;
                b.shape = c.dims;
                livein.erase(c.res);
            } else {
                // inside a loop or branch: keep the payload in a read-only buffer uploaded once
                PlanBuffer pb;
                pb.kind = PlanBuffer::CONSTPOOL;
                pb.name = c.res + ".init";
                pb.elems = std::max<int64_t>(ne, 1);
                pb.host = c.host;
                pb.host_elems = ne;
                plan->buffers.push_back(pb);
                Node* n = new_node(Op::UPLOAD, c.dims, {}, c.res);
                n->buffer = (int)plan->buffers.size() - 1;
                bind_val(c.res, n, c.dims);
            }
            return;
        }
        case T_CREATE_CONSTANT: {
            Binding& b = env[c.res];
            b = Binding();
            b.kind = Binding::CONST;
            b.c = c.f;
            b.shape = c.dims;
            return;
        }
        case T_ELW_MULTIPLY: case T_ELW_ADD: case T_ELW_MULTIPLY_EQ: case T_ELW_ADD_EQ: {
            const bool mul = c.tag == T_ELW_MULTIPLY || c.tag == T_ELW_MULTIPLY_EQ;
            Binding& ba = lookup(c.a);
            Binding& bb = lookup(c.b);
            if (ba.kind == Binding::CONST && bb.kind == Binding::CONST) {
                // constant (x) constant folds on the host (reference src/kernel/trackers/constant.rs:26-56;
                // its `+=` case multiplies, the evident intent -- add -- is followed here)
                float r = mul ? ba.c * bb.c : ba.c + bb.c;
                Shape sh = ba.shape;
                Binding& br = env[c.res];
                br = Binding();
                br.kind = Binding::CONST;
                br.c = r;
                br.shape = sh;
                return;
            }
            // result takes a's shape (reference src/kernel/trackers/shape.rs:31-34); a constant's
            // shape is nominal, so the tensor operand decides then
            Shape sh = ba.kind == Binding::CONST ? bb.shape : ba.shape;
            TRef ta = operand(c.a, &sh), tb = operand(c.b, &sh);
            Node* n = new_node(mul ? Op::MUL : Op::ADD, sh, {ta, tb}, c.res);
            bind_val(c.res, n, sh);
            return;
        }
        case T_EQUAL_ZERO: case T_MORE_ZERO: case T_LESS_ZERO: case T_EXP2: case T_LOG2: case T_SIN: case T_RECIP:
        case T_SQRT: case T_CONTIGIOUS: {
            Shape sh = lookup(c.a).shape;
            TRef ta = operand(c.a);
            Op op = Op::COPY;
            switch (c.tag) {
            case T_EQUAL_ZERO: op = Op::EQ0; break;
            case T_MORE_ZERO: op = Op::GT0; break;
            case T_LESS_ZERO: op = Op::LT0; break;
            case T_EXP2: op = Op::EXP2; break;
            case T_LOG2: op = Op::LOG2; break;
            case T_SIN: op = Op::SIN; break;
            case T_RECIP: op = Op::RECIP; break;
            case T_SQRT: op = Op::SQRT; break;
            default: break;
            }
            Node* n = new_node(op, sh, {ta}, c.res, 0.f, c.tag != T_CONTIGIOUS);
            if (c.tag == T_CONTIGIOUS) n->force_root = true;
            bind_val(c.res, n, sh);
            return;
        }
        case T_SUM: case T_MAX: {
            TRef ta = operand(c.a);
            ADHIP_CHECK(ta.shape.size() == 2, "%s: operand '%s' has shape %s, expected 2-D", tag_name(c.tag), c.a.c_str(), shape_str(ta.shape).c_str());
            ADHIP_CHECK(c.tag == T_SUM || ta.shape[1] > 0, "Max: operand '%s' has no elements to take the largest of", c.a.c_str());
            Shape sh{ta.shape[0]};
            Node* n = new_node(c.tag == T_SUM ? Op::SUM : Op::MAX, sh, {ta}, c.res);
            bind_val(c.res, n, sh);
            return;
        }
        case T_DOT_PRODUCT: {
            TRef ta = operand(c.a), tb = operand(c.b);
            ADHIP_CHECK(ta.shape.size() == 2 && tb.shape.size() == 2, "DotProduct: operands must be 2-D");
            ADHIP_CHECK(ta.shape[1] == tb.shape[0], "DotProduct: %s x %s", shape_str(ta.shape).c_str(), shape_str(tb.shape).c_str());
            Shape sh{ta.shape[0], tb.shape[1]};
            Node* n = new_node(Op::DOT, sh, {ta, tb}, c.res);
            bind_val(c.res, n, sh);
            return;
        }
        case T_VIEW: case T_INDEX: case T_PERMUTE: case T_BROADCAST: case T_CONCAT: {
            TRef a = sym_ref(c.a);
            TRef r;
            if (c.tag == T_VIEW) r = tr_reshape(a, c.dims);
            else if (c.tag == T_INDEX) r = tr_index(a, c.i0, c.i1);
            else if (c.tag == T_PERMUTE) r = tr_permute(a, c.dims);
            else if (c.tag == T_BROADCAST) r = tr_broadcast(a, c.i0, c.i1);
            else r = tr_concat(a, sym_ref(c.b), c.i0);
            Binding& b = env[c.res];
            b = Binding();
            b.kind = Binding::ALIAS;
            b.shape = r.shape;
            b.alias = std::move(r);
            return;
        }
        default: throw Error(strf("internal: unexpected command %s in a region", tag_name(c.tag)));
        }
    }

    // -----------------------------------------------------------------------------------
    // region flush: choose roots, form kernels, assign buffers, emit launches
    // -----------------------------------------------------------------------------------
    static void for_each_src(const Node* n, const std::function<void(Node*, const Piece&, const TRef&)>& f) {
        for (const TRef& t : n->in)
            for (const Piece& p : t.pieces)
                if (p.src.kind == Src::NODE) f(p.src.node, p, t);
    }

    static bool in_mem(const Node* n) { return op_is_leaf(n->op) || n->root; }

    static bool identity_piece(const Piece& p, const TRef& t) {
        if (!t.single_full()) return false;
        for (const Stage& s : p.view.st)
            if (!stage_is_identity(s)) return false;
        return true;
    }

    // A SUM whose operand is the transpose of an element-wise value E seen as [R, V] (a sum over the
    // rows of E: `x.sum(0)`, bias gradients) can be produced by the pass that computes E.
    static Node* colsum_source(const Node* s, int64_t& rows, int64_t& cols) {
        if (s->op != Op::SUM) return nullptr;
        Affine2D a;
        if (!tref_affine2d(s->in[0], a)) return nullptr;
        const int64_t V = s->in[0].shape[0], R = s->in[0].shape[1];
        if (!(op_is_elw(a.base->op) || in_mem(a.base)) || a.offset != 0 || a.s0 != 1 || a.s1 != V) return nullptr;
        if (numel(a.base->shape) != V * R || V % 4 != 0 || R < 16 || V * R < (int64_t(1) << 16)) return nullptr;
        rows = R;
        cols = V;
        return a.base;
    }

    // The element-wise (or in-memory) value E with rows*cols elements whose rows the reduction `s` adds up, if `s` is
    // such a plain row sum over a space large enough for the 2-D element-wise layout.
    static Node* rowsum_source(const Node* s, int64_t& rows, int64_t& cols) {
        if (s->op != Op::SUM) return nullptr;
        Affine2D a;
        if (!tref_affine2d(s->in[0], a)) return nullptr;
        const int64_t V = s->in[0].shape[0], R = s->in[0].shape[1];
        if (!(op_is_elw(a.base->op) || in_mem(a.base)) || a.offset != 0 || a.s0 != R || a.s1 != 1) return nullptr;
        if (numel(a.base->shape) != V * R || R % 4 != 0 || R < 256 || V < 16 || V * R < (int64_t(1) << 16)) return nullptr;
        rows = V;
        cols = R;
        return a.base;
    }

    // True when, below the reduction `sum` over a [V,R] space, every read of `old` (V values) is the broadcast
    // (v, r) -> old[v] reached through element-for-element references only.
    static bool reads_at_kept_coordinate_only(Node* sum, Node* old, int64_t V, int64_t R) {
        if (numel(old->shape) != V) return false;
        bool ok = true;
        std::set<Node*> seen;
        std::function<bool(Node*)> reaches = [&](Node* n) {
            bool r = false;
            for_each_src(n, [&](Node* s, const Piece&, const TRef&) {
                if (s == old) r = true;
                else if (!in_mem(s) && !r) r = reaches(s);
            });
            return r;
        };
        std::function<void(Node*)> walk = [&](Node* n) {
            for_each_src(n, [&](Node* s, const Piece& p, const TRef& t) {
                if (!ok) return;
                if (s == old) {
                    const bool row = t.single_full() && t.shape == Shape{V, R} && p.view.st.size() == 1 &&
                                     p.view.st[0].shape == Shape{V, R} && p.view.st[0].stride == Shape{1, 0} &&
                                     p.view.st[0].offset == 0;
                    if (!row) ok = false;
                    return;
                }
                if (in_mem(s)) return;
                if (!(identity_piece(p, t) && numel(s->shape) == V * R)) {
                    if (reaches(s)) ok = false;
                    return;
                }
                if (seen.insert(s).second) walk(s);
            });
        };
        walk(sum);
        return ok;
    }

    // in-memory nodes a root reads (through folded nodes); value = every path is an identity view
    void collect_reads(Node* r, std::map<Node*, bool>& reads, std::set<Node*>* folded = nullptr) {
        std::map<std::pair<Node*, bool>, bool> seen;
        std::function<void(Node*, bool)> walk = [&](Node* n, bool ident) {
            for_each_src(n, [&](Node* s, const Piece& p, const TRef& t) {
                bool id2 = ident && identity_piece(p, t) && numel(s->shape) == numel(n->shape);
                if (in_mem(s)) {
                    auto it = reads.find(s);
                    if (it == reads.end()) reads[s] = id2;
                    else it->second = it->second && id2;
                } else {
                    if (folded && id2) folded->insert(s);
                    if (seen.insert({{s, id2}, true}).second) walk(s, id2);
                }
            });
        };
        walk(r, true);
    }

    // Kernels are told apart by their text with the entry name blanked: the per-head kernels of multi-head attention
    // (and the same epilogue generated for two layers) differ in nothing but the position in the program that their
    // name carries, and then share the first one's code object instead of being compiled once each.
    int add_kernel(const std::string& entry, const std::string& source, const std::string& kind) {
        std::string key;
        key.reserve(source.size());
        auto ident = [](char c) { return isalnum((unsigned char)c) || c == '_'; };
        for (size_t pos = 0; pos < source.size();) {
            const size_t hit = source.find(entry, pos);
            if (hit == std::string::npos) { key.append(source, pos, std::string::npos); break; }
            const size_t end = hit + entry.size();
            const bool whole = (hit == 0 || !ident(source[hit - 1])) && (end >= source.size() || !ident(source[end]));
            key.append(source, pos, hit - pos);
            if (whole) key += "@entry@";
            else key.append(source, hit, entry.size());
            pos = end;
        }
        auto it = kernel_by_source.find(key);
        if (it != kernel_by_source.end()) {
            std::vector<int>& rg = plan->kernels[(size_t)it->second].regions;
            if (std::find(rg.begin(), rg.end(), cur_region) == rg.end()) rg.push_back(cur_region);
            return it->second;
        }
        KernelDef d;
        d.entry = entry;
        d.source = source;
        d.kind = kind;
        d.regions.push_back(cur_region);
        plan->kernels.push_back(std::move(d));
        kernel_by_source[key] = (int)plan->kernels.size() - 1;
        return (int)plan->kernels.size() - 1;
    }

    // The variant of a generated kernel that runs `cnt` instances of it in one launch: the kernel becomes a device
    // function, and the new entry hands it the buffers of instance blockIdx.z.  Every parameter after `guard` is a
    // pointer; the variant takes cnt of each, in the order p0_0 .. p0_<cnt-1>, p1_0 ...
    int add_layered_kernel(int kernel, int cnt) {
        auto it = layered_kernels.find({kernel, cnt});
        if (it != layered_kernels.end()) return it->second;
        const KernelDef base = plan->kernels[kernel];
        const std::string& src = base.source;
        const std::string head = "extern \"C\" __global__ __launch_bounds__(";
        const size_t at = src.find(head);
        ADHIP_CHECK(at != std::string::npos && src.find(head, at + 1) == std::string::npos, "internal: kernel '%s' has no single entry", base.entry.c_str());
        const size_t lb_end = src.find(')', at + head.size());
        const std::string bounds = src.substr(at + head.size(), lb_end - (at + head.size()));
        const size_t open = src.find('(', lb_end + 1), close = src.find(") {", open);
        ADHIP_CHECK(open != std::string::npos && close != std::string::npos, "internal: kernel '%s' has no parameter list", base.entry.c_str());
        std::vector<std::pair<std::string, std::string>> params;  // (type, name) after guard
        {
            const std::string list = src.substr(open + 1, close - open - 1);
            size_t pos = 0;
            bool first = true;
            while (pos < list.size()) {
                size_t comma = list.find(',', pos);
                if (comma == std::string::npos) comma = list.size();
                std::string prm = list.substr(pos, comma - pos);
                pos = comma + 1;
                while (!prm.empty() && prm.front() == ' ') prm.erase(prm.begin());
                while (!prm.empty() && prm.back() == ' ') prm.pop_back();
                if (first) { first = false; continue; }  // guard
                const size_t sp = prm.find_last_of(" *");
                ADHIP_CHECK(sp != std::string::npos && prm.find('*') != std::string::npos, "internal: kernel '%s' takes a non-pointer argument", base.entry.c_str());
                params.push_back({prm.substr(0, sp + 1), prm.substr(sp + 1)});
            }
        }
        const std::string entry = base.entry + strf("_x%d", cnt);
        std::string out = src.substr(0, at);
        out += "static __device__ __forceinline__ void " + base.entry + "_one" + src.substr(open);
        out += "\nextern \"C\" __global__ __launch_bounds__(" + bounds + ") void " + entry + "(const int* __restrict__ guard";
        for (auto& pr : params)
            for (int q = 0; q < cnt; ++q) out += ", " + pr.first + pr.second + strf("_%d", q);
        out += ") {\n";
        for (auto& pr : params) out += "    " + pr.first + pr.second + ";\n";
        out += "    switch (blockIdx.z) {\n";
        for (int q = 0; q < cnt; ++q) {
            out += strf("    case %d:", q);
            for (auto& pr : params) out += " " + pr.second + " = " + pr.second + strf("_%d;", q);
            out += " break;\n";
        }
        out += "    default: return;\n    }\n    " + base.entry + "_one(guard";
        for (auto& pr : params) out += ", " + pr.second;
        out += ");\n}\n";
        const int idx = add_kernel(entry, out, base.kind);
        layered_kernels[{kernel, cnt}] = idx;
        return idx;
    }

    void push_launch(std::vector<Step>& out, Launch l, const std::string& kind) {
        KernelStat st;
        st.label = l.label;
        st.kind = kind;
        st.kernel = l.kernel;
        st.bytes = l.bytes;
        st.flops = l.flops;
        plan->stats.push_back(st);
        l.stat = (int)plan->stats.size() - 1;
        l.guard = cur_guard;
        Step s;
        s.kind = Step::LAUNCH;
        s.launch = std::move(l);
        out.push_back(std::move(s));
    }

    void emit_copy(std::vector<Step>& out, int dst, int src, int64_t n, const std::string& label) {
        if (fixed_copy < 0) fixed_copy = add_kernel("adhip_copy", fixed_kernels_source(), "copy");
        Launch l;
        l.kernel = fixed_copy;
        l.block[0] = 256;
        l.grid[0] = (unsigned)((n + 255) / 256);
        Arg a; a.kind = Arg::BUF; a.buf = dst; l.args.push_back(a);
        a.buf = src; l.args.push_back(a);
        Arg c; c.kind = Arg::I64; c.iv = n; l.args.push_back(c);
        l.label = label;
        l.bytes = 8.0 * (double)n;
        push_launch(out, l, "copy");
    }

    // -----------------------------------------------------------------------------------
    // attention: dot(softmax(scale * dot(Q, K^T)), V) as one kernel
    //
    // The caller writes attention with ordinary commands (reference src/nn/transformer.rs:10-18): a product, a scaling, a
    // row maximum, exp2((x - max) * log2 e), a row sum, a reciprocal, a multiplication, a product.  When a product's
    // first operand is exactly that chain, and nothing else looks at the chain's intermediate values, the product node
    // is turned into an ATTN node over (Q, K^T, V): the fused kernel computes the same arithmetic without the [Sq, Sk]
    // matrices ever reaching memory.  Anything that does not match to the letter stays what it was.
    // -----------------------------------------------------------------------------------
    static Node* whole_value(const TRef& t) {
        if (!t.single_full() || t.pieces[0].src.kind != Src::NODE || !identity_piece(t.pieces[0], t)) return nullptr;
        Node* n = t.pieces[0].src.node;
        return numel(n->shape) == numel(t.shape) ? n : nullptr;
    }
    // `t` of shape [V,R] is a [V] vector repeated along the columns
    static Node* column_broadcast(const TRef& t, int64_t V, int64_t R) {
        if (!t.single_full() || t.shape != Shape{V, R} || t.pieces[0].src.kind != Src::NODE) return nullptr;
        const View& v = t.pieces[0].view;
        if (v.st.empty()) return nullptr;
        for (size_t i = 0; i + 1 < v.st.size(); ++i)
            if (!stage_is_identity(v.st[i])) return nullptr;
        const Stage& s = v.st.back();
        if (s.shape != Shape{V, R} || s.stride != Shape{1, 0} || s.offset != 0) return nullptr;
        Node* n = t.pieces[0].src.node;
        return numel(n->shape) == V ? n : nullptr;
    }
    static bool constant_operand(const TRef& t, float& c) {
        if (t.pieces.size() != 1 || t.pieces[0].src.kind != Src::CONST) return false;
        c = t.pieces[0].src.c;
        return true;
    }
    // n = MUL(x, constant) in either order
    static Node* times_constant(Node* n, float& c) {
        if (n->op != Op::MUL || n->in.size() != 2) return nullptr;
        for (int k = 0; k < 2; ++k)
            if (constant_operand(n->in[(size_t)(1 - k)], c)) return whole_value(n->in[(size_t)k]);
        return nullptr;
    }

    struct AttentionKey {
        int64_t sq = 0, sk = 0, d = 0, dv = 0, q_ld = 0, k_ld = 0, v_ld = 0, m_ld = 0;  // m_ld: 0 without a mask
        float scale = 0.f;
        bool operator==(const AttentionKey& o) const {
            return sq == o.sq && sk == o.sk && d == o.d && dv == o.dv && q_ld == o.q_ld && k_ld == o.k_ld && v_ld == o.v_ld &&
                   m_ld == o.m_ld && scale == o.scale;
        }
    };
    // shape and strides of an ATTN node's operands, if they are what the kernel reads: unit stride inside a row of Q,
    // K and V, rows of K and V 16-byte aligned
    // A fourth operand is a [Sq, Sk] mask the scaled scores are multiplied with before the softmax (reference
    // src/nn/transformer.rs:21-30); `mask` receives its description.
    static bool attention_key(const Node* n, AttentionKey& k, Affine2D& q, Affine2D& kt, Affine2D& v, Affine2D* mask = nullptr) {
        if ((n->in.size() != 3 && n->in.size() != 4) || !tref_affine2d(n->in[0], q) || !tref_affine2d(n->in[1], kt) || !tref_affine2d(n->in[2], v)) return false;
        k.sq = n->in[0].shape[0];
        k.d = n->in[0].shape[1];
        k.sk = n->in[1].shape[1];
        k.dv = n->in[2].shape[1];
        if (n->in[1].shape[0] != k.d || n->in[2].shape[0] != k.sk) return false;
        if (k.d % 4 != 0 || k.d < 4 || k.d > 256 || k.dv % 16 != 0 || k.dv < 16 || k.dv > 256 || k.sq < 1 || k.sk < 1) return false;
        if ((q.s1 != 1 && k.d > 1) || kt.s0 != 1 || v.s1 != 1) return false;
        if (q.offset % 4 || q.s0 % 4 || kt.offset % 4 || kt.s1 % 4 || v.offset % 4 || v.s0 % 4) return false;
        // a thread's position inside a tile of 64 rows is a 32-bit offset
        if (q.s0 >= (int64_t(1) << 24) || kt.s1 >= (int64_t(1) << 24) || v.s0 >= (int64_t(1) << 24)) return false;
        k.q_ld = q.s0;
        k.k_ld = kt.s1;
        k.v_ld = v.s0;
        k.m_ld = 0;
        if (n->in.size() == 4) {
            Affine2D m;
            if (!tref_affine2d(n->in[3], m) || n->in[3].shape != Shape{k.sq, k.sk}) return false;
            if ((m.s1 != 1 && k.sk > 1) || m.s0 < 1 || m.s0 >= (int64_t(1) << 31)) return false;
            k.m_ld = m.s0;
            if (mask) *mask = m;
        }
        k.scale = n->cval;
        return true;
    }

    void fuse_attention(std::vector<Node*>& topo, const std::set<Node*>& wanted_nodes) {
        std::map<Node*, std::set<Node*>> consumers;
        for (Node* n : topo) for_each_src(n, [&](Node* s, const Piece&, const TRef&) { consumers[s].insert(n); });
        auto only_for = [&](Node* n, std::initializer_list<Node*> users) {
            if (wanted_nodes.count(n) || n->force_root) return false;
            std::set<Node*> u(users.begin(), users.end());
            return consumers[n] == u;
        };
        const float kLog2e = 1.44269502162933349609375f;
        for (Node* O : topo) {
            if (O->op != Op::DOT) continue;
            Node* P = whole_value(O->in[0]);
            if (!P || P->op != Op::MUL || P->shape.size() != 2) continue;
            const int64_t Sq = P->shape[0], Sk = P->shape[1];
            // P = E * (1 / sum(E)) broadcast along the row
            Node *E = nullptr, *R = nullptr;
            for (int k = 0; k < 2 && !R; ++k) {
                Node* e = whole_value(P->in[(size_t)k]);
                Node* r = column_broadcast(P->in[(size_t)(1 - k)], Sq, Sk);
                if (e && r && e->op == Op::EXP2 && r->op == Op::RECIP) { E = e; R = r; }
            }
            if (!E || !R) continue;
            Node* S = whole_value(R->in[0]);
            if (!S || S->op != Op::SUM || whole_value(S->in[0]) != E) continue;
            // E = exp2((X - max(X)) * log2 e)
            float c = 0.f;
            Node* E1 = whole_value(E->in[0]);
            Node* Dn = E1 ? times_constant(E1, c) : nullptr;
            if (!Dn || c != kLog2e || Dn->op != Op::ADD) continue;
            Node *X = nullptr, *N1 = nullptr, *M = nullptr;
            // the maximum is negated either as a vector (and repeated along the row afterwards) or after the repetition
            for (int k = 0; k < 2 && !M; ++k) {
                Node* x = whole_value(Dn->in[(size_t)k]);
                if (!x) continue;
                const TRef& other = Dn->in[(size_t)(1 - k)];
                Node* n1 = column_broadcast(other, Sq, Sk);
                const bool negated_vector = n1 != nullptr;
                if (!n1) n1 = whole_value(other);
                if (!n1 || n1->op != Op::MUL || n1->in.size() != 2) continue;
                float minus = 0.f;
                for (int q = 0; q < 2 && !M; ++q) {
                    Node* m = negated_vector ? whole_value(n1->in[(size_t)q]) : column_broadcast(n1->in[(size_t)q], Sq, Sk);
                    if (m && m->op == Op::MAX && constant_operand(n1->in[(size_t)(1 - q)], minus) && minus == -1.0f && whole_value(m->in[0]) == x) {
                        X = x; N1 = n1; M = m;
                    }
                }
            }
            if (!M) continue;
            // X = scale * (Q K^T), or that times a mask of the scores' shape
            float scale = 0.f;
            Node* D1 = times_constant(X, scale);
            Node* X0 = nullptr;   // the scaled scores under a mask
            const TRef* mask = nullptr;
            if (!D1 && X->op == Op::MUL && X->in.size() == 2) {
                for (int k = 0; k < 2 && !D1; ++k) {
                    Node* x0 = whole_value(X->in[(size_t)k]);
                    if (!x0 || X->in[(size_t)(1 - k)].shape != Shape{Sq, Sk}) continue;
                    Node* d1 = times_constant(x0, scale);
                    if (d1 && d1->op == Op::DOT) { D1 = d1; X0 = x0; mask = &X->in[(size_t)(1 - k)]; }
                }
            }
            if (!D1 || D1->op != Op::DOT) continue;
            if (!only_for(P, {O}) || !only_for(E, {P, S}) || !only_for(R, {P}) || !only_for(S, {R}) || !only_for(E1, {E}) ||
                !only_for(Dn, {E1}) || !only_for(N1, {Dn}) || !only_for(M, {N1}) || !only_for(X, {Dn, M}))
                continue;
            if (X0 ? (!only_for(X0, {X}) || !only_for(D1, {X0})) : !only_for(D1, {X})) continue;
            // would the kernel accept the operands as they are?
            Node probe;
            probe.in = {D1->in[0], D1->in[1], O->in[1]};
            if (mask) probe.in.push_back(*mask);
            probe.cval = scale;
            AttentionKey key;
            Affine2D q, kt, v, mk;
            if (!attention_key(&probe, key, q, kt, v, &mk)) continue;
            auto in_memory_able = [](const Affine2D& a) { return op_is_leaf(a.base->op) || op_is_elw(a.base->op) || a.base->root || op_is_reduce(a.base->op) || a.base->op == Op::DOT || a.base->op == Op::ATTN; };
            if (!in_memory_able(q) || !in_memory_able(kt) || !in_memory_able(v) || (mask && !in_memory_able(mk))) continue;
            O->op = Op::ATTN;
            O->in = probe.in;
            O->cval = scale;
            O->key.clear();
        }
    }

    // ---------------------------------------------------------------------------------------------------------
    // A straight-line region is lowered by a sequence of passes over one RegionPlan.  Each pass names, in the
    // references at its top, the parts of the plan it reads or changes.
    // ---------------------------------------------------------------------------------------------------------
    struct GroupKernels {
        GeneratedKernel k;
        std::vector<GeneratedKernel> extra;
        std::vector<Node*> extra_nodes;
        DotEpilogueCode dot_epi;   // DOT groups with an epilogue
        bool dot_store = true;     // ... and whether the product itself is still written
        // row sums riding along with an element-wise group: per sum the [rows][runs] partial buffer, the node that
        // stands for the second pass over it, and that pass's kernel
        std::vector<Node*> row_partials;
        // what the group's kernel was generated from, should it be generated again with a loop flag to latch
        int spec_kind = 0;  // 1: elw_spec + spec_members, 2: red_spec
        ElwKernelSpec elw_spec;
        std::set<const Node*> spec_members;
        ReduceKernelSpec red_spec;
    };
    struct Commit { int dst, src; int64_t n; std::string id; };
    struct RegionPlan {
        std::vector<std::pair<std::string, Node*>> wanted;  // (id, node) that must be in the id's home buffer at the end
        std::set<Node*> wanted_nodes;
        std::vector<Node*> topo;                             // every needed node, producers first
        std::map<Node*, std::map<Node*, bool>> reads;        // per root: in-memory values it reads (true: element for element only)
        std::map<Node*, std::set<Node*>> folded_in;          // per root: folded nodes it evaluates at its own index
        std::map<Node*, std::set<uint64_t>> sites;           // per value: the places its expression, evaluated in place, loads from
        std::vector<Group> groups;                           // kernels, in launch order
        std::map<Node*, int> group_of;
        std::map<Node*, std::string> home_of;                // wanted node -> id
        std::vector<GroupKernels> gks;                       // per group: generated code
        std::vector<std::map<Node*, bool>> greads;           // per group: reads, for hazard analysis
        std::vector<int> set_end;                            // per group: last group of the shared launches it runs in
        std::vector<Commit> commits;                         // results computed beside their home buffer, copied in at the end
    };

    void order_nodes(RegionPlan& rp) {
        rp.topo.clear();
        std::set<Node*> seen;
        std::function<void(Node*)> dfs = [&](Node* n) {
            if (!seen.insert(n).second) return;
            for_each_src(n, [&](Node* s, const Piece&, const TRef&) { dfs(s); });
            rp.topo.push_back(n);
        };
        for (auto& w : rp.wanted) dfs(w.second);
    }

    void flush_region(const IdSet& live, bool final_region, std::vector<Step>& out) {
        cur_region = region_counter++;
        const size_t first_step = out.size();
        flush_region_launches(live, final_region, out);
        if (opt.fuse && opt.merge_small) merge_single_block_runs(out, first_step);
    }

    // Consecutive launches of one region that are a single block each (the kernels of a program on tiny tensors: the
    // reference's README example is eleven of them) run as the phases of one launch instead: every kernel's translation
    // unit goes into a namespace of its own with its entry turned into a device function, and a new entry calls them
    // in order with a block-wide barrier in between, which is also what makes one phase's global writes visible to the
    // next.  Only kernel kinds in which no thread leaves before a barrier the others still reach.
    void merge_single_block_runs(std::vector<Step>& out, size_t from) {
        static const std::set<std::string> mergeable = {"elw", "reduce_row", "reduce_row_store", "reduce_col", "dot_naive", "copy", "rowchain"};
        auto single_block = [&](const Step& st) {
            if (st.kind != Step::LAUNCH) return false;
            const Launch& l = st.launch;
            if (l.grid[0] != 1 || l.grid[1] != 1 || l.grid[2] != 1 || l.block[0] != 256 || l.block[1] != 1 || l.block[2] != 1 || l.lds_bytes != 0) return false;
            return mergeable.count(plan->kernels[(size_t)l.kernel].kind) > 0;
        };
        for (size_t i = from; i < out.size(); ++i) {
            if (!single_block(out[i])) continue;
            size_t j = i, nargs = 0;
            while (j < out.size() && single_block(out[j]) && out[j].launch.guard == out[i].launch.guard &&
                   nargs + out[j].launch.args.size() <= 160) {
                nargs += out[j].launch.args.size();
                ++j;
            }
            if (j - i < 2) continue;
            std::string src, calls, params = "const int* guard";
            Launch merged;
            merged.block[0] = 256;
            merged.guard = out[i].launch.guard;
            bool ok = true;
            for (size_t q = i; q < j && ok; ++q) {
                const Launch& l = out[q].launch;
                const KernelDef& kd = plan->kernels[(size_t)l.kernel];
                std::string body = kd.source;
                const std::string head = "extern \"C\" __global__", bounds = "__launch_bounds__(", noalias = "__restrict__";
                for (size_t at = body.find(head); at != std::string::npos; at = body.find(head)) body.replace(at, head.size(), "static __device__");
                for (size_t at = body.find(bounds); at != std::string::npos; at = body.find(bounds)) body.erase(at, body.find(')', at) + 1 - at);
                // a buffer one phase writes is another phase's input: no parameter may promise that nothing else names its memory
                for (size_t at = body.find(noalias); at != std::string::npos; at = body.find(noalias)) body.erase(at, noalias.size());
                const size_t fn = body.find(" void " + kd.entry + "(");
                const size_t open = fn == std::string::npos ? fn : body.find('(', fn);
                const size_t close = open == std::string::npos ? open : body.find(") {", open);
                if (close == std::string::npos) { ok = false; break; }
                std::string list = body.substr(open + 1, close - open - 1), args;
                size_t pos = 0, index = 0;
                while (pos < list.size()) {
                    size_t comma = list.find(',', pos);
                    if (comma == std::string::npos) comma = list.size();
                    std::string prm = list.substr(pos, comma - pos);
                    pos = comma + 1;
                    while (!prm.empty() && isspace((unsigned char)prm.front())) prm.erase(prm.begin());
                    while (!prm.empty() && isspace((unsigned char)prm.back())) prm.pop_back();
                    if (index++ == 0) continue;  // guard
                    const size_t sp = prm.find_last_of(" *");
                    if (sp == std::string::npos) { ok = false; break; }
                    const std::string name = strf("s%zu_%s", q - i, prm.substr(sp + 1).c_str());
                    params += ", " + prm.substr(0, sp + 1) + name;
                    args += ", " + name;
                }
                if (index != l.args.size() + 1) ok = false;  // the launch must pass exactly the entry's parameters
                src += strf("namespace seg%zu {\n", q - i) + body + "\n}\n";
                calls += strf("    seg%zu::%s(guard%s);\n", q - i, kd.entry.c_str(), args.c_str());
                if (q + 1 < j) calls += "    __syncthreads();\n";
                merged.args.insert(merged.args.end(), l.args.begin(), l.args.end());
                merged.bytes += l.bytes;
                merged.flops += l.flops;
            }
            if (!ok) continue;
            const std::string entry = strf("run%d_%s_x%zu", kernel_counter++, out[i].launch.label.c_str(), j - i);
            src += "extern \"C\" __global__ __launch_bounds__(256) void " + entry + "(" + params + ") {\n" + calls + "}\n";
            merged.kernel = add_kernel(entry, src, "merged");
            merged.label = entry;
            KernelStat st;
            st.label = entry;
            st.kind = "merged";
            st.kernel = merged.kernel;
            st.bytes = merged.bytes;
            st.flops = merged.flops;
            plan->stats.push_back(st);
            merged.stat = (int)plan->stats.size() - 1;
            Step ms;
            ms.kind = Step::LAUNCH;
            ms.launch = std::move(merged);
            out.erase(out.begin() + (std::ptrdiff_t)i, out.begin() + (std::ptrdiff_t)j);
            out.insert(out.begin() + (std::ptrdiff_t)i, std::move(ms));
        }
    }

    void flush_region_launches(const IdSet& live, bool final_region, std::vector<Step>& out) {
        RegionPlan rp;
        collect_wanted(rp, live, final_region);
        order_nodes(rp);
        if (rp.topo.empty()) { end_region(rp.wanted); return; }
        if (opt.fuse && opt.fuse_attention) {
            fuse_attention(rp.topo, rp.wanted_nodes);
            order_nodes(rp);
        }
        force_roots(rp);
        narrow_references(rp);
        if (opt.fuse) plan_transposed_copies(rp);
        keep_shared_values(rp);
        cut_long_expressions(rp);
        form_groups(rp);
        if (opt.fuse) {
            attach_column_sums(rp);
            if (opt.row_chains) form_row_chains(rp);
            attach_row_sum_operands(rp);
            fold_transposed_copies(rp);
            attach_row_sums(rp);
            if (opt.group_dots) group_independent_products(rp);
        }
        generate_kernels(rp);
        if (opt.fuse && opt.layer_kernels) share_launches(rp);
        assign_buffers(rp);
        emit_launches(rp, out);
        end_region(rp.wanted);
    }

    // ---- 1. what has to be in a home buffer when the region ends
    void collect_wanted(RegionPlan& rp, const IdSet& live, bool final_region) {
        auto& wanted = rp.wanted;
        auto& wanted_nodes = rp.wanted_nodes;
        auto want = [&](const std::string& id, Node* n) {
            if (numel(n->shape) == 0) return;
            if (op_is_leaf(n->op) || wanted_nodes.count(n)) n = new_node(Op::COPY, n->shape, {tr_node(n, n->shape)}, id, 0.f, false);
            wanted_nodes.insert(n);
            wanted.push_back({id, n});
        };
        for (const std::string& id : live) {
            auto it = env.find(id);
            if (it == env.end()) continue;
            Binding& b = it->second;
            if (b.kind == Binding::VAL) {
                if (b.node->op == Op::LIVEIN && b.node->name == id) continue;
                want(id, b.node);
            } else if ((b.kind == Binding::ALIAS || b.kind == Binding::CONST) &&
                       ((final_region && deps.count(id)) || cond_ids.count(id))) {
                if (numel(b.shape) == 0) continue;
                Node* n;
                if (b.kind == Binding::CONST) n = new_node(Op::FILL, b.shape, {}, id, b.c, false);
                else {
                    TRef r = resolve(b.alias);
                    // a kept view that is just another name for a whole computed value (same linear
                    // layout) needs no copy: that value is written straight into this id's buffer
                    if (r.single_full() && r.pieces[0].src.kind == Src::NODE && identity_piece(r.pieces[0], r) &&
                        !op_is_leaf(r.pieces[0].src.node->op) && numel(r.pieces[0].src.node->shape) == numel(r.shape) &&
                        !wanted_nodes.count(r.pieces[0].src.node)) {
                        bool bound_elsewhere = false;  // ... unless the value must also live under its own id
                        for (const std::string& other : live) {
                            auto io = env.find(other);
                            if (io != env.end() && io->second.kind == Binding::VAL && io->second.node == r.pieces[0].src.node) bound_elsewhere = true;
                        }
                        if (!bound_elsewhere) {
                            n = r.pieces[0].src.node;
                            wanted_nodes.insert(n);
                            wanted.push_back({id, n});
                            continue;
                        }
                    }
                    n = new_node(Op::COPY, r.shape, {r}, id, 0.f, false);
                }
                wanted_nodes.insert(n);
                wanted.push_back({id, n});
            }
        }
    }

    // ---- 3. values that get a kernel and a buffer of their own whatever happens; product operands that are not
    // strided 2-D views of memory are copied first
    // A product whose left operand is a Concat of row blocks, each of them a strided view of one value in memory (the
    // heads of an attention layer side by side, transposed: the weight gradient of the projection behind them), would
    // need the Concat written out first -- against the grain, through transposed copies.  Rows of a product depend on
    // the same rows of its left operand only: it is computed as one product per block (they share a grouped launch) and
    // is itself the Concat of their results.
    void split_row_concat_products(RegionPlan& rp) {
        if (!opt.fuse || !opt.group_dots) return;
        bool changed = false;
        std::vector<Node*> work = rp.topo;
        for (Node* n : work) {
            if (n->op != Op::DOT || n->in.size() != 2) continue;
            const TRef A = n->in[0], B = n->in[1];
            Affine2D a2, b2;
            if (tref_affine2d(A, a2) || !tref_affine2d(B, b2)) continue;
            if (A.pieces.size() < 2 || (int)A.pieces.size() > kGemmGroupSlots) continue;
            const int64_t M = A.shape[0], K = A.shape[1], N = B.shape[1];
            std::vector<const Piece*> blocks;
            for (const Piece& pc : A.pieces) blocks.push_back(&pc);
            std::sort(blocks.begin(), blocks.end(), [](const Piece* x, const Piece* y) { return x->lo[0] < y->lo[0]; });
            bool ok = true;
            int64_t at = 0;
            std::vector<TRef> parts_a;
            for (const Piece* pc : blocks) {
                ok = ok && pc->lo[0] == at && pc->lo[1] == 0 && pc->hi[1] == K && pc->hi[0] - pc->lo[0] >= 64 && pc->src.kind == Src::NODE;
                if (!ok) break;
                at = pc->hi[0];
                TRef ai;
                ai.shape = {pc->hi[0] - pc->lo[0], K};
                Piece q = *pc;
                q.lo = {0, 0};
                q.hi = ai.shape;
                ai.pieces.push_back(std::move(q));
                Affine2D pa;
                ok = ok && tref_affine2d(ai, pa) && (op_is_leaf(pa.base->op) || op_is_elw(pa.base->op) || op_is_reduce(pa.base->op) ||
                                                     pa.base->op == Op::DOT || pa.base->op == Op::ATTN || pa.base->root);
                parts_a.push_back(std::move(ai));
            }
            if (!ok || at != M) continue;
            TRef whole;
            whole.shape = n->shape;
            int64_t row = 0;
            for (size_t i = 0; i < parts_a.size(); ++i) {
                const Shape sh{parts_a[i].shape[0], N};
                Node* d = new_node(Op::DOT, sh, {parts_a[i], B}, strf("%s.rows%zu", n->name.c_str(), i));
                d->order = std::min(d->order, n->order - 0.25 + 0.01 * (double)i);
                Piece q;
                q.lo = {row, 0};
                q.hi = {row + sh[0], N};
                q.view.st.push_back(contiguous_stage(sh));
                q.src.kind = Src::NODE;
                q.src.node = d;
                whole.pieces.push_back(std::move(q));
                row += sh[0];
            }
            n->op = Op::COPY;
            n->in = {whole};
            n->key.clear();
            changed = true;
        }
        if (changed) order_nodes(rp);
    }

    void force_roots(RegionPlan& rp) {
        split_row_concat_products(rp);
        auto& wanted = rp.wanted;
        auto& topo = rp.topo;
        for (auto& w : wanted) w.second->root = true;
        for (size_t i = 0; i < topo.size(); ++i) {
            Node* n = topo[i];
            if (op_is_reduce(n->op) || n->op == Op::DOT || n->op == Op::ATTN || n->force_root) n->root = true;
            if (!opt.fuse && op_is_elw(n->op)) n->root = true;
            if (numel(n->shape) == 0) n->root = false;
        }
        // matmul operands must be strided 2-D views of memory
        for (size_t i = 0; i < topo.size(); ++i) {
            Node* n = topo[i];
            if (n->op != Op::DOT && n->op != Op::ATTN) continue;
            for (TRef& t : n->in) {
                Affine2D a2;
                if (tref_affine2d(t, a2) && (op_is_leaf(a2.base->op) || op_is_elw(a2.base->op) || a2.base->root)) {
                    if (!op_is_leaf(a2.base->op)) a2.base->root = true;
                    continue;
                }
                Node* c = new_node(Op::COPY, t.shape, {t}, n->name + ".operand", 0.f, false);
                c->root = true;
                c->order = n->order - 0.5;
                t = tr_node(c, t.shape);
            }
        }
        order_nodes(rp);  // copies were added
    }

    // ---- 3b. large operands read against the grain (unit stride on a dim that is not the innermost one
    // of the consumer) are first copied densely by the tiled transposing kernel
    void plan_transposed_copies(RegionPlan& rp) {
        auto& topo = rp.topo;
        std::vector<Node*> work = topo;
        std::stable_sort(work.begin(), work.end(), [](Node* a, Node* b) { return a->order < b->order; });
        std::map<std::string, Node*> transposed;  // region of a source node -> its dense copy
        bool added = false;
        for (Node* n : work) {
            if (!op_is_elw(n->op) || n->transpose) continue;
            for (TRef& t : n->in) {
                for (Piece& pc : t.pieces) {
                    if (pc.src.kind != Src::NODE || !in_mem(pc.src.node) || pc.view.st.empty()) continue;
                    // the last stage is the one that addresses the buffer; earlier stages only
                    // produce a row-major index into its shape, which a dense copy keeps valid
                    const Stage st = pc.view.st.back();
                    int last = -1, u = -1, nbatch = 0;
                    for (int d = (int)st.shape.size() - 1; d >= 0; --d)
                        if (st.shape[d] > 1) { last = d; break; }
                    if (last < 0 || st.stride[last] <= 1) continue;
                    for (int d = 0; d < last; ++d)
                        if (st.shape[d] > 1 && st.stride[d] == 1) u = d;
                    if (u < 0 || st.shape[u] < 16 || st.shape[last] < 16 || numel(st.shape) < (int64_t(1) << 18)) continue;
                    for (int d = 0; d < last; ++d)
                        if (d != u && st.shape[d] > 1) ++nbatch;
                    if (nbatch > 3) continue;
                    {
                        // every 64x64 tile of every batch is one block along grid dimension x
                        int64_t blocks = ((st.shape[u] + 63) / 64) * ((st.shape[last] + 63) / 64);
                        for (int d = 0; d < last; ++d)
                            if (d != u && st.shape[d] > 1) blocks *= st.shape[d];
                        if (blocks > 0x7fffffff) continue;
                    }
                    // a dense copy of exactly this region that must be in memory anyway (Contigious, a kept view)
                    // is written by the transposing kernel itself; later readers of the region read that copy
                    const std::string region_key = std::to_string(pc.src.node->id) + "@" + stage_str(st);
                    Node* T = nullptr;
                    auto known = transposed.find(region_key);
                    if (known != transposed.end() && known->second->order < n->order) T = known->second;
                    if (!T && n->root && n->op == Op::COPY && t.single_full() && pc.view.st.size() == 1 && t.shape == st.shape &&
                        n->shape == st.shape) {
                        n->transpose = true;
                        n->transpose_u = u;
                        transposed[region_key] = n;
                        added = true;
                        continue;
                    }
                    if (!T) {
                        TRef region;
                        region.shape = st.shape;
                        Piece whole;
                        whole.lo.assign(st.shape.size(), 0);
                        whole.hi = st.shape;
                        whole.view.st = {st};
                        whole.src = pc.src;
                        region.pieces.push_back(whole);
                        T = new_node(Op::COPY, st.shape, {region}, pc.src.node->name + ".t", 0.f, true);
                        T->root = true;
                        T->transpose = true;
                        T->transpose_u = u;
                        T->order = std::min(T->order, n->order - 0.25);
                        transposed[region_key] = T;
                    }
                    pc.view.st.back() = contiguous_stage(st.shape);
                    pc.src = Src();
                    pc.src.kind = Src::NODE;
                    pc.src.node = T;
                    added = true;
                }
            }
        }
        if (added) order_nodes(rp);
    }

    // ---- 4. folded nodes used by several kernels: keep in memory when recomputing costs more
    void keep_shared_values(RegionPlan& rp) {
        auto& topo = rp.topo;
        std::map<Node*, std::set<std::string>> users;
        std::map<Node*, std::set<Node*>> bigleaves;
        for (Node* n : topo) {  // producers first
            if (in_mem(n)) continue;
            std::set<Node*>& bl = bigleaves[n];
            for_each_src(n, [&](Node* s, const Piece&, const TRef&) {
                if (in_mem(s)) { if (numel(s->shape) * 2 >= numel(n->shape)) bl.insert(s); }
                else bl.insert(bigleaves[s].begin(), bigleaves[s].end());
            });
        }
        for (size_t i = topo.size(); i-- > 0;) {  // consumers first
            Node* n = topo[i];
            std::set<std::string> mine;
            int64_t csr = 0, csc = 0;
            if (n->root && opt.fuse && colsum_source(n, csr, csc)) mine.insert("E" + std::to_string(csr * csc));
            else if (n->root) mine.insert(op_is_elw(n->op) ? "E" + std::to_string(numel(n->shape)) : "K" + std::to_string(n->id));
            else mine = users[n];
            if (!n->root && op_is_elw(n->op) && users[n].size() >= 2 && bigleaves[n].size() >= 3) {
                n->root = true;
                mine.clear();
                mine.insert("E" + std::to_string(numel(n->shape)));
            }
            for_each_src(n, [&](Node* s, const Piece&, const TRef&) {
                if (!in_mem(s)) users[s].insert(mine.begin(), mine.end());
            });
        }
    }

    // ---- 3a. A tensor reference with many pieces (a Concat of many values, or of many slices that do not continue one
    // another) costs its reader one predicated load per piece.  A reference with more pieces than the bound is cut,
    // by planes that no piece straddles (every Concat leaves one), into parts of at most that many pieces; a part with
    // more than one piece becomes a dense copy of its box, written by a kernel of its own, and the reference reads the
    // copies.  Repeated until the reference itself is narrow enough.
    TRef narrow_reference(const TRef& t, int64_t limit, double order, const std::string& name) {
        if ((int64_t)t.pieces.size() <= limit) return t;
        struct Part { Shape lo, hi; std::vector<const Piece*> pieces; };
        std::vector<Part> work, done;
        {
            Part whole;
            whole.lo.assign(t.shape.size(), 0);
            whole.hi = t.shape;
            for (const Piece& p : t.pieces) whole.pieces.push_back(&p);
            work.push_back(std::move(whole));
        }
        while (!work.empty()) {
            Part part = std::move(work.back());
            work.pop_back();
            if ((int64_t)part.pieces.size() <= limit) { done.push_back(std::move(part)); continue; }
            // the plane that divides the part's pieces most evenly
            int best_dim = -1;
            int64_t best_at = 0;
            size_t best_low = 0;
            for (size_t d = 0; d < t.shape.size(); ++d) {
                std::vector<int64_t> cuts;
                for (const Piece* p : part.pieces)
                    if (p->hi[d] < part.hi[d]) cuts.push_back(p->hi[d]);
                std::sort(cuts.begin(), cuts.end());
                cuts.erase(std::unique(cuts.begin(), cuts.end()), cuts.end());
                for (int64_t c : cuts) {
                    size_t low = 0;
                    bool clean = true;
                    for (const Piece* p : part.pieces) {
                        if (p->hi[d] <= c) ++low;
                        else if (p->lo[d] < c) { clean = false; break; }
                    }
                    if (!clean || low == 0 || low == part.pieces.size()) continue;
                    const size_t half = part.pieces.size() / 2;
                    auto off = [&](size_t v) { return v > half ? v - half : half - v; };
                    if (best_dim < 0 || off(low) < off(best_low)) { best_dim = (int)d; best_at = c; best_low = low; }
                }
            }
            if (best_dim < 0) { done.push_back(std::move(part)); continue; }  // no such plane: stays as wide as it is
            Part lo_part, hi_part;
            lo_part.lo = hi_part.lo = part.lo;
            lo_part.hi = hi_part.hi = part.hi;
            lo_part.hi[(size_t)best_dim] = best_at;
            hi_part.lo[(size_t)best_dim] = best_at;
            for (const Piece* p : part.pieces) (p->hi[(size_t)best_dim] <= best_at ? lo_part : hi_part).pieces.push_back(p);
            work.push_back(std::move(hi_part));
            work.push_back(std::move(lo_part));
        }
        if (done.size() < 2) return t;
        TRef o;
        o.shape = t.shape;
        for (const Part& part : done) {
            if (part.pieces.size() == 1) { o.pieces.push_back(*part.pieces[0]); continue; }
            TRef sub;
            for (size_t d = 0; d < t.shape.size(); ++d) sub.shape.push_back(part.hi[d] - part.lo[d]);
            for (const Piece* p : part.pieces) {
                Piece q = *p;
                for (size_t d = 0; d < t.shape.size(); ++d) { q.lo[d] -= part.lo[d]; q.hi[d] -= part.lo[d]; }
                sub.pieces.push_back(std::move(q));
            }
            Node* c = new_node(Op::COPY, sub.shape, {sub}, name + ".part");
            c->root = true;
            c->order = std::min(c->order, order - 0.5);
            Piece q;
            q.lo = part.lo;
            q.hi = part.hi;
            q.view.st.push_back(contiguous_stage(sub.shape));
            q.src.kind = Src::NODE;
            q.src.node = c;
            o.pieces.push_back(std::move(q));
        }
        std::sort(o.pieces.begin(), o.pieces.end(), [](const Piece& x, const Piece& y) { return x.lo < y.lo; });
        if (o.pieces.size() >= t.pieces.size()) return o;
        return narrow_reference(o, limit, order, name);
    }

    void narrow_references(RegionPlan& rp) {
        const int64_t limit = bound(opt.max_pieces);
        bool added = false;
        std::vector<Node*> work = rp.topo;
        for (size_t i = 0; i < work.size(); ++i) {
            Node* n = work[i];
            for (TRef& t : n->in) {
                if ((int64_t)t.pieces.size() <= limit) continue;
                const size_t before = arena.size();
                t = narrow_reference(t, limit, n->order, n->name);
                n->key.clear();
                // the copies' own operands are narrow by construction (at most `limit` pieces each)
                added = added || arena.size() != before;
            }
        }
        if (added) order_nodes(rp);
    }

    // ---- 4b. A kernel is bounded in what drives its register pressure.  A folded expression may load from at most
    // max_inline_sites places (a load site: one piece of a tensor reference onto a value in memory, reached along
    // one chain of views) and from at most max_inline_loads distinct values; a kernel may load from at most
    // max_kernel_sites places and name at most max_kernel_pointers buffers (operands and outputs of all its members).
    // Slices spelled as one Index per line joined by Concats, summed up by a backward pass, fold into expressions
    // with thousands of predicated loads of as many operands: the compiler needs minutes for the branches.  A pointer
    // takes two scalar registers and the lane mask of every predicate two more, of the 102 a wavefront has: kernels
    // of 60 and more buffers used all 512 vector registers, kept some 200 scalar registers in lanes of vector
    // registers and spilled vector registers to scratch on top, and three of them were seen to produce wrong elements.
    // Walking producers first, a value whose expression would exceed a limit gets a buffer and a kernel of its own
    // (its largest folded operands first, then itself), so that its consumers read it as one operand.
    static uint64_t mix(uint64_t h, uint64_t v) {
        h ^= v + 0x9e3779b97f4a7c15ull + (h << 6) + (h >> 2);
        return h;
    }
    static uint64_t hash_str(const std::string& s) {
        uint64_t h = 1469598103934665603ull;
        for (unsigned char c : s) { h ^= c; h *= 1099511628211ull; }
        return h;
    }
    // load sites of the expression of `n` evaluated in place, given those of the folded values below it
    std::set<uint64_t> expression_sites(Node* n, const std::map<Node*, std::set<uint64_t>>& below) {
        std::set<uint64_t> out;
        std::set<std::string> seen_refs;
        for (const TRef& t : n->in) {
            if (!seen_refs.insert(tref_str(t)).second) continue;  // x * x: one set of loads
            for (const Piece& p : t.pieces) {
                if (p.src.kind != Src::NODE) continue;
                Node* s = p.src.node;
                const bool ident = identity_piece(p, t) && numel(s->shape) == numel(n->shape);
                uint64_t path = 0;
                if (!ident) {
                    std::string v = shape_str(p.lo) + shape_str(p.hi);
                    for (const Stage& st : p.view.st) v += stage_str(st);
                    path = hash_str(v);
                }
                if (in_mem(s)) out.insert(mix((uint64_t)s->id + 1, path));
                else {
                    auto it = below.find(s);
                    if (it == below.end()) continue;
                    for (uint64_t k : it->second) out.insert(ident ? k : mix(k, path));
                }
            }
        }
        return out;
    }

    void cut_long_expressions(RegionPlan& rp) {
        if (!opt.fuse) return;
        const int64_t max_loads = bound(opt.max_inline_loads), max_sites = bound(opt.max_inline_sites);
        std::map<Node*, std::vector<Node*>> operands;  // per folded value: the in-memory values its expression reads (sorted)
        auto& sites = rp.sites;
        auto gather = [&](Node* n) {
            std::vector<Node*> u;
            for_each_src(n, [&](Node* s, const Piece&, const TRef&) {
                if (in_mem(s)) u.push_back(s);
                else { auto& o = operands[s]; u.insert(u.end(), o.begin(), o.end()); }
            });
            std::sort(u.begin(), u.end());
            u.erase(std::unique(u.begin(), u.end()), u.end());
            return u;
        };
        for (Node* n : rp.topo) {
            if (op_is_leaf(n->op) || numel(n->shape) == 0) continue;
            std::vector<Node*> u = gather(n);
            std::set<uint64_t> st = expression_sites(n, sites);
            auto too_long = [&] { return (int64_t)u.size() > max_loads || (int64_t)st.size() > max_sites; };
            if (too_long()) {
                std::vector<std::pair<size_t, Node*>> parts;
                for_each_src(n, [&](Node* s, const Piece&, const TRef&) {
                    if (!in_mem(s) && op_is_elw(s->op) && numel(s->shape) > 0) parts.push_back({sites[s].size(), s});
                });
                std::sort(parts.begin(), parts.end(), [](const std::pair<size_t, Node*>& x, const std::pair<size_t, Node*>& y) {
                    return x.first != y.first ? x.first > y.first : x.second->order < y.second->order;
                });
                parts.erase(std::unique(parts.begin(), parts.end()), parts.end());
                for (auto& pt : parts) {
                    if (!too_long()) break;
                    if (pt.second->root || pt.first <= 1) continue;
                    pt.second->root = true;
                    operands.erase(pt.second);
                    u = gather(n);
                    st = expression_sites(n, sites);
                }
                if (too_long() && op_is_elw(n->op)) n->root = true;
            }
            if (!in_mem(n)) operands[n] = std::move(u);
            sites[n] = std::move(st);
        }
    }

    // the buffers a kernel of this group (with one more member, if given) names: distinct operands, outputs, sums
    int64_t group_pointers(RegionPlan& rp, const Group& G, Node* extra = nullptr) {
        std::set<Node*> u;
        for (Node* m : G.members)
            for (auto& kv : rp.reads[m]) u.insert(kv.first);
        if (extra)
            for (auto& kv : rp.reads[extra]) u.insert(kv.first);
        return (int64_t)(u.size() + G.members.size() + (extra ? 1 : 0) + G.colsums.size() + G.rowsums.size());
    }
    // the places a kernel of this group (with one more member, if given) loads from
    int64_t group_sites(RegionPlan& rp, const Group& G, Node* extra = nullptr) {
        std::set<uint64_t> u;
        auto add = [&](Node* m) {
            auto it = rp.sites.find(m);
            if (it != rp.sites.end()) u.insert(it->second.begin(), it->second.end());
        };
        for (Node* m : G.members) add(m);
        for (auto& cs : G.riders()) add(cs.first);
        if (extra) add(extra);
        return (int64_t)u.size();
    }
    bool group_fits(RegionPlan& rp, const Group& G, Node* extra) {
        return group_pointers(rp, G, extra) <= bound(opt.max_kernel_pointers) && group_sites(rp, G, extra) <= bound(opt.max_kernel_sites);
    }
    // the pass with sums runs 1024 threads a block, which leaves a lane 128 vector registers: a pass that loads from
    // more places or names more buffers than this would spill them, so its sums get kernels of their own
    bool can_carry_sums(RegionPlan& rp, const Group& G, Node* value = nullptr) {
        if (tight()) return false;
        return group_pointers(rp, G) < bound(opt.max_carrier_pointers) && group_sites(rp, G, value) <= bound(opt.max_carrier_sites);
    }

    void form_groups(RegionPlan& rp) {
        auto& topo = rp.topo;
        auto& reads = rp.reads;
        auto& folded_in = rp.folded_in;
        auto& groups = rp.groups;
        auto& group_of = rp.group_of;
        // kernels run in program order: it is a valid topological order, and it keeps in-place updates
        // after the reads of the old value that precede them in the program
        std::vector<Node*> roots;
        for (Node* n : topo)
            if (n->root && !op_is_leaf(n->op)) roots.push_back(n);
        std::stable_sort(roots.begin(), roots.end(), [](Node* a, Node* b) { return a->order < b->order; });
        for (Node* r : roots) collect_reads(r, reads[r], &folded_in[r]);
        for (Node* r : roots) {
            int chosen = -1;
            if (op_is_elw(r->op) && opt.fuse && !r->transpose) {
                for (int g = (int)groups.size() - 1; g >= 0; --g) {
                    if (groups[g].kind != Group::ELW || groups[g].n != numel(r->shape)) continue;
                    if (!group_fits(rp, groups[g], r)) continue;  // a kernel's size is bounded too
                    bool ok = true;
                    for (auto& rd : reads[r]) {
                        if (op_is_leaf(rd.first->op)) continue;
                        int gd = group_of[rd.first];
                        if (gd == g) { if (!rd.second) { ok = false; break; } }
                        else if (gd > g) { ok = false; break; }
                    }
                    if (ok) { chosen = g; break; }
                }
            }
            if (chosen < 0) {
                Group g;
                g.n = numel(r->shape);
                g.kind = op_is_reduce(r->op) ? Group::SUM : (r->op == Op::DOT ? Group::DOT : (r->op == Op::ATTN ? Group::ATTN : (r->transpose ? Group::TRANSPOSE : Group::ELW)));
                groups.push_back(g);
                chosen = (int)groups.size() - 1;
            }
            groups[chosen].members.push_back(r);
            group_of[r] = chosen;
        }
        for (auto& w : rp.wanted) rp.home_of[w.second] = w.first;
    }

    // does kernel group H read `what` from memory?
    bool group_reads(RegionPlan& rp, const Group& H, Node* what) {
        auto& reads = rp.reads;
        std::vector<Node*> rs = H.members;
        for (Node* sd : H.side) rs.push_back(sd);
        for (Node* ep : H.epi) rs.push_back(ep);
        for (Node* m : rs)
            if (reads[m].count(what)) return true;
        for (auto& cs : H.riders()) {
            std::map<Node*, bool> er;
            if (in_mem(cs.first)) er[cs.first] = true;
            else collect_reads(cs.first, er);
            if (er.count(what)) return true;
        }
        return false;
    }

    // The element-wise group that can run as the epilogue of group g, whose result P has n_elems elements: the
    // first later group that reads P, provided it is element-wise over n_elems, reads P element for element only,
    // and may be moved up to g's position: everything else it reads exists before g runs, and no group in between
    // reads the old contents of a buffer it overwrites in place.  -1 if there is none.
    int find_epilogue(RegionPlan& rp, size_t g, Node* P, int64_t n_elems) {
        auto& reads = rp.reads;
        auto& groups = rp.groups;
        auto& group_of = rp.group_of;
        const auto& home_of = rp.home_of;
        auto reads_node = [&](const Group& H, Node* what) { return group_reads(rp, H, what); };
        if (tight()) return -1;  // a region asked to keep its kernels small fuses nothing across kernel kinds
        for (size_t ge = g + 1; ge < groups.size(); ++ge) {
            Group& E = groups[ge];
            if (E.dead) continue;
            if (!reads_node(E, P)) continue;
            if (E.kind != Group::ELW || E.rides() || E.n != n_elems) return -1;
            for (Node* m : E.members) {
                auto it = reads[m].find(P);
                if (it != reads[m].end() && !it->second) return -1;
                for (auto& rd : reads[m]) {
                    if (rd.first == P) continue;
                    auto gi = group_of.find(rd.first);
                    if (gi != group_of.end() && gi->second >= (int)g && gi->second != (int)ge) return -1;
                }
                auto ho = home_of.find(m);
                if (ho == home_of.end()) continue;
                auto li = livein.find(ho->second);
                if (li == livein.end()) continue;
                for (size_t h = g + 1; h < ge; ++h)
                    if (!groups[h].dead && reads_node(groups[h], li->second)) return -1;
            }
            return (int)ge;
        }
        return -1;
    }

    // ---- 5b. column sums ride along with the element-wise pass that computes their operand
    void attach_column_sums(RegionPlan& rp) {
        auto& reads = rp.reads;
        auto& folded_in = rp.folded_in;
        auto& groups = rp.groups;
        auto& group_of = rp.group_of;
        for (size_t gs = 0; gs < groups.size(); ++gs) {
            if (groups[gs].kind != Group::SUM) continue;
            Node* S = groups[gs].members[0];
            int64_t R = 0, C = 0;
            Node* E = colsum_source(S, R, C);
            if (!E) continue;
            int target = -1;
            for (size_t g = 0; g < groups.size() && target < 0; ++g) {
                Group& G = groups[g];
                if (G.dead || G.kind != Group::ELW || G.n != R * C || !can_carry_sums(rp, G, E)) continue;
                if (G.rides() && (G.cs_rows != R || G.cs_cols != C)) continue;
                for (Node* m : G.members)
                    if (m == E || folded_in[m].count(E)) { target = (int)g; break; }
            }
            if (target < 0) {
                // no pass computes E itself; one that already loads, element for element, everything E is made
                // of can still produce the sum without reading anything more (x.sum(0) next to dx = f(x))
                std::map<Node*, bool> er;
                if (in_mem(E)) er[E] = true;
                else collect_reads(E, er);
                bool ident = !er.empty();
                for (auto& kv : er) ident = ident && kv.second;
                for (size_t g = 0; ident && g < groups.size() && target < 0; ++g) {
                    Group& G = groups[g];
                    if (G.dead || G.kind != Group::ELW || G.n != R * C || !can_carry_sums(rp, G, E)) continue;
                    if (G.rides() && (G.cs_rows != R || G.cs_cols != C)) continue;
                    bool all = true;
                    for (auto& kv : er) {
                        bool found = false;
                        for (Node* m : G.members) {
                            auto it = reads[m].find(kv.first);
                            if (it != reads[m].end() && it->second) { found = true; break; }
                        }
                        all = all && found;
                    }
                    if (all) target = (int)g;
                }
            }
            if (target < 0) continue;
            // everything that reads S must run after the pass that now produces it
            bool ok = true;
            for (size_t g = 0; g < groups.size(); ++g) {
                if (groups[g].dead) continue;
                for (Node* m : groups[g].members)
                    if (reads[m].count(S) && (int)g <= target) ok = false;
            }
            if (!ok) continue;
            groups[target].colsums.push_back({E, S});
            groups[target].cs_rows = R;
            groups[target].cs_cols = C;
            groups[gs].dead = true;
            group_of[S] = target;
        }
    }

    // ---- 5b'. row sums ride along too: a plain row sum over an element-wise value E of [rows, cols] is produced by an
    // element-wise pass over the same space that computes E anyway or already loads, element for element, everything
    // E is made of (s = (x*x).sum(1) next to dx = f(x): x is read once for both).  Every wavefront of the 2-D layout
    // adds up its run of a row; a second pass adds a row's runs.  When the pass comes later in the program than the
    // sum did, it is moved up to the sum's place, which needs everything it reads to exist there already and nobody in
    // between to read the old contents of a buffer it overwrites.
    void attach_row_sums(RegionPlan& rp) {
        auto& reads = rp.reads;
        auto& folded_in = rp.folded_in;
        auto& groups = rp.groups;
        auto& group_of = rp.group_of;
        for (size_t gs = 0; gs < groups.size(); ++gs) {
            if (groups[gs].dead || groups[gs].kind != Group::SUM || groups[gs].members.size() != 1 || !groups[gs].side.empty()) continue;
            Node* S = groups[gs].members[0];
            int64_t R = 0, C = 0;
            Node* E = rowsum_source(S, R, C);
            if (!E) continue;
            std::map<Node*, bool> er;
            if (in_mem(E)) er[E] = true;
            else collect_reads(E, er);
            bool ident = !er.empty();
            for (auto& kv : er) ident = ident && kv.second;
            int target = -1;
            for (size_t g = 0; g < groups.size() && target < 0; ++g) {
                Group& G = groups[g];
                if (g == gs || G.dead || G.tiled || G.kind != Group::ELW || G.n != R * C || !G.side.empty() || !can_carry_sums(rp, G, E)) continue;
                if (G.rides() && (G.cs_rows != R || G.cs_cols != C)) continue;
                bool computes = false;
                for (Node* m : G.members) computes = computes || m == E || folded_in[m].count(E);
                bool loads_all = ident;
                for (auto& kv : er) {
                    if (!loads_all) break;
                    bool found = false;
                    for (Node* m : G.members) {
                        auto it = reads[m].find(kv.first);
                        if (it != reads[m].end() && it->second) { found = true; break; }
                    }
                    loads_all = found;
                }
                if (!computes && !loads_all) continue;
                // the pass must not need the sum itself, directly or through what it reads
                bool independent = true;
                for (Node* m : G.members) independent = independent && !reads[m].count(S);
                for (auto& cs : G.riders()) {
                    std::map<Node*, bool> cr;
                    if (in_mem(cs.first)) cr[cs.first] = true;
                    else collect_reads(cs.first, cr);
                    independent = independent && !cr.count(S);
                }
                if (!independent) continue;
                if (g > gs) {
                    // moving the pass up to the sum's place
                    bool movable = true;
                    auto early_enough = [&](const std::map<Node*, bool>& rd) {
                        for (auto& kv : rd) {
                            if (op_is_leaf(kv.first->op)) continue;
                            auto it = group_of.find(kv.first);
                            if (it != group_of.end() && it->second >= (int)gs && it->second != (int)g) movable = false;
                        }
                    };
                    std::vector<Node*> produced = G.members;
                    for (Node* m : G.members) early_enough(reads[m]);
                    for (auto& cs : G.riders()) {
                        std::map<Node*, bool> cr;
                        if (in_mem(cs.first)) cr[cs.first] = true;
                        else collect_reads(cs.first, cr);
                        early_enough(cr);
                        produced.push_back(cs.second);
                    }
                    for (Node* m : produced) {
                        auto ho = rp.home_of.find(m);
                        if (ho == rp.home_of.end()) continue;
                        auto li = livein.find(ho->second);
                        if (li == livein.end()) continue;
                        for (size_t h = gs; h < g; ++h)
                            if (!groups[h].dead && group_reads(rp, groups[h], li->second)) movable = false;
                    }
                    // whatever reads a result of the pass keeps coming after it; whatever the pass overwrites in place
                    // was checked above
                    if (!movable) continue;
                }
                target = (int)g;
            }
            if (target < 0) continue;
            if (target > (int)gs) {
                // everything that reads S runs after gs already; the pass takes the place right after the (now dead) sum
                Group moved = std::move(groups[(size_t)target]);
                groups.erase(groups.begin() + target);
                groups.insert(groups.begin() + (std::ptrdiff_t)gs + 1, std::move(moved));
                for (auto& kv : group_of) {
                    if (kv.second == target) kv.second = (int)gs + 1;
                    else if (kv.second > (int)gs && kv.second < target) kv.second += 1;
                }
                target = (int)gs + 1;
            } else {
                // the sum is produced earlier than it was: its readers all come after gs, hence after the pass
            }
            Group& G = groups[(size_t)target];
            G.rowsums.push_back({E, S});
            G.cs_rows = R;
            G.cs_cols = C;
            groups[gs].dead = true;
            group_of[S] = target;
        }
    }

    // ---- 5b''. Row chains: a row reduction whose result the following kernels use row by row -- a softmax (max, the
    // sum of the exponentials, the division), a LayerNorm (mean, the centred value, the variance, the scaling), the
    // backward pass of either -- runs as one kernel in which a wavefront or a block owns a row (gen_rowchain_kernel):
    // the row is read from memory once, and what only the chain itself uses is never written.  A chain is a run of
    // consecutive kernels over one [V, R] space: plain row reductions, element-wise kernels of V * R elements and
    // element-wise kernels of V elements, each of which reads what the chain produced before it only at its own row
    // (the same element of a full-size value, element x of a per-row value).
    bool chain_reads_rowwise(RegionPlan& rp, Node* m, const std::set<Node*>& produced, int64_t V, int64_t R) {
        bool ok = true;
        std::function<bool(Node*)> reaches = [&](Node* n) {
            bool r = false;
            for_each_src(n, [&](Node* s, const Piece&, const TRef&) {
                if (r) return;
                if (produced.count(s)) r = true;
                else if (!in_mem(s)) r = reaches(s);
            });
            return r;
        };
        std::set<std::pair<Node*, bool>> seen;
        std::function<void(Node*, bool)> walk = [&](Node* n, bool row_level) {
            for (const TRef& t : n->in) {
                for (const Piece& p : t.pieces) {
                    if (!ok || p.src.kind != Src::NODE) continue;
                    Node* s = p.src.node;
                    const bool mine = produced.count(s) != 0;
                    if (!mine && in_mem(s)) continue;                       // an operand from outside: read however it likes
                    const RowAccess ra = row_access(t, V, R, row_level);
                    const int64_t ns = numel(s->shape);
                    const bool aligned = (ra == RowAccess::FULL && ns == V * R) || (ra == RowAccess::ROW && ns == V);
                    if (mine) { if (!aligned) ok = false; continue; }
                    // a folded value: followed at the coordinates it is evaluated at, if those are a row's
                    if (aligned) { if (seen.insert({s, ra == RowAccess::ROW}).second) walk(s, ra == RowAccess::ROW); }
                    else if (reaches(s)) ok = false;
                }
            }
        };
        walk(m, !op_is_reduce(m->op) && numel(m->shape) == V);
        (void)rp;
        return ok;
    }

    void form_row_chains(RegionPlan& rp) {
        if (tight()) return;
        auto& groups = rp.groups;
        auto& reads = rp.reads;
        auto plain_reduction = [&](const Group& H, int64_t& V, int64_t& R) {
            if (H.dead || H.kind != Group::SUM || H.members.size() != 1 || !H.side.empty() || !H.epi.empty() || H.lead >= 0) return false;
            const Node* n = H.members[0];
            if (!op_is_reduce(n->op) || n->in.size() != 1 || n->in[0].shape.size() != 2) return false;
            V = n->in[0].shape[0];
            R = n->in[0].shape[1];
            return true;
        };
        for (size_t g0 = 0; g0 < groups.size(); ++g0) {
            int64_t V = 0, R = 0;
            if (!plain_reduction(groups[g0], V, R) || V < 2 || !rowchain_fits(V, R)) continue;
            std::vector<size_t> run;
            std::set<Node*> produced, streamed;
            auto acceptable = [&](const Group& H) {
                int64_t v2 = 0, r2 = 0;
                if (H.kind == Group::SUM) {
                    if (!plain_reduction(H, v2, r2) || v2 != V || r2 != R) return false;
                } else if (H.kind == Group::ELW) {
                    if (H.rides() || H.tiled || !H.side.empty() || H.lead >= 0 || (H.n != V * R && H.n != V)) return false;
                } else {
                    return false;
                }
                for (Node* m : H.members)
                    if (!chain_reads_rowwise(rp, m, produced, V, R)) return false;
                // it belongs to the chain if it uses what the chain made, or streams a full-size operand the chain
                // streams anyway; independent work on other data stays a kernel of its own
                if (produced.empty()) return true;
                for (Node* m : H.members)
                    for (auto& rd : reads[m])
                        if (produced.count(rd.first) || (streamed.count(rd.first) && numel(rd.first->shape) * 2 >= V * R)) return true;
                return false;
            };
            for (size_t h = g0; h < groups.size(); ++h) {
                if (groups[h].dead) continue;
                if (!acceptable(groups[h])) break;
                run.push_back(h);
                for (Node* m : groups[h].members) {
                    produced.insert(m);
                    for (auto& rd : reads[m]) streamed.insert(rd.first);
                }
            }
            // the chain pays when something that works on whole rows uses what the chain made before it; it ends with
            // the last such kernel (per-row arithmetic that follows gains nothing from sharing the launch)
            auto members_of = [&](size_t upto) {
                std::vector<Node*> ms;
                for (size_t i = 0; i < upto; ++i) {
                    std::vector<Node*> part = groups[run[i]].members;
                    std::stable_sort(part.begin(), part.end(), [](Node* a, Node* b) { return a->order < b->order; });
                    ms.insert(ms.end(), part.begin(), part.end());
                }
                return ms;
            };
            size_t len = run.size();
            for (; len >= 2; --len) {
                std::vector<Node*> ms = members_of(len);
                std::set<Node*> earlier(ms.begin(), ms.end());
                for (Node* m : groups[run[len - 1]].members) earlier.erase(m);
                Node* tail = ms.back();
                bool uses = false;
                if (op_is_reduce(tail->op) || numel(tail->shape) == V * R)
                    for (Node* m : groups[run[len - 1]].members)
                        for (auto& rd : reads[m]) uses = uses || earlier.count(rd.first) != 0;
                if (!uses) continue;
                // the kernel's size is bounded like any other's
                Group probe;
                probe.members = ms;
                if (!group_fits(rp, probe, nullptr)) continue;
                // and it has to generate (a reference the generator cannot follow ends the attempt, not the lowering)
                RowChainSpec spec;
                spec.V = V;
                spec.R = R;
                spec.name = "probe";
                spec.order = ms;
                for (Node* m : ms) spec.stored.insert(m);
                try {
                    (void)gen_rowchain_kernel(spec);
                } catch (const Error&) {
                    continue;
                }
                break;
            }
            if (len < 2) continue;
            Group& G = groups[g0];
            G.kind = Group::ROWCHAIN;
            G.members = members_of(len);
            G.n = V * R;
            G.cs_rows = V;
            G.cs_cols = R;
            for (size_t i = 1; i < len; ++i) groups[run[i]].dead = true;
            for (Node* m : G.members) rp.group_of[m] = (int)g0;
        }
    }

    // ---- 5c. a row sum over an element-wise value produced by the kernel just before it: the
    // reduction computes, stores and sums that value in one pass
    void attach_row_sum_operands(RegionPlan& rp) {
        auto& groups = rp.groups;
        auto& group_of = rp.group_of;
        if (tight()) return;
        for (size_t gs = 1; gs < groups.size(); ++gs) {
            Group& GS = groups[gs];
            if (GS.dead || GS.kind != Group::SUM) continue;
            Node* S = GS.members[0];
            const TRef& t = S->in[0];
            if (!t.single_full() || t.pieces[0].src.kind != Src::NODE) continue;
            Node* E = t.pieces[0].src.node;
            if (!E->root || !op_is_elw(E->op) || E->transpose || !identity_piece(t.pieces[0], t)) continue;
            if (numel(E->shape) != numel(t.shape) || t.shape[1] % 4 != 0 || t.shape[1] < 256) continue;
            int ge = group_of[E];
            int prev = (int)gs - 1;
            while (prev >= 0 && groups[prev].dead) --prev;
            if (ge != prev) continue;
            Group& GE = groups[ge];
            if (GE.kind != Group::ELW || GE.members.size() != 1 || GE.rides()) continue;
            GS.side.push_back(E);
            GE.dead = true;
            group_of[E] = (int)gs;
        }
    }

    // ---- 5c'. a dense transposed copy that a single element-wise kernel reads is not made at all when that kernel
    // can fetch the operand's tiles through LDS itself (gen_elw_kernel then answers with its tiled form): the
    // copy's round trip through memory -- twice the operand's size -- goes away
    void fold_transposed_copies(RegionPlan& rp) {
        auto& wanted_nodes = rp.wanted_nodes;
        auto& reads = rp.reads;
        auto& folded_in = rp.folded_in;
        auto& groups = rp.groups;
        auto& group_of = rp.group_of;
        for (size_t tg = 0; tg < groups.size(); ++tg) {
            Group& TG = groups[tg];
            if (TG.dead || TG.kind != Group::TRANSPOSE) continue;
            Node* T = TG.members[0];
            if (wanted_nodes.count(T) || T->force_root) continue;  // has to be in memory for its own sake
            int consumer = -1;
            bool fusable = true;
            for (size_t g = 0; g < groups.size() && fusable; ++g) {
                if (groups[g].dead || g == tg) continue;
                bool rd = false;
                for (Node* m : groups[g].members) rd = rd || reads[m].count(T);
                for (Node* sd : groups[g].side) rd = rd || reads[sd].count(T);
                for (auto& cs : groups[g].riders()) {
                    std::map<Node*, bool> er;
                    if (in_mem(cs.first)) er[cs.first] = true;
                    else collect_reads(cs.first, er);
                    if (er.count(T)) fusable = false;
                }
                if (!rd) continue;
                if (consumer >= 0 || groups[g].kind != Group::ELW || groups[g].rides() || !groups[g].side.empty() || g < tg) fusable = false;
                consumer = (int)g;
            }
            if (!fusable || consumer < 0) continue;
            Group& G = groups[consumer];
            T->root = false;
            std::map<Node*, std::map<Node*, bool>> saved_reads;
            std::map<Node*, std::set<Node*>> saved_folded;
            for (Node* m : G.members) {
                saved_reads[m] = reads[m];
                saved_folded[m] = folded_in[m];
                reads[m].clear();
                folded_in[m].clear();
                collect_reads(m, reads[m], &folded_in[m]);
            }
            ElwKernelSpec probe_spec;
            probe_spec.outputs = G.members;
            probe_spec.name = "probe";
            bool tiled = false;
            try {
                tiled = gen_elw_kernel(probe_spec, std::set<const Node*>(G.members.begin(), G.members.end())).kind == "elw_tiled";
            } catch (const Error&) {
                tiled = false;
            }
            if (tiled) {
                G.tiled = true;
                TG.dead = true;
                group_of.erase(T);  // T is no kernel's product any more: its consumer computes it in place
            } else {
                T->root = true;
                for (Node* m : G.members) { reads[m] = saved_reads[m]; folded_in[m] = saved_folded[m]; }
            }
        }
    }

    // ---- 5d. matrix-core products of one shape that each fill only part of the chip and do not depend on one
    // another (the per-head projections, scores and weighted values of multi-head attention, and their
    // gradients) become one grouped launch.  Products are independent when they sit at the same depth, counted
    // in products along the longest chain of dependencies; ordering the kernels by that depth, products last
    // within a depth, puts everything such a set reads before all of it and everything that reads it after.
    // Dependencies are the values a kernel reads plus, for a kernel that overwrites an id's buffer, the earlier
    // kernels that still read the id's old contents.  Regions without such a set keep program order.
    void group_independent_products(RegionPlan& rp) {
        auto& groups = rp.groups;
        // a product that fills the chip by itself gives up an epilogue only for nothing: it stays out of grouped
        // launches when an element-wise consumer could run on its accumulators
        auto keeps_epilogue = [&](int g) {
            Node* D = groups[g].members[0];
            const int64_t M = D->shape[0], N = D->shape[1];
            if (((M + 127) / 128) * ((N + 127) / 128) < 256) return false;
            return find_epilogue(rp, (size_t)g, D, numel(D->shape)) >= 0;
        };
        group_products(groups, rp.group_of, rp.reads, rp.home_of, [&](const Group& H, Node* what) { return group_reads(rp, H, what); }, keeps_epilogue);

    }

    // ---- 6. generate code per group (no buffers needed yet)
    void generate_kernels(RegionPlan& rp) {
        auto& reads = rp.reads;
        auto& groups = rp.groups;
        auto& group_of = rp.group_of;
        auto& gks = rp.gks;
        auto& greads = rp.greads;
        const auto& home_of = rp.home_of;
        gks.assign(groups.size(), GroupKernels());
        greads.assign(groups.size(), {});
        for (size_t g = 0; g < groups.size(); ++g) {
            Group& G = groups[g];
            if (G.dead) continue;
            std::set<const Node*> members(G.members.begin(), G.members.end());
            std::vector<Node*> readers = G.members;
            for (Node* sd : G.side) { members.insert(sd); readers.push_back(sd); }
            for (Node* m : readers)
                for (auto& rd : reads[m]) {
                    if (members.count(rd.first)) continue;
                    auto it = greads[g].find(rd.first);
                    if (it == greads[g].end()) greads[g][rd.first] = rd.second;
                    else it->second = it->second && rd.second;
                }
            std::string name = strf("k%d_%s", kernel_counter++, G.members[0]->name.empty() ? "t" : G.members[0]->name.c_str());
            for (char& ch : name) if (!isalnum((unsigned char)ch) && ch != '_') ch = '_';
            if (G.kind == Group::ELW) {
                ElwKernelSpec spec;
                spec.outputs = G.members;
                spec.name = name;
                spec.rows = G.cs_rows;
                spec.cols = G.cs_cols;
                if (G.rides()) {
                    G.cs_streams = (int)G.members.size();
                    for (auto& rd : greads[g])
                        if (numel(rd.first->shape) * 2 >= G.cs_rows * G.cs_cols) ++G.cs_streams;
                    spec.streams = G.cs_streams;
                }
                for (auto& cs : G.colsums) {
                    // partial sums [tiles][cols], added by the fixed second-pass kernel
                    const int64_t tiles = elw_colsum_tiles(G.cs_rows, G.cs_cols, G.cs_streams);
                    Node* S = cs.second;
                    Node* partial = new_node(Op::COPY, Shape{tiles, G.cs_cols}, {}, S->name + ".partial", 0.f, false);
                    partial->root = true;
                    spec.colsums.push_back({cs.first, partial});
                    gks[g].extra_nodes.push_back(partial);
                }
                for (auto& rs : G.rowsums) {
                    // one partial sum per (row, run of 256 columns), added by the fixed second-pass kernel
                    const int64_t runs = elw_rowsum_runs(G.cs_cols);
                    Node* S = rs.second;
                    Node* partial = new_node(Op::COPY, Shape{G.cs_rows, runs}, {}, S->name + ".runs", 0.f, false);
                    partial->root = true;
                    spec.rowsums.push_back({rs.first, partial});
                    gks[g].row_partials.push_back(partial);
                }
                gks[g].k = gen_elw_kernel(spec, members);
                gks[g].spec_kind = 1;
                gks[g].elw_spec = spec;
                gks[g].spec_members = members;
            } else if (G.kind == Group::DOT) {
                // the element-wise group scheduled right after a matrix-core product, if all it needs from the
                // product is the result element for element, runs on the accumulators before they are stored (the
                // reference's DotProd + ELW fusion, src/kernel/fusion/dp_elw.rs:13-149); the product itself is
                // written only if something else still reads it
                Node* D = G.members[0];
                DotLaunchPlan dpl;
                const bool grouped = G.members.size() > 1;  // one launch for all of them: whole k, no epilogue
                if (dot_uses_mfma(D) && !grouped) dpl = plan_dot(D);
                int nx = (grouped || dpl.splits > 1 || !opt.fuse || !dot_uses_mfma(D)) ? -1 : find_epilogue(rp, g, D, numel(D->shape));
                if (nx >= 0) {
                    // an epilogue streams its other operands in the accumulator layout (32 floats of a row per half
                    // wave); with many of them (a sum over all heads' gradients) a separate element-wise pass, with
                    // 128-bit accesses, is faster than the product kernel held up by them
                    std::set<Node*> big;
                    for (Node* m : groups[nx].members)
                        for (auto& rd : reads[m])
                            if (rd.first != D && numel(rd.first->shape) * 2 >= numel(D->shape)) big.insert(rd.first);
                    if (big.size() > 8) nx = -1;
                }
                if (grouped) {
                    const DotLaunchPlan gpl = plan_dot_group(D, (int)G.members.size());
                    if (gpl.splits > 1) {
                        Node* partial = new_node(Op::COPY, Shape{(int64_t)G.members.size() * gpl.splits, numel(D->shape)}, {},
                                                 D->name + ".slices", 0.f, false);
                        partial->root = true;
                        gks[g].extra_nodes.push_back(partial);
                    }
                } else if (dpl.splits > 1) {
                    Node* partial = new_node(Op::COPY, Shape{dpl.splits, numel(D->shape)}, {}, D->name + ".slices", 0.f, false);
                    partial->root = true;
                    gks[g].extra_nodes.push_back(partial);
                } else if (nx >= 0) {
                    {
                        gks[g].dot_epi = gen_dot_epilogue(D, groups[nx].members);
                        G.epi = groups[nx].members;
                        groups[nx].dead = true;
                        std::set<Node*> own(G.epi.begin(), G.epi.end());
                        own.insert(D);
                        for (Node* m : G.epi) {
                            group_of[m] = (int)g;
                            for (auto& rd : reads[m]) {
                                if (own.count(rd.first)) continue;
                                auto it = greads[g].find(rd.first);
                                if (it == greads[g].end()) greads[g][rd.first] = rd.second;
                                else it->second = it->second && rd.second;
                            }
                        }
                        // is the product itself still needed in memory?
                        bool needed = home_of.count(D) != 0;
                        for (size_t g2 = 0; g2 < groups.size() && !needed; ++g2) {
                            if (groups[g2].dead || g2 == g) continue;
                            std::vector<Node*> rs = groups[g2].members;
                            for (Node* sd : groups[g2].side) rs.push_back(sd);
                            for (Node* ep : groups[g2].epi) rs.push_back(ep);
                            for (Node* m : rs)
                                if (reads[m].count(D)) needed = true;
                            for (auto& cs : groups[g2].riders()) {
                                std::map<Node*, bool> er;
                                if (in_mem(cs.first)) er[cs.first] = true;
                                else collect_reads(cs.first, er);
                                if (er.count(D)) needed = true;
                            }
                        }
                        gks[g].dot_store = needed;
                    }
                }
            } else if (G.kind == Group::ROWCHAIN) {
                // a member is written to memory only if an id holds it or a kernel outside the chain reads it
                RowChainSpec spec;
                spec.V = G.cs_rows;
                spec.R = G.cs_cols;
                spec.name = name;
                spec.order = G.members;
                for (Node* m : G.members) {
                    bool needed = home_of.count(m) != 0;
                    for (size_t g2 = 0; g2 < groups.size() && !needed; ++g2)
                        if (g2 != g && !groups[g2].dead && group_reads(rp, groups[g2], m)) needed = true;
                    if (needed) spec.stored.insert(m);
                    else G.unstored.insert(m);
                }
                gks[g].k = gen_rowchain_kernel(spec);
            } else if (G.kind == Group::SUM) {
                ReduceKernelSpec spec;
                spec.node = G.members[0];
                spec.name = name;
                spec.side_outputs = G.side;
                // the element-wise group scheduled right after this reduction, if all it needs from it is the result
                // element for element, becomes the reduction's epilogue (the reference's Reduce + ELW fusion,
                // src/kernel/fusion/reduce_elw.rs:12-143)
                const int ge = opt.fuse ? find_epilogue(rp, g, G.members[0], numel(G.members[0]->shape)) : -1;
                if (ge >= 0) spec.epilogue_outputs = groups[ge].members;
                gks[g].k = gen_reduce_kernel(spec);
                gks[g].spec_kind = 2;
                gks[g].red_spec = spec;
                ADHIP_CHECK(G.side.empty() || gks[g].k.side_done, "internal: row reduction did not take over its operand's store");
                if (ge >= 0 && gks[g].k.epilogue_done) {
                    G.epi = groups[ge].members;
                    groups[ge].dead = true;
                    std::set<Node*> own(G.epi.begin(), G.epi.end());
                    own.insert(G.members[0]);
                    for (Node* m : G.epi) {
                        group_of[m] = (int)g;
                        for (auto& rd : reads[m]) {
                            if (own.count(rd.first)) continue;
                            auto it = greads[g].find(rd.first);
                            if (it == greads[g].end()) greads[g][rd.first] = rd.second;
                            else it->second = it->second && rd.second;
                        }
                    }
                }
                if (gks[g].k.chunks > 1) {
                    // second pass over the partial sums [chunks][V]
                    Node* n = G.members[0];
                    const int64_t V = n->shape[0], C = gks[g].k.chunks;
                    Node* partial = new_node(Op::COPY, Shape{C, V}, {}, n->name + ".partial", 0.f, false);
                    partial->root = true;
                    Node* fin = new_node(n->op, Shape{V}, {tr_permute(tr_node(partial, Shape{C, V}), Shape{1, 0})}, n->name, 0.f, false);
                    fin->root = true;
                    ReduceKernelSpec s2;
                    s2.node = fin;
                    s2.name = name + "_fin";
                    gks[g].extra.push_back(gen_reduce_kernel(s2, 1));
                    gks[g].extra_nodes = {partial, fin};
                }
            }
        }
    }

    // ---- 6b. groups that run the same kernels on other buffers (every attention head's softmax passes) share
    // their launches: block layer blockIdx.z works on member z.  A follower is moved up behind its lead, which
    // needs everything it reads to exist before the lead runs; groups that update a live id's buffer in place
    // stay where they are.
    void share_launches(RegionPlan& rp) {
        auto& groups = rp.groups;
        auto& group_of = rp.group_of;
        auto& gks = rp.gks;
        auto& greads = rp.greads;
        const auto& home_of = rp.home_of;
        const size_t n_groups = groups.size();
        auto updates_in_place = [&](const Group& H) {
            std::vector<Node*> produced = H.members;
            for (Node* sd : H.side) produced.push_back(sd);
            for (Node* ep : H.epi) produced.push_back(ep);
            for (Node* m : produced) {
                auto ho = home_of.find(m);
                if (ho != home_of.end() && livein.count(ho->second)) return true;
            }
            return false;
        };
        std::map<std::vector<int64_t>, std::vector<size_t>> by_signature;
        for (size_t g = 0; g < n_groups; ++g) {
            Group& H = groups[g];
            if (H.dead || (H.kind != Group::ELW && H.kind != Group::SUM && H.kind != Group::ROWCHAIN) || H.rides() || updates_in_place(H)) continue;
            std::vector<int64_t> sig;
            bool ok = true;
            auto add = [&](const GeneratedKernel& k) {
                if (k.source.find("blockIdx.z") != std::string::npos || !k.int_args.empty()) ok = false;
                sig.push_back(add_kernel(k.entry, k.source, k.kind));
                for (int d = 0; d < 3; ++d) { sig.push_back(k.grid[d]); sig.push_back(k.block[d]); }
                sig.push_back(k.lds_bytes);
                sig.push_back((int64_t)k.buffer_args.size());
                sig.push_back(k.chunks);
            };
            add(gks[g].k);
            for (const GeneratedKernel& e : gks[g].extra) add(e);
            if (ok && gks[g].k.grid[2] == 1) by_signature[sig].push_back(g);
        }
        std::vector<std::vector<size_t>> followers(n_groups);
        bool any = false;
        // sets in the order of their first member, so that a set whose members read the results of another
        // (the pass after each head's reduction) sees where those have moved to
        std::vector<const std::pair<const std::vector<int64_t>, std::vector<size_t>>*> sets;
        for (auto& kv : by_signature) sets.push_back(&kv);
        std::sort(sets.begin(), sets.end(), [](auto* x, auto* y) { return x->second[0] < y->second[0]; });
        std::vector<size_t> position(n_groups);  // the old index of the group a group will run behind (its own if it stays)
        for (size_t g = 0; g < n_groups; ++g) position[g] = g;
        for (auto* set : sets) {
            auto& kv = *set;
            if (kv.second.size() < 2) continue;
            const size_t n_buf = (size_t)kv.first[8];
            const size_t cap = std::max<size_t>(1, std::min<size_t>(16, 96 / std::max<size_t>(1, n_buf)));
            std::vector<size_t> leads;
            for (size_t f : kv.second) {
                bool placed = false;
                for (size_t h : leads) {
                    if (followers[h].size() + 1 >= cap) continue;
                    bool ready = true;
                    for (auto& rd : greads[f]) {
                        if (op_is_leaf(rd.first->op)) continue;
                        auto it = group_of.find(rd.first);
                        if (it != group_of.end() && position[it->second] >= h) { ready = false; break; }
                    }
                    if (!ready) continue;
                    followers[h].push_back(f);
                    position[f] = h;
                    placed = any = true;
                    break;
                }
                if (!placed) leads.push_back(f);
            }
        }
        if (any) {
            std::vector<char> is_follower(n_groups, 0);
            for (auto& fs : followers)
                for (size_t f : fs) is_follower[f] = 1;
            std::vector<int> new_index(n_groups, -1);
            std::vector<Group> sorted;
            std::vector<GroupKernels> sorted_gks;
            std::vector<std::map<Node*, bool>> sorted_reads;
            auto take = [&](size_t g, int lead) {
                new_index[g] = (int)sorted.size();
                sorted.push_back(std::move(groups[g]));
                sorted.back().lead = lead;
                sorted_gks.push_back(std::move(gks[g]));
                sorted_reads.push_back(std::move(greads[g]));
            };
            for (size_t g = 0; g < n_groups; ++g) {
                if (is_follower[g]) continue;
                take(g, -1);
                const int lead = new_index[g];
                for (size_t f : followers[g]) take(f, lead);
            }
            for (auto& kv : group_of) kv.second = new_index[kv.second];
            groups.swap(sorted);
            gks.swap(sorted_gks);
            greads.swap(sorted_reads);
        }
    }

    // ---- 7. buffers: homes, temporaries, in-place hazards
    void assign_buffers(RegionPlan& rp) {
        auto& groups = rp.groups;
        auto& gks = rp.gks;
        auto& greads = rp.greads;
        auto& set_end = rp.set_end;
        auto& commits = rp.commits;
        const auto& home_of = rp.home_of;
        // the last group of the shared launches a group runs in (itself if it runs alone)
        set_end.assign(groups.size(), 0);
        for (size_t g = 0; g < groups.size(); ++g) {
            set_end[g] = (int)g;
            const int lead = groups[g].lead;
            if (lead >= 0)
                for (int q = lead; q <= (int)g; ++q) set_end[q] = (int)g;
        }
        std::vector<int> last_use(arena.size() + 16, -1);
        std::map<Node*, int> last_reader;
        for (size_t g = 0; g < groups.size(); ++g)
            if (!groups[g].dead)
                for (auto& rd : greads[g]) last_reader[rd.first] = (int)g;
        std::vector<std::vector<Node*>> free_after(groups.size());
        std::vector<int> scratch_to_free;
        for (size_t g = 0; g < groups.size(); ++g) {
            if (groups[g].dead) continue;
            std::vector<Node*> produced = groups[g].members;
            for (auto& cs : groups[g].riders()) produced.push_back(cs.second);
            for (Node* sd : groups[g].side) produced.push_back(sd);
            for (Node* ep : groups[g].epi) produced.push_back(ep);
            if (groups[g].kind == Group::DOT && !gks[g].dot_store) produced.erase(produced.begin());  // lives in registers only
            if (groups[g].kind == Group::ROWCHAIN)
                produced.erase(std::remove_if(produced.begin(), produced.end(), [&](Node* m) { return groups[g].unstored.count(m) != 0; }), produced.end());
            for (Node* m : produced) {
                auto ho = home_of.find(m);
                bool direct = false;
                if (ho != home_of.end()) {
                    const std::string& id = ho->second;
                    direct = true;
                    auto li = livein.find(id);
                    if (li != livein.end()) {
                        Node* old = li->second;
                        const bool is_side = std::find(groups[g].side.begin(), groups[g].side.end(), m) != groups[g].side.end() ||
                                             std::find(groups[g].epi.begin(), groups[g].epi.end(), m) != groups[g].epi.end();
                        const bool is_member = is_side || (groups[g].kind == Group::ELW &&
                            std::find(groups[g].members.begin(), groups[g].members.end(), m) != groups[g].members.end());
                        // a row chain reads all it needs of a row before it stores any of it: it may overwrite a value
                        // of the same extent that its members read only at the row (and element) they work on (an id
                        // redefined with another extent lays its rows out differently: another row's store could
                        // land on what this row still has to read)
                        bool chain_in_place = groups[g].kind == Group::ROWCHAIN && numel(old->shape) == numel(m->shape);
                        if (chain_in_place)
                            for (Node* cm : groups[g].members)
                                chain_in_place = chain_in_place && chain_reads_rowwise(rp, cm, std::set<Node*>{old}, groups[g].cs_rows, groups[g].cs_cols);
                        for (size_t g2 = 0; g2 < groups.size(); ++g2) {
                            if (groups[g2].dead) continue;
                            auto it = greads[g2].find(old);
                            if (it == greads[g2].end()) continue;
                            if (g2 > g) direct = false;
                            if (g2 == g && !(it->second && is_member) && !chain_in_place) {
                                // a reduction may still update its result in place when it reads the old result only
                                // at the position it is about to write (s = Sum(f(x, s broadcast along the reduced
                                // dim))): the block that owns an output element loads before it stores, and a
                                // chunked reduction stores in its second pass
                                const bool own_sum = groups[g].kind == Group::SUM && m == groups[g].members[0] && op_is_reduce(m->op) &&
                                                     m->in[0].shape.size() == 2 &&
                                                     reads_at_kept_coordinate_only(m, old, m->in[0].shape[0], m->in[0].shape[1]);
                                if (!own_sum) direct = false;
                            }
                        }
                    }
                    int hb = home(id, numel(m->shape));
                    if (direct) m->buffer = hb;
                    else {
                        m->buffer = alloc_temp(numel(m->shape), id + ".new");
                        commits.push_back({hb, m->buffer, numel(m->shape), id});
                        // released after the commits
                    }
                } else {
                    m->buffer = alloc_temp(numel(m->shape), m->name + ".tmp");
                    auto lr = last_reader.find(m);
                    int when = lr == last_reader.end() ? (int)g : std::max(lr->second, (int)g);
                    free_after[set_end[when]].push_back(m);  // groups that share launches run at the same time
                }
            }
            // partial-sum scratch of chunked reductions lives only inside this group
            for (Node* e : gks[g].extra_nodes) {
                if (e->op == Op::COPY) e->buffer = alloc_temp(numel(e->shape), e->name);
            }
            for (Node* e : gks[g].extra_nodes)
                if (e->op == Op::COPY) scratch_to_free.push_back(e->buffer);
            for (Node* e : gks[g].row_partials) {
                e->buffer = alloc_temp(numel(e->shape), e->name);
                scratch_to_free.push_back(e->buffer);
            }
            if (set_end[g] != (int)g) continue;
            for (int b : scratch_to_free) free_temp(b);
            scratch_to_free.clear();
            for (Node* f : free_after[g]) free_temp(f->buffer);
        }
    }

    // ---- 8. launches
    void emit_launches(RegionPlan& rp, std::vector<Step>& out) {
        auto& groups = rp.groups;
        auto& gks = rp.gks;
        auto& commits = rp.commits;
        auto buf_arg = [&](Node* n) {
            ADHIP_CHECK(n->buffer >= 0, "internal: node %d (%s, %s) has no buffer", n->id, n->name.c_str(), op_name(n->op));
            Arg a;
            a.kind = Arg::BUF;
            a.buf = n->buffer;
            return a;
        };
        auto launch_generated = [&](GeneratedKernel& gk) {
            Launch l2;
            l2.kernel = add_kernel(gk.entry, gk.source, gk.kind);
            memcpy(l2.grid, gk.grid, sizeof l2.grid);
            memcpy(l2.block, gk.block, sizeof l2.block);
            l2.lds_bytes = gk.lds_bytes;
            l2.label = gk.entry;
            l2.bytes = gk.bytes;
            l2.flops = gk.flops;
            for (Node* n : gk.buffer_args) l2.args.push_back(buf_arg(n));
            push_launch(out, l2, gk.kind);
        };
        // the launches of an element-wise group without column sums or of a reduction, with their statistics kinds
        auto group_launches = [&](size_t g) {
            Group& G = groups[g];
            GeneratedKernel& k = gks[g].k;
            std::vector<std::pair<Launch, std::string>> ls;
            Launch l;
            l.kernel = add_kernel(k.entry, k.source, k.kind);
            memcpy(l.grid, k.grid, sizeof l.grid);
            memcpy(l.block, k.block, sizeof l.block);
            l.lds_bytes = k.lds_bytes;
            l.label = k.entry;
            l.bytes = k.bytes;
            l.flops = k.flops;
            if (G.kind == Group::SUM && k.chunks > 1) {
                Node* partial = gks[g].extra_nodes[0];
                Node* fin = gks[g].extra_nodes[1];
                fin->buffer = G.members[0]->buffer;
                for (size_t i = 0; i < k.buffer_args.size(); ++i)
                    l.args.push_back(buf_arg(i == 0 ? partial : k.buffer_args[i]));
                ls.push_back({l, k.kind});
                GeneratedKernel& k2 = gks[g].extra[0];
                Launch l2;
                l2.kernel = add_kernel(k2.entry, k2.source, k2.kind);
                memcpy(l2.grid, k2.grid, sizeof l2.grid);
                memcpy(l2.block, k2.block, sizeof l2.block);
                l2.label = k2.entry;
                l2.bytes = k2.bytes;
                l2.flops = k2.flops;
                for (Node* n : k2.buffer_args) l2.args.push_back(buf_arg(n));
                ls.push_back({l2, k2.kind});
            } else {
                for (Node* n : k.buffer_args) l.args.push_back(buf_arg(n));
                ls.push_back({l, k.kind});
            }
            return ls;
        };
        for (size_t g = 0; g < groups.size(); ++g) {
            Group& G = groups[g];
            if (G.dead) continue;
            if (G.kind == Group::DOT) {
                if (G.members.size() > 1) emit_dot_group(G.members, out, gks[g].extra_nodes.empty() ? nullptr : gks[g].extra_nodes[0]);
                else if (!G.epi.empty()) emit_dot(G.members[0], out, &gks[g].dot_epi, gks[g].dot_store);
                else emit_dot(G.members[0], out, nullptr, true, gks[g].extra_nodes.empty() ? nullptr : gks[g].extra_nodes[0]);
                continue;
            }
            if (G.kind == Group::TRANSPOSE) {
                emit_transpose(G.members[0], out);
                continue;
            }
            if (G.kind == Group::ATTN) {
                emit_attention(G.members, out);
                continue;
            }
            GeneratedKernel& k = gks[g].k;
            if (G.kind == Group::ELW && G.rides()) {
                launch_generated(k);
                const int64_t tiles = elw_colsum_tiles(G.cs_rows, G.cs_cols, G.cs_streams);
                auto B = [&](Node* x) { Arg q; q.kind = Arg::BUF; ADHIP_CHECK(x->buffer >= 0, "internal: riding sum without buffer"); q.buf = x->buffer; return q; };
                auto I = [&](int64_t v) { Arg q; q.kind = Arg::I64; q.iv = v; return q; };
                size_t cols_done = 0;
                // row sums: one launch of the fixed second-pass kernel per two of them, which also takes up to four of
                // the column sums along
                for (size_t r0 = 0; r0 < G.rowsums.size(); r0 += 2) {
                    const size_t nr = std::min<size_t>(2, G.rowsums.size() - r0);
                    const size_t nc = std::min<size_t>(4, G.colsums.size() - cols_done);
                    const int64_t runs = elw_rowsum_runs(G.cs_cols);
                    const int64_t col_blocks = nc ? (G.cs_cols + 63) / 64 : 0, row_blocks = (G.cs_rows + 1023) / 1024;
                    if (fixed_sums_finalize < 0) fixed_sums_finalize = add_kernel("adhip_sums_finalize", fixed_kernels_source(), "sums_finalize");
                    Launch lf;
                    lf.kernel = fixed_sums_finalize;
                    lf.block[0] = 1024;
                    lf.grid[0] = (unsigned)(col_blocks + row_blocks);
                    lf.grid[1] = (unsigned)std::max(nr, std::max<size_t>(nc, 1));
                    // unused slots repeat a valid buffer: the kernel never touches them
                    for (size_t j = 0; j < 4; ++j) lf.args.push_back(nc ? B(G.colsums[cols_done + std::min(j, nc - 1)].second) : B(G.rowsums[r0].second));
                    for (size_t j = 0; j < 4; ++j) lf.args.push_back(nc ? B(gks[g].extra_nodes[cols_done + std::min(j, nc - 1)]) : B(gks[g].row_partials[r0]));
                    lf.args.push_back(I(tiles));
                    lf.args.push_back(I(G.cs_cols));
                    lf.args.push_back(I((int64_t)nc));
                    for (size_t j = 0; j < 2; ++j) lf.args.push_back(B(G.rowsums[r0 + std::min(j, nr - 1)].second));
                    for (size_t j = 0; j < 2; ++j) lf.args.push_back(B(gks[g].row_partials[r0 + std::min(j, nr - 1)]));
                    lf.args.push_back(I(G.cs_rows));
                    lf.args.push_back(I(runs));
                    lf.args.push_back(I((int64_t)nr));
                    lf.args.push_back(I(col_blocks));
                    lf.label = k.entry + "_rs0";
                    lf.bytes = 4.0 * (double)nc * (double)G.cs_cols * (double)(tiles + 1) + 4.0 * (double)nr * (double)G.cs_rows * (double)(runs + 1);
                    lf.flops = (double)nc * (double)G.cs_cols * (double)tiles + (double)nr * (double)G.cs_rows * (double)runs;
                    push_launch(out, lf, "sums_finalize");
                    cols_done += nc;
                }
                // the column sums that are left: one launch of the fixed second-pass kernel per four sums
                if (cols_done < G.colsums.size() && fixed_finalize < 0) fixed_finalize = add_kernel("adhip_colsum_finalize", fixed_kernels_source(), "colsum_finalize");
                for (size_t i0 = cols_done; i0 < G.colsums.size(); i0 += 4) {
                    const size_t cnt = std::min<size_t>(4, G.colsums.size() - i0);
                    Launch lf;
                    lf.kernel = fixed_finalize;
                    lf.block[0] = 1024;
                    lf.grid[0] = (unsigned)((G.cs_cols + 63) / 64);
                    lf.grid[1] = (unsigned)cnt;
                    for (size_t j = 0; j < 4; ++j) lf.args.push_back(B(G.colsums[i0 + std::min(j, cnt - 1)].second));
                    for (size_t j = 0; j < 4; ++j) lf.args.push_back(B(gks[g].extra_nodes[i0 + std::min(j, cnt - 1)]));
                    Arg t; t.kind = Arg::I64; t.iv = tiles; lf.args.push_back(t);
                    t.iv = G.cs_cols; lf.args.push_back(t);
                    lf.label = k.entry + "_cs";
                    lf.bytes = 4.0 * (double)cnt * (double)G.cs_cols * (double)(tiles + 1);
                    lf.flops = (double)cnt * (double)G.cs_cols * (double)tiles;
                    push_launch(out, lf, "colsum_finalize");
                }
                continue;
            }
            // groups that share their launches: one launch per kernel of the lead, block layer z for member z
            size_t last = g;
            while (last + 1 < groups.size() && groups[last + 1].lead == (int)g) ++last;
            std::vector<std::vector<std::pair<Launch, std::string>>> per_member;
            for (size_t q = g; q <= last; ++q) per_member.push_back(group_launches(q));
            for (size_t j = 0; j < per_member[0].size(); ++j) {
                if (last == g) {
                    push_launch(out, per_member[0][j].first, per_member[0][j].second);
                    continue;
                }
                Launch l = per_member[0][j].first;
                const int cnt = (int)per_member.size();
                l.kernel = add_layered_kernel(l.kernel, cnt);
                l.grid[2] = (unsigned)cnt;
                l.args.clear();
                for (size_t a = 0; a < per_member[0][j].first.args.size(); ++a)
                    for (int q = 0; q < cnt; ++q) {
                        const Launch& lq = per_member[q][j].first;
                        ADHIP_CHECK(lq.kernel == per_member[0][j].first.kernel && lq.args.size() == per_member[0][j].first.args.size() &&
                                        lq.args[a].kind == Arg::BUF, "internal: groups that share a launch differ");
                        l.args.push_back(lq.args[a]);
                    }
                l.bytes *= cnt;
                l.flops *= cnt;
                l.label += strf("_x%d", cnt);
                push_launch(out, l, per_member[0][j].second);
            }
            g = last;
        }
        if (latch_region && latch_slot >= 0 && commits.empty() && opt.fuse) attach_latch(rp, out);
        for (auto& c : commits) emit_copy(out, c.dst, c.src, c.n, "commit_" + c.id);
        for (auto& c : commits) free_temp(c.src);
    }

    // The region is the last one of a device-predicated loop's body.  When its last launch is the generated kernel
    // that produces the loop's predicate (a one-element value), that kernel is generated once more with the loop flag
    // as a trailing argument: the thread that stores the predicate also stores `predicate != 0` into the flag, for the
    // next iteration's kernels to see.  Nothing may run after it in the iteration (it would see the new flag), which is
    // why the region must end with it and have no commits.
    void attach_latch(RegionPlan& rp, std::vector<Step>& out) {
        if (out.empty() || out.back().kind != Step::LAUNCH) return;
        Node* n = nullptr;
        for (auto& w : rp.wanted)
            if (w.first == latch_id) n = w.second;
        if (!n || numel(n->shape) != 1) return;
        auto it = rp.group_of.find(n);
        if (it == rp.group_of.end()) return;
        const size_t g = (size_t)it->second;
        Group& G = rp.groups[g];
        if (G.dead || G.lead >= 0) return;
        for (size_t h = g + 1; h < rp.groups.size(); ++h)
            if (!rp.groups[h].dead) return;
        GroupKernels& gk = rp.gks[g];
        GeneratedKernel nk;
        if (G.kind == Group::ELW && gk.spec_kind == 1 && !G.rides() && !G.tiled) {
            ElwKernelSpec spec = gk.elw_spec;
            spec.latch = n;
            spec.name += "_latch";
            nk = gen_elw_kernel(spec, gk.spec_members);
        } else if (G.kind == Group::SUM && gk.spec_kind == 2 && gk.k.epilogue_done && gk.k.chunks == 1) {
            ReduceKernelSpec spec = gk.red_spec;
            spec.latch = n;
            spec.name += "_latch";
            nk = gen_reduce_kernel(spec);
        } else {
            return;
        }
        Launch& l = out.back().launch;
        if (!nk.latch_done || l.label != gk.k.entry || nk.buffer_args.size() != gk.k.buffer_args.size()) return;
        l.kernel = add_kernel(nk.entry, nk.source, nk.kind);
        l.label = nk.entry;
        plan->stats[(size_t)l.stat].label = nk.entry;
        plan->stats[(size_t)l.stat].kernel = l.kernel;
        Arg a;
        a.kind = Arg::FLAG;
        a.iv = latch_slot;
        l.args.push_back(a);
        latch_attached = true;
    }

    void emit_transpose(Node* n, std::vector<Step>& out) {
        const Piece& pc = n->in[0].pieces[0];
        const Stage& st = pc.view.st[0];
        const int nd = (int)st.shape.size();
        int last = -1;
        for (int d = nd - 1; d >= 0; --d)
            if (st.shape[d] > 1) { last = d; break; }
        const int u = n->transpose_u;
        Shape dense = row_major_strides(st.shape);
        int64_t nb[3] = {1, 1, 1}, ib[3] = {0, 0, 0}, ob[3] = {0, 0, 0};
        int k = 0;
        for (int d = 0; d < last; ++d)
            if (d != u && st.shape[d] > 1) { nb[k] = st.shape[d]; ib[k] = st.stride[d]; ob[k] = dense[d]; ++k; }
        const int64_t U = st.shape[u], V = st.shape[last];
        const int64_t batches = nb[0] * nb[1] * nb[2];
        const int64_t ut = (U + 63) / 64, vt = (V + 63) / 64;
        ADHIP_CHECK(ut * vt * batches <= 0x7fffffff, "internal: transpose grid too large");
        // the source region must lie inside the source buffer
        int64_t hi = st.offset;
        for (int d = 0; d < nd; ++d) hi += (st.shape[d] - 1) * st.stride[d];
        ADHIP_CHECK(st.offset >= 0 && hi < numel(pc.src.node->shape), "internal: transposing copy reads outside its source");
        bool v4 = (U % 4 == 0) && (V % 4 == 0) && (st.offset % 4 == 0) && (st.stride[last] % 4 == 0) && (dense[u] % 4 == 0);
        for (int q = 0; q < 3; ++q) v4 = v4 && (ib[q] % 4 == 0) && (ob[q] % 4 == 0);
        if (fixed_transpose < 0) fixed_transpose = add_kernel("adhip_transpose_copy", fixed_kernels_source(), "transpose");
        if (fixed_transpose4 < 0) fixed_transpose4 = add_kernel("adhip_transpose_copy4", fixed_kernels_source(), "transpose");
        Launch l;
        l.kernel = v4 ? fixed_transpose4 : fixed_transpose;
        l.block[0] = 256;
        l.grid[0] = (unsigned)(ut * vt * batches);
        auto B = [&](Node* x) { Arg q; q.kind = Arg::BUF; ADHIP_CHECK(x->buffer >= 0, "internal: transpose operand without buffer"); q.buf = x->buffer; return q; };
        auto I = [&](int64_t v) { Arg q; q.kind = Arg::I64; q.iv = v; return q; };
        l.args = {B(n), B(pc.src.node), I(st.offset), I(nb[0]), I(nb[1]), I(nb[2]), I(ib[0]), I(ib[1]), I(ib[2]),
                  I(ob[0]), I(ob[1]), I(ob[2]), I(U), I(V), I(st.stride[last]), I(dense[u]), I(ut), I(vt)};
        l.label = "transpose_" + n->name;
        l.bytes = 8.0 * (double)numel(st.shape);
        push_launch(out, l, "transpose");
    }

    // How a matrix-core product is launched: tile, bounds checking, and how many ranges of k it is split into.
    struct DotLaunchPlan {
        GemmConfig cfg;
        int bn_tile = 128;
        int64_t splits = 1, k_chunk = 0;
    };

    // What must agree for products to share a grouped launch: sizes, strides and whether operands are 16-byte
    // aligned.  False for products that do not go to the matrix cores.
    static bool dot_group_key(const Node* n, std::array<int64_t, 8>& key) {
        if (!dot_uses_mfma(n)) return false;
        Affine2D a, b;
        tref_affine2d(n->in[0], a);
        tref_affine2d(n->in[1], b);
        const int64_t M = n->shape[0], N = n->shape[1], K = n->in[0].shape[1];
        key = {M, N, K, a.s0, a.s1, b.s0, b.s1, dot_alignment(a, b, M, N, K)};
        return true;
    }

    // 0: both operands are 16-byte aligned line by line and k is a multiple of the tile depth (the kernel without
    // bounds checks, if M and N fit the tile as well); 1: not so, but a line of either operand holds at least four
    // elements (128-bit reads of whatever alignment, single elements on the ragged rim); 2: single elements only
    static int dot_alignment(const Affine2D& a, const Affine2D& b, int64_t M, int64_t N, int64_t K) {
        const bool a_k = a.s1 == 1, b_k = b.s0 == 1;
        const int64_t a_ld = a_k ? a.s0 : a.s1, b_ld = b_k ? b.s1 : b.s0;
        if ((a_k ? K : M) < 4 || (b_k ? K : N) < 4) return 2;
        // (the kernel without bounds checks addresses a tile by 32-bit offsets from its corner: lines of 2^22 elements
        // and more take the checked variant, whose index arithmetic is 64 bits wide)
        const int64_t widest = int64_t(1) << 22;
        return ((a.offset % 4) || (b.offset % 4) || (a_ld % 4) || (b_ld % 4) || (K % 16) || a_ld >= widest || b_ld >= widest) ? 1 : 0;
    }

    template <class ReadsNode, class KeepsEpilogue>
    void group_products(std::vector<Group>& groups, std::map<Node*, int>& group_of, std::map<Node*, std::map<Node*, bool>>& reads,
                        const std::map<Node*, std::string>& home_of, ReadsNode&& reads_node, KeepsEpilogue&& keeps_epilogue) {
        const int G = (int)groups.size();
        std::vector<std::array<int64_t, 8>> key(G);
        std::vector<char> cand(G, 0);
        int ncand = 0;
        for (int g = 0; g < G; ++g) {
            if (groups[g].dead) continue;
            if (groups[g].kind == Group::DOT && dot_group_key(groups[g].members[0], key[g]) && !keeps_epilogue(g)) {
                cand[g] = 1;
                ++ncand;
            } else if (groups[g].kind == Group::ATTN) {
                // the heads of multi-head attention: same shapes and strides, one launch (bit 40 keeps these keys
                // apart from those of plain products)
                AttentionKey ak;
                Affine2D q, kt, v;
                if (!attention_key(groups[g].members[0], ak, q, kt, v)) continue;
                uint32_t sb;
                memcpy(&sb, &ak.scale, 4);
                key[g] = {ak.sq, ak.sk, ak.d, ak.dv + (ak.m_ld << 10), ak.q_ld, ak.k_ld, ak.v_ld, (int64_t)sb | (int64_t(1) << 40)};
                cand[g] = 1;
                ++ncand;
            }
        }
        if (ncand < 2) return;
        // depth of every kernel
        std::vector<int> level(G, 0);
        for (int g = 0; g < G; ++g) {
            Group& H = groups[g];
            if (H.dead) continue;
            std::set<int> preds;
            bool ok = true;
            auto add_reads = [&](const std::map<Node*, bool>& rd) {
                for (auto& kv : rd) {
                    if (op_is_leaf(kv.first->op)) continue;
                    auto it = group_of.find(kv.first);
                    if (it == group_of.end() || it->second == g) continue;
                    if (it->second > g) ok = false;
                    preds.insert(it->second);
                }
            };
            std::vector<Node*> produced = H.members;
            for (Node* sd : H.side) produced.push_back(sd);
            for (Node* m : produced) add_reads(reads[m]);
            for (auto& cs : H.riders()) {
                std::map<Node*, bool> er;
                if (in_mem(cs.first)) er[cs.first] = true;
                else collect_reads(cs.first, er);
                add_reads(er);
                produced.push_back(cs.second);
            }
            if (!ok) return;  // not in dependency order as it stands: leave the region alone
            for (Node* m : produced) {
                auto ho = home_of.find(m);
                if (ho == home_of.end()) continue;
                auto li = livein.find(ho->second);
                if (li == livein.end()) continue;
                for (int r = 0; r < g; ++r)
                    if (!groups[r].dead && reads_node(groups[r], li->second)) preds.insert(r);
            }
            for (int p : preds) level[g] = std::max(level[g], level[p] + (groups[p].kind == Group::DOT || groups[p].kind == Group::ATTN ? 1 : 0));
        }
        // sets of at least two
        std::map<std::pair<int, std::array<int64_t, 8>>, std::vector<int>> sets;
        for (int g = 0; g < G; ++g)
            if (cand[g]) sets[{level[g], key[g]}].push_back(g);
        bool any = false;
        for (auto& kv : sets) any = any || kv.second.size() >= 2;
        if (!any) return;
        // new order
        std::vector<int> order;
        for (int g = 0; g < G; ++g)
            if (!groups[g].dead) order.push_back(g);
        std::stable_sort(order.begin(), order.end(), [&](int x, int y) {
            if (level[x] != level[y]) return level[x] < level[y];
            auto product = [&](int g) { return groups[g].kind == Group::DOT || groups[g].kind == Group::ATTN; };
            return product(x) < product(y);
        });
        std::vector<int> new_index(G, -1);
        std::vector<Group> sorted;
        for (int g : order) {
            new_index[g] = (int)sorted.size();
            sorted.push_back(groups[g]);
        }
        for (auto& kv : group_of) {
            ADHIP_CHECK(kv.second >= 0 && kv.second < G && new_index[kv.second] >= 0, "internal: value produced by a dropped kernel");
            kv.second = new_index[kv.second];
        }
        groups.swap(sorted);
        // merge each set into its first member, at most kGemmGroupSlots products per launch, evenly
        for (auto& kv : sets) {
            const std::vector<int>& set = kv.second;
            if (set.size() < 2) continue;
            const size_t launches = (set.size() + kGemmGroupSlots - 1) / kGemmGroupSlots;
            const size_t per = (set.size() + launches - 1) / launches;
            for (size_t i0 = 0; i0 < set.size(); i0 += per) {
                const size_t i1 = std::min(set.size(), i0 + per);
                if (i1 - i0 < 2) continue;
                const int head = new_index[set[i0]];
                for (size_t i = i0 + 1; i < i1; ++i) {
                    Group& T = groups[new_index[set[i]]];
                    groups[head].members.push_back(T.members[0]);
                    group_of[T.members[0]] = head;
                    T.dead = true;
                }
            }
        }
    }

    // Tile and k ranges of a grouped launch of `cnt` products shaped like `first`: by the number of blocks the whole
    // launch has, as plan_dot does for a single product.
    static DotLaunchPlan plan_dot_group(const Node* first, int cnt) {
        std::array<int64_t, 8> key{};
        ADHIP_CHECK(dot_group_key(first, key), "internal: grouped launch of a product that does not qualify");
        const int64_t M = key[0], N = key[1], K = key[2];
        DotLaunchPlan pl;
        GemmConfig& cfg = pl.cfg;
        cfg.a_kcontig = key[4] == 1;
        cfg.b_kcontig = key[5] == 1;
        cfg.grouped = true;
        const int64_t blocks128 = ((M + 127) / 128) * ((N + 127) / 128) * cnt;
        const int64_t max_splits = std::min<int64_t>(K / 256, 32);
        auto splits_for = [&](int64_t blocks) {
            if (blocks >= 256 || max_splits < 2) return (int64_t)1;
            return std::max<int64_t>(std::min<int64_t>((512 + blocks - 1) / blocks, max_splits), 1);
        };
        // three 64x64 blocks per CU without cutting k beat 128x128 blocks with k cut and the slice sum that follows
        // (12 x 2048x128x1024: 66 us against 77 + 8); with two per CU it is the other way round (8 x 2048x128x2048:
        // 105-118 us against 80 + 7)
        const int64_t blocks64 = ((M + 63) / 64) * ((N + 63) / 64) * cnt;
        const bool small_whole = blocks128 < 256 && blocks64 >= 768;
        cfg.bm = (!small_whole && blocks128 * splits_for(blocks128) >= 256) ? 128 : 64;
        pl.bn_tile = cfg.bm == 64 ? 64 : 128;
        if (cfg.bm == 128 && blocks128 < 512 && splits_for(blocks128) == 1) { pl.bn_tile = 64; cfg.bn = 64; }
        cfg.edge = key[7] || (M % cfg.bm) || (N % pl.bn_tile);
        cfg.edge_vec = key[7] != 2;
        const int64_t blocks = ((M + cfg.bm - 1) / cfg.bm) * ((N + pl.bn_tile - 1) / pl.bn_tile) * cnt;
        const int64_t want = small_whole ? 1 : splits_for(blocks);
        if (want > 1) {
            pl.k_chunk = (((K + want - 1) / want) + 15) / 16 * 16;
            pl.splits = (K + pl.k_chunk - 1) / pl.k_chunk;
            cfg.split_k = pl.splits > 1;
            if (!cfg.split_k) pl.splits = 1;
        }
        return pl;
    }

    // One launch for several products of the same shape (see group_products): problem y is block row y; with k cut
    // into ranges, range z is block layer z and `partial` holds [problem][range][M*N] partial products, added by one
    // grouped launch of the slice sum.
    void emit_dot_group(const std::vector<Node*>& dots, std::vector<Step>& out, Node* partial) {
        const int cnt = (int)dots.size();
        ADHIP_CHECK(cnt >= 2 && cnt <= kGemmGroupSlots, "internal: grouped product launch of %d products", cnt);
        std::array<int64_t, 8> key0{};
        ADHIP_CHECK(dot_group_key(dots[0], key0), "internal: grouped launch of a product that does not qualify");
        const int64_t M = key0[0], N = key0[1], K = key0[2];
        const DotLaunchPlan pl = plan_dot_group(dots[0], cnt);
        const GemmConfig& cfg = pl.cfg;
        ADHIP_CHECK(cfg.split_k == (partial != nullptr), "internal: split grouped product and its slice buffer disagree");
        ADHIP_CHECK(!partial || numel(partial->shape) == (int64_t)cnt * pl.splits * M * N, "internal: slice buffer of the wrong size");
        std::string entry = strf("adhip_gemm_%c%c_%d%s%s%s_grouped", cfg.a_kcontig ? 'k' : 'm', cfg.b_kcontig ? 'k' : 'n', cfg.bm,
                                 cfg.bn == 64 && cfg.bm != 64 ? "x64" : "", cfg.edge ? (cfg.edge_vec ? "_rim" : "_edge") : "", cfg.split_k ? "_splitk" : "");
        Launch l;
        l.kernel = add_kernel(entry, gemm_kernel_source(cfg, entry), "dot_mfma");
        l.block[0] = cfg.bm == 64 ? 256u : (unsigned)(cfg.bm * 2);
        l.grid[0] = (unsigned)(((M + cfg.bm - 1) / cfg.bm) * ((N + pl.bn_tile - 1) / pl.bn_tile));
        l.grid[1] = (unsigned)cnt;
        l.grid[2] = (unsigned)pl.splits;
        auto B = [&](Node* x, int64_t off) {
            Arg q;
            q.kind = Arg::BUF;
            ADHIP_CHECK(x->buffer >= 0, "internal: matmul operand without buffer");
            q.buf = x->buffer;
            q.off = off;
            return q;
        };
        auto I = [&](int64_t v) { Arg q; q.kind = Arg::I64; q.iv = v; return q; };
        for (int i = 0; i < kGemmGroupSlots; ++i) {
            const int pi = std::min(i, cnt - 1);  // unused slots repeat the last problem; no block reads them
            Node* n = dots[pi];
            std::array<int64_t, 8> key{};
            ADHIP_CHECK(dot_group_key(n, key) && key == key0, "internal: grouped products differ in shape or strides");
            Affine2D a, b;
            tref_affine2d(n->in[0], a);
            tref_affine2d(n->in[1], b);
            l.args.push_back(partial ? B(partial, (int64_t)pi * pl.splits * M * N) : B(n, 0));
            l.args.push_back(B(a.base, a.offset));
            l.args.push_back(B(b.base, b.offset));
        }
        for (int q = 0; q < 7; ++q) l.args.push_back(I(key0[q]));
        if (cfg.split_k) l.args.push_back(I(pl.k_chunk));
        l.label = strf("dots_%s_%dx_%lldx%lldx%lld", dots[0]->name.c_str(), cnt, (long long)M, (long long)N, (long long)K);
        l.bytes = 4.0 * cnt * ((double)M * K + (double)K * N + (double)M * N * (double)pl.splits);
        l.flops = 2.0 * cnt * (double)M * (double)N * (double)K;
        push_launch(out, l, "dot_mfma");
        if (cfg.split_k) {
            if (fixed_sum_slices_grouped < 0)
                fixed_sum_slices_grouped = add_kernel("adhip_sum_slices_grouped", fixed_kernels_source(), "sum_slices");
            Launch lf;
            lf.kernel = fixed_sum_slices_grouped;
            lf.block[0] = 256;
            lf.grid[0] = (unsigned)((M * N + 1023) / 1024);
            lf.grid[1] = (unsigned)cnt;
            for (int i = 0; i < kGemmGroupSlots; ++i) lf.args.push_back(B(dots[std::min(i, cnt - 1)], 0));
            lf.args.push_back(B(partial, 0));
            lf.args.push_back(I(pl.splits));
            lf.args.push_back(I(M * N));
            lf.label = l.label + "_sum";
            lf.bytes = 4.0 * cnt * (double)M * (double)N * (double)(pl.splits + 1);
            lf.flops = (double)cnt * (double)M * (double)N * (double)pl.splits;
            push_launch(out, lf, "sum_slices");
        }
    }

    // One launch of the fused attention kernel for up to 16 problems of one shape (block row y works on problem y).
    void emit_attention(const std::vector<Node*>& atts, std::vector<Step>& out) {
        const int cnt = (int)atts.size();
        ADHIP_CHECK(cnt >= 1 && cnt <= kAttentionSlots, "internal: attention launch of %d problems", cnt);
        AttentionKey key0;
        Affine2D q0, k0, v0;
        ADHIP_CHECK(attention_key(atts[0], key0, q0, k0, v0), "internal: attention node whose operands the kernel cannot read");
        AttentionConfig cfg;
        cfg.d = (int)key0.d;
        cfg.dv = (int)key0.dv;
        cfg.mask = key0.m_ld > 0;
        const int64_t row_blocks = (key0.sq + 63) / 64;
        // A launch with two or more blocks per CU runs blocks of four wavefronts on tiles of 32 keys, two of which fit
        // a CU's LDS while the heads are not too wide; a smaller launch splits every tile between two groups of four
        // wavefronts instead, so that a SIMD still has two wavefronts to switch between.  Tiles of 64 keys where two
        // stages of them fit in LDS.
        const bool narrow = cfg.d + cfg.dv <= 256;
        if (row_blocks * cnt >= 512 && narrow) { cfg.bn = 32; cfg.wg = 1; }
        else { cfg.bn = narrow ? 64 : 32; cfg.wg = 2; }
        ADHIP_CHECK(attention_lds_bytes(cfg) <= 160 * 1024, "internal: attention tiles of %d keys do not fit in LDS", cfg.bn);
        const std::string entry = strf("adhip_attention_d%d_v%d_k%d_w%d%s", cfg.d, cfg.dv, cfg.bn, cfg.wg, cfg.mask ? "_mask" : "");
        Launch l;
        l.kernel = add_kernel(entry, attention_kernel_source(cfg, entry), "attention");
        l.block[0] = 256u * (unsigned)cfg.wg;
        ADHIP_CHECK(row_blocks * cnt <= 0x7fffffff, "internal: attention grid too large");
        l.grid[0] = (unsigned)(row_blocks * cnt);
        auto B = [&](Node* x, int64_t off) {
            Arg a;
            a.kind = Arg::BUF;
            ADHIP_CHECK(x->buffer >= 0, "internal: attention operand without buffer");
            a.buf = x->buffer;
            a.off = off;
            return a;
        };
        auto I = [&](int64_t v) { Arg a; a.kind = Arg::I64; a.iv = v; return a; };
        for (int i = 0; i < kAttentionSlots; ++i) {
            Node* n = atts[(size_t)std::min(i, cnt - 1)];  // unused slots repeat the last problem; no block reads them
            AttentionKey key;
            Affine2D q, kt, v, mk;
            ADHIP_CHECK(attention_key(n, key, q, kt, v, &mk) && key == key0, "internal: attention problems of one launch differ");
            l.args.push_back(B(n, 0));
            l.args.push_back(B(q.base, q.offset));
            l.args.push_back(B(kt.base, kt.offset));
            l.args.push_back(B(v.base, v.offset));
            if (cfg.mask) l.args.push_back(B(mk.base, mk.offset));
        }
        for (int64_t v : {key0.sq, key0.sk, key0.q_ld, key0.k_ld, key0.v_ld}) l.args.push_back(I(v));
        if (cfg.mask) l.args.push_back(I(key0.m_ld));
        Arg sc;
        sc.kind = Arg::F32;
        sc.fv = key0.scale;
        l.args.push_back(sc);
        for (int64_t v : {row_blocks, (int64_t)cnt}) { Arg a; a.kind = Arg::I32; a.iv = v; l.args.push_back(a); }
        l.label = strf("attention_%s_%dx_%lldx%lldx%lldx%lld", atts[0]->name.c_str(), cnt, (long long)key0.sq, (long long)key0.sk,
                       (long long)key0.d, (long long)key0.dv);
        l.bytes = 4.0 * cnt * ((double)key0.sq * key0.d + (double)key0.sk * key0.d + (double)key0.sk * key0.dv + (double)key0.sq * key0.dv) +
                  (cfg.mask ? 4.0 * (double)key0.sq * (double)key0.sk : 0.0);
        l.flops = 2.0 * cnt * (double)key0.sq * (double)key0.sk * (double)(key0.d + key0.dv);
        push_launch(out, l, "attention");
    }

    // whether a product goes to the matrix-core kernel (else the one-thread-per-output kernel)
    static bool dot_uses_mfma(const Node* n) {
        Affine2D a, b;
        if (!tref_affine2d(n->in[0], a) || !tref_affine2d(n->in[1], b)) return false;
        const int64_t M = n->shape[0], N = n->shape[1], K = n->in[0].shape[1];
        const bool a_unit = a.s1 == 1 || a.s0 == 1, b_unit = b.s0 == 1 || b.s1 == 1;
        return M * N * K >= 64 * 64 * 64 && a_unit && b_unit;
    }

    static DotLaunchPlan plan_dot(const Node* n) {
        Affine2D a, b;
        tref_affine2d(n->in[0], a);
        tref_affine2d(n->in[1], b);
        const int64_t M = n->shape[0], N = n->shape[1], K = n->in[0].shape[1];
        DotLaunchPlan pl;
        GemmConfig& cfg = pl.cfg;
        cfg.a_kcontig = a.s1 == 1;
        cfg.b_kcontig = b.s0 == 1;
        const int alignment = dot_alignment(a, b, M, N, K);
        const bool unaligned = alignment != 0;
        // the largest block tile that still puts enough blocks on the chip's 256 CUs: 256x128 (8 waves) with at
        // least two blocks per CU, 128x128 with at least one -- counting the ranges k can be cut into (each at
        // least 256 deep; the slices are added afterwards) -- else 64x64, cut the same way.  A block that has a CU
        // to itself cannot hide the latency of its operand loads, hence the target of about 512 blocks.
        const int64_t blocks128 = ((M + 127) / 128) * ((N + 127) / 128);
        const int64_t max_splits = std::min<int64_t>(K / 256, 32);
        auto splits_for = [&](int64_t blocks) {
            if (blocks >= 256 || max_splits < 2) return (int64_t)1;
            return std::max<int64_t>(std::min<int64_t>((512 + blocks - 1) / blocks, max_splits), 1);
        };
        // An output of 512 and more 64x64 tiles but fewer than 256 of 128x128, with k up to 2048: the small tile, whole,
        // beats the large one with k cut in four and the slices added afterwards (2048 x 1024 x 1024: 38.5 us against
        // 39.1 + 6.4; at k = 4096 the large tile's better rate has made up for the slice sum: 139.6 against 131.3 + 6.4).
        const int64_t blocks64 = ((M + 63) / 64) * ((N + 63) / 64);
        const bool small_whole = blocks128 < 256 && blocks64 >= 512 && K <= 2048;
        if (!unaligned && M % 256 == 0 && N % 128 == 0 && (M / 256) * (N / 128) >= 512) cfg.bm = 256;
        else if (!small_whole && blocks128 * splits_for(blocks128) >= 256) cfg.bm = 128;
        else cfg.bm = 64;
        pl.bn_tile = cfg.bm == 64 ? 64 : 128;
        // one 128x128 block per CU is too few to hide its own latencies: halve the tile's width for two per CU
        if (cfg.bm == 128 && blocks128 < 512 && splits_for(blocks128) == 1) { pl.bn_tile = 64; cfg.bn = 64; }
        // diagnostic: ADHIP_DOT_PLAN=<bm>,<bn>,<splits> forces tile and k ranges of every aligned product the tile divides
        int64_t forced_splits = 0;
        if (const char* e = getenv("ADHIP_DOT_PLAN")) {
            long fbm = 0, fbn = 0, fs = 0;
            if (sscanf(e, "%ld,%ld,%ld", &fbm, &fbn, &fs) == 3 && !unaligned && (fbm == 256 || fbm == 128 || fbm == 64) &&
                (fbn == 128 || fbn == 64) && M % fbm == 0 && N % fbn == 0 && fs >= 1 && !(fbm == 256 && fbn != 128) && !(fbm == 64 && fbn != 64)) {
                cfg.bm = (int)fbm;
                pl.bn_tile = (int)fbn;
                cfg.bn = (fbm == 128 && fbn == 64) ? 64 : 0;
                forced_splits = fs;
            }
        }
        cfg.edge = unaligned || (M % cfg.bm) || (N % pl.bn_tile);
        cfg.edge_vec = alignment != 2;
        const int64_t blocks = ((M + cfg.bm - 1) / cfg.bm) * ((N + pl.bn_tile - 1) / pl.bn_tile);
        const int64_t want = forced_splits ? std::min<int64_t>(forced_splits, std::max<int64_t>(K / 64, 1)) : (cfg.bm == 256 || small_whole ? 1 : splits_for(blocks));
        if (want > 1) {
            pl.k_chunk = (((K + want - 1) / want) + 15) / 16 * 16;
            pl.splits = (K + pl.k_chunk - 1) / pl.k_chunk;
            cfg.split_k = pl.splits > 1;
            if (!cfg.split_k) pl.splits = 1;
        }
        return pl;
    }

    void emit_dot(Node* n, std::vector<Step>& out, const DotEpilogueCode* epi = nullptr, bool store_c = true,
                  Node* partial = nullptr) {
        Affine2D a, b;
        ADHIP_CHECK(tref_affine2d(n->in[0], a) && tref_affine2d(n->in[1], b), "internal: matmul operand is not a strided view");
        const int64_t M = n->shape[0], N = n->shape[1], K = n->in[0].shape[1];
        auto B = [&](Node* x) { Arg q; q.kind = Arg::BUF; ADHIP_CHECK(x->buffer >= 0, "internal: matmul operand without buffer"); q.buf = x->buffer; return q; };
        auto I = [&](int64_t v) { Arg q; q.kind = Arg::I64; q.iv = v; return q; };
        const bool a_unit = a.s1 == 1 || a.s0 == 1, b_unit = b.s0 == 1 || b.s1 == 1;
        ADHIP_CHECK(!epi || dot_uses_mfma(n), "internal: product epilogue on the small-product kernel");
        if (M * N * K >= 64 * 64 * 64 && a_unit && b_unit) {
            // matrix-core kernel; operands keep their strides (x^T, W^T are never copied)
            DotLaunchPlan pl = plan_dot(n);
            GemmConfig cfg = pl.cfg;
            const int bn_tile = pl.bn_tile;
            ADHIP_CHECK(!cfg.split_k || (partial && !epi), "internal: split product without its slice buffer");
            std::string entry = strf("adhip_gemm_%c%c_%d%s%s%s", cfg.a_kcontig ? 'k' : 'm', cfg.b_kcontig ? 'k' : 'n', cfg.bm,
                                     cfg.bn == 64 && cfg.bm != 64 ? "x64" : "", cfg.edge ? (cfg.edge_vec ? "_rim" : "_edge") : "", cfg.split_k ? "_splitk" : "");
            Launch l;
            if (epi) {
                // the element-wise group that followed the product runs on the accumulators; every distinct
                // epilogue is its own kernel
                entry += strf("_e%d", dot_epilogue_counter++);
                GemmEpilogue ge;
                ge.prelude = kernel_prelude();
                ge.params = epi->params;
                ge.code = epi->code;
                ge.store_c = store_c;
                l.kernel = add_kernel(entry, gemm_kernel_source(cfg, entry, &ge), "dot_mfma");
            } else {
                l.kernel = add_kernel(entry, gemm_kernel_source(cfg, entry), "dot_mfma");
            }
            l.block[0] = cfg.bm == 64 ? 256u : (unsigned)(cfg.bm * 2);
            l.grid[0] = (unsigned)(((M + cfg.bm - 1) / cfg.bm) * ((N + bn_tile - 1) / bn_tile));
            // a product that is not stored has no buffer; the kernel never touches C then
            Node* c_arg = cfg.split_k ? partial : (store_c ? n : (epi ? epi->buffer_args[0] : n));
            l.args = {B(c_arg), B(a.base), B(b.base), I(M), I(N), I(K), I(a.offset), I(a.s0), I(a.s1), I(b.offset), I(b.s0), I(b.s1)};
            if (cfg.split_k) {
                l.args.push_back(I(pl.k_chunk));
                l.grid[1] = (unsigned)pl.splits;
            }
            l.label = strf("dot_%s_%lldx%lldx%lld", n->name.c_str(), (long long)M, (long long)N, (long long)K);
            l.bytes = 4.0 * ((double)M * K + (double)K * N + (store_c ? (double)M * N : 0.0));
            l.flops = 2.0 * (double)M * (double)N * (double)K;
            if (epi) {
                for (Node* x : epi->buffer_args) {
                    l.args.push_back(B(x));
                    l.bytes += 4.0 * (double)std::min<int64_t>(numel(x->shape), M * N);
                }
                l.flops += epi->flops * (double)M * (double)N;
            }
            push_launch(out, l, "dot_mfma");
            if (cfg.split_k) {
                // add the slices in a fixed order
                if (fixed_sum_slices < 0) fixed_sum_slices = add_kernel("adhip_sum_slices", fixed_kernels_source(), "sum_slices");
                Launch lf;
                lf.kernel = fixed_sum_slices;
                lf.block[0] = 256;
                lf.grid[0] = (unsigned)((M * N + 1023) / 1024);
                lf.args = {B(n), B(partial), I(pl.splits), I(M * N)};
                lf.label = l.label + "_sum";
                lf.bytes = 4.0 * (double)M * (double)N * (double)(pl.splits + 1);
                lf.flops = (double)M * (double)N * (double)pl.splits;
                push_launch(out, lf, "sum_slices");
            }
            return;
        }
        if (fixed_dot < 0) fixed_dot = add_kernel("adhip_dot_naive", fixed_kernels_source(), "dot_naive");
        Launch l;
        l.kernel = fixed_dot;
        l.block[0] = 256;
        l.grid[0] = (unsigned)((M * N + 255) / 256);
        l.args = {B(n), B(a.base), B(b.base), I(M), I(N), I(K), I(a.offset), I(a.s0), I(a.s1), I(b.offset), I(b.s0), I(b.s1)};
        l.label = strf("dot_%s_%lldx%lldx%lld", n->name.c_str(), (long long)M, (long long)N, (long long)K);
        l.bytes = 4.0 * ((double)M * K + (double)K * N + (double)M * N);
        l.flops = 2.0 * (double)M * (double)N * (double)K;
        push_launch(out, l, "dot_naive");
    }

    void end_region(const std::vector<std::pair<std::string, Node*>>& wanted) {
        std::set<std::string> homed;
        for (auto& w : wanted) homed.insert(w.first);
        for (auto& kv : env) {
            Binding& b = kv.second;
            if (b.kind == Binding::VAL) {
                const bool is_own_livein = b.node->op == Op::LIVEIN && b.node->name == kv.first;
                if (homed.count(kv.first) || is_own_livein || numel(b.shape) == 0) { b.kind = Binding::HOME; b.node = nullptr; }
                else { b.kind = Binding::NONE; b.node = nullptr; }
            }
        }
        rnodes.clear();
        cse.clear();
        livein.clear();
    }

    // -----------------------------------------------------------------------------------
    // structured walk
    // -----------------------------------------------------------------------------------
    int cond_buffer(const std::string& id) {
        Binding& b = lookup(id);
        ADHIP_CHECK(numel(b.shape) == 1, "control predicate '%s' must have one element, has shape %s", id.c_str(), shape_str(b.shape).c_str());
        return home(id, 1);
    }

    // Recognise `x += inc; t = x + add; cond = t < 0` at the top level of a loop body.
    bool counted_loop(const Cmd& w, Step& step) {
        const Proc& body = *w.block;
        std::map<std::string, float> consts;
        for (auto& kv : env)
            if (kv.second.kind == Binding::CONST) consts[kv.first] = kv.second.c;
        const Cmd* lt = nullptr;
        const Cmd* add = nullptr;
        const Cmd* inc = nullptr;
        std::function<bool(const Proc&)> has_ex = [&](const Proc& p) {
            for (const Cmd& c : p.cmds) {
                if (c.tag == T_EX) return true;
                if (c.tag == T_WHILE && has_ex(*c.block)) return true;
                if (c.tag == T_IF) {
                    for (auto& arm : c.conds) if (has_ex(*arm.second)) return true;
                    if (c.else_block && has_ex(*c.else_block)) return true;
                }
            }
            return false;
        };
        if (has_ex(body)) return false;
        for (const Cmd& c : body.cmds) {
            if (c.tag == T_CREATE_CONSTANT) consts[c.res] = c.f;
            else if ((c.tag == T_ELW_MULTIPLY || c.tag == T_ELW_ADD) && consts.count(c.a) && consts.count(c.b))
                consts[c.res] = c.tag == T_ELW_MULTIPLY ? consts[c.a] * consts[c.b] : consts[c.a] + consts[c.b];
            else if (!c.res.empty()) consts.erase(c.res);
            if (c.tag == T_LESS_ZERO && c.res == w.a) lt = &c;
        }
        if (!lt) return false;
        for (const Cmd& c : body.cmds)
            if (c.tag == T_ELW_ADD && c.res == lt->a) add = &c;
        if (!add) return false;
        std::string x, kadd;
        if (consts.count(add->b) && !consts.count(add->a)) { x = add->a; kadd = add->b; }
        else if (consts.count(add->a) && !consts.count(add->b)) { x = add->b; kadd = add->a; }
        else return false;
        auto bx = env.find(x);
        if (bx == env.end() || numel(bx->second.shape) != 1 || bx->second.kind == Binding::ALIAS || bx->second.kind == Binding::CONST) return false;
        // writes to x, t, cond: exactly the pattern, in this order, all at the top level
        int pos_inc = -1, pos_add = -1, pos_lt = -1;
        std::function<bool(const Proc&, bool)> scan = [&](const Proc& p, bool top) -> bool {
            for (size_t i = 0; i < p.cmds.size(); ++i) {
                const Cmd& c = p.cmds[i];
                if (c.tag == T_WHILE) { if (!scan(*c.block, false)) return false; continue; }
                if (c.tag == T_IF) {
                    for (auto& arm : c.conds) if (!scan(*arm.second, false)) return false;
                    if (c.else_block && !scan(*c.else_block, false)) return false;
                    continue;
                }
                const bool writes = c.res == x || c.res == add->res || c.res == lt->res;
                if (!writes) continue;
                if (!top) return false;
                if (c.res == x) {
                    if (c.tag != T_ELW_ADD_EQ || !consts.count(c.b) || pos_inc >= 0) return false;
                    inc = &c; pos_inc = (int)i;
                } else if (c.res == add->res) {
                    if (&c != add || pos_add >= 0) return false;
                    pos_add = (int)i;
                } else {
                    if (&c != lt || pos_lt >= 0) return false;
                    pos_lt = (int)i;
                }
            }
            return true;
        };
        if (!scan(body, true)) return false;
        if (!(pos_inc >= 0 && pos_inc < pos_add && pos_add < pos_lt)) return false;
        // The increment and the offset must have one value on every trip at the command that uses them: the id is
        // either not defined in the body at all (the value it has before the loop), or defined only by CreateConstant
        // at the top level, every definition with the same value, and -- when the first of them comes after the use --
        // the same value as before the loop too.
        auto invariant_constant = [&](const std::string& id, int use_pos, float& value) -> bool {
            bool ok = true, have = false, defined_before_use = false;
            float v = 0.f;
            std::function<void(const Proc&, bool)> defs = [&](const Proc& p, bool top) {
                for (size_t i = 0; i < p.cmds.size(); ++i) {
                    const Cmd& c = p.cmds[i];
                    if (c.tag == T_WHILE) { defs(*c.block, false); continue; }
                    if (c.tag == T_IF) {
                        for (auto& arm : c.conds) defs(*arm.second, false);
                        if (c.else_block) defs(*c.else_block, false);
                        continue;
                    }
                    if (c.res != id) continue;
                    if (!top || c.tag != T_CREATE_CONSTANT) { ok = false; continue; }
                    if (have && c.f != v) ok = false;
                    have = true;
                    v = c.f;
                    if ((int)i < use_pos) defined_before_use = true;
                }
            };
            defs(body, true);
            if (!ok) return false;
            if (!defined_before_use) {
                auto it = env.find(id);
                if (it == env.end() || it->second.kind != Binding::CONST) return false;
                if (have && it->second.c != v) return false;
                v = it->second.c;
            }
            value = v;
            return true;
        };
        float inc_value = 0.f, add_value = 0.f;
        if (!invariant_constant(inc->b, pos_inc, inc_value) || !invariant_constant(kadd, pos_add, add_value)) return false;
        step.counter_buf = home(x, 1);
        step.counter_inc = inc_value;
        step.counter_add = add_value;
        return true;
    }

    static bool has_loop_or_exit(const Proc& p) {
        for (const Cmd& c : p.cmds) {
            if (c.tag == T_EX || c.tag == T_WHILE) return true;
            if (c.tag == T_IF) {
                for (auto& arm : c.conds)
                    if (has_loop_or_exit(*arm.second)) return true;
                if (c.else_block && has_loop_or_exit(*c.else_block)) return true;
            }
        }
        return false;
    }

    void lower_block(const Proc& p, std::vector<Step>& out, bool once) {
        size_t i = 0;
        const size_t n = p.cmds.size();
        while (true) {
            size_t j = i;
            while (j < n && !is_control(p.cmds[j].tag)) ++j;
            for (size_t k = i; k < j; ++k) build_cmd(p.cmds[k], once);
            IdSet live = region_live[{&p, i}];
            const bool final_region = (j == n && &p == &prog) || (j < n && p.cmds[j].tag == T_EX);
            if (final_region)
                for (auto& d : deps) live.insert(d);
            latch_region = j == n && &p == latch_block;
            flush_region(live, final_region, out);
            latch_region = false;
            if (j == n) break;
            const Cmd& c = p.cmds[j];
            if (c.tag == T_EX) {
                Step s;
                s.kind = Step::EXIT;
                out.push_back(std::move(s));
                break;  // nothing after EX executes
            } else if (c.tag == T_WHILE) {
                Step s;
                s.kind = Step::LOOP;
                s.cond_buf = cond_buffer(c.a);
                s.parent_guard = cur_guard;
                const bool counted = counted_loop(c, s);
                const int saved = cur_guard;
                // a data-dependent loop whose body has no inner loop and no exit runs device-predicated
                if (!counted && cur_guard < 0 && !has_loop_or_exit(*c.block)) {
                    s.flag_slot = plan->n_flags++;
                    cur_guard = s.flag_slot;
                    latch_block = c.block.get();
                    latch_id = c.a;
                    latch_slot = s.flag_slot;
                    latch_attached = false;
                }
                lower_block(*c.block, s.body, false);
                if (s.flag_slot >= 0) {
                    s.latch_in_body = latch_attached;
                    latch_block = nullptr;
                    latch_attached = false;
                }
                cur_guard = saved;
                out.push_back(std::move(s));
            } else {
                Step s;
                s.kind = Step::BRANCH;
                s.parent_guard = cur_guard;
                const int saved = cur_guard;
                const bool predicated = cur_guard >= 0;  // inside a predicated loop the host cannot decide
                if (predicated) s.taken_slot = plan->n_flags++;
                // Bindings are threaded through the arms in program order (shapes follow the last definition in the
                // text, as the reference's trackers do).  An arm drops the binding of an id that is dead after the
                // branch; the next arm, which starts from the state before the branch, may still use it, and so may
                // dead code after the branch: what was bound before the branch stays bound.
                const std::unordered_map<std::string, Binding> before_branch = env;
                auto rebind_dropped = [&]() {
                    for (auto& kv : before_branch) {
                        if (kv.second.kind == Binding::NONE) continue;
                        auto it = env.find(kv.first);
                        if (it == env.end() || it->second.kind == Binding::NONE) env[kv.first] = kv.second;
                    }
                };
                for (auto& arm : c.conds) {
                    std::vector<Step> body;
                    rebind_dropped();
                    int cb = cond_buffer(arm.first);
                    if (predicated) {
                        s.arm_slots.push_back(plan->n_flags++);
                        cur_guard = s.arm_slots.back();
                    }
                    lower_block(*arm.second, body, false);
                    cur_guard = saved;
                    s.arms.emplace_back(cb, std::move(body));
                }
                if (c.else_block) {
                    if (predicated) {
                        s.else_slot = plan->n_flags++;
                        cur_guard = s.else_slot;
                    }
                    rebind_dropped();
                    lower_block(*c.else_block, s.else_body, false);
                    cur_guard = saved;
                }
                rebind_dropped();
                out.push_back(std::move(s));
            }
            i = j + 1;
        }
    }

    std::unique_ptr<Plan> run() {
        collect_alias_srcs(prog);
        if (opt.fuse) {
            AvState st;
            av_block(st, prog, true);
            if (av_poison) reuse.clear();
        }
        IdSet end_live;
        for (auto& d : deps) end_live.insert(d);
        const IdSet start_live = live_block(prog, end_live);
        lower_block(prog, plan->steps, true);
        // an id that is live when the program starts can be read before it is written (defined only on some paths,
        // or only inside a loop that may run zero times): its buffer starts as zeros.  Every other buffer is fully
        // written by a kernel or an upload before its first read and needs no clearing.
        for (const std::string& id : start_live) {
            auto hb = home_buf.find(id);
            if (hb != home_buf.end()) plan->buffers[hb->second].zero_init = true;
        }
        // results
        for (const std::string& d : deps) {
            auto it = env.find(d);
            if (it == env.end()) continue;
            auto hb = home_buf.find(d);
            if (hb == home_buf.end()) continue;
            ResultDesc r;
            r.buf = hb->second;
            r.shape = it->second.shape;
            plan->results[d] = r;
        }
        for (auto& s : slots) plan->slot_elems.push_back(s.first);
        drop_unused_kernels();
        return std::move(plan);
    }

    // Kernels and statistics entries that no launch refers to any more (their launches became phases of a merged
    // launch, or were generated again with a loop flag) are left out of the plan: they would only be compiled.
    void drop_unused_kernels() {
        std::vector<int> kernel_map(plan->kernels.size(), -1), stat_map(plan->stats.size(), -1);
        std::function<void(std::vector<Step>&, bool)> walk = [&](std::vector<Step>& steps, bool assign) {
            for (Step& st : steps) {
                if (st.kind == Step::LAUNCH) {
                    if (!assign) {
                        kernel_map[(size_t)st.launch.kernel] = 0;
                        if (st.launch.stat >= 0) stat_map[(size_t)st.launch.stat] = 0;
                    } else {
                        st.launch.kernel = kernel_map[(size_t)st.launch.kernel];
                        if (st.launch.stat >= 0) st.launch.stat = stat_map[(size_t)st.launch.stat];
                    }
                }
                walk(st.body, assign);
                for (auto& arm : st.arms) walk(arm.second, assign);
                walk(st.else_body, assign);
            }
        };
        walk(plan->steps, false);
        std::vector<KernelDef> kernels;
        for (size_t i = 0; i < plan->kernels.size(); ++i)
            if (kernel_map[i] == 0) { kernel_map[i] = (int)kernels.size(); kernels.push_back(std::move(plan->kernels[i])); }
        std::vector<KernelStat> stats;
        for (size_t i = 0; i < plan->stats.size(); ++i)
            if (stat_map[i] == 0) {
                stat_map[i] = (int)stats.size();
                stats.push_back(std::move(plan->stats[i]));
                stats.back().kernel = kernel_map[(size_t)stats.back().kernel];
            }
        plan->kernels.swap(kernels);
        plan->stats.swap(stats);
        walk(plan->steps, true);
    }
};

void describe_steps(const std::vector<Step>& steps, const Plan& p, int indent, std::string& o) {
    std::string pad((size_t)indent * 2, ' ');
    for (const Step& s : steps) {
        switch (s.kind) {
        case Step::LAUNCH: {
            const Launch& l = s.launch;
            o += pad + strf("launch %s [%s] kernel=%s grid=(%u,%u,%u) block=%u bytes=%.0f flops=%.0f args:", l.label.c_str(),
                            p.kernels[l.kernel].kind.c_str(), p.kernels[l.kernel].entry.c_str(), l.grid[0], l.grid[1], l.grid[2],
                            l.block[0], l.bytes, l.flops);
            for (const Arg& a : l.args) {
                if (a.kind == Arg::BUF) o += " " + p.buffers[a.buf].name + "#" + std::to_string(a.buf) + (a.off ? strf("+%lld", (long long)a.off) : std::string());
                else if (a.kind == Arg::F32) o += strf(" %g", a.fv);
                else if (a.kind == Arg::FLAG) o += strf(" flag%lld", (long long)a.iv);
                else o += strf(" %lld", (long long)a.iv);
            }
            o += "\n";
            break;
        }
        case Step::LOOP:
            o += pad + strf("while %s#%d != 0", p.buffers[s.cond_buf].name.c_str(), s.cond_buf);
            if (s.flag_slot >= 0) o += strf("   [device-predicated, flag %d%s]", s.flag_slot, s.latch_in_body ? ", latched by the body's last kernel" : "");
            if (s.counter_buf >= 0) o += strf("   [counted: %s += %g; cond = (%s + %g) < 0]", p.buffers[s.counter_buf].name.c_str(), s.counter_inc, p.buffers[s.counter_buf].name.c_str(), s.counter_add);
            o += " {\n";
            describe_steps(s.body, p, indent + 1, o);
            o += pad + "}\n";
            break;
        case Step::BRANCH:
            for (size_t i = 0; i < s.arms.size(); ++i) {
                o += pad + strf("%s %s#%d == 1 {\n", i ? "else if" : "if", p.buffers[s.arms[i].first].name.c_str(), s.arms[i].first);
                describe_steps(s.arms[i].second, p, indent + 1, o);
                o += pad + "}\n";
            }
            if (!s.else_body.empty()) {
                o += pad + "else {\n";
                describe_steps(s.else_body, p, indent + 1, o);
                o += pad + "}\n";
            }
            break;
        case Step::EXIT: o += pad + "exit\n"; break;
        }
    }
}

}  // namespace

std::string Plan::describe() const {
    std::string o;
    o += strf("buffers: %zu (temp slots: %zu), kernels: %zu\n", buffers.size(), slot_elems.size(), kernels.size());
    for (size_t i = 0; i < buffers.size(); ++i) {
        const PlanBuffer& b = buffers[i];
        o += strf("  #%zu %s %s elems=%lld%s%s\n", i, b.kind == PlanBuffer::HOME ? "home" : (b.kind == PlanBuffer::TEMP ? "temp" : "const"),
                  b.name.c_str(), (long long)b.elems, b.kind == PlanBuffer::TEMP ? strf(" slot=%d", b.slot).c_str() : "", b.host ? " upload" : "");
    }
    describe_steps(steps, *this, 0, o);
    return o;
}

std::string lowering_switches() {
    std::string out;
    for (const char* name : {"ADHIP_GROUP_DOTS", "ADHIP_LAYER_KERNELS", "ADHIP_MERGE_SMALL", "ADHIP_FUSE_ATTENTION", "ADHIP_ROW_CHAINS",
                             "ADHIP_TIGHTEN", "ADHIP_KERNEL_BOUNDS", "ADHIP_DOT_PLAN", "ADHIP_TILED_SHAPE", "ADHIP_GEMM_AHEAD", "ADHIP_GRAPHS"}) {
        const char* e = getenv(name);
        out += e ? e : "";
        out.push_back(';');
    }
    return out;
}

std::unique_ptr<Plan> lower_program(const Proc& prog, const std::vector<std::string>& dep_ids, const LowerOptions& opt_in) {
    LowerOptions opt = opt_in;
    if (const char* e = getenv("ADHIP_GROUP_DOTS")) opt.group_dots = opt.group_dots && atoi(e) != 0;
    if (const char* e = getenv("ADHIP_LAYER_KERNELS")) opt.layer_kernels = opt.layer_kernels && atoi(e) != 0;
    if (const char* e = getenv("ADHIP_MERGE_SMALL")) opt.merge_small = opt.merge_small && atoi(e) != 0;
    if (const char* e = getenv("ADHIP_FUSE_ATTENTION")) opt.fuse_attention = opt.fuse_attention && atoi(e) != 0;
    if (const char* e = getenv("ADHIP_ROW_CHAINS")) opt.row_chains = opt.row_chains && atoi(e) != 0;
    // diagnostic: every region lowered the way a region is after that many kernels of it spilled vector registers
    if (const char* e = getenv("ADHIP_TIGHTEN")) opt.min_shift = std::max(0, std::min(atoi(e), 4));
    // diagnostic: the seven kernel-size bounds, in the order LowerOptions declares them ("24,48,32,96,40,24,20")
    if (const char* e = getenv("ADHIP_KERNEL_BOUNDS")) {
        int* field[7] = {&opt.max_pieces, &opt.max_inline_sites, &opt.max_inline_loads, &opt.max_kernel_sites, &opt.max_kernel_pointers,
                         &opt.max_carrier_sites, &opt.max_carrier_pointers};
        for (int i = 0; i < 7 && *e; ++i) {
            char* end = nullptr;
            const long v = strtol(e, &end, 10);
            if (end == e) break;
            if (v >= 2) *field[i] = (int)std::min<long>(v, 1 << 20);
            e = *end == ',' ? end + 1 : end;
        }
    }
    Lowerer l(prog, dep_ids, opt);
    return l.run();
}

}  // namespace adhip
