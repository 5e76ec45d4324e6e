#include "codegen.hpp"

#include <algorithm>
#include <cctype>
#include <climits>
#include <cstdlib>
#include <cstring>
#include <functional>

namespace adhip {

const char* op_name(Op o) {
    switch (o) {
    case Op::LIVEIN: return "livein";
    case Op::UPLOAD: return "upload";
    case Op::ADD: return "add";
    case Op::MUL: return "mul";
    case Op::EXP2: return "exp2";
    case Op::LOG2: return "log2";
    case Op::SIN: return "sin";
    case Op::RECIP: return "recip";
    case Op::SQRT: return "sqrt";
    case Op::EQ0: return "eq0";
    case Op::GT0: return "gt0";
    case Op::LT0: return "lt0";
    case Op::COPY: return "copy";
    case Op::FILL: return "fill";
    case Op::SUM: return "sum";
    case Op::MAX: return "max";
    case Op::DOT: return "dot";
    case Op::ATTN: return "attention";
    }
    return "?";
}

const char* kernel_prelude() {
    // Everything the generated kernels need besides what hipRTC provides by itself.
    return R"(
typedef float float4_t __attribute__((ext_vector_type(4)));
static __device__ __forceinline__ float u2f(unsigned u) { return __builtin_bit_cast(float, u); }
// Sums and maxima over a wavefront: within each row of 16 lanes by data-parallel-primitive moves (neighbour, other
// pair, other quad mirrored, other half mirrored: register-to-register, no LDS round trip), then across the four rows.
// Every lane ends up with the same bits.
template <int CTRL> static __device__ __forceinline__ float wave_dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
static __device__ __forceinline__ float wave_sum(float v) {
    v += wave_dpp<0xB1>(v);
    v += wave_dpp<0x4E>(v);
    v += wave_dpp<0x141>(v);
    v += wave_dpp<0x140>(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
static __device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, wave_dpp<0xB1>(v));
    v = fmaxf(v, wave_dpp<0x4E>(v));
    v = fmaxf(v, wave_dpp<0x141>(v));
    v = fmaxf(v, wave_dpp<0x140>(v));
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}
// sin(x) for |x| <= 2^15 in ~15 instructions: x = k*pi + r with pi split in three floats (each fma is exact or rounds
// once, so r keeps full relative accuracy next to a multiple of pi), an odd polynomial of degree 11 on
// [-pi/2, pi/2], sign from the parity of k.  At most 2.1 ulp from the exact value (checked on the host over
// 4e7 arguments per binade range).  Larger, infinite arguments take the library routine; NaN passes through.
static __device__ __forceinline__ float adhip_sinf(float x) {
    const float k = __builtin_rintf(x * 0.318309886183790672f);
    float r = __builtin_fmaf(-k, 3.14159274101257324f, x);
    r = __builtin_fmaf(-k, -8.74227765734758577e-08f, r);
    r = __builtin_fmaf(-k, -3.4302490200117637e-15f, r);
    const float s = r * r;
    float p = __builtin_fmaf(-2.381510633e-08f, s, 2.752115961e-06f);
    p = __builtin_fmaf(p, s, -1.984078554e-04f);
    p = __builtin_fmaf(p, s, 8.333330043e-03f);
    p = __builtin_fmaf(p, s, -1.666666716e-01f);
    float res = __builtin_fmaf(r * s, p, r);
    res = __builtin_bit_cast(float, __builtin_bit_cast(unsigned, res) ^ ((unsigned)(int)k << 31));
    if (__builtin_expect(!(__builtin_fabsf(x) <= 32768.0f), 0)) res = sinf(x);
    return res;
}
)";
}

namespace {

// Buffers at least this large (elements) are read and written with non-temporal accesses: they cannot stay in the
// 256 MiB last-level cache until their next use anyway, and streaming them through it evicts (and, for dirty lines,
// writes back) whatever the neighbouring kernels could have reused.  ADHIP_NONTEMPORAL_MIB overrides the size in MiB;
// 0 turns non-temporal accesses off.
// Row length, in bytes, of the bands large flat element-wise kernels are cut into (see gen_elw_kernel); 0 turns the
// banded order off.  ADHIP_ELW_BAND_KIB overrides the default of 32 KiB (multiples of 1 KiB).
int64_t elw_band_bytes() {
    static const int64_t v = [] {
        int64_t kib = 32;
        if (const char* e = getenv("ADHIP_ELW_BAND_KIB")) kib = atoll(e);
        return kib < 0 ? 0 : kib * 1024;
    }();
    return v;
}

int64_t nontemporal_min_elems() {
    static const int64_t v = [] {
        int64_t mib = 256;
        if (const char* e = getenv("ADHIP_NONTEMPORAL_MIB")) mib = atoll(e);
        return mib <= 0 ? LLONG_MAX : mib * (int64_t(1) << 20) / 4;
    }();
    return v;
}

// ---------------------------------------------------------------------------------------
// symbolic integer index arithmetic: c + sum(coef * atom), atoms with known ranges
// ---------------------------------------------------------------------------------------

struct Atom {
    std::string name;
    int64_t range = 1;  // value in [0, range) whenever the access it feeds is selected
    bool lane = false;  // differs between the lanes of one thread's vector
    std::string code;   // derived atoms: the expression (over earlier atoms) that defines them
};

struct Aff {
    int64_t c = 0;
    std::vector<std::pair<int, int64_t>> t;  // (atom, coef), sorted by atom, coef != 0
};

Aff aff_const(int64_t c) { Aff a; a.c = c; return a; }
Aff aff_atom(int id, int64_t coef = 1) { Aff a; if (coef) a.t.push_back({id, coef}); return a; }

Aff aff_add(const Aff& a, const Aff& b) {
    Aff r;
    r.c = a.c + b.c;
    size_t i = 0, j = 0;
    while (i < a.t.size() || j < b.t.size()) {
        if (j >= b.t.size() || (i < a.t.size() && a.t[i].first < b.t[j].first)) r.t.push_back(a.t[i++]);
        else if (i >= a.t.size() || b.t[j].first < a.t[i].first) r.t.push_back(b.t[j++]);
        else {
            int64_t k = a.t[i].second + b.t[j].second;
            if (k) r.t.push_back({a.t[i].first, k});
            ++i; ++j;
        }
    }
    return r;
}

Aff aff_scale(const Aff& a, int64_t k) {
    Aff r;
    if (k == 0) return r;
    r.c = a.c * k;
    for (auto& x : a.t) r.t.push_back({x.first, x.second * k});
    return r;
}

std::string aff_key(const Aff& a) {
    std::string s = std::to_string(a.c);
    for (auto& x : a.t) s += "+" + std::to_string(x.second) + "*" + std::to_string(x.first);
    return s;
}

struct Val {
    std::string expr;
    bool lane = false;
};

struct LoadRec {
    const Node* node;
    Aff idx;
    bool predicated;
    std::string key;
};

struct Gen {
    int vec = 1;
    int lane_atom = -1;
    bool wide = false;
    std::vector<Atom> atoms;
    std::vector<std::string> codeA, codeB;  // per-thread / per-lane statements
    std::map<std::string, int> atom_memo;
    std::map<std::string, Val> val_memo;
    std::map<std::string, bool> pred_lane;
    std::map<const Node*, int> buf_index;
    std::vector<GenBuffer> bufs;
    std::set<const Node*> members;  // computed in this kernel, never loaded
    std::map<const Node*, std::string> preset;  // nodes whose value is a variable the kernel already holds
    std::map<const Node*, std::string> preset_at;  // ... and, where given, the only index (aff_key) that variable stands for
    std::vector<LoadRec> loads;
    std::vector<Aff> recorded;  // every index expression over base atoms, for dim merging
    // Tiled element-wise kernels: loads whose key is in `stage_keys` are not issued by the thread that needs the value;
    // the block reads the 64x64 tile they come from through LDS (see gen_elw_tiled_kernel).  `index_code` collects, in
    // order, every statement that defines an index atom or a predicate (no loads, no arithmetic on values), so that
    // the staging phase can evaluate the same index at other coordinates.
    std::set<std::string> stage_keys;
    struct Staged { std::string key, param, index, pred; int slot; };
    std::vector<Staged> staged;
    std::vector<std::string> index_code;
    std::string tile_row_origin, tile_col_origin;  // expressions of the tile's first row / first column
    int tile_rows = 64, tile_cols = 64;
    int row_atom = -1;
    int tmp = 0;
    double flops = 0;  // per lane element
    // Row-chain kernels: a 128-bit load whose key is in `keep_keys` is held in a per-thread array indexed by the
    // (fully unrolled) sweep counter `keep_index`, so that a later sweep takes it from registers; `sweep_loads`
    // collects the keys of the vector loads the current sweep makes.
    std::set<std::string> keep_keys, sweep_loads;
    std::map<std::string, std::string> kept_arrays;
    std::vector<std::string> kept_decls;
    std::string keep_index;

    const char* idx_t() const { return wide ? "unsigned long long" : "unsigned int"; }

    int add_atom(const std::string& name, int64_t range, bool lane) {
        atoms.push_back({name, range, lane});
        return (int)atoms.size() - 1;
    }

    int64_t aff_max(const Aff& a) const {
        int64_t m = a.c;
        for (auto& x : a.t)
            if (x.second > 0) m += x.second * (atoms[x.first].range - 1);
        return m;
    }
    int64_t aff_min(const Aff& a) const {
        int64_t m = a.c;
        for (auto& x : a.t)
            if (x.second < 0) m += x.second * (atoms[x.first].range - 1);
        return m;
    }
    // whether atom `a` is atom `base` or is computed from it
    bool atom_depends_on(int a, int base) const {
        if (a == base) return true;
        const std::string& code = atoms[(size_t)a].code;
        if (code.empty()) return false;
        auto mentions = [&](const std::string& name) {
            for (size_t pos = code.find(name); pos != std::string::npos; pos = code.find(name, pos + 1)) {
                const bool left = pos == 0 || !(isalnum((unsigned char)code[pos - 1]) || code[pos - 1] == '_');
                const size_t end = pos + name.size();
                const bool right = end >= code.size() || !(isalnum((unsigned char)code[end]) || code[end] == '_');
                if (left && right) return true;
            }
            return false;
        };
        for (int b = 0; b < a; ++b)
            if (mentions(atoms[(size_t)b].name) && atom_depends_on(b, base)) return true;
        return false;
    }
    bool aff_lane(const Aff& a) const {
        for (auto& x : a.t)
            if (atoms[x.first].lane) return true;
        return false;
    }

    std::string aff_str(const Aff& a) {
        recorded.push_back(a);
        if (a.t.empty()) return strf("(%s)%lld", idx_t(), (long long)a.c) + (wide ? "ull" : "u");
        std::string s = "(";
        bool first = true;
        for (auto& x : a.t) {
            if (!first) s += " + ";
            first = false;
            if (x.second == 1) s += atoms[x.first].name;
            else s += strf("%lld%s * %s", (long long)x.second, wide ? "ull" : "u", atoms[x.first].name.c_str());
        }
        if (a.c) s += strf(" + %lld%s", (long long)a.c, wide ? "ull" : "u");
        return s + ")";
    }

    void emit(bool lane, const std::string& stmt) { (lane ? codeB : codeA).push_back(stmt); }

    // an atom defined by an expression over other atoms
    int expr_atom(const std::string& code, int64_t range, bool lane) {
        auto it = atom_memo.find(code);
        if (it != atom_memo.end()) return it->second;
        std::string name = "a" + std::to_string(tmp++);
        emit(lane, strf("const %s %s = %s;", idx_t(), name.c_str(), code.c_str()));
        index_code.push_back(strf("const %s %s = %s;", idx_t(), name.c_str(), code.c_str()));
        int id = add_atom(name, range, lane);
        atoms[(size_t)id].code = code;
        atom_memo[code] = id;
        return id;
    }

    // exact a / k when every term divides, else an opaque quotient atom
    Aff aff_div(const Aff& a, int64_t k) {
        if (k == 1) return a;
        bool exact = a.c % k == 0;
        for (auto& x : a.t) exact = exact && (x.second % k == 0);
        if (exact) {
            Aff r;
            r.c = a.c / k;
            for (auto& x : a.t) r.t.push_back({x.first, x.second / k});
            return r;
        }
        int64_t mx = aff_max(a);
        if (mx < k && aff_min(a) >= 0) return aff_const(0);
        std::string code = strf("%s / %lld%s", aff_str(a).c_str(), (long long)k, wide ? "ull" : "u");
        return aff_atom(expr_atom(code, mx / k + 1, aff_lane(a)));
    }

    Aff aff_mod(const Aff& a, int64_t k) {
        if (aff_max(a) < k && aff_min(a) >= 0) return a;
        std::string code = strf("%s %% %lld%s", aff_str(a).c_str(), (long long)k, wide ? "ull" : "u");
        return aff_atom(expr_atom(code, k, aff_lane(a)));
    }

    // Split a linear row-major index over `shape` into coordinates.
    std::vector<Aff> split(const Aff& e, const Shape& shape) {
        const size_t n = shape.size();
        std::vector<Aff> out(n);
        if (n == 0) return out;
        if (n == 1) { out[0] = e; return out; }
        Shape r = row_major_strides(shape);
        Aff rem = e;
        for (size_t j = n - 1; j >= 1; --j) {
            const int64_t M = r[j] * shape[j];
            Aff low, high;
            bool ok = rem.c >= 0;
            low.c = rem.c >= 0 ? rem.c % M : 0;
            high.c = rem.c - low.c;
            if (low.c % r[j] != 0) ok = false;
            for (auto& x : rem.t) {
                if (x.second < 0) { ok = false; break; }
                if (x.second % M == 0) high.t.push_back(x);
                else if (x.second < M && x.second % r[j] == 0) low.t.push_back(x);
                else { ok = false; break; }
            }
            if (ok && aff_max(low) < M) {
                out[j] = aff_div(low, r[j]);
                rem = high;
                continue;
            }
            // Fall back to explicit div/mod from this dim outwards.
            Aff q = aff_div(rem, r[j]);
            for (size_t jj = j; jj >= 1; --jj) {
                out[jj] = aff_mod(q, shape[jj]);
                q = aff_div(q, shape[jj]);
            }
            out[0] = q;
            return out;
        }
        out[0] = aff_div(rem, r[0]);
        return out;
    }

    static bool stage_row_major(const Stage& s) {
        int64_t expect = 1;
        for (int i = (int)s.shape.size() - 1; i >= 0; --i) {
            if (s.shape[i] == 1) continue;
            if (s.stride[i] != expect) return false;
            expect *= s.shape[i];
        }
        return true;
    }

    Aff apply_stage_coords(const Stage& s, const std::vector<Aff>& coords) {
        Aff l = aff_const(s.offset);
        for (size_t i = 0; i < s.shape.size(); ++i) {
            if (s.shape[i] == 1 || s.stride[i] == 0) continue;
            l = aff_add(l, aff_scale(coords[i], s.stride[i]));
        }
        return l;
    }

    Aff apply_view_from(const View& v, size_t k, Aff l) {
        for (; k < v.st.size(); ++k) {
            const Stage& s = v.st[k];
            if (stage_row_major(s)) { l = aff_add(l, aff_const(s.offset)); continue; }
            l = apply_stage_coords(s, split(l, s.shape));
        }
        return l;
    }

    int buffer_of(const Node* n) {
        auto it = buf_index.find(n);
        if (it != buf_index.end()) return it->second;
        // the lowering bounds what a kernel reads long before this; a kernel that names hundreds of buffers would
        // take minutes to compile and could only run by spilling registers
        ADHIP_CHECK(bufs.size() < 192, "internal: a generated kernel names more than 192 operand buffers");
        GenBuffer b;
        b.node = const_cast<Node*>(n);
        b.param = "b" + std::to_string(bufs.size());
        bufs.push_back(b);
        buf_index[n] = (int)bufs.size() - 1;
        return (int)bufs.size() - 1;
    }

    static std::string flit(float f) {
        unsigned u;
        memcpy(&u, &f, 4);
        return strf("u2f(0x%08xu)", u);
    }

    bool vectorizable(const Aff& idx) const {
        if (vec == 1 || lane_atom < 0) return false;
        if (idx.c % vec != 0) return false;
        bool has_lane = false;
        for (auto& x : idx.t) {
            if (x.first == lane_atom) {
                if (x.second != 1) return false;
                has_lane = true;
            } else {
                if (atoms[x.first].lane) return false;
                if (x.second % vec != 0) return false;
            }
        }
        return has_lane;
    }

    Val load(const Node* n, const Aff& idx, const std::string& pred) {
        const bool plane = !pred.empty() && pred_lane[pred];
        std::string key = "L" + std::to_string(n->id) + "@" + aff_key(idx) + "?" + pred;
        auto it = val_memo.find(key);
        if (it != val_memo.end()) return it->second;
        const int64_t ne = numel(n->shape);
        ADHIP_CHECK(aff_min(idx) >= 0 && aff_max(idx) < ne,
                    "internal: generated load of node %d (%s) spans [%lld,%lld] outside its %lld elements", n->id,
                    n->name.c_str(), (long long)aff_min(idx), (long long)aff_max(idx), (long long)ne);
        loads.push_back({n, idx, !pred.empty(), key});
        const std::string& bp = bufs[buffer_of(n)].param;
        std::string name = "l" + std::to_string(tmp++);
        Val v;
        const bool ilane = aff_lane(idx);
        const bool nt = ne >= nontemporal_min_elems();
        if (stage_keys.count(key)) {
            // the value was put into LDS by the staging phase: tile[column within the tile][row within the tile]
            ADHIP_CHECK(lane_atom >= 0 && row_atom >= 0 && vec == 4, "internal: staged load outside a tiled kernel");
            const int slot = (int)staged.size();
            staged.push_back({key, bp, aff_str(idx), pred, slot});
            const std::string& last = atoms[(size_t)lane_atom - 1].name;  // the atom of the innermost dim (float4 index)
            emit(true, strf("const float %s = tile%d[(4u * %s + %s) - %s][%s - %s];", name.c_str(), slot, last.c_str(),
                            atoms[lane_atom].name.c_str(), tile_col_origin.c_str(), atoms[row_atom].name.c_str(), tile_row_origin.c_str()));
            v = {name, true};
            val_memo[key] = v;
            return v;
        }
        if (!ilane && !plane) {
            if (pred.empty()) emit(false, strf("const float %s = %s[%s];", name.c_str(), bp.c_str(), aff_str(idx).c_str()));
            else emit(false, strf("const float %s = %s ? %s[%s] : 0.0f;", name.c_str(), pred.c_str(), bp.c_str(), aff_str(idx).c_str()));
            v = {name, false};
        } else if (!plane && vectorizable(idx)) {
            Aff base = idx;
            for (auto it2 = base.t.begin(); it2 != base.t.end(); ++it2)
                if (it2->first == lane_atom) { base.t.erase(it2); break; }
            const std::string at = aff_str(base);
            std::string addr = nt ? strf("__builtin_nontemporal_load((const float4_t*)(%s + %s))", bp.c_str(), at.c_str())
                                  : strf("*(const float4_t*)(%s + %s)", bp.c_str(), at.c_str());
            if (pred.empty()) sweep_loads.insert(key);
            if (pred.empty() && keep_keys.count(key)) {
                auto kept = kept_arrays.find(key);
                if (kept == kept_arrays.end()) {
                    const std::string arr = "rk" + std::to_string(kept_arrays.size());
                    kept_arrays[key] = arr;
                    kept_decls.push_back(arr);
                    emit(false, strf("const float4_t %sv = (%s[%s] = %s);", name.c_str(), arr.c_str(), keep_index.c_str(), addr.c_str()));
                } else {
                    emit(false, strf("const float4_t %sv = %s[%s];", name.c_str(), kept->second.c_str(), keep_index.c_str()));
                }
            } else if (pred.empty()) emit(false, strf("const float4_t %sv = %s;", name.c_str(), addr.c_str()));
            else emit(false, strf("float4_t %sv = {0.f, 0.f, 0.f, 0.f}; if (%s) %sv = %s;", name.c_str(), pred.c_str(), name.c_str(), addr.c_str()));
            if (pred.empty()) {
                emit(false, strf("const float %s[4] = {%sv.x, %sv.y, %sv.z, %sv.w};", name.c_str(), name.c_str(), name.c_str(), name.c_str(), name.c_str()));
                v = {name + "[" + atoms[lane_atom].name + "]", true};
            } else {
                // no array of the four elements here: a select between elements of two such arrays under the loads'
                // own predicates is turned into a load through a selected address, which puts the arrays into scratch
                v = {name + "v[" + atoms[lane_atom].name + "]", true};
            }
        } else {
            if (pred.empty()) emit(true, strf("const float %s = %s[%s];", name.c_str(), bp.c_str(), aff_str(idx).c_str()));
            else emit(true, strf("const float %s = %s ? %s[%s] : 0.0f;", name.c_str(), pred.c_str(), bp.c_str(), aff_str(idx).c_str()));
            v = {name, true};
        }
        val_memo[key] = v;
        return v;
    }

    std::string and_pred(const std::string& pred, const std::string& cond, bool cond_lane) {
        std::string key = "P" + pred + "&" + cond;
        auto it = val_memo.find(key);
        if (it != val_memo.end()) return it->second.expr;
        std::string name = "p" + std::to_string(tmp++);
        bool lane = cond_lane || (!pred.empty() && pred_lane[pred]);
        emit(lane, strf("const bool %s = %s%s;", name.c_str(), pred.empty() ? "" : (pred + " && ").c_str(), cond.c_str()));
        index_code.push_back(strf("const bool %s = %s%s;", name.c_str(), pred.empty() ? "" : (pred + " && ").c_str(), cond.c_str()));
        pred_lane[name] = lane;
        val_memo[key] = {name, lane};
        return name;
    }

    Val gen_src(const Piece& p, const Aff& idx, const std::string& pred) {
        switch (p.src.kind) {
        case Src::CONST: return {flit(p.src.c), false};
        case Src::NODE: return gen_node(p.src.node, idx, pred);
        default: throw Error("internal: unresolved tensor reference reached code generation");
        }
    }

    // value of tensor reference `t` at linear (row-major over t.shape) index l
    Val gen_tref(const TRef& t, const Aff& l, const std::string& pred) {
        ADHIP_CHECK(!t.pieces.empty(), "internal: empty tensor reference in code generation");
        if (t.single_full()) {
            const Piece& p = t.pieces[0];
            if (p.src.kind == Src::CONST) return {flit(p.src.c), false};
            return gen_src(p, apply_view_from(p.view, 0, l), pred);
        }
        std::vector<Aff> coords = split(l, t.shape);
        std::vector<Val> vals;
        std::vector<std::string> conds;
        std::vector<bool> cond_lanes;
        for (size_t pi = 0; pi < t.pieces.size(); ++pi) {
            const Piece& p = t.pieces[pi];
            std::string cond;
            bool clane = false;
            std::vector<Aff> local(coords.size());
            for (size_t d = 0; d < coords.size(); ++d) {
                const bool partial = p.lo[d] != 0 || p.hi[d] != t.shape[d];
                if (!partial) { local[d] = coords[d]; continue; }
                if (vec > 1 && p.lo[d] % vec == 0 && (p.hi[d] - p.lo[d]) % vec == 0 && vectorizable(coords[d])) {
                    // The elements of one 128-bit access lie on the same side of a boundary at a multiple of four: the
                    // condition and the piece's own coordinate are the quad's, so the loads under the condition stay
                    // vector loads (a Concat of heads along the last dim, the gathered halves of a row).
                    Aff base = coords[d];
                    for (auto it2 = base.t.begin(); it2 != base.t.end(); ++it2)
                        if (it2->first == lane_atom) { base.t.erase(it2); break; }
                    const std::string bs = aff_str(base);
                    if (p.lo[d] != 0) cond += strf("%s%s >= %lldu", cond.empty() ? "" : " && ", bs.c_str(), (long long)p.lo[d]);
                    if (p.hi[d] != t.shape[d]) cond += strf("%s%s < %lldu", cond.empty() ? "" : " && ", bs.c_str(), (long long)p.hi[d]);
                    const std::string code = p.lo[d] != 0 ? strf("(%s - %lld%s) / %d%s", bs.c_str(), (long long)p.lo[d], wide ? "ull" : "u", vec, wide ? "ull" : "u")
                                                          : strf("%s / %d%s/*<%lld*/", bs.c_str(), vec, wide ? "ull" : "u", (long long)(p.hi[d] / vec));
                    const int qa = expr_atom(code, (p.hi[d] - p.lo[d]) / vec, false);
                    local[d] = aff_add(aff_atom(qa, vec), aff_atom(lane_atom, 1));
                    continue;
                }
                clane = clane || aff_lane(coords[d]);
                std::string cs = aff_str(coords[d]);
                if (p.lo[d] != 0) cond += strf("%s%s >= %lldu", cond.empty() ? "" : " && ", cs.c_str(), (long long)p.lo[d]);
                if (p.hi[d] != t.shape[d]) cond += strf("%s%s < %lldu", cond.empty() ? "" : " && ", cs.c_str(), (long long)p.hi[d]);
                if (p.lo[d] != 0) {
                    std::string code = strf("%s - %lld%s", cs.c_str(), (long long)p.lo[d], wide ? "ull" : "u");
                    local[d] = aff_atom(expr_atom(code, p.hi[d] - p.lo[d], aff_lane(coords[d])));
                } else {
                    // same variable, tighter range while this piece is selected
                    std::string code = strf("%s + 0u", cs.c_str());
                    local[d] = aff_atom(expr_atom(code + strf("/*<%lld*/", (long long)p.hi[d]), p.hi[d], aff_lane(coords[d])));
                }
            }
            std::string ppred = cond.empty() ? pred : and_pred(pred, "(" + cond + ")", clane);
            Val v;
            if (p.src.kind == Src::CONST) v = {flit(p.src.c), false};
            else {
                Aff idx = apply_stage_coords(p.view.st[0], local);
                idx = apply_view_from(p.view, 1, idx);
                v = gen_src(p, idx, ppred);
            }
            vals.push_back(v);
            conds.push_back(cond.empty() ? "" : ppred);
            cond_lanes.push_back(!cond.empty() && pred_lane[ppred]);
        }
        // select chain; the last piece is the default
        std::string e = vals.back().expr;
        bool lane = vals.back().lane;
        for (size_t pi = t.pieces.size() - 1; pi-- > 0;) {
            if (conds[pi].empty()) { e = vals[pi].expr; lane = vals[pi].lane; continue; }
            e = "(" + conds[pi] + " ? " + vals[pi].expr + " : " + e + ")";
            lane = lane || vals[pi].lane || cond_lanes[pi];
        }
        std::string name = "s" + std::to_string(tmp++);
        emit(lane, strf("const float %s = %s;", name.c_str(), e.c_str()));
        return {name, lane};
    }

    bool in_memory(const Node* n) const { return (op_is_leaf(n->op) || n->root) && !members.count(n); }

    Val gen_node(const Node* n, const Aff& l, const std::string& pred) {
        {
            auto ps = preset.find(n);
            if (ps != preset.end()) {
                auto at = preset_at.find(n);
                ADHIP_CHECK(at == preset_at.end() || at->second == aff_key(l), "internal: node %d is held for index %s, wanted at %s", n->id,
                            at->second.c_str(), aff_key(l).c_str());
                return {ps->second, false};
            }
        }
        if (in_memory(n)) return load(n, l, pred);
        if (n->op == Op::FILL) return {flit(n->cval), false};
        ADHIP_CHECK(op_is_elw(n->op), "internal: node %d (%s) is neither in memory nor element-wise", n->id, op_name(n->op));
        std::string key = "N" + std::to_string(n->id) + "@" + aff_key(l) + "?" + pred;
        auto it = val_memo.find(key);
        if (it != val_memo.end()) return it->second;
        std::vector<Val> a;
        for (const TRef& t : n->in) a.push_back(gen_tref(t, l, pred));
        bool lane = false;
        for (auto& v : a) lane = lane || v.lane;
        std::string e;
        const std::string& x = a[0].expr;
        switch (n->op) {
        case Op::ADD: e = x + " + " + a[1].expr; break;
        case Op::MUL: e = x + " * " + a[1].expr; break;
        case Op::EXP2: e = "exp2f(" + x + ")"; break;
        case Op::LOG2: e = "log2f(" + x + ")"; break;
        case Op::SIN: e = "adhip_sinf(" + x + ")"; break;
        case Op::RECIP: e = "1.0f / " + x; break;
        case Op::SQRT: e = "sqrtf(fabsf(" + x + "))"; break;
        case Op::EQ0: e = "(" + x + " == 0.0f) ? 1.0f : 0.0f"; break;
        case Op::GT0: e = "(" + x + " > 0.0f) ? 1.0f : 0.0f"; break;
        case Op::LT0: e = "(" + x + " < 0.0f) ? 1.0f : 0.0f"; break;
        case Op::COPY: e = x; break;
        default: throw Error("internal: unexpected op in element-wise code generation");
        }
        if (n->op != Op::COPY) flops += op_is_transcendental(n->op) ? 8 : 1;
        std::string name = "v" + std::to_string(tmp++);
        emit(lane, strf("const float %s = %s;", name.c_str(), e.c_str()));
        Val v{name, lane};
        val_memo[key] = v;
        return v;
    }
};

// statement that stores the four floats w[0..3] at `addr` (a float pointer expression), 128 bits wide
std::string store4_stmt(const std::string& w, const std::string& addr, bool nontemporal) {
    std::string q = strf("{ float4_t q = {%s[0], %s[1], %s[2], %s[3]}; ", w.c_str(), w.c_str(), w.c_str(), w.c_str());
    if (nontemporal) return q + "__builtin_nontemporal_store(q, (float4_t*)(" + addr + ")); }";
    return q + "*(float4_t*)(" + addr + ") = q; }";
}

std::string join(const std::vector<std::string>& v, const char* indent) {
    std::string s;
    for (auto& x : v) s += std::string(indent) + x + "\n";
    return s;
}

bool needs_wide(const std::vector<Node*>& nodes) {
    int64_t m = 0;
    std::set<const Node*> seen;
    std::function<void(const Node*)> walk = [&](const Node* n) {
        if (!seen.insert(n).second) return;
        m = std::max(m, numel(n->shape));
        for (auto& t : n->in)
            for (auto& p : t.pieces)
                if (p.src.kind == Src::NODE) walk(p.src.node);
    };
    for (auto n : nodes) walk(n);
    return m >= (int64_t(1) << 31) - 1024;
}

Shape drop_ones(const Shape& s) {
    Shape r;
    for (auto d : s)
        if (d != 1) r.push_back(d);
    if (r.empty()) r.push_back(1);
    return r;
}

// bytes moved by a kernel, counting each distinct buffer once
double traffic_bytes(const Gen& g, int64_t work_elems) {
    double b = 0;
    for (auto& gb : g.bufs) b += 4.0 * (double)std::min<int64_t>(numel(gb.node->shape), gb.written ? numel(gb.node->shape) : std::max<int64_t>(work_elems, 1));
    return b;
}

// Iteration shapes: merge adjacent dims whose atoms always appear as one linear combination.
Shape merge_dims(const Shape& shape, const std::vector<Aff>& recorded, const std::vector<int>& dim_atoms) {
    // dim_atoms[i] = atom id of dim i (base atoms); returns merged shape
    std::vector<bool> merge_with_next(shape.size(), false);
    for (size_t i = 0; i + 1 < shape.size(); ++i) {
        bool ok = true;
        for (const Aff& a : recorded) {
            int64_t ci = 0, cn = 0;
            for (auto& x : a.t) {
                if (x.first == dim_atoms[i]) ci = x.second;
                if (x.first == dim_atoms[i + 1]) cn = x.second;
            }
            if (ci != cn * shape[i + 1]) { ok = false; break; }
        }
        merge_with_next[i] = ok;
    }
    Shape out;
    int64_t cur = shape.empty() ? 1 : shape[0];
    for (size_t i = 0; i + 1 < shape.size(); ++i) {
        if (merge_with_next[i]) cur *= shape[i + 1];
        else { out.push_back(cur); cur = shape[i + 1]; }
    }
    out.push_back(cur);
    return out;
}

}  // namespace

// ---------------------------------------------------------------------------------------
// element-wise kernels
// ---------------------------------------------------------------------------------------

namespace {

struct ElwBody {
    Gen g;
    std::vector<std::string> out_exprs;
    std::vector<std::string> cs_exprs;
    std::vector<std::string> rs_exprs;
    std::vector<int> dim_atoms;
    Shape iter_shape;
};

ElwBody elw_body(const ElwKernelSpec& spec, const std::set<const Node*>& members, const Shape& iter_shape, int vec,
                 bool wide, const std::function<void(Gen&)>& setup = nullptr) {
    ElwBody b;
    b.iter_shape = iter_shape;
    Gen& g = b.g;
    g.vec = vec;
    g.wide = wide;
    g.members = members;
    if (setup) setup(g);
    const size_t nd = iter_shape.size();
    Shape rs = row_major_strides(iter_shape);
    Aff lin;
    for (size_t i = 0; i < nd; ++i) {
        const bool last = i + 1 == nd;
        int64_t range = last ? iter_shape[i] / vec : iter_shape[i];
        int a = g.add_atom("c" + std::to_string(i), range, false);
        b.dim_atoms.push_back(a);
        lin = aff_add(lin, aff_atom(a, last ? vec : rs[i]));
    }
    if (vec > 1) {
        g.lane_atom = g.add_atom("j", vec, true);
        lin = aff_add(lin, aff_atom(g.lane_atom, 1));
    }
    for (Node* out : spec.outputs) {
        // an output is computed from its operands even though it ends up in memory
        ADHIP_CHECK(op_is_elw(out->op), "internal: element-wise kernel asked to produce %s", op_name(out->op));
        Val v = g.gen_node(out, lin, "");
        b.out_exprs.push_back(v.expr);
    }
    for (auto& cs : spec.colsums) {
        Val v = g.gen_node(cs.value, lin, "");
        b.cs_exprs.push_back(v.expr);
    }
    for (auto& rs : spec.rowsums) {
        Val v = g.gen_node(rs.value, lin, "");
        b.rs_exprs.push_back(v.expr);
    }
    return b;
}

}  // namespace

// Rows one block of the column-sum layout covers: 16 (one per wavefront), times the number of rows each wavefront
// walks.  That is 1 until the partial sums would exceed 1024 rows -- except for passes that move few streams (at most
// three of: results stored, full-size operands read), where a block's closing steps (the sums across the wavefront,
// the 16 rows through LDS) weigh more against its streaming: two rows per wavefront then, if that still leaves eight
// blocks per CU.  Measured on 16384 x 4096 with one operand, one result, row and column sums: 103 -> 96 us a step
// (three and four rows: 98 and 100); on the 3-read + 4-write pass over 8192 x 8192 two rows per wavefront cost 1.5 %
// instead.
static int64_t elw_colsum_rows_per_wave(int64_t rows, int64_t cols, int streams) {
    const int64_t base = std::max<int64_t>(1, (rows + 16 * 1024 - 1) / (16 * 1024));
    if (base == 1 && streams <= 3 && ((cols / 4 + 63) / 64) * ((rows + 31) / 32) >= 2048) return 2;
    return base;
}

int64_t elw_rowsum_runs(int64_t cols) { return (cols / 4 + 63) / 64; }

int64_t elw_colsum_tiles(int64_t rows, int64_t cols, int streams) {
    const int64_t per_block = 16 * elw_colsum_rows_per_wave(rows, cols, streams);
    return std::max<int64_t>(1, (rows + per_block - 1) / per_block);
}

// Element-wise pass over a [rows, cols] space that also accumulates column sums.  A block is 16 wavefronts; each
// wavefront takes one row (lane = four adjacent columns, so a wavefront reads and writes 1 KiB runs) and the 16 row
// results are added through LDS in a fixed order, which leaves one partial row per block row for a second pass.
// There is no loop over rows in the common case: wavefronts are short-lived, the dispatcher hands out blocks in
// address order (the 16-row bands of one block row are contiguous in memory), and the chip as a whole streams through
// every operand front to back -- which is what keeps DRAM pages open for the four output streams.  A thread that
// walks down a column tile instead (fewer partial rows) was measured 20 % slower on the 3-read + 4-write pass of
// 8192 x 8192: long-lived loops drift apart and scatter the writes.
static GeneratedKernel gen_elw_colsum_kernel(const ElwKernelSpec& spec, const std::set<const Node*>& members) {
    const int64_t R = spec.rows, C = spec.cols, N = R * C;
    ADHIP_CHECK(C % 4 == 0 && R > 0, "internal: column-sum fusion needs cols %% 4 == 0");
    for (Node* o : spec.outputs) ADHIP_CHECK(numel(o->shape) == N, "internal: fused outputs differ in size");
    std::vector<Node*> all = spec.outputs;
    for (auto& cs : spec.colsums) all.push_back(cs.value);
    for (auto& rs : spec.rowsums) all.push_back(rs.value);
    const bool wide = needs_wide(all);
    const int64_t runs = elw_rowsum_runs(C);
    ElwBody b = elw_body(spec, members, Shape{R, C}, 4, wide);
    Gen& g = b.g;
    const int64_t K = elw_colsum_rows_per_wave(R, C, spec.streams);
    const int64_t tiles = elw_colsum_tiles(R, C, spec.streams);
    GeneratedKernel k;
    k.kind = "elw_colsum";
    k.entry = spec.name;
    std::string sig = "const int* __restrict__ guard";
    std::vector<Node*> order;
    // no __restrict__: an output may share its buffer with an input it replaces in place
    for (size_t i = 0; i < spec.outputs.size(); ++i) { sig += strf(", float* o%zu", i); order.push_back(spec.outputs[i]); }
    for (size_t i = 0; i < spec.colsums.size(); ++i) { sig += strf(", float* q%zu", i); order.push_back(spec.colsums[i].partial); }
    for (size_t i = 0; i < spec.rowsums.size(); ++i) { sig += strf(", float* r%zu", i); order.push_back(spec.rowsums[i].partial); }
    for (auto& gb : g.bufs) { sig += strf(", const float* %s", gb.param.c_str()); order.push_back(gb.node); }
    const char* it = g.idx_t();
    const char* sfx = wide ? "ull" : "u";
    const bool nt_out = N >= nontemporal_min_elems();
    std::string src = kernel_prelude();
    src += strf("extern \"C\" __global__ __launch_bounds__(1024) void %s(%s) {\n", k.entry.c_str(), sig.c_str());
    src += "    if (guard && *guard == 0) return;\n";
    if (!spec.colsums.empty()) src += "    __shared__ float4_t part[2][16][64];\n";
    src += "    const unsigned lane = threadIdx.x & 63u, wv = threadIdx.x >> 6;\n";
    src += strf("    const %s %s = (%s)blockIdx.x * 64u + lane;\n", it, (K >= 2 && K <= 4) ? "c1_raw" : "c1", it);
    src += strf("    const bool col_ok = %s < %lld%s;\n", (K >= 2 && K <= 4) ? "c1_raw" : "c1", (long long)(C / 4), sfx);
    for (size_t i = 0; i < spec.colsums.size(); ++i) src += strf("    float cs%zu[4] = {0.f, 0.f, 0.f, 0.f};\n", i);
    if (K >= 2 && K <= 4) {
        // A few rows per wavefront, in two phases: all rows' operands are loaded and everything is computed, then all
        // rows are stored.  A result may share its buffer with an operand, so the compiler cannot move a later
        // row's loads above an earlier row's stores by itself; and the rows are clamped to the last one rather than
        // skipped, because loads under a condition would not be issued together either.
        for (size_t i = 0; i < spec.outputs.size(); ++i) src += strf("    float keep%zu[%lld][4];\n", i, (long long)K);
        for (size_t i = 0; i < spec.rowsums.size(); ++i) src += strf("    float rsk%zu[%lld];\n", i, (long long)K);
        src += strf("    const %s c1 = col_ok ? c1_raw : %lld%s;\n", it, (long long)(C / 4 - 1), sfx);
        src += strf("#pragma unroll\n    for (unsigned kk = 0; kk < %lldu; ++kk) {\n", (long long)K);
        src += strf("        const %s row = (%s)blockIdx.y * %lld%s + kk * 16u + wv;\n", it, it, (long long)(16 * K), sfx);
        src += strf("        const bool live = col_ok && row < %lld%s;\n", (long long)R, sfx);
        src += strf("        const %s c0 = row < %lld%s ? row : %lld%s;\n", it, (long long)R, sfx, (long long)(R - 1), sfx);
        for (size_t i = 0; i < spec.rowsums.size(); ++i) src += strf("        float rs%zu = 0.f;\n", i);
        src += join(g.codeA, "        ");
        src += "#pragma unroll\n        for (int j = 0; j < 4; ++j) {\n";
        src += join(g.codeB, "            ");
        for (size_t i = 0; i < spec.outputs.size(); ++i) src += strf("            keep%zu[kk][j] = %s;\n", i, b.out_exprs[i].c_str());
        for (size_t i = 0; i < spec.colsums.size(); ++i) src += strf("            cs%zu[j] += live ? (%s) : 0.0f;\n", i, b.cs_exprs[i].c_str());
        for (size_t i = 0; i < spec.rowsums.size(); ++i) src += strf("            rs%zu += live ? (%s) : 0.0f;\n", i, b.rs_exprs[i].c_str());
        src += "        }\n";
        for (size_t i = 0; i < spec.rowsums.size(); ++i) src += strf("        rsk%zu[kk] = rs%zu;\n", i, i);
        src += "    }\n";
        src += strf("#pragma unroll\n    for (unsigned kk = 0; kk < %lldu; ++kk) {\n", (long long)K);
        src += strf("        const %s c0 = (%s)blockIdx.y * %lld%s + kk * 16u + wv;\n", it, it, (long long)(16 * K), sfx);
        src += strf("        if (col_ok && c0 < %lld%s) {\n", (long long)R, sfx);
        for (size_t i = 0; i < spec.outputs.size(); ++i)
            src += "            " + store4_stmt(strf("keep%zu[kk]", i), strf("o%zu + (c0 * %lld%s + c1 * 4u)", i, (long long)C, sfx), nt_out) + "\n";
        src += "        }\n";
        for (size_t i = 0; i < spec.rowsums.size(); ++i) {
            src += strf("        const float rs%zu = wave_sum(rsk%zu[kk]);\n", i, i);
            src += strf("        if (lane == 0u && c0 < %lld%s) r%zu[c0 * %lld%s + blockIdx.x] = rs%zu;\n", (long long)R, sfx, i, (long long)runs, sfx, i);
        }
        src += "    }\n";
    } else {
        if (K == 1) src += strf("    {\n        const %s c0 = (%s)blockIdx.y * 16u + wv;\n", it, it);
        else src += strf("%s\n    for (unsigned kk = 0; kk < %lldu; ++kk) {\n        const %s c0 = (%s)blockIdx.y * %lld%s + kk * 16u + wv;\n",
                         K <= 2 ? "#pragma unroll" : "#pragma unroll 1", (long long)K, it, it, (long long)(16 * K), sfx);
        for (size_t i = 0; i < spec.rowsums.size(); ++i) src += strf("        float rs%zu = 0.f;\n", i);
        src += strf("        if (col_ok && c0 < %lld%s) {\n", (long long)R, sfx);
        src += join(g.codeA, "            ");
        for (size_t i = 0; i < spec.outputs.size(); ++i) src += strf("            float w%zu[4];\n", i);
        src += "#pragma unroll\n            for (int j = 0; j < 4; ++j) {\n";
        src += join(g.codeB, "                ");
        for (size_t i = 0; i < spec.outputs.size(); ++i) src += strf("                w%zu[j] = %s;\n", i, b.out_exprs[i].c_str());
        for (size_t i = 0; i < spec.colsums.size(); ++i) src += strf("                cs%zu[j] += %s;\n", i, b.cs_exprs[i].c_str());
        for (size_t i = 0; i < spec.rowsums.size(); ++i) src += strf("                rs%zu += %s;\n", i, b.rs_exprs[i].c_str());
        src += "            }\n";
        for (size_t i = 0; i < spec.outputs.size(); ++i)
            src += "            " + store4_stmt(strf("w%zu", i), strf("o%zu + (c0 * %lld%s + c1 * 4u)", i, (long long)C, sfx), nt_out) + "\n";
        src += "        }\n";
        // a wavefront's run of a row: lanes outside the columns hold 0; one value per (row, run)
        for (size_t i = 0; i < spec.rowsums.size(); ++i) {
            src += strf("        rs%zu = wave_sum(rs%zu);\n", i, i);
            src += strf("        if (lane == 0u && c0 < %lld%s) r%zu[c0 * %lld%s + blockIdx.x] = rs%zu;\n", (long long)R, sfx, i, (long long)runs, sfx, i);
        }
        src += "    }\n";
    }
    // the 16 wavefronts' sums, added in wavefront order; two sums per round through LDS (wavefronts 0 and 1 add them)
    for (size_t i0 = 0; i0 < spec.colsums.size(); i0 += 2) {
        const size_t cnt = std::min<size_t>(2, spec.colsums.size() - i0);
        if (i0) src += "    __syncthreads();\n";
        for (size_t q = 0; q < cnt; ++q)
            src += strf("    part[%zu][wv][lane] = float4_t{cs%zu[0], cs%zu[1], cs%zu[2], cs%zu[3]};\n", q, i0 + q, i0 + q, i0 + q, i0 + q);
        src += "    __syncthreads();\n";
        src += strf("    if (wv < %zuu && col_ok) {\n        float4_t s = part[wv][0][lane];\n#pragma unroll\n        for (int r = 1; r < 16; ++r) s += part[wv][r][lane];\n", cnt);
        if (cnt == 2) src += strf("        float* q = wv ? q%zu : q%zu;\n", i0 + 1, i0);
        else src += strf("        float* q = q%zu;\n", i0);
        src += strf("        *(float4_t*)(q + ((%s)blockIdx.y * %lld%s + c1 * 4u)) = s;\n    }\n", it, (long long)C, sfx);
    }
    src += "}\n";
    k.source = src;
    k.buffer_args = order;
    k.block[0] = 1024;
    k.grid[0] = (unsigned)((C / 4 + 63) / 64);
    k.grid[1] = (unsigned)tiles;
    k.chunks = tiles;
    k.bytes = 4.0 * (double)N * (double)spec.outputs.size() + 4.0 * (double)tiles * C * spec.colsums.size() +
              4.0 * (double)R * (double)runs * spec.rowsums.size();
    for (auto& gb : g.bufs) k.bytes += 4.0 * (double)std::min<int64_t>(numel(gb.node->shape), N);
    k.flops = (g.flops + spec.colsums.size() + spec.rowsums.size()) * (double)N;
    return k;
}

// Element-wise kernel over 64x64 tiles of the two innermost iteration dims, for passes that read a large operand
// against the grain: consecutive *rows* of the result are adjacent in the operand's memory, consecutive columns are
// far apart (a permuted operand of a gather or an addition).  Read directly, every lane of a wavefront would touch its
// own cache line.  Here the block first fetches the operand's tile with the rows as the fast index (256-byte runs per
// wavefront), parks it in LDS, and every thread then takes its four values from there; everything else in the kernel,
// including the 128-bit accesses of all other operands and of the results, is the ordinary generated body.  The
// staging phase evaluates the very index expression the body would have used, at the coordinates of the element it
// fetches, so whatever view or concat piece the operand sits behind is handled by construction.
// Returns false (and leaves `k` alone) when the pass has no such operand or not the shape for it.
// Tile of the tiled element-wise kernel: 64 rows x 64 columns of the two innermost iteration extents.  The staged
// operand is read in runs of the tile's rows, the results are written in runs of its columns.  Measured on the gather
// stage of the manipulation workload (1 staged operand, 2 results, 453 MB): 64x64 77.3 us, 64x128 77.0, 128x64 77.9,
// 128x128 77.5, 64x256 80.3 -- the length of the runs is not what bounds it.  ADHIP_TILED_SHAPE=<rows>x<cols>
// (64 or 128 rows; 64, 128 or 256 columns) picks another tile, as a diagnostic.
static void tiled_shape(int64_t& TR, int64_t& TC) {
    TR = 64;
    TC = 64;
    if (const char* e = getenv("ADHIP_TILED_SHAPE")) {
        long r = 0, c = 0;
        if (sscanf(e, "%ldx%ld", &r, &c) == 2 && (r == 64 || r == 128) && (c == 64 || c == 128 || c == 256)) { TR = r; TC = c; }
    }
}

static bool gen_elw_tiled_kernel(const ElwKernelSpec& spec, const std::set<const Node*>& members, const Shape& shape, bool wide,
                                 GeneratedKernel& k) {
    const size_t nd = shape.size();
    if (nd < 2) return false;
    const int64_t I = shape[nd - 1], Rws = shape[nd - 2];
    if (I % 4 != 0 || I < 32 || Rws < 32) return false;   // tiles are at least 64x64: smaller extents leave most of a block idle
    int64_t TR = 64, TC = 64;
    tiled_shape(TR, TC);
    if ((TR * TC / 1024) * (int64_t)spec.outputs.size() > 32) { TR = 64; TC = 64; }   // a thread's share of the results stays in registers
    const int64_t N = numel(spec.outputs[0]->shape);
    std::set<std::string> keys;
    {
        ElwBody probe = elw_body(spec, members, shape, 4, wide);
        const int row_atom = probe.dim_atoms[nd - 2];
        for (const LoadRec& l : probe.g.loads) {
            if (numel(l.node->shape) < (int64_t(1) << 18)) continue;
            // unit stride along the rows (directly, or through a quotient / remainder of the row index), none along
            // the thread's own four columns
            bool unit_rows = false;
            for (auto& x : l.idx.t)
                if (x.second == 1 && !probe.g.atoms[(size_t)x.first].lane && probe.g.atom_depends_on(x.first, row_atom)) unit_rows = true;
            if (!unit_rows || !probe.g.aff_lane(l.idx) || probe.g.vectorizable(l.idx)) continue;
            keys.insert(l.key);
        }
    }
    if (keys.empty() || keys.size() > 2) return false;
    if (keys.size() * (size_t)(TC * (TR + 1) * 4) > 80 * 1024) { TR = 64; TC = 64; }   // two blocks' staging tiles fit a CU's 160 KB
    const std::string sfx = wide ? "ull" : "u";
    ElwBody b = elw_body(spec, members, shape, 4, wide, [&](Gen& g) {
        g.stage_keys = keys;
        g.row_atom = (int)nd - 2;
        g.tile_row_origin = "row0";
        g.tile_col_origin = "col0";
        g.tile_rows = (int)TR;
        g.tile_cols = (int)TC;
    });
    Gen& g = b.g;
    if (g.staged.empty()) return false;
    const char* it = g.idx_t();
    k = GeneratedKernel();
    k.kind = "elw_tiled";
    k.entry = spec.name;
    std::string sig = "const int* __restrict__ guard";
    std::vector<Node*> order;
    for (size_t i = 0; i < spec.outputs.size(); ++i) { sig += strf(", float* o%zu", i); order.push_back(spec.outputs[i]); }
    for (auto& gb : g.bufs) { sig += ", const float* " + gb.param; order.push_back(gb.node); }
    const int64_t TI = (I + TC - 1) / TC, TJ = (Rws + TR - 1) / TR;
    const int64_t NS = TR * TC / 256;          // staging loads per thread
    const int64_t QC = TC / 4;                 // float4 columns of a tile
    const int64_t RP = 256 / QC;               // rows of a tile that one pass of the block covers
    const int64_t NP = TR / RP;                // passes
    int64_t outer = 1;
    for (size_t d = 0; d + 2 < nd; ++d) outer *= shape[d];
    const int64_t blocks = TI * TJ * outer;
    if (blocks > 0x7fffffff) return false;
    const std::string rowv = "c" + std::to_string(nd - 2), colv = "c" + std::to_string(nd - 1);
    std::string src = kernel_prelude();
    src += strf("extern \"C\" __global__ __launch_bounds__(256) void %s(%s) {\n", k.entry.c_str(), sig.c_str());
    src += "    if (guard && *guard == 0) return;\n";
    for (auto& st : g.staged) src += strf("    __shared__ float tile%d[%lld][%lld];\n", st.slot, (long long)TC, (long long)(TR + 1));
    src += "    const unsigned tid = threadIdx.x;\n";
    src += strf("    %s bid = blockIdx.x;\n", it);
    src += strf("    const %s col0 = (bid %% %lld%s) * %lldu;\n    bid /= %lld%s;\n", it, (long long)TI, sfx.c_str(), (long long)TC, (long long)TI, sfx.c_str());
    src += strf("    const %s row0 = (bid %% %lld%s) * %lldu;\n    bid /= %lld%s;\n", it, (long long)TJ, sfx.c_str(), (long long)TR, (long long)TJ, sfx.c_str());
    for (size_t d = nd - 2; d-- > 0;) {
        if (d == 0) src += strf("    const %s c0 = bid;\n", it);
        else src += strf("    const %s c%zu = bid %% %lld%s;\n    bid /= %lld%s;\n", it, d, (long long)shape[d], sfx.c_str(), (long long)shape[d], sfx.c_str());
    }
    // staging: lane = row within the tile, so that a wavefront reads one 256-byte run of the operand per column
    // All 16 loads of a thread are issued before the first value is parked: the loads are unconditional (an element
    // outside the tensor or the operand's piece reads index 0 and is replaced by 0 afterwards), because a load under
    // a condition becomes a branch with a wait behind it, and the 16 memory latencies of a block then add up (that
    // version ran at 0.60 of the HBM peak with every wavefront waiting 88 % of its life).
    for (auto& st : g.staged) src += strf("    float sv%d[%lld];\n", st.slot, (long long)NS);
    src += strf("#pragma unroll\n    for (unsigned k = 0; k < %lldu; ++k) {\n", (long long)NS);
    src += strf("        const unsigned lj = tid %% %lldu, li = tid / %lldu + %lldu * k;\n", (long long)TR, (long long)TR, (long long)(256 / TR));
    src += strf("        const %s %s = row0 + lj;\n        const %s ii = col0 + li;\n", it, rowv.c_str(), it);
    src += strf("        const %s %s = ii >> 2;\n        const %s j = ii & 3u;\n", it, colv.c_str(), it);
    src += strf("        const bool inside = %s < %lld%s && ii < %lld%s;\n", rowv.c_str(), (long long)Rws, sfx.c_str(), (long long)I, sfx.c_str());
    src += join(g.index_code, "        ");
    for (auto& st : g.staged) {
        src += strf("        { const bool ok = inside%s%s; const float v = %s[ok ? (%s) : 0]; sv%d[k] = ok ? v : 0.0f; }\n",
                    st.pred.empty() ? "" : " && ", st.pred.c_str(), st.param.c_str(), st.index.c_str(), st.slot);
    }
    src += "    }\n";
    src += strf("#pragma unroll\n    for (unsigned k = 0; k < %lldu; ++k) {\n", (long long)NS);
    for (auto& st : g.staged) src += strf("        tile%d[tid / %lldu + %lldu * k][tid %% %lldu] = sv%d[k];\n", st.slot, (long long)TR, (long long)(256 / TR), (long long)TR, st.slot);
    src += "    }\n    __syncthreads();\n";
    // compute: a thread owns four adjacent columns of four rows of the tile
    src += strf("    const unsigned lc = tid %% %lldu, lr = tid / %lldu;\n", (long long)QC, (long long)QC);
    // the four rows' values are computed first and stored afterwards: a result may share its buffer with an operand,
    // so the compiler cannot move the next row's loads above this row's stores by itself, and the rows' memory
    // latencies would add up
    for (size_t i = 0; i < spec.outputs.size(); ++i) src += strf("    float keep%zu[%lld][4];\n", i, (long long)NP);
    src += strf("    %s at[%lld];\n    bool live[%lld];\n", it, (long long)NP, (long long)NP);
    src += strf("#pragma unroll\n    for (unsigned k = 0; k < %lldu; ++k) {\n", (long long)NP);
    // (a row or column quad beyond the edge works on the last valid one instead and is not stored: no branch)
    src += strf("        const %s row_k = row0 + lr + %lldu * k, quad_k = (col0 >> 2) + lc;\n", it, (long long)RP);
    src += strf("        live[k] = row_k < %lld%s && quad_k < %lld%s;\n", (long long)Rws, sfx.c_str(), (long long)(I / 4), sfx.c_str());
    src += strf("        const %s %s = row_k < %lld%s ? row_k : %lld%s;\n        const %s %s = quad_k < %lld%s ? quad_k : %lld%s;\n", it, rowv.c_str(),
                (long long)Rws, sfx.c_str(), (long long)(Rws - 1), sfx.c_str(), it, colv.c_str(), (long long)(I / 4), sfx.c_str(), (long long)(I / 4 - 1), sfx.c_str());
    src += join(g.codeA, "        ");
    for (size_t i = 0; i < spec.outputs.size(); ++i) src += strf("        float w%zu[4];\n", i);
    src += "#pragma unroll\n        for (int j = 0; j < 4; ++j) {\n";
    src += join(g.codeB, "            ");
    for (size_t i = 0; i < spec.outputs.size(); ++i) src += strf("            w%zu[j] = %s;\n", i, b.out_exprs[i].c_str());
    src += "        }\n";
    // linear float4 index of the thread's element: row-major over the iteration shape
    std::string lin = "c0";
    for (size_t d = 1; d < nd; ++d)
        lin = strf("(%s * %lld%s + c%zu)", lin.c_str(), (long long)(d + 1 == nd ? I / 4 : shape[d]), sfx.c_str(), d);
    src += strf("        at[k] = %s;\n", lin.c_str());
    for (size_t i = 0; i < spec.outputs.size(); ++i)
        src += strf("#pragma unroll\n        for (int j = 0; j < 4; ++j) keep%zu[k][j] = w%zu[j];\n", i, i);
    src += "    }\n";
    src += strf("#pragma unroll\n    for (unsigned k = 0; k < %lldu; ++k) {\n        if (!live[k]) continue;\n", (long long)NP);
    for (size_t i = 0; i < spec.outputs.size(); ++i)
        src += "        " + store4_stmt(strf("keep%zu[k]", i), strf("o%zu + at[k] * 4u", i), N >= nontemporal_min_elems()) + "\n";
    src += "    }\n}\n";
    k.source = src;
    k.buffer_args = order;
    k.block[0] = 256;
    k.grid[0] = (unsigned)blocks;
    k.bytes = 4.0 * (double)N * (double)spec.outputs.size();
    for (auto& gb : g.bufs) k.bytes += 4.0 * (double)std::min<int64_t>(numel(gb.node->shape), N);
    k.flops = g.flops * (double)N;
    return true;
}

GeneratedKernel gen_elw_kernel(const ElwKernelSpec& spec, const std::set<const Node*>& members) {
    if (!spec.colsums.empty() || !spec.rowsums.empty()) return gen_elw_colsum_kernel(spec, members);
    ADHIP_CHECK(!spec.outputs.empty(), "internal: element-wise kernel without outputs");
    const int64_t N = numel(spec.outputs[0]->shape);
    for (Node* o : spec.outputs) ADHIP_CHECK(numel(o->shape) == N, "internal: fused outputs differ in size");
    ADHIP_CHECK(N > 0, "internal: empty element-wise kernel");
    const bool wide = needs_wide(spec.outputs);

    // pass 1: natural shape, scalar lanes, to learn which dims can be merged
    Shape shape = drop_ones(spec.outputs[0]->shape);
    {
        ElwBody dry = elw_body(spec, members, shape, 1, wide);
        // atom definitions are recorded through aff_str as well
        shape = merge_dims(shape, dry.g.recorded, dry.dim_atoms);
    }
    int vec = (shape.back() % 4 == 0 && N >= 1024) ? 4 : 1;
    if (vec == 4) {
        GeneratedKernel tiled;
        if (gen_elw_tiled_kernel(spec, members, shape, wide, tiled)) return tiled;
    }
    ElwBody b = elw_body(spec, members, shape, vec, wide);
    Gen& g = b.g;

    GeneratedKernel k;
    k.kind = "elw";
    k.entry = spec.name;
    const int64_t threads = N / vec;
    std::string sig = "const int* __restrict__ guard";
    std::vector<Node*> order;
    // outputs first, then inputs
    std::vector<std::string> out_params;
    for (size_t i = 0; i < spec.outputs.size(); ++i) {
        out_params.push_back("o" + std::to_string(i));
        sig += ", float* o" + std::to_string(i);
        order.push_back(spec.outputs[i]);
    }
    for (auto& gb : g.bufs) {
        // a buffer that is also written in this kernel (in-place update) must not be restrict-qualified
        sig += ", const float* " + gb.param;
        order.push_back(gb.node);
    }
    int latch_output = -1;
    if (spec.latch && vec == 1 && N == 1)
        for (size_t i = 0; i < spec.outputs.size(); ++i)
            if (spec.outputs[i] == spec.latch) latch_output = (int)i;
    if (latch_output >= 0) {
        // the flag the kernel latches is the one that guards it: the two parameters name the same word
        sig.replace(sig.find("const int* __restrict__ guard"), strlen("const int* __restrict__ guard"), "const int* guard");
        sig += ", int* latch";
        k.latch_done = true;
    }
    std::string src = kernel_prelude();
    // Large kernels do not walk through memory block after block.  A block is 16 wavefronts; wavefront w takes a 1 KiB
    // run (64 float4) in band row w, where a band is 16 rows of `band` bytes, and consecutive blocks take consecutive
    // runs of the same 16 rows.  With rows of 32 KiB the 3-read + 4-write stream mix over 8192 x 8192 floats runs at
    // 0.80 of the HBM peak instead of 0.70 (plain copy 7.0 instead of 6.76 TB/s); 16 and 64 KiB rows give 0.79 and 0.77.
    // It is the access pattern the column-sum kernel has by construction on rows of 8192 floats.
    const int64_t run4 = elw_band_bytes() / 16;
    const bool banded = run4 >= 64 && vec == 4 && threads >= (int64_t(1) << 20);
    const int64_t bands = banded ? (threads + 16 * run4 - 1) / (16 * run4) : 0;
    if (banded) {
        src += strf("extern \"C\" __global__ __launch_bounds__(1024) void %s(%s) {\n", k.entry.c_str(), sig.c_str());
        src += "    if (guard && *guard == 0) return;\n";
        src += strf("    const %s band = (%s)blockIdx.x / %lldu, run = (%s)blockIdx.x %% %lldu;\n", g.idx_t(), g.idx_t(), (long long)(run4 / 64),
                    g.idx_t(), (long long)(run4 / 64));
        src += strf("    const %s t = (band * 16u + (threadIdx.x >> 6)) * %lldu + run * 64u + (threadIdx.x & 63u);\n", g.idx_t(), (long long)run4);
    } else {
        src += strf("extern \"C\" __global__ __launch_bounds__(256) void %s(%s) {\n", k.entry.c_str(), sig.c_str());
        src += "    if (guard && *guard == 0) return;\n";
        src += strf("    const %s t = (%s)blockIdx.x * 256u + threadIdx.x;\n", g.idx_t(), g.idx_t());
    }
    src += strf("    if (t >= %lld%s) return;\n", (long long)threads, wide ? "ull" : "u");
    // decompose t into iteration atoms
    {
        std::string rem = "t";
        for (size_t i = shape.size(); i-- > 0;) {
            int64_t range = (i + 1 == shape.size()) ? shape[i] / vec : shape[i];
            if (i == 0) src += strf("    const %s c0 = %s;\n", g.idx_t(), rem.c_str());
            else {
                src += strf("    const %s c%zu = %s %% %lld%s;\n", g.idx_t(), i, rem.c_str(), (long long)range, wide ? "ull" : "u");
                src += strf("    const %s r%zu = %s / %lld%s;\n", g.idx_t(), i, rem.c_str(), (long long)range, wide ? "ull" : "u");
                rem = "r" + std::to_string(i);
            }
        }
    }
    src += join(g.codeA, "    ");
    for (size_t i = 0; i < spec.outputs.size(); ++i) src += strf("    float w%zu[%d];\n", i, vec);
    if (vec > 1) src += strf("#pragma unroll\n    for (int j = 0; j < %d; ++j) {\n", vec);
    else src += "    {\n";
    src += join(g.codeB, "        ");
    for (size_t i = 0; i < spec.outputs.size(); ++i)
        src += strf("        w%zu[%s] = %s;\n", i, vec > 1 ? "j" : "0", b.out_exprs[i].c_str());
    src += "    }\n";
    for (size_t i = 0; i < spec.outputs.size(); ++i) {
        if (vec == 4) src += "    " + store4_stmt(strf("w%zu", i), strf("o%zu + t * 4u", i), N >= nontemporal_min_elems()) + "\n";
        else src += strf("    o%zu[t] = w%zu[0];\n", i, i);
    }
    if (latch_output >= 0) src += strf("    latch[0] = w%d[0] != 0.0f ? 1 : 0;\n", latch_output);
    src += "}\n";
    k.source = src;
    k.buffer_args = order;
    k.block[0] = 256;
    k.grid[0] = (unsigned)((threads + 255) / 256);
    if (banded) {
        k.block[0] = 1024;
        k.grid[0] = (unsigned)(bands * (run4 / 64));
    }
    k.bytes = 4.0 * (double)N * (double)spec.outputs.size();
    for (auto& gb : g.bufs) k.bytes += 4.0 * (double)std::min<int64_t>(numel(gb.node->shape), N);
    k.flops = g.flops * (double)N;
    return k;
}

DotEpilogueCode gen_dot_epilogue(const Node* dot, const std::vector<Node*>& outputs) {
    ADHIP_CHECK(dot->op == Op::DOT && dot->shape.size() == 2, "internal: malformed product for an epilogue");
    const int64_t M = dot->shape[0], N = dot->shape[1];
    Gen g;
    g.vec = 1;
    std::vector<Node*> all(outputs.begin(), outputs.end());
    g.wide = needs_wide(all) || M * N >= (int64_t(1) << 31) - 1024;
    const int ar = g.add_atom("er", M, false), ac = g.add_atom("ec", N, false);
    const Aff lin = aff_add(aff_atom(ar, N), aff_atom(ac, 1));
    g.preset[dot] = "sum_value";
    for (Node* o : outputs) {
        ADHIP_CHECK(numel(o->shape) == M * N && op_is_elw(o->op), "internal: product epilogue output of the wrong kind");
        g.members.insert(o);
    }
    std::vector<std::string> exprs;
    for (Node* o : outputs) exprs.push_back(g.gen_node(o, lin, "").expr);
    ADHIP_CHECK(g.codeB.empty(), "internal: product epilogue produced per-lane code");
    DotEpilogueCode e;
    e.code = strf("const %s er = (%s)row, ec = (%s)col;\n", g.idx_t(), g.idx_t(), g.idx_t());
    e.code += join(g.codeA, "");
    for (size_t i = 0; i < outputs.size(); ++i) {
        e.code += strf("e%zu[er * %lld%s + ec] = %s;\n", i, (long long)N, g.wide ? "ull" : "u", exprs[i].c_str());
        e.params += strf(", float* e%zu", i);
        e.buffer_args.push_back(outputs[i]);
    }
    for (auto& gb : g.bufs) {
        e.params += ", const float* " + gb.param;
        e.buffer_args.push_back(gb.node);
    }
    e.flops = g.flops;
    return e;
}

// ---------------------------------------------------------------------------------------
// reductions
// ---------------------------------------------------------------------------------------

namespace {

enum class RedLayout { ROW, COL };

struct RedBody {
    Gen g;
    std::vector<std::string> side_exprs;
    std::string value;  // per-lane value expression
    bool value_lane = false;
};

// atoms: ROW: x, yv (+ lane j along y); COL: xv, y (+ lane j along x)
RedBody red_body(const Node* n, RedLayout layout, int vec, bool wide, const std::vector<Node*>& side = {}) {
    RedBody b;
    Gen& g = b.g;
    g.vec = vec;
    g.wide = wide;
    for (Node* s : side) g.members.insert(s);
    const TRef& t = n->in[0];
    const int64_t V = t.shape[0], R = t.shape[1];
    Aff lin;
    if (layout == RedLayout::ROW) {
        int ax = g.add_atom("x", V, false);
        int ay = g.add_atom("yv", R / vec, false);
        lin = aff_add(aff_atom(ax, R), aff_atom(ay, vec));
    } else {
        int ax = g.add_atom("xv", V / vec, false);
        int ay = g.add_atom("y", R, false);
        lin = aff_add(aff_atom(ax, R * vec), aff_atom(ay, 1));
    }
    if (vec > 1) {
        g.lane_atom = g.add_atom("j", vec, true);
        lin = aff_add(lin, aff_atom(g.lane_atom, layout == RedLayout::ROW ? 1 : R));
    }
    Val v = g.gen_tref(t, lin, "");
    b.value = v.expr;
    b.value_lane = v.lane;
    for (Node* s : side) b.side_exprs.push_back(g.gen_node(s, lin, "").expr);
    return b;
}

}  // namespace

GeneratedKernel gen_reduce_kernel(const ReduceKernelSpec& spec, int64_t force_chunks) {
    const Node* n = spec.node;
    ADHIP_CHECK(op_is_reduce(n->op) && n->in.size() == 1 && n->in[0].shape.size() == 2, "internal: malformed reduction");
    // Sum and Max share everything but the combining step: `acc (+)= v`, the identity lanes start from, and how two
    // partial results are merged.  fmaxf returns the other operand when one is NaN, so NaN is the identity of the
    // maximum: a row's maximum is NaN exactly when all of it is (a row of -inf gives -inf), and lanes that hold no
    // element of the row drop out of every combination.
    const bool mx = n->op == Op::MAX;
    const char* ident = mx ? "__builtin_nanf(\"\")" : "0.0f";
    auto comb = [&](const std::string& a, const std::string& b) { return mx ? "fmaxf(" + a + ", " + b + ")" : a + " + " + b; };
    auto comb4 = [&](const std::string& a, const std::string& b, const std::string& c, const std::string& d) {
        return mx ? "fmaxf(fmaxf(" + a + ", " + b + "), fmaxf(" + c + ", " + d + "))" : "(" + a + " + " + b + ") + (" + c + " + " + d + ")";
    };
    const char* wave_comb = mx ? "wave_max" : "wave_sum";
    const int64_t V = n->in[0].shape[0], R = n->in[0].shape[1];
    ADHIP_CHECK(V > 0 && R > 0, "internal: empty reduction");
    std::vector<Node*> roots{const_cast<Node*>(n)};
    const bool wide = needs_wide(roots);

    // Decide the thread layout from how the largest operand is addressed.
    RedLayout layout = RedLayout::ROW;
    {
        RedBody dry = red_body(n, RedLayout::ROW, 1, wide);
        int64_t best = -1;
        int64_t cx = 0, cy = 0;
        for (auto& l : dry.g.loads) {
            int64_t ne = numel(l.node->shape);
            if (ne <= best) continue;
            best = ne;
            cx = cy = 0;
            for (auto& x : l.idx.t) {
                if (x.first == 0) cx = x.second;
                if (x.first == 1) cy = x.second;
            }
        }
        if (cy != 1 && cx == 1 && V >= 64) layout = RedLayout::COL;
    }
    GeneratedKernel k;
    k.entry = spec.name;
    int vec;
    std::string src = kernel_prelude();
    if (layout == RedLayout::ROW) {
        vec = (R % 4 == 0 && R >= 256) ? 4 : 1;
        const bool side = !spec.side_outputs.empty() && vec == 4;
        RedBody b = red_body(n, layout, vec, wide, side ? spec.side_outputs : std::vector<Node*>());
        Gen& g = b.g;
        k.side_done = side;
        const int64_t RV = R / vec;
        // threads per row: one wavefront per row (no barrier, no LDS) up to 2048 elements, a whole block beyond that
        // (16384 x 4096: 41 us with a wavefront per row, 38 us with a block per row)
        int T = RV <= 512 ? 64 : 256;
        if (V < 64 && RV >= 4096) T = 256;
        const int rows_per_block = 256 / T;
        // split long rows over several blocks when there are too few rows to fill the GPU
        int64_t chunks = 1;
        if (force_chunks > 0) chunks = force_chunks;
        else if (V * T < 131072 && RV >= (int64_t)T * 128) {
            chunks = std::min<int64_t>((131072 + V * T - 1) / (V * T), RV / ((int64_t)T * 8));
            chunks = std::max<int64_t>(chunks, 1);
        }
        const int64_t CH = (RV + chunks - 1) / chunks;  // vector elements per chunk
        k.kind = side ? "reduce_row_store" : "reduce_row";
        // Epilogue: element-wise consumers of the finished sums, evaluated at index x by the lane that stores the sum.
        // Generated with the same buffer table; its statements are taken out of the loop body's lists, and nothing
        // memoised inside the loop is visible to it.
        std::vector<std::string> epi_code, epi_exprs;
        const bool epi = !spec.epilogue_outputs.empty() && chunks == 1;
        if (epi) {
            auto memo = g.val_memo;
            g.val_memo.clear();
            auto atom_memo = g.atom_memo;  // index pieces split off x inside the loop are declared in the loop's scope
            g.atom_memo.clear();
            const int vec_saved = g.vec, lane_saved = g.lane_atom;
            g.vec = 1;
            g.lane_atom = -1;
            const size_t a0 = g.codeA.size(), b0 = g.codeB.size();
            const double flops_saved = g.flops;
            g.preset[n] = "sum_value";
            for (Node* e : spec.epilogue_outputs) g.members.insert(e);
            const Aff at_x = aff_atom(0, 1);  // atom 0 is x
            for (Node* e : spec.epilogue_outputs) epi_exprs.push_back(g.gen_node(e, at_x, "").expr);
            ADHIP_CHECK(g.codeB.size() == b0, "internal: reduction epilogue produced per-lane code");
            epi_code.assign(g.codeA.begin() + (long)a0, g.codeA.end());
            g.codeA.resize(a0);
            g.flops = flops_saved;
            g.vec = vec_saved;
            g.lane_atom = lane_saved;
            g.val_memo = memo;
            g.atom_memo = atom_memo;
            k.epilogue_done = true;
        }
        // no __restrict__: the result (and a stored operand) may share a buffer with an input it replaces in place
        std::string sig = "const int* __restrict__ guard, float* out";
        std::vector<Node*> order{const_cast<Node*>(n)};
        if (side)
            for (size_t i = 0; i < spec.side_outputs.size(); ++i) { sig += strf(", float* w%zu", i); order.push_back(spec.side_outputs[i]); }
        if (epi)
            for (size_t i = 0; i < spec.epilogue_outputs.size(); ++i) { sig += strf(", float* e%zu", i); order.push_back(spec.epilogue_outputs[i]); }
        for (auto& gb : g.bufs) { sig += std::string(", const float* ") + gb.param; order.push_back(gb.node); }
        int latch_epi = -1;
        if (epi && spec.latch && V == 1)
            for (size_t i = 0; i < spec.epilogue_outputs.size(); ++i)
                if (spec.epilogue_outputs[i] == spec.latch) latch_epi = (int)i;
        if (latch_epi >= 0) {
            sig.replace(sig.find("const int* __restrict__ guard"), strlen("const int* __restrict__ guard"), "const int* guard");
            sig += ", int* latch";
            k.latch_done = true;
        }
        src += strf("extern \"C\" __global__ __launch_bounds__(256) void %s(%s) {\n", k.entry.c_str(), sig.c_str());
        src += "    if (guard && *guard == 0) return;\n";
        src += strf("    const unsigned lane = threadIdx.x %% %du;\n", T);
        src += strf("    const %s x = (%s)blockIdx.x * %du + threadIdx.x / %du;\n", g.idx_t(), g.idx_t(), rows_per_block, T);
        src += "    const unsigned chunk = blockIdx.y;\n";
        src += strf("    const bool row_ok = x < %lld%s;\n", (long long)V, wide ? "ull" : "u");
        src += strf("    float acc[%d];\n#pragma unroll\n    for (int j = 0; j < %d; ++j) acc[j] = %s;\n", vec, vec, ident);
        // A row that is also stored, in a few iterations per lane: every iteration's loads are issued and the values
        // computed before the first one is stored.  A stored value may share its buffer with an operand, so the
        // compiler has to keep each iteration's loads behind the previous iteration's store, and the iterations'
        // memory latencies would add up (the body of the data-dependent loop of the manipulation workload is such a
        // kernel: three iterations).  Iterations past the end of the row are clamped to its last element, not skipped.
        const int64_t iters = (RV + T - 1) / T;
        const bool phased = side && chunks == 1 && vec == 4 && iters * (int64_t)b.side_exprs.size() <= 8;
        if (phased) {
            const char* it_t = g.idx_t();
            for (size_t i = 0; i < b.side_exprs.size(); ++i) src += strf("    float keep%zu[%lld][4];\n", i, (long long)iters);
            src += "    if (row_ok) {\n";
            src += strf("#pragma unroll\n    for (unsigned it = 0; it < %lldu; ++it) {\n", (long long)iters);
            src += strf("        const %s yv_raw = lane + it * %du;\n        const bool live = yv_raw < %lldu;\n        const %s yv = live ? yv_raw : %lldu;\n",
                        it_t, T, (long long)RV, it_t, (long long)(RV - 1));
            src += join(g.codeA, "        ");
            src += "#pragma unroll\n        for (int j = 0; j < 4; ++j) {\n";
            src += join(g.codeB, "            ");
            for (size_t i = 0; i < b.side_exprs.size(); ++i) src += strf("            keep%zu[it][j] = %s;\n", i, b.side_exprs[i].c_str());
            src += strf("            if (live) acc[j] = %s;\n        }\n    }\n", comb("acc[j]", b.value).c_str());
            src += strf("#pragma unroll\n    for (unsigned it = 0; it < %lldu; ++it) {\n        const %s yv = lane + it * %du;\n        if (yv < %lldu) {\n",
                        (long long)iters, it_t, T, (long long)RV);
            for (size_t i = 0; i < b.side_exprs.size(); ++i)
                src += "            " + store4_stmt(strf("keep%zu[it]", i), strf("w%zu + (%lldu * x + 4u * yv)", i, (long long)R), V * R >= nontemporal_min_elems()) + "\n";
            src += "        }\n    }\n    }\n";
        }
        if (phased) {
        } else if (chunks == 1) {
            // constant trip count: the loads of several iterations can be in flight together
            src += strf("    if (row_ok)\n#pragma unroll 8\n    for (%s yv = lane; yv < %lldu; yv += %du) {\n", g.idx_t(), (long long)RV, T);
        } else {
            src += strf("    const %s y_end = min((%s)(chunk + 1u) * %lldu, (%s)%lldu);\n", g.idx_t(), g.idx_t(), (long long)CH, g.idx_t(), (long long)RV);
            src += strf("    if (row_ok)\n#pragma unroll 4\n    for (%s yv = (%s)chunk * %lldu + lane; yv < y_end; yv += %du) {\n", g.idx_t(), g.idx_t(), (long long)CH, T);
        }
        if (!phased) {
        src += join(g.codeA, "        ");
        if (side)
            for (size_t i = 0; i < b.side_exprs.size(); ++i) src += strf("        float sv%zu[4];\n", i);
        if (vec > 1) src += strf("#pragma unroll\n        for (int j = 0; j < %d; ++j) {\n", vec);
        else src += "        { const int j = 0;\n";
        src += join(g.codeB, "            ");
        if (side)
            for (size_t i = 0; i < b.side_exprs.size(); ++i) src += strf("            sv%zu[j] = %s;\n", i, b.side_exprs[i].c_str());
        src += strf("            acc[j] = %s;\n        }\n", comb("acc[j]", b.value).c_str());
        if (side)
            for (size_t i = 0; i < b.side_exprs.size(); ++i)
                src += "        " + store4_stmt(strf("sv%zu", i), strf("w%zu + (%lldu * x + 4u * yv)", i, (long long)R), V * R >= nontemporal_min_elems()) + "\n";
        src += "    }\n";
        }
        if (vec == 4) src += "    float s = " + comb4("acc[0]", "acc[1]", "acc[2]", "acc[3]") + ";\n";
        else src += "    float s = acc[0];\n";
        std::string epilogue;
        if (epi) {
            epilogue = join(epi_code, "        ");
            for (size_t i = 0; i < epi_exprs.size(); ++i) epilogue += strf("        e%zu[x] = %s;\n", i, epi_exprs[i].c_str());
            if (latch_epi >= 0) epilogue += strf("        latch[0] = (%s) != 0.0f ? 1 : 0;\n", epi_exprs[(size_t)latch_epi].c_str());
        }
        if (T == 64) {
            src += strf("    s = %s(s);\n", wave_comb);
            src += "    if (lane == 0 && row_ok) {\n        const float sum_value = s;\n";
            src += strf("        out[(%s)chunk * %lldu + x] = sum_value;\n", g.idx_t(), (long long)V);
            src += epilogue + "    }\n";
        } else {
            src += strf("    __shared__ float part[4];\n    s = %s(s);\n", wave_comb);
            src += "    if ((threadIdx.x & 63u) == 0) part[threadIdx.x >> 6] = s;\n    __syncthreads();\n";
            src += "    if (threadIdx.x == 0 && row_ok) {\n        const float sum_value = " + comb4("part[0]", "part[1]", "part[2]", "part[3]") + ";\n";
            src += strf("        out[(%s)chunk * %lldu + x] = sum_value;\n", g.idx_t(), (long long)V);
            src += epilogue + "    }\n";
        }
        src += "}\n";
        k.buffer_args = order;
        k.block[0] = 256;
        k.grid[0] = (unsigned)((V + rows_per_block - 1) / rows_per_block);
        k.grid[1] = (unsigned)chunks;
        k.chunks = chunks;
        k.bytes = 4.0 * (double)V * (double)chunks;
        if (side) k.bytes += 4.0 * (double)V * (double)R * (double)spec.side_outputs.size();
        for (auto& gb : g.bufs) k.bytes += 4.0 * (double)std::min<int64_t>(numel(gb.node->shape), V * R);
        k.flops = (g.flops + 1) * (double)V * (double)R;
    } else {
        // one column per thread when the problem is small (more blocks beat wider loads there)
        vec = (V % 4 == 0 && V >= 1024 && V * R >= (int64_t(1) << 22)) ? 4 : 1;
        RedBody b = red_body(n, layout, vec, wide);
        Gen& g = b.g;
        const int64_t XV = V / vec;
        const int64_t bx = (XV + 63) / 64;
        // Large inputs: blocks of 16 wavefronts that live for one or two rows each, as in the element-wise pass with
        // column sums riding along (gen_elw_colsum_kernel) -- wavefront w adds up row 16 k + w of the block's rows over
        // 256 columns (four per lane), the 16 wavefronts' sums are added through LDS in a fixed order, and one partial
        // row per block goes to the second pass.  The chip then streams through the operand front to back; threads
        // that walk down 32 rows each in a loop reached 0.62 of the HBM peak on 16384 x 4096, this form 0.84.
        // A reduction on its own stores nothing per element, so more rows per wavefront -- four while that leaves four
        // blocks for every CU -- mean more loads in flight and fewer partial rows for the second pass (x.sum(0) over
        // 16384 x 4096: one row 55.2 us, two 43.7, four 40.0, eight 40.6, sixteen 42.9).
        int64_t KW = elw_colsum_rows_per_wave(R, V, 1);
        while (KW < 4 && bx * ((R + 32 * KW - 1) / (32 * KW)) >= 1024) KW *= 2;
        const int64_t tiles = (R + 16 * KW - 1) / (16 * KW);
        if (force_chunks == 0 && vec == 4 && KW <= 4 && tiles >= 2 && bx * tiles >= 512) {
            k.kind = "reduce_col";
            std::string sig = "const int* __restrict__ guard, float* out";
            std::vector<Node*> order{const_cast<Node*>(n)};
            for (auto& gb : g.bufs) { sig += ", const float* " + gb.param; order.push_back(gb.node); }
            const char* it = g.idx_t();
            const char* sfx = wide ? "ull" : "u";
            src += strf("extern \"C\" __global__ __launch_bounds__(1024) void %s(%s) {\n", k.entry.c_str(), sig.c_str());
            src += "    if (guard && *guard == 0) return;\n";
            src += "    __shared__ float4_t part[16][64];\n";
            src += "    const unsigned lane = threadIdx.x & 63u, wv = threadIdx.x >> 6;\n";
            src += strf("    const %s xv_raw = (%s)blockIdx.x * 64u + lane;\n", it, it);
            src += strf("    const bool col_ok = xv_raw < %lld%s;\n    const %s xv = col_ok ? xv_raw : %lld%s;\n", (long long)XV, sfx, it, (long long)(XV - 1), sfx);
            src += strf("    float acc[4] = {%s, %s, %s, %s};\n", ident, ident, ident, ident);
            // rows beyond the last one are clamped to it and left out of the sum: every load is unconditional, so a
            // wavefront's loads are all in flight together
            src += strf("#pragma unroll\n    for (unsigned kk = 0; kk < %lldu; ++kk) {\n", (long long)KW);
            src += strf("        const %s y_raw = (%s)blockIdx.y * %lld%s + kk * 16u + wv;\n", it, it, (long long)(16 * KW), sfx);
            src += strf("        const bool live = col_ok && y_raw < %lld%s;\n        const %s y = y_raw < %lld%s ? y_raw : %lld%s;\n", (long long)R, sfx, it,
                        (long long)R, sfx, (long long)(R - 1), sfx);
            src += join(g.codeA, "        ");
            src += "#pragma unroll\n        for (int j = 0; j < 4; ++j) {\n";
            src += join(g.codeB, "            ");
            src += strf("            if (live) acc[j] = %s;\n        }\n    }\n", comb("acc[j]", b.value).c_str());
            src += "    part[wv][lane] = float4_t{acc[0], acc[1], acc[2], acc[3]};\n    __syncthreads();\n";
            src += "    if (wv == 0u && col_ok) {\n        float4_t s = part[0][lane];\n#pragma unroll\n        for (int r = 1; r < 16; ++r) {\n            const float4_t q = part[r][lane];\n";
            src += "#pragma unroll\n            for (int j = 0; j < 4; ++j) s[j] = " + comb("s[j]", "q[j]") + ";\n        }\n";
            src += strf("        *(float4_t*)(out + ((%s)blockIdx.y * %lld%s + xv * 4u)) = s;\n    }\n}\n", it, (long long)V, sfx);
            k.buffer_args = order;
            k.block[0] = 1024;
            k.grid[0] = (unsigned)bx;
            k.grid[1] = (unsigned)tiles;
            k.chunks = tiles;
            k.bytes = 4.0 * (double)V * (double)tiles;
            for (auto& gb : g.bufs) k.bytes += 4.0 * (double)std::min<int64_t>(numel(gb.node->shape), V * R);
            k.flops = (g.flops + 1) * (double)V * (double)R;
            k.source = src;
            return k;
        }
        int64_t chunks = 1;
        if (force_chunks > 0) chunks = force_chunks;
        else {
            chunks = (2048 + bx - 1) / bx;
            chunks = std::min<int64_t>(chunks, std::max<int64_t>(R / (4 * 8), 1));
            chunks = std::max<int64_t>(chunks, 1);
        }
        const int64_t CH = (R + chunks - 1) / chunks;
        // row groups per block (block = 64 x YG threads): a launch with few blocks gets 16, so that every thread has
        // only a handful of rows to walk and all its loads are in flight together
        const int YG = (bx * chunks < 1024 && CH >= 64) ? 16 : 4;
        k.kind = "reduce_col";
        std::string sig = "const int* __restrict__ guard, float* out";
        std::vector<Node*> order{const_cast<Node*>(n)};
        for (auto& gb : g.bufs) { sig += ", const float* " + gb.param; order.push_back(gb.node); }
        src += strf("extern \"C\" __global__ __launch_bounds__(%d) void %s(%s) {\n", 64 * YG, k.entry.c_str(), sig.c_str());
        src += "    if (guard && *guard == 0) return;\n";
        src += strf("    __shared__ float part[%d][64][%d];\n", YG, vec);
        src += "    const unsigned lx = threadIdx.x & 63u, ly = threadIdx.x >> 6;\n";
        src += strf("    const %s xv = (%s)blockIdx.x * 64u + lx;\n", g.idx_t(), g.idx_t());
        src += "    const unsigned chunk = blockIdx.y;\n";
        src += strf("    const bool col_ok = xv < %lld%s;\n", (long long)XV, wide ? "ull" : "u");
        src += strf("    float acc[%d];\n#pragma unroll\n    for (int j = 0; j < %d; ++j) acc[j] = %s;\n", vec, vec, ident);
        src += strf("    const %s y_end = min((%s)(chunk + 1u) * %lldu, (%s)%lldu);\n", g.idx_t(), g.idx_t(), (long long)CH, g.idx_t(), (long long)R);
        src += strf("    if (col_ok)\n#pragma unroll 8\n    for (%s y = (%s)chunk * %lldu + ly; y < y_end; y += %du) {\n", g.idx_t(), g.idx_t(), (long long)CH, YG);
        src += join(g.codeA, "        ");
        if (vec > 1) src += strf("#pragma unroll\n        for (int j = 0; j < %d; ++j) {\n", vec);
        else src += "        { const int j = 0;\n";
        src += join(g.codeB, "            ");
        src += strf("            acc[j] = %s;\n        }\n    }\n", comb("acc[j]", b.value).c_str());
        src += strf("#pragma unroll\n    for (int j = 0; j < %d; ++j) part[ly][lx][j] = acc[j];\n    __syncthreads();\n", vec);
        src += "    if (ly == 0 && col_ok) {\n";
        src += strf("#pragma unroll\n        for (int j = 0; j < %d; ++j) {\n", vec);
        if (YG == 4)
            src += "            float s = " + comb4("part[0][lx][j]", "part[1][lx][j]", "part[2][lx][j]", "part[3][lx][j]") + ";\n";
        else {
            src += "            float s4[4];\n#pragma unroll\n            for (int q = 0; q < 4; ++q)\n";
            src += "                s4[q] = " + comb4("part[4 * q][lx][j]", "part[4 * q + 1][lx][j]", "part[4 * q + 2][lx][j]", "part[4 * q + 3][lx][j]") + ";\n";
            src += "            float s = " + comb4("s4[0]", "s4[1]", "s4[2]", "s4[3]") + ";\n";
        }
        src += strf("            out[(%s)chunk * %lldu + xv * %du + j] = s;\n        }\n    }\n}\n", g.idx_t(), (long long)V, vec);
        k.buffer_args = order;
        k.block[0] = 64u * YG;
        k.grid[0] = (unsigned)bx;
        k.grid[1] = (unsigned)chunks;
        k.chunks = chunks;
        k.bytes = 4.0 * (double)V * (double)chunks;
        for (auto& gb : g.bufs) k.bytes += 4.0 * (double)std::min<int64_t>(numel(gb.node->shape), V * R);
        k.flops = (g.flops + 1) * (double)V * (double)R;
    }
    k.source = src;
    return k;
}

// ---------------------------------------------------------------------------------------
// row chains
// ---------------------------------------------------------------------------------------

RowAccess row_access(const TRef& t, int64_t V, int64_t R, bool row_level) {
    if (!t.single_full() || t.pieces[0].src.kind != Src::NODE) return RowAccess::OTHER;
    Gen g;
    g.wide = true;
    const int ax = g.add_atom("x", V, false);
    Aff lin = row_level ? aff_atom(ax, 1) : aff_atom(ax, R);
    int ay = -1;
    if (!row_level) {
        ay = g.add_atom("y", R, false);
        lin = aff_add(lin, aff_atom(ay, 1));
    }
    const size_t before = g.atoms.size();
    Aff idx;
    try {
        idx = g.apply_view_from(t.pieces[0].view, 0, lin);
    } catch (const Error&) {
        return RowAccess::OTHER;
    }
    if (g.atoms.size() != before || idx.c != 0) return RowAccess::OTHER;
    if (idx.t.size() == 1 && idx.t[0].first == ax && idx.t[0].second == 1) return RowAccess::ROW;
    if (!row_level && idx.t.size() == 2 && idx.t[0].first == ax && idx.t[0].second == R && idx.t[1].first == ay && idx.t[1].second == 1)
        return RowAccess::FULL;
    return RowAccess::OTHER;
}

// 128-bit quads of a row up to which a wavefront owns the row of a row chain; a longer row belongs to a block of four
// wavefronts.  Measured on the softmax of 8 heads of 2048 x 2048 scores (512 quads a row): a wavefront per row 44.0 us
// forward and 76.4 us backward, a block per row 39.7 and 64.8 (a thread keeps two loads of a stream in registers
// instead of eight); LayerNorm over rows of 1024 elements is as fast either way (7-8 us).
static int64_t rowchain_wave_quads() { return 256; }

bool rowchain_fits(int64_t V, int64_t R) {
    if (V < 1 || R < 4 || R % 4 != 0) return false;
    const int64_t RV = R / 4;
    const int64_t T = RV <= rowchain_wave_quads() ? 64 : 256;
    return (RV + T - 1) / T <= 8;
}

GeneratedKernel gen_rowchain_kernel(const RowChainSpec& spec) {
    const int64_t V = spec.V, R = spec.R, RV = R / 4;
    ADHIP_CHECK(rowchain_fits(V, R), "internal: rows of %lld elements do not fit a row-chain kernel", (long long)R);
    const int T = RV <= rowchain_wave_quads() ? 64 : 256;             // threads per row: a wavefront, or the whole block
    const int64_t K = (RV + T - 1) / T;             // sweeps' trip count: 128-bit pieces of the row per thread
    const int rows_per_block = 256 / T;
    const bool ragged = RV % T != 0;
    const bool wide = needs_wide(spec.order) || V * R >= (int64_t(1) << 31) - 1024;
    const bool nt_out = V * R >= nontemporal_min_elems();
    int n_reduce = 0;
    for (Node* m : spec.order) n_reduce += op_is_reduce(m->op) ? 1 : 0;

    struct Sweep {
        std::vector<std::string> codeA, codeB;
        std::string value;          // reductions: the operand's value at this element
        const Node* reduce = nullptr;
        std::vector<std::string> after;                       // row-uniform statements that follow the sweep
        std::vector<std::pair<const Node*, std::string>> row_values;  // stored one-per-row members: (node, expression)
        std::vector<std::pair<const Node*, std::string>> outputs;     // last sweep: stored full-size members
    };
    struct Built {
        Gen g;
        std::vector<Sweep> sweeps;
        std::map<std::string, int> load_sweeps;   // vector load key -> number of sweeps that make it
        std::vector<std::string> head;             // row-uniform statements before the first sweep
    };
    auto build = [&](const std::set<std::string>& keep) {
        Built b;
        Gen& g = b.g;
        g.vec = 4;
        g.wide = wide;
        g.keep_keys = keep;
        g.keep_index = "it";
        const int ax = g.add_atom("x", V, false), ay = g.add_atom("yv", RV, false);
        g.lane_atom = g.add_atom("j", 4, true);
        const Aff lin = aff_add(aff_add(aff_atom(ax, R), aff_atom(ay, 4)), aff_atom(g.lane_atom, 1));
        const Aff at_x = aff_atom(ax, 1);
        for (Node* m : spec.order) g.members.insert(m);
        size_t a0 = 0, b0 = 0;
        auto begin = [&] {
            g.val_memo.clear();
            g.atom_memo.clear();
            g.sweep_loads.clear();
            a0 = g.codeA.size();
            b0 = g.codeB.size();
        };
        auto take = [&](std::vector<std::string>& A, std::vector<std::string>& B) {
            A.assign(g.codeA.begin() + (long)a0, g.codeA.end());
            B.assign(g.codeB.begin() + (long)b0, g.codeB.end());
            g.codeA.resize(a0);
            g.codeB.resize(b0);
            for (const std::string& k : g.sweep_loads) b.load_sweeps[k] += 1;
        };
        Sweep* last = nullptr;       // the sweep whose `after` list takes row-uniform values
        int ri = 0;
        for (Node* m : spec.order) {
            if (op_is_reduce(m->op)) {
                ADHIP_CHECK(m->in.size() == 1 && m->in[0].shape == (Shape{V, R}), "internal: row-chain reduction over another space");
                b.sweeps.emplace_back();
                Sweep& sw = b.sweeps.back();
                sw.reduce = m;
                begin();
                sw.value = g.gen_tref(m->in[0], lin, "").expr;
                take(sw.codeA, sw.codeB);
                const std::string name = strf("red%d", ri++);
                g.preset[m] = name;
                g.preset_at[m] = aff_key(at_x);
                if (spec.stored.count(m)) sw.row_values.push_back({m, name});
                last = &sw;
            } else if (numel(m->shape) == V && V != V * R) {
                // one value per row: row-uniform code behind the sweep that finished what it needs
                ADHIP_CHECK(op_is_elw(m->op), "internal: row-chain member of the wrong kind");
                begin();
                const int vec_saved = g.vec, lane_saved = g.lane_atom;
                g.vec = 1;
                g.lane_atom = -1;
                const Val v = g.gen_node(m, at_x, "");
                g.vec = vec_saved;
                g.lane_atom = lane_saved;
                std::vector<std::string> A, B;
                take(A, B);
                ADHIP_CHECK(B.empty(), "internal: a per-row value produced per-lane code");
                const std::string name = strf("rv%d", g.tmp++);
                A.push_back(strf("const float %s = %s;", name.c_str(), v.expr.c_str()));
                g.preset[m] = name;
                g.preset_at[m] = aff_key(at_x);
                std::vector<std::string>& dst = last ? last->after : b.head;
                dst.insert(dst.end(), A.begin(), A.end());
                if (spec.stored.count(m)) {
                    ADHIP_CHECK(last, "internal: a stored per-row value before the first sweep of a row chain");
                    last->row_values.push_back({m, name});
                }
            } else {
                ADHIP_CHECK(op_is_elw(m->op) && numel(m->shape) == V * R, "internal: row-chain member of the wrong size");
            }
        }
        // the last sweep evaluates and stores the full-size members
        b.sweeps.emplace_back();
        Sweep& fin = b.sweeps.back();
        begin();
        for (Node* m : spec.order)
            if (!op_is_reduce(m->op) && numel(m->shape) == V * R && spec.stored.count(m)) fin.outputs.push_back({m, g.gen_node(m, lin, "").expr});
        take(fin.codeA, fin.codeB);
        return b;
    };
    std::set<std::string> keep;
    {
        Built dry = build({});
        for (auto& kv : dry.load_sweeps)
            if (kv.second >= 2) keep.insert(kv.first);
        // a kept stream costs 4 K registers a thread
        while ((int64_t)keep.size() * 4 * K > 160) keep.erase(std::prev(keep.end()));
    }
    Built b = build(keep);
    Gen& g = b.g;
    if (b.sweeps.back().outputs.empty()) b.sweeps.pop_back();

    GeneratedKernel k;
    k.kind = "rowchain";
    k.entry = spec.name;
    const char* it_t = g.idx_t();
    const char* sfx = wide ? "ull" : "u";
    // no __restrict__: a stored member may share its buffer with an operand it replaces in place
    std::string sig = "const int* __restrict__ guard";
    std::vector<Node*> order;
    std::map<const Node*, std::string> out_param;
    for (Node* m : spec.order)
        if (spec.stored.count(m)) {
            out_param[m] = strf("w%zu", out_param.size());
            sig += ", float* " + out_param[m];
            order.push_back(m);
        }
    for (auto& gb : g.bufs) { sig += ", const float* " + gb.param; order.push_back(gb.node); }
    std::string src = kernel_prelude();
    src += strf("extern \"C\" __global__ __launch_bounds__(256) void %s(%s) {\n", k.entry.c_str(), sig.c_str());
    src += "    if (guard && *guard == 0) return;\n";
    if (T == 256 && n_reduce > 0) src += strf("    __shared__ float part[%d][4];\n", n_reduce);
    src += strf("    const unsigned lane = threadIdx.x %% %du;\n", T);
    src += strf("    const %s x_raw = (%s)blockIdx.x * %du + threadIdx.x / %du;\n", it_t, it_t, rows_per_block, T);
    // a row beyond the last one works on the last one and stores nothing: no thread leaves early
    src += strf("    const bool row_ok = x_raw < %lld%s;\n    const %s x = row_ok ? x_raw : %lld%s;\n", (long long)V, sfx, it_t, (long long)(V - 1), sfx);
    for (const std::string& arr : g.kept_decls) src += strf("    float4_t %s[%lld];\n", arr.c_str(), (long long)K);
    src += join(b.head, "    ");
    int ri = 0;
    for (size_t si = 0; si < b.sweeps.size(); ++si) {
        Sweep& sw = b.sweeps[si];
        const bool mx = sw.reduce && sw.reduce->op == Op::MAX;
        const char* ident = mx ? "__builtin_nanf(\"\")" : "0.0f";
        if (sw.reduce) src += strf("    float acc%d[4] = {%s, %s, %s, %s};\n", ri, ident, ident, ident, ident);
        src += strf("#pragma unroll\n    for (unsigned it = 0; it < %lldu; ++it) {\n", (long long)K);
        if (ragged) src += strf("        const %s yv_raw = lane + it * %du;\n        const bool live = yv_raw < %lldu;\n        const %s yv = live ? yv_raw : %lldu;\n",
                                it_t, T, (long long)RV, it_t, (long long)(RV - 1));
        else src += strf("        const %s yv = lane + it * %du;\n", it_t, T);
        src += join(sw.codeA, "        ");
        for (size_t i = 0; i < sw.outputs.size(); ++i) src += strf("        float o%zu[4];\n", i);
        src += "#pragma unroll\n        for (int j = 0; j < 4; ++j) {\n";
        src += join(sw.codeB, "            ");
        if (sw.reduce) {
            const std::string a = strf("acc%d[j]", ri);
            const std::string c = mx ? "fmaxf(" + a + ", " + sw.value + ")" : a + " + " + sw.value;
            src += strf("            %s%s = %s;\n", ragged ? "if (live) " : "", a.c_str(), c.c_str());
        }
        for (size_t i = 0; i < sw.outputs.size(); ++i) src += strf("            o%zu[j] = %s;\n", i, sw.outputs[i].second.c_str());
        src += "        }\n";
        if (!sw.outputs.empty()) {
            src += strf("        if (row_ok%s) {\n", ragged ? " && live" : "");
            for (size_t i = 0; i < sw.outputs.size(); ++i)
                src += "            " + store4_stmt(strf("o%zu", i), strf("%s + (%lld%s * x + 4u * yv)", out_param[sw.outputs[i].first].c_str(), (long long)R, sfx), nt_out) + "\n";
            src += "        }\n";
        }
        src += "    }\n";
        if (sw.reduce) {
            const std::string a = strf("acc%d", ri);
            const std::string s4 = mx ? strf("fmaxf(fmaxf(%s[0], %s[1]), fmaxf(%s[2], %s[3]))", a.c_str(), a.c_str(), a.c_str(), a.c_str())
                                      : strf("(%s[0] + %s[1]) + (%s[2] + %s[3])", a.c_str(), a.c_str(), a.c_str(), a.c_str());
            if (T == 64) {
                src += strf("    const float red%d = %s(%s);\n", ri, mx ? "wave_max" : "wave_sum", s4.c_str());
            } else {
                src += strf("    { const float s = %s(%s); if ((threadIdx.x & 63u) == 0) part[%d][threadIdx.x >> 6] = s; }\n    __syncthreads();\n",
                            mx ? "wave_max" : "wave_sum", s4.c_str(), ri);
                src += mx ? strf("    const float red%d = fmaxf(fmaxf(part[%d][0], part[%d][1]), fmaxf(part[%d][2], part[%d][3]));\n", ri, ri, ri, ri, ri)
                          : strf("    const float red%d = (part[%d][0] + part[%d][1]) + (part[%d][2] + part[%d][3]);\n", ri, ri, ri, ri, ri);
            }
            ++ri;
        }
        src += join(sw.after, "    ");
    }
    // one value per row: stored last, by the row's first lane, when every thread of the row has read what it needed
    bool any_row_value = false;
    for (Sweep& sw : b.sweeps) any_row_value = any_row_value || !sw.row_values.empty();
    if (any_row_value) {
        if (T == 256) src += "    __syncthreads();\n";
        src += "    if (lane == 0u && row_ok) {\n";
        for (Sweep& sw : b.sweeps)
            for (auto& rv : sw.row_values) src += strf("        %s[x] = %s;\n", out_param[rv.first].c_str(), rv.second.c_str());
        src += "    }\n";
    }
    src += "}\n";
    k.source = src;
    k.buffer_args = order;
    k.block[0] = 256;
    k.grid[0] = (unsigned)((V + rows_per_block - 1) / rows_per_block);
    k.bytes = 0;
    for (Node* m : spec.order)
        if (spec.stored.count(m)) k.bytes += 4.0 * (double)numel(m->shape);
    for (auto& gb : g.bufs) k.bytes += 4.0 * (double)std::min<int64_t>(numel(gb.node->shape), V * R);
    k.flops = (g.flops + n_reduce) * (double)V * (double)R;
    return k;
}

bool tref_affine2d(const TRef& t, Affine2D& out) {
    if (t.shape.size() != 2 || !t.single_full()) return false;
    const Piece& p = t.pieces[0];
    if (p.src.kind != Src::NODE) return false;
    Gen g;
    g.wide = true;
    int ar = g.add_atom("r", t.shape[0], false);
    int ak = g.add_atom("k", t.shape[1], false);
    Aff lin = aff_add(aff_atom(ar, t.shape[1]), aff_atom(ak, 1));
    const size_t before = g.atoms.size();
    Aff idx;
    try {
        idx = g.apply_view_from(p.view, 0, lin);
    } catch (const Error&) {
        return false;
    }
    if (g.atoms.size() != before) return false;
    out.base = p.src.node;
    out.offset = idx.c;
    out.s0 = out.s1 = 0;
    for (auto& x : idx.t) {
        if (x.first == ar) out.s0 = x.second;
        else if (x.first == ak) out.s1 = x.second;
    }
    if (out.s0 < 0 || out.s1 < 0) return false;
    return true;
}

}  // namespace adhip
