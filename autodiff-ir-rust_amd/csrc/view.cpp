#include "view.hpp"

#include <algorithm>

#include "graph.hpp"

namespace adhip {

bool Src::same(const Src& o) const {
    if (kind != o.kind) return false;
    switch (kind) {
    case NODE: return node == o.node;
    case SYM: return sym == o.sym;
    case CONST: return c == o.c || (c != c && o.c != o.c);
    case NESTED: return nested.get() == o.nested.get();
    }
    return false;
}

bool TRef::single_full() const {
    if (pieces.size() != 1) return false;
    const Piece& p = pieces[0];
    for (size_t i = 0; i < shape.size(); ++i)
        if (p.lo[i] != 0 || p.hi[i] != shape[i]) return false;
    return true;
}

Stage contiguous_stage(const Shape& shape) {
    Stage s;
    s.shape = shape;
    s.stride = row_major_strides(shape);
    s.offset = 0;
    return s;
}

bool stage_is_identity(const Stage& s) {
    if (s.offset != 0) return false;
    int64_t expect = 1;
    for (int i = (int)s.shape.size() - 1; i >= 0; --i) {
        if (s.shape[i] == 1) continue;
        if (s.stride[i] != expect) return false;
        expect *= s.shape[i];
    }
    return true;
}

bool stage_try_reshape(const Stage& in, const Shape& new_shape, Stage& out) {
    // Classic no-copy reshape: walk groups of old and new dims with equal products; an old group
    // can be re-split only if it is contiguous within itself.
    Shape os, ost;
    for (size_t i = 0; i < in.shape.size(); ++i)
        if (in.shape[i] != 1) { os.push_back(in.shape[i]); ost.push_back(in.stride[i]); }
    out.shape = new_shape;
    out.stride.assign(new_shape.size(), 0);
    out.offset = in.offset;
    if (numel(new_shape) == 0 || numel(in.shape) == 0) return numel(new_shape) == numel(in.shape);
    size_t oi = 0, ni = 0;
    const size_t on = os.size(), nn = new_shape.size();
    while (ni < nn && new_shape[ni] == 1) ++ni;
    while (oi < on && ni < nn) {
        int64_t op = os[oi], np = new_shape[ni];
        size_t oj = oi + 1, nj = ni + 1;
        while (op != np) {
            if (op < np) { if (oj >= on) return false; op *= os[oj++]; }
            else { if (nj >= nn) return false; np *= new_shape[nj++]; }
        }
        for (size_t k = oi; k + 1 < oj; ++k)
            if (ost[k] != ost[k + 1] * os[k + 1]) return false;
        int64_t st = ost[oj - 1];
        for (size_t k = nj; k-- > ni;) {
            out.stride[k] = st;
            st *= new_shape[k];
        }
        oi = oj;
        ni = nj;
        while (ni < nn && new_shape[ni] == 1) ++ni;
    }
    return oi == on && ni == nn;
}

void view_reshape(View& v, const Shape& new_shape) {
    Stage out;
    if (stage_try_reshape(v.st.front(), new_shape, out)) {
        v.st.front() = out;
    } else {
        v.st.insert(v.st.begin(), contiguous_stage(new_shape));
    }
}

static Piece full_piece(const Shape& shape, Src src) {
    Piece p;
    p.lo.assign(shape.size(), 0);
    p.hi = shape;
    p.view.st.push_back(contiguous_stage(shape));
    p.src = std::move(src);
    return p;
}

TRef tr_sym(const std::string& id, const Shape& shape) {
    Src s; s.kind = Src::SYM; s.sym = id;
    TRef t; t.shape = shape; t.pieces.push_back(full_piece(shape, s));
    return t;
}

TRef tr_node(Node* n, const Shape& shape) {
    Src s; s.kind = Src::NODE; s.node = n;
    TRef t; t.shape = shape; t.pieces.push_back(full_piece(shape, s));
    return t;
}

TRef tr_const(float c, const Shape& shape) {
    Src s; s.kind = Src::CONST; s.c = c;
    TRef t; t.shape = shape; t.pieces.push_back(full_piece(shape, s));
    return t;
}

TRef tr_permute(const TRef& t, const Shape& p) {
    const size_t n = t.shape.size();
    ADHIP_CHECK(p.size() == n, "Permute: rank mismatch (%zu vs %zu)", p.size(), n);
    std::vector<bool> seen(n, false);
    for (auto v : p) {
        ADHIP_CHECK(v >= 0 && (size_t)v < n && !seen[v], "Permute: not a permutation");
        seen[v] = true;
    }
    TRef r;
    r.shape.resize(n);
    for (size_t i = 0; i < n; ++i) r.shape[i] = t.shape[p[i]];
    for (const Piece& pc : t.pieces) {
        Piece q = pc;
        const Stage& s0 = pc.view.st.front();
        Stage& d0 = q.view.st.front();
        for (size_t i = 0; i < n; ++i) {
            q.lo[i] = pc.lo[p[i]];
            q.hi[i] = pc.hi[p[i]];
            d0.shape[i] = s0.shape[p[i]];
            d0.stride[i] = s0.stride[p[i]];
        }
        r.pieces.push_back(std::move(q));
    }
    return r;
}

TRef tr_broadcast(const TRef& t, int64_t dim, int64_t r) {
    ADHIP_CHECK(dim >= 0 && (size_t)dim < t.shape.size(), "Broadcast: dim out of range");
    ADHIP_CHECK(t.shape[dim] == 1 || t.shape[dim] == r, "Broadcast: source extent %lld is not 1",
                (long long)t.shape[dim]);
    TRef o = t;
    if (t.shape[dim] == r) return o;
    o.shape[dim] = r;
    for (Piece& p : o.pieces) {
        p.hi[dim] = r;
        p.view.st.front().shape[dim] = r;
        p.view.st.front().stride[dim] = 0;
    }
    return o;
}

TRef tr_index(const TRef& t, int64_t index, int64_t dim) {
    ADHIP_CHECK(dim >= 0 && (size_t)dim < t.shape.size(), "Index: dim out of range");
    ADHIP_CHECK(index >= 0 && index < t.shape[dim], "Index: index %lld out of range %lld", (long long)index,
                (long long)t.shape[dim]);
    TRef o;
    o.shape = t.shape;
    o.shape.erase(o.shape.begin() + dim);
    for (const Piece& pc : t.pieces) {
        if (index < pc.lo[dim] || index >= pc.hi[dim]) continue;
        Piece q = pc;
        Stage& s0 = q.view.st.front();
        s0.offset += (index - pc.lo[dim]) * s0.stride[dim];
        s0.shape.erase(s0.shape.begin() + dim);
        s0.stride.erase(s0.stride.begin() + dim);
        q.lo.erase(q.lo.begin() + dim);
        q.hi.erase(q.hi.begin() + dim);
        o.pieces.push_back(std::move(q));
    }
    return o;
}

// Try to fuse q into p when both are the same strided walk over the same source and q continues p
// along `dim`.  This is what collapses a range-select (one Index + unsqueeze + Concat per row,
// reference src/graph/data/index.rs:84-89) back into a single slice.
static bool try_merge(Piece& p, const Piece& q, size_t dim) {
    if (!p.src.same(q.src)) return false;
    if (p.src.kind == Src::CONST) {
        // constants have no addressing; boxes only need to line up
    } else if (p.view.st.size() != 1 || q.view.st.size() != 1) {
        return false;
    }
    const size_t n = p.lo.size();
    for (size_t i = 0; i < n; ++i) {
        if (i == dim) continue;
        if (p.lo[i] != q.lo[i] || p.hi[i] != q.hi[i]) return false;
    }
    if (p.hi[dim] != q.lo[dim]) return false;
    if (p.src.kind != Src::CONST) {
        const Stage& a = p.view.st[0];
        const Stage& b = q.view.st[0];
        for (size_t i = 0; i < n; ++i) {
            if (i == dim) continue;
            if (a.shape[i] > 1 && a.stride[i] != b.stride[i]) return false;
        }
        const int64_t la = a.shape[dim], lb = b.shape[dim];
        int64_t sd;
        if (la > 1) sd = a.stride[dim];
        else if (lb > 1) sd = b.stride[dim];
        else sd = b.offset - a.offset;
        if (sd < 0) return false;
        if (la > 1 && lb > 1 && a.stride[dim] != b.stride[dim]) return false;
        if (b.offset != a.offset + la * sd) return false;
        p.view.st[0].stride[dim] = sd;
    }
    p.hi[dim] = q.hi[dim];
    p.view.st[0].shape[dim] = p.hi[dim] - p.lo[dim];
    return true;
}

TRef tr_concat(const TRef& a, const TRef& b, int64_t dim) {
    const size_t n = a.shape.size();
    ADHIP_CHECK(b.shape.size() == n, "Concat: rank mismatch");
    ADHIP_CHECK(dim >= 0 && (size_t)dim < n, "Concat: dim out of range");
    for (size_t i = 0; i < n; ++i)
        ADHIP_CHECK((int64_t)i == dim || a.shape[i] == b.shape[i], "Concat: shapes %s and %s differ outside dim %lld",
                    shape_str(a.shape).c_str(), shape_str(b.shape).c_str(), (long long)dim);
    TRef o;
    o.shape = a.shape;
    o.shape[dim] += b.shape[dim];
    auto nonempty = [](const Piece& p) {
        for (size_t i = 0; i < p.lo.size(); ++i)
            if (p.hi[i] <= p.lo[i]) return false;
        return true;
    };
    for (const Piece& p : a.pieces)
        if (nonempty(p)) o.pieces.push_back(p);
    for (const Piece& p0 : b.pieces) {
        if (!nonempty(p0)) continue;
        Piece q = p0;
        q.lo[dim] += a.shape[dim];
        q.hi[dim] += a.shape[dim];
        bool merged = false;
        for (Piece& p : o.pieces) {
            if (try_merge(p, q, (size_t)dim)) { merged = true; break; }
        }
        if (!merged) o.pieces.push_back(std::move(q));
    }
    return o;
}

static TRef nested_reshape(const TRef& t, const Shape& new_shape) {
    Src s;
    s.kind = Src::NESTED;
    s.nested = std::make_shared<TRef>(t);
    TRef o;
    o.shape = new_shape;
    o.pieces.push_back(full_piece(new_shape, s));
    return o;
}

TRef tr_reshape(const TRef& t, const Shape& new_shape) {
    ADHIP_CHECK(numel(t.shape) == numel(new_shape), "View: %s cannot be viewed as %s", shape_str(t.shape).c_str(),
                shape_str(new_shape).c_str());
    if (t.shape == new_shape) return t;
    if (numel(new_shape) == 0) {
        TRef o; o.shape = new_shape; return o;
    }
    if (t.single_full()) {
        TRef o = t;
        o.shape = new_shape;
        Piece& p = o.pieces[0];
        p.lo.assign(new_shape.size(), 0);
        p.hi = new_shape;
        if (p.src.kind == Src::CONST) p.view.st = {contiguous_stage(new_shape)};
        else view_reshape(p.view, new_shape);
        return o;
    }
    // Several pieces: map every box through the reshape when each dim group allows it.
    const Shape& os = t.shape;
    const size_t on = os.size(), nn = new_shape.size();
    struct Group { size_t o0, o1, n0, n1; };
    std::vector<Group> groups;
    {
        size_t oi = 0, ni = 0;
        while (oi < on || ni < nn) {
            Group g{oi, oi, ni, ni};
            int64_t op = 1, np = 1;
            if (oi < on) { op = os[oi]; g.o1 = ++oi; }
            if (ni < nn) { np = new_shape[ni]; g.n1 = ++ni; }
            while (op != np) {
                if (op < np) { if (oi >= on) return nested_reshape(t, new_shape); op *= os[oi]; g.o1 = ++oi; }
                else { if (ni >= nn) return nested_reshape(t, new_shape); np *= new_shape[ni]; g.n1 = ++ni; }
            }
            groups.push_back(g);
        }
    }
    TRef o;
    o.shape = new_shape;
    for (const Piece& pc : t.pieces) {
        Piece q;
        q.src = pc.src;
        q.lo.assign(nn, 0);
        q.hi = new_shape;
        for (const Group& g : groups) {
            // find the first old dim of the group where the piece is partial; everything after it
            // inside the group must be full
            int64_t lo_lin = 0, hi_lin = 0;  // box along the group's linearised extent, as [lo, hi)
            bool partial_seen = false;
            int64_t inner = 1;
            for (size_t k = g.o1; k-- > g.o0;) {
                bool full = pc.lo[k] == 0 && pc.hi[k] == os[k];
                if (!full) {
                    if (partial_seen) return nested_reshape(t, new_shape);
                    partial_seen = true;
                    lo_lin = pc.lo[k] * inner;
                    hi_lin = pc.hi[k] * inner;
                    // all outer dims of the group must then have extent 1
                    for (size_t m = g.o0; m < k; ++m)
                        if (os[m] != 1) return nested_reshape(t, new_shape);
                }
                inner *= os[k];
            }
            if (!partial_seen) continue;  // full in this group: new dims stay full
            // place [lo_lin, hi_lin) on the new dims of the group: it must be a range of one new dim
            // with everything inside it full
            int64_t ninner = 1;
            bool placed = false;
            for (size_t k = g.n1; k-- > g.n0;) {
                int64_t ext = new_shape[k];
                if (!placed && lo_lin % ninner == 0 && hi_lin % ninner == 0 && hi_lin / ninner <= ext) {
                    // candidate: this dim takes the range; outer new dims must have extent 1
                    bool ok = true;
                    for (size_t m = g.n0; m < k; ++m)
                        if (new_shape[m] != 1) ok = false;
                    if (ok) {
                        q.lo[k] = lo_lin / ninner;
                        q.hi[k] = hi_lin / ninner;
                        placed = true;
                        break;
                    }
                }
                ninner *= ext;
            }
            if (!placed) return nested_reshape(t, new_shape);
        }
        Shape local(nn);
        for (size_t i = 0; i < nn; ++i) local[i] = q.hi[i] - q.lo[i];
        q.view = pc.view;
        if (q.src.kind == Src::CONST) q.view.st = {contiguous_stage(local)};
        else view_reshape(q.view, local);
        o.pieces.push_back(std::move(q));
    }
    return o;
}

std::string stage_str(const Stage& s) {
    return "{" + shape_str(s.shape) + "*" + shape_str(s.stride) + "+" + std::to_string(s.offset) + "}";
}

std::string tref_str(const TRef& t) {
    std::string o = shape_str(t.shape) + "<";
    for (size_t i = 0; i < t.pieces.size(); ++i) {
        const Piece& p = t.pieces[i];
        if (i) o += " | ";
        if (!t.single_full()) o += shape_str(p.lo) + ".." + shape_str(p.hi) + ":";
        switch (p.src.kind) {
        case Src::NODE: o += "n" + std::to_string(p.src.node ? p.src.node->id : -1); break;
        case Src::SYM: o += "$" + p.src.sym; break;
        case Src::CONST: o += strf("%g", p.src.c); break;
        case Src::NESTED: o += "(" + tref_str(*p.src.nested) + ")"; break;
        }
        if (p.src.kind != Src::CONST)
            for (const Stage& s : p.view.st) o += stage_str(s);
    }
    return o + ">";
}

}  // namespace adhip
