#include "ir.hpp"

#include <cstring>

namespace adhip {

namespace {
// Largest extent, index or repeat count a command may carry (2^40); products of extents are checked where they are formed.
constexpr int64_t kMaxExtent = int64_t(1) << 40;

struct Reader {
    int64_t bounded() {
        const int64_t v = (int64_t)u64();
        ADHIP_CHECK(v >= -kMaxExtent && v <= kMaxExtent, "index or count %lld out of range", (long long)v);
        return v;
    }
    const uint8_t* p;
    const uint8_t* end;
    const uint8_t* base = nullptr;
    std::vector<size_t>* payload_offsets = nullptr;
    void need(size_t n) { ADHIP_CHECK((size_t)(end - p) >= n, "program stream truncated"); }
    uint8_t u8() { need(1); return *p++; }
    uint32_t u32() { need(4); uint32_t v; memcpy(&v, p, 4); p += 4; return v; }
    uint64_t u64() { need(8); uint64_t v; memcpy(&v, p, 8); p += 8; return v; }
    float f32() { need(4); float v; memcpy(&v, p, 4); p += 4; return v; }
    std::string str() {
        uint32_t n = u32();
        need(n);
        std::string s((const char*)p, n);
        p += n;
        return s;
    }
    Shape dims() {
        uint32_t n = u32();
        ADHIP_CHECK(n <= 64, "tensor rank %u too large", n);
        Shape s(n);
        for (uint32_t i = 0; i < n; ++i) {
            s[i] = (int64_t)u64();
            ADHIP_CHECK(s[i] >= -1 && s[i] <= kMaxExtent, "tensor extent %lld out of range", (long long)s[i]);
        }
        return s;
    }
};

std::unique_ptr<Proc> parse_proc(Reader& r, int depth) {
    ADHIP_CHECK(depth < 64, "procedures nested too deeply");
    auto proc = std::make_unique<Proc>();
    proc->id = r.str();
    uint32_t n = r.u32();
    ADHIP_CHECK((size_t)(r.end - r.p) >= n, "program stream truncated");  // every command takes at least one byte
    proc->cmds.reserve(n);
    for (uint32_t i = 0; i < n; ++i) {
        Cmd c;
        uint8_t t = r.u8();
        ADHIP_CHECK(t < T_COUNT, "unknown IR command tag %u", (unsigned)t);
        c.tag = (Tag)t;
        switch (c.tag) {
        case T_CREATE_MAT: {
            c.res = r.str();
            c.dims = r.dims();
            if (r.payload_offsets) r.payload_offsets->push_back((size_t)(r.p - r.base));
            c.host = (const float*)(uintptr_t)r.u64();
            c.count = r.u64();
            ADHIP_CHECK((int64_t)c.count == numel(c.dims), "CreateMat %s: %llu values for dim %s", c.res.c_str(),
                        (unsigned long long)c.count, shape_str(c.dims).c_str());
            ADHIP_CHECK(c.count == 0 || c.host != nullptr, "CreateMat %s: null contents", c.res.c_str());
            break;
        }
        case T_CREATE_CONSTANT:
            c.f = r.f32();
            c.res = r.str();
            c.dims = r.dims();
            break;
        case T_ELW_MULTIPLY: case T_ELW_ADD: case T_DOT_PRODUCT:
            c.a = r.str(); c.b = r.str(); c.res = r.str();
            break;
        case T_ELW_MULTIPLY_EQ: case T_ELW_ADD_EQ:
            c.a = r.str(); c.b = r.str(); c.res = c.a;
            break;
        case T_EQUAL_ZERO: case T_MORE_ZERO: case T_LESS_ZERO: case T_SUM: case T_MAX: case T_CONTIGIOUS:
        case T_EXP2: case T_LOG2: case T_SIN: case T_RECIP: case T_SQRT:
            c.a = r.str(); c.res = r.str();
            break;
        case T_VIEW:
            c.a = r.str(); c.dims = r.dims(); c.res = r.str();
            break;
        case T_INDEX:
            c.a = r.str(); c.i0 = r.bounded(); c.i1 = r.bounded(); c.res = r.str();
            break;
        case T_CONCAT:
            c.a = r.str(); c.b = r.str(); c.i0 = r.bounded(); c.res = r.str();
            break;
        case T_PERMUTE:
            c.a = r.str(); c.dims = r.dims(); c.res = r.str();
            break;
        case T_BROADCAST:
            c.a = r.str(); c.i0 = r.bounded(); c.i1 = r.bounded(); c.res = r.str();
            break;
        case T_WHILE:
            c.a = r.str();
            c.block = parse_proc(r, depth + 1);
            break;
        case T_IF: {
            uint32_t nc = r.u32();
            for (uint32_t k = 0; k < nc; ++k) {
                std::string cond = r.str();
                c.conds.emplace_back(cond, parse_proc(r, depth + 1));
            }
            if (r.u8()) c.else_block = parse_proc(r, depth + 1);
            break;
        }
        case T_EX:
            break;
        case T_HEADING:
            c.text = r.str();
            break;
        default:
            throw Error("unreachable");
        }
        proc->cmds.push_back(std::move(c));
    }
    return proc;
}
}  // namespace

std::unique_ptr<Proc> parse_program(const uint8_t* data, size_t len, std::vector<size_t>* payload_offsets) {
    ADHIP_CHECK(data != nullptr && len >= 8, "program stream too short");
    ADHIP_CHECK(memcmp(data, "ADIR", 4) == 0, "bad program magic");
    Reader r{data + 4, data + len, data, payload_offsets};
    uint32_t ver = r.u32();
    ADHIP_CHECK(ver == 1, "unsupported program version %u", ver);
    auto p = parse_proc(r, 0);
    ADHIP_CHECK(r.p == r.end, "trailing bytes after program");
    return p;
}

const char* tag_name(Tag t) {
    static const char* names[] = {"CreateMat", "CreateConstant", "ElwMultiply", "ElwAdd", "ElwMultiplyEq",
                                  "ElwAddEq", "EqualZero", "MoreZero", "LessZero", "Sum", "DotProduct", "View",
                                  "Index", "Concat", "Permute", "Broadcast", "Contigious", "Exp2", "Log2", "Sin",
                                  "Recip", "Sqrt", "While", "If", "EX", "Heading", "Max"};
    return t < T_COUNT ? names[t] : "?";
}

}  // namespace adhip
