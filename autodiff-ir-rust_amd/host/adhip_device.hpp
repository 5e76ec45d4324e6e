// C++ host-side mirror of the reference's device boundary, over the C ABI of include/adhip.h.
//
//   Device      <->  trait Device { execute, get_tensor, ir_callback, dot_prod_shape }   reference src/core/ir.rs:126-143
//   IRCmd/IRProcedure <-> enum IRCmds / struct IRProcedure                              reference src/core/ir.rs:8-112
//   ValueData   <->  struct ValueData                                                    reference src/core/value_data.rs:6-11
//
// A Rust `impl Device` would do exactly what HipDevice does here: serialise the IR procedure, call
// adhip_execute with the keep list, and turn adhip_get_tensor's borrowed pointers into an owned ValueData.
#pragma once
#include <cstdint>
#include <cstring>
#include <memory>
#include <set>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/adhip.h"

namespace adhip_host {

enum Tag : uint8_t {
    CreateMat = 0, CreateConstant, ElwMultiply, ElwAdd, ElwMultiplyEq, ElwAddEq, EqualZero, MoreZero, LessZero, Sum,
    DotProduct, View, Index, Concat, Permute, Broadcast, Contigious, Exp2, Log2, Sin, Recip, Sqrt, While, If, EX, Heading,
    // not a variant of the reference's enum: the row maximum it declares (ReduceOp::Max, reference
    // src/kernel/kernel_decl.rs:75-78) but never emits; same fields as Sum
    Max
};

struct IRProcedure;

// One IR command; which fields are meaningful depends on the tag (names follow the reference's fields).
struct IRCmd {
    Tag tag = EX;
    std::string a, b, res;               // a/b/res; s/o of the *Eq forms are a/b; id of Create* is res
    std::vector<uint64_t> dim;           // dim / target_dim / p
    uint64_t index = 0, dim_index = 0, r = 0;
    float constant = 0.f;
    std::shared_ptr<std::vector<float>> contents;  // CreateMat
    std::string cmt;
    std::shared_ptr<IRProcedure> block;                                       // While
    std::vector<std::pair<std::string, std::shared_ptr<IRProcedure>>> conditions;  // If
    std::shared_ptr<IRProcedure> else_proc;
};

struct IRProcedure {
    std::string id = "main";
    std::vector<IRCmd> main;
    void push(IRCmd c) { main.push_back(std::move(c)); }
};

struct ValueData {
    std::vector<size_t> dim;
    std::vector<float> data;
    std::string id;
    bool is_none = true;
};

// command constructors, named after the reference's variants
inline IRCmd create_mat(std::string id, std::vector<uint64_t> dim, std::vector<float> data) {
    IRCmd c; c.tag = CreateMat; c.res = std::move(id); c.dim = std::move(dim);
    c.contents = std::make_shared<std::vector<float>>(std::move(data)); return c;
}
inline IRCmd create_constant(std::string id, float v, std::vector<uint64_t> dim) {
    IRCmd c; c.tag = CreateConstant; c.res = std::move(id); c.constant = v; c.dim = std::move(dim); return c;
}
inline IRCmd binary(Tag t, std::string a, std::string b, std::string res) {
    IRCmd c; c.tag = t; c.a = std::move(a); c.b = std::move(b); c.res = std::move(res); return c;
}
inline IRCmd op_eq(Tag t, std::string s, std::string o) { IRCmd c; c.tag = t; c.a = std::move(s); c.b = std::move(o); return c; }
inline IRCmd unary(Tag t, std::string a, std::string res) { IRCmd c; c.tag = t; c.a = std::move(a); c.res = std::move(res); return c; }
inline IRCmd view(std::string a, std::vector<uint64_t> target, std::string res) {
    IRCmd c; c.tag = View; c.a = std::move(a); c.dim = std::move(target); c.res = std::move(res); return c;
}
inline IRCmd permute(std::string a, std::vector<uint64_t> p, std::string res) {
    IRCmd c; c.tag = Permute; c.a = std::move(a); c.dim = std::move(p); c.res = std::move(res); return c;
}
inline IRCmd broadcast(std::string a, uint64_t dim, uint64_t r, std::string res) {
    IRCmd c; c.tag = Broadcast; c.a = std::move(a); c.dim_index = dim; c.r = r; c.res = std::move(res); return c;
}
inline IRCmd index(std::string a, uint64_t idx, uint64_t dim, std::string res) {
    IRCmd c; c.tag = Index; c.a = std::move(a); c.index = idx; c.dim_index = dim; c.res = std::move(res); return c;
}
inline IRCmd concat(std::string a, std::string b, uint64_t dim, std::string res) {
    IRCmd c; c.tag = Concat; c.a = std::move(a); c.b = std::move(b); c.dim_index = dim; c.res = std::move(res); return c;
}
inline IRCmd while_(std::string cond, IRProcedure body) {
    IRCmd c; c.tag = While; c.a = std::move(cond); c.block = std::make_shared<IRProcedure>(std::move(body)); return c;
}
inline IRCmd if_(std::string cond, IRProcedure then_block, const IRProcedure* else_block = nullptr) {
    IRCmd c; c.tag = If; c.conditions.emplace_back(std::move(cond), std::make_shared<IRProcedure>(std::move(then_block)));
    if (else_block) c.else_proc = std::make_shared<IRProcedure>(*else_block);
    return c;
}
inline IRCmd if_arms(std::vector<std::pair<std::string, IRProcedure>> arms, const IRProcedure* else_block = nullptr) {
    IRCmd c; c.tag = If;
    for (auto& arm : arms) c.conditions.emplace_back(std::move(arm.first), std::make_shared<IRProcedure>(std::move(arm.second)));
    if (else_block) c.else_proc = std::make_shared<IRProcedure>(*else_block);
    return c;
}
inline IRCmd heading(std::string cmt) { IRCmd c; c.tag = Heading; c.cmt = std::move(cmt); return c; }
inline IRCmd ex() { IRCmd c; c.tag = EX; return c; }

namespace detail {
inline void put(std::vector<uint8_t>& o, const void* p, size_t n) { const uint8_t* b = (const uint8_t*)p; o.insert(o.end(), b, b + n); }
inline void u32(std::vector<uint8_t>& o, uint32_t v) { put(o, &v, 4); }
inline void u64(std::vector<uint8_t>& o, uint64_t v) { put(o, &v, 8); }
inline void str(std::vector<uint8_t>& o, const std::string& s) { u32(o, (uint32_t)s.size()); put(o, s.data(), s.size()); }
inline void dims(std::vector<uint8_t>& o, const std::vector<uint64_t>& d) { u32(o, (uint32_t)d.size()); for (auto v : d) u64(o, v); }
inline void proc(std::vector<uint8_t>& o, const IRProcedure& p, std::vector<size_t>* payload_offsets) {
    str(o, p.id);
    u32(o, (uint32_t)p.main.size());
    for (const IRCmd& c : p.main) {
        o.push_back((uint8_t)c.tag);
        switch (c.tag) {
        case CreateMat:
            str(o, c.res); dims(o, c.dim);
            if (payload_offsets) payload_offsets->push_back(o.size());
            u64(o, (uint64_t)(uintptr_t)c.contents->data()); u64(o, c.contents->size());
            break;
        case CreateConstant: put(o, &c.constant, 4); str(o, c.res); dims(o, c.dim); break;
        case ElwMultiply: case ElwAdd: case DotProduct: str(o, c.a); str(o, c.b); str(o, c.res); break;
        case ElwMultiplyEq: case ElwAddEq: str(o, c.a); str(o, c.b); break;
        case View: case Permute: str(o, c.a); dims(o, c.dim); str(o, c.res); break;
        case Index: str(o, c.a); u64(o, c.index); u64(o, c.dim_index); str(o, c.res); break;
        case Concat: str(o, c.a); str(o, c.b); u64(o, c.dim_index); str(o, c.res); break;
        case Broadcast: str(o, c.a); u64(o, c.dim_index); u64(o, c.r); str(o, c.res); break;
        case While: str(o, c.a); proc(o, *c.block, payload_offsets); break;
        case If:
            u32(o, (uint32_t)c.conditions.size());
            for (auto& arm : c.conditions) { str(o, arm.first); proc(o, *arm.second, payload_offsets); }
            o.push_back(c.else_proc ? 1 : 0);
            if (c.else_proc) proc(o, *c.else_proc, payload_offsets);
            break;
        case EX: break;
        case Heading: str(o, c.cmt); break;
        default: str(o, c.a); str(o, c.res); break;  // the two-id commands
        }
    }
}
}  // namespace detail

// Flat little-endian stream understood by adhip_execute.  CreateMat payloads are referenced by pointer: the
// procedure must stay alive (and unmodified) until the call returns.  `payload_offsets`, when given, receives the byte
// offset of every such pointer field (the only bytes of the stream that differ from run to run).
inline std::vector<uint8_t> serialize(const IRProcedure& p, std::vector<size_t>* payload_offsets = nullptr) {
    std::vector<uint8_t> o{'A', 'D', 'I', 'R'};
    detail::u32(o, 1);
    detail::proc(o, p, payload_offsets);
    return o;
}

struct Device {
    virtual ~Device() = default;
    virtual void execute(const IRProcedure& proc, const std::set<std::string>& dep_list) = 0;
    virtual ValueData get_tensor(const std::string& id) const = 0;
    virtual void ir_callback(IRProcedure&) const {}
    virtual std::vector<size_t> dot_prod_shape(const std::vector<size_t>& a, const std::vector<size_t>& b) const {
        return {a.front(), b.back()};
    }
};

class HipDevice : public Device {
public:
    explicit HipDevice(int ordinal = 0) {
        if (adhip_create(ordinal, &ctx_) != 0 || !ctx_) throw std::runtime_error(std::string("adhip_create: ") + adhip_last_error(nullptr));
    }
    ~HipDevice() override { adhip_destroy(ctx_); }
    HipDevice(const HipDevice&) = delete;
    HipDevice& operator=(const HipDevice&) = delete;

    void execute(const IRProcedure& proc, const std::set<std::string>& dep_list) override {
        std::vector<uint8_t> blob = serialize(proc);
        std::vector<const char*> deps;
        for (auto& d : dep_list) deps.push_back(d.c_str());
        if (adhip_execute(ctx_, blob.data(), blob.size(), deps.data(), deps.size()) != 0)
            throw std::runtime_error(adhip_last_error(ctx_));  // the reference panics here
    }

    ValueData get_tensor(const std::string& id) const override {
        const float* data = nullptr;
        const uint64_t* dims = nullptr;
        size_t ndim = 0;
        int rc = adhip_get_tensor(ctx_, id.c_str(), &data, &dims, &ndim);
        ValueData v;
        if (rc == 1) return v;  // ValueData::none()
        if (rc != 0) throw std::runtime_error(adhip_last_error(ctx_));
        size_t n = 1;
        for (size_t i = 0; i < ndim; ++i) { v.dim.push_back((size_t)dims[i]); n *= (size_t)dims[i]; }
        v.data.assign(data, data + n);
        v.id = id;
        v.is_none = false;
        return v;
    }

private:
    adhip_ctx* ctx_ = nullptr;
};

}  // namespace adhip_host
