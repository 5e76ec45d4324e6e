// Builds the "every command once" program (the one tests/golden/make_wire_fixture.py builds in Python) through the
// C++ host mirror, serialises it, sets the CreateMat pointer fields to zero and writes the bytes to stdout.
// tests/test_wire_format.py compares them with tests/golden/wire_every_command.bin.  No GPU, no library call.
#include <cstdio>

#include "../../autodiff-ir-rust_amd/host/adhip_device.hpp"

using namespace adhip_host;

int main() {
    IRProcedure body;
    body.id = "loop";
    body.push(op_eq(ElwAddEq, "k", "m1"));
    body.push(unary(MoreZero, "k", "cond"));
    IRProcedure arm0;
    arm0.id = "arm0";
    arm0.push(op_eq(ElwMultiplyEq, "e", "c"));
    IRProcedure arm1;
    arm1.id = "arm1";
    arm1.push(create_constant("two", 2.0f, {2, 3}));
    arm1.push(op_eq(ElwAddEq, "e", "two"));
    IRProcedure other;
    other.id = "other";
    other.push(heading("neither predicate held"));

    IRProcedure p;
    p.push(heading("every command once"));
    p.push(create_mat("a", {2, 3}, {1, 2, 3, 4, 5, 6}));
    p.push(create_mat("b", {3, 2}, {1, 0, -1, 2, 0.5f, 4}));
    p.push(create_constant("c", 0.5f, {2, 3}));
    p.push(binary(ElwMultiply, "a", "c", "d"));
    p.push(binary(ElwAdd, "a", "d", "e"));
    p.push(op_eq(ElwMultiplyEq, "e", "c"));
    p.push(op_eq(ElwAddEq, "e", "a"));
    p.push(unary(EqualZero, "e", "f"));
    p.push(unary(MoreZero, "e", "g"));
    p.push(unary(LessZero, "e", "h"));
    p.push(unary(Sum, "e", "s"));
    p.push(binary(DotProduct, "a", "b", "p"));
    p.push(view("a", {3, 2}, "v"));
    p.push(index("a", 1, 0, "i"));
    p.push(concat("a", "a", 0, "cc"));
    p.push(permute("a", {1, 0}, "t"));
    p.push(view("s", {2, 1}, "s1"));
    p.push(broadcast("s1", 1, 3, "sb"));
    p.push(unary(Contigious, "t", "tc"));
    p.push(unary(Exp2, "a", "x2"));
    p.push(unary(Log2, "x2", "l2"));
    p.push(unary(Sin, "a", "sn"));
    p.push(unary(Recip, "x2", "rc"));
    p.push(unary(Sqrt, "x2", "sq"));
    p.push(create_mat("k", {1}, {2}));
    p.push(create_constant("m1", -1.0f, {1}));
    p.push(unary(MoreZero, "k", "cond"));
    p.push(while_("cond", body));
    p.push(unary(EqualZero, "k", "is0"));
    p.push(unary(LessZero, "k", "neg"));
    p.push(if_arms({{"neg", arm0}, {"is0", arm1}}, &other));
    p.push(unary(Max, "e", "mx"));
    p.push(ex());

    std::vector<size_t> offsets;
    std::vector<uint8_t> blob = serialize(p, &offsets);
    for (size_t o : offsets)
        for (int i = 0; i < 8; ++i) blob[o + i] = 0;
    return fwrite(blob.data(), 1, blob.size(), stdout) == blob.size() ? 0 : 1;
}
