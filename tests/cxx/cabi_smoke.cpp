// Drives the C ABI from C++ with no Python in between: the program a Rust `impl Device` would hand over.
//   c = dot(a, b); d = c + bias(broadcast);  for i in 0..3 { d += c }  ;  s = sum over columns of d^T
// Expected values are computed on the host in double precision.
#include <cmath>
#include <cstdio>

#include "../../autodiff-ir-rust_amd/host/adhip_device.hpp"

using namespace adhip_host;

static int fail(const char* what) { std::printf("FAIL: %s\n", what); return 1; }

int main() {
    const int M = 96, K = 80, N = 64;
    std::vector<float> a(M * K), b(K * N), bias(N);
    for (int i = 0; i < M * K; ++i) a[i] = (float)((i * 37 % 101) - 50) / 64.0f;
    for (int i = 0; i < K * N; ++i) b[i] = (float)((i * 53 % 97) - 48) / 32.0f;
    for (int i = 0; i < N; ++i) bias[i] = (float)i / 8.0f;

    IRProcedure p;
    p.push(create_mat("a", {(uint64_t)M, (uint64_t)K}, a));
    p.push(create_mat("b", {(uint64_t)K, (uint64_t)N}, b));
    p.push(create_mat("bias", {(uint64_t)N}, bias));
    p.push(binary(DotProduct, "a", "b", "c"));
    p.push(view("bias", {1, (uint64_t)N}, "bv"));
    p.push(broadcast("bv", 0, M, "bb"));
    p.push(binary(ElwAdd, "c", "bb", "d"));
    // counted loop in the shape ir_for emits: x = 0; cond = (x + -3) < 0; while cond { d += c; x += 1; cond = ... }
    p.push(create_mat("x", {1}, {0.0f}));
    p.push(create_constant("m3", -3.0f, {1}));
    p.push(binary(ElwAdd, "x", "m3", "t"));
    p.push(unary(LessZero, "t", "cond"));
    IRProcedure body;
    body.id = "a";
    body.push(op_eq(ElwAddEq, "d", "c"));
    body.push(create_constant("one", 1.0f, {1}));
    body.push(op_eq(ElwAddEq, "x", "one"));
    body.push(binary(ElwAdd, "x", "m3", "t"));
    body.push(unary(LessZero, "t", "cond"));
    p.push(while_("cond", body));
    p.push(permute("d", {1, 0}, "dt"));
    p.push(unary(Sum, "dt", "s"));  // [N, M] summed over its last dim -> [N]
    p.push(ex());

    HipDevice dev(0);
    dev.execute(p, {"d", "s", "x", "missing"});
    ValueData d = dev.get_tensor("d"), s = dev.get_tensor("s"), x = dev.get_tensor("x");
    if (d.is_none || s.is_none || x.is_none) return fail("kept tensor is none");
    if (!dev.get_tensor("missing").is_none) return fail("unknown id is not none");
    if (!dev.get_tensor("c").is_none) return fail("id that was not kept is not none");
    if (d.dim != std::vector<size_t>{(size_t)M, (size_t)N} || s.dim != std::vector<size_t>{(size_t)N}) return fail("dims");
    if (x.data[0] != 3.0f) return fail("loop counter");
    std::vector<double> colsum(N, 0.0);
    double worst = 0;
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            double acc = 0;
            for (int k = 0; k < K; ++k) acc += (double)a[i * K + k] * (double)b[k * N + j];
            double want = 4.0 * acc + bias[j];
            colsum[j] += want;
            worst = std::fmax(worst, std::fabs(want - d.data[i * N + j]) / std::fmax(1.0, std::fabs(want)));
        }
    if (worst > 1e-5 * std::sqrt((double)K)) { std::printf("d error %g\n", worst); return fail("d"); }
    for (int j = 0; j < N; ++j)
        if (std::fabs(colsum[j] - s.data[j]) > 1e-5 * std::sqrt((double)M) * std::fmax(1.0, std::fabs(colsum[j]))) return fail("s");
    // errors come back as exceptions with the library's message, never as a crash
    IRProcedure bad;
    bad.push(binary(ElwAdd, "nope", "nope", "y"));
    bad.push(ex());
    try {
        dev.execute(bad, {"y"});
        return fail("malformed program accepted");
    } catch (const std::runtime_error& e) {
        if (std::string(e.what()).find("used before it is defined") == std::string::npos) return fail("error message");
    }
    std::printf("cabi_smoke ok (max rel err %.3g)\n", worst);
    return 0;
}
