"""Runs the text of a generated element-wise kernel on the host: the generator writes HIP C++ whose only device
specifics are qualifiers and a handful of builtins, so with those defined away (and blockIdx / threadIdx as globals
that a loop steps through the launch's grid) the same text compiles as ordinary C++.  What the host computes from the
text and the device computes from it can then be told apart: a wrong result here is a generator bug, a right one
clears the text.  Only kernels whose threads do not communicate (kind "elw": no LDS, no barriers, no wavefront
operations) can be run this way."""
import os
import re
import subprocess
import tempfile

import numpy as np

from adhip.device import lower_describe

CLANG = "/opt/rocm/lib/llvm/bin/clang++"

_SHIM = r'''
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
struct dim3_ { unsigned x, y, z; };
static dim3_ blockIdx, threadIdx;
#define __global__
#define __device__
#define __forceinline__ inline
#define __launch_bounds__(x)
#define __restrict__
#define __shared__ static
#define __builtin_amdgcn_update_dpp(a, b, c, d, e, f) (b)
#define __shfl_xor(v, m, w) (v)
#define __builtin_nontemporal_load(p) (*(p))
#define __builtin_nontemporal_store(v, p) (*(p) = (v))
'''


def generated_kernels(proc, keep):
    """(plan text, {entry: (kind, source)}) of the lowered program."""
    old = os.environ.get("ADHIP_DUMP_SOURCE")
    os.environ["ADHIP_DUMP_SOURCE"] = "1"
    try:
        text = lower_describe(proc, keep)
    finally:
        if old is None:
            del os.environ["ADHIP_DUMP_SOURCE"]
        else:
            os.environ["ADHIP_DUMP_SOURCE"] = old
    parts = re.split(r"// ===== (\S+) \[(\w+)\] =====\n", text)
    return parts[0], {parts[i]: (parts[i + 1], parts[i + 2]) for i in range(1, len(parts), 3)}


def launch_of(plan, entry):
    """(grid, block, [(id the buffer holds, plan buffer, elements)]) of the launch of kernel `entry`."""
    line = [l for l in plan.splitlines() if l.strip().startswith(f"launch {entry} ")][0]
    m = re.search(r"grid=\((\d+),(\d+),(\d+)\) block=(\d+)", line)
    elems = {int(b): int(n) for b, n in re.findall(r"#(\d+) \w+ \S+ elems=(\d+)", plan)}
    args = []
    for a in line.split("args:")[1].split():
        name, buf = a.rsplit("#", 1)
        for suffix in (".tmp", ".new"):
            if name.endswith(suffix):
                name = name[: -len(suffix)]
        args.append((name, int(buf), elems[int(buf)]))
    return [int(m.group(k)) for k in (1, 2, 3)], int(m.group(4)), args


def run_on_host(entry, source, grid, block, arrays, n_out):
    """Calls kernel `entry` of `source` once per thread of the launch with `arrays` (float32, one per buffer
    argument; the first n_out are outputs) and returns the outputs."""
    with tempfile.TemporaryDirectory() as work:
        decl, names = [], []
        for i, a in enumerate(arrays):
            np.asarray(a, np.float32).ravel().tofile(f"{work}/arg{i}.bin")
            decl.append(f'    float* p{i} = load("{work}/arg{i}.bin", {a.size});')
            names.append(f"p{i}")
        body = _SHIM + source + r'''
static float* load(const char* path, long n) {
    float* p = (float*)aligned_alloc(64, ((n * 4 + 63) / 64) * 64 + 64);
    FILE* f = fopen(path, "rb");
    if (!f || fread(p, 4, n, f) != (size_t)n) abort();
    fclose(f);
    return p;
}
int main() {
''' + "\n".join(decl) + "\n" + "\n".join(f"    memset(p{i}, 0xff, {arrays[i].size} * 4);" for i in range(n_out)) + f'''
    for (unsigned bz = 0; bz < {grid[2]}u; ++bz) for (unsigned by = 0; by < {grid[1]}u; ++by) for (unsigned bx = 0; bx < {grid[0]}u; ++bx)
        for (unsigned tx = 0; tx < {block}u; ++tx) {{
            blockIdx = {{bx, by, bz}};
            threadIdx = {{tx, 0, 0}};
            {entry}(nullptr, {", ".join(names)});
        }}
''' + "\n".join(f'    {{ FILE* f = fopen("{work}/out{i}.bin", "wb"); fwrite(p{i}, 4, {arrays[i].size}, f); fclose(f); }}'
                for i in range(n_out)) + "\n    return 0;\n}\n"
        open(f"{work}/main.cpp", "w").write(body)
        subprocess.check_call([CLANG, "-x", "c++", "-std=c++17", "-O1", "-ffp-contract=off", "-o", f"{work}/main", f"{work}/main.cpp"])
        subprocess.check_call([f"{work}/main"])
        return [np.fromfile(f"{work}/out{i}.bin", np.float32) for i in range(n_out)]
