"""The command-stream parser and the lowering under AddressSanitizer + UndefinedBehaviorSanitizer (host code only, no
GPU): tests/cxx/lowering_sanitized.cpp is built together with the library's sources and fed the programs of the
differential generators and the workloads, intact and damaged.  A sanitizer report fails the test."""
import glob
import os
import subprocess

import pytest

from adhip import ir as IR
from adhip import workloads as W
from adhip.core import ValueData
from adhip.device import Device
from oracle.interp import OracleDevice

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "autodiff-ir-rust_amd", "csrc")
DRIVER_SRC = os.path.join(ROOT, "tests", "cxx", "lowering_sanitized.cpp")
DRIVER = os.path.join(ROOT, "tests", "cxx", "lowering_sanitized")


class _Capture(Device):
    def execute(self, proc, deps):
        self.proc, self.deps = proc, deps

    def get_tensor(self, id):
        return ValueData.none()


def _build_driver():
    sources = sorted(glob.glob(os.path.join(CSRC, "*.cpp")))
    newest = max(os.path.getmtime(p) for p in sources + [DRIVER_SRC] + glob.glob(os.path.join(CSRC, "*.hpp")))
    if os.path.exists(DRIVER) and os.path.getmtime(DRIVER) >= newest:
        return
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    # host sanitizers only: each -fsanitize directly after -Xarch_host
    cmd = [hipcc, "--offload-arch=gfx950", "-std=c++17", "-O1", "-g", "-Xarch_host", "-fsanitize=address", "-Xarch_host",
           "-fsanitize=undefined", "-fno-omit-frame-pointer", "-o", DRIVER, DRIVER_SRC] + sources + ["-lhiprtc"]
    subprocess.check_call(cmd, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)


def _dump(directory, name, proc, keep):
    blob, keepalive = IR.serialize(proc)
    with open(os.path.join(directory, name + ".blob"), "wb") as f:
        f.write(blob)
    with open(os.path.join(directory, name + ".deps"), "w") as f:
        f.write("\n".join(sorted(keep)))
    del keepalive
    return os.path.join(directory, name)


def test_parser_and_lowering_under_host_sanitizers(tmp_path):
    from fuzz_control import (random_control_program, random_epilogue_program, random_grouped_products_program,
                              random_layered_program)
    from fuzz_programs import random_program
    if not os.path.exists(os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")):
        pytest.skip("no hipcc to build the sanitized driver with")
    _build_driver()
    bases = []
    for seed in range(24):
        dev = _Capture()
        try:
            random_program(dev, seed)
        except Exception:
            pass   # the capture device returns no values; the program was handed over before that matters
        if hasattr(dev, "proc"):
            bases.append(_dump(str(tmp_path), f"prog{seed}", dev.proc, dev.deps))
        proc, keep, _ = random_control_program(seed)
        bases.append(_dump(str(tmp_path), f"ctrl{seed}", proc, keep))
        for tag, gen in (("epi", random_epilogue_program), ("grp", random_grouped_products_program), ("lay", random_layered_program)):
            proc, keep = gen(seed)
            bases.append(_dump(str(tmp_path), f"{tag}{seed}", proc, keep))
    builders = {
        "encoder": lambda d: W.encoder_layer(d, 256, 256, 4, 512),
        "encoder_train": lambda d: W.encoder_train(d, 128, 128, 2, 256, iters=2),
        "mlp_train": lambda d: W.mlp_train(d, 256, (256, 256, 256, 128), 2),
        "manip_loop": lambda d: W.manip_loop(d, 2, 16, 32, 16, 8, 24, 4),
        "fused_elw": lambda d: W.fused_elw(d, 256, 1024),
        "reductions": lambda d: W.reductions(d, 1024, 512),
    }
    for name, build in builders.items():
        proc, deps = build(OracleDevice()).finish()
        bases.append(_dump(str(tmp_path), name, proc, deps))
    _run_driver(bases, 60)


def _run_driver(bases, mutations, extra_env=None):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1", UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    env.update(extra_env or {})
    res = subprocess.run([DRIVER, str(mutations)] + bases, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=900)
    tail = res.stdout[-4000:]
    assert res.returncode == 0, tail
    assert "runtime error" not in res.stdout and "AddressSanitizer" not in res.stdout, tail
    assert "intact:" in res.stdout and " 0 failed" in res.stdout, tail


@pytest.mark.parametrize("tighten", ["0", "2"])
def test_model_and_adversarial_programs_under_host_sanitizers(tighten, tmp_path):
    """The passes that model-shaped and oversized programs bring into play -- row chains, products of concatenated row
    blocks, wide references cut into parts, long expressions cut, the tightened lowering that follows a vector spill
    (forced with ADHIP_TIGHTEN) -- under the same sanitizers."""
    import adversarial_programs as A
    from fuzz_models import random_model_program
    if not os.path.exists(os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")):
        pytest.skip("no hipcc to build the sanitized driver with")
    _build_driver()
    bases = []
    for scale, seeds in ((1, range(16)), (16, [0, 3, 8, 27]), (48, [2])):
        for seed in seeds:
            dev = _Capture()
            try:
                random_model_program(dev, seed, scale)
            except AttributeError:
                pass   # the capture device returns no values; the program was handed over before that matters
            bases.append(_dump(str(tmp_path), f"model{scale}_{seed}", dev.proc, dev.deps))
    for name, made in (("wide", A.wide_concat(100)), ("pieces", A.one_buffer_pieces(200)), ("gathers", A.gathers(39)), ("rider", A.rider(19))):
        bases.append(_dump(str(tmp_path), name, made[0], made[1]))
    _run_driver(bases, 8, {"ADHIP_TIGHTEN": tighten} if tighten != "0" else None)
