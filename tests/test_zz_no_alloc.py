"""adhip_program_enqueue_noalloc against adhip_program_enqueue, through the C ABI.

The same resident program is run twice from the same uploaded state: once with its temporaries in its own allocations
(`enqueue`), once with them in the library's static device array (`enqueue_noalloc`).  Both run the same kernels in the
same order, so every kept tensor must come back bit for bit equal.  Two programs in a row, the second smaller than
the first (it finds the first one's data in the array), then a program with device-side control-flow flags, then one
whose temporaries exceed the array, which must be refused with an error that names the limit."""
import numpy as np
import pytest

from adhip import workloads as W
from parity import assert_exact

pytestmark = pytest.mark.gpu


def _both_ways(dev, builder):
    wl = builder(dev)
    proc, deps = wl.finish()
    prog = dev.compile(proc, deps)
    text = prog.describe()
    out = []
    for how in ("enqueue", "enqueue_noalloc"):
        prog.upload()
        getattr(prog, how)()
        prog.sync()
        prog.readback()
        out.append({k: dev.get_tensor(v.id) for k, v in wl.outputs.items()})
    prog.close()
    return out[0], out[1], text


def _compare(plain, static, what):
    assert set(plain) == set(static)
    for k in plain:
        assert not static[k].is_none and static[k].dim == plain[k].dim, f"{what}: {k}"
        assert_exact(static[k].data, plain[k].data, f"{what}: {k}")


def test_noalloc_matches_enqueue_on_two_programs_in_a_row(hip_device):
    print("[case] noalloc: reductions 2048x1024, then 256x512", flush=True)
    plain, static, text = _both_ways(hip_device, lambda d: W.reductions(d, 2048, 1024, seed=21))
    assert " temp " in text, "the program was expected to use temporaries"
    _compare(plain, static, "reductions 2048x1024")
    x = W.reductions(hip_device, 2048, 1024, seed=21).inputs["x"].astype(np.float64)
    np.testing.assert_allclose(static["s1"].data, x.sum(0), rtol=0, atol=1e-5 * np.sqrt(2048) * float(np.abs(x).sum(0).max()))
    plain, static, _ = _both_ways(hip_device, lambda d: W.reductions(d, 256, 512, seed=22))
    _compare(plain, static, "reductions 256x512")


def test_noalloc_with_split_products_and_training_loop(hip_device):
    print("[case] noalloc: mlp_train 256, (512,256,128,64), 3 iterations", flush=True)
    plain, static, text = _both_ways(hip_device, lambda d: W.mlp_train(d, 256, (512, 256, 128, 64), 3, seed=23))
    assert " temp " in text
    _compare(plain, static, "mlp_train")


def test_noalloc_with_device_predicated_loop(hip_device):
    print("[case] noalloc: manip_loop with device-side flags", flush=True)
    plain, static, text = _both_ways(hip_device, lambda d: W.manip_loop(d, 2, 16, 32, 16, 8, 24, 6, seed=24))
    assert "device-predicated" in text
    _compare(plain, static, "manip_loop")


def test_noalloc_with_row_chains_and_grouped_products(hip_device):
    print("[case] noalloc: encoder layer 128x64, 4 heads (row chains, grouped and split products, layered launches)", flush=True)
    plain, static, text = _both_ways(hip_device, lambda d: W.encoder_layer(d, 128, 64, 4, 128, seed=26))
    assert " temp " in text and "[rowchain]" in text
    _compare(plain, static, "encoder_layer")


def test_noalloc_refuses_programs_beyond_the_static_area(hip_device):
    print("[case] noalloc: program with 64 MiB of temporaries", flush=True)
    wl = W.mlp_train(hip_device, 2048, (2048, 2048, 2048, 512), 1, seed=25)
    proc, deps = wl.finish()
    prog = hip_device.compile(proc, deps)
    prog.upload()
    with pytest.raises(RuntimeError, match=r"needs \d+ bytes of scratch memory, the static area holds 33554432"):
        prog.enqueue_noalloc()
    prog.enqueue()      # the ordinary entry point still runs it
    prog.sync()
    prog.close()
