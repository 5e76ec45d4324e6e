"""The wire format of the IR program, fixed independently of its writers: one program that uses every command once
(tests/golden/make_wire_fixture.py) must serialise to the committed bytes (tests/golden/wire_every_command.bin, with
the CreateMat pointer fields zeroed) from the Python writer (adhip/ir.py) and from the C++ writer
(autodiff-ir-rust_amd/host/adhip_device.hpp, through tests/cxx/wire_fixture.cpp); the reader (csrc/ir.cpp) must accept
the stream and see every command.  A Rust writer (autodiff-ir-rust_amd/host/hip_device.rs) is held to the same bytes
by whoever builds it."""
import os
import struct
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))

from make_wire_fixture import KEEP, blanked, every_command_program  # noqa: E402

from adhip import ir as IR  # noqa: E402
from adhip.device import lower_describe  # noqa: E402

GOLDEN = os.path.join(ROOT, "tests", "golden", "wire_every_command.bin")


def test_python_writer_matches_the_committed_bytes():
    offs = []
    blob, _keep = IR.serialize(every_command_program(), offs)
    assert len(offs) == 3
    assert blanked(blob, offs) == open(GOLDEN, "rb").read()


def test_committed_bytes_have_the_documented_layout():
    """Spot checks written against the format description, not against a writer: magic, version, the first commands'
    tags and field order, and that every one of the 27 tags occurs."""
    b = open(GOLDEN, "rb").read()
    assert b[:4] == b"ADIR" and struct.unpack_from("<I", b, 4)[0] == 1
    pos = 8
    n = struct.unpack_from("<I", b, pos)[0]
    assert b[pos + 4:pos + 4 + n] == b"main"
    pos += 4 + n
    ncmds = struct.unpack_from("<I", b, pos)[0]
    assert ncmds == 34
    pos += 4
    assert b[pos] == 25                                   # Heading: str(cmt)
    n = struct.unpack_from("<I", b, pos + 1)[0]
    assert b[pos + 5:pos + 5 + n] == b"every command once"
    pos += 5 + n
    assert b[pos] == 0                                    # CreateMat: str(id) dims u64(pointer) u64(count)
    assert struct.unpack_from("<I", b, pos + 1)[0] == 1 and b[pos + 5:pos + 6] == b"a"
    assert struct.unpack_from("<IQQ", b, pos + 6) == (2, 2, 3)
    assert struct.unpack_from("<QQ", b, pos + 26) == (0, 6)
    tags = set()
    # a command's tag byte always follows the previous command's last field; walking the whole stream needs the
    # grammar, which the library's reader has: here only the presence of every tag value is checked
    for t in range(27):
        assert bytes([t]) in b, t
        tags.add(t)
    assert len(tags) == 27


def test_cxx_writer_matches_the_committed_bytes(tmp_path):
    exe = str(tmp_path / "wire_fixture")
    src = os.path.join(ROOT, "tests", "cxx", "wire_fixture.cpp")
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-Wall", "-o", exe, src])
    out = subprocess.run([exe], capture_output=True, check=True).stdout
    assert out == open(GOLDEN, "rb").read()


def test_reader_accepts_the_stream_and_sees_every_command(monkeypatch):
    monkeypatch.setenv("ADHIP_MERGE_SMALL", "0")   # one launch per kernel, so that each shows in the plan by name
    text = lower_describe(every_command_program(), set(KEEP))
    # the program lowers: every kept id has a home buffer, the loop and the branch are there
    for k in KEEP:
        assert f" home {k} " in text, k
    assert "while cond#" in text and "if neg#" in text and "else if is0#" in text
    assert "[reduce_row] kernel=k8_mx" in text and "[dot_naive]" in text


def test_fixture_without_the_max_command_is_the_rust_shim_fixture():
    """The Rust shim's enum has no Max: its unit test (host/hip_device.rs) edits the fixture -- 12 bytes before the
    final EX byte removed, command count 33 -- and expects its own output to equal that.  Here the Python writer
    confirms that the edited bytes are what the program without its Max command serialises to."""
    prog = every_command_program()
    assert isinstance(prog.main[-2], IR.Max)
    del prog.main[-2]
    offs = []
    blob, _keep = IR.serialize(prog, offs)
    want = bytearray(open(GOLDEN, "rb").read())
    cut = len(want) - 1 - 12
    assert want[cut] == 26
    del want[cut:cut + 12]
    want[16:20] = struct.pack("<I", 33)
    assert blanked(blob, offs) == bytes(want)
