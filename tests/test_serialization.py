"""Object serialization of the three LUT layers (`.bb_net` object bytes; reference layout include/bb/Object.h:145-179,
StochasticLutN.h:170-223, DifferentiableLutN.h:266-334, BinaryLutN.h:481-519), CPU only.

The host classes are driven through tests/cpp/object_tool.  Pins: bytes written by the reference's own DumpObject
(tests/golden/objects.npz) are reproduced bit for bit from the same contents, survive load -> dump unchanged and come
apart into the contents they were made from; where oracle/_ref is built, fresh objects written here are read by the
reference's LoadObject and the two writers are compared on new contents; damaged objects are rejected."""
import os
import struct
import subprocess

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
TOOL = os.path.join(HERE, "cpp", "object_tool")
GOLD = np.load(os.path.join(HERE, "golden", "objects.npz"))
KIND_NAMES = {v: k for k, v in oracle.LUT_OBJECT_KINDS.items()}


@pytest.fixture(scope="module", autouse=True)
def built_tool():
    if not os.path.exists(TOOL):
        from binarybrain_amd.build import build_cpp_tests
        build_cpp_tests()


def tool(*args, check=True):
    p = subprocess.run([TOOL] + [str(a) for a in args], capture_output=True, text=True, timeout=60)
    if check:
        assert p.returncode == 0, p.stderr
    return p


def write_contents(prefix, idx, params, mean, var):
    idx.astype(np.int32).tofile(prefix + ".idx")
    params.tofile(prefix + ".params")
    mean.astype(np.float32).tofile(prefix + ".mean")
    var.astype(np.float32).tofile(prefix + ".var")


def read_contents(prefix, kind, O):
    out = {"idx": np.fromfile(prefix + ".idx", np.int32).reshape(O, 6)}
    out["params"] = np.fromfile(prefix + ".params", np.int32).reshape(O, 2) if kind == 2 else np.fromfile(prefix + ".params", np.float32).reshape(O, 64)
    if kind == 1:
        out["mean"] = np.fromfile(prefix + ".mean", np.float32); out["var"] = np.fromfile(prefix + ".var", np.float32)
    return out


def gold_case(k):
    q = "o%d_" % k
    kind, bit, I, O, flags = [int(v) for v in GOLD[q + "desc"]]
    return dict(kind=kind, bit=bit, I=I, O=O, flags=flags, name=GOLD[q + "name"].tobytes().decode(), idx=GOLD[q + "idx"],
                params=GOLD[q + "params"], mean=GOLD[q + "mean"], var=GOLD[q + "var"], data=GOLD[q + "bytes"].tobytes())


@pytest.mark.parametrize("k", range(int(GOLD["object_count"][0])))
def test_same_contents_give_the_reference_bytes(tmp_path, k):
    c = gold_case(k)
    prefix = str(tmp_path / "in")
    write_contents(prefix, c["idx"], c["params"], c["mean"], c["var"])
    out = str(tmp_path / "made.bb_net")
    tool("make", c["kind"], c["bit"], c["I"], c["O"], c["flags"], c["name"] or "-", prefix, out)
    assert open(out, "rb").read() == c["data"]


@pytest.mark.parametrize("k", range(int(GOLD["object_count"][0])))
def test_reference_bytes_load_and_survive_a_round_trip(tmp_path, k):
    c = gold_case(k)
    src = str(tmp_path / "ref.bb_net"); open(src, "wb").write(c["data"])
    again = str(tmp_path / "again.bb_net")
    tool("roundtrip", c["kind"], c["bit"], src, again)
    assert open(again, "rb").read() == c["data"]
    prefix = str(tmp_path / "out")
    I, O, name = tool("describe", c["kind"], c["bit"], src, prefix).stdout.split()
    assert (int(I), int(O)) == (c["I"], c["O"])
    assert name == (c["name"] or {0: "StochasticLut6", 1: "DifferentiableLut6", 2: "BinaryLut6"}[c["kind"]])
    got = read_contents(prefix, c["kind"], c["O"])
    assert np.array_equal(got["idx"], c["idx"]) and np.array_equal(got["params"], c["params"])
    if c["kind"] == 1:
        assert np.array_equal(got["mean"], c["mean"]) and np.array_equal(got["var"], c["var"])


def test_header_layout():
    # "BB_OBJ", int64 1, uint64 length, name: the part of the layout that does not depend on a layer (Object.h:145-157)
    data = gold_case(0)["data"]
    assert data[:6] == b"BB_OBJ" and struct.unpack("<q", data[6:14])[0] == 1
    n = struct.unpack("<Q", data[14:22])[0]
    assert data[22:22 + n] == b"StochasticLut6_fp32_fp32"
    names = [gold_case(k)["data"][22:22 + struct.unpack("<Q", gold_case(k)["data"][14:22])[0]].decode() for k in range(int(GOLD["object_count"][0]))]
    assert names == ["StochasticLut6_fp32_fp32", "StochasticLut6_bit_fp32", "DifferentiableLut6_fp32_fp32", "DifferentiableLut6_bit_fp32",
                     "DifferentiableLut6_fp32_fp32", "BinaryLut6_bit_fp32"]


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built")
@pytest.mark.parametrize("kind,bit,flags", [(0, 0, 0), (0, 1, 3), (1, 0, 7), (1, 1, 5), (2, 1, 0)])
def test_objects_written_here_load_in_the_reference(tmp_path, kind, bit, flags):
    rng = np.random.default_rng(100 + kind * 10 + bit)
    I, O = 40, 13
    idx = np.stack([rng.choice(I, 6, replace=False) for _ in range(O)]).astype(np.int32)
    params = rng.integers(-2**31, 2**31, (O, 2)).astype(np.int32) if kind == 2 else rng.standard_normal((O, 64)).astype(np.float32)
    mean = rng.standard_normal(O).astype(np.float32); var = (rng.random(O) + 0.1).astype(np.float32)
    prefix = str(tmp_path / "in")
    write_contents(prefix, idx, params, mean, var)
    out = str(tmp_path / "made.bb_net")
    tool("make", kind, bit, I, O, flags, "fresh", prefix, out)
    data = open(out, "rb").read()
    got = oracle.ref_load_lut_object(KIND_NAMES[kind], bit, data, O)
    assert got["input_nodes"] == I and got["name"] == "fresh"
    assert np.array_equal(got["idx"], idx) and np.array_equal(got["params"], params)
    if kind == 1:
        assert np.array_equal(got["mean"], mean) and np.array_equal(got["var"], var)
    # and the reference's writer, given the same contents, produces the same bytes
    assert oracle.ref_dump_lut_object(KIND_NAMES[kind], bit, I, idx, params, mean, var, flags, (0.75, 0.4, 0.6), "fresh") == data


def test_damaged_objects_are_rejected(tmp_path):
    c = gold_case(0)
    data = bytearray(c["data"])

    def rejected(blob, kind=c["kind"], bit=c["bit"]):
        src = str(tmp_path / "bad.bb_net"); open(src, "wb").write(bytes(blob))
        p = tool("roundtrip", kind, bit, src, str(tmp_path / "bad_out.bb_net"), check=False)
        return p.returncode != 0 and "rejected" in p.stderr

    assert rejected(data[: len(data) // 2])                    # truncated
    assert rejected(b"XX" + data[2:])                          # not an object
    assert rejected(data, kind=1)                              # another class
    assert rejected(data, kind=0, bit=1)                       # another element type
    # wiring that points outside the input nodes must not reach a kernel: the first table entry follows the table's own
    # header, found here through its value
    first = struct.pack("<i", int(c["idx"][0, 0])) + struct.pack("<i", int(c["idx"][0, 1]))
    at = bytes(data).find(first)
    assert at > 0
    bad = bytearray(data); bad[at:at + 4] = struct.pack("<i", c["I"] + 5)
    assert rejected(bad)
    bad = bytearray(data); bad[at:at + 4] = struct.pack("<i", -1)
    assert rejected(bad)
