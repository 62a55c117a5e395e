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


# ----------------------------------------------------------------------------------------------
#  container objects: Convolution2d (include/bb/Convolution2d.h:355-409), Sequential (Sequential.h:239-288),
#  ConvolutionIm2Col (:492-563), ConvolutionCol2Im (:334-367)
# ----------------------------------------------------------------------------------------------
CONTAINERS = np.load(os.path.join(HERE, "golden", "container_objects.npz"))
CONTAINER_NAMES = {0: "Convolution2d_fp32_fp32", 1: "Convolution2d_fp32_fp32", 2: "Sequential", 3: "ConvolutionIm2Col_fp32_fp32",
                   4: "ConvolutionCol2Im_fp32_fp32"}


def container_shapes(kind, c, h, w, fh, fw, ys, xs, same, o1, o2):
    """(input nodes, output nodes) that the loaded object must report"""
    oh = (h + ys - 1) // ys if same else ((h - fh + 1) + (ys - 1)) // ys
    ow = (w + xs - 1) // xs if same else ((w - fw + 1) + (xs - 1)) // xs
    if kind in (0, 1):
        return c * h * w, o2 * oh * ow
    if kind == 2:
        return c * fh * fw, o2
    if kind == 3:
        return c * h * w, c * fh * fw
    return o2, o2 * h * w


@pytest.mark.parametrize("k", range(int(CONTAINERS["count"][0])))
def test_reference_container_objects_load_and_survive_a_round_trip(tmp_path, k):
    """Bytes written by the reference are rebuilt here from the type names they carry (bb::Object_Load), report the shapes and the
    name they were made with, and are written again unchanged — the layers inside (wiring, tables, statistics) included."""
    p = "c%d_" % k
    kind, c, h, w, fh, fw, ys, xs, same, o1, o2, seed = [int(v) for v in CONTAINERS[p + "args"]]
    data = CONTAINERS[p + "bytes"].tobytes()
    name = CONTAINERS[p + "name"].tobytes().decode()
    src, dst = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    open(src, "wb").write(data)
    out = tool("reload", src, dst).stdout.split()
    assert out[0] == CONTAINER_NAMES[kind]
    # (the convolution wrapper does not store a name of its own; the other objects do)
    assert out[1] == (name if (name and kind in (2, 3, 4)) else CONTAINER_NAMES[kind].split("_")[0])
    assert (int(out[3]), int(out[5])) == container_shapes(kind, c, h, w, fh, fw, ys, xs, same, o1, o2)
    assert open(dst, "rb").read() == data


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref is not built")
def test_container_objects_against_the_reference(tmp_path):
    """Fresh objects from the reference (new geometry and seeds each): loaded and re-written here they keep their bytes, and the
    reference loads what was written here — rebuilding it from the type names — and writes the same bytes again."""
    rng = np.random.default_rng(2718)
    borders = ["constant", "reflect", "reflect_101", "replicate", "wrap"]
    for trial in range(12):
        kind = trial % 5
        c, fh, fw = int(rng.integers(1, 5)), int(rng.integers(1, 4)), int(rng.integers(1, 4))
        h, w = int(rng.integers(fh + 1, 12)), int(rng.integers(fw + 1, 12))
        ys, xs, same = int(rng.integers(1, 3)), int(rng.integers(1, 3)), bool(rng.integers(0, 2))
        o1, o2, seed = int(rng.integers(6, 40)), int(rng.integers(1, 20)), int(rng.integers(1, 1000))
        data = oracle.ref_dump_container_object(kind, c, h, w, fh, fw, ys, xs, same, borders[trial % 5], o1, o2, seed, "n%d" % trial)
        src, dst = str(tmp_path / ("in%d.bin" % trial)), str(tmp_path / ("out%d.bin" % trial))
        open(src, "wb").write(data.tobytes())
        tool("reload", src, dst)
        mine = np.frombuffer(open(dst, "rb").read(), np.uint8)
        assert np.array_equal(mine, data), (trial, kind)
        back = oracle.ref_reload_container_object(mine)
        assert back is not None and np.array_equal(back, data), (trial, kind)


def test_damaged_container_objects_are_rejected(tmp_path):
    data = bytearray(CONTAINERS["c2_bytes"].tobytes())          # a convolution over a list of two layers
    for cut in (20, len(data) // 2, len(data) - 3):
        p = str(tmp_path / ("cut%d.bin" % cut))
        open(p, "wb").write(bytes(data[:cut]))
        assert tool("reload", p, str(tmp_path / "x.bin"), check=False).returncode != 0
    # a layer type that is not known here inside a known container
    bad = bytes(data).replace(b"DifferentiableLut6_fp32_fp32", b"DifferentiableLut9_fp32_fp32")
    p = str(tmp_path / "unknown.bin")
    open(p, "wb").write(bad)
    assert tool("reload", p, str(tmp_path / "x.bin"), check=False).returncode != 0


# ----------------------------------------------------------------------------------------------
#  StochasticBatchNormalization (include/bb/StochasticBatchNormalization.h:143-183): the objects that the reference's class wrote
#  after a training pass (tests/golden/bn.npz), running statistics included
# ----------------------------------------------------------------------------------------------
BN = np.load(os.path.join(HERE, "golden", "bn.npz"))


@pytest.mark.parametrize("k", range(int(BN["count"][0])))
def test_reference_normalisation_objects_load_and_survive_a_round_trip(tmp_path, k):
    p = "b%d_" % k
    data = BN[p + "object"].tobytes()
    name = BN[p + "name"].tobytes().decode()
    nodes = int(BN[p + "geom"][0])
    src, dst = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    open(src, "wb").write(data)
    out = tool("reload", src, dst).stdout.split()
    assert out[0] == "StochasticBatchNormalization_fp32"
    assert out[1] == (name if name else "StochasticBatchNormalization")
    assert (int(out[3]), int(out[5])) == (nodes, nodes)
    assert open(dst, "rb").read() == data
    # the running statistics sit at the end of the object: two typed tensors of `nodes` floats each
    tail = np.frombuffer(data[-4 * nodes:], np.float32)
    assert np.array_equal(tail, BN[p + "running_var"])


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref is not built")
def test_normalisation_objects_against_the_reference(tmp_path):
    rng = np.random.default_rng(99)
    for trial in range(4):
        nodes, frames = int(rng.integers(1, 40)), int(rng.integers(2, 90))
        x = rng.random((nodes, frames)).astype(np.float32)
        r = oracle.ref_stochastic_bn(x, rng.standard_normal(nodes), rng.random(nodes) + 0.5, 0.1 + 0.1 * trial, 0.5, 0.8,
                                     train=True, name="bn%d" % trial if trial % 2 else "", want_object=True)
        src, dst = str(tmp_path / ("in%d.bin" % trial)), str(tmp_path / ("out%d.bin" % trial))
        open(src, "wb").write(r["object"].tobytes())
        tool("reload", src, dst)
        mine = np.frombuffer(open(dst, "rb").read(), np.uint8)
        assert np.array_equal(mine, r["object"]), trial
        back = oracle.ref_reload_container_object(mine)
        assert back is not None and np.array_equal(back, r["object"]), trial


# ----------------------------------------------------------------------------------------------
#  MaxLut (include/bb/MaxLut.h:428-465): objects written by the reference's class, fp32 and bit (tests/golden/maxlut.npz)
# ----------------------------------------------------------------------------------------------
MAXLUT = np.load(os.path.join(HERE, "golden", "maxlut.npz"))


@pytest.mark.parametrize("k", range(int(MAXLUT["count"][0])))
def test_reference_max_lut_objects_load_and_survive_a_round_trip(tmp_path, k):
    p = "m%d_" % k
    n, I, O, F, bin_out = [int(v) for v in MAXLUT[p + "geom"]]
    name = MAXLUT[p + "name"].tobytes().decode()
    for key, type_name in (("object", "MaxLut_fp32_fp32"), ("object_bit", "MaxLut_bit_fp32")):
        data = MAXLUT[p + key].tobytes()
        src, dst = str(tmp_path / (key + ".in")), str(tmp_path / (key + ".out"))
        open(src, "wb").write(data)
        out = tool("reload", src, dst).stdout.split()
        assert out[0] == type_name and out[1] == (name if name else "MaxLut")
        assert (int(out[3]), int(out[5])) == (I, O)
        assert open(dst, "rb").read() == data
        # the wiring sits at the end of the object
        assert np.array_equal(np.frombuffer(data[-4 * O * n:], np.int32).reshape(O, n), MAXLUT[p + "idx"])


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref is not built")
def test_max_lut_objects_against_the_reference(tmp_path):
    rng = np.random.default_rng(123)
    for trial in range(4):
        n, I, O, F = int(rng.integers(1, 9)), int(rng.integers(8, 60)), int(rng.integers(1, 30)), 5
        idx = rng.integers(0, I, (O, n)).astype(np.int32)
        bit = bool(trial % 2)
        x = np.zeros((I, 1), np.int32) if bit else np.zeros((I, F), np.float32)
        _, _, obj = oracle.ref_max_lut(x, idx, I, F, bit=bit, binarize_output=bool(trial // 2), name="m%d" % trial, want_object=True)
        src, dst = str(tmp_path / ("in%d.bin" % trial)), str(tmp_path / ("out%d.bin" % trial))
        open(src, "wb").write(obj.tobytes())
        tool("reload", src, dst)
        mine = np.frombuffer(open(dst, "rb").read(), np.uint8)
        assert np.array_equal(mine, obj), trial
        # (the reference's own loader does not know the type name MaxLut, include/bb/ObjectLoader.h, so there is no trip back
        # through it; equal bytes are what its LoadObject would read)
        assert oracle.ref_reload_container_object(mine) is None


# ----------------------------------------------------------------------------------------------
#  AverageLut (include/bb/AverageLut.h:412-458): the same layout as MaxLut (tests/golden/average_lut_objects.npz)
# ----------------------------------------------------------------------------------------------
AVERAGE = np.load(os.path.join(HERE, "golden", "average_lut_objects.npz"))


@pytest.mark.parametrize("k", range(int(AVERAGE["count"][0])))
def test_reference_average_lut_objects_load_and_survive_a_round_trip(tmp_path, k):
    p = "a%d_" % k
    n, I, O, bit, bin_in, bin_out = [int(v) for v in AVERAGE[p + "args"]]
    name = AVERAGE[p + "name"].tobytes().decode()
    data = AVERAGE[p + "bytes"].tobytes()
    src, dst = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    open(src, "wb").write(data)
    out = tool("reload", src, dst).stdout.split()
    assert out[0] == ("AverageLut_bit_fp32" if bit else "AverageLut_fp32_fp32") and out[1] == (name if name else "AverageLut")
    assert (int(out[3]), int(out[5])) == (I, O)
    assert open(dst, "rb").read() == data
    assert np.array_equal(np.frombuffer(data[-4 * O * n:], np.int32).reshape(O, n), AVERAGE[p + "idx"])
    # (as for MaxLut, the reference's own loader does not list this type name: equal bytes are what its LoadObject would read)


# ----------------------------------------------------------------------------------------------
#  Reduce (include/bb/Reduce.h:287-317): objects written by the reference's class, fp32 and bit (tests/golden/reduce_mse.npz)
# ----------------------------------------------------------------------------------------------
REDUCE = np.load(os.path.join(HERE, "golden", "reduce_mse.npz"))


@pytest.mark.parametrize("k", range(int(REDUCE["reduce_count"][0])))
def test_reference_reduce_objects_load_and_survive_a_round_trip(tmp_path, k):
    p = "r%d_" % k
    I, O, F, integ = [int(v) for v in REDUCE[p + "geom"]]
    name = REDUCE[p + "name"].tobytes().decode()
    for key, type_name in (("object", "Reduce_fp32_fp32"), ("object_bit", "Reduce_bit_fp32")):
        data = REDUCE[p + key].tobytes()
        src, dst = str(tmp_path / (key + ".in")), str(tmp_path / (key + ".out"))
        open(src, "wb").write(data)
        out = tool("reload", src, dst).stdout.split()
        assert out[0] == type_name and out[1] == (name if name else "Reduce")
        assert (int(out[3]), int(out[5])) == (I, O)
        assert open(dst, "rb").read() == data
        if oracle.have_ref():                           # the reference's loader lists this type: it reads what was written here
            back = oracle.ref_reload_container_object(np.frombuffer(open(dst, "rb").read(), np.uint8))
            assert back is not None and back.tobytes() == data


# ----------------------------------------------------------------------------------------------
#  RealToBinary, BinaryToReal, Binarize, HardTanh, BinaryModulation (include/bb/RealToBinary.h:501-548, BinaryToReal.h:352-380,
#  Binarize.h:286-308, HardTanh.h:262-289, BinaryModulation.h:370-420): objects written by the reference's classes
#  (tests/golden/modulation.npz) load here, report their shapes and names, and are written again byte for byte; the reference's
#  loader, which lists all of these type names, reads what was written here and writes the same bytes.
# ----------------------------------------------------------------------------------------------
MODULATION = np.load(os.path.join(HERE, "golden", "modulation.npz"))


def _reload_and_compare(tmp_path, data, type_name, name, default_name, in_nodes, out_nodes, through_reference=True):
    src, dst = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    open(src, "wb").write(data)
    out = tool("reload", src, dst).stdout.split()
    assert out[0] == type_name and out[1] == (name if name else default_name)
    assert (int(out[3]), int(out[5])) == (in_nodes, out_nodes)
    assert open(dst, "rb").read() == data
    if through_reference and oracle.have_ref():
        back = oracle.ref_reload_container_object(np.frombuffer(open(dst, "rb").read(), np.uint8))
        assert back is not None and back.tobytes() == data


@pytest.mark.parametrize("k", range(int(MODULATION["r2b_count"][0])))
def test_reference_real_to_binary_objects(tmp_path, k):
    q = "m%d_" % k
    d, p, F, fm, dm, _ = [int(v) for v in MODULATION[q + "geom"]]
    name = MODULATION[q + "name"].tobytes().decode()
    for key, type_name in (("object", "RealToBinary_fp32_fp32"), ("object_bit", "RealToBinary_bit_fp32")):
        _reload_and_compare(tmp_path, MODULATION[q + key].tobytes(), type_name, name, "RealToBinary", d * p, d * dm * p)


@pytest.mark.parametrize("k", range(int(MODULATION["b2r_count"][0])))
def test_reference_binary_to_real_objects(tmp_path, k):
    q = "b%d_" % k
    I, O, Fy, fm = [int(v) for v in MODULATION[q + "geom"]]
    name = MODULATION[q + "name"].tobytes().decode()
    for key, type_name in (("object", "BinaryToReal_fp32_fp32"), ("object_bit", "BinaryToReal_bit_fp32")):
        _reload_and_compare(tmp_path, MODULATION[q + key].tobytes(), type_name, name, "BinaryToReal", I, O)


@pytest.mark.parametrize("k", range(int(MODULATION["act_count"][0])))
def test_reference_activation_objects(tmp_path, k):
    q = "a%d_" % k
    kind = bytes(MODULATION[q + "kind"]).decode()
    nodes, F = [int(v) for v in MODULATION[q + "geom"]]
    name = MODULATION[q + "name"].tobytes().decode()
    model = "Binarize" if kind == "binarize" else "HardTanh"
    for key, suffix in (("object", "_fp32_fp32"), ("object_bit", "_bit_fp32")):
        _reload_and_compare(tmp_path, MODULATION[q + key].tobytes(), model + suffix, name, model, nodes, nodes)


@pytest.mark.parametrize("k", range(int(MODULATION["mod_count"][0])))
def test_reference_binary_modulation_objects(tmp_path, k):
    q = "n%d_" % k
    bit, I, o1, o2, tm, im, dm, seed, infer = [int(v) for v in MODULATION[q + "args"]]
    name = MODULATION[q + "name"].tobytes().decode()
    _reload_and_compare(tmp_path, MODULATION[q + "object"].tobytes(), "BinaryModulation_bit_fp32" if bit else "BinaryModulation_fp32_fp32",
                        name, "BinaryModulation", I, o2)


@pytest.mark.parametrize("k", range(int(MODULATION["discrete_count"][0])))
def test_reference_discrete_lut_objects(tmp_path, k):
    """DifferentiableLutDiscrete6 = StochasticLut6 -> StochasticBatchNormalization -> HardTanh (include/bb/DifferentiableLutDiscreteN.h:392-425)"""
    q = "d%d_" % k
    bit, I, O, seed, bn, saving = [int(v) for v in MODULATION[q + "args"]]
    name = MODULATION[q + "name"].tobytes().decode()
    _reload_and_compare(tmp_path, MODULATION[q + "object"].tobytes(), "DifferentiableLutDiscrete6_bit_fp32" if bit else "DifferentiableLutDiscrete6_fp32_fp32",
                        name, "DifferentiableLutDiscrete6", I, O, through_reference=False)
    # (no trip back through the reference's Object_Load: it builds this type with an empty output shape, which its own StochasticLutN
    # constructor refuses with an assertion that ends the process — include/bb/StochasticLutN.h:78; equal bytes are what LoadObject reads)


def test_truncated_modulation_objects_are_rejected(tmp_path):
    data = MODULATION["n1_object"].tobytes()
    for cut in (len(data) // 3, len(data) - 9):
        src = str(tmp_path / ("cut%d.bin" % cut))
        open(src, "wb").write(data[:cut])
        res = subprocess.run([TOOL, "reload", src, str(tmp_path / "out.bin")], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        assert res.returncode != 0


# ----------------------------------------------------------------------------------------------
#  MaxPooling, UpSampling (include/bb/MaxPooling.h:694-735, UpSampling.h:357-383): objects written by the reference's classes
#  (tests/golden/pooling.npz), fp32 and packed, load here and are written again byte for byte; the reference's loader reads them back.
# ----------------------------------------------------------------------------------------------
POOLING = np.load(os.path.join(HERE, "golden", "pooling.npz"))


@pytest.mark.parametrize("k", range(int(POOLING["pool_count"][0])))
def test_reference_max_pooling_objects(tmp_path, k):
    q = "p%d_" % k
    c, h, w, fh, fw, F = [int(v) for v in POOLING[q + "geom"]]
    name = POOLING[q + "name"].tobytes().decode()
    out_nodes = c * ((h + fh - 1) // fh) * ((w + fw - 1) // fw)
    for key, type_name in (("object", "MaxPooling_fp32_fp32"), ("object_bit", "MaxPooling_bit_fp32")):
        _reload_and_compare(tmp_path, POOLING[q + key].tobytes(), type_name, name, "MaxPooling", c * h * w, out_nodes)


@pytest.mark.parametrize("k", range(int(POOLING["up_count"][0])))
def test_reference_up_sampling_objects(tmp_path, k):
    q = "u%d_" % k
    c, h, w, fh, fw, fill, F = [int(v) for v in POOLING[q + "geom"]]
    name = POOLING[q + "name"].tobytes().decode()
    for key, type_name in (("object", "UpSampling_fp32_fp32"), ("object_bit", "UpSampling_bit_fp32")):
        _reload_and_compare(tmp_path, POOLING[q + key].tobytes(), type_name, name, "UpSampling", c * h * w, c * h * fh * w * fw)


#  Shuffle (include/bb/Shuffle.h:270-301): version, Model part, host_only, the two shapes, the unit
@pytest.mark.parametrize("k", range(int(POOLING["shuffle_count"][0])))
def test_reference_shuffle_objects(tmp_path, k):
    q = "s%d_" % k
    nodes, unit, F = [int(v) for v in POOLING[q + "geom"]]
    name = POOLING[q + "name"].tobytes().decode()
    _reload_and_compare(tmp_path, POOLING[q + "object"].tobytes(), "Shuffle", name, "Shuffle", nodes, nodes)
