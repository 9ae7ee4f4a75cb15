"""The native GGUF reader on the fixture file, asserting what the reference's own reader test asserts
(jitnn-gguf/src/test/java/ai/beestream/jitnn/gguf/GgufFileTest.java): header, metadata of every value type,
shapes in jitNN's axis order, types without a tensor type, rejected files.  Parsing needs no GPU; the tests
that move tensors to the device are marked gpu."""
import struct

import numpy as np
import pytest

from helpers import GOLDEN as GOLDEN_DIR

import jitnn_amd
from jitnn_amd import DType, GgufFile, UnsupportedTypeError

FIXTURE = GOLDEN_DIR / "fixture.gguf"
PATH_FORMATS = ["Q8_0", "Q4_0", "Q4_1", "Q4_K", "Q5_K", "Q6_K", "Q5_0", "Q5_1", "Q2_K", "Q3_K"]


@pytest.fixture(scope="module")
def f():
    g = GgufFile.open(FIXTURE)
    yield g
    g.close()


def test_header(f):  # GgufFileTest.java:41-49
    assert f.version() == 3
    assert f.alignment() == 32
    assert f.data_offset() % 32 == 0
    assert f.architecture() == "llama"
    assert len(f.tensor_infos()) == 30


def test_metadata_of_every_type(f):  # GgufFileTest.java:51-82
    assert f.integer("test.u8") == 250
    assert f.integer("test.i8") == -100
    assert f.integer("test.u16") == 60000
    assert f.integer("test.i16") == -30000
    assert f.long_value("test.u32") == 3_000_000_000
    with pytest.raises(ValueError):
        f.integer("test.u32")
    assert f.integer("test.i32") == -2_000_000_000
    assert f.float_value("test.f32") == 1.5
    assert f.bool("test.bool") is True
    assert f.string("test.string") == "héllo, wörld"
    assert f.long_value("test.u64") == (1 << 40) + 3
    assert f.long_value("test.i64") == -(1 << 40)
    assert f.float_value("test.f64") == 2.25
    assert f.ints("test.ints").tolist() == [1, -2, 3]
    assert f.floats("test.floats").tolist() == [0.5, -1.25]
    assert f.strings("test.strings") == ["a", "βγ", ""]
    assert f.get("test.bools") == [True, False]
    assert f.get("test.nested") == [[1, 2], [3]]
    assert f.longs("test.u32s").tolist() == [7, 4_000_000_000]
    with pytest.raises(ValueError):
        f.ints("test.u32s")
    assert f.get("test.f64s") == [0.125, -3.5]
    assert f.integer("llama.block_count") == 2
    assert f.integer("llama.missing", 7) == 7
    assert f.get("llama.missing") is None
    with pytest.raises(ValueError):
        f.string("llama.missing")
    with pytest.raises(ValueError):
        f.string("test.u8")
    with pytest.raises(ValueError):
        f.integer("test.bool")


def test_shapes_in_jitnn_order(f):  # GgufFileTest.java:84-102
    q = f.info("w.Q4_K")
    assert q.shape == (3, 512) and q.type == "Q4_K" and q.bytes == 3 * 512 // 256 * 144
    assert f.info("axes.1d").shape == (5,)
    assert f.info("axes.3d").shape == (2, 3, 4)
    t = f.tensor("axes.3d")
    assert (t.dim(0), t.dim(1), t.dim(2)) == (2, 3, 4)
    assert t.to_float_array().tolist() == [float(i) for i in range(24)]  # numpy's row-major order is jitNN's
    assert t.numpy()[1, 2, 3] == 23.0
    assert f.tensor("axes.1d").to_float_array().tolist() == [0, 1, 2, 3, 4]
    ints = f.tensor("ints.I32")
    assert ints.dtype() == DType.I32
    assert ints.to_int_array().tolist() == [1, -2, 3, 4, 5, -6]


def test_every_tensor_lies_inside_the_file(f):
    size = FIXTURE.stat().st_size
    for t in f.tensor_infos().values():
        assert t.offset % f.alignment() == 0 and t.offset >= f.data_offset()
        assert t.bytes >= 0 and t.offset + t.bytes <= size, t


def test_raw_bytes_are_the_files(f):
    whole = FIXTURE.read_bytes()
    for name in ("w.Q4_K", "w.Q6_K", "expect.Q8_0", "ints.I32"):
        t = f.info(name)
        assert f.raw(name).tobytes() == whole[t.offset:t.offset + t.bytes]


def test_types_without_tensor_type(f):  # GgufFileTest.java:104-112
    assert f.info("w.Q8_K").type == "Q8_K"
    with pytest.raises(UnsupportedTypeError):
        f.tensor("w.Q8_K")
    assert f.raw("w.Q8_K").size == 3 * 512 // 256 * 292
    with pytest.raises(ValueError):
        f.tensor("no.such.tensor")
    with pytest.raises(ValueError):
        f.raw("no.such.tensor")


def test_rejects_other_files(tmp_path):  # GgufFileTest.java:114-123
    not_gguf = tmp_path / "a.bin"
    not_gguf.write_bytes(bytes(64))
    with pytest.raises(OSError):
        GgufFile.open(not_gguf)
    truncated = tmp_path / "t.gguf"
    truncated.write_bytes(FIXTURE.read_bytes()[:600])
    with pytest.raises(OSError):
        GgufFile.open(truncated)
    with pytest.raises(OSError):
        GgufFile.open(tmp_path / "missing.gguf")
    empty = tmp_path / "empty.gguf"
    empty.write_bytes(b"")
    with pytest.raises(OSError):
        GgufFile.open(empty)
    v1 = tmp_path / "v1.gguf"
    v1.write_bytes(struct.pack("<IIQQ", 0x46554747, 1, 0, 0) + bytes(64))
    with pytest.raises(OSError):
        GgufFile.open(v1)


def crafted(dim, offset, metadata=b"", kv_count=0, ttype=0):
    """A GGUF header with one tensor "w" of the given dimension, type and offset, and optional metadata bytes."""
    b = struct.pack("<IIQQ", 0x46554747, 3, 1, kv_count) + metadata
    b += struct.pack("<Q", 1) + b"w" + struct.pack("<IQIQ", 1, dim & 0xFFFFFFFFFFFFFFFF, ttype, offset & 0xFFFFFFFFFFFFFFFF)
    return b + bytes(64)


def test_crafted_file_opens(tmp_path):
    ok = tmp_path / "ok.gguf"
    ok.write_bytes(crafted(4, 0))
    g = GgufFile.open(ok)
    assert g.info("w").shape == (4,) and g.info("w").bytes == 16
    assert g.raw("w").tobytes() == bytes(16)


def test_rejects_crafted_sizes(tmp_path):  # GgufFileTest.java:135-155
    huge_dim = tmp_path / "dim.gguf"
    huge_dim.write_bytes(crafted(-1, 0))
    with pytest.raises(OSError):
        GgufFile.open(huge_dim)
    huge_offset = tmp_path / "offset.gguf"
    huge_offset.write_bytes(crafted(4, (1 << 63) - 1 - 31))
    with pytest.raises(OSError):
        GgufFile.open(huge_offset)
    past_end = tmp_path / "past.gguf"
    past_end.write_bytes(crafted(1 << 20, 0))
    with pytest.raises(OSError):
        GgufFile.open(past_end)
    ragged = tmp_path / "ragged.gguf"  # a row of a block type must hold whole blocks
    ragged.write_bytes(crafted(48, 0, ttype=8))
    with pytest.raises(OSError):
        GgufFile.open(ragged)
    kv = struct.pack("<Q", 4) + b"deep" + struct.pack("<I", 9)
    for _ in range(200):  # arrays nested 200 deep: rejected instead of overflowing the stack
        kv += struct.pack("<IQ", 9, 1)
    kv += struct.pack("<IQ", 4, 0)
    deep = tmp_path / "deep.gguf"
    deep.write_bytes(crafted(4, 0, kv, 1))
    with pytest.raises(OSError):
        GgufFile.open(deep)
    long_string = tmp_path / "str.gguf"
    long_string.write_bytes(crafted(4, 0, struct.pack("<Q", 1) + b"k" + struct.pack("<IQ", 8, 1 << 40), 1))
    with pytest.raises(OSError):
        GgufFile.open(long_string)
    long_array = tmp_path / "arr.gguf"
    long_array.write_bytes(crafted(4, 0, struct.pack("<Q", 1) + b"k" + struct.pack("<IIQ", 9, 4, 1 << 60), 1))
    with pytest.raises(OSError):
        GgufFile.open(long_array)


def test_mapping_leaves_the_file_unchanged(tmp_path):  # GgufFileTest.java:166-178 (host part)
    rw = tmp_path / "rw.gguf"
    rw.write_bytes(FIXTURE.read_bytes())
    g = GgufFile.open(rw)
    for name, t in g.tensor_infos().items():
        g.raw(name)
    g.close()
    assert rw.read_bytes() == FIXTURE.read_bytes()


def test_tensor_upload_needs_a_device(f):
    try:
        jitnn_amd.init()
    except jitnn_amd.JitnnError:
        pass
    else:
        pytest.skip("a device is present")
    with pytest.raises(jitnn_amd.JitnnError):
        f.tensor("w.Q4_K")


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", PATH_FORMATS)
def test_weights_from_file_dequantise_bit_exact(f, fmt):  # GgufChecks.weights, GgufChecks.java:58-75
    w = f.tensor("w." + fmt)
    assert w.dtype() == DType[fmt] and w.shape() == (3, 512)
    got = w.to_float_array()
    expect = f.tensor("expect." + fmt).to_float_array()
    assert np.array_equal(got.view(np.uint32), expect.view(np.uint32))


@pytest.mark.gpu
def test_read_only_file(tmp_path):  # GgufFileTest.java:157-164
    ro = tmp_path / "ro.gguf"
    ro.write_bytes(FIXTURE.read_bytes())
    ro.chmod(0o444)
    g = GgufFile.open(ro)
    assert np.array_equal(g.tensor("w.Q4_K").to_float_array(), g.tensor("expect.Q4_K").to_float_array())


@pytest.mark.gpu
def test_linear_on_file_weights(f):  # GgufChecks.java:76-110: the linear of each file weight against its expected values
    from jitnn_amd import Gguf, Tensor
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 512)).astype(np.float32)
    for fmt in PATH_FORMATS:
        w = f.tensor("w." + fmt)
        e = f.tensor("expect." + fmt).numpy().astype(np.float64)
        ref = x.astype(np.float64) @ e.T
        y = Gguf.linear(Tensor.of(x), w, None).numpy()
        assert np.abs(y - ref).max() <= 1e-4 * np.abs(ref).max(), fmt


@pytest.mark.gpu
def test_tensors_stops_at_unsupported_type(f):
    with pytest.raises(UnsupportedTypeError):
        f.tensors()
