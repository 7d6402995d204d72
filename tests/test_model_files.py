"""Model files on the CPU: the `.otter` parser and the ncnn `.bin` reader of the host layer against the compiled
reference (where oracle/_ref is built) and against the committed fixture of the reference's parse."""
import glob
import os

import numpy as np
import pytest

from tensor_amd import calibration, hostnet, modelfile

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")


def test_parser_reproduces_the_reference_parse_of_the_syntax_cases():
    """Quoted values with blanks, `key:value` / `key :value` / `key : value`, `Name{`, comments, nested blocks whose
    parameters reach the layer, the `$` terminator: the committed dump is the reference's own reading."""
    got = hostnet.otter_dump(os.path.join(GOLDEN, "otter_syntax_cases.otter"))
    with open(os.path.join(GOLDEN, "otter_syntax_cases.dump")) as f:
        want = f.read()
    assert got == want
    assert "never_read" not in got and "P input=data, conv_a" in got


def test_parser_on_the_int8_detection_model():
    dump = hostnet.otter_dump(os.path.join(GOLDEN, "nanodet-plus-m-1.5x_416_int8_fused.otter")).splitlines()
    blocks = [l[2:] for l in dump if l.startswith("T ")]
    assert len(blocks) == 190 and blocks.count("Convolution") == 110 and blocks[0] == "Input"
    assert sum(l.startswith("P int8_scale_term=") for l in dump) == 110
    # a nested Param block's keys arrive after the block's own keys
    i = dump.index("P name=conv_1")
    assert dump[i - 1] == "P activation=LRelu" and "P out_channels=24" in dump[i:i + 6]


def test_parser_equals_the_compiled_reference_on_every_description(ref):
    files = sorted(glob.glob(os.path.join(GOLDEN, "*.otter"))) + sorted(glob.glob("/root/reference/benchmark/*.otter"))
    assert files
    for f in files:
        assert hostnet.otter_dump(f) == ref.otter_dump(f), f


def _write_bin(path, rng):
    """One tensor of every form the reader knows, then plain vectors; returns (shapes, kinds, expected arrays)."""
    w8 = rng.integers(-127, 128, size=(5, 3, 3, 3)).astype(np.int8)      # 135 bytes: padded to 136
    w16 = rng.normal(0, 1, (4, 7)).astype(np.float16)                    # 56 bytes
    w16[0, :4] = [0.0, -0.0, 6.1e-5, 5.96e-8]                            # zero, smallest normal, a subnormal
    w16b = rng.normal(0, 30, (3, 3)).astype(np.float16)                  # 18 bytes: padded to 20
    w32 = rng.normal(0, 1, (2, 3, 1, 1)).astype(np.float32)
    table = rng.normal(0, 1, 256).astype(np.float32)
    index = rng.integers(0, 256, size=(6, 5)).astype(np.uint8)           # 30 bytes: padded to 32
    bias = rng.normal(0, 1, 5).astype(np.float32)
    scale = np.array([31.5], np.float32)
    blob = (modelfile.weight_int8(w8) + modelfile.vector(bias) + modelfile.weight_fp16(w16) + modelfile.weight_fp16(w16b) +
            modelfile.weight_fp32(w32) + modelfile.weight_fp32(w32, tagged=True) + modelfile.weight_table(table, index) +
            modelfile.vector(scale) + b"tail")
    with open(path, "wb") as f:
        f.write(blob)
    shapes = [w8.shape, bias.shape, w16.shape, w16b.shape, w32.shape, w32.shape, index.shape, scale.shape]
    kinds = [0, 1, 0, 0, 0, 0, 0, 1]
    want = [w8, bias, w16.astype(np.float32), w16b.astype(np.float32), w32, w32, table[index], scale]
    return shapes, kinds, want


def test_ncnn_bin_reader_every_tensor_form(tmp_path):
    path = str(tmp_path / "forms.bin")
    shapes, kinds, want = _write_bin(path, np.random.default_rng(5))
    got, remain = hostnet.ncnn_read(path, shapes, kinds)
    assert remain == 4  # the four bytes of "tail"
    for g, w in zip(got, want):
        assert g.dtype == w.dtype
        np.testing.assert_array_equal(g, w)
    # a truncated file: the tensor that cannot be read completely comes back undefined
    with open(path, "rb") as f:
        data = f.read()
    short = str(tmp_path / "short.bin")
    with open(short, "wb") as f:
        f.write(data[:100])
    got, remain = hostnet.ncnn_read(short, shapes[:2], kinds[:2])
    assert got[0] is None


def test_ncnn_bin_reader_equals_the_compiled_reference(ref, tmp_path):
    path = str(tmp_path / "forms.bin")
    shapes, kinds, _ = _write_bin(path, np.random.default_rng(6))
    ours, remain_ours = hostnet.ncnn_read(path, shapes, kinds)
    fn, err = ref.ncnn_read_entry
    theirs, remain_ref = hostnet.ncnn_read(path, shapes, kinds, reader=fn, err=err)
    assert remain_ours == remain_ref
    for a, b in zip(ours, theirs):
        assert a.dtype == b.dtype
        np.testing.assert_array_equal(a, b)


def test_conv_record_layout():
    """weight (tag + bytes + pad), bias, weight scales, bottom scale, top scale only when int8_scale_term > 100."""
    wq = np.arange(-5, 5, dtype=np.int8).reshape(2, 5, 1, 1)
    rec = modelfile.conv_record(wq, np.zeros(2, np.float32), np.ones(2, np.float32), 3.0, 4.0, 101)
    assert len(rec) == 4 + 12 + 8 + 8 + 4 + 4
    assert np.frombuffer(rec[:4], np.uint32)[0] == 0x000D4B38
    rec1 = modelfile.conv_record(wq, None, np.ones(2, np.float32), 3.0, 4.0, 1)
    assert len(rec1) == 4 + 12 + 8 + 4


def test_quantize_weights_definition():
    w = np.array([[[[0.5, -1.0]]], [[[0.2, 0.1]]], [[[0.0, 0.0]]]], np.float32)
    wq, ws = calibration.quantize_weights(w)
    np.testing.assert_array_equal(wq.reshape(3, 2), [[64, -127], [127, 64], [0, 0]])  # 63.5 rounds away from zero
    np.testing.assert_allclose(ws, [127.0, 635.0, 127.0])
    wq1, ws1 = calibration.quantize_weights(w, per_channel=False)
    assert ws1.shape == (1,) and wq1.reshape(-1)[1] == -127 and wq1.reshape(-1)[2] == 25


@pytest.mark.gpu
def test_host_net_refuses_the_mixed_description_by_name():
    """The library's own Net runs int8 convolutions only: it refuses a graph with an fp32 convolution when it is compiled,
    naming the layer, rather than fail inside a forward pass."""
    net = hostnet.Net()
    with pytest.raises(hostnet.HostError, match="conv_1.*fp32 convolution"):
        net.load_otter(os.path.join(GOLDEN, "nanodet-plus-m-1.5x_416_int8_mixed.otter"))
    net.close()
