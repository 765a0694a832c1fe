"""MCLTEN tensor files (src/serialization.cpp:21-63,121-136 of MotifCL): the Python writer and reader
against a hand-assembled file -- the same literal bytes the C++ host test holds -- plus the
version-1 form and the refusals."""
import numpy as np
import pytest

from motifcl_amd import checkpoint as ck

LITERAL_V2 = bytes(
    [ord(c) for c in "MCLTEN2"] + [0] +
    [3, 0, 0, 0] +                    # dtype U8
    [1, 0, 0, 0, 0, 0, 0, 0] +        # ndim
    [6, 0, 0, 0, 0, 0, 0, 0] +        # dims[0]
    [6, 0, 0, 0, 0, 0, 0, 0] +        # nbytes
    [0x00, 0x00, 0x80, 0x3f] +        # quant_scale 1.0f
    [0, 0, 0, 0] +                    # has_quant_scales
    [0xff, 0xff, 0xff, 0xff] +        # quant_scale_axis -1
    [0, 0, 0, 0, 0, 0, 0, 0] +        # quant_block_size
    [0, 1, 2, 3, 4, 5])


def test_written_bytes_match_the_stated_layout(tmp_path):
    p = str(tmp_path / "t.mt")
    ck.save_tensor(np.arange(6, dtype=np.uint8), p)
    assert open(p, "rb").read() == LITERAL_V2
    back = ck.load_tensor(p)
    assert back.dtype == np.uint8 and back.tolist() == [0, 1, 2, 3, 4, 5]


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int32, np.uint8])
def test_round_trip(tmp_path, dtype):
    rng = np.random.default_rng(3)
    a = (rng.standard_normal((5, 7, 2)) * 50).astype(dtype)
    p = str(tmp_path / "a.mt")
    ck.save_tensor(a, p)
    b = ck.load_tensor(p)
    assert b.dtype == a.dtype and b.shape == a.shape and np.array_equal(a, b)


def test_version_1_files_load(tmp_path):
    p = tmp_path / "v1.mt"
    p.write_bytes(b"MCLTEN1\0" + bytes([3, 0, 0, 0, 1, 0, 0, 0, 0, 0, 0, 0, 3, 0, 0, 0, 0, 0, 0, 0,
                                        3, 0, 0, 0, 0, 0, 0, 0, 9, 8, 7]))
    assert ck.load_tensor(str(p)).tolist() == [9, 8, 7]


@pytest.mark.parametrize("mutate, message", [
    (lambda b: b[:6] + b"9" + b[7:], "magic mismatch"),
    (lambda b: b[:28] + bytes([7]) + b[29:], "does not match dtype/shape"),
    (lambda b: b[:-2], "failed to read tensor payload"),
    (lambda b: b[:8] + bytes([5]) + b[9:], "dtype"),
    (lambda b: b[:40] + bytes([1]) + b[41:], "quantization scales"),
    (lambda b: b[:20], "failed to read"),
])
def test_damaged_files_are_refused(tmp_path, mutate, message):
    p = tmp_path / "bad.mt"
    p.write_bytes(mutate(LITERAL_V2))
    with pytest.raises(ck.CheckpointError, match=message):
        ck.load_tensor(str(p))


def test_counter_layer_files(tmp_path, oracle):
    n_in, n_out, C = 16, 6, 11
    rng = np.random.default_rng(0)
    state = oracle.pack_codes(rng.integers(0, 63, (n_out, n_in)).astype(np.uint8))
    scale = rng.random(n_out).astype(np.float32)
    v = rng.random(n_out).astype(np.float32)
    prefix = str(tmp_path / "l0_wq")
    ck.save_counter_layer(prefix, state, scale, v)
    s2, sc2, v2 = ck.load_counter_layer(prefix, n_in, n_out)
    assert np.array_equal(s2, state) and np.array_equal(sc2, scale) and np.array_equal(v2, v)
    with pytest.raises(ck.CheckpointError, match="does not fit"):
        ck.load_counter_layer(prefix, n_in, n_out + 1)
