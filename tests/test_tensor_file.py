"""The reference's raw tensor file format (test/utils/dsp/include/tensor.h:235-260): byte-exact header and data for
a hand-built file, round trips for every type id, and the error cases. Runs without a GPU."""
import struct
import sys
import os

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "hexagon-mlir_amd"))
from hexmi.tensor_file import load_tensor, save_tensor  # noqa: E402


def test_bytes_of_a_known_tensor(tmp_path):
    # f32 [2,3] holding 0..5: id 2, rank 2, shape 2 3, then six little-endian floats, nothing else
    t = torch.arange(6, dtype=torch.float32).reshape(2, 3)
    p = tmp_path / "t.bin"
    save_tensor(str(p), t)
    want = struct.pack("<i", 2) + struct.pack("<q", 2) + struct.pack("<qq", 2, 3) + struct.pack("<6f", 0, 1, 2, 3, 4, 5)
    assert p.read_bytes() == want
    # and a file written by hand in that layout reads back
    q = tmp_path / "h.bin"
    q.write_bytes(struct.pack("<iq", 4, 1) + struct.pack("<q", 5) + bytes([1, 2, 253, 254, 255]))
    got = load_tensor(str(q))
    assert got.dtype == torch.int8 and got.tolist() == [1, 2, -3, -2, -1]


@pytest.mark.parametrize("dtype", [torch.bool, torch.float16, torch.float32, torch.float64, torch.int8, torch.int16,
                                   torch.int32, torch.int64, torch.uint8])
def test_round_trip(tmp_path, dtype):
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(3, 5, 7, generator=g) * 50)
    x = (x > 0) if dtype == torch.bool else x.to(dtype)
    p = str(tmp_path / "x.bin")
    save_tensor(p, x)
    y = load_tensor(p)
    assert y.dtype == dtype and y.shape == x.shape and torch.equal(x, y)
    assert os.path.getsize(p) == 4 + 8 + 8 * 3 + x.numel() * x.element_size()


def test_rank_zero_and_non_contiguous(tmp_path):
    p = str(tmp_path / "s.bin")
    save_tensor(p, torch.tensor(2.5))
    y = load_tensor(p)
    assert y.shape == () and float(y) == 2.5 and os.path.getsize(p) == 16
    x = torch.arange(12, dtype=torch.int32).reshape(3, 4).t()      # strided view: stored row-major
    save_tensor(p, x)
    assert torch.equal(load_tensor(p), x.contiguous())
    save_tensor(p, np.arange(4, dtype=np.uint16))
    assert np.array_equal(load_tensor(p).numpy(), np.arange(4, dtype=np.uint16))


def test_errors(tmp_path):
    p = tmp_path / "bad.bin"
    with pytest.raises(TypeError):
        save_tensor(str(p), torch.zeros(2, dtype=torch.bfloat16))
    p.write_bytes(struct.pack("<iq", 42, 0))
    with pytest.raises(ValueError):
        load_tensor(str(p))
    p.write_bytes(struct.pack("<iq", 2, 1) + struct.pack("<q", 4) + b"\0" * 15)      # one byte short
    with pytest.raises(ValueError):
        load_tensor(str(p))
    p.write_bytes(b"\1\0\0")
    with pytest.raises(ValueError):
        load_tensor(str(p))
