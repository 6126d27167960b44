"""The reference's raw tensor file format, for tensors that cross a process boundary (inputs and outputs of its
device wrappers; here also a place to keep pre-packed weights).

Layout, little endian (test/utils/dsp/include/tensor.h:235-260): int32 data type id, int64 rank, rank x int64
shape, then the elements row-major with no padding. Type ids (tensor.h:26-38 = qcom_hexagon_backend/backend/
utils.py:36-54): 0 bool, 1 f16, 2 f32, 3 f64, 4 i8, 5 i16, 6 i32, 7 i64, 8 u8, 9 u16, 10 u32. bfloat16 has no id in
the reference and is refused.
"""
import struct

import numpy as np
import torch

_ID_TO_NP = {0: np.bool_, 1: np.float16, 2: np.float32, 3: np.float64, 4: np.int8, 5: np.int16, 6: np.int32,
             7: np.int64, 8: np.uint8, 9: np.uint16, 10: np.uint32}
_NP_TO_ID = {np.dtype(v): k for k, v in _ID_TO_NP.items()}


def save_tensor(path, tensor):
    """Write a torch tensor (any device; copied to the host) or numpy array in the reference's format."""
    if isinstance(tensor, torch.Tensor):
        if tensor.dtype == torch.bfloat16:
            raise TypeError("tensor_file: the format has no type id for bfloat16")
        arr = tensor.detach().cpu().contiguous().numpy()
    else:
        arr = np.ascontiguousarray(tensor)
    if arr.dtype not in _NP_TO_ID:
        raise TypeError("tensor_file: no type id for dtype %s" % arr.dtype)
    with open(path, "wb") as f:
        f.write(struct.pack("<iq", _NP_TO_ID[arr.dtype], arr.ndim))
        f.write(struct.pack("<%dq" % arr.ndim, *arr.shape))
        f.write(arr.astype(arr.dtype.newbyteorder("<"), copy=False).tobytes())


def load_tensor(path):
    """Read a file in the reference's format into a CPU torch tensor (uint16 / uint32 need a torch that has them)."""
    with open(path, "rb") as f:
        head = f.read(12)
        if len(head) != 12:
            raise ValueError("tensor_file: %s is shorter than its header" % path)
        type_id, rank = struct.unpack("<iq", head)
        if type_id not in _ID_TO_NP:
            raise ValueError("tensor_file: unknown data type id %d in %s" % (type_id, path))
        if rank < 0 or rank > 64:
            raise ValueError("tensor_file: implausible rank %d in %s" % (rank, path))
        dims = f.read(8 * rank)
        if len(dims) != 8 * rank:
            raise ValueError("tensor_file: %s ends inside its shape" % path)
        shape = struct.unpack("<%dq" % rank, dims)
        if any(d < 0 for d in shape):
            raise ValueError("tensor_file: negative extent in %s" % path)
        dt = np.dtype(_ID_TO_NP[type_id]).newbyteorder("<")
        count = int(np.prod(shape, dtype=np.int64)) if rank else 1
        data = f.read(count * dt.itemsize)
        if len(data) != count * dt.itemsize:
            raise ValueError("tensor_file: %s holds %d of %d data bytes" % (path, len(data), count * dt.itemsize))
    arr = np.frombuffer(data, dtype=dt).astype(dt.newbyteorder("="), copy=True).reshape(shape)
    return torch.from_numpy(arr)
