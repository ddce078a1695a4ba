"""Raw tensor files of the reference's examples.

`load_tensor` mirrors loadTensor (runtime/source/utils/utils.cpp:71-101): a `.bin` file is the little-endian bytes
of a dense tensor as `numpy.ndarray.tofile` writes them, with shape and element type given by the caller (e.g. the
RNNT encoder input `feature.bin`, fp16 [341, 1, 240], examples/runtime/source/pipeline_manager.cpp:105).
Unlike the reference, a missing or short file is an error instead of being ignored.
"""
import os

import numpy as np
import torch

# DataType names of ir/include/types.h used by loadTensor.
_DTYPES = {
    "INT64": (np.dtype("<i8"), torch.int64),
    "FLOAT32": (np.dtype("<f4"), torch.float32),
    "FLOAT16": (np.dtype("<f2"), torch.float16),
    "BOOL": (np.dtype("?"), torch.bool),
}


def load_tensor(bin_file, shape, dtype, device=None):
    """Returns a torch tensor of `shape` read from `bin_file`.  dtype: "INT64" | "FLOAT32" | "FLOAT16" | "BOOL"."""
    if dtype not in _DTYPES:
        raise ValueError(f"unsupported data type {dtype!r}")
    np_dtype, _ = _DTYPES[dtype]
    if not os.path.isfile(bin_file):
        raise FileNotFoundError(bin_file)
    count = int(np.prod(shape)) if len(shape) else 1
    need = count * np_dtype.itemsize
    if os.path.getsize(bin_file) < need:
        raise ValueError(f"{bin_file} holds {os.path.getsize(bin_file)} bytes, {need} are needed for shape {list(shape)}")
    data = np.fromfile(bin_file, dtype=np_dtype, count=count).reshape(shape)
    t = torch.from_numpy(data.copy())
    return t.to(device) if device is not None else t


def save_tensor(tensor, bin_file):
    """The inverse: dense little-endian bytes of `tensor`."""
    tensor.detach().cpu().contiguous().numpy().tofile(bin_file)
