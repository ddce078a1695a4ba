"""The raw `.bin` tensor loader (loadTensor, runtime/source/utils/utils.cpp:71-101) on the reference's own input files."""
import os

import numpy as np
import pytest
import torch

from pimaicompiler_amd import io

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def test_rnnt_feature_files_load_with_the_documented_shapes():
    # examples/runtime/resource/rnnt/inputs/README.md: feature.bin fp16 [341, 1, 240], feature_len.bin int64 [1] = 341
    feat = io.load_tensor(os.path.join(GOLDEN, "rnnt_feature_341x1x240_f16.bin"), [341, 1, 240], "FLOAT16")
    n = io.load_tensor(os.path.join(GOLDEN, "rnnt_feature_len_i64.bin"), [1], "INT64")
    assert feat.dtype == torch.float16 and list(feat.shape) == [341, 1, 240] and int(n[0]) == 341
    assert torch.isfinite(feat.float()).all() and float(feat.float().std()) > 0.5   # normalised features


def test_round_trip_and_errors(tmp_path):
    for dtype, t in [("FLOAT16", torch.randn(3, 5).half()), ("FLOAT32", torch.randn(7)), ("INT64", torch.arange(12).reshape(3, 4)),
                     ("BOOL", torch.tensor([True, False, True]))]:
        f = str(tmp_path / f"{dtype}.bin")
        io.save_tensor(t, f)
        assert torch.equal(io.load_tensor(f, list(t.shape), dtype), t)
    f = str(tmp_path / "short.bin")
    np.zeros(3, np.float16).tofile(f)
    with pytest.raises(ValueError):
        io.load_tensor(f, [4], "FLOAT16")
    with pytest.raises(FileNotFoundError):
        io.load_tensor(str(tmp_path / "missing.bin"), [1], "FLOAT16")
    with pytest.raises(ValueError):
        io.load_tensor(f, [3], "FLOAT64")
