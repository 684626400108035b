"""The safetensors reader against files written by the safetensors package and against hand-built bytes."""
import json
import struct

import numpy as np
import pytest
import torch

from juliavision_amd import safetensors as ST


def _write(path, header: dict, data: bytes, pad=0):
    h = json.dumps(header).encode() + b" " * pad
    path.write_bytes(struct.pack("<Q", len(h)) + h + data)


def test_reads_what_the_safetensors_package_writes(tmp_path):
    from safetensors.torch import save_file
    torch.manual_seed(0)
    want = {"w": torch.randn(5, 7).half(), "b": torch.randn(7), "idx": torch.arange(6, dtype=torch.int64).view(2, 3),
            "flag": torch.tensor([True, False, True]), "scalar": torch.tensor(3.5), "bf": torch.randn(4, 2).bfloat16(),
            "empty": torch.zeros((0, 4), dtype=torch.float16), "u8": torch.arange(10, dtype=torch.uint8)}
    p = tmp_path / "m.safetensors"
    save_file(want, str(p), metadata={"format": "pt"})
    assert sorted(ST.names(str(p))) == sorted(want)
    got = ST.read(str(p))
    assert set(got) == set(want)
    for k, t in want.items():
        assert got[k].dtype == t.dtype and tuple(got[k].shape) == tuple(t.shape), k      # shapes as stored: torch is row-major like the file
        assert torch.equal(got[k], t), k
    sub = ST.read(str(p), only=["w", "b"])
    assert set(sub) == {"w", "b"}
    with pytest.raises(KeyError):
        ST.read(str(p), only=["nope"])
    got["w"][0, 0] = 99.0                                    # copy-on-write mapping: the file is untouched
    assert torch.equal(ST.read(str(p))["w"], want["w"])


def test_hand_built_file_and_row_major_order(tmp_path):
    a = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    c = (np.arange(4) + 1j * np.arange(4)).astype(np.complex64)
    data = a.tobytes() + c.tobytes()
    p = tmp_path / "h.safetensors"
    _write(p, {"__metadata__": {"k": "v"}, "a": {"dtype": "F32", "shape": [2, 3, 4], "data_offsets": [0, 96]},
               "c": {"dtype": "C64", "shape": [4], "data_offsets": [96, 128]}}, data, pad=5)
    got = ST.read(str(p))
    assert got["a"][1, 2, 3] == 23.0 and got["a"][0, 1, 0] == 4.0 and got["a"].stride() == (12, 4, 1)
    assert np.array_equal(got["c"].numpy(), c)
    assert ST.names(str(p)) == ["a", "c"]


def test_malformed_files_are_refused_by_name(tmp_path):
    p = tmp_path / "bad.safetensors"
    p.write_bytes(b"\x01\x02")
    with pytest.raises(ST.SafetensorsError, match="shorter"):
        ST.read(str(p))
    p.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(ST.SafetensorsError, match="exceeds"):
        ST.read(str(p))
    _write(p, {"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 12]}}, b"\0" * 16)
    with pytest.raises(ST.SafetensorsError, match="byte range"):
        ST.read(str(p))
    _write(p, {"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}, b"\0" * 8)
    with pytest.raises(ST.SafetensorsError, match="byte range"):
        ST.read(str(p))
    _write(p, {"a": {"dtype": "F8_E4M3", "shape": [4], "data_offsets": [0, 4]}}, b"\0" * 4)
    with pytest.raises(ST.SafetensorsError, match="dtype"):
        ST.read(str(p))
    p.write_bytes(struct.pack("<Q", 4) + b"nope")
    with pytest.raises(ST.SafetensorsError, match="JSON"):
        ST.read(str(p))
