"""Host-only validation of optimizer-state checkpoints (mxopt_checkpoint_inspect): runs without a GPU.
Valid files come from the `safetensors` package; malformed ones are hand-made or fuzzed, and must be
refused with a message, never crash and never be accepted with ranges outside the file."""
import ctypes as C
import json
import os
import struct
import sys

import numpy as np
import pytest
from hypothesis import HealthCheck, given, settings
from hypothesis import strategies as st

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "mlx-node_amd"))
F = np.float32
META = {"format": "mxopt-optimizer-state", "optimizer": "adamw", "step": "1230"}


@pytest.fixture(scope="module")
def lib():
    from mxopt import _lib
    return _lib.load()


def inspect(lib, path):
    kind = C.create_string_buffer(32)
    step, tensors, elements = C.c_int64(), C.c_uint64(), C.c_uint64()
    rc = lib.mxopt_checkpoint_inspect(str(path).encode(), kind, 32, C.byref(step), C.byref(tensors), C.byref(elements))
    return rc, kind.value.decode(), step.value, tensors.value, elements.value, lib.mxopt_last_error(None).decode()


def raw_file(path, header: bytes, data: bytes = b""):
    path.write_bytes(struct.pack("<Q", len(header)) + header + data)
    return path


def test_accepts_what_the_safetensors_package_writes(lib, tmp_path):
    from safetensors.numpy import save_file
    p = tmp_path / "ok.safetensors"
    save_file({"layers.0.w.m": np.zeros(1000, F), "layers.0.w.v": np.ones(1000, F), "b.m": np.zeros(7, F),
               "b.v": np.zeros(7, F)}, str(p), metadata=META)
    rc, kind, step, tensors, elements, _ = inspect(lib, p)
    assert (rc, kind, step, tensors, elements) == (0, "adamw", 1230, 4, 2014)


def test_refuses_malformed_files(lib, tmp_path):
    entry = {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}
    ok_header = json.dumps({"w.m": entry, "__metadata__": META}).encode()
    assert inspect(lib, raw_file(tmp_path / "ok", ok_header, b"\0" * 16))[0] == 0
    cases = {
        "missing file": None,
        "too short": b"\x01\x02",
        "data cut": (ok_header, b"\0" * 15),
        "no metadata": (json.dumps({"w.m": entry}).encode(), b"\0" * 16),
        "model file": (json.dumps({"w": entry, "__metadata__": {"format": "pt"}}).encode(), b"\0" * 16),
        "bf16 moments": (json.dumps({"w.m": dict(entry, dtype="BF16"), "__metadata__": META}).encode(), b"\0" * 16),
        "reversed range": (json.dumps({"w.m": dict(entry, data_offsets=[16, 0]), "__metadata__": META}).encode(), b"\0" * 16),
        "negative offset": (json.dumps({"w.m": dict(entry, data_offsets=[-4, 12]), "__metadata__": META}).encode(), b"\0" * 16),
        "huge offset": (json.dumps({"w.m": dict(entry, data_offsets=[0, 1e30]), "__metadata__": META}).encode(), b"\0" * 16),
        "ragged floats": (json.dumps({"w.m": dict(entry, data_offsets=[0, 15]), "__metadata__": META}).encode(), b"\0" * 16),
        "offsets are strings": (json.dumps({"w.m": dict(entry, data_offsets=["0", "16"]), "__metadata__": META}).encode(), b"\0" * 16),
        "entry is a list": (json.dumps({"w.m": [1, 2], "__metadata__": META}).encode(), b"\0" * 16),
        "not json": (b"{not json" + b" " * 7, b""),
        "deep nesting": (b"[" * 200 + b"]" * 200, b""),
        "unterminated string": (b'{"abc', b""),
        "optimizer name with a byte that is no text": (ok_header.replace(b'"adamw"', b'"\x80damw"'), b"\0" * 16),
        "optimizer name with a control character": (ok_header.replace(b'"adamw"', b'"ada\\nw"'), b"\0" * 16),
    }
    for name, spec in cases.items():
        path = tmp_path / "bad"
        if spec is None:
            path = tmp_path / "nothing-here"
        elif isinstance(spec, bytes):
            path.write_bytes(spec)
        else:
            raw_file(path, *spec)
        rc, *_, msg = inspect(lib, path)
        assert rc != 0 and msg, name
    # a header length that points past the end of the file
    (tmp_path / "len").write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    assert inspect(lib, tmp_path / "len")[0] != 0


@settings(max_examples=300, deadline=None, derandomize=True, suppress_health_check=list(HealthCheck))
@given(blob=st.binary(max_size=200), flips=st.lists(st.tuples(st.integers(0, 400), st.integers(0, 255)), max_size=6))
def test_fuzzed_files_never_crash_and_never_overrun(lib, tmp_path_factory, blob, flips):
    d = tmp_path_factory.mktemp("fuzz")
    # raw junk
    (d / "junk").write_bytes(blob)
    inspect(lib, d / "junk")
    # a valid file with a few bytes overwritten
    header = json.dumps({"a.m": {"dtype": "F32", "shape": [8], "data_offsets": [0, 32]},
                         "a.v": {"dtype": "F32", "shape": [8], "data_offsets": [32, 64]}, "__metadata__": META}).encode()
    good = bytearray(struct.pack("<Q", len(header)) + header + b"\0" * 64)
    for pos, val in flips:
        if pos < len(good):
            good[pos] = val
    (d / "mut").write_bytes(bytes(good))
    rc, kind, step, tensors, elements, _ = inspect(lib, d / "mut")
    if rc == 0:   # whatever was accepted must fit inside the file
        assert elements * 4 <= len(good)
