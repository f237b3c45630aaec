"""CPU-only checks: the C-ABI library loads and exports every symbol that
include/nxhip.h declares (no compute calls without a GPU), the product fails
loudly without a device, and the host-side view algebra follows the
reference's (packages/nx/lib/core/view.ml)."""

import ctypes
import re
from pathlib import Path

import numpy as np
import pytest

from raven_amd import _ffi
from raven_amd import dtype as dt
from raven_amd.view import View

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols():
    text = (ROOT / "include" / "nxhip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nxh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _ffi.load()
    names = declared_symbols()
    assert len(names) >= 31
    for n in names:
        assert hasattr(lib, n), n
    assert set(names) == set(_ffi.SIGNATURES), set(names) ^ set(_ffi.SIGNATURES)


def test_descriptor_layout_matches_header():
    # void* + 2*int32 + int64 + 2 * 32 * int64
    assert ctypes.sizeof(_ffi.NxhTensor) == 8 + 8 + 8 + 2 * 32 * 8
    assert _ffi.NxhTensor.offset.offset == 16 and _ffi.NxhTensor.shape.offset == 24
    assert _ffi.NxhTensor.strides.offset == 24 + 32 * 8


def test_dtype_bytes_without_a_device():
    lib = _ffi.load()
    for d in dt.ALL:
        assert lib.nxh_dtype_bytes(d.tag, 7) == d.nbytes(7)
    assert lib.nxh_dtype_bytes(dt.int4.tag, 7) == 4
    assert lib.nxh_dtype_bytes(99, 1) == -1
    assert [d.tag for d in dt.ALL] == list(range(19))  # nx_c.h:197-200


def test_no_device_is_a_loud_failure_not_a_fallback():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from raven_amd.nx_backend import Backend

    with pytest.raises(RuntimeError, match="no HIP device"):
        Backend()


def test_view_algebra():
    v = View.create((64, 512, 512))
    p = v.permute((0, 2, 1))
    assert p.strides == (262144, 1, 512) and not p.is_c_contiguous()
    assert View.create((1, 512, 1)).expand((64, 512, 512)).strides == (0, 1, 0)
    assert View.create(()).expand((3, 4)).strides == (0, 0)
    s = v.shrink([(1, 3), (0, 512), (5, 9)])
    assert s.offset == 262144 + 5 and s.shape == (2, 512, 4)
    f = View.create((3, 4)).flip((True, False))
    assert f.offset == 8 and f.strides == (-4, 1)
    assert View.create((4, 6)).reshape((2, 2, 6)).strides == (12, 6, 1)
    t = View.create((4, 6)).permute((1, 0))
    assert t.reshape((6, 2, 2)).strides == (1, 12, 6)       # split of a strided dim
    assert t.reshape((1, 6, 4, 1)).strides == (0, 1, 6, 0)  # squeeze/unsqueeze only
    with pytest.raises(ValueError, match="call contiguous"):
        t.reshape((24,))
    with pytest.raises(ValueError):
        View.create((2, 3)).expand((4, 3))
    with pytest.raises(ValueError):
        View.create((2, 3)).permute((0, 0))
    with pytest.raises(ValueError):
        View.create((2, 3)).shrink([(0, 3), (0, 3)])
    assert View.create((3, 1, 5), (5, 99, 1)).is_c_contiguous()  # size-1 strides are free
    assert View.create((0, 3)).reshape((0,)).offset == 0
    # merging broadcast dims keeps them broadcast
    b = View.create((1, 1)).expand((3, 4))
    assert b.reshape((12,)).strides == (0,)


def test_scalar_encoding_matches_oracle_converters():
    from oracle.nx_oracle import lib
    from raven_amd.nx_backend import encode_scalar

    L = lib()
    for v in (0.0, 1.0, 0.5, -2.0, 1.00390625, 257.0, 3.14159, float("inf"), 1e-40):
        assert int(encode_scalar(dt.bfloat16, v)[0]) == L.nxo_f32_to_bf16(np.float32(v))
        with np.errstate(all="ignore"):
            assert int(encode_scalar(dt.float16, v).view(np.uint16)[0]) == L.nxo_f32_to_f16(np.float32(v))


@pytest.mark.gpu
def test_the_abi_from_plain_c():
    """tests/abi_c/nxh_abi_check.c drives the library the way the OCaml stubs do
    (dlopen, descriptors, statuses), with no Python or torch in the process, and
    checks every result against the same arithmetic on the host."""
    import subprocess

    from raven_amd import _ffi, build

    assert build.ABI_CHECK_BIN.exists(), "run __graft_entry__.build() first"
    r = subprocess.run([str(build.ABI_CHECK_BIN), str(_ffi.LIB_PATH)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and r.stdout.strip().endswith("all ok"), r.stdout + r.stderr
    assert "FAIL" not in r.stdout
