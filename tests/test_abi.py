"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol that
include/difflogic_hip.h declares, the Python binding declares the same set, and argument
validation that happens before any launch returns the documented status codes."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "difflogic_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dl_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from difflogic_amd import _lib
    names = declared_symbols()
    assert "dl_logic_eval" in names and "dl_groupbitsum" in names and len(names) >= 9
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(_lib.SIGNATURES) == names
    assert _lib.load().dl_version() >= 100
    assert _lib.status_string(0) == "ok"
    assert "bit_count" in _lib.status_string(_lib.DL_ERR_BIT_COUNT)


def test_argument_validation_without_launch():
    from difflogic_amd import _lib
    lib = _lib.load()
    null = ctypes.c_void_p(0)
    one = ctypes.c_void_p(16)     # never dereferenced: every call below must fail before a launch
    assert lib.dl_logic_eval(one, one, one, one, one, 4, 4, 4, 12, null) == _lib.DL_ERR_BIT_COUNT
    assert lib.dl_logic_eval(null, one, one, one, one, 4, 4, 4, 64, null) == _lib.DL_ERR_INVALID_ARGUMENT
    assert lib.dl_logic_eval(one, one, one, one, one, 4, -1, 4, 64, null) == _lib.DL_ERR_INVALID_ARGUMENT
    assert lib.dl_logic_eval(null, null, null, null, null, 4, 0, 4, 64, null) == _lib.DL_OK      # empty: no work
    assert lib.dl_groupbitsum(one, one, 10, 4, 64, 0, 3, null) == _lib.DL_ERR_NOT_DIVISIBLE
    assert lib.dl_groupbitsum(one, one, 10, 4, 64, 0, 0, null) == _lib.DL_ERR_INVALID_ARGUMENT
    assert lib.dl_groupbitsum(one, one, 10, 4, 64, 257, 2, null) == _lib.DL_ERR_INVALID_ARGUMENT
    assert lib.dl_groupbitsum(one, one, 10, 4, 7, 0, 2, null) == _lib.DL_ERR_BIT_COUNT
    pad = ctypes.c_int64(-1)
    assert lib.dl_tensor_packbits(null, null, 3, 0, 32, ctypes.byref(pad), null) == _lib.DL_OK and pad.value == 0
    assert lib.dl_tensor_packbits(null, one, 3, 70, 32, ctypes.byref(pad), null) == _lib.DL_ERR_INVALID_ARGUMENT
    assert pad.value == 26
    assert lib.dl_tensor_packbits_batch_major(null, null, 0, 3, 64, ctypes.byref(pad), null) == _lib.DL_OK
    assert lib.dl_tensor_packbits(one, one, 3, 70, 5, None, null) == _lib.DL_ERR_BIT_COUNT
    assert lib.dl_logic_forward(one, one, one, one, one, 4, 4, 4, 9, null) == _lib.DL_ERR_DTYPE
    assert lib.dl_logic_forward(one, null, one, one, one, 4, 4, 4, _lib.DL_F32, null) == _lib.DL_ERR_INVALID_ARGUMENT
    assert lib.dl_logic_backward_w(one, one, one, one, null, 4, 4, 4, _lib.DL_F32, null) == _lib.DL_ERR_INVALID_ARGUMENT
    assert lib.dl_logic_backward_x(one, one, one, one, one, null, one, one, 4, 4, 4, 1.0, _lib.DL_F32,
                                   null) == _lib.DL_ERR_INVALID_ARGUMENT


def test_binding_rejects_cpu_tensors_and_bad_arguments():
    import torch

    from difflogic_amd import difflogic_cuda as ext
    x = torch.zeros(4, 2, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ext.eval(x, torch.zeros(3, dtype=torch.int64), torch.zeros(3, dtype=torch.int64), torch.zeros(3, dtype=torch.uint8))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ext.forward(torch.zeros(4, 2), torch.zeros(3, dtype=torch.int64), torch.zeros(3, dtype=torch.int64),
                    torch.zeros(3, 16))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ext.groupbitsum(x, 0, 2)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ext.tensor_packbits_cuda(torch.zeros(2, 8, dtype=torch.bool), 8)


def test_library_shares_torchs_hip_runtime_whatever_the_import_order():
    """Importing the package before torch must not bring a second HIP runtime into the process."""
    import subprocess
    import sys
    code = ("import difflogic_amd, torch\n"
            "libs = {l.split()[-1] for l in open('/proc/self/maps') if 'libamdhip64' in l}\n"
            "print(len(libs), sorted(libs))")
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert out.returncode == 0, out.stderr
    assert out.stdout.split()[0] == "1", out.stdout
