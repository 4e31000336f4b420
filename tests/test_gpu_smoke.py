"""The driver's smoke entry and the loud failure when the native library is missing."""

import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_smoke_entry():
    sys.path.insert(0, ROOT)
    import __graft_entry__

    __graft_entry__.smoke()


def test_no_silent_fallback_when_the_kernel_library_cannot_be_loaded(tmp_path):
    """With an unloadable kernel library the engine raises; it never computes on another path."""
    code = (
        "import sys; sys.path.insert(0, %r)\n"
        "from mini_gpt_inference_amd.csrc import build\n"
        "build.ensure_kernels = lambda: %r\n"
        "from mini_gpt_inference_amd.ops import library\n"
        "try:\n"
        "    library.kernels()\n"
        "except library.NativeLibraryError as e:\n"
        "    print('LOUD', e)\n"
    ) % (ROOT, str(tmp_path / "missing.so"))
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert "LOUD" in proc.stdout and "cannot load native library" in proc.stdout
