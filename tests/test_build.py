"""The native libraries are rebuilt when a source has changed since they were built (CPU, with a
stubbed compiler)."""

import os

from mini_gpt_inference_amd.csrc import build


def _sandbox(tmp_path, monkeypatch):
    hip = tmp_path / "hip"
    hip.mkdir()
    (hip / "a.hip").write_text("// kernel a\n")
    (hip / "common.h").write_text("// header\n")
    lib = tmp_path / "libmgpt_kernels.so"
    monkeypatch.setattr(build, "HIP_DIR", str(hip))
    monkeypatch.setattr(build, "KERNEL_LIB", str(lib))
    monkeypatch.setattr(build, "_find", lambda tool, extra=(): tool)
    calls = []

    def fake_run(cmd, what):
        calls.append(what)
        out = cmd[cmd.index("-o") + 1]
        with open(out, "wb") as fh:
            fh.write(b"built")

    monkeypatch.setattr(build, "_run", fake_run)
    return hip, lib, calls


def test_ensure_builds_once_and_again_after_a_source_or_header_changed(tmp_path, monkeypatch):
    hip, lib, calls = _sandbox(tmp_path, monkeypatch)
    assert build.ensure_kernels() == str(lib) and os.path.isfile(lib)
    first = len(calls)
    assert first > 0
    assert build.ensure_kernels() == str(lib)
    assert len(calls) == first, "nothing changed: nothing is compiled"
    (hip / "common.h").write_text("// header, edited\n")
    build.ensure_kernels()
    assert len(calls) == 2 * first, "a changed header makes the library stale"
    (hip / "a.hip").write_text("// kernel a, edited\n")
    build.ensure_kernels()
    assert len(calls) == 3 * first
    # the same text again under a new modification time is no change
    os.utime(hip / "a.hip", (1, 1))
    build.ensure_kernels()
    assert len(calls) == 3 * first


def test_a_library_without_its_digest_counts_as_stale(tmp_path, monkeypatch):
    hip, lib, calls = _sandbox(tmp_path, monkeypatch)
    lib.write_bytes(b"from somewhere")
    build.ensure_kernels()
    assert calls, "a library of unknown origin is rebuilt"
    assert build.is_current(str(lib), build.sources_digest(build.kernel_sources(), build.HIP_FLAGS))
