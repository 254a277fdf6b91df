"""The argument types that the Python side sets on the HIP library's entry points are read from the sources:
every entry point must be read, with the types its declaration has."""
import ctypes

import pytest


def test_signatures_are_read_from_the_sources():
    from inferx_amd.csrc import build
    sig = build.signatures()
    assert len(sig) >= 30 and all(name.startswith("ix_") for name in sig)
    p, i, q, f = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
    # int ix_embed(void* h, const void* table, int dtype, const int32_t* ids, int64_t tokens, int64_t width,
    #              int64_t rows, float scale, hipStream_t stream)
    assert sig["ix_embed"] == (i, [p, p, i, p, q, q, q, f, p])
    assert sig["ix_last_error"] == (ctypes.c_char_p, [])
    assert sig["ix_abi_version"] == (i, [])
    # the entry point that allocates nothing is the other one without its workspace arguments
    with_ws, without = sig["ix_attention_mfma"][1], sig["ix_attention_mfma_noalloc"][1]
    assert len(with_ws) == len(without) + 2 and with_ws[-3:] == without[-3:]
    # a double* (the flops that a probe reports) and a stream are pointers
    assert sig["ix_probe_mfma"] == (i, [i, i, p, p, p])


def test_every_declared_entry_point_is_read():
    import os
    import re
    from inferx_amd.csrc import build
    declared = set()
    for name in build.sources():
        with open(os.path.join(build.HERE, name)) as fh:
            declared |= set(re.findall(r'extern\s+"C"[^(;{]*?\b(ix_\w+)\s*\(', fh.read()))
    assert declared == set(build.signatures())


def test_a_missing_compiler_or_a_stale_library_is_said_plainly(monkeypatch):
    """Without hipcc the build fails with an error that says where it looked; a library built from other sources
    than the present ones is not taken."""
    from inferx_amd.csrc import build
    monkeypatch.setattr(build, "_digest", lambda: "not-the-digest-of-any-build")
    assert build.find_built() is None
    monkeypatch.undo()
    monkeypatch.setenv("HIPCC", "/nonexistent/hipcc")
    monkeypatch.setattr(build.shutil, "which", lambda name: None)
    monkeypatch.setattr(build.os.path, "isfile", lambda p: False)
    with pytest.raises(build.BuildError, match="hipcc not found"):
        build.build(verbose=False)
