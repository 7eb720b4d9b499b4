"""The kernel library's build script: where it may put (and find) a built library."""
import importlib.util
import os
import stat
import tempfile

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def build_module():
    path = os.path.join(HERE, "..", "hector-engine_amd", "csrc", "build.py")
    spec = importlib.util.spec_from_file_location("_hector_csrc_build_for_test", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_private_folder_is_created_for_this_user_only(tmp_path, monkeypatch):
    monkeypatch.setattr(tempfile, "tempdir", str(tmp_path))
    b = build_module()
    folder = b.private_folder()
    st = os.stat(folder)
    assert folder.startswith(str(tmp_path)) and st.st_uid == os.getuid()
    assert stat.S_IMODE(st.st_mode) == 0o700
    assert b.private_folder() == folder        # a second call finds it again


def test_a_folder_others_may_write_is_refused(tmp_path, monkeypatch):
    """A library found in the fallback folder is loaded as code: a folder of that name that anyone may
    write to is not trusted, and the candidates for a build then leave it out."""
    monkeypatch.setattr(tempfile, "tempdir", str(tmp_path))
    b = build_module()
    planted = tmp_path / f"hector-engine_amd-{os.getuid()}"
    planted.mkdir()
    os.chmod(planted, 0o777)
    with pytest.raises(RuntimeError, match="not a private folder"):
        b.private_folder()
    assert b._candidate_dirs() == [b.CSRC]


def test_the_hash_follows_sources_and_flags():
    b = build_module()
    h = b.source_hash()
    assert h == b.source_hash() and len(h) == 64
    flags = list(b.HIPCC_FLAGS)
    try:
        b.HIPCC_FLAGS.append("-DX")
        assert b.source_hash() != h
    finally:
        b.HIPCC_FLAGS[:] = flags
    # packed fp32 instructions stay switched off for all device code
    assert "-packed-fp32-ops" in " ".join(b.HIPCC_FLAGS)
