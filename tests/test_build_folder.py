"""Where built kernel libraries are looked for: the source tree's own folder, and a folder under
the temp folder only if it is this user's alone."""
import os
import stat

import pytest

from kappai_amd.kernels import lib


def test_writable_tree_means_no_other_folder_is_consulted(monkeypatch, tmp_path):
    monkeypatch.setattr(lib, "CSRC", tmp_path)
    monkeypatch.setattr(lib.tempfile, "gettempdir", lambda: str(tmp_path / "tmp"))
    (tmp_path / "tmp").mkdir()
    hostile = tmp_path / "tmp" / f"kappai_amd_build_{os.getuid()}"
    hostile.mkdir()
    assert lib._build_dirs() == [tmp_path / "_build"]
    assert lib._writable_build_dir() == tmp_path / "_build"


def test_temp_folder_must_be_ours_alone(monkeypatch, tmp_path):
    monkeypatch.setattr(lib, "_dir_writable", lambda d: d.name != "_build" and os.access(d, os.W_OK))
    monkeypatch.setattr(lib, "CSRC", tmp_path)
    monkeypatch.setattr(lib.tempfile, "gettempdir", lambda: str(tmp_path / "tmp"))
    (tmp_path / "tmp").mkdir()
    d = tmp_path / "tmp" / f"kappai_amd_build_{os.getuid()}"
    # made by us: mode 0700
    assert lib._writable_build_dir() == d
    assert stat.S_IMODE(os.lstat(d).st_mode) == 0o700
    # a folder that others can write is refused, for building and for loading
    os.chmod(d, 0o777)
    with pytest.raises(lib.KernelBuildError, match="only they can write"):
        lib._writable_build_dir()
    with pytest.raises(lib.KernelBuildError, match="only they can write"):
        lib._find_built("gemm", "0" * 64)
    # so is a symbolic link in its place
    os.chmod(d, 0o700)
    d.rmdir()
    (tmp_path / "elsewhere").mkdir(mode=0o700)
    os.symlink(tmp_path / "elsewhere", d)
    with pytest.raises(lib.KernelBuildError, match="only they can write"):
        lib._writable_build_dir()
