"""Where the kernel library may be loaded from: the tree, or a folder under the temporary directory that is
this user's alone."""
import os

from tessweave_engine_amd.kernels import build


def test_a_shared_temporary_folder_is_used_only_if_it_is_this_users_alone(tmp_path, monkeypatch):
    mine = tmp_path / "mine"
    monkeypatch.setattr(build, "_user_dir", lambda: mine)
    monkeypatch.setattr(build, "_in_tree_dir", lambda: tmp_path / "missing" / "tree")
    assert build.find_library() is None
    mine.mkdir(mode=0o700)
    (mine / build.library_name()).write_bytes(b"x")
    assert build.find_library() == mine / build.library_name()
    os.chmod(mine, 0o777)                                   # anyone could have put the file there
    assert build.find_library() is None
    os.chmod(mine, 0o700)
    link = tmp_path / "link"
    link.symlink_to(mine)                                   # a link is not a folder of ours
    monkeypatch.setattr(build, "_user_dir", lambda: link)
    assert build.find_library() is None
    # building goes to the private folder, created with mode 0700, when the tree cannot be written
    fresh = tmp_path / "fresh"
    monkeypatch.setattr(build, "_user_dir", lambda: fresh)
    blocked = tmp_path / "file"
    blocked.write_bytes(b"")
    monkeypatch.setattr(build, "_in_tree_dir", lambda: blocked / "sub")
    assert build._writable_dir() == fresh and (os.stat(fresh).st_mode & 0o777) == 0o700


def test_block_size_is_checked_when_the_engine_configuration_is_made():
    import pytest
    from tessweave_engine_amd.config import EngineConfig
    assert EngineConfig(block_size=12).block_size == 12
    with pytest.raises(ValueError, match="multiple of 4"):
        EngineConfig(block_size=6)
