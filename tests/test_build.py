"""Where the kernel library may be written to and loaded from (no compiler involved)."""

from __future__ import annotations

import os

from tinyserve_llm_amd.csrc import build


def test_a_fallback_folder_must_be_the_users_own(tmp_path, monkeypatch):
    """The per-user folder under the shared temporary directory has a name anyone can guess, and a
    library found in it is loaded into the process: it is made closed to others, and one that is
    open to others, or is a link to somewhere else, is neither searched nor written to."""
    mine = tmp_path / "mine"
    assert build._usable(str(mine), create=True) and (os.stat(mine).st_mode & 0o777) == 0o700
    assert build._usable(str(mine), create=False)
    shared = tmp_path / "shared"
    shared.mkdir()
    os.chmod(shared, 0o777)
    assert not build._usable(str(shared), create=False) and not build._usable(str(shared), create=True)
    link = tmp_path / "link"
    link.symlink_to(mine)
    assert not build._usable(str(link), create=False)
    assert not build._usable(str(tmp_path / "missing"), create=False)
    # a library with the right stamp in a folder that is open to others is not found
    monkeypatch.setattr(build, "candidate_dirs", lambda: [str(shared)])
    (shared / build.LIB_NAME).write_bytes(b"")
    (shared / (build.LIB_NAME + ".hash")).write_text(build.source_hash())
    assert build.find_current() is None
    os.chmod(shared, 0o700)
    assert build.find_current() == str(shared / build.LIB_NAME)


def test_the_source_folder_is_taken_as_it_is():
    assert build.candidate_dirs()[0] == build.HERE and build._usable(build.HERE, create=False)
