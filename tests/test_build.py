"""The build helpers that need no compiler."""
from concurrent.futures import ThreadPoolExecutor

from nanospec_amd.kernels import build


def test_every_thread_builds_into_the_same_folder(monkeypatch):
    """``build_all`` runs several compilers side by side; each asks where to build.  All of them get the folder beside the
    sources (a thread that found it unwritable by accident once built into the temporary folder and left a stale library
    behind)."""
    monkeypatch.setattr(build, "_build_dir_found", None)
    with ThreadPoolExecutor(max_workers=16) as pool:
        found = list(pool.map(lambda _: build._build_dir(), range(200)))
    assert len(set(found)) == 1
    assert found[0] == build.CSRC / "_build" or not (build.CSRC / "_build").exists()


def test_a_library_is_stale_when_a_header_or_a_flag_changes(tmp_path, monkeypatch):
    monkeypatch.setattr(build, "CSRC", tmp_path)
    (tmp_path / "a.hip").write_text("// a")
    (tmp_path / "h.h").write_text("// h")
    d0 = build._digest(["a.hip"], ["-DX=1"])
    assert d0 == build._digest(["a.hip"], ["-DX=1"])
    assert d0 != build._digest(["a.hip"], ["-DX=2"])
    (tmp_path / "h.h").write_text("// h changed")
    assert d0 != build._digest(["a.hip"], ["-DX=1"])
