"""The kernel library and its sources: a library built from other sources than those beside it is
never called (entry points gain parameters; an old binary would read shifted arguments)."""
import pytest

from bare_cuda_4gib_amd.csrc import build, library
from bare_cuda_4gib_amd.errors import KernelError


def test_the_built_library_carries_the_digest_of_its_sources():
    if not build.is_built():
        pytest.skip("the kernel library is not built here")
    assert len(build.sources_digest()) == 64
    assert build.built_digest() == build.sources_digest() and not build.is_stale()


def test_a_stale_library_is_rebuilt_or_refused(monkeypatch):
    if not build.is_built():
        pytest.skip("the kernel library is not built here")
    monkeypatch.setattr(library, "_lib", None)
    monkeypatch.setattr(build, "sources_digest", lambda: "0" * 64)          # as if a source had been edited
    assert build.is_stale()
    with pytest.raises(KernelError, match="other sources"):
        library.load(build_if_missing=False)
    monkeypatch.setattr(build, "can_build", lambda: False)                  # no compiler on this machine
    with pytest.raises(KernelError, match="other sources"):
        library.load()
    calls = []
    monkeypatch.setattr(build, "can_build", lambda: True)
    monkeypatch.setattr(build, "build", lambda verbose=True: calls.append(1))
    with pytest.raises(KernelError, match="digest"):                        # "rebuilt" (here: not really), checked again
        library.load()
    assert calls == [1]


def test_where_the_library_lives(monkeypatch, tmp_path):
    """Beside its sources, where that folder can be written or already holds a library of these sources; else in a
    folder that belongs to this user alone under the temporary folder -- and never in one that others can write."""
    import os
    import tempfile
    in_tree = (os.path.join(build.HERE, "_build"), os.path.join(build.HERE, "libbc4g.so"))
    monkeypatch.setattr(build, "BUILD_DIR", in_tree[0])
    monkeypatch.setattr(build, "LIB_PATH", in_tree[1])
    monkeypatch.setattr(tempfile, "tempdir", str(tmp_path))
    monkeypatch.setattr(os, "access", lambda path, mode: True)
    build._settle()
    assert (build.BUILD_DIR, build.LIB_PATH) == in_tree
    monkeypatch.setattr(os, "access", lambda path, mode: False)          # a checkout that belongs to someone else
    monkeypatch.setattr(build, "built_digest", lambda path="": build.sources_digest())
    build._settle()                                                      # ... with a library of these sources
    assert (build.BUILD_DIR, build.LIB_PATH) == in_tree
    monkeypatch.setattr(build, "built_digest", lambda path="": "")       # ... without
    build._settle()
    home = os.path.join(str(tmp_path), f"bc4g-{os.getuid()}")
    assert build.LIB_PATH == os.path.join(home, "libbc4g.so") and build.BUILD_DIR == os.path.join(home, "_build")
    assert os.stat(home).st_mode & 0o777 == 0o700
    monkeypatch.setattr(build, "BUILD_DIR", in_tree[0])
    monkeypatch.setattr(build, "LIB_PATH", in_tree[1])
    os.chmod(home, 0o777)
    with pytest.raises(KernelError, match="nowhere to build"):
        build._settle()
