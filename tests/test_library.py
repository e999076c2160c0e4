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
