"""Which built library is loaded (no GPU, nothing compiled): only one that was made from the sources
as they are, and from the temporary directory only out of a folder that is this user's alone."""
import os

import pytest

from torchless_rs_amd.kernels import build


def test_a_library_older_than_its_sources_is_built_again(tmp_path):
    lib = str(tmp_path / "lib.so")
    open(lib, "w").close()
    calls = []

    def rebuild():
        calls.append(1)
        return "fresh"

    assert build._current_or_rebuilt(lib, "abc", rebuild, "lib") == "fresh"         # no stamp at all
    build._write_stamp(lib, "abc")
    assert build._current_or_rebuilt(lib, "abc", rebuild, "lib") == lib and len(calls) == 1
    assert build._current_or_rebuilt(lib, "abd", rebuild, "lib") == "fresh" and len(calls) == 2
    assert build._current_or_rebuilt(None, "abc", rebuild, "lib") == "fresh"

    def cannot():
        raise build.ExtensionMissing("hipcc not found")

    with pytest.raises(build.ExtensionMissing, match="older than its sources"):
        build._current_or_rebuilt(lib, "abd", cannot, "lib")


def test_the_digest_follows_sources_and_flags(tmp_path):
    f = tmp_path / "k.hip"
    f.write_text("a")
    d0 = build._digest([str(f)], ["-O3"])
    assert d0 == build._digest([str(f)], ["-O3"]) and d0 != build._digest([str(f)], ["-O2"])
    f.write_text("b")
    assert d0 != build._digest([str(f)], ["-O3"])
    assert len({build.kernels_digest(), build.host_digest(), build.measure_digest()}) == 3


def test_the_measuring_kernels_are_no_part_of_the_library_that_a_step_loads():
    """What a model's first step compiles is what the model needs: the kernels that measure the
    machine's ceilings have a folder and a library of their own."""
    names = [os.path.basename(f) for f in build.sources()]
    assert names and "ceilings.hip" not in names
    assert [os.path.basename(f) for f in build.measure_sources()] == ["ceilings.hip"]
    assert build.LIB_NAME != build.MEASURE_LIB_NAME


def test_a_shared_folder_under_tmp_is_not_trusted(tmp_path):
    mine = tmp_path / "mine"
    mine.mkdir(mode=0o700)
    assert build._own_private_dir(str(mine))
    os.chmod(mine, 0o777)
    assert not build._own_private_dir(str(mine))
    assert not build._own_private_dir(str(tmp_path / "absent"))


def test_a_current_library_in_the_private_folder_goes_before_a_stale_one_in_the_package(tmp_path, monkeypatch):
    """A package folder that cannot be written keeps its stale library for good; the current one that an
    earlier process built into the private folder must be found, not built again by every process."""
    pkg, private = tmp_path / "pkg", tmp_path / "private"
    pkg.mkdir()
    private.mkdir(mode=0o700)
    monkeypatch.setattr(build, "build_dirs", lambda: [str(pkg), str(private)])
    stale, fresh = str(pkg / "lib.so"), str(private / "lib.so")
    open(stale, "w").close()
    build._write_stamp(stale, "old")
    assert build.built_library("lib.so", "new") == stale          # nothing current anywhere: the first found
    open(fresh, "w").close()
    build._write_stamp(fresh, "new")
    assert build.built_library("lib.so", "new") == fresh
    assert build.built_library("lib.so") == stale                  # without a digest: the order of preference
    assert build.built_library("lib.so", "old") == stale
    os.chmod(private, 0o777)                                        # a folder others can write to is never looked into
    assert build.built_library("lib.so", "new") == stale
    os.remove(stale)
    assert build.built_library("lib.so", "new") is None
