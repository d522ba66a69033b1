"""Where compiled kernel libraries may be loaded from."""

import os

from burn_transformers_amd.kernels import build


def test_fallback_folder_must_be_ones_own_and_closed_to_others(tmp_path, monkeypatch):
    package_dir, fallback = str(tmp_path / "package"), str(tmp_path / "fallback")
    monkeypatch.setattr(build, "lib_dirs", lambda: [package_dir, fallback])
    os.makedirs(fallback, mode=0o777)
    os.chmod(fallback, 0o777)                      # somebody else could have put a library here
    with open(os.path.join(fallback, "core.so"), "w") as handle:
        handle.write("not a library")
    with open(os.path.join(fallback, "core.hash"), "w") as handle:
        handle.write("h")
    assert build._find("core", "h") is None and not build._writable(fallback)
    os.chmod(fallback, 0o700)
    assert build._find("core", "h") == os.path.join(fallback, "core.so") and build._writable(fallback)
    assert build._find("core", "another hash") is None
