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


def test_a_part_can_bring_a_kernel_module_of_its_own(tmp_path):
    """``register_module``: a source outside the package, with headers of its own, known to
    ``ensure`` / ``build_all`` by name; its launch-list entry points are read from its source."""
    import pytest
    source, header = tmp_path / "mine.hip", tmp_path / "mine.h"
    header.write_text("#define MINE 1\n")
    source.write_text('#include "host.h"\n#include "mine.h"\n'
                      'BT_EXPORT int bt_mine_call(void* stream, const void* c) { return 0; }\n'
                      'BT_EXPORT int bt_other_thing_call (void* stream, const void* c) { return 0; }\n'
                      'BT_EXPORT int bt_mine(void* stream) { return 0; }\n')
    name = f"test_mine_{os.getpid()}"
    try:
        spec = build.register_module(name, str(source), flags=["-DX=1"], headers=[str(header)])
        assert build.register_module(name, str(source), flags=["-DX=1"], headers=[str(header)]) is spec   # again: a no-op
        with pytest.raises(ValueError, match="registered already"):
            build.register_module(name, str(source), flags=["-DX=2"], headers=[str(header)])
        assert name in build.all_modules() and "core" in build.all_modules()
        assert build.entry_points(name) == ["bt_mine_call", "bt_other_thing_call"]
        before = build._hash(name)
        header.write_text("#define MINE 2\n")             # a change to its own header rebuilds it
        assert build._hash(name) != before
    finally:
        build._registered.pop(name, None)
    with pytest.raises(ValueError, match="unknown kernel module"):
        build.module_spec(name)
    with pytest.raises(ValueError, match="no bfloat16 attention kernel for head size 24"):
        build.module_spec("attention_bf16_hd24")


def test_the_packages_own_modules_are_registered_like_any_other():
    for name in ("core", "gemm_mfma", "gemm_library", "program", "attention_f32", "attention_bf16_hd64"):
        assert build.module_spec(name).own
    assert "bt_gemm_skinny_call" in build.entry_points("gemm_mfma")
    assert build.module_spec("attention_bf16_hd96").flags == ("-DBT_HEAD_DIM=96",)
