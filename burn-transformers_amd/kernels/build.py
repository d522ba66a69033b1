"""Compiles the HIP sources under ``csrc/`` for gfx950, one shared library per kernel module.

A module is one ``.hip`` file plus compile-time definitions (the bfloat16 attention is built
once per head size).  Libraries are kept in ``_lib/`` inside the package, or in a per-user
folder below the system's temporary directory when the package folder is not writable.  A
library is rebuilt when the hash of its sources and flags changes, so a run compiles exactly
the modules it needs and a stale library is never loaded.
"""

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

PACKAGE_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC_DIR = os.path.join(PACKAGE_DIR, "csrc")
ARCH = "gfx950"
# -packed-fp32-ops is switched off for every kernel: some packed 32-bit forms have produced
# wrong values on this hardware generation.
FLAGS = ["-O3", "-std=c++17", "--offload-arch=" + ARCH, "-fPIC", "-shared",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
ATTENTION_HEAD_SIZES = tuple(range(16, 129, 16))


class ModuleSpec:
    """One kernel module: a source file, the definitions and link options it is compiled with, and
    headers of its own beside the package's (which every module may include)."""

    def __init__(self, name, source, flags=(), headers=(), own=False):
        self.name, self.source, self.flags, self.headers, self.own = name, source, tuple(flags), tuple(headers), own

    def same_as(self, other):
        return (self.source, self.flags, self.headers) == (other.source, other.flags, other.headers)


_registered = {}
_registry_lock = threading.Lock()


def register_module(name, source, flags=(), headers=(), _own=False):
    """Makes a kernel module known under ``name``: ``ensure`` compiles it when it is first needed,
    ``build_all`` compiles it with the package's own, ``kernels.library`` loads it and types every
    ``bt_*_call(stream, structure)`` entry point its source defines.  This is how a part brings
    kernels of its own, without a change to the package.

    source: the ``.hip`` / ``.cpp`` file (absolute, or relative to the package's ``csrc/``); it may
    include the package's headers (``common.h``, ``host.h`` for error reporting, ``calls.h``, ...).
    flags: definitions (``-DNAME=1``) and link options (``-lfoo``) beyond the package's own.
    headers: further files the source includes; a change to any of them rebuilds the module.
    Registering a name again with the same description is a no-op; with another it is an error."""
    if not os.path.isabs(source):
        source = os.path.join(CSRC_DIR, source)
    spec = ModuleSpec(name, source, flags, [os.path.abspath(h) for h in headers], _own)
    with _registry_lock:
        held = _registered.get(name)
        if held is not None and not held.same_as(spec):
            raise ValueError(f"kernel module {name!r} is registered already, from {held.source}")
        _registered[name] = held or spec
    return _registered[name]


def module_spec(name):
    spec = _registered.get(name)
    if spec is None:
        if name.startswith("attention_bf16_hd"):
            raise ValueError(
                f"no bfloat16 attention kernel for head size {name[len('attention_bf16_hd'):]}: "
                f"sizes {ATTENTION_HEAD_SIZES[0]}..{ATTENTION_HEAD_SIZES[-1]} in steps of 16 are built")
        raise ValueError(f"unknown kernel module {name!r}; registered: {sorted(_registered)}")
    return spec


def package_headers():
    """Every header of the package's ``csrc/``: each is part of every module's hash."""
    return sorted(os.path.join(CSRC_DIR, f) for f in os.listdir(CSRC_DIR) if f.endswith(".h"))


def entry_points(name):
    """The ``bt_*_call`` entry points a module's source defines (its launch-list forms)."""
    import re
    with open(module_spec(name).source, errors="replace") as handle:
        return sorted(set(re.findall(r"\b(bt_\w+_call)\s*\(", handle.read())))


# the package's own modules
for _name in ("core", "gemm_mfma", "attention_f32"):
    register_module(_name, _name + ".hip", _own=True)
register_module("gemm_library", "gemm_library.hip", ["-ldl"], _own=True)   # host code around hipBLASLt, opened at run time
register_module("program", "program.cpp", _own=True)                       # the host loop that walks a launch list
for _size in ATTENTION_HEAD_SIZES:                                         # the bfloat16 attention, once per head size
    register_module(f"attention_bf16_hd{_size}", "attention_bf16.hip", [f"-DBT_HEAD_DIM={_size}"], _own=True)


def all_modules():
    """Every registered module: the package's own and what parts have brought so far."""
    return list(_registered)


def _hash(name):
    spec = module_spec(name)
    digest = hashlib.sha256()
    for path in package_headers() + list(spec.headers) + [spec.source]:
        with open(path, "rb") as handle:
            digest.update(handle.read())
    digest.update(" ".join(FLAGS + list(spec.flags)).encode())
    return digest.hexdigest()


def _own_private(path):
    """True for a folder that belongs to this user and that nobody else can write to.  The
    per-user fallback has a name anyone can guess and lies in a folder everyone can write to:
    a library found there is loaded into this process, so a folder that somebody else made, or
    can write to, is never read from and never written to."""
    try:
        status = os.stat(path, follow_symlinks=False)
    except OSError:
        return False
    import stat
    return stat.S_ISDIR(status.st_mode) and status.st_uid == os.getuid() and not (status.st_mode & 0o022)


def _writable(path):
    try:
        os.makedirs(path, mode=0o700, exist_ok=True)
        if path == lib_dirs()[1] and not _own_private(path):
            return False
        probe = os.path.join(path, f".probe-{os.getpid()}-{threading.get_ident()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def lib_dirs():
    """Places a library may be in: the package first, then the per-user fallback."""
    fallback = os.path.join(tempfile.gettempdir(), f"burn_transformers_amd-{os.getuid()}")
    return [os.path.join(PACKAGE_DIR, "_lib"), fallback]


def _find(name, wanted_hash):
    package_dir, fallback = lib_dirs()
    for folder in (package_dir, fallback):
        if folder == fallback and not _own_private(folder):
            continue
        lib = os.path.join(folder, name + ".so")
        stamp = os.path.join(folder, name + ".hash")
        try:
            with open(stamp) as handle:
                if handle.read().strip() == wanted_hash and os.path.exists(lib):
                    return lib
        except OSError:
            continue
    return None


def hipcc():
    for candidate in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.exists(candidate):
            return candidate
    raise RuntimeError("hipcc was not found: the HIP kernels of burn_transformers_amd cannot be built")


def compile_module(name, verbose=True):
    """Compiles one module and returns the path of its library."""
    spec = module_spec(name)
    target_dir = next((d for d in lib_dirs() if _writable(d)), None)
    if target_dir is None:
        raise RuntimeError(f"no writable folder for compiled kernels among {lib_dirs()}")
    lib = os.path.join(target_dir, name + ".so")
    partial = os.path.join(target_dir, f".{name}.{os.getpid()}.{threading.get_ident()}.so")
    options = [d for d in spec.flags if not d.startswith("-l")]
    libraries = [d for d in spec.flags if d.startswith("-l")]
    command = [hipcc()] + FLAGS + ["-I", CSRC_DIR] + options + ["-o", partial, spec.source] + libraries
    if verbose:
        print(f"[burn_transformers_amd] compiling {name} for {ARCH} ...", file=sys.stderr, flush=True)
    started = time.time()
    done = threading.Event()

    def heartbeat():
        while not done.wait(10.0):
            print(f"[burn_transformers_amd] still compiling {name} ({time.time() - started:.0f} s)",
                  file=sys.stderr, flush=True)

    if verbose:
        threading.Thread(target=heartbeat, daemon=True).start()
    try:
        env = dict(os.environ)
        env.setdefault("HOME", tempfile.gettempdir())
        result = subprocess.run(command, capture_output=True, text=True, env=env)
    finally:
        done.set()
    if result.returncode != 0:
        noise = "is not a recognized feature for this target"
        message = "\n".join(l for l in (result.stdout + result.stderr).splitlines() if noise not in l)
        raise RuntimeError(f"hipcc failed for {name}:\n{message}")
    os.replace(partial, lib)
    with open(os.path.join(target_dir, name + ".hash"), "w") as handle:
        handle.write(_hash(name))
    if verbose:
        print(f"[burn_transformers_amd] compiled {name} in {time.time() - started:.1f} s",
              file=sys.stderr, flush=True)
    return lib


def ensure(name, verbose=True):
    """Path of an up-to-date library of the module, compiling it if there is none."""
    found = _find(name, _hash(name))
    return found if found else compile_module(name, verbose)


def ensure_many(names, verbose=True, jobs=8):
    """The same for several modules; those that have to be compiled are compiled side by side."""
    from concurrent.futures import ThreadPoolExecutor
    missing = [name for name in dict.fromkeys(names) if _find(name, _hash(name)) is None]
    if len(missing) > 1:
        with ThreadPoolExecutor(max_workers=min(jobs, len(missing))) as pool:
            list(pool.map(lambda n: compile_module(n, verbose), missing))
    return {name: ensure(name, verbose) for name in names}


def build_all(verbose=True, jobs=8):
    """Compiles every registered module anew (the build check of the repository)."""
    from concurrent.futures import ThreadPoolExecutor
    names = all_modules()
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        return dict(zip(names, pool.map(lambda n: compile_module(n, verbose), names)))
