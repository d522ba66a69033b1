"""ctypes bindings of the HIP kernel modules.

Every function here launches kernels on torch's current HIP stream and takes torch tensors
on the GPU.  There is no fallback: a module that cannot be built or loaded raises, and a size
that a kernel does not take raises :class:`KernelError` with the kernel's own message.
"""

import ctypes
import os
import sys
import threading

import torch  # imported first: the kernel libraries bind to the HIP runtime torch has loaded

from . import build

FLOAT32, BFLOAT16 = 0, 1
DTYPE_CODES = {torch.float32: FLOAT32, torch.bfloat16: BFLOAT16}

EPI_STORE, EPI_ACT, EPI_F32, EPI_QKV, EPI_RESIDUAL = 0, 1, 2, 3, 4
ACTIVATIONS = {"gelu_tanh": 0, "gelu_erf": 1}
NORM_KINDS = {"layer_norm": 0, "rms_norm": 1}
KV_BLOCK = 64

_c_int, _c_i64, _c_ptr, _c_float, _c_u64 = (ctypes.c_int, ctypes.c_int64, ctypes.c_void_p,
                                           ctypes.c_float, ctypes.c_uint64)


class KernelError(RuntimeError):
    """A kernel refused its operands or a launch failed."""


class KvView(ctypes.Structure):
    """One layer of one group of the paged key/value storage, as the kernels see it."""
    _fields_ = [("keys", _c_ptr), ("values", _c_ptr), ("blocks", _c_ptr),
                ("max_blocks", _c_int), ("kv_heads", _c_int), ("head_dim", _c_int),
                ("block_stride", _c_i64), ("head_stride", _c_i64)]


class Epilogue(ctypes.Structure):
    _fields_ = [("mode", _c_int), ("act", _c_int), ("bias", _c_ptr), ("out", _c_ptr),
                ("ldo", _c_i64), ("split_stride", _c_i64), ("n_q", _c_int), ("n_kv", _c_int),
                ("tok_seq", _c_ptr), ("tok_pos", _c_ptr), ("kv", KvView), ("out_rows", _c_int)]


class AttnArgs(ctypes.Structure):
    _fields_ = [("q", _c_ptr), ("ldq", _c_i64), ("out", _c_ptr), ("ldo", _c_i64),
                ("tok_seq", _c_ptr), ("tok_pos", _c_ptr), ("seq_off", _c_ptr), ("seq_start", _c_ptr),
                ("kv", KvView), ("q_heads", _c_int), ("n_tokens", _c_int), ("n_seqs", _c_int),
                ("max_count", _c_int), ("window", _c_int), ("scale", _c_float), ("splits", _c_int),
                ("partial", _c_ptr), ("out_rows", _c_int)]


class NormOperand(ctypes.Structure):
    _fields_ = [("x", _c_ptr), ("ldx", _c_i64), ("gamma", _c_ptr), ("beta", _c_ptr), ("eps", _c_float),
                ("kind", _c_int)]


class EmbedCall(ctypes.Structure):
    _fields_ = [("dtype", _c_int), ("tokens", _c_int), ("width", _c_int), ("ids", _c_ptr), ("pos", _c_ptr),
                ("table", _c_ptr), ("positions", _c_ptr), ("out", _c_ptr)]


class AddNormCall(ctypes.Structure):
    _fields_ = [("out_dtype", _c_int), ("n_delta", _c_int), ("kind", _c_int), ("n_rows", _c_int), ("width", _c_int),
                ("write_back", _c_int), ("out_rows", _c_int), ("eps", _c_float), ("x", _c_ptr), ("delta", _c_ptr),
                ("delta_stride", _c_i64), ("bias", _c_ptr), ("gamma", _c_ptr), ("beta", _c_ptr), ("out", _c_ptr),
                ("rows", _c_ptr)]


class GemmCall(ctypes.Structure):
    _fields_ = [("dtype", _c_int), ("M", _c_int), ("N", _c_int), ("K", _c_int), ("splits", _c_int), ("variant", _c_int),
                ("packed_columns", _c_int), ("a_rows", _c_int), ("has_norm", _c_int), ("A", _c_ptr), ("lda", _c_i64),
                ("W", _c_ptr), ("epi", Epilogue), ("norm", NormOperand)]


class AttentionCall(ctypes.Structure):
    _fields_ = [("dtype", _c_int), ("args", AttnArgs)]


class KvCopyCall(ctypes.Structure):
    _fields_ = [("dtype", _c_int), ("tokens", _c_int), ("to_cache", _c_int), ("k_rows", _c_ptr), ("v_rows", _c_ptr),
                ("ld", _c_i64), ("tok_seq", _c_ptr), ("tok_pos", _c_ptr), ("kv", KvView)]


class LaunchEntry(ctypes.Structure):
    _fields_ = [("call", _c_ptr), ("args", _c_ptr)]


class Chunked:
    """Activations of a step of few rows kept chunk-major: the chunks of 64 bytes of the columns (32
    bfloat16 or 16 float32 values) one after the other, each with that chunk of every row,
    [columns / chunk][rows][chunk] (``activation_offset`` in csrc/common.h).  The skinny product
    reads its rows sixteen at a time, 64 bytes of each: from row-major rows those lie a whole row
    apart, from this layout they are one contiguous KiB (for 64 rows of 1,600 columns a work-group
    needs 1 us instead of 5.8 us to read them).  Written by the norm kernel, the decode attention
    kernel and the products' store / activation epilogues; read by the skinny product only.  It
    stands where a tensor [rows, columns] would; whoever only hands it on to ``gemm``, ``add_norm``
    or ``attention_args`` needs to know nothing of it."""

    # Steps of 9 to 64 rows use it.  Up to 8 rows it loses: the norm's rows are written by one
    # work-group each, and two rows share every 128-byte line of a chunk (measured at 8 rows: the
    # norm 4.0 -> 4.6 us, the products behind it 6.3 -> 6.8 us; at 64 rows a step gains 5 %).
    # Measured as ms a decode step, row-major / chunk-major, at three widths (12 layers of width 768,
    # 24 of 1,024, 12 of 1,600): 12 rows 0.413 / 0.406, 0.837 / 0.823, 0.619 / 0.611; 16 rows
    # 0.433 / 0.423, 0.908 / 0.888, 0.654 / 0.638.
    MIN_ROWS, MAX_ROWS = 9, 64
    enabled = True        # tests switch it off to compare with row-major activations

    @classmethod
    def wanted(cls, rows):
        return cls.enabled and cls.MIN_ROWS <= rows <= cls.MAX_ROWS

    def __init__(self, data, rows, columns):
        self.data, self.shape = data, (rows, columns)
        self.dtype, self.device = data.dtype, data.device

    @classmethod
    def take(cls, step, key, rows, columns, dtype):
        """A chunk-major buffer [rows, columns] from the step's workspace."""
        chunk = 64 // (2 if dtype == torch.bfloat16 else 4)
        padded = (columns + chunk - 1) // chunk * chunk
        return cls(step.buffer(key + ".chunked", rows, padded, dtype), rows, columns)

    def to_rows(self):
        """The same values as a row-major tensor (tests)."""
        rows, columns = self.shape
        chunk = 64 // self.data.element_size()
        return self.data.view(-1, rows, chunk).permute(1, 0, 2).reshape(rows, -1)[:, :columns]

    def stride(self, dim):
        return self.shape[1] if dim == 0 else 1

    def data_ptr(self):
        return self.data.data_ptr()


class Normalized:
    """Rows of the float32 residual stream that are still to be normalised: handed to ``gemm`` in
    place of its activations, the skinny product kernel normalises them itself (up to 16 rows of
    bfloat16 products, width up to 2048), which saves the norm's own kernel in front of it."""

    MAX_ROWS, MAX_WIDTH = 16, 2048          # what the kernel takes
    # What pays: every work-group normalises all rows, a wave one row after the other from nine rows
    # on, so the fold is worth it while a wave has at most this many elements to normalise; beyond,
    # the norm as a kernel of its own in front of an ordinary product is faster again.  Measured as
    # ms a decode step with the norm folded up to 8 rows / up to 16 rows: width 768 (12 layers) 0.425 /
    # 0.413 at batch 12 and 0.438 / 0.433 at 16; width 1,024 (24 layers) 0.847 / 0.837 and 0.908 / 0.908;
    # width 1,600 (12 layers) 0.651 / 0.666 at batch 12 and 0.681 / 0.724 at 16.
    WORTH_ELEMENTS = 2048

    def __init__(self, x, gamma, beta, eps, kind):
        self.x, self.gamma, self.beta, self.eps, self.kind = x, gamma, beta, eps, kind
        self.shape = x.shape
        self.dtype = torch.bfloat16
        self.device = x.device

    @classmethod
    def possible(cls, rows, width):
        """Whether the kernel takes such rows."""
        return rows <= cls.MAX_ROWS and width <= cls.MAX_WIDTH and width % 8 == 0

    @classmethod
    def worth_it(cls, rows, width):
        """Whether a norm in front of a product should be folded into it."""
        return cls.possible(rows, width) and (rows + 7) // 8 * width <= cls.WORTH_ELEMENTS


# Every kernel of a step is called through its structure form, bt_<kernel>_call(stream, structure)
# (csrc/calls.h): the same pair can be called now or kept in a launch list (:class:`Program`).  A
# module's entry points of that form are found in its source when it is loaded (``build.entry_points``).

_modules = {}
_lock = threading.Lock()


def _module(name):
    lib = _modules.get(name)          # (a dict read is atomic; the lock is for building and loading)
    if lib is not None:
        return lib
    with _lock:
        lib = _modules.get(name)
        if lib is None:
            path = build.ensure(name)
            try:
                lib = ctypes.CDLL(path)
            except OSError as error:
                raise RuntimeError(f"cannot load the kernel library {path}: {error}") from error
            if hasattr(lib, "bt_last_error"):
                lib.bt_last_error.restype = ctypes.c_char_p
            for entry in build.entry_points(name):
                if hasattr(lib, entry):
                    getattr(lib, entry).argtypes = [_c_ptr, _c_ptr]
            _modules[name] = lib
        return lib


def _check(lib, code):
    if code != 0:
        raise KernelError(lib.bt_last_error().decode() if hasattr(lib, "bt_last_error")
                          else f"a kernel module's entry point returned {code}")


register_module = build.register_module      # how a part brings kernels of its own: see there


def launch(module, entry, call):
    """Calls ``entry`` (an entry point ``int bt_*_call(void* stream, const Structure*)``) of the
    registered module ``module`` with the ctypes structure ``call``, on the current stream: now,
    or, while a launch list is being recorded, as one more call of that list.  The structure must
    name only addresses that stay where they are (weights, the step's workspaces and tables)."""
    _launch(_module(module), entry, call)


class _Recorder(threading.local):
    """The Program that this thread's kernel calls are being written into, if any: a list records
    what the thread that opened it issues, and nothing that another thread launches meanwhile."""
    program = None


_recorder = _Recorder()


def _launch(lib, name, call):
    """Calls a kernel's structure form now, or, while a launch list is being recorded, keeps the
    pair for later."""
    program = _recorder.program
    if program is not None:
        program.add(lib, name, call)
        if not program.launch_while_recording:
            return
    _check(lib, getattr(lib, name)(_stream(), ctypes.byref(call)))


# The fields of the call structures that hold a step's number of tokens ("tokens") or the most tokens
# one of its sequences brings ("max_count"): what differs between the launch lists of two steps of
# one class (``engine.step.token_capacity``).  A part that brings a kernel of its own says the same of
# its structure with a class attribute ``_step_fields_ = {"field": "tokens"}``; a structure that says
# nothing keeps a list from serving any step but the one it was recorded for.
def _step_fields(call):
    kind = type(call)
    if kind is GemmCall:
        return (("M", "tokens"),)
    if kind is AddNormCall:
        return () if call.rows else (("n_rows", "tokens"),)        # (with a selection of rows: the wanted rows)
    if kind is EmbedCall or kind is KvCopyCall:
        return (("tokens", "tokens"),)
    if kind is AttentionCall:
        return (("args.n_tokens", "tokens"), ("args.max_count", "max_count"))
    declared = getattr(kind, "_step_fields_", None)
    return None if declared is None else tuple(declared.items())


def _field(call, path):
    """(the structure that holds the field, its name) of a dotted path."""
    *outer, name = path.split(".")
    for part in outer:
        call = getattr(call, part)
    return call, name


class Program:
    """A launch list: the kernel calls of one step, in order, each as (entry point, argument
    structure).  ``run`` hands the whole list to one C++ loop (csrc/program.cpp), so a step costs
    the host one call from Python plus the launches themselves.

        program = Program()
        with program.recording():
            model.forward(step, cache)        # nothing is launched; every kernels.library call is kept
        program.run()                         # launches them all, now and as often as wanted

    ``recording(launch=True)`` keeps the calls AND launches each as it comes: the first step of a
    shape then starts on the GPU at once, as it would without a list, and leaves its list behind.

    What the list holds is only addresses and sizes: it stays valid as long as every buffer, table
    and weight it names stays where it is, and gives the same results as calling the kernels one
    by one, bit for bit (they are the same calls)."""

    def __init__(self):
        self.calls = []             # (module, entry point name, structure); the structures are kept alive here
        self._entries = None
        self.launch_while_recording = False
        self.patches = None         # see ``for_any_step_of_its_class``
        self.shape = None           # (tokens, max_count) the structures hold now

    def for_any_step_of_its_class(self, tokens, max_count, wanted_rows):
        """Finds the fields of the list's calls that hold the step's counts, so that the list can
        be run for another step of the same class (``set_shape``).  ``tokens``, ``max_count`` and
        ``wanted_rows`` are those of the step it was recorded for.  Returns False, and leaves the
        list good for steps of exactly that shape only, if a call does not say which of its fields
        they are, or holds a row count that is neither the step's tokens nor its wanted rows (or
        could be either)."""
        patches = []
        for _, _, call in self.calls:
            fields = _step_fields(call)
            if fields is None:
                return False
            for path, what in fields:
                holder, name = _field(call, path)
                value = getattr(holder, name)
                if what == "max_count":
                    if value != max_count:
                        return False
                elif value == tokens and tokens != wanted_rows:
                    pass
                elif value == wanted_rows and tokens != wanted_rows and type(call) is GemmCall:
                    continue                   # the readout's product: its rows are the wanted ones
                else:
                    return False
                patches.append((holder, name, what))
        self.patches, self.shape = patches, (tokens, max_count)
        return True

    def set_shape(self, tokens, max_count):
        """Makes the list that of a step of ``tokens`` tokens, ``max_count`` at most of one sequence."""
        if self.shape != (tokens, max_count):
            for holder, name, what in self.patches:
                setattr(holder, name, tokens if what == "tokens" else max_count)
            self.shape = (tokens, max_count)

    def add(self, lib, name, call):
        self.calls.append((lib, name, call))
        self._entries = None

    def recording(self, launch=False):
        self.launch_while_recording = launch
        return _Recording(self)

    def __len__(self):
        return len(self.calls)

    def _freeze(self):
        entries = (LaunchEntry * max(len(self.calls), 1))()
        for i, (lib, name, call) in enumerate(self.calls):
            entries[i].call = ctypes.cast(getattr(lib, name), _c_ptr).value
            entries[i].args = ctypes.addressof(call)
        self._entries = entries

    def run(self):
        """Launches every call of the list on the current stream."""
        if self._entries is None:
            self._freeze()
        runner = _module("program")
        failed = _c_int(-1)
        code = runner.bt_program_run(_c_ptr(_stream()), self._entries, _c_int(len(self.calls)), ctypes.byref(failed))
        if code != 0:
            lib, name, _ = self.calls[failed.value]
            message = lib.bt_last_error().decode() if hasattr(lib, "bt_last_error") else f"returned {code}"
            raise KernelError(f"{message} (call {failed.value} of {len(self.calls)}, {name})")


class _Recording:
    def __init__(self, program):
        self.program = program

    def __enter__(self):
        if _recorder.program is not None:
            raise RuntimeError("a launch list is already being recorded")
        _recorder.program = self.program
        return self.program

    def __exit__(self, *exc):
        _recorder.program = None
        return False


_held_stream = [None]


def _stream():
    held = _held_stream[0]
    return held if held is not None else torch.cuda.current_stream().cuda_stream


class one_stream:
    """While this context is open every kernel goes to the stream that was current when it was
    entered, looked up once: asking torch for the current stream costs more host time than a launch
    does, and a step is hundreds of launches.  Enter it inside whatever chose the stream (a
    ``torch.cuda.stream`` or ``torch.cuda.graph`` context), never around it.  One thread issues
    kernels at a time (the same holds for the workspaces this module keeps per device)."""

    def __enter__(self):
        self.before = _held_stream[0]
        _held_stream[0] = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        _held_stream[0] = self.before
        return False


def _ptr(tensor):
    return None if tensor is None else tensor.data_ptr()


def loaded_modules():
    return sorted(_modules)


def require_gpu():
    if not torch.cuda.is_available():
        raise RuntimeError("burn_transformers_amd runs on an AMD GPU only (no HIP device is visible); "
                           "there is no CPU path")


def prepare(dtype, modules=()):
    """Builds and loads what every model of this dtype needs, and the modules its parts ask for
    (``Part.kernel_modules``)."""
    names = ["core", "gemm_mfma", "program"]
    if dtype == torch.bfloat16 and os.environ.get(PRODUCTS_ENV, "") != "own":
        names.append("gemm_library")
    names += [name for name in modules if name not in names]
    with _lock:
        build.ensure_many(names)        # what is missing is compiled side by side
    for name in names:
        if name != "gemm_library":
            _module(name)
    if dtype == torch.bfloat16:
        library_products()


# --- the vendor's GEMM library for steps with many rows ---------------------------------------

_library_state = {"tried": False, "lib": None}
PRODUCTS_ENV = "BURN_TRANSFORMERS_AMD_PRODUCTS"     # "own": never use the vendor's GEMM library


def library_products():
    """The module that runs prompt-sized bfloat16 products through hipBLASLt, or None.

    The reference leaves its matrix products to its backend's library (src/attention.rs:481-513
    and the feed-forward call ``linear``); here the vendor's library takes the products of steps
    with more than 256 rows (512 for those that add to the residual stream: ``deep_form_rows``),
    where it is about 1.6 times as fast as the tile kernel of this package at GPT-2 XL sizes, and
    the hand-written kernels keep everything else.  The library is
    opened from the copy that came with torch's HIP runtime and checked once against the tile
    kernel; if it cannot be opened, or disagrees, the tile kernel does those products too, and
    a line on stderr says so.
    """
    state = _library_state
    if state["tried"]:
        return state["lib"]
    state["tried"] = True
    if os.environ.get(PRODUCTS_ENV, "") == "own":
        return None
    try:
        lib = _module("gemm_library")
        candidates = [os.path.join(os.path.dirname(torch.__file__), "lib", "libhipblaslt.so"), "libhipblaslt.so"]
        version, errors = ctypes.c_int(0), []
        for path in candidates:
            if lib.bt_gemm_library_open(path.encode(), ctypes.byref(version)) == 0:
                break
            errors.append(lib.bt_last_error().decode())
        else:
            raise RuntimeError("; ".join(errors))
        state["lib"] = lib
        _check_library_products()
    except Exception as error:   # the library is an optimisation: without it the own kernels run
        state["lib"] = None
        print(f"[burn_transformers_amd] hipBLASLt is not used ({error}); the tile kernel takes its products",
              file=sys.stderr, flush=True)
    return state["lib"]


def _check_library_products():
    """One small product with each epilogue the library is given, against the tile kernel."""
    gen = torch.Generator(device="cuda").manual_seed(0)
    m, n, k = 96, 80, 64
    a = torch.randn(m, k, generator=gen, device="cuda").to(torch.bfloat16)
    w = (torch.randn(n, k, generator=gen, device="cuda") / 8).to(torch.bfloat16)
    bias = torch.randn(n, generator=gen, device="cuda")
    for make, dtype in ((epilogue_store, torch.bfloat16), (lambda o, b: epilogue_act(o, "gelu_tanh", b), torch.bfloat16),
                        (epilogue_residual, torch.float32)):
        mine = torch.ones(m, n, dtype=dtype, device="cuda")
        theirs = torch.ones(m, n, dtype=dtype, device="cuda")
        gemm(a, w, make(mine, bias), impl="tile")
        gemm(a, w, make(theirs, bias), impl="library")
        error = float((mine.float() - theirs.float()).abs().max())
        if not error < 0.05:
            raise RuntimeError(f"its result differs from the tile kernel's by {error}")


_library_refused = set()     # (rows, columns, k, epilogue mode, bias?) the library had no algorithm for


def _library_takes(epilogue):
    if epilogue.out_rows:            # chunk-major results are written by this package's kernels only
        return False
    return epilogue.mode in (EPI_STORE, EPI_RESIDUAL, EPI_F32) or (epilogue.mode == EPI_ACT and epilogue.act == 0)


# --- epilogues -------------------------------------------------------------------------------

def _out_rows(out):
    return out.shape[0] if isinstance(out, Chunked) else 0


def epilogue_store(out, bias=None):
    """``out`` [M, N] in the products' dtype, or a :class:`Chunked` of that shape."""
    return Epilogue(mode=EPI_STORE, bias=_ptr(bias), out=out.data_ptr(), ldo=out.stride(0), out_rows=_out_rows(out))


def epilogue_act(out, activation, bias=None):
    return Epilogue(mode=EPI_ACT, act=ACTIVATIONS[activation], bias=_ptr(bias), out=out.data_ptr(),
                    ldo=out.stride(0), out_rows=_out_rows(out))


def epilogue_f32(out, bias=None):
    """``out`` is float32 [splits, M, N] (or [M, N] for one split)."""
    split_stride = out.stride(0) if out.dim() == 3 else 0
    return Epilogue(mode=EPI_F32, bias=_ptr(bias), out=out.data_ptr(), ldo=out.stride(-2),
                    split_stride=split_stride)


def epilogue_residual(x, bias=None):
    """x[m][n] += acc + bias, with x the float32 residual stream [M, N] itself."""
    return Epilogue(mode=EPI_RESIDUAL, bias=_ptr(bias), out=x.data_ptr(), ldo=x.stride(0))


def epilogue_qkv(q_out, n_q, n_kv, kv_view, tok_seq, tok_pos, bias=None):
    return Epilogue(mode=EPI_QKV, bias=_ptr(bias), out=q_out.data_ptr(), ldo=q_out.stride(0), n_q=n_q,
                    n_kv=n_kv, tok_seq=tok_seq.data_ptr(), tok_pos=tok_pos.data_ptr(), kv=kv_view)


# --- kernels ---------------------------------------------------------------------------------

def embed(ids, positions, table, position_table, out):
    """out[t] = table[ids[t]] (+ position_table[positions[t]]); out is the float32 stream."""
    _launch(_module("core"), "bt_embed_call",
            EmbedCall(dtype=DTYPE_CODES[table.dtype], tokens=ids.numel(), width=table.shape[1], ids=ids.data_ptr(),
                      pos=_ptr(positions), table=table.data_ptr(), positions=_ptr(position_table), out=out.data_ptr()))


def add_norm(x, out, gamma, beta, eps, kind="layer_norm", delta=None, bias=None, rows=None,
             write_back=True):
    """x[t] += sum(delta[:, t]) + bias (kept when ``write_back``); out[r] = norm(x[t]) * gamma + beta
    with t = rows[r] if rows is given else r.  ``out`` may be None (only the add) or a :class:`Chunked`."""
    lib = _module("core")
    width = x.shape[1]
    if delta is None:
        n_delta, stride = 0, 0
    elif delta.dim() == 3:
        n_delta, stride = delta.shape[0], delta.stride(0)
    else:
        n_delta, stride = 1, 0
    n_rows = rows.numel() if rows is not None else x.shape[0]
    if delta is None and bias is None:
        write_back = False      # nothing is added: the stream already holds what would be written
    out_dtype = DTYPE_CODES[out.dtype] if out is not None else FLOAT32
    _launch(lib, "bt_add_norm_call",
            AddNormCall(out_dtype=out_dtype, n_delta=n_delta, kind=NORM_KINDS[kind], n_rows=n_rows, width=width,
                        write_back=1 if write_back else 0, out_rows=_out_rows(out), eps=eps, x=x.data_ptr(),
                        delta=_ptr(delta), delta_stride=stride, bias=_ptr(bias), gamma=_ptr(gamma), beta=_ptr(beta),
                        out=out.data_ptr() if out is not None else None, rows=_ptr(rows)))


def pack_columns(w, columns):
    """[N, K] -> the skinny kernel's packed form for ``columns`` output columns per work-group:
    [groups, chunks, columns, chunk] with chunks of 32 bfloat16 (16 float32) K values, K and the last
    group padded with zeros.  A wave then loads a chunk of its columns as one contiguous run of
    bytes, and a work-group reads its share of the matrix as one block, front to back."""
    n, k = w.shape
    chunk = 32 if w.dtype == torch.bfloat16 else 16
    groups, chunks = (n + columns - 1) // columns, (k + chunk - 1) // chunk
    padded = w.new_zeros((groups * columns, chunks * chunk))
    padded[:n, :k] = w
    return padded.view(groups, columns, chunks, chunk).permute(0, 2, 1, 3).contiguous()


def skinny_columns(m, n, k, splits, dtype, units):
    """The output columns per work-group the skinny kernel's launcher chooses for this product
    (the same rule as in ``bt_gemm_skinny``: the busiest compute unit pulls the least)."""
    chunk = 32 if dtype == torch.bfloat16 else 16
    per = ((k + chunk - 1) // chunk + splits - 1) // splits
    best, columns = -1, 16 if m <= 16 else 32
    for c in range(32, 7, -4):
        groups = (n + c - 1) // c * splits
        cost = (groups + units - 1) // units * (per * (c + m) + 160)
        if best < 0 or cost < best:
            best, columns = cost, c
    return columns


class PackedWeight:
    """Second copies of a matrix in the skinny kernel's packed form (``pack_columns``), one for each
    column count the launcher chooses for steps of a few rows with the given splits of K (a product
    that adds to the residual stream runs with a split of K or, behind a folded norm, without).
    Decode steps read weights and little else, and from a packed copy a product of up to 16 rows
    takes about a seventh less time (6.9 -> 6.0 us for 4800 x 1600, 7.9 -> 6.5 us for 6400 x 1600
    at 8 rows); results are bitwise the same.  ``for_step`` hands out the copy that fits a step."""

    ROWS = 8            # the step the copies are laid out for; other small steps choose the same columns almost always
    enabled = True      # tests switch it off to run the plain layout too

    def __init__(self, w, splits=(1,)):
        self.shape, self.dtype = tuple(w.shape), w.dtype
        self.units = torch.cuda.get_device_properties(w.device).multi_processor_count
        self.copies = {}                 # columns per work-group -> packed tensor
        for count in ((splits,) if isinstance(splits, int) else splits):
            columns = skinny_columns(self.ROWS, w.shape[0], w.shape[1], count, w.dtype, self.units)
            if columns not in self.copies:
                self.copies[columns] = pack_columns(w, columns)
        self._fits = {}

    def for_step(self, m, splits):
        """(packed tensor, columns) if a product of ``m`` rows and ``splits`` slices runs on the
        skinny kernel with the columns of one of the copies, else None (the caller then reads the
        plain matrix)."""
        if not PackedWeight.enabled or m > 64:
            return None
        fits = self._fits.get((m, splits))
        if fits is None:
            columns = skinny_columns(m, self.shape[0], self.shape[1], splits, self.dtype, self.units)
            fits = (self.copies[columns], columns) if columns in self.copies else False
            self._fits[(m, splits)] = fits
        return fits or None


def gemm(a, w, epilogue, splits=1, impl="auto", variant=0, packed=None):
    """C = a . w^T handed to ``epilogue``.  a: [M, K] (rows may be strided), w: [N, K] contiguous.

    impl: "auto" (skinny up to 64 rows; beyond that the tile kernel, or for bfloat16 the vendor's
    library where it is usable and has the epilogue; float32 operands that are not multiples of
    four wide go to the plain kernel), or one of "plain", "tile", "skinny", "library" to force one.
    variant picks one of the tile kernel's forms (0: the fastest the operands allow, 1: any K,
    2: lean, 3: direct to LDS) or, for the skinny kernel, the output columns a work-group owns
    (8, 12, ... 32; 0: chosen for balance).  ``a`` may be a :class:`Normalized`.
    packed: a :class:`PackedWeight` of ``w`` (or directly (``pack_columns(w, columns)``, columns)), read in
    place of ``w`` where the skinny kernel runs and the copy fits the step.
    """
    m, k = a.shape
    n = w.shape[0]
    if isinstance(packed, PackedWeight):
        packed = packed.for_step(m, splits) if variant == 0 and impl in ("auto", "skinny") else None
    a_rows = 0
    if isinstance(a, Chunked):          # read by the skinny product only
        if impl not in ("auto", "skinny") or m > Chunked.MAX_ROWS or w.shape[1] != k or not w.is_contiguous() or a.dtype != w.dtype:
            raise KernelError(f"gemm: chunk-major activations [{m},{k}] {a.dtype} go to the skinny kernel "
                              f"(up to {Chunked.MAX_ROWS} rows) with weights [{n},{k}] of the same type")
        impl, a_rows = "skinny", m
    if isinstance(a, Normalized):
        if w.shape[1] != k or not w.is_contiguous() or w.dtype != torch.bfloat16 or impl not in ("auto", "skinny"):
            raise KernelError(f"gemm: rows to be normalised [{m},{k}] go with bfloat16 weights [{n},{k}] on the skinny kernel only")
        operand = NormOperand(x=a.x.data_ptr(), ldx=a.x.stride(0), gamma=a.gamma.data_ptr(), beta=_ptr(a.beta),
                              eps=a.eps, kind=NORM_KINDS[a.kind])
        weights, columns = (packed[0].data_ptr(), packed[1]) if packed is not None else (w.data_ptr(), 0)
        _launch(_module("gemm_mfma"), "bt_gemm_skinny_call",
                GemmCall(dtype=BFLOAT16, M=m, N=n, K=k, splits=splits, variant=variant, packed_columns=columns,
                         has_norm=1, W=weights, epi=epilogue, norm=operand))
        return
    if w.shape[1] != k or a.stride(1) != 1 or not w.is_contiguous() or a.dtype != w.dtype:
        raise KernelError(f"gemm: operands [{m},{k}] {a.dtype} and [{n},{w.shape[1]}] {w.dtype} do not fit")
    dtype = DTYPE_CODES[a.dtype]
    if impl == "auto":
        if dtype == FLOAT32 and (k % 4 or a.stride(0) % 4):
            impl = "plain"                       # the MFMA kernels read 16 bytes at a time
        elif m <= 64:
            impl = "skinny"
        elif dtype == FLOAT32:
            impl = "tile"
        elif deep_form_rows(m, k, a.stride(0), n, sliced=splits > 1, scatters=epilogue.mode == EPI_QKV):
            # short prompts and chunks: the tile kernel's deep forms (see ``deep_form_rows``)
            impl = "tile"
            if variant == 0:
                # tiles of 64 x 64 in four stages, two work-groups to a compute unit.  (Tiles of 128 x
                # 64 in three stages beyond 128 rows were the choice once: alone they measure the same
                # at 256 rows, 19.9 against 19.5 us for 4800 x 1600, and lose at 129 to 192 rows, where
                # the small tiles still have a compute unit each, 18.9 against 12.9 us; a prompt of 160
                # tokens through 12 layers 1.08 -> 0.97 ms, of 256 tokens 1.20 -> 1.17 ms.)
                variant = 5
        else:
            impl = "library" if splits == 1 and _library_takes(epilogue) and library_products() \
                and _library_has_algorithm(a.stride(0), m, n, k, epilogue) else "tile"
    call = GemmCall(dtype=dtype, M=m, N=n, K=k, splits=splits, variant=variant, A=a.data_ptr(), lda=a.stride(0),
                    W=w.data_ptr(), epi=epilogue)
    if impl == "plain":
        if splits != 1:
            raise KernelError("gemm: the plain kernel does not split K")
        _launch(_module("core"), "bt_gemm_plain_call", call)
    elif impl == "library":
        if dtype != BFLOAT16 or epilogue.out_rows:
            raise KernelError("gemm: the library product takes bfloat16 only and writes row-major results")
        lib = _library_state["lib"] or library_products()
        if lib is None:
            raise KernelError("gemm: the vendor's GEMM library is not available")
        if splits != 1:
            raise KernelError("gemm: the library product does not split K")
        _launch(lib, "bt_gemm_library_call", call)
    elif impl == "tile":
        _launch(_module("gemm_mfma"), "bt_gemm_tile_call", call)
    else:
        call.a_rows = a_rows
        if packed is not None:          # (only here: the other kernels read the plain matrix)
            call.W, call.packed_columns = packed[0].data_ptr(), packed[1]
        _launch(_module("gemm_mfma"), "bt_gemm_skinny_call", call)


DEEP_FORM_ROWS = 256          # most rows of a bfloat16 product that the tile kernel's deep forms take ...
DEEP_FORM_SLICED_ROWS = 512   # ... and of one that leaves partial sums of slices of K pending ...
DEEP_FORM_SCATTER_ROWS = 384  # ... and of one that scatters keys and values into the cache


def deep_form_rows(m, k, lda, n, sliced=False, scatters=False):
    """Whether a bfloat16 product of ``m`` rows is one for the tile kernel's deep forms (tiles of
    64 x 64 or 128 x 64 brought straight into LDS, several of them on their way at once): 65 to
    256 rows, where it has too few tiles of 128 x 128 to fill the chip and the vendor's library
    takes 16 to 24 us whatever the shape (measured at widths 1,600 and 6,400: these forms take a
    quarter to a third less); where the product may leave slices of K pending (``sliced``: the two
    products that add to the residual stream) up to 512 rows, and up to 45 % less.  Beyond, the
    library wins.  The fused projection of a mixer (``scatters``) stays up to 384 rows: the
    library's product cannot scatter keys and values into the cache, and the copy behind it costs
    5 us (4800 x 1600 at 320 and 384 rows: 19.5 and 19.7 us here, 18.7 and 18.9 + 5.1 there; at 512
    rows 28.4 against 20.8 + 5.0).  The forms read K in tiles of 64 and address their operands with
    32 bits."""
    limit = DEEP_FORM_SLICED_ROWS if sliced else DEEP_FORM_SCATTER_ROWS if scatters else DEEP_FORM_ROWS
    return 64 < m <= limit and k % 64 == 0 and m * lda * 2 < (1 << 32) and n * k * 2 < (1 << 32)


def deep_split_count(rows, columns, k, units=256):
    """Into how many slices of pending partial sums a residual-writing bfloat16 product of 65 to
    ``DEEP_FORM_SLICED_ROWS`` rows cuts its K range: as many as still give every work-group (a tile
    of 64 x 64 of one slice) a compute unit of its own, or, where even two slices are too many for
    that, as many as leave at most two work-groups to a unit; at most four (the norm behind the
    product reads them all), each at least four tiles of K long.  Measured at width 1,600 on 256
    units (us for 1600 x 1600 and 1600 x 6400, slices 2 / 3 / 4): 128 rows 7.1 / 6.3 / 5.9 and 18.9 /
    14.5 / 12.1; 192 rows 7.3 / 6.5 / 7.2 and 18.8 / 14.7 / 18.8; 256 rows 7.4 / 7.9 / 7.5 and 19.2 /
    22.4 / 18.8; 384 rows 9.3 / 8.4 / 10.9 and 29.3 / 23.1 / 26.5; 512 rows 9.5 / 12.1 / 12.1 and 30.7 /
    32.2 / 31.0 (the vendor's library: 11.1 to 12.2 and 18.3 to 32.4).  Measured and not taken: tiles
    of 128 x 128 in four slices for 1600 x 6400 at 512 rows (25.2 us alone against 30.3, but 29.5 in
    the step, where the norm behind it also reads four slices instead of two), and slices beyond 512
    rows (640 rows: 10.1 and 30.7 against the library's 12.2 and 32.7, which the norm's second
    reading of two slices takes back)."""
    if not deep_form_rows(rows, k, k, columns, sliced=True):
        return 1
    tiles = ((rows + 63) // 64) * ((columns + 63) // 64)
    splits = units // tiles
    if splits < 2:
        splits = 2 * units // tiles
    return max(1, min(4, splits, (k // 64) // 4))


def prompt_products_in_library(m, n, k, lda, scatters=False):
    """Whether a bfloat16 product of a step of ``m`` rows goes to the vendor's library (which cannot
    scatter keys and values into the cache: the caller then copies them)."""
    return m > 64 and not deep_form_rows(m, k, lda, n, scatters=scatters) and library_products() is not None


def _library_has_algorithm(lda, m, n, k, epilogue):
    """Whether the vendor's library has an algorithm for this product (asked without running
    anything; the library keeps what it found).  A shape it has none for is remembered and runs on
    the package's tile kernel, with a line on stderr the first time."""
    shape = (m, n, k, int(epilogue.mode), bool(epilogue.bias))
    if shape in _library_refused:
        return False
    lib = _library_state["lib"]
    if lib.bt_gemm_library_plan(_c_i64(lda), _c_int(m), _c_int(n), _c_int(k), ctypes.byref(epilogue)) == 0:
        return True
    refusal = lib.bt_last_error().decode()
    if "no algorithm" not in refusal:
        raise KernelError(refusal)
    _library_refused.add(shape)
    print(f"[burn_transformers_amd] {refusal}; this shape runs on the package's tile kernel",
          file=sys.stderr, flush=True)
    return False


def attention_args(q, out, kv_view, tok_seq, tok_pos, seq_off, seq_start, q_heads, n_seqs, max_count,
                   scale, window=0, partial=None, runs=None):
    """``partial``: float32 [rows * q_heads * runs, head_dim + 2] for a step whose keys are cut into
    runs that separate work-groups take.  Decode steps (long contexts in small batches): rows are
    the sequences, and ``runs`` follows from the shape.  Prompt steps (few query tiles behind a long
    context): rows are the step's tokens, the buffer may be longer than this step needs, and
    ``runs`` is given.  ``out`` may be a :class:`Chunked` for the bfloat16 decode kernels."""
    splits = 1
    if partial is not None:
        rows = n_seqs if runs is None else q.shape[0]
        splits = partial.shape[0] // (rows * q_heads) if runs is None else runs
        if partial.dtype != torch.float32 or not partial.is_contiguous() or partial.shape[1] != kv_view.head_dim + 2 \
                or (splits * rows * q_heads != partial.shape[0] if runs is None else splits * rows * q_heads > partial.shape[0]):
            raise KernelError(f"attention: partial results of shape {tuple(partial.shape)} do not fit "
                              f"{rows} rows of {q_heads} heads of {kv_view.head_dim} in {splits} runs")
    return AttnArgs(splits=splits, partial=partial.data_ptr() if partial is not None and splits > 1 else None,
                    q=q.data_ptr(), ldq=q.stride(0), out=out.data_ptr(), ldo=out.stride(0), out_rows=_out_rows(out),
                    tok_seq=tok_seq.data_ptr(), tok_pos=tok_pos.data_ptr(), seq_off=seq_off.data_ptr(),
                    seq_start=seq_start.data_ptr(), kv=kv_view, q_heads=q_heads, n_tokens=q.shape[0],
                    n_seqs=n_seqs, max_count=max_count, window=window or 0, scale=scale)


def attention(args, dtype, decode, impl="auto"):
    """Attention of the step's tokens over the cache.  impl: "auto" (bfloat16: the MFMA kernels;
    float32: the tiled kernel for head sizes up to 128, else the plain one), "plain", "tiled"
    (float32) or "mfma" (bfloat16)."""
    code = DTYPE_CODES[dtype]
    if impl == "auto":
        if code == BFLOAT16:
            impl = "mfma"
        else:
            impl = "tiled" if args.kv.head_dim <= 128 and args.kv.head_dim % 16 == 0 and args.ldq % 4 == 0 \
                and (decode or args.ldo % 4 == 0) else "plain"
    call = AttentionCall(dtype=code, args=args)
    if impl == "plain":
        _launch(_module("core"), "bt_attention_plain_call", call)
        return
    if impl == "tiled":
        if code != FLOAT32:
            raise KernelError("attention: the tiled kernel takes float32 only")
        _launch(_module("attention_f32"), "bt_attention_f32_call", call)
        return
    if code != BFLOAT16:
        raise KernelError("attention: the MFMA kernels take bfloat16 only")
    _launch(_module(f"attention_bf16_hd{args.kv.head_dim}"),
            "bt_attention_decode_bf16_call" if decode else "bt_attention_prefill_bf16_call", call)


def kv_copy(k_rows, v_rows, tok_seq, tok_pos, kv_view, to_cache):
    """Copies [tokens, kv_heads * head_dim] rows into the paged cache, or back out of it."""
    _launch(_module("core"), "bt_kv_copy_call",
            KvCopyCall(dtype=DTYPE_CODES[k_rows.dtype], tokens=k_rows.shape[0], to_cache=1 if to_cache else 0,
                       k_rows=k_rows.data_ptr(), v_rows=v_rows.data_ptr(), ld=k_rows.stride(0),
                       tok_seq=tok_seq.data_ptr(), tok_pos=tok_pos.data_ptr(), kv=kv_view))


_sample_workspaces = {}


def sample(logits, ids, logp, temperature=None, seed=0, first_draw=0, draw_rows=None):
    """Greedy (temperature None) or temperature sampling of each row of float32 logits.  Row r uses
    draw number first_draw + (draw_rows[r] if draw_rows is given else r) of the seed's stream."""
    lib = _module("core")
    rows, vocab = logits.shape
    sampling = temperature is not None
    lib.bt_sample_workspace_bytes.restype = ctypes.c_int64
    need = lib.bt_sample_workspace_bytes(_c_int(rows), _c_int(vocab))
    workspace = _sample_workspaces.get(logits.device)
    if workspace is None or workspace.numel() < need:       # partial results of the first kernel
        workspace = torch.empty(max(need, 1 << 16), dtype=torch.uint8, device=logits.device)
        _sample_workspaces[logits.device] = workspace
    _check(lib, lib.bt_sample(_c_ptr(_stream()), _c_ptr(logits.data_ptr()), _c_i64(logits.stride(0)),
                              _c_int(rows), _c_int(vocab), _c_int(1 if sampling else 0),
                              _c_float(temperature if sampling else 1.0), _c_u64(seed & (2 ** 64 - 1)),
                              _c_u64(first_draw & (2 ** 64 - 1)), _c_ptr(_ptr(draw_rows)), _c_ptr(ids.data_ptr()),
                              _c_ptr(logp.data_ptr()), _c_ptr(workspace.data_ptr())))


class ProcessArgs(ctypes.Structure):
    _fields_ = [("logits", _c_ptr), ("ld", _c_i64), ("vocab", _c_int), ("bias", _c_ptr),
                ("counts_all", _c_ptr), ("counts_add", _c_ptr), ("counts_ld", _c_i64),
                ("batch_rows", _c_ptr), ("ban_ids", _c_ptr), ("ban_offsets", _c_ptr),
                ("repetition", _c_float), ("presence", _c_float), ("frequency", _c_float),
                ("sample", _c_int), ("temperature", _c_float), ("clamp", _c_int),
                ("top_k", _c_int), ("top_p", _c_float), ("min_p", _c_float),
                ("seed", _c_u64), ("first_draw", _c_u64), ("ids", _c_ptr), ("logp", _c_ptr)]


def select_processed(logits, ids, logp, *, bias=None, counts_all=None, counts_add=None, batch_rows=None,
                     ban_ids=None, ban_offsets=None, repetition=1.0, presence=0.0, frequency=0.0,
                     temperature=None, clamp=False, top_k=0, top_p=1.0, min_p=0.0, seed=0, first_draw=0):
    """One token per row of float32 logits after bias, penalties, temperature, banned tokens and (when
    sampling: ``temperature`` given) top-k / top-p / min-p; see ``select_processed_kernel``.
    ``batch_rows`` (int32) names each row's number in the batch as it started: its row in the
    count tensors and its draw."""
    lib = _module("core")
    rows, vocab = logits.shape
    counts = counts_all if counts_all is not None else counts_add
    sampling = temperature is not None
    truncating = sampling and ((top_k or 0) > 0 or (top_p is not None and top_p < 1.0) or (min_p or 0.0) > 0.0)
    args = ProcessArgs(
        logits=logits.data_ptr(), ld=logits.stride(0), vocab=vocab, bias=_ptr(bias),
        counts_all=_ptr(counts_all), counts_add=_ptr(counts_add), counts_ld=counts.stride(0) if counts is not None else 0,
        batch_rows=_ptr(batch_rows), ban_ids=_ptr(ban_ids), ban_offsets=_ptr(ban_offsets),
        repetition=repetition, presence=presence, frequency=frequency,
        sample=1 if sampling else 0, temperature=temperature if sampling else 1.0,
        clamp=1 if clamp else 0, top_k=top_k or 0, top_p=top_p if top_p is not None else 1.0,
        min_p=min_p or 0.0, seed=seed & (2 ** 64 - 1), first_draw=first_draw & (2 ** 64 - 1),
        ids=ids.data_ptr(), logp=logp.data_ptr())
    if truncating:          # one work-group holds the row in registers: processing, thresholds and the draw in one kernel
        _check(lib, lib.bt_select_processed(_c_ptr(_stream()), ctypes.byref(args), _c_int(rows)))
        return
    # Nothing is cut off: the processing alone by many work-groups per row into processed scores
    # (one compute unit pulls a row's logits and counts no faster than in 25 us), then the plain
    # selection: the lowest index of the maximum, or a draw at temperature 1 (it is applied already).
    held = _processed_scores.get(logits.device)
    if held is None or held.shape[0] < rows or held.shape[1] != vocab:
        held = torch.empty((max(rows, 8), vocab), dtype=torch.float32, device=logits.device)
        _processed_scores[logits.device] = held
    scores = held[:rows]
    _check(lib, lib.bt_process_scores(_c_ptr(_stream()), ctypes.byref(args), _c_int(rows),
                                      _c_ptr(scores.data_ptr()), _c_i64(scores.stride(0))))
    sample(scores, ids, logp, temperature=1.0 if sampling else None, seed=seed, first_draw=first_draw,
           draw_rows=batch_rows)


_processed_scores = {}


def count_tokens(counts, rows, tokens):
    """counts[rows[i]][tokens[i]] += 1 (int32 counts on the GPU; rows and tokens: Python lists)."""
    lib = _module("core")
    pairs = torch.tensor([list(rows), list(tokens)], dtype=torch.int32).to(counts.device, non_blocking=True)
    _check(lib, lib.bt_count_tokens(_c_ptr(_stream()), _c_ptr(counts.data_ptr()), _c_i64(counts.stride(0)),
                                    _c_ptr(pairs[0].data_ptr()), _c_ptr(pairs[1].data_ptr()), _c_int(len(rows))))
