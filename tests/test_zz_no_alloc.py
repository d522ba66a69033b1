"""bt_sample_no_alloc, the entry point for callers that cannot allocate, called through ctypes
exactly as such a caller would: against bt_sample (which takes a workspace) on the same logits,
twice in a row, the second call with a smaller input, so that what the first call left in the
library's fixed scratch array is there when the second runs."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

from burn_transformers_amd.kernels import build  # noqa: E402

c_int, c_i64, c_ptr, c_float, c_u64 = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p, ctypes.c_float, ctypes.c_uint64


def library():
    lib = ctypes.CDLL(build.ensure("core"))
    lib.bt_last_error.restype = ctypes.c_char_p
    lib.bt_sample_workspace_bytes.restype = c_i64
    lib.bt_sample_no_alloc_capacity.restype = c_i64
    common = [c_ptr, c_ptr, c_i64, c_int, c_int, c_int, c_float, c_u64, c_u64, c_ptr, c_ptr, c_ptr]
    lib.bt_sample.argtypes = common + [c_ptr]
    lib.bt_sample_no_alloc.argtypes = common
    return lib


def both(lib, logits, temperature, seed, first_draw):
    """(ids, log-probabilities) of the entry point with a workspace and of the one without."""
    rows, vocab = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    sampling = temperature is not None
    args = (stream, logits.data_ptr(), logits.stride(0), rows, vocab, 1 if sampling else 0,
            temperature if sampling else 1.0, seed, first_draw, None)
    out = []
    workspace = torch.empty(lib.bt_sample_workspace_bytes(rows, vocab), dtype=torch.uint8, device=logits.device)
    for entry, extra in ((lib.bt_sample, (workspace.data_ptr(),)), (lib.bt_sample_no_alloc, ())):
        ids = torch.full((rows,), -1, dtype=torch.int32, device=logits.device)
        logp = torch.full((rows,), float("nan"), dtype=torch.float32, device=logits.device)
        code = entry(*args, ids.data_ptr(), logp.data_ptr(), *extra)
        assert code == 0, lib.bt_last_error().decode()
        torch.cuda.synchronize()
        out.append((ids.cpu(), logp.cpu()))
    return out


@pytest.mark.parametrize("temperature", [None, 0.7])
def test_two_calls_in_a_row_the_second_smaller(temperature):
    lib = library()
    gen = torch.Generator().manual_seed(5)
    first = (torch.randn(37, 50257, generator=gen) * 3).to("cuda:0")
    second = (torch.randn(5, 1000, generator=gen) * 3).to("cuda:0")       # fewer rows, fewer chunks' worth of logits
    for call, logits in enumerate((first, second)):
        (want_ids, want_logp), (ids, logp) = both(lib, logits, temperature, seed=99, first_draw=1000 * call)
        assert torch.equal(ids, want_ids), f"call {call}"
        assert torch.equal(logp, want_logp), f"call {call}"
        if temperature is None:
            assert torch.equal(ids.long(), logits.cpu().argmax(-1))
        reference = torch.log_softmax(logits.cpu().double() / (temperature or 1.0), -1)
        assert (logp.double() - reference.gather(1, ids.long()[:, None])[:, 0]).abs().max() < 1e-4


def test_sizes_beyond_the_fixed_array_are_refused_with_a_message():
    lib = library()
    capacity = lib.bt_sample_no_alloc_capacity()
    assert capacity == 4096
    rows = capacity // 16 + 1                     # 16 chunks a row up to 65,536 logits
    logits = torch.zeros(rows, 64, device="cuda:0")
    ids = torch.zeros(rows, dtype=torch.int32, device="cuda:0")
    logp = torch.zeros(rows, dtype=torch.float32, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    code = lib.bt_sample_no_alloc(stream, logits.data_ptr(), 64, rows, 64, 0, 1.0, 0, 0, None, ids.data_ptr(), logp.data_ptr())
    assert code == 1 and b"fixed scratch array holds 4096" in lib.bt_last_error()
    code = lib.bt_sample_no_alloc(stream, logits.data_ptr(), 64, rows - 1, 64, 0, 1.0, 0, 0, None, ids.data_ptr(), logp.data_ptr())
    assert code == 0, lib.bt_last_error().decode()
    torch.cuda.synchronize()
    assert int(ids[:rows - 1].abs().max()) == 0          # all logits equal: the lowest index
