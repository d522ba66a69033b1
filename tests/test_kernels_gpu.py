"""Each kernel alone against a plain float64 reference, at sizes other than the engine's."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

from burn_transformers_amd.kernels import library as K  # noqa: E402
from kernel_helpers import PagedCase, gelu_erf, gelu_tanh  # noqa: E402

DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def rel_err(got, want):
    got, want = got.detach().cpu().to(torch.float64), want.detach().cpu().to(torch.float64)
    return float((got - want).abs().max() / (want.abs().max() + 1e-30))


def operands(m, n, k, dtype, seed=0, lda=None):
    gen = torch.Generator().manual_seed(seed)
    lda = lda or k
    a_full = (torch.randn(m, lda, generator=gen)).to(dtype).to(DEV)
    a = a_full[:, :k]
    w = (torch.randn(n, k, generator=gen) / math.sqrt(k)).to(dtype).to(DEV)
    bias = torch.randn(n, generator=gen).to(DEV)
    want = a.cpu().double() @ w.cpu().double().t()
    return a, w, bias, want


GEMM_CASES = [("plain", "float32", 1, 50, 24), ("plain", "float32", 70, 131, 40), ("plain", "bfloat16", 33, 67, 72),
              ("tile", "bfloat16", 128, 128, 64), ("tile", "bfloat16", 200, 300, 136),
              ("tile", "bfloat16", 300, 517, 1600), ("tile", "bfloat16", 65, 50257 // 16, 96),
              ("skinny", "bfloat16", 1, 100, 136), ("skinny", "bfloat16", 7, 48, 1600),
              ("skinny", "bfloat16", 16, 333, 72), ("skinny", "bfloat16", 17, 64, 320),
              ("skinny", "bfloat16", 33, 1000, 64), ("skinny", "bfloat16", 64, 517, 6400),
              ("tile", "float32", 128, 128, 32), ("tile", "float32", 200, 300, 132), ("tile", "float32", 300, 517, 1600),
              ("tile", "float32", 65, 50257 // 16, 100), ("skinny", "float32", 1, 100, 132),
              ("skinny", "float32", 7, 48, 1600), ("skinny", "float32", 16, 333, 76), ("skinny", "float32", 17, 64, 320),
              ("skinny", "float32", 33, 1000, 64), ("skinny", "float32", 64, 517, 6400)]


@pytest.mark.parametrize("impl,dtype,m,n,k", GEMM_CASES)
def test_gemm_epilogues(impl, dtype, m, n, k):
    dt = DTYPES[dtype]
    tol = 2e-6 if dtype == "float32" else 6e-3
    a, w, bias, want = operands(m, n, k, dt, seed=m + n + k, lda=k + 8)
    out = torch.full((m, n), float("nan"), dtype=dt, device=DEV)
    K.gemm(a, w, K.epilogue_store(out, bias), impl=impl)
    assert rel_err(out, want + bias.cpu().double()) < tol
    for name, fn in (("gelu_tanh", gelu_tanh), ("gelu_erf", gelu_erf)):
        out = torch.full((m, n), float("nan"), dtype=dt, device=DEV)
        K.gemm(a, w, K.epilogue_act(out, name, bias), impl=impl)
        assert rel_err(out, fn(want + bias.cpu().double())) < tol
    out32 = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
    K.gemm(a, w, K.epilogue_f32(out32), impl=impl)
    assert rel_err(out32, want) < (2e-6 if dtype == "float32" else 2e-5 * math.sqrt(k))
    if dtype == "float32" and impl != "plain":
        # true 32-bit products: operands with 24 significant bits whose low bits decide the sum
        gen = torch.Generator().manual_seed(5)
        a2 = (1.0 + torch.rand(m, k, generator=gen) * 2 ** -12).to(DEV)
        w2 = (torch.where(torch.arange(k) % 2 == 0, 1.0, -1.0) * (1.0 + torch.rand(n, k, generator=gen) * 2 ** -12)).to(DEV)
        want2 = a2.cpu().double() @ w2.cpu().double().t()           # sums of +-1 nearly cancel: what is left is the low bits
        K.gemm(a2, w2, K.epilogue_f32(out32), impl=impl)
        assert float((out32.cpu().double() - want2).abs().max()) < 1e-5 * math.sqrt(k)


@pytest.mark.parametrize("variant", [1, 2, 3, 4, 5, 6, 7])
@pytest.mark.parametrize("m,n,k", [(128, 128, 64), (300, 517, 1600), (130, 96, 192), (1000, 1600, 6400), (65, 40, 128)])
def test_tile_gemm_forms_agree(variant, m, n, k):
    """The forms of the tile kernel (any K; lean; direct to LDS; direct to LDS with tiles of 64 x 64
    and of 128 x 64 in more stages than K has tiles, or fewer) against float64."""
    a, w, bias, want = operands(m, n, k, torch.bfloat16, seed=variant, lda=k + 64)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    K.gemm(a, w, K.epilogue_act(out, "gelu_erf", bias), impl="tile", variant=variant)
    assert rel_err(out, gelu_erf(want + bias.cpu().double())) < 6e-3
    parts = torch.full((3, m, n), float("nan"), dtype=torch.float32, device=DEV)
    K.gemm(a, w, K.epilogue_f32(parts), impl="tile", variant=variant, splits=3)
    assert rel_err(parts.sum(0), want) < 2e-5 * math.sqrt(k)
    if variant > 1:
        a2, w2, _, _ = operands(70, 40, 96, torch.bfloat16)
        with pytest.raises(K.KernelError, match="multiple of 64"):
            K.gemm(a2, w2, K.epilogue_store(torch.empty(70, 40, dtype=torch.bfloat16, device=DEV)), impl="tile",
                   variant=variant)


@pytest.mark.parametrize("m,n,k", [(65, 48, 72), (200, 300, 136), (300, 517, 1600), (2048, 1600, 320),
                                   (5000, 136, 72), (32768, 96, 64)])
def test_vendor_library_products(m, n, k):
    """Prompt-sized products through hipBLASLt with the three epilogues it is given, against float64;
    the tall ones go to the library in runs of rows, with and without a shorter last run."""
    if K.library_products() is None:
        pytest.skip("hipBLASLt could not be opened; the tile kernel takes these products")
    a, w, bias, want = operands(m, n, k, torch.bfloat16, seed=m, lda=k + 8)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    K.gemm(a, w, K.epilogue_store(out, bias), impl="library")
    assert rel_err(out, want + bias.cpu().double()) < 6e-3
    K.gemm(a, w, K.epilogue_store(out), impl="library")
    assert rel_err(out, want) < 6e-3
    K.gemm(a, w, K.epilogue_act(out, "gelu_tanh", bias), impl="library")
    assert rel_err(out, gelu_tanh(want + bias.cpu().double())) < 6e-3
    gen = torch.Generator().manual_seed(1)
    x0 = torch.randn(m, n, generator=gen)
    x = x0.clone().to(DEV)
    K.gemm(a, w, K.epilogue_residual(x, bias), impl="library")
    assert rel_err(x, x0.double() + want + bias.cpu().double()) < 2e-5 * math.sqrt(k)
    out32 = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
    K.gemm(a, w, K.epilogue_f32(out32), impl="library")
    assert rel_err(out32, want) < 2e-5 * math.sqrt(k)
    with pytest.raises(K.KernelError, match="not one the library has"):
        K.gemm(a, w, K.epilogue_act(out, "gelu_erf", bias), impl="library")
    # what "auto" picks for these rows gives the same
    auto = torch.empty_like(out)
    K.gemm(a, w, K.epilogue_act(out, "gelu_tanh", bias), impl="library")
    K.gemm(a, w, K.epilogue_act(auto, "gelu_tanh", bias))
    assert torch.equal(auto, out)


def test_a_shape_the_library_refuses_runs_on_the_tile_kernel(monkeypatch, capfd):
    """When the library has no algorithm for a shape, "auto" says so once and takes the tile kernel."""
    if K.library_products() is None:
        pytest.skip("hipBLASLt could not be opened")
    m, n, k = 130, 72, 136
    a, w, bias, want = operands(m, n, k, torch.bfloat16, seed=4)
    calls = []

    class Refusing:
        def __getattr__(self, name):
            return getattr(K._library_state["real"], name)

        def bt_gemm_library_plan(self, *args):        # what "auto" asks before it names the library
            calls.append(1)
            return 1

        def bt_last_error(self):
            return b"gemm_library: no algorithm without workspace for this test"

    monkeypatch.setitem(K._library_state, "real", K._library_state["lib"])
    monkeypatch.setitem(K._library_state, "lib", Refusing())
    monkeypatch.setattr(K, "_library_refused", set())
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    for _ in range(2):
        K.gemm(a, w, K.epilogue_store(out, bias))
        assert rel_err(out, want + bias.cpu().double()) < 6e-3
    assert len(calls) == 1                       # asked once; the refusal is remembered for the shape
    assert "tile kernel" in capfd.readouterr().err


@pytest.mark.parametrize("m,n,k,splits", [(1, 100, 136, 1), (8, 4800, 1600, 2), (16, 1600, 1600, 4),
                                          (7, 333, 6400, 8), (3, 50, 1760, 1), (16, 517, 1608, 3),
                                          (2, 16, 8, 1), (9, 40, 3400, 1)])
@pytest.mark.parametrize("columns", [0, 16, 12, 8, 20, 28, 32])
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_skinny_gemm_at_decode_sizes(m, n, k, splits, columns, dtype):
    """Up to 16 rows, K with a short last chunk, slices of K that do not divide evenly; 16, 12 or 8
    to 32 output columns per work-group (0: chosen for balance)."""
    variant = columns
    dt = DTYPES[dtype]
    a, w, bias, want = operands(m, n, k, dt, seed=k, lda=k + 24)
    parts = torch.full((splits, m, n), float("nan"), dtype=torch.float32, device=DEV)
    K.gemm(a, w, K.epilogue_f32(parts, bias), splits=splits, impl="skinny", variant=variant)
    assert rel_err(parts.sum(0), want + bias.cpu().double()) < (2e-6 if dtype == "float32" else 2e-5 * math.sqrt(k))
    if splits == 1:
        out = torch.full((m, n), float("nan"), dtype=dt, device=DEV)
        K.gemm(a, w, K.epilogue_act(out, "gelu_tanh", bias), impl="skinny", variant=variant)
        assert rel_err(out, gelu_tanh(want + bias.cpu().double())) < (2e-6 if dtype == "float32" else 6e-3)


@pytest.mark.parametrize("m,n,k,splits", [(1, 100, 136, 1), (8, 4800, 1600, 1), (16, 1600, 1608, 4), (7, 333, 6400, 5),
                                          (3, 50, 40, 1), (33, 517, 1760, 1), (64, 96, 320, 2)])
@pytest.mark.parametrize("columns", [8, 12, 20, 32])
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_skinny_gemm_reads_packed_weights(m, n, k, splits, columns, dtype):
    """The same product from the packed copy of the weights (chunks of K one after the other for
    each work-group's columns, K and the last group padded): right against float64, and bitwise
    what the plain layout gives, because only the addresses differ."""
    dt = DTYPES[dtype]
    a, w, bias, want = operands(m, n, k, dt, seed=k + columns, lda=k + 8)
    packed = K.pack_columns(w, columns)
    chunk = 32 if dtype == "bfloat16" else 16
    assert packed.shape == ((n + columns - 1) // columns, (k + chunk - 1) // chunk, columns, chunk)
    plain = torch.full((splits, m, n), float("nan"), dtype=torch.float32, device=DEV)
    from_packed = torch.full((splits, m, n), float("nan"), dtype=torch.float32, device=DEV)
    K.gemm(a, w, K.epilogue_f32(plain, bias), splits=splits, impl="skinny", variant=columns)
    K.gemm(a, w, K.epilogue_f32(from_packed, bias), splits=splits, impl="skinny", packed=(packed, columns))
    assert torch.equal(plain, from_packed)
    assert rel_err(from_packed.sum(0), want + bias.cpu().double()) < (2e-6 if dtype == "float32" else 2e-5 * math.sqrt(k))


def test_packed_weight_is_used_only_where_it_fits():
    """A PackedWeight is laid out for one column count; steps whose launcher would choose another
    (another split of K, many rows) read the plain matrix, and so does every other kernel."""
    gen = torch.Generator().manual_seed(5)
    w = (torch.randn(1600, 640, generator=gen) / 25).to(torch.bfloat16).to(DEV)
    packed = K.PackedWeight(w, splits=2)
    units = torch.cuda.get_device_properties(DEV).multi_processor_count
    columns = K.skinny_columns(8, 1600, 640, 2, torch.bfloat16, units)
    assert list(packed.copies) == [columns]
    assert packed.for_step(8, 2) is not None and packed.for_step(8, 2)[1] == columns
    assert packed.for_step(65, 2) is None
    other = [s for s in (1, 2, 3, 4, 5) if K.skinny_columns(8, 1600, 640, s, torch.bfloat16, units) != columns]
    both = K.PackedWeight(w, splits=(2, 1))
    assert set(both.copies) == {columns, K.skinny_columns(8, 1600, 640, 1, torch.bfloat16, units)}
    assert both.for_step(2, 1) is not None
    for splits in other:
        assert packed.for_step(8, splits) is None
    for m, splits in ((1, 2), (8, 2), (16, 1), (40, 2), (100, 1)):
        a = (torch.randn(m, 640, generator=gen)).to(torch.bfloat16).to(DEV)
        with_copy = torch.full((splits, m, 1600), float("nan"), dtype=torch.float32, device=DEV)
        without = torch.full((splits, m, 1600), float("nan"), dtype=torch.float32, device=DEV)
        K.gemm(a, w, K.epilogue_f32(with_copy), splits=splits, packed=packed, impl="auto" if splits == 1 else "skinny" if m <= 64 else "tile")
        K.gemm(a, w, K.epilogue_f32(without), splits=splits, impl="auto" if splits == 1 else "skinny" if m <= 64 else "tile")
        assert torch.equal(with_copy, without)
    try:
        K.PackedWeight.enabled = False
        assert packed.for_step(8, 2) is None
    finally:
        K.PackedWeight.enabled = True


@pytest.mark.parametrize("m,n,k", [(1, 100, 136), (8, 6400, 1600), (16, 333, 1608), (9, 517, 64), (13, 4800, 2048),
                                   (3, 48, 1024), (16, 96, 1032)])
@pytest.mark.parametrize("kind,with_shift", [("layer_norm", True), ("rms_norm", False)])
@pytest.mark.parametrize("columns", [0, 8, 16, 28])
def test_skinny_gemm_normalises_its_rows_itself(m, n, k, kind, with_shift, columns):
    """The product of rows of the float32 residual stream that the kernel normalises itself against
    float64, and against the norm kernel followed by the plain product."""
    gen = torch.Generator().manual_seed(m * n + k)
    x = (torch.randn(m, k + 12, generator=gen) * 3.0 + 0.7).to(DEV)[:, :k]        # pitch unlike the width
    gamma = (1.0 + 0.2 * torch.randn(k, generator=gen)).to(DEV)
    beta = (0.3 * torch.randn(k, generator=gen)).to(DEV) if with_shift else None
    w = (torch.randn(n, k, generator=gen) / math.sqrt(k)).to(torch.bfloat16).to(DEV)
    bias = torch.randn(n, generator=gen).to(DEV)
    eps = 1e-5
    xd = x.cpu().double()
    if kind == "layer_norm":
        h = (xd - xd.mean(-1, keepdim=True)) / torch.sqrt(xd.var(-1, unbiased=False, keepdim=True) + eps)
    else:
        h = xd / torch.sqrt((xd ** 2).mean(-1, keepdim=True) + eps)
    h = h * gamma.cpu().double() + (beta.cpu().double() if with_shift else 0.0)
    want = gelu_tanh(h @ w.cpu().double().t() + bias.cpu().double())
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    operand = K.Normalized(x, gamma, beta, eps, kind)
    assert operand.shape == (m, k) and K.Normalized.possible(m, k)
    K.gemm(operand, w, K.epilogue_act(out, "gelu_tanh", bias), variant=columns)
    assert rel_err(out, want) < 6e-3
    normed = torch.empty(m, k, dtype=torch.bfloat16, device=DEV)
    K.add_norm(x.contiguous(), normed, gamma, beta, eps, kind)
    apart = torch.empty_like(out)
    K.gemm(normed, w, K.epilogue_act(apart, "gelu_tanh", bias), impl="skinny", variant=columns)
    assert rel_err(out, apart.double()) < 4e-3            # the statistics are summed in another order: a last bit of a row's values
    parts = torch.full((2, m, n), float("nan"), dtype=torch.float32, device=DEV)
    if k >= 256:
        K.gemm(operand, w, K.epilogue_f32(parts), splits=2, variant=columns)
        assert rel_err(parts.sum(0), h @ w.cpu().double().t()) < 6e-3
    with pytest.raises(K.KernelError, match="up to 16 rows"):
        K.gemm(K.Normalized(torch.zeros(17, k, device=DEV), gamma, beta, eps, kind), w,
               K.epilogue_store(torch.empty(17, n, dtype=torch.bfloat16, device=DEV)))


@pytest.mark.parametrize("impl,m,n,k,splits", [("skinny", 5, 96, 1600, 4), ("skinny", 64, 50, 6400, 8),
                                               ("skinny", 20, 1600, 320, 2), ("tile", 150, 200, 1600, 3),
                                               ("tile", 600, 1600, 6400, 3), ("tile", 512, 1600, 6400, 4)])
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_gemm_split_k_partials(impl, m, n, k, splits, dtype):
    a, w, bias, want = operands(m, n, k, DTYPES[dtype], seed=splits)
    parts = torch.full((splits, m, n), float("nan"), dtype=torch.float32, device=DEV)
    K.gemm(a, w, K.epilogue_f32(parts, bias), splits=splits, impl=impl)
    assert rel_err(parts.sum(0), want + bias.cpu().double()) < (2e-6 if dtype == "float32" else 2e-5 * math.sqrt(k))


@pytest.mark.parametrize("impl,dtype,m,n,k", [("plain", "float32", 9, 50, 24), ("tile", "bfloat16", 130, 96, 200),
                                               ("skinny", "bfloat16", 8, 1600, 6400), ("skinny", "bfloat16", 3, 40, 96),
                                               ("tile", "float32", 130, 96, 200), ("skinny", "float32", 8, 1600, 6400),
                                               ("skinny", "float32", 3, 40, 100)])
def test_gemm_adds_into_the_residual_stream(impl, dtype, m, n, k):
    a, w, bias, want = operands(m, n, k, DTYPES[dtype], seed=77)
    gen = torch.Generator().manual_seed(1)
    x0 = torch.randn(m, n, generator=gen)
    x = x0.clone().to(DEV)
    K.gemm(a, w, K.epilogue_residual(x, bias), impl=impl)
    tol = 2e-6 if dtype == "float32" else 2e-5 * math.sqrt(k)
    assert rel_err(x, x0.double() + want + bias.cpu().double()) < tol


def test_gemm_refuses_what_it_cannot_take():
    a, w, bias, _ = operands(4, 32, 20, torch.bfloat16)
    out = torch.empty(4, 32, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(K.KernelError, match="multiples of 8"):
        K.gemm(a, w, K.epilogue_store(out), impl="skinny")
    a, w, bias, _ = operands(80, 32, 64, torch.bfloat16)
    out = torch.empty(80, 32, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(K.KernelError, match="at most 64"):
        K.gemm(a, w, K.epilogue_store(out), impl="skinny")
    with pytest.raises(K.KernelError, match="partial sums"):
        K.gemm(a, w, K.epilogue_store(out), impl="tile", splits=2)
    a, w, bias, _ = operands(4, 32, 18, torch.float32)
    out = torch.empty(4, 32, dtype=torch.float32, device=DEV)
    with pytest.raises(K.KernelError, match="multiples of 4"):
        K.gemm(a, w, K.epilogue_store(out), impl="skinny")
    K.gemm(a, w, K.epilogue_store(out))                       # "auto" gives such float32 operands to the plain kernel
    assert rel_err(out, a.cpu().double() @ w.cpu().double().t()) < 2e-6
    with pytest.raises(K.KernelError, match="general form only"):
        a, w, bias, _ = operands(128, 128, 64, torch.float32)
        K.gemm(a, w, K.epilogue_store(torch.empty(128, 128, device=DEV)), impl="tile", variant=2)


@pytest.mark.parametrize("impl,dtype,counts", [("plain", "float32", [3, 1, 70]), ("plain", "bfloat16", [5, 2]),
                                               ("tile", "bfloat16", [100, 1, 37]), ("skinny", "bfloat16", [1, 1, 1]),
                                               ("skinny", "bfloat16", [9, 30]), ("tile", "float32", [100, 1, 37]),
                                               ("skinny", "float32", [1, 1, 1]), ("skinny", "float32", [9, 30])])
def test_fused_projection_scatters_into_the_cache(impl, dtype, counts):
    dt = DTYPES[dtype]
    q_heads, kv_heads, hd, width = 4, 2, 32, 72
    totals = [c + 61 + 7 * i for i, c in enumerate(counts)]
    case = PagedCase(totals, counts, kv_heads, hd, dt, DEV, seed=1)
    n_q, n_kv = q_heads * hd, kv_heads * hd
    a, w, bias, want = operands(case.n_tokens, n_q + 2 * n_kv, width, dt, seed=9)
    want = want + bias.cpu().double()
    q = torch.full((case.n_tokens, n_q), float("nan"), dtype=dt, device=DEV)
    before_k, before_v = case.read_back()
    K.gemm(a, w, K.epilogue_qkv(q, n_q, n_kv, case.view(), case.tok_seq, case.tok_pos, bias), impl=impl,
           variant=12 if impl == "skinny" and case.n_tokens <= 16 else 0)
    after_k, after_v = case.read_back()
    tol = 2e-6 if dtype == "float32" else 6e-3
    assert rel_err(q, want[:, :n_q]) < tol
    row, base = 0, 0
    for total, count in zip(totals, counts):
        new = slice(base + total - count, base + total)
        old = slice(base, base + total - count)
        assert rel_err(after_k[new], want[row:row + count, n_q:n_q + n_kv]) < tol
        assert rel_err(after_v[new], want[row:row + count, n_q + n_kv:]) < tol
        assert torch.equal(after_k[old], before_k[old]) and torch.equal(after_v[old], before_v[old])
        row, base = row + count, base + total


ATTN_CASES = [
    # q_heads, kv_heads, head_dim, totals, counts, window
    (2, 2, 16, [5, 11, 17], [5, 11, 17], 0),          # whole prompts
    (3, 1, 48, [70, 130], [1, 1], 0),                 # decode, grouped heads, two blocks
    (4, 2, 32, [200, 64, 65], [40, 64, 1], 0),        # chunks on non-empty caches, block edges
    (2, 2, 64, [300, 129], [300, 2], 50),             # window
    (5, 5, 80, [33], [33], 0),
    (2, 1, 128, [260, 31], [1, 1], 100),              # decode with a window
    (4, 2, 64, [200, 64, 65, 131], [40, 64, 1, 131], 0),   # heads of 64 without a window: keys and values go through LDS
    (3, 3, 64, [33, 700], [33, 129], 0),
]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("q_heads,kv_heads,hd,totals,counts,window", ATTN_CASES)
def test_attention_plain(dtype, q_heads, kv_heads, hd, totals, counts, window):
    dt = DTYPES[dtype]
    case = PagedCase(totals, counts, kv_heads, hd, dt, DEV, seed=2, poison=True)
    gen = torch.Generator().manual_seed(5)
    q = torch.randn(case.n_tokens, q_heads * hd, generator=gen).to(dt).to(DEV)
    out = torch.full((case.n_tokens, q_heads * hd), float("nan"), dtype=dt, device=DEV)
    scale = 0.37 / math.sqrt(hd)
    args = K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                            q_heads, len(totals), max(counts), scale, window)
    K.attention(args, dt, decode=max(counts) == 1, impl="plain")
    want = case.reference(q, q_heads, scale, window)
    assert rel_err(out, want) < (3e-6 if dtype == "float32" else 8e-3)


@pytest.mark.parametrize("q_heads,kv_heads,hd,totals,counts,window",
                         ATTN_CASES + [(2, 1, 112, [500, 64, 1], [500, 33, 1], 0), (1, 1, 96, [130], [70], 33),
                                       # heads of 128: the one size whose LDS passes 64 KiB, prompts and chunks
                                       (2, 1, 128, [300, 129], [171, 129], 0), (3, 3, 128, [70, 200, 64], [70, 40, 64], 0)])
def test_attention_tiled_float32(q_heads, kv_heads, hd, totals, counts, window):
    """The float path's tiled kernel: prompts, chunks and single tokens through the same code; a
    query's result is bitwise the same whether it comes alone or among others."""
    dt = torch.float32
    case = PagedCase(totals, counts, kv_heads, hd, dt, DEV, seed=2, poison=True)
    gen = torch.Generator().manual_seed(5)
    q = torch.randn(case.n_tokens, q_heads * hd, generator=gen).to(DEV)
    out = torch.full((case.n_tokens, q_heads * hd), float("nan"), dtype=dt, device=DEV)
    scale = 0.37 / math.sqrt(hd)
    args = K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                            q_heads, len(totals), max(counts), scale, window)
    K.attention(args, dt, decode=max(counts) == 1, impl="tiled")
    want = case.reference(q, q_heads, scale, window)
    assert rel_err(out, want) < 3e-6
    # the last token of every sequence alone, as a decode step brings it (a kernel of its own)
    last = [int(case.seq_off[i + 1]) - 1 for i in range(len(totals))]
    alone = PagedCase(totals, [1] * len(totals), kv_heads, hd, dt, DEV, seed=2, poison=True)
    q1 = q[last].contiguous()
    out1 = torch.full((len(totals), q_heads * hd), float("nan"), dtype=dt, device=DEV)
    args = K.attention_args(q1, out1, alone.view(), alone.tok_seq, alone.tok_pos, alone.seq_off, alone.seq_start,
                            q_heads, len(totals), 1, scale, window)
    K.attention(args, dt, decode=True, impl="tiled")
    assert rel_err(out1, want[last]) < 3e-6
    # the last two tokens of every sequence that has two: the tiled kernel again, and bitwise what
    # it gave the same queries among the others of their step
    pairs = [i for i, c in enumerate(counts) if c >= 2]
    if pairs:
        sub_totals = [totals[i] for i in pairs]
        two = PagedCase(totals, [2 if i in pairs else 1 for i in range(len(totals))], kv_heads, hd, dt, DEV, seed=2,
                        poison=True)
        rows = []
        for i in range(len(totals)):
            rows += [last[i] - 1, last[i]] if i in pairs else [last[i]]
        q2 = q[rows].contiguous()
        out2 = torch.full((len(rows), q_heads * hd), float("nan"), dtype=dt, device=DEV)
        args = K.attention_args(q2, out2, two.view(), two.tok_seq, two.tok_pos, two.seq_off, two.seq_start,
                                q_heads, len(totals), 2, scale, window)
        K.attention(args, dt, decode=False, impl="tiled")
        keep = [r for r, row in enumerate(rows) if (row in last and any(row == last[i] for i in pairs)) or row + 1 in last]
        assert torch.equal(out2[keep], out[[rows[r] for r in keep]])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("totals,counts", [([5, 70], [5, 3]), ([130, 67, 9, 260], [130, 66, 2, 77]),
                                           ([300], [299])])
@pytest.mark.parametrize("kv_heads,hd", [(3, 16), (41, 64)])      # the second: more than one round of 8 x 256 channels
def test_kv_copy_round_trip(dtype, totals, counts, kv_heads, hd):
    """Rows written into the paged cache (a few tokens: element by element; a prompt in bfloat16: runs
    of four positions at a time, starting anywhere) come back unchanged, and nothing else is touched."""
    dt = DTYPES[dtype]
    case = PagedCase(totals, counts, kv_heads, hd, dt, DEV, seed=4)
    before_k, before_v = case.read_back()
    gen = torch.Generator().manual_seed(8)
    pitch = 2 * kv_heads * hd + 8
    rows = torch.randn(case.n_tokens, pitch, generator=gen).to(dt).to(DEV)
    new_k, new_v = rows[:, :kv_heads * hd], rows[:, kv_heads * hd:2 * kv_heads * hd]
    K.kv_copy(new_k, new_v, case.tok_seq, case.tok_pos, case.view(), True)
    after_k, after_v = case.read_back()
    row, begin = 0, 0
    for total, count in zip(totals, counts):
        old = slice(begin, begin + total - count)
        new = slice(begin + total - count, begin + total)
        assert torch.equal(after_k[old], before_k[old]) and torch.equal(after_v[old], before_v[old])
        assert torch.equal(after_k[new], new_k[row:row + count]) and torch.equal(after_v[new], new_v[row:row + count])
        row, begin = row + count, begin + total


# More query tiles than the GPU has compute units: the prefill kernel then pairs a late tile
# with an early one in each work-group (an even and an odd number of tiles, sequences shorter
# than the longest, chunks on non-empty caches, a window).
PAIRED_CASES = [
    (8, 4, 32, [700, 300, 650, 129, 640, 513], [700, 300, 650, 129, 640, 513], 0),
    (4, 4, 64, [600] * 13 + [100], [600] * 13 + [100], 0),
    (8, 4, 32, [900, 800, 700, 650, 600, 560, 520, 512, 1000], [500, 500, 300, 129, 128, 1, 64, 500, 512], 0),
    (6, 6, 64, [400] * 12, [400] * 12, 100),
]


@pytest.mark.parametrize("q_heads,kv_heads,hd,totals,counts,window", ATTN_CASES + PAIRED_CASES)
def test_attention_mfma(q_heads, kv_heads, hd, totals, counts, window):
    dt = torch.bfloat16
    case = PagedCase(totals, counts, kv_heads, hd, dt, DEV, seed=3, poison=True)
    gen = torch.Generator().manual_seed(6)
    q = torch.randn(case.n_tokens, q_heads * hd, generator=gen).to(dt).to(DEV)
    scale = 0.37 / math.sqrt(hd)
    want = case.reference(q, q_heads, scale, window)
    kinds = [False] + ([True] if max(counts) == 1 else [])
    for decode in kinds:
        out = torch.full((case.n_tokens, q_heads * hd), float("nan"), dtype=dt, device=DEV)
        args = K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                                q_heads, len(totals), max(counts), scale, window)
        K.attention(args, dt, decode=decode, impl="mfma")
        assert rel_err(out, want) < 1.2e-2, f"decode kernel={decode}"


def test_attention_finds_one_far_key_among_hundreds():
    """One key far back is made to dominate; an off-by-one in block or tile addressing loses it."""
    hd, total = 64, 700
    for dt, target in [(torch.bfloat16, t) for t in (0, 63, 64, 333, 671, 672, 698, 699)] + [(torch.float32, t) for t in (0, 64, 333, 698, 699)]:
        case = PagedCase([total], [1], 1, hd, dt, DEV, seed=target)
        q = torch.zeros(1, hd)
        q[0, 3] = 8.0
        case.k_rows[0][:] *= 0.05
        case.k_rows[0][target, 3] = 8.0
        seq = torch.zeros(total, dtype=torch.int32, device=DEV)
        pos = torch.arange(total, dtype=torch.int32, device=DEV)
        K.kv_copy(case.k_rows[0].to(DEV), case.v_rows[0].to(DEV), seq, pos, case.view(), True)
        q = q.to(dt).to(DEV)
        want = case.reference(q, 1, 1.0)
        assert (want[0] - case.v_rows[0][target].double()).abs().max() < 1e-3
        impls = (("plain", True), ("mfma", True), ("mfma", False)) if dt == torch.bfloat16 else (("plain", True), ("tiled", True))
        for impl, decode in impls:
            out = torch.empty(1, hd, dtype=dt, device=DEV)
            args = K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                                    1, 1, 1, 1.0, 0)
            K.attention(args, dt, decode=decode, impl=impl)
            assert rel_err(out, want) < 1e-2, (target, impl, decode)


def _dominant_target(row, pos):
    """The one key query ``row`` at position ``pos`` looks at: its own position, the one before, the
    first key of its block of 64, the last key of the tile of 32 before its own, key 0, or a key
    of an odd block of 64 far back."""
    kind = row % 6
    if kind == 0:
        return pos
    if kind == 1:
        return max(pos - 1, 0)
    if kind == 2:
        return pos // 64 * 64
    if kind == 3:
        return max(pos // 32 * 32 - 1, 0)
    if kind == 4:
        return 0
    return 64 * (2 * (pos // 128) - 1) + pos % 64 if pos >= 128 else pos // 2


@pytest.mark.parametrize("dtype,q_heads,kv_heads,hd,totals,counts", [
    ("bfloat16", 2, 2, 64, [700, 450, 333], [517, 450, 70]),        # chunks that start at 183 and 263
    ("bfloat16", 4, 2, 32, [700, 450, 333], [517, 450, 70]),
    ("bfloat16", 4, 4, 64, [600] * 13 + [100], [600] * 13 + [100]),   # more query tiles than compute units
    ("bfloat16", 2, 1, 128, [300, 129], [171, 129]),
    ("float32", 2, 2, 64, [700, 450, 333], [517, 450, 70]),
    ("float32", 3, 3, 48, [300, 129], [171, 129]),
    ("float32", 2, 1, 128, [300, 129], [171, 129]),
])
def test_prefill_attention_every_query_finds_its_one_key(dtype, q_heads, kv_heads, hd, totals, counts):
    """Every query of a prompt (or chunk) is given ONE key that takes all the weight, at a place
    chosen to sit on the edges of the kernels' tiles: on the diagonal, just before it, at the first
    key of the query's block, at the last key of the tile before, at key 0, in an odd block far
    back.  A key that a tile edge, the bound of the unmasked tiles, or the hand-over between the two
    halves of a work-group loses or counts twice changes the query's output from that key's value
    row to some other's, which no tolerance hides."""
    dt = DTYPES[dtype]
    case = PagedCase(totals, counts, kv_heads, hd, dt, DEV, seed=31, poison=True)
    group = q_heads // kv_heads
    q = torch.zeros(case.n_tokens, q_heads * hd)
    row = 0
    for s, (total, count) in enumerate(zip(totals, counts)):
        keys = case.k_rows[s].float().view(total, kv_heads, hd)
        keys = keys / keys.norm(dim=-1, keepdim=True)          # unit keys: a key's score with itself is the largest
        case.k_rows[s] = keys.reshape(total, kv_heads * hd).to(dt)
        stored = case.k_rows[s].float().view(total, kv_heads, hd)
        for i in range(count):
            pos = total - count + i
            for head in range(q_heads):
                q[row, head * hd:(head + 1) * hd] = stored[_dominant_target(row + head, pos), head // group]
            row += 1
    seq = torch.cat([torch.full((t,), s, dtype=torch.int32) for s, t in enumerate(totals)]).to(DEV)
    pos = torch.cat([torch.arange(t, dtype=torch.int32) for t in totals]).to(DEV)
    K.kv_copy(torch.cat(case.k_rows).to(DEV), torch.cat(case.v_rows).to(DEV), seq, pos, case.view(), True)
    q = q.to(dt).to(DEV)
    scale = 60.0           # the target scores 60, any other key 60 cos(angle): below 40 among random directions
    want = case.reference(q, q_heads, scale)
    # the premise: every output row IS (nearly) one value row
    row = 0
    for s, (total, count) in enumerate(zip(totals, counts)):
        values = case.v_rows[s].double().view(total, kv_heads, hd)
        for i in range(0, count, 37):
            target = _dominant_target(row + i, total - count + i)
            assert (want[row + i, :hd] - values[target, 0]).abs().max() < 2e-2
        row += count
    impl = "mfma" if dtype == "bfloat16" else "tiled"
    out = torch.full((case.n_tokens, q_heads * hd), float("nan"), dtype=dt, device=DEV)
    args = K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                            q_heads, len(totals), max(counts), scale, 0)
    K.attention(args, dt, decode=False, impl=impl)
    error = (out.detach().cpu().double() - want).abs().max(dim=1).values
    worst = int(error.argmax())
    assert float(error.max()) < (2e-2 if dtype == "bfloat16" else 1e-4), \
        f"query row {worst} (position {int(case.tok_pos[worst])} of sequence {int(case.tok_seq[worst])}) is off by {float(error.max())}"


@pytest.mark.parametrize("dtype,hd,window,totals,counts", [
    ("bfloat16", 64, 100, [700, 333], [517, 70]),
    ("bfloat16", 32, 64, [300, 200], [300, 1]),
    ("bfloat16", 64, 33, [500, 90, 41], [1, 1, 1]),            # a decode step
    ("float32", 64, 100, [700, 333], [517, 70]),
    ("float32", 48, 33, [500, 90, 41], [1, 1, 1]),
    ("float32", 128, 70, [400, 150], [333, 70]),
    ("bfloat16", 128, 70, [400, 150], [333, 70]),
])
def test_attention_at_the_edge_of_a_window(dtype, hd, window, totals, counts):
    """A query with a window of w sees keys pos - w + 1 ... pos.  Every even query is given one key
    that takes all the weight at the first position it still sees, every odd query at the position
    just before, which it must not see: counted in, that key would turn the output into its value
    row; left out, the output is the softmax over the window.  An off-by-one at either edge shows
    as an error of the size of a value, in the kernels for prompts and for single tokens."""
    dt = DTYPES[dtype]
    q_heads = kv_heads = 2
    case = PagedCase(totals, counts, kv_heads, hd, dt, DEV, seed=41, poison=True)
    q = torch.zeros(case.n_tokens, q_heads * hd)
    row, inside, outside = 0, 0, 0
    for s, (total, count) in enumerate(zip(totals, counts)):
        keys = case.k_rows[s].float().view(total, kv_heads, hd)
        keys = keys / keys.norm(dim=-1, keepdim=True)
        case.k_rows[s] = keys.reshape(total, kv_heads * hd).to(dt)
        stored = case.k_rows[s].float().view(total, kv_heads, hd)
        for i in range(count):
            pos = total - count + i
            target = pos - window + 1 if row % 2 == 0 else pos - window
            if target >= 0:
                q[row] = stored[target].reshape(-1)
                inside, outside = inside + (row % 2 == 0), outside + (row % 2 == 1)
            else:
                q[row] = stored[pos].reshape(-1)
            row += 1
    assert inside > 0 and outside > 0
    seq = torch.cat([torch.full((t,), s, dtype=torch.int32) for s, t in enumerate(totals)]).to(DEV)
    pos = torch.cat([torch.arange(t, dtype=torch.int32) for t in totals]).to(DEV)
    K.kv_copy(torch.cat(case.k_rows).to(DEV), torch.cat(case.v_rows).to(DEV), seq, pos, case.view(), True)
    q = q.to(dt).to(DEV)
    scale = 60.0
    want = case.reference(q, q_heads, scale, window)
    decode = max(counts) == 1
    impls = (["mfma"] if dtype == "bfloat16" else ["tiled"]) + ["plain"]
    for impl in impls:
        for as_decode in ([False, True] if decode and impl == "mfma" else [decode]):
            out = torch.full((case.n_tokens, q_heads * hd), float("nan"), dtype=dt, device=DEV)
            args = K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                                    q_heads, len(totals), max(counts), scale, window)
            K.attention(args, dt, decode=as_decode, impl=impl)
            error = (out.detach().cpu().double() - want).abs().max(dim=1).values
            worst = int(error.argmax())
            assert float(error.max()) < (3e-2 if dtype == "bfloat16" else 1e-4), \
                f"{impl} (decode kernel: {as_decode}): query row {worst} at position {int(case.tok_pos[worst])} is off by {float(error.max())}"


@pytest.mark.parametrize("dtype,hd,window", [("bfloat16", 64, 0), ("bfloat16", 32, 0), ("bfloat16", 64, 3000),
                                             ("float32", 64, 0), ("float32", 112, 0), ("float32", 48, 1500)])
def test_attention_decode_in_runs(dtype, hd, window):
    """Long contexts of a small batch cut into runs that separate work-groups take and a second
    kernel joins: every number of runs gives the result of the undivided kernel, also where a run
    is empty (a short sequence beside long ones), and a single dominant key is found in whichever
    run it falls."""
    dt = DTYPES[dtype]
    q_heads, kv_heads = 4, 2
    totals = [5000, 2100, 70, 4097, 1]
    case = PagedCase(totals, [1] * len(totals), kv_heads, hd, dt, DEV, seed=21, poison=True)
    gen = torch.Generator().manual_seed(22)
    q = torch.randn(len(totals), q_heads * hd, generator=gen) * 0.3
    # sequence 0: head 0 looks at key 4321 alone, head 3 at key 17; sequence 3: head 1 at its last block
    targets = [(0, 0, 4321), (0, 3, 17), (3, 1, 4040)]
    seq = torch.cat([torch.full((t,), s, dtype=torch.int32) for s, t in enumerate(totals)]).to(DEV)
    pos = torch.cat([torch.arange(t, dtype=torch.int32) for t in totals]).to(DEV)
    for s, head, key in targets:
        channels = slice((head // 2) * hd, (head // 2) * hd + hd)
        case.k_rows[s][:, channels] *= 0.05
        case.k_rows[s][key, (head // 2) * hd + 3] = 8.0
        q[s, head * hd:(head + 1) * hd] = 0.0
        q[s, head * hd + 3] = 8.0
    K.kv_copy(torch.cat(case.k_rows).to(DEV), torch.cat(case.v_rows).to(DEV), seq, pos, case.view(), True)
    q = q.to(dt).to(DEV)
    want = case.reference(q, q_heads, 1.0, window)
    for s, head, key in targets:
        if window == 0 or key > totals[s] - 1 - window:
            value = case.v_rows[s][key, (head // 2) * hd:(head // 2) * hd + hd].double()
            assert (want[s, head * hd:(head + 1) * hd] - value).abs().max() < 1e-3
    impl = "mfma" if dtype == "bfloat16" else "tiled"
    bound = 1.2e-2 if dtype == "bfloat16" else 3e-6
    for runs in (1, 2, 5, 19, 64):
        out = torch.full((len(totals), q_heads * hd), float("nan"), dtype=dt, device=DEV)
        partial = torch.full((len(totals) * q_heads * runs, hd + 2), float("nan"), device=DEV) if runs > 1 else None
        args = K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                                q_heads, len(totals), 1, 1.0, window, partial)
        K.attention(args, dt, decode=True, impl=impl)
        assert rel_err(out, want) < bound, runs
    with pytest.raises(K.KernelError, match="do not fit"):
        K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                         q_heads, len(totals), 1, 1.0, window, torch.zeros(7, hd + 2, device=DEV))


@pytest.mark.parametrize("q_heads,kv_heads", [(2, 2), (4, 2)])
def test_prompt_attention_in_runs_of_keys(q_heads, kv_heads):
    """A chunk of a prompt behind a long context has few tiles of queries and many keys for each: the
    keys of every tile are cut into runs that separate work-groups take and a second kernel joins.
    Every number of runs gives what the undivided kernel gives (a chunk that starts off the block
    grid, a sequence with nothing behind its chunk, one shorter than a tile, runs that are empty for
    the early tiles), queries that look at ONE key find it in whichever run it falls, and the
    records are written into a buffer full of NaN, longer than the step needs."""
    dt, hd = torch.bfloat16, 64
    totals, counts = [3000, 300, 1183, 70], [256, 300, 200, 3]
    case = PagedCase(totals, counts, kv_heads, hd, dt, DEV, seed=31, poison=True)
    gen = torch.Generator().manual_seed(32)
    q = torch.randn(case.n_tokens, q_heads * hd, generator=gen) * 0.3
    # queries of sequence 0 (positions 2744 ...): row 5 of head 0 looks at key 9 alone, row 130 at
    # key 1500, row 255 of the last head at its own position, row 200 at key 2688 (its tile's last block but one)
    group = q_heads // kv_heads
    targets = [(0, 5, 0, 9), (0, 130, 0, 1500), (0, 255, q_heads - 1, 2999), (0, 200, 0, 2688)]
    offsets = [0]
    for c in counts:
        offsets.append(offsets[-1] + c)
    for s, row, head, key in targets:
        kv_head = head // group
        case.k_rows[s][:, kv_head * hd:(kv_head + 1) * hd] *= 0.05
    for index, (s, row, head, key) in enumerate(targets):      # (a channel of its own for each, so that no query sees two)
        kv_head = head // group
        case.k_rows[s][key, kv_head * hd + 3 + 5 * index] = 8.0
        q[offsets[s] + row, head * hd:(head + 1) * hd] = 0.0
        q[offsets[s] + row, head * hd + 3 + 5 * index] = 8.0
    seq = torch.cat([torch.full((t,), i, dtype=torch.int32) for i, t in enumerate(totals)]).to(DEV)
    pos = torch.cat([torch.arange(t, dtype=torch.int32) for t in totals]).to(DEV)
    K.kv_copy(torch.cat(case.k_rows).to(DEV), torch.cat(case.v_rows).to(DEV), seq, pos, case.view(), True)
    q = q.to(dt).to(DEV)
    want = case.reference(q, q_heads, 1.0, 0)
    for s, row, head, key in targets:
        kv_head = head // group
        value = case.v_rows[s][key, kv_head * hd:(kv_head + 1) * hd].double()
        assert (want[offsets[s] + row, head * hd:(head + 1) * hd] - value).abs().max() < 2e-3, (row, key)
    results = {}
    for runs in (1, 2, 3, 8, 64):
        out = torch.full((case.n_tokens, q_heads * hd), float("nan"), dtype=dt, device=DEV)
        partial = torch.full(((case.n_tokens + 9) * q_heads * runs, hd + 2), float("nan"), device=DEV) if runs > 1 else None
        args = K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                                q_heads, len(totals), max(counts), 1.0, 0, partial, runs=runs if runs > 1 else None)
        K.attention(args, dt, decode=False, impl="mfma")
        assert rel_err(out, want) < 1.2e-2, runs
        for s, row, head, key in targets:
            got = out[offsets[s] + row, head * hd:(head + 1) * hd].double().cpu()
            assert (got - want[offsets[s] + row, head * hd:(head + 1) * hd].cpu()).abs().max() < 3e-2, (runs, row, key)
        results[runs] = out
    # runs are refused where the kernel that takes them does not run: a window, another head size
    partial = torch.zeros(case.n_tokens * q_heads * 2, hd + 2, device=DEV)
    args = K.attention_args(q, results[1].clone(), case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                            q_heads, len(totals), max(counts), 1.0, 100, partial, runs=2)
    with pytest.raises(K.KernelError, match="runs of keys"):
        K.attention(args, dt, decode=False, impl="mfma")
    with pytest.raises(K.KernelError, match="do not fit"):
        K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                         q_heads, len(totals), max(counts), 1.0, 0, torch.zeros(7, hd + 2, device=DEV), runs=2)


@pytest.mark.parametrize("pattern", ["ramp", "jumps", "falling"])
def test_attention_with_scores_that_rise_and_jump(pattern):
    """The running maximum is allowed to lag a little before sums are rescaled: scores that creep
    up (never rescaled after the first tile, probabilities above one), jump (rescaled at once)
    or fall (the first tile dominates) must all give the plain result."""
    dt = torch.bfloat16
    hd, total = 64, 600
    case = PagedCase([total], [total], 1, hd, dt, DEV, seed=11)
    position = torch.arange(total, dtype=torch.float32)
    if pattern == "ramp":
        gain = position / total * 30.0                    # about 1.6 per tile of 32 keys
    elif pattern == "jumps":
        gain = (position // 97) * 25.0 + (position % 7)
    else:
        gain = 40.0 - position / total * 40.0
    case.k_rows[0][:] *= 0.05
    case.k_rows[0][:, 5] = gain.to(dt)
    seq = torch.zeros(total, dtype=torch.int32, device=DEV)
    pos = torch.arange(total, dtype=torch.int32, device=DEV)
    K.kv_copy(case.k_rows[0].to(DEV), case.v_rows[0].to(DEV), seq, pos, case.view(), True)
    gen = torch.Generator().manual_seed(12)
    q = torch.randn(total, hd, generator=gen) * 0.1
    q[:, 5] = 1.0
    q = q.to(dt).to(DEV)
    want = case.reference(q, 1, 1.0)
    out = torch.empty(total, hd, dtype=dt, device=DEV)
    args = K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                            1, 1, total, 1.0, 0)
    K.attention(args, dt, decode=False, impl="mfma")
    assert rel_err(out, want) < 1.2e-2
    # the last query alone, through the decode kernel (its waves meet with their own maxima)
    one = PagedCase([total], [1], 1, hd, dt, DEV, seed=11)
    K.kv_copy(case.k_rows[0].to(DEV), case.v_rows[0].to(DEV), seq, pos, one.view(), True)
    out1 = torch.empty(1, hd, dtype=dt, device=DEV)
    args = K.attention_args(q[-1:], out1, one.view(), one.tok_seq, one.tok_pos, one.seq_off, one.seq_start,
                            1, 1, 1, 1.0, 0)
    K.attention(args, dt, decode=True, impl="mfma")
    assert rel_err(out1, want[-1:]) < 1.2e-2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width,rows", [(64, 3), (96, 17), (1600, 5), (50, 2), (1600, 515), (96, 1030),
                                        (2052, 513), (4096, 512), (50, 600)])
def test_add_norm(dtype, width, rows):
    """Few rows: a work-group per row; 512 rows and more: a wave per row."""
    dt = DTYPES[dtype]
    gen = torch.Generator().manual_seed(width)
    x = (torch.randn(rows, width, generator=gen) * 2 + 0.5).to(DEV)
    more = torch.randn(5, rows, width, generator=gen).to(DEV)
    delta = more[:3].contiguous()
    bias = torch.randn(width, generator=gen).to(DEV)
    gamma = (1 + 0.1 * torch.randn(width, generator=gen)).to(DEV)
    beta = torch.randn(width, generator=gen).to(DEV)
    total = x.double() + delta.double().sum(0) + bias.double()
    want = torch.nn.functional.layer_norm(total, (width,), gamma.double(), beta.double(), 1e-3)
    tol = 3e-6 if dtype == "float32" else 5e-3
    xs = x.clone()
    out = torch.empty(rows, width, dtype=dt, device=DEV)
    K.add_norm(xs, out, gamma, beta, 1e-3, "layer_norm", delta=delta, bias=bias)
    assert rel_err(out, want) < tol
    assert rel_err(xs, total) < 1e-6
    # other numbers of pending sums (the wave-per-row kernel has a form for each up to four, and a loop)
    for n in (1, 2, 4, 5):
        xs = x.clone()
        K.add_norm(xs, out, gamma, beta, 1e-3, "layer_norm", delta=more[:n].contiguous(), bias=bias)
        summed = x.double() + more[:n].double().sum(0) + bias.double()
        assert rel_err(xs, summed) < 1e-6, n
        assert rel_err(out, torch.nn.functional.layer_norm(summed, (width,), gamma.double(), beta.double(), 1e-3)) < tol, n
    # selected rows: nothing is written back
    pick = torch.tensor([rows - 1, 0], dtype=torch.int32, device=DEV)
    xs = x.clone()
    out = torch.empty(2, width, dtype=dt, device=DEV)
    K.add_norm(xs, out, gamma, beta, 1e-3, "layer_norm", delta=delta, bias=bias, rows=pick, write_back=False)
    assert rel_err(out, want[[rows - 1, 0]]) < tol
    assert torch.equal(xs, x)
    if rows >= 512:     # many selected rows, in another order
        pick = torch.arange(rows - 1, -1, -1, dtype=torch.int32, device=DEV)
        out = torch.empty(rows, width, dtype=dt, device=DEV)
        K.add_norm(xs, out, gamma, beta, 1e-3, "layer_norm", delta=delta, bias=bias, rows=pick, write_back=False)
        assert rel_err(out, want.flip(0)) < tol
        assert torch.equal(xs, x)
    # root-mean-square norm, no shift
    xs = x.clone()
    out = torch.empty(rows, width, dtype=dt, device=DEV)
    K.add_norm(xs, out, gamma, None, 1e-3, "rms_norm")
    want = x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-3) * gamma.double()
    assert rel_err(out, want) < tol


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed(dtype):
    dt = DTYPES[dtype]
    gen = torch.Generator().manual_seed(0)
    table = torch.randn(37, 50, generator=gen).to(dt).to(DEV)
    positions = torch.randn(20, 50, generator=gen).to(dt).to(DEV)
    ids = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32, device=DEV)
    pos = torch.tensor([19, 0, 3, 4, 7], dtype=torch.int32, device=DEV)
    out = torch.empty(5, 50, dtype=torch.float32, device=DEV)
    K.embed(ids, pos, table, positions, out)
    assert torch.equal(out, table[ids.long()].float() + positions[pos.long()].float())
    K.embed(ids, None, table, None, out)
    assert torch.equal(out, table[ids.long()].float())


def test_greedy_takes_the_lowest_index_of_the_maximum():
    gen = torch.Generator().manual_seed(0)
    logits = torch.randn(4, 50257, generator=gen)
    logits[0, 777] = logits[0, 40000] = 9.0
    logits[1, 50256] = 11.0
    logits[2, 0] = 12.0
    dev = logits.to(DEV)
    ids = torch.empty(4, dtype=torch.int32, device=DEV)
    logp = torch.empty(4, dtype=torch.float32, device=DEV)
    K.sample(dev, ids, logp)
    want = [777, 50256, 0, int(logits[3].argmax())]
    assert ids.tolist() == want
    ref = torch.log_softmax(logits.double(), -1)
    for r in range(4):
        assert abs(float(logp[r]) - float(ref[r, want[r]])) < 1e-4
    # other widths: a handful of logits, and more than 65,536 (more chunks per row); rows with a pitch
    for vocab in (3, 100, 70001):
        wide = torch.randn(5, vocab + 3, generator=gen)
        wide[1, vocab - 1] = wide[1, 0] = 20.0
        view = wide.to(DEV)[:, :vocab]
        ids = torch.empty(5, dtype=torch.int32, device=DEV)
        logp = torch.empty(5, dtype=torch.float32, device=DEV)
        K.sample(view, ids, logp)
        assert ids.tolist() == [int(x) for x in wide[:, :vocab].argmax(-1)] and int(ids[1]) == 0
        ref = torch.log_softmax(wide[:, :vocab].double(), -1)
        assert all(abs(float(logp[r]) - float(ref[r, int(ids[r])])) < 1e-4 for r in range(5))


@pytest.mark.parametrize("rows,vocab", [(64, 517), (5, 17), (9, 50257), (3, 70001)])
def test_sampling_is_the_inverse_cdf_of_the_tempered_softmax(rows, vocab):
    import plain_gpt2 as plain
    gen = torch.Generator().manual_seed(1)
    temperature, seed, first = 0.8, 1234567, 40
    logits = torch.randn(rows, vocab, generator=gen) * 3
    ids = torch.empty(rows, dtype=torch.int32, device=DEV)
    logp = torch.empty(rows, dtype=torch.float32, device=DEV)
    draw_rows = torch.arange(rows - 1, -1, -1, dtype=torch.int32, device=DEV)
    K.sample(logits.to(DEV), ids, logp, temperature=temperature, seed=seed, first_draw=first, draw_rows=draw_rows)
    exact = 0
    for r in range(rows):
        u = plain.interior_unit(plain.splitmix64(seed, first + rows - 1 - r))
        p = torch.softmax(logits[r].double() / temperature, -1)
        c = torch.cumsum(p, -1)
        k = int(ids[r])
        # the chosen index satisfies c[k-1] < u <= c[k] up to float32 rounding of the running sum
        lo = float(c[k - 1]) if k > 0 else 0.0
        assert lo - 1e-5 <= u <= float(c[k]) + 1e-5, (r, k, u, lo, float(c[k]))
        exact += k == plain.sample_index(logits[r], temperature, u)
        assert abs(float(logp[r]) - math.log(float(p[k]))) < 1e-4
    assert exact >= rows - 2
    # the same seed gives the same tokens; another seed does not
    again = torch.empty_like(ids)
    K.sample(logits.to(DEV), again, logp, temperature=temperature, seed=seed, first_draw=first, draw_rows=draw_rows)
    assert torch.equal(ids, again)
    K.sample(logits.to(DEV), again, logp, temperature=temperature, seed=seed + 1, first_draw=first, draw_rows=draw_rows)
    assert not torch.equal(ids, again)


class _Workspace:
    """Stands in for a step where only its buffers are asked for."""

    def buffer(self, key, rows, cols, dtype):
        return torch.full((rows, cols), float("nan"), dtype=dtype, device=DEV)


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("m,n,k,splits", [(1, 100, 136, 1), (8, 4800, 1600, 1), (16, 96, 1608, 3), (17, 333, 320, 1),
                                          (40, 517, 1760, 2), (64, 1600, 6400, 5), (64, 50, 40, 1)])
def test_chunk_major_activations_through_the_kernels_that_write_and_read_them(dtype, m, n, k, splits):
    """Activations of a small step in the chunk-major layout ([columns / chunk][rows][chunk], 64-byte
    chunks): written by the norm kernel and by a product's store and activation epilogues, read by
    the skinny product; every value is bitwise what the row-major path gives, only addresses differ."""
    dt = DTYPES[dtype]
    gen = torch.Generator().manual_seed(m * 1000 + k)
    x = (torch.randn(m, k, generator=gen) * 2 + 0.3).to(DEV)
    gamma = (1 + 0.1 * torch.randn(k, generator=gen)).to(DEV)
    beta = torch.randn(k, generator=gen).to(DEV)
    w = (torch.randn(n, k, generator=gen) / math.sqrt(k)).to(dt).to(DEV)
    bias = torch.randn(n, generator=gen).to(DEV)
    # the norm writes it
    rows_out = torch.empty(m, k, dtype=dt, device=DEV)
    K.add_norm(x.clone(), rows_out, gamma, beta, 1e-5, "layer_norm")
    chunked = K.Chunked.take(_Workspace(), "test", m, k, dt)
    K.add_norm(x.clone(), chunked, gamma, beta, 1e-5, "layer_norm")
    assert chunked.shape == (m, k) and torch.equal(chunked.to_rows(), rows_out)
    # the skinny product reads it, from the plain and from the packed weights
    plain = torch.full((splits, m, n), float("nan"), dtype=torch.float32, device=DEV)
    K.gemm(rows_out, w, K.epilogue_f32(plain, bias), splits=splits, impl="skinny")
    for packed in (None, K.PackedWeight(w, splits)):
        got = torch.full((splits, m, n), float("nan"), dtype=torch.float32, device=DEV)
        K.gemm(chunked, w, K.epilogue_f32(got, bias), splits=splits, packed=packed)
        assert torch.equal(got, plain)
    assert rel_err(plain.sum(0), rows_out.double().cpu() @ w.double().cpu().t() + bias.double().cpu()) < (
        2e-6 if dtype == "float32" else 2e-5 * math.sqrt(k))
    # a product's epilogues write it
    if splits == 1:
        for make in (K.epilogue_store, lambda o, b: K.epilogue_act(o, "gelu_tanh", b)):
            want = torch.full((m, n), float("nan"), dtype=dt, device=DEV)
            K.gemm(rows_out, w, make(want, bias), impl="skinny")
            got = K.Chunked.take(_Workspace(), "test", m, n, dt)
            K.gemm(chunked, w, make(got, bias))
            assert torch.equal(got.to_rows(), want)
    # what cannot read or write it says so
    with pytest.raises(K.KernelError, match="skinny kernel"):
        K.gemm(chunked, w, K.epilogue_f32(plain), impl="tile")
    if dtype == "bfloat16":
        big = torch.zeros(100, k, dtype=dt, device=DEV)
        with pytest.raises(K.KernelError, match="row-major"):
            K.gemm(big, w, K.epilogue_store(K.Chunked.take(_Workspace(), "test", 100, n, dt)), impl="library")


@pytest.mark.parametrize("q_heads,kv_heads,hd,totals", [(4, 4, 16, [5, 70, 1]), (6, 2, 48, [300, 64, 65, 1000]),
                                                        (25, 25, 64, [590] * 8), (8, 1, 128, [33, 2000])])
def test_decode_attention_writes_chunk_major_rows(q_heads, kv_heads, hd, totals):
    """The bfloat16 decode kernel (and the kernel that joins runs of keys) leaves its rows in the
    chunk-major layout when asked: the same bits as row-major; the other attention kernels refuse."""
    dt = torch.bfloat16
    case = PagedCase(totals, [1] * len(totals), kv_heads, hd, dt, DEV, seed=hd)
    gen = torch.Generator().manual_seed(hd + 1)
    q = (torch.randn(len(totals), q_heads * hd, generator=gen) * 0.5).to(dt).to(DEV)
    for runs in (1, 3):
        partial = torch.full((len(totals) * q_heads * runs, hd + 2), float("nan"), device=DEV) if runs > 1 else None
        want = torch.full((len(totals), q_heads * hd), float("nan"), dtype=dt, device=DEV)
        args = K.attention_args(q, want, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                                q_heads, len(totals), 1, 0.3, 0, partial)
        K.attention(args, dt, decode=True)
        got = K.Chunked.take(_Workspace(), "test", len(totals), q_heads * hd, dt)
        args = K.attention_args(q, got, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                                q_heads, len(totals), 1, 0.3, 0, partial)
        K.attention(args, dt, decode=True)
        assert torch.equal(got.to_rows(), want), runs
    assert rel_err(want, case.reference(q, q_heads, 0.3, 0)) < 1.2e-2
    for impl, decode in (("mfma", False), ("plain", True)):
        with pytest.raises(K.KernelError, match="chunk-major"):
            K.attention(args, dt, decode=decode, impl=impl)
