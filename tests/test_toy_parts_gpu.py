"""More toy parts, defined and registered here without touching the library's files: a
feed-forward that routes (two experts mixed by a softmax gate computed in float32), a position
encoding of another kind (sinusoids added to the token embedding), and, in a second model, a
norm of another kind (by the mean absolute value) with a readout that has a table of its own, a
bias and a soft cap.  All work on device tensors only, so the engine replays their decode steps
from a HIP graph like GPT-2's."""

from dataclasses import dataclass

import pytest
import torch

pytestmark = pytest.mark.gpu

import burn_transformers_amd as bt  # noqa: E402
import plain_gpt2 as plain  # noqa: E402
from burn_transformers_amd.engine.plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry  # noqa: E402
from burn_transformers_amd.kernels import library as K  # noqa: E402
from burn_transformers_amd.parts import Delta, Embedding, FeedForward, Norm, Readout, ResidualStream, register, unregister  # noqa: E402


class GatedExperts(FeedForward):
    """y = sum_e softmax(h . R^T)[e] * down_e(gelu(up_e(h))): the gate in float32, the experts
    through the library's own product kernel."""

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.inner, self.experts = params["width"], params["inner"], params["experts"]
        self.router = tensors["router"]
        self.up = [tensors[f"up{e}"] for e in range(self.experts)]
        self.down = [tensors[f"down{e}"] for e in range(self.experts)]

    def forward(self, h, step, stream):
        tokens = h.shape[0]
        gate = torch.softmax(h.float() @ self.router.float().t(), dim=-1)           # [tokens, experts], float32
        out = torch.zeros(1, tokens, self.width, dtype=torch.float32, device=h.device)
        for e in range(self.experts):
            hidden = step.buffer(f"toy.hidden{e}", tokens, self.inner, step.dtype)
            K.gemm(h, self.up[e], K.epilogue_act(hidden, "gelu_tanh"))
            y = step.buffer(f"toy.y{e}", tokens, self.width, "float32")
            K.gemm(hidden, self.down[e], K.epilogue_f32(y))
            out[0] += gate[:, e:e + 1] * y
        return Delta(out, None)


class SinusoidEmbedding(Embedding):
    """x0[t] = tokens[id[t]] + [sin(pos * f_i), cos(pos * f_i)], f_i = base^(-2i / width)."""

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.base = params["width"], params["base"]
        self.max_positions = params["max_positions"]
        self.token_table = tensors["tokens"]
        half = self.width // 2
        self.freq = torch.pow(torch.tensor(float(self.base)), -torch.arange(half, dtype=torch.float64) * 2 / self.width) \
            .to(torch.float32).to(self.token_table.device)

    def embed(self, step):
        x = step.buffer("stream.x", step.n_tokens, self.width, "float32")
        K.embed(step.tok_ids, None, self.token_table, None, x)
        angle = step.tok_pos.to(torch.float32)[:, None] * self.freq[None, :]
        x += torch.cat([torch.sin(angle), torch.cos(angle)], dim=-1)
        return ResidualStream(x)


@dataclass(frozen=True)
class RoutedConfig:
    width: int = 48
    inner: int = 80
    vocab_size: int = 61
    max_positions: int = 128
    heads: int = 3
    base: float = 50.0

    @classmethod
    def from_dict(cls, data):
        return cls(**{k: data[k] for k in cls.__dataclass_fields__ if k in data})

    def to_dict(self):
        return dict(architectures=["ToyRoutedLM"], **{k: getattr(self, k) for k in self.__dataclass_fields__})


def routed_plan(c):
    hd = c.width // c.heads
    norm = lambda p: PartSpec("layer_norm", {"width": c.width, "eps": 1e-5}, {"weight": p + ".g", "bias": p + ".b"})
    attention = PartSpec("attention", {"width": c.width, "heads": c.heads, "kv_heads": c.heads, "head_dim": hd,
                                       "scale": hd ** -0.5, "window": 0}, {"qkv_weight": "qkv", "out_weight": "out"})
    experts = PartSpec("toy_gated_experts", {"width": c.width, "inner": c.inner, "experts": 2},
                       {"router": "router", "up0": "up0", "up1": "up1", "down0": "down0", "down1": "down1"})
    layer = LayerPlan("pre_norm", {"mixer_norm": norm("n1"), "mixer": attention, "ff_norm": norm("n2"), "ff": experts})
    return ModelPlan(c.width, c.vocab_size, c.max_positions,
                     PartSpec("toy_sinusoid", {"width": c.width, "base": c.base, "max_positions": c.max_positions},
                              {"tokens": "tok"}),
                     [layer], [ScheduleEntry(0, 0)], norm("final"),
                     PartSpec("linear_readout", {"width": c.width, "vocab_size": c.vocab_size}, {"weight": "tok"}))


def routed_contract(c):
    d = c.width
    specs = [("tok", (c.vocab_size, d), "table"), ("qkv", (3 * d, d), "out_in"), ("out", (d, d), "out_in"),
             ("router", (2, d), "out_in"), ("up0", (c.inner, d), "out_in"), ("up1", (c.inner, d), "out_in"),
             ("down0", (d, c.inner), "out_in"), ("down1", (d, c.inner), "out_in")]
    for p in ("n1", "n2", "final"):
        specs += [(p + ".g", (d,), "vector"), (p + ".b", (d,), "vector")]
    return bt.Contract([bt.TensorSpec(*s) for s in specs])


def routed_init(c, generator):
    out = {}
    for spec in routed_contract(c).tensors:
        t = torch.randn(spec.shape, generator=generator) * (0.5 if spec.layout == "table" else spec.shape[-1] ** -0.5)
        out[spec.name] = (1 + 0.1 * t if spec.name.endswith(".g") else 0.1 * t) if spec.layout == "vector" else t
    out["router"] *= 3.0        # gates far from one half, so that a wrong gate shows
    return out


def routed_reference(ids, w, c):
    """Whole sequence in float64."""
    ln = lambda x, p: plain.layer_norm(x, w[p + ".g"], w[p + ".b"], 1e-5)
    d, hd, half = c.width, c.width // c.heads, c.width // 2
    pos = torch.arange(len(ids), dtype=torch.float64)
    freq = torch.pow(torch.tensor(c.base, dtype=torch.float64), -torch.arange(half, dtype=torch.float64) * 2 / d)
    x = w["tok"][ids] + torch.cat([torch.sin(pos[:, None] * freq), torch.cos(pos[:, None] * freq)], dim=-1)
    qkv = ln(x, "n1") @ w["qkv"].t()
    q, k, v = (plain.split_heads(qkv[:, i * d:(i + 1) * d], c.heads) for i in range(3))
    x = x + plain.merge_heads(plain.attention(q, k, v, hd ** -0.5)) @ w["out"].t()
    h = ln(x, "n2")
    gate = torch.softmax(h @ w["router"].t(), dim=-1)
    for e in range(2):
        x = x + gate[:, e:e + 1] * (plain.gelu_tanh(h @ w[f"up{e}"].t()) @ w[f"down{e}"].t())
    return ln(x, "final") @ w["tok"].t()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_routed_feed_forward_and_sinusoid_positions(dtype, tmp_path):
    register("feed_forward", "toy_gated_experts", GatedExperts)
    register("embedding", "toy_sinusoid", SinusoidEmbedding)
    bt.register_family(bt.Family("toy_routed", ("ToyRoutedLM",), (), RoutedConfig, routed_plan, routed_contract,
                                 routed_init))
    try:
        config = RoutedConfig()
        stored = bt.write_random_model(str(tmp_path), config.to_dict(), seed=5)
        model = bt.load_model(str(tmp_path), dtype=dtype)
        engine = bt.Engine(model, max_tokens=512, graphs="always")
        assert engine.use_graphs
        w = {k: v.double() for k, v in stored.items()}
        gen = torch.Generator().manual_seed(1)
        requests = [torch.randint(0, config.vocab_size, (n,), generator=gen).tolist() for n in (50, 12, 77)]
        wants = [routed_reference(torch.tensor(r), w, config) for r in requests]
        scale = max(float(x.abs().max()) for x in wants)
        tol = 2e-5 * (1 + scale) if dtype == "float32" else 2e-2 * scale
        gates = torch.softmax(plain.layer_norm(w["tok"][requests[0]], w["n2.g"], w["n2.b"], 1e-5) @ w["router"].t(), -1)
        assert float((gates[:, 0] - 0.5).abs().mean()) > 0.1           # the routing is not a formality
        # prompts of unequal length in one step, then one token each until the shortest ends, and on
        slots = [engine.open() for _ in requests]
        cut = [len(r) - 10 for r in requests]
        logits = engine.step([(s, r[:c]) for s, r, c in zip(slots, requests, cut)],
                             want=[list(range(c)) for c in cut]).clone()
        got, at = [[] for _ in requests], 0
        for i, c in enumerate(cut):
            got[i].append(logits[at:at + c])
            at += c
        for t in range(10):
            logits = engine.step([(s, [r[c + t]]) for s, r, c in zip(slots, requests, cut)]).clone()
            for i in range(len(requests)):
                got[i].append(logits[i:i + 1])
        assert engine.graph_replays >= 8
        for i, want in enumerate(wants):
            assert float((torch.cat(got[i]).cpu().double() - want).abs().max()) <= tol, f"request {i}"
    finally:
        unregister("feed_forward", "toy_gated_experts")
        unregister("embedding", "toy_sinusoid")
        bt.unregister_family("toy_routed")


class MeanAbsNorm(Norm):
    """y = x / (mean |x| + eps) * scale: statistics in float32 on what the stream holds once the
    pending sums are added."""

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.eps, self.scale = params["eps"], tensors["weight"]

    def apply(self, stream, step, rows=None):
        stream.flush()                                   # (adds what the part before left pending)
        x = stream.x if rows is None else stream.x[rows.long()]
        y = x / (x.abs().mean(dim=-1, keepdim=True) + self.eps) * self.scale
        return y.to(step.dtype)


class CappedReadout(Readout):
    """logits = cap * tanh((h . table^T + bias) / cap): a table of its own, a bias and a soft cap."""

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.cap, self.table, self.bias = params["cap"], tensors["weight"], tensors["bias"]

    def logits(self, h, step):
        out = step.buffer("toy.logits", h.shape[0], self.table.shape[0], "float32")
        K.gemm(h, self.table, K.epilogue_f32(out, self.bias))
        return self.cap * torch.tanh(out / self.cap)


@dataclass(frozen=True)
class CappedConfig:
    width: int = 64
    inner: int = 72
    vocab_size: int = 53
    max_positions: int = 96
    heads: int = 2
    cap: float = 3.0
    eps: float = 1e-3

    @classmethod
    def from_dict(cls, data):
        return cls(**{k: data[k] for k in cls.__dataclass_fields__ if k in data})

    def to_dict(self):
        return dict(architectures=["ToyCappedLM"], **{k: getattr(self, k) for k in self.__dataclass_fields__})


def capped_plan(c):
    hd = c.width // c.heads
    norm = lambda p: PartSpec("toy_mean_abs_norm", {"width": c.width, "eps": c.eps}, {"weight": p})
    attention = PartSpec("attention", {"width": c.width, "heads": c.heads, "kv_heads": c.heads, "head_dim": hd,
                                       "scale": hd ** -0.5, "window": 0}, {"qkv_weight": "qkv", "out_weight": "out"})
    ff = PartSpec("dense", {"width": c.width, "inner": c.inner, "activation": "gelu_tanh"},
                  {"up_weight": "up", "up_bias": "up.b", "down_weight": "down", "down_bias": "down.b"})
    layer = LayerPlan("pre_norm", {"mixer_norm": norm("n1"), "mixer": attention, "ff_norm": norm("n2"), "ff": ff})
    return ModelPlan(c.width, c.vocab_size, c.max_positions,
                     PartSpec("learned_positions", {"width": c.width, "vocab_size": c.vocab_size,
                                                    "max_positions": c.max_positions}, {"tokens": "tok", "positions": "pos"}),
                     [layer, layer], [ScheduleEntry(0, 0), ScheduleEntry(1, 1)], norm("final"),
                     PartSpec("toy_capped_readout", {"cap": c.cap}, {"weight": "head", "bias": "head.b"}))


def capped_contract(c):
    d = c.width
    specs = [("tok", (c.vocab_size, d), "table"), ("pos", (c.max_positions, d), "table"), ("head", (c.vocab_size, d), "out_in"),
             ("head.b", (c.vocab_size,), "vector"), ("qkv", (3 * d, d), "out_in"), ("out", (d, d), "out_in"),
             ("up", (c.inner, d), "out_in"), ("up.b", (c.inner,), "vector"), ("down", (d, c.inner), "out_in"),
             ("down.b", (d,), "vector"), ("n1", (d,), "vector"), ("n2", (d,), "vector"), ("final", (d,), "vector")]
    return bt.Contract([bt.TensorSpec(*s) for s in specs])


def capped_init(c, generator):
    out = {}
    for spec in capped_contract(c).tensors:
        t = torch.randn(spec.shape, generator=generator)
        if spec.layout == "vector":
            out[spec.name] = 1 + 0.2 * t if spec.name in ("n1", "n2", "final") else 0.3 * t
        else:
            out[spec.name] = t * (0.5 if spec.layout == "table" else spec.shape[-1] ** -0.5)
    out["head"] *= 4.0          # logits beyond the cap, so that a readout without it shows
    return out


def capped_reference(ids, w, c):
    """Whole sequence in float64; both layers share their tensors (the plan names one layer twice)."""
    norm = lambda x, p: x / (x.abs().mean(-1, keepdim=True) + c.eps) * w[p]
    d, hd = c.width, c.width // c.heads
    x = w["tok"][ids] + w["pos"][:len(ids)]
    for _ in range(2):
        qkv = norm(x, "n1") @ w["qkv"].t()
        q, k, v = (plain.split_heads(qkv[:, i * d:(i + 1) * d], c.heads) for i in range(3))
        x = x + plain.merge_heads(plain.attention(q, k, v, hd ** -0.5)) @ w["out"].t()
        x = x + plain.gelu_tanh(norm(x, "n2") @ w["up"].t() + w["up.b"]) @ w["down"].t() + w["down.b"]
    return c.cap * torch.tanh((norm(x, "final") @ w["head"].t() + w["head.b"]) / c.cap)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_norm_and_a_readout_of_other_kinds(dtype, tmp_path):
    register("norm", "toy_mean_abs_norm", MeanAbsNorm)
    register("readout", "toy_capped_readout", CappedReadout)
    bt.register_family(bt.Family("toy_capped", ("ToyCappedLM",), (), CappedConfig, capped_plan, capped_contract,
                                 capped_init))
    try:
        config = CappedConfig()
        stored = bt.write_random_model(str(tmp_path), config.to_dict(), seed=8)
        model = bt.load_model(str(tmp_path), dtype=dtype)
        engine = bt.Engine(model, max_tokens=512, graphs="always")
        w = {k: v.double() for k, v in stored.items()}
        gen = torch.Generator().manual_seed(2)
        requests = [torch.randint(0, config.vocab_size, (n,), generator=gen).tolist() for n in (70, 9, 33)]
        wants = [capped_reference(torch.tensor(r), w, config) for r in requests]
        assert max(float(x.abs().max()) for x in wants) > 0.9 * config.cap          # the cap is at work
        # bfloat16: the logits before the cap reach 10 and more and rounded weights move them by a per cent
        # (measured: 0.05 to 0.08; a missing cap or another norm is off by 0.5 and more)
        tol = 2e-5 if dtype == "float32" else 0.15
        slots = [engine.open() for _ in requests]
        cut = [len(r) - 6 for r in requests]
        logits = engine.step([(s, r[:c]) for s, r, c in zip(slots, requests, cut)],
                             want=[list(range(c)) for c in cut]).clone()
        got, at = [[] for _ in requests], 0
        for i, c in enumerate(cut):
            got[i].append(logits[at:at + c])
            at += c
        for t in range(6):
            logits = engine.step([(s, [r[c + t]]) for s, r, c in zip(slots, requests, cut)]).clone()
            for i in range(len(requests)):
                got[i].append(logits[i:i + 1])
        assert engine.graph_replays >= 4
        for i, want in enumerate(wants):
            error = float((torch.cat(got[i]).cpu().double() - want).abs().max())
            print(f"[toy norm and readout] {dtype} request {i}: max error {error:.3g}", flush=True)
            assert error <= tol, f"request {i}"
    finally:
        unregister("norm", "toy_mean_abs_norm")
        unregister("readout", "toy_capped_readout")
        bt.unregister_family("toy_capped")
