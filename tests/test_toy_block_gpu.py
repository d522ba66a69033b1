"""Toy arrangements of parts, defined and registered here without touching the library's files:

* a block whose parts carry other names than the library's own block uses ("tokens" and
  "channels" instead of "mixer" and "ff") and run side by side from ONE norm,
  x + mixer(norm(x)) + feed_forward(norm(x));
* a block without any mixer (norm and feed-forward only), which has no cache entry;
* a mixer with a position encoding of its own: it rotates queries and keys by their positions
  before the keys go into the cache (the token table gets no positions at all), with a kernel
  file of its own (``tests/toy_kernels/rotary_turn.hip``) that the package's build compiles and
  whose calls go into launch lists like the package's own.

The engine asks a block which of its parts mix tokens (``Block.mixers``) and what a run of it
keeps (``Block.cache_needs``); it knows no part by name."""

from dataclasses import dataclass

import pytest
import torch

pytestmark = pytest.mark.gpu

import burn_transformers_amd as bt  # noqa: E402
import plain_gpt2 as plain  # noqa: E402
from burn_transformers_amd.cache.storage import KVSpec  # noqa: E402
from burn_transformers_amd.engine.plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry  # noqa: E402
from burn_transformers_amd.kernels import library as K  # noqa: E402
from burn_transformers_amd.parts import Block, Mixer, register, unregister  # noqa: E402
import toy_kernels  # noqa: E402


class SideBySideBlock(Block):
    ROLES = {"norm": "norm", "tokens": "mixer", "channels": "feed_forward"}
    only_launches_kernels = True

    def forward(self, stream, step, memory):
        h = self.parts["norm"].apply(stream, step)
        for delta in (self.parts["tokens"].forward(h, step, memory, stream),
                      self.parts["channels"].forward(h, step, stream)):
            if delta is not None:
                stream.add(delta)


class ChannelsOnlyBlock(Block):
    ROLES = {"norm": "norm", "channels": "feed_forward"}
    only_launches_kernels = True

    def forward(self, stream, step, memory):
        assert memory is None
        delta = self.parts["channels"].forward(self.parts["norm"].apply(stream, step), step, stream)
        if delta is not None:
            stream.add(delta)


class RotatingAttention(Mixer):
    """Attention whose queries and keys are turned by their positions: channel pair (i, i + h/2) of
    a head by the angle pos * base^(-2i/h), computed in float32; keys are cached turned.  The turn
    is a kernel this test brings (``toy_kernels``): the part asks for its module by name, and does
    nothing in a step but launch kernels, so its steps are kept as launch lists."""

    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.heads, self.base = params["width"], params["heads"], params["base"]
        self.head_dim = self.width // self.heads
        self.qkv, self.out = tensors["qkv"], tensors["out"]
        half = self.head_dim // 2
        self.freq = torch.pow(torch.tensor(float(self.base), dtype=torch.float64),
                              -torch.arange(half, dtype=torch.float64) * 2 / self.head_dim).float().to(self.qkv.device)

    def kv_spec(self):
        return KVSpec(self.heads, self.head_dim, 0)

    def kernel_modules(self, dtype):
        attention = f"attention_bf16_hd{self.head_dim}" if dtype == torch.bfloat16 else "attention_f32"
        return [attention] + toy_kernels.register()

    def forward(self, h, step, memory, stream):
        tokens, d = h.shape[0], self.width
        qkv = step.buffer("toy.qkv", tokens, 3 * d, step.dtype)
        K.gemm(h, self.qkv, K.epilogue_store(qkv))
        K.launch("toy_rotary_turn", "bt_toy_rotary_turn_call", toy_kernels.RotaryTurnCall(
            dtype=K.DTYPE_CODES[step.dtype], tokens=tokens, parts=2, heads=self.heads, head_dim=self.head_dim,
            ld=qkv.stride(0), rows=qkv.data_ptr(), positions=step.tok_pos.data_ptr(), freq=self.freq.data_ptr()))
        kv = memory.kv()
        K.kv_copy(qkv[:, d:2 * d], qkv[:, 2 * d:], step.tok_seq, step.tok_pos, kv, to_cache=True)
        mixed = step.buffer("toy.mixed", tokens, d, step.dtype)
        K.attention(K.attention_args(qkv[:, :d], mixed, kv, step.tok_seq, step.tok_pos, step.seq_off, step.seq_start,
                                     self.heads, step.n_seqs, step.max_count, self.head_dim ** -0.5), step.dtype, step.decode)
        stream.add_product(step, mixed, self.out)


@dataclass(frozen=True)
class SideConfig:
    width: int = 64
    inner: int = 96
    vocab_size: int = 83
    max_positions: int = 256
    heads: int = 2
    base: float = 100.0

    @classmethod
    def from_dict(cls, data):
        return cls(**{k: data[k] for k in cls.__dataclass_fields__ if k in data})

    def to_dict(self):
        return dict(architectures=["ToySideBySideLM"], **{k: getattr(self, k) for k in self.__dataclass_fields__})


def side_plan(c):
    norm = lambda p: PartSpec("rms_norm", {"width": c.width, "eps": 1e-5}, {"weight": p})
    dense = lambda p: PartSpec("dense", {"width": c.width, "inner": c.inner, "activation": "gelu_tanh"},
                               {"up_weight": p + ".up", "down_weight": p + ".down"})
    turning = PartSpec("toy_rotating_attention", {"width": c.width, "heads": c.heads, "base": c.base},
                       {"qkv": "qkv", "out": "out"})
    layers = [LayerPlan("toy_side_by_side", {"norm": norm("n0"), "tokens": turning, "channels": dense("f0")}),
              LayerPlan("toy_channels_only", {"norm": norm("n1"), "channels": dense("f1")})]
    # the layer with the mixer runs twice, each run with keys and values of its own; between them the
    # layer that keeps nothing
    schedule = [ScheduleEntry(0, 0), ScheduleEntry(1, None), ScheduleEntry(0, 1)]
    return ModelPlan(c.width, c.vocab_size, c.max_positions,
                     PartSpec("token_only", {"width": c.width, "vocab_size": c.vocab_size,
                                             "max_positions": c.max_positions}, {"tokens": "tok"}),
                     layers, schedule, norm("final"),
                     PartSpec("linear_readout", {"width": c.width, "vocab_size": c.vocab_size}, {"weight": "tok"}))


def side_contract(c):
    d = c.width
    specs = [("tok", (c.vocab_size, d), "table"), ("qkv", (3 * d, d), "out_in"), ("out", (d, d), "out_in")]
    for p in ("f0", "f1"):
        specs += [(p + ".up", (c.inner, d), "out_in"), (p + ".down", (d, c.inner), "out_in")]
    specs += [(p, (d,), "vector") for p in ("n0", "n1", "final")]
    return bt.Contract([bt.TensorSpec(*s) for s in specs])


def side_init(c, generator):
    out = {}
    for spec in side_contract(c).tensors:
        t = torch.randn(spec.shape, generator=generator)
        out[spec.name] = 1 + 0.1 * t if spec.layout == "vector" else t * (0.5 if spec.layout == "table" else 1.5 * spec.shape[-1] ** -0.5)
    return out


def side_reference(ids, w, c, first_position=0):
    """Whole sequence in float64."""
    rms = lambda x, p: x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w[p]
    ff = lambda h, p: plain.gelu_tanh(h @ w[p + ".up"].t()) @ w[p + ".down"].t()
    d, hd = c.width, c.width // c.heads
    pos = torch.arange(len(ids), dtype=torch.float64) + first_position
    freq = torch.pow(torch.tensor(c.base, dtype=torch.float64), -torch.arange(hd // 2, dtype=torch.float64) * 2 / hd)
    cos, sin = torch.cos(pos[:, None] * freq), torch.sin(pos[:, None] * freq)

    def turn(x):          # [heads, tokens, hd]
        a, b = x[..., :hd // 2], x[..., hd // 2:]
        return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)

    def side_by_side(x):
        h = rms(x, "n0")
        qkv = h @ w["qkv"].t()
        q, k, v = (plain.split_heads(qkv[:, i * d:(i + 1) * d], c.heads) for i in range(3))
        mixed = plain.merge_heads(plain.attention(turn(q), turn(k), v, hd ** -0.5))
        return x + mixed @ w["out"].t() + ff(h, "f0")

    x = side_by_side(w["tok"][ids])
    x = x + ff(rms(x, "n1"), "f1")
    x = side_by_side(x)
    return rms(x, "final") @ w["tok"].t()


def test_the_toy_reference_depends_on_distances_only():
    """What pins the rotation in the float64 reference of this file: shifting every position by the
    same amount changes nothing (a wrong sign or a wrong pairing of channels would), and the
    rotation is not a formality."""
    c = SideConfig()
    w = {k: v.double() for k, v in side_init(c, torch.Generator().manual_seed(2)).items()}
    ids = torch.randint(0, c.vocab_size, (40,), generator=torch.Generator().manual_seed(3))
    base = side_reference(ids, w, c)
    assert float((side_reference(ids, w, c, first_position=77) - base).abs().max()) < 1e-9
    still = SideConfig(base=1e30)          # angles of (almost) zero for all but the first pair
    assert float((side_reference(ids, w, still) - base).abs().max()) > 1e-3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_blocks_with_other_roles_no_mixer_and_a_turning_mixer(dtype, tmp_path):
    register("block", "toy_side_by_side", SideBySideBlock)
    register("block", "toy_channels_only", ChannelsOnlyBlock)
    register("mixer", "toy_rotating_attention", RotatingAttention)
    bt.register_family(bt.Family("toy_side", ("ToySideBySideLM",), (), SideConfig, side_plan, side_contract, side_init))
    try:
        config = SideConfig()
        stored = bt.write_random_model(str(tmp_path), config.to_dict(), seed=7)
        model = bt.load_model(str(tmp_path), dtype=dtype)
        assert [len(block.mixers()) for block in model.blocks] == [1, 0]
        assert model.blocks[1].cache_needs() == (None, None) and model.cache_entries == 2
        engine = bt.Engine(model, max_tokens=1024, graphs="always")
        assert engine.use_graphs
        w = {k: v.double() for k, v in stored.items()}
        gen = torch.Generator().manual_seed(4)
        requests = [torch.randint(0, config.vocab_size, (n,), generator=gen).tolist() for n in (150, 9, 70)]
        wants = [side_reference(torch.tensor(r), w, config) for r in requests]
        scale = max(float(x.abs().max()) for x in wants)
        tol = 2e-5 * (1 + scale) if dtype == "float32" else 2e-2 * scale
        for round_ in range(2):                 # the second round takes the slots of the first
            slots = [engine.open() for _ in requests]
            cut = [len(r) - 8 for r in requests]
            logits = engine.step([(s, r[:c]) for s, r, c in zip(slots, requests, cut)],
                                 want=[list(range(c)) for c in cut]).clone()
            got, at = [[] for _ in requests], 0
            for i, c in enumerate(cut):
                got[i].append(logits[at:at + c])
                at += c
            for t in range(8):
                logits = engine.step([(s, [r[c + t]]) for s, r, c in zip(slots, requests, cut)]).clone()
                for i in range(len(requests)):
                    got[i].append(logits[i:i + 1])
            for i, want in enumerate(wants):
                err = float((torch.cat(got[i]).cpu().double() - want).abs().max())
                assert err <= tol, f"round {round_} request {i}: {err} > {tol}"
            for slot in slots:
                engine.close(slot)
        assert engine.graph_replays >= 8
        engine.cache.ledger.check()
        # The model only launches kernels (the toy's own among them), so its steps are kept as launch
        # lists: walked in C++ they give the bits that the same calls give one by one from Python.
        assert model.recordable and "toy_rotary_turn" in K.loaded_modules()
        listed = bt.Engine(model, max_tokens=1024, graphs=False)
        direct = bt.Engine(model, max_tokens=1024, graphs=False, programs=False)
        assert listed.use_programs and not direct.use_programs
        for round_ in range(3):                 # the last round's steps are all walked from their lists
            runs_before = listed.program_runs
            pairs = [(listed.open(), direct.open()) for _ in requests]
            for begin, end in ((0, 5), (5, 6), (6, 7), (7, 9)):
                a = listed.step([(p[0], r[begin:end]) for p, r in zip(pairs, requests)]).clone()
                b = direct.step([(p[1], r[begin:end]) for p, r in zip(pairs, requests)]).clone()
                assert torch.equal(a, b), f"round {round_} tokens {begin}..{end}"
            if round_ == 2:            # (earlier steps may have made workspaces grow, which drops the lists kept till then)
                assert any(name == "bt_toy_rotary_turn_call" for _, name, _ in listed.last_program.calls)
                assert listed.program_runs - runs_before == 4
            for a, b in pairs:
                listed.close(a)
                direct.close(b)
        assert direct.program_runs == 0
    finally:
        unregister("block", "toy_side_by_side")
        unregister("block", "toy_channels_only")
        unregister("mixer", "toy_rotating_attention")
        bt.unregister_family("toy_side")
