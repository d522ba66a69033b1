"""Each part alone, at sizes of its own; schedules that name a layer twice or share a cache;
and a toy mixer with state of its own that is registered from here, without touching the
library's files."""

import math
from dataclasses import dataclass

import pytest
import torch

pytestmark = pytest.mark.gpu

import burn_transformers_amd as bt  # noqa: E402
import plain_gpt2 as plain  # noqa: E402
from burn_transformers_amd.cache.storage import Cache, KVSpec, StateSpec  # noqa: E402
from burn_transformers_amd.engine.model import CausalLM  # noqa: E402
from burn_transformers_amd.engine.plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry  # noqa: E402
from burn_transformers_amd.parts import Delta, Memory, Mixer, ResidualStream, lookup, register, unregister  # noqa: E402
from burn_transformers_amd.weights.loader import WeightStore  # noqa: E402
from model_helpers import TINY_A, model_folder, prompts_for  # noqa: E402
from step_helpers import make_step  # noqa: E402

DEV = torch.device("cuda:0")
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 3e-6, "bfloat16": 1e-2}


def rel_err(got, want):
    got, want = got.detach().cpu().double(), want.detach().cpu().double()
    return float((got - want).abs().max() / (want.abs().max() + 1e-30))


def rnd(gen, *shape, scale=1.0):
    return torch.randn(*shape, generator=gen) * scale


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["layer_norm", "rms_norm"])
def test_norm_adds_what_is_pending_then_normalises(kind, dtype):
    gen = torch.Generator().manual_seed(1)
    width, tokens, eps = 88, 6, 3e-4
    weight, bias = 1 + rnd(gen, width, scale=0.2), rnd(gen, width)
    tensors = {"weight": weight.to(DEV)}
    if kind == "layer_norm":
        tensors["bias"] = bias.to(DEV)
    norm = lookup("norm", kind)({"width": width, "eps": eps}, tensors)
    x, parts, pbias = rnd(gen, tokens, width, scale=2), rnd(gen, 2, tokens, width), rnd(gen, width)
    stream = ResidualStream(x.clone().to(DEV))
    stream.add(Delta(parts.to(DEV), pbias.to(DEV)))
    step = make_step(DTYPES[dtype], [tokens])
    out = norm.apply(stream, step)
    total = x.double() + parts.double().sum(0) + pbias.double()
    if kind == "layer_norm":
        want = plain.layer_norm(total, weight.double(), bias.double(), eps)
    else:
        want = total / torch.sqrt((total ** 2).mean(-1, keepdim=True) + eps) * weight.double()
    assert rel_err(out, want) < TOL[dtype] and stream.pending is None
    assert rel_err(stream.x, total) < 1e-6
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    assert rel_err(norm.apply(stream, step, rows=rows), want[[4, 1]]) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width,inner,activation,tokens", [(80, 200, "gelu_erf", 5), (48, 72, "gelu_tanh", 70),
                                                           (64, 100, "gelu_tanh", 3), (48, 37, "gelu_erf", 70)])
def test_dense_feed_forward_alone(dtype, width, inner, activation, tokens):
    gen, dt = torch.Generator().manual_seed(2), DTYPES[dtype]
    up, down = rnd(gen, inner, width, scale=width ** -0.5).to(dt), rnd(gen, width, inner, scale=inner ** -0.5).to(dt)
    up_b, down_b = rnd(gen, inner), rnd(gen, width)
    part = lookup("feed_forward", "dense")(
        {"width": width, "inner": inner, "activation": activation},
        {"up_weight": up.to(DEV), "up_bias": up_b.to(DEV), "down_weight": down.to(DEV), "down_bias": down_b.to(DEV)})
    h = rnd(gen, tokens, width).to(dt)
    start = rnd(gen, tokens, width)
    stream = ResidualStream(start.clone().to(DEV))
    assert part.forward(h.to(DEV), make_step(dt, [tokens]), stream) is None
    stream.flush()
    act = plain.gelu_erf if activation == "gelu_erf" else plain.gelu_tanh
    want = act(h.double() @ up.double().t() + up_b.double()) @ down.double().t() + down_b.double()
    assert rel_err(stream.x.cpu().double() - start.double(), want) < TOL[dtype]
    with pytest.raises(ValueError, match="projections are"):
        lookup("feed_forward", "dense")({"width": width, "inner": inner + 8, "activation": activation}, part.tensors)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding_and_readout_alone(dtype):
    gen, dt = torch.Generator().manual_seed(3), DTYPES[dtype]
    vocab, width, positions = 123, 40, 30
    table, ptable = rnd(gen, vocab, width).to(dt), rnd(gen, positions, width).to(dt)
    embedding = lookup("embedding", "learned_positions")(
        {"width": width, "vocab_size": vocab, "max_positions": positions},
        {"tokens": table.to(DEV), "positions": ptable.to(DEV)})
    ids = [5, 122, 0, 7, 7]
    step = make_step(dt, [3, 2], starts=[10, 28], ids=ids)
    stream = embedding.embed(step)
    want = table[ids].double() + ptable[[10, 11, 12, 28, 29]].double()
    assert rel_err(stream.x, want) < 1e-7
    readout = lookup("readout", "linear_readout")({"width": width, "vocab_size": vocab}, {"weight": table.to(DEV)})
    h = rnd(gen, 4, width).to(dt)
    assert rel_err(readout.logits(h.to(DEV), step), h.double() @ table.double().t()) < TOL[dtype]


def attention_reference(x, qkv_w, qkv_b, out_w, out_b, heads, kv_heads, hd, scale, window):
    """Whole-sequence float64 attention with grouped heads; weights held [out, in]."""
    qkv = x @ qkv_w.t() + qkv_b
    n_q, n_kv = heads * hd, kv_heads * hd
    q = plain.split_heads(qkv[:, :n_q], heads)
    k = plain.split_heads(qkv[:, n_q:n_q + n_kv], kv_heads).repeat_interleave(heads // kv_heads, 0)
    v = plain.split_heads(qkv[:, n_q + n_kv:], kv_heads).repeat_interleave(heads // kv_heads, 0)
    mixed = plain.attention(q, k, v, scale, True, window or None)
    return plain.merge_heads(mixed) @ out_w.t() + out_b


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv_heads,hd,width,window", [(6, 2, 32, 104, 0), (3, 3, 16, 40, 5), (4, 1, 48, 64, 70)])
def test_attention_mixer_alone(dtype, heads, kv_heads, hd, width, window):
    gen, dt = torch.Generator().manual_seed(4), DTYPES[dtype]
    n_q, n_kv, scale = heads * hd, kv_heads * hd, 0.9 / math.sqrt(hd)
    qkv_w = rnd(gen, n_q + 2 * n_kv, width, scale=width ** -0.5).to(dt)
    out_w = rnd(gen, width, n_q, scale=n_q ** -0.5).to(dt)
    qkv_b, out_b = rnd(gen, n_q + 2 * n_kv, scale=0.3), rnd(gen, width)
    mixer = lookup("mixer", "attention")(
        {"width": width, "heads": heads, "kv_heads": kv_heads, "head_dim": hd, "scale": scale, "window": window},
        {"qkv_weight": qkv_w.to(DEV), "qkv_bias": qkv_b.to(DEV), "out_weight": out_w.to(DEV), "out_bias": out_b.to(DEV)})
    assert mixer.kv_spec() == KVSpec(kv_heads, hd, window)
    bt.kernels.library.prepare(dt, mixer.kernel_modules(dt))
    cache = Cache([mixer.kv_spec()], [None], max_tokens=512, max_sequence_length=256, dtype=dt, device=DEV)
    lengths = [90, 7]
    xs = [rnd(gen, n, width).to(dt) for n in lengths]
    want = [attention_reference(x.double(), qkv_w.double(), qkv_b.double(), out_w.double(), out_b.double(),
                                heads, kv_heads, hd, scale, window) for x in xs]
    slots = [cache.acquire() for _ in lengths]
    got = [[] for _ in lengths]
    # a chunk, a ragged second chunk, then single tokens for the longer sequence
    cuts = [[(0, 60), (60, 88), (88, 89), (89, 90)], [(0, 3), (3, 7)]]
    for round_ in range(4):
        live = [i for i in range(2) if round_ < len(cuts[i])]
        spans = [cuts[i][round_] for i in live]
        for i, (a, b) in zip(live, spans):
            cache.ledger.reserve(slots[i], b)
        step = make_step(dt, [b - a for a, b in spans], starts=[a for a, _ in spans], cache=cache,
                         slots=[slots[i] for i in live])
        h = torch.cat([xs[i][a:b] for i, (a, b) in zip(live, spans)]).to(DEV)
        stream = ResidualStream(torch.zeros(h.shape[0], width, device=DEV))
        assert mixer.forward(h, step, Memory(cache, 0, True, step), stream) is None
        stream.flush()
        out = stream.x.double().cpu()
        at = 0
        for i, (a, b) in zip(live, spans):
            got[i].append(out[at:at + b - a])
            cache.ledger.commit(slots[i], b)
            at += b - a
    for i in range(2):
        assert rel_err(torch.cat(got[i]), want[i]) < TOL[dtype], f"sequence {i}"


def gpt2_store(name, dtype):
    folder, config_json, weights = model_folder(name)
    family = bt.resolve_family(config_json)
    config = family.config_class.from_dict(config_json)
    from burn_transformers_amd.weights.loader import store_from_tensors
    store = store_from_tensors(weights, family.contract(config), dtype, DEV)
    return family, config, store, weights, config_json


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_schedule_may_name_a_layer_twice_and_share_a_cache(dtype):
    """Order of layers is data: layer 0 runs, layer 1 runs, layer 0 runs again with a cache entry
    of its own, then layer 1 runs reading the keys and values that layer 0's first run wrote."""
    family, config, store, weights, cfg = gpt2_store("A", DTYPES[dtype])
    plan = family.plan(config)
    plan.schedule = [ScheduleEntry(0, 0), ScheduleEntry(1, 1), ScheduleEntry(0, 2), ScheduleEntry(1, 0, writes=False)]
    model = CausalLM(plan, store, config, family)
    assert model.cache_entries == 3
    engine = bt.Engine(model, max_tokens=512)
    ids = prompts_for("A", [70], seed=8)[0]

    # the same schedule with the plain parts, whole sequence in float64
    w = {k: v.double() for k, v in weights.items()}
    x = plain.embed(torch.tensor(ids), torch.arange(len(ids)), w["wte.weight"], w["wpe.weight"])
    x = plain.block(x, w, 0, cfg)
    kv_source = plain.layer_norm(plain.embed(torch.tensor(ids), torch.arange(len(ids)), w["wte.weight"], w["wpe.weight"]),
                                 w["h.0.ln_1.weight"], w["h.0.ln_1.bias"], cfg["layer_norm_epsilon"])
    x = plain.block(x, w, 1, cfg)
    x = plain.block(x, w, 0, cfg)
    # layer 1 once more: its queries, but keys and values of layer 0's first run
    d, heads = cfg["n_embd"], cfg["n_head"]
    h = plain.layer_norm(x, w["h.1.ln_1.weight"], w["h.1.ln_1.bias"], cfg["layer_norm_epsilon"])
    q = (h @ w["h.1.attn.c_attn.weight"] + w["h.1.attn.c_attn.bias"])[:, :d]
    kv = kv_source @ w["h.0.attn.c_attn.weight"] + w["h.0.attn.c_attn.bias"]
    mixed = plain.attention(plain.split_heads(q, heads), plain.split_heads(kv[:, d:2 * d], heads),
                            plain.split_heads(kv[:, 2 * d:], heads), 1 / math.sqrt(d // heads))
    y = x + plain.merge_heads(mixed) @ w["h.1.attn.c_proj.weight"] + w["h.1.attn.c_proj.bias"]
    z = y + plain.mlp(plain.layer_norm(y, w["h.1.ln_2.weight"], w["h.1.ln_2.bias"], cfg["layer_norm_epsilon"]),
                      w["h.1.mlp.c_fc.weight"], w["h.1.mlp.c_fc.bias"], w["h.1.mlp.c_proj.weight"],
                      w["h.1.mlp.c_proj.bias"], "gelu_new")
    want = plain.layer_norm(z, w["ln_f.weight"], w["ln_f.bias"], cfg["layer_norm_epsilon"]) @ w["wte.weight"].t()

    slot = engine.open()
    rows = [engine.step([(slot, ids[:40])], want=[list(range(40))]).clone()]
    rows += [engine.step([(slot, [t])]).clone() for t in ids[40:]]
    got = torch.cat(rows).cpu().double()
    tol = (2e-5 + 1e-5 * float(want.abs().max())) if dtype == "float32" else 1e-2 * float(want.abs().max())
    assert float((got - want).abs().max()) <= tol

    bad = family.plan(config)
    bad.schedule = [ScheduleEntry(0, 0, writes=False)]
    with pytest.raises(ValueError, match="before it is written"):
        CausalLM(bad, store, config, family)
    bad.schedule = [ScheduleEntry(0, 0), ScheduleEntry(1, 0)]
    with pytest.raises(ValueError, match="two writers"):
        CausalLM(bad, store, config, family)


# --- a toy architecture defined here: one attention layer, then a layer whose mixer keeps a
# --- running sum per sequence as fixed-size state -------------------------------------------

class RunningSumMixer(Mixer):
    """out[t] = (state + sum of h[0..t]) . W^T, state += sum of the step's h.  Torch ops driven by
    the step's host tables: a toy, and therefore never graph-replayed."""
    graph_safe = False

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.weight = params["width"], tensors["weight"]

    def state_spec(self):
        return StateSpec((self.width,), "float32")

    def forward(self, h, step, memory, stream):
        state = memory.state()
        out = torch.empty(1, h.shape[0], self.width, dtype=torch.float32, device=h.device)
        at = 0
        for slot, count in zip(step.host.slots, step.host.counts):
            sums = state[slot] + torch.cumsum(h[at:at + count].float(), 0)
            out[0, at:at + count] = sums @ self.weight.float().t()
            state[slot] = sums[-1]
            at += count
        return Delta(out, None)


@dataclass(frozen=True)
class ToyConfig:
    width: int = 64
    vocab_size: int = 97
    max_positions: int = 96
    heads: int = 2

    @classmethod
    def from_dict(cls, data):
        return cls(**{k: data[k] for k in ("width", "vocab_size", "max_positions", "heads") if k in data})

    def to_dict(self):
        return {"architectures": ["ToyRunningSumLM"], "width": self.width, "vocab_size": self.vocab_size,
                "max_positions": self.max_positions, "heads": self.heads}


def toy_plan(c):
    norm = lambda p: PartSpec("rms_norm", {"width": c.width, "eps": 1e-5}, {"weight": p + ".scale"})
    ff = lambda p: PartSpec("dense", {"width": c.width, "inner": 2 * c.width, "activation": "gelu_tanh"},
                            {"up_weight": p + ".up", "down_weight": p + ".down"})
    attention = PartSpec("attention", {"width": c.width, "heads": c.heads, "kv_heads": 1, "head_dim": c.width // c.heads,
                                       "scale": (c.width // c.heads) ** -0.5, "window": 0},
                         {"qkv_weight": "l0.qkv", "out_weight": "l0.out"})
    toy = PartSpec("toy_running_sum", {"width": c.width}, {"weight": "l1.mix"})
    layers = [LayerPlan("pre_norm", {"mixer_norm": norm("l0.n1"), "mixer": attention, "ff_norm": norm("l0.n2"), "ff": ff("l0")}),
              LayerPlan("pre_norm", {"mixer_norm": norm("l1.n1"), "mixer": toy, "ff_norm": norm("l1.n2"), "ff": ff("l1")})]
    return ModelPlan(c.width, c.vocab_size, c.max_positions,
                     PartSpec("learned_positions", {"width": c.width, "vocab_size": c.vocab_size,
                                                    "max_positions": c.max_positions},
                              {"tokens": "tok", "positions": "pos"}),
                     layers, [ScheduleEntry(0, 0), ScheduleEntry(1, 1)], norm("final"),
                     PartSpec("linear_readout", {"width": c.width, "vocab_size": c.vocab_size}, {"weight": "tok"}))


def toy_contract(c):
    d, hd = c.width, c.width // c.heads
    specs = [("tok", (c.vocab_size, d), "table"), ("pos", (c.max_positions, d), "table"), ("final.scale", (d,), "vector"),
             ("l0.qkv", (d + 2 * hd, d), "out_in"), ("l0.out", (d, d), "out_in"), ("l1.mix", (d, d), "out_in")]
    for p in ("l0", "l1"):
        specs += [(p + ".n1.scale", (d,), "vector"), (p + ".n2.scale", (d,), "vector"),
                  (p + ".up", (2 * d, d), "out_in"), (p + ".down", (d, 2 * d), "out_in")]
    return bt.Contract([bt.TensorSpec(*s) for s in specs])


def toy_init(c, generator):
    out = {}
    for spec in toy_contract(c).tensors:
        t = torch.randn(spec.shape, generator=generator) * (0.3 if spec.layout == "table" else spec.shape[-1] ** -0.5)
        out[spec.name] = 1 + 0.1 * t if spec.layout == "vector" else t
    out["l1.mix"] *= 0.05
    return out


def toy_reference(ids, w, c):
    """Whole sequence in float64, from the plain parts."""
    rms = lambda x, g: x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * g
    ff = lambda x, p: plain.gelu_tanh(x @ w[p + ".up"].t()) @ w[p + ".down"].t()
    d, hd = c.width, c.width // c.heads
    x = w["tok"][ids] + w["pos"][torch.arange(len(ids))]
    qkv = rms(x, w["l0.n1.scale"]) @ w["l0.qkv"].t()
    q, k, v = plain.split_heads(qkv[:, :d], c.heads), qkv[:, d:d + hd], qkv[:, d + hd:]
    mixed = plain.attention(q, k.expand(c.heads, -1, -1), v.expand(c.heads, -1, -1), hd ** -0.5)
    x = x + plain.merge_heads(mixed) @ w["l0.out"].t()
    x = x + ff(rms(x, w["l0.n2.scale"]), "l0")
    x = x + torch.cumsum(rms(x, w["l1.n1.scale"]), 0) @ w["l1.mix"].t()
    x = x + ff(rms(x, w["l1.n2.scale"]), "l1")
    return rms(x, w["final.scale"]) @ w["tok"].t()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_mixer_with_state_is_registered_built_and_stepped(dtype, tmp_path):
    register("mixer", "toy_running_sum", RunningSumMixer)
    family = bt.Family("toy_running_sum", ("ToyRunningSumLM",), (), ToyConfig, toy_plan, toy_contract, toy_init)
    bt.register_family(family)
    try:
        stored = bt.write_random_model(str(tmp_path), ToyConfig().to_dict(), seed=3)
        model = bt.load_model(str(tmp_path), dtype=dtype)          # chosen by config.json, like GPT-2
        assert model.kv_specs == [KVSpec(1, 32, 0), None] and model.state_specs == [None, StateSpec((64,), "float32")]
        engine = bt.Engine(model, max_tokens=512)
        assert not engine.use_graphs
        w = {k: v.double() for k, v in stored.items()}
        gen = torch.Generator().manual_seed(0)
        requests = [torch.randint(0, 97, (n,), generator=gen).tolist() for n in (40, 9, 70, 23)]
        scale = max(float(toy_reference(torch.tensor(r), w, ToyConfig()).abs().max()) for r in requests)
        tol = 2e-5 * (1 + scale) if dtype == "float32" else 1.5e-2 * scale
        # two batches after one another: the second reuses the slots, whose state must start at zero
        for batch in (requests[:2], requests[2:]):
            slots = [engine.open() for _ in batch]
            got = [[] for _ in batch]
            cut = [len(r) // 2 for r in batch]
            logits = engine.step([(s, r[:c]) for s, r, c in zip(slots, batch, cut)],
                                 want=[list(range(c)) for c in cut]).clone()
            at = 0
            for i, c in enumerate(cut):
                got[i].append(logits[at:at + c])
                at += c
            position, live = list(cut), list(range(len(batch)))
            while live:
                logits = engine.step([(slots[i], [batch[i][position[i]]]) for i in live]).clone()
                for row, i in enumerate(live):
                    got[i].append(logits[row:row + 1])
                    position[i] += 1
                for i in [i for i in live if position[i] == len(batch[i])]:
                    engine.close(slots[i])
                    live.remove(i)
            for i, r in enumerate(batch):
                want = toy_reference(torch.tensor(r), w, ToyConfig())
                assert float((torch.cat(got[i]).cpu().double() - want).abs().max()) <= tol
    finally:
        unregister("mixer", "toy_running_sum")
        bt.unregister_family("toy_running_sum")
