"""Plain, slow GPT-2 used only as the oracle of the tests.

Whole sequences, no cache, one sequence at a time, one function per part, written from
the formulas of the reference (cited as path:line of the reference) and sharing no
code with the product path.  Weights are a dict of torch tensors under the checkpoint's
own names and Conv1D ``[in, out]`` layout (``h.N.attn.c_attn.weight`` ...).  Everything
is evaluated in ``dtype`` (float64 unless asked otherwise).
"""

import math

import torch


def embed(ids, positions, wte, wpe):
    """x0[t] = wte[id[t]] + wpe[pos[t]]  (src/models/gpt2/model.rs:447-448)."""
    return wte[ids] + wpe[positions]


def layer_norm(x, gamma, beta, eps):
    """y = (x - mean) / sqrt(var + eps) * gamma + beta over the last axis, var = E[(x-mean)^2]
    (src/models/gpt2/model.rs:8, src/models/gpt2.rs:128; built at model.rs:143-148)."""
    mean = x.mean(dim=-1, keepdim=True)
    centered = x - mean
    var = (centered * centered).mean(dim=-1, keepdim=True)
    return centered / torch.sqrt(var + eps) * gamma + beta


def linear(x, weight_in_out, bias):
    """y = x W + b with W stored [in, out] (src/operations.rs:529-643; model.rs:136-137)."""
    return x @ weight_in_out + bias


def split_qkv(qkv, width):
    """q, k, v are the thirds of the fused projection, in that order
    (src/models/gpt2/checkpoint.rs:131-152)."""
    return qkv[..., :width], qkv[..., width:2 * width], qkv[..., 2 * width:3 * width]


def split_heads(x, heads):
    """[S, d] -> [H, S, h]; head j owns channels j*h .. (j+1)*h-1 (src/attention.rs:484,531)."""
    tokens, width = x.shape
    return x.reshape(tokens, heads, width // heads).permute(1, 0, 2)


def merge_heads(x):
    """[H, S, h] -> [S, H*h] with head-major channels (src/attention.rs:882-897)."""
    heads, tokens, size = x.shape
    return x.permute(1, 0, 2).reshape(tokens, heads * size)


def attention_scale(head_size, layer_index, scale_attn_weights, scale_by_inverse_layer):
    """(1/sqrt(h) if scale_attn_weights) / (layer+1 if scale_attn_by_inverse_layer_idx),
    layer index zero-based (src/models/gpt2/model.rs:121-133)."""
    scale = 1.0 / math.sqrt(head_size) if scale_attn_weights else 1.0
    if scale_by_inverse_layer:
        scale = scale / float(layer_index + 1)
    return scale


def attention(q, k, v, scale, causal=True, window=None):
    """softmax_k((q k^T) * scale, excluded -> -inf) v per head.

    Scores: the product is scaled (src/attention/dispatch.rs:314-328).  Excluded keys are
    replaced by -inf, never biased (dispatch.rs:365-367); causal exclusion is key > query
    with bottom-right alignment (src/attention/mask.rs:28-40); ``window`` additionally
    excludes keys at distance >= window.  Softmax with max subtraction (dispatch.rs:390-406).
    q: [H, Q, h], k, v: [H, K, h]; query row i sits at key position i + K - Q.
    """
    heads, queries, _ = q.shape
    keys = k.shape[1]
    scores = torch.matmul(q, k.transpose(1, 2)) * scale
    q_pos = torch.arange(queries).unsqueeze(1) + (keys - queries)
    k_pos = torch.arange(keys).unsqueeze(0)
    excluded = torch.zeros(queries, keys, dtype=torch.bool)
    if causal:
        excluded |= k_pos > q_pos
    if window is not None:
        excluded |= k_pos <= q_pos - window
    scores = scores.masked_fill(excluded.unsqueeze(0), float("-inf"))
    top = scores.max(dim=-1, keepdim=True).values
    weights = torch.exp(scores - top)
    weights = weights / weights.sum(dim=-1, keepdim=True)
    return torch.matmul(weights, v)


def gelu_tanh(x):
    """0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))  (src/feed_forward.rs:351-387)."""
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x * x * x)))


def gelu_erf(x):
    """x (1 + erf(x / sqrt 2)) / 2  (src/models/gpt2.rs:50-51)."""
    return x * (1.0 + torch.erf(x / math.sqrt(2.0))) / 2.0


ACTIVATIONS = {"gelu_new": gelu_tanh, "gelu": gelu_erf}


def mlp(x, w_fc, b_fc, w_proj, b_proj, activation):
    """down(act(up(x)))  (src/feed_forward.rs:111-114)."""
    return linear(ACTIVATIONS[activation](linear(x, w_fc, b_fc)), w_proj, b_proj)


def self_attention(x, w, prefix, heads, scale, causal=True, window=None):
    """Fused QKV projection, per-head attention, merge, output projection
    (src/attention.rs:481-513, 882-897)."""
    width = x.shape[-1]
    qkv = linear(x, w[prefix + "c_attn.weight"], w[prefix + "c_attn.bias"])
    q, k, v = split_qkv(qkv, width)
    mixed = attention(split_heads(q, heads), split_heads(k, heads), split_heads(v, heads),
                      scale, causal, window)
    return linear(merge_heads(mixed), w[prefix + "c_proj.weight"], w[prefix + "c_proj.bias"])


def block(x, w, layer, cfg, taps=None):
    """y = x + attn(ln_1 x); z = y + mlp(ln_2 y)  (src/models/gpt2/model.rs:218-270)."""
    p = f"h.{layer}."
    eps = cfg["layer_norm_epsilon"]
    heads = cfg["n_head"]
    scale = attention_scale(x.shape[-1] // heads, layer, cfg.get("scale_attn_weights", True),
                            cfg.get("scale_attn_by_inverse_layer_idx", False))
    normed = layer_norm(x, w[p + "ln_1.weight"], w[p + "ln_1.bias"], eps)
    y = x + self_attention(normed, w, p + "attn.", heads, scale, cfg.get("causal", True))
    normed = layer_norm(y, w[p + "ln_2.weight"], w[p + "ln_2.bias"], eps)
    f = mlp(normed, w[p + "mlp.c_fc.weight"], w[p + "mlp.c_fc.bias"],
            w[p + "mlp.c_proj.weight"], w[p + "mlp.c_proj.bias"],
            cfg.get("activation_function", "gelu_new"))
    if taps is not None:
        taps.setdefault("mlp", []).append(f)
    return y + f


class _Converted:
    """The weights in ``dtype``, each tensor converted when it is used (a model of a billion
    parameters is not held a second time)."""

    def __init__(self, tensors, dtype):
        self.tensors, self.dtype = tensors, dtype

    def __getitem__(self, name):
        return self.tensors[name].to(self.dtype)


def forward(ids, w, cfg, dtype=torch.float64, taps=None, rows=None):
    """Logits [S, V] of one whole sequence: embed, blocks, ln_f, tied readout
    (src/models/gpt2/model.rs:385-420, 500-513).  With ``rows``, only those positions are read out:
    the selection comes after the final norm and before the product (src/models/shared/logits.rs:58-80)."""
    w = _Converted(w, dtype)
    ids = torch.as_tensor(ids, dtype=torch.long)
    x = embed(ids, torch.arange(ids.numel()), w["wte.weight"], w["wpe.weight"])
    if taps is not None:
        taps["hidden"] = [x]
    for layer in range(cfg["n_layer"]):
        x = block(x, w, layer, cfg, taps)
        if taps is not None:
            taps["hidden"].append(x)
    x = layer_norm(x, w["ln_f.weight"], w["ln_f.bias"], cfg["layer_norm_epsilon"])
    if taps is not None:
        taps["final"] = x
    if rows is not None:
        x = x[torch.as_tensor(rows, dtype=torch.long)]
    return x @ w["wte.weight"].t()


def greedy(ids, w, cfg, steps, dtype=torch.float64):
    """Reference greedy continuation: recompute the whole sequence for every new token;
    ties go to the lowest index (src/generation.rs:655-664)."""
    ids = list(ids)
    out = []
    for _ in range(steps):
        token = int(torch.argmax(forward(ids, w, cfg, dtype)[-1]))
        out.append(token)
        ids.append(token)
    return out


def splitmix64(seed, index):
    """Output ``index`` of the SplitMix64 stream (src/generation/random.rs:232-237)."""
    mask = (1 << 64) - 1
    value = (seed + 0x9E3779B97F4A7C15 * ((index + 1) & mask)) & mask
    value = ((value ^ (value >> 30)) * 0xBF58476D1CE4E5B9) & mask
    value = ((value ^ (value >> 27)) * 0x94D049BB133111EB) & mask
    return value ^ (value >> 31)


def interior_unit(bits):
    """Midpoint of one of 2^23 intervals of (0,1) (src/generation/random.rs:244-247)."""
    return ((bits >> 41) + 0.5) / float(1 << 23)


def sample_index(logits, temperature, u):
    """Inverse-CDF choice #{k : c_k < u * c_last} on softmax(z / T)
    (src/generation.rs:632-637, 1148-1165)."""
    z = logits.to(torch.float64) / temperature
    p = torch.softmax(z, dim=-1)
    c = torch.cumsum(p, dim=-1)
    return int((c < u * c[-1]).sum())


def log_probability(logits, index, temperature=None):
    """log_softmax of the processed logits at the chosen id (src/generation.rs:732-743)."""
    z = logits.to(torch.float64)
    if temperature is not None:
        z = z / temperature
    return float(torch.log_softmax(z, dim=-1)[index])


# --- processing of the logits before a token is chosen (src/generation.rs:18-44) -------------------

F32_MAX = 3.4028234663852886e38


def banned_by_ngrams(tokens, size):
    """Tokens that would complete an n-gram the row already holds: whatever followed the last
    size - 1 tokens earlier (src/generation/ngram.rs:1-12, 57-100)."""
    if size <= 0 or len(tokens) < size - 1:
        return []
    prefix = list(tokens[len(tokens) - (size - 1):]) if size > 1 else []
    out = set()
    for end in range(size - 1, len(tokens)):            # tokens[end] is the last token of an n-gram
        if list(tokens[end - (size - 1):end]) == prefix:
            out.add(tokens[end])
    return sorted(out)


def process_logits(z, sampling, temperature=1.0, logit_bias=None, repetition_penalty=1.0, presence_penalty=0.0,
                   frequency_penalty=0.0, seen_counts=None, additive_counts=None, banned=()):
    """Bias, penalties, temperature, overflow clamp, hard constraints, in that order
    (src/generation.rs:608-640; penalties :838-923; bias :767-795; constraints :797-836)."""
    z = z.to(torch.float64).clone()
    adjusts = bool(logit_bias) or repetition_penalty != 1.0 or presence_penalty != 0.0 or frequency_penalty != 0.0
    for token, bias in (logit_bias or {}).items():
        z[token] += bias
    if repetition_penalty != 1.0:
        seen = seen_counts > 0
        penalized = torch.where(z < 0, z * repetition_penalty, z / repetition_penalty)
        z = torch.where(seen, penalized, z)
    if frequency_penalty != 0.0:
        z = z - (additive_counts.to(torch.float64) * frequency_penalty).clamp(-F32_MAX, F32_MAX)
    if presence_penalty != 0.0:
        z = z - (additive_counts > 0).to(torch.float64) * presence_penalty
    if sampling:
        z = z / temperature
    if adjusts or (sampling and temperature < 1.0):
        z = z.clamp(max=F32_MAX)
    for token in banned:
        z[token] = -math.inf
    return z


def filter_top_k(z, k):
    """Every score below the k-th greatest becomes -inf; ties with it survive (generation.rs:1189-1208)."""
    boundary = torch.sort(z, descending=True).values[k - 1]
    return torch.where(z < boundary, torch.full_like(z, -math.inf), z)


def filter_top_p(z, p):
    """Ranked by score, an item survives when the mass before it is below p (generation.rs:1210-1233).
    Items with equal scores are ranked by index here; the reference leaves that to its backend's sort."""
    order = torch.sort(z, descending=True, stable=True).indices
    mass = torch.softmax(z[order], dim=-1)
    before = torch.cumsum(mass, dim=-1) - mass
    keep = torch.zeros_like(z, dtype=torch.bool)
    keep[order[before < p]] = True
    return torch.where(keep, z, torch.full_like(z, -math.inf))


def filter_min_p(z, min_p):
    """p_i >= min_p * max p, as z_i >= max z + ln(min_p) (generation.rs:1235-1253)."""
    threshold = z.max() + math.log(min_p)
    return torch.where(z < threshold, torch.full_like(z, -math.inf), z)


def truncate(z, top_k=None, top_p=None, min_p=None):
    """top-k, then top-p, then min-p, each only when it is not a no-op (generation.rs:926-948)."""
    if top_k is not None and top_k < z.numel():
        z = filter_top_k(z, top_k)
    if top_p is not None and top_p < 1.0:
        z = filter_top_p(z, top_p)
    if min_p is not None and min_p > 0.0:
        z = filter_min_p(z, min_p)
    return z
