"""Plain, slow, whole-sequence Bozisun in torch: the oracle of the test-suite for that design.

No cache, no batching, no kernels, one function per mechanism, nothing imported from the
product package.  A model is ``(config dict, {tensor name: tensor})``; every function works
in the type of the tensors it is given (float32, or float64 for a tighter oracle).

The design in this file's notation (n tokens, width w):

* embedding:  x_t = E[id_t] + B[r_t],  r_t = (id_{t-1} a + id_t b) mod m for t > 0, r_0 = m (the spare last row);
* order:      the layers [start, stop) of ``loop`` run ``times`` times in a row (same weights), then the rest;
* layer:      u = N(x);  x += mixer(u) + ff(u);  then the token's own share:
              y = P (gelu(G x) * s_t),  s_t = columns [i d, (i + 1) d) of S[id_t] for layer i;  x += N'(y)
* N(x):       x / sqrt(mean(x^2) + eps) * weight
* attention:  grouped-query, q and k normed per head with one shared weight, the first ``dims`` elements of
              each head turned by position (half-split pairs, frequencies blended for longer contexts), causal
              softmax, the concatenated heads times sigmoid(W_g u), output projection;
* feed-forward: gated (silu), or routed experts: logits = R u + b, the ``top`` largest chosen, weights = softmax
              over the chosen logits, sum of the weighted experts' outputs;
* output:     logits = c tanh(H N(x) / c).
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# --------------------------------------------------------------------------- files
def read_config(folder) -> dict:
    return json.loads((Path(folder) / "config.json").read_text())


def read_weights(folder, dtype=torch.float32) -> dict:
    from safetensors.torch import load_file

    out = {}
    for shard in sorted(Path(folder).glob("*.safetensors")):
        for k, v in load_file(str(shard)).items():
            out[k] = v.to(dtype) if v.is_floating_point() else v
    return out


# --------------------------------------------------------------------------- small pieces
def rms_norm(x, weight, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


_ROUND_PRODUCTS_TO = None     # see ``rounded_products``


def linear(x, w):
    """w is stored [out, in]."""
    y = x @ w.T
    return y if _ROUND_PRODUCTS_TO is None else y.to(_ROUND_PRODUCTS_TO).to(y.dtype)


class rounded_products:
    """Within this context every matrix product's result is rounded to ``dtype`` (and widened again): what
    an implementation that keeps its activations in bfloat16 does to the numbers at the least."""

    def __init__(self, dtype=torch.bfloat16):
        self.dtype = dtype

    def __enter__(self):
        global _ROUND_PRODUCTS_TO
        self.before, _ROUND_PRODUCTS_TO = _ROUND_PRODUCTS_TO, self.dtype

    def __exit__(self, *exc):
        global _ROUND_PRODUCTS_TO
        _ROUND_PRODUCTS_TO = self.before


# --------------------------------------------------------------------------- embedding
def bigram_rows(tokens, bigram: dict) -> list:
    m, a, b = int(bigram["buckets"]), int(bigram["mul_prev"]), int(bigram["mul_cur"])
    return [m if t == 0 else (int(tokens[t - 1]) * a + int(tokens[t]) * b) % m for t in range(len(tokens))]


def embed(w: dict, cfg: dict, tokens):
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    x = w["embed"][ids]
    bigram = (cfg.get("embedding") or {}).get("bigram")
    if bigram:
        x = x + w["bigram"][torch.as_tensor(bigram_rows(tokens, bigram), dtype=torch.long)]
    return x


# --------------------------------------------------------------------------- rotation
def rotary_frequencies(rot: dict):
    """One frequency per pair, as float64."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    amp = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, original = float(sc["factor"]), float(sc["original"])

        def pair_of(turns):
            return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))

        lo = max(math.floor(pair_of(float(sc["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(sc["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / factor * ramp + f * (1 - ramp)
        amp = 0.1 * math.log(factor) + 1.0
    return f, amp


def rotate(x, positions, rot: dict):
    """x [n, heads, d]: the first rot.dims elements of every head turn, element i with element i + dims / 2."""
    dims = int(rot["dims"])
    if dims == 0:
        return x
    f, amp = rotary_frequencies(rot)
    ang = torch.as_tensor(list(positions), dtype=torch.float64)[:, None] * f[None, :]
    cos, sin = (torch.cos(ang) * amp).to(x.dtype)[:, None, :], (torch.sin(ang) * amp).to(x.dtype)[:, None, :]
    half = dims // 2
    u, v, rest = x[..., :half], x[..., half:dims], x[..., dims:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, rest], dim=-1)


# --------------------------------------------------------------------------- mixer
_ONLY_LAST_KEYS = None     # see ``only_last_keys``


class only_last_keys:
    """Within this context every query sees its last ``n`` keys only.  The design has no such limit: a test uses
    this to show that its rows do hang on keys further back, so that an engine that loses them would be caught."""

    def __init__(self, n: int):
        self.n = int(n)

    def __enter__(self):
        global _ONLY_LAST_KEYS
        self.before, _ONLY_LAST_KEYS = _ONLY_LAST_KEYS, self.n

    def __exit__(self, *exc):
        global _ONLY_LAST_KEYS
        _ONLY_LAST_KEYS = self.before


def attention(w: dict, p: str, m: dict, u, eps: float):
    """u [n, width], the layer's normed input; positions 0 .. n - 1."""
    n = u.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = linear(u, w[p + "q"]).view(n, H, d)
    k = linear(u, w[p + "k"]).view(n, G, d)
    v = linear(u, w[p + "v"]).view(n, G, dv)
    q, k = rms_norm(q, w[p + "q.norm"], eps), rms_norm(k, w[p + "k.norm"], eps)
    rot = m.get("rot")
    if rot:
        q, k = rotate(q, range(n), rot), rotate(k, range(n), rot)
    out = torch.zeros(n, H, dv, dtype=u.dtype)
    causal = torch.ones(n, n, dtype=torch.bool).tril()
    if _ONLY_LAST_KEYS is not None:
        causal &= torch.ones(n, n, dtype=torch.bool).triu(1 - _ONLY_LAST_KEYS)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * float(m["scale"])
        s = s.masked_fill(~causal, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    out = out.reshape(n, H * dv) * torch.sigmoid(linear(u, w[p + "g"]))
    return linear(out, w[p + "o"])


# --------------------------------------------------------------------------- feed-forward
def gated_ff(w: dict, p: str, u):
    return linear(silu(linear(u, w[p + "gate"])) * linear(u, w[p + "up"]), w[p + "down"])


def router_choice(z, top: int):
    """(indices [n, top], weights [n, top]): the largest logits, softmax over the chosen ones alone."""
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def routed_ff(w: dict, p: str, f: dict, u):
    top = int(f["router"]["top"])
    z = u @ w[p + "router"].T + w[p + "router.b"]
    idx, wgt = router_choice(z, top)
    out = torch.zeros_like(u)
    for t in range(u.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            out[t] += wgt[t, j] * gated_ff(w, f"{p}e{e}.", u[t:t + 1])[0]
    return out


def feed_forward(w: dict, p: str, f: dict, u):
    return gated_ff(w, p, u) if f.get("kind", "dense") == "dense" else routed_ff(w, p, f, u)


# --------------------------------------------------------------------------- the token's own share of a layer
def token_side(w: dict, cfg: dict, i: int, x, tokens):
    d, eps = int(cfg["token_side"]["dim"]), float(cfg["norm"]["eps"])
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    s = w["side.embed"][ids][:, i * d:(i + 1) * d]
    y = linear(gelu_tanh(linear(x, w[f"l{i}.side.gate"])) * s, w[f"l{i}.side.proj"])
    return rms_norm(y, w[f"l{i}.side.norm"], eps)


# --------------------------------------------------------------------------- the model
def layer_order(cfg: dict) -> list:
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def layer(w: dict, cfg: dict, i: int, x, tokens):
    spec, eps = cfg["layers"][i], float(cfg["norm"]["eps"])
    u = rms_norm(x, w[f"l{i}.norm1"], eps)
    share = attention(w, f"l{i}.mix.", spec["mixer"], u, eps)
    if spec.get("mlp"):
        share = share + feed_forward(w, f"l{i}.mlp.", spec["mlp"], u)
    x = x + share
    if cfg.get("token_side"):
        x = x + token_side(w, cfg, i, x, tokens)
    return x


def forward(w: dict, cfg: dict, tokens, streams=None):
    """Logits [n, vocab] of one sequence from its first token on.  ``streams``: a list that receives x after
    every layer run."""
    x = embed(w, cfg, tokens)
    for i in layer_order(cfg):
        x = layer(w, cfg, i, x, tokens)
        if streams is not None:
            streams.append(x)
    z = linear(rms_norm(x, w["final.norm"], float(cfg["norm"]["eps"])), w["head"])
    cap = cfg.get("logit_softcap")
    return float(cap) * torch.tanh(z / float(cap)) if cap else z
