"""Plain, slow, whole-sequence Zeripel in torch: the oracle of the test-suite for that design.

No cache, no batching, no kernels, one function per mechanism, nothing imported from the
product package.  A model is ``(config dict, {tensor name: tensor})``; every function works
in the type of the tensors it is given (float32, or float64 for a tighter oracle).

The design in this file's notation (n tokens, width d, m = ``residual_mult``):

* embedding:  x_t = a E[id_t] + B[r_t],  r_t = (id_{t-1} p + id_t c) mod b for t > 0, r_0 = b (the spare last row);
* layer:      x += m mixer(N1(x));  x += m ff(N2(x))   (the second line only with a feed-forward)
* N(x):       x / sqrt(mean(x^2) + eps) * weight
* wkv:        with u_t the mixer's input and u_{t-1} the one before (zeros before the first), every one of r, k, v,
              g, w reads its own blend u_t + (u_{t-1} - u_t) mu;  decay_t = exp(-exp(W2 tanh(W1 blend_w) + w0));
              per head, with S the [key, value] state:  o_t = (S + diag(bonus) k_t v_t^T)^T r_t,
              S <- diag(decay_t) S + k_t v_t^T;  o / rms(o) per head, times a weight, times silu(W_g blend_g), then W_o;
* attention:  grouped-query; the values are the projected keys (before their norm); q and k normed per head with one
              shared weight; q at position p times 1 + coef ln(floor((p + 1) / every) + 1); no rotation; causal softmax;
* latent attention: q = W_q u laid out per head [plain | turned];  W_dkv u = [latent | shared turned key part];  the
              latent is normed;  per head k = [W_uk c | turned part], v = W_uv c;  pairs (2i, 2i + 1) of the turned
              parts rotate by p base^(-2i / dims);  causal softmax whose denominator also holds exp(sink_h);  head h's
              output times sigmoid(W_g u)_h;  a layer with ``kv_from`` j takes c and the turned key part of layer j;
* feed-forward: dense: W_down(gelu_tanh(W_gate u) * W_up u);  routed: s = sigmoid(W_router u), the ``top`` largest
              s + correction chosen, weights s / (sum of the chosen s + 1e-20) * scale, experts with silu;  a shared
              expert for every token times sigmoid(W_sg u);
* output:     logits = H N(x).
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
def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return rms(x, eps) * weight


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
def pair_rows(tokens, bigram: dict) -> list:
    b, p, c = bigram["buckets"], bigram["mul_prev"], bigram["mul_cur"]
    return [b if t == 0 else (tokens[t - 1] * p + tokens[t] * c) % b for t in range(len(tokens))]


def embed(w: dict, cfg: dict, tokens):
    e = cfg.get("embedding") or {}
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)] * e.get("scale", 1.0)
    if e.get("bigram"):
        x = x + w["bigram"][torch.tensor(pair_rows(list(tokens), e["bigram"]), dtype=torch.long)]
    return x


# --------------------------------------------------------------------------- mixers
def wkv(w: dict, p: str, m: dict, u, eps: float, keep=None):
    """``keep``: a list that receives the state after every token (tests of the recurrence alone)."""
    n, H, D = u.shape[0], m["heads"], m["dim"]
    before = torch.cat([torch.zeros_like(u[:1]), u[:-1]])
    blend = {s: u + (before - u) * w[f"{p}mu.{s}"] for s in "rkvgw"}
    r = linear(blend["r"], w[p + "r"]).view(n, H, D)
    k = linear(blend["k"], w[p + "k"]).view(n, H, D)
    v = linear(blend["v"], w[p + "v"]).view(n, H, D)
    gate = silu(linear(blend["g"], w[p + "g"]))
    rate = linear(torch.tanh(linear(blend["w"], w[p + "w1"])), w[p + "w2"]) + w[p + "w0"]
    decay = torch.exp(-torch.exp(rate)).view(n, H, D)
    bonus = w[p + "u"].view(H, D)
    S = torch.zeros((H, D, D), dtype=u.dtype)
    out = torch.empty((n, H, D), dtype=u.dtype)
    for t in range(n):
        kv = k[t].unsqueeze(2) * v[t].unsqueeze(1)                       # [H, key, value]
        out[t] = ((S + bonus.unsqueeze(2) * kv) * r[t].unsqueeze(2)).sum(1)
        S = decay[t].unsqueeze(2) * S + kv
        if keep is not None:
            keep.append(S.clone())
    o = rms(out, eps).reshape(n, H * D) * w[p + "norm"] * gate
    return linear(o, w[p + "o"])


def query_temperature(positions, q_temp):
    if not q_temp:
        return torch.ones(len(positions), dtype=torch.float64)
    steps = torch.tensor([(int(p) + 1) // q_temp["every"] for p in positions], dtype=torch.float64)
    return 1.0 + q_temp["coef"] * torch.log(steps + 1.0)


def causal_softmax(scores, sink=None):
    """scores [heads, n, n]; ``sink`` [heads]: one more term exp(sink) in every row's denominator."""
    n = scores.shape[-1]
    mask = torch.ones((n, n), dtype=torch.bool).tril()
    scores = scores.masked_fill(~mask, float("-inf"))
    if sink is None:
        return torch.softmax(scores, dim=-1)
    full = torch.cat([scores, sink.view(-1, 1, 1).expand(-1, n, 1).to(scores.dtype)], dim=-1)
    return torch.softmax(full, dim=-1)[..., :n]


def attention(w: dict, p: str, m: dict, u, eps: float, only_last_keys=None):
    n, H, G, D = u.shape[0], m["heads"], m["kv_heads"], m["dim"]
    q = linear(u, w[p + "q"]).view(n, H, D)
    k = linear(u, w[p + "k"]).view(n, G, D)
    v = k                                                                  # the values are the keys as projected
    q = rms_norm(q, w[p + "q.norm"], eps) * query_temperature(range(n), m.get("q_temp")).to(u.dtype).view(n, 1, 1)
    k = rms_norm(k, w[p + "k.norm"], eps)
    kh = k.repeat_interleave(H // G, dim=1)
    vh = v.repeat_interleave(H // G, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, kh) * m["scale"]
    if only_last_keys is not None:       # a test's question: what if keys further back were lost?
        i, j = torch.arange(n).view(n, 1), torch.arange(n).view(1, n)
        scores = scores.masked_fill((i - j >= only_last_keys).unsqueeze(0), float("-inf"))
    probs = causal_softmax(scores)
    o = torch.einsum("hij,jhd->ihd", probs, vh).reshape(n, H * D)
    return linear(o, w[p + "o"])


def rotate_pairs(x, positions, rot: dict):
    """x [n, ..., size]: the pairs (2i, 2i + 1) below ``dims`` turn by position * base^(-2i / dims)."""
    dims = rot["dims"]
    i = torch.arange(dims // 2, dtype=torch.float64)
    freq = torch.tensor(float(rot["base"]), dtype=torch.float64) ** (-2.0 * i / dims)
    ang = torch.tensor(list(positions), dtype=torch.float64).view(-1, 1) * freq
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    cos, sin = torch.cos(ang).to(x.dtype).view(shape), torch.sin(ang).to(x.dtype).view(shape)
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def latent_cache(w: dict, p: str, m: dict, u, eps: float):
    """(normed latent [n, rank], turned key part [n, rot_dim]) that a latent layer with a W_dkv keeps per token."""
    rank = m["kv_rank"]
    down = linear(u, w[p + "dkv"])
    c = rms_norm(down[:, :rank], w[p + "dkv.norm"], eps)
    kr = down[:, rank:]
    if m["rot_dim"]:
        kr = rotate_pairs(kr, range(u.shape[0]), m["rot"])
    return c, kr


def latent_attention(w: dict, p: str, m: dict, u, eps: float, cache, only_last_keys=None):
    n, H, D, R, V = u.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, kr = cache
    q = linear(u, w[p + "q"]).view(n, H, D + R)
    q_plain, q_rot = q[..., :D], q[..., D:]
    if R:
        q_rot = rotate_pairs(q_rot, range(n), m["rot"])
    k_plain = linear(c, w[p + "uk"]).view(n, H, D)
    v = linear(c, w[p + "uv"]).view(n, H, V)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihr,jr->hij", q_rot, kr)) * m["scale"]
    if only_last_keys is not None:
        i, j = torch.arange(n).view(n, 1), torch.arange(n).view(1, n)
        scores = scores.masked_fill((i - j >= only_last_keys).unsqueeze(0), float("-inf"))
    probs = causal_softmax(scores, w[p + "sink"])
    o = torch.einsum("hij,jhv->ihv", probs, v)
    o = o * torch.sigmoid(linear(u, w[p + "g"])).view(n, H, 1)
    return linear(o.reshape(n, H * V), w[p + "o"])


# --------------------------------------------------------------------------- feed-forwards
def gated_ff(w: dict, p: str, u, act):
    return linear(act(linear(u, w[p + "gate"])) * linear(u, w[p + "up"]), w[p + "down"])


def router(w: dict, p: str, f: dict, u):
    """(chosen experts [n, top], their weights [n, top])."""
    r = f["router"]
    s = torch.sigmoid(u @ w[p + "router"].T)                               # never rounded
    choice = torch.topk(s + w[p + "correction"], r["top"], dim=-1).indices
    chosen = torch.gather(s, 1, choice)
    return choice, chosen / (chosen.sum(-1, keepdim=True) + 1e-20) * r.get("scale", 1.0)


def routed_ff(w: dict, p: str, f: dict, u):
    choice, weight = router(w, p, f, u)
    out = torch.zeros_like(u)
    for t in range(u.shape[0]):
        for e, g in zip(choice[t].tolist(), weight[t]):
            out[t] += g * gated_ff(w, f"{p}e{e}.", u[t:t + 1], silu)[0]
    if f.get("shared"):
        out = out + gated_ff(w, p + "shared.", u, silu) * torch.sigmoid(linear(u, w[p + "shared.sg"]))
    return out


def feed_forward(w: dict, p: str, f: dict, u):
    if f.get("kind", "dense") == "dense":
        return gated_ff(w, p, u, gelu_tanh)
    return routed_ff(w, p, f, u)


# --------------------------------------------------------------------------- the model
def forward(w: dict, cfg: dict, tokens, streams=None, only_last_keys=None):
    """Logits [n, vocab] of one sequence from its first token; ``streams``: a list that receives the residual
    stream after every layer."""
    eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x = embed(w, cfg, tokens)
    caches = {}
    for i, layer in enumerate(cfg["layers"]):
        p, mix = f"l{i}.mix.", layer["mixer"]
        u = rms_norm(x, w[f"l{i}.norm1"], eps)
        if layer["type"] == "wkv":
            y = wkv(w, p, mix, u, eps)
        elif layer["type"] == "attention":
            y = attention(w, p, mix, u, eps, only_last_keys)
        elif layer["type"] == "latent_attention":
            src = mix.get("kv_from")
            if src is None:
                caches[i] = latent_cache(w, p, mix, u, eps)
            y = latent_attention(w, p, mix, u, eps, caches[i if src is None else src], only_last_keys)
        else:
            raise ValueError(layer["type"])
        x = x + m * y
        if layer.get("mlp"):
            x = x + m * feed_forward(w, f"l{i}.mlp.", layer["mlp"], rms_norm(x, w[f"l{i}.norm2"], eps))
        if streams is not None:
            streams.append(x.clone())
    return linear(rms_norm(x, w["final.norm"], eps), w["head"])
