"""Zeripel: a decoder whose layers are listed one by one in ``config.json``, every layer with one of three token
mixers and a dense or routed feed-forward (or none).  A scaled token embedding plus a row chosen by the pair
(previous token, token); pre-norm layers whose sublayers join the float stream under one constant
(``residual_mult``); a final norm and a linear head.  This file reads that configuration and turns it into a
``ModelSpec``; the mechanisms are parts of their own:

* ``wkv``: ``parts/recurrent.py: TimeMix`` (token shift, a decay per key channel, a bonus for the current token);
* ``attention``: ``parts/attention.py`` with the values taken from the keys as projected, a per-head q/k norm, a query
  temperature that grows with position and no rotation;
* ``latent_attention``: ``parts/latent_attention.py`` with queries projected directly, interleaved rotation of the
  rotated parts, a sink per head in the softmax denominator and one output gate per head; a layer with ``kv_from`` j
  has no down-projection and reads layer j's cache (``LayerRun.cache_of``);
* feed-forward: ``parts/mlp.py: GatedMLP`` (tanh-form gelu) or ``parts/moe.py`` (sigmoid scores, a correction that
  takes part in the choice only, weights normed over the chosen and scaled, a shared expert under a gate per token).

``config.json``: ``architecture`` "Zeripel", ``vocab``, ``width``, ``norm.eps``, ``residual_mult`` (default 1),
``embedding`` ``{scale (default 1), bigram: {buckets, mul_prev, mul_cur} (optional)}`` and ``layers``: a list of
``{type, mixer, mlp}`` with

* type "wkv": mixer ``{heads, dim}`` (``decay_rank`` optional: the checkpoint's shape of ``w1`` gives it);
* type "attention": mixer ``{heads, kv_heads, dim, vdim (= dim), scale, q_temp: {coef, every} (optional)}``;
* type "latent_attention": mixer ``{heads, dim, rot_dim, vdim, kv_rank, scale, rot: {base, dims}, kv_from (optional)}``;
* mlp ``{kind: "dense", ff}``, ``{kind: "moe", router: {experts, top, scale (default 1)}, expert: {ff},
  shared: {ff} (optional)}`` or null.

Tensor names: ``embed``, ``bigram``, ``final.norm``, ``head``, and per layer ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.{mu.r,mu.k,mu.v,mu.g,mu.w,r,k,v,g,w1,w2,w0,u,norm,o}`` (wkv), ``l<i>.mix.{q,k,q.norm,k.norm,o}`` (attention),
``l<i>.mix.{q,dkv,dkv.norm,uk,uv,sink,g,o}`` (latent attention), ``l<i>.mlp.{gate,up,down}`` or
``l<i>.mlp.{router,correction,e<j>.gate,e<j>.up,e<j>.down,shared.gate,shared.up,shared.down,shared.sg}``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional

from ..config.errors import ConfigError
from ..config.model import config_value, read_config_json
from ..config.registry import register_architecture
from ..parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

MIXERS = ("wkv", "attention", "latent_attention")


def _positive(where: str, c: Mapping, key: str) -> int:
    v = config_value(c, key, int)
    if v <= 0:
        raise ConfigError(f"{where}.{key} must be positive, got {v}")
    return v


def _section(where: str, c: Mapping, key: str, required: bool = True) -> Optional[Mapping]:
    v = c.get(key)
    if v is None:
        if required:
            raise ConfigError(f"config.json lacks {where}.{key}")
        return None
    if not isinstance(v, Mapping):
        raise ConfigError(f"{where}.{key} must be an object")
    return v


@dataclass(frozen=True)
class ZeripelLayer:
    kind: str                       # one of MIXERS
    mixer: Mapping[str, Any]        # the mixer's sizes and constants, checked
    mlp: Optional[Mapping[str, Any]]


@dataclass(frozen=True)
class ZeripelConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    embedding_scale: float
    bigram: Optional[tuple]         # (buckets, mul_prev, mul_cur)
    layers: tuple
    raw: Mapping[str, Any]

    @classmethod
    def from_dict(cls, c: Mapping[str, Any]) -> "ZeripelConfig":
        vocab, width = _positive("config", c, "vocab"), _positive("config", c, "width")
        eps = config_value(_section("config", c, "norm"), "eps", float)
        if not eps >= 0.0:
            raise ConfigError("norm.eps must be non-negative")
        mult = config_value(c, "residual_mult", float, default=1.0, required=False)
        emb = _section("config", c, "embedding", required=False) or {}
        scale = config_value(emb, "scale", float, default=1.0, required=False)
        bigram = None
        b = emb.get("bigram")
        if b is not None:
            if not isinstance(b, Mapping):
                raise ConfigError("embedding.bigram must be an object")
            bigram = (_positive("embedding.bigram", b, "buckets"), config_value(b, "mul_prev", int),
                      config_value(b, "mul_cur", int))
            if min(bigram[1:]) < 0 or max(bigram[1:]) >= 2 ** 31:
                raise ConfigError("embedding.bigram.mul_prev and mul_cur must lie in [0, 2^31)")
        listed = c.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json needs a non-empty list 'layers'")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{where} must be an object")
            kind = config_value(entry, "type", str)
            if kind not in MIXERS:
                raise ConfigError(f"{where}.type {kind!r} is not one of {MIXERS}")
            m = _section(where, entry, "mixer")
            {"wkv": _check_wkv, "attention": _check_attention, "latent_attention": _check_latent}[kind](where + ".mixer", m)
            mlp = _section(where, entry, "mlp", required=False)
            if mlp is not None:
                _check_mlp(where + ".mlp", mlp)
            layers.append(ZeripelLayer(kind, m, mlp))
        for i, layer in enumerate(layers):
            if layer.kind == "latent_attention" and layer.mixer.get("kv_from") is not None:
                _check_kv_from(i, layers)
        return cls(vocab, width, eps, mult, scale, bigram, tuple(layers), dict(c))

    @classmethod
    def from_folder(cls, path) -> "ZeripelConfig":
        return cls.from_dict(read_config_json(path))

    def to_dict(self) -> dict:
        return dict(self.raw)


def _check_wkv(where: str, m: Mapping) -> None:
    _positive(where, m, "heads")
    _positive(where, m, "dim")
    if m.get("decay_rank") is not None:
        _positive(where, m, "decay_rank")


def _check_attention(where: str, m: Mapping) -> None:
    heads, kv = _positive(where, m, "heads"), _positive(where, m, "kv_heads")
    if heads % kv:
        raise ConfigError(f"{where}.heads = {heads} is not a multiple of kv_heads = {kv}")
    dim = _positive(where, m, "dim")
    vdim = config_value(m, "vdim", int, default=dim, required=False)
    if vdim != dim:
        raise ConfigError(f"{where}.vdim = {vdim}: the values are the keys, so vdim equals dim = {dim}")
    if not config_value(m, "scale", float) > 0:
        raise ConfigError(f"{where}.scale must be positive")
    qt = _section(where, m, "q_temp", required=False)
    if qt is not None:
        config_value(qt, "coef", float)
        _positive(where + ".q_temp", qt, "every")


def _check_latent(where: str, m: Mapping) -> None:
    for key in ("heads", "dim", "vdim", "kv_rank"):
        _positive(where, m, key)
    rot_dim = config_value(m, "rot_dim", int)
    if rot_dim < 0:
        raise ConfigError(f"{where}.rot_dim must not be negative")
    if not config_value(m, "scale", float) > 0:
        raise ConfigError(f"{where}.scale must be positive")
    rot = _section(where, m, "rot", required=rot_dim > 0)
    if rot is not None:
        dims = config_value(rot, "dims", int)
        if dims < 0 or dims % 2 or dims > rot_dim:
            raise ConfigError(f"{where}.rot.dims must be even and at most rot_dim = {rot_dim}, got {dims}")
        if not config_value(rot, "base", float) > 1.0:
            raise ConfigError(f"{where}.rot.base must be above 1")
    if m.get("kv_from") is not None:
        config_value(m, "kv_from", int)


def _check_kv_from(i: int, layers: list) -> None:
    m = layers[i].mixer
    j = m["kv_from"]
    where = f"layers[{i}].mixer.kv_from"
    if not 0 <= j < i:
        raise ConfigError(f"{where} = {j} must name an earlier layer")
    other = layers[j]
    if other.kind != "latent_attention" or other.mixer.get("kv_from") is not None:
        raise ConfigError(f"{where} = {j}: that layer keeps no latent cache of its own")
    for key in ("kv_rank", "rot_dim", "rot"):
        if other.mixer.get(key) != m.get(key):
            raise ConfigError(f"{where} = {j}: {key} differs between the two layers")


def _check_mlp(where: str, f: Mapping) -> None:
    kind = f.get("kind", "dense")
    if kind == "dense":
        _positive(where, f, "ff")
        return
    if kind != "moe":
        raise ConfigError(f"{where}.kind {kind!r}: this architecture's feed-forward is 'dense' or 'moe'")
    router = _section(where, f, "router")
    experts, top = _positive(where + ".router", router, "experts"), _positive(where + ".router", router, "top")
    if top > experts:
        raise ConfigError(f"{where}.router.top = {top} exceeds its {experts} experts")
    config_value(router, "scale", float, default=1.0, required=False)
    _positive(where + ".expert", _section(where, f, "expert"), "ff")
    shared = _section(where, f, "shared", required=False)
    if shared is not None:
        _positive(where + ".shared", shared, "ff")


def _mixer_spec(cfg: ZeripelConfig, layer: ZeripelLayer):
    """(PartSpec of the mixer, local tensor name -> name below the layer's prefix)."""
    m = layer.mixer
    if layer.kind == "wkv":
        spec = PartSpec("time_mix", {"hidden_size": cfg.width, "num_heads": m["heads"], "head_dim": m["dim"],
                                     "decay_rank": m.get("decay_rank"), "norm_eps": cfg.eps})
        names = {f"mu.{s}": f"mu.{s}" for s in "rkvgw"}
        names.update({"r_proj.weight": "r", "k_proj.weight": "k", "v_proj.weight": "v", "gate.weight": "g",
                      "decay_down.weight": "w1", "decay_up.weight": "w2", "decay_base": "w0", "bonus": "u",
                      "norm.weight": "norm", "o_proj.weight": "o"})
        return spec, names
    if layer.kind == "attention":
        qt = m.get("q_temp")
        spec = PartSpec("gqa_attention", {
            "hidden_size": cfg.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
            "qk_norm_eps": cfg.eps, "qk_norm": "head", "position": None, "scale": float(m["scale"]),
            "values_are_keys": True, "q_temperature": (float(qt["coef"]), int(qt["every"])) if qt else None})
        return spec, {"q_proj.weight": "q", "k_proj.weight": "k", "q_norm.weight": "q.norm", "k_norm.weight": "k.norm",
                      "o_proj.weight": "o"}
    rot = m.get("rot")
    position = None
    if m["rot_dim"] and rot and rot["dims"]:
        position = PartSpec("rotary", {"head_dim": m["rot_dim"], "theta": float(rot["base"]), "rotary_dim": rot["dims"],
                                       "interleaved": True})
    own = m.get("kv_from") is None
    spec = PartSpec("latent_attention", {
        "hidden_size": cfg.width, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"],
        "v_dim": m["vdim"], "q_rank": 0, "kv_rank": m["kv_rank"], "scale": float(m["scale"]), "norm_eps": cfg.eps,
        "position": position, "output_gate": "head", "sinks": True, "own_cache": own})
    names = {"q_proj.weight": "q", "k_up.weight": "uk", "v_up.weight": "uv", "sinks": "sink", "gate.weight": "g",
             "o_proj.weight": "o"}
    if own:
        names.update({"kv_down.weight": "dkv", "kv_norm.weight": "dkv.norm"})
    return spec, names


def _mlp_spec(cfg: ZeripelConfig, f: Mapping):
    dense = {"gate_proj.weight": "gate", "up_proj.weight": "up", "down_proj.weight": "down"}
    if f.get("kind", "dense") == "dense":
        spec = PartSpec("gated_mlp", {"hidden_size": cfg.width, "intermediate_size": f["ff"], "activation": "gelu_tanh"})
        return spec, dense
    router = f["router"]
    experts = router["experts"]
    shared = f.get("shared")
    spec = PartSpec("routed_experts", {
        "hidden_size": cfg.width, "num_experts": experts, "top": router["top"], "expert_size": f["expert"]["ff"],
        "activation": "silu", "weight_on_input": False, "score": "sigmoid_normed", "choice_correction": True,
        "weight_scale": float(router.get("scale", 1.0)),
        "shared": PartSpec("gated_mlp", {"hidden_size": cfg.width, "intermediate_size": shared["ff"],
                                         "activation": "silu"}) if shared else None,
        "shared_gate": bool(shared)})
    names = {"router.weight": "router", "router.correction": "correction"}
    for e in range(experts):
        for part in ("gate", "up", "down"):
            names[f"experts.{e}.{part}.weight"] = f"e{e}.{part}"
    if shared:
        names.update({"shared." + k: "shared." + v for k, v in dense.items()})
        names["shared_gate.weight"] = "shared.sg"
    return spec, names


def build_spec(cfg: ZeripelConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps})
    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        mixer, mixer_names = _mixer_spec(cfg, layer)
        rename = {"mix." + k: "mix." + v for k, v in mixer_names.items()}
        ffn = None
        if layer.mlp is not None:
            ffn, ffn_names = _mlp_spec(cfg, layer.mlp)
            rename.update({"mlp." + k: "mlp." + v for k, v in ffn_names.items()})
        rename["norm1.weight"] = "norm1"
        rename["norm2.weight"] = "norm2"
        block = PartSpec("prenorm", {"norm": norm, "mixer_norm_name": "norm1", "feed_forward_norm_name": "norm2",
                                     "residual_scale": cfg.residual_mult, "has_feed_forward": ffn is not None})
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=mixer, feed_forward=ffn, block=block, mixer_prefix="mix.",
                                feed_forward_prefix="mlp.", rename=rename))
        schedule.append(LayerRun(i, cache_of=layer.mixer.get("kv_from") if layer.kind == "latent_attention" else None))
    if cfg.bigram is not None:
        embedding = PartSpec("token_pair_embedding", {
            "vocab_size": cfg.vocab, "hidden_size": cfg.width, "buckets": cfg.bigram[0], "mul_prev": cfg.bigram[1],
            "mul_cur": cfg.bigram[2], "scale": cfg.embedding_scale})
    else:
        embedding = PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width,
                                                 "scale": cfg.embedding_scale})
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=cfg.width, embedding=embedding, embedding_prefix="embed.",
        final_norm=norm, final_norm_prefix="final.norm.",
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width}),
        head_prefix="head.", layers=layers, schedule=schedule,
        rename={"embed.weight": "embed", "embed.pair.weight": "bigram", "final.norm.weight": "final.norm",
                "head.weight": "head"},
    )


register_architecture("Zeripel", ZeripelConfig.from_dict, build_spec)
