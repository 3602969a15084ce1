"""Bozisun: a decoder whose layers are listed one by one in ``config.json``.  An embedding that adds a row chosen
by the pair (previous token, token); layers whose attention and feed-forward read one normed input and join the
stream together, followed by an input of the token's own (a slice of a table that all layers share); a range of
layers that runs several times in a row with the same weights, every pass with a cache of its own; logits
under a soft cap.  This file reads that configuration and turns it into a ``ModelSpec``; the mechanisms are
parts of their own (``parts/embedding.py: TokenPairEmbedding``, ``parts/block.py: ParallelBlock``,
``parts/token_input.py``, ``parts/attention.py`` with its output gate, ``parts/moe.py`` with a router bias and
the softmax over the chosen logits, ``parts/rotary.py``, ``parts/embedding.py: LinearHead`` with its cap).

``config.json``: ``architecture`` "Bozisun", ``vocab``, ``width``, ``norm.eps``, ``embedding.bigram``
``{buckets, mul_prev, mul_cur}`` (optional), ``token_side.dim`` (optional), ``loop`` ``{start, stop, times}``
(optional), ``logit_softcap`` (optional) and ``layers``: a list of ``{type: "attention", mixer: {heads, kv_heads,
dim, vdim, scale, rot: {base, dims, scaling: {factor, original, fast, slow} | absent} | absent}, mlp: {kind: "dense",
ff} | {kind: "moe", router: {experts, top}, expert: {ff}} | null}``.  Tensor names: ``embed``, ``bigram``,
``side.embed``, ``final.norm``, ``head``, and per layer ``l<i>.norm1``, ``l<i>.mix.{q,k,v,g,o,q.norm,k.norm}``,
``l<i>.mlp.{gate,up,down}`` or ``l<i>.mlp.{router,router.b,e<j>.gate,e<j>.up,e<j>.down}``,
``l<i>.side.{gate,proj,norm}``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional

from ..config.errors import ConfigError
from ..config.model import config_value, read_config_json
from ..config.registry import register_architecture
from ..parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

MIXERS = ("attention",)


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
class BozisunLayer:
    kind: str                       # one of MIXERS
    mixer: Mapping[str, Any]        # the mixer's sizes and constants, checked
    mlp: Optional[Mapping[str, Any]]


@dataclass(frozen=True)
class BozisunConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple
    bigram: Optional[tuple]         # (buckets, mul_prev, mul_cur)
    side_dim: Optional[int]
    loop: Optional[tuple]           # (start, stop, times)
    softcap: Optional[float]
    raw: Mapping[str, Any]

    @classmethod
    def from_dict(cls, c: Mapping[str, Any]) -> "BozisunConfig":
        vocab, width = _positive("config", c, "vocab"), _positive("config", c, "width")
        eps = config_value(_section("config", c, "norm"), "eps", float)
        if not eps >= 0.0:
            raise ConfigError("norm.eps must be non-negative")
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
            _check_attention(where + ".mixer", m)
            mlp = _section(where, entry, "mlp", required=False)
            if mlp is not None:
                _check_mlp(where + ".mlp", mlp)
            layers.append(BozisunLayer(kind, m, mlp))
        bigram = None
        b = (_section("config", c, "embedding", required=False) or {}).get("bigram")
        if b is not None:
            if not isinstance(b, Mapping):
                raise ConfigError("embedding.bigram must be an object")
            bigram = (_positive("embedding.bigram", b, "buckets"), config_value(b, "mul_prev", int),
                      config_value(b, "mul_cur", int))
            if min(bigram[1:]) < 0 or max(bigram[1:]) >= 2 ** 31:
                raise ConfigError("embedding.bigram.mul_prev and mul_cur must lie in [0, 2^31)")
        side = _section("config", c, "token_side", required=False)
        side_dim = _positive("token_side", side, "dim") if side is not None else None
        loop = None
        lp = _section("config", c, "loop", required=False)
        if lp is not None:
            loop = (config_value(lp, "start", int), config_value(lp, "stop", int), _positive("loop", lp, "times"))
            if not 0 <= loop[0] <= loop[1] <= len(layers):
                raise ConfigError(f"loop.start .. loop.stop = {loop[0]} .. {loop[1]} does not lie within the {len(layers)} layers")
        softcap = config_value(c, "logit_softcap", float, required=False)
        if softcap is not None and not softcap > 0:
            raise ConfigError("logit_softcap must be positive")
        return cls(vocab, width, eps, tuple(layers), bigram, side_dim, loop, softcap, dict(c))

    @classmethod
    def from_folder(cls, path) -> "BozisunConfig":
        return cls.from_dict(read_config_json(path))

    def to_dict(self) -> dict:
        return dict(self.raw)

    def layer_order(self) -> list:
        """Indices of the layers in the order they run: the looped range ``times`` times in a row."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        a, b, times = self.loop
        return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def _check_attention(where: str, m: Mapping) -> None:
    heads, kv = _positive(where, m, "heads"), _positive(where, m, "kv_heads")
    if heads % kv:
        raise ConfigError(f"{where}.heads = {heads} is not a multiple of kv_heads = {kv}")
    dim = _positive(where, m, "dim")
    _positive(where, m, "vdim")
    if not config_value(m, "scale", float) > 0:
        raise ConfigError(f"{where}.scale must be positive")
    rot = _section(where, m, "rot", required=False)
    if rot is not None:
        dims = config_value(rot, "dims", int)
        if dims < 0 or dims % 2 or dims > dim:
            raise ConfigError(f"{where}.rot.dims must be even and at most dim = {dim}, got {dims}")
        if not config_value(rot, "base", float) > 1.0:
            raise ConfigError(f"{where}.rot.base must be above 1")
        sc = _section(where + ".rot", rot, "scaling", required=False)
        if sc is not None:
            for key in ("factor", "original", "fast", "slow"):
                if not config_value(sc, key, float) > 0:
                    raise ConfigError(f"{where}.rot.scaling.{key} must be positive")


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
    _positive(where + ".expert", _section(where, f, "expert"), "ff")


def _mixer_spec(cfg: BozisunConfig, m: Mapping):
    """(PartSpec of the mixer, local tensor name -> name below the layer's prefix)."""
    position = None
    rot = m.get("rot")
    if rot and rot["dims"]:
        sc = rot.get("scaling")
        position = PartSpec("rotary", {
            "head_dim": m["dim"], "theta": float(rot["base"]), "rotary_dim": rot["dims"],
            "rescale": {k: float(sc[k]) for k in ("factor", "original", "fast", "slow")} if sc else None})
    spec = PartSpec("gqa_attention", {
        "hidden_size": cfg.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
        "v_head_dim": m["vdim"], "qk_norm_eps": cfg.eps, "qk_norm": "head", "position": position,
        "scale": float(m["scale"]), "output_gate": True})
    names = {"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "q_norm.weight": "q.norm",
             "k_norm.weight": "k.norm", "gate.weight": "g", "o_proj.weight": "o"}
    return spec, names


def _mlp_spec(cfg: BozisunConfig, f: Mapping):
    if f.get("kind", "dense") == "dense":
        spec = PartSpec("gated_mlp", {"hidden_size": cfg.width, "intermediate_size": f["ff"], "activation": "silu"})
        return spec, {"gate_proj.weight": "gate", "up_proj.weight": "up", "down_proj.weight": "down"}
    experts, top, ff = f["router"]["experts"], f["router"]["top"], f["expert"]["ff"]
    spec = PartSpec("routed_experts", {
        "hidden_size": cfg.width, "num_experts": experts, "top": top, "expert_size": ff, "activation": "silu",
        "weight_on_input": False, "router_bias": True, "score": "softmax_chosen"})
    names = {"router.weight": "router", "router.bias": "router.b"}
    for e in range(experts):
        for part in ("gate", "up", "down"):
            names[f"experts.{e}.{part}.weight"] = f"e{e}.{part}"
    return spec, names


def build_spec(cfg: BozisunConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps})
    layers = []
    n = len(cfg.layers)
    for i, layer in enumerate(cfg.layers):
        mixer, mixer_names = _mixer_spec(cfg, layer.mixer)
        rename = {"mix." + k: "mix." + v for k, v in mixer_names.items()}
        ffn = None
        if layer.mlp is not None:
            ffn, ffn_names = _mlp_spec(cfg, layer.mlp)
            rename.update({"mlp." + k: "mlp." + v for k, v in ffn_names.items()})
        rename["norm1.weight"] = "norm1"
        side, shared = None, {}
        if cfg.side_dim is not None:
            # layer i reads its own dim columns of the one table; a layer that runs several times reads the same ones
            side = PartSpec("gated_token_input", {
                "hidden_size": cfg.width, "vocab_size": cfg.vocab, "dim": cfg.side_dim, "table_width": n * cfg.side_dim,
                "offset": i * cfg.side_dim, "eps": cfg.eps, "activation": "gelu_tanh"})
            rename.update({"side.gate.weight": "side.gate", "side.proj.weight": "side.proj", "side.norm.weight": "side.norm"})
            shared = {"side.table": "side.embed"}
        block = PartSpec("parallel", {"norm": norm, "has_feed_forward": ffn is not None, "token_input": side})
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=mixer, feed_forward=ffn, block=block, mixer_prefix="mix.",
                                feed_forward_prefix="mlp.", rename=rename, shared=shared))
    if cfg.bigram is not None:
        embedding = PartSpec("token_pair_embedding", {
            "vocab_size": cfg.vocab, "hidden_size": cfg.width, "buckets": cfg.bigram[0], "mul_prev": cfg.bigram[1],
            "mul_cur": cfg.bigram[2]})
    else:
        embedding = PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width})
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=cfg.width, embedding=embedding, embedding_prefix="embed.",
        final_norm=norm, final_norm_prefix="final.norm.",
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "softcap": cfg.softcap}),
        head_prefix="head.", layers=layers,
        schedule=[LayerRun(i) for i in cfg.layer_order()],      # every pass of the loop keeps a cache of its own
        rename={"embed.weight": "embed", "embed.pair.weight": "bigram", "final.norm.weight": "final.norm",
                "head.weight": "head"},
    )


register_architecture("Bozisun", BozisunConfig.from_dict, build_spec)
