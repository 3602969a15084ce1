"""Small Zeripel configurations of the test-suite and what the tests of that design share.

The configurations differ from one another in every size and constant: widths (also no multiple of 4), head counts and
ratios, head sizes (below, at and above a wave), latent sizes whose cached vector is and is not a size of the
matrix-core attention kernels, rotated parts that turn whole or in part, several layers reading one layer's latent
cache, the order of the three mixers, feed-forwards (gated, routed with one, some or all experts chosen, with and
without the shared expert, none), with and without the row per token pair, the embedding's scale and the constant on
the sublayers.
"""
import numpy as np
import torch

from tests.lomozen_util import check_rows  # noqa: F401  (the same judgement of rows serves every design)
from tests.plain import zeripel_plain as P


def wkv(heads, dim, rank):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim, "decay_rank": rank}}


def attention(heads, kv_heads, dim, scale=None, q_temp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale if scale is not None else dim ** -0.5}
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention", "mixer": m}


def latent(heads, dim, rot_dim, vdim, rank, scale=None, rot=None, kv_from=None):
    """``rot`` (dims, base)."""
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if rot_dim:
        m["rot"] = {"dims": rot[0] if rot else rot_dim, "base": rot[1] if rot else 10000.0}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None, scale=None):
    f = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if scale is not None:
        f["router"]["scale"] = scale
    if shared:
        f["shared"] = {"ff": shared}
    return f


def layer(mixer, mlp=None):
    return dict(mixer, mlp=mlp)


def config(width, vocab, layers, eps=1e-5, bigram=None, scale=None, mult=None):
    c = {"architecture": "Zeripel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    emb = {}
    if bigram:
        emb["bigram"] = dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))
    if scale is not None:
        emb["scale"] = scale
    if emb:
        c["embedding"] = emb
    if mult is not None:
        c["residual_mult"] = mult
    return c


# everything at once: the three mixers, a second latent layer on the first one's cache, part of the rotated part turned,
# gated and routed feed-forwards with and without the shared expert, a layer without a feed-forward
SMALL_A = dict(name="A", seed=3, std=0.25, norm_std=0.1, page_size=8, config=config(48, 131, [
    layer(wkv(3, 8, 5), dense(40)),
    layer(latent(3, 8, 4, 12, 20, scale=0.3, rot=(2, 100.0)), moe(6, 2, 24, shared=16, scale=1.5)),
    layer(attention(4, 2, 12, scale=0.4, q_temp=(0.5, 16)), moe(4, 4, 16)),
    layer(latent(2, 6, 4, 10, 20, rot=(2, 100.0), kv_from=1), None),
    layer(wkv(2, 16, 3), moe(5, 3, 12, shared=8)),
], bigram=(37, 5, 3), scale=0.5, mult=0.3))
# nothing optional, sizes that are no multiples of 4, one expert chosen of five, attention first
SMALL_B = dict(name="B", seed=4, std=0.2, norm_std=0.2, page_size=16, config=config(90, 301, [
    layer(attention(3, 1, 10), moe(5, 1, 18, shared=14)),
    layer(wkv(5, 6, 7), None),
    layer(latent(3, 10, 6, 14, 18, rot=(6, 10.0)), dense(50)),
], eps=1e-6))
# one bucket, multipliers near 2^31, heads above a wave, a cached vector of 128 and heads of 64 (the matrix-core
# attention kernels in bfloat16), three layers on one latent cache, a temperature that steps at every fourth position
SMALL_C = dict(name="C", seed=5, std=0.3, norm_std=0.05, page_size=32, config=config(64, 97, [
    layer(latent(2, 32, 32, 48, 96, rot=(32, 250000.0)), dense(96)),
    layer(latent(4, 16, 32, 16, 96, scale=0.2, rot=(32, 250000.0), kv_from=0), moe(3, 2, 40, shared=24, scale=2.5)),
    layer(wkv(1, 72, 16), moe(4, 2, 24)),
    layer(latent(1, 8, 32, 80, 96, rot=(32, 250000.0), kv_from=0), None),
    layer(attention(4, 2, 64, scale=0.1, q_temp=(1.0, 4)), dense(72)),
], eps=1e-4, bigram=(1, 2147483629, 1000003), scale=2.0, mult=0.7))
ALL_SMALL = [SMALL_A, SMALL_B, SMALL_C]


def make_folder(small, tmp_path, patch=None):
    """A model folder with random weights; ``patch`` {tensor name: value or function of the tensor} rewrites some.
    Sinks and the corrections of the experts' choice are drawn wider than the random-weights mode draws them, so
    that they count."""
    from jax_vllm_amd import write_random_model
    from safetensors.torch import load_file, save_file

    folder = write_random_model(tmp_path, small["config"], seed=small["seed"], std=small["std"], norm_std=small["norm_std"])
    path = str(folder / "model.safetensors")
    tensors = load_file(path)
    g = torch.Generator().manual_seed(small["seed"])
    for name, t in tensors.items():
        if name.endswith(".mix.sink"):
            tensors[name] = (torch.randn(t.shape, generator=g) * 1.5 + 1.0).to(t.dtype)
        if name.endswith(".mlp.correction"):
            tensors[name] = (torch.randn(t.shape, generator=g) * 0.3).to(t.dtype)
    for name, change in (patch or {}).items():
        t = tensors[name]
        new = change(t.float()) if callable(change) else torch.full_like(t.float(), float(change))
        tensors[name] = new.to(t.dtype).contiguous()
    save_file(tensors, path)
    return folder


def plain_of(folder, dtype=torch.float64):
    return P.read_config(folder), P.read_weights(folder, dtype)


def plain_logits(cfg, w, tokens, **kw):
    return P.forward(w, cfg, tokens, **kw).to(torch.float32).numpy()


def expected(cfg, w, tokens, dtype):
    """What ``check_rows`` compares with: the plain logits, and for bfloat16 also the plain logits with every
    matrix product rounded to bfloat16 (the model's own sensitivity to that rounding)."""
    want = plain_logits(cfg, w, tokens)
    if dtype in ("float32", "fp32"):
        return want
    with P.rounded_products(torch.bfloat16):
        return want, plain_logits(cfg, w, tokens)


def tokens_of(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], size=n).tolist()
