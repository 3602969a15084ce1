"""Small Bozisun configurations of the test-suite and what the tests of that design share.

The configurations differ from one another in every size and constant: widths (also no multiple of 4), head counts and
ratios, key and value sizes (equal, larger, smaller, above a wave), rotated dimensions (none, part of a head, all of it),
rescaled and plain frequencies, feed-forwards (gated, routed with one, some or all experts chosen, none), with and
without the row per token pair, the per-layer token input, the loop (from the first layer, over all layers, once) and
the cap on the logits.
"""
import numpy as np
import torch

from tests.lomozen_util import check_rows  # noqa: F401  (the same judgement of rows serves every design)
from tests.plain import bozisun_plain as P


def rot(dims, base=10000.0, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling:
        r["scaling"] = scaling
    return r


def attention(heads, kv_heads, dim, vdim, scale=None, rot_=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if rot_:
        m["rot"] = rot_
    return {"type": "attention", "mixer": m}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def layer(mixer, mlp=None):
    return dict(mixer, mlp=mlp)


def config(width, vocab, layers, eps=1e-5, bigram=None, side=None, loop=None, softcap=None):
    c = {"architecture": "Bozisun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if bigram:
        c["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))}
    if side:
        c["token_side"] = {"dim": side}
    if loop:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    if softcap:
        c["logit_softcap"] = softcap
    return c


YARN = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}

# everything at once: value heads larger than key heads, one to three q heads a kv head, part of a head rotated with
# rescaled frequencies, a whole head rotated with plain ones, no rotation; gated, routed and no feed-forward; the two
# middle layers run twice
SMALL_A = dict(name="A", seed=3, std=0.25, norm_std=0.1, page_size=8, config=config(48, 131, [
    layer(attention(3, 3, 8, 12, scale=0.4, rot_=rot(6, 100.0, YARN)), dense(40)),
    layer(attention(4, 2, 12, 20, rot_=rot(12, 500.0)), moe(6, 2, 24)),
    layer(attention(3, 1, 16, 16, scale=0.3), None),
    layer(attention(2, 2, 8, 4, rot_=rot(4, 50.0, dict(YARN, factor=1.5))), moe(4, 4, 16)),
], bigram=(37, 5, 3), side=6, loop=(1, 3, 2), softcap=8.0))
# nothing optional, sizes that are no multiples of 4, one expert chosen of five
SMALL_B = dict(name="B", seed=4, std=0.2, norm_std=0.2, page_size=16, config=config(90, 301, [
    layer(attention(3, 1, 10, 6, rot_=rot(10, 1e4)), moe(5, 1, 18)),
    layer(attention(2, 2, 6, 14, scale=0.9), dense(50)),
    layer(attention(5, 5, 2, 2, rot_=rot(2, 10.0)), None),
], eps=1e-6))
# one bucket, multipliers near 2^31, a token input of five columns, the loop over all layers three times, heads
# above a wave, a value size above and below the key size
SMALL_C = dict(name="C", seed=5, std=0.3, norm_std=0.05, page_size=32, config=config(64, 97, [
    layer(attention(1, 1, 72, 80, rot_=rot(32, 1e6, dict(YARN, original=32))), dense(96)),
    layer(attention(4, 2, 32, 16, scale=0.7, rot_=rot(32, 250000.0)), moe(3, 2, 40)),
], eps=1e-4, bigram=(1, 2147483629, 1000003), side=5, loop=(0, 2, 3), softcap=30.0))
ALL_SMALL = [SMALL_A, SMALL_B, SMALL_C]


def make_folder(small, tmp_path, patch=None):
    """A model folder with random weights; ``patch`` {tensor name: value or function of the tensor} rewrites some."""
    from jax_vllm_amd import write_random_model

    folder = write_random_model(tmp_path, small["config"], seed=small["seed"], std=small["std"], norm_std=small["norm_std"])
    if patch:
        from safetensors.torch import load_file, save_file

        path = str(folder / "model.safetensors")
        tensors = load_file(path)
        for name, change in patch.items():
            t = tensors[name]
            new = change(t.float()) if callable(change) else torch.full_like(t.float(), float(change))
            tensors[name] = new.to(t.dtype).contiguous()
        save_file(tensors, path)
    return folder


def plain_of(folder, dtype=torch.float64):
    return P.read_config(folder), P.read_weights(folder, dtype)


def plain_logits(cfg, w, tokens):
    return P.forward(w, cfg, tokens).to(torch.float32).numpy()


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
