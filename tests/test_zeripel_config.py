"""Zeripel on the host: its configuration reader, the tensors its ``ModelSpec`` asks for, which layers read another
layer's cache, what a request keeps (pages, state), a random model folder written and read back (also with the one
size that only the checkpoint gives), and the plain implementation's own consistency."""
import copy
import json

import pytest
import torch

from tests.zeripel_util import ALL_SMALL, SMALL_A, SMALL_B, SMALL_C, attention, config, latent, layer, make_folder, moe, wkv
from tests.plain import zeripel_plain as P


def spec_of(cfg_dict):
    from jax_vllm_amd.config.registry import resolve
    from jax_vllm_amd.parts.model import DecoderModel

    arch, cfg, _ = resolve(cfg_dict)
    return arch, cfg, DecoderModel(arch.build_spec(cfg))


def expected_tensors(c):
    """Names and shapes from the configuration alone, written out independently of the product."""
    w = c["width"]
    out = {"embed": (c["vocab"], w), "final.norm": (w,), "head": (c["vocab"], w)}
    if (c.get("embedding") or {}).get("bigram"):
        out["bigram"] = (c["embedding"]["bigram"]["buckets"] + 1, w)
    for i, l in enumerate(c["layers"]):
        p, m = f"l{i}.", l["mixer"]
        out[p + "norm1"] = (w,)
        H, d = m["heads"], m["dim"]
        if l["type"] == "wkv":
            out.update({p + f"mix.mu.{s}": (w,) for s in "rkvgw"})
            out.update({p + f"mix.{s}": (H * d, w) for s in "rkvg"})
            out.update({p + "mix.w1": (m["decay_rank"], w), p + "mix.w2": (H * d, m["decay_rank"]), p + "mix.w0": (H * d,),
                        p + "mix.u": (H, d), p + "mix.norm": (H * d,), p + "mix.o": (w, H * d)})
        elif l["type"] == "attention":
            out.update({p + "mix.q": (H * d, w), p + "mix.k": (m["kv_heads"] * d, w), p + "mix.q.norm": (d,),
                        p + "mix.k.norm": (d,), p + "mix.o": (w, H * d)})
        else:
            r, rank, dv = m["rot_dim"], m["kv_rank"], m["vdim"]
            out.update({p + "mix.q": (H * (d + r), w), p + "mix.uk": (H * d, rank), p + "mix.uv": (H * dv, rank),
                        p + "mix.sink": (H,), p + "mix.g": (H, w), p + "mix.o": (w, H * dv)})
            if m.get("kv_from") is None:
                out.update({p + "mix.dkv": (rank + r, w), p + "mix.dkv.norm": (rank,)})
        f = l.get("mlp")
        if f:
            out[p + "norm2"] = (w,)
        if f and f["kind"] == "dense":
            out.update({p + "mlp.gate": (f["ff"], w), p + "mlp.up": (f["ff"], w), p + "mlp.down": (w, f["ff"])})
        elif f:
            e, ff = f["router"]["experts"], f["expert"]["ff"]
            out.update({p + "mlp.router": (e, w), p + "mlp.correction": (e,)})
            for j in range(e):
                out.update({f"{p}mlp.e{j}.gate": (ff, w), f"{p}mlp.e{j}.up": (ff, w), f"{p}mlp.e{j}.down": (w, ff)})
            if f.get("shared"):
                s = f["shared"]["ff"]
                out.update({p + "mlp.shared.gate": (s, w), p + "mlp.shared.up": (s, w), p + "mlp.shared.down": (w, s),
                            p + "mlp.shared.sg": (1, w)})
    return out


@pytest.mark.parametrize("small", ALL_SMALL, ids=[s["name"] for s in ALL_SMALL])
def test_tensors_schedule_and_memory_plan_follow_the_configuration(small):
    c = small["config"]
    _, cfg, model = spec_of(c)
    got = {k: tuple(v.shape) for k, v in model.tensor_specs().items()}
    assert got == expected_tensors(c)
    assert [run.layer for run in model.spec.schedule] == list(range(len(c["layers"])))
    plan = model.memory_plan()
    for p, l in zip(plan, c["layers"]):
        m = l["mixer"]
        if l["type"] == "wkv":
            assert p.cache is None and p.cache_of is None
            assert {s.name: s.shape for s in p.state} == {"S": (m["heads"], m["dim"], m["dim"]), "shift": (c["width"],)}
            assert all(s.dtype == "float32" for s in p.state)
        elif l["type"] == "attention":
            assert p.state is None and p.cache_of is None and p.cache.window is None
            assert [t.token_shape for t in p.cache.tensors] == [(m["kv_heads"], -(-m["dim"] // 16) * 16)] * 2
        else:
            assert p.state is None and p.cache_of == m.get("kv_from") and p.cache.window is None
            assert [t.token_shape for t in p.cache.tensors] == [(1, m["kv_rank"] + m["rot_dim"])] * 2
    assert model.replayable()


def test_layers_that_read_another_layers_cache_keep_none():
    from jax_vllm_amd.cache.storage import cache_bytes_per_token

    _, _, model = spec_of(SMALL_C["config"])
    plan = model.memory_plan()
    assert [p.cache_of for p in plan] == [None, 0, None, 0, None]
    # per token: one latent vector of 128 in two layouts, keys and values of 2 heads of 64
    assert cache_bytes_per_token(plan, torch.bfloat16) == 2 * (2 * 128 + 2 * 2 * 64)


def test_configuration_errors_name_the_place():
    from jax_vllm_amd.config.errors import ConfigError
    from jax_vllm_amd.config.registry import resolve

    def broken(change):
        c = copy.deepcopy(SMALL_A["config"])
        change(c)
        with pytest.raises(ConfigError) as e:
            resolve(c)
        return str(e.value)

    assert "layers[2].mixer" in broken(lambda c: c["layers"][2]["mixer"].update(kv_heads=3))
    assert "layers[2].mixer.vdim" in broken(lambda c: c["layers"][2]["mixer"].update(vdim=16))
    assert "layers[1].mixer.rot.dims" in broken(lambda c: c["layers"][1]["mixer"]["rot"].update(dims=6))
    assert "layers[1].mixer.rot.dims" in broken(lambda c: c["layers"][1]["mixer"]["rot"].update(dims=3))
    assert "layers[1].mlp.router.top" in broken(lambda c: c["layers"][1]["mlp"]["router"].update(top=7))
    assert "layers[2].type" in broken(lambda c: c["layers"][2].update(type="retention"))
    assert "layers[0].mlp.kind" in broken(lambda c: c["layers"][0]["mlp"].update(kind="sparse"))
    assert "layers[3].mixer.kv_from" in broken(lambda c: c["layers"][3]["mixer"].update(kv_from=3))
    assert "layers[3].mixer.kv_from" in broken(lambda c: c["layers"][3]["mixer"].update(kv_from=2))
    assert "kv_rank differs" in broken(lambda c: c["layers"][3]["mixer"].update(kv_rank=24))
    assert "rot differs" in broken(lambda c: c["layers"][3]["mixer"].update(rot={"dims": 2, "base": 50.0}))
    assert "q_temp" in broken(lambda c: c["layers"][2]["mixer"]["q_temp"].update(every=0))
    assert "bigram" in broken(lambda c: c["embedding"]["bigram"].update(buckets=0))
    assert "scale" in broken(lambda c: c["layers"][1]["mixer"].pop("scale"))
    assert "layers[0].mixer.heads" in broken(lambda c: c["layers"][0]["mixer"].update(heads=0))
    assert "shared" in broken(lambda c: c["layers"][1]["mlp"]["shared"].update(ff=0))


def test_random_folder_is_read_back_and_the_decay_rank_comes_from_the_checkpoint(tmp_path):
    from jax_vllm_amd import write_random_model
    from jax_vllm_amd.weights.loader import check_against_specs
    from jax_vllm_amd.weights.safetensors_io import open_shards

    folder = write_random_model(tmp_path, SMALL_C["config"], seed=1, std=0.1, norm_std=0.05)
    w = P.read_weights(folder)
    assert {k: tuple(v.shape) for k, v in w.items()} == expected_tensors(SMALL_C["config"])
    assert 0.0 <= float(w["l2.mix.mu.k"].min()) and float(w["l2.mix.mu.k"].max()) <= 1.0
    assert P.forward(w, P.read_config(folder), [1, 2, 3]).shape == (3, 97)
    # a configuration that leaves the decay's inner size out: any checkpoint size fits, random weights need it
    bare = copy.deepcopy(SMALL_C["config"])
    del bare["layers"][2]["mixer"]["decay_rank"]
    _, _, model = spec_of(bare)
    specs = model.tensor_specs()
    assert tuple(specs["l2.mix.w1"].shape) == (None, 64) and tuple(specs["l2.mix.w2"].shape) == (72, None)
    shard = next(iter(open_shards(folder)))
    assert check_against_specs(folder, specs, set(), dict(shard.entries)) == []
    shard.close()
    with pytest.raises(ValueError, match="random weights need every size"):
        write_random_model(tmp_path / "bare", bare, seed=1)


def test_plain_pieces():
    """The plain implementation against itself: the latent form of attention equals attention over keys and values
    written out per head; the recurrence's outputs do not depend on where a sequence is cut when the state and the
    row before are carried; a sink of minus infinity is no sink; the router's weights sum to its scale."""
    torch.manual_seed(0)
    folder_cfg = SMALL_A["config"]
    import tempfile
    from pathlib import Path

    with tempfile.TemporaryDirectory() as d:
        folder = make_folder(SMALL_A, Path(d))
        cfg, w = P.read_config(folder), P.read_weights(folder, torch.float64)
    assert cfg == json.loads(json.dumps(folder_cfg))
    n, eps = 23, cfg["norm"]["eps"]
    u = torch.randn(n, cfg["width"], dtype=torch.float64)
    # latent attention, written out with explicit keys and values
    m = cfg["layers"][1]["mixer"]
    p = "l1.mix."
    cache = P.latent_cache(w, p, m, u, eps)
    got = P.latent_attention(w, p, m, u, eps, cache)
    H, D, R, V = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, kr = cache
    q = (u @ w[p + "q"].T).view(n, H, D + R)
    q = torch.cat([q[..., :D], P.rotate_pairs(q[..., D:], range(n), m["rot"])], -1)
    k = torch.cat([(c @ w[p + "uk"].T).view(n, H, D), kr.unsqueeze(1).expand(n, H, R)], -1)
    v = (c @ w[p + "uv"].T).view(n, H, V)
    gate = torch.sigmoid(u @ w[p + "g"].T)
    out = torch.zeros(n, H, V, dtype=torch.float64)
    for h in range(H):
        for i in range(n):
            s = (k[:i + 1, h] @ q[i, h]) * m["scale"]
            e = torch.exp(s - s.max())
            denom = e.sum() + torch.exp(w[p + "sink"][h] - s.max())
            out[i, h] = (e / denom) @ v[:i + 1, h] * gate[i, h]
    assert torch.allclose(got, out.reshape(n, H * V) @ w[p + "o"].T, atol=1e-10)
    # only pairs below rot.dims turn
    x = torch.randn(5, 3, 4, dtype=torch.float64)
    turned = P.rotate_pairs(x, [0, 1, 2, 3, 4], {"dims": 2, "base": 100.0})
    assert torch.equal(turned[..., 2:], x[..., 2:]) and torch.equal(turned[0], x[0]) and not torch.allclose(turned[1:, :, :2], x[1:, :, :2])
    # the recurrence: the state after every token is decay * the one before + k v^T, and the first output has the bonus alone
    keep = []
    m0 = cfg["layers"][0]["mixer"]
    P.wkv(w, "l0.mix.", m0, u, eps, keep)
    assert len(keep) == n and keep[0].shape == (m0["heads"], m0["dim"], m0["dim"])
    b = u[:1] * (1 - w["l0.mix.mu.k"])          # the first token blends with zeros
    k0 = (b @ w["l0.mix.k"].T).view(m0["heads"], m0["dim"])
    bv = u[:1] * (1 - w["l0.mix.mu.v"])
    v0 = (bv @ w["l0.mix.v"].T).view(m0["heads"], m0["dim"])
    assert torch.allclose(keep[0], k0.unsqueeze(2) * v0.unsqueeze(1), atol=1e-12)
    # the causal softmax with and without a sink
    s = torch.randn(2, 4, 4, dtype=torch.float64)
    assert torch.allclose(P.causal_softmax(s, torch.full((2,), -1e9, dtype=torch.float64)), P.causal_softmax(s))
    assert float(P.causal_softmax(s, torch.zeros(2, dtype=torch.float64))[0, 0, 0]) == pytest.approx(
        float(torch.exp(s[0, 0, 0]) / (torch.exp(s[0, 0, 0]) + 1)))
    # the router: weights of the chosen sum to the scale, the correction changes the choice and not the weights
    f = cfg["layers"][1]["mlp"]
    choice, weight = P.router(w, "l1.mlp.", f, u)
    assert torch.allclose(weight.sum(-1), torch.full((n,), f["router"]["scale"], dtype=torch.float64))
    w2 = dict(w)
    w2["l1.mlp.correction"] = w["l1.mlp.correction"] + torch.tensor([5.0, 0, 0, 0, 0, 0], dtype=torch.float64)
    choice2, weight2 = P.router(w2, "l1.mlp.", f, u)
    assert (choice2 == 0).any(-1).all()
    sig = torch.sigmoid(u @ w["l1.mlp.router"].T)
    picked = torch.gather(sig, 1, choice2)
    assert torch.allclose(weight2, picked / picked.sum(-1, keepdim=True) * f["router"]["scale"])
    # the temperature counts position + 1
    t = P.query_temperature(range(40), {"coef": 0.5, "every": 16})
    assert float(t[14]) == 1.0 and float(t[15]) == pytest.approx(1 + 0.5 * 0.6931471805599453) and float(t[31]) == pytest.approx(1 + 0.5 * 1.0986122886681098)


def test_registry_knows_the_design():
    from jax_vllm_amd.config.registry import supported_architectures

    assert "Zeripel" in supported_architectures()
    assert SMALL_B["config"]["architecture"] == "Zeripel"
