"""Bozisun on the host: its configuration reader, the tensors its ``ModelSpec`` asks for, the order in which looped
layers run and their caches, a random model folder written and read back, the rescaled frequencies of its rotation,
the previous token that the cache manager keeps for the embedding, and the plain implementation's own consistency."""
import copy

import pytest
import torch

from tests.bozisun_util import ALL_SMALL, SMALL_A, SMALL_B, SMALL_C, YARN, attention, config, dense, layer, moe, rot
from tests.plain import bozisun_plain as P


def spec_of(cfg_dict):
    from jax_vllm_amd.config.registry import resolve
    from jax_vllm_amd.parts.model import DecoderModel

    arch, cfg, _ = resolve(cfg_dict)
    return arch, cfg, DecoderModel(arch.build_spec(cfg))


def expected_tensors(c):
    """Names and shapes from the configuration alone, written out independently of the product."""
    w, n = c["width"], len(c["layers"])
    out = {"embed": (c["vocab"], w), "final.norm": (w,), "head": (c["vocab"], w)}
    if c.get("embedding"):
        out["bigram"] = (c["embedding"]["bigram"]["buckets"] + 1, w)
    side = (c.get("token_side") or {}).get("dim")
    if side:
        out["side.embed"] = (c["vocab"], n * side)
    for i, l in enumerate(c["layers"]):
        p, m = f"l{i}.", l["mixer"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        out.update({p + "norm1": (w,), p + "mix.q": (H * d, w), p + "mix.k": (G * d, w), p + "mix.v": (G * dv, w),
                    p + "mix.q.norm": (d,), p + "mix.k.norm": (d,), p + "mix.g": (H * dv, w), p + "mix.o": (w, H * dv)})
        f = l.get("mlp")
        if f and f["kind"] == "dense":
            out.update({p + "mlp.gate": (f["ff"], w), p + "mlp.up": (f["ff"], w), p + "mlp.down": (w, f["ff"])})
        elif f:
            e, ff = f["router"]["experts"], f["expert"]["ff"]
            out.update({p + "mlp.router": (e, w), p + "mlp.router.b": (e,)})
            for j in range(e):
                out.update({f"{p}mlp.e{j}.gate": (ff, w), f"{p}mlp.e{j}.up": (ff, w), f"{p}mlp.e{j}.down": (w, ff)})
        if side:
            out.update({p + "side.gate": (side, w), p + "side.proj": (w, side), p + "side.norm": (w,)})
    return out


@pytest.mark.parametrize("small", ALL_SMALL, ids=[s["name"] for s in ALL_SMALL])
def test_tensors_schedule_and_memory_plan_follow_the_configuration(small):
    c = small["config"]
    _, cfg, model = spec_of(c)
    got = {k: tuple(v.shape) for k, v in model.tensor_specs().items()}
    assert got == expected_tensors(c)
    order = [run.layer for run in model.spec.schedule]
    assert order == P.layer_order(c) == cfg.layer_order()
    plan = model.memory_plan()
    assert len(plan) == len(order) and all(p.cache_of is None for p in plan)       # every pass keeps its own keys
    for p in plan:
        m = c["layers"][p.layer]["mixer"]
        padded = -(-max(m["dim"], m["vdim"]) // 16) * 16
        assert p.state is None and p.cache.window is None
        assert [t.token_shape for t in p.cache.tensors] == [(m["kv_heads"], padded)] * 2
    assert model.replayable()


def test_the_order_of_looped_layers():
    from jax_vllm_amd.config.registry import resolve

    def order(n, loop):
        c = config(16, 20, [layer(attention(1, 1, 4, 4))] * n, loop=loop)
        return resolve(c)[1].layer_order()

    assert order(5, (2, 4, 3)) == [0, 1, 2, 3, 2, 3, 2, 3, 4]
    assert order(3, None) == [0, 1, 2]
    assert order(3, (0, 3, 2)) == [0, 1, 2, 0, 1, 2]
    assert order(3, (2, 3, 1)) == [0, 1, 2]
    assert order(4, (1, 1, 5)) == [0, 1, 2, 3]                # an empty range
    assert order(2, (1, 2, 4)) == [0, 1, 1, 1, 1]


def test_configuration_errors_name_the_place():
    from jax_vllm_amd.config.errors import ConfigError
    from jax_vllm_amd.config.registry import resolve

    def broken(change):
        c = copy.deepcopy(SMALL_A["config"])
        change(c)
        with pytest.raises(ConfigError) as e:
            resolve(c)
        return str(e.value)

    assert "layers[1].mixer" in broken(lambda c: c["layers"][1]["mixer"].update(kv_heads=3))
    assert "layers[0].mixer.rot.dims" in broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10))
    assert "layers[0].mixer.rot.dims" in broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=5))
    assert "layers[1].mlp.router.top" in broken(lambda c: c["layers"][1]["mlp"]["router"].update(top=7))
    assert "layers[2].type" in broken(lambda c: c["layers"][2].update(type="retention"))
    assert "layers[0].mlp.kind" in broken(lambda c: c["layers"][0]["mlp"].update(kind="sparse"))
    assert "loop" in broken(lambda c: c["loop"].update(stop=9))
    assert "loop" in broken(lambda c: c["loop"].update(times=0))
    assert "bigram" in broken(lambda c: c["embedding"]["bigram"].update(buckets=0))
    assert "token_side" in broken(lambda c: c["token_side"].update(dim=0))
    assert "logit_softcap" in broken(lambda c: c.update(logit_softcap=-1.0))
    assert "scale" in broken(lambda c: c["layers"][0]["mixer"].pop("scale"))


def test_random_folder_is_read_back(tmp_path):
    from jax_vllm_amd import write_random_model
    from jax_vllm_amd.weights.safetensors_io import open_shards

    folder = write_random_model(tmp_path, SMALL_C["config"], seed=1, std=0.1, norm_std=0.05)
    w = P.read_weights(folder)
    assert {k: tuple(v.shape) for k, v in w.items()} == expected_tensors(SMALL_C["config"])
    assert abs(float(w["l1.side.norm"].mean()) - 1.0) < 0.05 and abs(float(w["l0.mix.q.norm"].mean()) - 1.0) < 0.05
    shard = next(iter(open_shards(folder)))
    assert set(shard.entries) == set(w)
    shard.close()
    assert P.forward(w, P.read_config(folder), [1, 2, 3]).shape == (3, 97)


def test_frequencies_of_the_rotation_part_follow_the_rescaling_rule():
    from jax_vllm_amd.parts.rotary import RotaryEncoding

    for dims, base, sc in ((6, 100.0, YARN), (32, 1e6, dict(YARN, original=32)), (48, 40000.0, dict(YARN, original=2048, factor=6.0, fast=16.0)),
                           (12, 500.0, None)):
        part = RotaryEncoding(dims + 4, base, dims, rescale=sc)
        want, amp = P.rotary_frequencies(rot(dims, base, sc))
        got = part.inverse_frequencies().double()
        assert got.shape == (dims // 2,) and float(((got - want) / want).abs().max()) < 3e-7
        assert abs(part.amplitude - amp) < 1e-12
    # the three branches all occur: a pair that keeps its frequency, one slowed down by the factor, one blended
    f = 40000.0 ** (-2.0 * torch.arange(24, dtype=torch.float64) / 48)
    ratio = P.rotary_frequencies(rot(48, 40000.0, dict(YARN, original=2048, factor=6.0, fast=16.0)))[0] / f
    assert float(ratio[0]) == 1.0 and abs(float(ratio[-1]) - 1 / 6) < 1e-12 and any(0.18 < float(r) < 0.99 for r in ratio)


def test_the_cache_manager_keeps_the_previous_token():
    from jax_vllm_amd.cache.manager import CacheManager

    cache = CacheManager([("full",)], 4, 8, 2, enable_prefix_cache=False)
    cache.start("a")
    assert cache.last_token("a") == -1                  # nothing before a sequence's first token
    cache.reserve("a", 3)
    cache.commit("a", [7, 8, 9])
    assert cache.last_token("a") == 9
    cache.start("b")
    assert cache.last_token("b") == -1
    cache.finish("a")
    cache.start("a")                                    # the id again: a new sequence
    assert cache.last_token("a") == -1


def test_the_cache_manager_keeps_the_previous_token_behind_a_cached_prefix():
    from jax_vllm_amd.cache.manager import CacheManager

    cache = CacheManager([("full",)], 4, 8, 2, enable_prefix_cache=True)
    prompt = list(range(10, 23))
    cache.start("a", prompt)
    cache.reserve("a", len(prompt))
    cache.commit("a", prompt)
    cache.finish("a")
    assert cache.start("b", prompt) == 12               # three full pages are taken over
    assert cache.last_token("b") == prompt[11]


def test_plain_pieces():
    """The oracle's own sanity: no position looks ahead; the row of a token pair; the router's choice; the order of
    the looped layers; the cap."""
    c = SMALL_A["config"]
    torch.manual_seed(0)
    _, _, model = spec_of(c)
    w = {k: torch.randn(v.shape, dtype=torch.float64) * 0.3 for k, v in model.tensor_specs().items()}
    toks = list(range(1, 20))
    full = P.forward(w, c, toks)
    assert torch.allclose(P.forward(w, c, toks[:11]), full[:11], atol=1e-12)
    assert float(full.abs().max()) < c["logit_softcap"]
    assert P.bigram_rows([4, 9, 9], {"buckets": 37, "mul_prev": 5, "mul_cur": 3}) == [37, (20 + 27) % 37, (45 + 27) % 37]
    big = {"buckets": 61, "mul_prev": 2147483629, "mul_cur": 1000003}
    assert P.bigram_rows([96, 95], big) == [61, (96 * 2147483629 + 95 * 1000003) % 61]
    idx, wgt = P.router_choice(torch.tensor([[0.0, 3.0, 1.0, 2.0]], dtype=torch.float64), 2)
    assert idx.tolist() == [[1, 3]] and torch.allclose(wgt, torch.softmax(torch.tensor([[3.0, 2.0]], dtype=torch.float64), -1))
    # a first token's logits differ from the same token's behind another one: the pair row and the attention both see it
    assert not torch.allclose(P.forward(w, c, [5])[0], P.forward(w, c, [6, 5])[1])
    # layers outside the loop run once: with times = 1 the loop changes nothing
    once = copy.deepcopy(c)
    once["loop"]["times"] = 1
    none = copy.deepcopy(c)
    none.pop("loop")
    assert torch.equal(P.forward(w, once, toks), P.forward(w, none, toks))
    assert not torch.allclose(P.forward(w, c, toks), P.forward(w, none, toks))
    # every optional piece can be left out
    bare = config(48, 131, [layer(attention(3, 3, 8, 12)), layer(attention(4, 2, 12, 20, rot_=rot(12)), dense(8)),
                            layer(attention(1, 1, 4, 4), moe(2, 1, 4))])
    _, _, model = spec_of(bare)
    wb = {k: torch.randn(v.shape, dtype=torch.float64) * 0.3 for k, v in model.tensor_specs().items()}
    assert "bigram" not in wb and "side.embed" not in wb
    assert P.forward(wb, bare, toks).shape == (19, 131)


def test_registry_knows_the_design():
    from jax_vllm_amd.config.registry import supported_architectures

    assert "Bozisun" in supported_architectures()
    assert SMALL_B["config"]["architecture"] == "Bozisun"
