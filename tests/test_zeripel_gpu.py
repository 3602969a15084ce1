"""Zeripel on the GPU against its plain implementation (``tests/plain/zeripel_plain.py``): each mechanism alone, whole
prompts against portions and token-by-token decoding, unequal requests in one batch against each alone, pages and
slots that are used again, keys at page borders and one far key among hundreds, a state that remembers a token from
hundreds of steps back, the row before a portion's first one, the positions at which the query temperature steps,
sinks that carry the denominator, layers that read another layer's latent cache, long decoding through recorded
steps, sizes that are no multiples of anything, greedy generation through the entry point and its scheduler, and the
kernels alone."""
import math

import numpy as np
import pytest
import torch

from tests.zeripel_util import (ALL_SMALL, SMALL_A, SMALL_B, SMALL_C, attention, check_rows, config, dense, expected, latent,
                                layer, make_folder, moe, plain_logits, plain_of, tokens_of, wkv)
from tests.plain import zeripel_plain as P

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {s["name"]: make_folder(s, tmp_path_factory.mktemp(f"zp{s['name']}")) for s in ALL_SMALL}


def entry(rid, tokens, want=None):
    from jax_vllm_amd.engine.entries import StepEntry

    return StepEntry(rid, tokens, range(len(tokens)) if want is None else want)


def make_core(folder, dtype, page_size, pages=64, seqs=4, graphs=False):
    from jax_vllm_amd.config import EngineConfig
    from jax_vllm_amd.engine.core import EngineCore
    from jax_vllm_amd.weights import load_model

    model, _ = load_model(folder, dtype, "cuda")
    cfg = EngineConfig(dtype=dtype, block_size=page_size, num_blocks=pages + 1, max_num_seqs=seqs,
                       max_model_len=pages * page_size, max_num_batched_tokens=4096, enable_prefix_cache=False,
                       use_hip_graphs=graphs)
    return EngineCore(model, cfg)


def run_cut(core, rid, tokens, cuts):
    """The request's logits at every position, its tokens fed in portions of the given sizes."""
    core.start_request(rid)
    out, at = [], 0
    for n in cuts:
        out.append(core.run([entry(rid, tokens[at:at + n])]).cpu().numpy())
        at += n
    assert at == len(tokens)
    core.finish_request(rid)
    return np.concatenate(out)


# ------------------------------------------------------------------ each mechanism alone
TINY = attention(1, 1, 4)            # the smallest mixer, beside the feed-forward under test
ALONE = {
    "time_mix": dict(layers=[layer(wkv(3, 8, 5))]),
    "time_mix_one_head_above_a_wave": dict(layers=[layer(wkv(1, 80, 2))]),
    "attention_groups_and_temperature": dict(layers=[layer(attention(4, 2, 12, scale=1.5, q_temp=(0.7, 8)))]),
    "attention_one_kv_head_no_temperature": dict(layers=[layer(attention(6, 1, 16, scale=0.2))]),
    "latent_attention": dict(layers=[layer(latent(3, 8, 4, 12, 20, scale=0.5, rot=(4, 100.0)))]),
    "latent_attention_part_of_the_part_turned": dict(layers=[layer(latent(2, 6, 8, 5, 11, rot=(2, 30.0)))]),
    "latent_attention_nothing_turned": dict(layers=[layer(latent(2, 6, 0, 5, 12))]),
    "latent_cache_read_by_two_layers": dict(layers=[layer(latent(2, 8, 4, 6, 16, rot=(4, 50.0))), layer(TINY),
                                                    layer(latent(3, 4, 4, 10, 16, scale=0.7, rot=(4, 50.0), kv_from=0)),
                                                    layer(latent(1, 12, 4, 8, 16, rot=(4, 50.0), kv_from=0))]),
    "gated_feed_forward": dict(layers=[layer(TINY, dense(72))]),
    "routed_experts": dict(layers=[layer(TINY, moe(7, 3, 24, scale=1.5))]),
    "routed_experts_one_chosen": dict(layers=[layer(TINY, moe(4, 1, 10))]),
    "routed_experts_all_chosen": dict(layers=[layer(TINY, moe(3, 3, 16, scale=0.5))]),
    "shared_expert_under_its_gate": dict(layers=[layer(TINY, moe(4, 2, 8, shared=20))]),
    "token_pair_rows_and_scale": dict(layers=[layer(TINY)], bigram=(23, 7, 11), scale=3.0),
    "scale_without_pair_rows": dict(layers=[layer(TINY)], scale=0.25),
    "constant_on_the_sublayers": dict(layers=[layer(TINY, dense(16)), layer(TINY)], mult=0.3),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", sorted(ALONE))
def test_one_mechanism_at_a_time(tmp_path, dtype, which):
    """A model of one or a few layers with one mechanism beside the smallest mixer and nothing else optional: a prompt
    of 70 tokens whole, and again in portions down to two tokens and single ones."""
    small = dict(name=which, seed=11, std=0.3, norm_std=0.2, config=config(40, 61, **ALONE[which]))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 70, 1)
    want = expected(cfg, w, toks, dtype)
    core = make_core(folder, dtype, 8)
    check_rows(dtype, run_cut(core, "whole", toks, [70]), want, "whole")
    check_rows(dtype, run_cut(core, "cut", toks, [2, 3, 1, 17, 2, 31, 1, 1, 2, 10]), want, "portions")


def test_the_corrected_choice_differs_from_the_largest_scores(tmp_path):
    """The correction decides which experts run, the weights do not contain it: with corrections as large as the
    scores' spread many tokens choose other experts than their largest scores (seen on the plain implementation), and
    the engine follows."""
    small = dict(name="corr", seed=19, std=0.3, norm_std=0.2, config=config(40, 61, [layer(TINY, moe(6, 2, 12, shared=8, scale=1.5))]))
    folder = make_folder(small, tmp_path, {"l0.mlp.correction": lambda t: torch.tensor([0.4, -0.4, 0.3, -0.3, 0.2, 0.0])})
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 60, 2)
    u = torch.randn(60, 40, dtype=torch.float64)
    choice, _ = P.router(w, "l0.mlp.", cfg["layers"][0]["mlp"], u)
    plain_top = torch.topk(torch.sigmoid(u @ w["l0.mlp.router"].T), 2, dim=-1).indices
    assert (choice.sort(-1).values != plain_top.sort(-1).values).any(-1).float().mean() > 0.2
    core = make_core(folder, "float32", 8)
    check_rows("float32", run_cut(core, "whole", toks, [60]), expected(cfg, w, toks, "float32"), "whole")
    check_rows("float32", run_cut(core, "cut", toks, [1, 2, 30, 27]), expected(cfg, w, toks, "float32"), "portions")


# ------------------------------------------------------------------ portions, decoding, first tokens
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("small", ALL_SMALL, ids=[s["name"] for s in ALL_SMALL])
def test_whole_prompt_portions_and_decoding_agree(folders, dtype, small):
    cfg, w = plain_of(folders[small["name"]])
    toks = tokens_of(cfg, 75, 2)
    want = expected(cfg, w, toks, dtype)
    core = make_core(folders[small["name"]], dtype, small["page_size"])
    check_rows(dtype, run_cut(core, "whole", toks, [75]), want, "whole")
    check_rows(dtype, run_cut(core, "single", toks, [1] * 75), want, "token by token")
    check_rows(dtype, run_cut(core, "twos", toks, [2] * 37 + [1]), want, "portions of two")
    check_rows(dtype, run_cut(core, "mixed", toks, [7, 9, 16, 1, 1, 33, 8]), want, "portions of several sizes")
    check_rows(dtype, run_cut(core, "prompt+decode", toks, [40] + [1] * 35), want, "prompt, then decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("small", ALL_SMALL, ids=[s["name"] for s in ALL_SMALL])
def test_first_tokens_of_a_sequence(folders, dtype, small):
    """The first token takes the spare row of the pair table, blends with a row of zeros, starts from an empty state and
    sees one key beside the sink: prompts of one to five tokens in every cut."""
    cfg, w = plain_of(folders[small["name"]])
    toks = [5, 1, 9, 2, 7]
    want = expected(cfg, w, toks, dtype)
    core = make_core(folders[small["name"]], dtype, small["page_size"])
    for rid, cuts in (("one", [1, 1, 1, 1, 1]), ("two", [1, 2, 2]), ("three", [3, 2]), ("whole", [5])):
        check_rows(dtype, run_cut(core, rid, toks, cuts), want, rid)
    check_rows(dtype, run_cut(core, "alone", toks[:1], [1]), expected(cfg, w, toks[:1], dtype), "a prompt of one token")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_row_before_a_portion_decides_its_first_row(tmp_path, dtype):
    """One time-mixing layer whose blends read the row before alone (every mu is 1), two requests with the same tokens
    but for one in the middle: the row behind the changed token differs by much (checked on the plain implementation),
    so a row before that is lost at a portion's start, taken from the batch's neighbour or from the slot's last owner
    shows.  Both requests run cut at different places, side by side, and a third in a slot that was used before."""
    small = dict(name="shift", seed=13, std=0.3, norm_std=0.1, config=config(32, 50, [layer(wkv(2, 8, 4))], bigram=(41, 13, 29)))
    ones = {f"l0.mix.mu.{s}": 1.0 for s in "rkvgw"}
    folder = make_folder(small, tmp_path, dict(ones, **{"l0.mix.w0": 1.5}))      # a fast decay: the state forgets within a few tokens
    cfg, w = plain_of(folder)
    a = tokens_of(cfg, 40, 3)
    b = list(a)
    b[19] = (a[19] + 7) % 50
    c = [(t + 3) % 50 for t in a]
    plain_a, plain_b = plain_logits(cfg, w, a), plain_logits(cfg, w, b)
    moved = np.abs(plain_a[20] - plain_b[20]).max()
    assert moved > 0.05 * np.abs(plain_a).max()
    core = make_core(folder, dtype, 8, seqs=2)
    for rid, toks in (("a", a), ("b", b)):
        check_rows(dtype, run_cut(core, rid, toks, [1, 1, 2, 5, 1, 1, 9, 2, 18]), expected(cfg, w, toks, dtype), rid)
    core.start_request("a")
    core.start_request("b")
    got = {"a": [], "b": []}
    at = {"a": 0, "b": 0}
    for na, nb in ((20, 1), (1, 19), (2, 1), (1, 1), (16, 18)):
        es = []
        for r, toks, n in (("a", a, na), ("b", b, nb)):
            es.append(entry(r, toks[at[r]:at[r] + n]))
            at[r] += n
        out = core.run(es).cpu().numpy()
        got["a"].append(out[:na])
        got["b"].append(out[na:])
    core.finish_request("a")
    core.finish_request("b")
    check_rows(dtype, np.concatenate(got["a"]), expected(cfg, w, a, dtype), "a beside b")
    check_rows(dtype, np.concatenate(got["b"]), expected(cfg, w, b, dtype), "b beside a")
    check_rows(dtype, run_cut(core, "c", c, [1] * 6 + [34]), expected(cfg, w, c, dtype), "a slot used again")


# ------------------------------------------------------------------ far keys, page borders, a long memory
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mixer", ["attention", "latent"])
def test_one_far_key_among_hundreds_and_page_borders(tmp_path, dtype, mixer):
    """Scores sharp enough that single keys carry a row, as often as not far ones: rows beyond position 200 change by
    much when the plain implementation is kept from seeing keys more than 150 back.  300 tokens over 19 pages: whole,
    in portions that end at, one before and one after page borders, and with the last 40 decoded."""
    mix = attention(4, 2, 16, scale=3.0, q_temp=(0.3, 100)) if mixer == "attention" else \
        latent(4, 16, 8, 8, 24, scale=3.0, rot=(8, 1e4))
    small = dict(name="far", seed=23, std=0.3, norm_std=0.1, config=config(32, 50, [layer(mix)]))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 300, 12)
    want = expected(cfg, w, toks, dtype)
    plain = plain_logits(cfg, w, toks)
    near = plain_logits(cfg, w, toks, only_last_keys=150)
    assert np.median(np.abs(near[200:] - plain[200:]).max(axis=-1)) > 0.01 * np.abs(plain).max()
    core = make_core(folder, dtype, 16, pages=20)
    check_rows(dtype, run_cut(core, "whole", toks, [300]), want, "whole")
    check_rows(dtype, run_cut(core, "portions", toks, [64, 63, 1, 17, 47, 2, 66] + [1] * 40), want, "portions and decoding")
    assert core.cache.num_free_pages(0) == 20       # every page came back


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_state_remembers_a_token_from_hundreds_of_steps_back(tmp_path, dtype):
    """A time-mixing layer that hardly decays (the decay's base far below zero): the rows at the end change when the
    fourth token is another one (seen on the plain implementation), so a state that is lost, reset or handed to the
    wrong request between portions shows there.  260 tokens whole, in portions, and with a decoded tail."""
    small = dict(name="mem", seed=29, std=0.3, norm_std=0.05, config=config(32, 50, [layer(wkv(2, 16, 3))]))
    folder = make_folder(small, tmp_path, {"l0.mix.w0": -7.0, "l0.mix.w2": lambda t: t * 0.1})
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 260, 5)
    other = list(toks)
    other[3] = (toks[3] + 1) % 50
    plain, without = plain_logits(cfg, w, toks), plain_logits(cfg, w, other)
    assert np.median(np.abs(plain[200:] - without[200:]).max(axis=-1)) > 0.003 * np.abs(plain).max()
    want = expected(cfg, w, toks, dtype)
    core = make_core(folder, dtype, 16, pages=20)
    check_rows(dtype, run_cut(core, "whole", toks, [260]), want, "whole")
    check_rows(dtype, run_cut(core, "cut", toks, [3, 1, 12, 16, 15, 2, 31, 110] + [1] * 70), want, "portions and decoding")


@pytest.mark.parametrize("dtype", DTYPES)
def test_sinks_carry_the_denominator(tmp_path, dtype):
    """Sinks of +4 with small scores: most of every softmax denominator is the sink (without it the plain logits move
    by much), in prompts, for the first tokens and in decoding."""
    small = dict(name="sink", seed=31, std=0.3, norm_std=0.1, config=config(32, 50, [layer(latent(3, 8, 4, 8, 12, scale=0.2, rot=(4, 1e3)))]))
    folder = make_folder(small, tmp_path, {"l0.mix.sink": lambda t: torch.tensor([4.0, 2.0, -1.0])})
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 80, 4)
    plain = plain_logits(cfg, w, toks)
    w_off = dict(w)
    w_off["l0.mix.sink"] = torch.full_like(w["l0.mix.sink"], -40.0)
    assert np.abs(plain - plain_logits(cfg, w_off, toks)).max() > 0.1 * np.abs(plain).max()
    want = expected(cfg, w, toks, dtype)
    core = make_core(folder, dtype, 8)
    check_rows(dtype, run_cut(core, "whole", toks, [80]), want, "whole")
    check_rows(dtype, run_cut(core, "cut", toks, [1, 1, 2, 30, 6] + [1] * 40), want, "portions and decoding")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_positions_at_which_the_temperature_steps(tmp_path, dtype):
    """The query temperature grows at positions every - 1, 2 every - 1, ... (the count is of position + 1): a large
    coefficient, portions that begin and end just before, at and behind those positions, and decoding across them."""
    small = dict(name="temp", seed=37, std=0.3, norm_std=0.1, config=config(32, 50, [layer(attention(2, 1, 16, scale=0.5, q_temp=(2.0, 16)))]))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 70, 6)
    plain = plain_logits(cfg, w, toks)
    flat = {**cfg, "layers": [{**cfg["layers"][0], "mixer": {k: v for k, v in cfg["layers"][0]["mixer"].items() if k != "q_temp"}}]}
    moved = np.abs(plain - plain_logits(flat, w, toks)).max(axis=-1)
    assert moved[:15].max() == 0 and moved[15] > 0.01 * np.abs(plain).max()
    want = expected(cfg, w, toks, dtype)
    core = make_core(folder, dtype, 8)
    check_rows(dtype, run_cut(core, "whole", toks, [70]), want, "whole")
    check_rows(dtype, run_cut(core, "cut", toks, [14, 1, 1, 15, 2, 14] + [1] * 23), want, "portions and decoding")


# ------------------------------------------------------------------ batches, pages and slots used again
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("small", [SMALL_A, SMALL_C], ids=["A", "C"])
def test_unequal_requests_in_one_batch_with_pages_and_slots_used_again(folders, dtype, small):
    """Seven requests of 1 to 90 tokens through two slots and a small pool of pages, portions of some beside single
    tokens of others; each request's logits equal the plain implementation's of it alone."""
    cfg, w = plain_of(folders[small["name"]])
    ps = small["page_size"]
    lengths = [33, 1, 90, 17, 64, 5, 48]
    reqs = {f"r{i}": tokens_of(cfg, n, 10 + i) for i, n in enumerate(lengths)}
    want = {r: expected(cfg, w, t, dtype) for r, t in reqs.items()}
    pages = max(14, 2 * (-(-90 // ps)) + 2)
    core = make_core(folders[small["name"]], dtype, ps, pages=pages, seqs=2)
    got = {r: [] for r in reqs}
    at = {r: 0 for r in reqs}
    waiting, live = list(reqs), []
    rng = np.random.default_rng(5)
    slots_seen = []
    while waiting or live:
        while waiting and len(live) < 2:
            r = waiting.pop(0)
            core.start_request(r)
            slots_seen.append(core.cache.slot(r))
            live.append(r)
        entries = []
        for r in live:
            left = len(reqs[r]) - at[r]
            n = 1 if (at[r] > 0 and rng.integers(2)) else int(min(left, rng.choice([1, 2, 3, 8, 21])))
            entries.append(entry(r, reqs[r][at[r]:at[r] + n]))
            at[r] += n
        logits = core.run(entries).cpu().numpy()
        k = 0
        for e in entries:
            got[e.request_id].append(logits[k:k + len(e.tokens)])
            k += len(e.tokens)
        for r in list(live):
            if at[r] == len(reqs[r]):
                core.finish_request(r)
                live.remove(r)
        core.cache.check_invariants()
    assert sorted(set(slots_seen)) == [0, 1] and len(slots_seen) == 7         # slots were used again
    assert core.cache.num_free_pages(0) == pages
    if dtype == "float32":
        for r in reqs:
            check_rows(dtype, np.concatenate(got[r]), want[r], r)
    else:       # few rows a request: the shares of rows that rounding moves far are judged over all of them
        check_rows(dtype, np.concatenate([x for r in reqs for x in got[r]]),
                   tuple(np.concatenate([want[r][k] for r in reqs]) for k in (0, 1)), "all requests")


# ------------------------------------------------------------------ long decoding, recorded steps
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "recorded"])
def test_long_decoding(folders, dtype, graphs):
    """260 decoded tokens behind a prompt of 9, over many pages; with recorded steps two requests decode side by side
    (the shorter one leaves a padded row, whose state goes to the spare slot)."""
    cfg, w = plain_of(folders["A"])
    a, b = tokens_of(cfg, 269, 6), tokens_of(cfg, 150, 7)
    want_a, want_b = expected(cfg, w, a, dtype), expected(cfg, w, b, dtype)
    core = make_core(folders["A"], dtype, SMALL_A["page_size"], pages=60, graphs=graphs)
    core.start_request("a")
    core.start_request("b")
    got_a = [core.run([entry("a", a[:9])]).cpu().numpy()]
    got_b = [core.run([entry("b", b[:30])]).cpu().numpy()]
    for i in range(9, 269):
        es = [entry("a", a[i:i + 1])]
        j = 30 + i - 9
        if j < 150:
            es.append(entry("b", b[j:j + 1]))
        out = core.run(es).cpu().numpy()
        got_a.append(out[:1])
        if j < 150:
            got_b.append(out[1:2])
    check_rows(dtype, np.concatenate(got_a), want_a, "a")
    check_rows(dtype, np.concatenate(got_b), want_b, "b")
    if graphs:
        assert core.graph_replays > 200


# ------------------------------------------------------------------ the entry point
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["A", "C"])
def test_greedy_generation_through_the_entry_point(folders, dtype, which):
    """Four prompts through ``LLM.generate`` with two slots, a small token budget (prompts are cut) and few pages, decode
    steps recorded and following each other without the host in between: in float32 every token is the plain
    implementation's argmax; in bfloat16 each token is within a margin of the plain maximum given what came before."""
    from jax_vllm_amd import LLM, SamplingParams

    small = {"A": SMALL_A, "C": SMALL_C}[which]
    cfg, w = plain_of(folders[which])
    prompts = [tokens_of(cfg, n, 30 + n) for n in (3, 41, 18, 70)]
    llm = LLM(folders[which], dtype=dtype, block_size=small["page_size"], max_num_seqs=2, max_model_len=128,
              max_num_batched_tokens=24, num_blocks=max(9, 256 // small["page_size"] + 1))
    assert llm.prewarm() > 0.0
    got = llm.generate(prompts, SamplingParams(max_new_tokens=12))
    assert [len(g) for g in got] == [12] * 4
    for p, g in zip(prompts, got):
        seq = list(p)
        for i, t in enumerate(g):
            logits = P.forward(w, cfg, seq)[-1]
            if dtype == "float32":
                assert int(torch.argmax(logits)) == t, f"token {i}: engine {t}, plain {int(torch.argmax(logits))}"
            else:
                assert float(logits.max() - logits[t]) <= 0.06 * float(logits.abs().max()), f"token {i} is far below the maximum"
            seq.append(t)


def test_command_line_runs_the_design(folders, capsys):
    from jax_vllm_amd.engine.cli import main

    cfg, w = plain_of(folders["B"])
    prompt = tokens_of(cfg, 12, 40)
    code = main(["--model-path", str(folders["B"]), "--dtype", "fp32", "--block-size", "16", "--max-model-len", "64",
                 "--max-prefill-len", "32", "--max-new-tokens", "5", "--no-prewarm", "--prompt-ids",
                 " ".join(map(str, prompt))])
    assert code == 0
    got = [int(t) for t in capsys.readouterr().out.split()]
    seq = list(prompt)
    for t in got:
        assert int(torch.argmax(P.forward(w, cfg, seq)[-1])) == t
        seq.append(t)
    assert len(got) == 5


class _Both:
    """(plain logits, plain logits with rounded products) of a request, indexed by position as one."""

    def __init__(self, pair):
        self.pair = pair

    def __getitem__(self, pos):
        return self.pair


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_with_four_slots_and_a_pool_for_the_live_requests_only(folders, dtype, tmp_path):
    """``bin/trace_run`` on a mixed schedule: nine requests of 20 to 150 tokens, at most four live, portions of some
    beside single tokens of others, some sitting a step out; the pool holds what the live requests hold at the peak, so
    pages and slots are used again; then one request whole, one with its tail decoded, one in portions down to two."""
    from tests.replay_util import Trace, compare, mixed, portions, run_trace, tail_one_by_one, whole

    cfg, w = plain_of(folders["A"])
    rng = np.random.default_rng(17)
    reqs = {f"q{i}": tokens_of(cfg, n, 50 + i) for i, n in enumerate((150, 20, 77, 64, 33, 129, 48, 90, 65))}
    trace = Trace()
    peak = mixed(trace, reqs, rng)
    whole(trace, "q0#w", reqs["q0"])
    tail_one_by_one(trace, "q2#t", reqs["q2"], tail=40)
    portions(trace, "q5#p", reqs["q5"], (2, 31, 3, 17))
    got = run_trace(folders["A"], dtype, trace, max(peak, 192), tmp_path / "out", block_size=SMALL_A["page_size"])
    want = {r: expected(cfg, w, t, dtype) for r, t in reqs.items()}
    rows_got, rows_plain, rows_rounded = [], [], []

    def collect(name, pos, got_row, want_row):
        rows_got.append(got_row)
        if dtype == "float32":
            rows_plain.append(want_row)
        else:
            rows_plain.append(want_row[0][pos])
            rows_rounded.append(want_row[1][pos])

    if dtype == "float32":
        n = compare(trace, got, want, collect)
        check_rows(dtype, np.stack(rows_got), np.stack(rows_plain), "trace")
    else:
        n = compare(trace, got, {r: _Both(v) for r, v in want.items()}, collect)
        check_rows(dtype, np.stack(rows_got), (np.stack(rows_plain), np.stack(rows_rounded)), "trace")
    assert n == sum(len(t) for t in reqs.values()) + 150 + 41 + 129


# ------------------------------------------------------------------ other sizes
@pytest.mark.parametrize("dtype", DTYPES)
def test_odd_sizes_and_heads_beyond_the_matrix_core_kernels(tmp_path, dtype):
    """A width that is no multiple of 4, a cached latent vector of 263 elements (above the matrix-core attention
    kernels: the float kernel runs in bfloat16 too), heads of 6 and 10, a decay through one channel, feed-forwards and
    experts of odd sizes, three buckets, seven q heads on one kv head."""
    small = dict(name="odd", seed=31, std=0.25, norm_std=0.2, config=config(50, 61, [
        layer(latent(2, 10, 6, 7, 257, rot=(6, 77.0)), dense(21)),
        layer(wkv(3, 6, 1), moe(5, 2, 13, shared=9, scale=0.7)),
        layer(attention(7, 1, 18, q_temp=(0.2, 1)), None),
        layer(latent(3, 5, 6, 3, 257, rot=(6, 77.0), kv_from=0), moe(3, 1, 5)),
        layer(wkv(1, 10, 9), dense(33)),
    ], bigram=(3, 1, 1), scale=1.5, mult=0.9))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 70, 8)
    want = expected(cfg, w, toks, dtype)
    core = make_core(folder, dtype, 16)
    check_rows(dtype, run_cut(core, "whole", toks, [70]), want, "whole")
    check_rows(dtype, run_cut(core, "cut", toks, [33, 2, 1, 17, 1, 1, 15]), want, "portions")


@pytest.mark.parametrize("dtype", DTYPES)
def test_wider_layers_and_a_long_prompt(tmp_path, dtype):
    """Six layers at a width of 256 with heads of 32 to 128 and cached vectors of 96 and 192 (the sizes at which the
    matrix-core attention kernels, the matrix-core expert products and the streaming products all run), a prompt of
    420 tokens: whole, in portions that end inside pages, and with a decoded tail."""
    small = dict(name="wide", seed=41, std=0.08, norm_std=0.1, config=config(256, 500, [
        layer(latent(8, 32, 32, 64, 160, scale=0.2, rot=(32, 5e4)), dense(320)),
        layer(wkv(4, 64, 32), moe(8, 2, 96, shared=64, scale=2.0)),
        layer(attention(8, 2, 64, scale=0.15, q_temp=(0.5, 128)), None),
        layer(latent(4, 64, 32, 32, 160, rot=(32, 5e4), kv_from=0), moe(16, 4, 64)),
        layer(latent(2, 16, 16, 128, 80, rot=(8, 1e4)), dense(192)),
        layer(wkv(2, 128, 8), dense(64)),
    ], bigram=(211, 31, 17), scale=0.7, mult=0.4))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 420, 9)
    want = expected(cfg, w, toks, dtype)
    core = make_core(folder, dtype, 16, pages=40)
    whole, cut = run_cut(core, "whole", toks, [420]), run_cut(core, "cut", toks, [100, 31, 2, 64, 33, 7, 129, 14] + [1] * 40)
    if dtype == "bfloat16":
        check_rows(dtype, whole, want, "whole")
        check_rows(dtype, cut, want, "portions and decoding")
        return
    # a few positions are badly conditioned (a close choice between experts, a small output in front of a norm): the
    # plain implementation in float32 is itself off there, so a row may be off by three times that on top of the bound
    own = np.abs(P.forward(P.read_weights(folder, torch.float32), cfg, toks).numpy().astype(np.float64) - want).max(axis=-1)
    scale = float(np.abs(want).max())
    for what, got in (("whole", whole), ("portions and decoding", cut)):
        err = np.abs(got.astype(np.float64) - want).max(axis=-1)
        worst = int((err - 3 * own).argmax())
        assert (err <= 3e-5 * scale + 1e-5 + 3 * own).all(), f"{what}: row {worst} is off by {err[worst]}, plain float32 by {own[worst]}"
        assert np.median(err) <= 1e-5 * scale, f"{what}: median error {np.median(err)}"


# ------------------------------------------------------------------ the kernels alone
def _dev(x, dtype=None):
    return x.to("cuda").to(dtype) if dtype is not None else x.to("cuda")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("hidden", [50, 64, 520])
def test_kernel_blends_with_the_row_before(dtype, hidden):
    """Three requests of 5, 1 and 12 rows in slots 2, 0 and 3: the first row of each blends with its slot's state row,
    which then holds the request's last row; other slots stay as they were."""
    from jax_vllm_amd.ops import kernels as K

    g = torch.Generator().manual_seed(1)
    lens, slots = [5, 1, 12], [2, 0, 3]
    n = sum(lens)
    x = torch.randn(n, hidden, generator=g).to(dtype)
    mu = torch.rand(5, hidden, generator=g)
    state = torch.randn(5, hidden, generator=g)
    cu = np.cumsum([0] + lens)
    before = torch.empty(n, hidden)
    for r, s in enumerate(slots):
        before[cu[r]] = state[s]
        before[cu[r] + 1:cu[r + 1]] = x[cu[r]:cu[r + 1] - 1].float()
    want = x.float().unsqueeze(0) + (before - x.float()).unsqueeze(0) * mu.unsqueeze(1)
    want_state = state.clone()
    for r, s in enumerate(slots):
        want_state[s] = x[cu[r + 1] - 1].float()
    st = _dev(state.clone())
    token_req = torch.repeat_interleave(torch.arange(3), torch.tensor(lens)).to(torch.int32)
    got = K.token_shift_mix(_dev(x), _dev(mu), st, _dev(torch.tensor(slots, dtype=torch.int32)),
                            _dev(torch.tensor(cu, dtype=torch.int32)), _dev(token_req))
    tol = 1e-6 if dtype == torch.float32 else 2e-2
    assert torch.allclose(got.float().cpu(), want, atol=tol, rtol=tol)
    assert torch.equal(st.cpu(), want_state)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("chunks", [False, True], ids=["steps", "chunks"])
@pytest.mark.parametrize("shape", [(3, 8, 8), (1, 80, 80), (2, 128, 128), (5, 6, 6), (2, 64, 72)])
def test_kernel_recurrence_with_a_decay_per_channel_and_a_bonus(dtype, chunks, shape):
    """Three requests (7, 1 and 100 rows: chunks that are full, short and single) that continue states of their own
    against the recurrence written out token by token; the outputs and the states that the step leaves.  Some decays
    are next to nothing (rates far above zero), some next to one."""
    from types import SimpleNamespace

    from jax_vllm_amd.ops import kernels as K

    H, d, dv = shape
    g = torch.Generator().manual_seed(2)
    lens, slots = [7, 1, 100], [1, 3, 0]
    n = sum(lens)
    r, k, v = (torch.randn(n, H * s, generator=g).to(dtype) for s in (d, d, dv))
    rate = (torch.randn(n, H * d, generator=g) * 0.5).to(dtype)
    rate[40:44] = 6.0           # these tokens wipe the state: log decays of -e^4 and below
    w0 = torch.randn(H * d, generator=g) - 2.0
    bonus = torch.randn(H * d, generator=g)
    state = torch.randn(5, H, d, dv, generator=g)
    want, want_state = torch.empty(n, H * dv, dtype=torch.float64), state.double().clone()
    cu = np.cumsum([0] + lens)
    for q, s in enumerate(slots):
        S = want_state[s]
        for t in range(cu[q], cu[q + 1]):
            rt, kt, vt = r[t].double().view(H, d), k[t].double().view(H, d), v[t].double().view(H, dv)
            wt = torch.exp(-torch.exp(rate[t].double() + w0.double())).view(H, d)
            kv = kt.unsqueeze(2) * vt.unsqueeze(1)
            want[t] = ((S + bonus.double().view(H, d, 1) * kv) * rt.unsqueeze(2)).sum(1).reshape(-1)
            S = wt.unsqueeze(2) * S + kv
        want_state[s] = S
    st = _dev(state.clone())
    plan = None
    if chunks:
        ctx = SimpleNamespace(captured=False, max_q_len=max(lens), plans={}, q_lens_host=lens, positions=st)
        plan = K.wkv_chunk_plan(ctx, d)
        assert plan is not None and plan[2] == 1 + 1 + 4
    got = K.wkv_steps(_dev(r), _dev(k), _dev(v), _dev(rate), _dev(w0), _dev(bonus), st,
                      _dev(torch.tensor(slots, dtype=torch.int32)), _dev(torch.tensor(cu, dtype=torch.int32)), H, d, dv,
                      chunk_plan=plan)
    scale = float(want.abs().max())
    assert float((got.double().cpu() - want).abs().max()) <= 2e-5 * scale
    assert float((st.double().cpu() - want_state).abs().max()) <= 2e-5 * float(want_state.abs().max())
    assert torch.equal(st[2].cpu(), state[2]) and torch.equal(st[4].cpu(), state[4])


@pytest.mark.parametrize("n", [5, 40, 300])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_kernel_router_with_a_corrected_choice_and_normed_weights(n, dtype):
    from jax_vllm_amd.ops import kernels as K

    g = torch.Generator().manual_seed(3)
    hidden, experts, top = 48, 9, 3
    x = torch.randn(n, hidden, generator=g).to(dtype)
    wr = (torch.randn(experts, hidden, generator=g) * 0.3).to(dtype)
    corr = torch.randn(experts, generator=g) * 0.3
    s = torch.sigmoid(x.double() @ wr.double().T)
    choice = torch.topk(s + corr.double(), top, dim=-1).indices
    chosen = torch.gather(s, 1, choice)
    weights = chosen / (chosen.sum(-1, keepdim=True) + 1e-20) * 1.7
    plan = K.moe_route(None, top, x=_dev(x), w_router=_dev(wr), score="sigmoid_normed", correction=_dev(corr), weight_scale=1.7)
    ids, wts = plan.ids.view(n, top).cpu().long(), plan.weights.view(n, top).cpu().double()
    # rows whose choice is not a close call
    margin = (s + corr.double()).sort(-1, descending=True).values
    clear = (margin[:, top - 1] - margin[:, top]) > 1e-4
    assert clear.float().mean() > 0.9
    assert torch.equal(ids[clear].sort(-1).values, choice[clear].sort(-1).values)
    order_got, order_want = ids.argsort(-1), choice.argsort(-1)
    assert torch.allclose(torch.gather(wts, 1, order_got)[clear], torch.gather(weights, 1, order_want)[clear], atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("shape", [(13, 5, 1, 12, 8), (300, 8, 2, 64, 16), (70, 4, 4, 96, 16)])
def test_kernel_attention_input_with_the_keys_as_values_and_a_temperature(dtype, shape):
    """q and k normed per head, q times its temperature, the k columns as projected into the value pages."""
    from jax_vllm_amd.ops import kernels as K

    n, nq, nkv, dk, page = shape
    g = torch.Generator().manual_seed(4)
    dp = K.padded_head_dim(dk, dk)
    rows = torch.randn(n, (nq + nkv) * dk + 8, generator=g).to(dtype)
    qw, kw = torch.rand(dk, generator=g) + 0.5, torch.rand(dk, generator=g) + 0.5
    positions = torch.randint(0, 100, (n,), generator=g, dtype=torch.int32)
    pages = -(-n // page) + 1
    slot = torch.randperm(pages * page, generator=g)[:n].to(torch.int32) + page       # page 0 stays the null page
    kp = torch.zeros(pages + 1, nkv, page, dp, dtype=dtype, device="cuda")
    vp = torch.zeros(pages + 1, nkv, dp, page, dtype=dtype, device="cuda")
    q = K.attn_prepare_wide(_dev(rows), None, _dev(qw), _dev(kw), 1e-5, None, 0, _dev(slot), kp, vp, page, nq, nkv, dk, dk, dp,
                            norm_per_head=True, values_are_keys=True, positions=_dev(positions), q_temperature=(0.6, 7))
    x = rows.float()
    qh, kh = x[:, :nq * dk].view(n, nq, dk), x[:, nq * dk:(nq + nkv) * dk].view(n, nkv, dk)
    norm = lambda a, wt: a / torch.sqrt((a * a).mean(-1, keepdim=True) + 1e-5) * wt      # noqa: E731
    temp = 1.0 + 0.6 * torch.log(torch.div(positions + 1, 7, rounding_mode="floor").float() + 1.0)
    want_q = norm(qh, qw) * temp.view(n, 1, 1)
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    assert torch.allclose(q.float().cpu().view(n, nq, dp)[..., :dk], want_q, atol=tol, rtol=tol)
    pg, off = (slot // page).long(), (slot % page).long()
    got_k = kp.float().cpu()[pg, :, off, :dk]
    got_v = vp.float().cpu()[pg, :, :dk, off]
    assert torch.allclose(got_k, norm(kh, kw), atol=tol, rtol=tol)
    assert torch.equal(got_v, kh.to(dtype).float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("head_dim", [40, 64, 160])
def test_kernel_attention_with_sinks(dtype, head_dim):
    """Prompt portions and single tokens of three requests over a paged cache, with one sink per q head in the
    denominator: the float kernel, and in bfloat16 the matrix-core kernels for prompts and for decoded tokens (with the
    keys of the long request shared out to several blocks)."""
    from types import SimpleNamespace

    from jax_vllm_amd.ops import kernels as K
    from jax_vllm_amd.parts import attention_backend
    from jax_vllm_amd.parts.spec import LayerMemory, StepContext

    g = torch.Generator().manual_seed(5)
    nq, nkv, page, D = 4, 2, 16, head_dim
    for q_lens, ctx_lens in (([37, 5, 1], [0, 20, 700]), ([1, 1, 1], [3, 900, 64])):
        R, n = len(q_lens), sum(q_lens)
        total = [c + q for c, q in zip(ctx_lens, q_lens)]
        width = max(-(-t // page) for t in total)
        tables = torch.zeros(R, width, dtype=torch.int32)
        nxt = 1
        for r, t in enumerate(total):
            for p in range(-(-t // page)):
                tables[r, p] = nxt
                nxt += 1
        keys = [torch.randn(t, nkv, D, generator=g) * 0.5 for t in total]
        vals = [torch.randn(t, nkv, D, generator=g) for t in total]
        kp = torch.zeros(nxt, nkv, page, D)
        vp = torch.zeros(nxt, nkv, D, page)
        for r, t in enumerate(total):
            for j in range(t):
                kp[tables[r, j // page], :, j % page] = keys[r][j]
                vp[tables[r, j // page], :, :, j % page] = vals[r][j]
        kp, vp = kp.to(dtype), vp.to(dtype)
        q = (torch.randn(n, nq * D, generator=g) * 0.5).to(dtype)
        sinks = torch.tensor([1.5, -0.5, 3.0, 0.0])
        scale = 0.3
        want = torch.empty(n, nq, D, dtype=torch.float64)
        cu = np.cumsum([0] + q_lens)
        positions, token_req = [], []
        for r in range(R):
            kk = kp.double()[tables[r].long()].permute(0, 2, 1, 3).reshape(-1, nkv, D)[:total[r]]
            vv = vp.double()[tables[r].long()].permute(0, 3, 1, 2).reshape(-1, nkv, D)[:total[r]]
            for i in range(q_lens[r]):
                pos = ctx_lens[r] + i
                positions.append(pos)
                token_req.append(r)
                for h in range(nq):
                    s = (kk[:pos + 1, h // (nq // nkv)] @ q[cu[r] + i].double().view(nq, D)[h]) * scale
                    full = torch.cat([s, sinks[h:h + 1].double()])
                    p = torch.softmax(full, 0)[:-1]
                    want[cu[r] + i, h] = p @ vv[:pos + 1, h // (nq // nkv)]
        i32 = lambda a: _dev(torch.tensor(a, dtype=torch.int32))      # noqa: E731
        ctx = StepContext(num_tokens=n, num_requests=R, positions=i32(positions), token_req=i32(token_req), cu_seqlens=i32(cu),
                          context_lens=i32(ctx_lens), slot_ids=i32([0] * R), block_tables=[_dev(tables)], slot_mappings=[None],
                          page_size=page, q_lens_host=q_lens, context_lens_host=ctx_lens, slot_ids_host=[0] * R,
                          max_q_len=max(q_lens), max_kv_len=max(total))
        att = SimpleNamespace(nq=nq, nkv=nkv, d=D, scale=scale, window=None, q_row_stride=nq * D, sinks=_dev(sinks))
        out = torch.empty(n, nq * D, dtype=dtype, device="cuda")
        attention_backend.run(att, out, _dev(q), ctx, LayerMemory(pages={"k": _dev(kp), "v": _dev(vp)}, group=0))
        tol = 2e-5 if dtype == torch.float32 else 3e-2
        assert float((out.double().cpu().view(n, nq, D) - want).abs().max()) <= tol * max(1.0, float(want.abs().max()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_kernel_latent_input_with_neighbouring_pairs_turned(dtype):
    """The cached vector [normed latent | key part with the pairs (2i, 2i + 1) turned] behind directly projected
    queries, and the queries' turned parts."""
    from jax_vllm_amd.ops import kernels as K

    g = torch.Generator().manual_seed(6)
    n, H, dim, rot, dims, rank, page = 21, 3, 8, 6, 4, 20, 8
    q_width = H * (dim + rot)
    rows = torch.randn(n, q_width + rank + rot + 5, generator=g).to(dtype)
    wkv_ = torch.rand(rank, generator=g) + 0.5
    positions = torch.randint(0, 500, (n,), generator=g, dtype=torch.int32)
    inv_freq = 1.0 / (50.0 ** (torch.arange(0, dims, 2).float() / dims))
    cos_sin = K.rope_table(_dev(positions), _dev(inv_freq))
    pages = -(-n // page) + 1
    slot = torch.randperm(pages * page, generator=g)[:n].to(torch.int32) + page
    E = rank + rot
    kp = torch.zeros(pages + 1, 1, page, E, dtype=dtype, device="cuda")
    vp = torch.zeros(pages + 1, 1, E, page, dtype=dtype, device="cuda")
    assert K.latent_prepare(_dev(rows), 0, rank, rot, dims, None, _dev(wkv_), 1e-5, cos_sin, _dev(slot), kp, vp, page,
                            kv_off=q_width, interleaved=True) is None
    qe = torch.zeros(n, H * E, dtype=dtype, device="cuda")
    K.latent_query_rope(_dev(rows), qe, H, dim, rot, dims, rank, cos_sin, interleaved=True)

    def turn(a):
        ang = positions.double().view(-1, *([1] * (a.dim() - 1))) * inv_freq.double()
        out = a.double().clone()
        u, v = a.double()[..., 0:dims:2], a.double()[..., 1:dims:2]
        out[..., 0:dims:2] = u * torch.cos(ang) - v * torch.sin(ang)
        out[..., 1:dims:2] = v * torch.cos(ang) + u * torch.sin(ang)
        return out

    x = rows.float()
    c = x[:, q_width:q_width + rank]
    want_e = torch.cat([(c / torch.sqrt((c * c).mean(-1, keepdim=True) + 1e-5) * wkv_).double(),
                        turn(x[:, q_width + rank:q_width + E])], dim=-1)
    pg, off = (slot // page).long(), (slot % page).long()
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    assert torch.allclose(kp.double().cpu()[pg, 0, off], want_e, atol=tol, rtol=tol)
    assert torch.allclose(vp.double().cpu()[pg, 0, :, off], want_e, atol=tol, rtol=tol)
    want_q = turn(x[:, :q_width].view(n, H, dim + rot)[..., dim:])
    assert torch.allclose(qe.double().cpu().view(n, H, E)[..., rank:], want_q, atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_kernel_gates_of_a_head_and_of_a_row(dtype):
    """One matrix per head under one gate per head; rows into a float share under one gate per row."""
    from jax_vllm_amd.ops import kernels as K

    g = torch.Generator().manual_seed(7)
    n, H, N, Kd = 37, 3, 10, 16
    x = torch.randn(n, H * Kd, generator=g).to(dtype)
    w = (torch.randn(H, N, Kd, generator=g) * 0.3).to(dtype)
    gates = torch.randn(n, H + 3, generator=g).to(dtype)
    y = torch.empty(n, H * N, dtype=dtype, device="cuda")
    K.head_linear(y, N, _dev(x), Kd, _dev(w), gate=_dev(gates)[:, 1:1 + H])
    want = torch.einsum("thk,hnk->thn", x.double().view(n, H, Kd), w.double()) * torch.sigmoid(gates.double()[:, 1:1 + H]).unsqueeze(-1)
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    assert torch.allclose(y.double().cpu().view(n, H, N), want, atol=tol, rtol=tol)
    for width in (50, 64):
        rows = torch.randn(n, width, generator=g).to(dtype)
        out = torch.empty(n, width, dtype=torch.float32, device="cuda")
        K.row_gate(out, _dev(rows), _dev(gates)[:, 2:3])
        assert torch.allclose(out.cpu().double(), rows.double() * torch.sigmoid(gates.double()[:, 2:3]), atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_kernel_a_sublayer_joins_the_stream_under_a_constant(dtype):
    """h += c * (rows + float shares) and the norm of the new stream in one pass; with a list of rows the stream stays."""
    from jax_vllm_amd.ops import kernels as K

    g = torch.Generator().manual_seed(8)
    for hidden in (48, 50):
        n = 19
        h = torch.randn(n, hidden, generator=g)
        y = torch.randn(n, hidden, generator=g).to(dtype)
        parts = torch.randn(3, n, hidden, generator=g)
        weight = torch.rand(hidden, generator=g) + 0.5
        new = h.double() + 0.3 * (y.double() + parts.double().sum(0))
        want = new / torch.sqrt((new * new).mean(-1, keepdim=True) + 1e-5) * weight.double()
        hd, out = _dev(h.clone()), torch.empty(n, hidden, dtype=dtype, device="cuda")
        K.postnorm_add_rmsnorm(hd, _dev(y), _dev(parts), None, 0.0, _dev(weight), out, out_eps=1e-5, plain_scale=0.3)
        tol = 1e-5 if dtype == torch.float32 else 3e-2
        assert torch.allclose(hd.double().cpu(), new, atol=1e-5, rtol=1e-5)
        assert torch.allclose(out.double().cpu(), want, atol=tol, rtol=tol)
        rows = _dev(torch.tensor([4, 0, 18], dtype=torch.int32))
        hd2, out2 = _dev(h.clone()), torch.empty(3, hidden, dtype=dtype, device="cuda")
        K.postnorm_add_rmsnorm(hd2, _dev(y), _dev(parts), None, 0.0, _dev(weight), out2, rows, out_eps=1e-5, plain_scale=0.3)
        assert torch.equal(hd2.cpu(), h)
        assert torch.allclose(out2.double().cpu(), want[[4, 0, 18]], atol=tol, rtol=tol)
