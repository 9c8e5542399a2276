"""Tedulorn through the framework's step function, cache manager and scheduler, on the CPU with the
stand-in kernels, against the plain implementation in ``plain_tedulorn``: every mechanism alone and in
mixtures; whole prompts, token-by-token decoding, portions down to two tokens, mixed batches in a pool so
small that pages and state rows are used again; the edges of the window and of the kept first tokens;
the added weight of the softmax; the choice of experts; the configuration and the weights' names."""

import json

import pytest
import torch

import plain_tedulorn as plain
from helpers import make_runner, random_prompts
from tedulorn_models import (BLOCK, CUTS, MODELS, attention, check_trace, compare, dense, drawn_model, model, moe, oracle,
                             random_weights, read_folder, retention, tensor_shapes, write_model)
from socrates_amd.config import ConfigError, load_config
from socrates_amd.config.tedulorn import TedulornConfig
from socrates_amd.engine import StepEntry
from socrates_amd.parts import cache_needs, expected_tensors
from socrates_amd.parts.registry import PagedKV, RowState
from torch_kernels import TorchKernels

TOL = 2e-4          # float32 stand-in kernels against the float64 oracle, in units of the logits' spread


def ops32():
    return TorchKernels(torch.float32, "cpu")


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("tedulorn")
    return {name: write_model(base / name, cfg, seed=i + 1) for i, (name, cfg) in enumerate(MODELS.items())}


# ---- configuration, plan, names ---------------------------------------------------------------------
def test_plan_follows_the_configuration(folders):
    cfg = load_config(folders["A"])
    assert isinstance(cfg, TedulornConfig) and cfg.to_dict() == MODELS["A"]
    plan = cfg.plan()
    needs = cache_needs(plan)
    assert isinstance(needs[0], RowState) and needs[0].shape == (2 * 16 * 32,)
    # keys of 32 and values of 16 share pools of 32; keys of 40 need 48
    assert needs[1] == PagedKV(1, 32, 9, 3) and needs[2] == PagedKV(2, 32, 5, 1) and needs[3] == PagedKV(2, 48, 12, 0)
    blends = [getattr(b.mixer, "value_blend", None) for b in plan.layers]
    assert blends == [None, None, "first", "later", None]
    assert plan.layers[2].ffn is None and "l2.norm2" in plan.ignorable and "l1.mix.vmix" in plan.ignorable
    assert plan.embedding_scale == 2.0
    names = expected_tensors(plan)
    want = tensor_shapes(MODELS["A"])
    assert set(names) == set(want)
    assert all(names[n].fits(want[n]) for n in want)
    # a model without the side input has no table
    assert "side.embed" not in expected_tensors(load_config(folders["B"]).plan())


def test_configuration_errors():
    good = MODELS["A"]

    def broken(change):
        bad = json.loads(json.dumps(good))
        change(bad)
        return bad
    with pytest.raises(ConfigError, match="unknown type"):
        TedulornConfig.from_dict(broken(lambda c: c["layers"][0].update(type="conv")))
    with pytest.raises(ConfigError, match="decay"):
        TedulornConfig.from_dict(broken(lambda c: c["layers"][0]["mixer"].update(decay=[0.5])))
    with pytest.raises(ConfigError, match="blended"):
        TedulornConfig.from_dict(broken(lambda c: c["layers"][3]["mixer"].update(vdim=8)))
    with pytest.raises(ConfigError, match="groups"):
        TedulornConfig.from_dict(broken(lambda c: c["layers"][0]["mlp"]["router"].update(top=5)))
    with pytest.raises(ConfigError, match="rot.dims"):
        TedulornConfig.from_dict(broken(lambda c: c["layers"][1]["mixer"]["rot"].update(dims=34)))
    with pytest.raises(ConfigError, match="kv heads"):
        TedulornConfig.from_dict(broken(lambda c: c["layers"][1]["mixer"].update(kv_heads=2)))
    with pytest.raises(ConfigError, match="lacks"):
        TedulornConfig.from_dict(broken(lambda c: c.pop("norm")))


# ---- each mechanism of the stand-in kernel set against the plain function ---------------------------------
def test_the_choice_of_experts():
    """Negative choice scores, groups whose best expert decides, experts of dropped groups that would
    otherwise win: the stand-in's choice and weights are the plain function's."""
    g = torch.Generator().manual_seed(3)
    for E, top, count, keep in ((12, 3, 4, 2), (6, 2, 3, 1), (8, 8, 2, 2), (5, 1, 5, 2), (9, 4, 1, 1)):
        z = torch.randn(50, E, generator=g, dtype=torch.float64) * 2
        corr = torch.randn(E, generator=g, dtype=torch.float64) * 0.3 - 0.2
        h = torch.eye(E, dtype=torch.float64)
        want = plain.route(z, {"router": h, "correction": corr}, {"top": top, "groups": {"count": count, "keep": keep}})
        idx, w = TorchKernels(torch.float64, "cpu", acc=torch.float64).moe_route(z, corr, top, count, keep)
        got = torch.zeros_like(want).scatter_(1, idx.long(), w)
        assert torch.allclose(got, want, atol=1e-12)
        assert (want > 0).sum(-1).eq(top).all()
        if keep < count and top > 1:
            # somewhere an expert of a dropped group has a better choice score than a chosen one
            free = (torch.softmax(z, -1) + corr).topk(top, dim=-1).indices
            assert (want.gather(1, free) == 0).any()


def test_the_added_weight_and_the_kept_first_tokens_show(tmp_path):
    """A sharp softmax: the key just inside the window or among the kept first tokens often carries the
    weight, so a window or a count one off moves the logits by far more than the tolerance, and so does
    a softmax without the added weight. The plain model with the constants changed is the proof that the
    test can see each; the framework matches the unchanged one under every cut, in prompts and decoding."""
    size, keep = 6, 3
    cfg = model(48, 50, [attention(2, 1, 16, 8, window=size, keep_first=keep, scale=2.0, rot=8)], [dense(64)], side=4)
    folder = write_model(tmp_path / "m", cfg, seed=21)
    prompts = random_prompts([60], cfg["vocab"], seed=22)
    want = oracle(folder, prompts)
    for cut in ("whole", "tail", "portions"):
        check_trace(folder, ops32(), prompts, CUTS[cut](prompts), TOL, want=want, block_size=4, max_len=64, what=f"edges {cut}")
    pcfg, w = read_folder(folder)
    mask = pcfg["layers"][0]["mixer"]["mask"]
    for key, other in (("size", size - 1), ("size", size + 1), ("keep_first", keep - 1), ("keep_first", keep + 1)):
        was, mask[key] = mask[key], other
        off = plain.forward(pcfg, w, prompts[0]).float()
        mask[key] = was
        with pytest.raises(AssertionError):
            compare(off[size + keep:], want[0][size + keep:], 50 * TOL)
        compare(off[:size - 1], want[0][:size - 1], TOL)           # the first tokens see everything either way
    # without the added weight the weights of one key sum to one: the very first token shows it
    q = torch.randn(1, 5, dtype=torch.float64)
    assert float(torch.softmax(q, -1).sum()) == pytest.approx(1.0)
    lone = plain.forward(pcfg, w, prompts[0][:1])
    W = plain.sub(w, "l0.mix.")
    h = plain.rms(w["embed"][prompts[0][:1]] * pcfg["embedding"]["scale"], pcfg["norm"]["eps"]) * w["l0.norm1"]
    y, _ = plain.attention(h, W, pcfg["layers"][0]["mixer"], pcfg["norm"]["eps"], None)
    v = (h @ W["v"].T).repeat_interleave(2, dim=1) * torch.sigmoid(h @ W["g"].T).repeat_interleave(8, dim=1)
    assert not torch.allclose(y, v @ W["o"].T, rtol=1e-3) and lone.shape == (1, 50)


# ---- every mixer alone and mixtures, cut in every way -----------------------------------------------
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("name", list(MODELS))
def test_cuts_match_the_plain_model(folders, name, cut):
    cfg = MODELS[name]
    prompts = random_prompts([3, 41, 70, 26, 1, 58], cfg["vocab"], seed=7)
    pool = {}
    if cut == "mixed":
        # a pool that cannot hold all requests at once: pages come back and are used again
        pool = dict(num_blocks=4 * (-(-72 // BLOCK[name])))
    check_trace(folders[name], ops32(), prompts, CUTS[cut](prompts), TOL, block_size=BLOCK[name], max_len=128,
                what=f"{name} {cut}", **pool)


def test_a_batch_equals_each_request_alone(folders):
    cfg = MODELS["A"]
    prompts = random_prompts([37, 2, 19, 64], cfg["vocab"], seed=9)
    runner = make_runner(folders["A"], ops32(), max_len=128)
    alone = []
    for p in prompts:
        row = runner.cache.open_row()
        alone.append(runner.step([StepEntry(row, p, list(range(len(p))))]))
        runner.cache.close_row(row)
    rows = [runner.cache.open_row() for _ in prompts]
    together = runner.step([StepEntry(r, p, list(range(len(p)))) for r, p in zip(rows, prompts)])
    compare(together, torch.cat(alone), 1e-5, "batch against alone")


def test_rows_and_pages_used_again_start_clean(folders):
    """A state row and pages that another request left are taken by the next: its logits are those of a
    fresh run (the retention state is cleared, the kept first pages are the new request's own)."""
    cfg = MODELS["A"]
    a, b = random_prompts([50, 33], cfg["vocab"], seed=11)
    runner = make_runner(folders["A"], ops32(), max_rows=1, max_len=64, block_size=4, num_blocks=16)
    want = oracle(folders["A"], [b])[0]
    for first in (a, b, a):
        row = runner.cache.open_row()
        runner.step([StepEntry(row, first, [])])
        runner.cache.close_row(row)
    row = runner.cache.open_row()
    assert row == 0
    got = torch.cat([runner.step([StepEntry(row, b[:20], list(range(20)))]), runner.step([StepEntry(row, b[20:], list(range(13)))])])
    compare(got, want, TOL, "a row used again")


def test_pages_behind_the_window_come_back_but_the_first_stay(folders):
    """120 tokens in pages of 4 would be 30 pages per layer; behind windows of at most 12 tokens with at most
    3 kept first ones, a pool of 14 serves portions of up to 33 tokens, and the page of the kept first tokens
    is still the row's at the end."""
    cfg = MODELS["A"]
    prompts = random_prompts([120], cfg["vocab"], seed=24)
    runner = make_runner(folders["A"], ops32(), max_rows=1, max_len=128, block_size=4, num_blocks=14)
    want = oracle(folders["A"], prompts)[0]
    row = runner.cache.open_row()
    got, t = [], 0
    for n in [33, 2, 17, 1, 1, 30, 5, 31]:
        got.append(runner.step([StepEntry(row, prompts[0][t:t + n], list(range(n)))]))
        t += n
        runner.cache.check()
    assert t == 120
    compare(torch.cat(got), want, TOL, "a small pool")
    kept = [g for g in runner.cache.groups if g.kept_blocks]
    assert kept and all(g.host_table[row, 0] != 0 and g.first_live[row] > g.kept_blocks for g in kept)
    none_kept = [g for g in runner.cache.groups if not g.kept_blocks]
    assert none_kept and all(g.host_table[row, 0] == 0 for g in none_kept)
    runner.cache.close_row(row)
    runner.cache.check()
    assert all(g.allocator.n_free == 14 for g in runner.cache.groups)


def test_a_token_far_back_reaches_through_the_state(tmp_path):
    """A slow decay and no attention: what the first token was still shows 150 tokens later, in the plain
    model by far more than the tolerance, and the framework carries it through portions and single tokens."""
    cfg = model(48, 50, [retention(2, 24, 16, (0.995, 1.0), rot=24), retention(3, 8, 20, (0.99, 0.98, 0.999), rot=4)],
                [dense(64), None])
    folder = write_model(tmp_path / "m", cfg, 31)
    prompt = random_prompts([160], cfg["vocab"], seed=32)[0]
    other = [(prompt[0] + 7) % cfg["vocab"]] + prompt[1:]
    want, moved = oracle(folder, [prompt, other])
    with pytest.raises(AssertionError):
        compare(moved[150:], want[150:], 50 * TOL)
    for cut in ("portions", "tail"):
        check_trace(folder, ops32(), [prompt], CUTS[cut]([prompt]), TOL, want=[want], max_len=192, what=f"far {cut}")


def test_a_far_key_among_many(tmp_path):
    """No window to speak of (longer than the prompt), 200 keys, and one query-key pair made to stand out: the
    key matrix is the query matrix behind a map that sends the input of the token at position 3 to that of the
    token at position 190, so that key is what position 190 looks at, across page borders, in a prompt and
    decoded. Changing the token at position 3 moves the logits at 190 by far more than the tolerance."""
    cfg = model(32, 40, [attention(1, 1, 16, 16, window=500, keep_first=0, scale=1.5, rot=0)], [None])
    w = random_weights(cfg, 41)
    prompt = [t % 38 for t in random_prompts([200], cfg["vocab"], seed=42)[0]]
    prompt[3], prompt[190] = 38, 39                        # two tokens that appear nowhere else
    h = plain.rms(w["embed"][[38, 39]].double() * cfg["embedding"]["scale"], cfg["norm"]["eps"]) * w["l0.norm1"].double()
    turn = torch.eye(32, dtype=torch.float64) + torch.outer(h[1] - h[0], h[0]) / h[0].dot(h[0])
    w["l0.mix.k"] = (w["l0.mix.q"].double() @ turn).float()
    folder = write_model(tmp_path / "m", cfg, 41, w)
    want = oracle(folder, [prompt])
    moved = oracle(folder, [[1 if i == 3 else t for i, t in enumerate(prompt)]])
    with pytest.raises(AssertionError):
        compare(moved[0][190:191], want[0][190:191], 50 * TOL)
    compare(moved[0][4:190], want[0][4:190], 0.2)          # elsewhere that key is one among many
    for cut in ("whole", "tail", "portions"):
        check_trace(folder, ops32(), [prompt], CUTS[cut]([prompt]), TOL, want=want, block_size=16, max_len=256, what=f"far key {cut}")


@pytest.mark.parametrize("seed", range(12))
def test_drawn_configurations(tmp_path, seed):
    cfg = drawn_model(seed)
    folder = write_model(tmp_path / "m", cfg, seed=100 + seed)
    prompts = random_prompts([23, 1, 40, 9], cfg["vocab"], seed=seed)
    block = [2, 4, 16][seed % 3]
    # (such models can be touchy in float32: a sharp softmax, a width of 24, a decay of one; a fault is larger by far)
    check_trace(folder, ops32(), prompts, CUTS[["mixed", "portions", "tail"][seed % 3]](prompts), 5 * TOL, block_size=block,
                max_len=64, what=f"drawn {seed}")


def test_long_decoding(folders):
    """225 tokens one by one: the windows pass over decoded tokens, pages come back, the state runs on."""
    cfg = MODELS["B"]
    prompts = random_prompts([230], cfg["vocab"], seed=25)
    steps = [([("r0", prompts[0][:5], list(range(5)))], [])]
    steps += [([("r0", [t], [0])], []) for t in prompts[0][5:]]
    steps[-1] = (steps[-1][0], ["r0"])
    check_trace(folders["B"], ops32(), prompts, steps, TOL, max_len=256, what="225 decoded tokens")


def test_greedy_generation_through_the_engine(folders):
    """The framework's own entry point and scheduler over this model: more requests than rows, prompts cut
    into portions, rows used again; the tokens are the plain model's greedy ones."""
    from socrates_amd.engine import Engine
    cfg, w = read_folder(folders["A"])
    prompts = random_prompts([12, 3, 29, 7, 18], cfg["vocab"], seed=26)
    want = [plain.greedy(cfg, w, p, 6) for p in prompts]
    runner = make_runner(folders["A"], ops32(), max_rows=3, max_len=64, block_size=4)
    engine = Engine(runner, device="cpu", dtype=torch.float32, compile=False, max_batch=3, max_len=64, max_new_tokens=6,
                    block_size=4, chunk=8)
    assert engine.generate(prompts, max_new_tokens=6) == want
