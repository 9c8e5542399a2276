"""Mitisun through the framework's step function, cache manager and scheduler, on the CPU with
the stand-in kernels, against the plain implementation in ``plain_mitisun``: every mixer alone
and in mixtures; whole prompts, token-by-token decoding, portions down to two tokens, mixed
batches in a pool so small that pages and state rows are used again; windows' edges; the
configuration and the weights' names."""

import json

import pytest
import torch

import plain_mitisun as plain
from helpers import random_prompts, replay, make_runner
from mitisun_models import BLOCK, CUTS, MODELS, check_trace, compare, drawn_model, latent, model, oracle, random_weights, write_model, wkv, mamba2
from socrates_amd.config import ConfigError, MitisunConfig, load_config
from socrates_amd.engine import StepEntry
from socrates_amd.parts import cache_needs, expected_tensors
from socrates_amd.parts.registry import PagedLatent, RowState
from torch_kernels import TorchKernels

TOL = 2e-4          # float32 stand-in kernels against the float64 oracle, in units of the logits' spread


def ops32():
    return TorchKernels(torch.float32, "cpu")


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("mitisun")
    return {name: write_model(base / name, cfg, seed=i + 1) for i, (name, cfg) in enumerate(MODELS.items())}


# ---- configuration, plan, names ---------------------------------------------------------------------
def test_plan_follows_the_configuration(folders):
    cfg = load_config(folders["A"])
    assert isinstance(cfg, MitisunConfig) and cfg.to_dict() == MODELS["A"]
    plan = cfg.plan()
    assert [s.cache for s in plan.order] == [0, 1, 2, 1, 4] and [s.write for s in plan.order] == [True, True, True, False, True]
    needs = cache_needs(plan)
    # the shared slot keeps the wider of its two readers' windows
    assert needs[1] == PagedLatent(32, 9) and needs[3] is None and isinstance(needs[0], RowState)
    assert plan.layers[3].mixer.window == 5 and plan.layers[3].mixer.keep == 9 and not plan.layers[3].mixer.own_kv
    assert plan.layers[2].ffn is None and "l2.norm2" in plan.ignorable
    names = expected_tensors(plan)
    from mitisun_models import tensor_shapes
    want = tensor_shapes(MODELS["A"])
    assert set(names) == set(want)
    assert all(names[n].fits(want[n]) for n in want)


def test_configuration_errors():
    good = MODELS["A"]
    bad = json.loads(json.dumps(good)); bad["layers"][3]["mixer"]["kv_from"] = 2
    with pytest.raises(ConfigError, match="kv_from"):
        MitisunConfig.from_dict(bad)
    bad = json.loads(json.dumps(good)); bad["layers"][3]["mixer"]["kv_rank"] = 40
    with pytest.raises(ConfigError, match="differ"):
        MitisunConfig.from_dict(bad)
    bad = json.loads(json.dumps(good)); bad["layers"][0]["type"] = "conv"
    with pytest.raises(ConfigError, match="unknown type"):
        MitisunConfig.from_dict(bad)
    bad = json.loads(json.dumps(good)); del bad["layers"][0]["mixer"]["state"]
    with pytest.raises(ConfigError, match="state"):
        MitisunConfig.from_dict(bad)
    bad = json.loads(json.dumps(good)); del bad["residual_mult"]
    with pytest.raises(ConfigError, match="residual_mult"):
        MitisunConfig.from_dict(bad)


def test_a_layer_without_feed_forward_may_store_its_unused_tensors(tmp_path):
    cfg = MODELS["A"]
    w = random_weights(cfg, 3)
    w["l2.norm2"], w["l2.rg2.b"] = torch.ones(()), torch.zeros(cfg["width"])
    folder = write_model(tmp_path / "m", cfg, 3, w)
    make_runner(folder, ops32(), max_len=32)


# ---- every mixer alone and mixtures, cut in every way -----------------------------------------------
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("name", list(MODELS))
def test_cuts_match_the_plain_model(folders, name, cut):
    cfg = MODELS[name]
    prompts = random_prompts([3, 41, 70, 26, 1, 58], cfg["vocab"], seed=7)
    if cut == "mixed":
        # a pool that cannot hold all requests at once: pages come back and are used again
        check_trace(folders[name], ops32(), prompts, CUTS[cut](prompts), TOL, block_size=BLOCK[name],
                    num_blocks=4 * (-(-72 // BLOCK[name])), max_len=128, what=f"{name} {cut}")
    else:
        check_trace(folders[name], ops32(), prompts, CUTS[cut](prompts), TOL, block_size=BLOCK[name], max_len=128,
                    what=f"{name} {cut}")


def test_a_batch_equals_each_request_alone(folders):
    """Unequal requests in one step against each alone: the same bits per position are not asked
    for, the same logits up to rounding are."""
    cfg = MODELS["B"]
    prompts = random_prompts([37, 2, 19, 64], cfg["vocab"], seed=9)
    runner = make_runner(folders["B"], ops32(), max_len=128)
    alone = []
    for p in prompts:
        row = runner.cache.open_row()
        alone.append(runner.step([StepEntry(row, p, list(range(len(p))))]))
        runner.cache.close_row(row)
    rows = [runner.cache.open_row() for _ in prompts]
    together = runner.step([StepEntry(r, p, list(range(len(p)))) for r, p in zip(rows, prompts)])
    compare(together, torch.cat(alone), 1e-5, "batch against alone")


def test_rows_and_pages_used_again_start_clean(folders):
    """A state row and pages that another request left are taken by the next: its logits are
    those of a fresh run."""
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


# ---- windows ----------------------------------------------------------------------------------------
def test_window_edges_show(tmp_path):
    """A sharp softmax (a large scale): the key just inside the window often carries the weight, so a
    window one off changes the logits by far more than the tolerance. The oracle with the window one
    larger or smaller is the proof that the test can see it."""
    w_size = 6
    cfg = model(48, 50, [latent(2, 16, 8, 16, 24, 16, window=w_size, scale=3.0)], mult=1.0)
    folder = write_model(tmp_path / "m", cfg, seed=21)
    prompts = random_prompts([60], cfg["vocab"], seed=22)
    want = oracle(folder, prompts)
    for cut in ("whole", "tail", "portions"):
        check_trace(folder, ops32(), prompts, CUTS[cut](prompts), TOL, want=want, block_size=4, max_len=64, what=f"window {cut}")
    pcfg, w = plain.read_folder(folder, torch.float64)
    for other in (w_size - 1, w_size + 1):
        pcfg["layers"][0]["mixer"]["mask"]["size"] = other
        off = plain.forward(pcfg, w, prompts[0]).float()
        with pytest.raises(AssertionError):
            compare(off[w_size - 1:], want[0][w_size - 1:], 50 * TOL)
        compare(off[:w_size - 1], want[0][:w_size - 1], TOL)       # the first tokens see everything either way


def test_two_windows_on_one_cache(folders):
    """Model A's second attention layer reads the first one's cache with a smaller window, model B's
    with a much smaller one than its writer's: pages are kept for the wider, each layer masks its own."""
    for name, n in (("A", 40), ("B", 120)):
        cfg = MODELS[name]
        prompts = random_prompts([n], cfg["vocab"], seed=23)
        runner = check_trace(folders[name], ops32(), prompts, CUTS["portions"](prompts), TOL, block_size=4, max_len=128, what=name)
        assert len(runner.cache.groups) == 1


def test_pages_behind_the_window_come_back(folders):
    cfg = MODELS["A"]
    prompts = random_prompts([100], cfg["vocab"], seed=24)
    # 100 tokens in pages of 4 would be 25 pages; a portion of up to 33 tokens behind a window of 9 needs 12
    check_trace(folders["A"], ops32(), prompts, CUTS["portions"](prompts), TOL, block_size=4, num_blocks=12, max_len=128)


def test_a_token_far_back_reaches_through_the_states(tmp_path):
    """Slow decays (a state that forgets a hundredth per token) and no attention: what the first token was still
    shows 150 tokens later, in the plain model by far more than the tolerance, and the framework carries it
    through portions of every size and through single tokens."""
    cfg = model(48, 50, [wkv(2, 24), mamba2(3, 16, 12, conv=2)], mult=1.0)
    w = random_weights(cfg, 31)
    w["l0.mix.w0"] = torch.full_like(w["l0.mix.w0"], -4.6)          # decay exp(-exp(-4.6)) = 0.99
    w["l1.mix.A_log"] = torch.full_like(w["l1.mix.A_log"], -2.3)    # rate 0.1 ...
    w["l1.mix.dt_bias"] = torch.full_like(w["l1.mix.dt_bias"], -2.2)  # ... times steps of about 0.1
    folder = write_model(tmp_path / "m", cfg, 31, w)
    prompt = random_prompts([160], cfg["vocab"], seed=32)[0]
    other = [(prompt[0] + 7) % cfg["vocab"]] + prompt[1:]
    want, moved = oracle(folder, [prompt, other])
    with pytest.raises(AssertionError):
        compare(moved[150:], want[150:], 50 * TOL)
    for cut in ("portions", "tail"):
        check_trace(folder, ops32(), [prompt], CUTS[cut]([prompt]), TOL, want=[want], max_len=192, what=f"far {cut}")


@pytest.mark.parametrize("seed", range(12))
def test_drawn_configurations(tmp_path, seed):
    cfg = drawn_model(seed)
    folder = write_model(tmp_path / "m", cfg, seed=100 + seed)
    prompts = random_prompts([23, 1, 40, 9], cfg["vocab"], seed=seed)
    block = [2, 4, 16][seed % 3]
    check_trace(folder, ops32(), prompts, CUTS[["mixed", "portions", "tail"][seed % 3]](prompts), TOL, block_size=block,
                max_len=64, what=f"drawn {seed}")


def test_long_decoding(folders):
    cfg = MODELS["B"]
    prompts = random_prompts([230], cfg["vocab"], seed=25)
    steps = [([("r0", prompts[0][:5], list(range(5)))], [])]
    steps += [([("r0", [t], [0])], []) for t in prompts[0][5:]]
    steps[-1] = (steps[-1][0], ["r0"])
    check_trace(folders["B"], ops32(), prompts, steps, TOL, max_len=256, what="225 decoded tokens")


def test_greedy_tokens_of_the_plain_model_through_the_step(folders):
    cfg, w = plain.read_folder(folders["A"], torch.float64)
    prompt = random_prompts([12], cfg["vocab"], seed=26)[0]
    want = plain.greedy(cfg, w, prompt, 10)
    runner = make_runner(folders["A"], ops32(), max_len=64, block_size=4)
    row = runner.cache.open_row()
    logits = runner.step([StepEntry(row, prompt, [len(prompt) - 1])])
    got = []
    for _ in range(10):
        got.append(int(logits[0].argmax()))
        logits = runner.step([StepEntry(row, [got[-1]], [0])])
    assert got == want
