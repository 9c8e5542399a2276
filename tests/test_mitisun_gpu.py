"""Mitisun on the GPU: the HIP kernels under the framework's step function, cache manager,
scheduler and entry points, in float32 and bfloat16, against the plain implementation in
``plain_mitisun``. The same small models and cuts as on the CPU, then greedy generation through
``Engine`` (captured decode steps, steps queued ahead, rows used again) and the trace runner as a
user starts it."""

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_mitisun as plain
from helpers import make_runner, random_prompts, replay, trace_mixed, trace_tail_decode
from mitisun_models import BLOCK, CUTS, MODELS, check_trace, compare, drawn_model, row_errors, latent, mamba2, model, oracle, wkv, write_model

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]
DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# in units of the logits' spread per position
TOL = {"float32": 3e-4, "bfloat16": (0.2, 0.05)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("mitisun_gpu")
    return {name: write_model(base / name, cfg, seed=i + 1) for i, (name, cfg) in enumerate(MODELS.items())}


@pytest.fixture(scope="module")
def kernel_sets():
    from socrates_amd.kernels import HipKernels
    return {name: HipKernels(dt, DEV) for name, dt in DTYPES.items()}


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("name", list(MODELS))
def test_cuts_match_the_plain_model(folders, kernel_sets, name, cut, dtype):
    cfg = MODELS[name]
    prompts = random_prompts([3, 41, 70, 26, 1, 58], cfg["vocab"], seed=7)
    pool = dict(num_blocks=4 * (-(-72 // BLOCK[name]))) if cut == "mixed" else {}
    check_trace(folders[name], kernel_sets[dtype], prompts, CUTS[cut](prompts), TOL[dtype], block_size=BLOCK[name], max_len=128,
                what=f"{name} {cut} {dtype}", **pool)


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("seed", range(24))
def test_drawn_configurations(tmp_path, kernel_sets, seed, dtype):
    """Configurations drawn from everything config.json can say (layer order, every size, windows of one token
    and longer than the prompts, one to five taps, shared caches, layers without feed-forward), each under one
    way of cutting its requests, captured decode steps included. Such models can be touchy (a width of 24, a
    sharp softmax, a large eps): in bfloat16 a request is judged against what rounding alone does to it, which
    the stand-in kernels in bfloat16 on the CPU say (they round where the HIP kernels round): within three times
    that, per request, for the worst row and for nine rows in ten."""
    cfg = drawn_model(seed)
    folder = write_model(tmp_path / "m", cfg, seed=100 + seed)
    prompts = random_prompts([23, 1, 40, 9], cfg["vocab"], seed=seed)
    block = [2, 4, 16][seed % 3]
    runner = make_runner(folder, kernel_sets[dtype], max_rows=4, max_len=64, block_size=block)
    if seed % 2:
        runner.enable_graphs(4)
    got = replay(runner, CUTS[["mixed", "portions", "tail"][seed % 3]](prompts))
    want = oracle(folder, prompts)
    if dtype == "float32":
        for i in range(len(prompts)):
            compare(got[f"r{i}"], want[i], TOL[dtype], f"drawn {seed} {dtype} request {i}")
        return
    from torch_kernels import TorchKernels
    rounded = replay(make_runner(folder, TorchKernels(torch.bfloat16, "cpu"), max_rows=4, max_len=64, block_size=block),
                     CUTS[["mixed", "portions", "tail"][seed % 3]](prompts))
    for i in range(len(prompts)):
        mine, noise = row_errors(got[f"r{i}"], want[i]), row_errors(rounded[f"r{i}"], want[i])
        nine = max(1, int(0.9 * mine.numel()))
        assert float(mine.max()) <= 3 * float(noise.max()) + 0.03, f"drawn {seed} request {i}: {float(mine.max()):.3g} against {float(noise.max()):.3g}"
        assert float(mine.kthvalue(nine).values) <= 3 * float(noise.kthvalue(nine).values) + 0.03, f"drawn {seed} request {i}, nine rows in ten"


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_a_wider_model_with_long_prompts(tmp_path, kernel_sets, dtype):
    """Width 320, six layers, heads of 48 and 96, states of 64 and 128, a latent of 96 + 24 (padded to 128 in its
    pages), windows of 100 and 37 on one cache, prompts of up to 700 tokens: decoded at the end, mixed, and in
    portions of 2 to 200 tokens, through captured decode steps."""
    from helpers import trace_mixed, trace_portions
    cfg = model(320, 500, [latent(5, 48, 24, 40, 96, 64, window=100, scale=0.15), wkv(5, 48),
                           mamba2(6, 40, 64, groups=2, conv=3, norm_groups=2),
                           latent(7, 32, 24, 56, 96, 72, window=37, scale=0.2, kv_from=0), wkv(4, 96),
                           mamba2(4, 64, 128, groups=1, conv=4, norm_groups=1)], ff=520, limit=2.0, mult=0.7, no_ff=(4,))
    folder = write_model(tmp_path / "m", cfg, seed=5)
    prompts = random_prompts([700, 333, 64, 150], cfg["vocab"], seed=6)
    want = oracle(folder, prompts)
    tol = TOL[dtype] if dtype == "float32" else (0.2, 0.06)
    for name, steps in (("tail", trace_tail_decode(prompts, 40)), ("mixed", trace_mixed(prompts, seed=7)),
                        ("portions", trace_portions(prompts, seed=8, sizes=(2, 3, 64, 65, 128, 200)))):
        runner = make_runner(folder, kernel_sets[dtype], max_rows=4, max_len=768, block_size=16, num_blocks=4 * 48)
        runner.enable_graphs(4)
        got = replay(runner, steps)
        for i in range(len(prompts)):
            compare(got[f"r{i}"], want[i], tol, f"{name} {dtype} request {i}")


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("heads", [17, 20, 33])
def test_many_heads_on_one_cached_vector(tmp_path, kernel_sets, heads, dtype):
    """All heads of a latent-attention layer share one cached vector, one "kv head" for the attention kernels:
    more than sixteen of them, which is more than one row block of the MFMA kernels per token."""
    cfg = model(64, 60, [latent(heads, 8, 8, 8, 24, 16, window=21, scale=0.8), wkv(2, 16)], mult=0.7)
    folder = write_model(tmp_path / "m", cfg, seed=60 + heads)
    prompts = random_prompts([50, 3, 33], cfg["vocab"], seed=heads)
    for cut in ("whole", "tail", "mixed"):
        check_trace(folder, kernel_sets[dtype], prompts, CUTS[cut](prompts), TOL[dtype], block_size=16, max_len=64,
                    what=f"{heads} heads {cut} {dtype}")


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_window_edges_and_long_decoding(tmp_path, kernel_sets, dtype):
    """A window of 6 (in float32 under a sharp softmax, so the key at the edge often carries the weight;
    in bfloat16 a flat one, where every key of six counts and rounding moves little), pages of 4, 150
    tokens decoded one by one from captured steps, so the window passes over decoded tokens and pages
    behind it come back."""
    scale = 3.0 if dtype == "float32" else 0.5
    cfg = model(48, 50, [latent(2, 16, 8, 16, 24, 16, window=6, scale=scale), wkv(1, 48), mamba2(2, 24, 8)], mult=1.0)
    folder = write_model(tmp_path / "m", cfg, seed=21)
    prompts = random_prompts([160], cfg["vocab"], seed=22)
    want = oracle(folder, prompts)
    runner = make_runner(folder, kernel_sets[dtype], max_rows=2, max_len=192, block_size=4, num_blocks=8)
    runner.enable_graphs(2)
    got = replay(runner, trace_tail_decode(prompts, 150))
    compare(got["r0"], want[0], TOL[dtype], "decoded behind a window")
    # the test sees a window that is one off: the plain model with such a window is far outside the limits
    pcfg, w = plain.read_folder(folder, torch.float64)
    pcfg["layers"][0]["mixer"]["mask"]["size"] = 7
    with pytest.raises(AssertionError):
        compare(plain.forward(pcfg, w, prompts[0]).float(), want[0], TOL[dtype])


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_captured_decode_steps_equal_eager_ones(folders, kernel_sets, dtype):
    cfg = MODELS["A"]
    prompts = random_prompts([30, 45, 9], cfg["vocab"], seed=31)
    steps = trace_mixed(prompts, seed=32, max_live=3, prefill_frac=0.3)
    eager = replay(make_runner(folders["A"], kernel_sets[dtype], max_len=64, block_size=4), steps)
    runner = make_runner(folders["A"], kernel_sets[dtype], max_len=64, block_size=4)
    runner.enable_graphs(4)
    assert runner.graphs_refused is None
    captured = replay(runner, steps)
    assert runner._graphs, "no decode step was captured"
    for rid in eager:
        torch.testing.assert_close(captured[rid], eager[rid], atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("name", ["A", "wkv", "B"])
def test_greedy_generation_through_the_engine(folders, name):
    """``Engine(folder)`` finds the model class by config.json; float32 greedy tokens are the plain model's,
    with more requests than rows, so rows, states and pages are used again."""
    from socrates_amd.engine import Engine
    cfg, w = plain.read_folder(folders[name], torch.float64)
    prompts = random_prompts([5, 17, 33, 2, 21, 11], cfg["vocab"], seed=41)
    want = [plain.greedy(cfg, w, p, 8) for p in prompts]
    engine = Engine(str(folders[name]), device=DEV, dtype=torch.float32, max_batch=3, max_len=64, max_new_tokens=8,
                    block_size=BLOCK[name], chunk=16)
    assert engine.generate(prompts, max_new_tokens=8) == want
    engine.cache.check()


def test_trace_runner_on_a_model_folder(tmp_path, folders):
    cfg = MODELS["B"]
    prompts = random_prompts([70, 33, 100, 12, 64], cfg["vocab"], seed=51)
    want = oracle(folders["B"], prompts)
    steps = trace_mixed(prompts, seed=52)
    lines, wanted, fed = [], [], {}
    for n, (entries, ends) in enumerate(steps):
        lines.append(json.dumps({"step": n, "entries": [{"id": r, "tokens": t, "want": w} for r, t, w in entries], "end": ends}))
        here = []
        for r, t, w in entries:
            here.append((int(r[1:]), [fed.get(r, 0) + j for j in w]))
            fed[r] = fed.get(r, 0) + len(t)
        wanted.append(here)
    max_tokens = sum(-(-len(p) // 64) * 64 for p in sorted(prompts, key=len)[-4:])
    for dtype in DTYPES:
        out = tmp_path / dtype
        proc = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folders["B"]), "--dtype", dtype,
                               "--out", str(out), "--max-tokens", str(max_tokens)], input="\n".join(lines) + "\n",
                              capture_output=True, text=True, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert proc.stdout.split("\n")[:-1] == [f"done {i}" for i in range(len(lines))]
        for n, here in enumerate(wanted):
            rows = sum(len(pos) for _, pos in here)
            if rows:
                got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(rows, cfg["vocab"]).copy())
                compare(got, torch.cat([want[i][pos] for i, pos in here]), TOL[dtype], f"step {n} {dtype}")
