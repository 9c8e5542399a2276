"""Small Mitisun configurations and seeded weights for the tests, and the checks that the CPU
and the GPU tests share. Sizes differ from model to model in everything that can differ: layer
order, head counts and sizes (also none a multiple of 16), groups, norm parts, taps, windows
(also two layers on one cache with different windows), ranks, residual multiplier, eps, a layer
without feed-forward, a rotation over part of the rotated dimensions."""

import json
import math
from pathlib import Path

import torch
from safetensors.torch import save_file

import plain_mitisun as plain
from helpers import make_runner, replay, trace_mixed, trace_portions, trace_tail_decode, trace_whole


def wkv(heads, dim):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}}


def mamba2(heads, vdim, state, groups=1, conv=4, norm_groups=1):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}}


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, window, base=10000.0, scale=None, kv_from=None, dims=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5, "rot": {"base": base, "dims": dims or rot_dim},
         "mask": {"size": window}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def model(width, vocab, layers, ff=None, limit=2.0, mult=1.0, eps=1e-5, no_ff=()):
    out = []
    for i, layer in enumerate(layers):
        layer = dict(layer)
        layer["mlp"] = None if i in no_ff else {"kind": "dense", "ff": ff or 2 * width, "limit": limit}
        out.append(layer)
    return {"architecture": "Mitisun", "vocab": vocab, "width": width, "layers": out, "norm": {"eps": eps},
            "residual_mult": mult}


# every mixer alone, then mixtures
ONE_WKV = model(48, 61, [wkv(3, 16)], mult=0.8)
ONE_MAMBA = model(40, 53, [mamba2(4, 8, 12, groups=2, conv=3, norm_groups=2)], eps=1e-6)
ONE_LATENT = model(56, 71, [latent(3, 20, 8, 12, 24, 28, window=7, scale=1.5)], mult=0.6)
MIX_A = model(64, 97, [mamba2(4, 16, 16, groups=2, conv=3, norm_groups=2),
                       latent(3, 16, 8, 24, 24, 20, window=9, scale=0.9),
                       wkv(2, 32),
                       latent(3, 16, 8, 24, 24, 36, window=5, scale=1.2, kv_from=1),
                       wkv(3, 16)], ff=96, limit=1.0, mult=0.5, no_ff=(2,))
MIX_B = model(96, 130, [wkv(4, 24),
                        latent(2, 40, 12, 40, 52, 30, window=200, base=500.0, dims=8),
                        mamba2(6, 16, 20, groups=1, conv=2, norm_groups=1),
                        latent(5, 16, 12, 16, 52, 48, window=33, base=500.0, dims=8, kv_from=1)],
              ff=200, limit=3.0, mult=1.0, eps=3e-6)
MODELS = {"wkv": ONE_WKV, "mamba2": ONE_MAMBA, "latent": ONE_LATENT, "A": MIX_A, "B": MIX_B}
BLOCK = {"wkv": 16, "mamba2": 16, "latent": 4, "A": 4, "B": 16}


def drawn_model(seed):
    """A configuration drawn from everything config.json can say: 2 to 6 layers in any order, sizes that are
    no multiples of anything, windows of one token up to longer than the prompts, one to five taps, a layer
    now and then without feed-forward, attention layers that read an earlier one's cache."""
    import random
    rng = random.Random(seed)
    width = rng.choice([24, 40, 56, 64, 88, 128])
    layers, writers, no_ff = [], [], []
    for i in range(rng.randint(2, 6)):
        kind = rng.choice(["wkv", "mamba2", "latent", "latent"])
        if kind == "wkv":
            layers.append(wkv(rng.randint(1, 5), rng.choice([8, 12, 16, 24, 40, 64])))
            layers[-1]["mixer"]["decay_rank"] = rng.choice([1, 3, 8, 20])
        elif kind == "mamba2":
            groups = rng.choice([1, 2, 3])
            layers.append(mamba2(groups * rng.randint(1, 3), rng.choice([4, 8, 20, 32]), rng.choice([4, 8, 16, 24, 40, 64]),
                                 groups=groups, conv=rng.randint(1, 5), norm_groups=1))
            m = layers[-1]["mixer"]
            m["norm_groups"] = rng.choice([g for g in (1, 2, 3, 4) if (m["heads"] * m["vdim"]) % g == 0])
        else:
            window = rng.choice([1, 2, 5, 17, 64, 300])
            if writers and rng.random() < 0.5:
                j = rng.choice(writers)
                src = layers[j]["mixer"]
                layers.append(latent(rng.randint(1, 6), rng.choice([4, 8, 16, 24, 48]), src["rot_dim"], rng.choice([4, 8, 20, 32]),
                                     src["kv_rank"], rng.choice([4, 12, 32]), window, base=src["rot"]["base"],
                                     scale=rng.choice([0.3, 1.0, 2.5]), kv_from=j, dims=src["rot"]["dims"]))
            else:
                rot_dim = rng.choice([2, 4, 6, 8, 16, 32])
                layers.append(latent(rng.randint(1, 6), rng.choice([4, 8, 16, 24, 48]), rot_dim, rng.choice([4, 8, 20, 32]),
                                     rng.choice([8, 12, 24, 40, 64, 100]), rng.choice([4, 12, 32]), window,
                                     base=rng.choice([100.0, 10000.0, 250000.0]), scale=rng.choice([0.3, 1.0, 2.5]),
                                     dims=rng.choice([d for d in (2, 4, 6, 8, 16, 32) if d <= rot_dim])))
                writers.append(i)
        if rng.random() < 0.2:
            no_ff.append(i)
    return model(width, rng.choice([37, 64, 101]), layers, ff=rng.choice([24, 50, 96]), limit=rng.choice([0.5, 2.0, 6.0]),
                 mult=rng.choice([0.3, 0.7, 1.0]), eps=rng.choice([1e-6, 1e-5, 1e-3]), no_ff=tuple(no_ff))


def tensor_shapes(cfg):
    d = cfg["width"]
    t = {"embed": (cfg["vocab"], d), "head": (cfg["vocab"], d), "final.norm": ()}
    for i, layer in enumerate(cfg["layers"]):
        L, m = f"l{i}.", layer["mixer"]
        t.update({L + "norm1": (), L + "norm1b": (), L + "rg1": (d, d), L + "rg1.b": (d,)})
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            t.update({L + "norm2": (), L + "norm2b": (), L + "rg2": (d, d), L + "rg2.b": (d,),
                      L + "mlp.gate": (ff, d), L + "mlp.up": (ff, d), L + "mlp.down": (d, ff)})
        p = L + "mix."
        if layer["type"] == "wkv":
            C, rank = m["heads"] * m["dim"], m.get("decay_rank", 6)
            t.update({p + "mu." + s: (d,) for s in "rkvgw"})
            t.update({p + s: (C, d) for s in "rkvg"})
            t.update({p + "w1": (rank, d), p + "w2": (C, rank), p + "w0": (C,), p + "u": (m["heads"], m["dim"]),
                      p + "norm": (C,), p + "o": (d, C)})
        elif layer["type"] == "mamba2":
            H, inner = m["heads"], m["heads"] * m["vdim"]
            C = inner + 2 * m["groups"] * m["state"]
            t.update({p + "in": (inner + C + H, d), p + "conv": (C, m["conv"]), p + "conv.b": (C,), p + "dt_bias": (H,),
                      p + "A_log": (H,), p + "D": (H,), p + "norm": (inner,), p + "o": (d, inner)})
        else:
            H, R = m["heads"], m["kv_rank"]
            t.update({p + "dq": (m["q_rank"], d), p + "dq.norm": (m["q_rank"],), p + "uq": (H * (m["dim"] + m["rot_dim"]), m["q_rank"]),
                      p + "uk": (H * m["dim"], R), p + "uv": (H * m["vdim"], R), p + "o": (d, H * m["vdim"])})
            if m.get("kv_from") is None:
                t.update({p + "dkv": (R + m["rot_dim"], d), p + "dkv.norm": (R,)})
    return t


def random_weights(cfg, seed):
    """Weights in float32 that already hold bfloat16 values. Matrices are scaled so that every
    branch has results of order one; blends, decays, gains and biases are spread widely."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if shape == ():
            t = 0.5 + torch.rand((), generator=g)
        elif name.endswith("norm") and len(shape) == 1:
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif ".mu." in name:
            t = torch.rand(shape, generator=g)
        elif leaf in ("w0", "A_log", "dt_bias", "b", "D", "u"):
            t = torch.randn(shape, generator=g)
        elif leaf == "conv":
            t = torch.randn(shape, generator=g) * 0.5
        elif name in ("embed",):
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.5 / math.sqrt(shape[-1]))
        out[name] = t.to(torch.bfloat16).float()
    return out


def write_model(folder, cfg, seed, weights=None):
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    weights = weights if weights is not None else random_weights(cfg, seed)
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in weights.items()}, str(folder / "model.safetensors"))
    return folder


def oracle(folder, prompts):
    cfg, w = plain.read_folder(folder, torch.float64)
    return [plain.forward(cfg, w, p).float() for p in prompts]


def row_errors(got, want):
    """Per row: the difference of the logits, mean taken off, root mean square over the vocabulary, in units of
    the row's spread."""
    got, want = got.double(), want.double()
    d = (got - got.mean(-1, keepdim=True)) - (want - want.mean(-1, keepdim=True))
    return d.pow(2).mean(-1).sqrt() / want.std(-1)


def compare(got, want, tol, what=""):
    """Logits with their mean taken off (a shift of all logits changes no choice), by rows, in units of
    the row's spread. ``tol``: a limit for every row, or (limit for every row, limit that nine rows in
    ten keep): rounding to bfloat16 moves a row here and there by several times the typical error,
    a fault of a window, a state or a page moves most rows by far more."""
    got, want = got.double(), want.double()
    d = (got - got.mean(-1, keepdim=True)) - (want - want.mean(-1, keepdim=True))
    err = d.pow(2).mean(-1).sqrt() / want.std(-1)
    worst = int(err.argmax())
    top, usual = tol if isinstance(tol, tuple) else (tol, tol)
    assert float(err.max()) <= top, f"{what}: row {worst} differs by {float(err.max()):.3g} of the logits' spread (limit {top})"
    if err.numel() >= 10:
        nine_in_ten = float(err.kthvalue(int(0.9 * err.numel())).values)
        assert nine_in_ten <= usual, f"{what}: one row in ten differs by {nine_in_ten:.3g} or more (limit {usual})"


def check_trace(folder, ops, prompts, steps, tol, want=None, max_rows=4, block_size=16, num_blocks=None, max_len=512, what=""):
    """Replay ``steps`` through the framework's step function and compare every position with the oracle."""
    runner = make_runner(folder, ops, max_rows=max_rows, max_len=max_len, block_size=block_size, num_blocks=num_blocks)
    got = replay(runner, steps)
    want = want or oracle(folder, prompts)
    for i, p in enumerate(prompts):
        compare(got[f"r{i}"], want[i], tol, f"{what} request {i}")
    assert runner.cache.open_rows == []
    return runner


CUTS = {"whole": lambda p: trace_whole(p), "tail": lambda p: trace_tail_decode(p, 24),
        "portions": lambda p: trace_portions(p, seed=5, sizes=(2, 3, 5, 7, 16, 17, 33)),
        "mixed": lambda p: trace_mixed(p, seed=6)}
