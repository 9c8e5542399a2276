"""Small Tedulorn configurations and seeded weights for the tests, and the checks that the CPU and
the GPU tests share. Sizes differ from model to model in everything that can differ: layer order,
head counts and groups, key and value sizes (also none a multiple of 16, also equal), rotations over
part of a head or none, windows and kept first tokens, blended and unblended values, decays, dense
and routed feed-forwards (with and without groups and shared expert), a layer without feed-forward,
models with and without the per-token side input."""

import json
import math
import random
from pathlib import Path

import torch
from safetensors.torch import load_file, save_file

import plain_tedulorn as plain
from helpers import make_runner, replay
from mitisun_models import CUTS, compare, row_errors  # noqa: F401  (shared by the test files)


def attention(heads, kv_heads, dim, vdim, window, keep_first, scale=None, rot=None, base=10000.0, v_mix=True):
    return {"type": "attention", "mixer": {
        "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5,
        "rot": {"base": base, "dims": dim if rot is None else rot}, "mask": {"size": window, "keep_first": keep_first},
        "v_mix": v_mix}}


def retention(heads, dim, vdim, decay, rot=None, base=10000.0):
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay),
                                           "rot": {"base": base, "dims": dim if rot is None else rot}}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit, groups=None, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if groups is not None:
        out["router"]["groups"] = {"count": groups[0], "keep": groups[1]}
    if shared is not None:
        out["shared"] = {"ff": shared[0], "limit": shared[1]}
    return out


def model(width, vocab, layers, mlps, side=None, eps=1e-5, scale=1.0):
    out = []
    for layer, mlp in zip(layers, mlps):
        layer = json.loads(json.dumps(layer))
        layer["mlp"] = mlp
        out.append(layer)
    cfg = {"architecture": "Tedulorn", "vocab": vocab, "width": width, "layers": out, "norm": {"eps": eps},
           "embedding": {"scale": scale}}
    if side is not None:
        cfg["token_side"] = {"dim": side}
    return cfg


ONE_ATTENTION = model(40, 61, [attention(4, 2, 24, 12, window=7, keep_first=2, scale=0.3, rot=8, base=1000.0)], [dense(56)],
                      side=6, scale=3.0)
ONE_RETENTION = model(48, 53, [retention(3, 20, 28, (0.9, 0.97, 0.99), rot=12)],
                      [moe(6, 2, 24, 1.2, groups=(3, 2), shared=(40, 0.8))], eps=1e-6)
MIX_A = model(64, 97, [retention(2, 16, 32, (0.95, 0.995)),
                       attention(3, 1, 32, 16, window=9, keep_first=3, v_mix=False, rot=16),
                       attention(4, 2, 16, 24, window=5, keep_first=1, base=500.0),
                       attention(2, 2, 40, 24, window=12, keep_first=0, scale=0.2, rot=20),
                       retention(4, 8, 8, (0.5, 0.9, 0.99, 1.0), rot=0)],
              [moe(8, 3, 16, 1.0, groups=(4, 2), shared=(24, 2.0)), dense(80), None, moe(4, 1, 32, 0.7), dense(48)],
              side=5, scale=2.0)
MIX_B = model(96, 130, [attention(8, 2, 16, 16, window=200, keep_first=4, base=250000.0),
                        retention(1, 48, 80, (0.98,), rot=24, base=100.0),
                        attention(6, 2, 48, 16, window=33, keep_first=40, scale=0.25)],
              [moe(5, 5, 20, 3.0, groups=(5, 5)), moe(12, 2, 24, 1.5, groups=(2, 1), shared=(16, 1.0)), dense(200)],
              eps=3e-6, scale=8.0)
MODELS = {"attention": ONE_ATTENTION, "retention": ONE_RETENTION, "A": MIX_A, "B": MIX_B}
BLOCK = {"attention": 4, "retention": 16, "A": 4, "B": 16}


def drawn_model(seed):
    """A configuration drawn from everything config.json can say: 2 to 5 layers in any order, sizes that are no
    multiples of anything (and sometimes 1), windows of one token up to longer than the prompts, kept first tokens
    from none to more than the window, groups of one expert and one group of all, layers without feed-forward."""
    rng = random.Random(seed)
    width = rng.choice([24, 36, 40, 50, 56, 64, 88, 128])
    layers, mlps = [], []
    blended = None
    for _ in range(rng.randint(2, 5)):
        if rng.random() < 0.4:
            heads = rng.randint(1, 4)
            dim = rng.choice([4, 8, 12, 16, 24, 40, 64])
            layers.append(retention(heads, dim, rng.choice([4, 8, 20, 32, 48]),
                                    [rng.choice([0.5, 0.9, 0.97, 0.995, 1.0]) for _ in range(heads)],
                                    rot=rng.choice([r for r in (0, 2, 4, 8, 12, 16, 24, 40, 64) if r <= dim]),
                                    base=rng.choice([100.0, 10000.0, 1e6])))
        else:
            kv = rng.randint(1, 3)
            dim = rng.choice([4, 8, 12, 16, 24, 40, 64])
            v_mix = rng.random() < 0.7
            vdim = rng.choice([4, 8, 20, 32, 48])
            if v_mix and blended is None:
                blended = (kv, vdim)
            elif v_mix:
                kv, vdim = blended
            layers.append(attention(kv * rng.randint(1, 3), kv, dim, vdim, window=rng.choice([1, 2, 5, 17, 64, 300]),
                                    keep_first=rng.choice([0, 1, 3, 8, 20]), scale=rng.choice([0.1, 0.3, 1.0]) * 4 / dim ** 0.5,
                                    rot=rng.choice([r for r in (0, 2, 4, 8, 12, 16, 24, 40, 64) if r <= dim]),
                                    base=rng.choice([100.0, 10000.0, 1e6]), v_mix=v_mix))
        kind = rng.random()
        if kind < 0.15:
            mlps.append(None)
        elif kind < 0.45:
            mlps.append(dense(rng.choice([24, 50, 96])))
        else:
            count = rng.choice([1, 2, 3, 4])
            per = rng.choice([1, 2, 3])
            keep = rng.randint(1, count)
            mlps.append(moe(count * per, rng.randint(1, keep * per), rng.choice([8, 20, 32]), rng.choice([0.5, 1.0, 4.0]),
                            groups=None if count == 1 and rng.random() < 0.5 else (count, keep),
                            shared=None if rng.random() < 0.4 else (rng.choice([8, 24]), rng.choice([0.5, 2.0]))))
    return model(width, rng.choice([37, 64, 101]), layers, mlps, side=rng.choice([None, 1, 4, 10]),
                 eps=rng.choice([1e-6, 1e-5, 1e-3]), scale=rng.choice([1.0, 4.0]))


def tensor_shapes(cfg):
    d, L = cfg["width"], len(cfg["layers"])
    t = {"embed": (cfg["vocab"], d), "head": (cfg["vocab"], d), "final.norm": (d,)}
    side = (cfg.get("token_side") or {}).get("dim")
    if side:
        t["side.embed"] = (cfg["vocab"], L * side)
    for i, layer in enumerate(cfg["layers"]):
        P, m, mlp = f"l{i}.", layer["mixer"], layer["mlp"]
        t[P + "norm1"] = (d,)
        p = P + "mix."
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        if layer["type"] == "attention":
            G = m["kv_heads"]
            t.update({p + "q": (H * D, d), p + "k": (G * D, d), p + "v": (G * Dv, d), p + "q.norm": (D,), p + "k.norm": (D,),
                      p + "g": (H, d), p + "o": (d, H * Dv)})
            if m.get("v_mix"):
                t[p + "vmix"] = ()
        else:
            t.update({p + "q": (H * D, d), p + "k": (H * D, d), p + "v": (H * Dv, d), p + "g": (H * Dv, d), p + "o": (d, H * Dv)})
        if mlp is not None:
            t[P + "norm2"] = (d,)
            p = P + "mlp."
            if mlp["kind"] == "dense":
                t.update({p + "up": (mlp["ff"], d), p + "down": (d, mlp["ff"])})
            else:
                E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
                t.update({p + "router": (E, d), p + "correction": (E,)})
                for e in range(E):
                    t.update({f"{p}e{e}.gate": (ff, d), f"{p}e{e}.up": (ff, d), f"{p}e{e}.down": (d, ff)})
                if mlp.get("shared"):
                    ff = mlp["shared"]["ff"]
                    t.update({p + "shared.gate": (ff, d), p + "shared.up": (ff, d), p + "shared.down": (d, ff)})
        if side:
            t.update({P + "side.gate": (side, d), P + "side.proj": (d, side), P + "side.norm": (d,)})
    return t


def random_weights(cfg, seed):
    """Weights in float32 that already hold bfloat16 values. Matrices are scaled so that every branch has results
    of order one; routers are sharp (a choice rarely hangs on the last bits), corrections of both signs."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if leaf == "vmix":
            t = 0.2 + 0.6 * torch.rand((), generator=g)
        elif leaf == "norm" and len(shape) == 1 or leaf in ("norm1", "norm2"):
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif leaf == "correction":
            t = 0.1 * torch.randn(shape, generator=g)
        elif leaf == "router":
            t = torch.randn(shape, generator=g) * (3.0 / math.sqrt(shape[-1]))
        elif name in ("embed", "side.embed"):
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


def read_folder(folder):
    folder = Path(folder)
    return json.loads((folder / "config.json").read_text()), {k: v.double() for k, v in load_file(str(folder / "model.safetensors")).items()}


def oracle(folder, prompts):
    cfg, w = read_folder(folder)
    return [plain.forward(cfg, w, p).float() for p in prompts]


def check_trace(folder, ops, prompts, steps, tol, want=None, max_rows=4, block_size=16, num_blocks=None, max_len=512, what="",
                graphs=0):
    """Replay ``steps`` through the framework's step function and compare every position with the oracle."""
    runner = make_runner(folder, ops, max_rows=max_rows, max_len=max_len, block_size=block_size, num_blocks=num_blocks)
    if graphs:
        runner.enable_graphs(graphs)
    got = replay(runner, steps)
    want = want or oracle(folder, prompts)
    for i, p in enumerate(prompts):
        compare(got[f"r{i}"], want[i], tol, f"{what} request {i}")
    assert runner.cache.open_rows == []
    return runner
