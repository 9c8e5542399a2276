"""Typed configuration of Mitisun (``"architecture": "Mitisun"``).

A decoder whose layers differ: ``layers`` lists them, each with the ``type`` of its mixer
(``wkv``: time mixing with a matrix state; ``mamba2``: a state-space mixer; ``latent_attention``:
windowed softmax attention over one cached latent per token, which a layer may also read from
another layer's cache, ``kv_from``), the mixer's sizes, and its feed-forward (or none). Every
layer is arranged as x <- x + m * norm_b(gate(h) * branch(h)) with h = norm(x): norms with one
stored number as gain, a sigmoid gate per branch, ``residual_mult`` m. Tensor names: layer i's
start with ``l<i>.``, the mixer's with ``l<i>.mix.``, the feed-forward's with ``l<i>.mlp.``.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Tuple

from .qwen3 import ConfigError
from .specs import (BlockSpec, ClampedGLUSpec, LatentAttentionSpec, Mamba2Spec, ModelPlan, PairRopeSpec,
                    RunStep, ScalarRMSNormSpec, SigmoidGateSpec, WkvSpec)

_NAMES = (("norm1", "norm1"), ("mixer", "mix"), ("norm2", "norm2"), ("ffn", "mlp"),
          ("post_norm1", "norm1b"), ("post_norm2", "norm2b"), ("gate1", "rg1"), ("gate2", "rg2"))
_MIXER_KEYS = {
    "wkv": ("heads", "dim"),
    "mamba2": ("heads", "vdim", "state", "groups", "conv", "norm_groups"),
    "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "scale", "rot"),
}


def _positive_int(where, key, value):
    if not isinstance(value, int) or isinstance(value, bool) or value < 1:
        raise ConfigError(f"{where}: {key} must be a positive integer, found {value!r}")
    return value


@dataclass(frozen=True)
class MitisunConfig:
    vocab: int
    width: int
    layers: Tuple[dict, ...]          # as config.json lists them (validated)
    norm_eps: float
    residual_mult: float
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Mitisun"

    # ---- reading -----------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: dict) -> "MitisunConfig":
        missing = [k for k in ("vocab", "width", "layers", "norm", "residual_mult") if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks {missing} (required for Mitisun)")
        _positive_int("config", "vocab", d["vocab"])
        _positive_int("config", "width", d["width"])
        if not isinstance(d["norm"], dict) or not d["norm"].get("eps", 0) > 0:
            raise ConfigError("norm.eps must be positive")
        if not isinstance(d["layers"], (list, tuple)) or not d["layers"]:
            raise ConfigError("layers must list at least one layer")
        layers = []
        for i, layer in enumerate(d["layers"]):
            where = f"layer {i}"
            kind = layer.get("type")
            if kind not in _MIXER_KEYS:
                raise ConfigError(f"{where}: unknown type {kind!r}; known: {sorted(_MIXER_KEYS)}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"{where}: no mixer sizes")
            lacking = [k for k in _MIXER_KEYS[kind] if k not in m]
            if lacking:
                raise ConfigError(f"{where} ({kind}): mixer lacks {lacking}")
            for k in _MIXER_KEYS[kind]:
                if k not in ("scale", "rot"):
                    _positive_int(where, k, m[k])
            if kind == "latent_attention":
                rot = m["rot"]
                if not isinstance(rot, dict) or "base" not in rot or "dims" not in rot:
                    raise ConfigError(f"{where}: rot needs base and dims")
                size = (m.get("mask") or {}).get("size")
                if size is not None:
                    _positive_int(where, "mask.size", size)
                src = m.get("kv_from")
                if src is not None:
                    if not isinstance(src, int) or not 0 <= src < i:
                        raise ConfigError(f"{where}: kv_from must name an earlier layer, found {src!r}")
                    other = d["layers"][src]
                    om = other.get("mixer") or {}
                    if other.get("type") != "latent_attention" or om.get("kv_from") is not None:
                        raise ConfigError(f"{where}: kv_from {src} is not a latent-attention layer with a cache of its own")
                    if any(om.get(k) != m.get(k) for k in ("kv_rank", "rot_dim", "rot")):
                        raise ConfigError(f"{where}: latent size and rotation differ from layer {src}'s, whose cache it reads")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{where}: feed-forward kind {mlp.get('kind')!r} is not supported (dense)")
                _positive_int(where, "mlp.ff", mlp.get("ff"))
                if not mlp.get("limit", 0) > 0:
                    raise ConfigError(f"{where}: mlp.limit must be positive")
            layers.append(json.loads(json.dumps(layer)))       # a copy of plain values
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        return cls(vocab=d["vocab"], width=d["width"], layers=tuple(_freeze(x) for x in layers),
                   norm_eps=float(d["norm"]["eps"]), residual_mult=float(d["residual_mult"]),
                   eos_token_ids=eos_ids, architecture=d.get("architecture", "Mitisun"))

    @classmethod
    def from_json(cls, path) -> "MitisunConfig":
        path = Path(path)
        if path.is_dir():
            path = path / "config.json"
        return cls.from_dict(json.loads(path.read_text()))

    # ---- writing -----------------------------------------------------------------
    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "layers": [_thaw(x) for x in self.layers],
               "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult,
               "vocab": self.vocab, "width": self.width}
        if self.eos_token_ids:
            out["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return out

    # ---- the layer recipe -------------------------------------------------------------
    def _mixer(self, i, layers):
        d, eps = self.width, self.norm_eps
        layer = layers[i]
        kind, m = layer["type"], layer["mixer"]
        if kind == "wkv":
            return WkvSpec(hidden=d, n_heads=m["heads"], head_dim=m["dim"], eps=eps, decay_rank=m.get("decay_rank", 0))
        if kind == "mamba2":
            return Mamba2Spec(hidden=d, n_heads=m["heads"], head_dim=m["vdim"], state=m["state"], n_groups=m["groups"],
                              conv_taps=m["conv"], norm_groups=m["norm_groups"], eps=eps)
        writer = m.get("kv_from")
        slot_of = i if writer is None else writer
        # the cache slot keeps what the widest window of its readers still sees
        windows = [(layers[j]["mixer"].get("mask") or {}).get("size") for j in range(len(layers))
                   if layers[j]["type"] == "latent_attention"
                   and (j == slot_of or layers[j]["mixer"].get("kv_from") == slot_of)]
        keep = None if any(w is None for w in windows) else max(windows)
        return LatentAttentionSpec(
            hidden=d, n_heads=m["heads"], head_dim=m["dim"], rot_dim=m["rot_dim"], v_dim=m["vdim"],
            kv_rank=m["kv_rank"], q_rank=m["q_rank"], scale=float(m["scale"]),
            position=PairRopeSpec(dims=m["rot"]["dims"], base=float(m["rot"]["base"])), eps=eps,
            window=(m.get("mask") or {}).get("size"), keep=keep, own_kv=writer is None)

    def plan(self) -> ModelPlan:
        d, eps = self.width, self.norm_eps
        layers = [_thaw(x) for x in self.layers]
        norm = ScalarRMSNormSpec(d, eps)
        blocks, order, ignorable = [], [], []
        for i, layer in enumerate(layers):
            mlp = layer.get("mlp")
            ffn = None if mlp is None else ClampedGLUSpec(d, mlp["ff"], float(mlp["limit"]))
            blocks.append(BlockSpec(
                mixer=self._mixer(i, layers), ffn=ffn, norm1=norm, norm2=None if ffn is None else norm,
                prefix=f"l{i}.", names=_NAMES, arrangement="sandwich",
                post_norm1=norm, post_norm2=None if ffn is None else norm,
                gate1=SigmoidGateSpec(d), gate2=None if ffn is None else SigmoidGateSpec(d),
                residual_mult=self.residual_mult))
            if ffn is None:
                ignorable += [f"l{i}.norm2", f"l{i}.norm2b", f"l{i}.rg2", f"l{i}.rg2.b"]
            src = layer["mixer"].get("kv_from") if layer["type"] == "latent_attention" else None
            order.append(RunStep(layer=i, cache=i if src is None else src, write=src is None))
        return ModelPlan(
            architecture=self.architecture, vocab_size=self.vocab, hidden=d, layers=tuple(blocks),
            order=tuple(order), final_norm=norm, embedding_name="embed", final_norm_prefix="final.norm",
            head_name="head", eos_token_ids=self.eos_token_ids,
            ignorable=tuple(ignorable))

    # ---- byte and flop counts ---------------------------------------------------------
    def param_counts(self) -> dict:
        from ..parts import expected_tensors
        total = per_step = 0
        for name, decl in expected_tensors(self.plan()).items():
            n = 1
            for s in decl.shape:
                n *= max(s, 1)
            total += n
            per_step += 0 if name == "embed" else n
        return {"total": total, "read_per_step": per_step}

    def step_cache_bytes(self, batch: int, context: int, item: int) -> int:
        """Bytes of cache and state a decode step of ``batch`` requests behind ``context`` tokens reads:
        the recurrent layers' float32 states, and per attention layer the cached vectors its window sees."""
        from ..parts import cache_needs
        from ..parts.registry import PagedLatent, RowState
        plan = self.plan()
        needs = cache_needs(plan)
        total = 0
        for step in plan.order:
            need = needs[step.cache]
            if isinstance(need, RowState):
                total += 4 * need.shape[0]
            elif isinstance(need, PagedLatent):
                window = plan.layers[step.layer].mixer.window
                total += item * need.width * min(context, window or context)
        return batch * total

    def prefill_flops(self, tokens: int) -> float:
        """Multiply-adds times two of one prompt of ``tokens`` tokens from position 0: the matrices
        (every stored matrix once per token; the head at one position), attention scores and sums over
        each window, and the two recurrences (per token and head, state size times four)."""
        from ..parts import expected_tensors
        plan = self.plan()
        matrices = sum(decl.shape[0] * decl.shape[1] for name, decl in expected_tensors(plan).items()
                       if decl.kind == "matrix" and len(decl.shape) == 2 and name not in ("embed", "head") and -1 not in decl.shape)
        flops = 2.0 * tokens * matrices + 2.0 * self.vocab * self.width
        for block in plan.layers:
            m = block.mixer
            if isinstance(m, LatentAttentionSpec):
                seen = sum(min(p + 1, m.window or p + 1) for p in range(tokens))
                flops += 2.0 * seen * m.n_heads * (m.cache_width + m.kv_rank)
            elif isinstance(m, WkvSpec):
                flops += 4.0 * tokens * m.n_heads * m.head_dim * m.head_dim
            elif isinstance(m, Mamba2Spec):
                flops += 4.0 * tokens * m.n_heads * m.state * m.head_dim
        return flops


def _freeze(x):
    if isinstance(x, dict):
        return tuple(sorted((k, _freeze(v)) for k, v in x.items()))
    if isinstance(x, list):
        return ("__list__",) + tuple(_freeze(v) for v in x)
    return x


def _thaw(x):
    if isinstance(x, tuple) and x and x[0] == "__list__":
        return [_thaw(v) for v in x[1:]]
    if isinstance(x, tuple):
        return {k: _thaw(v) for k, v in x}
    return x
