"""Typed configuration of Tedulorn (``"architecture": "Tedulorn"``).

A decoder whose layers differ: ``layers`` lists them, each with the ``type`` of its mixer
(``attention``: grouped-query softmax attention over a window that keeps the first tokens visible,
with one more weight of score 0 in the softmax, values blended with the first such layer's and a
gate per head; ``retention``: linear attention with a fixed decay per head), the mixer's sizes, and
its feed-forward (``dense``: squared relu; ``moe``: routed experts chosen among groups, beside a
shared one; or none). Layers are pre-norm; where ``token_side`` is given, every layer ends with an
input that depends on the token alone. Tensor names: layer i's start with ``l<i>.``, the mixer's
with ``l<i>.mix.``, the feed-forward's with ``l<i>.mlp.``, the side input's with ``l<i>.side.``.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Optional, Tuple

from .mitisun import _freeze, _positive_int, _thaw
from .qwen3 import ConfigError
from .specs import (BlockSpec, ClampedGLUSpec, GatedWindowAttentionSpec, ModelPlan, ReluSquaredSpec, RetentionSpec,
                    RMSNormSpec, RopeSpec, RoutedExpertsSpec, RunStep, TokenSideSpec)

_NAMES = (("norm1", "norm1"), ("mixer", "mix"), ("norm2", "norm2"), ("ffn", "mlp"), ("side", "side"))
_MIXER_KEYS = {
    "attention": ("heads", "kv_heads", "dim", "vdim", "scale", "rot", "mask"),
    "retention": ("heads", "dim", "vdim", "decay", "rot"),
}
_INT_KEYS = ("heads", "kv_heads", "dim", "vdim")


def _number(where, key, value, positive=True):
    if isinstance(value, bool) or not isinstance(value, (int, float)) or (positive and not value > 0):
        raise ConfigError(f"{where}: {key} must be a {'positive ' if positive else ''}number, found {value!r}")
    return float(value)


def _rotation(where, rot, dim):
    if not isinstance(rot, dict) or "base" not in rot or "dims" not in rot:
        raise ConfigError(f"{where}: rot needs base and dims")
    dims = rot["dims"]
    if not isinstance(dims, int) or isinstance(dims, bool) or dims < 0 or dims % 2 or dims > dim:
        raise ConfigError(f"{where}: rot.dims must be even and at most the head size {dim}, found {dims!r}")
    _number(where, "rot.base", rot["base"])


def _glu(where, d, what):
    if not isinstance(d, dict):
        raise ConfigError(f"{where}: {what} needs ff and limit")
    _positive_int(where, f"{what}.ff", d.get("ff"))
    _number(where, f"{what}.limit", d.get("limit"))


@dataclass(frozen=True)
class TedulornConfig:
    vocab: int
    width: int
    layers: Tuple[tuple, ...]         # as config.json lists them (validated, frozen)
    norm_eps: float
    embedding_scale: float
    side_dim: Optional[int]
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Tedulorn"

    # ---- reading -----------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: dict) -> "TedulornConfig":
        missing = [k for k in ("vocab", "width", "layers", "norm") if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks {missing} (required for Tedulorn)")
        _positive_int("config", "vocab", d["vocab"])
        _positive_int("config", "width", d["width"])
        if not isinstance(d["norm"], dict) or not d["norm"].get("eps", 0) > 0:
            raise ConfigError("norm.eps must be positive")
        if not isinstance(d["layers"], (list, tuple)) or not d["layers"]:
            raise ConfigError("layers must list at least one layer")
        scale = 1.0
        if d.get("embedding") is not None:
            scale = _number("config", "embedding.scale", (d["embedding"] or {}).get("scale", 1.0))
        side = d.get("token_side")
        side_dim = None
        if side is not None:
            side_dim = _positive_int("config", "token_side.dim", (side or {}).get("dim"))
        blended = None                        # the sizes of the first layer whose values are blended
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
            for k in _INT_KEYS:
                if k in _MIXER_KEYS[kind]:
                    _positive_int(where, k, m[k])
            _rotation(where, m["rot"], m["dim"])
            if kind == "attention":
                _number(where, "scale", m["scale"])
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"{where}: {m['heads']} heads do not divide into {m['kv_heads']} kv heads")
                mask = m["mask"]
                if mask is not None:
                    if not isinstance(mask, dict):
                        raise ConfigError(f"{where}: mask needs size and keep_first")
                    _positive_int(where, "mask.size", mask.get("size"))
                    kf = mask.get("keep_first", 0)
                    if not isinstance(kf, int) or isinstance(kf, bool) or kf < 0:
                        raise ConfigError(f"{where}: mask.keep_first must be a whole number, not negative, found {kf!r}")
                if m.get("v_mix"):
                    sizes = (m["kv_heads"], m["vdim"])
                    if blended is None:
                        blended = sizes
                    elif blended != sizes:
                        raise ConfigError(f"{where}: values of {sizes[0]} x {sizes[1]} cannot be blended with the first "
                                          f"blended layer's {blended[0]} x {blended[1]}")
            else:
                decay = m["decay"]
                if not isinstance(decay, (list, tuple)) or len(decay) != m["heads"]:
                    raise ConfigError(f"{where}: decay lists one number per head ({m['heads']})")
                for x in decay:
                    _number(where, "decay", x, positive=False)
            mlp = layer.get("mlp")
            if mlp is not None:
                kind_ff = mlp.get("kind")
                if kind_ff == "dense":
                    _positive_int(where, "mlp.ff", mlp.get("ff"))
                elif kind_ff == "moe":
                    _glu(where, mlp.get("expert"), "mlp.expert")
                    if mlp.get("shared") is not None:
                        _glu(where, mlp["shared"], "mlp.shared")
                    r = mlp.get("router")
                    if not isinstance(r, dict):
                        raise ConfigError(f"{where}: mlp.router is missing")
                    E = _positive_int(where, "router.experts", r.get("experts"))
                    top = _positive_int(where, "router.top", r.get("top"))
                    g = r.get("groups") or {"count": 1, "keep": 1}
                    count = _positive_int(where, "router.groups.count", g.get("count"))
                    keep = _positive_int(where, "router.groups.keep", g.get("keep"))
                    if top > E or E % count or keep > count or keep * (E // count) < top:
                        raise ConfigError(f"{where}: {top} of {E} experts from {keep} of {count} groups is not possible")
                else:
                    raise ConfigError(f"{where}: feed-forward kind {kind_ff!r} is not known (dense, moe)")
            layers.append(json.loads(json.dumps(layer)))       # a copy of plain values
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        return cls(vocab=d["vocab"], width=d["width"], layers=tuple(_freeze(x) for x in layers),
                   norm_eps=float(d["norm"]["eps"]), embedding_scale=scale, side_dim=side_dim,
                   eos_token_ids=eos_ids, architecture=d.get("architecture", "Tedulorn"))

    @classmethod
    def from_json(cls, path) -> "TedulornConfig":
        path = Path(path)
        if path.is_dir():
            path = path / "config.json"
        return cls.from_dict(json.loads(path.read_text()))

    # ---- writing -----------------------------------------------------------------
    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
               "layers": [_thaw(x) for x in self.layers], "norm": {"eps": self.norm_eps},
               "vocab": self.vocab, "width": self.width}
        if self.side_dim is not None:
            out["token_side"] = {"dim": self.side_dim}
        if self.eos_token_ids:
            out["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return out

    # ---- the layer recipe -------------------------------------------------------------
    def _mixer(self, layer, first_blended):
        d, eps = self.width, self.norm_eps
        m = layer["mixer"]
        rot = m["rot"]
        position = RopeSpec(head_dim=m["dim"], theta=float(rot["base"]), rotary_dim=rot["dims"]) if rot["dims"] else None
        if layer["type"] == "retention":
            return RetentionSpec(hidden=d, n_heads=m["heads"], head_dim=m["dim"], v_dim=m["vdim"],
                                 decays=tuple(float(x) for x in m["decay"]), eps=eps, position=position)
        mask = m["mask"]
        blend = None
        if m.get("v_mix"):
            blend = "first" if first_blended else "later"
        return GatedWindowAttentionSpec(
            hidden=d, n_heads=m["heads"], n_kv_heads=m["kv_heads"], head_dim=m["dim"], v_dim=m["vdim"],
            scale=float(m["scale"]), qk_norm_eps=eps, position=position,
            window=None if mask is None else mask["size"], keep_first=0 if mask is None else mask.get("keep_first", 0),
            sink=True, value_blend=blend, head_gate=True)

    def _ffn(self, mlp):
        d = self.width
        if mlp is None:
            return None
        if mlp["kind"] == "dense":
            return ReluSquaredSpec(d, mlp["ff"])
        r = mlp["router"]
        g = r.get("groups") or {"count": 1, "keep": 1}
        shared = mlp.get("shared")
        return RoutedExpertsSpec(
            hidden=d, n_experts=r["experts"], top=r["top"],
            expert=ClampedGLUSpec(d, mlp["expert"]["ff"], float(mlp["expert"]["limit"])),
            n_groups=g["count"], keep_groups=g["keep"],
            shared=None if shared is None else ClampedGLUSpec(d, shared["ff"], float(shared["limit"])))

    def plan(self) -> ModelPlan:
        d, eps = self.width, self.norm_eps
        layers = [_thaw(x) for x in self.layers]
        norm = RMSNormSpec(d, eps, tensor="")
        blocks, ignorable = [], []
        seen_blend = False
        for i, layer in enumerate(layers):
            blends = layer["type"] == "attention" and bool(layer["mixer"].get("v_mix"))
            mixer = self._mixer(layer, first_blended=blends and not seen_blend)
            seen_blend = seen_blend or blends
            ffn = self._ffn(layer.get("mlp"))
            side = None
            if self.side_dim is not None:
                side = TokenSideSpec(hidden=d, dim=self.side_dim, index=i, n_layers=len(layers), vocab=self.vocab, eps=eps)
            blocks.append(BlockSpec(mixer=mixer, ffn=ffn, norm1=norm, norm2=None if ffn is None else norm,
                                    prefix=f"l{i}.", names=_NAMES, arrangement="prenorm_side", side=side))
            if ffn is None:
                ignorable.append(f"l{i}.norm2")
            if layer["type"] == "attention" and not blends:
                ignorable.append(f"l{i}.mix.vmix")
        return ModelPlan(
            architecture=self.architecture, vocab_size=self.vocab, hidden=d, layers=tuple(blocks),
            order=tuple(RunStep(layer=i, cache=i) for i in range(len(blocks))), final_norm=norm,
            embedding_name="embed", final_norm_prefix="final.norm", head_name="head",
            eos_token_ids=self.eos_token_ids, ignorable=tuple(ignorable), embedding_scale=self.embedding_scale)

    # ---- byte and flop counts ---------------------------------------------------------
    def param_counts(self) -> dict:
        """Elements stored, and elements a decode step of one token reads (of the experts only a token's
        share; of the tables one row)."""
        from ..parts import expected_tensors
        total = per_step = 0
        plan = self.plan()
        share = {}
        for i, block in enumerate(plan.layers):
            if isinstance(block.ffn, RoutedExpertsSpec):
                share[f"l{i}.mlp.e"] = block.ffn.top / block.ffn.n_experts
        for name, decl in expected_tensors(plan).items():
            n = 1
            for s in decl.shape:
                n *= max(s, 1)
            total += n
            if name in ("embed", "side.embed"):
                continue
            per_step += n * next((f for p, f in share.items() if name.startswith(p)), 1.0)
        return {"total": total, "read_per_step": int(per_step)}

    def step_weight_bytes(self, batch: int, item: int) -> int:
        """Bytes of weights that a decode step of ``batch`` tokens reads if its tokens choose their experts
        independently and evenly: of E experts, E (1 - (1 - top / E)^batch) on average."""
        from ..parts import expected_tensors
        plan = self.plan()
        share = {}
        for i, block in enumerate(plan.layers):
            if isinstance(block.ffn, RoutedExpertsSpec):
                share[f"l{i}.mlp.e"] = 1.0 - (1.0 - block.ffn.top / block.ffn.n_experts) ** batch
        total = 0.0
        for name, decl in expected_tensors(plan).items():
            if name in ("embed", "side.embed"):
                continue
            n = 1
            for s in decl.shape:
                n *= max(s, 1)
            total += n * next((f for p, f in share.items() if name.startswith(p)), 1.0)
        return int(total * item)

    def step_cache_bytes(self, batch: int, context: int, item: int) -> int:
        """Bytes of cache and state that a decode step of ``batch`` requests behind ``context`` tokens reads."""
        total = 0
        for block in self.plan().layers:
            m = block.mixer
            if isinstance(m, RetentionSpec):
                total += 4 * m.n_heads * m.head_dim * m.v_dim
            else:
                seen = context if m.window is None else min(context, m.window + m.keep_first)
                total += item * 2 * m.n_kv_heads * m.cache_width * seen
        return batch * total

    def prefill_flops(self, tokens: int) -> float:
        """Multiply-adds times two of one prompt of ``tokens`` tokens from position 0: every matrix a token
        uses (of the experts a token's share; the head at one position), attention scores and sums over what
        each token sees, and the recurrence (per token and head, state size times four)."""
        from ..parts import expected_tensors
        plan = self.plan()
        share = {}
        for i, block in enumerate(plan.layers):
            if isinstance(block.ffn, RoutedExpertsSpec):
                share[f"l{i}.mlp.e"] = block.ffn.top / block.ffn.n_experts
        matrices = 0.0
        for name, decl in expected_tensors(plan).items():
            if decl.kind == "matrix" and len(decl.shape) == 2 and name not in ("embed", "head", "side.embed"):
                matrices += decl.shape[0] * decl.shape[1] * next((f for p, f in share.items() if name.startswith(p)), 1.0)
        flops = 2.0 * tokens * matrices + 2.0 * self.vocab * self.width
        for block in plan.layers:
            m = block.mixer
            if isinstance(m, RetentionSpec):
                flops += 4.0 * tokens * m.n_heads * m.head_dim * m.v_dim
            else:
                seen = sum(min(p + 1, p + 1 if m.window is None else m.window + min(m.keep_first, max(0, p + 1 - m.window)))
                           for p in range(tokens))
                flops += 2.0 * seen * m.n_heads * (m.head_dim + m.v_dim)
        return flops
