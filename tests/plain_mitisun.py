"""A plain, slow Mitisun in PyTorch: one whole sequence from position 0, no cache, no batches.

It is the oracle the framework's Mitisun is compared with, written from the design's
equations with one function per mechanism, and shares no code with ``socrates_amd``.
``w`` maps tensor names to tensors (any float dtype; everything is computed in the dtype
of ``x``, float64 in the tests), ``cfg`` is the dict of ``config.json``.

Notation: T tokens, d the model's width, H heads. A linear weight W is stored [out, in] and
applied as x @ W.T.
"""

import json
import math
from pathlib import Path

import torch
from safetensors import safe_open


def read_folder(folder, dtype=torch.float64):
    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    w = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            w[name] = f.get_tensor(name).to(dtype)
    return cfg, w


# ---- norms ------------------------------------------------------------------------------------
def unit_rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def scalar_gain_norm(x, g, eps):
    """RMS norm whose gain is one number for all coordinates."""
    return unit_rms(x, eps) * g


def rms_norm(x, weight, eps):
    return unit_rms(x, eps) * weight


# ---- activations ------------------------------------------------------------------------------
def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


# ---- mixer: RWKV-style time mixing with per-channel decay --------------------------------------
def shifted(h):
    """Row t holds h[t - 1]; row 0 holds zeros."""
    return torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)


def wkv_recurrence(r, k, v, decay, bonus):
    """r, k, decay [T, H, K]; v [T, H, V]; bonus [H, K]. Returns o [T, H, V].

    o_t = (S + diag(bonus) k_t v_t^T)^T r_t with the state before token t, then
    S <- diag(decay_t) S + k_t v_t^T. The state starts at zero."""
    T, H, K = k.shape
    S = torch.zeros(H, K, v.shape[-1], dtype=r.dtype)
    out = []
    for t in range(T):
        kv = k[t].unsqueeze(-1) * v[t].unsqueeze(-2)                  # [H, K, V]
        out.append(torch.einsum("hk,hkv->hv", r[t], S + bonus.unsqueeze(-1) * kv))
        S = decay[t].unsqueeze(-1) * S + kv
    return torch.stack(out)


def wkv_mixer(h, w, p, m, eps):
    H, D = m["heads"], m["dim"]
    T = h.shape[0]
    diff = shifted(h) - h
    mix = {s: h + diff * w[f"{p}mu.{s}"] for s in "rkvgw"}
    r = (mix["r"] @ w[p + "r"].T).view(T, H, D)
    k = (mix["k"] @ w[p + "k"].T).view(T, H, D)
    v = (mix["v"] @ w[p + "v"].T).view(T, H, D)
    gate = silu(mix["g"] @ w[p + "g"].T)
    log_decay = torch.tanh(mix["w"] @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"]
    decay = torch.exp(-torch.exp(log_decay)).view(T, H, D)
    o = wkv_recurrence(r, k, v, decay, w[p + "u"])
    o = unit_rms(o, eps).reshape(T, H * D) * w[p + "norm"] * gate
    return o @ w[p + "o"].T


# ---- mixer: latent attention -------------------------------------------------------------------
def rotate_pairs(x, positions, base, dims):
    """Rotary positions in the interleaved layout over the first ``dims`` coordinates of the
    last axis: coordinates 2i and 2i + 1 are one pair, turned by position * base^(-2i/dims).
    x [T, ..., D]; positions [T]."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    angle = positions.to(torch.float64).unsqueeze(-1) * base ** (-2.0 * i / dims)       # [T, dims/2]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    cos, sin = angle.cos().to(x.dtype).view(shape), angle.sin().to(x.dtype).view(shape)
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def latent_kv(h, w, p, m, eps, positions):
    """What a latent-attention layer keeps per token: the normed latent [T, kv_rank] and the
    rotated key part that all heads share [T, rot_dim]."""
    R = m["kv_rank"]
    down = h @ w[p + "dkv"].T
    latent = rms_norm(down[:, :R], w[p + "dkv.norm"], eps)
    shared_key = rotate_pairs(down[:, R:], positions, m["rot"]["base"], m["rot"]["dims"])
    return latent, shared_key


def windowed_softmax(scores, window):
    """scores [H, T, T] (query, key); key j is visible to query i if 0 <= i - j < window."""
    T = scores.shape[-1]
    i, j = torch.arange(T).unsqueeze(1), torch.arange(T).unsqueeze(0)
    visible = (i - j >= 0) & (i - j < window)
    return torch.softmax(scores.masked_fill(~visible, float("-inf")), dim=-1)


def latent_attention_mixer(h, w, p, m, eps, kept):
    """``kept``: (latent, shared key) of the layer this one reads, from ``latent_kv``."""
    H, D, Dr, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    positions = torch.arange(T)
    latent, shared_key = kept
    q = (rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps) @ w[p + "uq"].T).view(T, H, D + Dr)
    q_plain = q[..., :D]
    q_turned = rotate_pairs(q[..., D:], positions, m["rot"]["base"], m["rot"]["dims"])
    k_plain = (latent @ w[p + "uk"].T).view(T, H, D)
    value = (latent @ w[p + "uv"].T).view(T, H, Dv)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain)
              + torch.einsum("ihd,jd->hij", q_turned, shared_key)) * m["scale"]
    weights = windowed_softmax(scores, m["mask"]["size"])
    o = torch.einsum("hij,jhd->ihd", weights, value).reshape(T, H * Dv)
    return o @ w[p + "o"].T


# ---- mixer: Mamba-2 -----------------------------------------------------------------------------
def causal_conv(x, kernel, bias):
    """Per channel: y[t, c] = bias[c] + sum_j kernel[c, j] x[t - (taps - 1) + j, c], zeros before
    the start (the last column of the kernel meets the current token). x [T, C]."""
    T, taps = x.shape[0], kernel.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=x.dtype), x], dim=0)
    y = bias.expand(T, -1).clone()
    for j in range(taps):
        y = y + padded[j:j + T] * kernel[:, j]
    return y


def ssd_recurrence(x, dt, a, B, C, skip):
    """x [T, H, P]; dt [T, H]; a [H] (positive rates); B, C [T, H, N] (already spread from
    groups to heads); skip [H]. S_t = exp(-a dt_t) S_(t-1) + dt_t B_t x_t^T, y_t = S_t^T C_t +
    skip x_t."""
    T, H, P = x.shape
    S = torch.zeros(H, B.shape[-1], P, dtype=x.dtype)
    out = []
    for t in range(T):
        S = torch.exp(-a * dt[t]).view(H, 1, 1) * S + (dt[t].unsqueeze(-1) * B[t]).unsqueeze(-1) * x[t].unsqueeze(-2)
        out.append(torch.einsum("hn,hnp->hp", C[t], S) + skip.unsqueeze(-1) * x[t])
    return torch.stack(out)


def mamba2_mixer(h, w, p, m, eps):
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner, T = H * P, h.shape[0]
    proj = h @ w[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    per_group = H // G
    B = xbc[:, inner:inner + G * N].view(T, G, N).repeat_interleave(per_group, dim=1)
    C = xbc[:, inner + G * N:].view(T, G, N).repeat_interleave(per_group, dim=1)
    dt = softplus(dt + w[p + "dt_bias"])
    y = ssd_recurrence(x, dt, torch.exp(w[p + "A_log"]), B, C, w[p + "D"]).reshape(T, inner)
    y = y * silu(z)
    parts = m["norm_groups"]
    y = unit_rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w[p + "norm"]
    return y @ w[p + "o"].T


# ---- feed-forward -------------------------------------------------------------------------------
def clamped_glu(h, w, p, limit):
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w[p + "down"].T


# ---- the model ----------------------------------------------------------------------------------
def forward(cfg, w, ids, trace=None):
    """Logits [T, vocab] of the whole sequence ``ids``. ``trace``: a list that receives the
    residual stream after every layer."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = w["embed"][torch.as_tensor(ids, dtype=torch.long)]
    positions = torch.arange(x.shape[0])
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        L, m = f"l{i}.", layer["mixer"]
        h = scalar_gain_norm(x, w[L + "norm1"], eps)
        if layer["type"] == "wkv":
            a = wkv_mixer(h, w, L + "mix.", m, eps)
        elif layer["type"] == "mamba2":
            a = mamba2_mixer(h, w, L + "mix.", m, eps)
        elif layer["type"] == "latent_attention":
            if "kv_from" in m and m["kv_from"] is not None:
                src = kept[m["kv_from"]]
            else:
                src = kept[i] = latent_kv(h, w, L + "mix.", m, eps, positions)
            a = latent_attention_mixer(h, w, L + "mix.", m, eps, src)
        else:
            raise ValueError(layer["type"])
        a = a * torch.sigmoid(h @ w[L + "rg1"].T + w[L + "rg1.b"])
        x = x + mult * scalar_gain_norm(a, w[L + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = scalar_gain_norm(x, w[L + "norm2"], eps)
            f = clamped_glu(h, w, L + "mlp.", layer["mlp"]["limit"])
            f = f * torch.sigmoid(h @ w[L + "rg2"].T + w[L + "rg2.b"])
            x = x + mult * scalar_gain_norm(f, w[L + "norm2b"], eps)
        if trace is not None:
            trace.append(x.clone())
    return scalar_gain_norm(x, w["final.norm"], eps) @ w["head"].T


def greedy(cfg, w, prompt, n_new):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(forward(cfg, w, ids)[-1].argmax()))
    return ids[len(prompt):]
