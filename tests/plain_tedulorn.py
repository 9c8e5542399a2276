"""Tedulorn the plain way: whole sequences in float64, no cache, no batches, one function per
mechanism, written from the design's equations. It shares no code with ``socrates_amd``; the
tests compare the framework with it.

A model is (config dict as config.json holds it, {tensor name: torch tensor}).
"""

import math

import torch

F = torch.float64


def rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def turn(x, positions, dims, base):
    """x [T, H, D]: element i < dims/2 of a head is paired with element i + dims/2 and the pair
    is turned by position * base^(-2i/dims); elements from dims on pass."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    a = positions.to(F)[:, None] * freq[None, :]
    c, s = a.cos()[:, None, :], a.sin()[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def retention(h, W, m, eps):
    """Linear attention with a fixed decay per head: S <- decay S + k v^T, o = S^T q."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = turn((h @ W["q"].T).view(T, H, D), pos, m["rot"]["dims"], m["rot"]["base"])
    k = turn((h @ W["k"].T).view(T, H, D), pos, m["rot"]["dims"], m["rot"]["base"]) * D ** -0.5
    v = (h @ W["v"].T).view(T, H, Dv)
    decay = torch.tensor(m["decay"], dtype=F)
    S = torch.zeros(H, D, Dv, dtype=F)
    o = torch.empty(T, H, Dv, dtype=F)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = rms(o, eps).reshape(T, H * Dv)
    g = h @ W["g"].T
    return (o * g * torch.sigmoid(g)) @ W["o"].T


def attention(h, W, m, eps, v_first):
    """Softmax attention over a window plus the first tokens, with one more weight of score 0 in
    the denominator, values blended with an earlier layer's, a gate per head. Returns (result,
    the values that a later layer may blend with: this layer's own, before any blend)."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = rms((h @ W["q"].T).view(T, H, D), eps) * W["q.norm"]
    k = rms((h @ W["k"].T).view(T, G, D), eps) * W["k.norm"]
    q = turn(q, pos, m["rot"]["dims"], m["rot"]["base"])
    k = turn(k, pos, m["rot"]["dims"], m["rot"]["base"])
    v = (h @ W["v"].T).view(T, G, Dv)
    own = v
    if m.get("v_mix") and v_first is not None:
        lam = W["vmix"]
        v = (1.0 - lam) * v + lam * v_first
    size, keep = m["mask"]["size"], m["mask"]["keep_first"]
    i, j = pos[:, None], pos[None, :]
    seen = (j <= i) & ((i - j < size) | (j < keep))
    out = torch.empty(T, H, Dv, dtype=F)
    for a in range(H):
        b = a // (H // G)
        s = (q[:, a] @ k[:, b].T) * m["scale"]
        s = torch.where(seen, s, torch.full_like(s, -math.inf))
        top = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)       # the added weight's score is 0
        e = torch.exp(s - top)
        p = e / (torch.exp(-top) + e.sum(-1, keepdim=True))
        out[:, a] = p @ v[:, b]
    gate = torch.sigmoid(h @ W["g"].T)                     # [T, H]
    return (out * gate[:, :, None]).reshape(T, H * Dv) @ W["o"].T, own


def dense(h, W):
    return torch.relu(h @ W["up"].T) ** 2 @ W["down"].T


def expert(h, W, limit):
    g = torch.clamp(h @ W["gate"].T, max=limit)
    u = torch.clamp(h @ W["up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W["down"].T


def route(h, W, r):
    """[T, experts] weights: zero for the experts a token does not use."""
    s = torch.softmax(h @ W["router"].T, dim=-1)
    choice = s + W["correction"]
    T, E = s.shape
    groups = r.get("groups") or {"count": 1, "keep": 1}
    per = E // groups["count"]
    best = choice.view(T, groups["count"], per).max(-1).values
    kept = best.topk(groups["keep"], dim=-1).indices
    allowed = torch.zeros(T, groups["count"], dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    choice = torch.where(allowed.repeat_interleave(per, dim=1), choice, torch.full_like(choice, -math.inf))
    chosen = choice.topk(r["top"], dim=-1).indices
    picked = torch.gather(s, 1, chosen)
    w = torch.zeros_like(s)
    w.scatter_(1, chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20))
    return w


def sub(tensors, prefix):
    return {k[len(prefix):]: v.to(F) for k, v in tensors.items() if k.startswith(prefix)}


def moe(h, W, mlp):
    w = route(h, W, mlp["router"])
    y = torch.zeros_like(h)
    for e in range(mlp["router"]["experts"]):
        y = y + w[:, e:e + 1] * expert(h, sub(W, f"e{e}."), mlp["expert"]["limit"])
    if mlp.get("shared"):
        y = y + expert(h, sub(W, "shared."), mlp["shared"]["limit"])
    return y


def token_side(x, tokens, i, tensors, dim, eps):
    W = sub(tensors, f"l{i}.side.")
    e = tensors["side.embed"].to(F)[tokens][:, i * dim:(i + 1) * dim]
    y = (gelu_tanh(x @ W["gate"].T) * e) @ W["proj"].T
    return rms(y, eps) * W["norm"]


def forward(config, tensors, tokens, streams=None):
    """float64 logits [T, vocab] of the whole sequence; ``streams``: a list that receives the
    residual stream after every layer."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = config["norm"]["eps"]
    x = tensors["embed"].to(F)[tokens] * config["embedding"]["scale"]
    v_first = None
    for i, layer in enumerate(config["layers"]):
        m, mlp = layer["mixer"], layer.get("mlp")
        h = rms(x, eps) * tensors[f"l{i}.norm1"].to(F)
        W = sub(tensors, f"l{i}.mix.")
        if layer["type"] == "retention":
            x = x + retention(h, W, m, eps)
        else:
            y, own = attention(h, W, m, eps, v_first)
            if m.get("v_mix") and v_first is None:
                v_first = own
            x = x + y
        if mlp is not None:
            h = rms(x, eps) * tensors[f"l{i}.norm2"].to(F)
            W = sub(tensors, f"l{i}.mlp.")
            x = x + (dense(h, W) if mlp["kind"] == "dense" else moe(h, W, mlp))
        if config.get("token_side"):
            x = x + token_side(x, tokens, i, tensors, config["token_side"]["dim"], eps)
        if streams is not None:
            streams.append(x.clone())
    x = rms(x, eps) * tensors["final.norm"].to(F)
    return x @ tensors["head"].to(F).T


def greedy(config, tensors, prompt, n):
    out = list(prompt)
    for _ in range(n):
        out.append(int(forward(config, tensors, out)[-1].argmax()))
    return out[len(prompt):]
