"""Float64 oracle for the Voborax design, written from its equations.

Whole sequences, no caches, one function per mechanism. Shares no code with
``kserve_amd``. Weights come in as a dict name -> float64 tensor with the
checkpoint's tensor names; the config is the plain dict of config.json.

Notation: ``W x`` for a stored [out, in] matrix; sequences are [T, width].
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rotate_interleaved(x, positions, dims, base):
    """x [..., T, n]: coordinates (2i, 2i+1), i < dims/2, turned by
    position * base^(-2i/dims); the rest unchanged. positions [T]."""
    out = x.clone()
    half = dims // 2
    i = torch.arange(half, dtype=F64)
    freq = base ** (-2.0 * i / dims)
    ang = positions.to(F64)[:, None] * freq[None, :]          # [T, half]
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def visible(T, window):
    """[T, T] bool: query i sees key j iff 0 <= i - j (< window if window)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window:
        ok &= (i - j) < window
    return ok


def softmax_sink(scores, mask, sink=None):
    """Row softmax over the visible keys; with ``sink`` (one number per row)
    the denominator has one more term exp(sink) that carries no value."""
    s = scores.masked_fill(~mask, -math.inf)
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink[..., None])
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink[..., None] - m)
    return e / den


def latent_kv(h, w, p, mx, eps, positions):
    """The two things a latent-attention layer caches: the normed latent
    [T, kv_rank] and the shared rotated key part [T, rot_dim] (None without)."""
    R = int(mx["kv_rank"])
    rd = int(mx.get("rot_dim", 0))
    t = h @ w[p + "dkv"].T
    c = rms_unit(t[:, :R], eps) * w[p + "dkv.norm"]
    kr = None
    if rd:
        rot = mx["rot"]
        kr = rotate_interleaved(t[:, R:R + rd], positions, int(rot["dims"]), float(rot["base"]))
    return c, kr


def latent_attention(h, w, p, mx, eps, positions, kv):
    """Both latent mixers: queries through a normed latent, keys and values
    expanded per head from the cached latent ``kv`` = (c, rotated key part);
    window, sink and output gate are used where the layer has them."""
    T = h.shape[0]
    H, D, DV = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
    rd = int(mx.get("rot_dim", 0))
    c, kr = kv
    cq = rms_unit(h @ w[p + "dq"].T, eps) * w[p + "dq.norm"]
    q = (cq @ w[p + "uq"].T).view(T, H, D + rd).transpose(0, 1)       # [H, T, D+rd]
    k = (c @ w[p + "uk"].T).view(T, H, D).transpose(0, 1)
    v = (c @ w[p + "uv"].T).view(T, H, DV).transpose(0, 1)
    scores = q[..., :D] @ k.transpose(1, 2)
    if rd:
        rot = mx["rot"]
        qr = rotate_interleaved(q[..., D:], positions, int(rot["dims"]), float(rot["base"]))
        scores = scores + qr @ kr.T[None]
    scores = scores * float(mx["scale"])
    window = int((mx.get("mask") or {}).get("size", 0))
    mask = visible(T, window)[None].expand(H, T, T)
    sink = None
    if (p + "sink") in w:
        sink = w[p + "sink"][:, None].expand(H, T)
    o = softmax_sink(scores, mask, sink) @ v                           # [H, T, DV]
    if (p + "g") in w:
        o = o * torch.sigmoid(h @ w[p + "g"].T).T[:, :, None]
    return o.transpose(0, 1).reshape(T, H * DV) @ w[p + "o"].T


def dense_ff(h, w, p):
    z = h @ w[p + "up"].T + w[p + "up.b"]
    return gelu_tanh(z) @ w[p + "down"].T + w[p + "down.b"]


def glu_expert(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, w, p, ml):
    """-> (chosen [T, top], weights [T, top]); expert numbers at or past
    ``experts`` are identity experts."""
    top = int(ml["router"]["top"])
    s = torch.softmax(h @ w[p + "router"].T, dim=-1)
    choice = s + w[p + "correction"]
    idx = torch.topk(choice, top, dim=-1).indices
    sel = torch.gather(s, 1, idx)
    return idx, sel / (sel.sum(-1, keepdim=True) + 1e-20)


def moe_ff(h, w, p, ml):
    E = int(ml["router"]["experts"])
    idx, wt = route(h, w, p, ml)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(idx.shape[1]):
            e = int(idx[t, k])
            y = glu_expert(h[t:t + 1], w, f"{p}e{e}.")[0] if e < E else h[t]
            out[t] += wt[t, k] * y
    if ml.get("shared"):
        out = out + glu_expert(h, w, p + "shared.")
    return out


def forward(cfg, w, tokens):
    """-> (logits [T, vocab], list of the residual stream after every layer)."""
    eps = float(cfg["norm"]["eps"])
    m = float(cfg["residual_mult"])
    tok = torch.as_tensor(tokens, dtype=torch.long)
    pos = torch.arange(tok.shape[0])
    x = w["embed"][tok] * float(cfg["embedding"]["scale"])
    kept = {}
    stream = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        mx = L["mixer"]
        if "kv_from" in mx and mx["kv_from"] is not None:
            kv = kept[int(mx["kv_from"])]
        else:
            kv = kept[i] = latent_kv(x, w, p + "mix.", mx, eps, pos)
        a = latent_attention(x, w, p + "mix.", mx, eps, pos, kv)
        x = x + m * layer_norm(a, w[p + "norm1"], eps)
        ml = L.get("mlp")
        if ml:
            f = moe_ff(x, w, p + "mlp.", ml) if ml.get("kind") == "moe" else dense_ff(x, w, p + "mlp.")
            x = x + m * layer_norm(f, w[p + "norm2"], eps)
        stream.append(x.clone())
    y = layer_norm(x, w["final.norm"], eps)
    return y @ w["head"].T, stream
