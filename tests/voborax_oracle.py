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


# -- small configurations and random checkpoints for the tests ----------------

def mixer(heads=2, dim=8, vdim=8, kv_rank=16, q_rank=16, scale=None, rot_dim=0,
          rot_base=10000.0, window=0, kv_from=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank,
         "q_rank": q_rank, "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if rot_dim:
        m["rot_dim"] = rot_dim
        m["rot"] = {"base": rot_base, "dims": rot_dim}
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense_cfg(ff=32):
    return {"kind": "dense", "ff": ff}


def moe_cfg(experts=4, top=2, ff=16, identity=0, shared_ff=0):
    d = {"kind": "moe", "expert": {"ff": ff},
         "router": {"experts": experts, "identity": identity, "top": top}}
    if shared_ff:
        d["shared"] = {"ff": shared_ff}
    return d


def windowed(mlp="dense", **kw):
    """A layer with rotated key part, sliding window and output gate."""
    kw.setdefault("rot_dim", 8)
    kw.setdefault("window", 16)
    return {"type": "latent_attention", "mixer": mixer(**kw),
            "mlp": dense_cfg() if mlp == "dense" else mlp}


def sinked(mlp="dense", **kw):
    """A layer without positions: causal, with a sink."""
    return {"type": "latent_attention_2", "mixer": mixer(**kw),
            "mlp": dense_cfg() if mlp == "dense" else mlp}


def make_config(layers, vocab=48, width=32, eps=1e-5, emb_scale=1.0, mult=1.0):
    return {"architecture": "Voborax", "vocab": vocab, "width": width,
            "embedding": {"scale": emb_scale}, "norm": {"eps": eps},
            "residual_mult": mult, "layers": layers}


def random_weights(cfg, seed=0, dtype=torch.float32):
    """name -> tensor, values rounded to ``dtype`` and returned as float64."""
    g = torch.Generator().manual_seed(seed)
    W = int(cfg["width"])
    out = {}

    def mat(name, rows, cols, gain=1.0):
        out[name] = torch.randn(rows, cols, generator=g) * gain * cols ** -0.5

    def vec(name, n, mean=0.0, std=0.3):
        out[name] = mean + torch.randn(n, generator=g) * std

    out["embed"] = torch.randn(int(cfg["vocab"]), W, generator=g)
    mat("head", int(cfg["vocab"]), W)
    vec("final.norm", W, 1.0)
    for i, L in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", L["mixer"]
        H, D, DV = mx["heads"], mx["dim"], mx["vdim"]
        R, Q, rd = mx["kv_rank"], mx["q_rank"], mx.get("rot_dim", 0)
        vec(p + "norm1", W, 1.0)
        mat(p + "mix.dq", Q, W)
        vec(p + "mix.dq.norm", Q, 1.0)
        mat(p + "mix.uq", H * (D + rd), Q, 2.0)
        if mx.get("kv_from") is None:
            mat(p + "mix.dkv", R + rd, W)
            vec(p + "mix.dkv.norm", R, 1.0)
        mat(p + "mix.uk", H * D, R, 2.0)
        mat(p + "mix.uv", H * DV, R)
        mat(p + "mix.o", W, H * DV)
        if L["type"] == "latent_attention":
            mat(p + "mix.g", H, W, 2.0)
        else:
            vec(p + "mix.sink", H, 0.0, 1.0)
        ml = L.get("mlp")
        if not ml:
            continue
        vec(p + "norm2", W, 1.0)
        q = p + "mlp."
        if ml["kind"] == "dense":
            mat(q + "up", ml["ff"], W)
            vec(q + "up.b", ml["ff"])
            mat(q + "down", W, ml["ff"])
            vec(q + "down.b", W)
            continue
        r = ml["router"]
        n_out = r["experts"] + r.get("identity", 0)
        mat(q + "router", n_out, W, 3.0)
        vec(q + "correction", n_out, 0.0, 0.1)
        names = [f"e{e}." for e in range(r["experts"])]
        ffs = [ml["expert"]["ff"]] * r["experts"]
        if ml.get("shared"):
            names.append("shared.")
            ffs.append(ml["shared"]["ff"])
        for n, ff in zip(names, ffs):
            mat(q + n + "gate", ff, W)
            mat(q + n + "up", ff, W)
            mat(q + n + "down", W, ff)
    return {k: v.to(dtype).to(F64) for k, v in out.items()}
