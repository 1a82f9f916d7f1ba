"""Plain float64 implementation of the Laperax design, written from its
equations: one function per mechanism, whole sequences, no caches, no
batching. Shares no code with ``kserve_amd``.

Notation: T tokens, positions 0..T-1; linear weights are [out, in].

  rms(x)         = x / sqrt(mean(x^2) + eps)
  rotate(x, p)   : for i < n/2 the pair (x_i, x_{i+n/2}) of the first n
                   coordinates of a head turns by the angle p * base^(-2i/n)
  retention      : S_t = d_h S_{t-1} + k_t v_t^T, o_t = S_t^T q_t, k scaled by
                   dim^-1/2; o -> rms per head, times silu(W_g h), W_o
  attention      : q, k rotated then rms-normed per head; softmax over the
                   keys j with 0 <= i - j < window; grouped KV heads
  delta          : q, k, v through a causal depthwise convolution and silu;
                   q, k unit vectors (q times dim^-1/2); g_t = exp(-exp(A)
                   softplus(W_a h + dt)); S <- g S; u = sigmoid(W_b h) (v - S^T k);
                   S <- S + k u^T; o = S^T q; o -> rms per head times a weight,
                   times silu(W_g h), W_o
  experts        : s = sigmoid(W_r h); the `top` largest; weights s / (sum +
                   1e-20) * scale; sum of weight * W_down relu(W_up h)^2
  layer          : h = rms(x) * w; x <- x + (mixer(h) + experts(h))
  model          : x = rms(embed[tok]) * w_e; layers; rms(x) * w_f; head;
                   times logit_scale; cap * tanh(. / cap)
"""

import numpy as np
import torch


def _np(t):
    return t.detach().to(torch.float64).cpu().numpy()


def rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def rotate(x, pos, n, base):
    """x [T, heads, dim]; the first n coordinates of each head are turned."""
    if not n:
        return x
    half = n // 2
    f = float(base) ** (-2.0 * np.arange(half) / n)
    ang = pos[:, None] * f[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:n]
    out = x.copy()
    out[..., :half] = u * c - v * s
    out[..., half:n] = v * c + u * s
    return out


def visible(T, window):
    i = np.arange(T)[:, None]
    j = np.arange(T)[None, :]
    ok = j <= i
    if window:
        ok &= i - j < window
    return ok


def retention(h, W, p, m, eps):
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m.get("vdim", m["dim"])
    pos = np.arange(T, dtype=np.float64)
    rot = m.get("rot") or {}
    n, base = rot.get("dims", 0), rot.get("base", 10000.0)
    q = rotate((h @ W[p + "q"].T).reshape(T, H, D), pos, n, base)
    k = rotate((h @ W[p + "k"].T).reshape(T, H, D), pos, n, base) * D ** -0.5
    v = (h @ W[p + "v"].T).reshape(T, H, V)
    o = np.zeros((T, H, V))
    for a in range(H):
        S = np.zeros((D, V))
        for t in range(T):
            S = m["decay"][a] * S + np.outer(k[t, a], v[t, a])
            o[t, a] = S.T @ q[t, a]
    o = rms(o, eps).reshape(T, H * V) * silu(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def attention(h, W, p, m, eps):
    T = h.shape[0]
    H, G = m["heads"], m.get("kv_heads", m["heads"])
    D, V = m["dim"], m.get("vdim", m["dim"])
    pos = np.arange(T, dtype=np.float64)
    rot = m.get("rot") or {}
    n, base = rot.get("dims", 0), rot.get("base", 10000.0)
    q = rms(rotate((h @ W[p + "q"].T).reshape(T, H, D), pos, n, base), eps)
    k = rms(rotate((h @ W[p + "k"].T).reshape(T, G, D), pos, n, base), eps)
    v = (h @ W[p + "v"].T).reshape(T, G, V)
    ok = visible(T, (m.get("mask") or {}).get("size", 0))
    o = np.zeros((T, H, V))
    for a in range(H):
        g = a // (H // G)
        s = np.where(ok, (q[:, a] @ k[:, g].T) * m["scale"], -np.inf)
        w = np.exp(s - s.max(axis=1, keepdims=True))
        o[:, a] = (w / w.sum(axis=1, keepdims=True)) @ v[:, g]
    return o.reshape(T, H * V) @ W[p + "o"].T


def conv_silu(x, w):
    """x [T, C]; w [C, taps], the last column weighs the current token."""
    T, C = x.shape
    taps = w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, C)), x], axis=0)
    y = np.zeros((T, C))
    for j in range(taps):
        y += padded[j : j + T] * w[:, j][None, :]
    return silu(y)


def unit(x):
    return x / np.sqrt((x * x).sum(-1, keepdims=True) + 1e-6)


def delta(h, W, p, m, eps):
    T = h.shape[0]
    H, G = m["heads"], m.get("kv_heads", m["heads"])
    D, V = m["dim"], m.get("vdim", m["dim"])
    q = unit(conv_silu(h @ W[p + "q"].T, W[p + "q.conv"]).reshape(T, G, D)) * D ** -0.5
    k = unit(conv_silu(h @ W[p + "k"].T, W[p + "k.conv"]).reshape(T, G, D))
    v = conv_silu(h @ W[p + "v"].T, W[p + "v.conv"]).reshape(T, H, V)
    beta = sigmoid(h @ W[p + "b"].T)
    g = np.exp(
        -np.exp(W[p + "A_log"])[None, :]
        * softplus(h @ W[p + "a"].T + W[p + "dt_bias"][None, :])
    )
    o = np.zeros((T, H, V))
    for a in range(H):
        c = a // (H // G)
        S = np.zeros((D, V))
        for t in range(T):
            S = g[t, a] * S
            u = beta[t, a] * (v[t, a] - S.T @ k[t, c])
            S = S + np.outer(k[t, c], u)
            o[t, a] = S.T @ q[t, c]
    o = rms(o, eps) * W[p + "norm"][None, None, :]
    return (o.reshape(T, H * V) * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def route(h, W, p, r):
    """-> list per token of (expert, weight)."""
    s = sigmoid(h @ W[p + "router"].T)
    out = []
    for t in range(h.shape[0]):
        order = sorted(range(r["experts"]), key=lambda e: (-s[t, e], e))[: r["top"]]
        tot = sum(s[t, e] for e in order) + 1e-20
        out.append([(e, s[t, e] / tot * r.get("scale", 1.0)) for e in order])
    return out


def expert(x, W, p):
    return W[p + "down"] @ (np.maximum(W[p + "up"] @ x, 0.0) ** 2)


def experts(h, W, p, m):
    out = np.zeros((h.shape[0], W[p + "e0.down"].shape[0]))
    for t, picks in enumerate(route(h, W, p, m["router"])):
        for e, w in picks:
            out[t] += w * expert(h[t], W, f"{p}e{e}.")
    return out


MIXERS = {"retention": retention, "attention": attention, "delta": delta}


def forward(cfg, sd, tokens, streams=None):
    """Logits [T, vocab] (float64 torch); ``streams`` collects the residual
    stream after every layer."""
    W = {k: _np(v) for k, v in sd.items()}
    eps = cfg["norm"]["eps"]
    x = rms(W["embed"][np.asarray(tokens)], eps) * W["embed.norm"]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms(x, eps) * W[p + "norm1"]
        add = MIXERS[layer["type"]](h, W, p + "mix.", layer["mixer"], eps)
        if layer.get("mlp"):
            add = add + experts(h, W, p + "mlp.", layer["mlp"])
        x = x + add
        if streams is not None:
            streams.append(torch.from_numpy(x.copy()))
    lg = (rms(x, eps) * W["final.norm"]) @ W["head"].T * cfg.get("logit_scale", 1.0)
    cap = cfg.get("logit_softcap", 0.0)
    if cap:
        lg = cap * np.tanh(lg / cap)
    return torch.from_numpy(lg)


# -- builders -----------------------------------------------------------------

def moe(experts=4, top=2, ff=24, scale=1.5):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "scale": scale}}


def retention_layer(heads=2, dim=8, vdim=12, decay=None, rot_dims=4, base=100.0, mlp=None):
    decay = decay or [1.0 - 2.0 ** -(3 + i) for i in range(heads)]
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
    return {"type": "retention", "mixer": m, "mlp": mlp}


def attention_layer(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.4, window=9,
                    rot_dims=4, base=50.0, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": scale, "mask": {"size": window}}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def delta_layer(heads=4, kv_heads=2, dim=8, vdim=12, conv=4, mlp=None):
    return {"type": "delta", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                      "vdim": vdim, "conv": conv}}


def make_config(layers, vocab=61, width=32, eps=1e-5, logit_scale=0.7, softcap=8.0):
    return {"architecture": "Laperax", "vocab": vocab, "width": width,
            "norm": {"eps": eps}, "logit_scale": logit_scale,
            "logit_softcap": softcap, "layers": layers}


def random_weights(cfg, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain * i ** -0.5).to(dtype)

    def around_one(n):
        return (1.0 + 0.1 * torch.randn(n, generator=g)).to(dtype)

    sd = {"embed": torch.randn(cfg["vocab"], W, generator=g).to(dtype),
          "embed.norm": around_one(W), "final.norm": around_one(W),
          "head": mat(cfg["vocab"], W)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        sd[p + "norm1"] = around_one(W)
        H, D, V = m["heads"], m["dim"], m.get("vdim", m["dim"])
        G = m.get("kv_heads", H)
        x = p + "mix."
        if layer["type"] == "retention":
            sd[x + "q"], sd[x + "k"] = mat(H * D, W), mat(H * D, W)
            sd[x + "v"], sd[x + "g"] = mat(H * V, W), mat(H * V, W, 2.0)
            sd[x + "o"] = mat(W, H * V)
        elif layer["type"] == "attention":
            sd[x + "q"], sd[x + "k"] = mat(H * D, W), mat(G * D, W)
            sd[x + "v"], sd[x + "o"] = mat(G * V, W), mat(W, H * V)
        else:
            taps = m["conv"]
            for n, rows in (("q", G * D), ("k", G * D), ("v", H * V)):
                sd[x + n] = mat(rows, W, 2.0)
                sd[x + n + ".conv"] = (torch.randn(rows, taps, generator=g) * 0.5).to(dtype)
            sd[x + "g"], sd[x + "o"] = mat(H * V, W, 2.0), mat(W, H * V)
            sd[x + "b"], sd[x + "a"] = mat(H, W, 2.0), mat(H, W, 2.0)
            sd[x + "A_log"] = (torch.rand(H, generator=g) * 2 - 2).to(dtype)
            sd[x + "dt_bias"] = (torch.rand(H, generator=g) * 2 - 1).to(dtype)
            sd[x + "norm"] = around_one(V)
        if layer.get("mlp"):
            f, r = layer["mlp"]["expert"]["ff"], layer["mlp"]["router"]
            y = p + "mlp."
            sd[y + "router"] = mat(r["experts"], W, 2.0)
            for e in range(r["experts"]):
                sd[f"{y}e{e}.up"], sd[f"{y}e{e}.down"] = mat(f, W), mat(W, f)
    return sd
