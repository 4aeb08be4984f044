"""Plain whole-sequence implementation of the Fikizen design, used as the oracle of
``tests/test_fikizen.py``. One function per mechanism, float64 by default, token by token
where the design is recurrent, no cache, no batching, and no code shared with ``hipserve``.

A model is (config dict as in ``config.json``, dict of tensors under the checkpoint's names).
"""
from __future__ import annotations

import math

import torch

DT = torch.float64


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def unit(x):
    """x / sqrt(sum(x^2) + 1e-6) over the last axis."""
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def silu(x):
    return x * torch.sigmoid(x)


def rotate(x, pos, dims, base):
    """x [n, heads, d]: rotate-half over the first ``dims`` of every head, angle pos * base^(-2i/dims)."""
    if dims <= 0:
        return x
    half = dims // 2
    i = torch.arange(half, dtype=DT)
    ang = pos.to(DT)[:, None] * base ** (-2.0 * i / dims)[None]           # [n, half]
    c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def sink_softmax(s):
    """exp(s_j) / (1 + sum_j exp(s_j)) over the last axis (entries at -inf get 0)."""
    m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def window_attention(q, k, v, scale, window):
    """q [n, H, d], k [n, G, d], v [n, G, dv]: position i sees j with 0 <= i - j < window; sink softmax."""
    n, H, _ = q.shape
    G = k.shape[1]
    i = torch.arange(n)
    d = i[:, None] - i[None]
    ok = (d >= 0) & (d < window)
    out = torch.zeros(n, H, v.shape[-1], dtype=DT)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].t()) * scale
        s = s.masked_fill(~ok, float("-inf"))
        out[:, h] = sink_softmax(s) @ v[:, g]
    return out


def attention_mixer(h, m, W, pre, eps, gated, biased, normed):
    """The attention mixer; ``gated``: per-head sigmoid output gate; ``biased``: projection biases;
    ``normed``: RMS norm over the whole q / k projection (weights) and unit-rms values per head."""
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ W[pre + "q"].t(), h @ W[pre + "k"].t(), h @ W[pre + "v"].t()
    if biased:
        q, k, v = q + W[pre + "q.b"], k + W[pre + "k.b"], v + W[pre + "v.b"]
    if normed:
        q = rms(q, eps) * W[pre + "q.norm"]
        k = rms(k, eps) * W[pre + "k.norm"]
    q, k, v = q.view(n, H, d), k.view(n, G, d), v.view(n, G, dv)
    pos = torch.arange(n)
    rot = m.get("rot") or {}
    q = rotate(q, pos, int(rot.get("dims", 0)), float(rot.get("base", 10000.0)))
    k = rotate(k, pos, int(rot.get("dims", 0)), float(rot.get("base", 10000.0)))
    if normed:
        v = rms(v, eps)
    o = window_attention(q, k, v, m["scale"], m["mask"]["size"])
    if gated:
        o = o * torch.sigmoid(h @ W[pre + "g"].t())[:, :, None]
    return o.reshape(n, H * dv) @ W[pre + "o"].t()


def causal_conv(x, w):
    """x [n, C], w [C, taps] (last column = current token), zeros before the start."""
    n, taps = x.shape[0], w.shape[1]
    xp = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=DT), x])
    return sum(xp[j:j + n] * w[:, j] for j in range(taps))


def gated_delta_mixer(h, m, W, pre, eps):
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ W[pre + "q"].t(), W[pre + "q.conv"])).view(n, G, d)
    k = silu(causal_conv(h @ W[pre + "k"].t(), W[pre + "k.conv"])).view(n, G, d)
    v = silu(causal_conv(h @ W[pre + "v"].t(), W[pre + "v.conv"])).view(n, H, dv)
    q = unit(q) * d ** -0.5
    k = unit(k)
    beta = torch.sigmoid(h @ W[pre + "b"].t())                                         # [n, H]
    g = torch.exp(-torch.exp(W[pre + "A_log"]) * softplus(h @ W[pre + "a"].t() + W[pre + "dt_bias"]))
    o = torch.zeros(n, H, dv, dtype=DT)
    for hd in range(H):
        kh = hd // (H // G)
        S = torch.zeros(d, dv, dtype=DT)
        for t in range(n):
            S = g[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.t() @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            o[t, hd] = S.t() @ q[t, kh]
    o = rms(o, eps) * W[pre + "norm"] * silu(h @ W[pre + "g"].t()).view(n, H, dv)
    return o.reshape(n, H * dv) @ W[pre + "o"].t()


def delta_rule_mixer(h, m, W, pre, eps):
    """Generalized delta rule with per-channel decay and removal."""
    n = h.shape[0]
    H, d = m["heads"], m["dim"]
    r = (h @ W[pre + "r"].t()).view(n, H, d)
    k = (h @ W[pre + "k"].t()).view(n, H, d)
    v = (h @ W[pre + "v"].t()).view(n, H, d)
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ W[pre + "w1"].t()) @ W[pre + "w2"].t() + W[pre + "w0"]))
    w = w.view(n, H, d)
    a = torch.sigmoid(h @ W[pre + "a"].t() + W[pre + "a.b"]).view(n, H, d)
    u = unit(k)
    o = torch.zeros(n, H, d, dtype=DT)
    for hd in range(H):
        S = torch.zeros(d, d, dtype=DT)                                  # [key, value]
        for t in range(n):
            uS = u[t, hd] @ S
            S = w[t, hd][:, None] * S - torch.outer(a[t, hd] * u[t, hd], uS) + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.t() @ r[t, hd]
    o = rms(o, eps).reshape(n, H * d) * W[pre + "norm"] * torch.sigmoid(h @ W[pre + "g"].t())
    return o @ W[pre + "o"].t()


def parallel_mixer(h, m, W, pre, eps):
    left = attention_mixer(h, m["left"], W, pre + "left.", eps, gated=False, biased=True, normed=True)
    right = delta_rule_mixer(h, m["right"], W, pre + "right.", eps)
    return m["left_scale"] * left + m["right_scale"] * right


def xielu(z, p, q):
    pos = softplus(p) * z * z + z / 2
    neg = (0.5 + softplus(q)) * (torch.expm1(torch.clamp(z, max=0.0)) - z) + z / 2
    return torch.where(z > 0, pos, neg)


def feed_forward(h, W, pre):
    act = W[pre + "act"]
    return xielu(h @ W[pre + "up"].t(), act[0], act[1]) @ W[pre + "down"].t()


def forward(cfg: dict, tensors: dict, tokens, capture: list | None = None):
    """Logits [n, vocab] of one sequence; ``capture`` gets the residual stream after every layer."""
    W = {k: (v.to(DT) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = float(cfg["norm"]["eps"])
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(cfg["layers"]):
        j = layer.get("weights_of", i)
        pre = f"l{j}."
        hn = rms(x, eps) * W[pre + "norm1"]
        kind = layer["type"]
        if kind == "attention":
            y = attention_mixer(hn, layer["mixer"], W, pre + "mix.", eps, gated=True, biased=False, normed=False)
        elif kind == "parallel":
            y = parallel_mixer(hn, layer["mixer"], W, pre + "mix.", eps)
        elif kind == "delta":
            y = gated_delta_mixer(hn, layer["mixer"], W, pre + "mix.", eps)
        else:
            raise ValueError(kind)
        x = x + y
        if layer.get("mlp") is not None:
            x = x + feed_forward(rms(x, eps) * W[pre + "norm2"], W, pre + "mlp.")
        if capture is not None:
            capture.append(x.clone())
    logits = (rms(x, eps) * W["final.norm"]) @ W["head"].t()
    cap = float(cfg.get("logit_softcap") or 0.0)
    if cap > 0:
        logits = cap * torch.tanh(logits / cap)
    return logits


# ---------------------------------------------------------------- test models
def attn_mixer(heads=4, kv_heads=2, dim=12, vdim=10, window=6, rot_dims=8, base=100.0, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window},
            "rot": {"base": base, "dims": rot_dims}, "scale": dim ** -0.5 if scale is None else scale}


def attn_layer(mlp=None, **kw):
    return {"type": "attention", "mixer": attn_mixer(**kw), "mlp": mlp}


def delta_layer(heads=4, kv_heads=2, dim=8, vdim=6, conv=3, mlp=None):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": mlp}


def parallel_layer(left=None, heads=3, dim=8, left_scale=0.7, right_scale=1.2, mlp=None):
    return {"type": "parallel", "mixer": {"left": attn_mixer(**(left or {})), "right": {"heads": heads, "dim": dim},
                                          "left_scale": left_scale, "right_scale": right_scale}, "mlp": mlp}


def shared(layers, j):
    """An entry that runs layer j's weights once more."""
    return dict(layers[j], weights_of=j)


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def make_config(layers, width=32, vocab=96, softcap=20.0, eps=1e-5):
    return {"architecture": "Fikizen", "layers": layers, "logit_softcap": softcap, "norm": {"eps": eps},
            "vocab": vocab, "width": width}


def make_weights(cfg, seed=0, gain=1.0, rank=5):
    """Random checkpoint tensors (values representable in bf16) under the design's names."""
    g = torch.Generator().manual_seed(seed)
    Wd, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).bfloat16().float()

    def lin(o, i):
        return rnd(o, i, std=gain / math.sqrt(i))

    def attn(p, m, full):
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        W[p + "q"], W[p + "k"], W[p + "v"], W[p + "o"] = lin(H * d, Wd) * 2, lin(G * d, Wd) * 2, lin(G * dv, Wd), lin(Wd, H * dv)
        if full:
            W[p + "q.b"], W[p + "k.b"], W[p + "v.b"] = rnd(H * d, std=0.3), rnd(G * d, std=0.3), rnd(G * dv, std=0.3)
            W[p + "q.norm"], W[p + "k.norm"] = 1 + rnd(H * d, std=0.3), 1 + rnd(G * d, std=0.3)
        else:
            W[p + "g"] = lin(H, Wd) * 2

    W = {"embed": rnd(V, Wd), "head": lin(V, Wd) * 3, "final.norm": 1 + rnd(Wd, std=0.1)}
    for i, l in enumerate(cfg["layers"]):
        if "weights_of" in l:
            continue
        p, m = f"l{i}.", l["mixer"]
        W[p + "norm1"] = 1 + rnd(Wd, std=0.1)
        if l["type"] == "attention":
            attn(p + "mix.", m, False)
        elif l["type"] == "delta":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for n, c in (("q", G * d), ("k", G * d), ("v", H * dv)):
                W[p + "mix." + n] = lin(c, Wd) * 2
                W[p + "mix." + n + ".conv"] = rnd(c, m["conv"], std=0.6)
            W[p + "mix.b"], W[p + "mix.a"] = lin(H, Wd) * 2, lin(H, Wd) * 2
            W[p + "mix.A_log"], W[p + "mix.dt_bias"] = rnd(H, std=0.5) - 1.5, rnd(H, std=0.5)
            W[p + "mix.norm"], W[p + "mix.g"], W[p + "mix.o"] = 1 + rnd(dv, std=0.2), lin(H * dv, Wd) * 2, lin(Wd, H * dv)
        else:
            attn(p + "mix.left.", m["left"], True)
            q, N = p + "mix.right.", m["right"]["heads"] * m["right"]["dim"]
            for n in ("r", "k", "v", "a", "g"):
                W[q + n] = lin(N, Wd) * 2
            W[q + "a.b"], W[q + "w0"], W[q + "norm"] = rnd(N, std=0.5), rnd(N), 1 + rnd(N, std=0.2)
            W[q + "w1"], W[q + "w2"], W[q + "o"] = lin(rank, Wd) * 2, rnd(N, rank, std=0.7), lin(Wd, N)
        if l["mlp"] is not None:
            W[p + "norm2"] = 1 + rnd(Wd, std=0.1)
            W[p + "mlp.up"], W[p + "mlp.down"] = lin(l["mlp"]["ff"], Wd) * 2, lin(Wd, l["mlp"]["ff"])
            W[p + "mlp.act"] = rnd(2, std=0.7)
    return {k: v.bfloat16().float() for k, v in W.items()}


def save_checkpoint(path, cfg, W):
    import json
    import os

    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.bfloat16().contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return path
