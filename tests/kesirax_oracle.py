"""Plain, slow fp32 implementation of the Kesirax design for the tests: one function per
mechanism, written from the design's equations, whole sequences at once, no cache, no batching.
It reads the same ``config.json`` dictionary and checkpoint tensor names as the engine and
shares no code with it.

Notation: x [T, W] residual stream, h the layer's normed input, p_t = t the position.
"""
import json
import math
import os

import torch


# ------------------------------------------------------------------ mechanisms
def rms(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def group_rms(x, w, groups, eps):
    """The last axis cut into `groups` equal consecutive parts, each divided by its own rms."""
    parts = x.reshape(*x.shape[:-1], groups, x.shape[-1] // groups)
    parts = parts / torch.sqrt((parts * parts).mean(-1, keepdim=True) + eps)
    return parts.reshape(x.shape) * w


def rotate(v, pos, base, dims):
    """Rotary position on the first `dims` entries of the last axis; entry i pairs with i + dims/2;
    angle = pos * base^(-2i/dims). v [..., T, d], pos [T]."""
    half = dims // 2
    out = v.clone()
    for i in range(half):
        ang = pos.to(torch.float32) * torch.tensor(base, dtype=torch.float32) ** (-2.0 * i / dims)
        c, s = torch.cos(ang), torch.sin(ang)
        a, b = v[..., i], v[..., i + half]
        out[..., i] = a * c - b * s
        out[..., i + half] = b * c + a * s
    return out


def latent_attention(h, W, pre, m, eps, pos0=0):
    """h [T, width]; W tensors under prefix `pre`; m the mixer's config dictionary."""
    T = h.shape[0]
    H, d, r, vd, kr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    window = (m.get("mask") or {}).get("size")
    pos = torch.arange(pos0, pos0 + T)
    cq = rms(h @ W[pre + "dq"].T, W[pre + "dq.norm"], eps)
    q = (cq @ W[pre + "uq"].T).reshape(T, H, d + r)
    dkv = h @ W[pre + "dkv"].T
    c = rms(dkv[:, :kr], W[pre + "dkv.norm"], eps)
    k_rot = rotate(dkv[:, kr:], pos, base, dims)                       # shared by the heads
    k = (c @ W[pre + "uk"].T).reshape(T, H, d)
    v = (c @ W[pre + "uv"].T).reshape(T, H, vd)
    gate = torch.sigmoid(h @ W[pre + "g"].T)                           # [T, H]
    out = torch.zeros(T, H, vd)
    for hd in range(H):
        qr = rotate(q[:, hd, d:], pos, base, dims)
        s = (q[:, hd, :d] @ k[:, hd].T + qr @ k_rot.T) * m["scale"]    # [T, T]
        back = pos[:, None] - pos[None, :]                             # i - j
        hidden = (back < 0) | (back >= window) if window else (back < 0)
        s = s.masked_fill(hidden, -math.inf)
        out[:, hd] = (torch.softmax(s, -1) @ v[:, hd]) * gate[:, hd:hd + 1]
    return out.reshape(T, H * vd) @ W[pre + "o"].T


def mingru(h, W, pre, m, state=None):
    """Returns (output [T, width of the stream], last state)."""
    z = torch.sigmoid(h @ W[pre + "z"].T + W[pre + "z.b"])
    u = h @ W[pre + "x"].T + W[pre + "x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = h @ W[pre + "g"].T
    S = torch.zeros(m["width"]) if state is None else state
    rows = []
    for t in range(h.shape[0]):
        S = (1 - z[t]) * S + z[t] * cand[t]
        rows.append(S * (g[t] * torch.sigmoid(g[t])))
    return torch.stack(rows) @ W[pre + "o"].T, S


def table_moe(h, tokens, W, pre, f):
    top = f["router"]["top"]
    out = torch.zeros(h.shape[0], W[pre + "e0.down"].shape[0])
    for t, tok in enumerate(tokens):
        for e in W[pre + "table"][tok].tolist():
            a = torch.relu(W[f"{pre}e{e}.up"] @ h[t])
            out[t] += (W[f"{pre}e{e}.down"] @ (a * a)) / top
    return out


def layer_runs(cfg):
    n, lp = len(cfg["layers"]), cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b = lp["start"], lp["stop"]
    runs = [(i, False) for i in range(a)]
    for t in range(lp["times"]):
        runs += [(i, t > 0 and i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, W, tokens, streams=None):
    """Logits [T, vocab] of a whole sequence. `streams`: list that gets x after every layer run."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x0 = W["embed"][torch.tensor(tokens)]
    x = x0.clone()
    for i, again in layer_runs(cfg):
        if again:
            x = x + x0
        l = cfg["layers"][i]
        h = group_rms(x, W[f"l{i}.norm1"], groups, eps)
        if l["type"] == "latent_attention":
            y = latent_attention(h, W, f"l{i}.mix.", l["mixer"], eps)
        else:
            y, _ = mingru(h, W, f"l{i}.mix.", l["mixer"])
        y = y * W[f"l{i}.ls1"]
        if l.get("mlp") is not None:
            y = y + table_moe(h, tokens, W, f"l{i}.mlp.", l["mlp"]) * W[f"l{i}.ls2"]
        x = x + y
        if streams is not None:
            streams.append(x.clone())
    return group_rms(x, W["final.norm"], groups, eps) @ W["head"].T * cfg["logit_scale"]


# ------------------------------------------------------------------ test models
def attn_layer(heads=3, dim=8, rot_dim=4, vdim=8, q_rank=12, kv_rank=16, window=6, base=100.0, scale=None,
               rot_dims=None, mlp=None):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
             "scale": scale if scale is not None else (dim + rot_dim) ** -0.5,
             "rot": {"base": base, "dims": rot_dims or rot_dim}}
    if window:
        mixer["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def gru_layer(width=24, mlp=None):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": mlp}


def moe(experts=4, top=2, ff=12):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def make_config(layers, width=32, vocab=96, loop=(0, 0, 1), groups=4, logit_scale=0.75, eps=1e-6):
    return {"architecture": "Kesirax", "layers": layers, "logit_scale": logit_scale,
            "loop": {"start": loop[0], "stop": loop[1], "times": loop[2]},
            "norm": {"eps": eps, "groups": groups}, "vocab": vocab, "width": width}


def make_weights(cfg, seed=0, gain=1.0):
    """Random checkpoint tensors (values representable in bf16) under the design's names."""
    g = torch.Generator().manual_seed(seed)
    Wd, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).bfloat16().float()

    def lin(o, i):
        return rnd(o, i, std=gain / math.sqrt(i))

    W = {"embed": rnd(V, Wd), "head": lin(V, Wd), "final.norm": 1 + rnd(Wd, std=0.1)}
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        W[p + "norm1"] = 1 + rnd(Wd, std=0.1)
        W[p + "ls1"] = 0.6 + rnd(Wd, std=0.1)
        if l["type"] == "latent_attention":
            H, d, r, vd = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            W[p + "mix.dq"] = lin(m["q_rank"], Wd)
            W[p + "mix.dq.norm"] = 1 + rnd(m["q_rank"], std=0.1)
            W[p + "mix.uq"] = lin(H * (d + r), m["q_rank"]) * 2
            W[p + "mix.dkv"] = lin(m["kv_rank"] + r, Wd)
            W[p + "mix.dkv.norm"] = 1 + rnd(m["kv_rank"], std=0.1)
            W[p + "mix.uk"] = lin(H * d, m["kv_rank"]) * 2
            W[p + "mix.uv"] = lin(H * vd, m["kv_rank"])
            W[p + "mix.g"] = lin(H, Wd)
            W[p + "mix.o"] = lin(Wd, H * vd)
        else:
            n = m["width"]
            for k in ("z", "x", "g"):
                W[p + "mix." + k] = lin(n, Wd)
            W[p + "mix.z.b"] = rnd(n)
            W[p + "mix.x.b"] = rnd(n, std=0.5)
            W[p + "mix.o"] = lin(Wd, n)
        f = l.get("mlp")
        if f is not None:
            E, top, ff = f["router"]["experts"], f["router"]["top"], f["expert"]["ff"]
            W[p + "ls2"] = 0.6 + rnd(Wd, std=0.1)
            W[p + "mlp.table"] = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(V)]).int()
            for e in range(E):
                W[f"{p}mlp.e{e}.up"] = lin(ff, Wd)
                W[f"{p}mlp.e{e}.down"] = lin(Wd, ff)
    # what the checkpoint file holds: every float tensor rounded to bf16
    return {k: (v if v.dtype == torch.int32 else v.bfloat16().float()) for k, v in W.items()}


def save_checkpoint(path, cfg, W):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: (v if v.dtype == torch.int32 else v.bfloat16()).contiguous() for k, v in W.items()},
              os.path.join(path, "model.safetensors"))
    return path
