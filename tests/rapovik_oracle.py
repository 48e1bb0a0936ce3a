"""A slow, whole-sequence implementation of the Rapovik design in plain fp32 (or fp64) PyTorch: one function per
mechanism, written from the equations, sharing no code with the package.  ``forward`` runs one sequence from its
first token and returns the logits of every position (and, on request, the residual after every layer run).

Weights are a dict of tensors under the checkpoint's names; ``cfg`` is the parsed ``config.json``.
"""
from __future__ import annotations

import json
import math
import os

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    """RMS norm whose gain is stored as an offset from one."""
    return rms(x, eps) * (1.0 + w)


def rotate_pairs(x, pos, base, dims):
    """x [..., T, n]: dimensions (2i, 2i + 1), i < dims / 2, turn by pos * base^(-2i / dims); the rest pass."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=x.dtype)
    ang = pos.to(x.dtype)[:, None] * base ** (-2.0 * i / dims)[None, :]
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_attention(h, w, m, eps):
    """h [T, W].  Keys and values come from a low-rank latent; one rotated key part serves every head."""
    T = h.shape[0]
    H, D, P, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w["q"].T).view(T, H, D + P)
    down = h @ w["dkv"].T
    c = rms(down[:, :R], eps) * w["dkv.norm"]
    k_rot = down[:, R:]
    rot = m.get("rot") or {}
    pos = torch.arange(T)
    if rot:
        dims = int(rot.get("dims", P))
        k_rot = rotate_pairs(k_rot, pos, float(rot["base"]), dims)
        q_rot = rotate_pairs(q[:, :, D:].transpose(0, 1), pos, float(rot["base"]), dims).transpose(0, 1)
    else:
        q_rot = q[:, :, D:]
    k = (c @ w["uk"].T).view(T, H, D)
    v = (c @ w["uv"].T).view(T, H, Dv)
    sc = torch.einsum("ihd,jhd->hij", q[:, :, :D], k) + torch.einsum("ihd,jd->hij", q_rot, k_rot)
    sc = sc * float(m["scale"])
    i, j = pos[:, None], pos[None, :]
    seen = j <= i
    size = (m.get("mask") or {}).get("size")
    if size:
        seen = seen & (i - j < int(size))
    sc = sc.masked_fill(~seen[None], float("-inf"))
    o = torch.einsum("hij,jhd->ihd", torch.softmax(sc, -1), v)
    return o.reshape(T, H * Dv) @ w["o"].T


def silu(x):
    return x * torch.sigmoid(x)


def mamba2(h, w, m, eps):
    T = h.shape[0]
    H, Dv, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = H * Dv
    p = h @ w["in"].T
    z, xbc, dt = p[:, :inner], p[:, inner: 2 * inner + 2 * G * N], p[:, 2 * inner + 2 * G * N:]
    padded = torch.cat([xbc.new_zeros(taps - 1, xbc.shape[1]), xbc])
    conv = sum(padded[t: t + T] * w["conv"][:, t] for t in range(taps)) + w["conv.b"]
    xbc = silu(conv)
    x = xbc[:, :inner].view(T, H, Dv)
    B = xbc[:, inner: inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = torch.nn.functional.softplus(dt + w["dt_bias"], threshold=1e9)
    decay = torch.exp(-torch.exp(w["A_log"]) * dt)                   # [T, H]
    grp = torch.arange(H) // (H // G)
    S = h.new_zeros(H, N, Dv)
    ys = []
    for t in range(T):
        Bt, Ct = B[t, grp], C[t, grp]                                  # [H, N]
        S = decay[t, :, None, None] * S + dt[t, :, None, None] * Bt[:, :, None] * x[t, :, None, :]
        ys.append(torch.einsum("hnd,hn->hd", S, Ct) + w["D"][:, None] * x[t])
    y = torch.stack(ys).reshape(T, inner) * silu(z)
    parts = int(m.get("norm_groups", 1))
    y = rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w["norm"]
    return y @ w["o"].T


def mlstm(h, w, m, eps):
    T = h.shape[0]
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = (h @ w["q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w["k"].T).view(T, H, D)
    v = (h @ w["v"].T).view(T, H, Dv)
    ig = cap * torch.tanh((h @ w["i"].T + w["i.b"]) / cap)                                          # [T, H], log
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ w["f"].T + w["f.b"]) / cap))
    S = h.new_zeros(H, D, Dv)
    n = h.new_zeros(H, D)
    mx = h.new_zeros(H)
    outs = []
    for t in range(T):
        m_new = torch.maximum(fg[t] + mx, ig[t])
        a, b = torch.exp(fg[t] + mx - m_new), torch.exp(ig[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t, :, :, None] * v[t, :, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        mx = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        outs.append(num / den[:, None])
    o = rms(torch.stack(outs), eps).reshape(T, H * Dv) * w["norm"]
    o = o * torch.sigmoid(h @ w["g"].T)
    return o @ w["o"].T


def gated_ff(h, w, limit, bias):
    g = h @ w["gate"].T + (w["gate.b"] if bias else 0.0)
    u = h @ w["up"].T + (w["up.b"] if bias else 0.0)
    g = g.clamp(max=limit)
    u = u.clamp(-limit, limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    return y @ w["down"].T + (w["down.b"] if bias else 0.0)


def route(h, w, r):
    """Returns (chosen expert ids [T, top], their weights [T, top])."""
    s = torch.sigmoid(h @ w["router"].T)
    choice = s + w["correction"] if "correction" in w else s.clone()
    E = s.shape[1]
    groups = r.get("groups")
    if groups and int(groups["count"]) > 1:
        cnt, keep = int(groups["count"]), int(groups["keep"])
        per = choice.view(-1, cnt, E // cnt)
        gscore = per.topk(min(2, E // cnt), -1).values.sum(-1)
        best = gscore.topk(keep, -1).indices
        allow = torch.zeros_like(gscore, dtype=torch.bool).scatter_(1, best, True)
        choice = per.masked_fill(~allow[:, :, None], float("-inf")).reshape(-1, E)
    ids = choice.topk(int(r["top"]), -1).indices
    return ids, s.gather(1, ids)


def moe(h, w, mlp):
    ids, wts = route(h, w, mlp["router"])
    out = torch.zeros_like(h)
    lim = float(mlp["expert"]["limit"])
    for t in range(h.shape[0]):
        for e, a in zip(ids[t].tolist(), wts[t]):
            we = {k[len(f"e{e}."):]: v for k, v in w.items() if k.startswith(f"e{e}.")}
            out[t] += a * gated_ff(h[t: t + 1], we, lim, False)[0]
    if mlp.get("shared"):
        ws = {k[len("shared."):]: v for k, v in w.items() if k.startswith("shared.")}
        out = out + gated_ff(h, ws, float(mlp["shared"]["limit"]), False)
    return out


MIXERS = {"latent_attention": latent_attention, "mamba2": mamba2, "mlstm": mlstm}


def layer_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, dtype=torch.float32, want_layers=False):
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    trail = []
    for i in layer_order(cfg):
        spec = cfg["layers"][i]
        lw = sub(W, f"l{i}.")
        y = MIXERS[spec["type"]](norm_around_zero(x, lw["norm1"], eps), sub(lw, "mix."), spec["mixer"], eps)
        x = x + norm_around_zero(y, lw["norm1b"], eps)
        mlp = spec.get("mlp")
        if mlp is not None:
            hin = norm_around_zero(x, lw["norm2"], eps)
            if mlp.get("kind", "dense") == "dense":
                y = gated_ff(hin, sub(lw, "mlp."), float(mlp["limit"]), True)
            else:
                y = moe(hin, sub(lw, "mlp."), mlp)
            x = x + norm_around_zero(y, lw["norm2b"], eps)
        trail.append(x)
    logits = norm_around_zero(x, W["final.norm"], eps) @ W["head"].T
    return (logits, torch.stack(trail)) if want_layers else logits


# ---- small random models ---------------------------------------------------------------------------------------------
def attention_layer(heads=3, dim=12, rot_dim=8, vdim=20, kv_rank=24, window=9, base=100.0, rot_dims=None, scale=0.3,
                    mlp="dense"):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if base:
        m["rot"] = {"base": base, "dims": rot_dims or rot_dim}
    return {"type": "latent_attention", "mixer": m, "mlp": feed_forward(mlp)}


def mamba_layer(heads=4, vdim=12, state=16, groups=2, conv=4, norm_groups=2, mlp="moe"):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}, "mlp": feed_forward(mlp)}


def mlstm_layer(heads=2, dim=12, vdim=20, gate_cap=15.0, mlp="dense"):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap},
            "mlp": feed_forward(mlp)}


def feed_forward(kind, ff=40, limit=1.5, experts=6, top=2, groups=(3, 2), shared=24):
    if kind is None or isinstance(kind, dict):
        return kind
    if kind == "dense":
        return {"kind": "dense", "ff": ff, "limit": limit}
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "router": router, "expert": {"ff": ff // 2, "limit": limit}}
    if shared:
        out["shared"] = {"ff": shared, "limit": limit + 0.5}
    return out


def make_config(layers, vocab=96, width=48, eps=1e-5, loop=None):
    cfg = {"architecture": "Rapovik", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps}}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_weights(cfg, seed=0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    Wd, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, s=1.0):
        return torch.randn(*shape, generator=g) * s

    def lin(o, i, s=1.0):
        return rnd(o, i, s=s / math.sqrt(i))
    W = {"embed": rnd(V, Wd), "head": lin(V, Wd, 2.0), "final.norm": rnd(Wd, s=0.1)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        for n in ("norm1", "norm1b"):
            W[p + n] = rnd(Wd, s=0.1)
        if L["type"] == "latent_attention":
            H, D, P, E, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            W.update({p + "mix.q": lin(H * (D + P), Wd, 2.0), p + "mix.dkv": lin(R + P, Wd, 2.0),
                      p + "mix.dkv.norm": 1.0 + rnd(R, s=0.1), p + "mix.uk": lin(H * D, R, 2.0),
                      p + "mix.uv": lin(H * E, R), p + "mix.o": lin(Wd, H * E)})
        elif L["type"] == "mamba2":
            H, E, N, G, t = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            inner, ch = H * E, H * E + 2 * G * N
            W.update({p + "mix.in": lin(2 * inner + 2 * G * N + H, Wd, 1.5), p + "mix.conv": rnd(ch, t, s=0.5),
                      p + "mix.conv.b": rnd(ch, s=0.2), p + "mix.dt_bias": rnd(H) - 1.0, p + "mix.A_log": rnd(H, s=0.5),
                      p + "mix.D": 1.0 + rnd(H, s=0.2), p + "mix.norm": 1.0 + rnd(inner, s=0.1),
                      p + "mix.o": lin(Wd, inner)})
        else:
            H, D, E = m["heads"], m["dim"], m["vdim"]
            W.update({p + "mix.q": lin(H * D, Wd, 2.0), p + "mix.k": lin(H * D, Wd, 2.0), p + "mix.v": lin(H * E, Wd),
                      p + "mix.g": lin(H * E, Wd), p + "mix.o": lin(Wd, H * E), p + "mix.norm": 1.0 + rnd(H * E, s=0.1),
                      p + "mix.i": lin(H, Wd, 2.0), p + "mix.i.b": rnd(H), p + "mix.f": lin(H, Wd, 2.0),
                      p + "mix.f.b": rnd(H) + 3.0})
        mlp = L.get("mlp")
        if mlp is None:
            continue
        for n in ("norm2", "norm2b"):
            W[p + n] = rnd(Wd, s=0.1)
        if mlp.get("kind", "dense") == "dense":
            ff = mlp["ff"]
            W.update({p + "mlp.gate": lin(ff, Wd, 2.5), p + "mlp.gate.b": rnd(ff, s=0.3), p + "mlp.up": lin(ff, Wd, 2.5),
                      p + "mlp.up.b": rnd(ff, s=0.3), p + "mlp.down": lin(Wd, ff), p + "mlp.down.b": rnd(Wd, s=0.1)})
        else:
            E_, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            W[p + "mlp.router"] = lin(E_, Wd, 3.0)
            W[p + "mlp.correction"] = rnd(E_, s=0.3) - 0.5         # choice scores of either sign
            for e in range(E_):
                W.update({f"{p}mlp.e{e}.gate": lin(ff, Wd, 2.5), f"{p}mlp.e{e}.up": lin(ff, Wd, 2.5),
                          f"{p}mlp.e{e}.down": lin(Wd, ff)})
            if mlp.get("shared"):
                fs = mlp["shared"]["ff"]
                W.update({p + "mlp.shared.gate": lin(fs, Wd, 2.5), p + "mlp.shared.up": lin(fs, Wd, 2.5),
                          p + "mlp.shared.down": lin(Wd, fs)})
    # the checkpoint holds bfloat16: round once, so that oracle and engine read the same numbers
    return {k: v.to(dtype) for k, v in W.items()}


def save_checkpoint(folder, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def logit_error(got, want):
    """Root mean square difference over the vocabulary with the mean taken off, relative to the logits' own spread."""
    d = torch.as_tensor(got).float() - torch.as_tensor(want).float()
    d = d - d.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / torch.as_tensor(want).float().std(-1).clamp_min(1e-6)).max().item()
