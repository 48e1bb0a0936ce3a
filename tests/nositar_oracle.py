"""A plain, slow implementation of the Nositar design for the tests: one function per mechanism, whole sequences at
once, fp32, no cache and no state carried between calls.  It shares nothing with the package's code paths; the
tests compare the engine (CPU backend and HIP kernels) with it.

Notation: T tokens, W model width, H heads, G key/value (or query/key) heads, D key width, E value width.
"""
import json
import math
import os

import torch
import torch.nn.functional as F


# ---- mechanisms ------------------------------------------------------------------------------------------
def unit_rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def scalar_norm(x, gain, eps):
    return unit_rms(x, eps) * gain


def visible(T, window, keep_first):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window:
        ok = ok & ((i - j < window) | (j < keep_first))
    return ok


def sigmoid_attention(x, wq, wk, wv, wo, talk, bias, H, G, D, E, scale, window, keep_first, eps):
    T = x.shape[0]
    q = unit_rms((x @ wq.T).view(T, H, D), eps)
    k = unit_rms((x @ wk.T).view(T, G, D), eps)
    v = (x @ wv.T).view(T, G, E)
    out = torch.zeros(T, H, E)
    raw = torch.zeros(H, T, T)
    for h in range(H):
        raw[h] = (q[:, h] @ k[:, h // (H // G)].T) * scale
    mixed = torch.zeros(H, T, T)
    for h in range(H):
        for g in range(H):
            mixed[h] += talk[h, g] * raw[g]
    ok = visible(T, window, keep_first)
    for h in range(H):
        w = torch.sigmoid(mixed[h] + bias[h]) * ok
        out[:, h] = w @ v[:, h // (H // G)]
    return out.reshape(T, H * E) @ wo.T


def short_conv_silu(x, w):
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros(T, C)
    for t in range(T):
        for a in range(taps):
            s = t - (taps - 1) + a
            if s >= 0:
                y[t] += x[s] * w[:, a]
    return F.silu(y)


def delta_rule(x, P, H, G, D, E, eps):
    """P: dict of the mixer's tensors (q, k, v, q.conv, k.conv, v.conv, b, A_log, a1, a2, dt_bias, g1, g2, norm, o)."""
    T = x.shape[0]
    q = short_conv_silu(x @ P["q"].T, P["q.conv"]).view(T, G, D)
    k = short_conv_silu(x @ P["k"].T, P["k.conv"]).view(T, G, D)
    v = short_conv_silu(x @ P["v"].T, P["v.conv"]).view(T, H, E)
    q = q / torch.sqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) / math.sqrt(D)
    k = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(x @ P["b"].T)
    rate = F.softplus((x @ P["a1"].T) @ P["a2"].T + P["dt_bias"]).view(T, H, D)
    decay = torch.exp(-torch.exp(P["A_log"]).view(1, H, 1) * rate)
    gate = torch.sigmoid((x @ P["g1"].T) @ P["g2"].T).view(T, H, E)
    out = torch.zeros(T, H, E)
    for h in range(H):
        c = h // (H // G)
        S = torch.zeros(D, E)
        for t in range(T):
            S = decay[t, h][:, None] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, c])
            S = S + torch.outer(k[t, c], u)
            out[t, h] = S.T @ q[t, c]
    out = unit_rms(out, eps) * P["norm"] * gate
    return out.reshape(T, H * E) @ P["o"].T


def relu_mlp(x, gate, up, down):
    return (F.relu(x @ gate.T) * (x @ up.T)) @ down.T


# ---- the model ---------------------------------------------------------------------------------------------
def forward(cfg, Wt, tokens, layer_sums=None):
    """Logits [T, vocab] of a whole sequence.  ``Wt``: name -> tensor; everything runs in fp32."""
    W = {k: v.float() for k, v in Wt.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    n = cfg.get("streams")
    xs = [x.clone() for _ in range(n)] if n else None
    for i, L in enumerate(cfg["layers"]):
        m = L["mixer"]
        pre = f"l{i}."
        mix = {k[len(pre) + 4:]: v for k, v in W.items() if k.startswith(pre + "mix.")}

        def mixer(h):
            if L["type"] == "attention":
                mask = m.get("mask") or {}
                return sigmoid_attention(h, mix["q"], mix["k"], mix["v"], mix["o"], mix["talk"], mix["pb"], m["heads"],
                                         m["kv_heads"], m["dim"], m["vdim"], m["scale"], mask.get("size"),
                                         mask.get("keep_first", 0), eps)
            return delta_rule(h, mix, m["heads"], m["kv_heads"], m["dim"], m["vdim"], eps)

        subs = [(1, mixer)]
        if L.get("mlp") is not None:
            subs.append((2, lambda h: relu_mlp(h, W[pre + "mlp.gate"], W[pre + "mlp.up"], W[pre + "mlp.down"])))
        for qi, fn in subs:
            gain = W[f"{pre}norm{qi}"]
            if xs is None:
                x = x + fn(scalar_norm(x, gain, eps))
            else:
                a, b, M = W[f"{pre}hc{qi}.in"], W[f"{pre}hc{qi}.out"], W[f"{pre}hc{qi}.mix"]
                u = sum(a[s] * xs[s] for s in range(n))
                y = fn(scalar_norm(u, gain, eps))
                xs = [sum(M[s, t] * xs[s] for s in range(n)) + b[t] * y for t in range(n)]
        if layer_sums is not None:
            layer_sums.append(sum(xs) if xs is not None else x.clone())
    if xs is not None:
        x = sum(xs)
    logits = scalar_norm(x, W["final.norm"], eps) @ W["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


# ---- small random models -----------------------------------------------------------------------------------
def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, window=12, keep_first=2, ff=48, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5}
    if window:
        m["mask"] = {"size": window, "keep_first": keep_first}
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def delta_layer(heads=2, kv_heads=2, dim=16, vdim=8, conv=4, ff=48, kind="channel_delta"):
    return {"type": kind, "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def make_config(layers, vocab=96, width=32, streams=2, softcap=20.0, embed_scale=2.0, eps=1e-5):
    cfg = {"architecture": "Nositar", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
           "embedding": {"scale": embed_scale}}
    if streams:
        cfg["streams"] = streams
    if softcap:
        cfg["logit_softcap"] = softcap
    return cfg


def make_weights(cfg, seed=0, rank=6, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    Wd, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, s=1.0):
        return torch.randn(*shape, generator=g) * s

    def lin(o, i, s=1.0):
        return rnd(o, i, s=s / math.sqrt(i))
    W = {"embed": rnd(V, Wd), "head": lin(V, Wd, 2.0), "final.norm": torch.tensor(1.0 + 0.1 * rnd(1).item())}
    n = cfg.get("streams")
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        W[p + "norm1"] = torch.tensor(1.0 + 0.1 * rnd(1).item())
        if L["type"] == "attention":
            W.update({p + "mix.q": lin(H * D, Wd, 2.0), p + "mix.k": lin(G * D, Wd, 2.0), p + "mix.v": lin(G * E, Wd),
                      p + "mix.talk": torch.eye(H) + 0.3 * rnd(H, H), p + "mix.pb": rnd(H) - 2.0,
                      p + "mix.o": lin(Wd, H * E)})
        else:
            t = m["conv"]
            W.update({p + "mix.q": lin(G * D, Wd, 2.0), p + "mix.k": lin(G * D, Wd, 2.0), p + "mix.v": lin(H * E, Wd, 2.0),
                      p + "mix.q.conv": rnd(G * D, t, s=0.6), p + "mix.k.conv": rnd(G * D, t, s=0.6),
                      p + "mix.v.conv": rnd(H * E, t, s=0.6), p + "mix.b": lin(H, Wd, 2.0),
                      p + "mix.A_log": rnd(H, s=0.5) - 1.0, p + "mix.norm": 1.0 + 0.1 * rnd(E),
                      p + "mix.a1": lin(rank, Wd), p + "mix.a2": lin(H * D, rank, 2.0), p + "mix.dt_bias": rnd(H * D),
                      p + "mix.g1": lin(rank + 1, Wd), p + "mix.g2": lin(H * E, rank + 1, 2.0),
                      p + "mix.o": lin(Wd, H * E)})
        if L.get("mlp") is not None:
            ff = L["mlp"]["ff"]
            W[p + "norm2"] = torch.tensor(1.0 + 0.1 * rnd(1).item())
            W.update({p + "mlp.gate": lin(ff, Wd, 1.5), p + "mlp.up": lin(ff, Wd, 1.5), p + "mlp.down": lin(Wd, ff)})
        if n:
            for qi in (1, 2) if L.get("mlp") is not None else (1,):
                W[f"{p}hc{qi}.in"] = 1.0 / n + 0.2 * rnd(n)
                W[f"{p}hc{qi}.out"] = 1.0 + 0.2 * rnd(n)
                W[f"{p}hc{qi}.mix"] = torch.eye(n) + 0.15 * rnd(n, n)
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
