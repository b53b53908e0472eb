"""Plain token-by-token float64 oracle of the Dizepel design: one function
per mechanism, written from the equations, sharing no code with the
serving path. Weights arrive as a dict of checkpoint names -> tensors and
the configuration as the dict that ``config.json`` holds.

Every function walks a whole sequence from position 0 and keeps nothing
between calls; the serving path's caches, portions and batches are checked
against it.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


# ------------------------------------------------------------------ pieces
def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def causal_conv(u, w, bias=None):
    """u [T, C], w [C, K]: y_t = sum_j w[:, j] u_(t-K+1+j), zeros before
    the start."""
    T, C = u.shape
    K = w.shape[1]
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(K):
            s = t - K + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
        if bias is not None:
            y[t] += bias
    return y


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(x)))


def yarn_table(dims, base, scaling):
    """Per-pair frequencies and the multiplier of cos and sin."""
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    if not scaling:
        return f, 1.0
    factor, orig = scaling["factor"], scaling["original"]

    def corr(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (
            2.0 * math.log(base))

    lo = max(math.floor(corr(scaling["fast"])), 0)
    hi = min(math.ceil(corr(scaling["slow"])), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate(x, dims, freqs, mult):
    """x [T, heads, D]; pairs (i, i + dims/2) of the first ``dims``."""
    T = x.shape[0]
    half = dims // 2
    y = x.clone()
    fr = torch.tensor(freqs, dtype=F64)
    for t in range(T):
        a = t * fr
        c, s = torch.cos(a) * mult, torch.sin(a) * mult
        u, v = x[t, :, :half], x[t, :, half:dims]
        y[t, :, :half] = u * c - v * s
        y[t, :, half:dims] = v * c + u * s
    return y


# ------------------------------------------------------------------ mixers
def left_attention(h, W, pre, mc):
    """Causal softmax attention whose values are the unrotated keys, with
    short convolutions on q and k, partial rotation, capped scores and a
    learned sink in the denominator."""
    T = h.shape[0]
    H, G, D = mc["heads"], mc["kv_heads"], mc["dim"]
    q = h @ W[pre + "q"].T + W[pre + "q.b"]
    k = h @ W[pre + "k"].T + W[pre + "k.b"]
    q = causal_conv(q, W[pre + "q.conv"]).view(T, H, D)
    k = causal_conv(k, W[pre + "k.conv"]).view(T, G, D)
    v = k.clone()
    rot = mc.get("rot")
    if rot and rot["dims"]:
        fr, mult = yarn_table(rot["dims"], rot["base"], rot.get("scaling"))
        q = rotate(q, rot["dims"], fr, mult)
        k = rotate(k, rot["dims"], fr, mult)
    cap = mc.get("softcap")
    out = torch.zeros(T, H, D, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        sink = W[pre + "sink"][hh]
        for t in range(T):
            s = (k[:t + 1, g] @ q[t, hh]) * mc["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            m = torch.maximum(s.max(), sink)
            e = torch.exp(s - m)
            den = e.sum() + torch.exp(sink - m)
            out[t, hh] = (e / den) @ v[:t + 1, g]
    return out.reshape(T, H * D) @ W[pre + "o"].T


def right_ssd(h, W, pre, mc, eps):
    """Selective state-space recurrence with scalar decay per head."""
    T = h.shape[0]
    Hh, P, N, G = mc["heads"], mc["vdim"], mc["state"], mc["groups"]
    inner = Hh * P
    u = h @ W[pre + "in"].T
    z = u[:, :inner]
    xbc = u[:, inner:2 * inner + 2 * G * N]
    dt = u[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, W[pre + "conv"], W[pre + "conv.b"]))
    x = xbc[:, :inner].view(T, Hh, P)
    Bm = xbc[:, inner:inner + G * N].view(T, G, N)
    Cm = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + W[pre + "dt_bias"])
    A = -torch.exp(W[pre + "A_log"])
    y = torch.zeros(T, Hh, P, dtype=F64)
    for hh in range(Hh):
        g = hh // (Hh // G)
        S = torch.zeros(N, P, dtype=F64)
        for t in range(T):
            S = torch.exp(A[hh] * dt[t, hh]) * S + dt[t, hh] * torch.outer(
                Bm[t, g], x[t, hh])
            y[t, hh] = S.T @ Cm[t, g] + W[pre + "D"][hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)
    ng = mc["norm_groups"]
    y = unit_rms(y.view(T, ng, inner // ng), eps).reshape(T, inner)
    return (y * W[pre + "norm"]) @ W[pre + "o"].T


def parallel_mixer(h, W, pre, mc, eps):
    a = left_attention(h, W, pre + "left.", mc["left"])
    b = right_ssd(h, W, pre + "right.", mc["right"], eps)
    return 0.5 * (unit_rms(a, eps) * W[pre + "left.out"]
                  + unit_rms(b, eps) * W[pre + "right.out"])


def polynorm_ff(h, W, pre, eps):
    z = h @ W[pre + "up"].T
    a, b, c, e = W[pre + "act"]
    act = (a * unit_rms(z, eps) + b * unit_rms(z * z, eps)
           + c * unit_rms(z * z * z, eps) + e)
    return act @ W[pre + "down"].T


def layer(x, W, i, lc, cfg):
    eps = cfg["norm"]["eps"]
    h = layer_norm(x, W[f"l{i}.norm1"], eps)
    h = h + causal_conv(h, W[f"l{i}.canon1"])
    assert lc["type"] == "parallel"
    y = parallel_mixer(h, W, f"l{i}.mix.", lc["mixer"], eps)
    x = x + layer_norm(y, W[f"l{i}.norm1b"], eps)
    if lc.get("mlp") is not None:
        h = layer_norm(x, W[f"l{i}.norm2"], eps)
        h = h + causal_conv(h, W[f"l{i}.canon2"])
        y = polynorm_ff(h, W, f"l{i}.mlp.", eps)
        x = x + layer_norm(y, W[f"l{i}.norm2b"], eps)
    return x


def layer_runs(cfg):
    """[(layer index, pass number or None)] in execution order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t) for i in range(loop["start"], loop["stop"])]
    runs += [(i, None) for i in range(loop["stop"], n)]
    return runs


def model(tokens, W, cfg, want_layers=False):
    """Logits [T, vocab] (and the residual after every layer run)."""
    W = {k: v.to(F64) for k, v in W.items()}
    x = W["embed"][torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    sums = []
    loop = cfg.get("loop")
    for i, t in layer_runs(cfg):
        if t is not None and i == loop["start"]:
            x = x + W["loop.step"][t]
        x = layer(x, W, i, cfg["layers"][i], cfg)
        sums.append(x.clone())
    x = layer_norm(x, W["final.norm"], cfg["norm"]["eps"])
    logits = x @ W["head"].T
    return (logits, sums) if want_layers else logits
