"""Plain oracle of the Potosun design, written from its equations only: one
function per mechanism, float64 numpy throughout, whole sequences from
position 0, no cache, no batching, nothing shared with the serving path.

A model is (cfg, W): ``cfg`` the dictionary of config.json and ``W`` a
dictionary tensor name -> numpy array (float64; tables as given).
"""

import math

import numpy as np


def rms(x, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi)
                                    * (z + 0.044715 * z ** 3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


# ------------------------------------------------------------- positions
def plain_frequencies(dims, base):
    return [base ** (-2.0 * i / dims) for i in range(dims // 2)]


def scaled_frequencies(dims, base, sc):
    """Two-regime scaling: (frequencies, multiplier of cos and sin)."""
    def pair_index(turns):
        return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) \
            / (2.0 * math.log(base))
    lo = max(math.floor(pair_index(sc["fast"])), 0)
    hi = min(math.ceil(pair_index(sc["slow"])), dims - 1)
    out = []
    for i, f in enumerate(plain_frequencies(dims, base)):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / sc["factor"] * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(sc["factor"]) + 1.0


def rotate_pairs(x, pos, freqs, mult, first, second):
    """Rotate entries (first[i], second[i]) of the last axis of x by the
    angle pos * freqs[i]; cos and sin are multiplied by ``mult``."""
    out = x.copy()
    for i, f in enumerate(freqs):
        c, s = math.cos(pos * f) * mult, math.sin(pos * f) * mult
        u, v = x[..., first[i]], x[..., second[i]]
        out[..., first[i]] = u * c - v * s
        out[..., second[i]] = v * c + u * s
    return out


def rotate_interleaved(x, pos, dims, base):
    """Pairs (2i, 2i+1) among the first ``dims`` entries."""
    n = dims // 2
    return rotate_pairs(x, pos, plain_frequencies(dims, base), 1.0,
                        [2 * i for i in range(n)],
                        [2 * i + 1 for i in range(n)])


def rotate_halves(x, pos, dims, base, scaling=None):
    """Pairs (i, i + dims/2) among the first ``dims`` entries, optionally
    with the two-regime frequency scaling."""
    n = dims // 2
    if scaling:
        fr, mult = scaled_frequencies(dims, base, scaling)
    else:
        fr, mult = plain_frequencies(dims, base), 1.0
    return rotate_pairs(x, pos, fr, mult, list(range(n)),
                        [i + n for i in range(n)])


# ----------------------------------------------------------------- masks
# a layer without a mask (size None) sees every earlier position
def sees_window_keep(i, j, size, keep):
    return j <= i and (size is None or i - j < size or j < keep)


def sees_chunk(i, j, size):
    return j <= i and (size is None or i // size == j // size)


def sees_window(i, j, size):
    return 0 <= i - j and (size is None or i - j < size)


def mask_of(mc):
    m = mc.get("mask") or {}
    return m.get("size"), m.get("keep_first", 0)


def distance_bucket(n, rows, far):
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(
        math.log(n / half) / math.log(far / half) * (rows - half))))


# --------------------------------------------------------------- softmax
def softmax_rows(scores, sink=None):
    """Softmax of a 1-d score vector; ``sink`` adds exp(sink) to the
    denominator only."""
    m = scores.max() if sink is None else max(scores.max(), sink)
    e = np.exp(scores - m)
    den = e.sum() + (0.0 if sink is None else math.exp(sink - m))
    return e / den


def mix_values(v, mc, P, vmix):
    """Value mixing across layers: the first layer that mixes keeps its
    values and publishes them; later ones blend them in."""
    if not mc.get("v_mix"):
        return v
    if "first" not in vmix:
        vmix["first"] = v
        return v
    lam = float(P["vmix"])
    return (1.0 - lam) * v + lam * vmix["first"].reshape(v.shape)


# ---------------------------------------------------------------- mixers
def biased_attention(h, P, mc, eps, vmix):
    """Position-free scores plus a learned distance bias; sliding window
    that keeps the first tokens; element-wise output gate."""
    H, G, D, V = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    T = h.shape[0]
    q = rms((h @ P["q"].T).reshape(T, H, D), eps) * P["q.norm"]
    k = rms((h @ P["k"].T).reshape(T, G, D), eps) * P["k.norm"]
    v = mix_values((h @ P["v"].T).reshape(T, G, V), mc, P, vmix)
    rel = P["rel"]
    size, keep = mask_of(mc)
    o = np.zeros((T, H, V))
    for i in range(T):
        js = [j for j in range(i + 1) if sees_window_keep(i, j, size, keep)]
        bk = [distance_bucket(i - j, rel.shape[0], mc["bias_max"])
              for j in js]
        for hd in range(H):
            g = hd // (H // G)
            s = (k[js, g] @ q[i, hd]) * mc["scale"] + rel[bk, hd]
            p = softmax_rows(s)
            o[i, hd] = p @ v[js, g]
    o = o.reshape(T, H * V) * sigmoid(h @ P["g"].T)
    return o @ P["o"].T


def chunked_attention(h, P, mc, eps, vmix):
    """Interleaved rotation, attention inside chunks counted from the
    sequence's start, a learned sink logit per head."""
    H, G, D, V = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    T = h.shape[0]
    rot = mc["rot"]
    q = (h @ P["q"].T).reshape(T, H, D)
    k = (h @ P["k"].T).reshape(T, G, D)
    q = np.stack([rotate_interleaved(q[t], t, rot["dims"], rot["base"])
                  for t in range(T)])
    k = np.stack([rotate_interleaved(k[t], t, rot["dims"], rot["base"])
                  for t in range(T)])
    v = mix_values((h @ P["v"].T).reshape(T, G, V), mc, P, vmix)
    size, _ = mask_of(mc)
    o = np.zeros((T, H, V))
    for i in range(T):
        js = [j for j in range(i + 1) if sees_chunk(i, j, size)]
        for hd in range(H):
            g = hd // (H // G)
            s = (k[js, g] @ q[i, hd]) * mc["scale"]
            p = softmax_rows(s, sink=float(P["sink"][hd]))
            o[i, hd] = p @ v[js, g]
    return o.reshape(T, H * V) @ P["o"].T


def latent_attention(h, P, mc, eps):
    """Keys and values expanded per head from one normed latent per token
    plus one rotated key part shared by the heads; sliding window; sink
    logit per head; one output gate per head."""
    H, D, rd, V, R = (mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"],
                      mc["kv_rank"])
    T = h.shape[0]
    rot = mc["rot"]
    assert rot["dims"] == rd
    q = (h @ P["q"].T).reshape(T, H, D + rd)
    d = h @ P["dkv"].T
    c = rms(d[:, :R], eps) * P["dkv.norm"]
    kr = np.stack([rotate_halves(d[t, R:], t, rd, rot["base"],
                                 rot.get("scaling")) for t in range(T)])
    qr = np.stack([rotate_halves(q[t, :, D:], t, rd, rot["base"],
                                 rot.get("scaling")) for t in range(T)])
    ku = (c @ P["uk"].T).reshape(T, H, D)
    vv = (c @ P["uv"].T).reshape(T, H, V)
    gate = sigmoid(h @ P["g"].T)                       # [T, H]
    size, _ = mask_of(mc)
    o = np.zeros((T, H, V))
    for i in range(T):
        js = [j for j in range(i + 1) if sees_window(i, j, size)]
        for hd in range(H):
            s = (ku[js, hd] @ q[i, hd, :D] + kr[js] @ qr[i, hd]) * mc["scale"]
            p = softmax_rows(s, sink=float(P["sink"][hd]))
            o[i, hd] = (p @ vv[js, hd]) * gate[i, hd]
    return o.reshape(T, H * V) @ P["o"].T


def gated_ff(h, P):
    return (gelu_tanh(h @ P["gate"].T) * (h @ P["up"].T)) @ P["down"].T


# ----------------------------------------------------------------- model
def forward(cfg, W, tokens, layer_out=None):
    """Logits [T, vocab] for one sequence from position 0; ``layer_out``
    (a list) receives the residual after every layer."""
    W = {k: np.asarray(v, dtype=np.float64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    tokens = np.asarray(tokens, dtype=np.int64)
    x = W["embed"][tokens] * (cfg.get("embedding") or {}).get("scale", 1.0)
    vmix = {}
    for i, lc in enumerate(cfg["layers"]):
        mc = lc["mixer"]
        pre = f"l{i}.mix."
        P = {k[len(pre):]: v for k, v in W.items() if k.startswith(pre)}
        h = rms(x, eps) * W[f"l{i}.norm1"]
        if lc["type"] == "attention":
            y = biased_attention(h, P, mc, eps, vmix)
        elif lc["type"] == "attention_2":
            y = chunked_attention(h, P, mc, eps, vmix)
        elif lc["type"] == "latent_attention":
            y = latent_attention(h, P, mc, eps)
        else:
            raise KeyError(lc["type"])
        x = x + y
        if lc.get("mlp") is not None:
            assert lc["mlp"]["kind"] == "dense"
            pre = f"l{i}.mlp."
            F = {k[len(pre):]: v for k, v in W.items() if k.startswith(pre)}
            x = x + gated_ff(rms(x, eps) * W[f"l{i}.norm2"], F)
        if layer_out is not None:
            layer_out.append(x.copy())
    z = (rms(x, eps) * W["final.norm"]) @ W["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        z = cap * np.tanh(z / cap)
    return z
