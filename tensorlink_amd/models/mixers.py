"""Building blocks beyond the Llama shape: Dynamic-Tanh norm,
hyper-connected residual streams, matrix-memory (mLSTM) mixer,
differential attention with cross-layer KV sharing, and a group-limited
top-k mixture of experts with squared-ReLU experts.

Every block takes its sizes and constants as constructor arguments, runs
on flat ragged batches (:class:`tensorlink_amd.ops.mixers.RaggedMeta`) and
keeps its per-sequence memory in the slot/page cache handed to it
(:class:`tensorlink_amd.models.paged.HybridSlotCache`), so a model file
only assembles them by configuration.

Precision: what feeds a norm, a router, a gate of a recurrence, a score or
the residual is fp32 whatever the serving dtype; the big projections and
expert GEMMs run in the serving dtype with fp32 accumulation.
"""

from __future__ import annotations

import os
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from tensorlink_amd import ops
from tensorlink_amd.models.dense import TLLinear
from tensorlink_amd.ops import mixers as mx


class _F32Cache:
    """fp32 contiguous copies of small parameters, rebuilt when the
    parameter is written or moved (the module may be stored in bf16)."""

    def _f32(self, name: str) -> torch.Tensor:
        p = getattr(self, name)
        store = self.__dict__.setdefault("_f32_store", {})
        key = (p.data_ptr(), p._version, p.device, p.dtype)
        hit = store.get(name)
        if hit is None or hit[0] != key:
            hit = (key, p.detach().float().contiguous())
            store[name] = hit
        return hit[1]


class DynamicTanh(nn.Module, _F32Cache):
    """y = tanh(alpha * x) * weight + bias; no mean, no variance."""

    def __init__(self, width: int):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(width))
        self.bias = nn.Parameter(torch.zeros(width))
        self.alpha = nn.Parameter(torch.ones(()))

    def params(self):
        return (self._f32("alpha").reshape(1), self._f32("weight"),
                self._f32("bias"))


class HyperConnection(nn.Module, _F32Cache):
    """Read weights ``inw`` [ns], write weights ``out`` [ns] and stream
    mixing matrix ``mix`` [from, to] of one sublayer."""

    def __init__(self, streams: int):
        super().__init__()
        self.inw = nn.Parameter(torch.full((streams,), 1.0 / streams))
        self.out = nn.Parameter(torch.ones(streams))
        self.mix = nn.Parameter(torch.eye(streams))


class MLSTMMixer(nn.Module, _F32Cache):
    """Matrix-memory mixer: fused q|k|v|g projection, fp32 soft-capped
    gates, the slot-state recurrence kernel, output projection."""

    kind = "mlstm"

    def __init__(self, width: int, heads: int, dim: int, vdim: int,
                 gate_cap: float, eps: float):
        super().__init__()
        self.H, self.D, self.V = heads, dim, vdim
        self.cap, self.eps = float(gate_cap), float(eps)
        hd, hv = heads * dim, heads * vdim
        self.offs = (0, hd, 2 * hd, 2 * hd + hv)
        self.proj = TLLinear(width, 2 * hd + 2 * hv, bias=False)
        self.gate = nn.Linear(width, 2 * heads, bias=True)   # input | forget
        self.norm = nn.Parameter(torch.ones(hv))
        self.o_proj = TLLinear(hv, width, bias=False)

    def cache_spec(self):
        return {"kind": "mlstm", "H": self.H, "D": self.D, "V": self.V}

    def forward(self, h, meta, cache, layer_idx):
        proj = self.proj(h)
        gw = self.gate.weight
        if gw.dtype != torch.float32:
            store = self.__dict__.setdefault("_gate32", None)
            key = (gw.data_ptr(), gw._version, self.gate.bias._version)
            if store is None or store[0] != key:
                store = (key, gw.detach().float(),
                         self.gate.bias.detach().float())
                self.__dict__["_gate32"] = store
            gates = F.linear(h.float(), store[1], store[2])
        else:
            gates = F.linear(h.float(), gw, self.gate.bias)
        S, n, m = cache.state[layer_idx]
        o = mx.mlstm_scan(proj, self.offs, gates, self._f32("norm"), S, n, m,
                          meta, self.H, self.D, self.V, self.cap, self.eps)
        return self.o_proj(o)


class DiffAttention(nn.Module, _F32Cache):
    """Two-map (differential) softmax attention over the paged pool, GQA,
    position-free scores. ``kv_from`` = index of an earlier layer whose
    key/value pools this layer reads instead of projecting its own."""

    kind = "attention"

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int,
                 vdim: int, scale: float, diff: float, eps: float,
                 kv_from: Optional[int] = None):
        super().__init__()
        assert heads % kv_heads == 0
        self.H, self.G, self.D, self.V = heads, kv_heads, dim, vdim
        self.scale, self.diff, self.eps = float(scale), float(diff), float(eps)
        self.kv_from = kv_from
        self.q_cols = heads * 2 * dim
        self.k_cols = 0 if kv_from is not None else kv_heads * 2 * dim
        self.v_cols = 0 if kv_from is not None else kv_heads * vdim
        self.qkv = TLLinear(width, self.q_cols + self.k_cols + self.v_cols,
                            bias=False)
        self.lq1 = nn.Parameter(torch.zeros(dim))
        self.lk1 = nn.Parameter(torch.zeros(dim))
        self.lq2 = nn.Parameter(torch.zeros(dim))
        self.lk2 = nn.Parameter(torch.zeros(dim))
        self.o_proj = TLLinear(heads * vdim, width, bias=False)

    def cache_spec(self):
        if self.kv_from is not None:
            return {"kind": "kv_ref", "src": self.kv_from}
        return {"kind": "kv", "G": self.G, "DK": 2 * self.D, "V": self.V}

    def lam(self) -> torch.Tensor:
        """exp(lq1.lk1) - exp(lq2.lk2) + diff as a 1-element fp32 tensor,
        recomputed only when a lambda parameter changes."""
        key = tuple((p.data_ptr(), p._version) for p in
                    (self.lq1, self.lk1, self.lq2, self.lk2))
        hit = self.__dict__.get("_lam")
        if hit is None or hit[0] != key:
            v = (torch.exp((self.lq1.float() * self.lk1.float()).sum())
                 - torch.exp((self.lq2.float() * self.lk2.float()).sum())
                 + self.diff).reshape(1).detach()
            hit = (key, v)
            self.__dict__["_lam"] = hit
        return hit[1]

    def forward(self, h, meta, cache, layer_idx):
        proj = self.qkv(h)
        src = layer_idx if self.kv_from is None else self.kv_from
        kpool, vpool = cache.k[src], cache.v[src]
        if self.kv_from is None:
            mx.kv_append(proj, self.q_cols, self.q_cols + self.k_cols,
                         kpool, vpool, meta)
        o = mx.diff_attention(proj, 0, kpool, vpool, meta, self.lam(),
                              self.H, self.D, self.scale, self.diff,
                              self.eps)
        return self.o_proj(o)


class GroupLimitedMoE(nn.Module, _F32Cache):
    """Mixture of two-matrix experts (down(relu(up x)^2), no biases) under
    a softmax router with group-limited top-k selection."""

    def __init__(self, width: int, ff: int, experts: int, top: int,
                 n_groups: int, keep_groups: int, route_scale: float):
        super().__init__()
        assert experts % n_groups == 0 and keep_groups <= n_groups
        assert top <= keep_groups * (experts // n_groups)
        self.W, self.ff, self.E, self.top = width, ff, experts, top
        self.n_groups, self.keep = n_groups, keep_groups
        self.route_scale = float(route_scale)
        self.router = nn.Parameter(torch.zeros(experts, width))
        self.up = nn.Parameter(torch.zeros(experts, ff, width))
        self.down = nn.Parameter(torch.zeros(experts, width, ff))

    def _grouped_ok(self, h) -> bool:
        return (h.is_cuda and h.dtype == torch.bfloat16
                and ops.extension_loaded()
                and self.W % 64 == 0 and self.ff % 64 == 0
                and not os.environ.get("TL_NO_GROUPED_MOE"))

    def _tables(self, dev):
        key = (self.up.data_ptr(), self.down.data_ptr(), str(dev))
        hit = self.__dict__.get("_ptrs")
        if hit is None or hit[0] != key:
            mk = lambda p: torch.tensor(
                [p[e].data_ptr() for e in range(self.E)],
                dtype=torch.int64, device=dev)
            hit = (key, mk(self.up), mk(self.down))
            self.__dict__["_ptrs"] = hit
        return hit[1], hit[2]

    def forward(self, h):
        T = h.shape[0]
        logits = F.linear(h.float(), self._f32("router"))
        w, idx = mx.group_limited_router(logits, self.top, self.n_groups,
                                         self.keep, self.route_scale)
        if self._grouped_ok(h):
            # grouped expert GEMMs over expert-sorted (token, choice) pairs
            # (ops/csrc/moe_gemm.hip); fixed-order fp32 combine, no atomics
            C = ops._require_ext()
            dev = h.device
            up_p, down_p = self._tables(dev)
            fi = idx.reshape(-1)
            order = fi.argsort(stable=True)
            counts = torch.zeros(self.E, device=dev, dtype=torch.long)
            counts.scatter_add_(0, fi, torch.ones_like(fi))
            seg = torch.zeros(self.E + 1, device=dev, dtype=torch.int32)
            seg[1:] = counts.cumsum(0)
            pair_tok = (order // self.top).to(torch.int32)
            a = C.moe_gemm(h.contiguous(), pair_tok, seg, up_p, None,
                           self.ff, False)
            a = mx.relu_squared(a)
            y = C.moe_gemm(a, None, seg, down_p, None, self.W, False)
            y = y.float() * w.reshape(-1)[order].unsqueeze(1)
            inv = torch.empty_like(order)
            inv[order] = torch.arange(order.numel(), device=dev,
                                      dtype=order.dtype)
            return y[inv].view(T, self.top, self.W).sum(1).to(h.dtype)
        out = torch.zeros(T, self.W, device=h.device, dtype=torch.float32)
        for e in range(self.E):
            tok, choice = (idx == e).nonzero(as_tuple=True)
            if tok.numel() == 0:
                continue
            a = mx.relu_squared(F.linear(h[tok], self.up[e]))
            out.index_add_(0, tok, F.linear(a, self.down[e]).float()
                           * w[tok, choice, None])
        return out.to(h.dtype)


# ---------------------------------------------------------------------------
# blocks of the post-norm layered family: lightning (decayed linear)
# attention, latent attention, windowed attention with score mixing and a
# sink, plain two-matrix feed-forward, per-layer token input
# ---------------------------------------------------------------------------
class RMSWeight(nn.Module, _F32Cache):
    """Weight of an RMS norm; ``one_plus`` = stored around zero and
    applied as (1 + w)."""

    def __init__(self, width: int, one_plus: bool):
        super().__init__()
        self.one_plus = bool(one_plus)
        self.weight = nn.Parameter(torch.zeros(width) if one_plus
                                   else torch.ones(width))

    def w32(self):
        return self._f32("weight")


class LightningMixer(nn.Module, _F32Cache):
    """Linear attention with one fixed decay per head: fused q|k|v|g
    projection, silu on q, k, v, the slot-state recurrence
    S <- decay S + k v^T, read-out S^T q, one RMS norm over all heads
    together, sigmoid output gate, output projection."""

    kind = "lightning"

    def __init__(self, width: int, heads: int, dim: int, vdim: int,
                 decay, eps: float):
        super().__init__()
        assert len(decay) == heads
        self.H, self.D, self.V, self.eps = heads, dim, vdim, float(eps)
        hd, hv = heads * dim, heads * vdim
        self.offs = (0, hd, 2 * hd, 2 * hd + hv)
        self.proj = TLLinear(width, 2 * hd + 2 * hv, bias=False)
        self.norm = nn.Parameter(torch.ones(hv))
        self.o_proj = TLLinear(hv, width, bias=False)
        # a constant of the design, not a parameter: kept out of the
        # module's tensors so that a cast of the module to the serving
        # dtype cannot round it
        self.decay = tuple(float(x) for x in decay)

    def cache_spec(self):
        return {"kind": "state", "shapes": [(self.H, self.D, self.V)]}

    def _decay32(self, dev):
        hit = self.__dict__.get("_dec")
        if hit is None or hit.device != dev:
            hit = torch.tensor(self.decay, dtype=torch.float64).to(
                device=dev, dtype=torch.float32)
            self.__dict__["_dec"] = hit
        return hit

    def forward(self, h, meta, cache, layer_idx):
        proj = self.proj(h)
        (S,) = cache.state[layer_idx]
        o = mx.lightning_scan(proj, self.offs[:3], self._decay32(h.device),
                              S, meta, self.H, self.D, self.V)
        y = mx.rms_scale(o, self._f32("norm"), self.eps, False, gate=proj,
                         gate_col=self.offs[3], out_dtype=h.dtype)
        return self.o_proj(y)


class LatentAttention(nn.Module, _F32Cache):
    """Attention whose cache holds, per token, one normed latent c
    [kv_rank] and one rotated key part [rot_dim] shared by all heads.

    Keys and values are linear in c (k_h = W_uk,h c, v_h = W_uv,h c), so
    the heads' unrotated queries are carried into latent space
    (q'_h = W_uk,h^T q_h) and every head attends the SAME cached rows
    [c | k_rot] (one shared key head, values = the first kv_rank columns
    of the row); W_uv is applied to the attended latent afterwards. The
    per-head keys and values are never materialised. ``kv_from`` = index
    of an earlier latent layer whose cached rows this layer reads with its
    own W_uk / W_uv and queries.

    Options: ``window`` > 0 = sliding window; ``rot_scaling`` = two-regime
    frequency scaling of the rotation (see ``ops.mixers.yarn_freqs``);
    ``sink_logits`` = one learned logit per head in the softmax denominator
    (``sink``); ``head_gate`` = head h's output times sigmoid of one more
    projection of the input (``g`` rows of the fused projection, one per
    head). A scalar gate commutes with W_uv, so it is applied to the
    attended latent where the attention kernel writes it."""

    kind = "latent_attention"

    def __init__(self, width: int, heads: int, dim: int, rot_dim: int,
                 vdim: int, kv_rank: int, scale: float, rot_base: float,
                 eps: float, kv_from: Optional[int] = None, *,
                 window: int = 0, rot_scaling: Optional[dict] = None,
                 sink_logits: bool = False, head_gate: bool = False):
        super().__init__()
        assert rot_dim % 2 == 0
        self.H, self.D, self.RD, self.V, self.R = (heads, dim, rot_dim, vdim,
                                                   kv_rank)
        self.scale, self.eps, self.base = float(scale), float(eps), rot_base
        self.kv_from = kv_from
        self.window = int(window)
        self.rot_scaling = dict(rot_scaling) if rot_scaling else None
        self.q_cols = heads * (dim + rot_dim)
        self.kv_cols = 0 if kv_from is not None else kv_rank + rot_dim
        self.g_cols = heads if head_gate else 0
        self.qdkv = TLLinear(width, self.q_cols + self.kv_cols + self.g_cols,
                             bias=False)
        self.sink = nn.Parameter(torch.zeros(heads)) if sink_logits else None
        if kv_from is None:
            self.dkv_norm = nn.Parameter(torch.ones(kv_rank))
        self.uk = nn.Parameter(torch.zeros(heads * dim, kv_rank))
        self.uv = nn.Parameter(torch.zeros(heads * vdim, kv_rank))
        self.o_proj = TLLinear(heads * vdim, width, bias=False)

    def cache_spec(self):
        if self.kv_from is not None:
            return {"kind": "kv_ref", "src": self.kv_from}
        return {"kind": "kv", "G": 1, "DK": self.R + self.RD, "V": 0}

    def _freqs(self, dev):
        """(frequencies, multiplier of cos and sin)."""
        hit = self.__dict__.get("_fr")
        if hit is None or hit[0].device != dev:
            hit = mx.yarn_freqs(self.RD, self.base, self.rot_scaling, dev)
            self.__dict__["_fr"] = hit
        return hit

    def forward(self, h, meta, cache, layer_idx, shared=None):
        H, D, RD, R, V = self.H, self.D, self.RD, self.R, self.V
        T = h.shape[0]
        proj = self.qdkv(h)
        fr, mult = self._freqs(h.device)
        src = layer_idx if self.kv_from is None else self.kv_from
        pool = cache.k[src]
        if self.kv_from is None:
            mx.norm_rope_rows(proj, self.q_cols, 1, R + RD, meta,
                              norm_w=self._f32("dkv_norm"), norm_cols=R,
                              eps=self.eps, rot_off=R, rot_dims=RD,
                              freqs=fr, rot_mult=mult, pool=pool)
        q = mx.norm_rope_rows(proj, 0, H, D + RD, meta, rot_off=D,
                              rot_dims=RD, freqs=fr,
                              rot_mult=mult).view(T, H, D + RD)
        qa = torch.empty(T, H, R + RD, device=h.device, dtype=torch.float32)
        qa[:, :, R:] = q[:, :, D:]
        torch.bmm(q[:, :, :D].transpose(0, 1),
                  self._f32("uk").view(H, D, R),
                  out=qa[:, :, :R].transpose(0, 1))
        o = mx.flex_attention(
            qa.view(T, H * (R + RD)), pool, None, meta, H, self.scale,
            v_cols=R, window=self.window,
            sink_logits=self._f32("sink") if self.sink is not None else None,
            gate=proj if self.g_cols else None,
            gate_col=self.q_cols + self.kv_cols, gate_heads=True)
        o = torch.bmm(o.view(T, H, R).transpose(0, 1),
                      self._f32("uv").view(H, V, R).transpose(1, 2))
        return self.o_proj(o.transpose(0, 1).reshape(T, H * V).to(h.dtype))


class WindowAttention(nn.Module, _F32Cache):
    """Grouped-query softmax attention over the paged pool with: one RMS
    norm over the WHOLE query projection and one over the whole key
    projection (plain weights, before rotation); rotate-half positions on
    the first ``rot_dims`` dimensions of every head; a learned [H, H]
    mixing of the heads' scores before the softmax (``talk``); a sliding
    window (``window`` = 0: plain causal); a sink (one added to the
    softmax denominator).

    Further options, all off by default:
    ``head_norm``    the query / key norm is per head over ``dim`` with one
                     weight [dim] shared by the heads;
    ``interleaved``  rotation pairs are (2i, 2i+1) instead of halves;
    ``chunk``        instead of a window: a query sees the keys of its own
                     chunk of this many positions, counted from position 0;
    ``keep_first``   the first positions stay visible beyond the window;
    ``sink_logits``  a learned logit per head in the denominator (``sinks``)
                     instead of the constant one;
    ``rel_rows``, ``rel_far``  a learned distance bias ``rel``
                     [rel_rows, heads] added to the scaled score, distances
                     bucketed exactly up to rel_rows / 2 and geometrically up
                     to ``rel_far`` (``ops.mixers.log_distance_buckets``);
    ``out_gate``     the concatenated heads times sigmoid of one more
                     projection of the input (``g`` rows of the fused
                     projection);
    ``v_mix``        value mixing across layers: the first such layer of a
                     model publishes its values of the step's tokens in the
                     ``shared`` dictionary handed to forward, later ones
                     cache (1 - vmix) v + vmix v_first (``vmix`` a learned
                     scalar); the mixing layers must agree in kv_heads *
                     vdim."""

    kind = "attention"

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int,
                 vdim: int, scale: float, rot_dims: int, rot_base: float,
                 window: int, eps: float, sink: bool = True,
                 talk: bool = True, qk_norm: bool = True, *,
                 head_norm: bool = False, interleaved: bool = False,
                 chunk: int = 0, keep_first: int = 0,
                 sink_logits: bool = False, rel_rows: int = 0,
                 rel_far: float = 0.0, out_gate: bool = False,
                 v_mix: bool = False):
        super().__init__()
        assert heads % kv_heads == 0 and rot_dims % 2 == 0 and rot_dims <= dim
        assert not (chunk and window), "a chunked mask has no window"
        self.H, self.G, self.D, self.V = heads, kv_heads, dim, vdim
        self.scale, self.eps = float(scale), float(eps)
        self.rot_dims, self.base = int(rot_dims), rot_base
        self.window, self.sink = int(window), bool(sink or sink_logits)
        self.head_norm, self.interleaved = bool(head_norm), bool(interleaved)
        self.chunk, self.keep_first = int(chunk), int(keep_first)
        self.rel_rows, self.rel_far = int(rel_rows), float(rel_far)
        self.v_mix = bool(v_mix)
        self.q_cols, self.k_cols = heads * dim, kv_heads * dim
        self.v_cols = kv_heads * vdim
        self.g_cols = heads * vdim if out_gate else 0
        self.qkv = TLLinear(width, self.q_cols + self.k_cols + self.v_cols
                            + self.g_cols, bias=False)
        self.q_norm = nn.Parameter(torch.ones(
            dim if head_norm else self.q_cols)) if qk_norm else None
        self.k_norm = nn.Parameter(torch.ones(
            dim if head_norm else self.k_cols)) if qk_norm else None
        self.talk = nn.Parameter(torch.eye(heads)) if talk else None
        self.sinks = nn.Parameter(torch.zeros(heads)) if sink_logits \
            else None
        self.rel = nn.Parameter(torch.zeros(rel_rows, heads)) if rel_rows \
            else None
        self.vmix = nn.Parameter(torch.zeros(())) if v_mix else None
        if rel_rows:
            self.buckets = mx.log_distance_buckets(rel_rows, rel_far)
        self.o_proj = TLLinear(heads * vdim, width, bias=False)

    def cache_spec(self):
        return {"kind": "kv", "G": self.G, "DK": self.D, "V": self.V}

    def _freqs(self, dev):
        hit = self.__dict__.get("_fr")
        if hit is None or hit.device != dev:
            hit = mx.rope_freqs(self.rot_dims, self.base, dev)
            self.__dict__["_fr"] = hit
        return hit

    def _dist_bias(self, dev):
        """The distance bias spread over distances: fp32 [H, n] with
        entry [h, d] = rel[bucket(d), h]; the last column serves every
        larger distance. Rebuilt when ``rel`` changes."""
        p = self.rel
        key = (p.data_ptr(), p._version, p.device)
        hit = self.__dict__.get("_lut")
        if hit is None or hit[0] != key:
            idx = torch.tensor(self.buckets, dtype=torch.long,
                               device=p.device)
            hit = (key, p.detach().float().t()[:, idx].contiguous())
            self.__dict__["_lut"] = hit
        return hit[1]

    def forward(self, h, meta, cache, layer_idx, shared=None):
        proj = self.qkv(h)
        fr = self._freqs(h.device) if self.rot_dims else None
        qn = self._f32("q_norm") if self.q_norm is not None else None
        kn = self._f32("k_norm") if self.k_norm is not None else None
        kpool, vpool = cache.k[layer_idx], cache.v[layer_idx]
        v_col = self.q_cols + self.k_cols
        rot = dict(rot_dims=self.rot_dims, freqs=fr,
                   interleaved=self.interleaved, head_norm=self.head_norm,
                   eps=self.eps)
        mx.norm_rope_rows(proj, self.q_cols, self.G, self.D, meta,
                          norm_w=kn, norm_cols=self.k_cols, pool=kpool, **rot)
        first = None
        if self.v_mix:
            if shared is None:
                raise ValueError("value mixing needs the step's shared "
                                 "dictionary")
            first = shared.get("v_first")
            if first is None:
                shared["v_first"] = (proj, v_col, self.v_cols)
            elif first[2] != self.v_cols:
                raise ValueError("value-mixing layers differ in "
                                 "kv_heads * vdim")
        if first is None:
            mx.norm_rope_rows(proj, v_col, self.G, self.V, meta, pool=vpool)
        else:
            mx.norm_rope_rows(proj, v_col, self.G, self.V, meta, pool=vpool,
                              mix_src=first[0], mix_col=first[1],
                              mix_lam=self._f32("vmix").reshape(1))
        q = mx.norm_rope_rows(proj, 0, self.H, self.D, meta, norm_w=qn,
                              norm_cols=self.q_cols, **rot)
        o = mx.flex_attention(
            q, kpool, vpool, meta, self.H, self.scale, window=self.window,
            sink=self.sink,
            talk=self._f32("talk") if self.talk is not None else None,
            sink_logits=self._f32("sinks") if self.sinks is not None
            else None,
            chunk=self.chunk, keep_first=self.keep_first,
            dist_bias=self._dist_bias(h.device) if self.rel is not None
            else None,
            gate=proj if self.g_cols else None,
            gate_col=v_col + self.v_cols, out_dtype=h.dtype)
        return self.o_proj(o)


class DenseFF(nn.Module):
    """down(gelu(up x)), exact (erf) or tanh-form GELU, no biases."""

    def __init__(self, width: int, ff: int, tanh_form: bool = False):
        super().__init__()
        self.tanh_form = bool(tanh_form)
        self.up = TLLinear(width, ff, bias=False)
        self.down = TLLinear(ff, width, bias=False)

    def forward(self, h):
        return self.down(mx.gelu(self.up(h), self.tanh_form))


class GatedFF(nn.Module):
    """down(gelu(gate x) * (up x)), tanh-form or exact GELU, no biases;
    gate and up are one fused projection [gate | up]."""

    def __init__(self, width: int, ff: int, tanh_form: bool = True):
        super().__init__()
        self.ff, self.tanh_form = int(ff), bool(tanh_form)
        self.gate_up = TLLinear(width, 2 * ff, bias=False)
        self.down = TLLinear(ff, width, bias=False)

    def forward(self, h):
        return self.down(mx.gelu_gate(self.gate_up(h), self.tanh_form))


class TokenSide(nn.Module):
    """Per-layer token input: a slice of a second embedding table gates a
    narrow projection of the residual,
    y = proj(gelu_tanh(gate x) * table[token, col:col + dim]); the caller
    adds y through an RMS norm with the plain weight ``norm``."""

    def __init__(self, width: int, dim: int, col: int):
        super().__init__()
        self.dim, self.col = dim, col
        self.gate = TLLinear(width, dim, bias=False)
        self.proj = TLLinear(dim, width, bias=False)
        self.norm = RMSWeight(width, one_plus=False)

    def forward(self, h, table, tokens):
        g = mx.gelu(self.gate(h), True, table=table, tokens=tokens,
                    table_col=self.col)
        return self.proj(g)


# ---------------------------------------------------------------------------
# blocks of the parallel-mixer family: layer norm without bias, causal
# input convolution, softmax attention with short convolutions / a learned
# sink / capped scores whose values are its unrotated keys, a selective
# state-space (SSD) mixer, a pair of mixers on one input, and a PolyNorm
# feed-forward
# ---------------------------------------------------------------------------
class LayerNormWeight(nn.Module, _F32Cache):
    """Weight of a layer norm without bias."""

    def __init__(self, width: int):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(width))

    def w32(self):
        return self._f32("weight")


class CanonConv(nn.Module, _F32Cache):
    """Causal per-channel convolution over time added to a sublayer's
    input: h <- h + conv(h), taps [width, K], no bias. Its last K-1 inputs
    are per-sequence state (``state_shape``)."""

    def __init__(self, width: int, taps: int):
        super().__init__()
        self.taps = int(taps)
        self.weight = nn.Parameter(torch.zeros(width, taps))
        self.state_shape = (taps - 1, width)

    def w32(self):
        return self._f32("weight")


class ConvSinkAttention(nn.Module, _F32Cache):
    """Grouped-query softmax attention over the paged pool whose VALUES are
    its keys before rotation (no value projection). q and k (with biases,
    added by the caller's fused projection) pass a short causal
    convolution over time, then rotate-half positions on the first
    ``rot_dims`` dimensions of every head (optionally with a two-regime
    frequency scaling, see ``ops.mixers.yarn_freqs``); scores are scaled,
    optionally capped through tanh, and the softmax denominator holds one
    learned logit per head (``sink``): weight that attends to nothing.

    The module owns everything after the input projection; ``in_cols``
    columns [q | k] of the caller's projection feed it. Per-sequence
    memory: key pool (rotated), value pool (unrotated) and the last
    ``conv - 1`` projected rows (``state_shapes``)."""

    kind = "conv_sink_attention"

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int,
                 conv: int, scale: float, softcap: float, rot_dims: int,
                 rot_base: float, rot_scaling: Optional[dict]):
        super().__init__()
        assert heads % kv_heads == 0 and rot_dims % 2 == 0 \
            and rot_dims <= dim
        self.H, self.G, self.D, self.K = heads, kv_heads, dim, int(conv)
        self.scale, self.softcap = float(scale), float(softcap or 0.0)
        self.rot_dims, self.base = int(rot_dims), float(rot_base)
        self.rot_scaling = dict(rot_scaling) if rot_scaling else None
        self.q_cols, self.k_cols = heads * dim, kv_heads * dim
        self.in_cols = self.q_cols + self.k_cols
        self.bias_cols = self.in_cols
        self.qk_conv = nn.Parameter(torch.zeros(self.in_cols, self.K))
        self.sink = nn.Parameter(torch.zeros(heads))
        self.o_proj = TLLinear(heads * dim, width, bias=False)
        self.state_shapes = [(self.K - 1, self.in_cols)]

    def cache_spec(self):
        return {"kind": "kv", "G": self.G, "DK": self.D, "V": self.D}

    def _freqs(self, dev):
        hit = self.__dict__.get("_fr")
        if hit is None or hit[0].device != dev:
            hit = mx.yarn_freqs(self.rot_dims, self.base, self.rot_scaling,
                                dev)
            self.__dict__["_fr"] = hit
        return hit

    def forward(self, proj, col, meta, kpool, vpool, hist):
        fr, mult = (self._freqs(proj.device) if self.rot_dims
                    else (None, 1.0))
        q = mx.conv_rope_rows(proj, col, self.H + self.G, self.D,
                              self._f32("qk_conv"), hist, meta,
                              rot_dims=self.rot_dims, freqs=fr, rot_mult=mult,
                              pool=kpool, raw_pool=vpool, pool_heads=self.G)
        o = mx.flex_attention(q, kpool, vpool, meta, self.H, self.scale,
                              softcap=self.softcap,
                              sink_logits=self._f32("sink"),
                              out_dtype=proj.dtype)
        return self.o_proj(o)


class SSDMixer(nn.Module, _F32Cache):
    """Selective state-space mixer with one scalar decay per head
    (state-space duality form). Columns [z | x | B | C | dt] of the
    caller's projection feed it (``in_cols``); x, B, C pass a short causal
    convolution with bias and silu; dt = softplus(dt + dt_bias);
    S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T, y_t = S_t^T C_t +
    D x_t; y * silu(z) is RMS-normed in ``norm_groups`` equal parts, times
    ``norm``, then the output projection. Per-sequence memory: the state
    [heads, state, vdim] (fp32) and the convolution's last inputs."""

    kind = "ssd"

    def __init__(self, width: int, heads: int, vdim: int, state: int,
                 groups: int, conv: int, norm_groups: int, eps: float):
        super().__init__()
        assert heads % groups == 0 and (heads * vdim) % norm_groups == 0
        self.H, self.P, self.N, self.G = heads, vdim, state, groups
        self.K, self.norm_groups, self.eps = int(conv), norm_groups, float(eps)
        self.inner = heads * vdim
        self.conv_cols = self.inner + 2 * groups * state
        self.in_cols = self.inner + self.conv_cols + heads
        self.bias_cols = 0
        self.conv = nn.Parameter(torch.zeros(self.conv_cols, self.K))
        self.conv_b = nn.Parameter(torch.zeros(self.conv_cols))
        self.dt_bias = nn.Parameter(torch.zeros(heads))
        self.A_log = nn.Parameter(torch.zeros(heads))
        self.D = nn.Parameter(torch.ones(heads))
        self.norm = nn.Parameter(torch.ones(self.inner))
        self.o_proj = TLLinear(self.inner, width, bias=False)
        self.state_shapes = [(self.K - 1, self.conv_cols),
                             (heads, state, vdim)]

    def forward(self, proj, col, meta, hist, S):
        inner, GN = self.inner, self.G * self.N
        xbc = mx.conv_rope_rows(proj, col + inner, 1, self.conv_cols,
                                self._f32("conv"), hist, meta,
                                bias=self._f32("conv_b"), silu=True)
        y = mx.ssd_scan(xbc, (0, inner, inner + GN), proj,
                        col + inner + self.conv_cols, self._f32("dt_bias"),
                        self._f32("A_log"), self._f32("D"), S, meta, self.H,
                        self.P, self.N, self.G)
        u = mx.gated_group_rms(y, proj, col, self._f32("norm"),
                               self.norm_groups, self.eps,
                               out_dtype=proj.dtype)
        return self.o_proj(u)


class ParallelMixer(nn.Module, _F32Cache):
    """A pair of mixers fed by the same input: ``left`` (attention) and
    ``right`` (state-space), fed by ONE fused input projection. The result
    is half the sum of the two outputs after each is RMS-normed over the
    model width with its plain weight (``left_out`` / ``right_out``);
    ``forward`` returns the two raw outputs and the caller's residual
    update applies the norms and the half sum in the same pass."""

    kind = "parallel"

    def __init__(self, width: int, left: nn.Module, right: nn.Module):
        super().__init__()
        self.left, self.right = left, right
        self.proj = TLLinear(width, left.in_cols + right.in_cols, bias=True)
        self.left_out = nn.Parameter(torch.ones(width))
        self.right_out = nn.Parameter(torch.ones(width))
        self.state_shapes = list(left.state_shapes) + list(right.state_shapes)

    def cache_spec(self):
        return dict(self.left.cache_spec(), shapes=self.state_shapes)

    def forward(self, h, meta, kpool, vpool, states):
        proj = self.proj(h)
        nl = len(self.left.state_shapes)
        a = self.left(proj, 0, meta, kpool, vpool, *states[:nl])
        b = self.right(proj, self.left.in_cols, meta, *states[nl:])
        return a, b


class PolyNormFF(nn.Module, _F32Cache):
    """down(polynorm(up x)): the activation is a learned cubic in the
    row-normalised powers of its input, coefficients ``act`` [4]."""

    def __init__(self, width: int, ff: int, eps: float):
        super().__init__()
        self.eps = float(eps)
        self.up = TLLinear(width, ff, bias=False)
        self.down = TLLinear(ff, width, bias=False)
        self.act = nn.Parameter(torch.tensor([1.0, 0.0, 0.0, 0.0]))

    def forward(self, h):
        return self.down(mx.polynorm(self.up(h), self._f32("act"), self.eps))
