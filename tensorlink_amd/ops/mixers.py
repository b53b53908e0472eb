"""Sequence-mixer ops over ragged batches: hyper-connection + Dynamic-Tanh,
matrix-memory (mLSTM) recurrence with slot-resident state, differential
attention over the paged KV pool, group-limited top-k routing.

Same dispatch policy as the rest of :mod:`tensorlink_amd.ops`: tensors on
the GPU run the hand-written HIP kernels (``csrc/hyper_dyt.hip``,
``csrc/mlstm_scan.hip``, ``csrc/diff_attn.hip``) and a missing extension
raises; CPU tensors run the torch implementations below, which are the
CPU test tier's execution path.

A step's batch is *ragged*: sequence b contributes ``new[b]`` tokens that
continue ``pos0[b]`` cached ones. Tokens are flattened sequence after
sequence; :class:`RaggedMeta` carries the offsets on the host and on the
device, so a prompt portion and single decoded tokens of other requests
share one forward pass.
"""

from __future__ import annotations

import os
from typing import List, Optional, Sequence

import torch

PAGE = 128
SCAN_CHUNK = 64      # tokens per chunk of the chunk-parallel recurrence


class RaggedMeta:
    """Flat-token description of one step.

    ``new[b]`` tokens of sequence b start at flat offset ``cu[b]`` and at
    position ``pos0[b]``; ``slots[b]`` is its state slot and ``table[b]``
    its page-table row."""

    def __init__(self, new: Sequence[int], pos0: Sequence[int],
                 slots: Sequence[int], table: torch.Tensor, device):
        assert len(new) == len(pos0) == len(slots) == table.shape[0]
        self.new_h = [int(x) for x in new]
        self.pos0_h = [int(x) for x in pos0]
        self.slots_h = [int(x) for x in slots]
        self.B = len(self.new_h)
        cu = [0]
        for x in self.new_h:
            cu.append(cu[-1] + x)
        self.cu_h = cu
        self.T = cu[-1]
        seq, pos = [], []
        for b, (x, p) in enumerate(zip(self.new_h, self.pos0_h)):
            seq += [b] * x
            pos += range(p, p + x)
        i32 = dict(dtype=torch.int32, device=device)
        # ONE host->device copy for all the small index vectors
        packed = torch.tensor(cu + self.slots_h + self.pos0_h + seq + pos,
                              dtype=torch.int32).to(device)
        B, T = self.B, self.T
        self.cu = packed[:B + 1]
        self.slots = packed[B + 1:2 * B + 1]
        self.pos0 = packed[2 * B + 1:3 * B + 1]
        self.tok_seq = packed[3 * B + 1:3 * B + 1 + T]
        self.tok_pos = packed[3 * B + 1 + T:]
        self.table = table.to(**i32).contiguous()
        self.max_kv = max((p + x for p, x in zip(self.pos0_h, self.new_h)),
                          default=0)
        self._tiles = None
        self._device = device

    def query_tiles(self, size: int = 64) -> torch.Tensor:
        """[n, 4] int32 rows (sequence, first flat token, count <= size,
        first position): the step's tokens cut into per-sequence tiles for
        the tiled attention kernel."""
        if self._tiles is None:
            self._tiles = {}
        hit = self._tiles.get(size)
        if hit is None:
            rows = []
            for b in range(self.B):
                for o in range(0, self.new_h[b], size):
                    rows.append([b, self.cu_h[b] + o,
                                 min(size, self.new_h[b] - o),
                                 self.pos0_h[b] + o])
            hit = torch.tensor(rows, dtype=torch.int32).reshape(
                -1, 4).to(self._device)
            self._tiles[size] = hit
        return hit

    def scan_chunks(self, size: int):
        """The step's tokens cut into per-sequence chunks of ``size`` for
        the chunk-parallel recurrence: (cu [NC+1], chunk ids [NC], ones
        [NC], first chunk per sequence [B], chunk count per sequence [B],
        NC, largest count) — index tensors on the device, built once per
        step and shared by all layers."""
        hit = self.__dict__.setdefault("_chunks", {}).get(size)
        if hit is None:
            cu, base, cnt = [0], [], []
            for b in range(self.B):
                base.append(len(cu) - 1)
                n = 0
                for o in range(0, self.new_h[b], size):
                    cu.append(self.cu_h[b] + min(o + size, self.new_h[b]))
                    n += 1
                cnt.append(n)
            nc = len(cu) - 1
            packed = torch.tensor(cu + list(range(nc)) + [1] * nc + base
                                  + cnt, dtype=torch.int32).to(self._device)
            o1, o2, o3 = nc + 1, 2 * nc + 1, 3 * nc + 1
            hit = (packed[:o1], packed[o1:o2], packed[o2:o3],
                   packed[o3:o3 + self.B], packed[o3 + self.B:], nc,
                   max(cnt, default=0))
            self._chunks[size] = hit
        return hit

    def chunk_rows(self, size: int) -> torch.Tensor:
        """For every flat token its row in the chunk-major layout of
        ``scan_chunks(size)`` (chunk index * size + offset in the chunk):
        int64 [T] on the device."""
        hit = self.__dict__.setdefault("_chunk_rows", {}).get(size)
        if hit is None:
            rows, c = [], 0
            for b in range(self.B):
                for o in range(0, self.new_h[b], size):
                    n = min(size, self.new_h[b] - o)
                    rows += range(c * size, c * size + n)
                    c += 1
            hit = torch.tensor(rows, dtype=torch.int64).to(self._device)
            self._chunk_rows[size] = hit
        return hit

    @property
    def last_rows(self) -> List[int]:
        """Flat index of every sequence's last token."""
        return [c - 1 for c in self.cu_h[1:]]


def _ext():
    from tensorlink_amd import ops
    return ops._require_ext()


# ---------------------------------------------------------------------------
# hyper-connections + Dynamic Tanh
# ---------------------------------------------------------------------------
def hyper_dyt(X: torch.Tensor, y: Optional[torch.Tensor] = None,
              mix: Optional[torch.Tensor] = None,
              out: Optional[torch.Tensor] = None,
              inw: Optional[torch.Tensor] = None,
              alpha: Optional[torch.Tensor] = None,
              w: Optional[torch.Tensor] = None,
              b: Optional[torch.Tensor] = None,
              out_dtype=torch.float32, want_sum: bool = False):
    """One pass over the fp32 residual streams X [ns, T, W] (in place).

    If ``y`` is given, first X_t <- sum_s mix[s, t] X_s + out[t] * y. Then
    u = sum_s inw[s] X_s (plain sum without ``inw``); returns
    (tanh(alpha u) * w + b as ``out_dtype`` or None, u or None)."""
    if X.is_cuda:
        io32 = (y.dtype if y is not None else out_dtype) == torch.float32
        h, u = _ext().hyper_dyt(X, y, mix, out, inw, alpha, w, b, io32,
                                want_sum)
        return (h if w is not None else None, u if want_sum else None)
    if y is not None:
        X.copy_(torch.einsum("st,sij->tij", mix, X)
                + out.view(-1, 1, 1) * y.float())
    u = X.sum(0) if inw is None else (inw.view(-1, 1, 1) * X).sum(0)
    h = None
    if w is not None:
        h = (torch.tanh(alpha * u) * w + b).to(out_dtype)
    return h, (u if want_sum else None)


def relu_squared(x: torch.Tensor) -> torch.Tensor:
    if x.is_cuda:
        return _ext().relu_sq(x.contiguous())
    return torch.relu(x) ** 2


# ---------------------------------------------------------------------------
# matrix memory
# ---------------------------------------------------------------------------
def soft_cap(x: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(x / cap)


def mlstm_scan(proj: torch.Tensor, offs, gates: torch.Tensor,
               norm_w: torch.Tensor, S: torch.Tensor, n: torch.Tensor,
               m: torch.Tensor, meta: RaggedMeta, H: int, D: int, V: int,
               cap: float, eps: float) -> torch.Tensor:
    """Stabilised matrix-memory recurrence for every sequence of the step.

    proj [T, L] holds q | k | v | g at column offsets ``offs``; gates
    [T, 2H] fp32 are the raw input | forget pre-activations. State pools
    S [slots, H, D, V], n [slots, H, D], m [slots, H] (fp32) are read at
    ``meta.slots`` (zero for a sequence with no cached tokens) and written
    back. Returns [T, H*V]: per-head unit-RMS of the read-out, times
    ``norm_w``, times sigmoid(g)."""
    q_off, k_off, v_off, g_off = offs
    qscale = D ** -0.5
    if proj.is_cuda:
        C = _ext()
        gates = gates.contiguous()
        chunk = SCAN_CHUNK
        while max(meta.new_h) * H * D * V * 4 // chunk > (1 << 30):
            chunk *= 2                   # bound the chunk-state scratch
        if (max(meta.new_h) >= 4 * chunk
                and not os.environ.get("TL_NO_SCAN_CHUNKS")):
            # long prompt portions: chunk-parallel form. (1) every chunk's
            # own summary from the empty state, all chunks in parallel;
            # (2) a cheap sequential chain turns summaries into the state
            # BEFORE each chunk and updates the slots; (3) every chunk's
            # read-out from its start state, all chunks in parallel.
            cu_c, ids_c, ones_c, base, cnt, nc, cmax = meta.scan_chunks(chunk)
            if cmax <= 2048:
                f32 = dict(device=proj.device, dtype=torch.float32)
                S_t = torch.empty(nc, H, D, V, **f32)
                n_t = torch.empty(nc, H, D, **f32)
                m_t = torch.empty(nc, H, **f32)
                F_t = torch.empty(nc, H, **f32)
                C.mlstm_seq(proj, q_off, k_off, v_off, g_off, gates, norm_w,
                            S_t, n_t, m_t, cu_c, ids_c, ones_c, H, D, V, cap,
                            qscale, eps, F_t)
                C.mlstm_chain(S_t, n_t, m_t, F_t, S, n, m, base, cnt,
                              meta.slots, meta.pos0, cmax)
                return C.mlstm_seq(proj, q_off, k_off, v_off, g_off, gates,
                                   norm_w, S_t, n_t, m_t, cu_c, ids_c,
                                   ones_c, H, D, V, cap, qscale, eps, None)
        return C.mlstm_seq(proj, q_off, k_off, v_off, g_off, gates, norm_w,
                           S, n, m, meta.cu, meta.slots, meta.pos0, H, D, V,
                           cap, qscale, eps, None)
    T = proj.shape[0]
    pf = proj.float()
    q = pf[:, q_off:q_off + H * D].view(T, H, D) * qscale
    k = pf[:, k_off:k_off + H * D].view(T, H, D)
    v = pf[:, v_off:v_off + H * V].view(T, H, V)
    g = pf[:, g_off:g_off + H * V]
    li = soft_cap(gates[:, :H], cap)
    lf = torch.nn.functional.logsigmoid(soft_cap(gates[:, H:], cap))
    o = torch.empty(T, H, V)
    for b in range(meta.B):
        slot = meta.slots_h[b]
        if meta.pos0_h[b] == 0:
            Sb = torch.zeros(H, D, V)
            nb = torch.zeros(H, D)
            mb = torch.zeros(H)
        else:
            Sb, nb, mb = S[slot].clone(), n[slot].clone(), m[slot].clone()
        for t in range(meta.cu_h[b], meta.cu_h[b + 1]):
            m_new = torch.maximum(lf[t] + mb, li[t])
            a = torch.exp(lf[t] + mb - m_new)
            bb = torch.exp(li[t] - m_new)
            Sb = a[:, None, None] * Sb + bb[:, None, None] * (
                k[t].unsqueeze(-1) * v[t].unsqueeze(-2))
            nb = a[:, None] * nb + bb[:, None] * k[t]
            mb = m_new
            num = (Sb * q[t].unsqueeze(-1)).sum(1)
            den = torch.maximum((nb * q[t]).sum(-1).abs(),
                                torch.exp(-mb)) + 1e-6
            o[t] = num / den[:, None]
        if meta.new_h[b] > 0:
            S[slot], n[slot], m[slot] = Sb, nb, mb
    o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps)
    out = o.reshape(T, H * V) * norm_w * torch.sigmoid(g)
    return out.to(proj.dtype)


# ---------------------------------------------------------------------------
# differential attention over the paged pool
# ---------------------------------------------------------------------------
def kv_append(proj: torch.Tensor, k_off: int, v_off: int,
              kpool: torch.Tensor, vpool: torch.Tensor,
              meta: RaggedMeta) -> None:
    """Write the step's key rows [G*DK] and value rows [G*V] (columns
    ``k_off`` / ``v_off`` of proj) into pools [pages, G, PAGE, *]."""
    if proj.is_cuda:
        _ext().kv_append(proj, k_off, v_off, kpool, vpool, meta.tok_seq,
                         meta.tok_pos, meta.table)
        return
    G, DK, V = kpool.shape[1], kpool.shape[3], vpool.shape[3]
    T = proj.shape[0]
    pos = meta.tok_pos.long()
    page = meta.table.long()[meta.tok_seq.long(), pos // PAGE]
    r = pos % PAGE
    kpool[page, :, r] = proj[:, k_off:k_off + G * DK].view(T, G, DK)
    vpool[page, :, r] = proj[:, v_off:v_off + G * V].view(T, G, V)


def diff_attention(q: torch.Tensor, q_off: int, kpool: torch.Tensor,
                   vpool: torch.Tensor, meta: RaggedMeta, lam: torch.Tensor,
                   H: int, D: int, scale: float, diff: float,
                   eps: float) -> torch.Tensor:
    """Two-map attention of the step's tokens over their sequences' cached
    keys/values (the step's own rows already appended). Query rows are
    [H, 2, D] at column ``q_off``; returns [T, H*V] =
    unit_rms(a1 - lam * a2) * (1 - diff) per head."""
    if q.is_cuda:
        if (q.dtype == torch.bfloat16 and meta.T > meta.B
                and not os.environ.get("TL_NO_ATTN_TILES")):
            # a prompt portion is in the step: 64-query MFMA tiles
            out = torch.empty(q.shape[0], H * vpool.shape[3], device=q.device,
                              dtype=q.dtype)
            if _ext().diff_attn_tiles(q, q_off, kpool, vpool,
                                      meta.query_tiles(), meta.table, lam,
                                      out, H, D, scale, diff, eps):
                return out
        # few rows over long contexts (decoding): spread each row's keys
        # over several blocks so the chip is filled; a function of the
        # step's shape only
        n_split = 1
        while (n_split < 16 and meta.T * H * n_split < 1024
               and meta.max_kv > 512 * n_split):
            n_split *= 2
        return _ext().diff_attn_rows(q, q_off, kpool, vpool, meta.tok_seq,
                                     meta.tok_pos, meta.table, lam, H, D,
                                     scale, diff, eps, n_split)
    G, V = kpool.shape[1], vpool.shape[3]
    T = q.shape[0]
    out = torch.empty(T, H, V)
    qf = q[:, q_off:q_off + H * 2 * D].float().view(T, H, 2, D)
    rep = H // G
    for b in range(meta.B):
        t0, t1 = meta.cu_h[b], meta.cu_h[b + 1]
        if t1 == t0:
            continue
        L = meta.pos0_h[b] + (t1 - t0)
        pages = meta.table[b, :(L + PAGE - 1) // PAGE].long()
        # [L, G, *]
        kb = kpool[pages].float().permute(0, 2, 1, 3).reshape(
            -1, G, 2, D)[:L]
        vb = vpool[pages].float().permute(0, 2, 1, 3).reshape(-1, G, V)[:L]
        kb = kb.repeat_interleave(rep, 1)                  # [L, H, 2, D]
        vb = vb.repeat_interleave(rep, 1)
        sc = torch.einsum("thmd,jhmd->hmtj", qf[t0:t1], kb) * scale
        qpos = torch.arange(meta.pos0_h[b], L).view(-1, 1)
        mask = torch.arange(L).view(1, -1) > qpos
        sc = sc.masked_fill(mask, float("-inf"))
        a = torch.einsum("hmtj,jhv->mthv", torch.softmax(sc, -1), vb)
        out[t0:t1] = a[0] - lam.float() * a[1]
    out = out * torch.rsqrt((out * out).mean(-1, keepdim=True) + eps)
    return (out * (1.0 - diff)).reshape(T, H * V).to(q.dtype)


# ---------------------------------------------------------------------------
# routing
# ---------------------------------------------------------------------------
def group_limited_router(logits: torch.Tensor, top: int, n_groups: int,
                         keep_groups: int, scale: float):
    """Softmax scores over all experts; experts form ``n_groups`` equal
    groups of neighbours scored by their best member, and only the
    ``keep_groups`` best groups stay eligible. The ``top`` best eligible
    experts are chosen; weights = their scores / (sum + 1e-20) * scale.

    logits [T, E] fp32 -> (weights [T, top] fp32, indices [T, top])."""
    s = torch.softmax(logits.float(), -1)
    T, E = s.shape
    if keep_groups < n_groups:
        gs = s.view(T, n_groups, E // n_groups).amax(-1)
        kept = gs.topk(keep_groups, dim=-1).indices
        allow = torch.zeros(T, n_groups, dtype=torch.bool, device=s.device)
        allow.scatter_(1, kept, True)
        allow = allow.unsqueeze(-1).expand(T, n_groups, E // n_groups)
        masked = s.masked_fill(~allow.reshape(T, E), -1.0)
    else:
        masked = s
    idx = masked.topk(top, dim=-1).indices
    w = s.gather(1, idx)
    w = w / (w.sum(-1, keepdim=True) + 1e-20) * scale
    return w, idx


# ---------------------------------------------------------------------------
# post-norm residual, gated / plain RMS scaling, GELU, soft cap
# ---------------------------------------------------------------------------
def _rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)


def postnorm_add(X: torch.Tensor, y: torch.Tensor, w: torch.Tensor,
                 eps: float, one_plus: bool, out_dtype=torch.float32):
    """Residual with the norm on the sublayer's OUTPUT, in place on the
    fp32 residual X [T, W]:  X += y / rms(y) * (1 + w  |  w).
    Returns X in ``out_dtype`` (the next sublayer's input; X itself for
    fp32)."""
    assert X.dtype == torch.float32 and w.dtype == torch.float32
    if X.is_cuda:
        return _ext().postnorm_add(X, y.contiguous(), w, float(eps),
                                   bool(one_plus),
                                   out_dtype == torch.float32)
    X += _rms(y.float(), eps) * ((1.0 + w) if one_plus else w)
    return X if out_dtype == torch.float32 else X.to(out_dtype)


def rms_scale(x: torch.Tensor, w: torch.Tensor, eps: float, one_plus: bool,
              gate: Optional[torch.Tensor] = None, gate_col: int = 0,
              out_dtype=torch.float32) -> torch.Tensor:
    """x / rms(x) * (1 + w | w) over the last axis of x [T, N] (fp32),
    optionally times sigmoid(gate[:, gate_col:gate_col + N])."""
    assert x.dtype == torch.float32 and w.dtype == torch.float32
    if x.is_cuda:
        return _ext().rms_scale(x.contiguous(), w, float(eps),
                                bool(one_plus), gate, int(gate_col),
                                out_dtype == torch.float32)
    y = _rms(x, eps) * ((1.0 + w) if one_plus else w)
    if gate is not None:
        y = y * torch.sigmoid(
            gate[:, gate_col:gate_col + x.shape[-1]].float())
    return y.to(out_dtype)


def gelu(x: torch.Tensor, tanh_form: bool = False,
         table: Optional[torch.Tensor] = None,
         tokens: Optional[torch.Tensor] = None,
         table_col: int = 0) -> torch.Tensor:
    """GELU of x [T, N] — exact (erf) or the tanh form — evaluated in fp32,
    optionally times ``table[tokens, table_col:table_col + N]`` (a
    per-token embedding slice gathered in the same pass)."""
    if x.is_cuda:
        return _ext().gelu_mul(x.contiguous(), bool(tanh_form), table,
                               tokens, int(table_col))
    y = torch.nn.functional.gelu(x.float(),
                                 approximate="tanh" if tanh_form else "none")
    if table is not None:
        y = y * table[tokens.long(),
                      table_col:table_col + x.shape[-1]].float()
    return y.to(x.dtype)


def soft_cap_(z: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(z / cap) in place on fp32 logits."""
    assert z.dtype == torch.float32
    if z.is_cuda:
        _ext().soft_cap_(z, float(cap))
        return z
    return z.copy_(cap * torch.tanh(z / cap))


def add_rms(X: torch.Tensor, y: Optional[torch.Tensor],
            w: Optional[torch.Tensor], eps: float, out_dtype=torch.float32,
            x_scale: float = 1.0) -> torch.Tensor:
    """Pre-norm residual step, in place on the fp32 residual X [T, W]:
    X <- X * x_scale + y (``y`` = the previous sublayer's output, or None),
    then returns the next sublayer's input X / rms(X) * w in ``out_dtype``;
    without ``w`` (after the last sublayer) only the add is done and X is
    returned. Sum, statistic and scaling are fp32."""
    assert X.dtype == torch.float32
    assert w is None or w.dtype == torch.float32
    if X.is_cuda:
        return _ext().add_rms(
            X, None if y is None else y.contiguous(), w, float(eps),
            float(x_scale), out_dtype == torch.float32)
    if x_scale != 1.0:
        X *= x_scale
    if y is not None:
        X += y.float()
    return X if w is None else (_rms(X, eps) * w).to(out_dtype)


def gelu_gate(p: torch.Tensor, tanh_form: bool = True) -> torch.Tensor:
    """gelu(p[:, :N]) * p[:, N:] for a fused [gate | up] projection
    p [T, 2N]; evaluated in fp32, result in p's dtype."""
    if p.is_cuda:
        return _ext().gelu_gate(p.contiguous(), bool(tanh_form))
    N = p.shape[1] // 2
    f = p.float()
    y = torch.nn.functional.gelu(
        f[:, :N], approximate="tanh" if tanh_form else "none") * f[:, N:]
    return y.to(p.dtype)


# ---------------------------------------------------------------------------
# row preparation: RMS norm over a projection + rotate-half positions,
# written densely (queries) or into a page pool (keys, values, latents)
# ---------------------------------------------------------------------------
def rope_freqs(dims: int, base: float, device) -> torch.Tensor:
    """f_i = base^(-2i/dims), i < dims/2, evaluated in float64 and kept
    there (the angle p * f_i is formed in double by the kernels)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64),
                     -2.0 * i / dims).to(device)


def norm_rope_rows(src: torch.Tensor, col: int, n_heads: int, head_dim: int,
                   meta: RaggedMeta, *, norm_w: Optional[torch.Tensor] = None,
                   norm_cols: int = 0, eps: float = 0.0, rot_off: int = 0,
                   rot_dims: int = 0, freqs: Optional[torch.Tensor] = None,
                   pool: Optional[torch.Tensor] = None,
                   head_norm: bool = False, interleaved: bool = False,
                   rot_mult: float = 1.0,
                   mix_src: Optional[torch.Tensor] = None, mix_col: int = 0,
                   mix_lam: Optional[torch.Tensor] = None):
    """Take columns [col, col + n_heads*head_dim) of src [T, L]; RMS-norm
    the first ``norm_cols`` of them together (weight ``norm_w``, plain) or,
    with ``head_norm``, every head on its own with the one weight
    [head_dim]; rotate dims [rot_off, rot_off + rot_dims) of every head by
    the token's position (pairs (i, i + rot_dims/2), or (2i, 2i+1) with
    ``interleaved``; angle pos * freqs[i]; cos and sin times ``rot_mult``);
    with ``mix_src`` blend the result with the same token's columns
    [mix_col, mix_col + N) of that tensor, (1 - lam) x + lam m with lam =
    ``mix_lam`` (one fp32 element); all in fp32. Without ``pool`` returns
    the rows as fp32 [T, n_heads*head_dim]; with ``pool``
    [pages, n_heads, PAGE, head_dim] scatters them to the tokens' page rows
    in the pool's dtype and returns None."""
    N = n_heads * head_dim
    T = src.shape[0]
    if src.is_cuda:
        out = None if pool is not None else torch.empty(
            T, N, device=src.device, dtype=torch.float32)
        _ext().norm_rope_rows(src, int(col), int(n_heads), int(head_dim),
                              norm_w, int(norm_cols), float(eps),
                              int(rot_off), int(rot_dims), freqs,
                              meta.tok_seq, meta.tok_pos, meta.table, out,
                              pool, bool(head_norm), bool(interleaved),
                              float(rot_mult), mix_src, int(mix_col),
                              mix_lam)
        return out
    x = src[:, col:col + N].float()
    if norm_w is not None and head_norm:
        x = (_rms(x.reshape(T, n_heads, head_dim), eps)
             * norm_w).reshape(T, N)
    elif norm_w is not None:
        x = torch.cat([_rms(x[:, :norm_cols], eps) * norm_w,
                       x[:, norm_cols:]], 1)
    x = x.reshape(T, n_heads, head_dim).clone()
    pos = meta.tok_pos.long()
    if rot_dims:
        half = rot_dims // 2
        ang = pos.double().view(T, 1, 1) * freqs.double().view(1, 1, half)
        c = (torch.cos(ang) * rot_mult).float()
        s = (torch.sin(ang) * rot_mult).float()
        if interleaved:
            iu = slice(rot_off, rot_off + rot_dims, 2)
            iv = slice(rot_off + 1, rot_off + rot_dims, 2)
        else:
            iu = slice(rot_off, rot_off + half)
            iv = slice(rot_off + half, rot_off + rot_dims)
        u, v = x[:, :, iu].clone(), x[:, :, iv].clone()
        x[:, :, iu] = u * c - v * s
        x[:, :, iv] = v * c + u * s
    if mix_src is not None:
        lam = mix_lam.float().reshape(())
        x = (1.0 - lam) * x + lam * mix_src[
            :, mix_col:mix_col + N].float().reshape(T, n_heads, head_dim)
    if pool is None:
        return x.reshape(T, N)
    page = meta.table.long()[meta.tok_seq.long(), pos // PAGE]
    pool[page, :, pos % PAGE] = x.to(pool.dtype)
    return None


# ---------------------------------------------------------------------------
# softmax attention over the paged pool with the options layered models
# combine: GQA/MQA, sliding window, sink, cross-head score mixing, values
# that are a prefix of the key row (latent attention)
# ---------------------------------------------------------------------------
def flex_attention(q: torch.Tensor, kpool: torch.Tensor,
                   vpool: Optional[torch.Tensor], meta: RaggedMeta, H: int,
                   scale: float, *, window: int = 0, sink: bool = False,
                   talk: Optional[torch.Tensor] = None, v_cols: int = 0,
                   softcap: float = 0.0,
                   sink_logits: Optional[torch.Tensor] = None,
                   chunk: int = 0, keep_first: int = 0,
                   dist_bias: Optional[torch.Tensor] = None,
                   gate: Optional[torch.Tensor] = None, gate_col: int = 0,
                   gate_heads: bool = False,
                   out_dtype=torch.float32) -> torch.Tensor:
    """Causal attention of the step's tokens over their sequences' cached
    rows (the step's own rows already appended).

    q [T, H*DK] fp32 (normed / rotated); kpool [pages, G, PAGE, DK];
    values from vpool [pages, G, PAGE, V], or, without it, the first
    ``v_cols`` columns of the key row. score = q.k * scale; with ``talk``
    [H, H] the heads' scores are mixed, s_h <- sum_g talk[h, g] s_g;
    ``softcap`` > 0 replaces a score by softcap * tanh(score / softcap);
    ``window`` > 0 keeps keys with 0 <= i - j < window; ``sink`` adds one
    to the softmax denominator, ``sink_logits`` [H] (fp32) adds
    exp(sink_logits[h]) instead (a keyless, valueless entry that is neither
    scaled nor capped). ``chunk`` > 0 (instead of a window) keeps the keys
    of the query's own chunk, floor(j / chunk) = floor(i / chunk), chunks
    counted from position 0; ``keep_first`` > 0 keeps keys j < keep_first
    visible whatever the window or chunk says. ``dist_bias`` [H, n] (fp32)
    adds dist_bias[h, min(i - j, n - 1)] to the scaled score. ``gate``
    [T, L] multiplies the result by sigmoid of its columns from
    ``gate_col``: one per output column, or one per head with
    ``gate_heads``. Scores, weights and sums are fp32.
    Returns [T, H*V] in ``out_dtype``."""
    G, DK = kpool.shape[1], kpool.shape[3]
    V = vpool.shape[3] if vpool is not None else v_cols
    T = q.shape[0]
    assert q.dtype == torch.float32 and q.shape[1] == H * DK
    if sink_logits is not None:
        assert sink_logits.dtype == torch.float32 \
            and sink_logits.numel() == H
        sink = True
    if q.is_cuda:
        if (kpool.dtype == torch.bfloat16 and meta.T > meta.B
                and not os.environ.get("TL_NO_ATTN_TILES")
                and _ext().flex_attn_tiles_ok(H, G, talk is not None, DK,
                                              V)):
            # a prompt portion is in the step: 64-query MFMA tiles
            return _ext().flex_attn_tiles(
                q, kpool, vpool, meta.query_tiles(), meta.table, talk,
                int(H), float(scale), int(window), bool(sink), int(V),
                out_dtype == torch.float32, float(softcap), sink_logits,
                int(chunk), int(keep_first), dist_bias, gate, int(gate_col),
                bool(gate_heads))
        # few rows over long key ranges (decoding): spread each row's
        # keys over several blocks so the chip is filled; a function of
        # the step's shape only
        span = meta.max_kv
        if window > 0 or chunk > 0:
            span = min(span, max(window, chunk) + keep_first)
        n_split = 1
        while (n_split < 16 and meta.T * H * n_split < 2048
               and span > 256 * n_split):
            n_split *= 2
        return _ext().flex_attn_rows(q, kpool, vpool, meta.tok_seq,
                                     meta.tok_pos, meta.table, talk, int(H),
                                     float(scale), int(window), bool(sink),
                                     int(V), out_dtype == torch.float32,
                                     n_split, 1 if meta.T * H <= 512 else 8,
                                     float(softcap), sink_logits, int(chunk),
                                     int(keep_first), dist_bias, gate,
                                     int(gate_col), bool(gate_heads))
    out = torch.empty(T, H, V)
    qf = q.view(T, H, DK)
    rep = H // G
    for b in range(meta.B):
        t0, t1 = meta.cu_h[b], meta.cu_h[b + 1]
        if t1 == t0:
            continue
        L = meta.pos0_h[b] + (t1 - t0)
        pages = meta.table[b, :(L + PAGE - 1) // PAGE].long()
        kb = kpool[pages].float().permute(0, 2, 1, 3).reshape(-1, G, DK)[:L]
        vb = (vpool[pages].float().permute(0, 2, 1, 3).reshape(-1, G, V)[:L]
              if vpool is not None else kb[:, :, :V])
        kb = kb.repeat_interleave(rep, 1)                 # [L, H, DK]
        vb = vb.repeat_interleave(rep, 1)
        sc = torch.einsum("thd,jhd->htj", qf[t0:t1], kb) * scale
        if talk is not None:
            sc = torch.einsum("hg,gtj->htj", talk.float(), sc)
        if softcap:
            sc = softcap * torch.tanh(sc / softcap)
        qpos = torch.arange(meta.pos0_h[b], L).view(-1, 1)
        kpos = torch.arange(L).view(1, -1)
        if dist_bias is not None:
            d = (qpos - kpos).clamp(0, dist_bias.shape[1] - 1)
            sc = sc + dist_bias[:, d]
        hide = torch.zeros_like(kpos > qpos)
        if window > 0:
            hide = qpos - kpos >= window
        elif chunk > 0:
            hide = (kpos // chunk) != (qpos // chunk)
        if keep_first > 0:
            hide = hide & (kpos >= keep_first)
        hide = hide | (kpos > qpos)
        sc = sc.masked_fill(hide, float("-inf"))
        m = sc.amax(-1, keepdim=True)
        if sink:
            sl = (sink_logits.view(H, 1, 1) if sink_logits is not None
                  else torch.zeros(H, 1, 1))
            m = torch.maximum(m, sl)
        e = torch.exp(sc - m)
        den = e.sum(-1, keepdim=True)
        if sink:
            den = den + torch.exp(sl - m)
        out[t0:t1] = torch.einsum("htj,jhv->thv", e / den, vb)
    if gate is not None:
        n = H if gate_heads else H * V
        g = torch.sigmoid(gate[:, gate_col:gate_col + n].float())
        out = out * (g.view(T, H, 1) if gate_heads else g.view(T, H, V))
    return out.reshape(T, H * V).to(out_dtype)


# ---------------------------------------------------------------------------
# lightning attention: decayed outer-product memory per head
# ---------------------------------------------------------------------------
def lightning_scan(proj: torch.Tensor, offs, decay: torch.Tensor,
                   S: torch.Tensor, meta: RaggedMeta, H: int, D: int,
                   V: int) -> torch.Tensor:
    """S_t = decay_h S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t  per head, with
    q, k, v = silu of columns ``offs`` = (q, k, v) of proj [T, L]. The
    state pool S [slots, H, D, V] (fp32) is read at ``meta.slots`` (zeros
    for a sequence with no cached tokens) and written back. Returns the
    raw read-out [T, H*V] in fp32."""
    q_off, k_off, v_off = offs
    T = proj.shape[0]
    if proj.is_cuda:
        chunk = SCAN_CHUNK
        while meta.T * H * D * V * 4 // chunk > (1 << 31):
            chunk *= 2                   # bound the chunk-state scratch
        if (max(meta.new_h) >= 4 * chunk
                and not os.environ.get("TL_NO_SCAN_CHUNKS")):
            # long prompt portions: chunk form. Per chunk the intra-chunk
            # part (Q K^T with the decay mask, times V), the chunk summary
            # Kw^T V and the carried part Qd S0 are batched fp32 GEMMs over
            # all chunks at once; only the chain of summaries is sequential.
            C = _ext()
            cu_c, _, _, base, cnt, nc, _ = meta.scan_chunks(chunk)
            Qs, Qd, Ks, Kw, Vs = C.lightning_chunk_prep(
                proj, int(q_off), int(k_off), int(v_off), decay, cu_c,
                int(H), int(D), int(V), chunk)
            A = torch.bmm(Qs, Ks.transpose(1, 2))
            C.lightning_decay_mask_(A, decay)
            O = torch.bmm(A, Vs)
            U = torch.bmm(Kw.transpose(1, 2), Vs)
            C.lightning_chain_(U, S, decay, cu_c, base, cnt, meta.slots,
                               meta.pos0)
            O.baddbmm_(Qd, U)
            rows = meta.chunk_rows(chunk)
            return O.view(nc, H, chunk, V).transpose(1, 2).reshape(
                nc * chunk, H * V).index_select(0, rows)
        return _ext().lightning_scan(proj, int(q_off), int(k_off),
                                     int(v_off), decay, S, meta.cu,
                                     meta.slots, meta.pos0, int(H), int(D),
                                     int(V))
    silu = torch.nn.functional.silu
    pf = proj.float()
    q = silu(pf[:, q_off:q_off + H * D]).view(T, H, D)
    k = silu(pf[:, k_off:k_off + H * D]).view(T, H, D)
    v = silu(pf[:, v_off:v_off + H * V]).view(T, H, V)
    o = torch.empty(T, H, V)
    dec = decay.float().view(H, 1, 1)
    for b in range(meta.B):
        slot = meta.slots_h[b]
        Sb = (torch.zeros(H, D, V) if meta.pos0_h[b] == 0
              else S[slot].clone())
        for t in range(meta.cu_h[b], meta.cu_h[b + 1]):
            Sb = dec * Sb + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
            o[t] = (Sb * q[t].unsqueeze(-1)).sum(1)
        if meta.new_h[b] > 0:
            S[slot] = Sb
    return o.reshape(T, H * V)


# ---------------------------------------------------------------------------
# layer norm with a weight and no bias, causal per-channel convolutions
# whose last inputs live in the slot state, PolyNorm, grouped gated RMS,
# the selective state-space recurrence
# ---------------------------------------------------------------------------
CONV_TILE = 8        # tokens per block of the convolution kernels


def _ln(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    d = x - x.mean(-1, keepdim=True)
    return d * torch.rsqrt((d * d).mean(-1, keepdim=True) + eps) * w


def _conv_ragged(u: torch.Tensor, w: torch.Tensor, hist: torch.Tensor,
                 meta: RaggedMeta) -> torch.Tensor:
    """Torch form of the causal convolution over a ragged step:
    y_t = sum_j w[:, j] u_(t-K+1+j); inputs before a portion's start come
    from hist[slot] (zeros for a sequence with no cached tokens), which is
    left holding the sequence's last K-1 inputs."""
    K = w.shape[1]
    y = torch.empty_like(u)
    for b in range(meta.B):
        t0, t1 = meta.cu_h[b], meta.cu_h[b + 1]
        if t1 == t0:
            continue
        slot = meta.slots_h[b]
        prev = (torch.zeros(K - 1, u.shape[1]) if meta.pos0_h[b] == 0
                else hist[slot].clone())
        ext = torch.cat([prev, u[t0:t1]], 0)
        n = t1 - t0
        acc = torch.zeros(n, u.shape[1])
        for j in range(K):
            acc += w[:, j] * ext[j:j + n]
        y[t0:t1] = acc
        if K > 1:
            hist[slot] = ext[ext.shape[0] - (K - 1):]
    return y


def layer_norm_rows(x: torch.Tensor, w: torch.Tensor, eps: float,
                    out_dtype=torch.float32) -> torch.Tensor:
    """(x - mean) / sqrt(var + eps) * w over the last axis of x [T, W]
    (fp32; var = mean of squared deviations)."""
    assert x.dtype == torch.float32 and w.dtype == torch.float32
    if x.is_cuda:
        return _ext().layer_norm_rows(x.contiguous(), w, float(eps),
                                      out_dtype == torch.float32)
    return _ln(x, w, eps).to(out_dtype)


def ln_canon(X: torch.Tensor, w: torch.Tensor, eps: float,
             conv_w: torch.Tensor, hist: torch.Tensor, meta: RaggedMeta,
             out_dtype=torch.float32) -> torch.Tensor:
    """A sublayer's input: h = layer_norm(X) * w, then h + conv(h) with the
    causal per-channel taps conv_w [W, K]. hist [slots, K-1, W] (fp32)
    holds every sequence's last K-1 normed rows and is updated; a sequence
    with no cached tokens starts from zeros whatever its slot holds.
    Everything in fp32; returns [T, W] in ``out_dtype``."""
    assert X.dtype == torch.float32 and hist.dtype == torch.float32
    K = conv_w.shape[1]
    assert hist.shape[1] == K - 1 and K - 1 <= CONV_TILE
    if X.is_cuda:
        return _ext().ln_canon(X, w, float(eps), conv_w, hist,
                               meta.query_tiles(CONV_TILE), meta.cu,
                               meta.slots, meta.pos0,
                               out_dtype == torch.float32)
    h = _ln(X, w, eps)
    return (h + _conv_ragged(h, conv_w, hist, meta)).to(out_dtype)


def conv_rope_rows(src: torch.Tensor, col: int, n_heads: int, head_dim: int,
                   conv_w: torch.Tensor, hist: torch.Tensor,
                   meta: RaggedMeta, *, bias: Optional[torch.Tensor] = None,
                   silu: bool = False, rot_dims: int = 0,
                   freqs: Optional[torch.Tensor] = None,
                   rot_mult: float = 1.0,
                   pool: Optional[torch.Tensor] = None,
                   raw_pool: Optional[torch.Tensor] = None,
                   pool_heads: int = 0):
    """Short causal convolution over time on columns
    [col, col + n_heads*head_dim) of src [T, L] (taps conv_w [N, K], fp32;
    optional per-channel bias and silu), then rotate-half positions on the
    first ``rot_dims`` dimensions of every head (angle pos * freqs[i], cos
    and sin times ``rot_mult``). hist [slots, K-1, N] (fp32) holds every
    sequence's last K-1 projected rows and is updated. The first
    n_heads - pool_heads heads are returned densely as fp32
    [T, (n_heads - pool_heads)*head_dim]; the last ``pool_heads`` heads
    are scattered to the tokens' page rows of ``pool``
    [pages, pool_heads, PAGE, head_dim] after rotation and, with
    ``raw_pool``, the unrotated convolution output as well."""
    N = n_heads * head_dim
    T = src.shape[0]
    K = conv_w.shape[1]
    assert conv_w.shape[0] == N and hist.shape[1:] == (K - 1, N)
    assert K - 1 <= CONV_TILE and rot_dims % 2 == 0 and rot_dims <= head_dim
    assert (pool is None) == (pool_heads == 0) and pool_heads <= n_heads
    dense = n_heads - pool_heads
    if src.is_cuda:
        out = torch.empty(T, dense * head_dim, device=src.device,
                          dtype=torch.float32) if dense else None
        _ext().conv_rope_rows(src, int(col), int(n_heads), int(head_dim),
                              conv_w, bias, bool(silu), hist, int(rot_dims),
                              freqs, float(rot_mult),
                              meta.query_tiles(CONV_TILE), meta.cu,
                              meta.slots, meta.pos0, meta.table, out, pool,
                              raw_pool, int(pool_heads))
        return out
    y = _conv_ragged(src[:, col:col + N].float(), conv_w, hist, meta)
    if bias is not None:
        y = y + bias
    if silu:
        y = torch.nn.functional.silu(y)
    raw = y.reshape(T, n_heads, head_dim)
    x = raw.clone()
    pos = meta.tok_pos.long()
    if rot_dims:
        half = rot_dims // 2
        ang = pos.double().view(T, 1, 1) * freqs.double().view(1, 1, half)
        c = (torch.cos(ang) * rot_mult).float()
        s = (torch.sin(ang) * rot_mult).float()
        u, v = raw[:, :, :half], raw[:, :, half:rot_dims]
        x[:, :, :half] = u * c - v * s
        x[:, :, half:rot_dims] = v * c + u * s
    if pool is not None:
        page = meta.table.long()[meta.tok_seq.long(), pos // PAGE]
        pool[page, :, pos % PAGE] = x[:, dense:].to(pool.dtype)
        if raw_pool is not None:
            raw_pool[page, :, pos % PAGE] = raw[:, dense:].to(raw_pool.dtype)
    return x[:, :dense].reshape(T, dense * head_dim) if dense else None


def yarn_freqs(dims: int, base: float, scaling: Optional[dict], device):
    """Rotation frequencies (float64 [dims/2]) and the multiplier of cos and
    sin. Without ``scaling``: f_i = base^(-2i/dims), multiplier 1. With
    ``scaling`` = {factor, original, fast, slow}: pairs that turn more than
    ``fast`` times over ``original`` positions keep f_i, pairs that turn
    fewer than ``slow`` times get f_i / factor, a linear ramp over the pair
    index lies between; the multiplier is 0.1 ln(factor) + 1."""
    f = rope_freqs(dims, base, "cpu")
    if not scaling:
        return f.to(device), 1.0
    import math
    factor = float(scaling["factor"])

    def pair_of(turns):
        return dims * math.log(scaling["original"]
                               / (2.0 * math.pi * turns)) / (
                                   2.0 * math.log(base))

    lo = max(math.floor(pair_of(scaling["fast"])), 0)
    hi = min(math.ceil(pair_of(scaling["slow"])), dims - 1)
    i = torch.arange(dims // 2, dtype=torch.float64)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    f = f / factor * ramp + f * (1.0 - ramp)
    return f.to(device), 0.1 * math.log(factor) + 1.0


def log_distance_buckets(rows: int, far: float) -> List[int]:
    """Bucket of every distance n = 0, 1, ... up to the first that falls
    into the last bucket (all larger ones do too). With half = rows // 2:
    n < half has its own bucket n; beyond, buckets grow geometrically,
    half + floor(ln(n / half) / ln(far / half) * (rows - half)), capped at
    rows - 1. Evaluated in float64 on the host."""
    import math
    half = rows // 2
    if rows < 2 or far <= half:
        raise ValueError("distance buckets need rows >= 2 and a far "
                         "distance beyond rows // 2")
    out = []
    n = 0
    while True:
        if n < half:
            b = n
        else:
            b = min(rows - 1, half + int(math.floor(
                math.log(n / half) / math.log(far / half) * (rows - half))))
        out.append(b)
        if b == rows - 1:
            return out
        n += 1


def ssd_scan(xbc: torch.Tensor, offs, dt_src: torch.Tensor, dt_col: int,
             dt_bias: torch.Tensor, A_log: torch.Tensor, skip: torch.Tensor,
             S: torch.Tensor, meta: RaggedMeta, H: int, P: int, N: int,
             G: int) -> torch.Tensor:
    """Selective state-space recurrence with one scalar decay per head and
    token. xbc [T, *] (fp32) holds x [H*P] | B [G*N] | C [G*N] at columns
    ``offs``; the raw step sizes are columns [dt_col, dt_col + H) of
    dt_src. Per head h (group floor(h / (H/G))):

        dt = softplus(raw + dt_bias_h)
        S_t = exp(-exp(A_log_h) dt) S_(t-1) + dt B_t x_t^T     (S is [N, P])
        y_t = S_t^T C_t + skip_h x_t

    The state pool S [slots, H, N, P] (fp32) is read at ``meta.slots``
    (zeros for a sequence with no cached tokens) and written back. All in
    fp32; returns y [T, H*P] fp32."""
    x_off, b_off, c_off = offs
    T = xbc.shape[0]
    assert xbc.dtype == torch.float32 and S.dtype == torch.float32
    assert S.shape[1:] == (H, N, P) and H % G == 0
    if xbc.is_cuda:
        chunk = SCAN_CHUNK
        while meta.T * H * N * P * 4 // chunk > (1 << 31):
            chunk *= 2                   # bound the chunk-state scratch
        if (max(meta.new_h) >= 4 * chunk
                and not os.environ.get("TL_NO_SCAN_CHUNKS")):
            # long prompt portions: chunk form. The intra-chunk part
            # (C B^T with the decay mask, times dt x), the chunk summary
            # Bw^T (dt x) and the carried part Cd S0 are batched fp32 GEMMs
            # over all chunks at once; only the chain of summaries is
            # sequential.
            C = _ext()
            cu_c, _, _, base, cnt, nc, _ = meta.scan_chunks(chunk)
            Cs, Cd, Bs, Bw, Xd, Lc, tot = C.ssd_chunk_prep(
                xbc, int(x_off), int(b_off), int(c_off), dt_src, int(dt_col),
                dt_bias, A_log, cu_c, int(H), int(P), int(N), int(G), chunk)
            A = torch.bmm(Cs, Bs.transpose(1, 2))
            C.ssd_decay_mask_(A, Lc)
            O = torch.bmm(A, Xd)
            U = torch.bmm(Bw.transpose(1, 2), Xd)
            C.ssd_chain_(U, S, tot, base, cnt, meta.slots, meta.pos0)
            O.baddbmm_(Cd, U)
            y = O.view(nc, H, chunk, P).transpose(1, 2).reshape(
                nc * chunk, H * P).index_select(0, meta.chunk_rows(chunk))
            y.view(T, H, P).addcmul_(
                xbc[:, x_off:x_off + H * P].view(T, H, P),
                skip.view(1, H, 1))
            return y
        return _ext().ssd_scan(xbc, int(x_off), int(b_off), int(c_off),
                               dt_src, int(dt_col), dt_bias, A_log, skip, S,
                               meta.cu, meta.slots, meta.pos0, int(H),
                               int(P), int(N), int(G))
    x = xbc[:, x_off:x_off + H * P].view(T, H, P)
    rep = H // G
    Bm = xbc[:, b_off:b_off + G * N].view(T, G, N).repeat_interleave(rep, 1)
    Cm = xbc[:, c_off:c_off + G * N].view(T, G, N).repeat_interleave(rep, 1)
    dt = torch.nn.functional.softplus(
        dt_src[:, dt_col:dt_col + H].float() + dt_bias)
    dec = torch.exp(-torch.exp(A_log) * dt)                    # [T, H]
    y = torch.empty(T, H, P)
    for b in range(meta.B):
        t0, t1 = meta.cu_h[b], meta.cu_h[b + 1]
        if t1 == t0:
            continue
        slot = meta.slots_h[b]
        Sb = (torch.zeros(H, N, P) if meta.pos0_h[b] == 0
              else S[slot].clone())
        for t in range(t0, t1):
            Sb = dec[t].view(H, 1, 1) * Sb + (dt[t].view(H, 1) * Bm[t]
                                              ).unsqueeze(-1) * x[t].unsqueeze(1)
            y[t] = (Sb * Cm[t].unsqueeze(-1)).sum(1) + skip.view(H, 1) * x[t]
        S[slot] = Sb
    return y.reshape(T, H * P)


def gated_group_rms(y: torch.Tensor, gate: torch.Tensor, gate_col: int,
                    w: torch.Tensor, groups: int, eps: float,
                    out_dtype=torch.float32) -> torch.Tensor:
    """u = y * silu(gate[:, gate_col:gate_col + N]); every one of
    ``groups`` equal parts of a row of u is divided by its own root mean
    square; times w [N]. y [T, N] fp32; fp32 arithmetic."""
    N = y.shape[1]
    assert y.dtype == torch.float32 and N % groups == 0
    if y.is_cuda:
        return _ext().gated_group_rms(y.contiguous(), gate, int(gate_col), w,
                                      int(groups), float(eps),
                                      out_dtype == torch.float32)
    u = y * torch.nn.functional.silu(gate[:, gate_col:gate_col + N].float())
    u = _rms(u.view(-1, groups, N // groups), eps).reshape(-1, N)
    return (u * w).to(out_dtype)


def postln_add(X: torch.Tensor, y: torch.Tensor, w: torch.Tensor, eps: float,
               y2: Optional[torch.Tensor] = None,
               wy: Optional[torch.Tensor] = None,
               wy2: Optional[torch.Tensor] = None) -> None:
    """Residual with a layer norm on the sublayer's OUTPUT, in place on the
    fp32 residual X [T, W]:  X += layer_norm(u) * w.  u = y, or with two
    branch outputs u = (y / rms(y) * wy + y2 / rms(y2) * wy2) / 2."""
    assert X.dtype == torch.float32 and w.dtype == torch.float32
    if X.is_cuda:
        _ext().postln_add(X, y.contiguous(), w, float(eps),
                          None if y2 is None else y2.contiguous(), wy, wy2)
        return
    u = y.float()
    if y2 is not None:
        u = 0.5 * (_rms(u, eps) * wy + _rms(y2.float(), eps) * wy2)
    X += _ln(u, w, eps)


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """coef[0] N(z) + coef[1] N(z^2) + coef[2] N(z^3) + coef[3] with
    element-wise powers and N(u) = u / rms(u) over a row; fp32 arithmetic,
    result in z's dtype."""
    assert coef.dtype == torch.float32 and coef.numel() == 4
    if z.is_cuda:
        return _ext().polynorm(z.contiguous(), coef, float(eps))
    f = z.float()
    f2 = f * f
    out = (coef[0] * _rms(f, eps) + coef[1] * _rms(f2, eps)
           + coef[2] * _rms(f2 * f, eps) + coef[3])
    return out.to(z.dtype)
