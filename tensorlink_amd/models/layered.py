"""What the layered model families share: a stage whose ``config.json``
lists its layers one by one, whose mixers keep their per-sequence memory
in a :class:`~tensorlink_amd.models.paged.HybridSlotCache` (page pools per
layer, pools shared between layers, fp32 recurrent state per slot) and
which runs a flat ragged batch in one forward pass.

A family file derives its stage from :class:`LayeredStage`, gives every
layer a ``mix`` module with ``cache_spec()`` and fills ``forward``; the
runner, the continuous batcher and the engine then drive it through the
usual stage interface (embed / forward / head / make_kv_cache).
"""

from __future__ import annotations

import os
from typing import Dict, Iterable, Tuple

import torch
import torch.nn as nn

from tensorlink_amd.ops import mixers as mx


class LayeredStage(nn.Module):
    SUPPORTS_RAGGED = True      # one forward serves a mixed ragged batch
    GRAPH_CAPTURE = False       # host-built ragged metadata every step

    @property
    def num_layers(self):
        return len(self.layers)

    # ---------------------------------------------------------- cache
    def cache_specs(self):
        return [l.mix.cache_spec() for l in self.layers]

    def make_slot_cache(self, slots: int, pool_pages: int, max_seq: int,
                        device, dtype):
        from tensorlink_amd.models.paged import HybridSlotCache
        return HybridSlotCache(self.cache_specs(), slots, pool_pages,
                               max_seq, device, dtype)

    def make_kv_cache(self, batch: int, max_seq: int, device, dtype=None,
                      kv_mode: str = "paged"):
        """Rectangular-batch cache for ``PipelineRunner.generate``: one
        slot per row with its pages leased up front."""
        from tensorlink_amd.models.paged import PAGE
        if dtype is None:
            dtype = self.lm_head.weight.dtype
        pps = (max_seq + PAGE - 1) // PAGE
        cache = self.make_slot_cache(batch, batch * pps, max_seq, device,
                                     dtype)
        for s in range(batch):
            cache.ensure(s, max_seq)
        cache.static = True
        return cache

    def _meta(self, kv_cache, positions, B, S):
        meta = getattr(kv_cache, "ragged", None)
        if meta is not None:
            return meta
        # rectangular batch: B sequences of S new tokens each
        pos0 = positions.reshape(B, S)[:, 0].tolist()
        slots = getattr(kv_cache, "slot_ids", None)
        if slots is None:
            slots = list(range(B))
        return mx.RaggedMeta([S] * B, pos0, slots, kv_cache.table[:B],
                             positions.device)

    def embed(self, input_ids):
        return self.embed_tokens(input_ids)


def tensor_shapes(ckpt_dir: str) -> Dict[str, Tuple[int, ...]]:
    """Tensor name -> shape from the header of ``model.safetensors`` in
    ``ckpt_dir`` (an 8-byte little-endian length, then that many bytes of
    JSON); no tensor data is read. Empty if there is no such file."""
    import json
    import struct
    path = os.path.join(ckpt_dir, "model.safetensors")
    if not os.path.isfile(path):
        return {}
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
    return {k: tuple(v["shape"]) for k, v in header.items()
            if k != "__metadata__"}


@torch.no_grad()
def load_named_tensors(params: Dict[str, torch.Tensor],
                       names: Dict[str, Tuple[str, int]], ckpt_dir: str,
                       optional: Iterable[str] = (),
                       partial: Dict[str, int] = None) -> int:
    """Fill ``params`` from ``model.safetensors``. ``names`` maps a
    checkpoint tensor to (parameter, row offset — or expert index for a
    stacked 3-d parameter). Strict both ways: an unknown tensor raises and
    so does a parameter left (partly) unfilled, unless listed in
    ``optional`` and untouched; ``partial`` names parameters that the
    checkpoint fills only up to the given number of elements (the rest
    keeps the caller's values)."""
    from safetensors import safe_open
    filled = {k: 0 for k in params}
    loaded = 0
    with safe_open(os.path.join(ckpt_dir, "model.safetensors"),
                   framework="pt", device="cpu") as f:
        for key in f.keys():
            if key not in names:
                raise KeyError(f"unexpected tensor {key!r} in checkpoint")
            pname, off = names[key]
            t = f.get_tensor(key)
            p = params[pname]
            if p.dim() == 0:
                p.copy_(t.reshape(()))
            elif p.dim() == 3:                      # stacked experts
                p[off].copy_(t)
            else:
                if t.shape[1:] != p.shape[1:] or off + t.shape[0] > p.shape[0]:
                    raise KeyError(f"tensor {key!r} has shape "
                                   f"{tuple(t.shape)}, which does not fit "
                                   "the configuration")
                p[off:off + t.shape[0]].copy_(t)
            filled[pname] += t.numel()
            loaded += 1
    optional = set(optional)
    partial = partial or {}
    short = [k for k, n in filled.items()
             if n != partial.get(k, params[k].numel())
             and not (n == 0 and k in optional)]
    if short:
        raise KeyError(f"checkpoint leaves parameters unfilled: {short[:5]}")
    return loaded
