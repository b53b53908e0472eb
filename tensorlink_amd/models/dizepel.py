"""Dizepel model family: a layered decoder whose ``config.json`` lists
every layer. A layer's mixer is a pair of mixers fed by the same input
— softmax attention with short convolutions, a learned sink and capped
scores whose values are its unrotated keys, and a selective state-space
(SSD) mixer — followed by an optional PolyNorm feed-forward. Every
sublayer reads layer_norm(x) plus a causal convolution of it over time and
is added back through a second layer norm: x <- x + ln_b(f(h + conv(h))),
h = ln(x). A span of layers may run several times in a row with the same
weights (``loop``); each pass has its own cache pages and state and adds
its own learned vector to the residual first. The residual is fp32.

The blocks live in :mod:`tensorlink_amd.models.mixers`; this file reads
the configuration, assembles them, maps checkpoint tensor names and runs
the stage over a flat ragged batch through the stage interface of
:class:`~tensorlink_amd.models.layered.LayeredStage`. One stage (PP = 1).
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field
from typing import List, Optional, Tuple

import torch
import torch.nn as nn

from tensorlink_amd.models.configs import ModelConfig
from tensorlink_amd.models.dense import TLLinear
from tensorlink_amd.models.layered import LayeredStage, load_named_tensors
from tensorlink_amd.models.mixers import (CanonConv, ConvSinkAttention,
                                          LayerNormWeight, ParallelMixer,
                                          PolyNormFF, SSDMixer)
from tensorlink_amd.ops import mixers as mx

MIXERS = ("parallel",)


@dataclass
class DizepelConfig(ModelConfig):
    """Flat ModelConfig fields are filled for the planner and the engine;
    ``layer_specs`` (the checkpoint's ``layers`` list) is authoritative."""
    layer_specs: List[dict] = field(default_factory=list)
    embed_scale: float = 1.0
    canon_taps: int = 1
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 0                 # 0 = no looped span
    architecture: str = "dizepel"

    @classmethod
    def from_dict(cls, cfg: dict, name: str = "dizepel") -> "DizepelConfig":
        if "layer_specs" in cfg:                     # own to_json round trip
            known = {f.name for f in cls.__dataclass_fields__.values()}
            return cls(**{k: v for k, v in cfg.items() if k in known})
        layers = cfg["layers"]
        for i, lc in enumerate(layers):
            if lc["type"] not in MIXERS:
                raise KeyError(f"layer {i}: unknown mixer {lc['type']!r}")
            mlp = lc.get("mlp")
            if mlp is not None and mlp.get("kind") != "dense":
                raise KeyError(f"layer {i}: unknown feed-forward "
                               f"{mlp.get('kind')!r}")
            left, right = lc["mixer"]["left"], lc["mixer"]["right"]
            if left["vdim"] != left["dim"]:
                raise KeyError(f"layer {i}: the values are the keys, so "
                               "vdim must equal dim")
            if left["heads"] % left["kv_heads"]:
                raise KeyError(f"layer {i}: heads must be a multiple of "
                               "kv_heads")
            if right["heads"] % right["groups"] or \
                    (right["heads"] * right["vdim"]) % right["norm_groups"]:
                raise KeyError(f"layer {i}: heads / groups / norm_groups of "
                               "the state-space mixer do not divide")
        loop = cfg.get("loop") or {}
        n = len(layers)
        start, stop = int(loop.get("start", 0)), int(loop.get("stop", 0))
        times = int(loop.get("times", 0)) if loop else 0
        if loop and not (0 <= start <= stop <= n and times >= 1):
            raise KeyError("loop: need 0 <= start <= stop <= layers and "
                           "times >= 1")
        heads = max(lc["mixer"]["left"]["heads"] for lc in layers)
        kvh = max(lc["mixer"]["left"]["kv_heads"] for lc in layers)
        dim = max(lc["mixer"]["left"]["dim"] for lc in layers)
        inter = max((lc["mlp"]["ff"] for lc in layers
                     if lc.get("mlp") is not None), default=cfg["width"])
        return cls(
            name=name, vocab_size=cfg["vocab"], hidden_size=cfg["width"],
            intermediate_size=inter, num_hidden_layers=n,
            num_attention_heads=heads, num_key_value_heads=kvh,
            head_dim=dim, rms_norm_eps=cfg["norm"]["eps"],
            tie_word_embeddings=False, layer_specs=layers,
            embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
            canon_taps=int((cfg.get("canon") or {}).get("taps", 1)),
            loop_start=start, loop_stop=stop, loop_times=times)

    def layer_runs(self) -> List[Tuple[int, Optional[int]]]:
        """(layer index, pass number or None) in execution order; every
        run has its own cache entry."""
        n = len(self.layer_specs)
        if not self.loop_times:
            return [(i, None) for i in range(n)]
        runs = [(i, None) for i in range(self.loop_start)]
        for t in range(self.loop_times):
            runs += [(i, t) for i in range(self.loop_start, self.loop_stop)]
        return runs + [(i, None) for i in range(self.loop_stop, n)]

    def param_count(self, include_embeddings: bool = True) -> int:
        w = self.hidden_size
        total = w + self.loop_times * w
        for lc in self.layer_specs:
            L, R = lc["mixer"]["left"], lc["mixer"]["right"]
            qk = (L["heads"] + L["kv_heads"]) * L["dim"]
            inner = R["heads"] * R["vdim"]
            cc = inner + 2 * R["groups"] * R["state"]
            total += 2 * w + w * self.canon_taps
            total += qk * (w + 1 + L["conv"]) + L["heads"] \
                + w * L["heads"] * L["dim"]
            total += w * (inner + cc + R["heads"]) + cc * (R["conv"] + 1) \
                + 3 * R["heads"] + inner + w * inner + 2 * w
            if lc.get("mlp") is not None:
                total += 2 * w + w * self.canon_taps \
                    + 2 * w * lc["mlp"]["ff"] + 4
        if include_embeddings:
            total += 2 * self.vocab_size * w
        return total


def build_mixer(lc: dict, width: int, eps: float) -> nn.Module:
    L, R = lc["mixer"]["left"], lc["mixer"]["right"]
    rot = L.get("rot") or {"dims": 0, "base": 1.0}
    left = ConvSinkAttention(width, L["heads"], L["kv_heads"], L["dim"],
                             L["conv"], L["scale"], L.get("softcap") or 0.0,
                             rot["dims"], rot["base"], rot.get("scaling"))
    right = SSDMixer(width, R["heads"], R["vdim"], R["state"], R["groups"],
                     R["conv"], R["norm_groups"], eps)
    return ParallelMixer(width, left, right)


class DizepelLayer(nn.Module):
    def __init__(self, config: DizepelConfig, idx: int):
        super().__init__()
        lc = config.layer_specs[idx]
        w, eps = config.hidden_size, config.rms_norm_eps
        self.norm1 = LayerNormWeight(w)
        self.norm1b = LayerNormWeight(w)
        self.canon1 = CanonConv(w, config.canon_taps)
        self.mix = build_mixer(lc, w, eps)
        self.mlp = None
        if lc.get("mlp") is not None:
            self.norm2 = LayerNormWeight(w)
            self.norm2b = LayerNormWeight(w)
            self.canon2 = CanonConv(w, config.canon_taps)
            self.mlp = PolyNormFF(w, lc["mlp"]["ff"], eps)

    def cache_spec(self):
        """The mixer's pools and state, preceded by the histories of the
        layer's own input convolutions."""
        own = [self.canon1.state_shape]
        if self.mlp is not None:
            own.append(self.canon2.state_shape)
        sp = self.mix.cache_spec()
        return dict(sp, shapes=own + list(sp["shapes"]))

    def forward(self, X, meta, cache, run: int, eps: float, dtype):
        """One run of the layer on the fp32 residual X [T, W], in place;
        ``run`` names the cache entry of this pass."""
        st = cache.state[run]
        n_own = 2 if self.mlp is not None else 1
        h = mx.ln_canon(X, self.norm1.w32(), eps, self.canon1.w32(), st[0],
                        meta, dtype)
        a, b = self.mix(h, meta, cache.k[run], cache.v[run], st[n_own:])
        mx.postln_add(X, a, self.norm1b.w32(), eps, y2=b,
                      wy=self.mix._f32("left_out"),
                      wy2=self.mix._f32("right_out"))
        if self.mlp is not None:
            h = mx.ln_canon(X, self.norm2.w32(), eps, self.canon2.w32(),
                            st[1], meta, dtype)
            mx.postln_add(X, self.mlp(h), self.norm2b.w32(), eps)


class DizepelStageModel(LayeredStage):
    """Whole-model stage (embedding, every layer run, final norm + head)."""

    def __init__(self, config: DizepelConfig, layer_start: int,
                 layer_end: int, has_embedding: bool, has_head: bool):
        super().__init__()
        if not (has_embedding and has_head and layer_start == 0
                and layer_end == config.num_hidden_layers):
            raise ValueError("the Dizepel family runs as a single stage "
                             "(fp32 residual); use world=1")
        self.config = config
        self.layer_start, self.layer_end = layer_start, layer_end
        self.has_embedding = self.has_head = True
        w = config.hidden_size
        self.embed_tokens = nn.Embedding(config.vocab_size, w)
        self.layers = nn.ModuleList([DizepelLayer(config, i)
                                     for i in range(config.num_hidden_layers)])
        self.loop_step = (nn.Parameter(torch.zeros(config.loop_times, w))
                          if config.loop_times else None)
        self.norm = LayerNormWeight(w)
        self.lm_head = TLLinear(w, config.vocab_size, bias=False)
        self.runs = config.layer_runs()
        self.layer_sums = None      # list -> residual after every layer run

    def cache_specs(self):
        """One cache entry per layer RUN: a looped layer's passes do not
        share pages or state."""
        return [self.layers[i].cache_spec() for i, _ in self.runs]

    def head(self, hidden: torch.Tensor) -> torch.Tensor:
        """Final layer norm and vocabulary projection of residual rows
        [..., W] (fp32); fp32 logits."""
        shape = hidden.shape
        x = hidden.reshape(-1, shape[-1]).float()
        h = mx.layer_norm_rows(x, self.norm.w32(), self.config.rms_norm_eps,
                               out_dtype=self.lm_head.weight.dtype)
        return self.lm_head(h).float().reshape(*shape[:-1], -1)

    @torch.no_grad()
    def forward(self, hidden_or_ids, positions, kv_cache=None,
                training: bool = False, return_logits: bool = True):
        if training:
            raise NotImplementedError(
                "the Dizepel family is served, not trained, by this build")
        B, S = hidden_or_ids.shape[:2]
        dev = hidden_or_ids.device
        dtype = self.lm_head.weight.dtype
        cfg = self.config
        eps = cfg.rms_norm_eps
        if kv_cache is None:
            kv_cache = self.make_kv_cache(B, int(positions.max()) + 1, dev,
                                          dtype)
        meta = self._meta(kv_cache, positions, B, S)
        X = self.embed_tokens(hidden_or_ids.reshape(-1)).float()
        if cfg.embed_scale != 1.0:
            X = X * cfg.embed_scale
        X = X.contiguous()
        steps = (self.loop_step.detach().float()
                 if self.loop_step is not None else None)
        for run, (li, t) in enumerate(self.runs):
            if t is not None and li == cfg.loop_start:
                X += steps[t]
            self.layers[li](X, meta, kv_cache, run, eps, dtype)
            if self.layer_sums is not None:
                self.layer_sums.append(X.clone())
        if kv_cache is not None:
            kv_cache.advance(S)
        u = X.view(B, S, -1)
        return self.head(u) if return_logits else u


# ------------------------------------------------------------------ weights
def _name_map(stage: DizepelStageModel):
    """checkpoint tensor name -> (parameter, row offset)."""
    P = dict(stage.named_parameters())
    m = {"embed": ("embed_tokens.weight", 0), "head": ("lm_head.weight", 0),
         "final.norm": ("norm.weight", 0)}
    if stage.loop_step is not None:
        m["loop.step"] = ("loop_step", 0)
    for i, layer in enumerate(stage.layers):
        a, b = f"l{i}.", f"layers.{i}."
        for nm in ("norm1", "norm1b", "canon1"):
            m[a + nm] = (f"{b}{nm}.weight", 0)
        left, right = layer.mix.left, layer.mix.right
        m[f"{a}mix.left.q"] = (f"{b}mix.proj.weight", 0)
        m[f"{a}mix.left.k"] = (f"{b}mix.proj.weight", left.q_cols)
        m[f"{a}mix.right.in"] = (f"{b}mix.proj.weight", left.in_cols)
        m[f"{a}mix.left.q.b"] = (f"{b}mix.proj.bias", 0)
        m[f"{a}mix.left.k.b"] = (f"{b}mix.proj.bias", left.q_cols)
        m[f"{a}mix.left.q.conv"] = (f"{b}mix.left.qk_conv", 0)
        m[f"{a}mix.left.k.conv"] = (f"{b}mix.left.qk_conv", left.q_cols)
        m[f"{a}mix.left.sink"] = (f"{b}mix.left.sink", 0)
        m[f"{a}mix.left.o"] = (f"{b}mix.left.o_proj.weight", 0)
        m[f"{a}mix.right.conv"] = (f"{b}mix.right.conv", 0)
        m[f"{a}mix.right.conv.b"] = (f"{b}mix.right.conv_b", 0)
        for nm in ("dt_bias", "A_log", "D", "norm"):
            m[f"{a}mix.right.{nm}"] = (f"{b}mix.right.{nm}", 0)
        m[f"{a}mix.right.o"] = (f"{b}mix.right.o_proj.weight", 0)
        m[f"{a}mix.left.out"] = (f"{b}mix.left_out", 0)
        m[f"{a}mix.right.out"] = (f"{b}mix.right_out", 0)
        if layer.mlp is not None:
            for nm in ("norm2", "norm2b", "canon2"):
                m[a + nm] = (f"{b}{nm}.weight", 0)
            m[f"{a}mlp.up"] = (f"{b}mlp.up.weight", 0)
            m[f"{a}mlp.down"] = (f"{b}mlp.down.weight", 0)
            m[f"{a}mlp.act"] = (f"{b}mlp.act", 0)
    return m, P


@torch.no_grad()
def load_dizepel_weights(stage: DizepelStageModel, ckpt_dir: str,
                         dtype=torch.bfloat16) -> int:
    """Fill the stage from ``model.safetensors``; every tensor of the
    checkpoint must be consumed and every parameter filled. The fused
    projection's bias covers only the attention's columns; the rest stays
    zero."""
    names, P = _name_map(stage)
    partial = {}
    for i, layer in enumerate(stage.layers):
        P[f"layers.{i}.mix.proj.bias"].zero_()
        partial[f"layers.{i}.mix.proj.bias"] = layer.mix.left.bias_cols
    return load_named_tensors(P, names, ckpt_dir, partial=partial)


@torch.no_grad()
def init_dizepel_random(stage: DizepelStageModel, seed: int = 0) -> None:
    """Scaled-normal matrices, norm weights near one, taps near a delta on
    the current token, step sizes and decays in the usual range: finite
    activations at any depth for benchmarks and tests."""
    g = torch.Generator().manual_seed(seed)
    for name, p in stage.named_parameters():
        leaf = name.rsplit(".", 1)[-1]
        t = torch.empty(p.shape, dtype=torch.float32)
        if ".norm" in name and name.endswith(".weight") \
                or name == "norm.weight" \
                or leaf in ("norm", "left_out", "right_out"):
            t = 1.0 + 0.1 * torch.randn(p.shape, generator=g)
        elif ".canon" in name:
            t = 0.2 * torch.randn(p.shape, generator=g)
        elif leaf in ("qk_conv", "conv"):
            t = 0.3 * torch.randn(p.shape, generator=g)
            t[:, -1] += 1.0
        elif leaf in ("conv_b", "sink", "loop_step") or name.endswith(
                "proj.bias"):
            t = 0.2 * torch.randn(p.shape, generator=g)
        elif leaf == "dt_bias":
            t = torch.rand(p.shape, generator=g) * 3.0 - 4.0
        elif leaf == "A_log":
            t = torch.log(1.0 + 7.0 * torch.rand(p.shape, generator=g))
        elif leaf == "D":
            t = 1.0 + 0.2 * torch.randn(p.shape, generator=g)
        elif leaf == "act":
            t = torch.tensor([0.6, 0.3, 0.2, 0.05])
        elif name == "embed_tokens.weight":
            t.normal_(0.0, 1.0, generator=g)
        else:
            t.normal_(0.0, 1.0 / math.sqrt(p.shape[-1]), generator=g)
        p.copy_(t.to(p.dtype))


def read_config(path: str) -> Optional[DizepelConfig]:
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    if cfg.get("architecture") in ("Dizepel", "dizepel"):
        return DizepelConfig.from_dict(cfg, name=path)
    return None
