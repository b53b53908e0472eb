"""Potosun model family: a pre-norm layered decoder whose ``config.json``
lists every layer, x <- x + mixer(norm1(x)); x <- x + ff(norm2(x)), with RMS
norms (plain weights), an fp32 residual from the scaled embedding to the
soft-capped logits, and three attention mixers:

``attention``         position-free scores with per-head query/key norms, a
                      learned bucketed distance bias, a sliding window that
                      keeps the first tokens, an element-wise sigmoid output
                      gate;
``attention_2``       interleaved rotation, attention inside chunks counted
                      from the sequence's start, a learned sink logit per
                      head;
``latent_attention``  cached latents + one shared rotated key part
                      (rotate-half with an optional two-regime frequency
                      scaling), sliding window, sink logits, one output gate
                      per head.

Layers whose configuration says ``v_mix`` blend the values of the FIRST such
layer into their own before caching them. The feed-forward is
down(gelu_tanh(gate x) * up x).

The blocks live in :mod:`tensorlink_amd.models.mixers`; this file reads the
configuration, assembles them, maps checkpoint tensor names and runs the
stage over a flat ragged batch through the stage interface of
:class:`~tensorlink_amd.models.layered.LayeredStage`. One stage (PP = 1).
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field
from typing import List, Optional

import torch
import torch.nn as nn

from tensorlink_amd.models.configs import ModelConfig
from tensorlink_amd.models.dense import TLLinear
from tensorlink_amd.models.layered import (LayeredStage, load_named_tensors,
                                           tensor_shapes)
from tensorlink_amd.models.mixers import (GatedFF, LatentAttention, RMSWeight,
                                          WindowAttention)
from tensorlink_amd.ops import mixers as mx

MIXERS = ("attention", "attention_2", "latent_attention")


@dataclass
class PotosunConfig(ModelConfig):
    """Flat ModelConfig fields are filled for the planner and the engine;
    ``layer_specs`` (the checkpoint's ``layers`` list) is authoritative.
    The number of rows of a distance-bias table is no key of config.json:
    it is the table's shape, read from the checkpoint's header into the
    mixer's ``bias_rows`` (a configuration built by hand gives it)."""
    layer_specs: List[dict] = field(default_factory=list)
    embed_scale: float = 1.0
    logit_softcap: float = 0.0          # 0 = none
    architecture: str = "potosun"

    @classmethod
    def from_dict(cls, cfg: dict, name: str = "potosun") -> "PotosunConfig":
        if "layer_specs" in cfg:                     # own to_json round trip
            known = {f.name for f in cls.__dataclass_fields__.values()}
            return cls(**{k: v for k, v in cfg.items() if k in known})
        layers = json.loads(json.dumps(cfg["layers"]))       # own copy
        shapes = None
        mixed = None
        for i, lc in enumerate(layers):
            if lc["type"] not in MIXERS:
                raise KeyError(f"layer {i}: unknown mixer {lc['type']!r}")
            mlp = lc.get("mlp")
            if mlp is not None and mlp.get("kind") != "dense":
                raise KeyError(f"layer {i}: unknown feed-forward "
                               f"{mlp.get('kind')!r}")
            mc = lc["mixer"]
            if lc["type"] == "latent_attention":
                if mc["rot"]["dims"] != mc["rot_dim"] or mc["rot_dim"] % 2:
                    raise KeyError(f"layer {i}: the rotated part is rot_dim "
                                   "(even) wide")
                continue
            if mc["heads"] % mc["kv_heads"]:
                raise KeyError(f"layer {i}: heads must be a multiple of "
                               "kv_heads")
            if lc["type"] == "attention_2":
                rot = mc.get("rot") or {"dims": 0}
                if rot["dims"] % 2 or rot["dims"] > mc["dim"]:
                    raise KeyError(f"layer {i}: rot.dims must be even and "
                                   "at most dim")
            elif "bias_rows" not in mc:
                if shapes is None:
                    shapes = tensor_shapes(name)
                key = f"l{i}.mix.rel"
                if key not in shapes:
                    raise KeyError(f"layer {i}: the distance-bias table's "
                                   "size is neither configured nor in a "
                                   "checkpoint")
                mc["bias_rows"] = int(shapes[key][0])
            if mc.get("v_mix"):
                if mixed is None:
                    mixed = mc["kv_heads"] * mc["vdim"]
                elif mixed != mc["kv_heads"] * mc["vdim"]:
                    raise KeyError(f"layer {i}: value-mixing layers must "
                                   "agree in kv_heads * vdim")
        heads = max((lc["mixer"]["heads"] for lc in layers), default=1)
        kvh = max((lc["mixer"].get("kv_heads", 1) for lc in layers),
                  default=1)
        dim = max((lc["mixer"]["dim"] for lc in layers), default=1)
        inter = max((lc["mlp"]["ff"] for lc in layers
                     if lc.get("mlp") is not None), default=cfg["width"])
        return cls(
            name=name, vocab_size=cfg["vocab"], hidden_size=cfg["width"],
            intermediate_size=inter, num_hidden_layers=len(layers),
            num_attention_heads=heads, num_key_value_heads=kvh,
            head_dim=dim, rms_norm_eps=cfg["norm"]["eps"],
            tie_word_embeddings=False, layer_specs=layers,
            embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
            logit_softcap=float(cfg.get("logit_softcap") or 0.0))

    def param_count(self, include_embeddings: bool = True) -> int:
        w = self.hidden_size
        total = w
        for lc in self.layer_specs:
            mc = lc["mixer"]
            H, D, V = mc["heads"], mc["dim"], mc["vdim"]
            total += w + H * V * w
            if lc["type"] == "latent_attention":
                R, rd = mc["kv_rank"], mc["rot_dim"]
                total += w * (H * (D + rd) + R + rd + H) + R \
                    + H * (D + V) * R + H
            else:
                G = mc["kv_heads"]
                total += w * (H * D + G * D + G * V)
                if mc.get("v_mix"):
                    total += 1
                if lc["type"] == "attention":
                    total += 2 * D + mc["bias_rows"] * H + w * H * V
                else:
                    total += H
            if lc.get("mlp") is not None:
                total += w + 3 * w * lc["mlp"]["ff"]
        if include_embeddings:
            total += 2 * self.vocab_size * w
        return total


def build_mixer(lc: dict, width: int, eps: float) -> nn.Module:
    mc = lc["mixer"]
    mask = mc.get("mask") or {}
    if lc["type"] == "latent_attention":
        return LatentAttention(width, mc["heads"], mc["dim"], mc["rot_dim"],
                               mc["vdim"], mc["kv_rank"], mc["scale"],
                               mc["rot"]["base"], eps,
                               window=mask.get("size", 0),
                               rot_scaling=mc["rot"].get("scaling"),
                               sink_logits=True, head_gate=True)
    if lc["type"] == "attention":
        return WindowAttention(width, mc["heads"], mc["kv_heads"], mc["dim"],
                               mc["vdim"], mc["scale"], 0, 1.0,
                               mask.get("size", 0), eps, sink=False,
                               talk=False, qk_norm=True, head_norm=True,
                               keep_first=mask.get("keep_first", 0),
                               rel_rows=mc["bias_rows"],
                               rel_far=mc["bias_max"], out_gate=True,
                               v_mix=bool(mc.get("v_mix")))
    rot = mc.get("rot") or {"dims": 0, "base": 1.0}
    return WindowAttention(width, mc["heads"], mc["kv_heads"], mc["dim"],
                           mc["vdim"], mc["scale"], rot["dims"], rot["base"],
                           0, eps, sink=False, talk=False, qk_norm=False,
                           interleaved=True, chunk=mask.get("size", 0),
                           sink_logits=True, v_mix=bool(mc.get("v_mix")))


class PotosunLayer(nn.Module):
    def __init__(self, config: PotosunConfig, idx: int):
        super().__init__()
        lc = config.layer_specs[idx]
        w, eps = config.hidden_size, config.rms_norm_eps
        self.norm1 = RMSWeight(w, one_plus=False)
        self.mix = build_mixer(lc, w, eps)
        self.mlp = None
        if lc.get("mlp") is not None:
            self.norm2 = RMSWeight(w, one_plus=False)
            self.mlp = GatedFF(w, lc["mlp"]["ff"], tanh_form=True)


class PotosunStageModel(LayeredStage):
    """Whole-model stage (embedding, every layer, final norm + head)."""

    def __init__(self, config: PotosunConfig, layer_start: int,
                 layer_end: int, has_embedding: bool, has_head: bool):
        super().__init__()
        if not (has_embedding and has_head and layer_start == 0
                and layer_end == config.num_hidden_layers):
            raise ValueError("the Potosun family runs as a single stage "
                             "(fp32 residual); use world=1")
        self.config = config
        self.layer_start, self.layer_end = layer_start, layer_end
        self.has_embedding = self.has_head = True
        w = config.hidden_size
        self.embed_tokens = nn.Embedding(config.vocab_size, w)
        self.layers = nn.ModuleList([PotosunLayer(config, i)
                                     for i in range(config.num_hidden_layers)])
        self.norm = RMSWeight(w, one_plus=False)
        self.lm_head = TLLinear(w, config.vocab_size, bias=False)
        self.layer_sums = None      # list -> residual after every layer

    def head(self, hidden: torch.Tensor) -> torch.Tensor:
        """Final norm, vocabulary projection and soft cap of residual rows
        [..., W] (fp32); fp32 logits."""
        shape = hidden.shape
        x = hidden.reshape(-1, shape[-1]).float()
        h = mx.rms_scale(x, self.norm.w32(), self.config.rms_norm_eps, False,
                         out_dtype=self.lm_head.weight.dtype)
        z = self.lm_head(h).float()
        if self.config.logit_softcap:
            z = mx.soft_cap_(z, self.config.logit_softcap)
        return z.reshape(*shape[:-1], -1)

    @torch.no_grad()
    def forward(self, hidden_or_ids, positions, kv_cache=None,
                training: bool = False, return_logits: bool = True):
        if training:
            raise NotImplementedError(
                "the Potosun family is served, not trained, by this build")
        B, S = hidden_or_ids.shape[:2]
        dev = hidden_or_ids.device
        dtype = self.lm_head.weight.dtype
        cfg = self.config
        eps = cfg.rms_norm_eps
        if kv_cache is None:
            kv_cache = self.make_kv_cache(B, int(positions.max()) + 1, dev,
                                          dtype)
        meta = self._meta(kv_cache, positions, B, S)
        X = self.embed_tokens(hidden_or_ids.reshape(-1)).float().contiguous()
        # the embedding's scale rides on the first norm's pass over X; the
        # output of every sublayer is added by the NEXT sublayer's norm
        scale, y = cfg.embed_scale, None
        shared = {}                 # what layers of one step hand on
        for li, layer in enumerate(self.layers):
            h = mx.add_rms(X, y, layer.norm1.w32(), eps, dtype, x_scale=scale)
            scale = 1.0
            if self.layer_sums is not None and li > 0:
                self.layer_sums.append(X.clone())
            y = layer.mix(h, meta, kv_cache, li, shared)
            if layer.mlp is not None:
                h = mx.add_rms(X, y, layer.norm2.w32(), eps, dtype)
                y = layer.mlp(h)
        if y is not None or scale != 1.0:
            mx.add_rms(X, y, None, eps, dtype, x_scale=scale)
            if self.layer_sums is not None and y is not None:
                self.layer_sums.append(X.clone())
        if kv_cache is not None:
            kv_cache.advance(S)
        u = X.view(B, S, -1)
        return self.head(u) if return_logits else u


# ------------------------------------------------------------------ weights
def _name_map(stage: PotosunStageModel):
    """checkpoint tensor name -> (parameter, row offset)."""
    P = dict(stage.named_parameters())
    m = {"embed": ("embed_tokens.weight", 0), "head": ("lm_head.weight", 0),
         "final.norm": ("norm.weight", 0)}
    for i, layer in enumerate(stage.layers):
        a, b = f"l{i}.", f"layers.{i}."
        m[f"{a}norm1"] = (f"{b}norm1.weight", 0)
        mix = layer.mix
        if mix.kind == "latent_attention":
            m[f"{a}mix.q"] = (f"{b}mix.qdkv.weight", 0)
            m[f"{a}mix.dkv"] = (f"{b}mix.qdkv.weight", mix.q_cols)
            m[f"{a}mix.g"] = (f"{b}mix.qdkv.weight",
                              mix.q_cols + mix.kv_cols)
            m[f"{a}mix.dkv.norm"] = (f"{b}mix.dkv_norm", 0)
            m[f"{a}mix.uk"] = (f"{b}mix.uk", 0)
            m[f"{a}mix.uv"] = (f"{b}mix.uv", 0)
            m[f"{a}mix.sink"] = (f"{b}mix.sink", 0)
        else:
            v_col = mix.q_cols + mix.k_cols
            m[f"{a}mix.q"] = (f"{b}mix.qkv.weight", 0)
            m[f"{a}mix.k"] = (f"{b}mix.qkv.weight", mix.q_cols)
            m[f"{a}mix.v"] = (f"{b}mix.qkv.weight", v_col)
            if mix.g_cols:
                m[f"{a}mix.g"] = (f"{b}mix.qkv.weight", v_col + mix.v_cols)
            if mix.q_norm is not None:
                m[f"{a}mix.q.norm"] = (f"{b}mix.q_norm", 0)
                m[f"{a}mix.k.norm"] = (f"{b}mix.k_norm", 0)
            if mix.rel is not None:
                m[f"{a}mix.rel"] = (f"{b}mix.rel", 0)
            if mix.sinks is not None:
                m[f"{a}mix.sink"] = (f"{b}mix.sinks", 0)
            if mix.vmix is not None:
                m[f"{a}mix.vmix"] = (f"{b}mix.vmix", 0)
        m[f"{a}mix.o"] = (f"{b}mix.o_proj.weight", 0)
        if layer.mlp is not None:
            m[f"{a}norm2"] = (f"{b}norm2.weight", 0)
            m[f"{a}mlp.gate"] = (f"{b}mlp.gate_up.weight", 0)
            m[f"{a}mlp.up"] = (f"{b}mlp.gate_up.weight", layer.mlp.ff)
            m[f"{a}mlp.down"] = (f"{b}mlp.down.weight", 0)
    return m, P


@torch.no_grad()
def load_potosun_weights(stage: PotosunStageModel, ckpt_dir: str,
                         dtype=torch.bfloat16) -> int:
    """Fill the stage from ``model.safetensors``; every tensor of the
    checkpoint must be consumed and every parameter filled. The blending
    weight of the first value-mixing layer has no use; the checkpoint may
    or may not hold one."""
    names, P = _name_map(stage)
    first = next((f"layers.{i}.mix.vmix" for i, l in enumerate(stage.layers)
                  if getattr(l.mix, "vmix", None) is not None), None)
    return load_named_tensors(P, names, ckpt_dir,
                              optional=[first] if first else ())


@torch.no_grad()
def init_potosun_random(stage: PotosunStageModel, seed: int = 0) -> None:
    """Scaled-normal matrices, norm weights near one, small biases, sinks
    and blending weights: finite activations at any depth for benchmarks
    and tests."""
    g = torch.Generator().manual_seed(seed)
    scale = stage.config.embed_scale
    for name, p in stage.named_parameters():
        leaf = name.rsplit(".", 1)[-1]
        t = torch.empty(p.shape, dtype=torch.float32)
        if name.endswith((".norm1.weight", ".norm2.weight")) \
                or name == "norm.weight" \
                or leaf in ("q_norm", "k_norm", "dkv_norm"):
            t = 1.0 + 0.1 * torch.randn(p.shape, generator=g)
        elif leaf in ("sink", "sinks"):
            t = 0.5 * torch.randn(p.shape, generator=g)
        elif leaf == "rel":
            t = 0.5 * torch.randn(p.shape, generator=g)
        elif leaf == "vmix":
            t = 0.2 + 0.5 * torch.rand(p.shape, generator=g)
        elif name == "embed_tokens.weight":
            t.normal_(0.0, 1.0 / scale, generator=g)
        else:
            t.normal_(0.0, 1.0 / math.sqrt(p.shape[-1]), generator=g)
        p.copy_(t.to(p.dtype))


def read_config(path: str) -> Optional[PotosunConfig]:
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    if cfg.get("architecture") in ("Potosun", "potosun"):
        return PotosunConfig.from_dict(cfg, name=path)
    return None
