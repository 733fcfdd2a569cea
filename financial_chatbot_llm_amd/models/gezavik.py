"""Gezavik: a layered hybrid decoder of parallel blocks.

``config.json`` lists the layers; each has one sequence mixer (``mamba2`` or ``latent_attention``,
:mod:`.mixers`) and optionally one feed-forward (dense relu^2 or a routed mixture), both reading the
SAME normed input:

    h = RMSnorm(x) * w_norm1;   x <- x + residual_mult * (mixer(h) + ff(h))

and the model ends with RMSnorm * ``final.norm`` and the ``head`` projection.  The residual stream
``x`` is f32 whatever the activation dtype; each block's update is fused with the next block's norm
(one pass over ``x``), and the mixer's and feed-forward's input projections are one stacked GEMM.

Checkpoint tensors: ``embed``, ``l<i>.norm1``, ``l<i>.mix.<name>``, ``l<i>.mlp.<name>``,
``final.norm``, ``head`` (linear weights [out, in]).  Tensor parallelism is not implemented for this
design (TP = 1); data parallel replicas work as for every model.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F

from ..ops import mixers as mx
from .common import AttentionMetadata, HybridCache
from .configs import ModelConfig
from .layered import Layer, LayeredDecoder
from .mixers import DenseFF, RoutedFF


def example_config(width: int = 192, vocab: int = 1024, heads: int = 3, pattern: str = "amAm",
                   scale_up: bool = False) -> Dict:
    """A config.json-shaped dict for random-weight models (tests, benchmarks).  ``pattern``: one letter
    per layer -- a/A latent attention, m/M mamba2; lower case with a dense feed-forward, upper case
    with a routed one.  ``scale_up``: sizes in the range of a real model's layers."""
    if scale_up:
        att = {"dim": 96, "heads": heads, "kv_rank": 256, "mask": {"size": 1024}, "q_rank": 768,
               "rot": {"base": 10000.0, "dims": 32}, "rot_dim": 32, "scale": (96 + 32) ** -0.5, "vdim": 96}
        mam = {"conv": 4, "groups": 2, "heads": 2 * width // 64, "norm_groups": 2, "state": 128, "vdim": 64}
        dense = {"ff": 3 * width, "kind": "dense"}
        moe = {"expert": {"ff": width // 2, "limit": 7.0}, "kind": "moe",
               "router": {"experts": 32, "identity": 2, "top": 4}, "shared": {"ff": width, "limit": 7.0}}
    else:
        att = {"dim": 24, "heads": heads, "kv_rank": 40, "mask": {"size": 21}, "q_rank": 56,
               "rot": {"base": 10000.0, "dims": 8}, "rot_dim": 8, "scale": 32 ** -0.5, "vdim": 20}
        mam = {"conv": 3, "groups": 2, "heads": 6, "norm_groups": 2, "state": 24, "vdim": 20}
        dense = {"ff": 160, "kind": "dense"}
        moe = {"expert": {"ff": 48, "limit": 1.5}, "kind": "moe", "router": {"experts": 6, "identity": 2, "top": 3},
               "shared": {"ff": 72, "limit": 2.5}}
    layers = []
    for ch in pattern:
        layers.append({"type": "latent_attention" if ch in "aA" else "mamba2", "mixer": dict(att if ch in "aA" else mam),
                       "mlp": dict(moe if ch.isupper() else dense)})
    return {"architecture": "Gezavik", "layers": layers, "norm": {"eps": 1e-5}, "residual_mult": 0.5, "vocab": vocab,
            "width": width}


class _Layer(Layer):
    def __init__(self, i: int, spec: Dict, width: int, eps: float):
        super().__init__(i, spec, width, eps, GezavikModel.mixer_types)
        mlp = spec.get("mlp")
        if mlp is None:
            self.ff = None
        elif mlp["kind"] == "dense":
            self.ff = DenseFF(mlp, width, act="relu2")
        elif mlp["kind"] == "moe":
            self.ff = RoutedFF(mlp, width, alpha=1.702)
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")


class GezavikModel(LayeredDecoder):
    arch = "gezavik"
    mixer_types = ("mamba2", "latent_attention")

    def __init__(self, cfg: ModelConfig, device="cuda", dtype=torch.bfloat16):
        super().__init__(cfg, device, dtype)
        self.has_state = any(l.mixer.kind == "mamba2" for l in self.layers)
        self.mult = float(cfg.residual_mult)

    def make_layer(self, i: int, spec: Dict) -> Layer:
        return _Layer(i, spec, self.cfg.hidden_size, self.cfg.norm_eps)

    def load_layer(self, l: Layer, get) -> None:
        dt = self.dtype
        l.norm1 = get(l.prefix + ".norm1").float().contiguous()
        parts = [l.mixer.load(lambda k, p=l.prefix: get(f"{p}.mix.{k}"), dt)]
        if l.ff is not None:
            w = l.ff.load(lambda k, p=l.prefix: get(f"{p}.mlp.{k}"), dt)
            if w is not None:
                parts.append(w)
        l.w_in = torch.cat(parts, 0).contiguous()         # ONE in-projection per block

    # -- forward -----------------------------------------------------------------------------------
    def forward(self, ids: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, kv: HybridCache) -> torch.Tensor:
        """Final-normed hidden states [T, width] of every row of the step."""
        eps = self.cfg.norm_eps
        if meta.seg_cu is None:
            raise ValueError("this model needs the segment view of the step (AttentionMetadata.seg_*)")
        x = mx.embed_f32(ids, self.embed)
        h = mx.residual_norm(x, self.layers[0].norm1, eps, out_dtype=self.dtype)
        n = len(self.layers)
        for i, l in enumerate(self.layers):
            proj = F.linear(h, l.w_in)
            nm = l.mixer.in_rows
            a = l.mixer.forward(proj[:, :nm], positions, meta, kv.layers[i])
            b = l.ff.forward(h, proj[:, nm:]) if l.ff is not None else None
            w_next = self.layers[i + 1].norm1 if i + 1 < n else self.final_norm
            h = mx.residual_norm(x, w_next, eps, a, b, self.mult, out_dtype=self.dtype)
            if self.capture is not None:
                self.capture.append(x.clone())
        return h
