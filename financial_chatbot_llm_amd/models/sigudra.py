"""Sigudra: a layered decoder of sequential blocks with the norm on each sublayer's OUTPUT.

``config.json`` lists the layers; each has one sequence mixer -- ``channel_delta`` (gated delta rule
with per-channel decay), ``gla`` (gated linear attention) or ``parallel`` (sliding-window attention
beside a gated-LRU block), see :mod:`.mixers` -- and optionally one feed-forward (gated GeLU, or a
mixture of SiLU experts whose sigmoid score scales the expert's input):

    x <- x + LN(mixer(x)) * w_norm1;      x <- x + LN(ff(x)) * w_norm2

with LN the weight-only layer norm; the sublayers read ``x`` itself (rounded to the activation dtype
for the projections).  The embedding is ``embed[token]`` plus a hashed token-pair row
``bigram[(prev * mul_prev + token * mul_cur) mod buckets]`` (row ``buckets`` for a sequence's first
token); the previous token is kept per state slot between steps.  The model ends with
LN * ``final.norm`` and the ``head`` projection.  The residual stream ``x`` is f32 whatever the
activation dtype; each sublayer's norm, the residual add and the rounding of the next GEMM input are
one kernel.

Checkpoint tensors: ``embed``, ``bigram``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.<name>``,
``l<i>.mlp.<name>``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from typing import Dict

import torch
import torch.nn.functional as F

from ..ops import mixers as mx
from .common import AttentionMetadata, HybridCache
from .configs import ModelConfig
from .layered import Layer, LayeredDecoder
from .mixers import DenseFF, InputScaledRoutedFF


def example_config(width: int = 160, vocab: int = 640, pattern: str = "dGPd", scale_up: bool = False, heads: int = 0) -> Dict:
    """A config.json-shaped dict for random-weight models (tests, benchmarks).  ``pattern``: one letter
    per layer -- d/D channel_delta, g/G gla, p/P parallel; lower case with a dense feed-forward, upper
    case with a routed one.  ``scale_up``: sizes in the range of a real model's layers.  The
    ``decay_rank`` / ``gate_rank`` entries size the low-rank projections of random weights only (a
    checkpoint's tensors give them)."""
    if scale_up:
        H = heads or width // 128
        delta = {"conv": 4, "dim": 128, "heads": H, "kv_heads": H, "vdim": 128, "decay_rank": 64, "gate_rank": 64}
        gla = {"dim": 64, "heads": H, "tau": 16.0, "vdim": 128, "decay_rank": 32}
        par = {"left": {"dim": 128, "heads": H, "kv_heads": max(H // 4, 1), "mask": {"size": 1024}, "scale": 128 ** -0.5,
                        "vdim": 128},
               "right": {"blocks": max(width // 256, 1), "conv": 4, "width": width}}
        dense = {"ff": 3 * width, "kind": "dense"}
        moe = {"expert": {"ff": width // 2}, "kind": "moe", "router": {"experts": 32, "top": 4}}
    else:
        delta = {"conv": 4, "dim": 24, "heads": 4, "kv_heads": 2, "vdim": 20, "decay_rank": 12, "gate_rank": 10}
        gla = {"dim": 20, "heads": 3, "tau": 8.0, "vdim": 28, "decay_rank": 8}
        par = {"left": {"dim": 24, "heads": 4, "kv_heads": 2, "mask": {"size": 37}, "scale": 0.2, "vdim": 40},
               "right": {"blocks": 3, "conv": 3, "width": 96}}
        dense = {"ff": 224, "kind": "dense"}
        moe = {"expert": {"ff": 56}, "kind": "moe", "router": {"experts": 7, "top": 2}}
    kinds = {"d": ("channel_delta", delta), "g": ("gla", gla), "p": ("parallel", par)}
    layers = []
    for ch in pattern:
        t, m = kinds[ch.lower()]
        layers.append({"type": t, "mixer": {k: (dict(v) if isinstance(v, dict) else v) for k, v in m.items()},
                       "mlp": dict(moe if ch.isupper() else dense)})
    return {"architecture": "Sigudra", "embedding": {"bigram": {"buckets": 251, "mul_cur": 5, "mul_prev": 29}},
            "layers": layers, "norm": {"eps": 1e-5}, "vocab": vocab, "width": width}


class _Layer(Layer):
    def __init__(self, i: int, spec: Dict, width: int, eps: float):
        super().__init__(i, spec, width, eps, SigudraModel.mixer_types)
        mlp = spec.get("mlp")
        if mlp is None:
            self.ff = None
        elif mlp["kind"] == "dense":
            self.ff = DenseFF(mlp, width, act="gelu_tanh", gated=True)
        elif mlp["kind"] == "moe":
            self.ff = InputScaledRoutedFF(mlp, width, act="silu", score="sigmoid")
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
        self.w_ff = None
        self.norm2 = None

    def norms(self):
        return ("norm1", "norm2") if self.ff is not None else ("norm1",)


class SigudraModel(LayeredDecoder):
    arch = "sigudra"
    mixer_types = ("channel_delta", "gla", "parallel")
    slot_arrays = {"last_token": (torch.int32, ())}

    def __init__(self, cfg: ModelConfig, device="cuda", dtype=torch.bfloat16):
        super().__init__(cfg, device, dtype)
        pair = (cfg.embedding or {}).get("bigram")
        self.pair = (int(pair["buckets"]), int(pair["mul_prev"]), int(pair["mul_cur"])) if pair else None
        self.pair_table = None

    def make_layer(self, i: int, spec: Dict) -> Layer:
        return _Layer(i, spec, self.cfg.hidden_size, self.cfg.norm_eps)

    def extra_shapes(self) -> Dict[str, tuple]:
        return {"bigram": (self.pair[0] + 1, self.cfg.hidden_size)} if self.pair else {}

    def load_extra(self, get) -> None:
        if self.pair:
            self.pair_table = get("bigram").to(self.dtype).contiguous()

    def load_layer(self, l: Layer, get) -> None:
        dt = self.dtype
        l.norm1 = get(l.prefix + ".norm1").float().contiguous()
        l.w_in = l.mixer.load(lambda k, p=l.prefix: get(f"{p}.mix.{k}"), dt).contiguous()
        if l.ff is not None:
            l.norm2 = get(l.prefix + ".norm2").float().contiguous()
            w = l.ff.load(lambda k, p=l.prefix: get(f"{p}.mlp.{k}"), dt)
            l.w_ff = w.contiguous() if w is not None else None

    def weight_tensors(self):
        return super().weight_tensors() + ([self.pair_table] if self.pair_table is not None else [])

    # -- forward -----------------------------------------------------------------------------------
    def forward(self, ids: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, kv: HybridCache) -> torch.Tensor:
        """Final-normed hidden states [T, width] of every row of the step."""
        eps, dt = self.cfg.norm_eps, self.dtype
        if meta.seg_cu is None:
            raise ValueError("this model needs the segment view of the step (AttentionMetadata.seg_*)")
        if self.pair:
            x = mx.embed_pairs(ids, self.embed, self.pair_table, self.pair[1], self.pair[2], kv.model["last_token"],
                               meta.seg_cu, meta.seg_state, positions, meta.seg_max_len)
        else:
            x = mx.embed_f32(ids, self.embed)
        h = x if dt == torch.float32 else x.to(dt)
        for i, l in enumerate(self.layers):
            m = l.mixer.forward(F.linear(h, l.w_in), positions, meta, kv.layers[i])
            if isinstance(m, tuple):          # two mixers side by side: half the sum of their RMS norms
                h = mx.post_norm_add(x, m[0], l.norm1, eps, dt, b=m[1], wa=l.mixer.out_w[0], wb=l.mixer.out_w[1])
            else:
                h = mx.post_norm_add(x, m, l.norm1, eps, dt)
            if l.ff is not None:
                f = l.ff.forward(h, F.linear(h, l.w_ff) if l.w_ff is not None else None, x32=x)
                h = mx.post_norm_add(x, f, l.norm2, eps, dt)
            if self.capture is not None:
                self.capture.append(x.clone())
        return mx.layer_norm_out(x, self.final_norm, eps, dt)
