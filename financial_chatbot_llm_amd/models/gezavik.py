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
from .common import AttentionMetadata, HybridCache, param_seed
from .configs import ModelConfig
from .mixers import MIXERS, DenseFF, RoutedFF


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


class _Layer:
    def __init__(self, i: int, spec: Dict, width: int, eps: float):
        self.prefix = f"l{i}"
        if spec["type"] not in MIXERS:
            raise ValueError(f"layer {i}: unknown mixer type {spec['type']!r}; known: {sorted(MIXERS)}")
        self.mixer = MIXERS[spec["type"]](spec["mixer"], width, eps)
        mlp = spec.get("mlp")
        if mlp is None:
            self.ff = None
        elif mlp["kind"] == "dense":
            self.ff = DenseFF(mlp, width, act="relu2")
        elif mlp["kind"] == "moe":
            self.ff = RoutedFF(mlp, width, alpha=1.702)
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
        self.w_in: Optional[torch.Tensor] = None
        self.norm1: Optional[torch.Tensor] = None


class GezavikModel:
    segment_meta = True          # the runner builds the segment view of each step (AttentionMetadata.seg_*)
    has_state = True             # sequences hold a recurrent-state slot; no prefix reuse, no draft rows
    tp_size = 1
    tp_rank = 0

    def __init__(self, cfg: ModelConfig, device="cuda", dtype=torch.bfloat16):
        if cfg.arch != "gezavik" or not cfg.layers:
            raise ValueError(f"{cfg.name} is not a Gezavik config")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        self.layers: List[_Layer] = [_Layer(i, spec, cfg.hidden_size, cfg.norm_eps) for i, spec in enumerate(cfg.layers)]
        self.has_state = any(l.mixer.kind == "mamba2" for l in self.layers)
        self.mult = float(cfg.residual_mult)
        self.sequence_parallel = False
        self.capture: Optional[list] = None      # debugging: residual stream after every layer
        # head geometry the generic runner asks every decoder for (unused by the segment kernels)
        self.hq = self.hkv = 1
        self.D = 64

    # -- weights -----------------------------------------------------------------------------------
    def full_shapes(self) -> Dict[str, tuple]:
        c = self.cfg
        s = {"embed": (c.vocab_size, c.hidden_size), "final.norm": (c.hidden_size,), "head": (c.vocab_size, c.hidden_size)}
        for l in self.layers:
            s[l.prefix + ".norm1"] = (c.hidden_size,)
            s.update({f"{l.prefix}.mix.{k}": v for k, v in l.mixer.shapes().items()})
            if l.ff is not None:
                s.update({f"{l.prefix}.mlp.{k}": v for k, v in l.ff.shapes().items()})
        return s

    @staticmethod
    def _random(name: str, shape, seed: int, device="cpu") -> torch.Tensor:
        g = torch.Generator(device=device).manual_seed(param_seed(seed, name))
        randn = lambda: torch.randn(shape, generator=g, device=device)  # noqa: E731
        rand = lambda: torch.rand(shape, generator=g, device=device)  # noqa: E731
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("norm1", "norm") and len(shape) == 1:
            return 1.0 + 0.1 * randn()
        if leaf == "A_log":
            return torch.log(1.0 + 7.0 * rand())
        if leaf == "dt_bias":      # softplus^-1 of step sizes in [0.01, 0.2]
            dt = torch.exp(rand() * (math.log(0.2) - math.log(0.01)) + math.log(0.01))
            return dt + torch.log(-torch.expm1(-dt))
        if leaf == "D":
            return 1.0 + 0.2 * randn()
        if leaf == "correction":
            return 0.05 * randn()
        if leaf == "b":
            return 0.1 * randn()
        if leaf == "conv":
            return randn() * shape[1] ** -0.5
        if leaf == "embed":
            return randn()
        return randn() * shape[-1] ** -0.5

    def init_random(self, seed: int = 0, std: float = 0.02) -> "GezavikModel":
        """Deterministic per-name weights, rounded to bf16 as a checkpoint would hold them."""
        sd = {n: self._random(n, s, seed, self.device).to(torch.bfloat16) for n, s in self.full_shapes().items()}
        return self.load_state(sd)

    def load_state(self, sd: Dict[str, torch.Tensor]) -> "GezavikModel":
        missing = set(self.full_shapes()) - set(sd)
        if missing:
            raise KeyError(f"missing weights: {sorted(missing)[:5]}...")
        for n, shape in self.full_shapes().items():
            if tuple(sd[n].shape) != tuple(shape):
                raise ValueError(f"{n}: checkpoint shape {tuple(sd[n].shape)} != config shape {tuple(shape)}")
        dev, dt = self.device, self.dtype
        get = lambda n: sd[n].to(dev)  # noqa: E731
        self.embed = get("embed").to(dt).contiguous()
        self.head = get("head").to(dt).contiguous()
        self.final_norm = get("final.norm").float().contiguous()
        for l in self.layers:
            l.norm1 = get(l.prefix + ".norm1").float().contiguous()
            parts = [l.mixer.load(lambda k, p=l.prefix: get(f"{p}.mix.{k}"), dt)]
            if l.ff is not None:
                w = l.ff.load(lambda k, p=l.prefix: get(f"{p}.mlp.{k}"), dt)
                if w is not None:
                    parts.append(w)
            l.w_in = torch.cat(parts, 0).contiguous()         # ONE in-projection per block
        return self

    def num_bytes(self) -> int:
        b = sum(t.numel() * t.element_size() for t in (self.embed, self.head))
        for l in self.layers:
            b += l.w_in.numel() * l.w_in.element_size() + l.mixer.num_bytes() + (l.ff.num_bytes() if l.ff else 0)
        return b

    # -- cache -------------------------------------------------------------------------------------
    def cache_specs(self):
        return [l.mixer.cache_spec() for l in self.layers]

    def kv_bytes_per_block(self) -> int:
        return HybridCache.bytes_per_block(self.cache_specs(), 4 if self.dtype == torch.float32 else 2)

    def make_cache(self, num_blocks: int, num_slots: int) -> HybridCache:
        return HybridCache(self.cache_specs(), num_blocks, num_slots, self.dtype, self.device)

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

    def lm_weight(self) -> torch.Tensor:
        return self.head

    def logits(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(h, self.head)
