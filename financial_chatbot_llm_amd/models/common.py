"""Shared model plumbing: attention metadata, paged KV cache, deterministic weight init."""
from __future__ import annotations

import zlib
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

from ..ops.attention import KV_BS, DecodeWorkspace


@dataclass
class AttentionMetadata:
    """Per-step batch layout: ``num_prefill_tokens`` prefill tokens first, then one token per
    decoding sequence.  All tensors live on the model's device."""

    slots: torch.Tensor                      # [T] int32 KV slot per token (-1: no write)
    num_prefill_tokens: int = 0
    cu_q: Optional[torch.Tensor] = None      # [Sp+1] int32
    ctx_lens_p: Optional[torch.Tensor] = None  # [Sp] int32 total KV length after this step
    block_tables_p: Optional[torch.Tensor] = None  # [Sp, max_blocks] int32
    max_q_len: int = 0
    num_decode: int = 0
    ctx_lens_d: Optional[torch.Tensor] = None  # [Bd]
    block_tables_d: Optional[torch.Tensor] = None
    decode_ws: Optional[DecodeWorkspace] = None
    causal: bool = True
    prefill_work: Optional[torch.Tensor] = None  # [n, 2] int32 (ops.attention.prefill_work_list) or lean [., 6]
    prefill_lean: Optional[tuple] = None          # lean list counts (items, merges, slots), host ints
    # segment view of the same step for the sequence mixers (ops.mixers): every prefill chunk and every
    # decode row is one segment, in batch order
    seg_cu: Optional[torch.Tensor] = None         # [S+1] int32 row bounds
    seg_bt: Optional[torch.Tensor] = None         # [S, W] int32 page tables
    seg_state: Optional[torch.Tensor] = None      # [S] int32 recurrent-state slot (< 0: padding row)
    seg_max_len: int = 0                          # longest segment (host int)


class KVCache:
    """All layers' paged K/V in ONE HBM allocation: [L, 2, num_blocks, Hkv, 64*D] bf16.

    ``k(l)`` / ``v(l)`` are [num_blocks, Hkv, 64*D] tiles in MFMA-fragment-native order
    (csrc/kernels/kv_layout.h).
    """

    def __init__(self, num_layers: int, num_blocks: int, num_kv_heads: int, head_dim: int,
                 dtype=torch.bfloat16, device="cuda"):
        self.num_layers, self.num_blocks = num_layers, num_blocks
        self.num_kv_heads, self.head_dim = num_kv_heads, head_dim
        self.buf = torch.zeros((num_layers, 2, num_blocks, num_kv_heads, KV_BS * head_dim), dtype=dtype,
                               device=device)

    def k(self, layer: int) -> torch.Tensor:
        return self.buf[layer, 0]

    def v(self, layer: int) -> torch.Tensor:
        return self.buf[layer, 1]

    @staticmethod
    def bytes_per_block(num_layers: int, num_kv_heads: int, head_dim: int, elt: int = 2) -> int:
        return num_layers * 2 * num_kv_heads * KV_BS * head_dim * elt


class HybridCache:
    """Per-layer memory of a layered decoder: paged row caches for attention layers and state slot
    arrays for recurrent layers, behind the engine's one page table and one slot id per sequence.

    A layer's spec -> its entry in ``layers``:

    * ``("latent", w)`` / ``("rows", w)`` -> ``(kind, rows)``, rows [num_blocks * 64, w] in the
      activation dtype (one cache row per token: a key/value latent, or [keys | values]);
    * ``("state", taps, channels, heads, vdim, state)`` -> ``("state", conv, ssm)``, f32 conv
      [slots, taps - 1, channels] and ssm [slots, heads, vdim, state];
    * ``("slots", {name: shape})`` -> ``("slots", {name: f32 [slots, *shape]})``;
    * ``("pair", spec_a, spec_b)`` -> ``("pair", entry_a, entry_b)`` (two mixers side by side).

    ``slot_arrays`` ({name: (dtype, shape)}) are per-slot records of the model as a whole
    (``model[name]``: [slots, *shape]), e.g. the last token of each sequence.  Pages and slots are
    handed on uncleared: a cache row is written before any query may see it, and a sequence's
    first segment starts from zero state."""

    def __init__(self, specs, num_blocks: int, num_slots: int, dtype, device, slot_arrays=None):
        self.num_blocks, self.num_slots = num_blocks, num_slots
        self.dtype, self.device = dtype, device
        self.layers = [self._make(sp) for sp in specs]
        self.model = {n: torch.zeros((num_slots, *shape), dtype=dt, device=device)
                      for n, (dt, shape) in (slot_arrays or {}).items()}

    def _make(self, sp):
        nb, ns, dev = self.num_blocks, self.num_slots, self.device
        if sp[0] in ("latent", "rows"):
            return (sp[0], torch.zeros((nb * KV_BS, sp[1]), dtype=self.dtype, device=dev))
        if sp[0] == "state":
            _, taps, channels, heads, vdim, nstate = sp
            return ("state", torch.zeros((ns, max(taps - 1, 1), channels), dtype=torch.float32, device=dev),
                    torch.zeros((ns, heads, vdim, nstate), dtype=torch.float32, device=dev))
        if sp[0] == "slots":
            return ("slots", {n: torch.zeros((ns, *shape), dtype=torch.float32, device=dev) for n, shape in sp[1].items()})
        if sp[0] == "pair":
            return ("pair", self._make(sp[1]), self._make(sp[2]))
        return (sp[0],)

    @staticmethod
    def _flat(specs):
        for sp in specs:
            if sp[0] == "pair":
                yield from HybridCache._flat(sp[1:])
            else:
                yield sp

    @staticmethod
    def bytes_per_block(specs, elt: int) -> int:
        return max(1, sum(KV_BS * sp[1] * elt for sp in HybridCache._flat(specs) if sp[0] in ("latent", "rows")))

    @staticmethod
    def bytes_per_slot(specs) -> int:
        n = 0
        for sp in HybridCache._flat(specs):
            if sp[0] == "state":
                n += 4 * (max(sp[1] - 1, 1) * sp[2] + sp[3] * sp[4] * sp[5])
            elif sp[0] == "slots":
                for shape in sp[1].values():
                    k = 4
                    for d in shape:
                        k *= d
                    n += k
        return n


def param_seed(base: int, name: str) -> int:
    return (base * 1_000_003 + zlib.crc32(name.encode())) & 0x7FFFFFFF


def random_tensor(name: str, shape, seed: int, device, dtype=torch.bfloat16, std: float = 0.02,
                  kind: str = "normal") -> torch.Tensor:
    """Deterministic per-name init, identical on every rank (so TP shards agree)."""
    if kind == "ones":
        return torch.ones(shape, dtype=dtype, device=device)
    if kind == "zeros":
        return torch.zeros(shape, dtype=dtype, device=device)
    g = torch.Generator(device=device)
    g.manual_seed(param_seed(seed, name))
    t = torch.randn(shape, generator=g, device=device, dtype=torch.float32 if device == "cpu" else dtype)
    return t.mul_(std).to(dtype)
