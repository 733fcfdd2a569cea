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
    """Per-layer memory of a layered decoder: a paged latent cache for every attention layer and a
    state slot array for every recurrent layer, behind the engine's one page table and one slot id
    per sequence.

    ``layers[i]`` is ``("latent", rows)`` with rows [num_blocks * 64, row_width] in the activation
    dtype, or ``("state", conv, ssm)`` with f32 conv [slots, taps - 1, channels] and f32 ssm
    [slots, heads, vdim, state].  Pages and slots are handed on uncleared: a latent row is written
    before any query may see it, and a sequence's first segment starts from zero state."""

    def __init__(self, specs, num_blocks: int, num_slots: int, dtype, device):
        self.num_blocks, self.num_slots = num_blocks, num_slots
        self.layers = []
        for sp in specs:
            if sp[0] == "latent":
                self.layers.append(("latent", torch.zeros((num_blocks * KV_BS, sp[1]), dtype=dtype, device=device)))
            elif sp[0] == "state":
                _, taps, channels, heads, vdim, nstate = sp
                self.layers.append(("state",
                                    torch.zeros((num_slots, max(taps - 1, 1), channels), dtype=torch.float32, device=device),
                                    torch.zeros((num_slots, heads, vdim, nstate), dtype=torch.float32, device=device)))
            else:
                self.layers.append((sp[0],))

    @staticmethod
    def bytes_per_block(specs, elt: int) -> int:
        return max(1, sum(KV_BS * sp[1] * elt for sp in specs if sp[0] == "latent"))

    @staticmethod
    def bytes_per_slot(specs) -> int:
        return sum(4 * (max(sp[1] - 1, 1) * sp[2] + sp[3] * sp[4] * sp[5]) for sp in specs if sp[0] == "state")


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
