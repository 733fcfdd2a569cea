"""Building blocks of layered (hybrid) decoders: sequence mixers and feed-forwards that read one
normed input ``h`` and return a sublayer output, with their sizes and constants as parameters.

* :class:`Mamba2Mixer` -- state-space duality layer (causal short convolution + selective scan with
  an f32 state per sequence slot, gated grouped RMS norm, output projection).
* :class:`LatentAttentionMixer` -- attention whose keys and values are up-projections of one cached
  latent per token plus one shared rotated key part; runs in the latent space over a paged latent
  cache with a sliding window and a per-head sigmoid output gate.
* :class:`DenseFF` -- up, activation, down.
* :class:`RoutedFF` -- mixture of clamped gated experts with biased top-k choice, identity experts
  and an always-on shared expert.

Every block declares the rows it needs from a fused in-projection (``in_weight``): a layer stacks
its mixer's and its feed-forward's rows into ONE GEMM over ``h`` and hands each block its column
slice.  GEMMs are vendor matrix products (``F.linear`` / ``bmm``) on bf16 or f32 weights; everything
else runs on the kernels behind :mod:`..ops.mixers`.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import torch
import torch.nn.functional as F

from ..ops import mixers as mx
from .common import AttentionMetadata

Getter = Callable[[str], torch.Tensor]

# steps with at most this many (token, expert) pairs run every expert over every row (no host sync:
# hipGraph-capturable, and a decode step streams all expert weights anyway); larger steps bucket
# the rows by expert and read the bucket sizes on the host once per layer
DENSE_MAX_PAIRS = 512


def _capturing(t: torch.Tensor) -> bool:
    return t.is_cuda and torch.cuda.is_current_stream_capturing()


class Mamba2Mixer:
    kind = "mamba2"

    def __init__(self, spec: Dict, width: int, eps: float):
        self.H, self.P, self.N = int(spec["heads"]), int(spec["vdim"]), int(spec["state"])
        self.G, self.K = int(spec.get("groups", 1)), int(spec["conv"])
        self.norm_groups = int(spec.get("norm_groups", 1))
        self.inner = self.H * self.P
        self.C = self.inner + 2 * self.G * self.N          # convolved channels: x | B | C
        self.in_rows = 2 * self.inner + 2 * self.G * self.N + self.H   # z | x | B | C | dt
        self.width, self.eps = width, eps
        if self.H % self.G or self.inner % self.norm_groups:
            raise ValueError("mamba2: heads must split into groups and inner into norm_groups")
        if self.N > 256 or not 1 <= self.K <= 8:
            raise ValueError("mamba2: state <= 256 and 1 <= conv taps <= 8 are supported")

    def shapes(self) -> Dict[str, tuple]:
        return {"in": (self.in_rows, self.width), "conv": (self.C, self.K), "conv.b": (self.C,), "dt_bias": (self.H,),
                "A_log": (self.H,), "D": (self.H,), "norm": (self.inner,), "o": (self.width, self.inner)}

    def cache_spec(self):
        return ("state", self.K, self.C, self.H, self.P, self.N)

    def load(self, get: Getter, dtype) -> torch.Tensor:
        f32 = lambda n: get(n).float().contiguous()  # noqa: E731
        self.conv_w, self.conv_b = f32("conv"), f32("conv.b")
        self.dt_bias, self.A_log, self.D, self.norm_w = f32("dt_bias"), f32("A_log"), f32("D"), f32("norm")
        self.o = get("o").to(dtype).contiguous()
        return get("in").to(dtype)

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.conv_w, self.conv_b, self.norm_w, self.o))

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        _, conv_state, ssm_state = cache
        z = proj[:, :self.inner]
        xbc = proj[:, self.inner:self.inner + self.C]
        dt = proj[:, self.inner + self.C:self.inner + self.C + self.H]
        u = mx.conv_silu(xbc, self.conv_w, self.conv_b, conv_state, meta.seg_cu, meta.seg_state, positions,
                         meta.seg_max_len)
        y = mx.ssm_scan(u, dt, self.dt_bias, self.A_log, self.D, ssm_state, meta.seg_cu, meta.seg_state, positions,
                        self.H, self.P, self.N, self.G)
        # the gate comes before the norm: rms over silu(z) * y, in norm_groups equal parts
        yn = mx.group_norm(y, self.norm_w, self.eps, self.norm_groups, gate=z, out_dtype=proj.dtype)
        return F.linear(yn, self.o)


class LatentAttentionMixer:
    kind = "latent_attention"

    def __init__(self, spec: Dict, width: int, eps: float):
        self.H, self.dn, self.dr, self.dv = int(spec["heads"]), int(spec["dim"]), int(spec["rot_dim"]), int(spec["vdim"])
        self.R, self.q_rank = int(spec["kv_rank"]), int(spec["q_rank"])
        rot = spec.get("rot") or {}
        self.rot_dims = int(rot.get("dims", self.dr))
        self.rot_base = float(rot.get("base", 10000.0))
        mask = spec.get("mask") or {}
        self.window = int(mask["size"]) if mask.get("size") else 1 << 30      # no mask entry: plain causal
        self.scale = float(spec["scale"]) if "scale" in spec else (self.dn + self.dr) ** -0.5
        self.in_rows = self.q_rank + self.R + self.dr + self.H                # c_q | c, k_rot | gate
        self.width, self.eps = width, eps
        if self.rot_dims > self.dr or self.rot_dims % 2 or self.R > 512:
            raise ValueError("latent_attention: rot.dims must be even and <= rot_dim, kv_rank <= 512")

    def shapes(self) -> Dict[str, tuple]:
        H, dq = self.H, self.dn + self.dr
        return {"dq": (self.q_rank, self.width), "dq.norm": (self.q_rank,), "uq": (H * dq, self.q_rank),
                "dkv": (self.R + self.dr, self.width), "dkv.norm": (self.R,), "uk": (H * self.dn, self.R),
                "uv": (H * self.dv, self.R), "g": (H, self.width), "o": (self.width, H * self.dv)}

    def cache_spec(self):
        return ("latent", self.R + self.dr)

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.dq_norm = get("dq.norm").float().contiguous()
        self.dkv_norm = get("dkv.norm").float().contiguous()
        self.uq = get("uq").to(dtype).contiguous()
        self.uk = get("uk").to(dtype).view(self.H, self.dn, self.R).contiguous()      # [H, dn, R]
        self.uv_t = get("uv").to(dtype).view(self.H, self.dv, self.R).transpose(1, 2).contiguous()  # [H, R, dv]
        self.o = get("o").to(dtype).contiguous()
        self.inv_freq = mx.rope_inv_freq(self.rot_dims, self.rot_base, device=self.uq.device)
        return torch.cat([get("dq"), get("dkv"), get("g")], 0).to(dtype)

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.uq, self.uk, self.uv_t, self.o))

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        rows = cache[1]
        T = proj.shape[0]
        H, dn, dr, R = self.H, self.dn, self.dr, self.R
        a = self.q_rank
        cq = mx.group_norm(proj[:, :a], self.dq_norm, self.eps, 1)
        kv = proj[:, a:a + R + dr]
        gate = proj[:, a + R + dr:a + R + dr + H]
        q = F.linear(cq, self.uq)                                            # [T, H * (dn + dr)]
        # latent row + shared rotated key into the cache; every head's rotated query part
        q_rot = mx.latent_prep(kv, self.dkv_norm, self.eps, self.inv_freq, self.rot_dims, positions, meta.slots, rows,
                               q, H, dn + dr, dn, R, dr)
        # fold each head's key up-projection into its query: q_lat[h] = W_uk[h]^T q_nope[h]
        q_nope = q.view(T, H, dn + dr)[:, :, :dn]
        q_lat = torch.bmm(q_nope.transpose(0, 1), self.uk).transpose(0, 1).contiguous()   # [T, H, R]
        o_lat = mx.latent_attend(q_lat, q_rot, rows, meta.seg_cu, positions, meta.seg_bt, self.window, self.scale,
                                 meta.seg_max_len, gate=gate)
        o = torch.bmm(o_lat.transpose(0, 1), self.uv_t).transpose(0, 1).reshape(T, H * self.dv)
        return F.linear(o, self.o)


class DenseFF:
    """W_down act(W_up h); ``act``: "relu2" (the square of relu)."""

    def __init__(self, spec: Dict, width: int, act: str = "relu2"):
        self.ff, self.width, self.act = int(spec["ff"]), width, act
        self.in_rows = self.ff
        if act != "relu2":
            raise ValueError(f"unknown activation {act!r}")

    def shapes(self) -> Dict[str, tuple]:
        return {"up": (self.ff, self.width), "down": (self.width, self.ff)}

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.down = get("down").to(dtype).contiguous()
        return get("up").to(dtype)

    def num_bytes(self) -> int:
        return self.down.numel() * self.down.element_size()

    def forward(self, h: torch.Tensor, proj: torch.Tensor) -> torch.Tensor:
        return F.linear(mx.relu2(proj), self.down)


class RoutedFF:
    """Mixture of ``experts`` clamped gated feed-forwards, ``top`` per token.

    Router logits z = W_r h in f32; scores s = softmax(z) over the experts and the ``identity``
    experts that follow them; the ``top`` largest s + correction are chosen and weighted by s itself.
    An identity expert returns its input.  Expert: g = min(W_g h, limit), u = clamp(W_u h, +-limit),
    W_d (g * sigmoid(alpha g) * (u + 1)).  A shared expert of the same form runs for every token."""

    def __init__(self, spec: Dict, width: int, alpha: float = 1.702):
        r = spec["router"]
        self.E, self.I, self.top = int(r["experts"]), int(r.get("identity", 0)), int(r["top"])
        self.F = int(spec["expert"]["ff"])
        self.limit = float(spec["expert"]["limit"])
        sh = spec.get("shared")
        self.Fs = int(sh["ff"]) if sh else 0
        self.limit_s = float(sh["limit"]) if sh else 0.0
        self.alpha, self.width = alpha, width
        self.in_rows = 2 * self.Fs                                            # shared gate | up

    def shapes(self) -> Dict[str, tuple]:
        s = {"router": (self.E + self.I, self.width), "correction": (self.E + self.I,)}
        for e in range(self.E):
            s.update({f"e{e}.gate": (self.F, self.width), f"e{e}.up": (self.F, self.width),
                      f"e{e}.down": (self.width, self.F)})
        if self.Fs:
            s.update({"shared.gate": (self.Fs, self.width), "shared.up": (self.Fs, self.width),
                      "shared.down": (self.width, self.Fs)})
        return s

    def load(self, get: Getter, dtype) -> Optional[torch.Tensor]:
        self.router = get("router").float().contiguous()
        self.correction = get("correction").float().contiguous()
        self.w13 = torch.stack([torch.cat([get(f"e{e}.gate"), get(f"e{e}.up")], 0) for e in range(self.E)]).to(dtype)
        self.w2 = torch.stack([get(f"e{e}.down") for e in range(self.E)]).to(dtype).contiguous()
        if not self.Fs:
            return None
        self.down_s = get("shared.down").to(dtype).contiguous()
        return torch.cat([get("shared.gate"), get("shared.up")], 0).to(dtype)

    def num_bytes(self) -> int:
        ts = [self.router, self.w13, self.w2] + ([self.down_s] if self.Fs else [])
        return sum(t.numel() * t.element_size() for t in ts)

    def forward(self, h: torch.Tensor, proj: Optional[torch.Tensor]) -> torch.Tensor:
        T, W = h.shape
        E, top, Fe = self.E, self.top, self.F
        shared = None
        if self.Fs:
            shared = F.linear(mx.glu_clamp(proj[:, :self.Fs], proj[:, self.Fs:2 * self.Fs], self.limit_s, self.alpha),
                              self.down_s)
        wts, idx = mx.route_biased(F.linear(h.float(), self.router), self.correction, top)
        if T * top <= DENSE_MAX_PAIRS or _capturing(h):
            gu = torch.bmm(h.unsqueeze(0).expand(E, T, W), self.w13.transpose(1, 2)).view(E * T, 2 * Fe)
            act = mx.glu_clamp(gu[:, :Fe], gu[:, Fe:], self.limit, self.alpha)
            ys = torch.bmm(act.view(E, T, Fe), self.w2.transpose(1, 2)).view(E * T, W)
            rows = torch.arange(T, dtype=torch.int32, device=h.device)[:, None]
            pos = (idx.clamp(max=E - 1) * T + rows).to(torch.int32)
            return mx.moe_combine(ys, pos, idx, wts, h, shared, E)
        flat = idx.reshape(-1).long()
        order = torch.argsort(flat, stable=True)
        offs = [0] + torch.bincount(flat, minlength=E + self.I).cumsum(0).tolist()     # host read of the buckets
        xs = h.index_select(0, order // top)
        ys = torch.empty((T * top, W), dtype=h.dtype, device=h.device)
        for e in range(E):
            a, b = offs[e], offs[e + 1]
            if b > a:
                gu = F.linear(xs[a:b], self.w13[e])
                torch.mm(mx.glu_clamp(gu[:, :Fe], gu[:, Fe:], self.limit, self.alpha), self.w2[e].t(), out=ys[a:b])
        pos = torch.empty_like(order)
        pos[order] = torch.arange(order.numel(), device=order.device)
        return mx.moe_combine(ys, pos.view(T, top).to(torch.int32), idx, wts, h, shared, E)


MIXERS = {"mamba2": Mamba2Mixer, "latent_attention": LatentAttentionMixer}
