"""Sequence-mixer ops of the hybrid decoders (``csrc/mixers``): a 32-bit residual stream with a fused
parallel-block update + RMS norm, grouped / gated RMS norms, the Mamba-2 causal convolution and
state-space scan over a flat batch of segments, latent attention over a paged latent cache with a
sliding window, clamped gated units, and biased top-k routing.

Activations are bf16 or f32 (a model-wide choice); statistics, scores, softmax, recurrences and the
residual stream are f32 either way.  CUDA(HIP) tensors run the kernels of ``libpenny_mixers.so``
and fail loudly without it; CPU tensors run the fp32 PyTorch forms below (CI).

Batch layout: a step's rows are ``S`` segments, segment ``s`` owning rows ``cu[s]:cu[s+1]`` (a
prompt chunk, or a single decoded token), ``pos`` the position of every row, ``slot[s]`` the
segment's recurrent-state slot (< 0: padding, skipped) and ``bt[s]`` its cache page table.  A
segment whose first row is at position 0 starts from zero state whatever its slot holds.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from . import _native as N

PAGE = 64


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return 1
    if t.dtype == torch.bfloat16:
        return 0
    raise TypeError(f"mixer ops take bf16 or f32 tensors, got {t.dtype}")


def _rows(t: torch.Tensor) -> torch.Tensor:
    """A 2-D view whose last dimension is contiguous (column slices of a projection pass as is)."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError("expected a [rows, n] tensor with unit column stride")
    return t


# ----------------------------------------------------------------------------------------------
# residual stream
# ----------------------------------------------------------------------------------------------
def embed_f32(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """Token rows of ``table`` (bf16 or f32) as an f32 residual stream [T, W]."""
    T, (V, W) = ids.numel(), table.shape
    if N.use_native(table):
        out = torch.empty((T, W), dtype=torch.float32, device=table.device)
        N.mcall("mx_embed", N.ptr(ids.to(torch.int32).contiguous()), N.ptr(table), _dt(table), N.ptr(out), T, W, V,
                N.stream())
        return out
    return table[ids.long().clamp(0, V - 1)].float()


def residual_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float, a: Optional[torch.Tensor] = None,
                  b: Optional[torch.Tensor] = None, mult: float = 1.0,
                  out_dtype: torch.dtype = torch.bfloat16) -> Optional[torch.Tensor]:
    """``x`` (f32 [T, W], in place) <- x + mult * (a + b) when a sublayer output is given, then
    y = x / sqrt(mean(x^2) + eps) * w in ``out_dtype`` (``w`` None: the update only)."""
    T, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    ab = a if a is not None else b
    if N.use_native(x):
        out = torch.empty((T, W), dtype=out_dtype, device=x.device) if w is not None else None
        if a is not None and b is not None:
            assert a.dtype == b.dtype
        N.mcall("mx_residual_norm", N.ptr(x), N.ptr(_rows(a)) if a is not None else None,
                a.stride(0) if a is not None else 0, N.ptr(_rows(b)) if b is not None else None,
                b.stride(0) if b is not None else 0, _dt(ab) if ab is not None else 1, float(mult),
                N.ptr(w), float(eps), N.ptr(out), _dt(out) if out is not None else 1, T, W, N.stream())
        return out
    if ab is not None:
        s = torch.zeros_like(x)
        for t in (a, b):
            if t is not None:
                s = s + t.float()
        x.add_(mult * s)
    if w is None:
        return None
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def group_norm(inp: torch.Tensor, w: torch.Tensor, eps: float, groups: int = 1, gate: Optional[torch.Tensor] = None,
               out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """RMS norm of each of ``groups`` equal parts of every row of ``inp`` [T, n] (each part by its own
    root mean square), times ``w`` [n].  ``gate``: the row is multiplied by silu(gate) first."""
    T, n = inp.shape
    out_dtype = out_dtype or inp.dtype
    if n % groups:
        raise ValueError(f"{n} columns do not split into {groups} groups")
    if N.use_native(inp):
        out = torch.empty((T, n), dtype=out_dtype, device=inp.device)
        N.mcall("mx_group_norm", N.ptr(_rows(inp)), inp.stride(0), _dt(inp), N.ptr(_rows(gate)) if gate is not None else None,
                gate.stride(0) if gate is not None else 0, _dt(gate) if gate is not None else 1, N.ptr(w),
                float(eps), N.ptr(out), out.stride(0), _dt(out), T, groups, n // groups, N.stream())
        return out
    v = inp.float()
    if gate is not None:
        v = v * F.silu(gate.float())
    v = v.view(T, groups, n // groups)
    v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    return (v.reshape(T, n) * w.float()).to(out_dtype)


# ----------------------------------------------------------------------------------------------
# activations
# ----------------------------------------------------------------------------------------------
def relu2(x: torch.Tensor) -> torch.Tensor:
    """relu(x)^2, rows may be a column slice of a wider projection."""
    T, n = x.shape
    if N.use_native(x):
        out = torch.empty((T, n), dtype=x.dtype, device=x.device)
        N.mcall("mx_relu2", N.ptr(_rows(x)), x.stride(0), N.ptr(out), out.stride(0), _dt(x), T, n, N.stream())
        return out
    return torch.relu(x.float()).square().to(x.dtype)


def glu_clamp(gate: torch.Tensor, up: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
    """g = min(gate, limit), u = clamp(up, -limit, limit): g * sigmoid(alpha * g) * (u + 1)."""
    T, n = gate.shape
    if N.use_native(gate):
        out = torch.empty((T, n), dtype=gate.dtype, device=gate.device)
        N.mcall("mx_glu_clamp", N.ptr(_rows(gate)), gate.stride(0), N.ptr(_rows(up)), up.stride(0), float(limit),
                float(alpha), N.ptr(out), out.stride(0), _dt(gate), T, n, N.stream())
        return out
    g = gate.float().clamp(max=limit)
    u = up.float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1)).to(gate.dtype)


# ----------------------------------------------------------------------------------------------
# routing
# ----------------------------------------------------------------------------------------------
def route_biased(z: torch.Tensor, bias: Optional[torch.Tensor], top: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Scores s = softmax(z) over all entries (f32); the ``top`` entries with the largest s + bias are
    chosen, and their weights are the unbiased scores s (not renormalised).  Returns (weights f32
    [T, top], indices int32 [T, top])."""
    T, E = z.shape
    assert z.dtype == torch.float32
    if N.use_native(z):
        z = z.contiguous()
        w = torch.empty((T, top), dtype=torch.float32, device=z.device)
        i = torch.empty((T, top), dtype=torch.int32, device=z.device)
        N.mcall("mx_route_biased", N.ptr(z), N.ptr(bias), E, top, N.ptr(w), N.ptr(i), T, N.stream())
        return w, i
    s = torch.softmax(z, -1)
    c = s + bias.float() if bias is not None else s
    idx = torch.topk(c, top, dim=-1).indices
    return s.gather(1, idx), idx.to(torch.int32)


def moe_combine(ys: Optional[torch.Tensor], pos: torch.Tensor, idx: torch.Tensor, wts: torch.Tensor, h: torch.Tensor,
                shared: Optional[torch.Tensor], num_experts: int) -> torch.Tensor:
    """out[t] = sum_k wts[t, k] * src(t, k) (+ shared[t]): src is the token's own input ``h[t]`` for an
    identity expert (idx >= num_experts), else row ``pos[t, k]`` of the expert outputs ``ys``."""
    T, W = h.shape
    top = idx.shape[1]
    if N.use_native(h):
        out = torch.empty((T, W), dtype=h.dtype, device=h.device)
        N.mcall("mx_moe_combine", N.ptr(ys), N.ptr(pos.contiguous()), N.ptr(idx.contiguous()), N.ptr(wts.contiguous()),
                N.ptr(_rows(h)), h.stride(0), N.ptr(_rows(shared)) if shared is not None else None,
                shared.stride(0) if shared is not None else 0, num_experts, top, W, N.ptr(out), _dt(h), T, N.stream())
        return out
    acc = shared.float().clone() if shared is not None else torch.zeros((T, W), dtype=torch.float32)
    for k in range(top):
        e = idx[:, k].long()
        ident = e >= num_experts
        src = h.float().clone()
        if ys is not None and (~ident).any():
            rows = pos[:, k].long().clamp(0, ys.shape[0] - 1)
            src = torch.where(ident[:, None], src, ys.float()[rows])
        acc += wts[:, k:k + 1] * src
    return acc.to(h.dtype)


# ----------------------------------------------------------------------------------------------
# state-space mixer
# ----------------------------------------------------------------------------------------------
def conv_silu(inp: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
              cu: torch.Tensor, slot: torch.Tensor, pos: torch.Tensor, max_len: int) -> torch.Tensor:
    """Causal per-channel convolution + SiLU over every segment.  ``inp`` [T, C] (a column slice of the
    in-projection), ``w`` f32 [C, K] (last column: the current token's tap), ``state`` f32
    [slots, K-1, C]: the last K-1 inputs of each slot's sequence, read (unless the segment starts
    at position 0) and then replaced.  Returns f32 [T, C]."""
    T, C = inp.shape
    K = w.shape[1]
    S = cu.numel() - 1
    if N.use_native(inp):
        out = torch.empty((T, C), dtype=torch.float32, device=inp.device)
        N.mcall("mx_conv_silu", N.ptr(_rows(inp)), inp.stride(0), _dt(inp), N.ptr(w), N.ptr(bias), N.ptr(state),
                N.ptr(cu), N.ptr(slot), N.ptr(pos), N.ptr(out), S, int(max_len), C, K, N.stream())
        return out
    out = torch.zeros((T, C), dtype=torch.float32)
    cul, sll, pl = cu.tolist(), slot.tolist(), pos.tolist()
    x = inp.float()
    for s in range(S):
        a, b = cul[s], cul[s + 1]
        if sll[s] < 0 or b <= a:
            continue
        hist = torch.zeros((K - 1, C)) if pl[a] == 0 else state[sll[s]].clone()
        full = torch.cat([hist, x[a:b]])
        win = full.unfold(0, K, 1)                      # [n, C, K]
        acc = (win * w.float()[None]).sum(-1)
        if bias is not None:
            acc = acc + bias.float()
        out[a:b] = F.silu(acc)
        if K > 1:
            state[sll[s]] = full[-(K - 1):]
    return out


def ssm_scan(u: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, A_log: torch.Tensor, D: torch.Tensor,
             state: torch.Tensor, cu: torch.Tensor, slot: torch.Tensor, pos: torch.Tensor, heads: int, vdim: int,
             nstate: int, groups: int) -> torch.Tensor:
    """Mamba-2 recurrence, token by token, f32.  ``u`` f32 [T, H*P + 2*G*N] = [x | B | C] (after the
    convolution), ``dt_raw`` [T, H]; per head h of group h // (H / G):
    dt = softplus(dt_raw + dt_bias), S <- exp(-exp(A_log) dt) S + dt x B^T, y = S C + D x.
    ``state`` f32 [slots, H, P, N] is read (unless the segment starts at position 0) and replaced."""
    T, C = u.shape
    H, P, Ns, G = heads, vdim, nstate, groups
    S = cu.numel() - 1
    assert u.dtype == torch.float32 and u.is_contiguous() and C == H * P + 2 * G * Ns
    if N.use_native(u):
        y = torch.empty((T, H * P), dtype=torch.float32, device=u.device)
        N.mcall("mx_ssm_scan", N.ptr(u), C, N.ptr(_rows(dt_raw)), dt_raw.stride(0), _dt(dt_raw), N.ptr(dt_bias),
                N.ptr(A_log), N.ptr(D), N.ptr(state), N.ptr(cu), N.ptr(slot), N.ptr(pos), N.ptr(y), S, H, P, Ns, G, T,
                N.stream())
        return y
    y = torch.zeros((T, H * P), dtype=torch.float32)
    cul, sll, pl = cu.tolist(), slot.tolist(), pos.tolist()
    A = -torch.exp(A_log.float())
    rep = H // G
    for s in range(S):
        a, b = cul[s], cul[s + 1]
        if sll[s] < 0 or b <= a:
            continue
        St = torch.zeros((H, P, Ns)) if pl[a] == 0 else state[sll[s]].clone()
        dt = F.softplus(dt_raw[a:b].float() + dt_bias.float())          # [n, H]
        dec = torch.exp(A * dt)
        x = u[a:b, :H * P].view(-1, H, P)
        Bm = u[a:b, H * P:H * P + G * Ns].view(-1, G, Ns).repeat_interleave(rep, 1)
        Cm = u[a:b, H * P + G * Ns:].view(-1, G, Ns).repeat_interleave(rep, 1)
        for t in range(b - a):
            St = dec[t, :, None, None] * St + (dt[t, :, None] * x[t])[:, :, None] * Bm[t][:, None, :]
            y[a + t] = ((St * Cm[t][:, None, :]).sum(-1) + D.float()[:, None] * x[t]).reshape(-1)
        state[sll[s]] = St
    return y


# ----------------------------------------------------------------------------------------------
# latent attention
# ----------------------------------------------------------------------------------------------
def rope_inv_freq(dims: int, base: float, device=None) -> torch.Tensor:
    """f_i = base^(-2i / dims), i < dims / 2, f32."""
    i = torch.arange(0, dims, 2, dtype=torch.float32, device=device)
    return (1.0 / (base ** (i / dims))).contiguous()


def _rotate(v: torch.Tensor, ang: torch.Tensor, dims: int) -> torch.Tensor:
    """Interleaved-pair rotation of the first ``dims`` entries of the last axis; ``ang`` broadcasts
    against v[..., 0:dims:2]."""
    out = v.clone()
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    c, s = torch.cos(ang), torch.sin(ang)
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def latent_prep(kv: torch.Tensor, norm_w: torch.Tensor, eps: float, inv_freq: torch.Tensor, rot_dims: int,
                pos: torch.Tensor, slots: torch.Tensor, cache: torch.Tensor, q: torch.Tensor, heads: int,
                head_stride: int, rot_off: int, rank: int, rot_dim: int) -> torch.Tensor:
    """Per token: c = RMSnorm(kv[:rank]) * norm_w and the rotated shared key part rope(kv[rank:]) go to
    cache row ``slots[t]`` (< 0: no write; ``cache`` [rows, rank + rot_dim]); every head's rotated
    query part ``q[t, h*head_stride + rot_off : +rot_dim]`` is rotated into the returned
    [T, heads, rot_dim].  Angles are pos * inv_freq in f32, pairs interleaved."""
    T = kv.shape[0]
    R, Dr, H = rank, rot_dim, heads
    if N.use_native(kv):
        assert kv.dtype == cache.dtype == q.dtype
        q_rot = torch.empty((T, H, Dr), dtype=q.dtype, device=q.device)
        N.mcall("mx_latent_prep", N.ptr(_rows(kv)), kv.stride(0), N.ptr(norm_w), float(eps), N.ptr(inv_freq),
                int(rot_dims), N.ptr(pos), N.ptr(slots), N.ptr(cache), N.ptr(_rows(q)), q.stride(0), head_stride,
                rot_off, N.ptr(q_rot), _dt(kv), T, H, R, Dr, N.stream())
        return q_rot
    kvf = kv.float()
    c = kvf[:, :R]
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
    ang = pos.float()[:, None] * inv_freq.float()[None, :rot_dims // 2]
    kr = _rotate(kvf[:, R:R + Dr], ang, rot_dims)
    rows = torch.cat([c, kr], 1).to(cache.dtype)
    ok = slots >= 0
    cache.view(-1, R + Dr)[slots[ok].long()] = rows[ok]
    qr = torch.stack([q[:, h * head_stride + rot_off:h * head_stride + rot_off + Dr] for h in range(H)], 1).float()
    return _rotate(qr, ang[:, None, :], rot_dims).to(q.dtype)


def latent_attend(q_lat: torch.Tensor, q_rot: torch.Tensor, cache: torch.Tensor, cu: torch.Tensor, pos: torch.Tensor,
                  bt: torch.Tensor, window: int, scale: float, max_len: int,
                  gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Windowed causal attention in the latent space.  ``q_lat`` [T, H, R], ``q_rot`` [T, H, Dr];
    cache rows [c | k_rot]; the query at position p sees the keys j of its own sequence with
    0 <= p - j < window; score = (q_lat . c_j + q_rot . k_rot_j) * scale, f32 softmax,
    out[t, h] = sum_j p_j c_j, times sigmoid(gate[t, h]) when a gate [T, H] is given."""
    T, H, R = q_lat.shape
    Dr = q_rot.shape[2]
    S = cu.numel() - 1
    if N.use_native(q_lat):
        assert q_lat.is_contiguous() and q_rot.is_contiguous() and bt.is_contiguous()
        out = torch.empty((T, H, R), dtype=q_lat.dtype, device=q_lat.device)
        # decode-size steps (one row per segment) walk each row's keys with several blocks so that a
        # small batch still fills the chip; the split depends only on static sizes (graph-safe)
        nsplit, ws = 1, None
        if max_len == 1 and q_lat.dtype == torch.bfloat16:
            tiles = (min(window, bt.shape[1] * PAGE) + 31) // 32 + 1
            nsplit = max(1, min(16, tiles // 2, 1024 // max(S * ((H + 63) // 64), 1)))
            if nsplit > 1:
                ws = torch.empty((T, H, nsplit, R + 2), dtype=torch.float32, device=q_lat.device)
        N.mcall("mx_latent_attend", N.ptr(q_lat), N.ptr(q_rot), N.ptr(cache), N.ptr(cu), N.ptr(pos), N.ptr(bt),
                bt.shape[1], N.ptr(_rows(gate)) if gate is not None else None,
                gate.stride(0) if gate is not None else 0, int(min(window, 1 << 30)), float(scale), N.ptr(out),
                _dt(q_lat), S, int(max_len), H, R, Dr, nsplit, N.ptr(ws), N.stream())
        return out
    out = torch.zeros((T, H, R), dtype=torch.float32)
    rows = cache.view(-1, R + Dr).float()
    cul, pl = cu.tolist(), pos.tolist()
    for s in range(S):
        a, b = cul[s], cul[s + 1]
        if b <= a:
            continue
        ctx = pl[b - 1] + 1
        pages = bt[s, :(ctx + PAGE - 1) // PAGE].long()
        keys = rows.view(-1, PAGE, R + Dr)[pages].reshape(-1, R + Dr)[:ctx]
        qq = torch.cat([q_lat[a:b].float(), q_rot[a:b].float()], -1)       # [n, H, D]
        sc = torch.einsum("nhd,jd->nhj", qq, keys) * scale
        p = pos[a:b].long()[:, None]
        j = torch.arange(ctx)[None]
        vis = (j <= p) & (j > p - window)
        sc = sc.masked_fill(~vis[:, None, :], float("-inf"))
        out[a:b] = torch.einsum("nhj,jr->nhr", torch.softmax(sc, -1), keys[:, :R])
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[:, :, None]
    return out.to(q_lat.dtype)
