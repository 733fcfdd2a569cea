"""Plain whole-sequence float64 implementation of the Sigudra decoder, one function per mechanism.

Written from the design's equations only; shares no code with ``financial_chatbot_llm_amd``.  Every
function takes one sequence ([n, ...] tensors) and a dict of float64 weights keyed by the checkpoint
names without the layer prefix.  Slow on purpose: recurrences are token-by-token Python loops.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def sub(sd: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    """Tensors whose names start with ``prefix + '.'``, with that part cut off, as float64."""
    n = len(prefix) + 1
    return {k[n:]: (v.to(F64) if v.is_floating_point() else v) for k, v in sd.items() if k.startswith(prefix + ".")}


def layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.clamp(z, min=0) + torch.log1p(torch.exp(-z.abs()))


def causal_conv(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [n, C], w [C, K] with the last column on the current token; zeros before the sequence."""
    n, C = x.shape
    K = w.shape[1]
    out = torch.zeros_like(x)
    for t in range(n):
        for k in range(K):
            j = t - (K - 1) + k
            if j >= 0:
                out[t] += w[:, k] * x[j]
    if bias is not None:
        out = out + bias
    return out


def embed(tokens: List[int], sd: Dict[str, torch.Tensor], bigram: Optional[Dict]) -> torch.Tensor:
    x = sd["embed"].to(F64)[tokens]
    if bigram:
        B = int(bigram["buckets"])
        rows = [B] + [(tokens[i - 1] * int(bigram["mul_prev"]) + tokens[i] * int(bigram["mul_cur"])) % B
                      for i in range(1, len(tokens))]
        x = x + sd["bigram"].to(F64)[rows]
    return x


def channel_delta(h: torch.Tensor, w: Dict[str, torch.Tensor], m: Dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, G, D, P = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(causal_conv(h @ w["q"].T, w["q.conv"])).view(n, G, D)
    k = silu(causal_conv(h @ w["k"].T, w["k.conv"])).view(n, G, D)
    v = silu(causal_conv(h @ w["v"].T, w["v.conv"])).view(n, H, P)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w["b"].T)                                        # [n, H]
    dt = softplus((h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).view(n, H, D)
    g = torch.exp(-torch.exp(w["A_log"])[None, :, None] * dt)                 # [n, H, D]
    gate = torch.sigmoid((h @ w["g1"].T) @ w["g2"].T).view(n, H, P)
    out = torch.zeros(n, H, P, dtype=F64)
    for hd in range(H):
        kv = hd // (H // G)
        S = torch.zeros(D, P, dtype=F64)
        for t in range(n):
            S = g[t, hd][:, None] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            out[t, hd] = S.T @ q[t, kv]
    out = rms(out, eps) * w["norm"] * gate
    return out.reshape(n, H * P) @ w["o"].T


def gla(h: torch.Tensor, w: Dict[str, torch.Tensor], m: Dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, D, P, tau = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"])
    q = (h @ w["q"].T).view(n, H, D) * D ** -0.5
    k = (h @ w["k"].T).view(n, H, D)
    v = (h @ w["v"].T).view(n, H, P)
    z = (h @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / tau)).view(n, H, D)
    out = torch.zeros(n, H, P, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, P, dtype=F64)
        for t in range(n):
            S = alpha[t, hd][:, None] * S + torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = S.T @ q[t, hd]
    out = rms(out, eps) * w["norm"]
    return (out.reshape(n, H * P) * silu(h @ w["g"].T)) @ w["o"].T


def window_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: Dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, G, D, P = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    window = int(m["mask"]["size"]) if m.get("mask") else None
    q = rms(h @ w["q"].T, eps) * w["q.norm"]          # statistics over the whole projection
    k = rms(h @ w["k"].T, eps) * w["k.norm"]
    q, k = q.view(n, H, D), k.view(n, G, D)
    v = (h @ w["v"].T).view(n, G, P)
    gate = torch.sigmoid(h @ w["g"].T)                # [n, H]
    out = torch.zeros(n, H, P, dtype=F64)
    for hd in range(H):
        kv = hd // (H // G)
        for i in range(n):
            lo = 0 if window is None else max(0, i - window + 1)
            sc = (k[lo:i + 1, kv] @ q[i, hd]) * float(m["scale"])
            p = torch.softmax(sc, 0)
            out[i, hd] = (p[:, None] * v[lo:i + 1, kv]).sum(0) * gate[i, hd]
    return out.reshape(n, H * P) @ w["o"].T


def gated_lru(h: torch.Tensor, w: Dict[str, torch.Tensor], m: Dict) -> torch.Tensor:
    n = h.shape[0]
    R, B = int(m["width"]), int(m["blocks"])
    y = gelu_tanh(h @ w["y"].T + w["y.b"])
    u = causal_conv(h @ w["x"].T + w["x.b"], w["conv"], w["conv.b"])
    ub = u.view(n, B, R // B)
    r = torch.sigmoid(torch.einsum("boi,nbi->nbo", w["ra"], ub) + w["ra.b"]).reshape(n, R)
    i = torch.sigmoid(torch.einsum("boi,nbi->nbo", w["ri"], ub) + w["ri.b"]).reshape(n, R)
    a = torch.exp(-8.0 * r * softplus(w["lam"]))
    S = torch.zeros(R, dtype=F64)
    out = torch.zeros(n, R, dtype=F64)
    for t in range(n):
        S = a[t] * S + torch.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S
    return (out * y) @ w["o"].T


def parallel(h: torch.Tensor, w: Dict[str, torch.Tensor], m: Dict, eps: float) -> torch.Tensor:
    left = window_attention(h, sub(w, "left"), m["left"], eps)
    right = gated_lru(h, sub(w, "right"), m["right"])
    return 0.5 * (rms(left, eps) * w["left.out"] + rms(right, eps) * w["right.out"])


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    return (gelu_tanh(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def routed_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], spec: Dict) -> torch.Tensor:
    top = int(spec["router"]["top"])
    s = torch.sigmoid(h @ w["router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in torch.topk(s[t], top).indices.tolist():
            xin = s[t, e] * h[t]
            out[t] += (silu(w[f"e{e}.gate"] @ xin) * (w[f"e{e}.up"] @ xin)) @ w[f"e{e}.down"].T
    return out


MIXERS = {"channel_delta": channel_delta, "gla": gla, "parallel": parallel}


def forward(cfg: Dict, sd: Dict[str, torch.Tensor], tokens: List[int], streams: Optional[list] = None) -> torch.Tensor:
    """Logits [n, vocab] (float64) of one whole sequence; ``streams`` collects x after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = embed(tokens, sd, (cfg.get("embedding") or {}).get("bigram"))
    for i, spec in enumerate(cfg["layers"]):
        w = sub(sd, f"l{i}")
        m = MIXERS[spec["type"]](x, sub(w, "mix"), spec["mixer"], eps)
        x = x + layer_norm(m, w["norm1"], eps)
        mlp = spec.get("mlp")
        if mlp is not None:
            f = dense_ff(x, sub(w, "mlp")) if mlp["kind"] == "dense" else routed_ff(x, sub(w, "mlp"), mlp)
            x = x + layer_norm(f, w["norm2"], eps)
        if streams is not None:
            streams.append(x.clone())
    return layer_norm(x, sd["final.norm"].to(F64), eps) @ sd["head"].to(F64).T


def greedy(cfg: Dict, sd: Dict[str, torch.Tensor], prompt: List[int], n: int) -> List[int]:
    """``n`` greedy tokens after ``prompt``, each from a whole-sequence forward pass."""
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(forward(cfg, sd, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out
