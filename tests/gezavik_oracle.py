"""A plain, slow fp32/fp64 implementation of the Gezavik design, one function per mechanism, written
from the design's equations and sharing no code with the package: the oracle of tests/test_gezavik*.py.

Everything takes whole sequences (no cache, no state carried between calls); ``w`` maps checkpoint
tensor names to tensors, ``cfg`` is the config.json dict.
"""
import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x):
    return x * torch.sigmoid(x)


def expert(w, p, h, limit):
    g = torch.clamp(h @ w[p + ".gate"].T, max=limit)
    u = torch.clamp(h @ w[p + ".up"].T, -limit, limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1)
    return y @ w[p + ".down"].T


def ff(w, p, mlp, h):
    if mlp is None:
        return torch.zeros_like(h)
    if mlp["kind"] == "dense":
        return torch.relu(h @ w[p + ".up"].T) ** 2 @ w[p + ".down"].T
    r = mlp["router"]
    E, I, top = r["experts"], r.get("identity", 0), r["top"]
    z = h @ w[p + ".router"].T
    s = torch.softmax(z, -1)
    choice = s + w[p + ".correction"]
    idx = torch.topk(choice, top, -1).indices
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in idx[t].tolist():
            wt = s[t, e]
            if e >= E:
                out[t] += wt * h[t]
            else:
                out[t] += wt * expert(w, f"{p}.e{e}", h[t:t + 1], mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        out = out + expert(w, p + ".shared", h, mlp["shared"]["limit"])
    return out


def mamba2(w, p, m, h, eps):
    T = h.shape[0]
    H, P, N, G, K = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = H * P
    proj = h @ w[p + ".in"].T
    z, xBC, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    cw, cb = w[p + ".conv"], w[p + ".conv.b"]
    pad = torch.cat([torch.zeros(K - 1, xBC.shape[1], dtype=h.dtype), xBC])
    conv = torch.stack([(pad[t:t + K] * cw.T).sum(0) + cb for t in range(T)])
    xBC = silu(conv)
    x = xBC[:, :inner].reshape(T, H, P)
    B = xBC[:, inner:inner + G * N].reshape(T, G, N)
    C = xBC[:, inner + G * N:].reshape(T, G, N)
    dt = torch.nn.functional.softplus(dt + w[p + ".dt_bias"])
    A = -torch.exp(w[p + ".A_log"])
    S = torch.zeros(H, N, P, dtype=h.dtype)
    y = torch.zeros(T, H, P, dtype=h.dtype)
    for t in range(T):
        for hh in range(H):
            g = hh // (H // G)
            S[hh] = torch.exp(A[hh] * dt[t, hh]) * S[hh] + dt[t, hh] * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S[hh].T @ C[t, g] + w[p + ".D"][hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = rms(y.reshape(T, ng, inner // ng), eps).reshape(T, inner) * w[p + ".norm"]
    return y @ w[p + ".o"].T


def rope(v, pos, dims, base):
    # v [..., T, d]; rotate first dims, interleaved pairs
    i = torch.arange(dims // 2, dtype=v.dtype)
    f = base ** (-2 * i / dims)
    a = pos.to(v.dtype)[:, None] * f[None]
    c, s = torch.cos(a), torch.sin(a)
    out = v.clone()
    u, w_ = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - w_ * s
    out[..., 1:dims:2] = w_ * c + u * s
    return out


def latent_attention(w, p, m, h, eps):
    T = h.shape[0]
    H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms(h @ w[p + ".dq"].T, eps) * w[p + ".dq.norm"]
    q = (cq @ w[p + ".uq"].T).reshape(T, H, dn + dr)
    kv = h @ w[p + ".dkv"].T
    c = rms(kv[:, :R], eps) * w[p + ".dkv.norm"]
    kr = kv[:, R:]
    pos = torch.arange(T)
    rd, base = m["rot"]["dims"], m["rot"]["base"]
    kr = rope(kr, pos, rd, base)
    qn, qr = q[..., :dn], q[..., dn:]
    qr = rope(qr.transpose(0, 1), pos, rd, base).transpose(0, 1)
    kn = (c @ w[p + ".uk"].T).reshape(T, H, dn)
    v = (c @ w[p + ".uv"].T).reshape(T, H, dv)
    sc = (torch.einsum("ihd,jhd->hij", qn, kn) + torch.einsum("ihd,jd->hij", qr, kr)) * m["scale"]
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None]
    size = (m.get("mask") or {}).get("size") or T + 1
    vis = (i - j >= 0) & (i - j < size)
    sc = sc.masked_fill(~vis, float("-inf"))
    pr = torch.softmax(sc, -1)
    o = torch.einsum("hij,jhd->ihd", pr, v)
    gate = torch.sigmoid(h @ w[p + ".g"].T)
    o = o * gate[:, :, None]
    return o.reshape(T, H * dv) @ w[p + ".o"].T


def greedy(cfg, w, prompt, n, dtype=torch.float64):
    """n greedy tokens after ``prompt`` (each step re-runs the whole sequence)."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(torch.argmax(forward(cfg, w, toks, dtype)[-1]).item()))
    return toks[len(prompt):]


def forward(cfg, w, tokens, dtype=torch.float32, layers_out=None):
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens)]
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}"
        h = rms(x, eps) * w[p + ".norm1"]
        if L["type"] == "mamba2":
            a = mamba2(w, p + ".mix", L["mixer"], h, eps)
        else:
            a = latent_attention(w, p + ".mix", L["mixer"], h, eps)
        x = x + cfg["residual_mult"] * (a + ff(w, p + ".mlp", L["mlp"], h))
        if layers_out is not None:
            layers_out.append(x.clone())
    h = rms(x, eps) * w["final.norm"]
    return h @ w["head"].T
