"""Times the sequence-mixer kernels (``ops.mixers``) at the layer shapes of a hybrid decoder.

    python -m financial_chatbot_llm_amd.bench.mixer_kernels [--width 2048]

Two step shapes: a prefill step of two 2048-token prompts and a decode step of 64 single rows at
depth 1024.  Shapes follow ``models.gezavik.example_config(scale_up=True)``: Mamba-2 with inner =
2 * width, 64-wide heads, state 128, 2 groups, 4 taps; latent attention with width / 128 heads,
kv_rank 256, rot_dim 32, window 1024.  One JSON line per kernel and shape (microseconds, and the
arithmetic or byte rate the time corresponds to).
"""
from __future__ import annotations

import argparse
import json

import torch

from ..ops import mixers as mx


def _time(f, n: int = 20) -> float:
    for _ in range(3):
        f()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(n):
        f()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / n * 1e3


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--width", type=int, default=2048)
    a = ap.parse_args(argv)
    dev = "cuda"
    H, P, Ns, G, K = 2 * a.width // 64, 64, 128, 2, 4
    C = H * P + 2 * G * Ns
    Ha, R, Dr, window = max(a.width // 128, 2), 256, 32, 1024
    for name, lens, start in (("prefill 2x2048", [2048, 2048], 0), ("decode 64x1 at 1024", [1] * 64, 1024)):
        S, T = len(lens), sum(lens)
        cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32, device=dev)
        pos = torch.cat([torch.arange(start, start + n) for n in lens]).to(torch.int32).to(dev)
        slot = torch.arange(S, dtype=torch.int32, device=dev)
        inp = torch.randn(T, C, device=dev).bfloat16()
        cw, cb = torch.randn(C, K, device=dev), torch.randn(C, device=dev)
        cst = torch.zeros(S, K - 1, C, device=dev)
        us = _time(lambda: mx.conv_silu(inp, cw, cb, cst, cu, slot, pos, max(lens)))
        print(json.dumps({"shape": name, "kernel": "conv_silu", "us": round(us, 1),
                          "TB_per_s": round(T * C * 6 / us / 1e6, 2)}), flush=True)
        u = mx.conv_silu(inp, cw, cb, cst, cu, slot, pos, max(lens))
        dtr = torch.randn(T, H, device=dev).bfloat16()
        dtb, Al, Dd = torch.zeros(H, device=dev) - 3, torch.zeros(H, device=dev), torch.ones(H, device=dev)
        sst = torch.zeros(S, H, P, Ns, device=dev)
        us = _time(lambda: mx.ssm_scan(u, dtr, dtb, Al, Dd, sst, cu, slot, pos, H, P, Ns, G))
        print(json.dumps({"shape": name, "kernel": "ssm_scan", "us": round(us, 1),
                          "f32_TFLOP_per_s": round(T * H * P * Ns * 4 / us / 1e6, 2),
                          "state_TB_per_s": round(S * H * P * Ns * 8 / us / 1e6, 2)}), flush=True)
        pages = (start + max(lens) + 63) // 64
        cache = torch.randn(S * pages * 64, R + Dr, device=dev).bfloat16()
        bt = torch.arange(S * pages, dtype=torch.int32, device=dev).view(S, pages).contiguous()
        ql = torch.randn(T, Ha, R, device=dev).bfloat16() * .1
        qr = torch.randn(T, Ha, Dr, device=dev).bfloat16() * .1
        gate = torch.randn(T, Ha, device=dev).bfloat16()
        us = _time(lambda: mx.latent_attend(ql, qr, cache, cu, pos, bt, window, 0.1, max(lens), gate=gate), 5)
        pairs = sum(min(p + 1, window) for n in lens for p in range(start, start + n))
        print(json.dumps({"shape": name, "kernel": "latent_attend", "us": round(us, 1),
                          "bf16_TFLOP_per_s": round(pairs * Ha * 2 * (2 * R + Dr) / us / 1e6, 1),
                          "cache_TB_per_s": round(S * min(start + max(lens), window + max(lens)) * (R + Dr) * 2 / us / 1e6, 2)}),
              flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
