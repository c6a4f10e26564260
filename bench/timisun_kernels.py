"""Per-kernel rates of the Timisun design beside the like kernel of the Llama family, at layer shapes of
bench/timisun_compare.py: achieved TFLOP/s for the matrix-core kernels, TB/s for the memory-bound ones, each at a
prompt step (M tokens) and a decode step (B single tokens). Prints one JSON object.

    python bench/timisun_kernels.py [--size w2048] [--tokens 8192] [--batch 64] [--ctx 1024]
"""
import argparse
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "bench"))

PEAK_TFLOPS, PEAK_TBS = 2500.0, 8.0


def timed(fn, iters=20, warm=3):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    b.synchronize()
    return a.elapsed_time(b) / iters * 1e-3  # seconds


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--size", default="w2048")
    ap.add_argument("--tokens", type=int, default=8192)
    ap.add_argument("--seq", type=int, default=1024)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--ctx", type=int, default=1024)
    a = ap.parse_args()
    from timisun_compare import SIZES

    from llmss_amd import ops
    from llmss_amd.ops import hip as H

    s = SIZES[a.size]
    dev = torch.device("cuda", 0)
    bf = torch.bfloat16
    W, Hh, dim, vd, R, win = s["width"], s["heads"], s["dim"], s["vdim"], s["rank"], s["window"]
    E, top, F, Fd = s["experts"], s["top"], s["ff"], s["top"] * s["ff"] + s["shared"]
    g = torch.Generator(device=dev).manual_seed(0)

    def rn(*shape, dt=bf, std=1.0):
        return (torch.randn(*shape, device=dev, generator=g) * std).to(dt)

    H.reserve_workspace(dev, 64 << 20)
    rows = []

    def add(name, phase, sec, flops=0.0, bytes_=0.0, like=None):
        """``of_roofline``: the time the kernel's own roofline allows - the larger of flops / peak matrix rate and
        bytes / peak HBM rate - over the time measured."""
        r = dict(kernel=name, phase=phase, us=round(sec * 1e6, 1))
        if flops:
            r["tflops"] = round(flops / sec / 1e12, 1)
        if bytes_:
            r["tb_s"] = round(bytes_ / sec / 1e12, 3)
        if flops or bytes_:
            r["of_roofline"] = round(max(flops / (PEAK_TFLOPS * 1e12), bytes_ / (PEAK_TBS * 1e12)) / sec, 4)
        if like:
            r["like"] = like
        rows.append(r)
        print(json.dumps(r), file=sys.stderr, flush=True)
        return r

    for phase, M in (("prompt", a.tokens), ("decode", a.batch)):
        # ---------------- residual add + norm
        x32, a_bf, b32, w = rn(M, W, dt=torch.float32), rn(M, W), rn(M, W, dt=torch.float32), rn(W, std=0.1)
        t = timed(lambda: ops.resid_add_norm(x32, a_bf, b32, w, 1.0, 1e-6, bf))
        add("resid_add_norm", phase, t, bytes_=M * W * 16)
        xb, res = rn(M, W), rn(M, W)
        t = timed(lambda: ops.add_norm(xb, w, None, 1e-6, True, res))
        add("add_norm (bf16 residual)", phase, t, bytes_=M * W * 8, like="resid_add_norm")
        # ---------------- per-head absorbed / expanded projections vs a dense GEMM of similar work
        q, uk_t = rn(M, Hh * dim, std=0.3), rn(Hh, R, dim, std=dim ** -0.5)
        t = timed(lambda: ops.head_absorb(q, uk_t, bf))
        add("head_absorb (gemm_tile, batched)", phase, t, flops=2.0 * M * Hh * dim * R,
            bytes_=2.0 * (M * Hh * dim + M * Hh * R + Hh * R * dim))
        o, uv = rn(M, Hh, R, std=0.3), rn(Hh * vd, R, std=R ** -0.5)
        t = timed(lambda: ops.head_expand(o, uv, bf))
        add("head_expand (gemm_tile, batched)", phase, t, flops=2.0 * M * Hh * R * vd,
            bytes_=2.0 * (M * Hh * R + M * Hh * vd + Hh * vd * R))
        h, wo = rn(M, W, std=0.3), rn(W, W, std=W ** -0.5)
        t = timed(lambda: ops.linear(h, wo))
        add("dense o-projection (gemm.hip)", phase, t, flops=2.0 * M * W * W, bytes_=2.0 * (2 * M * W + W * W),
            like="head_absorb / head_expand")
        # ---------------- experts vs dense gated MLP
        router, corr = rn(E, W, std=W ** -0.5), rn(E, dt=torch.float32, std=0.1)
        gate, up, down = rn(E, F, W, std=W ** -0.5), rn(E, F, W, std=W ** -0.5), rn(E, W, F, std=F ** -0.5)
        t = timed(lambda: ops.moe_router(h, router, corr, top))
        add("router logits + route", phase, t)
        # every token draws its experts uniformly, so the grouped GEMMs see balanced groups and, in a decode step,
        # touch the experts a served batch would
        idx = torch.rand(M, E, device=dev, generator=g).topk(top, dim=-1).indices.to(torch.int32).contiguous()
        wts = torch.full((M, top), 1.0 / top, dtype=torch.float32, device=dev)
        t = timed(lambda: ops.moe_experts(h, idx, wts, gate, up, down, 7.0, 1.702, combine=False))
        touched = int(idx.unique().numel())
        add("experts: group + gate_up + down (gemm_tile grouped)", phase, t, flops=6.0 * M * top * F * W,
            bytes_=touched * 3 * F * W * 2 + M * top * (F * 2 * 2 + W * 4) + M * W * 2)
        wu = ops.glu_interleave(rn(Fd, W, std=W ** -0.5), rn(Fd, W, std=W ** -0.5), 0)
        wd = rn(W, Fd, std=Fd ** -0.5)
        t = timed(lambda: ops.linear(ops.linear(h, wu, None, "none", True), wd))
        add("dense gated MLP (gemm.hip, 2 launches)", phase, t, flops=6.0 * M * Fd * W,
            bytes_=3 * Fd * W * 2 + M * (Fd * 2 * 2 + W * 2 * 2), like="experts")
    # ---------------- attention, prompt: B sequences of `seq` tokens
    bs = 16
    B, S = max(1, a.tokens // a.seq), a.seq
    nblk = -(-S // bs)
    cache = rn(B * nblk, bs, R, std=0.3)
    bt = torch.arange(B * nblk, dtype=torch.int32, device=dev).view(B, nblk)
    cu = torch.arange(0, (B + 1) * S, S, dtype=torch.int32, device=dev)
    ctx = torch.full((B,), S, dtype=torch.int32, device=dev)
    qa = rn(B * S, Hh, R, std=0.1)
    t = timed(lambda: ops.latent_attn(qa, cache, bt, cu, ctx, win, dim ** -0.5, max_qlen=S))
    pairs = sum(min(i + 1, win) for i in range(S)) * B
    add(f"latent attention, prompt (extend kernel, rank {R}, window {win})", "prompt", t, flops=4.0 * Hh * R * pairs,
        bytes_=2.0 * (2 * B * S * Hh * R + B * S * R))
    D = W // Hh
    qkv = rn(B * S, 3 * Hh * D, std=0.3)
    t = timed(lambda: ops.attn_prefill(qkv, cu, S, Hh, Hh, D, D ** -0.5))
    add(f"dense causal attention, prompt (head_dim {D})", "prompt", t, flops=4.0 * Hh * D * B * S * (S + 1) / 2,
        bytes_=2.0 * 4 * B * S * Hh * D, like="latent attention, prompt")
    # ---------------- attention, decode: `batch` sequences with `ctx` cached tokens
    B, C = a.batch, a.ctx
    nblk = -(-C // bs)
    cache = rn(B * nblk, bs, R, std=0.3)
    bt = torch.nn.functional.pad(torch.arange(B * nblk, dtype=torch.int32, device=dev).view(B, nblk), (0, 8))
    cu = torch.arange(B + 1, dtype=torch.int32, device=dev)
    ctx = torch.full((B,), C, dtype=torch.int32, device=dev)
    qa = rn(B, Hh, R, std=0.1)
    t = timed(lambda: ops.latent_attn(qa, cache, bt, cu, ctx, win, dim ** -0.5, max_qlen=1, max_ctx=C + 64))
    add(f"latent attention, decode (extend kernel + key split, rank {R})", "decode", t,
        bytes_=B * min(C, win) * R * 2)
    kc, vc = rn(B * nblk, Hh, bs, D, std=0.3), rn(B * nblk, Hh, bs, D, std=0.3)
    qd = rn(B, 3 * Hh * D, std=0.3)
    t = timed(lambda: ops.attn_decode(qd, kc, vc, bt, ctx, Hh, Hh, D, D ** -0.5, C + 64))
    add(f"dense decode attention (head_dim {D}, {Hh} kv heads)", "decode", t, bytes_=B * C * Hh * D * 2 * 2,
        like="latent attention, decode")
    print(json.dumps(dict(size=a.size, shape=s, tokens=a.tokens, batch=a.batch, ctx=a.ctx, peak_tflops=PEAK_TFLOPS,
                          peak_tb_s=PEAK_TBS, kernels=rows)))


if __name__ == "__main__":
    main()
