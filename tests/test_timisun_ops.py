"""Each Timisun mechanism alone: the framework's ops (CPU definitions, and the HIP kernels on a GPU box in fp32 and
bf16) against the plain fp64 functions of timisun_oracle.py. Inputs are made so that a fault shows: one key's score
is made to stand out and placed far back, at page borders, and just inside / just outside the window, for rows of a
prompt portion and for a single decoded row; pages are scattered over the pool; expert limits are hit; some
experts get no token."""
import math

import numpy as np
import pytest
import torch

import timisun_oracle as oracle
from llmss_amd import ops

gpu = pytest.mark.gpu
RUNS = [pytest.param("cpu", torch.float32, id="cpu-fp32"), pytest.param("cuda", torch.float32, marks=gpu, id="gpu-fp32"),
        pytest.param("cuda", torch.bfloat16, marks=gpu, id="gpu-bf16")]


def rnd(*shape, seed=0, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16).double()  # exactly representable in bf16


def tol(dtype, f32=2e-5, bf16=2e-2):
    return f32 if dtype == torch.float32 else bf16


def rel(got, want):
    return float((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-9))


@pytest.mark.parametrize("device,dtype", RUNS)
def test_scaled_embedding_and_residual_norm(device, dtype):
    V, W, T = 37, 50, 9
    table, w = rnd(V, W, seed=1), rnd(W, seed=2, std=0.2)
    ids = torch.tensor([3, 36, 0, 5, 5, 7, 1, 2, 30])
    x = ops.embed_scaled(ids.to(device), table.to(device, dtype), 2.5)
    assert x.dtype == torch.float32 and rel(x, table[ids] * 2.5) < 1e-6
    a, b = rnd(T, W, seed=3), rnd(T, W, seed=4)
    x0 = x.double().cpu()
    y = ops.resid_add_norm(x, a.to(device, dtype), b.to(device, torch.float32), w.to(device, dtype), 1.0, 1e-5, dtype)
    assert rel(x, x0 + (a + b)) < 1e-6  # the stream itself stays fp32 and is updated in place
    assert rel(y, oracle.norm_around_zero(x0 + (a + b), w, 1e-5)) < tol(dtype, bf16=1e-2)
    x1 = x.double().cpu()
    y = ops.resid_add_norm(x, None, None, w.to(device, dtype), 0.0, 1e-5, dtype)  # plain weight, nothing added
    assert rel(x, x1) == 0 and rel(y, oracle.rms_unit(x1, 1e-5) * w) < tol(dtype, bf16=1e-2)


def run_attention(device, dtype, h, c, wq, wuk, wuv, wo, heads, dim, vdim, scale, window, block, portions):
    """The framework's latent attention for one sequence whose latent rows c are already known: c goes into pages
    scattered over a pool, and the rows are attended in the given portions (a portion of 1 = a decoded token)."""
    T, R = c.shape
    nblk = -(-T // block)
    perm = torch.randperm(nblk + 3, generator=torch.Generator().manual_seed(5))[:nblk]
    cache = torch.zeros(nblk + 3, block, R, dtype=dtype, device=device)
    for p in range(T):
        cache[perm[p // block], p % block] = c[p].to(dtype)
    bt = perm.to(torch.int32)[None].to(device)
    d = lambda t: t.to(device, dtype)  # noqa: E731
    out, at = [], 0
    for n in portions:
        q = ops.linear_f(d(h[at:at + n]), d(wq), dtype)
        uk_t = d(wuk.view(heads, dim, R).transpose(1, 2).contiguous())
        qa = ops.head_absorb(q, uk_t, ops.latent_qa_dtype(cache))
        o = ops.latent_attn(qa, cache, bt, torch.tensor([0, n], dtype=torch.int32, device=device),
                            torch.tensor([at + n], dtype=torch.int32, device=device), window, scale, max_qlen=n,
                            max_ctx=T + 70 if n == 1 else 0)  # a decoded row: its keys may be split over workgroups
        out.append(ops.linear_f(ops.head_expand(o, d(wuv), dtype), d(wo), dtype))
        at += n
    return torch.cat(out)


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("R", [24, 64])  # 64: in bf16 the matrix-core kernel runs; 24: the generic one
@pytest.mark.parametrize("window,back", [(0, 300), (0, 1), (33, 32), (33, 33), (33, 0), (16, 15), (16, 16), (17, 16),
                                         (1, 0), (1, 1), (64, 63), (65, 64), (130, 129), (129, 129)])
def test_latent_attention_standout_key(device, dtype, window, back, R):
    """Query row i = T - 1 (and, as a portion's row, i - 3) has one key `back` positions behind it whose score
    dominates; whether that key is seen decides the output."""
    heads, dim, vdim, W, block = 3, 8, 12, 40, 16
    T = max(back + 6, 40)
    scale = 0.3
    h, c = rnd(T, W, seed=6), rnd(T, R, seed=7, std=0.3)
    wq, wuk = rnd(heads * dim, W, seed=8, std=W ** -0.5), rnd(heads * dim, R, seed=9, std=R ** -0.5)
    wuv, wo = rnd(heads * vdim, R, seed=10, std=R ** -0.5), rnd(W, heads * vdim, seed=11, std=0.2)
    for i in (T - 1, T - 4):
        j = i - back
        for hd in range(heads):  # along each head's absorbed query: large positive score at (i, j)
            qa = (h[i] @ wq.T)[hd * dim:(hd + 1) * dim] @ wuk[hd * dim:(hd + 1) * dim]
            c[j] = c[j] + 4.0 * qa / qa.norm() / heads ** 0.5
    c = c.to(torch.bfloat16).double()
    want = oracle.latent_attention(h, c, wq, wuk, wuv, wo, heads, dim, vdim, scale, window)
    seen = oracle.latent_attention(h, c, wq, wuk, wuv, wo, heads, dim, vdim, scale, 0)
    if window and back >= window:  # the construction works: hiding the key changes the row
        assert float((want[T - 1] - seen[T - 1]).abs().max()) > 0.05 * float(seen[T - 1].abs().max())
    for portions in ([T], [T - 5, 4, 1], [T - 2] + [1, 1]):
        got = run_attention(device, dtype, h, c, wq, wuk, wuv, wo, heads, dim, vdim, scale, window, block, portions)
        assert rel(got, want) < tol(dtype, f32=5e-5, bf16=3e-2), (portions, rel(got, want))


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("R,window", [(600, 0), (520, 17), (130, 5)])
def test_latent_attention_ranks_beyond_the_matrix_core_kernel(device, dtype, R, window):
    heads, dim, vdim, W, block, T = 2, 8, 8, 24, 16, 37
    h, c = rnd(T, W, seed=30), rnd(T, R, seed=31, std=0.5)
    wq, wuk = rnd(heads * dim, W, seed=32, std=W ** -0.5), rnd(heads * dim, R, seed=33, std=R ** -0.5)
    wuv, wo = rnd(heads * vdim, R, seed=34, std=R ** -0.5), rnd(W, heads * vdim, seed=35, std=0.2)
    want = oracle.latent_attention(h, c, wq, wuk, wuv, wo, heads, dim, vdim, 0.4, window)
    for portions in ([T], [T - 3, 2, 1]):
        got = run_attention(device, dtype, h, c, wq, wuk, wuv, wo, heads, dim, vdim, 0.4, window, block, portions)
        assert rel(got, want) < tol(dtype, f32=5e-5, bf16=3e-2), (portions, rel(got, want))


@pytest.mark.parametrize("device,dtype", RUNS)
def test_latent_rows_are_normed_into_their_slots(device, dtype):
    T, R, off, block = 7, 24, 16, 4
    src, w = rnd(T, off + R + 8, seed=12, std=3.0), rnd(R, seed=13)
    cache = torch.full((5, block, R), 7.0, dtype=dtype, device=device)
    slots = torch.tensor([8, 9, -1, 17, 0, 3, 19])
    ops.latent_norm_cache(src.to(device, dtype), off, R, w.to(device, dtype), 1e-5, cache, slots.to(device))
    want = oracle.rms_unit(src[:, off:off + R], 1e-5) * w
    flat = cache.view(-1, R).double().cpu()
    keep = slots >= 0
    assert rel(flat[slots[keep]], want[keep]) < tol(dtype, bf16=1e-2)
    untouched = torch.ones(20, dtype=torch.bool)
    untouched[slots[keep]] = False
    assert bool((flat[untouched] == 7.0).all())  # the unslotted row wrote nothing, other slots are left alone


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("T,E,top,F,shared", [(1, 7, 2, 20, 12), (3, 4, 4, 8, None), (150, 7, 2, 20, 12),
                                              (70, 3, 1, 70, 5), (130, 9, 3, 33, None)])
def test_mixture_of_experts(device, dtype, T, E, top, F, shared):
    W = 40
    h = rnd(T, W, seed=14, std=1.5)
    sd = {"router": rnd(E, W, seed=15, std=0.3), "correction": rnd(E, seed=16, std=0.5)}
    sd["correction"][E - 1] = -5.0  # an expert nobody chooses (unless top == E)
    for e in range(E):
        sd[f"e{e}.gate"], sd[f"e{e}.up"] = rnd(F, W, seed=20 + e, std=0.4), rnd(F, W, seed=40 + e, std=0.4)
        sd[f"e{e}.down"] = rnd(W, F, seed=60 + e, std=F ** -0.5)
    spec = dict(router=dict(experts=E, top=top), expert=dict(ff=F, limit=1.5))
    if shared:
        spec["shared"] = dict(ff=shared, limit=0.75)
        sd["shared.gate"], sd["shared.up"] = rnd(shared, W, seed=80, std=0.4), rnd(shared, W, seed=81, std=0.4)
        sd["shared.down"] = rnd(W, shared, seed=82, std=shared ** -0.5)
    want = oracle.moe(h, sd, "", spec)
    g = (h @ sd["e0.gate"].T)
    assert float(g.max()) > 1.5 and float((h @ sd["e0.up"].T).min()) < -1.5  # the limits are hit
    d = lambda t: t.to(device, dtype)  # noqa: E731
    hd = d(h)
    z = ops.linear_f(hd, d(sd["router"]), torch.float32)
    assert z.dtype == torch.float32
    idx, wts = ops.moe_route(z, sd["correction"].to(device, torch.float32), top)
    ci, cw = oracle.route(h, sd["router"], sd["correction"], top)
    assert torch.equal(idx.cpu().long().sort(-1).values, ci.sort(-1).values)
    idx2, wts2 = ops.moe_router(hd, d(sd["router"]), sd["correction"].to(device, torch.float32), top)  # fused launch
    assert torch.equal(idx2.cpu().long().sort(-1).values, ci.sort(-1).values)
    assert rel(wts2.sort(-1).values, cw.sort(-1).values) < (1e-5 if dtype == torch.float32 else 1e-3)
    assert rel(wts.sum(-1), torch.ones(T, dtype=torch.double)) < 1e-5
    sh = None
    if shared:
        gu = ops.linear_f(hd, d(torch.cat([sd["shared.gate"], sd["shared.up"]])), dtype)
        sh = ops.linear_f(ops.glu_clamp(gu, shared, 0.75, 1.702), d(sd["shared.down"]), dtype)
    stack = lambda n: d(torch.stack([sd[f"e{e}.{n}"] for e in range(E)]))  # noqa: E731
    got = ops.moe_experts(hd, idx, wts, stack("gate"), stack("up"), stack("down"), 1.5, 1.702, shared=sh)
    assert got.dtype == torch.float32 and rel(got, want) < tol(dtype, f32=5e-5, bf16=3e-2)


@pytest.mark.parametrize("device,dtype", RUNS)
def test_router_choice_uses_the_correction_and_the_weights_do_not(device, dtype):
    z = torch.tensor([[2.0, 1.0, 0.0, -1.0], [0.0, 0.0, 0.0, 0.0]])
    corr = torch.tensor([-1.0, 0.0, 0.9, 0.0])
    idx, wts = ops.moe_route(z.to(device), corr.to(device), 2)
    s = torch.sigmoid(z)
    # row 0: choice values .88-1, .73, .5+.9, .27 -> experts 2 and 1; weights from the uncorrected scores
    assert sorted(idx[0].tolist()) == [1, 2]
    w = {int(e): float(x) for e, x in zip(idx[0], wts[0])}
    assert math.isclose(w[1], float(s[0, 1] / (s[0, 1] + s[0, 2])), rel_tol=1e-5)
    assert sorted(idx[1].tolist()) == [1, 2] or sorted(idx[1].tolist()) == [2, 3]  # .5 + .9 first, then a tie
    assert 2 in idx[1].tolist()


@pytest.mark.parametrize("device,dtype", RUNS)
def test_strided_products_of_odd_shapes(device, dtype):
    """linear_f on shapes no MFMA tile divides, and the per-head absorbed / expanded projections."""
    for M, N, K in ((1, 5, 7), (67, 129, 35), (130, 64, 16)):
        x, w = rnd(M, K, seed=M), rnd(N, K, seed=N + 1)
        got = ops.linear_f(x.to(device, dtype), w.to(device, dtype), torch.float32)
        assert rel(got, x @ w.T) < 1e-5
    H, dim, vd, R, T = 3, 5, 7, 11, 9
    q, uk, uv, o = rnd(T, H * dim + 4, seed=90), rnd(H * dim, R, seed=91), rnd(H * vd, R, seed=92), rnd(T, H, R, seed=93)
    qa = ops.head_absorb(q.to(device, dtype), uk.view(H, dim, R).transpose(1, 2).contiguous().to(device, dtype))
    want = torch.einsum("thd,hdr->thr", q[:, :H * dim].view(T, H, dim), uk.view(H, dim, R))
    assert rel(qa, want) < 1e-5
    y = ops.head_expand(o.to(device, torch.float32), uv.to(device, dtype), torch.float32)
    assert rel(y, torch.einsum("thr,hvr->thv", o, uv.view(H, vd, R)).reshape(T, -1)) < 1e-5
