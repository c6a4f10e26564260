"""Each mechanism of the Babotar design alone: the framework's op (CPU definition, and on a GPU box the HIP kernel in
fp32 and bf16 storage) against the plain float64 function in babotar_oracle.py, over pages that are scattered, state
slots that held something else before, portions cut at awkward places, and inputs built so that a fault shows (a far
key whose score stands out, scores so low that only the sink is left, scores far above the cap)."""
import math

import numpy as np
import pytest
import torch

import babotar_oracle as oracle
from llmss_amd import ops

gpu = pytest.mark.gpu
RUNS = [pytest.param("cpu", torch.float32, id="cpu-fp32"), pytest.param("cuda", torch.float32, marks=gpu, id="gpu-fp32"),
        pytest.param("cuda", torch.bfloat16, marks=gpu, id="gpu-bf16")]
F64 = torch.float64


def tol(dtype):
    return 2e-5 if dtype == torch.float32 else 2e-2


def close(got, want, dtype, what="", scale=None):
    got, want = got.detach().double().cpu(), want.double()
    s = float(want.abs().max()) if scale is None else scale
    err = float((got - want).abs().max()) / max(s, 1e-9)
    assert err < tol(dtype), f"{what}: error {err:.3g} of the largest value"


def rnd(*shape, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype).double()  # values the storage type holds exactly


def i32(x, device):
    return torch.tensor(x, dtype=torch.int32, device=device)


def steps_of(cuts_per_seq):
    """[(seq, first position, rows)] step lists: step k feeds portion k of every sequence that still has one."""
    at = [0] * len(cuts_per_seq)
    out = []
    for k in range(max(len(c) for c in cuts_per_seq)):
        step = []
        for s, cuts in enumerate(cuts_per_seq):
            if k < len(cuts):
                step.append((s, at[s], cuts[k]))
                at[s] += cuts[k]
        out.append(step)
    return out


def meta(step, slots, device):
    cu = np.cumsum([0] + [n for _, _, n in step])
    return (i32(cu.tolist(), device), i32([p0 + n for _, p0, n in step], device), i32([slots[s] for s, _, _ in step], device))


# ------------------------------------------------------------------------------------------------ streams and norms
@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("S,W,rms", [(1, 40, False), (2, 48, False), (3, 100, True), (4, 24, False)])
def test_stream_write_back_and_normed_read(device, dtype, S, W, rms):
    T = 7
    x0 = rnd(S, T, W, seed=1) * 3 + 0.5
    y, w = rnd(T, W, seed=2, dtype=dtype), (1 + 0.1 * rnd(W, seed=3)).to(dtype).double()
    mix, outw, inw = torch.eye(S).double() + 0.3 * rnd(S, S, seed=4), 1 + 0.3 * rnd(S, seed=5), rnd(S, seed=6)
    c, eps = 0.7, 1e-5
    x = x0.float().to(device).contiguous()
    h = ops.stream_add_norm(x, y.to(dtype).to(device), mix.float().to(device).contiguous(), outw.float().to(device),
                            c, inw.float().to(device), w.to(dtype).to(device), eps, rms, torch.float32)
    nx = torch.stack([sum(mix[s, t] * x0[s] for s in range(S)) + c * outw[t] * y for t in range(S)])
    u = sum(inw[s] * nx[s] for s in range(S))
    want = oracle.rms_div(u, eps) * w if rms else oracle.layer_norm(u, w, eps)
    close(x, nx, torch.float32, "streams after the write-back")
    close(h, want, torch.float32, "normed read")
    # read only (first sublayer), plain sum (final norm), output in the storage type
    h2 = ops.stream_add_norm(x, None, None, None, c, None, w.to(dtype).to(device), eps, rms, dtype)
    u2 = nx.sum(0)
    close(h2, oracle.rms_div(u2, eps) * w if rms else oracle.layer_norm(u2, w, eps), dtype, "plain sum read")
    close(x, nx, torch.float32, "a read leaves the streams alone")


@pytest.mark.parametrize("device,dtype", RUNS)
def test_embedding_fills_every_stream(device, dtype):
    tab, pos = rnd(13, 20, seed=1, dtype=dtype), rnd(9, 20, seed=2, dtype=dtype)
    ids, p = torch.tensor([3, 12, 0, 3]), torch.tensor([0, 8, 5, 1])
    x = ops.embed_streams(ids.to(device), p.to(device), tab.to(dtype).to(device), pos.to(dtype).to(device), 3)
    for s in range(3):
        close(x[s], tab[ids] + pos[p], torch.float32, f"stream {s}")
    x = ops.embed_streams(ids.to(device), p.to(device), tab.to(dtype).to(device), None, 1)
    close(x[0], tab[ids], torch.float32, "no position table")


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("groups,n,act", [(1, 96, "sigmoid"), (3, 20, "silu"), (2, 300, "silu"), (5, 1, "sigmoid")])
def test_gated_group_norm(device, dtype, groups, n, act):
    T, eps, c = 5, 1e-5, 0.9
    o, gate, w = rnd(T, groups * n, seed=1) * 4, rnd(T, groups * n + 3, seed=2, dtype=dtype), rnd(n, seed=3, dtype=dtype)
    g = gate[:, 3:]
    got = ops.gated_group_norm(o.float().to(device), gate.to(dtype).to(device)[:, 3:], w.to(dtype).to(device), eps, act,
                               c, out_dtype=dtype)
    a = torch.sigmoid(g) if act == "sigmoid" else oracle.silu(g)
    want = (oracle.rms_div(o.view(T, groups, n), eps) * w).view(T, -1) * a * c
    close(got, want, dtype, "gated norm")


@pytest.mark.parametrize("device,dtype", RUNS)
def test_gated_activation(device, dtype):
    gu = rnd(6, 2 * 37, seed=1, dtype=dtype) * 3
    got = ops.glu_act(gu.to(dtype).to(device), 37, "gelu_tanh")
    close(got, oracle.gelu_tanh(gu[:, :37]) * gu[:, 37:], dtype, "tanh-form GELU gate")


# ------------------------------------------------------------------------------------------------ convolution tails
@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("taps,res,silu", [(3, True, False), (4, False, True), (2, False, True), (1, True, False),
                                           (9, False, False)])
def test_causal_convolution_over_portions_and_reused_slots(device, dtype, taps, res, silu):
    C = 70
    lens = [23, 1, 12]
    xs = [rnd(n, C, seed=10 + i, dtype=dtype) for i, n in enumerate(lens)]
    w = rnd(C, taps, seed=3, dtype=dtype)
    cuts = [[2, 1, 1, 7, 1, 2, 9], [1], [5, 1, 6]]  # portions shorter than the tail, single rows, and a one-row sequence
    slots = [2, 0, 3]
    state = torch.full((4, max(taps - 1, 0), C), 77.0, device=device)  # whatever the slots held before
    got = [torch.zeros(n, C) for n in lens]
    for step in steps_of(cuts):
        cu, ctx, ss = meta(step, slots, device)
        x = torch.cat([xs[s][p0:p0 + n] for s, p0, n in step]).to(dtype).to(device)
        y = ops.causal_conv(x, w.to(dtype).to(device), state, cu, ctx, ss, res, silu, torch.float32).cpu()
        r = 0
        for s, p0, n in step:
            got[s][p0:p0 + n] = y[r:r + n]
            r += n
    for s, n in enumerate(lens):
        want = oracle.causal_conv(xs[s], w) + (xs[s] if res else 0)
        close(got[s], oracle.silu(want) if silu else want, torch.float32, f"sequence {s}")
    if taps > 1:  # the tail is the sequence's last inputs, zeros where it is shorter
        want = torch.cat([torch.zeros(max(taps - 1 - lens[2], 0), C, dtype=F64), xs[2][-(taps - 1):]])
        close(state[3], want, torch.float32, "tail after the last step")


# ------------------------------------------------------------------------------------------------------- recurrences
@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("H,d,dv", [(3, 8, 12), (1, 40, 70), (2, 160, 20), (2, 64, 64)])
def test_decay_recurrence_carries_its_state(device, dtype, H, d, dv):
    lens = [19, 6]
    decay = torch.tensor([0.5, 0.97, 0.999][:H]).double()
    data = [[rnd(n, H * k, seed=20 + 3 * i + j, dtype=dtype) for j, k in enumerate((d, d, dv))] for i, n in enumerate(lens)]
    cuts = [[1, 2, 9, 1, 6], [2, 4]]
    slots = [1, 0]
    state = torch.full((2, H, d, dv), 5.0, device=device)
    got = [torch.zeros(n, H * dv) for n in lens]
    for step in steps_of(cuts):
        cu, ctx, ss = meta(step, slots, device)
        q, k, v = (torch.cat([data[s][j][p0:p0 + n] for s, p0, n in step]).to(dtype).to(device) for j in range(3))
        y = ops.decay_recurrence(q, k, v, decay.float().to(device), state, cu, ctx, ss, H, d, dv, True).cpu()
        r = 0
        for s, p0, n in step:
            got[s][p0:p0 + n] = y[r:r + n]
            r += n
    for s, n in enumerate(lens):
        q, k, v = (oracle.silu(t) for t in data[s])
        want = oracle.lightning_scan(q.view(n, H, d), k.view(n, H, d), v.view(n, H, dv), decay.tolist())
        close(got[s], want.reshape(n, -1), torch.float32 if dtype == torch.float32 else dtype, f"sequence {s}")


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("H,G,d,dv", [(4, 2, 8, 12), (1, 1, 48, 40), (2, 2, 130, 24), (6, 2, 32, 64)])
def test_delta_rule_carries_its_state(device, dtype, H, G, d, dv):
    lens = [17, 5]
    A_log, dtb = rnd(H, seed=1) * 0.5 - 1, rnd(H, seed=2) * 0.3
    data = []
    for i, n in enumerate(lens):
        q, k, v = rnd(n, G * d, seed=30 + i), rnd(n, G * d, seed=40 + i) * 2, rnd(n, H * dv, seed=50 + i)
        ab = rnd(n, 2 * H, seed=60 + i, dtype=dtype) * 2
        data.append((q, k, v, ab))
    cuts = [[3, 1, 1, 12], [1, 4]]
    slots = [0, 2]
    state = torch.full((3, H, d, dv), -3.0, device=device)
    got = [torch.zeros(n, H * dv) for n in lens]
    for step in steps_of(cuts):
        cu, ctx, ss = meta(step, slots, device)
        q, k, v = (torch.cat([data[s][j][p0:p0 + n] for s, p0, n in step]).float().to(device) for j in range(3))
        ab = torch.cat([data[s][3][p0:p0 + n] for s, p0, n in step]).to(dtype).to(device)
        y = ops.delta_recurrence(q, k, v, ab[:, :H], ab[:, H:], A_log.float().to(device), dtb.float().to(device), state,
                                 cu, ctx, ss, H, G, d, dv).cpu()
        r = 0
        for s, p0, n in step:
            got[s][p0:p0 + n] = y[r:r + n]
            r += n
    for s, n in enumerate(lens):
        q, k, v, ab = data[s]
        q, k = q.view(n, G, d), k.view(n, G, d)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        beta = torch.sigmoid(ab[:, H:])
        g = torch.exp(-torch.exp(A_log) * torch.nn.functional.softplus(ab[:, :H] + dtb))
        want = oracle.delta_scan(q, k, v.view(n, H, dv), beta, g)
        close(got[s], want.reshape(n, -1), torch.float32, f"sequence {s}")


# ------------------------------------------------------------------------------------------- rotation and attention
@pytest.mark.parametrize("dims,scaling", [(8, None), (16, dict(factor=4.0, original=64, fast=16.0, slow=1.0)),
                                          (64, dict(factor=2.0, original=512, fast=8.0, slow=2.0))])
def test_angle_table(dims, scaling):
    rot = dict(dims=dims, base=5000.0, scaling=scaling)
    cos, sin = oracle.rotary_tables(rot, 300)
    tab = ops.rope_angle_table(300, dims, 5000.0, None if scaling is None else tuple(
        float(scaling[k]) for k in ("factor", "original", "fast", "slow")))
    assert float((tab[..., 0].double() - cos).abs().max()) < 1e-6 and float((tab[..., 1].double() - sin).abs().max()) < 1e-6


class Paged:
    """Keys and values of a few sequences in pages taken in a scattered order."""

    def __init__(self, lens, G, d, dv, bs, device, dtype, seed=0):
        self.bs, self.G, self.d, self.dv = bs, G, d, dv
        nb = sum(-(-n // bs) for n in lens) + 3
        order = np.random.default_rng(seed).permutation(nb).tolist()
        self.kc = torch.full((nb, bs, G * d), 9.0, dtype=dtype, device=device)
        self.vc = torch.full((nb, bs, G * dv), 9.0, dtype=dtype, device=device)
        self.tables = []
        for n in lens:
            self.tables.append([order.pop() for _ in range(-(-n // bs))])
        self.maxb = max(len(t) for t in self.tables)

    def slots(self, s, p0, n):
        return [self.tables[s][p // self.bs] * self.bs + p % self.bs for p in range(p0, p0 + n)]

    def bt(self, seqs, device):
        return i32([self.tables[s] + [0] * (self.maxb - len(self.tables[s])) for s in seqs], device)


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("H,G,d,dv,rot", [(4, 2, 16, 12, 8), (2, 2, 8, 8, 8), (3, 1, 24, 40, 0), (8, 2, 64, 128, 32)])
def test_rotation_bias_and_cache_write(device, dtype, H, G, d, dv, rot):
    T, bs = 11, 4
    pg = Paged([T], G, d, dv, bs, device, dtype)
    nq, nk, nv = H * d, G * d, G * dv
    proj = rnd(T, 5 + nq + nk + nv, seed=1, dtype=dtype)
    bias = rnd(nq + nk + nv, seed=2, dtype=dtype)
    pos = torch.arange(T) + 3
    sc = (2.0, 32.0, 8.0, 1.0)
    tab = ops.rope_angle_table(64, rot, 100.0, sc) if rot else None
    slots = torch.tensor(pg.slots(0, 0, T))
    slots[4] = -1  # a row that is not cached
    q = ops.rope_bias_cache(proj.to(dtype).to(device), 5, 5 + nq, 5 + nq + nk, bias.to(dtype).to(device), pos.to(device),
                            tab.to(device) if rot else None, rot, pg.kc, pg.vc, slots.to(device), H, G, d, dv)
    qw = (proj[:, 5:5 + nq] + bias[:nq]).view(T, H, d)
    kw = (proj[:, 5 + nq:5 + nq + nk] + bias[nq:nq + nk]).view(T, G, d)
    vw = proj[:, 5 + nq + nk:] + bias[nq + nk:]
    if rot:
        cos, sin = oracle.rotary_tables(dict(dims=rot, base=100.0, scaling=dict(factor=2.0, original=32.0, fast=8.0,
                                                                               slow=1.0)), 64)
        qw, kw = oracle.rotate(qw, cos[pos], sin[pos], rot), oracle.rotate(kw, cos[pos], sin[pos], rot)
    close(q, qw.reshape(T, nq), torch.float32 if dtype == torch.float32 else dtype, "q")
    keep = slots >= 0
    close(pg.kc.view(-1, nk)[slots[keep]], kw.reshape(T, nk)[keep], dtype, "cached k")
    close(pg.vc.view(-1, nv)[slots[keep]], vw[keep], dtype, "cached v")
    assert float(pg.kc.view(-1, nk).float().cpu()[[s for s in range(pg.kc.shape[0] * bs) if s not in slots.tolist()]].min()) == 9.0


def attention_case(device, dtype, H, G, d, dv, lens, cuts, scale, cap, talk, bs=16, boost=None, shift=0.0, seed=0):
    """Run sink_attn + talk_mix over portions and compare every row with the oracle. ``boost`` = (sequence, key
    position, factor): that key and the last query are scaled so that its score stands out."""
    pg = Paged(lens, G, d, dv, bs, device, dtype, seed)
    data = []
    for i, n in enumerate(lens):
        q, k, v = rnd(n, H, d, seed=seed + 3 * i + 1), rnd(n, G, d, seed=seed + 3 * i + 2, dtype=dtype), \
            rnd(n, G, dv, seed=seed + 3 * i + 3, dtype=dtype)
        if boost and boost[0] == i:  # the last two queries point along that key, which is made long
            for r in (-1, -2):
                q[r] = k[boost[1]].repeat_interleave(H // G, 0)
            k[boost[1]] *= boost[2]
        q = q + shift
        data.append((q, k, v))
    tk = (torch.eye(H).double() * 0.5 + 0.4 * rnd(H, H, seed=9)) if talk else None
    got = [torch.zeros(n, H * dv) for n in lens]
    for step in steps_of(cuts):
        step = sorted(step, key=lambda e: not (e[2] == 1 and e[1] > 0))  # single rows after a prefix come first
        nd = sum(1 for _, p0, n in step if n == 1 and p0 > 0)
        seqs = [s for s, _, _ in step]
        for s, p0, n in step:  # the step's keys and values are in the cache before it attends
            sl = torch.tensor(pg.slots(s, p0, n), device=device)
            pg.kc.view(-1, G * d)[sl] = data[s][1][p0:p0 + n].reshape(n, -1).to(dtype).to(device)
            pg.vc.view(-1, G * dv)[sl] = data[s][2][p0:p0 + n].reshape(n, -1).to(dtype).to(device)
        cu, ctx, _ = meta(step, [0] * len(lens), device)
        q = torch.cat([data[s][0][p0:p0 + n] for s, p0, n in step]).reshape(-1, H * d).float().to(device)
        O = ops.sink_attn(q, pg.kc, pg.vc, pg.bt(seqs, device), cu, ctx, H, G, d, dv, scale, cap, talk,
                          max_qlen=max(n for _, _, n in step), num_decode=nd)
        y = ops.talk_mix(O, tk.float().to(device).contiguous() if talk else None, 0.8, H, G, dv,
                         out_dtype=torch.float32).cpu()
        r = 0
        for s, p0, n in step:
            got[s][p0:p0 + n] = y[r:r + n]
            r += n
    for s, n in enumerate(lens):
        q, k, v = data[s]
        want = 0.8 * oracle.sink_talk_attention(q, k, v, scale, cap, tk).reshape(n, -1)
        close(got[s], want, dtype, f"sequence {s}", scale=float(v.abs().max()))
    return got, data


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("H,G,d,dv,talk", [(4, 2, 16, 12, True), (4, 4, 8, 20, True), (3, 1, 24, 40, False),
                                           (1, 1, 8, 8, True), (8, 2, 64, 72, True), (16, 2, 32, 8, False),
                                           (4, 2, 128, 64, True), (4, 1, 128, 40, False), (6, 2, 64, 160, True),
                                           (2, 2, 64, 128, False)])
def test_sink_attention_portions_decoding_and_batches(device, dtype, H, G, d, dv, talk):
    # key sizes 64 and 128 with value sizes in eights: in bf16 on a GPU the portions run on the matrix cores
    attention_case(device, dtype, H, G, d, dv, [70, 1, 33], [[16, 1, 15, 2, 1, 1, 30, 3, 1], [1], [2, 31]],
                   d ** -0.5, 30.0, talk)
    attention_case(device, dtype, H, G, d, dv, [150, 90], [[65, 64, 1, 20], [3, 87]], d ** -0.5, 0.0, talk, seed=7)


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("d", [16, 64])
@pytest.mark.parametrize("far", [0, 15, 16, 17, 63, 64, 200])
def test_a_far_key_among_hundreds_in_a_prompt_and_when_decoding(device, dtype, far, d):
    # the last query of the prompt portion and the decoded token both point at one key far back / at a page border
    H, G, dv, n = 2, 1, 8, 300
    got, data = attention_case(device, dtype, H, G, d, dv, [n], [[n - 1, 1]], 0.25, 0.0, False, boost=(0, far, 6.0),
                               seed=100 + far)
    q, k, v = data[0]
    s = (q[-1, 0] @ k[:, 0].T) * 0.25
    w = torch.exp(s) / (1 + torch.exp(s).sum())
    assert int(s.argmax()) == far and float(w[far]) > 0.9  # nearly all of the row's weight sits on that key
    assert float((got[0][-1].view(H, dv)[0].double() - 0.8 * v[far, 0]).abs().max()) < 0.15 * float(v.abs().max())


@pytest.mark.parametrize("device,dtype", RUNS)
def test_the_sink_takes_the_weight_when_every_score_is_low_and_the_cap_holds_high_scores(device, dtype):
    # scores around -40: without the unit in the denominator the weights would sum to one, with it they vanish
    H, G, d, dv = 2, 1, 8, 8
    pg = Paged([20], G, d, dv, 16, device, dtype)
    k = torch.ones(20, d).double()
    v = rnd(20, dv, seed=1, dtype=dtype)
    sl = torch.tensor(pg.slots(0, 0, 20), device=device)
    pg.kc.view(-1, d)[sl] = k.to(dtype).to(device)
    pg.vc.view(-1, dv)[sl] = v.to(dtype).to(device)
    cu, ctx = i32([0, 20], device), i32([20], device)
    q = torch.full((20, H * d), -5.0, device=device)
    O = ops.sink_attn(q, pg.kc, pg.vc, pg.bt([0], device), cu, ctx, H, G, d, dv, 1.0, 0.0, False).cpu()
    assert float(O.abs().max()) < 1e-12
    # scores of +400 are capped to just under 10: weights stay finite and nearly uniform over the visible keys
    q = torch.full((20, H * d), 50.0, device=device)
    O = ops.sink_attn(q, pg.kc, pg.vc, pg.bt([0], device), cu, ctx, H, G, d, dv, 1.0, 10.0, False).cpu()
    want = oracle.sink_talk_attention(torch.full((20, H, d), 50.0, dtype=F64), k.view(20, 1, d), v.view(20, 1, dv), 1.0,
                                      10.0, None)
    close(O.reshape(20, -1), want.reshape(20, -1), dtype, "capped scores")
    assert torch.isfinite(O).all()


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("H,G,d,dv", [(4, 2, 16, 12), (8, 1, 8, 40), (6, 2, 64, 72), (3, 3, 24, 8), (16, 4, 128, 128),
                                      (5, 1, 8, 8), (16, 2, 32, 300)])
def test_a_step_of_single_rows_mixes_heads_before_it_meets_the_values(device, dtype, H, G, d, dv):
    """Decoded rows only, one per sequence, contexts of unequal length (one of a single token): attention, head
    mixing and the scale in one op, written into a view of a wider buffer."""
    lens = [70, 33, 1, 129]
    pg = Paged(lens, G, d, dv, 16, device, dtype, seed=3)
    data = []
    for i, n in enumerate(lens):
        q, k, v = rnd(n, H, d, seed=50 + 3 * i), rnd(n, G, d, seed=51 + 3 * i, dtype=dtype), \
            rnd(n, G, dv, seed=52 + 3 * i, dtype=dtype)
        k[n // 2] *= 3.0  # one key stands out in the middle of each context
        sl = torch.tensor(pg.slots(i, 0, n), device=device)
        pg.kc.view(-1, G * d)[sl] = k.reshape(n, -1).to(dtype).to(device)
        pg.vc.view(-1, G * dv)[sl] = v.reshape(n, -1).to(dtype).to(device)
        data.append((q, k, v))
    tk = torch.eye(H).double() * 0.5 + 0.4 * rnd(H, H, seed=9)
    B = len(lens)
    q = torch.stack([data[i][0][-1] for i in range(B)]).reshape(B, H * d).float().to(device)
    out = torch.zeros(B, H * dv + 5, dtype=dtype, device=device)  # a view into a wider buffer, as the mixer passes
    ops.sink_attn_mix(q, pg.kc, pg.vc, pg.bt(list(range(B)), device), i32(list(range(B + 1)), device), i32(lens, device),
                      tk.float().to(device).contiguous(), 0.8, H, G, d, dv, d ** -0.5, 20.0, out[:, :H * dv],
                      max_qlen=1, num_decode=0, max_ctx=pg.maxb * 16)
    for i, n in enumerate(lens):
        qq, k, v = data[i]
        want = 0.8 * oracle.sink_talk_attention(qq, k, v, d ** -0.5, 20.0, tk)[-1].reshape(-1)
        close(out[i, :H * dv], want, dtype, f"sequence {i}", scale=float(v.abs().max()))
    assert float(out[:, H * dv:].float().abs().max()) == 0.0
