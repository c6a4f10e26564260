"""Plain definition of the Babotar design in float64: one function per mechanism, whole sequences, no cache, no
batching, nothing shared with the product path. ``forward`` takes the raw config dictionary and a name -> tensor
dictionary under the checkpoint's names and returns the logits of every position and the residual stream after
every layer."""
import math

import torch

F64 = torch.float64


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w


def rms_div(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def causal_conv(h, w):
    """h [T, C], w [C, taps]; column taps - 1 multiplies the current row, column 0 the row taps - 1 back."""
    T, C = h.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def rotary_tables(rot, T):
    """cos / sin [T, dims / 2] of a rotary description {base, dims, scaling: {factor, original, fast, slow}}."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    amp = 1.0
    sc = rot.get("scaling")
    if sc:
        factor = float(sc["factor"])

        def turn_dim(turns):
            return dims * math.log(float(sc["original"]) / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
        hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
        ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=F64)
        f = f / factor * ramp + f * (1.0 - ramp)
        amp = 0.1 * math.log(factor) + 1.0
    ang = torch.arange(T, dtype=F64)[:, None] * f[None, :]
    return torch.cos(ang) * amp, torch.sin(ang) * amp


def rotate(x, cos, sin, dims):
    """x [T, heads, dim]: the first ``dims`` dimensions of each head turn, pairing i with i + dims / 2."""
    half = dims // 2
    a, b = x[..., :half], x[..., half:dims]
    c, s = cos[:, None, :], sin[:, None, :]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], -1)


def sink_talk_attention(q, k, v, scale, softcap, talk):
    """q [T, H, d], k [T, G, d], v [T, G, dv]. Causal scores, optionally soft-capped; softmax whose denominator
    holds one extra unit; the heads' weights mixed by ``talk`` [H, H]; head h reads the values of its own group."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    P = torch.zeros(H, T, T, dtype=F64)
    for h in range(H):
        s = (q[:, h] @ k[:, h // rep].T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        e = torch.exp(s) * torch.tril(torch.ones(T, T, dtype=F64))
        P[h] = e / (1.0 + e.sum(-1, keepdim=True))
    if talk is not None:
        P = torch.einsum("hg,gij->hij", talk, P)
    return torch.stack([P[h] @ v[:, h // rep] for h in range(H)], 1)  # [T, H, dv]


def lightning_scan(q, k, v, decay):
    """Per head S <- decay_h S + k v^T, o = S^T q. q, k [T, H, d], v [T, H, dv]."""
    T, H, d = q.shape
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        S = torch.zeros(d, v.shape[2], dtype=F64)
        for t in range(T):
            S = decay[h] * S + torch.outer(k[t, h], v[t, h])
            out[t, h] = S.T @ q[t, h]
    return out


def delta_scan(q, k, v, beta, g):
    """Per head S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q. q, k [T, G, d], v [T, H, dv]."""
    T, H, dv = v.shape
    G, d = q.shape[1], q.shape[2]
    rep = H // G
    out = torch.zeros(T, H, dv, dtype=F64)
    for h in range(H):
        S = torch.zeros(d, dv, dtype=F64)
        for t in range(T):
            kk, qq = k[t, h // rep], q[t, h // rep]
            S = g[t, h] * S
            u = beta[t, h] * (v[t, h] - S.T @ kk)
            S = S + torch.outer(kk, u)
            out[t, h] = S.T @ qq
    return out


def mixer_lightning(h, W, p, m, eps):
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = silu(h @ W[p + "q"].T).view(T, H, d)
    k = silu(h @ W[p + "k"].T).view(T, H, d)
    v = silu(h @ W[p + "v"].T).view(T, H, dv)
    o = lightning_scan(q, k, v, [float(x) for x in m["decay"]]).reshape(T, H * dv)
    o = rms_div(o, eps) * W[p + "norm"] * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def softmax_branch(h, W, p, m):
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]

    def proj(n):
        y = h @ W[p + n].T
        return y + W[p + n + ".b"] if p + n + ".b" in W else y
    q, k, v = proj("q").view(T, H, d), proj("k").view(T, G, d), proj("v").view(T, G, dv)
    rot = m.get("rot")
    if rot:
        cos, sin = rotary_tables(rot, T)
        q, k = rotate(q, cos, sin, int(rot["dims"])), rotate(k, cos, sin, int(rot["dims"]))
    o = sink_talk_attention(q, k, v, float(m["scale"]), float(m.get("softcap") or 0.0), W.get(p + "talk"))
    return o.reshape(T, H * dv) @ W[p + "o"].T


def delta_branch(h, W, p, m, eps):
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]

    def short(n):
        return silu(causal_conv(h @ W[p + n].T, W[p + n + ".conv"]))
    q, k, v = short("q").view(T, G, d), short("k").view(T, G, d), short("v").view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    g = torch.exp(-torch.exp(W[p + "A_log"]) * torch.nn.functional.softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    o = delta_scan(q, k, v, beta, g)  # [T, H, dv]
    o = rms_div(o, eps) * W[p + "norm"] * silu(h @ W[p + "g"].T).view(T, H, dv)
    return o.reshape(T, H * dv) @ W[p + "o"].T


def mixer_parallel(h, W, p, m, eps):
    left = softmax_branch(h, W, p + "left.", m["left"])
    right = delta_branch(h, W, p + "right.", m["right"], eps)
    return float(m.get("left_scale", 1.0)) * left + float(m.get("right_scale", 1.0)) * right


def feed_forward(h, W, p):
    return (gelu_tanh(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def forward(cfg, W, tokens):
    W = {k: v.to(F64) for k, v in W.items()}
    eps = float(cfg["norm"]["eps"])
    mult = float(cfg.get("residual_mult", 1.0))
    S = int(cfg.get("streams") or 0)
    T = len(tokens)
    x0 = W["embed"][torch.tensor(tokens)]
    if "pos" in W:
        x0 = x0 + W["pos"][:T]
    xs = [x0.clone() for _ in range(max(S, 1))]
    after = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        for q in (1, 2):
            if q == 2 and L.get("mlp") is None:
                continue
            hc = f"{p}hc{q}."
            u = sum(W[hc + "in"][s] * xs[s] for s in range(S)) if S else xs[0]
            h = layer_norm(u, W[f"{p}norm{q}"], eps)
            if q == 1:
                if cfg.get("canon"):
                    h = h + causal_conv(h, W[p + "canon1"])
                if L["type"] == "lightning":
                    y = mixer_lightning(h, W, p + "mix.", L["mixer"], eps)
                elif L["type"] == "parallel":
                    y = mixer_parallel(h, W, p + "mix.", L["mixer"], eps)
                else:
                    raise ValueError(L["type"])
            else:
                y = feed_forward(h, W, p + "mlp.")
            if S:
                xs = [sum(W[hc + "mix"][s, t] * xs[s] for s in range(S)) + mult * W[hc + "out"][t] * y
                      for t in range(S)]
            else:
                xs = [xs[0] + mult * y]
        after.append(sum(xs))
    x = layer_norm(sum(xs), W["final.norm"], eps)
    return x @ W["head"].T, torch.stack(after)


def greedy(cfg, W, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(forward(cfg, W, seq)[0][-1].argmax()))
    return seq[len(prompt):]
