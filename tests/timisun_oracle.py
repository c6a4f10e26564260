"""Plain, slow definition of the Timisun design in fp64: one function per mechanism, whole sequences at once, no
cache, no batching, nothing shared with llmss_amd. The tests compare the framework (engine, scheduler, paged cache,
kernels) with it.

Notation: x residual [T, W]; h = normed x; c latent rows [T, R]; per head q, k [T, dim], v [T, vdim].
"""
import math

import torch


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    """RMS norm whose stored weight is the deviation from one."""
    return rms_unit(x, eps) * (1.0 + w)


def latent_rows(h, w_dkv, w_norm, eps):
    """The cached latent: down-projection, RMS norm with a plain weight."""
    return rms_unit(h @ w_dkv.T, eps) * w_norm


def visible(T, window):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window:
        ok = ok & (i - j < window)
    return ok


def latent_attention(h, c, w_q, w_uk, w_uv, w_o, heads, dim, vdim, scale, window):
    """Keys and values expanded from the latent rows c, ordinary softmax over the visible keys."""
    T = h.shape[0]
    q = (h @ w_q.T).view(T, heads, dim)
    k = (c @ w_uk.T).view(T, heads, dim)
    v = (c @ w_uv.T).view(T, heads, vdim)
    ok = visible(T, window)
    out = torch.zeros(T, heads, vdim, dtype=h.dtype)
    for hd in range(heads):
        s = (q[:, hd] @ k[:, hd].T) * scale
        s = s.masked_fill(~ok, -math.inf)
        out[:, hd] = torch.softmax(s, -1) @ v[:, hd]
    return out.reshape(T, heads * vdim) @ w_o.T


def expert(h, w_gate, w_up, w_down, limit):
    g = torch.clamp(h @ w_gate.T, max=limit)
    u = torch.clamp(h @ w_up.T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w_down.T


def route(h, w_router, correction, top):
    """(chosen experts [T, top], their weights [T, top])."""
    s = torch.sigmoid(h @ w_router.T)
    chosen = torch.topk(s + correction, top, dim=-1).indices
    w = torch.gather(s, 1, chosen)
    return chosen, w / (w.sum(-1, keepdim=True) + 1e-20)


def route_margin(h, w_router, correction, top):
    """How far the last chosen expert's choice score lies above the first one left out, per token (inf when every
    expert is chosen): rows with a tiny margin are close calls that rounding may decide either way."""
    ch = torch.sort(torch.sigmoid(h @ w_router.T) + correction, dim=-1, descending=True).values
    if top >= ch.shape[1]:
        return torch.full((h.shape[0],), math.inf, dtype=h.dtype)
    return ch[:, top - 1] - ch[:, top]


def moe(h, sd, p, spec):
    chosen, w = route(h, sd[p + "router"], sd[p + "correction"], spec["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(chosen.shape[1]):
            e = int(chosen[t, j])
            out[t] += w[t, j] * expert(h[t:t + 1], sd[f"{p}e{e}.gate"], sd[f"{p}e{e}.up"], sd[f"{p}e{e}.down"],
                                       spec["expert"]["limit"])[0]
    if spec.get("shared"):
        out = out + expert(h, sd[p + "shared.gate"], sd[p + "shared.up"], sd[p + "shared.down"],
                           spec["shared"]["limit"])
    return out


def forward(cfg, sd, tokens, margins=None):
    """cfg: the config.json dict; sd: name -> tensor. Returns (logits [T, V], [residual after each layer]); a list
    given as ``margins`` receives every feed-forward's route_margin."""
    sd = {k: v.double() for k, v in sd.items()}
    eps = cfg["norm"]["eps"]
    x = sd["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    latents, stream = {}, []
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = norm_around_zero(x, sd[p + "norm1"], eps)
        if m.get("kv_from") is None:
            latents[i] = latent_rows(h, sd[p + "mix.dkv"], sd[p + "mix.dkv.norm"], eps)
            c = latents[i]
        else:
            c = latents[m["kv_from"]]
        window = (m.get("mask") or {}).get("size") or 0
        a = latent_attention(h, c, sd[p + "mix.q"], sd[p + "mix.uk"], sd[p + "mix.uv"], sd[p + "mix.o"], m["heads"],
                             m["dim"], m["vdim"], m["scale"], window)
        f = moe(h, sd, p + "mlp.", L["mlp"]) if L.get("mlp") else torch.zeros_like(x)
        if margins is not None and L.get("mlp"):
            margins.append(route_margin(h, sd[p + "mlp.router"], sd[p + "mlp.correction"], L["mlp"]["router"]["top"]))
        x = x + (a + f)
        stream.append(x.clone())
    return norm_around_zero(x, sd["final.norm"], eps) @ sd["embed"].T, stream


def greedy(cfg, sd, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, sd, toks)[0][-1].argmax()))
    return toks[len(prompt):]
