"""A plain, slow implementation of the Duperax decoder: float64, whole sequences at once, one function
per mechanism, nothing shared with the package.  The GPU tests compare the engine with it.

Notation: rows are tokens; ``i`` is a query's position, ``j`` a key's; ``x_1 .. x_S`` are the residual streams.

* layer norm        ``ln(x) = (x - mean x) / sqrt(mean (x - mean x)^2 + eps) * w + b``
* streams           sublayer q of a layer reads ``u = sum_s in_q[s] x_s`` and writes, for every t at once,
                    ``x_t <- sum_s mix_q[s, t] x_s + out_q[t] f(ln(u))``; all streams start as the embedding row and
                    their sum enters the final norm.  Without streams: ``x <- x + f(ln(x))``.
* run order         layers ``start .. stop - 1`` run ``times`` times in a row (own cache and state each time)
* row norm          q and k are divided by the root mean square of their whole row (all heads side by side), times a weight
* attention         ``scale * q.k`` over ``0 <= i - j < window``; no rotation
* attention_2       biases on q, k, v; rotation of the first ``dims`` elements of a head (pairs ``(e, e + dims/2)``)
                    with YaRN's frequencies and magnitude; ``cap * tanh(scale * q.k / cap)``; ``j <= i`` in i's chunk
* rglru             ``y = gelu(W_y h + b)``, ``u = conv(W_x h + b)``; per block of channels ``r = sigmoid(A_r u + b_r)``,
                    ``g = sigmoid(A_i u + b_i)``; ``a = exp(-8 r softplus(lam))``; ``S <- a S + sqrt(1 - a^2) g u``; ``W_o (S y)``
* dense ff          ``g = min(W_g h, L)``, ``v = clamp(W_u h, -L, L)``, ``W_d (g sigmoid(1.702 g) (v + 1))``
* routed ff         ``s = sigmoid(W_r h)``; choice by ``s + correction`` inside the best groups (a group counts by the sum
                    of its two largest choice scores); weights ``s / (sum of the chosen s + 1e-20)``
"""
import math
from typing import Dict, List, Optional, Sequence

import torch

F = torch.float64


# ---------------------------------------------------------------- configurations
def attention_layer(heads, kv_heads, dim, vdim, window, scale=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window},
         "scale": scale if scale is not None else dim ** -0.5}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def attention2_layer(heads, kv_heads, dim, vdim, chunk, rot_dims, base=10000.0, factor=4.0, original=64, fast=32.0, slow=1.0,
                     softcap=20.0, scale=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": chunk},
         "rot": {"base": base, "dims": rot_dims, "scaling": {"factor": factor, "original": original, "fast": fast, "slow": slow}},
         "scale": scale if scale is not None else dim ** -0.5, "softcap": softcap}
    return {"type": "attention_2", "mixer": m, "mlp": mlp}


def rglru_layer(width, blocks, taps, mlp=None):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": taps}, "mlp": mlp}


def dense(ff, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, top, groups, keep, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}


def config(layers, vocab=97, width=64, eps=1e-5, streams: Optional[int] = 3, loop=None, logit_scale=0.7):
    cfg = {"architecture": "Duperax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers,
           "logit_scale": logit_scale}
    if streams is not None:
        cfg["streams"] = streams
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    e, out = cfg["width"], {}
    out["embed"] = (cfg["vocab"], e)
    s = cfg.get("streams")
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        for n in ("norm1", "norm2") if layer["mlp"] is not None else ("norm1",):
            out[p + n] = (e,)
            out[p + n + ".b"] = (e,)
        if s is not None:
            for q in ("hc1", "hc2") if layer["mlp"] is not None else ("hc1",):
                out[p + q + ".in"], out[p + q + ".out"], out[p + q + ".mix"] = (s,), (s,), (s, s)
        if layer["type"] in ("attention", "attention_2"):
            qd, kd, vd = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            out[p + "mix.q"], out[p + "mix.k"], out[p + "mix.v"] = (qd, e), (kd, e), (vd, e)
            out[p + "mix.q.norm"], out[p + "mix.k.norm"] = (qd,), (kd,)
            out[p + "mix.o"] = (e, m["heads"] * m["vdim"])
            if layer["type"] == "attention_2":
                out[p + "mix.q.b"], out[p + "mix.k.b"], out[p + "mix.v.b"] = (qd,), (kd,), (vd,)
        else:
            w, nb = m["width"], m["blocks"]
            out[p + "mix.y"], out[p + "mix.y.b"], out[p + "mix.x"], out[p + "mix.x.b"] = (w, e), (w,), (w, e), (w,)
            out[p + "mix.conv"], out[p + "mix.conv.b"] = (w, m["conv"]), (w,)
            for g in ("ra", "ri"):
                out[p + "mix." + g], out[p + "mix." + g + ".b"] = (nb, w // nb, w // nb), (nb, w // nb)
            out[p + "mix.lam"], out[p + "mix.o"] = (w,), (e, w)
        f = layer["mlp"]
        if f is None:
            continue
        if f["kind"] == "dense":
            out[p + "mlp.gate"], out[p + "mlp.up"], out[p + "mlp.down"] = (f["ff"], e), (f["ff"], e), (e, f["ff"])
        else:
            ff = f["expert"]["ff"]
            for x in range(f["router"]["experts"]):
                out[p + f"mlp.e{x}.gate"], out[p + f"mlp.e{x}.up"], out[p + f"mlp.e{x}.down"] = (ff, e), (ff, e), (e, ff)
            out[p + "mlp.router"], out[p + "mlp.correction"] = (f["router"]["experts"], e), (f["router"]["experts"],)
    out["final.norm"], out["final.norm.b"], out["head"] = (e,), (e,), (cfg["vocab"], e)
    return out


def random_weights(cfg: dict, seed: int, matrix_std: Optional[float] = None, decided_routing: bool = False) -> Dict[str, torch.Tensor]:
    """Weights that keep activations of order one through many layers, rounded to bfloat16 values (so that a
    bfloat16 checkpoint holds exactly these numbers).  ``decided_routing``: the corrections of the routers are
    different powers of two (no two pairs of them have the same sum, so groups do not tie either), so that no rounding
    of a score changes which experts are chosen."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name.endswith(".b"):
            t = 0.1 * torch.randn(shape, generator=g, dtype=F)
        elif last in ("norm1", "norm2") or name in ("final.norm", "mix.q.norm") or name.endswith(".norm"):
            t = 1.0 + 0.1 * torch.randn(shape, generator=g, dtype=F)
        elif last == "in":
            t = 1.0 / shape[0] + 0.2 * torch.randn(shape, generator=g, dtype=F)
        elif last == "out":
            t = 1.0 + 0.3 * torch.randn(shape, generator=g, dtype=F)
        elif last == "mix" and ".hc" in name:
            t = torch.eye(shape[0], dtype=F) + 0.15 * torch.randn(shape, generator=g, dtype=F)
        elif last == "lam":
            t = torch.randn(shape, generator=g, dtype=F) - 1.0
        elif last == "correction":
            t = 0.2 * torch.randn(shape, generator=g, dtype=F)
            if decided_routing:
                t = 0.5 * 2.0 ** torch.randperm(shape[0], generator=g).to(F)
        elif last == "conv":
            t = 0.5 * torch.randn(shape, generator=g, dtype=F)
        elif name == "embed":
            t = torch.randn(shape, generator=g, dtype=F)
        else:
            std = matrix_std if matrix_std is not None else 1.0 / math.sqrt(shape[-1])
            t = std * torch.randn(shape, generator=g, dtype=F)
        out[name] = t.to(torch.bfloat16).to(F)
    return out


# ---------------------------------------------------------------- mechanisms
def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def row_rms(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the whole row (all heads side by side)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def streams_read(xs, read):
    """u = sum_s read[s] x_s for streams xs [S, T, E]."""
    return torch.einsum("s,ste->te", read, xs)


def streams_write(xs, y, mix, write):
    """x_t <- sum_s mix[s, t] x_s + write[t] y, all t at once."""
    return torch.einsum("st,sne->tne", mix, xs) + write[:, None, None] * y[None]


def run_order(cfg: dict) -> List[int]:
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, t = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * t + list(range(b, n))


def yarn_frequencies(rot: dict):
    """(frequency per pair, factor on sine and cosine)."""
    dims, base = rot["dims"], rot["base"]
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F), 1.0

    def where(t):
        return dims * math.log(sc["original"] / (2.0 * math.pi * t)) / (2.0 * math.log(base))
    lo, hi = max(math.floor(where(sc["fast"])), 0), min(math.ceil(where(sc["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / sc["factor"] * ramp + fi * (1.0 - ramp))
    return torch.tensor(out, dtype=F), 0.1 * math.log(sc["factor"]) + 1.0


def rotate(x, positions, rot: dict):
    """x [T, heads, dim]: the first ``dims`` elements of every head, pairs (e, e + dims/2)."""
    dims = rot["dims"]
    freq, mag = yarn_frequencies(rot)
    ang = positions.to(F)[:, None] * freq[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    a, b = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], -1)


def visible(kind: str, size: int, T: int):
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    if kind == "attention":
        return (j <= i) & (i - j < size)
    return (j <= i) & (i // size == j // size)


def attention(h, w, p, m, kind, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ w[p + "q"].T, h @ w[p + "k"].T, h @ w[p + "v"].T
    if kind == "attention_2":
        q, k, v = q + w[p + "q.b"], k + w[p + "k.b"], v + w[p + "v.b"]
    q, k = row_rms(q, w[p + "q.norm"], eps), row_rms(k, w[p + "k.norm"], eps)
    q, k, v = q.view(T, H, d), k.view(T, G, d), v.view(T, G, dv)
    if kind == "attention_2":
        pos = torch.arange(T)
        q, k = rotate(q, pos, m["rot"]), rotate(k, pos, m["rot"])
    see = visible(kind, m["mask"]["size"], T) if m.get("mask") else visible("attention", T, T)
    cap = m.get("softcap") if kind == "attention_2" else None
    return softmax_attention(q, k, v, m["scale"], see, cap).reshape(T, H * dv) @ w[p + "o"].T


def softmax_attention(q, k, v, scale, see, softcap=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; head h reads key head h // (H / G); ``see`` [T, T] says which keys a
    query sees.  Returns [T, H, dv]."""
    T, H, G = q.shape[0], q.shape[1], k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~see, -math.inf)
        out[:, hh] = torch.softmax(s, -1) @ v[:, g]
    return out


def causal_conv(x, taps_w, bias):
    """x [T, C]; taps_w [C, taps], the last column is the current token's; zeros before the start."""
    T, taps = x.shape[0], taps_w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=F), x], 0)
    out = torch.zeros_like(x)
    for j in range(taps):
        out += pad[j:j + T] * taps_w[:, j]
    return out + bias


def rglru_gates(u, w_r, b_r, w_i, b_i, lam, c=8.0):
    """(a, gated input) from the convolved branch u [T, W]; the gate matrices are [blocks, out, in]."""
    T, nb = u.shape[0], w_r.shape[0]
    ub = u.view(T, nb, -1)
    r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w_r) + b_r).reshape(T, -1)
    g = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w_i) + b_i).reshape(T, -1)
    a = torch.exp(-c * r * torch.nn.functional.softplus(lam))
    return a, torch.sqrt(1.0 - a ** 2) * g * u


def linear_scan(a, x):
    """S_t = a_t S_(t-1) + x_t from S = 0; all S_t [T, W]."""
    S = torch.zeros(a.shape[1], dtype=F)
    out = torch.zeros_like(x)
    for t in range(a.shape[0]):
        S = a[t] * S + x[t]
        out[t] = S
    return out


def rglru(h, w, p, m):
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u = causal_conv(h @ w[p + "x"].T + w[p + "x.b"], w[p + "conv"], w[p + "conv.b"])
    a, x = rglru_gates(u, w[p + "ra"], w[p + "ra.b"], w[p + "ri"], w[p + "ri.b"], w[p + "lam"])
    return (linear_scan(a, x) * y) @ w[p + "o"].T


def dense_ff(h, w, p, f):
    L = f["limit"]
    g = torch.clamp(h @ w[p + "gate"].T, max=L)
    u = torch.clamp(h @ w[p + "up"].T, -L, L)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def route(h, w, p, f):
    """(chosen experts [T, top], their weights [T, top])."""
    r = f["router"]
    E, top = r["experts"], r["top"]
    groups, keep = (r["groups"]["count"], r["groups"]["keep"]) if r.get("groups") else (1, 1)
    s = torch.sigmoid(h @ w[p + "router"].T)
    c = s + w[p + "correction"]
    gs = E // groups
    gscore = c.view(-1, groups, gs).topk(min(2, gs), -1).values.sum(-1)
    open_g = torch.zeros_like(gscore, dtype=torch.bool)
    open_g.scatter_(1, gscore.topk(keep, -1).indices, True)
    c = c.masked_fill(~open_g.repeat_interleave(gs, 1), -math.inf)
    idx = c.topk(top, -1).indices
    sw = s.gather(1, idx)
    return idx, sw / (sw.sum(-1, keepdim=True) + 1e-20)


def routed_ff(h, w, p, f):
    idx, wt = route(h, w, p, f)
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), wt[t]):
            z = h[t] @ w[p + f"e{e}.gate"].T
            out[t] += a * ((z * torch.sigmoid(z) * (h[t] @ w[p + f"e{e}.up"].T)) @ w[p + f"e{e}.down"].T)
    return out


def mixer(h, w, i, layer, eps):
    p = f"l{i}.mix."
    if layer["type"] == "rglru":
        return rglru(h, w, p, layer["mixer"])
    return attention(h, w, p, layer["mixer"], layer["type"], eps)


def feed_forward(h, w, i, layer):
    p, f = f"l{i}.mlp.", layer["mlp"]
    return dense_ff(h, w, p, f) if f["kind"] == "dense" else routed_ff(h, w, p, f)


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: Sequence[int], layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  ``layers_out`` receives the residual stream (the streams' sum) after every
    layer run."""
    w = {k: v.to(F) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    S = cfg.get("streams")
    x = w["embed"][torch.tensor(list(tokens))]
    xs = x[None].repeat(S, 1, 1) if S is not None else None             # [S, T, E]
    for i in run_order(cfg):
        layer = cfg["layers"][i]
        subs = [(1, lambda h: mixer(h, w, i, layer, eps))]
        if layer["mlp"] is not None:
            subs.append((2, lambda h: feed_forward(h, w, i, layer)))
        for q, fn in subs:
            nw, nb = w[f"l{i}.norm{q}"], w[f"l{i}.norm{q}.b"]
            if S is None:
                x = x + fn(layer_norm(x, nw, nb, eps))
            else:
                hc = f"l{i}.hc{q}."
                y = fn(layer_norm(streams_read(xs, w[hc + "in"]), nw, nb, eps))
                xs = streams_write(xs, y, w[hc + "mix"], w[hc + "out"])
        if layers_out is not None:
            layers_out.append((xs.sum(0) if S is not None else x).clone())
    if S is not None:
        x = xs.sum(0)
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    return (x @ w["head"].T) * cfg.get("logit_scale", 1.0)


def argmax_first(row) -> int:
    """The first index of the largest value."""
    return int((row == row.max()).nonzero()[0])
