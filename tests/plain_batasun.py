"""A plain, slow implementation of the Batasun decoder: float64, whole sequences at once, one function
per mechanism, nothing shared with the package.  The GPU tests compare the engine with it.

Notation: rows are tokens; ``i`` is a query's position, ``j`` a key's.

* norm              ``rms(x) = x / sqrt(mean x^2 + eps)``; a layer's and the model's norms multiply by ``1 + w``,
                    the norms of the latents by ``w``
* model             ``x = rms(embed[token]) (1 + w_e)``; layers; ``logits = head (rms(x) (1 + w_f))``
* a layer           ``x += rms(mix(x)) (1 + w1);  x += rms(ff(x)) (1 + w2)``: no norm in front of a sublayer
* latent attention  ``cq = rms(W_dq x) w``, ``q = W_uq cq`` (per head ``dim`` plain and ``rot`` rotated elements);
                    ``W_dkv x = [c' | r]``, ``c = rms(c') w``, ``r`` rotated, one for all heads; head h's key is
                    ``[W_uk,h c | r]``, its value ``W_uv,h c``; causal softmax of ``scale q.k``; heads side by side
                    times ``sigmoid(W_g x)``; ``W_o``.  A layer with ``kv_from`` reads that layer's ``c`` and ``r``.
* rotation          element e < dims/2 pairs with e + dims/2; angle ``p base^(-2e/dims)``;
                    ``(u, v) -> (u cos - v sin, v cos + u sin)``
* mamba2            ``W_in x = [z | xs | B | C | dt]``; ``xs, B, C`` pass a causal convolution over time (bias, SiLU);
                    ``dt = softplus(dt + dt_bias)``; per head, with its group's B and C:
                    ``S <- exp(-exp(A_log) dt) S + dt B xs^T``, ``y = S^T C + D xs``; ``y silu(z)`` is divided by its root
                    mean square in ``norm_groups`` equal parts, times a weight; ``W_o``
* expert            ``g = min(W_gate x, L)``, ``u = clamp(W_up x, -L, L)``, ``W_down (g sigmoid(1.702 g) (u + 1))``
* routed ff         logits ``W_r x + b``; the ``top`` largest are chosen, weights = softmax over the chosen logits; a
                    shared expert of the same form times ``sigmoid(w_sg . x)`` is added
"""
import math
from typing import Dict, List, Optional, Sequence

import torch

F = torch.float64
SWISH = 1.702


# ---------------------------------------------------------------- configurations
def moe(experts, top, ff, limit, shared_ff=None, shared_limit=None):
    out = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if shared_ff is not None:
        out["shared"] = {"ff": shared_ff, "limit": shared_limit if shared_limit is not None else limit}
    return out


def latent_layer(heads, dim, rot_dim, vdim, q_rank, kv_rank, base=10000.0, scale=None, kv_from=None, mlp=None, rot_dims=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "rot": {"base": base, "dims": rot_dims if rot_dims is not None else rot_dim}, "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def mamba_layer(heads, vdim, state, groups, conv, norm_groups, mlp=None):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}, "mlp": mlp}


def config(layers, vocab=97, width=64, eps=1e-5):
    return {"architecture": "Batasun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


def tensor_shapes(cfg) -> Dict[str, tuple]:
    e, out = cfg["width"], {}
    out["embed"], out["embed.norm"], out["final.norm"], out["head"] = (cfg["vocab"], e), (e,), (e,), (cfg["vocab"], e)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (e,)
        if layer["type"] == "latent_attention":
            H, qd = m["heads"], m["dim"] + m["rot_dim"]
            out[p + "mix.dq"], out[p + "mix.dq.norm"], out[p + "mix.uq"] = (m["q_rank"], e), (m["q_rank"],), (H * qd, m["q_rank"])
            if m.get("kv_from") is None:
                out[p + "mix.dkv"], out[p + "mix.dkv.norm"] = (m["kv_rank"] + m["rot_dim"], e), (m["kv_rank"],)
            out[p + "mix.uk"], out[p + "mix.uv"] = (H * m["dim"], m["kv_rank"]), (H * m["vdim"], m["kv_rank"])
            out[p + "mix.g"], out[p + "mix.o"] = (H * m["vdim"], e), (e, H * m["vdim"])
        else:
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            ch = inner + 2 * gn
            out[p + "mix.in"] = (2 * inner + 2 * gn + m["heads"], e)
            out[p + "mix.conv"], out[p + "mix.conv.b"] = (ch, m["conv"]), (ch,)
            for n in ("dt_bias", "A_log", "D"):
                out[p + "mix." + n] = (m["heads"],)
            out[p + "mix.norm"], out[p + "mix.o"] = (inner,), (e, inner)
        f = layer["mlp"]
        if f is not None:
            out[p + "norm2"] = (e,)
            q = p + "mlp."
            for k in range(f["router"]["experts"]):
                out[q + f"e{k}.gate"], out[q + f"e{k}.up"], out[q + f"e{k}.down"] = (f["expert"]["ff"], e), (f["expert"]["ff"], e), (e, f["expert"]["ff"])
            out[q + "router"], out[q + "router.b"] = (f["router"]["experts"], e), (f["router"]["experts"],)
            if f.get("shared") is not None:
                s = f["shared"]["ff"]
                out[q + "shared.gate"], out[q + "shared.up"], out[q + "shared.down"], out[q + "shared.sg"] = (s, e), (s, e), (e, s), (1, e)
    return out


def random_weights(cfg, seed=0, decided_routing=False) -> Dict[str, torch.Tensor]:
    """Weights rounded to bfloat16 (so that a bfloat16 folder holds exactly these).  Matrices are drawn so that a
    row's product with a vector of unit root mean square has about unit size; ``decided_routing``: the router's bias
    spreads the experts apart and its matrix is small, so that rounding never changes the choice."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        if len(shape) == 2 and last != "conv":
            t = torch.randn(shape, generator=g, dtype=F) / math.sqrt(shape[1])
            if last in ("embed", "head"):
                t = torch.randn(shape, generator=g, dtype=F) * (1.0 if last == "embed" else 1.0 / math.sqrt(shape[1]))
        elif last == "conv":
            t = torch.randn(shape, generator=g, dtype=F) * 0.5
        elif last == "A_log":
            t = torch.log(torch.rand(shape, generator=g, dtype=F) * 1.5 + 0.05)
        elif last == "dt_bias":
            t = torch.randn(shape, generator=g, dtype=F) * 0.7 - 2.0
        elif last == "D":
            t = torch.randn(shape, generator=g, dtype=F) * 0.5 + 1.0
        elif name.endswith("router.b"):
            t = torch.randn(shape, generator=g, dtype=F) * 0.3
            if decided_routing:
                t = torch.arange(shape[0], dtype=F)[torch.randperm(shape[0], generator=g)] * 0.7
        elif name.endswith("conv.b"):
            t = torch.randn(shape, generator=g, dtype=F) * 0.2
        elif name.endswith("dq.norm") or name.endswith("dkv.norm") or name.endswith("mix.norm"):
            t = 1.0 + torch.randn(shape, generator=g, dtype=F) * 0.2          # plain weights
        else:
            t = torch.randn(shape, generator=g, dtype=F) * 0.2                # weights stored around zero
        if decided_routing and name.endswith("mlp.router"):
            t = t * 0.02
        w[name] = t.to(torch.bfloat16).to(F)
    return w


# ---------------------------------------------------------------- mechanisms
def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rotate(x, positions, base, dims):
    """x [T, ..., d]: the first ``dims`` elements of the last axis turn, the rest pass."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * e / dims) for e in range(half)], dtype=F)
    a = torch.as_tensor(positions, dtype=F)[:, None] * f[None, :]            # [T, half]
    while a.dim() < x.dim():
        a = a.unsqueeze(1)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * torch.cos(a) - v * torch.sin(a), v * torch.cos(a) + u * torch.sin(a), x[..., dims:]], -1)


def causal_softmax_attention(q, k, v, scale):
    """q, k [T, H, d], v [T, H, dv] -> [T, H, dv]."""
    T = q.shape[0]
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    s = s.masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool)), -math.inf)
    return torch.einsum("hij,jhd->ihd", torch.softmax(s, -1), v)


def latent_attention(m, w, p, x, eps, shared):
    """``shared``: {layer: (c, r)} as the layers with a projection of their own left them."""
    T, H, d, rd, vd = x.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    pos = list(range(T))
    cq = rms(x @ w[p + "dq"].T, eps) * w[p + "dq.norm"]
    q = (cq @ w[p + "uq"].T).view(T, H, d + rd)
    q = torch.cat([q[..., :d], rotate(q[..., d:], pos, m["rot"]["base"], m["rot"]["dims"])], -1)
    if m.get("kv_from") is None:
        ckv = x @ w[p + "dkv"].T
        c = rms(ckv[:, :m["kv_rank"]], eps) * w[p + "dkv.norm"]
        r = rotate(ckv[:, m["kv_rank"]:], pos, m["rot"]["base"], m["rot"]["dims"])
    else:
        c, r = shared[m["kv_from"]]
    k = torch.cat([(c @ w[p + "uk"].T).view(T, H, d), r[:, None, :].expand(T, H, rd)], -1)
    v = (c @ w[p + "uv"].T).view(T, H, vd)
    o = causal_softmax_attention(q, k, v, m["scale"]).reshape(T, H * vd)
    return (o * torch.sigmoid(x @ w[p + "g"].T)) @ w[p + "o"].T, (c, r)


def causal_conv(u, taps, bias):
    """u [T, C], taps [C, K] (the last column is the current token's), zeros before the start."""
    T, K = u.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, u.shape[1], dtype=F), u], 0)
    out = bias[None, :].expand(T, -1).clone()
    for j in range(K):
        out = out + padded[j:j + T] * taps[:, j][None, :]
    return out


def silu(x):
    return x * torch.sigmoid(x)


def state_space_steps(xs, B, C, dt, rate, skip):
    """xs [T, H, P], B and C [T, G, N] (head h reads group h // (H / G)), dt [T, H] (already positive), rate and skip
    [H]:  S_t = exp(-rate dt) S_(t-1) + dt B_t xs_t^T,  y_t = S_t^T C_t + skip xs_t.  Returns (y [T, H, P], the last
    states [H, N, P])."""
    T, H, P_ = xs.shape
    G, N = B.shape[1], B.shape[2]
    y = torch.zeros(T, H, P_, dtype=F)
    last = torch.zeros(H, N, P_, dtype=F)
    for h in range(H):
        g = h // (H // G)
        S = torch.zeros(N, P_, dtype=F)
        for t in range(T):
            S = torch.exp(-rate[h] * dt[t, h]) * S + dt[t, h] * torch.outer(B[t, g], xs[t, h])
            y[t, h] = S.T @ C[t, g] + skip[h] * xs[t, h]
        last[h] = S
    return y, last


def gated_norm_in_parts(y, z, weight, parts, eps):
    """y silu(z), each of the row's ``parts`` equal parts divided by its own root mean square, times ``weight``."""
    T, width = y.shape
    g = y * silu(z)
    return rms(g.view(T, parts, width // parts), eps).reshape(T, width) * weight


def mamba2(m, w, p, x, eps):
    T, H, P_, N, G = x.shape[0], m["heads"], m["vdim"], m["state"], m["groups"]
    inner, gn = H * P_, G * N
    proj = x @ w[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * gn], proj[:, 2 * inner + 2 * gn:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    xs, B, C = xbc[:, :inner].view(T, H, P_), xbc[:, inner:inner + gn].view(T, G, N), xbc[:, inner + gn:].view(T, G, N)
    dt = torch.nn.functional.softplus(dt + w[p + "dt_bias"], threshold=1e9)
    y, _ = state_space_steps(xs, B, C, dt, torch.exp(w[p + "A_log"]), w[p + "D"])
    return gated_norm_in_parts(y.reshape(T, inner), z, w[p + "norm"], m["norm_groups"], eps) @ w[p + "o"].T


def expert(w, p, x, limit):
    g = torch.clamp(x @ w[p + "gate"].T, max=limit)
    u = torch.clamp(x @ w[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(SWISH * g) * (u + 1.0)) @ w[p + "down"].T


def route(z, top):
    """(choice [T, top], weights [T, top]): the largest logits (the lower index among equals), softmax over them."""
    vals, idx = torch.sort(z, dim=-1, descending=True, stable=True)
    return idx[:, :top], torch.softmax(vals[:, :top], -1)


def routed_ff(f, w, p, x):
    z = x @ w[p + "router"].T + w[p + "router.b"]
    choice, weight = route(z, f["router"]["top"])
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for c, wt in zip(choice[t].tolist(), weight[t]):
            out[t] += wt * expert(w, f"{p}e{c}.", x[t:t + 1], f["expert"]["limit"])[0]
    if f.get("shared") is not None:
        out = out + torch.sigmoid(x @ w[p + "shared.sg"].T) * expert(w, p + "shared.", x, f["shared"]["limit"])
    return out


def forward(cfg, weights, tokens: Sequence[int], streams: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """float64 logits [T, vocab]; ``streams`` (a list) receives the residual stream after every layer."""
    w = {k: v.to(F) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = rms(w["embed"][torch.tensor(list(tokens))], eps) * (1.0 + w["embed.norm"])
    shared = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        if layer["type"] == "latent_attention":
            a, kv = latent_attention(layer["mixer"], w, p + "mix.", x, eps, shared)
            if layer["mixer"].get("kv_from") is None:
                shared[i] = kv
        else:
            a = mamba2(layer["mixer"], w, p + "mix.", x, eps)
        x = x + rms(a, eps) * (1.0 + w[p + "norm1"])
        if layer["mlp"] is not None:
            x = x + rms(routed_ff(layer["mlp"], w, p + "mlp.", x), eps) * (1.0 + w[p + "norm2"])
        if streams is not None:
            streams.append(x.clone())
    return (rms(x, eps) * (1.0 + w["final.norm"])) @ w["head"].T


def argmax_first(row: torch.Tensor) -> int:
    return int(torch.nonzero(row == row.max())[0])
