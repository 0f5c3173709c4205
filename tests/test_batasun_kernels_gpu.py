"""Each mechanism of the Batasun decoder alone, kernel by kernel, against the plain functions of ``plain_batasun``:
the latents' norms with the rotation of the shared key part, the small products per head around the attention (both
forms), the state-space recurrence fed whole, in pieces and token by token, the gated norm in parts, the convolution's
bias, the router that weighs by the softmax over the chosen logits, the clamped activation in every kernel that ends
in it, the gate on the shared expert, and the layer without a norm in front of its sublayers."""
import pytest
import torch

import plain_batasun as P
from test_sequence_kernels_gpu import cuts, feed, planner_for

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F64 = torch.float64


def rel(got, ref):
    return float((got.cpu().to(F64) - ref).abs().max()) / max(float(ref.abs().max()), 1e-30)


class Positions:
    """What the latent kernels read of a step: the tokens' positions."""

    def __init__(self, pos):
        self.n_tokens = len(pos)
        self.tok_pos = torch.tensor(pos, dtype=torch.int32, device=DEV)


# ---------------------------------------------------------------- the latents
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("q_rank, kv_rank, rot_dim, rot_dims", [(24, 40, 8, 8), (7, 19, 6, 4), (300, 513, 64, 64), (16, 16, 0, 0), (5, 1, 2, 2)])
def test_latent_norms_and_the_rotated_key_part(dtype, q_rank, kv_rank, rot_dim, rot_dims):
    from agave_amd.ops import latent as L
    n, eps, base = 11, 3e-4, 700.0
    g = torch.Generator().manual_seed(q_rank + kv_rank)
    pos = [0, 1, 2, 63, 64, 65, 1000, 5, 4095, 77, 128]
    wide = torch.randn(n, q_rank + kv_rank + rot_dim + 3, generator=g) * 3          # the raw rows are column slices
    qw, kw = 1 + 0.3 * torch.randn(q_rank, generator=g), 1 + 0.3 * torch.randn(kv_rank, generator=g)
    raw = wide.to(DEV)
    q_raw, kv_raw = raw[:, :q_rank], raw[:, q_rank:q_rank + kv_rank + rot_dim]
    freq = None
    if rot_dims:
        freq = torch.tensor([base ** (-2.0 * e / rot_dims) for e in range(rot_dims // 2)], dtype=torch.float32, device=DEV)
    cq = torch.empty(n, q_rank, dtype=dtype, device=DEV)
    row = torch.empty(n, kv_rank + rot_dim, dtype=dtype, device=DEV)
    L.latent_prepare(q_raw, qw.to(DEV), cq, kv_raw, kw.to(DEV), row, kv_rank, rot_dim, freq, Positions(pos), eps)
    w64 = wide.to(F64)
    want_q = P.rms(w64[:, :q_rank], eps) * qw.to(F64)
    want_c = P.rms(w64[:, q_rank:q_rank + kv_rank], eps) * kw.to(F64)
    r = w64[:, q_rank + kv_rank:q_rank + kv_rank + rot_dim]
    want_r = P.rotate(r, pos, base, rot_dims) if rot_dims else r
    tol = 2e-5 if dtype == torch.float32 else 6e-3
    assert rel(cq, want_q) < tol and rel(row[:, :kv_rank], want_c) < tol
    if rot_dim:
        # angles of thousands of radians in 32-bit: the product position * frequency is rounded once
        assert rel(row[:, kv_rank:], want_r) < (4e-4 if dtype == torch.float32 else 6e-3)
    # a mixer that reads another's rows norms its query latent alone
    cq2 = torch.empty_like(cq)
    L.latent_prepare(q_raw, qw.to(DEV), cq2, None, None, None, kv_rank, rot_dim, None, Positions(pos), eps)
    assert torch.equal(cq, cq2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n, heads, K, n_out, tail, rot", [(5, 3, 16, 40, 8, 8), (40, 3, 16, 40, 8, 8), (130, 2, 24, 70, 16, 12),
                                                          (70, 5, 19, 7, 6, 4), (33, 1, 96, 128, 0, 0), (64, 4, 40, 16, 2, 2)])
def test_products_per_head_with_trailing_elements_and_a_gate(dtype, n, heads, K, n_out, tail, rot):
    """Both forms (a workgroup per token and head; the matrix cores for bfloat16 rows of 16 and more tokens with K a
    multiple of 8) against one einsum: the fold of a query through its head's key matrix with the rotated elements
    copied behind it, and the values from a head's sum over latent rows, times a gate."""
    from agave_amd.ops import latent as L
    g = torch.Generator().manual_seed(n + K)
    pos = [(7 * t) % 300 for t in range(n)]
    x = torch.randn(n, heads * (K + tail) + 5, generator=g).to(dtype)
    w = (torch.randn(heads, n_out, K, generator=g) * K ** -0.5).to(dtype)
    gate = torch.randn(n, heads * n_out, generator=g)
    freq = torch.tensor([50.0 ** (-2.0 * e / rot) for e in range(rot // 2)], dtype=torch.float32, device=DEV) if rot else None
    x64 = x.to(F64)[:, :heads * (K + tail)].view(n, heads, K + tail)
    prod = torch.einsum("thk,hck->thc", x64[..., :K], w.to(F64))
    tails = P.rotate(x64[..., K:], pos, 50.0, rot) if rot else x64[..., K:]
    tol = 2e-5 if dtype == torch.float32 else 8e-3
    for plain in (True, False):
        y = torch.full((n, heads * (n_out + tail) + 3), 9.0, dtype=dtype, device=DEV)
        L.heads_product(x.to(DEV), w.to(DEV), y, heads, K + tail, n_out + tail, tail=tail, freq=freq,
                        tok_pos=Positions(pos).tok_pos if tail else None, force_plain=plain)
        got = y[:, :heads * (n_out + tail)].view(n, heads, n_out + tail)
        assert rel(got[..., :n_out], prod) < tol, plain
        if tail:
            assert rel(got[..., n_out:], tails) < (4e-4 if dtype == torch.float32 else 8e-3), plain
        assert bool((y[:, heads * (n_out + tail):] == 9.0).all())
        if not tail:
            y2 = torch.empty(n, heads * n_out, dtype=dtype, device=DEV)
            L.heads_product(x.to(DEV), w.to(DEV), y2, heads, K, n_out, gate=gate.to(DEV), force_plain=plain)
            assert rel(y2.view(n, heads, n_out), prod * torch.sigmoid(gate.to(F64)).view(n, heads, n_out)) < tol, plain


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, dim, rot_dim, rot, kv_rank", [(4, 32, 16, 16, 48), (3, 10, 6, 4, 7), (1, 128, 64, 64, 512), (5, 8, 0, 0, 16)])
def test_every_heads_key_row_from_the_parts_and_the_gate(dtype, heads, dim, rot_dim, rot, kv_rank):
    from agave_amd.ops import latent as L
    n, qd = 37, dim + rot_dim
    g = torch.Generator().manual_seed(dim)
    pos = [(11 * t) % 500 for t in range(n)]
    q = torch.randn(n, heads * qd, generator=g).to(dtype)
    k_plain = torch.randn(n, heads * dim, generator=g).to(dtype)
    k_row = torch.randn(n, kv_rank + rot_dim, generator=g).to(dtype)
    freq = torch.tensor([90.0 ** (-2.0 * e / rot) for e in range(rot // 2)], dtype=torch.float32, device=DEV) if rot else None
    qd_, k_full = q.to(DEV), torch.empty(n, heads * qd, dtype=dtype, device=DEV)
    L.latent_expand(qd_, k_plain.to(DEV), k_row.to(DEV), kv_rank, k_full, heads, dim, rot_dim, freq, Positions(pos).tok_pos)
    q64 = q.to(F64).view(n, heads, qd)
    want_q = torch.cat([q64[..., :dim], P.rotate(q64[..., dim:], pos, 90.0, rot) if rot else q64[..., dim:]], -1)
    want_k = torch.cat([k_plain.to(F64).view(n, heads, dim), k_row.to(F64)[:, None, kv_rank:].expand(n, heads, rot_dim)], -1)
    assert torch.equal(k_full.cpu().to(F64).view(n, heads, qd), want_k)
    assert rel(qd_.view(n, heads, qd), want_q) < (4e-4 if dtype == torch.float32 else 8e-3)
    wide = torch.randn(n, heads * qd + 3, generator=g) * 3
    x = q.to(DEV).clone()
    L.gate_rows(x, wide.to(DEV)[:, 1:1 + heads * qd])
    assert rel(x, q.to(F64) * torch.sigmoid(wide.to(F64)[:, 1:1 + heads * qd])) < (1e-5 if dtype == torch.float32 else 5e-3)


# ---------------------------------------------------------------- the state-space recurrence
def run_state_space(t, sizes, plan_rows, vectors):
    from agave_amd.cache import StateNeed
    from agave_amd.ops import sequence as S
    H, G, N, dv = sizes
    cache, planner = planner_for(state={0: StateNeed((H, dv, N))})
    cache.alloc_slot()
    slot = cache.alloc_slot()
    T = t["xs"].shape[0]
    out = torch.zeros(T, H * dv, device=DEV)
    v = {n: x.to(DEV) for n, x in vectors.items()}
    for lo, hi in plan_rows:
        step = feed(cache, planner, [slot], [hi - lo])
        d = {n: x[lo:hi].to(DEV).contiguous() for n, x in t.items()}
        S.gated_recurrence(S.SSD, d["C"], d["B"], d["xs"], out[lo:hi], cache.state[0], step, H, G, N, dv, dt_in=d["dt"],
                           a_log=v["a_log"], dt_bias=v["dt_bias"], skip=v["skip"])
        planner.commit(step)
    return out.cpu().to(F64), cache.state[0][slot].cpu().to(F64).transpose(1, 2)          # states as [H, N, dv]


def state_space_inputs(H, G, N, dv, T, seed):
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *s: torch.randn(*s, generator=g)
    t = {"xs": rnd(T, H * dv), "B": rnd(T, G * N), "C": rnd(T, G * N), "dt": rnd(T, H) * 2}
    vec = {"a_log": 0.7 * rnd(H) - 1.0, "dt_bias": rnd(H) - 0.5, "skip": rnd(H)}
    return t, vec


def plain_state_space(t, vec, H, G, N, dv):
    T = t["xs"].shape[0]
    dt = torch.nn.functional.softplus(t["dt"].to(F64) + vec["dt_bias"].to(F64), threshold=1e9)
    return P.state_space_steps(t["xs"].to(F64).view(T, H, dv), t["B"].to(F64).view(T, G, N), t["C"].to(F64).view(T, G, N), dt,
                               torch.exp(vec["a_log"].to(F64)), vec["skip"].to(F64))


@pytest.mark.parametrize("H, G, N, dv", [(4, 2, 16, 24), (6, 3, 20, 5), (6, 2, 32, 48), (2, 1, 64, 64), (3, 3, 128, 40), (1, 1, 8, 3), (8, 1, 24, 100)])
def test_state_space_whole_pieces_and_tokens(H, G, N, dv):
    T = 90
    t, vec = state_space_inputs(H, G, N, dv, T, N + dv)
    ref, S_ref = plain_state_space(t, vec, H, G, N, dv)
    for plan in (cuts(T, T, 1), cuts(T, 40, 1), cuts(T, 1, 2), cuts(T, 17, 16), cuts(T, 33, 31), cuts(T, 1, 1)):
        got, S_got = run_state_space(t, (H, G, N, dv), plan, vec)
        assert torch.allclose(got, ref.reshape(T, -1), atol=3e-5, rtol=1e-4), plan[:2]
        assert torch.allclose(S_got, S_ref, atol=3e-5, rtol=1e-4), plan[:2]


def test_state_space_step_sizes_without_a_clamp_and_a_write_far_back():
    """Step sizes from almost nothing to dozens (softplus of -20 to 40, neither clamped); and with a decay rate of
    almost nothing what token 3 wrote is read 600 tokens later among small writes, while a fast rate forgets it."""
    H, G, N, dv, T = 1, 1, 8, 4, 650
    g = torch.Generator().manual_seed(5)
    for a_log, kept in ((-12.0, True), (1.0, False)):
        t = {"xs": 0.01 * torch.randn(T, dv, generator=g), "B": torch.zeros(T, N), "C": torch.zeros(T, N),
             "dt": torch.linspace(-20.0, 40.0, T)[torch.randperm(T, generator=g)][:, None].contiguous()}
        t["B"][:, 1] = 0.01
        t["xs"][3] = torch.tensor([7.0, -3.0, 2.0, 1.0])
        t["B"][3, 5] = 1.0
        t["dt"][3] = 0.5
        t["C"][-1, 5] = 4.0
        vec = {"a_log": torch.tensor([a_log]), "dt_bias": torch.tensor([0.1]), "skip": torch.tensor([0.0])}
        ref, _ = plain_state_space(t, vec, H, G, N, dv)
        for plan in (cuts(T, T, 1), cuts(T, 600, 1)):
            got, _ = run_state_space(t, (H, G, N, dv), plan, vec)
            assert torch.allclose(got, ref.reshape(T, -1), atol=1e-5, rtol=1e-4)
            assert (float(got[-1, 0].abs()) > 5.0) == kept


def test_state_space_batch_of_unequal_sequences_against_each_alone_and_a_slot_used_again():
    from agave_amd.cache import StateNeed
    from agave_amd.ops import sequence as S
    H, G, N, dv = 4, 2, 12, 10
    cache, planner = planner_for(state={0: StateNeed((H, dv, N))}, slots=4)
    for round_ in range(2):
        lens = [1, 33, 2, 18]
        made = [state_space_inputs(H, G, N, dv, n, 10 * round_ + i) for i, n in enumerate(lens)]
        vec = made[0][1]
        slots = [cache.alloc_slot() for _ in lens]
        first = [1, 20, 1, 18]
        outs = [[] for _ in lens]
        at = list(first)

        def run(slots_, rows):
            step = feed(cache, planner, slots_, [hi - lo for lo, hi in rows])
            idx = [slots.index(s) for s in slots_]
            cat = {n: torch.cat([made[i][0][n][lo:hi] for i, (lo, hi) in zip(idx, rows)]).to(DEV) for n in ("xs", "B", "C", "dt")}
            out = torch.empty(sum(hi - lo for lo, hi in rows), H * dv, device=DEV)
            S.gated_recurrence(S.SSD, cat["C"], cat["B"], cat["xs"], out, cache.state[0], step, H, G, N, dv, dt_in=cat["dt"],
                               **{n: x.to(DEV) for n, x in vec.items()})
            planner.commit(step)
            o = 0
            for i, (lo, hi) in zip(idx, rows):
                outs[i].append(out[o:o + hi - lo].cpu())
                o += hi - lo
        run(slots, [(0, f) for f in first])
        while any(a < n for a, n in zip(at, lens)):               # then one token each, the finished ones drop out
            live = [i for i, (a, n) in enumerate(zip(at, lens)) if a < n]
            run([slots[i] for i in live], [(at[i], at[i] + 1) for i in live])
            for i in live:
                at[i] += 1
        for i, n in enumerate(lens):
            ref, _ = plain_state_space(made[i][0], vec, H, G, N, dv)
            assert torch.allclose(torch.cat(outs[i]).to(F64), ref.reshape(n, -1), atol=3e-5, rtol=1e-4), (round_, i)
        for s in slots:
            cache.free_slot(s)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width, parts", [(48, 2), (30, 5), (7, 7), (288, 1), (1024, 4), (6, 1)])
def test_gated_norm_in_parts(dtype, width, parts):
    from agave_amd.ops import sequence as S
    n, eps = 19, 1e-3
    g = torch.Generator().manual_seed(width)
    wide = torch.randn(n, 2 * width + 1, generator=g) * 2
    weight = 1 + 0.3 * torch.randn(width, generator=g)
    d = wide.to(DEV)
    out = torch.empty(n, width, dtype=dtype, device=DEV)
    S.gated_group_norm(d[:, :width], d[:, width:2 * width], weight.to(DEV), out, parts, eps)
    want = P.gated_norm_in_parts(wide[:, :width].to(F64), wide[:, width:2 * width].to(F64), weight.to(F64), parts, eps)
    assert rel(out, want) < (2e-5 if dtype == torch.float32 else 6e-3)


@pytest.mark.parametrize("taps", [1, 3, 4])
def test_convolution_with_a_bias(taps):
    from agave_amd.cache import StateNeed
    from agave_amd.ops import sequence as S
    C, T = 37, 29
    g = torch.Generator().manual_seed(taps)
    u, w, b = torch.randn(T, C, generator=g), torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
    ref = P.silu(P.causal_conv(u.to(F64), w.to(F64), b.to(F64)))
    for first, piece in ((T, 1), (11, 1), (1, 2), (2, 9)):
        cache, planner = planner_for(state={0: StateNeed((taps - 1, C))})
        cache.alloc_slot()
        slot = cache.alloc_slot()
        got = torch.zeros(T, C)
        for lo, hi in cuts(T, first, piece):
            step = feed(cache, planner, [slot], [hi - lo])
            y = torch.empty(hi - lo, C, device=DEV)
            S.short_conv(u[lo:hi].to(DEV).contiguous(), w.to(DEV), y, cache.state[0], step, True, b.to(DEV))
            planner.commit(step)
            got[lo:hi] = y.cpu()
        assert torch.allclose(got.to(F64), ref, atol=2e-5, rtol=1e-5), (first, piece)


# ---------------------------------------------------------------- the routed feed-forward
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("R, top, K, n, extra", [(16, 2, 64, 37, 1), (5, 5, 40, 9, 0), (1, 1, 33, 4, 1), (130, 9, 96, 19, 2), (8, 1, 200, 1, 1)])
def test_the_largest_logits_choose_and_weigh(dtype, R, top, K, n, extra):
    """Logits with a bias; the ``top`` largest; weights by the softmax over the chosen alone (a softmax over all the
    logits would give other weights, a sigmoid too); further rows of the router matrix come out as they are."""
    from agave_amd.ops import routed
    g = torch.Generator().manual_seed(R + K)
    x = torch.randn(n, K, generator=g).to(dtype)
    router = torch.randn(R + extra, K, generator=g) * K ** -0.5 * 2
    bias = torch.randn(R, generator=g)
    z = x.to(F64) @ router[:R].to(F64).T + bias.to(F64)
    want_e, want_w = P.route(z, top)
    ranked = z.sort(-1, descending=True).values[:, :top + 1]
    safe = torch.ones(n, dtype=torch.bool) if R == 1 else (ranked[:, :-1] - ranked[:, 1:]).min(-1).values > 1e-5
    choice = torch.empty(n, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(n, top, device=DEV)
    extra_out = torch.empty(n, extra, device=DEV) if extra else None
    routed.route_rows(x.to(DEV), router.to(DEV), bias.to(DEV), 1, 1, top, 1.0, choice, weight, softmax_top=True, extra_out=extra_out)
    assert int(safe.sum()) >= n - 2
    assert torch.equal(choice.cpu().long()[safe], want_e[safe])
    assert torch.allclose(weight.cpu().to(F64)[safe], want_w[safe], rtol=2e-4, atol=1e-6)
    assert torch.allclose(weight.cpu().sum(-1), torch.ones(n), atol=1e-5)
    if extra:
        assert torch.allclose(extra_out.cpu().to(F64), x.to(F64) @ router[R:].to(F64).T, rtol=1e-4, atol=1e-5)


def test_equal_logits_go_to_the_lower_index_and_the_bias_counts_in_the_weights():
    from agave_amd.ops import routed
    x = torch.zeros(2, 8)
    x[1, 0] = 1.0
    router = torch.zeros(4, 8)
    router[:, 0] = torch.tensor([0.0, 3.0, 0.0, 3.0])
    bias = torch.tensor([1.0, 1.0, 2.0, -2.0])
    choice = torch.empty(2, 2, dtype=torch.int32, device=DEV)
    weight = torch.empty(2, 2, device=DEV)
    routed.route_rows(x.to(DEV), router.to(DEV), bias.to(DEV), 1, 1, 2, 1.0, choice, weight, softmax_top=True)
    # token 0: logits are the bias alone, (1, 1, 2, -2): 2 first, then the lower of the two equal ones
    # token 1: (1, 4, 2, 1): 1, then 2
    assert choice.cpu().tolist() == [[2, 0], [1, 2]]
    e = torch.exp(torch.tensor([[2.0, 1.0], [4.0, 2.0]], dtype=F64))
    assert torch.allclose(weight.cpu().to(F64), e / e.sum(-1, keepdim=True), rtol=1e-5)


def clamped(g, u, limit):
    g = torch.clamp(g, max=limit)
    return g * torch.sigmoid(P.SWISH * g) * (torch.clamp(u, -limit, limit) + 1.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_clamped_activation_alone(dtype):
    """Gates and up values far outside the limit on both sides: the gate is capped from above only, the up value on
    both sides, and one is added to it after the clamp."""
    from agave_amd.ops import kernels as K
    g = torch.Generator().manual_seed(1)
    gate, up = (torch.randn(13, 70, generator=g) * 4).to(dtype), (torch.randn(13, 70, generator=g) * 4).to(dtype)
    gate[0, :4] = torch.tensor([-30.0, 30.0, 1.5, -1.5]).to(dtype)
    up[0, :4] = torch.tensor([30.0, -30.0, -1.5, 1.5]).to(dtype)
    for limit in (1.5, 7.0, 0.25):
        out = torch.empty(13, 70, dtype=dtype, device=DEV)
        K.gated_act(gate.to(DEV), up.to(DEV), out, "swish_clamped", limit, P.SWISH)
        want = clamped(gate.to(F64), up.to(F64), limit)
        assert rel(out, want) < (1e-5 if dtype == torch.float32 else 5e-3), limit
    assert float(clamped(torch.tensor(-30.0, dtype=F64), torch.tensor(30.0, dtype=F64), 1.5).abs()) < 1e-10


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E, top, ff, hidden, n, limit", [(5, 3, 20, 40, 33, 1.25), (3, 1, 70, 24, 5, 0.5), (8, 8, 16, 72, 130, 2.0),
                                                         (6, 2, 136, 200, 300, 1.5), (4, 3, 96, 256, 70, 7.0), (1, 1, 32, 64, 20, 1.0)])
def test_clamped_experts_and_the_gated_shared_row(dtype, E, top, ff, hidden, n, limit):
    from agave_amd.ops import kernels as K
    from agave_amd.ops import routed
    act = K.GATE_ACTIVATIONS["swish_clamped"]
    g = torch.Generator().manual_seed(E * 10 + top)
    rnd = lambda *s: (torch.randn(*s, generator=g) * 2 * s[-1] ** -0.5).to(dtype).float()
    x = (torch.randn(n, hidden, generator=g) * 1.5).to(dtype).float()
    wg, wu, wd = rnd(E, ff, hidden), rnd(E, ff, hidden), rnd(E, hidden, ff)
    shared = torch.randn(n, hidden, generator=g).to(dtype).float()
    shared_logit = torch.randn(n, generator=g) * 2
    choice = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(n)]).int()
    weight = torch.softmax(torch.randn(n, top, generator=g), -1)
    w = {}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = wg[e].to(F64), wu[e].to(F64), wd[e].to(F64)
    want = torch.sigmoid(shared_logit.to(F64))[:, None] * shared.to(F64)
    for t in range(n):
        for e, a in zip(choice[t].tolist(), weight[t].tolist()):
            want[t] += a * P.expert(w, f"e{e}.", x[t:t + 1].to(F64), limit)[0]
    d = lambda t: t.to(dtype).to(DEV).contiguous()
    tol = 3e-5 if dtype == torch.float32 else 3e-2
    act_rows = torch.empty(n * top, ff, dtype=dtype, device=DEV)
    y = torch.full((n * top, hidden), float("nan"), device=DEV)
    routed.experts_plain(d(x), choice.view(-1).to(DEV), d(wg), d(wu), d(wd), act_rows, y, top, act, limit, P.SWISH)
    out = torch.empty(n, hidden, dtype=dtype, device=DEV)
    routed.combine(y, None, choice.view(-1).to(DEV), weight.view(-1).to(DEV), d(x), d(shared), out, top, E, shared_logit.to(DEV))
    assert rel(out, want) < tol
    if dtype == torch.bfloat16 and routed.mfma_ok(d(x), ff):
        for tm in (16, 64):
            tiles = (n * top + tm - 1) // tm + E
            place = torch.full((n * top,), -7, dtype=torch.int32, device=DEV)
            sorted_pair = torch.full((tiles * tm,), -7, dtype=torch.int32, device=DEV)
            tile_expert = torch.full((tiles,), -7, dtype=torch.int32, device=DEV)
            routed.route_sort(choice.view(-1).to(DEV), E, tm, tiles, place, sorted_pair, tile_expert)
            act_rows = torch.empty(tiles * tm, ff, dtype=dtype, device=DEV)
            y2 = torch.full((tiles * tm, hidden), float("nan"), device=DEV)
            routed.experts_mfma(d(x), sorted_pair, tile_expert, d(wg), d(wu), d(wd), act_rows, y2, tm, tiles, top, act, p0=limit, p1=P.SWISH)
            out2 = torch.empty(n, hidden, dtype=dtype, device=DEV)
            routed.combine(y2, place, choice.view(-1).to(DEV), weight.view(-1).to(DEV), d(x), d(shared), out2, top, E, shared_logit.to(DEV))
            assert rel(out2, want) < tol, tm


# ---------------------------------------------------------------- one mechanism a model
def one_layer(layer, dtype, **kw):
    from agave_amd.engine import Engine
    cfg = P.config([layer], vocab=kw.pop("vocab", 70), width=kw.pop("width", 48), eps=kw.pop("eps", 1e-5))
    w = P.random_weights(cfg, 11, decided_routing=(dtype == "bfloat16"))
    eng = Engine.from_tensors(cfg, {k: v.bfloat16() for k, v in w.items()}, dtype=dtype, max_slots=2, max_context=256)
    return cfg, w, eng


LAYERS = {
    "latent": lambda: P.latent_layer(3, 16, 8, 24, 24, 40, base=3000.0, mlp=None),
    "latent, one head of other sizes": lambda: P.latent_layer(1, 5, 4, 9, 7, 11, base=20.0, scale=0.7, rot_dims=2, mlp=None),
    "state space": lambda: P.mamba_layer(4, 12, 8, 2, 4, 3, mlp=None),
    "state space, one of everything": lambda: P.mamba_layer(1, 7, 5, 1, 2, 1, mlp=None),
    "routed": lambda: P.mamba_layer(1, 8, 8, 1, 2, 1, mlp=P.moe(6, 2, 24, 1.25, shared_ff=16, shared_limit=3.0)),
    "routed, no shared expert": lambda: P.mamba_layer(1, 8, 8, 1, 2, 1, mlp=P.moe(4, 4, 20, 0.5)),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(LAYERS))
def test_a_model_of_one_layer(name, dtype):
    """One layer between the embedding's norm and the model's end: a prompt whole, its first tokens (positions 0, 1,
    2 alone), the prompt in pieces of two and three tokens, and the last 70 tokens decoded across a page's border."""
    import engine_utils as U
    cfg, w, eng = one_layer(LAYERS[name](), dtype)
    toks = U.random_tokens(140, cfg["vocab"], 2)
    ref = P.forward(cfg, w, toks)
    tol = 3e-5 if dtype == "float32" else 0.06
    scale = float(ref.abs().max())

    def near(got, want, what):
        assert float((got.double() - want).abs().max()) <= tol * scale, (name, what)
    near(U.run_whole(eng, toks), ref, "whole")
    for n in (1, 2, 3):
        near(U.run_whole(eng, toks[:n]), ref[:n], f"the first {n}")
    near(U.run_tail(eng, toks, 70), ref, "decoded")
    near(U.run_tail(eng, toks, 139), ref, "decoded from the second token")
    for piece in (2, 3):
        eng.prefill_chunk = piece
        near(U.run_whole(eng, toks[:67]), ref[:67], f"pieces of {piece}")
