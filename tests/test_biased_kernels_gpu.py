"""The kernels of the biased attention, the layer norm and the routed feed-forward alone, against the plain
functions of ``plain_gusedra``: sizes that are no powers of two, sequences fed whole, in pieces and token by
token through the framework's own cache and step planner, and inputs made so that a fault would show (one
key that dominates, just inside and just outside a window, among the kept first positions and just behind
them, at a page's border, far back)."""
import math

import pytest
import torch

import plain_gusedra as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F64 = torch.float64


def planner_for(key, slots=3, pages=40, dtype=torch.float32, context=2048):
    from agave_amd.cache import KVCache
    from agave_amd.engine.step import StepPlanner
    cache = KVCache({0: key}, {}, slots, {key: pages}, dtype, torch.device(DEV), context)
    return cache, StepPlanner(cache, 1000, torch.device(DEV))


def cuts(total, first, piece):
    out, at = [(0, first)], first
    while at < total:
        n = min(piece, total - at)
        out.append((at, at + n))
        at += n
    return out


class Case:
    """One attention layer's inputs and what the kernels take of it."""

    def __init__(self, H, G, d, vd, window, keep, bias, sink, gate, T, seed=0, buckets=12, D=90):
        from agave_amd.ops import attention_biased as A
        from agave_amd.parts.biased_attention import distance_table
        g = torch.Generator().manual_seed(seed)
        self.H, self.G, self.d, self.vd, self.window, self.keep, self.T = H, G, d, vd, window, keep, T
        self.force_plain = False            # bfloat16 shapes that the matrix-core kernel takes run on the plain one instead
        self.workspace, self.splits = None, None   # steps of one row: a row's pages shared among this many workgroups
        self.q = torch.randn(T, H, d, generator=g)
        self.k = torch.randn(T, G, d, generator=g)
        self.v = torch.randn(T, G, vd, generator=g)
        self.gate = torch.randn(T, H * vd, generator=g) if gate else None
        self.sink = torch.randn(H, generator=g) if sink else None
        self.scale = 0.7 * d ** -0.5
        self.rel = torch.randn(buckets, H, generator=g) if bias == "table" else None
        self.bias_kind, self.D = bias, D
        if bias == "none":
            self.mode, self.bias = A.BIAS_NONE, None
        elif bias == "slopes":
            self.mode = A.BIAS_SLOPES
            self.bias = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=torch.float32, device=DEV)
        else:
            self.mode, self.bias = A.BIAS_TABLE, distance_table(self.rel, buckets, D).to(DEV)

    def rounded(self, dtype):
        for name in ("q", "k", "v", "gate"):
            t = getattr(self, name)
            if t is not None:
                setattr(self, name, t.to(dtype).float())

    def plain(self):
        T, H = self.T, self.H
        if self.bias_kind == "slopes":
            bias = P.slope_bias(T, H)
        elif self.bias_kind == "table":
            bias = P.bucket_bias(T, self.rel.to(F64), self.D)
        else:
            bias = torch.zeros(H, T, T, dtype=F64)
        out = P.softmax_attention(self.q.to(F64), self.k.to(F64), self.v.to(F64), self.scale, bias,
                                  P.visible(T, self.window, self.keep), self.sink.to(F64) if self.sink is not None else None)
        out = out.reshape(T, H * self.vd)
        return out * torch.sigmoid(self.gate.to(F64)) if self.gate is not None else out

    def key(self):
        from agave_amd.cache import GroupKey
        return GroupKey(self.window, self.G, self.d, v_head_dim=self.vd, layout="rows_vt",
                        keep_first=self.keep if self.window is not None else 0)

    def run(self, ranges, dtype=torch.float32, cache=None, planner=None, slot=None, pages=40):
        """Feed the rows of ``ranges`` one step each; returns the context rows [T, H * vd]."""
        from agave_amd.ops import attention_biased as A
        key = self.key()
        own = cache is None
        if own:
            cache, planner = planner_for(key, dtype=dtype, pages=pages)
            cache.alloc_slot()
            slot = cache.alloc_slot()
        head = key.kept_pages
        got = torch.zeros(self.T, self.H * self.vd)
        sink = self.sink.to(DEV) if self.sink is not None else None
        for lo, hi in ranges:
            step = planner.plan([slot], [[0] * (hi - lo)], "all")
            kp, vp, packed = cache.pages_of(0)
            table, base = step.tables[0]
            dev = lambda t: t[lo:hi].reshape(hi - lo, -1).to(dtype).to(DEV).contiguous()
            A.kv_append_rows(dev(self.k), dev(self.v), kp, vp, table, base, head, step, self.G, self.d, self.vd, packed)
            out = torch.empty(hi - lo, self.H * self.vd, dtype=dtype, device=DEV)
            A.attention(dev(self.q), out, dev(self.gate) if self.gate is not None else None, kp, vp, table, base, head, step,
                        self.H, self.G, self.d, self.vd, self.scale, self.window, self.keep, self.mode, self.bias, sink,
                        packed, force_plain=self.force_plain, workspace=self.workspace, splits=self.splits)
            planner.commit(step)
            got[lo:hi] = out.float().cpu()
        if own:
            cache.free_slot(slot)
            assert cache.groups[0].pool.n_free == cache.groups[0].pool.n_pages - 0
        return got


def close(got, ref, dtype, what):
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    err = (got.to(F64) - ref).abs().max()
    assert float(err) <= tol * max(1.0, float(ref.abs().max())), f"{what}: error {float(err):.3e}"


SHAPES = [
    # H, G, d, vd, window, keep, bias, sink, gate
    (6, 3, 16, 24, 70, 5, "table", False, True),          # values wider than keys, a window over a page's border, kept positions
    (4, 4, 24, 8, 33, 0, "slopes", True, False),          # values narrower, no grouping, sinks
    (8, 2, 20, 20, None, 0, "slopes", True, True),        # every earlier key, sizes that are no multiples of 16
    (3, 1, 64, 64, 130, 70, "table", False, False),       # one key head, two kept pages
    (2, 2, 8, 40, 64, 64, "none", False, False),          # no bias; window and kept positions of a page each
    (5, 5, 32, 16, 1, 3, "none", True, True),             # a window of the token itself
    (8, 2, 128, 128, 200, 3, "table", True, True),        # the sizes of large models: the matrix cores in bfloat16
    (4, 1, 96, 48, 100, 0, "slopes", True, False),        # sizes that fill the matrix cores' steps only in part
    (34, 1, 32, 32, None, 0, "table", False, True),       # more heads to a key head than a wave has columns
    (2, 2, 256, 256, 64, 64, "slopes", False, False),     # the largest heads that two waves a SIMD hold
    (16, 1, 320, 272, None, 0, "none", False, False),     # wider: one key head of cached rows for all query heads
    (16, 1, 576, 512, None, 0, "none", False, True),      # the widest, Q in LDS
    (3, 1, 400, 304, 130, 70, "slopes", True, False),     # the widest kernel filled in part, with a window, kept pages and sinks
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_whole_in_pieces_and_token_by_token(shape, dtype):
    T = 300
    c = Case(*shape, T=T, seed=len(str(shape)))
    c.rounded(dtype)
    ref = c.plain()
    for first, piece in ((T, 1), (200, 1), (1, 1), (3, 2), (50, 37), (64, 64)):
        close(c.run(cuts(T, first, piece), dtype), ref, dtype, f"{shape} first {first} pieces of {piece}")
    if dtype == torch.bfloat16:
        c.force_plain = True
        close(c.run(cuts(T, 180, 1), dtype), ref, dtype, f"{shape} on the plain kernel")


@pytest.mark.parametrize("shape", [SHAPES[3], SHAPES[6], SHAPES[8], SHAPES[10], SHAPES[11], SHAPES[12]])
@pytest.mark.parametrize("splits", [None, 2, 5, 16])
def test_a_rows_pages_shared_among_workgroups(shape, splits):
    """Decode steps whose row's pages are shared among several workgroups (more of them than there are pages, too),
    merged by the second kernel: sinks count once, a window's and the kept pages are found by every share."""
    from agave_amd.ops import attention_biased as A
    from agave_amd.parts import Workspace
    T = 330
    c = Case(*shape, T=T, seed=5)
    c.rounded(torch.bfloat16)
    ref = c.plain()
    c.workspace, c.splits = Workspace(torch.device(DEV)), splits
    close(c.run(cuts(T, 1, 1)[:12] + [(12, 250)] + cuts(T, 250, 1)[1:], torch.bfloat16), ref, torch.bfloat16, f"{shape} in {splits}")
    assert 1 <= A.decode_splits(8, 1, 16, 512, 64) <= A.MAX_SPLITS and A.decode_splits(300, 4, 4, 128, 64) == 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_table_too_long_for_lds_is_read_from_memory(dtype):
    """A bias over distances up to 20,000: the table's row of a head does not fit the kernel's LDS allowance and is read
    from memory, in short steps, in a long prompt (pages through LDS, the table not) and token by token."""
    c = Case(40, 4, 32, 32, 600, 3, "table", False, False, T=1100, seed=11, buckets=24, D=20000)
    assert c.bias.shape[1] > 8192
    c.rounded(dtype)
    ref = c.plain()
    close(c.run(cuts(1100, 1100, 1), dtype), ref, dtype, "whole")
    close(c.run(cuts(1100, 1000, 7), dtype), ref, dtype, "1,000 and pieces of 7")
    close(c.run(cuts(1100, 1090, 1), dtype), ref, dtype, "the last ten one by one")


@pytest.mark.parametrize("shape", [
    (40, 4, 64, 64, 200, 70, "table", True, True),        # a window, two kept pages, sinks and a gate
    (40, 2, 32, 48, None, 0, "slopes", False, False),     # every earlier key
    (36, 36, 96, 16, 130, 0, "none", True, False),        # a head size that fills its last step in part
])
def test_long_prompts_share_pages_through_lds(shape):
    """Steps long enough that the matrix-core kernel takes 32 rows a wave and brings the pages into LDS once for a
    workgroup's four waves: a whole prompt, and a long piece behind a short one (the window reaches back into pages
    of the earlier step, and the kept pages are not the window's)."""
    T = 1100
    c = Case(*shape, T=T, seed=7)
    c.rounded(torch.bfloat16)
    ref = c.plain()
    close(c.run(cuts(T, T, 1), torch.bfloat16), ref, torch.bfloat16, f"{shape} whole")
    close(c.run([(0, 230), (230, T)], torch.bfloat16), ref, torch.bfloat16, f"{shape} 230 + 870")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_batch_against_each_alone_and_slots_and_pages_used_again(dtype):
    from agave_amd.ops import attention_biased as A
    shape = (4, 2, 16, 24, 50, 4, "table", False, True)
    lens, firsts = (140, 1, 77), (90, 1, 2)
    cases = [Case(*shape, T=n, seed=10 + i) for i, n in enumerate(lens)]
    for c in cases[1:]:
        c.rel, c.bias = cases[0].rel, cases[0].bias          # one layer: one table
    key = cases[0].key()
    cache, planner = planner_for(key, slots=3, pages=9, dtype=dtype)      # the pool only fits because pages come back
    for round_ in range(2):
        for c in cases:
            c.rounded(dtype)
        slots = [cache.alloc_slot() for _ in cases]
        got = [torch.zeros(c.T, c.H * c.vd) for c in cases]
        used = [0] * len(cases)
        live = list(range(len(cases)))
        first = True
        while live:
            n_new = [firsts[i] if first else 1 for i in live]
            step = planner.plan([slots[i] for i in live], [[0] * n for n in n_new], "all")
            kp, vp, packed = cache.pages_of(0)
            table, base = step.tables[0]
            cat = lambda name: torch.cat([getattr(cases[i], name)[used[i]:used[i] + n].reshape(n, -1)
                                          for i, n in zip(live, n_new)]).to(dtype).to(DEV).contiguous()
            A.kv_append_rows(cat("k"), cat("v"), kp, vp, table, base, key.kept_pages, step, 2, 16, 24, packed)
            out = torch.empty(sum(n_new), 4 * 24, dtype=dtype, device=DEV)
            A.attention(cat("q"), out, cat("gate"), kp, vp, table, base, key.kept_pages, step, 4, 2, 16, 24, cases[0].scale,
                        50, 4, cases[0].mode, cases[0].bias, None, packed)
            planner.commit(step)
            at = 0
            for i, n in zip(live, n_new):
                got[i][used[i]:used[i] + n] = out[at:at + n].float().cpu()
                at += n
                used[i] += n
            first = False
            for i in [i for i in live if used[i] >= cases[i].T]:
                cache.free_slot(slots[i])
            live = [i for i in live if used[i] < cases[i].T]
        for i, c in enumerate(cases):
            close(got[i], c.plain(), dtype, f"round {round_} request {i}")
        assert cache.groups[0].pool.n_free == 9 and cache.slots.n_free == 3


def one_key_stands_out(c, j0, marker):
    """Make key j0 the one that every query answers to, and give it a value no other key has."""
    c.q[:] = 0.05 * c.q
    c.k[:] = 0.05 * c.k
    c.q[:, :, 0] = 6.0
    c.k[j0, :, 0] = 6.0 / c.scale / 6.0 * 4.0        # score of j0: 6 * that * scale = 24, far above the rest and any bias
    c.v[:] = 0.1 * c.v
    c.v[j0, :, :] = marker


@pytest.mark.parametrize("window, keep", [(75, 7), (64, 1), (100, 64), (129, 65), (48, 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_dominant_key_just_inside_and_just_outside(window, keep, dtype):
    """The key is seen (the output is its value) up to the window's last query and not from the next on; a key among
    the kept first positions is seen from everywhere, the first key behind them is not, in a prompt and decoded."""
    T = 420
    for j0, inside_until in ([(150, 150 + window - 1)] + ([(keep - 1, T - 1), (keep, keep + window - 1)] if keep else [])):
        # (a slope on the distance would bury a key hundreds of positions back: the table's bias is bounded)
        # (values of 16 in bfloat16: the matrix-core kernel; of 8: the plain one)
        c = Case(4, 2, 16, 16 if (dtype == torch.bfloat16 and window != 100) else 8, window, keep,
                 "slopes" if window == 48 else "table", True, False, T=T, seed=j0)
        one_key_stands_out(c, j0, 5.0)
        c.rounded(dtype)
        ref = c.plain()
        assert float(ref[inside_until].min()) > 4.5, "the test's key does not dominate where it is seen"
        if inside_until + 1 < T:
            assert float(ref[inside_until + 1].abs().max()) < 1.0, "the test's key shows where it must not"
        for ranges in (cuts(T, T, 1), cuts(T, max(1, j0), 1), cuts(T, inside_until - 3, 5)):
            got = c.run(ranges, dtype)
            close(got, ref, dtype, f"window {window} keep {keep} key {j0}")
            assert float(got[inside_until].min()) > 4.5
            if inside_until + 1 < T:
                assert float(got[inside_until + 1].abs().max()) < 1.0


def test_a_far_key_among_hundreds_without_a_window():
    c = Case(2, 1, 32, 16, None, 0, "none", False, False, T=900, seed=4)
    one_key_stands_out(c, 3, -7.0)
    ref = c.plain()
    got = c.run(cuts(900, 880, 1))
    close(got, ref, torch.float32, "a key 896 positions back")
    assert float(got[899].max()) < -6.0


def test_the_sink_takes_its_share_and_the_bias_is_not_scaled():
    # one token, one key: the weight of its value is exp(s) / (exp(s) + exp(sink)), s = scale q.k + bias(0)
    from agave_amd.ops import attention_biased as A
    c = Case(2, 2, 8, 8, 10, 0, "table", True, False, T=1, seed=2, buckets=6, D=20)
    ref = c.plain()
    s = (c.q[0] * c.k[0]).sum(-1).to(F64) * c.scale + c.rel[0].to(F64)
    by_hand = (torch.exp(s) / (torch.exp(s) + torch.exp(c.sink.to(F64))))[:, None] * c.v[0].to(F64)
    assert torch.allclose(ref.view(2, 8), by_hand, atol=1e-12)
    close(c.run([(0, 1)]), ref, torch.float32, "one token with a sink")


# ---------------------------------------------------------------- layer norm around the residual stream
@pytest.mark.parametrize("e", [32, 257, 1000, 4096, 6000, 9000])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_residual_layernorm(e, dtype):
    from agave_amd.ops import kernels as K
    g = torch.Generator().manual_seed(e)
    n = 7
    h = torch.randn(n, e, generator=g) * 3 + 1.5
    br = (torch.randn(n, e, generator=g) * 2 - 0.7).to(dtype).float()
    w1, b1, w2, b2 = (torch.randn(e, generator=g) for _ in range(4))
    eps = 1e-3
    added = h.to(F64) + P.layer_norm(br.to(F64), w1.to(F64), b1.to(F64), eps)
    normed = P.layer_norm(added, w2.to(F64), b2.to(F64), eps)
    tol = dict(atol=3e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=4e-2, rtol=2e-2)
    d = lambda t: t.to(DEV).contiguous()
    # branch through the norm after the sublayer, then the norm before the next
    hd, out = d(h), torch.empty(n, e, dtype=dtype, device=DEV)
    K.residual_layernorm(hd, d(br.to(dtype)), d(w1), d(b1), eps, out, d(w2), d(b2), eps)
    assert torch.allclose(hd.cpu().to(F64), added, atol=3e-5, rtol=2e-5)
    assert torch.allclose(out.float().cpu().to(F64), normed, **tol)
    # the branch as three 32-bit slices; the stream read from another place
    parts = torch.randn(3, n, e, generator=g)
    parts[2] = br - parts[0] - parts[1]
    src, hd = d(h), torch.zeros(n, e, device=DEV)
    K.residual_layernorm(hd, d(parts), d(w1), d(b1), eps, out, d(w2), d(b2), eps, src=src)
    assert torch.allclose(hd.cpu().to(F64), added, atol=2e-4, rtol=2e-5)
    # chosen rows only, no branch, no bias
    rows = torch.tensor([5, 0, 5, 3], dtype=torch.int32, device=DEV)
    out4 = torch.empty(4, e, dtype=dtype, device=DEV)
    K.residual_layernorm(d(h), None, None, None, 0.0, out4, d(w2), None, eps, rows)
    want = P.layer_norm(h.to(F64), w2.to(F64), torch.zeros(e, dtype=F64), eps)[[5, 0, 5, 3]]
    assert torch.allclose(out4.float().cpu().to(F64), want, **tol)
    # a branch without a norm is added as it is
    hd = d(h)
    K.residual_layernorm(hd, d(br.to(dtype)), None, None, 0.0, None, None, None, 0.0)
    assert torch.allclose(hd.cpu(), h + br, atol=1e-6)


def test_a_constant_row_and_the_variance_as_the_mean_of_squared_deviations():
    from agave_amd.ops import kernels as K
    e = 96
    h = torch.full((2, e), 1000.0)
    h[1, ::2] += 0.5                 # deviations of a quarter around a large mean: a sum of squares minus a squared mean would lose them
    w, b = torch.ones(e), torch.full((e,), 0.25)
    out = torch.empty(2, e, device=DEV)
    K.residual_layernorm(h.to(DEV), None, None, None, 0.0, out, w.to(DEV), b.to(DEV), 1e-6)
    want = P.layer_norm(h.to(F64), w.to(F64), b.to(F64), 1e-6)
    assert torch.allclose(out.cpu().to(F64), want, atol=1e-3)
    assert torch.allclose(out[0].cpu(), torch.full((e,), 0.25))


# ---------------------------------------------------------------- the square of relu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_relu_squared(dtype):
    from agave_amd.ops import kernels as K
    x = torch.randn(9, 50).to(dtype)
    out = torch.empty(9, 50, dtype=dtype, device=DEV)
    K.unary_act(x.to(DEV), out, "relu2")
    want = torch.relu(x.float()) ** 2
    assert torch.allclose(out.float().cpu(), want.to(dtype).float(), atol=1e-6)


# ---------------------------------------------------------------- the router's choice
@pytest.mark.parametrize("R, groups, keep, top", [(10, 2, 1, 4), (12, 4, 2, 5), (7, 1, 1, 7), (64, 8, 3, 6), (5, 5, 2, 2), (130, 1, 1, 9)])
def test_route_topk(R, groups, keep, top):
    from agave_amd.ops import routed
    g = torch.Generator().manual_seed(R)
    n = 200
    z = torch.randn(n, R, generator=g) * 2
    for corr in (torch.randn(R, generator=g) * 0.05, torch.full((R,), -3.0) + torch.randn(R, generator=g) * 0.01):
        # (the second: every choice score is negative; an output outside the kept groups must not win with a zero)
        want_e, want_w = P.route(z.to(F64), corr.to(F64), groups, keep, top, 1.7)
        choice = torch.empty(n, top, dtype=torch.int32, device=DEV)
        weight = torch.empty(n, top, device=DEV)
        routed.route_topk(z.to(DEV), corr.to(DEV), torch.empty(n, R, device=DEV), groups, keep, top, 1.7, choice, weight)
        got_e, got_w = choice.cpu().long(), weight.cpu()
        assert torch.equal(got_e.sort(-1).values, want_e.sort(-1).values)
        assert torch.equal(got_e, want_e)                         # in the order of falling choice score
        assert torch.allclose(got_w.to(F64), want_w, rtol=1e-5, atol=1e-7)
        size = R // groups
        assert int((got_e // size != (got_e // size)[:, :1]).any(-1).sum()) == 0 or keep > 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("R, groups, keep, top, K, n", [(10, 2, 1, 4, 64, 37), (18, 2, 1, 4, 200, 8), (7, 1, 1, 3, 33, 1), (130, 5, 2, 6, 96, 19)])
def test_router_product_and_choice_in_one(dtype, R, groups, keep, top, K, n):
    """The fused kernel against the plain product and choice on the same rows; tokens whose choice is a close call in
    32-bit arithmetic are left out (none of these seeds has more than a few)."""
    from agave_amd.ops import routed
    g = torch.Generator().manual_seed(R + K)
    x = torch.randn(n, K, generator=g).to(dtype)
    router = torch.randn(R, K, generator=g) * K ** -0.5 * 2
    corr = torch.randn(R, generator=g) * 0.05
    z = x.to(F64) @ router.to(F64).T
    want_e, want_w = P.route(z, corr.to(F64), groups, keep, top, 2.0)
    c = torch.softmax(z, -1) + corr.to(F64)
    size = R // groups
    by_group = c.view(n, groups, size).max(-1).values.sort(-1, descending=True).values
    safe = torch.ones(n, dtype=torch.bool) if keep == groups else (by_group[:, keep - 1] - by_group[:, keep] > 1e-5)
    open_ = torch.zeros(n, groups, dtype=torch.bool).scatter_(1, c.view(n, groups, size).max(-1).values.topk(keep).indices, True)
    ranked = c.masked_fill(~open_.repeat_interleave(size, dim=1), -math.inf).sort(-1, descending=True).values[:, :top + 1]
    safe &= (ranked[:, :-1] - ranked[:, 1:]).min(-1).values > 1e-5
    choice = torch.empty(n, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(n, top, device=DEV)
    routed.route_rows(x.to(DEV), router.to(DEV), corr.to(DEV), groups, keep, top, 2.0, choice, weight)
    assert int(safe.sum()) >= n - 3
    assert torch.equal(choice.cpu().long()[safe], want_e[safe])
    assert torch.allclose(weight.cpu().to(F64)[safe], want_w[safe], rtol=2e-4, atol=1e-6)


def test_route_groups_decide_before_the_experts():
    """The single best output lies in a group whose other outputs are poor; with one group kept the choice must
    come from that group all the same (a group counts by its best output), and an output that is second best
    overall but lies in another group is not chosen."""
    from agave_amd.ops import routed
    z = torch.tensor([[5.0, -9.0, -8.0, 4.0, 3.9, 3.8]])
    corr = torch.zeros(6)
    choice = torch.empty(1, 2, dtype=torch.int32, device=DEV)
    weight = torch.empty(1, 2, device=DEV)
    routed.route_topk(z.to(DEV), corr.to(DEV), torch.empty(1, 6, device=DEV), 2, 1, 2, 1.0, choice, weight)
    assert choice.cpu().tolist() == [[0, 2]]
    want_e, _ = P.route(z.to(F64), corr.to(F64), 2, 1, 2, 1.0)
    assert choice.cpu().tolist() == want_e.tolist()
    # the correction moves the choice and not the weight
    corr = torch.tensor([0.0, 0.0, 0.0, 0.9, 0.0, 0.0])
    routed.route_topk(z.to(DEV), corr.to(DEV), torch.empty(1, 6, device=DEV), 2, 1, 2, 1.0, choice, weight)
    s = torch.softmax(z[0].to(F64), -1)
    assert choice.cpu().tolist() == [[3, 4]] and torch.allclose(weight.cpu()[0].to(F64), s[[3, 4]], rtol=1e-5)


# ---------------------------------------------------------------- the experts and their sum
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E, I, top, ff, hidden, n", [(5, 2, 3, 20, 40, 33), (3, 0, 1, 70, 24, 5), (8, 1, 8, 16, 72, 130), (0, 2, 2, 8, 16, 4),
                                                    (6, 1, 2, 136, 200, 300), (4, 2, 3, 256, 128, 70), (3, 1, 2, 96, 160, 200)])
def test_experts_and_their_weighted_sum(dtype, E, I, top, ff, hidden, n):
    from agave_amd.ops import routed
    g = torch.Generator().manual_seed(E * 10 + top)
    rnd = lambda *s: (torch.randn(*s, generator=g) * s[-1] ** -0.5).to(dtype).float()
    x = torch.randn(n, hidden, generator=g).to(dtype).float()
    wg, wu, wd = rnd(max(E, 1), ff, hidden), rnd(max(E, 1), ff, hidden), rnd(max(E, 1), hidden, ff)
    shared = torch.randn(n, hidden, generator=g).to(dtype).float()
    choice = torch.stack([torch.randperm(E + I, generator=g)[:top] for _ in range(n)]).int()
    weight = torch.rand(n, top, generator=g) + 0.1
    want = shared.to(F64).clone()
    w = {}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = wg[e].to(F64), wu[e].to(F64), wd[e].to(F64)
    for t in range(n):
        for e, a in zip(choice[t].tolist(), weight[t].tolist()):
            want[t] += a * (x[t].to(F64) if e >= E else P.gated_expert(w, f"e{e}.", x[t:t + 1].to(F64))[0])
    d = lambda t: t.to(dtype).to(DEV).contiguous()
    y = None
    if E:
        act_rows = torch.empty(n * top, ff, dtype=dtype, device=DEV)
        y = torch.full((n * top, hidden), float("nan"), device=DEV)
        routed.experts_plain(d(x), choice.view(-1).to(DEV), d(wg), d(wu), d(wd), act_rows, y, top, 1)
    out = torch.empty(n, hidden, dtype=dtype, device=DEV)
    routed.combine(y, None, choice.view(-1).to(DEV), weight.view(-1).to(DEV), d(x), d(shared), out, top, E)
    tol = 3e-5 if dtype == torch.float32 else 3e-2
    err = (out.float().cpu().to(F64) - want).abs().max()
    assert float(err) <= tol * float(want.abs().max()), f"error {float(err):.3e}"
    if dtype == torch.bfloat16 and E and routed.mfma_ok(d(x), ff):
        # the same through the pairs sorted by expert and the matrix-core kernels, with both sizes of tile
        for tm in (16, 64):
            tiles = (n * top + tm - 1) // tm + E
            place = torch.full((n * top,), -7, dtype=torch.int32, device=DEV)
            sorted_pair = torch.full((tiles * tm,), -7, dtype=torch.int32, device=DEV)
            tile_expert = torch.full((tiles,), -7, dtype=torch.int32, device=DEV)
            routed.route_sort(choice.view(-1).to(DEV), E, tm, tiles, place, sorted_pair, tile_expert)
            pl, sp, te = place.cpu(), sorted_pair.cpu(), tile_expert.cpu()
            flat = choice.view(-1)
            assert bool(((pl >= 0) == (flat < E)).all())
            for p_ in range(n * top):
                if flat[p_] < E:
                    assert int(sp[pl[p_]]) == p_ and int(te[pl[p_] // tm]) == int(flat[p_])
            assert int((sp >= 0).sum()) == int((flat < E).sum())
            act_rows = torch.empty(tiles * tm, ff, dtype=dtype, device=DEV)
            y2 = torch.full((tiles * tm, hidden), float("nan"), device=DEV)
            routed.experts_mfma(d(x), sorted_pair, tile_expert, d(wg), d(wu), d(wd), act_rows, y2, tm, tiles, top, 1)
            out2 = torch.empty(n, hidden, dtype=dtype, device=DEV)
            routed.combine(y2, place, choice.view(-1).to(DEV), weight.view(-1).to(DEV), d(x), d(shared), out2, top, E)
            err = (out2.float().cpu().to(F64) - want).abs().max()
            assert float(err) <= tol * float(want.abs().max()), f"tiles of {tm}: error {float(err):.3e}"
            if ff % 32 == 0 and hidden % 32 == 0:          # the same with the weights in tile order
                y3 = torch.full((tiles * tm, hidden), float("nan"), device=DEV)
                routed.experts_mfma(d(x), sorted_pair, tile_expert, routed.pack_expert_weights(d(wg)), routed.pack_expert_weights(d(wu)),
                                    routed.pack_expert_weights(d(wd)), act_rows, y3, tm, tiles, top, 1, tile_order=True)
                real = (sorted_pair >= 0)
                assert torch.equal(y3[real], y2[real]), "weights in tile order give other sums"
