"""Each mechanism of the Duperax decoder alone, kernel by kernel, against the plain functions of ``plain_duperax``:
the residual streams' write and read with the norm behind it, the norm over whole q and k rows with the scaled
rotation, the attention with chunks and a cap on the scores (fed whole, in pieces and token by token through the
framework's own cache and step planner, on the plain and the matrix-core kernel), the recurrence's gates and its scan
over ragged batches, and the router that scores by sigmoids and counts a group by its two largest."""
import math

import pytest
import torch

import plain_duperax as P
from test_sequence_kernels_gpu import cuts, feed, planner_for

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F64 = torch.float64


def rel(got, ref):
    return float((got.cpu().to(F64) - ref).abs().max()) / max(float(ref.abs().max()), 1e-30)


# ---------------------------------------------------------------- residual streams
@pytest.mark.parametrize("S, E", [(1, 24), (2, 60), (3, 257), (4, 1000), (8, 40)])
@pytest.mark.parametrize("norm", ["layer", "layer_no_bias", "rms", "none"])
def test_streams_write_then_read(S, E, norm):
    from agave_amd.ops import streams as K
    g = torch.Generator().manual_seed(S * E)
    n, eps = 13, 3e-4
    xs = torch.randn(S, n, E, generator=g) * 3 + 1.5
    mix, write, read = torch.eye(S) + 0.3 * torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
    w, b = 1 + 0.2 * torch.randn(E, generator=g), torch.randn(E, generator=g)
    kind = {"layer": K.NORM_LAYER, "layer_no_bias": K.NORM_LAYER, "rms": K.NORM_RMS, "none": K.NORM_NONE}[norm]

    def normed(u):
        if norm == "none":
            return u
        if norm == "rms":
            return P.row_rms(u, w.to(F64), eps)
        return P.layer_norm(u, w.to(F64), b.to(F64) if norm == "layer" else 0.0, eps)

    def device_streams():
        return xs.permute(1, 0, 2).reshape(n, S * E).contiguous().to(DEV)
    bias = b.to(DEV) if norm == "layer" else None
    for how in ("float32", "bfloat16", "slices"):
        y = torch.randn(n, E, generator=g)
        if how == "bfloat16":
            y = y.bfloat16().float()
        branch = y.to(DEV) if how == "float32" else y.bfloat16().to(DEV) if how == "bfloat16" else \
            torch.stack([0.25 * y, 0.5 * y, 0.25 * y]).to(DEV)
        want_xs = P.streams_write(xs.to(F64), y.to(F64), mix.to(F64), write.to(F64))
        want_out = normed(P.streams_read(want_xs, read.to(F64)))
        for out_dtype in (torch.float32, torch.bfloat16):
            h = device_streams()
            out = torch.empty(n, E, dtype=out_dtype, device=DEV)
            K.step(h, S, E, branch, mix.to(DEV), write.to(DEV), read.to(DEV), kind, w.to(DEV), bias, eps, out)
            assert rel(h.view(n, S, E).permute(1, 0, 2), want_xs) < 1e-6, how
            assert rel(out, want_out) < (2e-5 if out_dtype == torch.float32 else 6e-3), (how, out_dtype)
        # the write alone; then the read alone of chosen rows, which stores nothing
        h = device_streams()
        K.step(h, S, E, branch, mix.to(DEV), write.to(DEV), None, K.NORM_NONE, None, None, 0.0, None)
        assert rel(h.view(n, S, E).permute(1, 0, 2), want_xs) < 1e-6
        rows = torch.tensor([n - 1, 0, 5], dtype=torch.int32, device=DEV)
        out = torch.empty(3, E, dtype=torch.float32, device=DEV)
        before = h.clone()
        K.step(h, S, E, None, None, None, read.to(DEV), kind, w.to(DEV), bias, eps, out, rows=rows)
        assert torch.equal(h, before) and rel(out, want_out[[n - 1, 0, 5]]) < 2e-5
        # chosen rows with a result that is still to be written: the rows see it, the streams stay
        h = device_streams()
        before = h.clone()
        K.step(h, S, E, branch, mix.to(DEV), write.to(DEV), read.to(DEV), kind, w.to(DEV), bias, eps, out, rows=rows)
        assert torch.equal(h, before) and rel(out, want_out[[n - 1, 0, 5]]) < 2e-5
    x0 = torch.randn(n, E, generator=g).to(DEV)
    h = torch.empty(n, S * E, device=DEV)
    K.fill(x0, h, S)
    assert torch.equal(h.view(n, S, E), x0[:, None, :].expand(n, S, E))


# ---------------------------------------------------------------- q and k rows
class Positions:
    def __init__(self, pos):
        self.n_tokens = len(pos)
        self.tok_pos = torch.tensor(pos, dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, G, d, vd, dims, scaling, normed", [
    (4, 2, 16, 8, 8, True, True), (1, 1, 10, 6, 10, False, True), (8, 1, 64, 64, 0, False, True), (3, 3, 12, 20, 4, True, False),
    (5, 5, 128, 32, 128, True, True)])
def test_row_norm_and_rotation(dtype, H, G, d, vd, dims, scaling, normed):
    from agave_amd.config.spec import PositionSpec
    from agave_amd.ops import attention_biased as A
    from agave_amd.parts import BuildEnv, Workspace, lookup
    g = torch.Generator().manual_seed(H * d + dims)
    pos = [0, 1, 2, 63, 64, 65, 1000, 5, 4095, 77, 128]
    n, eps = len(pos), 1e-5
    wide = torch.randn(n, H * d + G * d + G * vd + 3, generator=g) * 2         # the raw rows are column slices
    qw, kw = 1 + 0.3 * torch.randn(H * d, generator=g), 1 + 0.3 * torch.randn(G * d, generator=g)
    rot = {"dims": dims, "base": 300.0}
    if scaling:
        rot["scaling"] = {"factor": 5.0, "original": 40, "fast": 8.0, "slow": 0.5}
    env = BuildEnv(dtype, torch.device(DEV), Workspace(torch.device(DEV)))
    freq, magnitude = None, 1.0
    if dims:
        spec = PositionSpec("rope_yarn", rotary_dim=dims, theta=300.0, yarn_factor=5.0, yarn_original=40, yarn_fast=8.0,
                            yarn_slow=0.5) if scaling else PositionSpec("rope", rotary_dim=dims, theta=300.0)
        part = lookup("position", spec.kind)(spec, env)
        freq, magnitude = part.rotation_table()[0], part.magnitude
        f64, mag = P.yarn_frequencies(rot)
        assert float((freq.cpu() - f64).abs().max()) < 1e-15 and abs(magnitude - mag) < 1e-7
        assert scaling == (magnitude != 1.0)
    raw = wide.to(DEV)
    q, k, v = raw[:, :H * d], raw[:, H * d:H * d + G * d], raw[:, H * d + G * d:H * d + G * d + G * vd]
    q_out = torch.empty(n, H * d, dtype=dtype, device=DEV)
    kv = torch.empty(n, G * d + G * vd, dtype=dtype, device=DEV)
    A.row_norm_rope(q, k, v, q_out, kv[:, :G * d], kv[:, G * d:], qw.to(DEV) if normed else None, kw.to(DEV) if normed else None,
                    eps, eps, freq, magnitude, Positions(pos), H, G, d, vd)
    w64 = wide.to(F64)
    want_q, want_k = w64[:, :H * d], w64[:, H * d:H * d + G * d]
    if normed:
        want_q, want_k = P.row_rms(want_q, qw.to(F64), eps), P.row_rms(want_k, kw.to(F64), eps)
    want_q, want_k = want_q.view(n, H, d), want_k.view(n, G, d)
    if dims:
        want_q, want_k = P.rotate(want_q, torch.tensor(pos), rot), P.rotate(want_k, torch.tensor(pos), rot)
    tol = 2e-6 if dtype == torch.float32 else 6e-3
    assert rel(q_out.view(n, H, d), want_q) < tol and rel(kv[:, :G * d].reshape(n, G, d), want_k) < tol
    assert rel(kv[:, G * d:], w64[:, H * d + G * d:H * d + G * d + G * vd]) < tol
    # biases added on the way, and k and v straight into cache pages: the same rows as the kernel that appends rows puts there
    from agave_amd.cache import GroupKey, KVCache
    from agave_amd.engine.step import StepPlanner
    key = GroupKey(None, G, d, v_head_dim=vd, layout="rows_vt")
    qb, kb, vb = torch.randn(H * d, generator=g), torch.randn(G * d, generator=g), torch.randn(G * vd, generator=g)
    stores = []
    for fused in (True, False):
        cache = KVCache({0: key}, {}, 2, {key: 4}, dtype, torch.device(DEV), 256)
        planner = StepPlanner(cache, 1000, torch.device(DEV))
        step = planner.plan([cache.alloc_slot()], [[0] * n], "all")
        kp, vp, packed = cache.pages_of(0)
        table, base = step.tables[0]
        qo = torch.empty_like(q_out)
        if fused:
            A.row_norm_rope(q, k, v, qo, None, None, qw.to(DEV) if normed else None, kw.to(DEV) if normed else None, eps, eps,
                            freq, magnitude, step, H, G, d, vd, biases=(qb.to(DEV), kb.to(DEV), vb.to(DEV)),
                            pages=(kp, vp, table, base, 0, packed))
        else:
            rows = torch.empty(n, G * d + G * vd, dtype=dtype, device=DEV)
            A.row_norm_rope(q + qb.to(DEV), k + kb.to(DEV), v + vb.to(DEV), qo, rows[:, :G * d], rows[:, G * d:],
                            qw.to(DEV) if normed else None, kw.to(DEV) if normed else None, eps, eps, freq, magnitude, step, H, G, d, vd)
            A.kv_append_rows(rows[:, :G * d], rows[:, G * d:], kp, vp, table, base, 0, step, G, d, vd, packed)
        stores.append((qo.float().cpu(), kp.float().cpu().clone(), vp.float().cpu().clone()))
    for got, ref in zip(*stores):
        assert float((got - ref).abs().max()) <= (1e-6 if dtype == torch.float32 else 2e-2) * max(1.0, float(ref.abs().max()))
    assert float(stores[0][1].abs().max()) > 0
    # a run that appends nothing norms and rotates its queries alone
    q2 = torch.empty_like(q_out)
    A.row_norm_rope(q, None, None, q2, None, None, qw.to(DEV) if normed else None, None, eps, eps, freq, magnitude,
                    Positions(pos), H, G, d, vd)
    assert torch.equal(q2, q_out)


# ---------------------------------------------------------------- attention: chunks and a cap on the scores
class Case:
    def __init__(self, H, G, d, vd, window, chunk, softcap, T, seed=0, big=1.0):
        g = torch.Generator().manual_seed(seed)
        self.H, self.G, self.d, self.vd, self.window, self.chunk, self.softcap, self.T = H, G, d, vd, window, chunk, softcap, T
        self.q = torch.randn(T, H, d, generator=g) * big           # (big: scores that the cap bends)
        self.k = torch.randn(T, G, d, generator=g)
        self.v = torch.randn(T, G, vd, generator=g)
        self.scale = 0.7 * d ** -0.5
        self.force_plain = False

    def rounded(self, dtype):
        for name in ("q", "k", "v"):
            setattr(self, name, getattr(self, name).to(dtype).float())

    def plain(self):
        T = self.T
        i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
        see = j <= i
        if self.window is not None:
            see &= P.visible("attention", self.window, T)
        if self.chunk is not None:
            see &= P.visible("attention_2", self.chunk, T)
        return P.softmax_attention(self.q.to(F64), self.k.to(F64), self.v.to(F64), self.scale, see, self.softcap or None).reshape(T, -1)

    def run(self, ranges, dtype):
        from agave_amd.cache import GroupKey, KVCache
        from agave_amd.engine.step import StepPlanner
        from agave_amd.ops import attention_biased as A
        from agave_amd.parts import Workspace
        key = GroupKey(self.window, self.G, self.d, chunk=self.chunk, v_head_dim=self.vd, layout="rows_vt")
        cache = KVCache({0: key}, {}, 3, {key: 12}, dtype, torch.device(DEV), 2048)
        planner = StepPlanner(cache, 1000, torch.device(DEV))
        cache.alloc_slot()
        slot = cache.alloc_slot()
        ws = Workspace(torch.device(DEV))
        got = torch.zeros(self.T, self.H * self.vd)
        for lo, hi in ranges:
            step = planner.plan([slot], [[0] * (hi - lo)], "all")
            kp, vp, packed = cache.pages_of(0)
            table, base = step.tables[0]
            dev = lambda t: t[lo:hi].reshape(hi - lo, -1).to(dtype).to(DEV).contiguous()
            A.kv_append_rows(dev(self.k), dev(self.v), kp, vp, table, base, 0, step, self.G, self.d, self.vd, packed)
            out = torch.empty(hi - lo, self.H * self.vd, dtype=dtype, device=DEV)
            A.attention(dev(self.q), out, None, kp, vp, table, base, 0, step, self.H, self.G, self.d, self.vd, self.scale,
                        self.window, 0, A.BIAS_NONE, None, None, packed, force_plain=self.force_plain, workspace=ws,
                        chunk=self.chunk, softcap=self.softcap)
            planner.commit(step)
            got[lo:hi] = out.float().cpu()
        cache.free_slot(slot)
        assert cache.groups[0].pool.n_free == cache.groups[0].pool.n_pages      # (pages of chunks that are over came back on the way)
        return got


def close(got, ref, dtype, what):
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    err = (got.to(F64) - ref).abs().max()
    assert float(err) <= tol * max(1.0, float(ref.abs().max())), f"{what}: error {float(err):.3e}"


SHAPES = [
    # H, G, d, vd, window, chunk, softcap, big
    (4, 2, 16, 8, None, 50, 12.0, 6.0),           # a chunk shorter than a page, capped scores
    (6, 1, 48, 48, None, 96, 5.0, 8.0),           # a chunk over page borders; the matrix cores in bfloat16
    (8, 2, 64, 32, None, 64, 0.0, 1.0),           # a chunk of exactly a page, no cap
    (3, 3, 20, 12, None, 7, 30.0, 1.0),           # sizes the matrix cores do not take
    (2, 1, 32, 64, 40, 100, 2.0, 10.0),           # a window inside chunks, a cap that bends every score
    (5, 5, 128, 128, None, 130, 20.0, 3.0),       # the sizes of large models
    (2, 2, 16, 16, None, 1, 0.0, 1.0),            # every token its own chunk
    (4, 4, 32, 32, 70, None, 15.0, 5.0),          # a window with capped scores
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_with_chunks_and_capped_scores(shape, dtype):
    T = 300
    c = Case(*shape[:7], T=T, seed=len(str(shape)), big=shape[7])
    c.rounded(dtype)
    ref = c.plain()
    if c.softcap:
        uncapped = Case(*shape[:6], 0.0, T=T, seed=len(str(shape)), big=shape[7])
        uncapped.rounded(dtype)
        assert float((uncapped.plain() - ref).abs().max()) > 1e-3          # the cap matters with these inputs
    for first, piece in ((T, 1), (200, 1), (1, 1), (3, 2), (50, 37), (64, 64), (97, 150)):
        close(c.run(cuts(T, first, piece), dtype), ref, dtype, f"{shape} first {first} pieces of {piece}")
    if dtype == torch.bfloat16:
        c.force_plain = True
        close(c.run(cuts(T, 180, 1), dtype), ref, dtype, f"{shape} on the plain kernel")


# ---------------------------------------------------------------- the recurrence
@pytest.mark.parametrize("W, blocks", [(48, 3), (32, 1), (160, 2), (36, 4), (256, 1), (70, 70)])
@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
def test_recurrence_gates(W, blocks, wdtype):
    from agave_amd.ops import rglru as R
    g = torch.Generator().manual_seed(W)
    bw = W // blocks
    w_r, w_i = (torch.randn(blocks, bw, bw, generator=g) * bw ** -0.5).to(wdtype), (torch.randn(blocks, bw, bw, generator=g) * bw ** -0.5).to(wdtype)
    b_r, b_i, lam = torch.randn(blocks, bw, generator=g), torch.randn(blocks, bw, generator=g), torch.randn(W, generator=g) * 2 - 2
    for n in (75, 1, 9, 16, 17, 64, 65):               # steps of up to 64 tokens run a kernel of their own
        wide = torch.randn(n, W + 5, generator=g) * 1.5
        want_a, want_x = P.rglru_gates(wide[:, 2:2 + W].to(F64).contiguous(), w_r.to(F64), b_r.to(F64), w_i.to(F64), b_i.to(F64), lam.to(F64), c=6.0)
        decay = (6.0 * torch.nn.functional.softplus(lam.to(F64))).float().to(DEV)
        a, x = torch.empty(n, W, device=DEV), torch.empty(n, W, device=DEV)
        R.gates(wide.to(DEV)[:, 2:2 + W], w_r.to(DEV), w_i.to(DEV), b_r.reshape(-1).to(DEV), b_i.reshape(-1).to(DEV), decay, a, x)
        # (bfloat16 matrices with blocks the matrix cores take: the inputs enter as two bfloat16 numbers, exact to 2^-16)
        split = wdtype == torch.bfloat16 and bw % 32 == 0 and n > 64
        assert rel(a, want_a) < (2e-5 if split else 3e-6) and rel(x, want_x) < (5e-5 if split else 1e-5), n
    want_a, want_x = P.rglru_gates(wide[:, 2:2 + W].to(F64).contiguous(), w_r.to(F64), b_r.to(F64), w_i.to(F64), b_i.to(F64), lam.to(F64), c=6.0)
    decay = (6.0 * torch.nn.functional.softplus(lam.to(F64))).float().to(DEV)
    a, x = torch.empty(n, W, device=DEV), torch.empty(n, W, device=DEV)
    R.gates(wide.to(DEV)[:, 2:2 + W], w_r.to(DEV), w_i.to(DEV), b_r.reshape(-1).to(DEV), b_i.reshape(-1).to(DEV), decay, a, x)
    assert rel(a, want_a) < 3e-6 and rel(x, want_x) < 1e-5
    # sqrt(1 - a^2) where a is within rounding of 1: the gated input does not vanish before its time
    small = torch.full((W,), -16.0)
    decay = (6.0 * torch.nn.functional.softplus(small.to(F64))).float().to(DEV)
    want_a, want_x = P.rglru_gates(wide[:, 2:2 + W].to(F64).contiguous(), w_r.to(F64), b_r.to(F64), w_i.to(F64), b_i.to(F64), small.to(F64), c=6.0)
    R.gates(wide.to(DEV)[:, 2:2 + W], w_r.to(DEV), w_i.to(DEV), b_r.reshape(-1).to(DEV), b_i.reshape(-1).to(DEV), decay, a, x)
    assert float(want_a.min()) > 1 - 1e-6 and rel(x, want_x) < 1e-4


@pytest.mark.parametrize("W", [37, 256, 700])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_recurrence_scan_whole_pieces_tokens_and_ragged_batches(W, dtype):
    """Sequences fed whole, in pieces and token by token, alone and three together with unequal counts (a sequence's
    rows start anywhere inside the kernel's chunks of rows), through slots that were used before."""
    from agave_amd.cache import StateNeed
    from agave_amd.ops import rglru as R
    from agave_amd.parts import Workspace
    g = torch.Generator().manual_seed(W)
    lens = [150, 29, 77]
    a = [torch.rand(T, W, generator=g) ** 0.2 for T in lens]
    x = [torch.randn(T, W, generator=g) for T in lens]
    y = [torch.randn(T, W + 3, generator=g) for T in lens]
    yb = torch.randn(W, generator=g)
    want = [P.linear_scan(ai.to(F64), xi.to(F64)) * P.gelu_tanh(yi[:, 1:1 + W].to(F64) + yb.to(F64)) for ai, xi, yi in zip(a, x, y)]
    ws = Workspace(torch.device(DEV))
    tol = 1e-5 if dtype == torch.float32 else 6e-3

    def run(cache, planner, slots, members, ranges):
        """``ranges[i]``: the row ranges that sequence ``members[i]`` brings, step by step (None: it has ended)."""
        got = [torch.zeros(lens[m], W) for m in members]
        for r in range(max(len(x) for x in ranges)):
            live = [i for i in range(len(members)) if r < len(ranges[i])]
            step = feed(cache, planner, [slots[i] for i in live], [ranges[i][r][1] - ranges[i][r][0] for i in live])
            cat = lambda ts: torch.cat([ts[members[i]][ranges[i][r][0]:ranges[i][r][1]] for i in live]).to(DEV).contiguous()
            out = torch.empty(step.n_tokens, W, dtype=dtype, device=DEV)
            R.scan(cat(a), cat(x), cat(y)[:, 1:1 + W], out, cache.state[0], step, ws, y_bias=yb.to(DEV))
            planner.commit(step)
            at = 0
            for i in live:
                lo, hi = ranges[i][r]
                got[i][lo:hi] = out[at:at + hi - lo].float().cpu()
                at += hi - lo
        return got
    for first, piece in ((10 ** 6, 1), (11, 1), (1, 1), (5, 2), (33, 40), (100, 31)):
        cache, planner = planner_for(state={0: StateNeed((W,))}, slots=4)
        cache.alloc_slot()
        for m in range(3):                                                     # each alone; the slot is used again
            slot = cache.alloc_slot()
            got = run(cache, planner, [slot], [m], [cuts(lens[m], min(first, lens[m]), piece)])
            assert rel(got[0], want[m]) < tol, (first, piece, m)
            cache.free_slot(slot)
        slots = [cache.alloc_slot() for _ in range(3)]                         # together: prompts of unequal lengths, then one token each
        firsts = [min(first, lens[m] - 1) if piece == 1 else lens[m] for m in range(3)]
        got = run(cache, planner, slots, [0, 1, 2], [cuts(lens[m], firsts[m], 1) for m in range(3)])
        for m in range(3):
            assert rel(got[m], want[m]) < tol, (first, piece, m, "together")


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_convolution_with_a_bias_on_its_inputs(taps):
    """The bias of the product that made the convolution's inputs is added on the way in: to every input of the
    sequence, not to the zeros before its start, whole, in pieces (also shorter than the taps) and token by token."""
    from agave_amd.cache import StateNeed
    from agave_amd.ops import sequence as S
    C, T = 37, 29
    g = torch.Generator().manual_seed(taps)
    u, w = torch.randn(T, C, generator=g), torch.randn(C, taps, generator=g)
    b_in, b_out = torch.randn(C, generator=g), torch.randn(C, generator=g)
    ref = P.causal_conv(u.to(F64) + b_in.to(F64), w.to(F64), b_out.to(F64))
    for first, piece in ((T, 1), (11, 1), (5, 2), (1, 3), (2, 9)):
        cache, planner = planner_for(state={0: StateNeed((taps - 1, C))})
        cache.alloc_slot()
        slot = cache.alloc_slot()
        got = torch.zeros(T, C)
        for lo, hi in cuts(T, first, piece):
            step = feed(cache, planner, [slot], [hi - lo])
            y = torch.empty(hi - lo, C, device=DEV)
            S.short_conv(u[lo:hi].to(DEV).contiguous(), w.to(DEV), y, cache.state[0], step, False, b_out.to(DEV), b_in.to(DEV))
            planner.commit(step)
            got[lo:hi] = y.cpu()
        assert rel(got, ref) < 1e-5, (first, piece)


# ---------------------------------------------------------------- the router
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts, top, groups, keep, width", [(8, 3, 4, 3, 64), (6, 2, 3, 2, 40), (5, 3, 5, 4, 60), (4, 4, 1, 1, 24),
                                                              (1, 1, 1, 1, 32), (64, 6, 8, 3, 128), (12, 5, 2, 1, 72)])
def test_router_with_sigmoid_scores_and_groups_by_their_two_largest(dtype, experts, top, groups, keep, width):
    from agave_amd.ops import routed as R
    g = torch.Generator().manual_seed(experts * width)
    n = 90
    x = torch.randn(n, width, generator=g).to(dtype)
    router = torch.randn(experts, width, generator=g) * width ** -0.5 * 2
    corr = torch.randn(experts, generator=g) * 0.5 - 0.3                        # choice scores of both signs
    f = {"router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}
    w = {"r.router": router.to(F64), "r.correction": corr.to(F64)}
    idx, wt = P.route(x.to(F64), w, "r.", f)
    # the margin by which the plain choice was made: rows where rounding could change it are compared by weight only
    choice = torch.empty(n, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(n, top, dtype=torch.float32, device=DEV)
    R.route_rows(x.to(DEV), router.to(DEV), corr.to(DEV), groups, keep, top, 1.0, choice, weight, sigmoid=True, group_top=2,
                 normalise=True)
    got_sets = [sorted(r) for r in choice.cpu().tolist()]
    want_sets = [sorted(r) for r in idx.tolist()]
    same = [a == b for a, b in zip(got_sets, want_sets)]
    assert sum(same) >= n - 1, f"{n - sum(same)} rows chose other experts"
    assert float((weight.sum(-1).cpu() - 1).abs().max()) < 1e-5
    for t in range(n):
        if same[t]:
            order = {e: i for i, e in enumerate(idx[t].tolist())}
            got_w = torch.zeros(top, dtype=F64)
            for e, v in zip(choice[t].cpu().tolist(), weight[t].cpu().tolist()):
                got_w[order[e]] = v
            assert float((got_w - wt[t]).abs().max()) < 2e-6
