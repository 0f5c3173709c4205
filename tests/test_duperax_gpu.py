"""The Duperax decoder through the engine, against ``plain_duperax``: whole prompts, decoding token by token, prompts
in pieces down to two tokens, batches of unequal requests, slots and pages used again, long decoding across page
borders, windows' and chunks' edges with a key made to stand out, an early token kept in a recurrence's state, other
sizes (also ones where the usual sizes coincide or are 1), the residual after every layer run, greedy generation
through the engine's entry point, the command line and the trace replay tool."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import engine_utils as U
import plain_duperax as P

pytestmark = pytest.mark.gpu

CONFIGS = {
    # all three mixers, both feed-forwards and none; three streams; the two middle layers run twice; key and value
    # heads of different sizes; a rotation of half a head; a chunk and a window that are no multiples of a page
    "mixed": lambda: P.config([
        P.attention2_layer(4, 2, 16, 8, 50, 8, base=500.0, factor=3.0, original=32, fast=16.0, slow=2.0, softcap=12.0,
                           mlp=P.moe(6, 2, 3, 2, 24)),
        P.rglru_layer(48, 3, 3, mlp=P.dense(56, limit=1.2)),
        P.attention_layer(3, 3, 8, 24, 37, mlp=None),
        P.rglru_layer(32, 1, 1, mlp=P.moe(4, 4, 1, 1, 16))],
        vocab=131, width=40, eps=2e-6, streams=3, loop=(1, 3, 2)),
    # a width that is no multiple of 8 (no matrix-core packing), one ordinary residual, no loop, a window of one
    # position, a chunk shorter than a page, a plain rotation of whole heads without a cap, one head, one expert
    "odd": lambda: P.config([
        P.attention_layer(1, 1, 10, 6, 1, mlp=P.moe(1, 1, 1, 1, 20)),
        odd_second(),
        P.rglru_layer(36, 4, 7, mlp=None),
        P.attention_layer(6, 2, 4, 2, 200, scale=0.9, mlp=P.dense(30, limit=0.4))], vocab=97, width=60, eps=1e-3, streams=None,
        logit_scale=1.0),
    # sizes the matrix cores take everywhere; two streams; the whole model runs twice; a window of exactly a page
    "even": lambda: P.config([
        P.attention_layer(8, 2, 32, 32, 64, mlp=P.moe(8, 2, 1, 1, 64)),
        P.attention2_layer(4, 4, 64, 16, 128, 32, factor=8.0, original=64, mlp=P.dense(256, limit=2.0)),
        P.rglru_layer(256, 2, 4, mlp=P.moe(8, 3, 4, 2, 32))], vocab=256, width=128, streams=2, loop=(0, 3, 2)),
    # one stream that is still mixed (1 x 1 coefficients), a loop that runs once
    "one": lambda: P.config([
        P.rglru_layer(16, 2, 2, mlp=P.dense(24, limit=5.0)),
        P.attention2_layer(2, 1, 8, 8, 33, 8, factor=1.5, original=16, softcap=3.0, mlp=None)],
        vocab=61, width=24, streams=1, loop=(0, 1, 1)),
}


def odd_second():
    layer = P.attention2_layer(5, 1, 12, 12, 7, 12, base=77.0, mlp=P.moe(5, 3, 5, 4, 8))
    del layer["mixer"]["rot"]["scaling"], layer["mixer"]["softcap"]
    return layer


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    made = {}

    def get(name, decided=False):
        if (name, decided) not in made:
            cfg = CONFIGS[name]()
            w = P.random_weights(cfg, seed=len(name), decided_routing=decided)
            folder = U.write_model(str(tmp_path_factory.mktemp(name)), cfg, w)
            made[(name, decided)] = (cfg, w, folder)
        return made[(name, decided)]
    return get


def engine(folder, dtype, **kw):
    from agave_amd.engine import Engine
    kw.setdefault("max_slots", 4)
    kw.setdefault("max_context", 512)
    return Engine.from_folder(folder, dtype=dtype, **kw)


def close(got, ref, dtype, what):
    """32-bit: every row within 3e-5 of the largest logit.  bfloat16: 4 % of the largest logit for all rows but one
    in twenty, twice that for those."""
    scale = float(ref.abs().max())
    err = (got.double() - ref).abs().max(dim=-1).values
    where = f"{what}: error {float(err.max()):.3e} of {scale:.3e} at row {int(err.argmax())}"
    if dtype == "float32":
        assert float(err.max()) <= 3e-5 * scale, where
    else:
        assert float(err.max()) <= 0.08 * scale, where
        assert int((err > 0.04 * scale).sum()) <= max(1, len(err) // 20), where


def model_for(models, name, dtype):
    # in bfloat16 the choice of experts is decided by the routers' corrections (a close call would go either way)
    return models(name, decided=(dtype == "bfloat16"))


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_tail_and_pieces(models, name, dtype):
    cfg, w, folder = model_for(models, name, dtype)
    eng = engine(folder, dtype)
    toks = U.random_tokens(200, cfg["vocab"], 1)
    ref = P.forward(cfg, w, toks)
    close(U.run_whole(eng, toks), ref, dtype, "whole")
    close(U.run_tail(eng, toks, 150), ref, dtype, "the last 150 one by one, across page, window and chunk borders")
    close(U.run_tail(eng, toks, 199), ref, dtype, "token by token from the first")
    for piece in (2, 7, 64, 100):                 # the prompt enters in pieces of this many tokens
        eng.prefill_chunk = piece
        close(U.run_whole(eng, toks[:170]), ref[:170], dtype, f"pieces of {piece}")
    eng.prefill_chunk = 0
    assert eng.cache.slots.n_free == eng.cache.max_slots
    assert all(g.pool.n_free == g.pool.n_pages for g in eng.cache.groups)


def test_residual_after_every_layer_run(models):
    """The streams' sum after each run of a layer (a looped layer counts each time), read off the engine between its
    blocks: a block's last result is still pending when the next block starts, so it is written into a copy first."""
    from agave_amd.parts.streams import write_and_read
    cfg, w, folder = models("mixed")
    eng = engine(folder, "float32")
    eng.use_graphs = False
    toks = U.random_tokens(90, cfg["vocab"], 4)
    want = []
    P.forward(cfg, w, toks, layers_out=want)
    seen, S, E = [], cfg["streams"], cfg["width"]
    for b in eng.model.blocks:
        def wrapped(h, pending, step, memory, writes, inner=b.forward):
            if pending is not None:
                copy = h.clone()
                write_and_read(copy, S, E, pending, None, None, None)
                seen.append(copy.view(-1, S, E).sum(1).cpu())
            return inner(h, pending, step, memory, writes)
        b.forward = wrapped
    U.run_whole(eng, toks)
    assert len(seen) == len(want) - 1 == len(P.run_order(cfg)) - 1
    for i, (got, ref) in enumerate(zip(seen, want)):
        assert float((got.double() - ref).abs().max()) < 3e-5 * float(ref.abs().max()), f"after layer run {i}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batches_of_unequal_requests_and_slots_used_again(models, dtype):
    """Three batches one after another over the same three slots, through pools of pages that only hold them because
    pages come back; the recurrences' states start at zero again in a slot that is used again."""
    cfg, w, folder = model_for(models, "mixed", dtype)
    eng = engine(folder, dtype, max_slots=3, max_context=256, cache_tokens=448)
    for b, (lens, first) in enumerate([((50, 1, 130), (30, 1, 2)), ((70, 33), (69, 1)), ((90, 9, 140), (5, 9, 101))]):
        reqs = [U.random_tokens(n, cfg["vocab"], 10 * b + i) for i, n in enumerate(lens)]
        outs = U.run_batched(eng, reqs, first)
        for i, (r, o) in enumerate(zip(reqs, outs)):
            close(o, P.forward(cfg, w, r), dtype, f"batch {b} request {i}")
    assert eng.cache.slots.n_free == eng.cache.max_slots
    assert all(g.pool.n_free == g.pool.n_pages for g in eng.cache.groups)


def test_the_cache_as_the_mixers_asked(models):
    cfg, w, folder = models("mixed")
    eng = engine(folder, "float32")
    order = P.run_order(cfg)
    assert order == [0, 1, 2, 1, 2, 3]
    # every run of a layer has its own memory: the attention layers' runs 0, 2 and 4 hold pages, the others state
    assert set(eng.cache.group_of_memory) == {0, 2, 4} and set(eng.cache.state) == {1, 3, 5}
    keys = {m: eng.cache.group_keys[g] for m, g in eng.cache.group_of_memory.items()}
    assert (keys[0].chunk, keys[0].window, keys[0].n_kv_heads, keys[0].head_dim, keys[0].v_head_dim) == (50, None, 2, 16, 8)
    assert keys[2] == keys[4] and (keys[2].window, keys[2].chunk, keys[2].head_dim, keys[2].v_head_dim) == (37, None, 8, 24)
    assert tuple(eng.cache.state[1]["S"].shape[1:]) == (48,) and tuple(eng.cache.state[1]["conv"].shape[1:]) == (2, 48)
    assert tuple(eng.cache.state[5]["conv"].shape[1:]) == (0, 32) and eng.cache.state[3]["S"].dtype == torch.float32
    from agave_amd.ops import library
    slot = eng.alloc_slot()
    eng.step([slot], [[1, 2]])
    eng.free_slot(slot)
    loaded = library.loaded_paths()
    for name in ("streams.so", "rglru.so", "attention_biased.so", "routed_ffn.so", "sequence.so"):
        assert any(p.endswith(name) for p in loaded), name


def test_long_decoding(models):
    cfg, w, folder = models("even")
    eng = engine(folder, "float32", max_slots=1, max_context=1024, cache_tokens=64 * 11)
    toks = U.random_tokens(700, cfg["vocab"], 9)
    ref = P.forward(cfg, w, toks)
    close(U.run_tail(eng, toks, 500), ref, "float32", "500 tokens decoded")


VOCAB_NEEDLE = 40


def needle_model(kind: str, size: int, boost=30.0, value=25.0):
    """One attention layer whose head 0 is made to look for one token: token ``A``'s key is turned towards token
    ``Q``'s query (in ``attention_2`` only in the elements that are not rotated) and its value is made large, so that
    the logits at a ``Q`` change much with whether ``A`` is seen.  A layer's input is a function of the token alone in
    a model of one layer, and there are fewer tokens than the width: the key and value matrices are changed along the
    part of ``A``'s input that is orthogonal to every other token's, so no other token's key or value moves."""
    A, Q = 0, 1
    if kind == "attention":
        layer = P.attention_layer(2, 1, 16, 8, size, scale=1.0)
    else:
        layer = P.attention2_layer(2, 1, 16, 8, size, 8, factor=2.0, original=16, softcap=50.0, scale=1.0)
    cfg = P.config([layer], vocab=VOCAB_NEEDLE, width=64, streams=2)
    w = P.random_weights(cfg, 3)
    eps = cfg["norm"]["eps"]
    u = w["embed"] * float(w["l0.hc1.in"].sum())
    h = P.layer_norm(u, w["l0.norm1"], w["l0.norm1.b"], eps)                 # [vocab, width]: every token's input
    others = h[1:]
    coef = torch.linalg.lstsq(others.T, h[A][:, None]).solution[:, 0]
    d = h[A] - others.T @ coef                                              # orthogonal to every other token's input
    d = d / float(d @ h[A])
    q = h[Q] @ w["l0.mix.q"].T + (w["l0.mix.q.b"] if kind == "attention_2" else 0.0)
    q0 = P.row_rms(q, w["l0.mix.q.norm"], eps)[:16].clone()
    if kind == "attention_2":
        q0[:8] = 0.0
    w["l0.mix.k"] = w["l0.mix.k"] + boost * torch.outer(q0 / q0.norm(), d)      # (kept in double: the tests hand the engine these values rounded)
    w["l0.mix.v"] = w["l0.mix.v"] + value * torch.outer(torch.ones(8, dtype=P.F), d)
    for n in ("l0.mix.k", "l0.mix.v"):
        w[n] = w[n].to(torch.float32).to(P.F)
    return cfg, w, A, Q


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind, size", [("attention", 70), ("attention", 64), ("attention", 300), ("attention_2", 96), ("attention_2", 64), ("attention_2", 50)])
def test_a_key_at_the_edges_of_windows_and_chunks(dtype, kind, size):
    """The key that the last queries look for stands just inside and just outside what the last query sees (the
    window's far end; the chunk's first position and the one before it), at the query's own place, at page borders,
    and at the sequence's first positions; the queries come in the prompt, in pieces of it, and decoded one by one."""
    from agave_amd.engine import Engine
    cfg, w, A, Q = needle_model(kind, size)
    # (the changed matrices are handed over in 32-bit, so that the orthogonal direction survives; a bfloat16 engine casts them)
    eng = Engine.from_tensors(cfg, {k: v.float() for k, v in w.items()}, dtype=dtype, max_slots=2, max_context=512,
                              keep_stored_precision=False)
    T = 430
    last = T - 1
    if kind == "attention":
        inside, outside = last - size + 1, last - size
    else:
        inside, outside = (last // size) * size, (last // size) * size - 1
    places = {inside: True, outside: False, last - 1: True, 0: False, 1: False, 63: False, 64: False}
    if kind == "attention" and size == 300:
        places.update({191: True, 192: True, 255: True, 256: True})
    moved_when_seen = []
    for at, seen in places.items():
        toks = [2 + t % (VOCAB_NEEDLE - 2) for t in U.random_tokens(T, 1000, at + 5)]
        toks[-1] = Q
        toks[at] = A
        without = list(toks)
        without[at] = 7
        ref, ref_without = P.forward(cfg, w, toks), P.forward(cfg, w, without)
        scale = float(ref.abs().max())
        moved = float((ref[-1] - ref_without[-1]).abs().max())
        if seen:
            assert moved > 0.1 * scale, (at, moved, scale)
            moved_when_seen.append(moved)
        else:
            assert moved < 1e-9 * scale, (at, moved, scale)
        eng.prefill_chunk = 0
        runs = {"whole": U.run_whole(eng, toks), "decoded": U.run_tail(eng, toks, 100 if at < 200 else T - at + 3)}
        eng.prefill_chunk = 50
        runs["pieces"] = U.run_whole(eng, toks)
        for what, got in runs.items():
            close(got, ref, dtype, f"key at {at}, {what}")
            if seen:
                assert float((got[-1].double() - ref[-1]).abs().max()) < (0.002 if dtype == "float32" else 0.25) * moved, (at, what)
    assert moved_when_seen


def test_an_early_token_stays_in_the_state():
    """A recurrence that forgets slowly: a change of the third token moves the logits 400 tokens later, and the engine
    follows, decoding or not, in pieces or whole."""
    from agave_amd.engine import Engine
    cfg = P.config([P.rglru_layer(32, 2, 3, mlp=None)], vocab=60, width=32, streams=2)
    w = P.random_weights(cfg, 3)
    w["l0.mix.lam"] = torch.full((32,), -9.0, dtype=P.F)             # almost nothing is forgotten
    eng = Engine.from_tensors(cfg, {k: v.bfloat16() for k, v in w.items()}, dtype="float32", max_slots=2, max_context=512)
    toks = U.random_tokens(430, 60, 3)
    other = list(toks)
    other[2] = (toks[2] + 11) % 60
    ref, ref_other = P.forward(cfg, w, toks), P.forward(cfg, w, other)
    moved = float((ref[-1] - ref_other[-1]).abs().max())
    assert moved > 1e-3 * float(ref.abs().max())
    for t, r in ((toks, ref), (other, ref_other)):
        got = U.run_tail(eng, t, 40)
        assert float((got[-1].double() - r[-1]).abs().max()) < 0.02 * moved
        close(got, r, "float32", "state")
        eng.prefill_chunk = 33
        close(U.run_whole(eng, t), r, "float32", "state, pieces of 33")
        eng.prefill_chunk = 0


def random_config(seed: int) -> dict:
    """A configuration drawn from a seed: two to five layers of any kind and order, head counts and sizes that the
    matrix cores take and ones they do not, windows and chunks around page borders, rotations of a part of a head,
    blocks of the recurrence from 8 to 128 channels, one to eight streams or one ordinary residual, with or without
    a stretch of layers that runs again."""
    import random
    rng = random.Random(seed)
    layers = []
    n_layers = rng.randint(2, 5)
    for _ in range(n_layers):
        kind = rng.choice(["attention", "attention_2", "rglru"])
        r = rng.random()
        if r < 0.2:
            mlp = None
        elif r < 0.55:
            mlp = P.dense(rng.choice([64, 96, 200]), limit=rng.choice([0.5, 1.5, 7.0]))
        else:
            groups, per = rng.choice([1, 2, 3, 4]), rng.choice([1, 2, 3, 4])
            keep = rng.randint(1, groups)
            mlp = P.moe(groups * per, rng.randint(1, min(keep * per, 6)), groups, keep, rng.choice([32, 48, 96]))
        if kind == "rglru":
            blocks = rng.choice([1, 2, 4, 5, 8])
            layers.append(P.rglru_layer(blocks * rng.choice([8, 20, 32, 64, 128]), blocks, rng.randint(1, 6), mlp=mlp))
            continue
        kv = rng.choice([1, 1, 2, 3, 4])
        heads, dim = kv * rng.choice([1, 2, 3, 4, 8]), rng.choice([8, 16, 24, 48, 64, 80, 128, 20, 36])
        vdim = rng.choice([dim, 16, 32, 48, 24, 40])
        size = rng.choice([1, 2, 7, 31, 63, 64, 65, 72, 100, 127, 128, 129, 200, 400])
        scale = rng.choice([dim ** -0.5, 0.125, 1.7 * dim ** -0.5])
        if kind == "attention":
            layers.append(P.attention_layer(heads, kv, dim, vdim, size, scale=scale, mlp=mlp))
        else:
            dims = max(2, rng.choice([dim, dim // 2, 2, dim - dim // 4]) // 2 * 2)
            layers.append(P.attention2_layer(heads, kv, dim, vdim, max(size, 2), dims, base=rng.choice([100.0, 1e4, 1e6]),
                                             factor=rng.choice([1.0, 2.0, 8.0, 32.0]), original=rng.choice([16, 64, 1024, 4096]),
                                             fast=rng.choice([32.0, 4.0]), slow=rng.choice([1.0, 0.5]),
                                             softcap=rng.choice([5.0, 25.0, 50.0]), scale=scale, mlp=mlp))
    loop = None
    if rng.random() < 0.6:
        a = rng.randint(0, n_layers - 1)
        loop = (a, rng.randint(a, n_layers), rng.randint(1, 3))
    return P.config(layers, vocab=rng.choice([97, 256, 1000]), width=rng.choice([64, 96, 128, 160, 320, 72, 100]),
                    eps=rng.choice([1e-6, 1e-5]), streams=rng.choice([None, 1, 2, 3, 4, 5, 8]), loop=loop,
                    logit_scale=rng.choice([0.5, 1.0, 2.0]))


@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15, 16])
def test_configurations_drawn_at_random(seed):
    from agave_amd.engine import Engine
    cfg = random_config(seed)
    toks = U.random_tokens(330, cfg["vocab"], seed)
    others = [U.random_tokens(n, cfg["vocab"], seed + 100 + n) for n in (1, 150)]
    for dtype in ("float32", "bfloat16"):
        w = P.random_weights(cfg, seed, decided_routing=(dtype == "bfloat16"))
        eng = Engine.from_tensors(cfg, {k: v.bfloat16() for k, v in w.items()}, dtype=dtype, max_slots=3, max_context=512)
        ref = P.forward(cfg, w, toks)
        close(U.run_tail(eng, toks, 140), ref, dtype, f"{cfg}: tail")
        outs = U.run_batched(eng, [toks] + others, (300, 1, 100))
        for o, r in zip(outs, [ref] + [P.forward(cfg, w, t) for t in others]):
            close(o, r, dtype, f"{cfg}: in a batch")


@pytest.mark.parametrize("dtype", ["float32"])
def test_greedy_generation_through_the_entry_point(models, dtype):
    from agave_amd.sampling import SamplingParams
    cfg, w, folder = models("mixed")
    eng = engine(folder, dtype, max_slots=2, max_context=128)
    prompts = [U.random_tokens(7, cfg["vocab"], 50), U.random_tokens(45, cfg["vocab"], 51), U.random_tokens(1, cfg["vocab"], 52)]
    res = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=8))      # three requests, two slots: a slot is used again
    for p, r in zip(prompts, res):
        seq = list(p)
        for _ in range(8):
            seq.append(P.argmax_first(P.forward(cfg, w, seq)[-1]))
        assert list(r.tokens) == seq[len(p):]


def test_command_line_and_trace_replay(models, tmp_path):
    cfg, w, folder = models("odd", decided=True)
    root = U.ROOT
    out = subprocess.run([sys.executable, os.path.join(root, "bin", "agave_amd"), folder, "3 17 5 80 2", "-n", "5", "--dtype", "float32",
                          "--json"], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    seq = [3, 17, 5, 80, 2]
    for _ in range(5):
        seq.append(P.argmax_first(P.forward(cfg, w, seq)[-1]))
    got = json.loads(out.stdout.strip().splitlines()[-1])
    assert got["outputs"][0]["tokens"] == seq[5:] and got["outputs"][0]["prompt_tokens"] == 5
    batches = [[U.random_tokens(n, cfg["vocab"], 70 + n) for n in (40, 3, 110)], [U.random_tokens(n, cfg["vocab"], 90 + n) for n in (25, 60)]]
    firsts = [(8, 3, 78), (1, 59)]
    records, where = U.trace_steps_batched(batches, firsts)
    for dtype in ("float32", "bfloat16"):
        steps = U.run_trace_tool(folder, dtype, records, str(tmp_path / dtype), 153, cfg["vocab"])
        for bi, reqs in enumerate(batches):
            for i, r in enumerate(reqs):
                got = torch.from_numpy(np.stack([steps[s][row] for s, row in where[(bi, i)]]))
                close(got, P.forward(cfg, w, r), dtype, f"replay {dtype} batch {bi} request {i}")
