"""The Batasun decoder through the engine, against ``plain_batasun``: whole prompts, decoding token by token,
prompts in pieces down to two tokens, batches of unequal requests, slots and pages used again, long decoding
across page borders, other sizes (also ones where the usual sizes coincide or are 1), layers that read another
layer's latent rows, greedy generation through the engine's entry point, the command line and the trace replay
tool."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import engine_utils as U
import plain_batasun as P

pytestmark = pytest.mark.gpu

CONFIGS = {
    # both mixers; a state-space layer first; two readers of one layer's latent rows with a recurrent layer between
    # them and other head counts and sizes than their source; layers without a feed-forward; ranks that differ
    "mixed": lambda: P.config([
        P.mamba_layer(4, 12, 8, 2, 4, 3, mlp=P.moe(5, 2, 24, 1.25, shared_ff=16, shared_limit=3.0)),
        P.latent_layer(3, 16, 8, 20, 24, 40, base=5000.0, mlp=None),
        P.mamba_layer(2, 6, 16, 1, 2, 1),
        P.latent_layer(5, 8, 8, 4, 12, 40, base=5000.0, kv_from=1, mlp=P.moe(3, 3, 8, 0.5)),
        P.latent_layer(2, 24, 8, 8, 16, 40, base=5000.0, kv_from=1, mlp=P.moe(4, 1, 16, 2.0, shared_ff=8, shared_limit=0.7))],
        vocab=131, width=40, eps=2e-6),
    # a width that is no multiple of 8 (no matrix-core packing), cached rows of 25 numbers, one head, one tap, one
    # group, one expert out of one, all experts chosen, a rotation of a part of the rotated elements only
    "odd": lambda: P.config([
        P.latent_layer(1, 12, 6, 10, 20, 19, base=300.0, rot_dims=4, mlp=P.moe(3, 3, 30, 1.0)),
        P.mamba_layer(3, 10, 12, 1, 1, 1, mlp=P.moe(1, 1, 20, 4.0, shared_ff=12)),
        P.mamba_layer(6, 5, 20, 3, 5, 5, mlp=None),
        P.latent_layer(7, 4, 2, 6, 9, 11, base=1e6, scale=0.9, mlp=None)], vocab=97, width=60, eps=1e-3),
    # sizes the matrix cores take everywhere, everything a multiple of 16
    "even": lambda: P.config([
        P.latent_layer(4, 32, 16, 32, 48, 48, mlp=P.moe(8, 2, 64, 1.5, shared_ff=64, shared_limit=2.5)),
        P.mamba_layer(4, 32, 64, 2, 4, 4, mlp=P.moe(8, 4, 32, 3.0)),
        P.latent_layer(8, 16, 16, 16, 32, 48, kv_from=0, mlp=None)], vocab=256, width=128),
}


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
    """32-bit: every row within 3e-5 of the largest logit.  bfloat16: rounding is what it is, and a row whose norms
    divide by something small carries several times the usual error (the 32-bit engine's largest error sits in the
    same rows): 4 % of the largest logit for all rows but one in twenty, twice that for those."""
    scale = float(ref.abs().max())
    err = (got.double() - ref).abs().max(dim=-1).values
    where = f"{what}: error {float(err.max()):.3e} of {scale:.3e} at row {int(err.argmax())}"
    if dtype == "float32":
        assert float(err.max()) <= 3e-5 * scale, where
    else:
        assert float(err.max()) <= 0.08 * scale, where
        assert int((err > 0.04 * scale).sum()) <= max(1, len(err) // 20), where


def model_for(models, name, dtype):
    # in bfloat16 the choice of experts is decided by the router's bias (a close call would go either way)
    return models(name, decided=(dtype == "bfloat16"))


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_tail_and_pieces(models, name, dtype):
    cfg, w, folder = model_for(models, name, dtype)
    eng = engine(folder, dtype)
    toks = U.random_tokens(200, cfg["vocab"], 1)
    ref = P.forward(cfg, w, toks)
    close(U.run_whole(eng, toks), ref, dtype, "whole")
    close(U.run_tail(eng, toks, 150), ref, dtype, "the last 150 one by one, across page borders")
    close(U.run_tail(eng, toks, 199), ref, dtype, "token by token from the first")
    for piece in (2, 7, 64, 100):                 # the prompt enters in pieces of this many tokens
        eng.prefill_chunk = piece
        close(U.run_whole(eng, toks[:170]), ref[:170], dtype, f"pieces of {piece}")
    eng.prefill_chunk = 0
    assert eng.cache.slots.n_free == eng.cache.max_slots
    assert all(g.pool.n_free == g.pool.n_pages for g in eng.cache.groups)


def test_streams_after_every_layer(models):
    """The residual stream after each layer, read off the engine between its blocks."""
    from agave_amd.parts.norm import add_branch
    cfg, w, folder = models("mixed")
    eng = engine(folder, "float32")
    eng.use_graphs = False
    toks = U.random_tokens(90, cfg["vocab"], 4)
    want = []
    P.forward(cfg, w, toks, streams=want)
    seen = []
    for b in eng.model.blocks[1:]:
        def wrapped(h, pending, step, memory, writes, inner=b.forward):
            copy = h.clone()
            add_branch(copy, pending)
            seen.append(copy.cpu())
            return inner(h, pending, step, memory, writes)
        b.forward = wrapped
    U.run_whole(eng, toks)
    assert len(seen) == len(want) - 1
    for i, (got, ref) in enumerate(zip(seen, want)):
        assert float((got.double() - ref).abs().max()) < 3e-5 * float(ref.abs().max()), f"after layer {i}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batches_of_unequal_requests_and_slots_used_again(models, dtype):
    """Three batches one after another over the same three slots, through a pool of pages that only holds them because
    pages come back; states of the recurrent layers start at zero again in a slot that is used again."""
    cfg, w, folder = model_for(models, "mixed", dtype)
    eng = engine(folder, dtype, max_slots=3, max_context=256, cache_tokens=448)
    for b, (lens, first) in enumerate([((50, 1, 130), (30, 1, 2)), ((70, 33), (69, 1)), ((90, 9, 140), (5, 9, 101))]):
        reqs = [U.random_tokens(n, cfg["vocab"], 10 * b + i) for i, n in enumerate(lens)]
        outs = U.run_batched(eng, reqs, first)
        for i, (r, o) in enumerate(zip(reqs, outs)):
            close(o, P.forward(cfg, w, r), dtype, f"batch {b} request {i}")
    assert eng.cache.slots.n_free == eng.cache.max_slots
    assert all(g.pool.n_free == g.pool.n_pages for g in eng.cache.groups)


def test_prompts_from_their_first_position_make_every_heads_keys(models):
    """In bfloat16, with head sizes the matrix cores take, a step of prompts that all start at position 0 runs the
    attention over every head's own keys and values instead of the cached latent rows; its pieces and the decoding
    after it read the latent rows.  Unequal prompts together (one shorter than a page, one ending on a page's border),
    a reader of another layer's rows among the layers, and the same prompts in pieces, against the plain logits."""
    cfg, w, folder = models("even", decided=True)
    eng = engine(folder, "bfloat16", max_slots=3, max_context=512)
    latent = [b.mixer for b in eng.model.blocks if hasattr(b.mixer, "fresh_prompt")]
    assert len(latent) == 2 and all(m.fresh_ok for m in latent)
    calls = []
    for m in latent:
        def counted(*a, inner=m.fresh_prompt, **k):
            calls.append(1)
            return inner(*a, **k)
        m.fresh_prompt = counted
    reqs = [U.random_tokens(n, cfg["vocab"], 40 + n) for n in (150, 40, 128)]
    refs = [P.forward(cfg, w, r) for r in reqs]
    for r, o in zip(refs, U.run_batched(eng, reqs, (141, 33, 128))):
        close(o, r, "bfloat16", "prompts together, then decoded")
    assert len(calls) == 2
    eng.prefill_chunk = 70                                  # the first piece from position 0, the others behind it
    close(U.run_whole(eng, reqs[0]), refs[0], "bfloat16", "pieces of 70")
    assert len(calls) == 4
    eng.prefill_chunk = 0
    close(U.run_tail(eng, reqs[2], 100), refs[2], "bfloat16", "28 tokens (the latent rows' form), then decoded")
    assert len(calls) == 4


def test_the_cache_as_the_mixers_asked(models):
    cfg, w, folder = models("mixed")
    eng = engine(folder, "float32")
    assert set(eng.cache.group_of_memory) == {1}                  # layers 3 and 4 read layer 1's memory
    key = eng.cache.group_keys[0]
    assert (key.n_kv_heads, key.head_dim, key.v_head_dim, key.window, key.layout) == (1, 48, 40, None, "rows_vt")
    assert set(eng.cache.state) == {0, 2}
    assert tuple(eng.cache.state[0]["S"].shape[1:]) == (4, 12, 8) and tuple(eng.cache.state[0]["conv"].shape[1:]) == (3, 80)
    assert eng.cache.state[0]["S"].dtype == torch.float32
    # a position costs one row of 48 numbers (and its first 40 again as the values' copy), whatever the heads
    per_position = sum(t.numel() for t in eng.cache.k_store + eng.cache.v_store) / (eng.cache.groups[0].pool.n_pages * 64)
    assert per_position == 48 + 40
    from agave_amd.ops import library
    slot = eng.alloc_slot()
    eng.step([slot], [[1, 2]])
    eng.free_slot(slot)
    loaded = library.loaded_paths()
    for name in ("latent.so", "attention_biased.so", "routed_ffn.so", "sequence.so"):
        assert any(p.endswith(name) for p in loaded), name


def test_long_decoding(models):
    cfg, w, folder = models("even")
    eng = engine(folder, "float32", max_slots=1, max_context=1024, cache_tokens=64 * 11)
    toks = U.random_tokens(700, cfg["vocab"], 9)
    ref = P.forward(cfg, w, toks)
    close(U.run_tail(eng, toks, 500), ref, "float32", "500 tokens decoded")


def far_key_model(boost=40.0):
    """One latent layer whose head 0 is made to look for one token: the unrotated key of token ``A`` is given
    ``boost`` more score against the unrotated query of token ``Q`` than it had, by a change of rank one in head 0's
    key matrix.  (A layer's input is a function of the token alone in a model of one layer, so the two vectors can be
    computed ahead.)  Other tokens' latents overlap with A's by chance and get a part of the boost; A stands out by
    more than ten among hundreds of keys."""
    A, Q = 0, 1
    cfg = P.config([P.latent_layer(2, 8, 8, 12, 16, 24, base=100.0, mlp=None)], vocab=60, width=32)
    w = P.random_weights(cfg, 3)
    m, eps = cfg["layers"][0]["mixer"], cfg["norm"]["eps"]
    x = P.rms(w["embed"][[A, Q]], eps) * (1.0 + w["embed.norm"])
    c_a = P.rms((x[0] @ w["l0.mix.dkv"].T)[:m["kv_rank"]], eps) * w["l0.mix.dkv.norm"]
    cq = P.rms(x[1] @ w["l0.mix.dq"].T, eps) * w["l0.mix.dq.norm"]
    q0 = (cq @ w["l0.mix.uq"].T).view(m["heads"], -1)[0, :m["dim"]]
    uk = w["l0.mix.uk"].clone().view(m["heads"], m["dim"], m["kv_rank"])
    uk[0] += boost / (m["scale"] * float(q0 @ q0) * float(c_a @ c_a)) * torch.outer(q0, c_a)
    w["l0.mix.uk"] = uk.reshape(-1, m["kv_rank"]).to(torch.bfloat16).to(P.F)
    return cfg, w, A, Q


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds(dtype):
    """The key that the last queries look for stands at the third position, at a page's last and first place, or far
    inside the prompt; the queries come in the prompt, in pieces of it, and decoded one by one.  Taking the key away
    moves the logits by much more than the engine may be off."""
    from agave_amd.engine import Engine
    cfg, w, A, Q = far_key_model()
    eng = Engine.from_tensors(cfg, {k: v.bfloat16() for k, v in w.items()}, dtype=dtype, max_slots=2, max_context=512)
    for at in (2, 63, 64, 300):
        toks = [2 + t % 58 for t in U.random_tokens(430, 1000, at)]
        for t in range(380, 430, 3):
            toks[t] = Q
        toks[-1] = Q
        toks[at] = A
        without = list(toks)
        without[at] = 7
        ref, ref_without = P.forward(cfg, w, toks), P.forward(cfg, w, without)
        scale = float(ref.abs().max())
        moved = float((ref[-1] - ref_without[-1]).abs().max())
        assert moved > 0.1 * scale, at
        eng.prefill_chunk = 0
        runs = {"whole": U.run_whole(eng, toks), "decoded": U.run_tail(eng, toks, 60)}
        eng.prefill_chunk = 50
        runs["pieces"] = U.run_whole(eng, toks)
        for what, got in runs.items():
            close(got, ref, dtype, f"key at {at}, {what}")
            assert float((got[-1].double() - ref[-1]).abs().max()) < (0.002 if dtype == "float32" else 0.2) * moved, (at, what)


def test_an_early_token_stays_in_the_state():
    """A state-space layer that forgets slowly: a change of the third token moves the logits 400 tokens later, and the
    engine follows, decoding or not."""
    from agave_amd.engine import Engine
    cfg = P.config([P.mamba_layer(2, 8, 16, 1, 3, 2, mlp=None)], vocab=60, width=32)
    w = P.random_weights(cfg, 3)
    w["l0.mix.A_log"] = torch.full((2,), -7.0, dtype=P.F)             # almost nothing is forgotten
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
        steps = U.run_trace_tool(folder, dtype, records, str(tmp_path / dtype), 153, cfg["vocab"])      # the tokens held, counted one by one: three requests need four pages
        for bi, reqs in enumerate(batches):
            for i, r in enumerate(reqs):
                got = torch.from_numpy(np.stack([steps[s][row] for s, row in where[(bi, i)]]))
                close(got, P.forward(cfg, w, r), dtype, f"replay {dtype} batch {bi} request {i}")
