"""Decode and prefill throughput of the Gemma 3 4B text decoder (random bf16 weights) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one decode step of the whole batch: planning on the host, every kernel of the
model, sampling (greedy) and the copy of the new token ids back to the host; as in generation,
a step is launched while the host still waits for the tokens of the step before.  The default run
has the layer sizes of the published Gemma 3 4B text configuration, a batch of 8, prompts of 1,024 tokens and
256 decoded tokens per sequence (W warm-up steps, then K timed ones).  One JSON line is
printed: ``value`` is decoded tokens a second; ``prefill`` is one 2,048-token prompt;
``roofline`` prices the decode step by the bytes it has to read (every weight once, and the
cache of the live requests) against 8 TB/s; ``points`` holds decode at batch 1 and 64 and
prompts of 256 and 512 tokens (tokens a second each);
``peaks_measured`` is what this machine delivered to a streaming read and to a loop of
matrix-core instructions on random data a moment before (the fractions stay against the
published peaks).

The other published shapes:

    python bench.py --model 12b --ragged 16 --context 8192        # 16 prompts of unequal lengths 64..4096
    python bench.py --model 27b --prompt-len 2048 --context 8192 --batch 1 --no-points
    python bench.py --model 27b --prompt-len 2048 --context 8192 --batch 32 --no-points

Another design beside the closest Gemma 3 shape of equal size (not the default run):

    python bench.py --design rilenex|gusedra|batasun|duperax [--design-size small|medium|large] [--design-layers 8]

prints one JSON line with, for that decoder and for a Gemma 3 decoder of the same width, depth,
heads and about as many weights: tokens a second of a 2,048-token prompt and of decode steps at
batch 8 and 1, and the time of every kind of kernel in one prompt and in one decode step.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

# Gemma 3 4B text decoder, as its config.json gives it
GEMMA3_4B = dict(
    architectures=["Gemma3ForCausalLM"], model_type="gemma3_text", vocab_size=262208, hidden_size=2560,
    num_hidden_layers=34, num_attention_heads=8, num_key_value_heads=4, head_dim=256,
    query_pre_attn_scalar=256, intermediate_size=10240, sliding_window=1024, sliding_window_pattern=6,
    rope_theta=1e6, rope_local_base_freq=1e4, rope_scaling={"rope_type": "linear", "factor": 8.0},
    rms_norm_eps=1e-6, tie_word_embeddings=True, hidden_activation="gelu_pytorch_tanh",
    max_position_embeddings=131072, bos_token_id=2, eos_token_id=1)

# the larger published sizes of the same architecture, for --model (not the default run)
GEMMA3_12B = dict(GEMMA3_4B, hidden_size=3840, num_hidden_layers=48, num_attention_heads=16, num_key_value_heads=8,
                  intermediate_size=15360)
GEMMA3_27B = dict(GEMMA3_4B, hidden_size=5376, num_hidden_layers=62, num_attention_heads=32, num_key_value_heads=16,
                  head_dim=128, query_pre_attn_scalar=168, intermediate_size=21504)
MODELS = {"4b": ("gemma3-4b-text", GEMMA3_4B), "12b": ("gemma3-12b-text", GEMMA3_12B),
          "27b": ("gemma3-27b-text", GEMMA3_27B)}

PROMPT_LEN, DECODE_LEN, CONTEXT, PREFILL_LEN = 1024, 256, 4096, 2048


def model_numbers(cfg: dict, n_layers: int):
    e, nh, nkv, hd = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    ff, v = cfg["intermediate_size"], cfg["vocab_size"]
    qd, kvd = nh * hd, nkv * hd
    pattern = cfg["sliding_window_pattern"]
    sliding = [(i + 1) % pattern != 0 for i in range(n_layers)]
    per_layer = e * (qd + 2 * kvd) + qd * e + 3 * e * ff
    norms = n_layers * (4 * e + 2 * hd) + e
    return dict(e=e, qd=qd, kvd=kvd, ff=ff, v=v, sliding=sliding, window=cfg["sliding_window"],
                linear_params=per_layer * n_layers, table_params=v * e, norm_params=norms)


def decode_step_bytes(m: dict, contexts) -> float:
    """Bytes one decode step has to read: every weight once (bf16; the tied table once, as the
    output matrix; norm gains in 32-bit) and the keys and values each live request attends to."""
    weights = 2 * (m["linear_params"] + m["table_params"]) + 4 * m["norm_params"]
    kv = 0
    for ctx in contexts:
        for s in m["sliding"]:
            kv += (min(ctx, m["window"]) if s else ctx) * m["kvd"] * 2 * 2
    return float(weights + kv)


def measured_peaks():
    """What the machine delivers just now: a streaming read of 2 GiB and a loop of bfloat16
    matrix-core instructions on normally distributed operands (the published peak holds for zeros)."""
    from agave_amd.ops import peaks
    return {"hbm_read_gbs": round(peaks.hbm_read_gbs(), 1), "mfma_bf16_tflops": round(peaks.mfma_bf16_tflops(), 1)}


def prefill_flops(m: dict, t: int) -> float:
    """Multiply-adds of one prompt of t tokens, twice: the linear layers on every token, the
    output matrix on the one wanted row, and attention over the visible pairs."""
    linear = 2.0 * t * m["linear_params"] + 2.0 * m["table_params"]
    attn = 0.0
    for s in m["sliding"]:
        pairs = sum(min(i + 1, m["window"]) for i in range(t)) if s else t * (t + 1) // 2
        attn += 4.0 * m["qd"] * pairs
    return linear + attn


def random_prompts(n: int, length: int, vocab: int, seed: int):
    import numpy as np
    rng = np.random.default_rng(seed)
    return [rng.integers(0, vocab, size=length).tolist() for _ in range(n)]


def ragged_lengths(n: int, lo: int, hi: int, seed: int):
    """n prompt lengths drawn uniformly from lo..hi, the two ends among them."""
    import numpy as np
    rng = np.random.default_rng(seed)
    lens = rng.integers(lo, hi + 1, size=n).tolist()
    if n >= 2:
        lens[0], lens[-1] = lo, hi
    return lens


def run_decode(engine, batch: int, steps: int, warmup: int, seed: int, prompt_len: int = PROMPT_LEN, lengths=None,
               first_step=None):
    """Prefill ``batch`` prompts of ``prompt_len`` tokens (or of the given unequal ``lengths``, then
    as one ragged step whose time goes into ``first_step``), then time ``steps`` decode steps."""
    import numpy as np
    import torch
    from agave_amd.engine.generate import RowSampling
    if lengths is None:
        prompts = random_prompts(batch, prompt_len, engine.vocab_size, seed)
    else:
        rng = np.random.default_rng(seed)
        prompts = [rng.integers(0, engine.vocab_size, size=n).tolist() for n in lengths]
    plens = [len(p) for p in prompts]
    slots = [engine.alloc_slot() for _ in range(batch)]
    rows = [RowSampling(0.0, 0, 1.0, 1.0, 0.0, []) for _ in range(batch)]
    try:
        engine.prefill_chunk = 2048 if (batch > 8 and lengths is None) else 0
        if lengths is not None:             # the unequal prompts in one step, as a batch starts
            engine.step_sample(slots, prompts, rows)            # once untimed: libraries, workspace
            for s in slots:
                engine.free_slot(s)
            slots[:] = [engine.alloc_slot() for _ in range(batch)]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            toks = engine.step_sample(slots, prompts, rows)
            torch.cuda.synchronize()
            if first_step is not None:
                first_step.update(tokens=sum(plens), ms=round((time.perf_counter() - t0) * 1e3, 3))
        elif batch > 8:                     # keep the untimed prefill's workspace small
            toks = None
            for i in range(0, batch, 8):
                part = engine.step_sample(slots[i:i + 8], prompts[i:i + 8], rows[i:i + 8])
                toks = part if toks is None else toks + part
        else:
            toks = engine.step_sample(slots, prompts, rows)
        for _ in range(warmup):
            toks = engine.step_sample(slots, [[t] for t in toks], rows)
        torch.cuda.synchronize()
        # the timed steps run as generation runs them: each is launched, its tokens taken on the
        # device from the step before, while the host still waits for that step's tokens
        carry = list(range(batch))
        t0 = time.perf_counter()
        running = engine.launch_step(slots, [[t] for t in toks], rows)
        for _ in range(steps - 1):
            following = engine.launch_step(slots, None, rows, carry)
            toks = engine.finish_step(running)
            running = following
        toks = engine.finish_step(running)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        # keys the first timed step attends to: the prompt, the warm-up steps' tokens and its own
        contexts = [n + warmup + 1 + (steps - 1) / 2.0 for n in plens]
        return dt, contexts
    finally:
        for s in slots:
            engine.free_slot(s)
        engine.prefill_chunk = 0


def run_prefill(engine, seed: int, repeats: int = 3, length: int = PREFILL_LEN):
    import torch
    from agave_amd.engine.generate import RowSampling
    prompt = random_prompts(1, length, engine.vocab_size, seed)
    row = [RowSampling(0.0, 0, 1.0, 1.0, 0.0, [])]
    times = []
    for r in range(repeats + 1):                     # the first pass warms up
        slot = engine.alloc_slot()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step_sample([slot], prompt, row)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        engine.free_slot(slot)
        if r > 0:
            times.append(dt)
    return min(times)


# ---------------------------------------------------------------- another design beside Gemma 3
# width, feed-forward, heads, key heads, head size, chunk of the attention side, inner size of the two-step projections
DESIGN_SIZES = {"small": (1024, 4096, 8, 2, 128, 128, 64), "medium": (2048, 8192, 16, 4, 128, 256, 128),
                "large": (4096, 16384, 32, 8, 128, 256, 256)}


def rilenex_config(size: str, layers: int) -> dict:
    """Three layers of HGRN2 to one with attention and the delta rule side by side, every layer with its
    dense feed-forward; heads of 128 on every side."""
    e, ff, h, g, d, chunk, rank = DESIGN_SIZES[size]
    hgrn2 = {"type": "hgrn2", "mixer": {"heads": h, "dim": d, "vdim": d}, "mlp": {"kind": "dense", "ff": ff}}
    par = {"type": "parallel", "mlp": {"kind": "dense", "ff": ff},
           "mixer": {"left": {"heads": h, "kv_heads": g, "dim": d, "vdim": d, "conv": 4, "scale": d ** -0.5,
                              "mask": {"size": chunk}, "rot": {"dims": d, "base": 10000.0}},
                     "right": {"heads": h, "kv_heads": g, "dim": d, "vdim": d, "conv": 4, "decay_rank": rank, "gate_rank": rank},
                     "left_scale": 1.0, "right_scale": 1.0}}
    return {"architecture": "Rilenex", "vocab": 32768, "width": e, "norm": {"eps": 1e-5},
            "layers": [par if i % 4 == 2 else hgrn2 for i in range(layers)]}


def gusedra_config(size: str, layers: int) -> dict:
    """Layers of both attention mixers in turn (a learned bias over buckets with kept first positions and a gate;
    slopes with sinks), every fourth one reading the keys and values of the layer before it; feed-forwards in
    turn dense (the square of ReLU) and routed (16 experts of a quarter of the dense inner size plus two identity
    experts in 2 groups of 9, 4 of them a token, and a shared expert): a token's routed layer computes as much as
    a dense one.  Heads of 128, windows of 1,024 as the Gemma 3 shape beside it."""
    e, ff, h, g, d, _, _ = DESIGN_SIZES[size]
    def mixer(kind, i):
        m = {"heads": h, "kv_heads": g, "dim": d, "vdim": d, "scale": d ** -0.5, "mask": {"size": 1024}}
        if kind == "attention_2":
            m["mask"]["keep_first"] = 4
            m["bias_max"] = 2048
        elif i % 4 == 3:
            m["kv_from"] = i - 2
        return m
    dense = {"kind": "dense", "ff": ff}
    moe = {"kind": "moe", "expert": {"ff": ff // 4}, "shared": {"ff": ff // 4},
           "router": {"experts": 16, "identity": 2, "top": 4, "scale": 2.0, "groups": {"count": 2, "keep": 1}}}
    out = []
    for i in range(layers):
        kind = "attention_2" if i % 2 == 0 else "attention"
        out.append({"type": kind, "mixer": mixer(kind, i), "mlp": moe if i % 2 else dense})
    return {"architecture": "Gusedra", "vocab": 32768, "width": e, "norm": {"eps": 1e-5}, "residual_mult": 0.5, "layers": out}


def batasun_config(size: str, layers: int) -> dict:
    """Of every four layers the first has latent attention with a projection of its own, the next two are state-space
    mixers and the fourth is latent attention again that reads the first one's cached rows; every layer has the routed
    feed-forward of the Gusedra shape beside it (16 experts of a quarter of the dense inner size, 4 of them a token,
    and a shared expert).  Latent attention in the proportions of the published models of that kind: heads of 128
    plain and 64 rotated elements, values of 128, a query latent of three quarters of the width, and a cached row of
    192 + 64 numbers at the small size, 512 + 64 at the others.  State-space mixers twice as wide as the model, in
    heads of 64 with a state of 128 per head, B and C shared by all heads."""
    e, ff, h, _, d, _, _ = DESIGN_SIZES[size]
    kv_rank = 192 if size == "small" else 512
    moe = {"kind": "moe", "expert": {"ff": ff // 4, "limit": 7.0}, "shared": {"ff": ff // 4, "limit": 7.0},
           "router": {"experts": 16, "top": 4}}
    def latent(source):
        m = {"heads": h, "dim": d, "rot_dim": d // 2, "vdim": d, "q_rank": 3 * e // 4, "kv_rank": kv_rank,
             "scale": (d + d // 2) ** -0.5, "rot": {"base": 10000.0, "dims": d // 2}}
        if source is not None:
            m["kv_from"] = source
        return {"type": "latent_attention", "mixer": m, "mlp": moe}
    ssm = {"type": "mamba2", "mlp": moe,
           "mixer": {"heads": 2 * e // 64, "vdim": 64, "state": 128, "groups": 1, "conv": 4, "norm_groups": 1}}
    out = []
    for i in range(layers):
        out.append(latent(None) if i % 4 == 0 else latent(i - 3) if i % 4 == 3 else ssm)
    return {"architecture": "Batasun", "vocab": 32768, "width": e, "norm": {"eps": 1e-5}, "layers": out}


def duperax_config(size: str, layers: int) -> dict:
    """Of every four layers the first has windowed attention whose q and k rows are normed whole, the third attention in
    chunks with biases, a YaRN rotation and capped scores, the second and fourth the gated linear recurrence (as wide
    as the model, gates in blocks of 128 channels, four taps); feed-forwards in turn dense (clamped swish) and routed
    (16 experts of a quarter of the dense inner size in 4 groups of which 2 are open, 4 experts a token, sigmoid
    scores): a token's routed layer computes as much as a dense one of two thirds the size.  Four residual streams.
    Heads of 128, a window and chunks of 1,024 positions as the Gemma 3 shape beside it."""
    e, ff, h, g, d, _, _ = DESIGN_SIZES[size]
    dense = {"kind": "dense", "ff": (2 * ff // 3) // 256 * 256, "limit": 7.0}
    moe = {"kind": "moe", "expert": {"ff": ff // 4}, "router": {"experts": 16, "top": 4, "groups": {"count": 4, "keep": 2}}}
    first = {"type": "attention", "mixer": {"heads": h, "kv_heads": g, "dim": d, "vdim": d, "scale": d ** -0.5, "mask": {"size": 1024}}}
    second = {"type": "attention_2",
              "mixer": {"heads": h, "kv_heads": g, "dim": d, "vdim": d, "scale": d ** -0.5, "mask": {"size": 1024}, "softcap": 30.0,
                        "rot": {"dims": d, "base": 10000.0, "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}}
    lru = {"type": "rglru", "mixer": {"width": e, "blocks": e // 128, "conv": 4}}
    out = []
    for i in range(layers):
        out.append(dict((first, lru, second, lru)[i % 4], mlp=moe if i % 2 else dense))
    return {"architecture": "Duperax", "vocab": 32768, "width": e, "norm": {"eps": 1e-5}, "streams": 4, "logit_scale": 1.0,
            "layers": out}


def gemma_like_config(size: str, layers: int) -> dict:
    """The same width, depth and heads as a Gemma 3 decoder; its gated feed-forward has three matrices,
    so two thirds of the inner size give as many weights."""
    e, ff, h, g, d, chunk, _ = DESIGN_SIZES[size]
    return dict(GEMMA3_4B, vocab_size=32768, hidden_size=e, num_hidden_layers=layers, num_attention_heads=h,
                num_key_value_heads=g, head_dim=d, query_pre_attn_scalar=d, intermediate_size=(2 * ff // 3) // 256 * 256,
                sliding_window=1024, tie_word_embeddings=False)


def op_times(engine, prompt_len: int, batch: int, seed: int):
    """ms of every kind of kernel call in one prompt of ``prompt_len`` tokens and in one decode step
    of ``batch`` sequences after such prompts (steps run eagerly, two events around each call)."""
    import torch
    from agave_amd.engine.generate import RowSampling
    out = {}
    prompts = random_prompts(batch, prompt_len, engine.vocab_size, seed)
    rows = [RowSampling(0.0, 0, 1.0, 1.0, 0.0, []) for _ in range(batch)]
    slots = [engine.alloc_slot() for _ in range(batch)]
    engine.enable_profiling(True)
    try:
        engine.step_sample(slots[:1], prompts[:1], rows[:1])
        out["prompt"] = {n: [c, round(ms, 4)] for n, c, ms in engine.profile_table()}
        toks = [1] * batch
        if batch > 1:
            engine.step_sample(slots[1:], prompts[1:], rows[1:])
        for _ in range(3):
            toks = engine.step_sample(slots, [[t] for t in toks], rows)
        from agave_amd.ops import library
        library.profile.reset()
        reps = 5
        for _ in range(reps):
            toks = engine.step_sample(slots, [[t] for t in toks], rows)
        out["decode_step"] = {n: [c // reps, round(ms / reps, 4)] for n, c, ms in engine.profile_table()}
    finally:
        engine.enable_profiling(False)
        for s in slots:
            engine.free_slot(s)
    return out


def compare_designs(args) -> int:
    import torch
    from agave_amd.engine import Engine
    size, layers = args.design_size, args.design_layers
    context, prompt_len, batch = 4096, 1024, 8
    result = {"metric": f"{args.design} beside Gemma 3 at equal size ({size}, {layers} layers): tokens/s", "unit": "tokens/s",
              "dtype": "bf16", "data": "synthetic: uniform-random token ids, random weights", "sizes": DESIGN_SIZES[size],
              "peaks_measured": measured_peaks()}
    makers = {"rilenex": rilenex_config, "gusedra": gusedra_config, "batasun": batasun_config, "duperax": duperax_config}
    runs = [(args.design, makers[args.design](size, layers))]
    if args.design in ("batasun", "duperax"):      # the design with the same attention kernels and routed feed-forwards stands beside it too
        runs.append(("gusedra_equal_size", gusedra_config(size, layers)))
    if args.design == "duperax":                   # and the one with recurrent layers
        runs.append(("rilenex_equal_size", rilenex_config(size, layers)))
    runs.append(("gemma3_equal_size", gemma_like_config(size, layers)))
    for name, cfg in runs:
        engine = Engine.from_random(cfg, seed=0, dtype="bfloat16", max_slots=batch, max_context=context,
                                    cache_tokens=batch * (PREFILL_LEN + 512), device="cuda:0")
        rec = {"weights_gb": round(engine.model.weight_bytes() / 1e9, 3)}
        pdt = run_prefill(engine, seed=2, length=PREFILL_LEN)
        rec["prefill_2048"] = {"tokens_per_s": round(PREFILL_LEN / pdt, 1), "ms": round(pdt * 1e3, 3)}
        for b in (batch, 1):
            dt, _ = run_decode(engine, b, args.steps, args.warmup, seed=1, prompt_len=prompt_len)
            rec[f"decode_b{b}"] = {"tokens_per_s": round(b * args.steps / dt, 1), "ms_per_step": round(dt / args.steps * 1e3, 4),
                                   "weights_gbs": round(engine.model.weight_bytes() / (dt / args.steps) / 1e9, 1)}
        rec["kernels"] = op_times(engine, PREFILL_LEN, batch, seed=4)
        result[name] = rec
        del engine
        torch.cuda.empty_cache()
    print(json.dumps(result), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--model", default="4b", choices=sorted(MODELS),
                    help="layer sizes: Gemma 3 4B (the default run), 12B or 27B")
    ap.add_argument("--layers", type=int, default=0,
                    help="run fewer layers of the same sizes (reported in config)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prompt-len", type=int, default=PROMPT_LEN,
                    help="tokens of every prompt before the decode steps (the default run: 1024)")
    ap.add_argument("--context", type=int, default=CONTEXT, help="longest sequence a slot may hold")
    ap.add_argument("--prefill-len", type=int, default=PREFILL_LEN, help="tokens of the prefill prompt (the default run: 2048)")
    ap.add_argument("--ragged", type=int, default=0, metavar="N",
                    help="N prompts of unequal lengths 64..4096 (seeded) as one first step, then decode steps; "
                         "replaces --batch and --prompt-len")
    ap.add_argument("--no-points", action="store_true", help="skip prefill and the batch 1 / 64 points")
    ap.add_argument("--prefill-only", action="store_true",
                    help="time only the 2048-token prefill and print its record (for profiles)")
    ap.add_argument("--design", choices=["rilenex", "gusedra", "batasun", "duperax"], help="measure this design beside a Gemma 3 decoder of equal size")
    ap.add_argument("--design-size", default="medium", choices=sorted(DESIGN_SIZES))
    ap.add_argument("--design-layers", type=int, default=8)
    args = ap.parse_args()
    world = int(os.environ.get("WORLD_SIZE", "1"))
    if args.gpus != 1 or world != 1:
        if int(os.environ.get("RANK", "0")) == 0:
            print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.design:
        if args.steps == 240:
            args.steps = 64
        return compare_designs(args)
    lengths = None
    if args.ragged:
        lengths = ragged_lengths(args.ragged, 64, min(4096, args.context // 2), seed=7)
        args.batch, args.prompt_len, args.no_points = args.ragged, max(lengths), True
    if args.steps + args.warmup > args.context - args.prompt_len:
        ap.error(f"--steps + --warmup must stay within {args.context - args.prompt_len} decoded tokens")

    import torch
    from agave_amd.engine import Engine

    model_name, full = MODELS[args.model]
    if args.layers <= 0:
        args.layers = full["num_hidden_layers"]
    cfg = dict(full, num_hidden_layers=args.layers)
    m = model_numbers(cfg, args.layers)
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    per_seq = -(-(args.prompt_len + max(DECODE_LEN, args.steps + args.warmup) + 64) // 64) * 64
    cache_tokens = max(max_batch * per_seq, -(-max(PREFILL_LEN, args.prefill_len) // 64) * 64 + 64)
    peaks = measured_peaks() if args.dtype == "bfloat16" else None
    engine = Engine.from_random(cfg, seed=0, dtype=args.dtype, max_slots=max_batch, max_context=args.context,
                                cache_tokens=cache_tokens, device="cuda:0")
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"
    if args.prefill_only:
        pdt = run_prefill(engine, seed=2, length=args.prefill_len)
        print(json.dumps({"prefill": {"value": round(args.prefill_len / pdt, 1), "tokens": args.prefill_len,
                                      "ms": round(pdt * 1e3, 3),
                                      "frac": round(prefill_flops(m, args.prefill_len) / pdt / PEAK_FLOPS[dkey], 4)}}),
              flush=True)
        return 0

    first_step = {}
    dt, contexts = run_decode(engine, args.batch, args.steps, args.warmup, seed=1, prompt_len=args.prompt_len,
                              lengths=lengths, first_step=first_step)
    ms_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    need = decode_step_bytes(m, contexts)
    achieved = need / (ms_step * 1e-3) / 1e9
    out = {
        "metric": f"decode tok/s, Gemma3-{args.model.upper()} {dkey}, batch {args.batch}, "
                  + (f"prompts of unequal lengths {min(lengths)}..{max(lengths)}" if lengths else f"{args.prompt_len}-token prompts")
                  + f" + {args.warmup + args.steps + 1} decoded ({args.steps} steps timed after {args.warmup} of warm-up)",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dkey, "data": "synthetic: uniform-random token ids, random N(0,0.02) weights",
        "config": {"model": model_name, "layers": args.layers, "layers_of_config": full["num_hidden_layers"],
                   "hidden": m["e"], "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
                   "head_dim": cfg["head_dim"], "intermediate": m["ff"], "vocab": m["v"],
                   "sliding_window": m["window"], "sliding_pattern": cfg["sliding_window_pattern"],
                   "global_batch": args.batch, "seq_len": args.prompt_len + args.warmup + args.steps + 1,
                   "prompt_len": args.prompt_len,
                   "context": args.context, "prefill_len": args.prefill_len, "parallelism": "single GPU",
                   "sampling": "greedy", "weights_gb": round(2 * (m["linear_params"] + m["table_params"]) / 1e9, 3)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if peaks is not None:
        out["peaks_measured"] = peaks
    if lengths:
        flops = sum(prefill_flops(m, n) for n in lengths)
        out["ragged_prefill"] = {"value": round(first_step["tokens"] / (first_step["ms"] * 1e-3), 1),
                                 "tokens": first_step["tokens"], "ms": first_step["ms"], "sequences": len(lengths),
                                 "frac": round(flops / (first_step["ms"] * 1e-3) / PEAK_FLOPS[dkey], 4)}
    if not args.no_points:
        pdt = run_prefill(engine, seed=2, length=args.prefill_len)
        flops = prefill_flops(m, args.prefill_len)
        out["prefill"] = {"value": round(args.prefill_len / pdt, 1), "tokens": args.prefill_len, "ms": round(pdt * 1e3, 3),
                          "frac": round(flops / pdt / PEAK_FLOPS[dkey], 4)}
        points = {}
        for b, k in ((1, 64), (64, 32)):
            d, _ = run_decode(engine, b, k, 8, seed=3 + b)
            points[f"decode_b{b}"] = round(b * k / d, 2)
        for n in (256, 512):                      # short prompts: tokens a second of one prompt of n tokens
            points[f"prefill_{n}"] = round(n / run_prefill(engine, seed=5, length=n), 1)
        out["points"] = points
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
