"""Decode and prefill throughput of GPT-2 XL layer sizes on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--dtype bfloat16]

Prints one JSON line.  ``value`` is decoded tokens a second at the given batch (default 8):
K timed decode steps, every request starting from a 512-token prompt, so that the first timed
step runs at context 512 and, with the default K, the last at the model's last position but one (511 steps)
(the reference's benchmark draws uniform random prompts and switches end-of-sequence off,
mlx_lm/benchmark.py:118-124; it warms up, then times five trials and reports their mean,
mlx_lm/benchmark.py:152-176).  The W warm-up steps run before, on requests of their own, so
that they do not move the timed steps' context.  ``config`` gives the context range as
``ctx_from``/``ctx_to``.  ``prefill`` is one step of 2 x 1,024 prompt tokens: W untimed
warm-up trials, three at least (a step whose shape keeps coming back is replayed from its
recorded graph, as in the serving path: the third trial records it), then the mean of five
timed ones, each listed in ``trials_ms``.
``points`` holds decode at batch 1, 16, 32, 48 and 64 over the same steps and, for batch 1, 8 and
64, at context 1,000; ``roofline`` the bytes a decode step has to read (every weight once, the live
requests' keys and values at each step's context) over its time, ``roofline_points`` the same
fraction for every point.  Times are the host's clock around the steps with the GPU drained on
both sides; ``gpu_ms_per_step`` (and ``prefill.gpu_ms``) is the same stretch between two events
on the GPU's stream, the reference's way of timing apart (mlx_lm/benchmark.py:152-176 times with
the host's clock around an evaluated result).  Weights are random (seeded), data synthetic.

``--n-positions 8192`` is a mode of its own for long contexts: the same layer sizes with 8,192
positions and, unless ``--layers`` says otherwise, 12 of the 48 layers (``config`` names both);
``value`` is decode at batch 8 from context 7,000, ``points`` hold batch 1 and 8 at contexts 4,000
and 7,000, ``prefill`` is one prompt of 8,192 tokens.

``--designs`` is another mode of its own (the default workload and its line are untouched by it):
Pafutar beside GPT-2 at equal sizes (the same width, heads, head size, inner size, layers,
vocabulary and positions; every Pafutar head with a key head of its own, as GPT-2's), random weights,
prefill of 2 x 1,024 tokens and decode at batch 1, 8 and 32 from context 512, for each of
``DESIGN_SIZES`` (``--design-size`` names one, ``--design-only`` one design, for a profile).  The
Pafutar model runs once without a window (like for like with GPT-2's attention) and once with a
window of 512 that keeps the first 64 tokens.  Ruzolorn runs at the same layer sizes too
(``ruzolorn_config``), without a window and with one of 512, and Zatinex (``zatinex_config``:
differential attention, gated linear attention and latent attention by turns, a dense gated
feed-forward), and Sazilorn (``sazilorn_config``: its parallel, HGRN2 and attention mixers by turns,
dense and expert feed-forwards).  It prints one JSON line of its own.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X, published: HBM3E 8 TB/s; dense MFMA bf16/fp16 2.5 PFLOP/s, fp32 157.3 TFLOP/s
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

XL = dict(model_type="gpt2", n_layer=48, n_embd=1600, n_head=25, n_inner=6400, vocab_size=50257,
          n_positions=1024, n_ctx=1024, layer_norm_epsilon=1e-5, activation_function="gelu_new")


# Layer sizes for --designs: width = heads x head size, as GPT-2 has it
DESIGN_SIZES = {
    "1024": dict(width=1024, heads=16, dim=64, ff=4096, layers=12),
    "2048": dict(width=2048, heads=16, dim=128, ff=8192, layers=8),
}
DESIGN_VOCAB, DESIGN_POSITIONS = 32000, 2048


def design_config(design, size, window=None):
    """The config.json of ``design`` ("gpt2", "pafutar") at one of ``DESIGN_SIZES``."""
    s = DESIGN_SIZES[size]
    if design == "gpt2":
        return dict(model_type="gpt2", n_layer=s["layers"], n_embd=s["width"], n_head=s["heads"], n_inner=s["ff"],
                    vocab_size=DESIGN_VOCAB, n_positions=DESIGN_POSITIONS, layer_norm_epsilon=1e-5,
                    activation_function="gelu_new")
    if design == "ruzolorn":
        return ruzolorn_config(s, window)
    if design == "zatinex":
        return zatinex_config(s)
    if design == "sazilorn":
        return sazilorn_config(s)
    mixer = {"heads": s["heads"], "kv_heads": s["heads"], "dim": s["dim"], "vdim": s["dim"], "scale": s["dim"] ** -0.5}
    if window:
        mixer["mask"] = {"size": window[0], "keep_first": window[1]}
    layer = {"type": "attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": s["ff"]}}
    return {"architecture": "Pafutar", "vocab": DESIGN_VOCAB, "width": s["width"], "max_positions": DESIGN_POSITIONS,
            "embedding": {"scale": s["width"] ** 0.5}, "norm": {"eps": 1e-6}, "postln_alpha": 2.0,
            "layers": [dict(layer) for _ in range(s["layers"])]}


def ruzolorn_config(s, window=None):
    """Ruzolorn at GPT-2's layer sizes: retention layers and parallel layers by turns, as many heads
    of the same size (a key head for every query head in the attention, as GPT-2 has; the state
    space as wide as the model, a state as large as a head), and a feed-forward of sixteen experts
    and two identity experts of which a token uses four, each an eighth of GPT-2's inner size, with
    a shared expert of a quarter of it: a token multiplies with 3 x (4/8 + 1/4) = 2.25 inner sizes
    of weights where GPT-2's does with 2."""
    H, d, D = s["heads"], s["dim"], s["width"]
    decay = [1.0 - 2.0 ** (-5.0 - 5.0 * h / max(1, H - 1)) for h in range(H)]
    retention = {"type": "retention", "mixer": {"heads": H, "dim": d, "vdim": d, "decay": decay,
                                                "rot": {"dims": d, "base": 10000.0}}}
    left = {"heads": H, "kv_heads": H, "dim": d, "vdim": d, "scale": d ** -0.5}
    if window:
        left["mask"] = {"size": window[0]}
    right = {"heads": H, "vdim": d, "state": d, "groups": 1, "conv": 4, "norm_groups": 1}
    parallel = {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": 1.0, "right_scale": 1.0}}
    mlp = {"kind": "moe", "expert": {"ff": s["ff"] // 8}, "router": {"experts": 16, "identity": 2, "top": 4},
           "shared": {"ff": s["ff"] // 4}}
    layers = [dict(retention if i % 2 == 0 else parallel, mlp=mlp) for i in range(s["layers"])]
    return {"architecture": "Ruzolorn", "vocab": DESIGN_VOCAB, "width": D, "max_positions": DESIGN_POSITIONS,
            "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5}, "residual_mult": 0.7, "layers": layers}


def zatinex_config(s):
    """Zatinex at GPT-2's layer sizes, its three mixers by turns.  Differential attention: half as
    many heads, each with two maps of a head's size over values twice as wide (the projections as
    large as GPT-2's), four taps, every column turning with interpolated frequencies.  Gated linear
    attention: as many heads of the same size (Ruzolorn's retention layers at the same sizes are
    its like), a decay through a middle of 16.  Latent attention: as many heads, a latent of 192
    columns and half a head of turning ones, queries through a latent of half the width; every
    second such layer reads the first one's latents.  A gated feed-forward of two thirds of GPT-2's
    inner size (three matrices where GPT-2 has two)."""
    H, d, D = s["heads"], s["dim"], s["width"]
    scaling = {"factor": 8.0, "original": 1024, "fast": 16.0, "slow": 2.0}
    attention = {"type": "attention", "mixer": {"heads": H // 2, "kv_heads": H // 2, "dim": d, "vdim": 2 * d, "conv": 4, "diff": 0.3,
                                                "scale": d ** -0.5, "rot": {"dims": d, "base": 10000.0, "scaling": scaling}}}
    gla = {"type": "gla", "mixer": {"heads": H, "dim": d, "vdim": d, "tau": 8.0}}
    latent = {"heads": H, "dim": d, "rot_dim": d // 2, "vdim": d, "q_rank": D // 2, "kv_rank": 192,
              "scale": (d + d // 2) ** -0.5, "rot": {"dims": d // 2, "base": 10000.0}}
    mlp = {"kind": "dense", "ff": s["ff"] * 2 // 3 // 64 * 64}
    layers, first_latent = [], None
    for i in range(s["layers"]):
        if i % 3 == 0:
            entry = dict(attention)
        elif i % 3 == 1:
            entry = dict(gla)
        else:
            m = dict(latent)
            if first_latent is None:
                first_latent = i
            elif (i // 3) % 2 == 1:
                m["kv_from"] = first_latent
            entry = {"type": "latent_attention", "mixer": m}
        layers.append(dict(entry, mlp=mlp))
    return {"architecture": "Zatinex", "vocab": DESIGN_VOCAB, "width": D, "max_positions": DESIGN_POSITIONS,
            "norm": {"eps": 1e-5}, "layers": layers}


def sazilorn_config(s):
    """Sazilorn at GPT-2's layer sizes, its three mixers by turns, four taps ahead of every mixer and
    the sum over depth behind every layer.  Parallel: capped, gated softmax attention with as many
    heads of the same size over a quarter as many key heads, beside lightning attention with half
    as many heads.  HGRN2: as many heads of the same size (Zatinex's gated linear attention and
    Ruzolorn's retention at the same sizes are its like).  Attention: grouped key heads as above,
    whole-projection norms, a distance table of 32 rows reaching to 128.  Feed-forwards by turns: a
    gelu-gated dense one of two thirds of GPT-2's inner size, and Ruzolorn's mixture at its sizes
    (sixteen experts of an eighth, four a token, a shared expert of a quarter)."""
    H, d, D = s["heads"], s["dim"], s["width"]
    G = max(1, H // 4)
    left = {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "scale": d ** -0.5, "softcap": 30.0}
    R = max(1, H // 2)
    right = {"heads": R, "dim": d, "vdim": d, "decay": [1.0 - 2.0 ** (-5.0 - 5.0 * h / max(1, R - 1)) for h in range(R)]}
    mixers = [("parallel", {"left": left, "right": right, "left_scale": 1.0, "right_scale": 1.0}),
              ("hgrn2", {"heads": H, "dim": d, "vdim": d}),
              ("attention", {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "scale": d ** -0.5, "bias_rows": 32, "bias_max": 128})]
    dense = {"kind": "dense", "ff": s["ff"] * 2 // 3 // 64 * 64}
    moe = {"kind": "moe", "expert": {"ff": s["ff"] // 8}, "router": {"experts": 16, "top": 4, "scale": 2.0}, "shared": {"ff": s["ff"] // 4}}
    layers = [{"type": mixers[i % 3][0], "mixer": mixers[i % 3][1], "mlp": moe if i % 3 == 1 else dense} for i in range(s["layers"])]
    return {"architecture": "Sazilorn", "vocab": DESIGN_VOCAB, "width": D, "max_positions": DESIGN_POSITIONS,
            "norm": {"eps": 1e-5}, "canon": {"taps": 4}, "layers": layers}


def bench_design(config, dtype, batches, steps, warmup):
    """Prefill of 2 x 1,024 tokens (three warm-up trials, the mean of five) and decode from
    context 512 at each of ``batches``, for the model that ``config`` describes."""
    import torch

    from mlx_lm_amd.engine import Engine, StepEntry

    model, _ = build_model(config, dtype, seed=2)
    V, P = model.decoder.vocab_size, model.decoder.max_positions
    engine = Engine(model, dtype=dtype, page_size=16, max_tokens=max(batches) * 1024 + 4096, max_requests=64,
                    record_prompt_steps=True)
    g = torch.Generator().manual_seed(0)
    prompts = torch.randint(0, V, (2, 1024), generator=g).tolist()
    ms = []
    for trial in range(8):
        for i in range(2):
            engine.add_request(("pre", i))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([StepEntry(("pre", i), prompts[i], [1023]) for i in range(2)])
        torch.cuda.synchronize()
        ms.append((time.perf_counter() - t0) * 1e3)
        for i in range(2):
            engine.end_request(("pre", i))
    pre = sum(ms[3:]) / 5
    out = {"prefill_ms": round(pre, 3), "prefill_tok_s": round(2048 / (pre / 1e3), 1),
           "weight_bytes": model.decoder.bytes_read_per_step(2 if dtype == "bfloat16" else 4)}
    for b in batches:
        dt, contexts = run_decode(engine, b, 512, min(steps, P - 514), warmup, V, seed=b)
        k = len(contexts)
        step_bytes = out["weight_bytes"] + b * (sum(contexts) / k) * engine.cache.bytes_per_token()
        out[f"decode_b{b}"] = {"tok_s": round(b * k / dt, 1), "ms_per_step": round(dt / k * 1e3, 4),
                               "hbm_frac": round(step_bytes / (dt / k) / 1e9 / PEAK_HBM_GBS, 4)}
    print(f"[bench] {config.get('model_type') or config.get('architecture')}: {out}", file=sys.stderr, flush=True)
    return out


def compare_designs(a):
    """The ``--designs`` mode: one JSON line with both designs' numbers at every size."""
    sizes = [a.design_size] if a.design_size else list(DESIGN_SIZES)
    batches = [1, 8, 32]
    line = {"metric": "prefill tok/s (2 x 1,024) and decode tok/s from context 512: Pafutar beside GPT-2 at equal sizes",
            "dtype": "bf16" if a.dtype == "bfloat16" else "fp32", "data": "synthetic token ids, random weights (seed 2)",
            "steps": a.steps, "warmup": a.warmup, "vocab": DESIGN_VOCAB, "positions": DESIGN_POSITIONS, "sizes": {}}
    for size in sizes:
        entry = {"layer_sizes": DESIGN_SIZES[size]}
        runs = {"gpt2": ("gpt2", None), "pafutar": ("pafutar", None), "pafutar_window_512_keep_64": ("pafutar", (512, 64)),
                "ruzolorn": ("ruzolorn", None), "ruzolorn_window_512": ("ruzolorn", (512, 0)), "zatinex": ("zatinex", None), "sazilorn": ("sazilorn", None)}
        for name, (design, window) in runs.items():
            if a.design_only and name != a.design_only:
                continue
            entry[name] = bench_design(design_config(design, size, window), a.dtype, batches, a.steps, a.warmup)
        line["sizes"][size] = entry
    print(json.dumps(line))


def build_model(config, dtype, seed):
    """Random weights under a checkpoint's names, loaded the way a folder's are."""
    from mlx_lm_amd.config import get_model_classes
    from mlx_lm_amd.utils import model_from_tensors

    model_cls, args_cls = get_model_classes(config)
    tensors = model_cls.random_weights(args_cls.from_dict(config), seed, "a")
    model = model_from_tensors(config, tensors, dtype=dtype, device="cuda:0")
    return model, model.args


def prefill_flops(args, n_seqs, seq_len):
    D, F, L, V = args.n_embd, args.n_inner, args.n_layer, args.vocab_size
    per_token = 2 * L * (3 * D * D + D * D + 2 * D * F)
    attn = n_seqs * L * 4 * D * seq_len * (seq_len + 1) / 2  # causal: half of QK^T and PV
    head = 2 * n_seqs * D * V
    return per_token * n_seqs * seq_len + attn + head


def _scheduler(engine, batch, prompt_len):
    from mlx_lm_amd.engine.scheduler import Scheduler
    from mlx_lm_amd.generate import make_sample_fn

    # all prompts go in one step, so that every request decodes from the same context on
    return Scheduler(engine, make_sample_fn(), max_num_seqs=batch,
                     max_num_batched_tokens=batch * (prompt_len + 1), prefill_step_size=prompt_len)


def _start(engine, sched, batch, prompt_len, vocab, seed, tag):
    import torch

    from mlx_lm_amd.engine.scheduler import Request

    g = torch.Generator().manual_seed(seed)
    prompts = torch.randint(0, vocab, (batch, prompt_len), generator=g).tolist()
    requests = [Request((tag, batch, i), prompts[i], max_tokens=10**6, seed=i)  # greedy; the caller ends it
                for i in range(batch)]
    for r in requests:
        sched.add(r)
    while sched.waiting or not all(r.decoding for r in sched.running):
        sched.step()
    return requests


def run_decode(engine, batch, prompt_len, steps, warmup, vocab, seed):
    """``batch`` requests of ``prompt_len`` tokens through the scheduler (the loop that generation
    uses: a step is launched while the host reads the tokens of the one before); times ``steps``
    decode steps.  Returns ``(seconds, contexts)``: the context each timed step ran at."""
    import torch

    sched = _scheduler(engine, batch, prompt_len)
    if warmup > 0:  # on requests of their own, so that the timed steps start at the prompt's end
        requests = _start(engine, sched, batch, prompt_len, vocab, seed + 1000, "warm")
        for _ in range(warmup):
            sched.step()
        torch.cuda.synchronize()
        for r in requests:
            sched.abort(r.request_id)
        while sched.has_work:
            sched.step()
    requests = _start(engine, sched, batch, prompt_len, vocab, seed, "bench")
    torch.cuda.synchronize()
    ctx0 = engine.context_len(requests[0].engine_id)
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    first.record()
    n_out = 0
    for _ in range(steps):
        n_out += len(sched.step())  # every step hands out one token per request
    last.record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    run_decode.gpu_seconds = first.elapsed_time(last) / 1e3
    if n_out != batch * steps:
        raise RuntimeError(f"{n_out} tokens came out of {steps} steps of {batch} requests")
    for r in requests:  # (a request that has reached the model's last position is over already)
        if r.live:
            sched.abort(r.request_id)
    while sched.has_work:
        sched.step()
    # steps overlap: the first timed call launches the step at the prompt's end, and every call
    # hands out the tokens of the step before, so `steps` calls ran `steps` steps
    return dt, list(range(ctx0, ctx0 + steps))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=512)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than GPT-2 XL has")
    ap.add_argument("--prompt-len", type=int, default=None)
    ap.add_argument("--n-positions", type=int, default=XL["n_positions"],
                    help="positions of the model; 8192: the long-context mode (12 layers unless --layers is given)")
    ap.add_argument("--no-points", action="store_true", help="skip the other batch sizes and contexts")
    ap.add_argument("--designs", action="store_true",
                    help="a mode of its own: Pafutar beside GPT-2 at equal layer sizes (prefill and decode)")
    ap.add_argument("--design-size", choices=sorted(DESIGN_SIZES), default=None, help="with --designs: one size only")
    ap.add_argument("--design-only", default=None, help="with --designs: one of gpt2, pafutar, pafutar_window_512_keep_64, ruzolorn, ruzolorn_window_512, zatinex, sazilorn")
    a = ap.parse_args()
    if a.designs:
        if a.gpus != 1:
            print("bench.py measures one GPU; this engine does not run on several (asked for %d)" % a.gpus)
            sys.exit(2)
        a.steps = min(a.steps, 128)
        return compare_designs(a)
    long_mode = a.n_positions != XL["n_positions"]
    if a.layers is None:
        a.layers = 12 if long_mode else XL["n_layer"]
    if a.prompt_len is None:
        a.prompt_len = a.n_positions * 7000 // 8192 if long_mode else 512
    if a.gpus != 1:
        print("bench.py measures one GPU; this engine does not run on several (asked for %d)" % a.gpus)
        sys.exit(2)

    import torch

    from mlx_lm_amd.engine import Engine, StepEntry

    config = dict(XL)
    config["n_layer"] = a.layers
    config["n_positions"] = config["n_ctx"] = a.n_positions
    t_build = time.perf_counter()
    model, args = build_model(config, a.dtype, seed=2)
    print(f"[bench] model built in {time.perf_counter() - t_build:.1f} s", file=sys.stderr, flush=True)
    P, V = args.n_positions, args.vocab_size
    # the step after a prompt of p tokens runs at context p; the token that takes the last position
    # (P - 1) is never fed, so the last step runs at context P - 2
    steps = max(1, min(a.steps, P - 1 - a.prompt_len))
    # (as the serving path makes it, generate.engine_for: steps of a shape that keeps coming back are recorded)
    engine = Engine(model, dtype=a.dtype, page_size=16, max_tokens=(8 if long_mode else 64) * P, max_requests=64,
                    record_prompt_steps=True)
    esize = 2 if a.dtype == "bfloat16" else 4
    kv_bytes_per_token = engine.cache.bytes_per_token()
    w_bytes = model.decoder.bytes_read_per_step(esize)

    # prefill: 2 x 1,024 tokens in one step (the long-context mode: one prompt of all the positions)
    g = torch.Generator().manual_seed(0)
    n_seqs, seq_len = (1, P) if long_mode else (2, 1024)
    prompts = torch.randint(0, V, (n_seqs, seq_len), generator=g).tolist()
    pre_ms, pre_gpu_ms = [], []
    # (the third sighting of the shape records it; the warm-up trials after it and the timed ones replay)
    warm_trials, timed_trials = max(3, a.warmup), 5
    for trial in range(warm_trials + timed_trials):
        for i in range(n_seqs):
            engine.add_request(("pre", i))
        torch.cuda.synchronize()
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        first.record()
        engine.step([StepEntry(("pre", i), prompts[i], [seq_len - 1]) for i in range(n_seqs)])
        last.record()
        torch.cuda.synchronize()
        pre_ms.append((time.perf_counter() - t0) * 1e3)
        pre_gpu_ms.append(first.elapsed_time(last))
        for i in range(n_seqs):
            engine.end_request(("pre", i))
    timed = pre_ms[warm_trials:]
    pre = sum(timed) / len(timed)
    flops = prefill_flops(args, n_seqs, seq_len)
    prefill = {"value": round(n_seqs * seq_len / (pre / 1e3), 1), "tokens": n_seqs * seq_len,
               "ms": round(pre, 3), "frac": round(flops / (pre / 1e3) / PEAK_FLOPS[a.dtype], 4),
               "trials_ms": [round(t, 3) for t in timed],
               "gpu_ms": round(sum(pre_gpu_ms[warm_trials:]) / timed_trials, 3)}
    print(f"[bench] prefill {prefill} (warm-up trials, ms: {[round(t, 2) for t in pre_ms[:warm_trials]]})",
          file=sys.stderr, flush=True)

    def measure(batch, prompt_len, k):
        dt, contexts = run_decode(engine, batch, prompt_len, k, a.warmup, V, seed=batch)
        ms = dt / k * 1e3
        gpu_ms = run_decode.gpu_seconds / k * 1e3
        step_bytes = w_bytes + batch * (sum(contexts) / len(contexts)) * kv_bytes_per_token
        gbs = step_bytes / (ms / 1e3) / 1e9
        print(f"[bench] decode batch {batch}, context {contexts[0]} to {contexts[-1]}: {batch * k / dt:.1f} tok/s, "
              f"{ms:.3f} ms/step ({gpu_ms:.3f} between events on the GPU), {gbs:.0f} GB/s", file=sys.stderr, flush=True)
        return {"tps": batch * k / dt, "ms": ms, "gpu_ms": gpu_ms, "gbs": gbs, "ctx": (contexts[0], contexts[-1]), "k": k}

    main_point = measure(a.batch, a.prompt_len, steps)
    points, fracs = {}, {f"decode_b{a.batch}": round(main_point["gbs"] / PEAK_HBM_GBS, 4)}
    if not a.no_points and long_mode:
        for b in sorted({1, a.batch}):
            for ctx in (P * 4000 // 8192, P * 7000 // 8192):
                r = main_point if (b, ctx) == (a.batch, a.prompt_len) else measure(b, ctx, min(steps, 128, P - 1 - ctx))
                points[f"decode_b{b}_ctx{ctx}"] = round(r["tps"], 1)
                fracs[f"decode_b{b}_ctx{ctx}"] = round(r["gbs"] / PEAK_HBM_GBS, 4)
    elif not a.no_points:
        for b in (1, 16, 32, 48, 64):
            r = main_point if b == a.batch else measure(b, a.prompt_len, steps)
            points[f"decode_b{b}"] = round(r["tps"], 1)
            fracs[f"decode_b{b}"] = round(r["gbs"] / PEAK_HBM_GBS, 4)
        late = min(1000, P - 8)
        for b in sorted({1, a.batch, 64}):
            r = measure(b, late, min(steps, P - 1 - late))
            points[f"decode_b{b}_ctx{late}"] = round(r["tps"], 1)
            fracs[f"decode_b{b}_ctx{late}"] = round(r["gbs"] / PEAK_HBM_GBS, 4)

    line = {
        "metric": "decode tok/s at batch 1/8/64; prefill tok/s at 2,048 tokens (GPT-2 XL)",
        "value": round(main_point["tps"], 1), "unit": "tokens/s", "n_gpus": 1, "steps": main_point["k"],
        "warmup": a.warmup, "ms_per_step": round(main_point["ms"], 4),
        "gpu_ms_per_step": round(main_point["gpu_ms"], 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if a.dtype == "bfloat16" else "fp32",
        "data": "synthetic uniform random token ids, random weights (seed 2)",
        "config": {"model": "gpt2-xl layer sizes", "n_layer": a.layers, "n_layer_full": XL["n_layer"],
                   "n_embd": args.n_embd, "n_head": args.n_head, "n_inner": args.n_inner,
                   "vocab_size": V, "n_positions": P, "layer_norm_epsilon": args.layer_norm_epsilon,
                   "global_batch": a.batch, "seq_len": P, "prompt_len": a.prompt_len,
                   "ctx_from": main_point["ctx"][0], "ctx_to": main_point["ctx"][1], "page_size": 16,
                   "parallelism": "none"},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(main_point["gbs"], 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(main_point["gbs"] / PEAK_HBM_GBS, 4)},
        "points": points,
        "roofline_points": fracs,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
