"""Decode and prefill throughput of the engine on one MI355X, at Qwen1.5-MoE-A2.7B layer sizes with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C]

A step is one decode step of the whole batch: the step function, greedy sampling on the GPU and the copy of the
chosen tokens to the host, exactly what the generation loop runs.  Prints one JSON line.

    python bench.py --sizes a14b --workload unequal         # 8 prompts of 512 to 4,096 tokens, then 256 decode steps
    python bench.py --dtype float32 --workload unequal      # true 32-bit: 64 prompts of 1 to 2,048 tokens, 64 steps

time the other two workloads: a batch of prompts of unequal lengths in one prompt step, then decode steps.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Qwen1.5-MoE-A2.7B layer sizes
A27B = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "vocab_size": 151936, "hidden_size": 2048, "num_hidden_layers": 24, "num_attention_heads": 16,
    "num_key_value_heads": 16, "intermediate_size": 5632, "moe_intermediate_size": 1408,
    "shared_expert_intermediate_size": 5632, "num_experts": 60, "num_experts_per_tok": 4, "norm_topk_prob": False,
    "decoder_sparse_step": 1, "mlp_only_layers": [], "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "use_sliding_window": False, "sliding_window": 32768, "max_window_layers": 24, "max_position_embeddings": 8192,
    "tie_word_embeddings": False, "torch_dtype": "bfloat16",
}
# the other Qwen2-MoE checkpoint's sizes, about 115 GB of bfloat16 weights (`--sizes a14b`)
A14B = dict(A27B, hidden_size=3584, num_hidden_layers=28, num_attention_heads=28, num_key_value_heads=4,
            intermediate_size=18944, moe_intermediate_size=2560, shared_expert_intermediate_size=20480, num_experts=64,
            num_experts_per_tok=8, sliding_window=131072, max_window_layers=28, max_position_embeddings=32768)
SIZES = {"a27b": (A27B, "Qwen1.5-MoE-A2.7B"), "a14b": (A14B, "Qwen2-57B-A14B")}
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
PREFILL_TOKENS = 2048


def layer_weight_elems(c, experts_used: float) -> float:
    H, Q = c["hidden_size"], c["num_attention_heads"] * (c["hidden_size"] // c["num_attention_heads"])
    KV = c["num_key_value_heads"] * (c["hidden_size"] // c["num_attention_heads"])
    attn = H * (Q + 2 * KV) + (Q + 2 * KV) + Q * H
    moe = c["num_experts"] * H + H + 3 * H * c["shared_expert_intermediate_size"] + experts_used * 3 * H * c["moe_intermediate_size"]
    return attn + moe + 2 * H


def decode_bytes(c, layers: int, batch: int, context: float, wbytes: int = 2, used: float | None = None) -> float:
    """Bytes a decode step has to read: every weight it uses once (`used` experts a layer, counted in a step of
    the run; without a count, what a batch of uniformly routed tokens reaches in expectation) and the keys and
    values of the live requests."""
    E, k = c["num_experts"], c["num_experts_per_tok"]
    if used is None:
        used = E * (1.0 - (1.0 - k / E) ** batch)
    hd = c["hidden_size"] // c["num_attention_heads"]
    w = layers * layer_weight_elems(c, used) + c["vocab_size"] * c["hidden_size"] + c["hidden_size"]
    kv = batch * context * layers * 2 * c["num_key_value_heads"] * hd
    return wbytes * (w + kv)


def prefill_flops(c, layers: int, T: int, rows_out: int = 1) -> float:
    H, nh = c["hidden_size"], c["num_attention_heads"]
    hd = H // nh
    Q, KV = nh * hd, c["num_key_value_heads"] * hd
    per_layer = (2 * T * H * (Q + 2 * KV) + 2 * T * Q * H + 4 * nh * hd * T * (T + 1) / 2
                 + 2 * T * H * (c["num_experts"] + 1)
                 + 2 * T * c["num_experts_per_tok"] * 3 * H * c["moe_intermediate_size"]
                 + 2 * T * 3 * H * c["shared_expert_intermediate_size"])
    return layers * per_layer + 2 * rows_out * H * c["vocab_size"]


def probe() -> int:
    """The measured counterparts of the published peaks: one JSON line."""
    import torch
    from turboquant_cpp_amd.csrc import ops
    dev = "cuda:0"

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e-3 / reps

    buf = torch.randint(0, 2 ** 31 - 1, (2 ** 28,), dtype=torch.int32, device=dev)      # 1 GiB
    nbytes = buf.numel() * 4
    out = {"metric": "measured peaks", "read_bytes": nbytes}
    for name, once in (("read_GBs", False), ("read_once_hint_GBs", True)):
        out[name] = round(nbytes / timed(lambda: ops.probe_stream(buf, once), 10) / 1e9, 0)
    del buf
    for shape in (32, 16):
        for name, seed in (("same_values", 0), ("random_values", 12345)):
            flop = [0.0]

            def run():
                flop[0] = ops.probe_mfma(shape, 512, 20000, seed, dev)
            t = timed(run, 3)
            out[f"mfma_{shape}_{name}_TFLOPs"] = round(flop[0] / t / 1e12, 0)
    out["published"] = {"hbm_GBs": PEAK_HBM_GBS, "bf16_TFLOPs": PEAK_FLOPS["bf16"] / 1e12}
    print(json.dumps(out))
    return 0


def plain_products(short: str) -> str:
    """Whose kernels run the plain products of a long prompt step (decode steps always run this library's own)."""
    from turboquant_cpp_amd.csrc import ops
    if short == "bf16" and ops._VENDOR:
        return f"hipBLASLt from {ops.VENDOR_MIN_ROWS} rows (TQ_PLAIN_PRODUCTS=own: this library's)"
    return "own kernels"


def count_experts(fn, engine):
    """Runs fn() (an eager decode step, part by part so that the routing can be watched) and returns the mean number of
    distinct experts a layer's router picked."""
    import torch
    from turboquant_cpp_amd.csrc import ops
    picked = []
    route = ops.route

    def counting_route(*a, **k):
        out = route(*a, **k)
        picked.append(int(torch.unique(out[0]).numel()))
        return out

    ops.route = counting_route
    executor, engine.native = engine.native, None
    try:
        result = fn()
    finally:
        ops.route = route
        engine.native = executor
    return result, sum(picked) / max(len(picked), 1)


def unequal_defaults(sizes: str) -> dict:
    """The two stated workloads of unequal prompts: the larger checkpoint's sizes in bfloat16 (8 prompts of 512 to 4,096
    tokens, seed 3, 256 decode steps) and the headline sizes in true 32-bit (64 prompts of 1 to 2,048, seed 4, 64 steps)."""
    big = sizes == "a14b"
    return {"batch": 8 if big else 64, "lo": 512 if big else 1, "hi": 4096 if big else 2048, "steps": 256 if big else 64,
            "seed": 3 if big else 4}


def unequal_workload(sizes: str, act: str, layers: int | None, wl: dict) -> dict:
    """A batch of prompts of unequal lengths in one prompt step, then decode steps; builds its own model with random
    weights and returns the record (the keys of the default run's line)."""
    import torch
    from turboquant_cpp_amd.csrc import ops
    from turboquant_cpp_amd.engine.model import random_model
    from turboquant_cpp_amd.engine.step import Engine
    from turboquant_cpp_amd.sampling.sampler import TokenFetch
    cfg, model_name = dict(SIZES[sizes][0]), SIZES[sizes][1]
    full_layers = cfg["num_hidden_layers"]
    layers = full_layers if layers is None else layers
    cfg["num_hidden_layers"] = cfg["max_window_layers"] = layers
    cfg["max_position_embeddings"] = wl["hi"] + wl["steps"] + 64
    short = "bf16" if act == "bfloat16" else "fp32"
    wbytes = 2 if act == "bfloat16" else 4
    dev = "cuda:0"
    t0 = time.time()
    model = random_model(cfg, seed=wl["seed"], act=act, device=dev)
    torch.cuda.synchronize()
    print(f"[bench] {model_name} sizes, {layers} layers, {short}: random weights on the device in {time.time() - t0:.1f}s "
          f"({model.weight_bytes / 1e9:.1f} GB)", file=sys.stderr, flush=True)
    V = cfg["vocab_size"]
    B = wl["batch"]
    g = torch.Generator().manual_seed(wl["seed"])
    lens = torch.randint(wl["lo"], wl["hi"] + 1, (B,), generator=g).tolist()
    prompts = [torch.randint(0, V, (n,), generator=g).tolist() for n in lens]
    page = 64
    engine = Engine(model, max_tokens=sum(-(-(n + wl["steps"] + 1) // page) * page for n in lens), page_size=page, max_slots=B)
    fetch = TokenFetch(dev, B)
    best = None
    for rep in range(2):                  # the first pass loads kernels and captures the decode graphs
        slots = engine.open(B)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = engine.step(slots, prompts)
        torch.cuda.synchronize()
        t_prompt = time.perf_counter() - t0
        tokens = ops.argmax(logits, act)
        used = None
        t0 = time.perf_counter()
        for i in range(wl["steps"]):
            fetch.start(tokens)
            if rep == 1 and i == 0:       # an eager step of the timed pass also counts the experts that are read
                graphs, engine.graphs = engine.graphs, None
                lg, used = count_experts(lambda: engine.step_from_device(slots, tokens), engine)
                engine.graphs = graphs
            else:
                lg = engine.step_from_device(slots, tokens)
            fetch.wait()
            tokens = ops.argmax(lg, act)
        torch.cuda.synchronize()
        t_decode = time.perf_counter() - t0
        engine.close(slots)
        best = (t_prompt, t_decode, used)
    t_prompt, t_decode, used = best
    T = sum(lens)
    sec = t_decode / wl["steps"]
    mean_total_ctx = T + B * (wl["steps"] + 1) / 2.0
    read = decode_bytes(cfg, layers, B, mean_total_ctx / B, wbytes, used)
    flops = sum(prefill_flops(cfg, layers, n, 0) for n in lens) + 2.0 * B * cfg["hidden_size"] * V
    out = {
        "metric": f"decode tok/s, batch {B} of unequal prompts ({wl['lo']}..{wl['hi']} tokens), {wl['steps']} steps "
                  f"({model_name} layer sizes, random weights)",
        "value": round(B / sec, 1), "unit": "tok/s", "n_gpus": 1, "steps": wl["steps"], "warmup": 0,
        "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic",
        "config": {"model": f"{model_name} sizes", "layers": layers, "layers_of_full_model": full_layers,
                   "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
                   "head_dim": cfg["hidden_size"] // cfg["num_attention_heads"], "vocab": V, "experts": cfg["num_experts"],
                   "top_k": cfg["num_experts_per_tok"], "expert_inner": cfg["moe_intermediate_size"],
                   "shared_inner": cfg["shared_expert_intermediate_size"], "global_batch": B,
                   "prompt_tokens": T, "longest_prompt": max(lens), "shortest_prompt": min(lens),
                   "weights": f"random N(0,0.02) seed {wl['seed']}", "kv_cache": short,
                   "experts_read_per_layer": round(used, 1), "parallelism": "single GPU"},
        "prefill": {"value": round(T / t_prompt, 1), "tokens": T, "ms": round(t_prompt * 1e3, 3),
                    "frac": round(flops / t_prompt / PEAK_FLOPS[short], 4), "plain_products": plain_products(short)},
        "roofline": {"bound": "hbm", "achieved": round(read / sec / 1e9, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(read / sec / 1e9 / PEAK_HBM_GBS, 4)},
        "decode": {"ms_total": round(t_decode * 1e3, 2), "gb_per_step": round(read / 1e9, 2)},
    }
    return out



def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--sizes", default="a27b", choices=sorted(SIZES), help="whose layer sizes (default: the headline model's)")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (default: all)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--points-context", type=int, default=2048)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true")
    ap.add_argument("--prefill-only", action="store_true", help="time only the prompt step (for profiles)")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                    help="length of the timed prompt (the contract's line has 2,048; other lengths are for profiles)")
    ap.add_argument("--one-stream", action="store_true",
                    help="no second stream in prompt steps: kernels run one after the other, so that a profile shows "
                         "each kernel's own time")
    ap.add_argument("--generate", action="store_true",
                    help="time the generation loop instead of bare steps: --batch prompts of 512 tokens, 256 new tokens "
                         "each, greedy and with the default sampling (temperature 0.7, top-p 0.9, repetition penalty)")
    ap.add_argument("--probe", action="store_true",
                    help="no model: what this GPU reaches on a plain read of memory and on the matrix instructions alone")
    ap.add_argument("--workload", default="steps", choices=["steps", "unequal"],
                    help="unequal: a batch of prompts of unequal lengths in one prompt step, then decode steps "
                         "(defaults per model: a14b 8 prompts of 512..4096, seed 3, 256 steps; float32 64 prompts of "
                         "1..2048, seed 4, 64 steps)")
    ap.add_argument("--prompt-min", type=int, default=None)
    ap.add_argument("--prompt-max", type=int, default=None)
    ap.add_argument("--decode-steps", type=int, default=None)
    ap.add_argument("--seed", type=int, default=None)
    ap.add_argument("--no-workloads", action="store_true",
                    help="leave out the two workloads of unequal prompts that the default run adds under \"workloads\"")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine runs on a single device)")
        return 2
    if args.probe:
        return probe()

    import torch
    from turboquant_cpp_amd.csrc import ops
    from turboquant_cpp_amd.engine.model import random_model
    from turboquant_cpp_amd.engine.step import Engine
    from turboquant_cpp_amd.sampling.sampler import TokenFetch

    cfg, model_name = dict(SIZES[args.sizes][0]), SIZES[args.sizes][1]
    full_layers = cfg["num_hidden_layers"]
    args.layers = full_layers if args.layers is None else args.layers
    cfg["num_hidden_layers"] = args.layers
    cfg["max_window_layers"] = args.layers
    n_prefill = args.prefill_tokens
    cfg["max_position_embeddings"] = max(args.context, args.points_context, n_prefill)
    act = args.dtype
    short = "bf16" if act == "bfloat16" else "fp32"
    dev = "cuda:0"
    ops.library(act)
    if args.workload == "unequal":
        wl = unequal_defaults(args.sizes)
        if args.batch != 8:
            wl["batch"] = args.batch
        for key, given in (("lo", args.prompt_min), ("hi", args.prompt_max), ("steps", args.decode_steps), ("seed", args.seed)):
            if given is not None:
                wl[key] = given
        print(json.dumps(unequal_workload(args.sizes, act, args.layers, wl)), flush=True)
        return 0
    t0 = time.time()
    model = random_model(cfg, seed=2, act=act, device=dev)
    torch.cuda.synchronize()
    print(f"[bench] {args.layers}-layer model with random weights on the device in {time.time() - t0:.1f}s "
          f"({model.weight_bytes / 1e9:.1f} GB)", file=sys.stderr, flush=True)
    V = cfg["vocab_size"]
    gen = torch.Generator().manual_seed(2)

    if args.generate:
        from turboquant_cpp_amd.engine.generate import GenerationOptions, generate
        P, N, B = 512, 256, args.batch
        engine = Engine(model, max_tokens=(P + N + 64) * B, page_size=64, max_slots=B)
        prompts = [torch.randint(0, V, (P,), generator=gen).tolist() for _ in range(B)]
        out = {"metric": f"generated tok/s, {B} prompts of {P} tokens, {N} new tokens each ({model_name}, random weights)",
               "unit": "tok/s", "dtype": short, "layers": args.layers}
        for name, opts in (("greedy", dict(temperature=0.0, rep_penalty=1.0)), ("default_sampling", dict())):
            for _ in range(2):      # the first pass loads kernels and captures the decode step
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                res = generate(engine, prompts, GenerationOptions(max_tokens=N, max_batch=B, loop_detection=False, **opts))
                torch.cuda.synchronize()
                dt = time.perf_counter() - t0
            n = sum(len(r.tokens) for r in res)
            out[name] = {"value": round(n / dt, 1), "tokens": n, "seconds": round(dt, 3)}
        print(json.dumps(out))
        return 0

    wbytes = 2 if act == "bfloat16" else 4

    def run_decode(batch: int, context: int, steps: int, warmup: int):
        """Prefills `batch` prompts so that the timed steps end at `context`, then times `steps` decode steps."""
        prompt_len = context - steps - warmup
        page = 64
        per_seq = -(-context // page) * page
        engine = Engine(model, max_tokens=per_seq * batch, page_size=page, max_slots=batch)
        if args.one_stream:
            engine.side_stream = None
        slots = engine.open(batch)
        prompts = [torch.randint(0, V, (prompt_len,), generator=gen).tolist() for _ in range(batch)]
        tp = time.time()
        logits = None
        # prompts go in one sequence at a time to bound the size of the activations
        for s, p in zip(slots, prompts):
            lg = engine.step([s], [p])
            logits = lg if logits is None else torch.cat([logits, lg])
        torch.cuda.synchronize()
        print(f"[bench] prefilled {batch} x {prompt_len} tokens in {time.time() - tp:.1f}s", file=sys.stderr, flush=True)
        tokens = ops.argmax(logits, act)
        fetch = TokenFetch(dev, batch)

        def one_step(ids):
            """As the generation loop does it: the step is issued from the tokens on the device, and the host
            reads those tokens (to look for end tokens) while the step runs."""
            fetch.start(ids)
            lg = engine.step_from_device(slots, ids)
            fetch.wait()
            return ops.argmax(lg, act)

        # the first warm-up step (which runs eagerly) also counts the distinct experts that each layer's router picks
        tokens, experts_used = count_experts(lambda: one_step(tokens), engine)
        for _ in range(warmup - 1):
            tokens = one_step(tokens)
        torch.cuda.synchronize()
        held = lambda: sum(engine.cache.length(s) for s in slots) / batch
        before = held()
        t = time.perf_counter()
        for _ in range(steps):
            tokens = one_step(tokens)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        # what a timed step read on average, from the cache's own count of positions: a step that finds L positions
        # writes one and reads L + 1; the first timed step finds `before`, the last one leaves `context`
        mean_ctx = (before + 1 + held()) / 2.0
        if held() != context or before != context - steps:
            raise RuntimeError(f"the timed steps ran from {before} to {held()} positions, not up to {context}")
        engine.close(slots)
        del engine
        torch.cuda.empty_cache()
        return dt / steps, mean_ctx, experts_used

    def run_prefill(T: int):
        engine = Engine(model, max_tokens=T + 64, page_size=64, max_slots=1)
        if args.one_stream:
            engine.side_stream = None
        prompt = torch.randint(0, V, (T,), generator=gen).tolist()
        times = []
        for i in range(4):
            slot = engine.open(1)
            torch.cuda.synchronize()
            t = time.perf_counter()
            engine.step(slot, [prompt])
            host = time.perf_counter() - t      # every launch is made; the chip may still be working
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t, host))
            engine.close(slot)
        del engine
        torch.cuda.empty_cache()
        return min(times[1:])

    pf, pf_host = run_prefill(n_prefill)
    if args.prefill_only:
        print(json.dumps({"metric": f"prefill tok/s at {n_prefill} tokens", "value": round(n_prefill / pf, 1),
                          "unit": "tok/s", "ms": round(pf * 1e3, 3), "host_ms": round(pf_host * 1e3, 3),
                          "layers": args.layers, "dtype": short,
                          "frac": round(prefill_flops(cfg, args.layers, n_prefill) / pf / PEAK_FLOPS[short], 4)}))
        return 0
    sec, mean_ctx, experts_used = run_decode(args.batch, args.context, args.steps, args.warmup)
    value = args.batch / sec
    read = decode_bytes(cfg, args.layers, args.batch, mean_ctx, wbytes, experts_used)
    achieved = read / sec / 1e9

    def point(b, ctx, s, mean, used):
        gb = decode_bytes(cfg, args.layers, b, mean, wbytes, used) / 1e9
        return {"tok_s": round(b / s, 1), "ms_per_step": round(s * 1e3, 4), "gb_per_step": round(gb, 2),
                "frac": round(gb / s / PEAK_HBM_GBS, 4)}

    # decode at batch 1 and 64 at the headline context, and every batch at the shorter context too
    points, detail = {}, {f"decode_b{args.batch}_ctx{args.context}": point(args.batch, args.context, sec, mean_ctx, experts_used)}
    if not args.no_points:
        for b in (1, 64):
            s, mean, used = run_decode(b, args.context, 32, 4)
            points[f"decode_b{b}"] = round(b / s, 1)
            detail[f"decode_b{b}_ctx{args.context}"] = point(b, args.context, s, mean, used)
        if args.points_context != args.context:
            for b in sorted({1, args.batch, 64}):
                s, mean, used = run_decode(b, args.points_context, 32, 4)
                detail[f"decode_b{b}_ctx{args.points_context}"] = point(b, args.points_context, s, mean, used)
    out = {
        "metric": f"decode tok/s at batch {args.batch}, context {args.context} ({model_name} layer sizes, random weights)",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic",
        "config": {
            "model": f"{model_name} sizes", "layers": args.layers, "layers_of_full_model": full_layers,
            "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
            "head_dim": cfg["hidden_size"] // cfg["num_attention_heads"], "vocab": V, "experts": cfg["num_experts"],
            "top_k": cfg["num_experts_per_tok"], "expert_inner": cfg["moe_intermediate_size"],
            "shared_inner": cfg["shared_expert_intermediate_size"], "global_batch": args.batch,
            "seq_len": args.context, "parallelism": "single GPU", "points_context": args.points_context,
            "prefill_tokens": n_prefill, "weights": "random N(0,0.02) seed 2", "kv_cache": short,
            "experts_read_per_layer": round(experts_used, 1),
        },
        "prefill": {"value": round(n_prefill / pf, 1), "tokens": n_prefill, "ms": round(pf * 1e3, 3),
                    "frac": round(prefill_flops(cfg, args.layers, n_prefill) / pf / PEAK_FLOPS[short], 4),
                    "plain_products": plain_products(short)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
        "points_detail": detail,
    }
    default_run = (args.sizes == "a27b" and act == "bfloat16" and args.layers == full_layers and not args.no_points
                   and not args.no_workloads)
    if default_run:
        # The two other stated workloads, each with a model of its own, once the headline model has left the device.
        # Whatever happens to them, the headline line is printed.
        import gc
        del model, run_decode, run_prefill
        gc.collect()
        torch.cuda.empty_cache()
        out["workloads"] = {}
        for name, sizes, dtype in (("a14b_bf16_unequal_b8", "a14b", "bfloat16"), ("a27b_fp32_unequal_b64", "a27b", "float32")):
            try:
                out["workloads"][name] = unequal_workload(sizes, dtype, None, unequal_defaults(sizes))
            except Exception as e:      # noqa: BLE001 - the record says what went wrong
                out["workloads"][name] = {"error": f"{type(e).__name__}: {e}"[:300]}
            gc.collect()
            torch.cuda.empty_cache()
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
