"""Command line in the manner of the reference's ``quant <model> [options]`` (/root/reference/tools/quant.c:126-163,
defaults :196-239): the model path first, then ``-p`` prompt, ``-n`` max tokens (256), ``-T`` temperature (0.7),
``-P`` top-p (0.9), ``-s`` seed (42), ``--ctx`` context length, ``--info``, ``--profile``, ``-M`` (the cache's memory per
token, :1382-1461), ``--bench-memory`` and ``--bench-prefill`` (:726-860), ``--version``.  There is no
tokenizer in this library, so a prompt is a list of token ids (``-p "5,17,3"``; several prompts are separated by
``;`` and run as one batch), or ``--random-prompt LEN[,LEN...]`` draws them.  ``--random-weights CONFIG.json --save
DIR`` is the random-weights mode: it writes a model folder for a configuration and a seed and exits.  ``--ppl FILE``
is the reference's teacher-forced perplexity (/root/reference/tools/quant.c:430-720) over a file of token ids, with its
report and, with ``--json``, its JSON; ``--save-logits FILE`` and ``--kl-baseline FILE`` go with it as in the reference
(:542-556, :594-636): the first writes every scored position's probabilities, the second reports the mean KL divergence
of such a file against this run (the 32-bit path against the bfloat16 path, for instance).  ``--save-kv FILE`` and
``--load-kv FILE`` are the reference's too (/root/reference/src/engine/tq_generate.c:268-362): the cache of one prompt
saved once it has run, and a later run that starts from it with its prompt behind the saved tokens.
"""
from __future__ import annotations

import argparse
import json
import sys
import time


def parse_prompts(text: str) -> list[list[int]]:
    prompts = []
    for part in text.split(";"):
        ids = [int(t) for t in part.replace(",", " ").split()]
        if ids:
            prompts.append(ids)
    if not prompts:
        raise ValueError("the prompt holds no token id")
    return prompts


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="turboquant_cpp_amd", description="Qwen2-MoE generation on one MI355X.")
    ap.add_argument("model", nargs="?", help="folder with config.json and model.safetensors")
    ap.add_argument("-p", dest="prompt", default=None, help='token ids of the prompt, e.g. "5,17,3"; ";" separates prompts')
    ap.add_argument("--tokens-file", default=None, metavar="FILE", help="prompts from a file: one prompt of token ids a line")
    ap.add_argument("--ppl", default=None, metavar="FILE", help="compute perplexity on a file of token ids (teacher-forced)")
    ap.add_argument("--save-kv", default=None, metavar="FILE",
                    help="one prompt: save the cache after the prompt has been run, before anything is generated")
    ap.add_argument("--load-kv", default=None, metavar="FILE",
                    help="one prompt: start from a saved cache; the prompt goes on behind its tokens")
    ap.add_argument("--save-logits", default=None, metavar="FILE",
                    help="with --ppl: write every scored position's probabilities (16-bit floats) to FILE")
    ap.add_argument("--kl-baseline", default=None, metavar="FILE",
                    help="with --ppl: mean KL(baseline || this run) against a file that --save-logits wrote")
    ap.add_argument("-n", dest="max_tokens", type=int, default=256, help="max tokens to generate (default: 256)")
    ap.add_argument("-T", dest="temperature", type=float, default=0.7, help="sampling temperature (default: 0.7)")
    ap.add_argument("-P", dest="top_p", type=float, default=0.9, help="top-p sampling (default: 0.9)")
    ap.add_argument("-s", dest="seed", type=int, default=42, help="random seed (default: 42)")
    ap.add_argument("-j", dest="threads", type=int, default=None, help="accepted for compatibility; the GPU does the work")
    ap.add_argument("--ctx", type=int, default=0, help="override max context length (default: the model's, at most 4096)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--f32-weights", default="bfloat16", choices=["bfloat16", "keep"],
                    help="with --dtype bfloat16: round matrices stored in 32 bits to bfloat16 at load (default), or keep them")
    ap.add_argument("--rep-penalty", type=float, default=1.1, help="repetition penalty over the last 32 tokens (default: 1.1)")
    ap.add_argument("--stop-id", type=int, action="append", default=None, help="stop token id (default: eos_token_id of config.json)")
    ap.add_argument("--random-prompt", default=None, metavar="LEN[,LEN...]", help="prompts of random token ids of these lengths")
    ap.add_argument("--max-batch", type=int, default=8, help="sequences that generate together")
    ap.add_argument("--info", action="store_true", help="print model info and exit")
    ap.add_argument("--bench-memory", action="store_true",
                    help="decode speed behind contexts of 10 to 500 tokens (BENCH_CSV lines) and exit")
    ap.add_argument("--bench-prefill", action="store_true", help="speed of a prompt of 200 tokens (a PREFILL_CSV line) and exit")
    ap.add_argument("-M", "--memory", action="store_true", help="print what the cache holds per token after the generation")
    ap.add_argument("--profile", action="store_true", help="time the prompt step and the decode steps")
    ap.add_argument("--json", action="store_true", help="print results as JSON")
    ap.add_argument("--version", action="store_true")
    ap.add_argument("--random-weights", metavar="CONFIG.json", default=None, help="write a model folder with random weights")
    ap.add_argument("--save", metavar="DIR", default=None, help="where --random-weights writes")
    ap.add_argument("--std", type=float, default=0.02)
    ap.add_argument("--norm-std", type=float, default=0.0)
    ap.add_argument("--file-dtype", default="bfloat16", choices=["bfloat16", "float32", "float16"])
    return ap


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.version:
        from . import __version__
        print(f"turboquant_cpp_amd v{__version__}")
        return 0
    if args.random_weights:
        if not args.save:
            print("--random-weights needs --save DIR", file=sys.stderr)
            return 2
        from .engine.model import write_random_model_dir
        with open(args.random_weights) as f:
            cfg = json.load(f)
        out = write_random_model_dir(args.save, cfg, args.seed, args.std, args.norm_std, args.file_dtype)
        print(f"wrote {out}", file=sys.stderr)
        return 0
    if not args.model:
        build_parser().print_usage(sys.stderr)
        return 2
    if args.info:
        from .config import config_from_dir
        arch, cfg = config_from_dir(args.model)
        print(f"architecture: {arch.name}")
        for k, v in vars(cfg).items():
            print(f"  {k}: {v}")
        return 0

    import torch
    from .api import Model
    t0 = time.time()
    model = Model(args.model, temperature=args.temperature, top_p=args.top_p, max_tokens=args.max_tokens,
                  context_length=args.ctx, dtype=args.dtype, seed=args.seed, rep_penalty=args.rep_penalty,
                  max_batch=args.max_batch, stop_tokens=args.stop_id, f32_matrices=args.f32_weights)
    print(f"loaded {args.model} in {time.time() - t0:.1f}s ({args.dtype}, context {model.context_length})", file=sys.stderr)
    if args.bench_memory or args.bench_prefill:
        # the reference's two small benchmarks (/root/reference/tools/quant.c:726-800, :804-860): one token, its token
        # 1, repeated as the context
        eng = model.engine
        tok = min(1, eng.vocab_size - 1)
        if args.bench_memory:
            print("\n=== Memory Bandwidth Benchmark ===", file=sys.stderr)
            print(f"KV type: {args.dtype}", file=sys.stderr)
            print(f"{'Context':<12} {'Tok/s':<12} {'Time(s)':<12}", file=sys.stderr)
            print("-------- -------- --------", file=sys.stderr)
            for ctx in (10, 50, 100, 200, 500):
                n_gen = min(20, model.context_length - ctx - 1)
                if ctx >= model.context_length or n_gen < 1:
                    continue
                for timed in (False, True):          # the first pass loads kernels and captures the decode step
                    slot = eng.open(1)
                    eng.step(slot, [[tok] * ctx], [[]])
                    torch.cuda.synchronize()
                    t1 = time.time()
                    for _ in range(n_gen):
                        eng.step(slot, [[tok]])
                    torch.cuda.synchronize()
                    elapsed = time.time() - t1
                    eng.close(slot)
                print(f"{ctx:<12d} {n_gen / elapsed:<12.1f} {elapsed:<12.3f}", file=sys.stderr)
                print(f"BENCH_CSV:{ctx},{n_gen / elapsed:.2f},{elapsed:.4f}", file=sys.stderr)
            print("==================================", file=sys.stderr)
        if args.bench_prefill:
            n = min(200, model.context_length - 1)
            print("\n=== Prefill Speed Benchmark ===", file=sys.stderr)
            print(f"Prefill length: {n} tokens", file=sys.stderr)
            print(f"{'KV Config':<28} {'Tok/s':<12} {'Time(s)':<12}", file=sys.stderr)
            print("---------------------------- ------------ ------------", file=sys.stderr)
            for timed in (False, True):
                slot = eng.open(1)
                torch.cuda.synchronize()
                t1 = time.time()
                eng.step(slot, [[tok] * n])
                torch.cuda.synchronize()
                elapsed = time.time() - t1
                eng.close(slot)
            name = f"{args.dtype} (no quant)"
            print(f"{name:<28} {n / elapsed:<12.1f} {elapsed:<12.3f}", file=sys.stderr)
            print(f"PREFILL_CSV:{name},{n},{n / elapsed:.2f},{elapsed:.4f}", file=sys.stderr)
            print("===============================", file=sys.stderr)
        model.close()
        return 0
    if args.ppl:
        with open(args.ppl) as f:
            ids = [int(t) for t in f.read().replace(",", " ").split()]
        print(f"PPL evaluation: {min(len(ids), model.context_length)} tokens from {args.ppl}", file=sys.stderr)
        torch.cuda.synchronize()
        t1 = time.time()
        res = model.perplexity(ids, save_logits=args.save_logits, kl_baseline=args.kl_baseline)
        elapsed = time.time() - t1
        rate = res["tokens_evaluated"] / elapsed if elapsed > 0 else 0.0
        print("\n=== Perplexity Results ===", file=sys.stderr)
        print(f"File:         {args.ppl}", file=sys.stderr)
        print(f"Tokens:       {res['tokens']} (evaluated {res['tokens_evaluated']})", file=sys.stderr)
        print(f"KV type:      {args.dtype}", file=sys.stderr)
        print(f"Avg NLL:      {res['avg_nll']:.6f}", file=sys.stderr)
        print(f"Perplexity:   {res['perplexity']:.4f}", file=sys.stderr)
        print(f"Time:         {elapsed:.1f}s ({rate:.1f} tok/s)", file=sys.stderr)
        print("==========================", file=sys.stderr)
        if args.kl_baseline and res["kl_tokens"]:
            print(f"KL divergence (baseline || this run): mean = {res['mean_kl']:.6f} over {res['kl_tokens']} tokens", file=sys.stderr)
        if args.save_logits:
            print(f"Saved logits to {args.save_logits}", file=sys.stderr)
        print(f"PPL_CSV:{res['tokens_evaluated']},{res['avg_nll']:.6f},{res['perplexity']:.4f}", file=sys.stderr)
        if args.json:
            print(json.dumps({"model": args.model, "benchmark": args.ppl, "tokens": res["tokens"],
                              "tokens_evaluated": res["tokens_evaluated"], "kv_type": args.dtype,
                              "perplexity": round(res["perplexity"], 4), "avg_nll": round(res["avg_nll"], 6),
                              "elapsed_s": round(elapsed, 2), "tok_per_s": round(rate, 1),
                              **({"mean_kl": res["mean_kl"], "kl_tokens": res["kl_tokens"]} if args.kl_baseline else {})},
                             indent=2))
        model.close()
        return 0
    if args.tokens_file:
        with open(args.tokens_file) as f:
            prompts = [p for line in f if line.strip() for p in parse_prompts(line)]
        if not prompts:
            raise ValueError(f"{args.tokens_file} holds no token id")
    elif args.random_prompt:
        g = torch.Generator().manual_seed(args.seed)
        V = model.engine.vocab_size
        prompts = [torch.randint(0, V, (int(n),), generator=g).tolist() for n in args.random_prompt.split(",")]
    else:
        prompts = parse_prompts(args.prompt if args.prompt is not None else "1")
    torch.cuda.synchronize()
    t1 = time.time()
    if args.save_kv or args.load_kv:
        # the reference's --load-kv / --save-kv (/root/reference/src/engine/tq_generate.c:268-362): the loaded cache
        # holds the first positions and the prompt goes on behind them; the cache is saved when the prompt has run
        from .engine.generate import GenerationResult
        if len(prompts) != 1:
            raise ValueError("--save-kv and --load-kv take one prompt")
        before = []
        if args.load_kv:
            model.load_context(args.load_kv)
            before = model.chat_tokens
            print(f"[load-kv] Loaded {len(before)} tokens from {args.load_kv}", file=sys.stderr)
        history = before + list(prompts[0])
        if args.save_kv:
            n = model.feed(history)
            model.save_context(args.save_kv)
            print(f"[save-kv] Saved {n} tokens to {args.save_kv}", file=sys.stderr)
        results = [GenerationResult(model.chat(history), model.last_finish_reason)]
    else:
        results = model.generate_detailed(prompts)
    torch.cuda.synchronize()
    elapsed = time.time() - t1
    n_generated = sum(len(r.tokens) for r in results)
    if args.json:
        print(json.dumps([{"tokens": r.tokens, "finish_reason": r.finish_reason} for r in results]))
    else:
        for i, r in enumerate(results):
            print(f"[{i}] {' '.join(str(t) for t in r.tokens)}  ({r.finish_reason})")
    if n_generated > 0 and elapsed > 0:
        print(f"{n_generated} tokens in {elapsed:.1f}s ({n_generated / elapsed:.1f} tok/s, {len(prompts)} sequences, "
              f"weights={args.dtype}, kv={args.dtype})", file=sys.stderr)
    if args.memory and n_generated > 0:
        # the reference's report (/root/reference/tools/quant.c:1382-1461), for a cache that is not compressed: what a
        # token costs in every layer that keeps keys and values, against keys and values in 16-bit floats
        cache = model.engine.cache
        esz = 4 if args.dtype == "float32" else 2
        # what the cache held of each sequence when it ended: a token that ended a sequence was never run, and a group
        # with a window has given its older pages back
        n_tok = sum(r.cached_positions for r in results) or sum(len(p) + len(r.tokens) for p, r in zip(prompts, results))
        k_per = sum(len(g.entries) * g.key.num_kv_heads * g.key.head_dim * esz for g in cache.groups)
        v_per = sum(len(g.entries) * g.key.num_kv_heads * g.key.value_dim * esz for g in cache.groups)
        f16_per = (k_per + v_per) // esz * 2
        if all(r.pages_held for r in results):
            held = [sum(min(r.cached_positions, r.pages_held[i] * cache.page_size) for r in results)
                    for i in range(len(cache.groups))]
            total = sum(len(g.entries) * g.key.num_kv_heads * (g.key.head_dim + g.key.value_dim) * esz * n
                        for g, n in zip(cache.groups, held))
            total16 = total // esz * 2
        else:
            total, total16 = (k_per + v_per) * n_tok, f16_per * n_tok
        ratio = total16 / total if total else 0.0
        print("\n=== KV Cache Memory Stats ===", file=sys.stderr)
        print(f"Tokens in cache:      {n_tok}", file=sys.stderr)
        print("Model config:         " + "; ".join(
            f"{len(g.entries)} layers, {g.key.num_kv_heads} kv_heads, head_dim={g.key.head_dim}"
            + (f", window={g.key.window}" if g.key.window else "") for g in cache.groups), file=sys.stderr)
        print(f"KV type:              {args.dtype}", file=sys.stderr)
        print(f"Per-token K ({args.dtype}): {k_per / 1024:.2f} KB", file=sys.stderr)
        print(f"Per-token V ({args.dtype}): {v_per / 1024:.2f} KB", file=sys.stderr)
        print(f"Per-token K+V total:  {(k_per + v_per) / 1024:.2f} KB", file=sys.stderr)
        print(f"Per-token K+V (FP16): {f16_per / 1024:.2f} KB", file=sys.stderr)
        print(f"Total K+V:            {total / 1024 / 1024:.2f} MB", file=sys.stderr)
        print(f"Total K+V (FP16):     {total16 / 1024 / 1024:.2f} MB", file=sys.stderr)
        print(f"Compression ratio:    {ratio:.2f}x (K+V combined)", file=sys.stderr)
        print(f"Weights:              {model._model.weight_bytes / 1024 / 1024:.2f} MB; cache pool: {cache.bytes() / 1024 / 1024:.2f} MB",
              file=sys.stderr)
        print("=============================", file=sys.stderr)
        print(f"MEMORY_CSV:{n_tok},{total},{total16},{ratio:.4f}", file=sys.stderr)
    if args.profile:
        # Where the time of a forward pass goes, by kind of work, in the reference's line
        # (/root/reference/src/engine/tq_transformer.c:2995-3020): steps run eagerly on one stream, an event behind
        # every launch.
        from .csrc import ops
        from .engine.step import Engine
        eng = Engine(model._model, max_tokens=sum(-(-(len(p) + 17) // 64) * 64 for p in prompts), page_size=64,
                     max_slots=len(prompts), use_graphs=False)
        eng.side_stream = None
        slots = eng.open(len(prompts))
        print("[Profile] steps are timed eagerly on one stream, an event behind every launch; generation replays its "
              "decode steps as graphs, which take less", file=sys.stderr)

        def report(phase, n_tok, steps):
            t = ops.profile_end()
            per = t["total"] / n_tok if n_tok else 0.0
            pct = {k: 100.0 * t[k] / t["total"] if t["total"] > 0 else 0.0 for k in ("matmul", "moe", "attn", "other")}
            print(f"[Profile {phase}, {n_tok} tok] matmul={pct['matmul']:.1f}% moe={pct['moe']:.1f}% attn={pct['attn']:.1f}% "
                  f"other={pct['other']:.1f}% | per-tok: {per:.4f}ms (mat={t['matmul'] / n_tok:.4f} moe={t['moe'] / n_tok:.4f} "
                  f"attn={t['attn'] / n_tok:.4f} other={t['other'] / n_tok:.4f}) | per-step: {t['total'] / steps:.3f}ms",
                  file=sys.stderr)
            print(f"PROFILE_CSV:{phase},{n_tok},{t['total']:.3f},{t['matmul']:.3f},{t['moe']:.3f},{t['attn']:.3f},{t['other']:.3f}",
                  file=sys.stderr)
            for name, (calls, ms) in sorted(t["kernels"].items(), key=lambda kv: -kv[1][1]):
                print(f"    {name:28s} {calls:6d} launches {ms:10.3f} ms {100.0 * ms / t['total']:5.1f}%", file=sys.stderr)

        eng.step(slots, [list(p) for p in prompts])            # the kernels' first launches are not timed
        eng.close(slots)
        slots = eng.open(len(prompts))
        ops.profile_begin()
        eng.step(slots, [list(p) for p in prompts])
        report("prompt", sum(len(p) for p in prompts), 1)
        eng.step(slots, [[1] for _ in prompts])
        ops.profile_begin()
        for _ in range(16):
            eng.step(slots, [[1] for _ in prompts])
        report("decode", 16 * len(prompts), 16)
        eng.close(slots)
    model.close()
    return 0
