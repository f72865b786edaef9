"""Decode and prefill throughput of the Qwen3-8B shape with random weights, as one JSON line.

Method after the reference's own bench (crates/leone/src/runtime.rs:1998-2002, 11342-11348;
crates/leone-cli/src/main.rs:4655-4802): fixed token ids, prefill timed to the synchronised end of
the step, decode timed over contiguous steps including the per-step copy of the chosen tokens to the
host, rate = tokens / duration, roofline = bytes a step must read / its time.
"""
from __future__ import annotations

import argparse
import json
import sys
import time
from typing import List, Optional

QWEN3_8B = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=36, hidden_size=4096,
                num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288,
                vocab_size=151936, max_position_embeddings=40960, rope_theta=1000000.0, rms_norm_eps=1e-6,
                tie_word_embeddings=False)
CONTEXT = 8192
PREFILL_TOKENS = 2048
STATED_PROMPT, STATED_NEW = 2048, 256     # the decode workload the configuration states
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def matmul_params(c) -> int:
    """Weights every token multiplies with, head excluded."""
    per_layer = (c.hidden_size * (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim
                 + c.num_attention_heads * c.head_dim * c.hidden_size + 3 * c.hidden_size * c.intermediate_size)
    return c.num_hidden_layers * per_layer


def prefill_flops(c, tokens: int, start: int = 0) -> float:
    gemm = 2.0 * tokens * matmul_params(c) + 2.0 * c.hidden_size * c.vocab_size          # head for one row
    keys = tokens * start + tokens * (tokens + 1) / 2.0                                   # causal pairs
    attention = c.num_hidden_layers * 4.0 * c.num_attention_heads * c.head_dim * keys
    return gemm + attention


def cache_bytes_per_token(model) -> int:
    """Bytes of keys and values one cached token takes over all cache slots of the model."""
    from .api import cache_bytes_per_token as per_token
    return per_token(model)


def decode_bytes(model, batch: int, context: float) -> float:
    """Bytes one decode step has to read: every weight it uses once (the model's own accounting), the rows
    of the stream, and the cache of the live requests."""
    size = 2 if str(model.dtype).endswith("bfloat16") else 4
    return (model.decode_step_weight_bytes(rows=batch) + batch * model.spec.hidden_size * size
            + batch * context * cache_bytes_per_token(model))


def measure_peaks(device: str = "cuda:0", megabytes: int = 1024, repeats: int = 5) -> dict:
    """What this GPU gives with nothing else going on: GB/s of a read and of a copy of a buffer several times
    the size of the caches, and TFLOP/s of a register-only loop of bfloat16 matrix instructions (own kernels,
    ``csrc/peaks.hip``; the reference's bench measures its stream rate the same way,
    crates/leone-cli/src/main.rs:4655-4802).  The best of ``repeats`` runs each."""
    import torch
    from .ops.library import call, library
    from . import ops
    count = megabytes * (1 << 20)
    src = torch.empty(count, dtype=torch.uint8, device=device)
    src.random_(0, 255)
    dst = torch.empty_like(src)
    sink = torch.zeros(4, dtype=torch.int32, device=device)
    units = ops.compute_units(device)
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def best_ms(launch):
        launch()
        found = None
        for _ in range(repeats):
            first.record()
            launch()
            last.record()
            torch.cuda.synchronize()
            ms = first.elapsed_time(last)
            found = ms if found is None else min(found, ms)
        return found

    stream = ops._stream()
    # how many workgroups a compute unit read fastest differs between a read and a copy: the best of a few
    read_ms = min(best_ms(lambda: call("leone_peak_read", src.data_ptr(), count, sink.data_ptr(), per * units, stream))
                  for per in (1, 2, 4, 8))
    copy_ms = min(best_ms(lambda: call("leone_peak_copy", src.data_ptr(), dst.data_ptr(), count, per * units, stream))
                  for per in (1, 2, 4, 8))
    iterations = 4000
    mfma_ms, blocks = min((best_ms(lambda: call("leone_peak_mfma", per * units, iterations, wide, sink.data_ptr(), stream)) / per,
                           per * units) for per in (4, 8) for wide in (0, 1))
    mfma_ms *= blocks // units
    flops = library().leone_peak_mfma_flops(blocks, iterations)
    return {"hbm_read_gbs": round(count / read_ms / 1e6, 1), "hbm_copy_gbs": round(2 * count / copy_ms / 1e6, 1),
            "mfma_bf16_tflops": round(flops / mfma_ms / 1e9, 1), "buffer_mb": megabytes}


def fill_cache(engine, batch: int, tokens: int, seed: int = 0):
    """Live requests with `tokens` positions each, their pages holding random keys and values (the
    timed steps read them; what they hold does not change the work)."""
    import torch
    gen = torch.Generator(device=engine.device)
    gen.manual_seed(seed)
    for k_pool, v_pool in ([] if getattr(engine, "_bench_filled", False) else engine.pools.kv.values()):
        for pool in (k_pool, v_pool):
            flat = pool.view(-1)
            for at in range(0, flat.numel(), 1 << 28):
                part = flat[at:at + (1 << 28)]
                part.copy_(torch.randn(part.numel(), generator=gen, device=engine.device, dtype=torch.float32) * 0.5)
    engine._bench_filled = True
    for b in range(batch):
        engine.admit(("bench", b))
        engine.cache.reserve(("bench", b), tokens)
        engine.cache.commit(("bench", b))


def time_decode(engine, batch: int, start_context: int, steps: int, warmup: int, seed: int = 1,
                profile_steps: int = 0, pipelined: bool = True):
    """(seconds of ``steps`` decode steps, mean context over them[, per-operation profile of further steps])."""
    import torch
    from .engine.engine import StepEntry
    from . import ops
    fill_cache(engine, batch, start_context)
    gen = torch.Generator().manual_seed(seed)
    tokens = torch.randint(0, engine.vocab_size, (batch,), generator=gen).tolist()

    # A step is issued with the tokens the step before it is choosing still on the device; then that step's tokens
    # are copied to the host (every step's are, one step late), as the generation loop does (``Generator``,
    # ``look_ahead``): what the host does for a step overlaps the step before it.  ``pipelined`` False: the step,
    # the choice and the copy one after the other, as the reference's loop.
    waiting, waiting_turn = [], []
    pinned = [torch.empty(batch, dtype=torch.int32).pin_memory() for _ in range(2)]

    def one_step(tokens):
        if not pipelined:
            out = engine.step([StepEntry(("bench", b), [tokens[b]], [0]) for b in range(batch)])
            return ops.argmax(out.logits).cpu().tolist()       # the per-step copy of the chosen tokens
        chosen, on_host, arrived = waiting.pop() if waiting else (None, None, None)
        out = engine.step([StepEntry(("bench", b), [tokens[b]], [0]) for b in range(batch)], device_tokens=chosen)
        picked = ops.argmax(out.logits)
        # the copy to the host is asked for at once and waited for by its event, one step later: asked for then, it
        # would queue behind the step issued meanwhile
        buffer = pinned[len(waiting_turn) % 2]
        waiting_turn.append(0)
        buffer.copy_(picked, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        waiting.append((picked, buffer, event))
        if chosen is None:
            return tokens
        arrived.synchronize()
        return on_host.tolist()

    for _ in range(warmup):
        tokens = one_step(tokens)
    torch.cuda.synchronize()
    started = time.perf_counter()
    for _ in range(steps):
        tokens = one_step(tokens)
    if waiting:
        waiting.pop()[2].synchronize()                       # the last step's tokens
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - started
    profiled = None
    pipelined = False
    if profile_steps:
        from .ops.profile import Recorder
        recorder = Recorder(profile_steps)
        for _ in range(profile_steps):
            recorder.begin_step()
            tokens = one_step(tokens)
            recorder.end_step(batch)
        profiled = recorder.profile
    for b in range(batch):
        engine.release(("bench", b))
    mean_context = start_context + warmup + (steps + 1) / 2.0
    return (elapsed, mean_context, profiled) if profile_steps else (elapsed, mean_context)


def time_generate(engine, batch: int, prompt_tokens: int, new_tokens: int, seed: int = 3, sampling=None) -> dict:
    """The stated workload through the generation loop itself, as the reference's bench runs it (prefill the
    prompt, sample, then time decoding: crates/leone/src/runtime.rs:2006-2050): ``batch`` prompts of
    ``prompt_tokens`` random tokens are submitted to a ``Generator`` (scheduler, real prefill a whole prompt a
    step, pages taken as tokens arrive, greedy choice on the device, tokens reported back), ``new_tokens``
    tokens each (``sampling``: another policy than greedy for all of them).  Timed, on the wall clock around ``Generator.step`` (planning, the step, sampling, the copy of
    the tokens, completion), are the steps that hold one decoded token of every request and nothing else: the
    same work as the bare step loop of ``time_decode`` plus everything the loop leaves out."""
    import torch
    from .engine.generate import Generator
    from .engine.scheduler import SchedulerPolicy
    from .sampling.sampler import SamplingParams
    gen = torch.Generator().manual_seed(seed)
    prompts = [torch.randint(0, engine.vocab_size, (prompt_tokens,), generator=gen).tolist() for _ in range(batch)]
    # a whole prompt beside the tokens the earlier requests decode meanwhile; a multiple of 256 (see SchedulerPolicy)
    policy = SchedulerPolicy(max_live_requests=batch, prefill_chunk_tokens=prompt_tokens,
                             max_step_tokens=prompt_tokens + 256 * -(-batch // 256))
    generator = Generator(engine, policy)
    for i, prompt in enumerate(prompts):
        generator.submit(("generate", i), prompt, new_tokens, sampling or SamplingParams(), None)
    seconds, tokens, steps, total_started = 0.0, 0, 0, time.perf_counter()
    while generator.scheduler.has_work():
        before = (generator.stats.decode_tokens, generator.stats.prefill_tokens)
        started = time.perf_counter()
        generator.step()
        elapsed = time.perf_counter() - started
        if generator.stats.decode_tokens - before[0] == batch and generator.stats.prefill_tokens == before[1]:
            steps += 1
            if steps > 4:                         # the first steps of a size record their graph
                seconds += elapsed
                tokens += batch
    torch.cuda.synchronize()
    engine.cache.check()
    assert not engine.cache.live_requests() and generator.stats.emitted_tokens == batch * new_tokens
    return {"tok_s": tokens / seconds if seconds else 0.0, "timed_steps": steps - 4,
            "prefill_tok_s": generator.stats.prefill_rate, "wall_s": time.perf_counter() - total_started}


def kernel_table(profiled, model, batch: int, context: float) -> dict:
    """Per operation of a decode step: microseconds a step and, where the operation streams something, the
    GB/s it reached (products: their weight bytes; attention: the cache of the live requests)."""
    steps = max(profiled.steps, 1)
    table = {}
    for name in profiled.operations():
        table[name] = {"us": round(profiled.seconds_by_operation[name] * 1e6 / steps, 1)}
    for (name, rows, columns, size), timing in sorted(profiled.products.items()):
        key = f"{name} {rows}x{columns}"
        table[key] = {"us": round(timing.seconds * 1e6 / steps, 1), "calls": timing.calls // steps,
                      "gbs": round(rows * columns * size * timing.calls / timing.seconds / 1e9, 1)}
    if "attention" in table:
        seconds = profiled.seconds_by_operation["attention"] / steps
        table["attention"]["gbs"] = round(batch * context * cache_bytes_per_token(model) / seconds / 1e9, 1)
    return table


def time_prefill(engine, tokens: int, repeats: int = 3, seed: int = 2, portion: Optional[int] = None):
    """Seconds of the best of ``repeats`` runs of a prompt of ``tokens`` tokens from position 0, in one step or
    (``portion``) in portions of that many tokens."""
    import torch
    from .engine.engine import StepEntry
    gen = torch.Generator().manual_seed(seed)
    prompt = torch.randint(0, engine.vocab_size, (tokens,), generator=gen).tolist()
    best = None
    for i in range(repeats + 1):
        torch.cuda.synchronize()
        started = time.perf_counter()
        for at in range(0, tokens, portion or tokens):
            part = prompt[at:at + (portion or tokens)]
            out = engine.step([StepEntry("prefill", part, [len(part) - 1] if at + len(part) == tokens else [])])
        out.logits.sum().item()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        engine.release("prefill")
        if i > 0:                                            # the first run warms up
            best = elapsed if best is None else min(best, elapsed)
    return best


QWEN3_14B = dict(QWEN3_8B, num_hidden_layers=40, hidden_size=5120, num_attention_heads=40, intermediate_size=17408)
QWEN3_32B = dict(QWEN3_8B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, intermediate_size=25600)

# Serving scenarios beside the headline figure: continuous batching with chunked prefill, and page pressure.
SCENARIOS = {
    # 32 requests, prompts uniform in 128..4096, prompt portions of 512, 128 greedy tokens each
    "mixed14b": dict(config=QWEN3_14B, requests=32, prompt=(128, 4096), new_tokens=128, chunk=512, temperature=None,
                     live=32, pool_fraction=1.0),
    # 16 requests of 4096 tokens, 256 tokens at temperature 0.7, the page pool at 60 % of what all would need
    "pressure32b": dict(config=QWEN3_32B, requests=16, prompt=(4096, 4096), new_tokens=256, chunk=1024,
                        temperature=0.7, live=16, pool_fraction=0.6),
    # one prompt of 32,768 tokens in portions of 512 (late portions: few rows over many keys), then 64 tokens
    "long32k": dict(config=QWEN3_8B, requests=1, prompt=(32768, 32768), new_tokens=64, chunk=512, temperature=None,
                    live=1, pool_fraction=1.0),
}


def trial_portion(engine, rows: int) -> None:
    """One prompt portion of ``rows`` tokens on a request of its own, released again: a process's first step of a
    size costs a quarter of a second more than any later one (the libraries load their kernels), which is not
    what a serving figure should hold."""
    import torch
    from .engine.engine import StepEntry
    rows = min(rows, engine.max_context)
    engine.step([StepEntry(("trial portion",), [(i * 7919) % engine.vocab_size for i in range(rows)], [rows - 1])])
    engine.release(("trial portion",))
    torch.cuda.synchronize()


def run_scenario(name: str, dtype: str = "bfloat16", layers: Optional[int] = None, tuned_products: bool = False) -> dict:
    import torch
    from .architectures import config_from_dict
    from .engine.engine import Engine
    from .engine.generate import Generator
    from .engine.scheduler import SchedulerPolicy
    from .runtime import random_model
    from .sampling.sampler import SamplingParams

    sc = SCENARIOS[name]
    raw = dict(sc["config"])
    full_layers = raw["num_hidden_layers"]
    if layers is not None:
        raw["num_hidden_layers"] = layers
    config = config_from_dict(raw)
    model = random_model(config, seed=0, dtype=dtype)
    gen = torch.Generator().manual_seed(7)
    lo, hi = sc["prompt"]
    lengths = [int(torch.randint(lo, hi + 1, (1,), generator=gen)) for _ in range(sc["requests"])]
    prompts = [torch.randint(0, config.vocab_size, (n,), generator=gen).tolist() for n in lengths]
    page_tokens = 64
    needed = sum((n + sc["new_tokens"] + page_tokens - 1) // page_tokens for n in lengths)
    pages = max(int(needed * sc["pool_fraction"]), (max(lengths) + sc["new_tokens"]) // page_tokens + 2)
    engine = Engine(model, num_pages=pages, page_tokens=page_tokens, max_requests=sc["live"],
                    max_context=max(lengths) + sc["new_tokens"] + 1)
    # The budget of a step is the portion size itself: decoded tokens take their rows out of the portion, and the
    # step keeps the row count the library's products do well with (a step of 544 rows of the 8B shape takes 11.8 ms,
    # one of 512 rows 10.0).
    policy = SchedulerPolicy(max_live_requests=sc["live"], prefill_chunk_tokens=sc["chunk"],
                             max_step_tokens=sc["chunk"])
    # before the clock starts: one trial portion, or (on request) the measured choice of the library's algorithms
    tuned = engine.tune_products(sc["chunk"]) if dtype == "bfloat16" and tuned_products else []
    if not tuned:
        trial_portion(engine, sc["chunk"])
    generator = Generator(engine, policy)
    sampling = SamplingParams(temperature=sc["temperature"], seed=11)
    for i, prompt in enumerate(prompts):
        generator.submit(i, prompt, sc["new_tokens"], sampling, None)
    torch.cuda.synchronize()
    started = time.perf_counter()
    finished = generator.run()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - started
    engine.cache.check()
    assert len(finished) == sc["requests"] and all(len(f.tokens) == sc["new_tokens"] for f in finished)
    assert not engine.cache.live_requests()
    stats, sched = generator.stats, generator.scheduler.stats
    return {"metric": f"generated tok/s, scenario {name}", "value": round(stats.emitted_tokens / elapsed, 2),
            "unit": "tok/s", "n_gpus": 1, "seconds": round(elapsed, 3), "dtype": "bf16" if dtype == "bfloat16" else "fp32",
            "data": "synthetic",
            "config": {"model": name, "layers": config.num_hidden_layers, "layers_of_configuration": full_layers,
                       "requests": sc["requests"], "prompt_tokens": sum(lengths), "new_tokens": sc["new_tokens"],
                       "prefill_chunk": sc["chunk"], "pages": pages, "pages_needed_for_all": needed,
                       "page_tokens": page_tokens,
                       "library_products": "measured choice" if any(r["kept"] for r in tuned) else "heuristic"},
            "steps": stats.steps, "prefill_tok_s": round(stats.prefill_rate, 1), "decode_tok_s": round(stats.decode_rate, 1),
            "preemptions": sched.preemptions, "max_step_rows": sched.max_step_rows, "max_live": sched.max_live}


def main(argv: Optional[List[str]] = None) -> int:
    parser = argparse.ArgumentParser(prog="bench.py")
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=CONTEXT)
    parser.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    parser.add_argument("--shape", default="8b", choices=["8b", "14b", "32b"],
                        help="layer sizes of which Qwen3 model (the headline figure is 8b)")
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 points")
    parser.add_argument("--no-generate", action="store_true",
                        help="skip the stated workload through the generation loop (points generate_b*)")
    parser.add_argument("--no-long", action="store_true",
                        help="skip the points of a second engine built for the model's whole context (context 32,768, "
                             "context 512 of 40,960, a prompt of 8,192 tokens)")
    parser.add_argument("--no-prefill", action="store_true")
    parser.add_argument("--no-kernels", action="store_true", help="skip the per-operation table of the decode step")
    parser.add_argument("--no-peaks", action="store_true", help="skip the measurement of this GPU's own peaks")
    parser.add_argument("--no-streamed-weights", action="store_true",
                        help="keep no second copy of the matrices in the decode kernels' order")
    parser.add_argument("--tuned-products", action="store_true",
                        help="let the prompt's products run with the vendor library's algorithms that are fastest when "
                             "timed now (Runtime(tune_products=True)); by default the library's heuristic chooses, as in "
                             "Runtime and `leone generate`")
    parser.add_argument("--peaks", action="store_true", help="only measure this GPU's own peaks and print them")
    parser.add_argument("--scenario", choices=sorted(SCENARIOS), help="run a serving scenario instead of the headline figure")
    args = parser.parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    if args.scenario:
        print(json.dumps(run_scenario(args.scenario, args.dtype, args.layers, args.tuned_products)), flush=True)
        return 0
    if args.peaks:
        print(json.dumps({"metric": "measured peaks", **measure_peaks()}), flush=True)
        return 0

    import torch
    from .architectures import config_from_dict
    from .engine.engine import Engine
    from .runtime import random_model

    raw = dict({"8b": QWEN3_8B, "14b": QWEN3_14B, "32b": QWEN3_32B}[args.shape])
    full_layers = raw["num_hidden_layers"]
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    config = config_from_dict(raw)
    size = 2 if args.dtype == "bfloat16" else 4
    dtype_name = "bf16" if args.dtype == "bfloat16" else "fp32"
    model = random_model(config, seed=0, dtype=args.dtype)
    page_tokens = 64
    points_batches = [] if args.no_points else [1, 64]
    largest = max([args.batch] + points_batches)
    pages = largest * (args.context // page_tokens + 1) + PREFILL_TOKENS // page_tokens
    # the cache takes requests of the context asked for and, for the prompt's figure, one of PREFILL_TOKENS
    engine = Engine(model, num_pages=pages, page_tokens=page_tokens, max_requests=largest + 1,
                    max_context=args.context if args.no_prefill else max(args.context, PREFILL_TOKENS),
                    streamed_weights=False if args.no_streamed_weights else None)

    peaks = None if args.no_peaks else measure_peaks()
    profile_steps = 0 if args.no_kernels else 4
    start = args.context - args.steps - args.warmup - 1 - profile_steps
    timed = time_decode(engine, args.batch, start, args.steps, args.warmup, profile_steps=profile_steps)
    elapsed, mean_context = timed[0], timed[1]
    ms_per_step = elapsed / args.steps * 1e3
    value = args.batch * args.steps / elapsed
    step_bytes = decode_bytes(model, args.batch, mean_context)
    achieved = step_bytes / (elapsed / args.steps) / 1e9
    record = {
        "metric": f"decode tok/s (Qwen3-{args.shape.upper()} shape)", "value": round(value, 2), "unit": "tok/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": dtype_name, "data": "synthetic",
        "config": {"model": f"Qwen3-{args.shape.upper()} shape, random weights", "layers": config.num_hidden_layers,
                   "layers_of_configuration": full_layers, "hidden": config.hidden_size,
                   "q_heads": config.num_attention_heads, "kv_heads": config.num_key_value_heads,
                   "head_dim": config.head_dim, "intermediate": config.intermediate_size, "vocab": config.vocab_size,
                   "global_batch": args.batch, "seq_len": args.context, "decode_start_context": start,
                   "prefill_tokens": PREFILL_TOKENS, "page_tokens": page_tokens, "rope_theta": config.rope_theta,
                   "tied_head": config.tie_word_embeddings, "parallelism": "single GPU",
                   "weight_copies": 2 if model.streamed_copy_bytes else 1,
                   "decode_loop": "a step is issued before the last step's tokens reach the host"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
    }
    weights = model.weight_accounting(rows=args.batch)
    record["bytes"] = {"weights_resident": weights["tensor_bytes"], "weights_a_step": sum(weights["decode"].values()),
                       "weights_second_copy": weights["streamed_copy_bytes"],
                       "cache_a_token": cache_bytes_per_token(model), "a_step": int(step_bytes)}
    if peaks is not None:
        record["peaks_measured"] = peaks
        record["roofline"]["frac_of_measured"] = round(achieved / peaks["hbm_read_gbs"], 4)
    if profile_steps:
        record["kernels"] = kernel_table(timed[2], model, args.batch, start + args.warmup + args.steps + 2)
    if not args.no_prefill:
        # on request the vendor library's products of the prompt run with the fastest of the library's algorithms,
        # found by timing them now on this model's matrices (Engine.tune_products)
        tuned = engine.tune_products(PREFILL_TOKENS) if args.tuned_products and args.dtype == "bfloat16" else []
        record["config"]["library_products"] = "measured choice" if any(r["kept"] for r in tuned) else "heuristic"
        seconds = time_prefill(engine, PREFILL_TOKENS)
        flops = prefill_flops(config, PREFILL_TOKENS)
        record["prefill"] = {"value": round(PREFILL_TOKENS / seconds, 1), "tokens": PREFILL_TOKENS,
                             "ms": round(seconds * 1e3, 3), "frac": round(flops / seconds / PEAK_FLOPS[dtype_name], 4)}
        if peaks is not None and dtype_name == "bf16":
            record["prefill"]["frac_of_measured"] = round(flops / seconds / (peaks["mfma_bf16_tflops"] * 1e12), 4)
    points = {}
    if not args.no_points:
        # the same steps one by one, as the reference's loop: step, choice, copy of the tokens, next step
        e, _ = time_decode(engine, args.batch, args.context - args.steps - args.warmup - 1, args.steps, args.warmup,
                           pipelined=False)
        points[f"decode_b{args.batch}_one_by_one"] = round(args.batch * args.steps / e, 2)
    for batch in points_batches:
        steps = max(8, args.steps // 2)
        warm = max(2, args.warmup // 2)
        e, _ = time_decode(engine, batch, args.context - steps - warm - 1, steps, warm)
        points[f"decode_b{batch}"] = round(batch * steps / e, 2)
    # The workload the configuration states: prompts of 2,048 tokens, 256 new tokens each.
    for batch in ([] if args.no_points else sorted({1, args.batch, 64})):
        if STATED_PROMPT + STATED_NEW + 1 > args.context:
            break
        e, _ = time_decode(engine, batch, STATED_PROMPT, STATED_NEW - 8, 8)
        points[f"decode_b{batch}_prompt{STATED_PROMPT}_new{STATED_NEW}"] = round(batch * (STATED_NEW - 8) / e, 2)
    # The same workload through the generation loop: scheduler, real prefill, page allocation, sampler.
    if not (args.no_points or args.no_generate) and STATED_PROMPT + STATED_NEW + 1 <= args.context:
        for batch in sorted({1, args.batch, 64}):
            run = time_generate(engine, batch, STATED_PROMPT, STATED_NEW)
            points[f"generate_b{batch}"] = round(run["tok_s"], 2)
        # and with a sampler that cuts: temperature 0.8, the 40 best, then 0.9 of their mass (chosen on the device)
        from .sampling.sampler import SamplingParams
        cut = SamplingParams(temperature=0.8, truncations=[("top_k", 40.0), ("top_p", 0.9)], seed=11)
        run = time_generate(engine, args.batch, STATED_PROMPT, STATED_NEW, sampling=cut)
        points[f"generate_b{args.batch}_top_k40_top_p0.9"] = round(run["tok_s"], 2)
    # A second engine, built for the model's whole context: decoding at context 32,768, decoding a short
    # context on an engine that could hold 40,960 positions (recordings are per context range), a long prompt.
    if not (args.no_points or args.no_long) and config.max_position_embeddings >= 32768 + 64:
        del engine
        torch.cuda.empty_cache()
        long_context, long_batch = 32768, 8
        engine = Engine(model, num_pages=long_batch * (long_context // page_tokens + 1), page_tokens=page_tokens,
                        max_requests=long_batch, streamed_weights=False if args.no_streamed_weights else None)
        assert engine.max_context == config.max_position_embeddings
        for batch in (1, long_batch):
            e, _ = time_decode(engine, batch, long_context - 40, 24, 8)
            points[f"decode_b{batch}_context{long_context}"] = round(batch * 24 / e, 2)
            e, _ = time_decode(engine, batch, 512 - 72, 64, 8)
            points[f"decode_b{batch}_context512_of_{engine.max_context}"] = round(batch * 64 / e, 2)
        if not args.no_prefill:
            seconds = time_prefill(engine, 8192, repeats=2)
            points["prefill_8192"] = round(8192 / seconds, 1)
    if points:
        record["points"] = points
    print(json.dumps(record), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
