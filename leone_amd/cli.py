"""Command line in the reference's manner: ``leone generate -m <model> -p <prompt> -n <tokens>``.

Subcommands and option names follow crates/leone-cli/src/main.rs:418-460 (generate, eval) and
crates/leone-cli/src/doctor.rs:303-346 (doctor).  Where the reference selects a backend or a
quantised cache (``--backend``, ``--kv``) this engine has ``--dtype bfloat16|float32``, which sets
weights, activations and cache alike.  A model without tokenizer.json takes ``--prompt-tokens``.
"""
from __future__ import annotations

import argparse
import json
import os
import signal
import struct
import sys
import time
from typing import List, Optional

# Decode steps that --profile-decode times (the reference's figure, crates/leone-cli/src/main.rs:2828-2830).
PROFILE_DECODE_STEPS = 64

_STAGE_FLAGS = {"--top-k": "top_k", "--top-p": "top_p", "--min-p": "min_p", "--top-a": "top_a", "--tfs": "tfs",
                "--typical": "typical", "--epsilon": "epsilon", "--eta": "eta", "--min-k": "min_k",
                "--top-n-sigma": "top_n_sigma"}


class _Stage(argparse.Action):
    """Truncation stages apply in the order their flags are given."""

    def __call__(self, parser, namespace, values, option_string=None):
        stages = list(getattr(namespace, "truncations", None) or [])
        stages.append((_STAGE_FLAGS[option_string], float(values)))
        namespace.truncations = stages


def _add_sampling(parser: argparse.ArgumentParser) -> None:
    parser.add_argument("--seed", type=int, default=0, help="Number the random draws are derived from (0 unless given)")
    parser.add_argument("--temp", "--temperature", dest="temp", type=float, default=None,
                        help="Sample at temperature t; left out, the best token is always taken")
    helps = {"--top-k": "Only the n likeliest tokens stay in the draw", "--top-p": "Likeliest tokens first, until their probabilities add up to p",
             "--min-p": "Drop what is less than p times as likely as the best token",
             "--top-a": "Drop what falls below a times the square of the best probability",
             "--tfs": "Cut the tail where the sorted probabilities flatten out (share z of the curvature kept)", "--typical": "Tokens whose surprise is nearest the entropy, up to mass p",
             "--epsilon": "Drop tokens whose probability is under e", "--eta": "Like --epsilon, with a bound that shrinks as the entropy grows (base e)",
             "--min-k": "Cut on the unscaled logits at their steepest drop; tau is the bound when none is found", "--top-n-sigma": "Unscaled logits no further than n standard deviations under the best"}
    for flag, text in helps.items():
        parser.add_argument(flag, action=_Stage, help=text)
    parser.add_argument("--repeat-penalty", type=float, default=1.0, help="Tokens already seen: a positive logit is divided by r, a negative one multiplied (1.0 does nothing)")
    parser.add_argument("--presence-penalty", type=float, default=0.0, help="Amount taken off the logit of every token already seen")
    parser.add_argument("--frequency-penalty", type=float, default=0.0, help="Amount taken off a logit for each time its token was seen")
    parser.add_argument("--penalty-window", type=int, default=64, help="How many of the latest tokens the three penalties look at (0: none)")
    parser.add_argument("--dry-multiplier", type=float, default=0.0, help="Strength of the penalty on continuing a repeated run of tokens (0.0: no such penalty)")
    parser.add_argument("--dry-base", type=float, default=1.75, help="Factor by which that penalty grows with every further matching token (1.75)")
    parser.add_argument("--dry-allowed-length", type=int, default=2, help="Matching tokens that go unpunished (2)")
    parser.add_argument("--dry-window", type=int, default=64, help="How far back repeated runs are looked for, in tokens (64)")


def _sampling_from(args):
    from .sampling.sampler import SamplingParams
    params = SamplingParams(args.temp, list(getattr(args, "truncations", None) or []), args.seed,
                            args.repeat_penalty, args.presence_penalty, args.frequency_penalty, args.penalty_window,
                            args.dry_multiplier, args.dry_base, args.dry_allowed_length, args.dry_window)
    if params.truncations and params.temperature is None:
        raise SystemExit("error: truncation flags need --temp; without it generation is greedy")
    params.validate()
    return params


def build_parser() -> argparse.ArgumentParser:
    from . import __version__
    parser = argparse.ArgumentParser(prog="leone", description="Qwen3 dense inference on MI355X")
    parser.add_argument("-V", "--version", action="version", version=f"leone {__version__}")
    parser.add_argument("--build-info", action="store_true",
                        help="Print where the two native libraries come from, as JSON")
    sub = parser.add_subparsers(dest="command")

    g = sub.add_parser("generate", help="Continue a prompt", usage="leone generate -m <model> -p <prompt> -n <tokens> [options]")
    g.add_argument("-m", "--model", required=True, help="Model folder (config.json, model.safetensors)")
    g.add_argument("-p", "--prompt", help="Prompt text (needs tokenizer.json in the model folder)")
    g.add_argument("--prompt-tokens", help="Prompt as comma-separated token ids")
    g.add_argument("-n", "--tokens", type=int, required=True, help="How many tokens to produce")
    g.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"], help="Weights, activations and cache")
    g.add_argument("--eager-decode", action="store_true", help="Launch every decode step kernel by kernel instead of replaying its recording")
    g.add_argument("--profile-decode", action="store_true",
                   help=f"Time the first {PROFILE_DECODE_STEPS} decode steps operation by operation")
    g.add_argument("--prefill-chunk", type=int, default=2048, help="Longest prompt portion per step")
    g.add_argument("--max-context", type=int, default=None, help="Context the cache is sized for")
    g.add_argument("--debug-tokens", help="File that receives the generated ids as a JSON list")
    g.add_argument("--debug-logits", help="File that receives, step by step, the five largest logits with their bits")
    g.add_argument("--ignore-eos", action="store_true", help="Do not stop at the end token")
    g.add_argument("--single-weight-copy", action="store_true",
                   help="Keep no second copy of the matrices in the decode kernels' order (half the weight memory, slower decoding)")
    g.add_argument("--tune-products", action="store_true",
                   help="Time the vendor library's algorithms for a full prompt portion first and use the fastest (a few seconds)")
    _add_sampling(g)

    d = sub.add_parser("doctor", help="Check the platform, the kernel library and a model folder")
    d.add_argument("-m", "--model", help="Model folder to check (metadata only)")
    d.add_argument("--probe", action="store_true", help="Also load the weights onto the GPU")
    d.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])

    e = sub.add_parser("eval", help="Feed given token ids and write the logits of every position")
    e.add_argument("-m", "--model", required=True)
    e.add_argument("--tokens", required=True, help="Input file: token ids, 32-bit unsigned, little-endian")
    e.add_argument("--logits", required=True, help="Output file: one row of 32-bit float logits per position, little-endian")
    e.add_argument("--metadata", help="Also write a JSON record of model, type, schedule and file digests")
    e.add_argument("--window", type=int, default=512, help="Tokens per window; a window starts on the last token of the one before, with an empty cache (512)")
    e.add_argument("--position-limit", type=int, default=None, help="Stop after n positions")
    e.add_argument("--prefill-chunk", type=int, default=None, help="Cut every window into portions of n tokens")
    e.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])

    r = sub.add_parser("random-model", help="Write a model folder with seeded random weights")
    r.add_argument("--config", required=True, help="config.json to build from")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--out", required=True)
    r.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])

    q = sub.add_parser("quality", help="Compare two logit files: KL divergence and top-1 agreement")
    q.add_argument("--oracle", required=True, help="Reference logits (row-major little-endian f32)")
    q.add_argument("--subject", required=True, help="Logits under test, same shape")
    q.add_argument("--vocab", type=int, help="Vocabulary size (or give -m)")
    q.add_argument("-m", "--model", help="Model folder to take the vocabulary size from")

    b = sub.add_parser("bench", help="Time decoding and prompt processing")
    b.add_argument("rest", nargs=argparse.REMAINDER)
    return parser


def cmd_generate(args) -> int:
    from .api import Runtime
    from .engine.scheduler import SchedulerPolicy

    sampling = _sampling_from(args)
    if args.tokens <= 0:
        raise SystemExit("error: -n must be positive")
    if (args.prompt is None) == (args.prompt_tokens is None):
        raise SystemExit("error: give exactly one of -p/--prompt and --prompt-tokens")
    runtime = Runtime.load(args.model, args.dtype, max_requests=1, max_context=args.max_context,
                           graphs=not args.eager_decode,
                           streamed_weights=False if args.single_weight_copy else None,
                           tune_products=args.tune_products,
                           policy=SchedulerPolicy(max_live_requests=1, prefill_chunk_tokens=args.prefill_chunk,
                                                  max_step_tokens=max(args.prefill_chunk, 1)))
    if args.prompt is not None:
        prompt = runtime.encode(args.prompt)
    else:
        prompt = [int(t) for t in args.prompt_tokens.replace(",", " ").split()]
    top_five: List[str] = []
    observe = None
    if args.debug_logits:
        def observe(request, position, row):
            values, ids = row.topk(min(5, row.numel()))
            top_five.append(" ".join(f"{int(i)}:{float(v):.6f}:0x{struct.unpack('<I', struct.pack('<f', float(v)))[0]:08x}"
                                     for v, i in zip(values.tolist(), ids.tolist())))

    def on_token(request, token):
        if runtime.tokenizer is not None:
            sys.stdout.write(runtime.decode([token]))
        else:
            sys.stdout.write(f"{token} ")
        sys.stdout.flush()

    eos = None if args.ignore_eos else "config"
    # Ctrl-C asks the run to stop after the step in hand; what was generated is still reported.
    interrupted = []
    earlier = signal.signal(signal.SIGINT, lambda *_: interrupted.append(True))
    try:
        results = runtime.generate_tokens([prompt], args.tokens, sampling, eos_token_id=eos, on_token=on_token,
                                          logit_observer=observe,
                                          profile_decode_steps=PROFILE_DECODE_STEPS if args.profile_decode else 0,
                                          cancelled=lambda: bool(interrupted))
    finally:
        signal.signal(signal.SIGINT, earlier)
    stats = runtime.last_stats
    sys.stdout.write("\n")
    if args.debug_tokens:
        with open(args.debug_tokens, "w") as handle:
            json.dump(results[0].tokens, handle)
    if args.debug_logits:
        with open(args.debug_logits, "w") as handle:
            handle.write("\n".join(top_five) + "\n")
    print(file=sys.stderr)
    print(f"decode: {stats.decode_rate:.2f} tok/s", file=sys.stderr)
    print(f"prefill: {stats.prefill_rate:.2f} tok/s", file=sys.stderr)
    print(f"tokens emitted: {stats.emitted_tokens}", file=sys.stderr)
    print(f"finish: {results[0].finish_reason}", file=sys.stderr)
    if args.tune_products:
        tuned = runtime.tuned_products
        print(f"library products of a portion of {tuned[0]['rows'] if tuned else 0} tokens: {len(tuned)} timed, "
              f"{sum(1 for r in tuned if r['kept'])} run with another algorithm than the heuristic's", file=sys.stderr)
    if runtime.last_decode_profile is not None:
        print("\n".join(runtime.last_decode_profile.lines()), file=sys.stderr)
    return 0


def cmd_doctor(args) -> int:
    import torch

    print(f"python {sys.version.split()[0]}, torch {torch.__version__}, hip {torch.version.hip}")
    ok = True
    if torch.cuda.is_available():
        props = torch.cuda.get_device_properties(0)
        print(f"gpu: {props.name}, {props.total_memory / 2**30:.1f} GiB, {props.multi_processor_count} CUs")
    else:
        print("gpu: none visible (this engine has no CPU path)")
        ok = False
    try:
        from .csrc import build
        path = build.library_path() or build.build(verbose=True)
        print(f"kernel library: {path}")
        if torch.cuda.is_available():
            from .ops.library import library
            found = library().leone_library_product_available()
            print("vendor library for the products of prompt portions: "
                  + ("hipBLASLt not found (torch's own calls of it remain; --tune-products has nothing to choose from)" if not found
                     else "hipBLASLt, algorithms by its heuristic's list" + (" or all of them" if found == 2 else "")))
    except Exception as error:  # noqa: BLE001 - doctor reports, it does not raise
        print(f"kernel library: FAILED: {error}")
        ok = False
    try:
        from .csrc import build
        path = build.host_library_path() or build.build_host(verbose=True)
        print(f"host library: {path}")
    except Exception as error:  # noqa: BLE001
        print(f"host library: FAILED: {error}")
        ok = False
    if args.model:
        from .architectures import config_from_dir, model_spec_for
        from .parts.model import DecoderModel
        from .weights import loader
        from .weights.safetensors_io import ModelFiles
        config = config_from_dir(args.model)
        print(f"architecture: {config.architecture}")
        print(f"context limit: {config.max_position_embeddings}")
        model = DecoderModel(model_spec_for(config), torch.float32, "cpu")
        files = ModelFiles(args.model)
        total = 0
        by_type = {}
        for entry in files.entries.values():
            total += entry.nbytes
            by_type[entry.dtype_name] = by_type.get(entry.dtype_name, 0) + entry.nbytes
        print(f"tensors: {len(files.entries)}, {total / 2**20:.1f} MiB " +
              ", ".join(f"{k} {v / 2**20:.1f} MiB" for k, v in sorted(by_type.items())))
        found = {n: (e.shape, e.dtype) for n, e in files.entries.items()}
        loader.check(model.tensor_specs(), found, args.model, model.spec.ignore_tensors)
        print("tensor names and shapes: ok")
        # bytes by class as the file stores them: in memory, and as one decode step reads them
        accounting = model.weight_accounting(lambda spec: files.entries[spec.name].nbytes)
        for family in sorted(accounting["resident"]):
            print(f"  {family:<13} resident {accounting['resident'][family] / 2**20:10.1f} MiB   "
                  f"a decode step {accounting['decode'][family] / 2**20:10.1f} MiB")
        print(f"weights a decode step reads: {sum(accounting['decode'].values()) / 2**20:.1f} MiB of "
              f"{accounting['tensor_bytes'] / 2**20:.1f} MiB")
        size = 2 if args.dtype == "bfloat16" else 4
        per_token = sum(need.bytes_per_token(size) for need in model.cache_needs().values() if getattr(need, "paged", False))
        print(f"cache bytes per token ({args.dtype}): {per_token}")
        # which attention kernels the layers' shapes get (pages of 64 tokens, the default)
        kinds = {}
        for layer in model.layers:
            mixer = getattr(layer, "mixer", None)
            if hasattr(mixer, "attention_kernels"):
                chosen = mixer.attention_kernels(torch.bfloat16 if args.dtype == "bfloat16" else torch.float32, 64)
                key = (mixer.q_heads, mixer.kv_heads, mixer.head_dim, chosen["decode"], chosen["prompt"])
                kinds[key] = kinds.get(key, 0) + 1
        names = {"projected": "split-KV matrix-core kernel that makes the heads itself", "split_kv": "split-KV matrix-core kernel",
                 "flash": "matrix-core prompt kernel", "rows": "row kernel in float arithmetic"}
        for (q_heads, kv_heads, head_dim, decode, prompt), count in kinds.items():
            print(f"attention, {count} layer(s) of {q_heads}/{kv_heads} heads of {head_dim}: decoded tokens on the "
                  f"{names[decode]}, prompt portions on the {names[prompt]}")
        # the second copy of the matrices that decode steps read (kept for bfloat16 when there is ample room)
        second = sum(v for family, v in accounting["decode"].items() if family not in ("embed", "norm"))
        second = second if args.dtype == "bfloat16" and model.spec.hidden_size % 64 == 0 else 0
        print(f"second copy of the matrices in the decode kernels' order: {second / 2**20:.1f} MiB "
              f"(kept if that is at most {model.STREAMED_SHARE_OF_DEVICE:.0%} of the device's memory)")
        if torch.cuda.is_available():
            free, device_total = torch.cuda.mem_get_info(0)
            room = free - total * (2 if args.dtype == "float32" else 1)
            if second <= model.STREAMED_SHARE_OF_DEVICE * device_total and second <= model.STREAMED_SHARE_OF_FREE * room:
                room -= second
            print(f"tokens of context that fit beside the weights: {max(0, int(room * 0.9) // max(1, per_token))}")
        if args.probe:
            from .runtime import load_model
            started = time.time()
            load_model(args.model, args.dtype)
            print(f"probe: weights loaded in {time.time() - started:.1f}s")
    return 0 if ok else 1


def cmd_eval(args) -> int:
    """Windows of W tokens, stride W-1, a fresh cache per window; the row after token i scores token i+1
    (crates/leone/src/runtime.rs:1673-1996, crates/leone-cli/src/eval.rs:526-558)."""
    import hashlib
    import numpy as np
    from .engine.engine import Engine, StepEntry
    from .runtime import load_model

    tokens = np.fromfile(args.tokens, dtype="<u4").astype(np.int64)
    if args.position_limit is not None:
        tokens = tokens[:args.position_limit]
    if tokens.size < 2:
        raise SystemExit("error: need at least two tokens")
    if args.window < 2:
        raise SystemExit("error: --window must be at least 2")
    model = load_model(args.model, args.dtype)
    window = min(args.window, model.spec.max_positions)
    engine = Engine(model, max_tokens=window + 64, page_tokens=64, max_requests=1, max_context=window)
    rows = 0
    digest = hashlib.sha256()
    with open(args.logits, "wb") as out:
        start = 0
        while start < tokens.size - 1:
            piece = tokens[start:start + window].tolist()
            feed = piece[:-1]   # the last token of a window is only a target
            chunk = args.prefill_chunk or 1
            at = 0
            while at < len(feed):
                part = feed[at:at + chunk]
                logits = engine.step([StepEntry("w", part, list(range(len(part))))]).logits
                data = logits.cpu().numpy().astype("<f4").tobytes()
                out.write(data)
                digest.update(data)
                rows += len(part)
                at += len(part)
            engine.release("w")
            start += window - 1
    if args.metadata:
        with open(args.metadata, "w") as handle:
            json.dump({"schema": "leone-amd.eval.v1", "model": os.path.abspath(args.model), "dtype": args.dtype,
                       "window": window, "prefill_chunk": args.prefill_chunk, "tokens": int(tokens.size),
                       "rows": rows, "vocab": model.spec.vocab_size,
                       "row_label": "row i of a window holds the logits after feeding its token i",
                       "logits_sha256": digest.hexdigest()}, handle, indent=2)
    print(f"wrote {rows} rows of {model.spec.vocab_size} logits", file=sys.stderr)
    return 0


def quality_stats(oracle, subject):
    """KL(oracle || subject) per row in nats (mean, median, 99th percentile, maximum) and how often the
    two agree on the highest logit: the reference's quality figures (crates/leone-cli/src/quality.rs:33-95)."""
    import numpy as np
    oracle = np.asarray(oracle, dtype=np.float64)
    subject = np.asarray(subject, dtype=np.float64)
    if oracle.shape != subject.shape or oracle.ndim != 2:
        raise ValueError(f"logit arrays differ in shape: {oracle.shape} and {subject.shape}")

    def log_softmax(x):
        x = x - x.max(axis=1, keepdims=True)
        return x - np.log(np.exp(x).sum(axis=1, keepdims=True))
    lo, ls = log_softmax(oracle), log_softmax(subject)
    kld = (np.exp(lo) * (lo - ls)).sum(axis=1)
    return {"samples": int(oracle.shape[0]), "kld_mean": float(kld.mean()), "kld_p50": float(np.percentile(kld, 50)),
            "kld_p99": float(np.percentile(kld, 99)), "kld_max": float(kld.max()),
            "top1_agreement": float((oracle.argmax(axis=1) == subject.argmax(axis=1)).mean()),
            "max_abs": float(np.abs(oracle - subject).max())}


def cmd_quality(args) -> int:
    import numpy as np
    vocab = args.vocab
    if vocab is None:
        if not args.model:
            raise SystemExit("error: give --vocab or -m")
        from .architectures import config_from_dir
        vocab = config_from_dir(args.model).vocab_size
    oracle = np.fromfile(args.oracle, dtype="<f4")
    subject = np.fromfile(args.subject, dtype="<f4")
    if oracle.size != subject.size or oracle.size % vocab:
        raise SystemExit(f"error: {oracle.size} and {subject.size} values do not make equal rows of {vocab}")
    stats = quality_stats(oracle.reshape(-1, vocab), subject.reshape(-1, vocab))
    print(f"samples: {stats['samples']}")
    print(f"KLD mean: {stats['kld_mean']:.9f} nats")
    print(f"KLD p50:  {stats['kld_p50']:.9f} nats")
    print(f"KLD p99:  {stats['kld_p99']:.9f} nats")
    print(f"KLD max:  {stats['kld_max']:.9f} nats")
    print(f"top1 agreement: {stats['top1_agreement']:.9f}")
    print(f"max abs difference: {stats['max_abs']:.6f}")
    return 0


def cmd_random_model(args) -> int:
    import torch
    from .architectures import config_from_dict
    from .weights.random_init import write_model_dir
    with open(args.config) as handle:
        config = config_from_dict(json.load(handle))
    write_model_dir(args.out, config, args.seed, torch.bfloat16 if args.dtype == "bfloat16" else torch.float32)
    print(args.out)
    return 0


def main(argv: Optional[List[str]] = None) -> int:
    parser = build_parser()
    args = parser.parse_args(argv)
    if args.build_info:
        from .csrc import build
        print(json.dumps(build.build_info()))
        return 0
    if args.command is None:
        parser.print_help()
        return 0
    if args.command == "generate":
        return cmd_generate(args)
    if args.command == "doctor":
        return cmd_doctor(args)
    if args.command == "eval":
        return cmd_eval(args)
    if args.command == "quality":
        return cmd_quality(args)
    if args.command == "random-model":
        return cmd_random_model(args)
    if args.command == "bench":
        from .benchmark import main as bench_main
        return bench_main(args.rest)
    parser.error(f"unknown command {args.command}")
    return 2


if __name__ == "__main__":
    sys.exit(main())
