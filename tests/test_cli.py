"""Command-line pieces that need no GPU."""
import json

import numpy as np
import pytest

from leone_amd import cli


def test_quality_statistics(tmp_path):
    rng = np.random.default_rng(0)
    oracle = rng.standard_normal((50, 40)).astype(np.float32)
    same = cli.quality_stats(oracle, oracle)
    assert same["kld_max"] == 0.0 and same["top1_agreement"] == 1.0 and same["samples"] == 50
    # a uniform row against a peaked one: KL(uniform || p) = -log(n) - mean(log p)
    uniform, peaked = np.zeros((1, 4)), np.array([[3.0, 0.0, 0.0, 0.0]])
    log_p = peaked - np.log(np.exp(peaked).sum())
    assert abs(cli.quality_stats(uniform, peaked)["kld_mean"] - (-np.log(4.0) - log_p.mean())) < 1e-12
    noisy = oracle + 0.01 * rng.standard_normal(oracle.shape).astype(np.float32)
    stats = cli.quality_stats(oracle, noisy)
    assert 0 < stats["kld_mean"] < 1e-3 and stats["kld_p50"] <= stats["kld_p99"] <= stats["kld_max"]
    a, b = tmp_path / "a.bin", tmp_path / "b.bin"
    oracle.astype("<f4").tofile(a); noisy.astype("<f4").tofile(b)
    assert cli.main(["quality", "--oracle", str(a), "--subject", str(b), "--vocab", "40"]) == 0
    with pytest.raises(SystemExit):
        cli.main(["quality", "--oracle", str(a), "--subject", str(b), "--vocab", "7"])


def test_truncation_flags_keep_their_order():
    args = cli.build_parser().parse_args(["generate", "-m", "x", "--prompt-tokens", "1", "-n", "2", "--temp", "0.7",
                                          "--top-p", "0.9", "--top-k", "40", "--min-p", "0.05", "--seed", "3"])
    assert args.truncations == [("top_p", 0.9), ("top_k", 40.0), ("min_p", 0.05)]
    params = cli._sampling_from(args)
    assert params.temperature == 0.7 and params.seed == 3 and params.truncations[0][0] == "top_p"
    greedy = cli.build_parser().parse_args(["generate", "-m", "x", "--prompt-tokens", "1", "-n", "2", "--top-k", "5"])
    with pytest.raises(SystemExit):
        cli._sampling_from(greedy)            # a truncation without a temperature
    dry = cli._sampling_from(cli.build_parser().parse_args(
        ["generate", "-m", "x", "--prompt-tokens", "1", "-n", "2", "--dry-multiplier", "0.8", "--dry-base", "2",
         "--dry-allowed-length", "3", "--dry-window", "16"]))
    assert (dry.dry_multiplier, dry.dry_base, dry.dry_allowed_length, dry.dry_window) == (0.8, 2.0, 3, 16)
    assert dry.dry_active and dry.penalties_active and not params.dry_active
    from leone_amd.engine.generate import device_kind
    from leone_amd.sampling.sampler import SamplingParams
    assert device_kind(dry) is None and device_kind(SamplingParams()) == "greedy"
    assert device_kind(params) is None                                        # top-p comes first: the whole row is needed
    assert device_kind(SamplingParams(temperature=0.7)) == "temperature"
    assert device_kind(SamplingParams(temperature=0.7, truncations=[("top_k", 40.0), ("top_p", 0.9)])) == "truncated"
    assert device_kind(SamplingParams(temperature=0.7, truncations=[("top_k", 300.0)])) is None
    assert device_kind(SamplingParams(temperature=0.7, truncations=[("top_k", 40.0), ("tfs", 0.9)])) is None
    assert device_kind(SamplingParams(temperature=0.7, truncations=[("top_k", 40.0)], mirostat=(3.0, 0.1))) is None


def test_bench_refuses_several_gpus(capsys):
    from leone_amd import benchmark
    assert benchmark.main(["--gpus", "2"]) == 2
    assert "one GPU" in capsys.readouterr().out


def test_bench_arithmetic():
    from leone_amd import benchmark
    from leone_amd.architectures import config_from_dict
    c = config_from_dict(benchmark.QWEN3_8B)
    assert benchmark.matmul_params(c) == 36 * (4096 * 6144 + 4096 * 4096 + 3 * 4096 * 12288)
    # weights 15.14 GB a step, cache 147,456 bytes a token of context: from the model's own accounting
    import torch
    from leone_amd.architectures import model_spec_for
    from leone_amd.parts.model import DecoderModel
    model = DecoderModel(model_spec_for(c), torch.bfloat16, "cpu")
    assert abs(benchmark.decode_bytes(model, 1, 0) / 1e9 - 15.14) < 0.01
    assert benchmark.decode_bytes(model, 8, 100) - benchmark.decode_bytes(model, 8, 0) == 8 * 100 * 147456
    assert benchmark.cache_bytes_per_token(model) == 147456
    accounting = model.weight_accounting(rows=8)
    table = 151936 * 4096 * 2
    assert accounting["resident"]["embed"] == table and accounting["resident"]["head"] == table
    assert accounting["decode"]["embed"] == 8 * 4096 * 2 and accounting["decode"]["head"] == table
    assert accounting["resident"]["feed_forward"] == 36 * 3 * 4096 * 12288 * 2
    assert accounting["resident"]["mixer"] == 36 * (4096 * 6144 + 4096 * 4096 + 2 * 128) * 2
    assert accounting["resident"]["norm"] == (36 * 2 + 1) * 4096 * 2
    assert model.weight_bytes() == sum(accounting["resident"].values())
    assert model.decode_step_weight_bytes(8) == model.weight_bytes() - table + 8 * 4096 * 2
    tied = DecoderModel(model_spec_for(config_from_dict(dict(benchmark.QWEN3_8B, tie_word_embeddings=True))),
                        torch.bfloat16, "cpu")
    assert tied.weight_accounting()["resident"]["head"] == 0 and tied.weight_accounting()["decode"]["head"] == table
    assert abs(benchmark.prefill_flops(c, 2048) / 2.97e13 - 1) < 0.01


def test_decode_profile_report():
    """The table of `generate --profile-decode`: totals, shares, the host gap, and weight GB/s by shape."""
    from leone_amd.ops.profile import ProductTiming, StepProfile
    profile = StepProfile(steps=4, tokens=4, wall_seconds=0.010, launches=40,
                          seconds_by_operation={"attention": 0.002, "gemv fused": 0.006, "zeta": 0.001},
                          products={("gemv fused", 1000, 500, 2): ProductTiming(calls=8, seconds=0.004)})
    assert abs(profile.gpu_seconds - 0.009) < 1e-12 and abs(profile.host_gap_seconds - 0.001) < 1e-12
    assert profile.operations() == ["gemv fused", "attention", "zeta"]          # known ones in their order, then the rest
    lines = profile.lines()
    assert "decode profile: 4 evaluations" in lines[1]
    fused = next(line for line in lines if line.strip().startswith("gemv fused") and "%" in line).split()
    assert fused[-3:] == ["6.000", "1500.000", "66.67%"]
    gap = next(line for line in lines if "host gap" in line).split()
    assert gap[-2:] == ["1.000", "250.000"]
    traffic = lines[-1].split()
    assert traffic[-5:] == ["1000", "500", "8", "4.000", "2.0"]                 # 8 calls x 1 MB in 4 ms


def test_key_ranges_of_the_prompt_kernel_are_chosen_by_rows_and_keys():
    from leone_amd import ops
    heads = 32
    assert ops.choose_prefill_splits(16, heads, 1024) == 1                       # 2,048 rows fill the chip by themselves
    assert ops.choose_prefill_splits(4, heads, 256) == 1                         # a prompt's first portion: few keys a row
    assert ops.choose_prefill_splits(4, heads, 30720 + 256) == 4                 # 512 rows far into a long prompt
    assert ops.choose_prefill_splits(1, heads, 8192) == 16
    assert ops.choose_prefill_splits(1, 1, 10**6) == ops.PREFILL_MAX_SPLITS
    assert ops.choose_prefill_splits(1, heads, 100000, window=128) == 1          # a window bounds the keys a row sees
    for groups in (1, 2, 3, 7, 16, 40):
        for keys in (1, 63, 64, 1000, 5000, 200000):
            splits = ops.choose_prefill_splits(groups, heads, keys)
            assert 1 <= splits <= ops.PREFILL_MAX_SPLITS
            assert splits == 1 or -(-keys // 64) // splits >= ops.PREFILL_SPLIT_MIN_STAGES
    assert ops.choose_prefill_splits(6, heads, 31000) == 5                       # 768 rows: 960 workgroups, two rounds of 512
    assert ops.choose_prefill_splits(8, heads, 512) == 1                         # 1,024 rows from position 0: the merge costs more
    assert ops.choose_prefill_splits(24, heads, 1536) == 1                       # and 3,072
    assert ops.choose_prefill_splits(12, heads, 31000) == 4


def test_version_and_build_info(capsys):
    from leone_amd import __version__, cli
    from leone_amd.csrc import build
    with pytest.raises(SystemExit) as stop:
        cli.main(["--version"])
    assert stop.value.code == 0 and capsys.readouterr().out.strip() == f"leone {__version__}"
    assert cli.main(["--build-info"]) == 0
    info = json.loads(capsys.readouterr().out)
    assert info["schema_version"] == "leone_amd.build-info.v1" and info["target"] == "gfx950"
    assert info["kernels"]["sources"] == build.sources() and "attention_decode.hip" in info["kernels"]["sources"]
    assert info["kernels"]["source_digest"] == build.source_digest()
    assert info["host"]["source_digest"] == build.host_digest() and "scheduler.cpp" in info["host"]["sources"]
    assert "-packed-fp32-ops" in info["kernels"]["flags"]
    # a change of a flag is a change of the digest: a library built otherwise does not pass for this one
    flags = list(build.FLAGS)
    try:
        build.FLAGS.append("-DSOMETHING")
        assert build.source_digest() != info["kernels"]["source_digest"]
    finally:
        build.FLAGS[:] = flags


def test_cache_bytes_per_token_ask_every_kind_of_cache():
    """The default size of the page pool and the roofline's cache bytes come from what each paged need says of
    itself, so a mixer with another kind of cache than keys and values is not counted as caching nothing."""
    from dataclasses import dataclass

    import torch

    from leone_amd.api import cache_bytes_per_token
    from leone_amd.parts.base import KvNeed, StateNeed

    @dataclass(frozen=True)
    class VectorNeed:                      # one vector of `width` elements a token; no kv_heads, no head_dim
        width: int
        paged = True

        def group_key(self):
            return self

        def bytes_per_token(self, element_size):
            return self.width * element_size

    class Model:
        dtype = torch.bfloat16

        def __init__(self, needs):
            self.needs = needs

        def cache_needs(self):
            return self.needs

    assert cache_bytes_per_token(Model({0: VectorNeed(24)})) == 48
    assert cache_bytes_per_token(Model({0: VectorNeed(24), 1: KvNeed(2, 16), 2: StateNeed((5,))})) == 48 + 2 * 2 * 16 * 2
    from leone_amd import benchmark
    assert benchmark.cache_bytes_per_token(Model({0: VectorNeed(10), 3: KvNeed(8, 128)})) == 20 + 2 * 8 * 128 * 2
