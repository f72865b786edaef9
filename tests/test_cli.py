"""Command-line pieces that need no GPU."""
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
    assert dry.dry_active and not dry.device_eligible and not params.dry_active


def test_bench_refuses_several_gpus(capsys):
    from leone_amd import benchmark
    assert benchmark.main(["--gpus", "2"]) == 2
    assert "one GPU" in capsys.readouterr().out


def test_bench_arithmetic():
    from leone_amd import benchmark
    from leone_amd.architectures import config_from_dict
    c = config_from_dict(benchmark.QWEN3_8B)
    assert benchmark.matmul_params(c) == 36 * (4096 * 6144 + 4096 * 4096 + 3 * 4096 * 12288)
    # weights 15.14 GB a step, cache 147,456 bytes a token of context
    assert abs(benchmark.decode_bytes(c, 1, 0, 2) / 1e9 - 15.14) < 0.01
    assert benchmark.decode_bytes(c, 8, 100, 2) - benchmark.decode_bytes(c, 8, 0, 2) == 8 * 100 * 147456
    assert abs(benchmark.prefill_flops(c, 2048) / 2.97e13 - 1) < 0.01
