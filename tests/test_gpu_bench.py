"""The measurement program's record: what a reader of its one line relies on."""
import json

import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def library_products_as_found():
    """The measurement programs choose the vendor library's algorithms by measurement for the process: what they
    chose goes back to the library's heuristic afterwards."""
    yield
    from leone_amd import ops
    ops.forget_tuned_products()


def test_the_record_of_a_short_run(capsys):
    """Two layers of the headline shape, a few steps: one line of JSON with the decode figure, the prompt's, the
    roofline's and the points', and a flat description of every size."""
    from leone_amd import benchmark
    assert benchmark.main(["--layers", "2", "--steps", "4", "--warmup", "1", "--batch", "8", "--context", "2560",
                           "--no-peaks"]) == 0
    lines = [line for line in capsys.readouterr().out.splitlines() if line.strip()]
    assert len(lines) == 1
    record = json.loads(lines[0])
    for key, kind in (("metric", str), ("value", float), ("unit", str), ("n_gpus", int), ("steps", int), ("warmup", int),
                      ("ms_per_step", float), ("higher_is_better", bool), ("scaling", str), ("dtype", str), ("data", str)):
        assert isinstance(record[key], kind), key
    assert record["n_gpus"] == 1 and record["steps"] == 4 and record["warmup"] == 1 and record["value"] > 0
    assert abs(record["value"] - 8 / record["ms_per_step"] * 1e3) / record["value"] < 1e-3      # decoded tokens a second
    config = record["config"]
    assert len(config) <= 20 and all(isinstance(v, (str, int, float, bool)) for v in config.values()), config
    assert config["layers"] == 2 and config["layers_of_configuration"] == 36 and config["global_batch"] == 8
    assert config["library_products"] in ("measured choice", "heuristic")
    prefill = record["prefill"]
    assert prefill["tokens"] == 2048 and prefill["ms"] > 0 and 0 < prefill["frac"] < 1
    assert abs(prefill["value"] - 2048 / prefill["ms"] * 1e3) / prefill["value"] < 1e-3
    roofline = record["roofline"]
    assert roofline["bound"] == "hbm" and roofline["unit"] == "GB/s" and roofline["peak"] == 8000.0
    assert abs(roofline["frac"] - roofline["achieved"] / roofline["peak"]) < 1e-3
    assert abs(roofline["achieved"] - record["bytes"]["a_step"] / record["ms_per_step"] / 1e6) / roofline["achieved"] < 1e-2
    assert {"decode_b1", "decode_b64"} <= set(record["points"]) and all(v > 0 for v in record["points"].values())
    # the stated workload as a bare step loop and through the generation loop, and the second engine's points
    for batch in (1, 8, 64):
        assert {f"decode_b{batch}_prompt2048_new256", f"generate_b{batch}"} <= set(record["points"])
    assert "generate_b8_top_k40_top_p0.9" in record["points"]
    assert {"decode_b1_context32768", "decode_b8_context32768", "decode_b1_context512_of_40960",
            "decode_b8_context512_of_40960", "prefill_8192"} <= set(record["points"])


@pytest.mark.parametrize("name", ["mixed14b", "pressure32b"])
def test_a_serving_scenario_with_one_layer(name):
    """The serving scenarios at their real widths and request mixes, one layer deep: every request finishes with
    all its tokens, no page is lost (the scenario checks both itself), steps stay within the budget, and the
    scenario with too few pages preempts."""
    from leone_amd import benchmark
    record = benchmark.run_scenario(name, layers=1)
    scenario = benchmark.SCENARIOS[name]
    assert record["value"] > 0 and record["config"]["layers"] == 1
    assert record["max_step_rows"] <= scenario["chunk"] and record["max_live"] <= scenario["live"]
    assert record["config"]["requests"] == scenario["requests"]
    assert (record["preemptions"] > 0) == (scenario["pool_fraction"] < 1.0)
    assert len(record["config"]) <= 20
