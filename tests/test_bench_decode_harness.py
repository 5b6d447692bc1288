"""Host logic of the decode benchmark harness (list parsing, aggregation, summary table, power parsing): the parts
that mirror src/nanoquant/kernel/test_decode.py:52-75, :720-800 and :880-1046, and a tiny sweep on the GPU."""
import csv

import pytest

from nanoquant_amd import bench_decode as bd


def test_list_parsing():
    assert bd.parse_int_list("1,4,16", "batch_size") == [1, 4, 16]
    assert bd.parse_int_list("128 512", "prompt_tokens") == [128, 512]
    assert bd.parse_int_list(8, "batch_size") == [8]
    assert bd.parse_int_list([1, 2], "x") == [1, 2]
    with pytest.raises(ValueError):
        bd.parse_int_list("", "batch_size")
    with pytest.raises(ValueError):
        bd.parse_int_list("-1", "batch_size")


def test_rank_rule():
    assert bd.nominal_rank(4096, 4096, 1.0) == 2048
    assert bd.nominal_rank(11008, 4096, 1.0) == 3008           # 2985 rounded up to whole words
    assert bd.nominal_rank(64, 64, 0.1) == 32


def _row(it, t, tokens, bs=2, energy="", peak=100):
    return {"iter": it, "model_shape": "tiny", "layers": 2, "batch_size": bs, "prompt_tokens": 16, "max_new_tokens": 5,
            "decode_tokens_total": tokens, "decode_time_s": f"{t:.6f}", "decode_tps_total": f"{tokens / t:.6f}",
            "decode_tps_per_seq": f"{tokens / t / bs:.6f}", "prefill_time_s": "0.5", "decode_energy_j": energy,
            "decode_energy_per_token_j": "", "gpu_mem_peak_alloc_bytes": peak, "gpu_mem_peak_reserved_bytes": peak * 2,
            "dtype": "float16"}


def test_aggregate_is_total_tokens_over_total_time_and_peak_is_max():
    rows = [_row(1, 1.0, 8, peak=100), _row(2, 3.0, 8, peak=300)]
    agg = bd.aggregate_config_rows(rows)
    assert agg["iter"] == "AGGREGATE"
    assert float(agg["decode_tps_total"]) == pytest.approx(16 / 4.0)        # not the mean of 8 and 2.67
    assert float(agg["decode_tps_per_seq"]) == pytest.approx(2.0)
    assert agg["gpu_mem_peak_alloc_bytes"] == 300 and agg["gpu_mem_peak_reserved_bytes"] == 600
    assert agg["dtype"] == "float16" and agg["batch_size"] == 2
    assert agg["decode_energy_per_token_j"] == ""                            # no energy samples: blank, as the reference
    rows = [_row(1, 1.0, 8, energy="40"), _row(2, 1.0, 8, energy="56")]
    agg = bd.aggregate_config_rows(rows)
    assert float(agg["decode_energy_per_token_j"]) == pytest.approx(96 / 16)
    assert bd.aggregate_config_rows([]) == {}


def test_summary_table_and_power_parse():
    table = bd.format_summary_table([{"batch_size": 1, "prompt_tokens": 128, "max_new_tokens": 64, "decode_tps_total": "1000.5"}])
    lines = table.splitlines()
    assert len(lines) == 3 and "decode_tps_total" in lines[0] and "1000.5" in lines[2]
    assert bd.PowerSampler.parse('{"card0": {"Average Graphics Package Power (W)": "312.0"}}') == 312.0
    assert bd.PowerSampler.parse('{"card0": {"Current Socket Graphics Package Power (W)": "95.5"}}') == 95.5
    assert bd.PowerSampler.parse("not json") is None


def test_parser_defaults_follow_the_reference_names():
    args = bd.build_parser().parse_args([])
    assert args.batch_size == "1" and args.max_new_tokens == "128" and args.output_csv is None
    assert args.quant_kernel_type == "runlist" and args.dtype == "float16"


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["runlist", "runlist-per-layer", "gemv", "gemv-group", "gemv-group-one-launch"])
def test_tiny_sweep_writes_rows_and_aggregates(dev, tmp_path, kind):
    out = tmp_path / "sweep.csv"
    rc = bd.main(["--model_shape", "tiny", "--batch_size", "1,2", "--prompt_tokens", "32", "--max_new_tokens", "5",
                  "--warmup", "1", "--iters", "2", "--quant_kernel_type", kind, "--output_csv", str(out)])
    assert rc == 0
    rows = list(csv.DictReader(open(out)))
    assert len(rows) == 2 * (2 + 1)                                          # two batches x (2 iterations + AGGREGATE)
    assert [r["iter"] for r in rows[:3]] == ["1", "2", "AGGREGATE"]
    for r in rows:
        assert float(r["decode_tps_total"]) > 0 and r["quant_kernel_type"] == kind
        assert int(r["decode_tokens_total"]) in (4, 8, 16)
    assert float(rows[2]["prefill_time_s"]) > 0


def test_prefill_harness_rank_and_gpu_requirement():
    import torch
    from nanoquant_amd import bench_prefill as bp
    assert bp.prefill_rank(4096, 4096, 1.0) == 2048
    assert bp.prefill_rank(11008, 4096, 1.0) == 2985
    assert bp.prefill_rank(64, 64, 0.1) == 32
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="needs a GPU"):
            bp.run(["--model_shape", "tiny", "--tokens", "32"])
