"""The final line of bench.py stays small and strict, whatever the rows are."""
import json

import bench


def _head():
    return {"metric": "achieved HBM GB/s, KV write (Llama-3-8B decode step)", "value": 5641.1, "unit": "GB/s",
            "n_gpus": 1, "steps": 320, "warmup": 32, "ms_per_step": 0.011897, "wall_ms_per_step": 0.012101,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u16", "data": "synthetic",
            "config": {"workload": "config 2: Llama-3-8B decode-step KV write, 256 seqs x 1 token, 32 layers, "
                                   "8 KV heads x 128, block_size 16, pool 65536 blocks (128 GiB)",
                       "entry": "kvc_reshape_and_cache_layers", "launch": "one eager launch per step",
                       "rotation": 16, "hw_queues": "runtime default", "cfg5_blocks": 8192},
            "roofline": {"bound": "hbm", "achieved": 5641.1, "peak": 8000.0, "unit": "GB/s", "frac": 0.7051,
                         "traffic": 67221046, "kernel": "write_planes_kernel<4 per lane>, 1024 wgs x 512 lanes",
                         "bytes_per_launch": 67110912, "us_per_launch": 11.897,
                         "plain_kernel_same_bytes": {"us": 13.51, "gbps": 4969}},
            "target": {"frac": 0.75, "met": False},
            "cpu_baseline": {"value": 40.92, "unit": "GB/s", "cores": 16, "kind": "port", "us_per_step": 1640.2,
                             "sample": "6097 decode-step writes (T=256, 32 layers) via oracle/torch_cpu.py, pool 2048 "
                                       "blocks/layer, 10.0 s",
                             "others_gbps": {"cfg3": 98.62, "cfg4": 8.92, "cfg5_out": 8.48, "cfg5_in": 32.07}},
            "details": "bench_out/bench_details.json"}


def _row(i):
    return {"id": f"cfg{2 + i % 4}", "entry": "kvc_append_paged_kv_cache_layers", "form": "per layer, plan, eager wall",
            "us": 12345.67, "gbps": 6463, "frac": 0.808, "traffic_ratio": 1.0016}


def test_a_full_default_run_fits_with_room_to_spare():
    text = bench.build_line(_head(), [_row(i) for i in range(17)])
    assert len(text.encode()) < 3900          # every row at its longest; a real run is ~3.2 KB
    line = json.loads(text)
    assert len(line["configs"]) == 17 and "configs_dropped" not in line
    assert line["configs"][0]["entry"] == "append_paged_kv_cache_layers"      # prefix dropped in the line
    assert line["roofline"]["frac"] == 0.7051 and line["cpu_baseline"]["cores"] == 16


def test_rows_beyond_the_limit_are_dropped_not_the_headline():
    text = bench.build_line(_head(), [_row(i) for i in range(200)])
    assert len(text.encode()) < bench.MAX_LINE_BYTES and "\n" not in text
    line = json.loads(text)
    assert line["configs_dropped"] == 200 - len(line["configs"]) > 0
    assert line["value"] == 5641.1 and line["roofline"] and line["cpu_baseline"]


def test_not_a_number_is_refused():
    import pytest
    head = _head()
    head["value"] = float("nan")
    with pytest.raises(ValueError):
        bench.build_line(head, [])


def test_default_sections_are_the_benchmarks_operations():
    args = bench.parse_args([])
    assert args.gpus == 1 and set(args.ops.split(",")) == {"write", "prefill", "copy", "swap", "step"}
    assert args.hw_queues == 0 and args.settle_seconds == 0.0


def test_every_section_module_imports_without_a_gpu():
    """The opt-in sections are imported lazily on the GPU box; a mistake in them must
    show here first. Every section the parser advertises has its function."""
    import bench
    import bench_sections
    import bench_util
    for name in ("bench_size_sweep", "bench_disk_tier", "bench_write_through_overlap", "bench_small_write_through",
                 "bench_two_process_swap", "bench_rope_decode", "bench_rope_prefill", "bench_index_prep",
                 "bench_calibration", "bench_slot_patterns", "bench_tp_shard", "bench_decode_step_graph",
                 "bench_load_policy", "bench_duplex_streams"):
        assert callable(getattr(bench_sections, name)), name
    assert callable(bench_util.time_region) and callable(bench.main)
    help_text = bench.parse_args(["--ops", "none"]) and bench.__doc__
    for op in ("rope", "shard", "index", "overlap", "twoproc", "disk", "sweep", "calib", "translation", "loads", "duplex"):
        assert op in help_text, op
