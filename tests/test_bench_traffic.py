"""bench.py's roofline.traffic comes from profiles/cfg3_traffic.json: the file must name kernels the benchmark
knows (by their algorithmic bytes), and bench.py must refuse a step that launches a kernel the file lacks."""
import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402

SHAPE = dict(L=5000000, U=2000000, G=1080000, G1=917000, Rm=550000, Gm=149000, Rb=548000, Gb=13500, T=2940000)
# side measurements of bench.py (combiner, ShowDecay, dense): profiled in the same runs, not part of the step
SIDE = ("k_show_decay", "k_reduce_pooled", "k_reduce_long", "k_combine_fwd", "k_lookup_keys", "k_example_rowptr",
        "k_place_lookups", "k_rank_short", "k_rank_mid", "k_order_huge", "k_dense_adam_v4", "k_dense_adagrad_v4",
        "k_probe", "k_load_rows", "k_export_rows", "k_finish_insert", "k_reset_status", "k_zero_f32", "k_fill_f32")


def test_traffic_file_names_known_kernels():
    with open(bench.TRAFFIC_FILE) as f:
        t = json.load(f)
    assert t["commit"] and t["fetch_factor"] > 0 and t["write_factor"] > 0
    names = t["bytes_per_launch"]
    assert names, "no kernels in the traffic file"
    for k, v in names.items():
        assert v > 0
        known = bench.kernel_algorithmic_bytes(k, "AdaGrad", 16, SHAPE) > 0
        assert known or k.startswith(SIDE) or k.startswith(bench.SMALL_STEP_KERNELS), "unknown kernel %s" % k
    # the kernels of the cfg3 step all have their figure
    step = ["k_tile_dedup", "k_lds_dedup<true>", "k_lds_flags", "k_lds_assign<false>", "k_lds_mapped",
            "k_group_count", "k_group_emit", "k_probe_recs", "k_gather_vars<4>", "k_verify_values<true, false>",
            "k_apply_single<KIND, 4>", "k_apply_vec<KIND, 4>", "k_apply_big_adagrad<DIM>", "k_stage_in", "k_publish"]
    per_launch, source = bench.measured_traffic(step)
    assert source["file"] == "profiles/cfg3_traffic.json" and source["profiled_at_commit"] == t["commit"]
    assert per_launch["k_apply_single"] > bench.kernel_algorithmic_bytes("k_apply_single", "AdaGrad", 16, SHAPE) * 0.5


def test_a_kernel_without_a_figure_is_refused():
    with pytest.raises(SystemExit) as e:
        bench.measured_traffic(["k_tile_dedup", "k_some_new_kernel<4>"])
    assert "k_some_new_kernel" in str(e.value)
