"""bench.py quotes HBM traffic and issued flops from earlier profiler runs (its COUNTER_TRAFFIC table).  These tests
hold every quoted number to the profile summary it names, so that refreshing a profile without the table (or the
reverse) fails here; and they check that the quantities the bench line measures itself are no longer typed in."""
import importlib.util
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# the kernels of the steady-state frame (the one-level scatter_kernel<0> only runs for a workspace's first frame there)
SHIPPED_SORT_KERNELS = ("tile_count_kernel", "slice_prefix_kernel", "tile_publish_kernel", "scatter_kernel<4",
                        "fine_scatter_kernel", "tile_sort_each_kernel", "tile_sort_list_kernel<512",
                        "tile_sort_list_1024x5_kernel")


def load_bench():
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def traffic_table(path):
    rows = {}
    for line in open(path):
        m = re.match(r"^(\S.*?)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s*$", line)
        if m:
            rows[m.group(1).strip()] = float(m.group(6))  # total MB per launch
    return rows


def test_quoted_traffic_matches_the_profile_it_names():
    bench = load_bench()
    table = bench.COUNTER_TRAFFIC
    path = os.path.join(ROOT, table["source"])
    if not os.path.exists(path):
        pytest.skip("profiles/ is not part of this checkout")
    rows = traffic_table(path)
    assert rows, "no kernel rows parsed from %s" % table["source"]
    want = {
        "blend": sum(v for k, v in rows.items() if k.startswith("blend_kernel")),
        "preprocess": sum(v for k, v in rows.items() if k.startswith("preprocess_kernel")),
        "keys_sort_ranges": sum(v for k, v in rows.items() if k.startswith(SHIPPED_SORT_KERNELS)),
    }
    for name, mb in want.items():
        assert mb > 0, name
        assert abs(table["bytes"][name] / 1e6 - mb) <= 0.002 * mb + 0.2, (name, table["bytes"][name] / 1e6, mb)


def test_quoted_decode_traffic_matches_the_profile_it_names():
    bench = load_bench()
    table = bench.COUNTER_TRAFFIC_C5
    path = os.path.join(ROOT, table["source"])
    if not os.path.exists(path):
        pytest.skip("profiles/ is not part of this checkout")
    # count + emit passes of the fp16-exact variant, which the named workload runs (<.., .., true> = fp32 weights)
    mb = sum(v for k, v in traffic_table(path).items() if k.startswith("decode_kernel") and k.endswith("false>"))
    assert mb > 0 and abs(table["bytes"]["decode"] / 1e6 - mb) <= 0.002 * mb + 0.2, (table["bytes"]["decode"] / 1e6, mb)


def test_quoted_issued_flops_match_the_profile_they_name():
    bench = load_bench()
    table = bench.COUNTER_TRAFFIC
    path = os.path.join(ROOT, table["blend_issued_flops_source"])
    if not os.path.exists(path):
        pytest.skip("profiles/ is not part of this checkout")
    text = open(path).read()
    block = text[text.index("blend_kernel<true>"):]
    block = block[:block.index("\n\n")] if "\n\n" in block else block
    c = {k: int(v) for k, v in re.findall(r"(SQ_INSTS_VALU_(?:FMA|MUL|ADD)_F32)\s+(\d+)", block)}
    flops = 64 * (2 * c["SQ_INSTS_VALU_FMA_F32"] + c["SQ_INSTS_VALU_MUL_F32"] + c["SQ_INSTS_VALU_ADD_F32"])
    assert abs(table["blend_issued_flops"] - flops) <= 0.005 * flops
    busy = float(re.search(r"VALU busy = .*? = ([\d.]+) %", block).group(1)) / 100.0
    assert abs(table["blend_valu_busy"] - busy) <= 0.01


def test_pair_counts_are_measured_not_typed():
    """The blend's algorithmic flops come from pair counts the C checker produces inside the bench run."""
    src = open(os.path.join(ROOT, "bench.py")).read()
    assert "BLEND_PAIRS" not in src
    assert not re.search(r"pairs[\"']?\s*[:=]\s*\{?\s*[\"']?evaluated[\"']?\s*:\s*[\d.]+e\d", src)
    assert "cpu_pair_stats" in src and "pairs_evaluated" in src


def test_pair_stats_of_a_small_frame_agree_with_the_checker():
    """bench.cpu_pair_stats is the checker's own count (same numbers as oracle.c_oracle.render on the same scene)."""
    from landmarksystem_amd import scenes
    from oracle import c_oracle as co
    from tests.helpers import oracle_frame, oracle_gaussians
    bench = load_bench()
    scene = scenes.config1(P=3000, width=128, height=96)
    got = bench.cpu_pair_stats(scene)
    ref = co.render(oracle_frame(scene), oracle_gaussians(scene), keep_intermediates=False)
    assert (got["evaluated"], got["accepted"], got["tile_work"], got["num_keys"]) == \
        (ref["pairs_evaluated"], ref["pairs_accepted"], ref["tile_work"], ref["num_keys"])
    assert got["evaluated"] >= got["accepted"] > 0 and got["tile_work"] >= got["evaluated"]
