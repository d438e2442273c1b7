"""bench.py's host-side helpers: the traffic figures of the roofline object come from the rocprofv3 summaries
under profiles/, keyed on the exact configuration a run measures."""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_default_workload_has_counter_traffic_on_file():
    import bench

    for kernel in ("k_app_feat", "k_march"):
        got = bench.measured_traffic("c4_1080p_multires_P3_base1024_shift0", 1044480, "f16x2", "auto", kernel)
        assert got is not None, f"no bench-traffic line for {kernel} of the default workload under profiles/"
        nbytes, where = got
        assert 1e9 < nbytes < 1e11 and where.startswith("profiles/") and ":" in where
        path, line = where.rsplit(":", 1)
        text = open(os.path.join(ROOT, path)).read().split("\n")[int(line) - 1]
        assert text.startswith("bench-traffic:") and f"kernel={kernel}" in text
    # any other configuration is not covered by that line: no figure rather than a stale one
    assert bench.measured_traffic("c4_1080p_multires_P3_base1024_shift0", 262144, "f16x2", "auto", "k_app_feat") is None
    assert bench.measured_traffic("c4_1080p_multires_P3_base1024_shift0", 1044480, "f16", "auto", "k_app_feat") is None
    assert bench.measured_traffic("c4_1080p_multires_P3_base1024_shift0", 1044480, "f16x2", "0", "k_app_feat") is None


def test_frame_chunks_are_whole_bands_within_32_bit_sample_indices():
    import bench

    class M:
        ray_row_length = -1

    m = M()
    assert bench.frame_chunks(m, 1920 * 1080, 128, 1920, 1 << 20) == 1044480 and m.ray_row_length == 1920
    assert bench.frame_chunks(m, 1920 * 1080, 128, 1920, 1 << 20, row_hint=False) == 1 << 20 and m.ray_row_length == 0
    c = bench.frame_chunks(m, 1920 * 1080, 3544, 1920, 1 << 21)
    assert c * 3544 < 2**32 and c % (8 * 1920) == 0
    assert bench.frame_chunks(m, 1000, 128, 50, 1 << 20) == 1000 and m.ray_row_length == 0  # 50 is no multiple of 8


def test_every_traffic_line_is_well_formed_and_found_by_its_own_key():
    """Each `bench-traffic:` line under profiles/ names workload, chunk, network mode, termination setting and kernel,
    carries positive byte counts, and is the line the lookup returns for that key (no two summaries claim one
    configuration); every summary says which commit it was taken at."""
    import re

    import bench

    prof = os.path.join(ROOT, "profiles")
    seen = {}
    for fn in sorted(os.listdir(prof)):
        if not fn.endswith(".txt"):
            continue
        text = open(os.path.join(prof, fn)).read()
        assert re.search(r"[Tt]aken at commit [0-9a-f]{7}", text), f"{fn}: no commit stamp"
        for ln, line in enumerate(text.split("\n"), 1):
            if not line.startswith("bench-traffic:"):
                continue
            kv = dict(tok.split("=", 1) for tok in line.split()[1:])
            assert set(kv) == {"workload", "chunk", "mlp", "term_eps", "kernel", "fetch_bytes", "write_bytes"}, (fn, ln)
            assert float(kv["fetch_bytes"]) > 0 and float(kv["write_bytes"]) > 0 and int(kv["chunk"]) > 0
            key = (kv["workload"], int(kv["chunk"]), kv["mlp"], kv["term_eps"], kv["kernel"])
            assert key not in seen, f"{fn}:{ln} repeats {seen[key]}"
            seen[key] = f"profiles/{fn}:{ln}"
            got = bench.measured_traffic(*key)
            assert got is not None and got[1] == seen[key]
            assert abs(got[0] - float(kv["fetch_bytes"]) - float(kv["write_bytes"])) < 1.0
    workloads = {k[0] for k in seen}
    assert any(w.startswith("c4_") for w in workloads) and any(w.startswith("c5_") for w in workloads) and any(w.startswith("prod_") for w in workloads)
