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
