"""The committed rocprofv3 summaries that bench.py quotes figures from (roofline.traffic) were taken with the kernel
sources the tree holds: each names the digest of those sources, and bench.py drops the figure when they differ."""
import os
import sys

from util import ROOT

sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_traffic_summaries_match_the_kernel_sources():
    for fname, key, sources in ((bench.TRAFFIC_PROFILE, "gemv_batch1_traffic_over_algorithmic", bench.GEMV_SOURCES),
                                (bench.CODEC_TRAFFIC_PROFILE, "pack_q8_0_traffic_over_algorithmic", bench.CODEC_SOURCES)):
        ratio, source = bench.profiled_ratio(fname, key, sources)
        assert ratio is not None, "%s: %s -- regenerate the summary with the command it names" % (fname, source)
        assert 0.9 < ratio < 1.2, (fname, ratio)
        assert source == "profiles/" + fname


def test_a_changed_source_makes_the_figure_stale(tmp_path, monkeypatch):
    # the same summary judged against another set of sources
    ratio, source = bench.profiled_ratio(bench.TRAFFIC_PROFILE, "gemv_batch1_traffic_over_algorithmic", ("codec.hip",))
    assert ratio is None and source.startswith("stale:")
    ratio, source = bench.profiled_ratio("no_such_summary.txt", "x", bench.GEMV_SOURCES)
    assert ratio is None and source == "absent"


def test_every_summary_names_its_command():
    d = os.path.join(ROOT, "profiles")
    names = [f for f in os.listdir(d) if f.endswith((".txt", ".md"))]
    assert names
    for f in names:
        text = open(os.path.join(d, f)).read()
        assert "rocprofv3 " in text and ("bench.py" in text), f
        assert "_work" not in text, f
