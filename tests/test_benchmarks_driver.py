"""The generic benchmark runner (mirror of examples/benchmarks.jl): discovery, the result / metric protocol of
the example modules, the table; on a GPU one full pass over two examples at their benchmark sizes."""
import io

import pytest


@pytest.fixture(scope="module")
def bm(ct):
    from cutile_jl_amd.examples import benchmarks
    return benchmarks


def test_discovery_finds_every_example(bm):
    """benchmarks.jl:68-80: all example files but the runner itself, sorted; names filter."""
    assert bm.discover_benchmarks() == ["batchmatmul", "fft", "fmha", "layernorm", "matmul", "moe", "softmax", "transpose", "vadd"]
    assert bm.discover_benchmarks("vadd", "fmha", "nothing") == ["fmha", "vadd"]


def test_throughput_formats(bm):
    """benchmarks.jl:26-38: GB/s rounded to an integer, TFLOPS to one digit, a latency in microseconds."""
    assert bm.format_throughput(3 * 2 ** 27 * 4, "GB/s", 0.25) == "6442 GB/s"
    assert bm.format_throughput(2 * 4096 ** 3, "TFLOPS", 0.13) == "1057.2 TFLOPS"
    assert bm.format_throughput(0, "us", 0.0113) == "11 \u03bcs"
    assert bm.format_throughput(1, "furlongs", 1.0) == ""


def test_summary_rows_follow_the_metric_protocol(bm):
    """benchmarks.jl:158-177: throughput from the minimum time; a (total, unit) metric applies to every row, a dict
    only to the rows it names; rows sorted by their minimum."""
    res = {"cuTile": [1.0, 2.0], "other": [0.5, 0.7]}
    assert bm.summarize(res, (1e9, "GB/s")) == [("other", 0.5, 0.6, "2000 GB/s"), ("cuTile", 1.0, 1.5, "1000 GB/s")]
    assert bm.summarize(res, {"cuTile": (2e12, "TFLOPS")}) == [("other", 0.5, 0.6, ""), ("cuTile", 1.0, 1.5, "2000.0 TFLOPS")]
    assert bm.summarize(res, None) == [("other", 0.5, 0.6, ""), ("cuTile", 1.0, 1.5, "")]
    out = io.StringIO()
    bm.print_table("demo", bm.summarize(res, (1e9, "GB/s")), file=out)
    lines = out.getvalue().splitlines()
    assert lines[2] == "  demo" and lines[4].startswith("Implementation") and lines[4].rstrip().endswith("Throughput")
    assert lines[6].split() == ["other", "0.500", "0.600", "2000", "GB/s"]


@pytest.mark.gpu
def test_runner_end_to_end_on_two_examples(bm):
    """One pass of the runner over transpose (one implementation row of ours + the vendor library's) and softmax
    (two rows of ours, named by the metric dict, + two others): 20 timed runs each, finite positive times."""
    ret = bm.run_benchmark("transpose")
    assert ret is not None
    results, metric = ret
    assert set(results) == {"cuTile", "torch copy_(x.t())"} and metric == (2 * 8192 * 8192 * 4, "GB/s")
    assert all(len(t) == bm.NRUNS and min(t) > 0 for t in results.values())
    results, metric = bm.run_benchmark("softmax")
    assert set(metric) == {"cuTile TMA", "cuTile Chunked"} and set(metric) < set(results)
    rows = bm.summarize(results, metric)
    assert [r[3] != "" for r in rows].count(True) == 2      # only the rows the metric names carry a throughput
    out = io.StringIO()
    bm.main("fft", file=out)
    text = out.getvalue()
    assert "Benchmarking fft..." in text and "rocFFT" in text and "Benchmark Complete" in text
