"""The synthetic benchmark harness on its smallest workloads (GPU)."""

import json

import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("argv", [
    ["--config", "c1", "--repeats", "1", "-ne", "5", "-k", "5,20"],
    ["--config", "c1", "--fit-query", "--host-inputs", "--repeats", "0", "-ne", "3", "-k", "10"],
    ["--config", "c3", "-n", "20000", "-nq", "200", "--repeats", "1", "-ne", "4", "-k", "10", "-bs", "64"],
    ["--config", "c4", "-n", "5000", "-nq", "100", "--repeats", "1", "-ne", "4", "-k", "10"],
    ["--config", "c4", "-n", "5000", "-nq", "100", "--repeats", "1", "-ne", "4", "-k", "10", "--prime", "2147483647"],
])
def test_benchmark_report(argv, capsys):
    from culsh_amd import benchmark

    assert benchmark.main(argv) == 0
    report = json.loads(capsys.readouterr().out)
    assert report["data"]["kind"] == "synthetic"
    if "--fit-query" in argv:
        assert report["runtimes"]["fit_query_time"] > 0
        # a row is always among its own candidates, and its own nearest neighbour
        assert report["recall_evaluation"]["queries_with_candidates"] == report["recall_evaluation"]["n_eval_queries"]
    else:
        assert report["runtimes"]["fit_time"] > 0 and report["runtimes"]["query_time"] > 0
        assert report["throughput"]["fit_mvec_per_s"] > 0
        assert report["index"]["n_total_buckets"] > 0
    if report["algorithm"] == "MinHashLSH":  # every MinHash report names its prime
        assert report["params"]["prime"] == (2147483647 if "--prime" in argv else 4294967291)
    rec = report["recall_evaluation"]
    for k, v in rec["recall_at_k"].items():
        assert 0.0 <= v <= 1.0
        assert len(rec["per_query_recall_at_k"][k]) == rec["n_eval_queries"]
