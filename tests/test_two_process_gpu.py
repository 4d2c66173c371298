"""llis_server and llis_app_client as two processes on the device (the deployment shape of the reference:
src/server/server.cpp:203-235 and app/client.cpp, driven by sosp23_artifact/gen_data_fig12_paella.sh:62-84).  The pair is
run once per session by tests/conftest.py, before the test interpreter touches the GPU; this file checks what it left."""
import pytest

import conftest

pytestmark = pytest.mark.gpu


def test_server_and_client_binaries_serve_the_two_tenant_mix_as_two_processes(cuda):
    r = conftest.TWO_PROCESS
    assert r, "the session-start run did not happen (GPU tests must be selected with -m gpu)"
    assert "error" not in r, r
    assert r["client_rc"] == 0, r.get("client_stderr")
    assert r["server_rc"] == 0
    s = r["stats"]
    assert s["num_jobs"] == 6000 and sum(s["per_type_count"]) == 5500
    assert 400 < s["per_type_count"][1] < 700                      # about one request in ten is Inception-v3
    # 6000 Poisson arrivals at 10 000 per second take 0.6 s; the served rate keeps up with the offered one
    assert 8000 < s["throughput_rps"] < 12000
    # stats row: x, num_jobs, elapsed, then mean/p50/p90/p95/p99/max/sd overall and per type (reference app/client.cpp:479-495)
    row = r["csv_row"].split(",")
    assert row[0] == "100" and row[1] == "6000" and len(row) == 3 + 7 * 3
    p50_small, p50_big = float(row[3 + 7 + 1]), float(row[3 + 14 + 1])
    assert 5 < p50_small < 2000 and 300 < p50_big < 20000
