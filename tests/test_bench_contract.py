"""bench.py on a machine without a GPU: what it must do before it touches one -- refuse more than one GPU with a
message that says why, know every measured workload, and keep the traffic table pointing at profiles that exist and at
kernel sources that exist (its figures are withheld, not wrong, when a digest no longer matches)."""
import os
import subprocess
import sys

ROOT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")


def test_more_than_one_gpu_is_refused_with_a_reason():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and "--gpus 2" in r.stderr


def test_traffic_table_names_existing_profiles_and_sources():
    sys.path.insert(0, ROOT)
    import bench
    from cuplayground_amd import workloads as wl
    assert {k.split("/")[0] for k in bench.MEASURED_TRAFFIC} <= set(wl.WORKLOADS)
    for key, t in bench.MEASURED_TRAFFIC.items():
        name = key.split("/")[0]       # "<workload>/<plan>": the same workload under a non-default plan
        assert os.path.isfile(os.path.join(ROOT, t["profile"])), t["profile"]
        for src in t["sources"]:
            assert os.path.isfile(os.path.join(ROOT, "cuplayground_amd", "csrc", src)), src
        assert len(t["kernel_digest"]) == 12 and t["bytes"] > 0
        text = open(os.path.join(ROOT, t["profile"])).read()
        assert "rocprofv3 --pmc FETCH_SIZE" in text and "--workload %s" % name in text or name == "mixtral"


def test_workloads_cover_the_five_measured_shapes():
    sys.path.insert(0, ROOT)
    from cuplayground_amd import workloads as wl
    tags = {w.tag for w in wl.WORKLOADS.values()}
    assert {"C1", "C2", "C3", "C4", "C5"} <= tags
    assert wl.WORKLOADS["mixtral"].config.tokens == 8192 and wl.WORKLOADS["mixtral"].bound == "mfma"
    assert wl.WORKLOADS["decode_fp8"].bound == "hbm"
