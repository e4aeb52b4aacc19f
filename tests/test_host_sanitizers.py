"""Host code of the library under AddressSanitizer + UndefinedBehaviorSanitizer (CPU only; GPU code is never built or
run with a sanitizer).  The knob-file loader is the one piece of the library that parses untrusted text, so it is the
piece compiled this way: csrc/config.cpp together with tests/host/config_sanitized.cpp, with g++."""
import json
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_config_loader_is_clean_under_asan_and_ubsan(tmp_path):
    exe = str(tmp_path / "config_sanitized")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=all", "-static-libasan", "-I", os.path.join(ROOT, "include"), "-o", exe,
           os.path.join(ROOT, "cuplayground_amd", "csrc", "config.cpp"), os.path.join(ROOT, "tests", "host", "config_sanitized.cpp")]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    ref = tmp_path / "aristos_config.json"
    ref.write_text(json.dumps({"capacity_factor": 1, "drop_tokens": 0, "expert_top_k": 1, "is_training": 0, "hidden_act": 0,
                               "hidden_size": 1024, "intermediate_size": 4096, "micro_batch": 4, "num_experts": 1,
                               "sequence_len": 2048, "torch_dtype": 0}, indent=2))
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    env.pop("LD_PRELOAD", None)     # the sanitizer runtime wants to come first
    r = subprocess.run([exe, str(ref)], capture_output=True, text=True, env=env, timeout=120)
    assert r.returncode == 0, (r.stdout + r.stderr)[-4000:]
    assert "0 failed checks" in r.stdout


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_queue_order_keeps_every_dependency_under_asan_and_ubsan(tmp_path):
    """csrc/queue_order.hpp is the code the routing kernel builds its merged task queue with; the same functions run here
    on the host for 20000 random layers: every row block's up-projection run stands in front of its down-projection run,
    the id space has no gaps, a rounded tail fills whole rounds of the workgroups, and with the last row blocks' tiles cut into
    partial sums every id of every queue decodes to each (row block, column tile, part) exactly once."""
    exe = str(tmp_path / "queue_order")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=all", "-static-libasan", "-I", os.path.join(ROOT, "cuplayground_amd", "csrc"), "-o", exe,
           os.path.join(ROOT, "tests", "host", "queue_order.cpp")]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    env.pop("LD_PRELOAD", None)
    r = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, (r.stdout + r.stderr)[-4000:]
    assert " 0 failed checks" in r.stdout and "with a rounded tail" in r.stdout and "with partial sums decoded id by id" in r.stdout
