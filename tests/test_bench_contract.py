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


def _undefined_names(path):
    """Names a module's functions load that are bound nowhere: not in the function (or an enclosing one), not at module
    level, not a builtin.  A small scope walk over the syntax tree -- enough to catch a variable pasted from another
    function, which only fails when the line that reads it finally runs."""
    import ast
    import builtins
    tree = ast.parse(open(path).read(), path)

    def bound_in(node):
        names = set()
        for n in ast.walk(node):
            if isinstance(n, ast.Name) and isinstance(n.ctx, (ast.Store, ast.Del)):
                names.add(n.id)
            elif isinstance(n, (ast.FunctionDef, ast.AsyncFunctionDef, ast.ClassDef)):
                names.add(n.name)
                if not isinstance(n, ast.ClassDef):
                    a = n.args
                    for arg in a.posonlyargs + a.args + a.kwonlyargs + [a.vararg, a.kwarg]:
                        if arg is not None:
                            names.add(arg.arg)
            elif isinstance(n, (ast.Import, ast.ImportFrom)):
                for al in n.names:
                    names.add((al.asname or al.name).split(".")[0])
            elif isinstance(n, ast.ExceptHandler) and n.name:
                names.add(n.name)
        return names

    module_names = set(dir(builtins))
    for stmt in tree.body:        # module level only: what a function binds is not visible to its neighbours
        if isinstance(stmt, (ast.FunctionDef, ast.AsyncFunctionDef, ast.ClassDef)):
            module_names.add(stmt.name)
        else:
            module_names |= bound_in(stmt)
    missing = []
    for fn in [n for n in tree.body if isinstance(n, (ast.FunctionDef, ast.AsyncFunctionDef))]:
        local = bound_in(fn)      # nested functions included: a superset of what any inner scope can see
        for n in ast.walk(fn):
            if isinstance(n, ast.Name) and isinstance(n.ctx, ast.Load) and n.id not in local and n.id not in module_names:
                missing.append((fn.name, n.id, n.lineno))
    return missing


def test_bench_reads_no_undefined_name():
    assert _undefined_names(os.path.join(ROOT, "bench.py")) == []
    assert _undefined_names(os.path.join(ROOT, "__graft_entry__.py")) == []


def test_undefined_name_check_sees_a_pasted_variable(tmp_path):
    p = tmp_path / "m.py"
    p.write_text("import os\n\ndef f(a):\n    b = a + 1\n    return b\n\ndef g(a):\n    return layer.plan if a else os.sep\n")
    assert _undefined_names(str(p)) == [("g", "layer", 8)]
