"""bench.py's command-line contract, checked without a GPU: more than one GPU is refused with a
message, the workload table names the configurations BASELINE.json lists, and the checker
(`oracle/`) is imported by the CPU-baseline leg only."""
import ast
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2
    assert "ONE GPU" in r.stderr and "--gpus 2" in r.stderr
    env = dict(os.environ, WORLD_SIZE="4")
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")], capture_output=True, text=True, env=env, timeout=120)
    assert r.returncode == 2 and "ONE GPU" in r.stderr


def test_workload_table_covers_the_baseline_configs():
    sys.path.insert(0, ROOT)
    import bench

    base = json.load(open(os.path.join(ROOT, "BASELINE.json")))
    assert len(base["configs"]) == len(bench.WORKLOADS) == 5
    family, cfg, batch, batch_cnt, splits, device_cnt, mixed = bench.WORKLOADS["vit_l16_fp16"]
    assert (family, batch, batch_cnt, splits, device_cnt, mixed) == ("vit", 64, 4, ["blocks.12"], 2, "fp16")
    assert bench.WORKLOADS["llama_1b_bf16"][2:] == (16, 8, ["layers.4", "layers.8", "layers.12"], 2, "bf16")
    assert bench.PEAK_HBM_GBS == 8000


def test_only_the_cpu_baseline_leg_imports_the_oracle():
    tree = ast.parse(open(os.path.join(ROOT, "bench.py")).read())
    users = set()
    for fn in [n for n in tree.body if isinstance(n, ast.FunctionDef)]:
        for node in ast.walk(fn):
            names = []
            if isinstance(node, ast.ImportFrom) and node.module:
                names = [node.module]
            elif isinstance(node, ast.Import):
                names = [a.name for a in node.names]
            if any(n == "oracle" or n.startswith("oracle.") for n in names):
                users.add(fn.name)
    top = [n for n in tree.body if isinstance(n, (ast.Import, ast.ImportFrom))]
    for node in top:
        mod = node.module if isinstance(node, ast.ImportFrom) else ",".join(a.name for a in node.names)
        assert "oracle" not in (mod or "")
    assert users == {"cpu_baseline"}, users


def test_the_product_package_never_imports_the_checker_or_scratch_files():
    """Nothing under pfeife_amd/ (nor the `pfeife` alias package) imports `oracle` or reads the scratch folder;
    `__graft_entry__.py` imports the oracle in smoke() only."""
    bad = []
    for top in ("pfeife_amd", "pfeife"):
        for dirpath, _, files in os.walk(os.path.join(ROOT, top)):
            for f in files:
                if not f.endswith(".py"):
                    continue
                path = os.path.join(dirpath, f)
                src = open(path).read()
                tree = ast.parse(src)
                for node in ast.walk(tree):
                    mods = []
                    if isinstance(node, ast.ImportFrom) and node.module:
                        mods = [node.module]
                    elif isinstance(node, ast.Import):
                        mods = [a.name for a in node.names]
                    if any(m == "oracle" or m.startswith("oracle.") for m in mods):
                        bad.append(path)
                if "_work/" in src or "_work\\\\" in src:
                    bad.append(path + " (_work)")
    assert not bad, bad
    tree = ast.parse(open(os.path.join(ROOT, "__graft_entry__.py")).read())
    users = set()
    for fn in [n for n in tree.body if isinstance(n, ast.FunctionDef)]:
        for node in ast.walk(fn):
            mods = []
            if isinstance(node, ast.ImportFrom) and node.module:
                mods = [node.module]
            elif isinstance(node, ast.Import):
                mods = [a.name for a in node.names]
            if any(m == "oracle" or m.startswith("oracle.") for m in mods):
                users.add(fn.name)
    assert users <= {"smoke", "build"}, users
