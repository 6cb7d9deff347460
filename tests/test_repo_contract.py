"""Repository-level rules that code review alone would have to re-check every time."""

import ast
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _node_imports(node):
    if isinstance(node, ast.Import):
        return [a.name for a in node.names]
    if isinstance(node, ast.ImportFrom):
        return [("." * node.level) + (node.module or "")]
    return []


def _imports(tree):
    return [m for node in ast.walk(tree) for m in _node_imports(node)]


def test_package_never_imports_the_oracle():
    """The oracle is test infrastructure: nothing under deconver_amd/ may import it."""
    pkg = os.path.join(ROOT, "deconver_amd")
    for name in os.listdir(pkg):
        if name.endswith(".py"):
            path = os.path.join(pkg, name)
            for module in _imports(ast.parse(open(path).read(), path)):
                assert not module.lstrip(".").startswith("oracle"), f"{name} imports {module}"


def test_bench_uses_the_oracle_only_for_the_cpu_baseline():
    path = os.path.join(ROOT, "bench.py")
    tree = ast.parse(open(path).read(), path)
    for func in ast.walk(tree):
        if isinstance(func, ast.FunctionDef):
            uses = [m for m in _imports(func) if m.startswith("oracle")]
            if uses:
                assert func.name == "cpu_baseline", f"bench.py:{func.name} imports {uses}"
    top_level = [m for node in tree.body for m in _node_imports(node) if m.startswith("oracle")]
    assert not top_level


def test_bench_refuses_more_than_one_gpu():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode != 0
    assert "one-GPU" in proc.stderr and proc.stdout.strip() == ""


def test_nothing_committed_reaches_into_the_working_folder():
    """_work/ holds the builder's scratch files; product, tests and docs must not use it."""
    tracked = subprocess.run(["git", "ls-files"], cwd=ROOT, stdout=subprocess.PIPE, text=True).stdout.split()
    for rel in tracked:
        if rel.endswith((".py", ".h", ".hip", ".cpp", ".c", "Makefile")) and rel != "tests/test_repo_contract.py":
            assert "_work/" not in open(os.path.join(ROOT, rel), errors="replace").read(), rel
