"""Host-side checks of the rules this repository keeps: the product never routes through the CPU oracle, the
benchmark refuses more than one GPU, and the bench's tables name workloads that exist."""
import ast
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _imports(path):
    tree = ast.parse(open(path).read())
    names = []
    for node in ast.walk(tree):
        if isinstance(node, ast.Import):
            names += [a.name for a in node.names]
        elif isinstance(node, ast.ImportFrom):
            names.append(("." * node.level) + (node.module or ""))
    return names


def test_the_product_package_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "matchattention_amd")
    files = [os.path.join(pkg, f) for f in os.listdir(pkg) if f.endswith(".py")] + [os.path.join(ROOT, "match_attention.py")]
    assert len(files) > 5
    for f in files:
        bad = [n for n in _imports(f) if n.split(".")[0] == "oracle" or n.lstrip(".").split(".")[0] == "oracle"]
        assert not bad, (f, bad)
        text = open(f).read()
        assert "import_module(\"oracle" not in text and "oracle/" not in text, f     # not by name or path either


def test_bench_reaches_the_oracle_only_in_its_cpu_baseline_legs():
    src = open(os.path.join(ROOT, "bench.py")).read()
    tree = ast.parse(src)
    users = set()
    for fn in [n for n in ast.walk(tree) if isinstance(n, ast.FunctionDef)]:
        for node in ast.walk(fn):
            if isinstance(node, (ast.Import, ast.ImportFrom)):
                mods = [a.name for a in node.names] if isinstance(node, ast.Import) else [node.module or ""]
                if any(m.split(".")[0] == "oracle" for m in mods):
                    users.add(fn.name)
    top = [n for n in tree.body if isinstance(n, (ast.Import, ast.ImportFrom))]
    assert not any((getattr(n, "module", None) or "").startswith("oracle") for n in top)
    assert users and all(name.startswith("_cpu_baseline") for name in users), users


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)


def test_measured_traffic_tables_name_existing_workloads():
    sys.path.insert(0, ROOT)
    import bench
    from matchattention_amd.workloads import WORKLOADS
    for (w, k), v in bench.MEASURED_TRAFFIC_BYTES.items():
        assert w in WORKLOADS and k.startswith("fwd_") and v > 0
    for (w, k), per_kernel in bench.MEASURED_BWD_TRAFFIC_BYTES.items():
        assert w in WORKLOADS and k.startswith("bwd_") and all(b > 0 for b in per_kernel.values())


def test_no_inline_assembly_instructions_in_the_kernel_that_uses_the_matrix_unit():
    """The compiler's hazard checks do not look into inline assembly, and its destination may be a register that a
    matrix instruction in flight still writes: the kernels of matchattn_fwd_tile.h (the only ones with matrix
    instructions) keep to builtins and plain code; empty asm statements that pin a register are fine."""
    import re
    src = open(os.path.join(ROOT, "matchattention_amd", "csrc", "matchattn_fwd_tile.h")).read()
    assert "__builtin_amdgcn_mfma" in src
    for m in re.finditer(r'asm\s*(?:volatile)?\s*\(\s*"([^"]*)"', src):
        assert m.group(1).strip() == "", m.group(0)
    # and the helper it would inherit inline assembly from is not called beside the matrix instructions
    body = src[src.index("if constexpr (kMatrixSum) {"):]
    assert "l1_sum" not in body[:body.index("} else {")]
