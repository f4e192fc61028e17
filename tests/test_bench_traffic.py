"""bench.py reports the HBM traffic of its kernels (`roofline.traffic`) from counter readings that are taken offline
and kept as text under profiles/. Each summary there ends in one line that states the figure in the form bench.py
holds it; this test reads those lines and compares, so a kernel that is profiled again without the benchmark's
table being brought along (or the other way round) fails here."""
import ast
import glob
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LINE = re.compile(r'^bench\.py TRAFFIC_BYTES\["(\w+)"\] = (.+) KiB$')


def traffic_table_of_bench():
    """TRAFFIC_BYTES as bench.py's source states it (read, not imported: the module needs a GPU stack to import)."""
    tree = ast.parse(open(os.path.join(ROOT, "bench.py")).read())
    for node in tree.body:
        if isinstance(node, ast.Assign) and getattr(node.targets[0], "id", None) == "TRAFFIC_BYTES":
            return {k.value: eval(compile(ast.Expression(v), "bench.py", "eval")) for k, v in zip(node.value.keys, node.value.values)}
    raise AssertionError("bench.py holds no TRAFFIC_BYTES table")


def traffic_lines_of_profiles():
    found = {}
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.txt"))):
        for line in open(path):
            m = LINE.match(line.strip())
            if m:
                expr = m.group(2).replace(",", "")
                assert re.fullmatch(r"[0-9+*() ]+", expr), (path, expr)
                assert m.group(1) not in found, f"{m.group(1)} stated twice"
                found[m.group(1)] = (eval(expr) * 1024, os.path.basename(path))
    return found


def test_the_traffic_figures_of_the_benchmark_are_the_profiles_figures():
    table, lines = traffic_table_of_bench(), traffic_lines_of_profiles()
    assert set(table) == set(lines), (sorted(table), sorted(lines))
    for key, value in table.items():
        assert value == lines[key][0], f"{key}: bench.py {value} B, {lines[key][1]} {lines[key][0]} B"
