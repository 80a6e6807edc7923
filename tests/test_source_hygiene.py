"""Source files must stand on their own: comments and docstrings state facts and cite the
reference by file and line, and never point at this build's planning documents, its
remote-run tooling or a stage of the build.  Also: nothing that ships imports the oracle."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCE_SUFFIXES = (".py", ".hip", ".cpp", ".h", ".c")
SKIP_DIRS = {".git", "_work", "gpurun_out", "__pycache__", ".pytest_cache", ".hypothesis"}


def _sources():
    for base, dirs, files in os.walk(ROOT):
        dirs[:] = [d for d in dirs if d not in SKIP_DIRS]
        for name in files:
            if name.endswith(SOURCE_SUFFIXES) or name == "Makefile":
                path = os.path.join(base, name)
                if os.path.abspath(path) != os.path.abspath(__file__):
                    yield path


def test_sources_name_no_planning_document_tool_or_stage():
    words = ["SUR" + "VEY", "DES" + "IGN.md", "INTEG" + "RATION.md", "BASE" + "LINE.md", "VER" + "DICT", "ADV" + "ICE.md",
             "gpu" + "run", "§"]
    pattern = re.compile("|".join(re.escape(w) for w in words) + r"|\b[Rr]ound[ -]\d")
    hits = []
    for path in _sources():
        for number, line in enumerate(open(path, encoding="utf-8", errors="replace"), 1):
            if pattern.search(line):
                hits.append(f"{os.path.relpath(path, ROOT)}:{number}: {line.strip()[:100]}")
    assert not hits, "\n".join(hits)


def test_only_tests_smoke_and_the_cpu_baseline_import_the_oracle():
    allowed = {"bench.py", "__graft_entry__.py"}
    hits = []
    for path in _sources():
        rel = os.path.relpath(path, ROOT)
        if rel.startswith(("tests" + os.sep, "oracle" + os.sep)) or rel in allowed or not rel.endswith(".py"):
            continue
        text = open(path, encoding="utf-8").read()
        if re.search(r"^\s*(import oracle|from oracle)", text, re.M):
            hits.append(rel)
    assert not hits, hits
    # inside bench.py the oracle is used by the CPU-baseline functions only
    bench = open(os.path.join(ROOT, "bench.py"), encoding="utf-8").read()
    for match in re.finditer(r"^(\s*)import oracle", bench, re.M):
        head = bench[:match.start()]
        owner = re.findall(r"^def (\w+)", head, re.M)[-1]
        assert "cpu_baseline" in owner, owner
