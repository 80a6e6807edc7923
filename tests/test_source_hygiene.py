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


def test_counter_summaries_are_of_the_kernels_as_they_are_now():
    """The traffic ratio bench.py reports comes from committed counter summaries; each names the
    kernel it was taken with and the digest of the kernel source it was built from.  A change
    to the kernels without new counter runs fails here (and makes bench.py report no traffic)."""
    import importlib.util
    import re

    spec = importlib.util.spec_from_file_location("bench_for_digest", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    now = bench.kernel_source_digest()
    assert re.fullmatch(r"[0-9a-f]{16}", now)
    for config in (2, 3, 4):
        path = os.path.join(ROOT, "profiles", f"kvm_copy_kernel_cfg{config}_pmc.txt")
        text = open(path).read()
        of_record = re.search(r"^KERNEL_OF_RECORD (.+)$", text, flags=re.M)
        digest = re.search(r"^KERNEL_SOURCE_DIGEST ([0-9a-f]+)$", text, flags=re.M)
        assert of_record and digest, path
        assert digest.group(1) == now, f"{path} was taken with other kernel source: take the counters again"
        traffic, source = bench.measured_traffic(config, of_record.group(1).strip(), 1e9)
        assert traffic is not None and 0.99e9 < traffic < 1.05e9 and "profiles/" in source
        # another kernel's name is refused
        assert bench.measured_traffic(config, "some_other_kernel", 1e9)[0] is None
