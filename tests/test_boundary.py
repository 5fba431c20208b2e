"""Who may import whom inside the package. The layers' parts know nothing of the cache or the
engine; a model knows parts and its configuration; the cache knows the parts' declarations only;
and of the engine, only `engine/interface.py` and the scheduler reach into `cache/` (the step
function, the loop and trace replay go through the interface). The reference keeps the same line
with tests/test_boundary.py:35-44 over its engine and model folders; here every folder has a row."""

from __future__ import annotations

import ast
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
PACKAGE = "tinyserve_llm_amd"

# folder -> the folders of the package it may import from (its own included)
MAY_IMPORT = {
    "config": {"config"},
    "csrc": {"csrc"},
    "ops": {"ops", "csrc"},
    "parts": {"parts", "ops"},
    "sampling": {"sampling", "ops"},
    "models": {"models", "parts", "config", "ops"},
    "weights": {"weights", "models", "parts"},
    "cache": {"cache", "parts", "ops"},
    "engine": {"engine", "models", "parts", "weights", "sampling", "ops", "cache", "config"},
}
CACHE_GATES = {"engine/interface.py", "engine/scheduler.py"}      # the engine modules that may name `cache/`


def imports_of(source: str) -> list[str]:
    """Every module of this package that `source` imports, as dotted names, wherever the import stands."""
    found = []
    for node in ast.walk(ast.parse(source)):
        if isinstance(node, ast.Import):
            names = [alias.name for alias in node.names]
        elif isinstance(node, ast.ImportFrom) and node.level == 0 and node.module:
            names = [node.module] if node.module != PACKAGE else [f"{PACKAGE}.{alias.name}" for alias in node.names]
        elif isinstance(node, ast.ImportFrom) and node.level:
            raise AssertionError("relative imports hide the layering; the package spells its imports out")
        else:
            continue
        found += [n for n in names if n == PACKAGE or n.startswith(PACKAGE + ".")]
    return found


def folder_of(module: str) -> str | None:
    parts = module.split(".")
    return parts[1] if len(parts) > 1 and parts[1] in MAY_IMPORT else None


def test_the_walker_sees_every_form_of_import():
    src = (f"import {PACKAGE}.cache.manager\nfrom {PACKAGE}.ops import hip\nfrom {PACKAGE} import models\nimport torch\n"
           f"def f():\n    from {PACKAGE}.engine.llm import LLM\n")
    assert imports_of(src) == [f"{PACKAGE}.cache.manager", f"{PACKAGE}.ops", f"{PACKAGE}.models", f"{PACKAGE}.engine.llm"]


def test_every_folder_imports_only_what_its_row_allows():
    violations = []
    seen = set()
    for path in sorted((ROOT / PACKAGE).rglob("*.py")):
        rel = path.relative_to(ROOT / PACKAGE)
        if len(rel.parts) < 2:
            continue                       # the package's own __init__ and its command line sit above the layers
        folder = rel.parts[0]
        seen.add(folder)
        assert folder in MAY_IMPORT, f"{folder}/ has no row in the table of this test"
        for module in imports_of(path.read_text()):
            target = folder_of(module)
            if target is not None and target not in MAY_IMPORT[folder]:
                violations.append(f"{rel}: {module}")
    assert not violations, violations
    assert seen == set(MAY_IMPORT)


def test_only_the_interface_and_the_scheduler_reach_into_the_cache():
    reaching = {str(p.relative_to(ROOT / PACKAGE)) for p in (ROOT / PACKAGE / "engine").glob("*.py")
                if any(folder_of(m) == "cache" for m in imports_of(p.read_text()))}
    assert reaching == CACHE_GATES
    for path in list((ROOT / PACKAGE / "cache").glob("*.py")):
        for module in imports_of(path.read_text()):
            if folder_of(module) == "parts":
                assert module == f"{PACKAGE}.parts.base", f"{path.name} needs the parts' declarations only, not {module}"
    for top in ("bench.py", f"{PACKAGE}/generate.py", "bin/trace_run"):
        assert not any(folder_of(m) == "cache" for m in imports_of((ROOT / top).read_text())), top
