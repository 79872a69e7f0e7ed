"""The C header and the binding notes at the repository root name the same surface: every function include/bm_moe.h
declares appears in the notes' extern "C" block with the same number of arguments under the same names, in the same
order, and the block binds nothing the header does not declare. (That the built library exports every declared symbol is
test_capi_cpu.py's part.)"""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NOTES = os.path.join(ROOT, "INTEGRATION.md")


def header_functions():
    src = open(os.path.join(ROOT, "include", "bm_moe.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    src = re.sub(r"^\s*#.*$", "", src, flags=re.M)
    src = re.sub(r"typedef struct \w+ \{.*?\} \w+;", "", src, flags=re.S)
    out = {}
    for name, params in re.findall(r"\b(bm_\w+)\s*\(([^;{}]*?)\)\s*;", src, flags=re.S):
        params = " ".join(params.split())
        names = [] if params in ("", "void") else [re.search(r"(\w+)$", p.strip()).group(1) for p in params.split(",")]
        assert name not in out, f"{name} declared twice"
        out[name] = names
    return out


def bound_functions():
    text = open(NOTES).read()
    block = re.search(r'extern "C" \{(.*?)\n\}', text, flags=re.S).group(1)
    out = {}
    for name, params in re.findall(r"pub fn (bm_\w+)\s*\((.*?)\)\s*(?:->[^;]*)?;", block, flags=re.S):
        params = " ".join(params.split())
        names = [] if not params else [p.split(":")[0].strip() for p in params.split(",")]
        assert name not in out, f"{name} bound twice"
        out[name] = names
    return out


def test_every_declared_function_is_bound_with_the_same_arguments():
    declared, bound = header_functions(), bound_functions()
    assert len(declared) > 60
    assert sorted(set(declared) - set(bound)) == [], "declared in include/bm_moe.h, missing from the binding notes"
    assert sorted(set(bound) - set(declared)) == [], "bound in the notes, not declared in include/bm_moe.h"
    for name, names in declared.items():
        assert bound[name] == names, f"{name}: the header has ({', '.join(names)}), the binding ({', '.join(bound[name])})"


def test_the_build_recipe_names_every_source_of_the_library():
    """The build.rs shown compiles what the Makefile compiles."""
    mk = open(os.path.join(ROOT, "bloomery_amd", "csrc", "Makefile")).read()
    srcs = re.search(r"^SRCS = (.*)$", mk, flags=re.M).group(1).split()
    text = open(NOTES).read()
    recipe = re.search(r"## build\.rs(.*?)## extern", text, flags=re.S).group(1)
    assert len(srcs) >= 7
    for s in srcs:
        assert f'"{s}"' in recipe, f"{s} is built by the Makefile and missing from the build.rs shown"
