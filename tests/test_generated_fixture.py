"""CPU checks of tests/golden/generated_steps.json (the reference generator's own output, see
tests/golden/make_generated_steps.py): each text compiles, and every name it reads is either bound by the text itself,
a builtin, or a name the exec dict of this package provides -- so a missing operator shows up here, without a GPU."""
import ast
import builtins
import json
import os

import pytest

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "generated_steps.json")) as _fh:
    RECIPES = json.load(_fh)["recipes"]


@pytest.mark.parametrize("recipe", RECIPES, ids=[r["name"] for r in RECIPES])
def test_generated_text_resolves_every_name_in_the_exec_dict(recipe):
    import mercury_artifact_amd as M

    tree = ast.parse(recipe["code"])
    compile(tree, recipe["name"], "exec")
    funcs = [n for n in tree.body if isinstance(n, ast.FunctionDef)]
    assert [f.name for f in funcs] == [recipe["function"]]
    bound = {a.arg for a in funcs[0].args.args}
    read = set()
    for node in ast.walk(funcs[0]):
        if isinstance(node, ast.Name):
            (bound if isinstance(node.ctx, (ast.Store, ast.Del)) else read).add(node.id)
    provided = set(M.namespace()) | set(M.namespace(lazy_merge=False)) | {"torch", "os", "dist", "SendRecv"}
    missing = {n for n in read - bound if not hasattr(builtins, n)} - provided
    assert not missing, missing


def test_fixture_names_the_reference_place_each_recipe_repeats():
    for r in RECIPES:
        assert ":" in r["source"] and r["source"].split(":")[0].endswith(".py"), r["name"]
        assert len(r["mesh"]) in (1, 2) and all(d < len(r["mesh"]) for d in r["q_dims"] + r["kv_dims"])


def test_harness_view_of_every_recipe_matches_its_text():
    """The I/O buffer table the reference's bench_program allocates from (mercury/search/bench.py:45-60) names exactly
    the tensor arguments of the generated function, with the shapes the text asserts."""
    import re

    for r in RECIPES:
        func = next(n for n in ast.parse(r["code"]).body if isinstance(n, ast.FunctionDef))
        tensors = [a.arg for a in func.args.args][: len(r["io_buffers"])]
        assert sorted(b["tensor"] for b in r["io_buffers"]) == sorted(tensors), r["name"]
        asserted = {name: list(ast.literal_eval(shape))
                    for name, shape in re.findall(r"assert (\w+)\.shape == (\([^)]*\))", r["code"])}
        for b in r["io_buffers"]:
            assert asserted[b["tensor"]] == b["shape"], (r["name"], b["tensor"])
            assert b["dtype"] == ("float32" if b["tensor"] == "lse" else "bfloat16")
        written = {b["tensor"] for b in r["io_buffers"] if b["write"]}
        assert written == ({"dq", "dkv"} if r["name"].startswith("backward") else {"o", "lse"}), r["name"]


@pytest.mark.skipif(not os.path.isdir("/root/reference/mercury"), reason="needs the reference tree (build container only)")
def test_mercury_lowering_runs_the_reference_generator_and_reproduces_the_fixture():
    """search_harness.mercury_lowering() for real: the four callables it imports from the reference, driven over the
    forward recipes of the fixture's generator, give the committed texts, buffer tables and byte counts."""
    import importlib.util
    import sys

    from mercury_artifact_amd import search_harness as SH

    spec = importlib.util.spec_from_file_location(
        "make_generated_steps", os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "make_generated_steps.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    sys.path.insert(0, gen.REFERENCE)
    try:
        made = gen.collect(lowering=SH.mercury_lowering(), backward=False)
    finally:
        sys.path.remove(gen.REFERENCE)
    stored = {r["name"]: r for r in RECIPES}
    assert len(made) == 11
    for r in made:
        assert r == stored[r["name"]], r["name"]
