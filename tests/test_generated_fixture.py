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
