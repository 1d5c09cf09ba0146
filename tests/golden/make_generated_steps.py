"""Writes tests/golden/generated_steps.json: the text Mercury's OWN generator emits for the schedules its tests
and its benchmark build, to be exec-ed unchanged against this package (tests/test_gpu_reference_generated.py).

Why the reference is run here: what the generated text looks like (names it resolves, keyword dict of the block
call, ring protocol, collective line, write-back hop) is the drop-in boundary of this build, and nothing else pins
it -- the reference holds no stored output of its generator.  This script runs in the build container only
(the reference tree is not on the GPU box); it imports `mercury.*` (frontend, IR, PyTorch emitter: pure Python
on ast / numpy / torch) from /root/reference.  The DSL templates are string constants of
utils/flash_attn_dsl.py and utils/attn_bwd_dsl.py; those two modules import flash-attn at their top, which is not
installed, so the strings are taken out of the files' syntax trees instead of importing them.  Nothing else of
the reference is executed, and no kernel of it exists to run.

Each recipe repeats the schedule calls of one place in the reference (cited), on a 4-rank mesh and small sizes:
the generator's output depends on mesh and sizes only through the constants it prints.

Usage:  python tests/golden/make_generated_steps.py       (rewrites the JSON next to it)
"""
import ast
import json
import os
import sys
import textwrap

REFERENCE = "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def template_strings(path):
    """Module-level string constants of a reference file, by name, without importing the file."""
    out = {}
    for node in ast.parse(open(path).read()).body:
        if isinstance(node, ast.Assign) and isinstance(node.value, ast.Constant) and isinstance(node.value.value, str):
            out[node.targets[0].id] = node.value.value
    return out


def collect(lowering=None, backward=True):
    """The recipes as a list of dicts.  ``lowering`` (four callables: eliminate_loops, generate_code, io_buffers,
    buffer_bytes -- the fields of mercury_artifact_amd.search_harness.Lowering) defaults to the reference's own
    functions, called directly; ``backward=False`` leaves out the searched backward programs."""
    if REFERENCE not in sys.path:
        sys.path.insert(0, REFERENCE)
    import mercury.ir.loop_eliminating as le
    import mercury.ir.primitives as sp
    from mercury.backend.pytorch.codegen import generate_pytorch_code
    from mercury.frontend.parser import IRBuilder
    from mercury.ir.distributed import DeviceMesh
    from mercury.ir.init_distributed import init_distributed
    from mercury.ir.nodes import AxisDef, GridLoop
    from mercury.ir.calculate_memory import get_buffer_size
    from mercury.ir.tile import tile_loop
    from mercury.ir.utils import get_io_buffers

    templates = template_strings(os.path.join(REFERENCE, "utils", "flash_attn_dsl.py"))
    templates.update(template_strings(os.path.join(REFERENCE, "utils", "attn_bwd_dsl.py")))

    B, S, H, D = 1, 1024, 4, 128          # global sizes the templates are formatted with
    KVH = 2

    def parse(name, **fmt):
        tree = ast.parse(textwrap.dedent(templates[name].format(**fmt)))
        for node in ast.walk(tree):
            if isinstance(node, ast.FunctionDef):
                return IRBuilder().visit(node)
        raise RuntimeError(name)

    def axes_of(program):
        return program.visit(lambda n: n.axis if isinstance(n, AxisDef) else None)

    def loops_of(program):
        loops = program.visit(lambda n: n if isinstance(n, GridLoop) else None)
        assert len(loops) == 2
        return loops

    def harness_view(program):
        """What the reference's bench_program (mercury/search/bench.py:45-60) takes from a lowered program besides
        its text: one entry per I/O buffer (argument name, per-rank shape, dtype, written or not) and the byte count."""
        buffers = [{"tensor": b.tensor, "shape": [int(d) for d in b.shape], "dtype": str(b.dtype).replace("torch.", ""),
                    "write": bool(b.write)} for b in io_buffers(program)]
        return {"io_buffers": buffers, "buffer_bytes": int(buffer_bytes(program))}

    if lowering is None:
        eliminate, generate = le.eliminate_loops, generate_pytorch_code
        io_buffers, buffer_bytes = (lambda program: program.visit(get_io_buffers)), get_buffer_size
    else:
        eliminate, generate = lowering.eliminate_loops, lowering.generate_code
        io_buffers, buffer_bytes = lowering.io_buffers, lowering.buffer_bytes

    def finish(program):
        eliminate(program)
        return program.name, generate(program), harness_view(program)

    fwd = dict(BATCH=B, SEQ_LEN=S, HEADS=H, HEAD_DIM=D)
    red = dict(fwd, RED_DIM=D + 1)
    recipes = []

    def recipe(name, source, mesh_shape, q_dims, kv_dims, heads_q=H, heads_kv=H):
        def deco(fn):
            program_name, code, view = fn()
            recipes.append({"name": name, "source": source, "mesh": list(mesh_shape), "function": program_name,
                            "q_dims": list(q_dims), "kv_dims": list(kv_dims), "B": B, "S": S, "Hq": heads_q,
                            "Hkv": heads_kv, "D": D, "code": code, **view})
            return fn
        return deco

    # ---- single ring with ring_divide (benchmark/bench_attn.py:115-163) -------------------------------------
    for divide in (1, 2, 4):
        @recipe(f"single_ring_divide_{divide}", "benchmark/bench_attn.py:115-163", (4,), (0,), (0,))
        def _(divide=divide):
            program = parse("flash_attn_pack_kv_template", **fwd)
            s_q = axes_of(program)[2]
            outer = next(l for l in loops_of(program) if len(l.axes) == 3)
            mesh = DeviceMesh(list(range(4)), (4,))
            init_distributed(program, mesh)
            sp.parallelize(program, outer, s_q, mesh, 0, 1)
            sp.shift(program, s_q, mesh, 0, 1, divide)
            return finish(program)

    # ---- double ring (tests/test_double_ring.py:26-84) -----------------------------------------------------------
    @recipe("double_ring_2x2", "tests/test_double_ring.py:26-84", (2, 2), (0, 1), (0, 1))
    def _():
        program = parse("flash_attn_pack_kv_double_ring_template", SEQ_LEN_IN=S // 2, SEQ_LEN_OUT=2, **fwd)
        mesh = DeviceMesh(list(range(4)), (2, 2))
        init_distributed(program, mesh)
        s_q = axes_of(program)[2]
        outer = next(l for l in loops_of(program) if len(l.axes) == 3)
        sp.parallelize(program, outer, s_q, mesh, 0, 2)
        sp.shift(program, s_q, mesh, 0, 2, 1)
        return finish(program)

    # ---- grouped K/V heads (tests/test_gqa.py:27-98) ---------------------------------------------------------------
    @recipe("gqa_single_ring", "tests/test_gqa.py:27-98", (4,), (0,), (0,), heads_q=H, heads_kv=KVH)
    def _():
        program = parse("gqa_pack_kv_template", KV_HEADS=KVH, HEADS_PER_GROUP=H // KVH, **fwd)
        mesh = DeviceMesh(list(range(4)), (4,))
        init_distributed(program, mesh)
        s_q = axes_of(program)[2]
        outer = next(l for l in loops_of(program) if len(l.axes) == 3)
        sp.parallelize(program, outer, s_q, mesh, 0, 1)
        sp.shift(program, s_q, mesh, 0, 1, 1)
        return finish(program)

    # ---- managed reduction: K/V sharded and not ringed -> the collective (tests/test_reduce.py:26-91) ------------
    @recipe("tree_attention", "tests/test_reduce.py:26-91", (4,), (), (0,))
    def _():
        program = parse("flash_attn_manage_reduction", **red)
        mesh = DeviceMesh(list(range(4)), (4,))
        init_distributed(program, mesh)
        s_kv = axes_of(program)[3]
        inner = loops_of(program)[1]
        sp.parallelize(program, inner, s_kv, mesh, 0, 1)
        return finish(program)

    # ---- managed reduction with a ring on its own axis (tests/test_reduce.py:93-159) ---------------------------------
    @recipe("reduce_ring", "tests/test_reduce.py:93-159", (4,), (0,), (0,))
    def _():
        program = parse("flash_attn_manage_reduction", **red)
        mesh = DeviceMesh(list(range(4)), (4,))
        init_distributed(program, mesh)
        s_kv = axes_of(program)[3]
        inner = loops_of(program)[1]
        sp.parallelize(program, inner, s_kv, mesh, 0, 1)
        sp.shift(program, s_kv, mesh, 0, 1, 1)
        return finish(program)

    # ---- K/V as a tree on mesh dimension 0, Q parallel on dimension 1 (tests/test_reduce.py:161-228) -----------------
    @recipe("tree_kv_parallel_q", "tests/test_reduce.py:161-228", (2, 2), (1,), (0,))
    def _():
        program = parse("flash_attn_manage_reduction", **red)
        mesh = DeviceMesh(list(range(4)), (2, 2))
        init_distributed(program, mesh)
        axes = axes_of(program)
        outer = next(l for l in loops_of(program) if len(l.axes) == 3)
        inner = loops_of(program)[1]
        sp.parallelize(program, inner, axes[3], mesh, 0, 1)
        sp.parallelize(program, outer, axes[2], mesh, 1, 2)
        return finish(program)

    # ---- managed reduction under a double ring of K/V on a 2-D mesh (tests/test_split.py:93-156) --------------------------------
    @recipe("managed_reduction_double_kv_ring_2x2", "tests/test_split.py:93-156", (2, 2), (0, 1), (0, 1))
    def _():
        program = parse("flash_attn_manage_reduction", **red)
        axes = axes_of(program)
        tile_loop(program, axes[3], S // 2)
        mesh = DeviceMesh(list(range(4)), (2, 2))
        init_distributed(program, mesh)
        outer = next(l for l in loops_of(program) if len(l.axes) == 3)
        sp.parallelize(program, outer, axes[2], mesh, 0, 2)
        sp.shift(program, axes[2], mesh, 0, 2, 1)
        return finish(program)

    # ---- the reduce buffer's own double ring (tests/test_split.py:26-91) -----------------------------------------------
    @recipe("double_reduce_ring_2x2", "tests/test_split.py:26-91", (2, 2), (0, 1), (0, 1))
    def _():
        program = parse("flash_attn_manage_reduction", **red)
        tile_loop(program, axes_of(program)[2], S // 2)
        mesh = DeviceMesh(list(range(4)), (2, 2))
        init_distributed(program, mesh)
        s_kv = axes_of(program)[4]
        inner = loops_of(program)[1]
        sp.parallelize(program, inner, s_kv, mesh, 0, 2)
        sp.shift(program, s_kv, mesh, 0, 2, 1)
        return finish(program)

    # ---- ring on the inner Q axis, tree on the outer K/V axis (tests/test_split.py:158-236) -----------------------------
    @recipe("tree_over_ring_2x2", "tests/test_split.py:158-236", (2, 2), (0,), (0, 1))
    def _():
        program = parse("flash_attn_manage_reduction", **red)
        tile_loop(program, axes_of(program)[3], S // 2)
        tile_loop(program, axes_of(program)[2], S // 2)
        mesh = DeviceMesh(list(range(4)), (2, 2))
        init_distributed(program, mesh)
        axes = axes_of(program)
        loops = loops_of(program)
        sp.parallelize(program, loops[0], axes[3], mesh, 0, 1)
        sp.shift(program, axes[3], mesh, 0, 1, 1)
        sp.parallelize(program, loops[1], axes[4], mesh, 1, 2)
        return finish(program)

    # ---- backward: the schedules the reference's search finds on a 1-D mesh (tests/test_attn_bwd.py:53-130 runs
    # every searched program); one of each kind, with all heads on every rank -----------------------------------------
    if not backward:
        return recipes
    import re

    from mercury.search.search import search

    program = parse("attn_backward_template", **fwd)
    found = {}
    for candidate in search(program, DeviceMesh(list(range(4)), (4,)), ["S_q", "S_kv"]):
        eliminate(candidate)
        found.setdefault(generate(candidate), harness_view(candidate))
    # The search also tiles the two sequence loops into sub-chunks.  Taken here: per kind the untiled program, and
    # the one whose K/V loop alone is tiled.  Left out: programs with a tiled QUERY loop around a travelling dK/dV
    # buffer -- their text restarts the buffer at every query tile (`reduce_dkv[...] = block_dkv...` at ring step
    # 0), so dK/dV keeps the last tile's share only; that is a property of the emitted text, not of the kernels
    # under it, and no test of the reference fixes what it should give.
    kinds = {}
    for code in sorted(found, key=lambda c: (len(c.splitlines()), c)):
        if "one_dim_to_n_dim(dist.get_rank(), (4,))" not in code or "S_q_outer" in code:
            continue
        shapes = dict(re.findall(r"assert (\w+)\.shape == (\([^)]*\))", code))
        if eval(shapes["q"])[2] != H:
            continue
        nq, nkv = S // eval(shapes["q"])[1], S // eval(shapes["kv"])[2]
        if "ring_comm_reduce_dq" in code:
            kind = "backward_q_ring"
        elif "ring_comm_reduce_dkv" in code:
            kind = "backward_kv_ring"
        elif "add_collective" in code and nq == 1:
            kind = "backward_kv_sharded_collective"
        elif "add_collective" in code and nkv == 1:
            kind = "backward_q_sharded_collective"
        else:
            continue
        if "S_kv_outer" in code:
            kind += "_kv_tiled"
        kinds.setdefault(kind, (code, nq, nkv))
    for kind, (code, nq, nkv) in sorted(kinds.items()):
        recipes.append({"name": kind, "source": "tests/test_attn_bwd.py:53-130 (mercury.search.search on a 4-rank mesh)",
                        "mesh": [4], "function": program.name, "q_dims": [0] if nq == 4 else [],
                        "kv_dims": [0] if nkv == 4 else [], "B": B, "S": S, "Hq": H, "Hkv": H, "D": D, "code": code,
                        **found[code]})

    return recipes


def main():
    recipes = collect()
    out = os.path.join(HERE, "generated_steps.json")
    with open(out, "w") as fh:
        json.dump({"made_by": "tests/golden/make_generated_steps.py", "recipes": recipes}, fh, indent=1)
    print(f"{len(recipes)} generated step functions -> {out}")
    for r in recipes:
        print(f"  {r['name']:32s} {r['function']:36s} {len(r['code'].splitlines()):4d} lines")


if __name__ == "__main__":
    main()
