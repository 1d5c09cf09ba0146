"""Host logic of the recording ``update_out_and_lse`` (mercury_artifact_amd/lazy.py) without a GPU.

The two kernel-backed functions the handles end in -- the one-pass fold and the literal merge -- are replaced
by CPU stand-ins built on the oracle, and the generated loop's call pattern (utils/flash_attn_dsl.py:176-179 and
its ``slice_`` sibling) is driven through the handles: what is checked here is the bookkeeping (what gets
recorded, when the fold is taken and when the chain, functional against in-place semantics, error behaviour),
not kernel arithmetic, which the GPU tests cover.
"""
import pytest
import torch

import oracle as O
from mercury_artifact_amd import lazy as L


class _Calls:
    def __init__(self):
        self.fold = 0
        self.chain = 0


@pytest.fixture
def cpu_merges(monkeypatch):
    """merge_many / update_out_and_lse of the merge module, restated on the CPU through the oracle."""
    calls = _Calls()

    def merge_many(block_outs, block_lses, final_out, final_lse, row_begin=None):
        calls.fold += 1
        begins = [0] * len(block_outs) if row_begin is None else list(row_begin)
        out = lse = None
        for bo, bl, sb in zip(block_outs, block_lses, begins):
            sl = None if sb == 0 else (slice(None), slice(sb, None))
            out, lse = O.update_out_and_lse(out, lse, bo.float(), bl.clone(), slice_=sl)
        final_out.copy_(out.to(final_out.dtype))
        final_lse.copy_(lse.squeeze(dim=-1).transpose(1, 2))

    def update_out_and_lse(out, lse, block_out, block_lse, slice_=None):
        calls.chain += 1
        # copies, as the kernel-backed first call makes them: the oracle's accumulators would otherwise be views
        # of the caller's block_lse, and a later in-place slice_ merge would write into it
        return O.update_out_and_lse(out, lse, block_out.float(), block_lse.clone(), slice_=slice_)

    monkeypatch.setattr(L._merge, "merge_many", merge_many)
    monkeypatch.setattr(L._merge, "update_out_and_lse", update_out_and_lse)
    return calls


def _blocks(n, B=2, S=24, H=3, D=64, seed=0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return ([torch.randn(B, S, H, D, generator=g).to(dtype) for _ in range(n)],
            [torch.randn(B, H, S, generator=g) * 3 for _ in range(n)])


def _epilogue(out, lse):
    """The two stores of the generated code (utils/flash_attn_dsl.py:178-179)."""
    return out.to(torch.bfloat16), lse.squeeze(dim=-1).transpose(1, 2)


def _reference(outs, lses, begins=None):
    begins = [0] * len(outs) if begins is None else begins
    out = lse = None
    for bo, bl, sb in zip(outs, lses, begins):
        sl = None if sb == 0 else (slice(None), slice(sb, None))
        out, lse = O.update_out_and_lse(out, lse, bo.float(), bl.clone(), slice_=sl)
    return out, lse


def test_generated_loop_folds_once(cpu_merges):
    outs, lses = _blocks(5)
    out = lse = None
    for bo, bl in zip(outs, lses):
        out, lse = L.update_out_and_lse_lazy(out, lse, bo, bl)
    assert isinstance(out, L.LazyOut) and isinstance(lse, L.LazyLse)
    assert (cpu_merges.fold, cpu_merges.chain) == (0, 0)              # nothing has run yet
    assert out.shape == (2, 24, 3, 64) and lse.shape == (2, 24, 3, 1) and out.dtype == torch.float32
    o, l = _epilogue(out, lse)
    assert (cpu_merges.fold, cpu_merges.chain) == (1, 0)              # ONE fold answers both expressions
    ro, rl = _reference(outs, lses)
    assert torch.equal(o, ro.to(torch.bfloat16))
    assert torch.allclose(l, rl.squeeze(-1).transpose(1, 2))
    assert o.dtype == torch.bfloat16 and l.shape == (2, 3, 24)


def test_functional_calls_leave_earlier_handles_alone(cpu_merges):
    outs, lses = _blocks(3, seed=1)
    o1, l1 = L.update_out_and_lse_lazy(None, None, outs[0], lses[0])
    o2, l2 = L.update_out_and_lse_lazy(o1, l1, outs[1], lses[1])
    o3, l3 = L.update_out_and_lse_lazy(o2, l2, outs[2], lses[2])
    # the pair after two blocks still stands for two blocks
    got2 = _epilogue(o2, l2)
    got3 = _epilogue(o3, l3)
    r2 = _reference(outs[:2], lses[:2])
    r3 = _reference(outs, lses)
    assert torch.equal(got2[0], r2[0].to(torch.bfloat16)) and torch.equal(got3[0], r3[0].to(torch.bfloat16))
    assert cpu_merges.fold == 2 and cpu_merges.chain == 0


def test_slice_updates_in_place_and_enters_the_fold(cpu_merges):
    S = 24
    outs, lses = _blocks(2, S=S, seed=2)
    tail_o, tail_l = _blocks(1, S=S - 8, seed=3)
    out, lse = L.update_out_and_lse_lazy(None, None, outs[0], lses[0])
    out, lse = L.update_out_and_lse_lazy(out, lse, outs[1], lses[1])
    same_o, same_l = L.update_out_and_lse_lazy(out, lse, tail_o[0], tail_l[0], slice_=(slice(None), slice(8, None)))
    assert same_o is out and same_l is lse                       # in place, as the reference's slice_ branch
    o, l = _epilogue(out, lse)
    assert (cpu_merges.fold, cpu_merges.chain) == (1, 0)
    ro, rl = _reference(outs + tail_o, lses + tail_l, [0, 0, 8])
    assert torch.equal(o, ro.to(torch.bfloat16))
    assert torch.allclose(l, rl.squeeze(-1).transpose(1, 2))


def test_anything_else_runs_the_literal_chain(cpu_merges):
    outs, lses = _blocks(3, seed=4)
    out = lse = None
    for bo, bl in zip(outs, lses):
        out, lse = L.update_out_and_lse_lazy(out, lse, bo, bl)
    ro, rl = _reference(outs, lses)
    total = torch.sum(out)                                        # a torch function on a handle
    assert cpu_merges.fold == 0 and cpu_merges.chain == 3
    assert torch.allclose(total, ro.sum(), rtol=1e-5)
    # from here on the handles behave like the accumulators: the epilogue is answered from them, not by a fold
    o, l = _epilogue(out, lse)
    assert cpu_merges.fold == 0
    assert torch.equal(o, ro.to(torch.bfloat16)) and torch.allclose(l, rl.squeeze(-1).transpose(1, 2))
    assert torch.allclose(out[0, 0], ro[0, 0]) and torch.allclose(lse.reshape(-1), rl.reshape(-1))


@pytest.mark.parametrize("what", ["fp32_blocks", "strided_rows", "odd_slice", "float_epilogue"])
def test_cases_the_fold_does_not_take(cpu_merges, what):
    outs, lses = _blocks(2, seed=5, dtype=torch.float32 if what == "fp32_blocks" else torch.bfloat16)
    if what == "strided_rows":
        wide = torch.randn(2, 24, 3, 128).bfloat16()
        outs[1] = wide[..., ::2]                                   # last dimension not contiguous
    out, lse = L.update_out_and_lse_lazy(None, None, outs[0], lses[0])
    if what == "odd_slice":
        out, lse = L.update_out_and_lse_lazy(out, lse, outs[1][:, :10], lses[1][:, :, :10],
                                             slice_=(slice(None), slice(0, 10)))     # rows 0..9: not "from a on"
        ro, rl = _reference([outs[0]], [lses[0]])
        so, sl = O.merge_closed_form(ro[:, :10], rl[:, :10], outs[1][:, :10].float(), lses[1][:, :, :10])
        ro[:, :10], rl[:, :10] = so, sl
    else:
        out, lse = L.update_out_and_lse_lazy(out, lse, outs[1], lses[1])
        ro, rl = _reference(outs, lses)
    o = out.to(torch.float32) if what == "float_epilogue" else out.to(torch.bfloat16)
    l = lse.squeeze(dim=-1).transpose(1, 2)
    assert cpu_merges.fold == 0 and cpu_merges.chain >= 1
    assert torch.allclose(o.float(), ro, atol=1e-2, rtol=1e-2)
    assert torch.allclose(l, rl.squeeze(-1).transpose(1, 2), atol=1e-5)


def test_more_blocks_than_one_fold_takes(cpu_merges, monkeypatch):
    monkeypatch.setattr(L._merge, "MAX_MERGE_MANY", 4)
    outs, lses = _blocks(6, seed=6)
    out = lse = None
    for bo, bl in zip(outs, lses):
        out, lse = L.update_out_and_lse_lazy(out, lse, bo, bl)
    o, l = _epilogue(out, lse)
    ro, rl = _reference(outs, lses)
    assert cpu_merges.fold == 0 and cpu_merges.chain == 6
    assert torch.equal(o, ro.to(torch.bfloat16))


def test_first_call_with_slice_raises_like_the_reference():
    outs, lses = _blocks(1, seed=7)
    with pytest.raises(RuntimeError, match="first update_out_and_lse should not pass slice_ args"):
        L.update_out_and_lse_lazy(None, None, outs[0], lses[0], slice_=(slice(None), slice(0, 4)))


def test_operators_on_handles_act_on_the_real_tensors(cpu_merges):
    """Python looks operators up on the type, not through __getattr__: arithmetic, comparisons, unary, in-place
    operators, len() and torch functions on a handle (and on the squeezed LSE) all give what the literal
    accumulators give."""
    outs, lses = _blocks(3, seed=9)
    h_out, h_lse = None, None
    for bo, bl in zip(outs, lses):
        h_out, h_lse = L.update_out_and_lse_lazy(h_out, h_lse, bo, bl)
    ref_out, ref_lse = _reference(outs, lses)            # fp32 (B,S,H,D), (B,S,H,1)
    assert torch.equal(h_out * 2.0, ref_out * 2.0)
    assert torch.equal(2.0 * h_out, ref_out * 2.0)
    assert torch.equal(-h_out, -ref_out)
    assert torch.equal(h_out / h_out.abs().clamp_min(1.0), ref_out / ref_out.abs().clamp_min(1.0))
    assert torch.equal(h_out - h_out, torch.zeros_like(ref_out))
    assert bool(((h_lse > -1e30) == (ref_lse > -1e30)).all())
    assert len(h_out) == ref_out.shape[0]
    sq = h_lse.squeeze(dim=-1)
    assert torch.equal(torch.transpose(sq, 1, 2), ref_lse.squeeze(-1).transpose(1, 2))      # a torch function on it
    assert torch.equal(sq + 1.0, ref_lse.squeeze(-1) + 1.0)
    assert torch.equal(sq[:, 2:5], ref_lse.squeeze(-1)[:, 2:5])
    # in place: the handle goes on standing for the updated accumulator
    same = h_out
    h_out *= 0.5
    assert h_out is same and torch.equal(h_out.materialize(), ref_out * 0.5)
    assert torch.equal(h_out.to(torch.bfloat16), (ref_out * 0.5).to(torch.bfloat16))
    assert cpu_merges.fold == 0
