"""Merge kernels (through the C ABI) against the CPU oracle.

fp32 elementwise arithmetic: the kernel evaluates the same sigmoid / softplus expressions with
different intrinsics, so the tolerance is a few fp32 ulps of the operands: atol = rtol = 2e-6 on
out and lse (the reference's own tests accept 1e-3)."""
import math

import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu
TOL = dict(atol=2e-6, rtol=2e-6)


def _blocks(B, Sq, H, D, seed=0):
    g = torch.Generator().manual_seed(seed)
    out = torch.randn(B, Sq, H, D, generator=g)
    lse = torch.randn(B, Sq, H, 1, generator=g) * 3 + 5
    bo = torch.randn(B, Sq, H, D, generator=g).bfloat16()
    bl = torch.randn(B, H, Sq, generator=g) * 3 + 5
    return out, lse, bo, bl


@pytest.mark.parametrize("B,Sq,H,D", [(1, 64, 4, 128), (2, 37, 3, 128), (1, 5, 1, 128), (2, 33, 5, 64),
                                      (1, 19, 2, 32), (1, 9, 2, 256), (1, 21, 3, 40)])
def test_update_out_and_lse_matches_reference_formula(B, Sq, H, D):
    import mercury_artifact_amd as M

    print(f"merge case {B} {Sq} {H} {D}", flush=True)
    out, lse, bo, bl = _blocks(B, Sq, H, D)
    ro, rl = O.merge_reference(out, lse, bo, bl)
    od, ld, bod, bld = out.cuda(), lse.cuda(), bo.cuda(), bl.cuda()
    # first call
    fo, fl = M.update_out_and_lse(None, None, bod, bld)
    assert torch.equal(fo.cpu(), bo.float()) and torch.equal(fl.cpu()[..., 0], bl.transpose(1, 2))
    # functional merge leaves its inputs alone
    no, nl = M.update_out_and_lse(od, ld, bod, bld)
    assert torch.equal(od.cpu(), out) and torch.equal(ld.cpu(), lse)
    assert torch.allclose(no.cpu(), ro, **TOL) and torch.allclose(nl.cpu(), rl, **TOL)
    # slice_ path merges in place on a row range
    if Sq >= 4:
        half = Sq // 2
        sl = (slice(None), slice(half, None))
        o2, l2 = od.clone(), ld.clone()
        r2o, r2l = M.update_out_and_lse(o2, l2, bod[:, half:].contiguous(), bld[:, :, half:].contiguous(), slice_=sl)
        assert r2o is o2 and r2l is l2
        eo, el = O.merge_reference(out[sl], lse[sl], bo[:, half:], bl[:, :, half:])
        assert torch.equal(o2.cpu()[:, :half], out[:, :half]) and torch.equal(l2.cpu()[:, :half], lse[:, :half])
        assert torch.allclose(o2.cpu()[sl], eo, **TOL) and torch.allclose(l2.cpu()[sl], el, **TOL)
    with pytest.raises(RuntimeError):
        M.update_out_and_lse(None, None, bod, bld, slice_=(slice(None), slice(0, 1)))


@pytest.mark.parametrize("D", [40, 130, 42])
def test_merge_in_place_generic_head_dim_beyond_residency(D):
    """dst == acc at head dimensions other than 32/64/128/256: multiples of 4 take the vector kernel with idle
    lanes (40), everything else (130, 42) the generic one (one row per 32 lanes of one wavefront: the row's lse
    is read by all its lanes before the one store).  The row count makes the grid far larger than what is
    resident at once, so that rows merged late would see lse values stored early if any thread read an lse it
    does not own."""
    import mercury_artifact_amd as M

    B, Sq, H = 2, 40000, 3
    out, lse, bo, bl = _blocks(B, Sq, H, D, seed=3)
    ro, rl = O.merge_reference(out, lse, bo, bl)
    od, ld = out.cuda(), lse.cuda()
    M.merge_into(od, ld, bo.cuda(), bl.cuda(), od, ld)                     # through mhip_lse_merge, dst = acc
    torch.cuda.synchronize()
    assert torch.allclose(od.cpu(), ro, **TOL) and torch.allclose(ld.cpu(), rl, **TOL)


@pytest.mark.parametrize("D", [128, 24])
def test_tree_merge_in_place(D):
    """mhip_tree_merge with dst == src (both phases) equals the out-of-place result bit for bit."""
    from mercury_artifact_amd import merge as MM

    torch.manual_seed(11)
    rows = 50001
    src = torch.randn(rows, D + 1).cuda()
    src[7, -1] = -math.inf
    row_max = (src[:, -1] + torch.rand(rows).cuda()).contiguous()
    row_max[7] = -math.inf
    for finish in (False, True):
        x = src.abs() if finish else src                                  # finish expects sum_d > 0 in the last column
        sep = torch.empty_like(x)
        MM._tree_merge(x, row_max, sep, finish)
        inplace = x.clone()
        MM._tree_merge(inplace, row_max, inplace, finish)
        torch.cuda.synchronize()
        assert torch.equal(sep.isnan(), inplace.isnan())
        assert torch.equal(sep.nan_to_num(), inplace.nan_to_num())


def test_merge_fused_final_epilogue():
    import mercury_artifact_amd as M

    B, Sq, H, D = 2, 70, 4, 128
    out, lse, bo, bl = _blocks(B, Sq, H, D, seed=1)
    ro, rl = O.merge_reference(out, lse, bo, bl)
    fo = torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
    fl = torch.empty(B, H, Sq, dtype=torch.float32, device="cuda")
    M.merge_into(out.cuda(), lse.cuda(), bo.cuda(), bl.cuda(), None, None, fo, fl)
    assert torch.allclose(fl.cpu(), rl.squeeze(-1).transpose(1, 2), **TOL)
    # the bf16 cast of a value within 2e-6 of the reference differs by at most one bf16 ulp
    assert (fo.float().cpu() - ro.bfloat16().float()).abs().max().item() <= 2 ** -7 * ro.abs().max().item()
    frac_equal = (fo.cpu() == ro.bfloat16()).float().mean().item()
    assert frac_equal > 0.999


def test_merge_infinite_lse_is_identity():
    import mercury_artifact_amd as M

    B, Sq, H, D = 1, 16, 2, 128
    out, lse, bo, bl = _blocks(B, Sq, H, D, seed=2)
    ninf_b = torch.full_like(bl, -math.inf)
    no, nl = M.update_out_and_lse(out.cuda(), lse.cuda(), bo.cuda(), ninf_b.cuda())
    assert torch.equal(no.cpu(), out) and torch.equal(nl.cpu(), lse)
    zo, zl = torch.zeros_like(out), torch.full_like(lse, -math.inf)
    no, nl = M.update_out_and_lse(zo.cuda(), zl.cuda(), bo.cuda(), bl.cuda())
    assert torch.equal(no.cpu(), bo.float()) and torch.equal(nl.cpu()[..., 0], bl.transpose(1, 2))
    no, nl = M.update_out_and_lse(zo.cuda(), zl.cuda(), torch.zeros_like(bo).cuda(), ninf_b.cuda())
    assert no.abs().max().item() == 0 and torch.isinf(nl).all() and not torch.isnan(no).any()


@pytest.mark.parametrize("rows,D", [(64, 128), (37, 128), (3, 128), (50, 64), (7, 5)])
def test_flash_reduce_and_pack(rows, D):
    import mercury_artifact_amd as M

    g = torch.Generator().manual_seed(rows)
    lhs = torch.randn(1, rows, 1, D + 1, generator=g)
    rhs = torch.randn(1, rows, 1, D + 1, generator=g)
    lhs[..., -1] = lhs[..., -1] * 3 + 4
    rhs[..., -1] = rhs[..., -1] * 3 + 4
    ref = O.flash_reduce(lhs, rhs)
    got = M.flash_reduce(lhs.cuda(), rhs.cuda())
    assert got.shape == lhs.shape and torch.allclose(got.cpu(), ref, **TOL)
    # pack, and pack fused with the reduce
    bo = torch.randn(1, rows, 1, D, generator=g).bfloat16()
    bl = torch.randn(1, 1, rows, generator=g) * 3 + 4
    packed = M.pack_block(bo.cuda(), bl.cuda())
    assert torch.equal(packed.cpu(), O.pack_block(bo, bl))
    fused = M.pack_block(bo.cuda(), bl.cuda(), reduce_into=lhs.cuda())
    assert torch.allclose(fused.cpu(), O.flash_reduce(lhs, O.pack_block(bo, bl)), **TOL)


def test_pack_multi_head_layout():
    import mercury_artifact_amd as M

    B, Sq, H, D = 2, 11, 3, 128
    _, _, bo, bl = _blocks(B, Sq, H, D, seed=4)
    assert torch.equal(M.pack_block(bo.cuda(), bl.cuda()).cpu(), O.pack_block(bo, bl))


@pytest.mark.parametrize("n", [4096, 1001, 3, 8, 4096 * 4096 + 13, 4096 * 2048 * 5 + 8])
def test_grad_accumulate(n):
    """Sizes below one group of 8, with a ragged tail, and large enough for the kernel's grid-stride loop to take one
    and two groups per pass; a block that is a view starting off a 16-byte boundary."""
    import mercury_artifact_amd as M

    g = torch.Generator().manual_seed(n % 1000)
    acc = torch.randn(n, generator=g)
    blk = torch.randn(n, generator=g).bfloat16()
    assert torch.equal(M.grad_accumulate(None, blk.cuda()).cpu(), blk.float())
    assert torch.equal(M.grad_accumulate(acc.cuda(), blk.cuda()).cpu(), acc + blk.float())
    if n > 8:
        view = blk.cuda()[3:]
        assert torch.equal(M.grad_accumulate(acc.cuda()[3:], view).cpu(), acc[3:] + blk[3:].float())


@pytest.mark.parametrize("op", ["all_reduce", "reduce"])
def test_tree_merge_collective_matches_oracle(op):
    """update_out_and_lse_collective over a group of four ranks (collectives replayed on the one GPU)
    against the CPU tree merge; one rank is all -inf, one row is -inf on every rank."""
    import math

    import mercury_artifact_amd as M

    torch.manual_seed(8)
    B, Sq, H, D, W = 2, 37, 3, 128, 4
    peers = []
    for r in range(W):
        out = torch.randn(B, Sq, H, D)
        lse = torch.randn(B, Sq, H, 1) * 3
        if r == 2:
            out.zero_()
            lse.fill_(-math.inf)
        lse[0, 5, 1] = -math.inf
        out[0, 5, 1] = 0
        peers.append(torch.cat([out, lse], dim=-1))
    ref = O.tree_merge(peers)
    dev = [p.cuda() for p in peers]
    mine = dev[1].clone()
    if op == "all_reduce":
        M.update_out_and_lse_collective(mine, torch.distributed.all_reduce, M.LocalGroup(dev, rank=1))
    else:
        M.update_out_and_lse_collective(mine, "reduce", M.LocalGroup(dev, rank=1), dst=1)
        other = dev[0].clone()
        M.update_out_and_lse_collective(other, "reduce", M.LocalGroup(dev, rank=0), dst=1)
        assert torch.equal(other, dev[0])                 # not the destination: untouched
    torch.cuda.synchronize()
    got = mine.cpu()
    assert torch.equal(torch.isinf(got[..., -1]), torch.isinf(ref[..., -1]))
    fin = ~torch.isinf(ref[..., -1])
    assert (got[..., :-1] - ref[..., :-1]).abs().max().item() <= 2e-6
    assert (got[..., -1][fin] - ref[..., -1][fin]).abs().max().item() <= 2e-6
    assert (got[0, 5, 1, :-1] == 0).all()
    for p, d in zip(peers, dev):
        assert torch.equal(d.cpu(), p)                    # the other ranks' operands are not modified
    with pytest.raises(RuntimeError):
        M.update_out_and_lse_collective(mine, "reduce_scatter", M.LocalGroup(dev, rank=1))


def test_add_collective_sums_the_group():
    import mercury_artifact_amd as M

    torch.manual_seed(9)
    peers = [torch.randn(2, 16, 4, 128).cuda() for _ in range(3)]
    mine = peers[0].clone()
    M.add_collective(mine, "all_reduce", M.LocalGroup(peers, rank=0))
    assert torch.allclose(mine, peers[0] + peers[1] + peers[2], atol=1e-6)
    with pytest.raises(ValueError):
        M.add_collective(mine, "reduce", M.LocalGroup(peers, rank=0))


@pytest.mark.parametrize("n", [1, 2, 3, 8, 16, 17, 32, 45, 64])
@pytest.mark.parametrize("B,Sq,H,D", [(2, 37, 3, 128), (1, 64, 4, 64), (1, 9, 2, 256), (2, 21, 3, 96), (1, 50, 2, 8)])
def test_merge_many_matches_the_chain(n, B, Sq, H, D):
    """One fold of all block results against the chain of reference merges in fp64 followed by the
    epilogue.  The output is bf16: atol 1e-3 + rtol 2^-8 (one bf16 rounding of the result); lse 1e-5."""
    import mercury_artifact_amd as M

    print(f"merge_many case n={n} {B} {Sq} {H} {D}", flush=True)
    g = torch.Generator().manual_seed(100 + n)
    outs = [torch.randn(B, Sq, H, D, generator=g).bfloat16() for _ in range(n)]
    lses = [torch.randn(B, H, Sq, generator=g) * 3 + 5 for _ in range(n)]
    # rows that are -inf in one block, in all but one, and in every block
    lses[0][0, 0, 0] = -math.inf
    if n == 1:
        outs[0][0, 0, 0] = 0           # a lone block's -inf row carries out = 0, as the block kernel writes it
    for i in range(1, n):
        lses[i][0, 0, 1] = -math.inf
    for i in range(n):
        lses[i][0, 0, 2] = -math.inf
        outs[i][0, 2, 0] = 0
    ro, rl = O.merge_chain(outs, lses)
    fo = torch.full((B, Sq, H, D), 7.0, dtype=torch.bfloat16, device="cuda")
    fl = torch.full((B, H, Sq), 7.0, dtype=torch.float32, device="cuda")
    M.merge_many([t.cuda() for t in outs], [t.cuda() for t in lses], fo, fl)
    fo, fl = fo.float().cpu(), fl.cpu()
    # the all -inf row: the chain NaNs (so does the reference), the kernel gives (0, -inf)
    assert torch.equal(fo[0, 2, 0], torch.zeros(D)) and fl[0, 0, 2].item() == -math.inf
    ro[0, 2, 0], rl[0, 0, 2] = 0, -math.inf
    assert not torch.isnan(fo).any() and not torch.isnan(fl).any()
    assert ((fo - ro.float()).abs() - (1e-3 + 2 ** -8 * ro.float().abs())).max().item() <= 0
    finite = torch.isfinite(rl)
    assert torch.equal(torch.isfinite(fl), finite)
    assert ((fl[finite] - rl[finite].float()).abs() / rl[finite].float().abs().clamp_min(1.0)).max().item() <= 1e-5


def test_merge_many_strided_blocks_and_errors():
    import mercury_artifact_amd as M

    B, Sq, H, D, n = 1, 50, 3, 128, 4
    g = torch.Generator().manual_seed(5)
    big = [torch.randn(B, Sq, 2 * H, D, generator=g).bfloat16().cuda() for _ in range(n)]
    outs = [t[:, :, H:] for t in big]                       # head-sliced views: same strides, offset base
    lses = [(torch.randn(B, H, Sq, generator=g) * 2).cuda() for _ in range(n)]
    ro, rl = O.merge_chain([t.cpu() for t in outs], [t.cpu() for t in lses])
    fo = torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
    fl = torch.empty(B, H, Sq, dtype=torch.float32, device="cuda")
    M.merge_many(outs, lses, fo, fl)
    assert ((fo.float().cpu() - ro.float()).abs() - (1e-3 + 2 ** -8 * ro.float().abs())).max().item() <= 0
    assert torch.allclose(fl.cpu(), rl.float(), atol=1e-5, rtol=1e-5)
    with pytest.raises(RuntimeError):
        M.merge_many(outs * 17, lses * 17, fo, fl)           # 68 blocks: one fold takes at most 64
    with pytest.raises(RuntimeError):
        M.merge_many(outs, lses[:-1], fo, fl)
    with pytest.raises(RuntimeError):
        M.merge_many([outs[0], big[1][:, :, :H].float()], lses[:2], fo, fl)
    with pytest.raises(RuntimeError):
        M.merge_many([t.cpu() for t in outs], lses, fo, fl)


def test_merge_many_with_partial_row_ranges():
    """Blocks that cover only the rows from ``row_begin`` on, as the slice_ merges of a zigzag schedule:
    against the chain with the same slices."""
    import mercury_artifact_amd as M

    B, Sq, H, D = 2, 40, 3, 128
    begins = [0, 20, 0, 20, 33, 40]                    # the last block starts past the end: no rows
    g = torch.Generator().manual_seed(9)
    outs = [torch.randn(B, Sq - sb, H, D, generator=g).bfloat16() for sb in begins]
    lses = [torch.randn(B, H, Sq - sb, generator=g) * 2 + 1 for sb in begins]
    out = lse = None
    for bo, bl, sb in zip(outs, lses, begins):
        sl = None if sb == 0 else (slice(None), slice(sb, None))
        if sb < Sq:
            out, lse = O.update_out_and_lse(out, lse, bo, bl, slice_=sl, acc_dtype=torch.float64)
    ro, rl = out.float(), lse.squeeze(-1).transpose(1, 2).float()
    fo = torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
    fl = torch.empty(B, H, Sq, dtype=torch.float32, device="cuda")
    M.merge_many([t.cuda() for t in outs], [t.cuda() for t in lses], fo, fl, row_begin=begins)
    assert ((fo.float().cpu() - ro).abs() - (1e-3 + 2 ** -8 * ro.abs())).max().item() <= 0
    assert torch.allclose(fl.cpu(), rl, atol=1e-5, rtol=1e-5)
    with pytest.raises(RuntimeError):
        M.merge_many([t.cuda() for t in outs], [t.cuda() for t in lses], fo, fl, row_begin=[0] * 6)


@pytest.mark.parametrize("B,Sq,H,D", [(2, 37, 3, 128), (1, 5, 2, 64), (1, 300, 1, 256)])
def test_unpack_matches_the_literal_epilogue(B, Sq, H, D):
    """buf[..., :-1].to(bf16) and buf[..., -1].transpose(1, 2) in one kernel: bit-exact (a cast and a copy)."""
    import mercury_artifact_amd as M

    g = torch.Generator().manual_seed(B + Sq)
    buf = torch.randn(B, Sq, H, D + 1, generator=g)
    buf[0, 0, 0, -1] = -math.inf
    o = torch.full((B, Sq, H, D), 3.0, dtype=torch.bfloat16, device="cuda")
    lse = torch.full((B, H, Sq), 3.0, dtype=torch.float32, device="cuda")
    M.unpack_into(buf.cuda(), o, lse)
    assert torch.equal(o.cpu(), buf[..., :-1].bfloat16())
    assert torch.equal(lse.cpu(), buf[..., -1].transpose(1, 2))
    with pytest.raises(RuntimeError):
        M.unpack_into(buf.cuda(), o.float(), lse)
