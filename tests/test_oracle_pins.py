"""Pins for the CPU oracle: each oracle function is checked against something that is NOT a
retyping of its own formula -- brute-force loops, torch library routines, closed forms and
invariants, a message-passing simulation.  The reference holds no golden vector for this path
(its tests compare two flash-attn CUDA results on unseeded data)."""
import itertools
import math

import pytest
import torch

import oracle as O

torch.manual_seed(0)


def _rand(*shape, dtype=torch.float64):
    return torch.randn(*shape, dtype=dtype)


# ----------------------------------------------------------------------------- block forward
def _brute_block(q, k, v, scale, causal):
    """Scalar loops, exponentials by math.exp: shares no code with the oracle."""
    B, Sq, Hq, D = q.shape
    _, Sc, Hkv, _ = k.shape
    out = torch.zeros(B, Sq, Hq, D, dtype=torch.float64)
    lse = torch.full((B, Hq, Sq), -math.inf, dtype=torch.float64)
    for b, h, i in itertools.product(range(B), range(Hq), range(Sq)):
        g = h // (Hq // Hkv)
        scores = []
        for j in range(Sc):
            if causal and j > i + (Sc - Sq):
                continue
            scores.append((j, scale * sum(float(q[b, i, h, d]) * float(k[b, j, g, d]) for d in range(D))))
        if not scores:
            continue
        m = max(s for _, s in scores)
        z = sum(math.exp(s - m) for _, s in scores)
        lse[b, h, i] = m + math.log(z)
        for j, s in scores:
            w = math.exp(s - m) / z
            for d in range(D):
                out[b, i, h, d] += w * float(v[b, j, g, d])
    return out, lse


@pytest.mark.parametrize("Sq,Sc,Hq,Hkv,causal", [
    (3, 5, 2, 2, False), (5, 3, 4, 2, False), (4, 4, 2, 1, True), (3, 6, 2, 2, True), (6, 3, 2, 2, True),
])
def test_block_attention_vs_brute_force(Sq, Sc, Hq, Hkv, causal):
    q, k, v = _rand(2, Sq, Hq, 4), _rand(2, Sc, Hkv, 4), _rand(2, Sc, Hkv, 4)
    out, lse = O.block_attention(q, k, v, 0.37, causal=causal, dtype=torch.float64)
    bo, bl = _brute_block(q, k, v, 0.37, causal)
    assert torch.allclose(out, bo, atol=1e-12)
    assert torch.equal(torch.isinf(lse), torch.isinf(bl))
    fin = ~torch.isinf(bl)
    assert torch.allclose(lse[fin], bl[fin], atol=1e-12)


@pytest.mark.parametrize("causal", [False, True])
def test_block_attention_vs_torch_sdpa(causal):
    """torch's own CPU attention is an independent library implementation."""
    B, S, Hq, Hkv, D = 2, 64, 8, 2, 32
    q, k, v = _rand(B, S, Hq, D), _rand(B, S, Hkv, D), _rand(B, S, Hkv, D)
    scale = D ** -0.5
    out, lse = O.block_attention(q, k, v, scale, causal=causal, dtype=torch.float64)
    kr = k.repeat_interleave(Hq // Hkv, dim=2)
    vr = v.repeat_interleave(Hq // Hkv, dim=2)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2), kr.transpose(1, 2), vr.transpose(1, 2), is_causal=causal, scale=scale)
    assert torch.allclose(out, ref.transpose(1, 2), atol=1e-10)
    s = torch.einsum("bihd,bjhd->bhij", q, kr) * scale
    if causal:
        s = s.masked_fill(torch.ones(S, S, dtype=torch.bool).triu(1), -math.inf)
    assert torch.allclose(lse, torch.logsumexp(s, -1), atol=1e-10)


def test_block_attention_empty_and_masked_rows():
    q, k, v = _rand(1, 4, 2, 8), _rand(1, 0, 2, 8), _rand(1, 0, 2, 8)
    out, lse = O.block_attention(q, k, v, 1.0)
    assert out.abs().max() == 0 and torch.isinf(lse).all() and (lse < 0).all()
    # Sq > Sc causal: the first Sq-Sc rows see no key at all
    q, k, v = _rand(1, 6, 1, 8), _rand(1, 2, 1, 8), _rand(1, 2, 1, 8)
    out, lse = O.block_attention(q, k, v, 1.0, causal=True)
    assert torch.isinf(lse[0, 0, :4]).all() and torch.isfinite(lse[0, 0, 4:]).all()
    assert out[0, :4].abs().max() == 0


# ----------------------------------------------------------------------------- merge
def _two_blocks(B=2, Sq=16, H=3, D=8, dtype=torch.float64):
    out = _rand(B, Sq, H, D, dtype=dtype)
    lse = _rand(B, Sq, H, 1, dtype=dtype) * 3
    bo = _rand(B, Sq, H, D, dtype=dtype)
    bl = _rand(B, H, Sq, dtype=dtype) * 3
    return out, lse, bo, bl


def test_merge_reference_equals_closed_form():
    """sigmoid/logsigmoid form (utils/flash_attn_dsl.py:46-47) == logaddexp form (its comment)."""
    out, lse, bo, bl = _two_blocks()
    a = O.merge_reference(out, lse, bo, bl)
    b = O.merge_closed_form(out, lse, bo, bl)
    assert torch.allclose(a[0], b[0], atol=1e-12) and torch.allclose(a[1], b[1], atol=1e-12)
    # and the textbook weights, written a third way
    blt = bl.transpose(-2, -1).unsqueeze(-1)
    w = torch.softmax(torch.cat([lse, blt], -1), -1)
    assert torch.allclose(a[0], w[..., :1] * out + w[..., 1:] * bo, atol=1e-12)
    assert torch.allclose(a[1], torch.logsumexp(torch.cat([lse, blt], -1), -1, keepdim=True), atol=1e-12)


def test_merge_commutative_associative_identity():
    out, lse, bo, bl = _two_blocks()
    lse_t = lse.squeeze(-1).transpose(1, 2)           # (B,H,Sq) form of the accumulator's lse
    blt = bl.transpose(-2, -1).unsqueeze(-1)
    ab = O.merge_closed_form(out, lse, bo, bl)
    ba = O.merge_closed_form(bo, blt, out, lse_t)
    assert torch.allclose(ab[0], ba[0], atol=1e-12) and torch.allclose(ab[1], ba[1], atol=1e-12)
    co, cl = _rand(*bo.shape), _rand(*bl.shape)
    left = O.merge_closed_form(*ab, co, cl)
    bc = O.merge_closed_form(bo, blt, co, cl)
    right = O.merge_closed_form(out, lse, bc[0], bc[1].squeeze(-1).transpose(1, 2))
    assert torch.allclose(left[0], right[0], atol=1e-12) and torch.allclose(left[1], right[1], atol=1e-12)
    # -inf block is the identity; -inf accumulator takes the block; both -inf stay (0, -inf)
    ninf = torch.full_like(bl, -math.inf)
    i = O.merge_closed_form(out, lse, bo, ninf)
    assert torch.equal(i[0], out) and torch.equal(i[1], lse)
    t = O.merge_closed_form(torch.zeros_like(out), torch.full_like(lse, -math.inf), bo, bl)
    assert torch.allclose(t[0], bo) and torch.allclose(t[1], blt)
    z = O.merge_closed_form(torch.zeros_like(out), torch.full_like(lse, -math.inf), torch.zeros_like(bo), ninf)
    assert z[0].abs().max() == 0 and torch.isinf(z[1]).all()


def test_flash_reduce_matches_update_on_packed():
    out, lse, bo, bl = _two_blocks(dtype=torch.float32)
    lhs = torch.cat([out, lse], -1)
    rhs = O.pack_block(bo, bl)
    assert rhs.shape[-1] == out.shape[-1] + 1
    red = O.flash_reduce(lhs, rhs)
    mo, ml = O.merge_reference(out, lse, bo, bl)
    assert torch.allclose(red[..., :-1], mo, atol=1e-6) and torch.allclose(red[..., -1:], ml, atol=1e-6)


def test_config0_chunks_merge_to_single_pass():
    """The CPU plumbing configuration: fp32, B1 H4 D64, Q 1024, K/V 1024 in 4 chunks of 256, seed 0."""
    torch.manual_seed(0)
    q, k, v = (torch.randn(1, 1024, 4, 64) for _ in range(3))
    scale = 64 ** -0.5
    chunks = [torch.stack([k[:, c * 256:(c + 1) * 256], v[:, c * 256:(c + 1) * 256]]) for c in range(4)]
    ref_o, ref_l = O.single_pass_attention(q, k, v, scale)
    for rank in range(4):
        for merge in (O.merge_reference, O.merge_closed_form):
            o, l = O.ring_forward(q, chunks, O.single_ring_order(rank, 4), scale, merge=merge)
            assert torch.allclose(o, ref_o, atol=2e-6) and torch.allclose(l, ref_l, atol=2e-6)
    o, l = O.ring_forward_packed(q, chunks, O.single_ring_order(1, 4), scale)
    assert torch.allclose(o, ref_o, atol=2e-6) and torch.allclose(l, ref_l, atol=2e-6)


def test_update_out_and_lse_dispatch():
    out, lse, bo, bl = _two_blocks(dtype=torch.float32)
    with pytest.raises(RuntimeError):
        O.update_out_and_lse(None, None, bo, bl, slice_=(slice(None), slice(0, 4)))
    o0, l0 = O.update_out_and_lse(None, None, bo.bfloat16(), bl)
    assert o0.dtype == torch.float32 and l0.shape == lse.shape
    assert torch.equal(o0, bo.bfloat16().float()) and torch.equal(l0[..., 0], bl.transpose(1, 2))
    sl = (slice(None), slice(8, None))
    o1, l1 = out.clone(), lse.clone()
    O.update_out_and_lse(o1, l1, bo[:, 8:], bl[:, :, 8:], slice_=sl)
    assert torch.equal(o1[:, :8], out[:, :8]) and torch.equal(l1[:, :8], lse[:, :8])
    eo, el = O.merge_closed_form(out[sl], lse[sl], bo[:, 8:], bl[:, :, 8:])
    assert torch.equal(o1[sl], eo) and torch.equal(l1[sl], el)


# ----------------------------------------------------------------------------- backward
@pytest.mark.parametrize("Hq,Hkv", [(2, 2), (4, 2)])
def test_block_backward_vs_autograd(Hq, Hkv):
    """Sum over chunks of block gradients taken with the GLOBAL lse/out == autograd of single-pass
    attention; each chunk's dk/dv is the matching slice of the full dk/dv."""
    B, Sq, S, D, W = 2, 12, 32, 8, 4
    q = _rand(B, Sq, Hq, D).requires_grad_()
    k = _rand(B, S, Hkv, D).requires_grad_()
    v = _rand(B, S, Hkv, D).requires_grad_()
    scale = 0.41
    kr, vr = (t.repeat_interleave(Hq // Hkv, dim=2) for t in (k, v))
    p = torch.softmax(torch.einsum("bihd,bjhd->bhij", q, kr) * scale, -1)
    out = torch.einsum("bhij,bjhd->bihd", p, vr)
    dout = _rand(*out.shape)
    gq, gk, gv = torch.autograd.grad(out, (q, k, v), dout)
    with torch.no_grad():
        o, lse = O.single_pass_attention(q, k, v, scale, dtype=torch.float64)
        assert torch.allclose(o, out, atol=1e-12)
        Sc = S // W
        chunks = [torch.stack([k[:, c * Sc:(c + 1) * Sc], v[:, c * Sc:(c + 1) * Sc]]) for c in range(W)]
        dq, dkv = O.ring_backward(q, chunks, O.single_ring_order(2, W), o, lse, dout, scale, dtype=torch.float64)
        assert torch.allclose(dq, gq, atol=1e-11)
        for c in range(W):
            assert torch.allclose(dkv[c][0], gk[:, c * Sc:(c + 1) * Sc], atol=1e-11)
            assert torch.allclose(dkv[c][1], gv[:, c * Sc:(c + 1) * Sc], atol=1e-11)


def test_block_backward_causal_vs_autograd():
    B, S, H, D = 1, 10, 2, 4
    q, k, v = (_rand(B, S, H, D).requires_grad_() for _ in range(3))
    s = torch.einsum("bihd,bjhd->bhij", q, k) * 0.5
    s = s.masked_fill(torch.ones(S, S, dtype=torch.bool).triu(1), -math.inf)
    out = torch.einsum("bhij,bjhd->bihd", torch.softmax(s, -1), v)
    dout = _rand(*out.shape)
    gq, gk, gv = torch.autograd.grad(out, (q, k, v), dout)
    with torch.no_grad():
        o, lse = O.block_attention(q, k, v, 0.5, causal=True, dtype=torch.float64)
        dq, dk, dv = O.block_backward(dout, q, k, v, o, lse, 0.5, causal=True, dtype=torch.float64)
    for a, b in ((dq, gq), (dk, gk), (dv, gv)):
        assert torch.allclose(a, b, atol=1e-11)


# ----------------------------------------------------------------------------- schedules
def _simulate_single(world):
    held = list(range(world))
    seen = [[] for _ in range(world)]
    for _ in range(world):
        for r in range(world):
            seen[r].append(held[r])
        held = [held[(r - 1) % world] for r in range(world)]      # everyone sends to r+1
    return seen


def _simulate_double(inner, outer):
    world = inner * outer
    held = list(range(world))
    seen = [[] for _ in range(world)]
    for o in range(outer):
        for i in range(inner):
            for r in range(world):
                seen[r].append(held[r])
            nxt = list(held)
            if i + 1 != inner:        # hop along mesh dim 0 (fastest digit)
                for r in range(world):
                    a, b = r % inner, r // inner
                    nxt[b * inner + (a + 1) % inner] = held[r]
            elif o + 1 != outer:      # hop along mesh dim 1
                for r in range(world):
                    a, b = r % inner, r // inner
                    nxt[((b + 1) % outer) * inner + a] = held[r]
            held = nxt
    return seen


@pytest.mark.parametrize("world", [1, 2, 4, 8])
def test_single_ring_order_vs_simulation(world):
    seen = _simulate_single(world)
    for r in range(world):
        assert O.single_ring_order(r, world) == seen[r]
        assert sorted(seen[r]) == list(range(world))


@pytest.mark.parametrize("inner,outer", [(4, 2), (2, 2), (2, 4), (1, 4), (4, 1)])
def test_double_ring_order_vs_simulation(inner, outer):
    seen = _simulate_double(inner, outer)
    for r in range(inner * outer):
        assert O.double_ring_order(r, inner, outer) == seen[r]
        assert sorted(seen[r]) == list(range(inner * outer))
    if (inner, outer) == (4, 2):
        assert O.double_ring_order(0, 4, 2) == [0, 3, 2, 1, 5, 4, 7, 6]


def test_ring_divide_order_covers_every_subchunk_once():
    order = O.ring_divide_order(3, 8, 4)
    assert len(order) == 32 and len(set(order)) == 32
    assert order[:8] == [(c, 0) for c in O.single_ring_order(3, 8)]


# ----------------------------------------------------------------------------- zigzag
@pytest.mark.parametrize("world", [2, 4])
def test_zigzag_ring_equals_global_causal(world):
    """Scatter every rank's result to global positions and compare with single-pass causal
    attention over the whole sequence."""
    B, Hq, Hkv, D, block = 1, 4, 2, 8, 6
    S = 2 * world * block
    q, k, v = _rand(B, S, Hq, D), _rand(B, S, Hkv, D), _rand(B, S, Hkv, D)
    scale = D ** -0.5
    ref_o, ref_l = O.single_pass_attention(q, k, v, scale, causal=True, dtype=torch.float64)
    pos = [O.zigzag_local_positions(r, world, block) for r in range(world)]
    chunks = [torch.stack([k[:, p], v[:, p]]) for p in pos]
    for r in range(world):
        o, l = O.zigzag_ring_forward(q[:, pos[r]], chunks, r, world, scale, dtype=torch.float64)
        assert torch.allclose(o, ref_o[:, pos[r]], atol=1e-11)
        assert torch.allclose(l, ref_l[:, :, pos[r]], atol=1e-11)
        kinds = [O.zigzag_step(r, i, world)[0] for i in range(world)]
        assert kinds[0] == "diag" and kinds.count("diag") == 1


# ----------------------------------------------------------------------------- fp8
def test_quantize_e4m3_is_nearest_representable():
    codes = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    grid = codes[torch.isfinite(codes)].unique()
    assert grid.max() == 448.0
    x = torch.randn(4096)
    xq, s = O.quantize_e4m3(x)
    assert torch.isclose(s, x.abs().max() / 448.0)
    y = x / s
    nearest = grid[(y.unsqueeze(1) - grid.unsqueeze(0)).abs().argmin(1)]
    got = xq.float()
    # equal to the nearest grid point except on exact ties (either neighbour is nearest)
    assert ((got - y).abs() <= (nearest - y).abs() + 1e-7).all()
    assert got.abs().max() == 448.0
    assert torch.allclose(O.dequantize(xq, s), x, rtol=2 ** -4, atol=float(s) * 2 ** -9)


def test_tree_merge_equals_pairwise_fold_and_single_pass():
    """The tree-attention form (max, exp, sum, divide) is pinned by two things it must equal: folding the
    same packed partials pairwise with the closed-form merge, and single-pass attention over all keys."""
    torch.manual_seed(5)
    B, Sq, H, D, W = 1, 24, 2, 16, 5
    q = torch.randn(B, Sq, H, D, dtype=torch.float64)
    k = torch.randn(B, W * 8, H, D, dtype=torch.float64)
    v = torch.randn(B, W * 8, H, D, dtype=torch.float64)
    parts = []
    for c in range(W):
        o, l = O.block_attention(q, k[:, c * 8:(c + 1) * 8], v[:, c * 8:(c + 1) * 8], 0.3, dtype=torch.float64)
        parts.append(torch.cat([o, l.transpose(1, 2).unsqueeze(-1)], dim=-1))
    tree = O.tree_merge(parts)
    fold = parts[0]
    for p in parts[1:]:
        fold = O.flash_reduce(fold, p)
    assert torch.allclose(tree, fold, atol=1e-12, rtol=1e-12)
    ro, rl = O.single_pass_attention(q, k, v, 0.3, dtype=torch.float64)
    assert torch.allclose(tree[..., :-1], ro, atol=1e-12)
    assert torch.allclose(tree[..., -1], rl.transpose(1, 2), atol=1e-12)
    # a rank that saw no key (lse = -inf) contributes nothing; all ranks empty -> (0 | -inf)
    empty = torch.cat([torch.zeros(B, Sq, H, D, dtype=torch.float64),
                       torch.full((B, Sq, H, 1), -math.inf, dtype=torch.float64)], dim=-1)
    assert torch.allclose(O.tree_merge(parts + [empty]), tree, atol=1e-12)
    both = O.tree_merge([empty, empty])
    assert torch.equal(both[..., :-1], torch.zeros(B, Sq, H, D, dtype=torch.float64))
    assert torch.isinf(both[..., -1]).all()
