"""GPU parity of the expert FFN (grouped SwiGLU GEMMs, forward / dgrad / wgrad) against the CPU oracle.

Shapes and tolerances of the first three tests are the ones the reference's own kernel test uses
(tests/test_megakernel.py:29-99): ragged counts with an empty expert and one longer than a tile,
fp32 atol = rtol = 1e-4 forward and 1e-3 on gradients, the row-weight epilogue, bf16 max |diff| < 5e-2.
"""

import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _mk(E, H, I, counts, dtype, seed, scale=0.1):
    g = torch.Generator().manual_seed(seed)
    N = int(sum(counts))
    x = torch.randn(N, H, generator=g).to(dtype)
    gw = (torch.randn(E, I, H, generator=g) * scale).to(dtype)
    uw = (torch.randn(E, I, H, generator=g) * scale).to(dtype)
    dw = (torch.randn(E, H, I, generator=g) * scale).to(dtype)
    return x, torch.tensor(counts, dtype=torch.int64), gw, uw, dw, g


def test_fwd_bwd_ragged_fp32(gpu):
    from picotron_amd.expert_parallel import megakernel

    x, counts, gw, uw, dw, g = _mk(4, 48, 96, [5, 0, 130, 17], torch.float32, 0)
    leaves = [t.cuda().requires_grad_(True) for t in (x, gw, uw, dw)]
    y = megakernel.fused_moe(leaves[0], counts.cuda(), *leaves[1:])
    yr = O.expert_ffn(x, counts, gw, uw, dw)
    assert torch.allclose(y.cpu(), yr, atol=1e-4, rtol=1e-4)
    assert (y.cpu() - yr).abs().max() <= 1e-5 * yr.abs().max()        # and the fp32 bar of this build
    dy = torch.randn(y.shape, generator=g)
    y.backward(dy.cuda())
    ref = O.expert_ffn_backward(x, counts, gw, uw, dw, dy)
    for got, want, name in zip([l.grad for l in leaves], ref, ("dx", "dgate", "dup", "ddown")):
        d = (got.cpu() - want).abs().max().item()
        assert d < 1e-3, (name, d)
        assert d <= 1e-5 * want.abs().max().item() + 1e-7, (name, d)
    assert torch.all(leaves[1].grad[1] == 0) and torch.all(leaves[3].grad[1] == 0)   # the empty expert


def test_row_weight_epilogue(gpu):
    from picotron_amd.expert_parallel import megakernel

    x, counts, gw, uw, dw, g = _mk(3, 32, 64, [20, 33, 7], torch.float32, 1)
    rw = torch.rand(60, generator=g)
    y = megakernel.fused_moe(x.cuda(), counts.cuda(), gw.cuda(), uw.cuda(), dw.cuda(), row_weight=rw.cuda())
    yr = O.expert_ffn(x, counts, gw, uw, dw, rw)
    assert torch.allclose(y.cpu(), yr, atol=1e-4)
    # and its gradient, including d row_weight
    leaves = [t.cuda().requires_grad_(True) for t in (x, gw, uw, dw, rw)]
    yy = megakernel.fused_moe(leaves[0], counts.cuda(), leaves[1], leaves[2], leaves[3], row_weight=leaves[4])
    dy = torch.randn(yy.shape, generator=g)
    yy.backward(dy.cuda())
    cl = [t.clone().requires_grad_(True) for t in (x, gw, uw, dw, rw)]
    O.expert_ffn(cl[0], counts, cl[1], cl[2], cl[3], cl[4]).backward(dy)
    for a, b in zip(leaves, cl):
        assert torch.allclose(a.grad.cpu(), b.grad, atol=1e-4, rtol=1e-4)


def test_backward_computes_only_what_autograd_asks_for(gpu):
    """Frozen experts (input gradient only), and a frozen input with one trainable matrix: the gradients that are asked
    for equal the oracle's, the others stay None."""
    from picotron_amd.expert_parallel import megakernel

    x, counts, gw, uw, dw, g = _mk(3, 32, 64, [9, 0, 40], torch.float32, 5)
    dy = torch.randn(49, 32, generator=g)
    ref = O.expert_ffn_backward(x, counts, gw, uw, dw, dy)
    xg = x.cuda().requires_grad_(True)
    megakernel.fused_moe(xg, counts.cuda(), gw.cuda(), uw.cuda(), dw.cuda()).backward(dy.cuda())
    assert torch.allclose(xg.grad.cpu(), ref[0], atol=1e-4, rtol=1e-4)
    for which in (1, 2, 3):
        leaves = [t.cuda() for t in (x, gw, uw, dw)]
        leaves[which].requires_grad_(True)
        megakernel.fused_moe(leaves[0], counts.cuda(), *leaves[1:]).backward(dy.cuda())
        assert torch.allclose(leaves[which].grad.cpu(), ref[which], atol=1e-4, rtol=1e-4)
        assert all(l.grad is None for i, l in enumerate(leaves) if i != which)


def test_bf16_small(gpu):
    from picotron_amd.expert_parallel import megakernel

    x, counts, gw, uw, dw, _ = _mk(4, 64, 128, [16, 16, 16, 16], torch.bfloat16, 2)
    y = megakernel.fused_moe(x.cuda(), counts.cuda(), gw.cuda(), uw.cuda(), dw.cuda())
    yr = O.expert_ffn(x, counts, gw, uw, dw)
    assert (y.cpu().float() - yr.float()).abs().max().item() < 5e-2


def test_empty_input_and_all_empty_but_one(gpu):
    from picotron_amd.expert_parallel import megakernel

    x, counts, gw, uw, dw, _ = _mk(3, 16, 32, [0, 0, 0], torch.float32, 3)
    y = megakernel.fused_moe(x.cuda(), counts.cuda(), gw.cuda(), uw.cuda(), dw.cuda())
    assert y.shape == (0, 16)
    grads = megakernel.fused_moe_backward(x.cuda(), counts.cuda(), gw.cuda(), uw.cuda(), dw.cuda(), y)
    assert all(torch.all(t == 0) for t in grads) and grads[1].shape == gw.shape
    x, counts, gw, uw, dw, _ = _mk(3, 16, 32, [0, 0, 9], torch.float32, 4)
    y = megakernel.fused_moe_forward(x.cuda(), counts.cuda(), gw.cuda(), uw.cuda(), dw.cuda())
    assert torch.allclose(y.cpu(), O.expert_ffn(x, counts, gw, uw, dw), atol=1e-5)


@pytest.mark.parametrize("dtype,H,I", [(torch.float32, 40, 72), (torch.bfloat16, 256, 384), (torch.bfloat16, 320, 192)])
def test_gate_and_up_weight_gradients_in_one_launch(gpu, dtype, H, I):
    """The autograd path computes d gate_w and d up_w with one launch ([dg | du] as the left operand in place, the result
    [E, 2I, H] split into two views); fused_moe_wgrad keeps one launch each.  Same tiles, same arithmetic: bit-equal, and
    every expert's slice of either gradient is contiguous (what the per-expert parameters receive)."""
    from picotron_amd.expert_parallel import megakernel

    E = 4
    x, counts, gw, uw, dw, g = _mk(E, H, I, [300, 0, 5, 257], dtype, 11)
    dy = torch.randn(x.shape, generator=g).to(dtype)
    leaves = [t.cuda().requires_grad_(True) for t in (x, gw, uw, dw)]
    megakernel.fused_moe(leaves[0], counts.cuda(), *leaves[1:]).backward(dy.cuda())
    _, a, d13 = megakernel.fused_moe_dgrad(x.cuda(), counts.cuda(), gw.cuda(), uw.cuda(), dw.cuda(), dy.cuda())
    dg, du, dd = megakernel.fused_moe_wgrad(x.cuda(), counts.cuda(), a, d13, dy.cuda())
    assert torch.equal(leaves[1].grad, dg) and torch.equal(leaves[2].grad, du) and torch.equal(leaves[3].grad, dd)
    # only one of the two asked for: the separate launches
    only_up = [t.cuda() for t in (x, gw, uw, dw)]
    only_up[2].requires_grad_(True)
    megakernel.fused_moe(only_up[0], counts.cuda(), *only_up[1:]).backward(dy.cuda())
    assert torch.equal(only_up[2].grad, du) and only_up[1].grad is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_explicit_dgrad_wgrad_api(gpu, dtype):
    """fused_moe_dgrad / fused_moe_wgrad return the intermediates the reference documents (a, d_inter13)."""
    from picotron_amd.expert_parallel import megakernel

    E, H, I = 3, 40, 72
    x, counts, gw, uw, dw, g = _mk(E, H, I, [33, 0, 70], dtype, 5)
    dy = torch.randn(x.shape, generator=g).to(dtype)
    dx, a, d13 = megakernel.fused_moe_dgrad(x.cuda(), counts.cuda(), gw.cuda(), uw.cuda(), dw.cuda(), dy.cuda())
    dg, du, dd = megakernel.fused_moe_wgrad(x.cuda(), counts.cuda(), a, d13, dy.cuda())
    xf, gf, uf, df, dyf = (t.float() for t in (x, gw, uw, dw, dy))
    rdx, rdg, rdu, rdd = O.expert_ffn_backward(xf, counts, gf, uf, df, dyf)
    # intermediates from their definitions
    owner = torch.repeat_interleave(torch.arange(E), counts)
    g13 = torch.cat([torch.einsum("nh,nih->ni", xf, gf[owner]), torch.einsum("nh,nih->ni", xf, uf[owner])], 1)
    ra = torch.nn.functional.silu(g13[:, :I]) * g13[:, I:]
    rd13 = O.silu_and_mul_bwd(g13, torch.einsum("nh,nhi->ni", dyf, df[owner]))
    for got, want in ((dx, rdx), (a, ra), (d13, rd13), (dg, rdg), (du, rdu), (dd, rdd)):
        if dtype == torch.float32:
            assert torch.allclose(got.cpu().float(), want, rtol=1e-4, atol=1e-5)
        else:  # bf16: every element within 1e-2 of the tensor's scale, the bar of the ragged tests below
            assert (got.cpu().float() - want).abs().max().item() <= 1e-2 * want.abs().max().item()


@pytest.mark.parametrize("H,I,counts", [(256, 512, [130, 128, 126, 0, 1, 64, 63, 0]), (100, 36, [7, 300]), (256, 384, [300, 0, 5, 257]), (512, 128, [1, 1000, 70]),
                                        (320, 192, [300, 0, 5, 257]), (128, 448, [129, 64, 1]), (704, 320, [33, 520, 0, 256]), (192, 128, [257, 3]),
                                        (512, 4096, [700, 3, 0, 129, 260, 515, 40, 1, 300, 256, 90, 130, 64, 257, 511, 33, 128, 127, 5, 600])])
def test_bf16_ragged_against_oracle(gpu, H, I, counts):
    """bf16: outputs and gradients within rtol 1e-2 of the oracle (measured against the magnitude of each tensor).
    Shapes five to eight are widths the 256-column tiles do not divide (hidden 320, 128, 704, 192; FFN 192, 448, 320): the
    MFMA kernels run them with clamped loads and masked stores in the last tile column.  The last one has enough tiles (twenty
    skewed experts, FFN 4096) for the tile walk to deal whole runs of 32 to the eight XCDs and still have tiles left over, in the
    row-grouped kernels (480 heavy tiles for gate/up) and in the weight gradients (640 and 1280 tiles)."""
    from picotron_amd.expert_parallel import megakernel

    E = len(counts)
    x, cnt, gw, uw, dw, g = _mk(E, H, I, counts, torch.bfloat16, 6, scale=0.05)
    leaves = [t.cuda().requires_grad_(True) for t in (x, gw, uw, dw)]
    y = megakernel.fused_moe(leaves[0], cnt.cuda(), *leaves[1:])
    yr = O.expert_ffn(x, cnt, gw, uw, dw)
    assert (y.cpu().float() - yr.float()).abs().max() <= 1e-2 * yr.float().abs().max()
    dy = torch.randn(y.shape, generator=g).bfloat16()
    y.backward(dy.cuda())
    ref = O.expert_ffn_backward(x.float(), cnt, gw.float(), uw.float(), dw.float(), dy.float())
    for got, want in zip([l.grad for l in leaves], ref):
        assert (got.cpu().float() - want).abs().max() <= 1e-2 * want.abs().max()


@pytest.mark.parametrize("H", [512, 320])
@pytest.mark.parametrize("counts", [[300, 260, 100, 515], [256, 512, 7, 129], [40, 0, 3, 1]])
def test_split_last_round_matches_whole_tiles(gpu, counts, H):
    """With a workspace the down and dgrad_x kernels cut the tiles of the last, partly filled round into 2 or 4 ranges of K
    (K here is 32 and 64 k-tiles, enough for 2 and 4 pieces) and add the fp32 partial tiles up in a second kernel: the
    result must agree with the whole-tile kernels to the rounding of the partial sums, and with the oracle at the bf16
    tolerance; rows past the tiles' segments must stay untouched."""
    from picotron_amd import _lib
    from picotron_amd.expert_parallel import megakernel as mk

    E, I = len(counts), 2048
    x, cnt, gw, uw, dw, g = _mk(E, H, I, counts, torch.bfloat16, 11, scale=0.03)
    N = x.shape[0]
    act = (torch.randn(N, I, generator=g) * 0.5).bfloat16().cuda()
    rw = torch.rand(N, generator=g).bfloat16().cuda()
    d13 = (torch.randn(N, 2 * I, generator=g) * 0.5).bfloat16().cuda()
    cntd, gwd, uwd, dwd = cnt.cuda(), gw.cuda(), uw.cuda(), dw.cuda()
    lib = _lib.load()
    ws = torch.empty(lib.picomoe_ffn_workspace_bytes(), dtype=torch.uint8, device="cuda")

    def down(workspace):
        y = torch.full((N, H), 7.0, dtype=torch.bfloat16, device="cuda")
        _lib.check(lib.picomoe_ffn_down(_lib.ptr(act), _lib.ptr(cntd), E, N, H, I, _lib.ptr(dwd), _lib.ptr(rw), _lib.dtype_code(act.dtype),
                                        _lib.ptr(y), _lib.ptr(workspace), workspace.numel() if workspace is not None else 0,
                                        _lib.stream_ptr()), "picomoe_ffn_down")
        return y

    def dgrad_x(workspace):
        dx = torch.full((N, H), 7.0, dtype=torch.bfloat16, device="cuda")
        _lib.check(lib.picomoe_ffn_dgrad_x(_lib.ptr(d13), _lib.ptr(cntd), E, N, H, I, _lib.ptr(gwd), _lib.ptr(uwd),
                                           _lib.dtype_code(d13.dtype), _lib.ptr(dx), _lib.ptr(workspace),
                                           workspace.numel() if workspace is not None else 0, _lib.stream_ptr()), "picomoe_ffn_dgrad_x")
        return dx

    owner = torch.repeat_interleave(torch.arange(E), cnt)
    want_y = torch.einsum("ni,nhi->nh", act.cpu().float(), dw.float()[owner]).bfloat16().float() * rw.cpu().float()[:, None]
    want_dx = torch.einsum("ni,nih->nh", d13.cpu().float()[:, :I], gw.float()[owner]) + torch.einsum(
        "ni,nih->nh", d13.cpu().float()[:, I:], uw.float()[owner])
    for fn, want in ((down, want_y), (dgrad_x, want_dx)):
        whole, split = fn(None).float().cpu(), fn(ws).float().cpu()
        scale = want.abs().max()
        assert (whole - want).abs().max() <= 1e-2 * scale and (split - want).abs().max() <= 1e-2 * scale
        assert (split - whole).abs().max() <= 2.0 ** -7 * scale       # one bf16 ulp of the largest value
        assert torch.equal(fn(ws).float().cpu(), split)               # fixed summation order: run to run identical


@pytest.mark.parametrize("H", [2048, 4096, 8192])
@pytest.mark.parametrize("counts", [[300, 260, 100, 515], [256, 512, 7, 129], [40, 0, 3, 1]])
def test_split_last_round_gate_up_and_dgrad_act(gpu, counts, H):
    """The same split for the two kernels whose epilogue is more than a store: gate/up (SwiGLU on the summed pieces, [g | u]
    kept) and dgrad_act (SwiGLU backward at [g | u] on the summed pieces, act rebuilt).  They split into four pieces from
    K = hidden = 64 k-tiles on (4096, 8192 here) and not below (2048: the workspace changes nothing); FFN width 384 gives the
    last tile column of dgrad_act only half its columns.  Whole-tile and split
    results agree to the rounding of the partial sums, both with the oracle's arithmetic at the bf16 tolerance, run to run
    identical, rows past the segments untouched."""
    from picotron_amd import _lib

    E, I = len(counts), 384
    x, cnt, gw, uw, dw, g = _mk(E, H, I, counts, torch.bfloat16, 17, scale=0.02)
    N, slack = x.shape[0], 5
    dy = torch.randn(N, H, generator=g).bfloat16()
    i13 = (torch.randn(N, 2 * I, generator=g) * 0.7).bfloat16()
    pad = lambda t: torch.cat([t, torch.full((slack, t.shape[1]), float("nan"), dtype=t.dtype)]).cuda()
    xd, dyd, i13d = pad(x), pad(dy), pad(i13)
    cntd, gwd, uwd, dwd = cnt.cuda(), gw.cuda(), uw.cuda(), dw.cuda()
    lib = _lib.load()
    ws = torch.empty(lib.picomoe_ffn_workspace_bytes(), dtype=torch.uint8, device="cuda")
    P, code, st = _lib.ptr, _lib.dtype_code(torch.bfloat16), _lib.stream_ptr()
    fill = lambda cols: torch.full((N + slack, cols), 7.0, dtype=torch.bfloat16, device="cuda")

    def gate_up(workspace):
        act, out13 = fill(I), fill(2 * I)
        _lib.check(lib.picomoe_ffn_gate_up(P(xd), P(cntd), E, N + slack, H, I, P(gwd), P(uwd), code, P(act), P(out13), P(workspace),
                                           workspace.numel() if workspace is not None else 0, st), "picomoe_ffn_gate_up")
        return torch.cat([act, out13], 1)

    def dgrad_act(workspace):
        d13, act = fill(2 * I), fill(I)
        _lib.check(lib.picomoe_ffn_dgrad_act(P(dyd), P(cntd), E, N + slack, H, I, P(dwd), P(i13d), code, P(d13), P(act), P(workspace),
                                             workspace.numel() if workspace is not None else 0, st), "picomoe_ffn_dgrad_act")
        return torch.cat([d13, act], 1)

    owner = torch.repeat_interleave(torch.arange(E), cnt)
    xf = x.float()
    g13 = torch.cat([torch.einsum("nh,nih->ni", xf, gw.float()[owner]), torch.einsum("nh,nih->ni", xf, uw.float()[owner])], 1)
    g13 = g13.bfloat16().float()
    want_gu = torch.cat([torch.nn.functional.silu(g13[:, :I]).bfloat16().float() * g13[:, I:], g13], 1)
    da = torch.einsum("nh,nhi->ni", dy.float(), dw.float()[owner]).bfloat16().float()
    gi, ui = i13.float()[:, :I], i13.float()[:, I:]
    want_da = torch.cat([O.silu_and_mul_bwd(i13.float(), da), torch.nn.functional.silu(gi).bfloat16().float() * ui], 1)
    for fn, want in ((gate_up, want_gu), (dgrad_act, want_da)):
        whole, split = fn(None).float().cpu(), fn(ws).float().cpu()
        assert torch.all(whole[N:] == 7.0) and torch.all(split[N:] == 7.0)          # slack rows: untouched
        whole, split = whole[:N], split[:N]
        scale = want.abs().max()
        assert (whole - want).abs().max() <= 1e-2 * scale and (split - want).abs().max() <= 1e-2 * scale
        assert (split - whole).abs().max() <= 2.0 ** -6 * scale       # two bf16 roundings (g or da, then the product) of the largest value
        assert torch.equal(fn(ws).float().cpu()[:N], split)           # fixed summation order: run to run identical


@pytest.mark.parametrize("H,I,dtype", [(256, 384, torch.bfloat16), (320, 192, torch.bfloat16), (96, 40, torch.bfloat16), (96, 40, torch.float32),
                                       (18, 10, torch.float32)])
def test_rows_past_the_segments_are_never_read_into_a_result(gpu, H, I, dtype):
    """n_rows > sum(counts), as in the capacity modes where the buffers are sized for every routed row and only the kept
    rows are laid out: the slack rows of every input hold NaN, the slack rows of every output are pre-filled.  Results
    for the valid rows and all three weight gradients must equal the run without slack bit for bit, and the slack rows
    of the outputs must come back untouched.  Covers the bf16 MFMA kernels (hidden 256; hidden 320 / FFN 192 with a partly
    filled last tile column), the fp32 MFMA kernels (hidden 96 / FFN 40 in fp32) and the generic ones (the same widths in
    bf16; hidden 18 / FFN 10 in fp32)."""
    from picotron_amd import _lib

    lib = _lib.load()
    counts = [70, 0, 300, 1, 129]
    E, n = len(counts), sum(counts)
    x, cnt, gw, uw, dw, g = _mk(E, H, I, counts, dtype, 13, scale=0.05)
    dy = torch.randn(n, H, generator=g).to(dtype)
    cntd, gwd, uwd, dwd = cnt.cuda(), gw.cuda(), uw.cuda(), dw.cuda()
    code, st = _lib.dtype_code(dtype), _lib.stream_ptr()

    def run(slack):
        N = n + slack
        pad = lambda t: torch.cat([t, torch.full((slack, t.shape[1]), float("nan"), dtype=dtype)]).cuda()
        fill = lambda cols: torch.full((N, cols), 7.0, dtype=dtype, device="cuda")
        xs, dys = pad(x), pad(dy)
        act, i13, y, d13, dx = fill(I), fill(2 * I), fill(H), fill(2 * I), fill(H)
        ws = torch.empty(lib.picomoe_ffn_workspace_bytes(), dtype=torch.uint8, device="cuda")
        P = _lib.ptr
        _lib.check(lib.picomoe_ffn_gate_up(P(xs), P(cntd), E, N, H, I, P(gwd), P(uwd), code, P(act), P(i13), P(ws), ws.numel(), st), "gate_up")
        out_rows = {"act": act.clone(), "inter13": i13.clone()}
        # slack rows of the intermediates a later kernel reads: NaN, like the caller's torch.empty may hold
        act[n:], i13[n:] = float("nan"), float("nan")
        _lib.check(lib.picomoe_ffn_down(P(act), P(cntd), E, N, H, I, P(dwd), None, code, P(y), P(ws), ws.numel(), st), "down")
        _lib.check(lib.picomoe_ffn_dgrad_act(P(dys), P(cntd), E, N, H, I, P(dwd), P(i13), code, P(d13), None, P(ws), ws.numel(), st), "dgrad_act")
        out_rows.update(y=y.clone(), d13=d13.clone())
        d13[n:] = float("nan")
        _lib.check(lib.picomoe_ffn_dgrad_x(P(d13), P(cntd), E, N, H, I, P(gwd), P(uwd), code, P(dx), P(ws), ws.numel(), st), "dgrad_x")
        out_rows["dx"] = dx.clone()
        grads = {}
        for name, lhs, ld_l, off, rhs, ld_r, p_dim, q_dim in (("d_down", dys, H, 0, act, I, H, I), ("d_gate", d13, 2 * I, 0, xs, H, I, H),
                                                              ("d_up", d13, 2 * I, I, xs, H, I, H)):
            o = torch.full((E, p_dim, q_dim), 7.0, dtype=dtype, device="cuda")
            lp = _lib.ctypes.c_void_p(lhs.data_ptr() + off * lhs.element_size())
            _lib.check(lib.picomoe_ffn_wgrad(lp, ld_l, P(rhs), ld_r, P(cntd), E, N, p_dim, q_dim, code, P(o), st), name)
            grads[name] = o
        torch.cuda.synchronize()
        return out_rows, grads

    base_rows, base_grads = run(0)
    rows, grads = run(37)
    for name, t in rows.items():
        assert torch.isfinite(t[:n]).all(), name
        assert torch.equal(t[:n], base_rows[name]), name          # valid rows: bit-identical to the run without slack
        assert torch.all(t[n:] == 7.0), name                       # slack rows of the outputs: untouched
    for name, t in grads.items():
        assert torch.isfinite(t).all(), name
        assert torch.equal(t, base_grads[name]), name
        assert torch.all(t[1] == 0), name                          # the empty expert
    # and the valid rows are the oracle's
    yr = O.expert_ffn(x, cnt, gw, uw, dw)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert (rows["y"][:n].cpu().float() - yr.float()).abs().max() <= tol * yr.float().abs().max()


def test_bf16_many_experts(gpu):
    """150 experts (more than one wave's worth in the tile lookup), counts 0..300 incl. empty experts, full tiles and
    tails of both classes: forward and gradients against the oracle."""
    from picotron_amd.expert_parallel import megakernel

    E, H, I = 150, 256, 128
    gen = torch.Generator().manual_seed(11)
    counts = torch.randint(0, 40, (E,), generator=gen).tolist()
    for e, c in ((3, 0), (64, 300), (65, 256), (66, 129), (149, 257), (100, 0)):
        counts[e] = c
    x, cnt, gw, uw, dw, g = _mk(E, H, I, counts, torch.bfloat16, 12, scale=0.05)
    leaves = [t.cuda().requires_grad_(True) for t in (x, gw, uw, dw)]
    y = megakernel.fused_moe(leaves[0], cnt.cuda(), *leaves[1:])
    yr = O.expert_ffn(x, cnt, gw, uw, dw)
    assert (y.cpu().float() - yr.float()).abs().max() <= 1e-2 * yr.float().abs().max()
    dy = torch.randn(y.shape, generator=g).bfloat16()
    y.backward(dy.cuda())
    ref = O.expert_ffn_backward(x.float(), cnt, gw.float(), uw.float(), dw.float(), dy.float())
    for got, want in zip([l.grad for l in leaves], ref):
        assert (got.cpu().float() - want).abs().max() <= 1e-2 * want.abs().max()
    assert torch.all(leaves[1].grad[3] == 0) and torch.all(leaves[3].grad[100] == 0)   # empty experts


def test_mlp_module_runs_the_kernels(gpu):
    import types

    from picotron_amd.model import MLP

    torch.manual_seed(0)
    m = MLP(types.SimpleNamespace(hidden_size=32, intermediate_size=80)).cuda()
    x = torch.randn(3, 5, 32)
    y = m(x.cuda())
    want = O.mlp(x, m.gate_proj.weight.detach().cpu(), m.up_proj.weight.detach().cpu(), m.down_proj.weight.detach().cpu())
    assert y.shape == (3, 5, 32) and torch.allclose(y.cpu(), want, atol=1e-5)
    y.sum().backward()
    assert all(p.grad is not None for p in m.parameters())


def test_workspace_cache_is_bounded(gpu):
    """The split-round workspaces are cached per stream; the cache keeps at most four and can be emptied."""
    from picotron_amd.expert_parallel import megakernel as mk

    mk.release_workspaces()
    dev = torch.device("cuda", torch.cuda.current_device())
    first = mk._ffn_workspace(dev)
    assert mk._ffn_workspace(dev) is first                     # same stream: same buffer
    for _ in range(6):
        with torch.cuda.stream(torch.cuda.Stream()):
            mk._ffn_workspace(dev)
    assert len(mk._workspaces) == mk._MAX_WORKSPACES
    mk.release_workspaces()
    assert len(mk._workspaces) == 0


@pytest.mark.parametrize("H,I,counts", [
    (256, 512, [5, 0, 130, 17, 300, 1, 127, 128]),   # the tiny configuration's widths; tails, an exact tile, an empty expert
    (132, 68, [7, 300]),                              # widths that are multiples of 4 only: a K tail in every GEMM
    (64, 36, [129, 64, 1]),                           # fewer output columns than a tile is wide
    (2048, 128, [33, 0, 200]),                        # a long contraction
])
def test_fp32_mfma_against_oracle(gpu, H, I, counts):
    """fp32 shapes the matrix-pipe kernels take (v_mfma_f32_32x32x2_f32, full fp32 products): forward and all four
    gradients within 1e-5 of each tensor's scale of the oracle's fp32 arithmetic, the explicit dgrad / wgrad entry points
    and their intermediates, and the row-weight epilogue with its gradient."""
    from picotron_amd.expert_parallel import megakernel

    assert megakernel.kernel_family(torch.float32, H, I) == "f32_mfma"
    E = len(counts)
    x, cnt, gw, uw, dw, g = _mk(E, H, I, counts, torch.float32, H + I, scale=0.05)
    dy = torch.randn(x.shape, generator=g)
    rw = torch.rand(x.shape[0], generator=g)

    def close(got, want, what):
        err, scale = (got.cpu() - want).abs().max().item(), want.abs().max().item()
        assert err <= 1e-5 * scale + 1e-9, f"{what}: max error {err:.3e} against a scale of {scale:.3e}"

    for with_rw in (False, True):
        leaves = [t.cuda().requires_grad_(True) for t in (x, gw, uw, dw)] + ([rw.cuda().requires_grad_(True)] if with_rw else [])
        y = megakernel.fused_moe(leaves[0], cnt.cuda(), leaves[1], leaves[2], leaves[3], row_weight=leaves[4] if with_rw else None)
        cl = [t.double().requires_grad_(True) for t in (x, gw, uw, dw)] + ([rw.double().requires_grad_(True)] if with_rw else [])
        yr = O.expert_ffn(cl[0], cnt, cl[1], cl[2], cl[3], cl[4] if with_rw else None)
        close(y.detach(), yr.detach().float(), "y")
        y.backward(dy.cuda())
        yr.backward(dy.double())
        for a, b, name in zip(leaves, cl, ("dx", "dgate", "dup", "ddown", "drow_weight")):
            close(a.grad, b.grad.float(), name)
        for e, c in enumerate(counts):
            if c == 0:
                assert torch.all(leaves[1].grad[e] == 0) and torch.all(leaves[3].grad[e] == 0)
    # the explicit entry points and what they hand on
    dx, a, d13 = megakernel.fused_moe_dgrad(x.cuda(), cnt.cuda(), gw.cuda(), uw.cuda(), dw.cuda(), dy.cuda())
    dg, du, dd = megakernel.fused_moe_wgrad(x.cuda(), cnt.cuda(), a, d13, dy.cuda())
    owner = torch.repeat_interleave(torch.arange(E), cnt)
    xd, gd, ud, dd_, dyd = (t.double() for t in (x, gw, uw, dw, dy))
    g13 = torch.cat([torch.einsum("nh,nih->ni", xd, gd[owner]), torch.einsum("nh,nih->ni", xd, ud[owner])], 1)
    close(a, (torch.nn.functional.silu(g13[:, :I]) * g13[:, I:]).float(), "a")
    close(d13, O.silu_and_mul_bwd(g13, torch.einsum("nh,nhi->ni", dyd, dd_[owner])).float(), "d_inter13")
    rdx, rdg, rdu, rdd = O.expert_ffn_backward(xd, cnt, gd, ud, dd_, dyd)
    for got, want, name in ((dx, rdx, "dx"), (dg, rdg, "dgate"), (du, rdu, "dup"), (dd, rdd, "ddown")):
        close(got, want.float(), "explicit " + name)


def test_kernel_family_and_the_generic_warning(gpu):
    """Which kernels a shape runs is a query of the library; a shape that lands on the scalar-FMA kernels warns, once."""
    import warnings

    from picotron_amd.expert_parallel import megakernel

    fam = megakernel.kernel_family
    assert fam(torch.bfloat16, 4096, 14336) == "bf16_mfma" and fam(torch.bfloat16, 320, 192) == "bf16_mfma"
    assert fam(torch.bfloat16, 96, 40) == "generic" and fam(torch.bfloat16, 100, 128) == "generic"
    assert fam(torch.float32, 256, 512) == "f32_mfma" and fam(torch.float32, 36, 68) == "f32_mfma"
    assert fam(torch.float32, 16, 32) == "generic" and fam(torch.float32, 130, 64) == "generic"
    x, counts, gw, uw, dw, _ = _mk(2, 24, 40, [3, 9], torch.bfloat16, 7)
    megakernel._warned_generic.discard((torch.bfloat16, 24, 40))
    with pytest.warns(RuntimeWarning, match="generic scalar-FMA"):
        megakernel.fused_moe_forward(x.cuda(), counts.cuda(), gw.cuda(), uw.cuda(), dw.cuda())
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        megakernel.fused_moe_forward(x.cuda(), counts.cuda(), gw.cuda(), uw.cuda(), dw.cuda())   # the second call is silent
        x2, c2, g2, u2, d2, _ = _mk(2, 256, 128, [3, 9], torch.bfloat16, 8)
        megakernel.fused_moe_forward(x2.cuda(), c2.cuda(), g2.cuda(), u2.cuda(), d2.cuda())      # an MFMA shape never warns
