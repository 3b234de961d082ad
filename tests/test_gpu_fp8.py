"""GPU parity of the FP8 E4M3 quantise / dequantise kernels against the CPU oracle: codes and
scales bit-exact (called through the C ABI via picotron_amd.expert_parallel.ep_communications)."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _c2_input(n, h, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, h, generator=g)
    mask = torch.rand(n, h, generator=g) < 0.001
    return torch.where(mask, 50 * torch.randn(n, h, generator=g), x)


def _check(x_cpu, gpu):
    from picotron_amd.expert_parallel import ep_communications as C

    q, s = C._per_token_quant_fp8(x_cpu.to(gpu))
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.float32
    q_ref, s_ref = O.quant_fp8(x_cpu)
    qc = q.view(torch.uint8).cpu()
    bad = (qc != q_ref).nonzero()
    assert bad.numel() == 0, f"{bad.shape[0]} code mismatches, first {bad[0].tolist()}: x={x_cpu[tuple(bad[0])].item()} got {qc[tuple(bad[0])].item()} want {q_ref[tuple(bad[0])].item()}"
    assert torch.equal(s.cpu().view(torch.int32), s_ref.view(torch.int32))
    d = C._dequant_fp8(q, s, x_cpu.dtype)
    d_ref = O.dequant_fp8(q_ref, s_ref, x_cpu.dtype)
    assert torch.equal(d.cpu().view(torch.int16 if x_cpu.dtype == torch.bfloat16 else torch.int32),
                       d_ref.view(torch.int16 if x_cpu.dtype == torch.bfloat16 else torch.int32))
    return q, s


def test_quant_full_benchmark_shape_bit_exact(gpu):
    """16384 x 4096 bf16, N(0,1) with 0.1% N(0,50) outliers: bytes and scales equal the reference cast."""
    x = _c2_input(16384, 4096).bfloat16()
    q, s = _check(x, gpu)
    # size-independent properties on the same data
    from picotron_amd.expert_parallel import ep_communications as C

    d = C._dequant_fp8(q, s, torch.bfloat16).float()
    xf = x.to(gpu).float()
    assert torch.all(d.abs().amax(-1) <= xf.abs().amax(-1).clamp_min(1e-4) * 1.005)
    rel = ((d - xf).norm() / xf.norm()).item()
    assert rel < 0.05, rel                       # the reference's own bound (tests/test_fp8_dispatch.py:85)
    assert q.element_size() * q.shape[1] + s.element_size() == 4100


@pytest.mark.parametrize("hidden", [8, 40, 256, 1000, 2048, 4104, 8192, 8200, 14336, 16384, 16392, 32768, 32776])
def test_quant_row_widths_bf16(gpu, hidden):
    """Every kernel of the quantiser: a wave per row up to 8192 values (with and without a partly filled last chunk
    round), a block per row up to 32768 (FFN 14336: the SwiGLU output of the FP8 down GEMM), the generic one beyond."""
    x = _c2_input(67, hidden, seed=hidden).bfloat16()
    _check(x, gpu)


def test_quant_long_rows_edge_cases(gpu):
    """Block-per-row kernel: a zero row (amax floor), a NaN, an inf, a huge finite value and the row maximum in the
    last chunk."""
    x = _c2_input(8, 14336, seed=3).bfloat16()
    x[0] = 0
    x[1, 14335] = float("nan")
    x[2, 9000] = float("inf")
    x[3, 14335] = 3.0e38
    x[4, 14335] = 1000.0
    x[5, 0] = -1000.0
    from picotron_amd.expert_parallel import ep_communications as C

    q, s = C._per_token_quant_fp8(x.to(gpu))
    q_ref, s_ref = O.quant_fp8(x)
    qc = q.view(torch.uint8).cpu()
    for r in (0, 3, 4, 5, 6, 7):
        assert torch.equal(qc[r], q_ref[r]) and s[r].item() == s_ref[r].item(), r
    # NaN / inf rows: the scale is NaN / inf as in the reference; codes of a NaN row are 0x7F by this build's convention
    assert torch.isnan(s[1]).item() and torch.all((qc[1] & 0x7F) == 0x7F)
    assert torch.isinf(s[2]).item()


def test_quant_edge_rows_bf16(gpu):
    x = _c2_input(16, 512, seed=5).bfloat16()
    x[0] = 0                               # amax floor 1e-4
    x[1] *= 1e-6                           # floor again, quotients below the smallest subnormal
    x[2] *= 1e-3
    x[3, 7] = 3.0e38                       # near bf16 max
    x[4] = torch.tensor(1e-4).bfloat16()   # exactly the floor
    x[5] = x[5].abs()
    x[6] = -x[6].abs()
    x[7, :] = 448.0
    x[8, ::2] = 1.0
    x[8, 1::2] = -1.0
    _check(x, gpu)


def test_quant_inf_row(gpu):
    x = _c2_input(4, 256, seed=6).bfloat16()
    x[1, 3] = float("inf")
    from picotron_amd.expert_parallel import ep_communications as C

    q, s = C._per_token_quant_fp8(x.to(gpu))
    q_ref, s_ref = O.quant_fp8(x)
    finite_cols = torch.isfinite(x[1])
    qc = q.view(torch.uint8).cpu()
    assert torch.equal(qc[[0, 2, 3]], q_ref[[0, 2, 3]])
    assert torch.equal(qc[1][finite_cols] & 0x7F, q_ref[1][finite_cols] & 0x7F)   # finite / inf = 0
    assert (qc[1][~finite_cols] & 0x7F).tolist() == [0x7F]                         # inf / inf = NaN
    assert torch.isinf(s.cpu()[1]) and torch.equal(s.cpu()[[0, 2, 3]], s_ref[[0, 2, 3]])


def test_quant_adversarial_scales(gpu):
    """Every bf16 value as an element, against scales whose mantissas stress the reciprocal trick
    (all-ones, one, alternating) plus random ones."""
    allv = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    allv = allv[torch.isfinite(allv)]
    rng = np.random.default_rng(0)
    amax_bits = [0x3F80, 0x3FFF, 0x407F, 0x4000, 0x3FD5, 0x3FAA, 0x7F7F, 0x38D2, 0x3900, 0x43E0, 0x4460]
    amax_bits += [int(b) for b in rng.integers(0x38D3, 0x7F7F, size=64)]
    rows = []
    for b in amax_bits:
        amax = torch.tensor([b], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        row = torch.where(allv.abs() <= amax, allv, torch.zeros_like(allv))
        row[0] = amax[0]
        rows.append(row)
    x = torch.stack(rows)[:, :65024]         # multiple of 8 columns -> generic path (hidden > 8192)
    _check(x, gpu)
    _check(x[:, :8192].contiguous(), gpu)    # vector path, row amax re-derived from the slice
    _check(x[:, 30000:38192].contiguous(), gpu)


@pytest.mark.parametrize("hidden", [16, 256, 1000])
def test_quant_fp32_rows(gpu, hidden):
    x = _c2_input(33, hidden, seed=hidden + 1)
    x[0] = 0
    _check(x, gpu)


def test_cpu_tensor_is_refused():
    from picotron_amd import _lib
    from picotron_amd.expert_parallel import ep_communications as C

    with pytest.raises(_lib.PicomoeError):
        C._per_token_quant_fp8(torch.randn(4, 8))


def test_round_trip_autograd_is_straight_through(gpu):
    from picotron_amd.expert_parallel import ep_communications as C

    x = _c2_input(32, 256, seed=9).bfloat16().to(gpu).requires_grad_(True)
    y = C.fp8_round_trip(x)
    g = torch.randn_like(y)
    y.backward(g)
    assert torch.equal(x.grad, g)


def _dispatch(x_cpu, inv, k, n_out, gpu, codes=True, wire=True, prefill=None):
    """picomoe_dispatch_fp8 through the C ABI with caller-owned, pre-filled outputs."""
    from picotron_amd import _lib

    lib = _lib.load()
    T, H = x_cpu.shape
    fill = 7.0 if prefill is None else prefill
    xs = torch.full((n_out, H), fill, dtype=x_cpu.dtype, device=gpu)
    qs = torch.full((n_out, H), 0x11, dtype=torch.uint8, device=gpu) if codes else None
    ss = torch.full((n_out,), fill, dtype=torch.float32, device=gpu) if codes else None
    q = torch.full((T, H), 0x11, dtype=torch.uint8, device=gpu) if wire else None
    s = torch.full((T,), fill, dtype=torch.float32, device=gpu) if wire else None
    P = _lib.ptr
    xd, invd = x_cpu.to(gpu), inv.to(gpu)     # named: the buffers must outlive the launch
    _lib.check(lib.picomoe_dispatch_fp8(P(xd), _lib.dtype_code(x_cpu.dtype), T, H, P(invd), k, n_out, P(xs), P(qs),
                                        P(ss), P(q), P(s), _lib.stream_ptr()), "picomoe_dispatch_fp8")
    torch.cuda.synchronize()
    del xd, invd
    return tuple(t.cpu() if t is not None else None for t in (xs, qs, ss, q, s))


@pytest.mark.parametrize("T,H,E,k,dtype", [
    (512, 4096, 8, 2, torch.bfloat16),     # the Mixtral row width: a wave per token, every chunk round full
    (300, 2048, 64, 6, torch.bfloat16),    # fine-grained: top-6
    (129, 1000, 4, 1, torch.bfloat16),     # a partly filled last chunk round, top-1
    (67, 8192, 8, 16, torch.bfloat16),     # the widest wave-per-token row, the largest top-k
    (40, 100, 4, 2, torch.bfloat16),       # rows that are not whole 16-byte chunks: the generic kernel
    (33, 8200, 4, 2, torch.bfloat16),      # rows longer than a wavefront holds: the generic kernel
    (65, 256, 8, 2, torch.float32),        # fp32 rows
])
def test_dispatch_fp8_is_quant_dequant_permute_in_one_pass(gpu, T, H, E, k, dtype):
    """picomoe_dispatch_fp8 against the oracle's quantise -> dequantise composed with its stable sort by expert:
    x_sorted == dequant(quant(tokens))[order // k], the sorted codes and scales likewise, the token-order codes and
    scales equal the quantiser's -- all bit for bit; edge rows (zeros, below the amax floor, huge, infinite) included."""
    x = _c2_input(T, H, seed=T + H).to(dtype)
    x[0] = 0
    x[1] = 1e-6
    x[2, 3] = 3e38 if dtype == torch.float32 else 3e38
    x[3, 5] = float("inf")
    g = torch.Generator().manual_seed(k)
    idx = torch.stack([torch.randperm(E, generator=g)[:k] if k <= E else torch.randint(0, E, (k,), generator=g) for _ in range(T)])
    order, inv, counts = O.permute_plan_fast(idx.reshape(-1), E)
    q_ref, s_ref = O.quant_fp8(x)
    d_ref = O.dequant_fp8(q_ref, s_ref, dtype)

    def bits(t):
        # bit patterns, with every NaN mapped to one pattern: the row with an infinite entry dequantises to NaN
        # (0 * inf), and which NaN a platform produces is not part of the contract
        b = t.view(torch.int16 if t.dtype == torch.bfloat16 else torch.int32)
        return torch.where(torch.isnan(t), torch.full_like(b, -1), b)

    xs, qs, ss, q, s = _dispatch(x, inv.int(), k, T * k, gpu)
    src = order // k
    assert torch.equal(q, q_ref) and torch.equal(s.view(torch.int32), s_ref.view(torch.int32))
    assert torch.isnan(d_ref[3]).all() and not torch.isnan(d_ref[:3]).any() and not torch.isnan(d_ref[4:]).any()
    assert torch.equal(bits(xs), bits(d_ref[src]))
    assert torch.equal(qs, q_ref[src]) and torch.equal(ss.view(torch.int32), s_ref[src].view(torch.int32))
    # without the optional outputs: the same rows
    xs2, _, _, _, _ = _dispatch(x, inv.int(), k, T * k, gpu, codes=False, wire=False)
    assert torch.equal(bits(xs2), bits(xs))
    # and it equals the three-pass form it replaces, kernel for kernel
    from picotron_amd import _ops
    from picotron_amd.expert_parallel import ep_communications as C

    three = _ops.gather_rows(C.fp8_round_trip(x.to(gpu)), order.int().to(gpu), k, T * k)
    assert torch.equal(bits(three.cpu()), bits(xs))


def test_dispatch_fp8_skips_rows_that_are_not_kept(gpu):
    """Negative positions (rows a capacity window dropped) and positions past n_out are skipped; what no kept row maps to
    is left as the caller filled it."""
    T, H, k = 50, 512, 2
    x = _c2_input(T, H, seed=3).bfloat16()
    g = torch.Generator().manual_seed(1)
    n_out = 70
    perm = torch.randperm(T * k, generator=g)
    inv = torch.full((T * k,), -1, dtype=torch.int32)
    inv[perm[:n_out]] = torch.arange(n_out, dtype=torch.int32)       # 70 kept rows, 30 dropped
    inv[perm[n_out]] = n_out + 5                                      # a position past the buffer: skipped too
    xs, qs, ss, _, _ = _dispatch(x, inv, k, n_out + 4, gpu)
    q_ref, s_ref = O.quant_fp8(x)
    d_ref = O.dequant_fp8(q_ref, s_ref, torch.bfloat16)
    src = perm[:n_out] // k
    assert torch.equal(xs[:n_out].view(torch.int16), d_ref[src].view(torch.int16))
    assert torch.equal(qs[:n_out], q_ref[src]) and torch.equal(ss[:n_out], s_ref[src])
    assert torch.all(xs[n_out:] == 7.0) and torch.all(qs[n_out:] == 0x11) and torch.all(ss[n_out:] == 7.0)


def test_dispatch_fp8_backward_is_the_gather_sum(gpu):
    """Autograd of the fused dispatch: straight through the quantiser, then d_tokens[t] = sum_j d_x_sorted[inv[t*k+j]]
    (the backward of expand + permute), equal to the three-pass form's gradient bit for bit."""
    from picotron_amd import _ops
    from picotron_amd.expert_parallel import ep_communications as C

    T, H, E, k = 96, 512, 8, 2
    x = _c2_input(T, H, seed=5).bfloat16()
    idx = torch.stack([torch.randperm(E, generator=torch.Generator().manual_seed(i))[:k] for i in range(T)])
    plan = _ops.permute_plan(idx.reshape(-1).to(gpu), E)
    up = torch.randn(T * k, H, generator=torch.Generator().manual_seed(6)).bfloat16().to(gpu)
    a = x.to(gpu).requires_grad_(True)
    ya, qa, sa = _ops.dispatch_fp8(a, plan.inv_order, k, T * k, with_codes=True)
    assert qa.dtype == torch.uint8 and sa.dtype == torch.float32 and not qa.requires_grad
    ya.backward(up)
    b = x.to(gpu).requires_grad_(True)
    yb = _ops.expand_permute(C.fp8_round_trip(b), plan.order, plan.inv_order, k, T * k)
    yb.backward(up)
    assert torch.equal(ya, yb) and torch.equal(a.grad, b.grad)
