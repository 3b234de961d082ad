"""Pins the FP8 E4M3 part of the CPU oracle (oracle/moe_oracle.py, oracle/moe_oracle.c).

What fixes the answers: the OCP E4M3FN format itself (closed-form value of each code, known
constants), torch's own ``float8_e4m3fn`` cast (a library routine present on every box), and the
statistics the reference holds for this path (rel-L2 ~0.023, picotron/expert_parallel/README.md:298;
``< 0.05`` in tests/test_fp8_dispatch.py:85; wire bytes H+4 per row, :77-78).
"""

import numpy as np
import torch

from oracle import c_oracle
from oracle import moe_oracle as O


def test_decode_table_known_values():
    t = O.e4m3_decode_table()
    assert t[0x00] == 0.0 and t[0x80] == 0.0
    assert t[0x7E] == 448.0 and t[0xFE] == -448.0          # largest finite
    assert np.isnan(t[0x7F]) and np.isnan(t[0xFF])          # the only NaN codes, no inf
    assert t[0x01] == 2.0 ** -9 and t[0x07] == 7 * 2.0 ** -9  # subnormals
    assert t[0x08] == 2.0 ** -6                             # smallest normal
    assert t[0x38] == 1.0 and t[0x3C] == 1.5 and t[0x40] == 2.0
    # strictly increasing over the positive finite codes
    assert np.all(np.diff(t[:0x7F]) > 0)
    # same table from torch's decoder and from the C oracle
    tt = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.nan_to_num(tt, nan=-1.0), np.nan_to_num(t, nan=-1.0))
    tc = np.array([c_oracle.lib().oracle_e4m3_decode(c) for c in range(256)], dtype=np.float32)
    assert np.array_equal(np.nan_to_num(tc, nan=-1.0), np.nan_to_num(t, nan=-1.0))


def _interesting_fp32():
    """Every code value, every midpoint between neighbours, and one-ulp neighbours of both."""
    t = O.e4m3_decode_table()[:0x7F].astype(np.float64)
    mids = (t[:-1] + t[1:]) / 2
    base = np.concatenate([t, mids, [464.0, 479.9, 2.0 ** -10, 2.0 ** -11, 3 * 2.0 ** -10]]).astype(np.float32)
    vals = [base, np.nextafter(base, np.float32(np.inf)), np.nextafter(base, np.float32(-np.inf))]
    rng = np.random.default_rng(0)
    vals.append(rng.standard_normal(200000).astype(np.float32) * 100)
    vals.append((rng.standard_normal(100000) * 0.01).astype(np.float32))
    v = np.concatenate(vals)
    v = v[np.abs(v) < 500.0]
    return np.concatenate([v, -v])


def test_encoders_match_torch_cast():
    v = _interesting_fp32()
    want = torch.from_numpy(v).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got_np = O.e4m3_encode_rne(v)
    assert np.array_equal(got_np, want)
    L = c_oracle.lib()
    sub = v[:: max(1, v.size // 20000)]
    want_sub = torch.from_numpy(sub).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got_c = np.array([L.oracle_e4m3_encode(float(x)) for x in sub], dtype=np.uint8)
    assert np.array_equal(got_c, want_sub)


def test_encoder_ties_and_overflow():
    enc = lambda x: int(O.e4m3_encode_rne(np.array([x], dtype=np.float32))[0])
    assert enc(2.0 ** -10) == 0x00            # tie between 0 and 2^-9 -> even (0)
    assert enc(3 * 2.0 ** -10) == 0x02        # tie between 1 and 2 (x 2^-9) -> even (2)
    assert enc(1.0625) == 0x38                # tie between 1.0 and 1.125 -> even mantissa
    assert enc(1.1875) == 0x3A                # tie between 1.125 and 1.25 -> even mantissa
    assert enc(448.0) == 0x7E and enc(463.9) == 0x7E and enc(464.0) == 0x7E  # 464 ties to the even 448
    assert enc(464.0001) == 0x7F and enc(480.0) == 0x7F   # why the reference clamps before the cast
    assert enc(-0.0) == 0x80


def _c2_like(n, h, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, h, generator=g)
    mask = torch.rand(n, h, generator=g) < 0.001
    x = torch.where(mask, 50 * torch.randn(n, h, generator=g), x)
    return x


def _reference_expression(x):
    """The cast exactly as the reference spells it (ep_communications.py:65-68), as a cross-check of
    the oracle's step-by-step version through the same library ops."""
    amax = x.abs().amax(dim=-1, keepdim=True).clamp_(min=1e-4)
    scale = amax / 448.0
    q = (x.float() / scale).clamp_(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q.view(torch.uint8), scale.squeeze(-1).float()


def test_quant_three_ways_bf16():
    x = _c2_like(64, 512).bfloat16()
    x[3] = 0                      # all-zero row hits the 1e-4 floor
    x[5] *= 1e-6                  # tiny row, floor again
    x[7, 11] = 3.0e38             # huge outlier
    q_ref, s_ref = _reference_expression(x)
    q_t, s_t = O.quant_fp8(x, encoder="torch")
    q_b, s_b = O.quant_fp8(x, encoder="bits")
    q_c, s_c = c_oracle.quant_rows_bf16(x.view(torch.int16).numpy().view(np.uint16))
    for q, s in ((q_t, s_t), (q_b, s_b), (torch.from_numpy(q_c), torch.from_numpy(s_c))):
        assert torch.equal(q, q_ref)
        assert torch.equal(s, s_ref)
    # the floor, in bf16, is 0x38D2
    assert s_ref[3].item() == (torch.tensor(1e-4).bfloat16() / 448.0).float().item()
    assert torch.tensor(1e-4).bfloat16().view(torch.int16).item() == 0x38D2


def test_quant_fp32_rows():
    x = _c2_like(32, 256, seed=1)
    q_ref, s_ref = _reference_expression(x)
    q_b, s_b = O.quant_fp8(x, encoder="bits")
    assert torch.equal(q_b, q_ref) and torch.equal(s_b, s_ref)


def test_dequant_and_round_trip_error():
    x = _c2_like(256, 1024, seed=2).bfloat16()
    q, s = O.quant_fp8(x)
    d = O.dequant_fp8(q, s, torch.bfloat16)
    want = q.view(torch.float8_e4m3fn).to(torch.bfloat16) * s.unsqueeze(-1).to(torch.bfloat16)  # ep_communications.py:100
    assert torch.equal(d, want)
    d_c = c_oracle.dequant_rows_bf16(q.numpy(), s.numpy())
    assert np.array_equal(d_c, d.view(torch.int16).numpy().view(np.uint16))
    # dequantised magnitude never exceeds the row amax; relative L2 error in the range the reference reports
    assert torch.all(d.float().abs().amax(-1) <= x.float().abs().amax(-1).clamp_min(1e-4) * 1.005)  # scale is bf16-rounded (2^-9 relative)
    plain = torch.randn(256, 1024, generator=torch.Generator().manual_seed(3)).bfloat16()
    qp, sp = O.quant_fp8(plain)
    rel = ((O.dequant_fp8(qp, sp, torch.bfloat16).float() - plain.float()).norm() / plain.float().norm()).item()
    assert 0.01 < rel < 0.05, rel


def test_wire_bytes_per_row():
    x = torch.randn(4, 4096).bfloat16()
    q, s = O.quant_fp8(x)
    assert q.element_size() * q.shape[1] + s.element_size() == 4100  # README.md:316, test_fp8_dispatch.py:78
