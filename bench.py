#!/usr/bin/env python3
"""Benchmark of the single-GPU MoE hot path on MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c5|c3|c4|c2|train_step]

A "step" is one pass of the hot path over one batch of synthetic input.  The default workload is the
Mixtral-shape MoE layer forward + backward with FP8 dispatch (8192 tokens, hidden 4096, FFN 14336, 8 experts,
top-2, bf16, aux-loss coefficient 0.01): zero_grad, forward, backward of loss = <out, g> + aux -- every gradient
the reference's autograd produces (input, router, 3 x 8 expert matrices) is computed inside the timed region.
Inputs and weights are resident in HBM before the clock starts.

`--workload train_step` instead times a whole optimizer step (forward, cross entropy + aux, backward, AdamW) of a
4-layer Llama whose feed-forward blocks are this MoE layer, the set-up of the reference's tests/bench_ep_train_step.py.

`--workload c2` times the FP8 quantise / dequantise round trip of a 16384 x 4096 bf16 activation on its own, with an
HBM `roofline` for the quantise kernel and the scalar C oracle as `cpu_baseline`.

Prints ONE JSON line on stdout: the layer's tokens/s as `value`, a `roofline` object for the grouped-GEMM
kernels (algorithmic FLOP / launch durations measured here with events on the launch stream), the FP8
quantise bandwidth and a `cpu_baseline` (the CPU oracle timed on this box's host cores on a bounded sample).
"""

import argparse
import json
import os
import sys
import time
import types

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
# L2 <-> memory bytes per step (c5: the grouped-GEMM launches of one layer step; c2: the quantise kernel alone), from
# two rocprofv3 --pmc runs of this script (FETCH_SIZE, WRITE_SIZE; scale factors from the --traffic-probe copy kernel).
# A counter run cannot happen inside a timed run, so the figure is carried here together with the digest of the kernel
# sources it was measured on: `traffic` is reported only while the sources are still those, otherwise it is null.
MEASURED_TRAFFIC = {
    "c5": {"bytes": 35.3e9, "algorithmic_bytes": 15.5e9, "sources": "6a7e161c91880ec2",
           "files": ("ffn_mfma.hip", "mfma_tiles.h", "ffn.h", "common.h"),
           "summary": "profiles/ffn_mfma_kernel_mixtral_hbm_traffic.txt"},
    "c2": {"bytes": 201.6e6, "algorithmic_bytes": 201.4e6, "sources": "567861dc6e2a9e36",
           "files": ("fp8_quant.hip", "common.h"),
           "summary": "profiles/quant_bf16_wave_per_row_fp8_round_trip.txt"},
}


def kernel_sources_digest(files):
    """sha256 over the named HIP kernel sources (names and contents, in name order), first 16 hex digits."""
    import hashlib

    h = hashlib.sha256()
    for name in sorted(files):
        h.update(name.encode())
        with open(os.path.join(ROOT, "picotron_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload):
    """(bytes or None, provenance dict) for the `roofline.traffic` field."""
    m = MEASURED_TRAFFIC.get(workload)
    if m is None:
        return None, None
    digest = kernel_sources_digest(m["files"])
    current = m["sources"] == digest
    return (m["bytes"] if current else None), {
        "summary": m["summary"], "measured_on_sources": m["sources"], "this_build": digest, "current": current,
        "algorithmic_bytes": m["algorithmic_bytes"]}


WORKLOADS = {
    # name: tokens, hidden, ffn, experts, top_k, shared, capacity_factor, fp8_dispatch, backward
    "c5": dict(T=8192, H=4096, I=14336, E=8, k=2, shared=0, cap=0.0, fp8=True, bwd=True,
               desc="Mixtral-shape MoE layer fwd+bwd, FP8 dispatch, aux 0.01: 8192 tok, H4096, I14336, E8, top-2, bf16"),
    "c3": dict(T=8192, H=4096, I=14336, E=8, k=2, shared=0, cap=0.0, fp8=False, bwd=False,
               desc="Mixtral-shape MoE layer fwd: 8192 tok, H4096, I14336, E8, top-2, bf16"),
    "c4": dict(T=16384, H=2048, I=1408, E=64, k=6, shared=2, cap=1.25, fp8=False, bwd=False,
               desc="fine-grained skewed MoE fwd: 16384 tok, H2048, I1408, E64, top-6, shared 2816, capacity 1.25 drop"),
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_layer(w, device, dtype, shared_stream=True):
    import torch

    from picotron_amd.expert_parallel.expert_parallel import MoELayer

    cfg = types.SimpleNamespace(
        hidden_size=w["H"], intermediate_size=w["I"], num_experts=w["E"], num_experts_per_tok=w["k"],
        num_shared_experts=w["shared"], norm_topk_prob=True, ep_fp8_dispatch=w["fp8"],
        ep_capacity_factor=w["cap"], ep_capacity_dropless=False, router_aux_loss_coef=0.01 if w["bwd"] else 0.0,
        ep_overlap=shared_stream,
    )
    with torch.device("meta"):
        moe = MoELayer(cfg)
    moe = moe.to_empty(device=device).to(dtype)
    g = torch.Generator(device=device).manual_seed(0)
    with torch.no_grad():
        for p in moe.parameters():
            p.copy_((0.02 * torch.randn(p.shape, generator=g, device=device, dtype=torch.float32)).to(dtype))
        moe.expert_bias.zero_()
        if w["cap"] > 0:  # Zipf(s=1.1) router bias -> load imbalance
            moe.gate.bias = torch.nn.Parameter(
                (-1.1 * torch.log(torch.arange(1, w["E"] + 1, device=device, dtype=torch.float32))).to(dtype))
    moe.train(w["bwd"])
    return moe


def time_events(fn, iters, warm=2):
    import torch

    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    st, en = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    st.record()
    for _ in range(iters):
        fn()
    en.record()
    torch.cuda.synchronize()
    return st.elapsed_time(en) / iters  # ms


class GemmTimer:
    """Records an event pair on the launch stream around every grouped-GEMM launch of the timed steps, so the
    launch durations come from the same region the throughput figure does."""

    FLOP = {"gate_up": 4.0, "down": 2.0, "dgrad_act": 2.0, "dgrad_x": 4.0, "wgrad": 2.0}  # x routed rows x H x I

    def __init__(self):
        self.records = []
        self.enabled = False
        self.pool = []
        self.shared_mult = 1

    def prepare(self, n_events):
        """Create the events before the clock starts (creating one costs far more than recording it)."""
        import torch

        self.pool = [torch.cuda.Event(enable_timing=True) for _ in range(n_events)]
        self.ref = torch.cuda.Event(enable_timing=True)

    def start(self):
        """Marks time zero of the timed region (the launch intervals are placed on one time axis from here)."""
        self.ref.record()
        self.enabled = True

    def busy_ms(self):
        """Length of the union of the launch intervals: the time during which at least one grouped GEMM was running.
        Launches of one stream follow each other, so without a second stream this is the sum of their durations; the
        shared expert's launches run on a second stream beside the routed ones and must not be counted twice."""
        spans = sorted((self.ref.elapsed_time(st), self.ref.elapsed_time(en)) for _, _, st, en, _ in self.records)
        total, cur_s, cur_e = 0.0, None, None
        for a, b in spans:
            if cur_e is None or a > cur_e:
                if cur_e is not None:
                    total += cur_e - cur_s
                cur_s, cur_e = a, b
            else:
                cur_e = max(cur_e, b)
        if cur_e is not None:
            total += cur_e - cur_s
        return total

    def install(self):
        import torch

        from picotron_amd.expert_parallel import megakernel as mk

        def wrap(name, fn):
            def timed(*a, **kw):
                if not self.enabled:
                    return fn(*a, **kw)
                if len(self.pool) < 2:
                    return fn(*a, **kw)
                st, en = self.pool.pop(), self.pool.pop()
                st.record()
                out = fn(*a, **kw)
                en.record()
                label = name
                if name == "wgrad":  # (lhs, ld_lhs, rhs, ld_rhs, counts, E, N, P, Q, dtype, device, lhs_offset)
                    label = "wgrad_" + kw["which"]  # down, gate, up, or gate_up: both in one launch
                    n_experts, rows = a[5], a[6]
                else:  # (x, counts, weight, ...): weight [E, ., .]
                    n_experts, rows = a[2].shape[0], a[0].shape[0]
                if n_experts == 1:
                    label = "shared_" + label  # the shared expert runs the same kernels with one expert
                self.records.append((label, name, st, en, rows))
                return out
            return timed

        for name in ("gate_up", "down", "dgrad_act", "dgrad_x", "wgrad"):
            setattr(mk, "_" + name, wrap(name, getattr(mk, "_" + name)))

    def summary(self, routed_rows, H, I):
        per = {}
        for label, name, st, en, rows in self.records:
            # routed launches: the rows that reach the GEMMs (kept rows under a capacity limit); shared: all tokens
            n_rows = rows if label.startswith("shared_") else routed_rows
            i_dim = I * self.shared_mult if label.startswith("shared_") else I
            flop_per = self.FLOP[name] * (2.0 if label.endswith("wgrad_gate_up") else 1.0)
            d = per.setdefault(label, {"ms": 0.0, "n": 0, "flop": flop_per * n_rows * H * i_dim})
            d["ms"] += st.elapsed_time(en)
            d["n"] += 1
        return {k: (v["ms"] / v["n"], v["flop"], v["n"]) for k, v in per.items()}


def outlier_activation(n, h, device, seed):
    """[n, h] bf16 ~ N(0, 1) with 0.1 % of the entries replaced by outliers ~ N(0, 50): the data of the FP8 round-trip
    configuration."""
    import torch

    g = torch.Generator(device=device).manual_seed(seed)
    x = torch.randn(n, h, generator=g, device=device)
    mask = torch.rand(n, h, generator=g, device=device) < 0.001
    return torch.where(mask, 50.0 * torch.randn(n, h, generator=g, device=device), x).bfloat16()


def fp8_quant_bandwidth(device, n=16384, h=4096, sets=6, iters=60):
    """FP8 E4M3 dispatch quantise at 16384 x 4096 bf16 on the round-trip configuration's data (0.1 % outliers of
    50 sigma), rotating over buffer sets larger than the 256 MB last-level cache so the figure is HBM traffic.
    Returns (GB/s quantise, GB/s dequantise, us quantise, us dequantise)."""
    import torch

    from picotron_amd import _lib

    lib = _lib.load()
    xs = [outlier_activation(n, h, device, seed) for seed in range(sets)]
    qs = [torch.empty(n, h, dtype=torch.uint8, device=device) for _ in range(sets)]
    ss = [torch.empty(n, dtype=torch.float32, device=device) for _ in range(sets)]
    os_ = [torch.empty(n, h, dtype=torch.bfloat16, device=device) for _ in range(sets)]
    st = _lib.stream_ptr()
    state = {"i": 0}

    def quant():
        i = state["i"] = (state["i"] + 1) % sets
        lib.picomoe_fp8_quant(_lib.ptr(xs[i]), 1, n, h, _lib.ptr(qs[i]), _lib.ptr(ss[i]), st)

    def dequant():
        i = state["i"] = (state["i"] + 1) % sets
        lib.picomoe_fp8_dequant(_lib.ptr(qs[i]), _lib.ptr(ss[i]), n, h, _lib.ptr(os_[i]), 1, st)

    nbytes = n * h * 3 + n * 4
    tq = time_events(quant, iters, warm=sets)
    td = time_events(dequant, iters, warm=sets)
    return nbytes / tq / 1e6, nbytes / td / 1e6, tq * 1e3, td * 1e3


def fp8_gemm_variant(moe, step, w, steps):
    """The same layer step with the forward GEMMs on FP8 MFMA (E4M3 dispatch codes x per-row quantised weights,
    re-quantised every step as in training): first gate/up alone, then gate/up and down (the SwiGLU output quantised per
    row by one more pass).  Step times, and the FP8 kernels and the quantisers timed with events."""
    import torch

    from picotron_amd.expert_parallel import megakernel as mk

    names = ("_gate_up_fp8", "_down_fp8", "quantize_expert_weights", "_quantize_rows")
    orig = {n: getattr(mk, n) for n in names}
    state = {"on": False, "times": None, "pool": []}

    def wrap(name, fn):
        def timed(*a, **kw):
            if not state["on"] or len(state["pool"]) < 2:
                return fn(*a, **kw)
            st, en = state["pool"].pop(), state["pool"].pop()
            st.record()
            out = fn(*a, **kw)
            en.record()
            state["times"][name].append((st, en))
            return out
        return timed

    for n in names:
        setattr(mk, n, wrap(n, orig[n]))
    rows = w["T"] * w["k"]
    out = {}
    layer_step = step

    def step():
        # a training step ends in an optimizer update, which changes every weight: the cached codes are dropped as that
        # update would drop them, so the weight quantisation is inside every timed step
        moe.invalidate_fp8_weights()
        layer_step()

    try:
        for mode in (True, "all"):
            moe.ep_fp8_gemm = mode
            state["times"] = {n: [] for n in names}
            state["pool"] = [torch.cuda.Event(enable_timing=True) for _ in range(2 * 6 * steps + 8)]
            for _ in range(3):
                step()
            torch.cuda.synchronize()
            state["on"] = True
            t0 = time.perf_counter()
            for _ in range(steps):
                step()
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) * 1e3 / steps
            state["on"] = False
            per_call = lambda n: sum(a.elapsed_time(b) for a, b in state["times"][n]) / max(len(state["times"][n]), 1)
            per_step = lambda n: sum(a.elapsed_time(b) for a, b in state["times"][n]) / max(steps, 1)
            gu_ms, q_ms = per_call("_gate_up_fp8"), per_step("quantize_expert_weights")
            gu_flop = 4.0 * rows * w["H"] * w["I"]
            if mode is True:
                log(f"[bench] fp8 gate/up GEMM variant: {ms:.3f} ms/step, gate_up_fp8 {gu_ms:.2f} ms ({gu_flop / gu_ms / 1e9:.0f} TFLOP/s), "
                    f"weight quantisation {q_ms:.2f} ms/step")
                out = {"ms_per_step": ms, "tokens_per_s": w["T"] / (ms * 1e-3), "gate_up_fp8_ms": gu_ms,
                       "gate_up_fp8_tflops": gu_flop / gu_ms / 1e9, "frac_fp8_mfma_peak": gu_flop / gu_ms / 1e9 / 5000.0,
                       "weight_quant_ms_per_step": q_ms,
                       "note": "forward gate/up on v_mfma_f32_16x16x128_f8f6f4; down, dgrad and wgrad stay bf16; not the headline value"}
            else:
                # _down_fp8 = the row quantiser of the SwiGLU output + the FP8 down kernel; the kernel alone is the difference
                d_ms, aq_ms = per_call("_down_fp8"), per_call("_quantize_rows")
                k_ms = d_ms - aq_ms
                d_flop = 2.0 * rows * w["H"] * w["I"]
                log(f"[bench] fp8 gate/up + down GEMM variant: {ms:.3f} ms/step, down_fp8 {k_ms:.2f} ms ({d_flop / k_ms / 1e9:.0f} TFLOP/s) "
                    f"+ {aq_ms:.2f} ms quantising its input, weight quantisation {q_ms:.2f} ms/step")
                out["all"] = {"ms_per_step": ms, "tokens_per_s": w["T"] / (ms * 1e-3), "gate_up_fp8_ms": gu_ms,
                              "down_fp8_ms": k_ms, "down_fp8_tflops": d_flop / k_ms / 1e9,
                              "down_frac_fp8_mfma_peak": d_flop / k_ms / 1e9 / 5000.0, "act_quant_ms": aq_ms,
                              "weight_quant_ms_per_step": q_ms,
                              "note": "forward gate/up and down on FP8 MFMA (SwiGLU output quantised per row); dgrad and wgrad stay bf16"}
    finally:
        state["on"] = False
        moe.ep_fp8_gemm = False
        for n in names:
            setattr(mk, n, orig[n])
    return out


MFMA_NOMINAL_CLOCK_GHZ = 2.4   # the shader clock the datasheet peaks are quoted at


def mfma_ceiling(device, launches=8):
    """What the matrix pipes sustain on this box under its power limit: the library's MFMA-only loop
    (`picomoe_diag_mfma_loop`: one block of 8 wavefronts per CU, 32 independent accumulator blocks per wavefront, no
    memory traffic inside the loop) on random operands, and on all-zero operands for scale.  TFLOP/s per MFMA shape,
    each from `launches` back-to-back launches of about 5 ms between two events on the launch stream."""
    import torch

    from picotron_amd import _lib

    lib = _lib.load()
    n_blocks = torch.cuda.get_device_properties(device).multi_processor_count
    g = torch.Generator(device=device).manual_seed(7)
    rand16 = torch.randn(8 << 20, generator=g, device=device).bfloat16()
    # random E4M3 codes, the two NaN codes (0x7F, 0xFF) replaced by 1.0
    rand8 = torch.randint(0, 256, (16 << 20,), generator=g, device=device, dtype=torch.int16).to(torch.uint8)
    rand8 = torch.where((rand8 & 0x7F) == 0x7F, torch.full_like(rand8, 0x38), rand8)
    zeros = torch.zeros(16 << 20, dtype=torch.uint8, device=device)
    st = _lib.stream_ptr()
    out = {}
    for name, shape, data, iters in (("bf16_16x16x32", 0, rand16, 5000), ("bf16_32x32x16", 1, rand16, 5000),
                                     ("fp8_16x16x128", 2, rand8, 5000), ("bf16_16x16x32_zero_operands", 0, zeros, 5000)):
        nbytes = data.numel() * data.element_size()
        flop = lib.picomoe_diag_mfma_loop_flop(shape, iters, n_blocks)

        def launch():
            _lib.check(lib.picomoe_diag_mfma_loop(_lib.ptr(data), nbytes, shape, iters, 0, 0, n_blocks, None, st), "picomoe_diag_mfma_loop")

        ms = time_events(launch, launches, warm=3)
        out[name] = flop / ms / 1e9
    # What a pause is worth: bursts of 40 iterations (about 40 us, the length of a k-loop of some 25 k-steps) with every
    # block idle for 5 / 10 / 20 us between them.  If the power limit alone set the pace the average rate would not move
    # (the clock would rise to use the budget the pause saves); if the clock did not react it would fall by the idle share.
    nbytes, iters, burst = rand16.numel() * 2, 4800, 40
    flop = lib.picomoe_diag_mfma_loop_flop(0, iters, n_blocks)
    duty = {}
    for idle_us in (5, 10, 20):
        def launch():
            _lib.check(lib.picomoe_diag_mfma_loop(_lib.ptr(rand16), nbytes, 0, iters, burst, idle_us, n_blocks, None, st), "picomoe_diag_mfma_loop")

        ms = time_events(launch, launches, warm=3)
        busy_ms = ms - (iters // burst) * idle_us * 1e-3
        duty[f"idle_{idle_us}us_per_40_iterations"] = {
            "average_tflops": flop / ms / 1e9, "tflops_inside_bursts": flop / busy_ms / 1e9, "idle_share": 1.0 - busy_ms / ms,
            "share_of_the_idle_time_won_back": 1.0 - (1.0 - flop / ms / 1e9 / out["bf16_16x16x32"]) / (1.0 - busy_ms / ms)}
    out["bursts_bf16_16x16x32"] = duty
    return out, n_blocks


def hipblaslt_dense(device, rows, H, I, iters=10):
    """The vendor comparator: the gate/up and the down GEMM of the layer as ONE dense library GEMM each over all routed
    rows (one weight matrix instead of one per expert, no SwiGLU, no ragged segments), `torch.nn.functional.linear` =
    hipBLASLt, on N(0, 1) activations and N(0, 0.02) weights.  TFLOP/s."""
    import torch

    g = torch.Generator(device=device).manual_seed(8)
    x = torch.randn(rows, H, generator=g, device=device).bfloat16()
    w13 = (0.02 * torch.randn(2 * I, H, generator=g, device=device)).bfloat16()
    t_gu = time_events(lambda: torch.nn.functional.linear(x, w13), iters, warm=3)
    del w13, x
    act = torch.randn(rows, I, generator=g, device=device).bfloat16()
    w2 = (0.02 * torch.randn(H, I, generator=g, device=device)).bfloat16()
    t_d = time_events(lambda: torch.nn.functional.linear(act, w2), iters, warm=3)
    return {"gate_up": 4.0 * rows * H * I / t_gu / 1e9, "down": 2.0 * rows * H * I / t_d / 1e9,
            "gate_up_ms": t_gu, "down_ms": t_d}


def cpu_baseline(w, moe, budget_s=25.0):
    """The CPU oracle (port of the reference's naive torch path) on this box's host cores, on a token-subsampled
    batch of the same layer shape (same H / I / E / k and the same weights)."""
    import torch

    from oracle import moe_oracle as O

    # the box's CPU share for one GPU is 16 cores, whatever os.cpu_count() shows; OMP_NUM_THREADS says so there
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")), 16)
    torch.set_num_threads(cores)
    c = lambda t: t.detach().to("cpu")
    ow = O.LayerWeights(
        c(moe.gate.weight), c(moe._stacks[0]) if moe._stacks else None, None, None,
        router_b=c(moe.gate.bias) if moe.gate.bias is not None else None,
    )
    ow.up_w, ow.down_w = c(moe._stacks[1]), c(moe._stacks[2])
    if moe.shared_expert is not None:
        s = moe.shared_expert
        ow.shared = (c(s.gate_proj.weight), c(s.up_proj.weight), c(s.down_proj.weight))

    def run(tokens):
        x = torch.randn(tokens, w["H"], generator=torch.Generator().manual_seed(0)).bfloat16()
        if w["bwd"]:
            for t in ow.tensors():
                t.requires_grad_(True)
                t.grad = None
            x.requires_grad_(True)
        t0 = time.perf_counter()
        out, info = O.moe_forward(x, ow, w["k"], fp8_dispatch=w["fp8"], capacity_factor=w["cap"], capacity_dropless=False,
                                  aux_coef=0.01 if w["bwd"] else 0.0, training=w["bwd"])
        if w["bwd"]:
            loss = (out.float() * torch.ones_like(out, dtype=torch.float32)).sum() + info["aux"]
            loss.backward()
        return time.perf_counter() - t0

    # grow the sample (x4 per round, up to the full batch) while the next round is predicted to fit the budget
    tokens = max(w["T"] // 64, 64)
    t = run(tokens)
    spent = t
    log(f"[cpu_baseline] {tokens} tokens: {t:.2f} s")
    while tokens * 4 <= w["T"] and spent + 4 * t < budget_s:
        tokens *= 4
        t = run(tokens)
        spent += t
        log(f"[cpu_baseline] {tokens} tokens: {t:.2f} s")
    return {
        "value": tokens / t, "unit": "tokens/s", "cores": cores, "kind": "port",
        "sample": f"{tokens} of {w['T']} tokens (same H/I/E/top-k and weights), one {'fwd+bwd' if w['bwd'] else 'fwd'} "
                  f"pass of the CPU oracle in {t:.2f} s ({spent:.1f} s of CPU work in all, growing samples)",
    }


def traffic_probe(device):
    """A plain copy kernel of known size (1 GiB read + 1 GiB written per launch, three launches): the reference that
    rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings of the other kernels are scaled by."""
    import torch

    src = torch.ones(1 << 29, dtype=torch.bfloat16, device=device)
    dst = torch.empty_like(src)
    for _ in range(3):
        torch.neg(src, out=dst)
    torch.cuda.synchronize()


def fp8_bench(args):
    """FP8 E4M3 per-token quantise / dequantise of a 16384 x 4096 bf16 activation (0.1 % outliers of 50 sigma), the
    dispatch wire format of the reference (picotron/expert_parallel/ep_communications.py:63-68, :100).  A step is one
    quantise and one dequantise pass over one of six buffer sets (rotated, so every pass comes from HBM and not from
    the 256 MB last-level cache)."""
    import numpy as np
    import torch

    from picotron_amd import _lib

    lib = _lib.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    device = torch.device("cuda:0")
    n, h, sets = 16384, 4096, 6
    xs = [outlier_activation(n, h, device, seed) for seed in range(sets)]
    qs = [torch.empty(n, h, dtype=torch.uint8, device=device) for _ in range(sets)]
    ss = [torch.empty(n, dtype=torch.float32, device=device) for _ in range(sets)]
    ys = [torch.empty(n, h, dtype=torch.bfloat16, device=device) for _ in range(sets)]
    st = _lib.stream_ptr()
    state = {"i": 0}

    def quant():
        i = state["i"] = (state["i"] + 1) % sets
        _lib.check(lib.picomoe_fp8_quant(_lib.ptr(xs[i]), 1, n, h, _lib.ptr(qs[i]), _lib.ptr(ss[i]), st), "fp8 quantise")

    def dequant():
        i = state["i"]
        _lib.check(lib.picomoe_fp8_dequant(_lib.ptr(qs[i]), _lib.ptr(ss[i]), n, h, _lib.ptr(ys[i]), 1, st), "fp8 dequantise")

    def step():
        quant()
        dequant()

    for _ in range(max(args.warmup, sets)):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    pass_bytes = n * h * 3 + n * 4
    # launch durations of each kernel on its own: back-to-back launches between two events on the launch stream
    tq = time_events(quant, 60, warm=sets)
    td = time_events(dequant, 60, warm=sets)
    if args.traffic_probe:
        traffic_probe(device)
    rel = float(((ys[0].float() - xs[0].float()).norm() / xs[0].float().norm()).item())
    log(f"[bench] c2: {ms * 1e3:.1f} us per quantise+dequantise step; quantise {tq * 1e3:.1f} us = "
        f"{pass_bytes / tq / 1e6:.0f} GB/s, dequantise {td * 1e3:.1f} us = {pass_bytes / td / 1e6:.0f} GB/s, round-trip rel-L2 {rel:.4f}")
    result = {
        "metric": "FP8 quant GB/s (per-token E4M3 quantise + dequantise round trip, algorithmic bytes)",
        "value": 2 * pass_bytes / ms / 1e6, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": "FP8 round trip: 16384 x 4096 bf16 -> e4m3 + fp32 row scale -> bf16, 0.1 % outliers",
                   "rows": n, "hidden": h, "bytes_per_pass": pass_bytes, "round_trip_rel_l2": rel},
        "roofline": {"bound": "hbm", "achieved": pass_bytes / tq / 1e6, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": pass_bytes / tq / 1e6 / HBM_PEAK_GBPS, "traffic": measured_traffic("c2")[0],
                     "traffic_source": measured_traffic("c2")[1],
                     "kernel": "quant_bf16_wave_per_row", "us": tq * 1e3,
                     "dequant": {"kernel": "dequant_bf16_wave_per_row", "achieved": pass_bytes / td / 1e6,
                                 "frac": pass_bytes / td / 1e6 / HBM_PEAK_GBPS, "us": td * 1e3}},
    }
    if not args.no_cpu_baseline:
        from oracle import c_oracle

        cores = 1
        rows = 4096  # a quarter of the batch: the scalar C port needs about a second for it
        bits = xs[0][:rows].cpu().view(torch.int16).numpy().view(np.uint16)
        t0 = time.perf_counter()
        q, scale = c_oracle.quant_rows_bf16(bits)
        c_oracle.dequant_rows_bf16(q, scale)
        t = time.perf_counter() - t0
        same = bool((torch.from_numpy(q) == qs[0][:rows].cpu()).all())  # every set was quantised in the timed loop
        result["cpu_baseline"] = {
            "value": 2 * (rows * h * 3 + rows * 4) / t / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"{rows} of {n} rows, one quantise + dequantise pass of the scalar C oracle in {t:.2f} s",
        }
        result["cpu_baseline"]["bytes_equal_gpu"] = same
    print(json.dumps(result), flush=True)


def train_step_bench(args):
    """One optimizer step of a small Llama with MoE feed-forward blocks, the recipe and default sizes of the
    reference's tests/bench_ep_train_step.py:27-44, 54-60, 82-93 (hidden 2048, FFN 2048, 4 layers, 16 heads / 4 kv
    heads, 8 experts top-2 + 1 shared, sequence 2048, micro-batch 1, vocabulary 32000, bf16, AdamW lr 1e-4)."""
    import torch
    import torch.nn.functional as F

    from picotron_amd import _lib
    from picotron_amd.expert_parallel.expert_parallel import collect_aux_loss
    from picotron_amd.model import Llama

    _lib.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    cfg = types.SimpleNamespace(
        vocab_size=32000, hidden_size=2048, intermediate_size=2048, num_attention_heads=16, num_key_value_heads=4,
        num_hidden_layers=4, max_position_embeddings=2048, rms_norm_eps=1e-5, rope_theta=10000.0, num_experts=8,
        num_experts_per_tok=2, num_shared_experts=1, norm_topk_prob=True, ep_overlap=not args.no_shared_stream)
    seq, mbs = 2048, 1
    torch.manual_seed(0)
    model = Llama(cfg).to(torch.bfloat16).cuda().train()
    # fused=True: one pass over the 626 M parameters instead of the default implementation's seven (measured: 8.1 ms
    # of a 19.1 ms step went to the unfused update)
    optimizer = torch.optim.AdamW(model.parameters(), lr=1e-4, fused=True, capturable=args.hip_graph)
    torch.manual_seed(42)
    input_ids = torch.randint(0, cfg.vocab_size, (mbs, seq), device="cuda")
    target_ids = torch.randint(0, cfg.vocab_size, (mbs, seq), device="cuda")

    def step():
        optimizer.zero_grad(set_to_none=True)
        logits = model(input_ids)
        loss = F.cross_entropy(logits.view(-1, logits.size(-1)).float(), target_ids.view(-1))
        aux = collect_aux_loss(model)
        if aux is not None:
            loss = loss + aux.float()
        loss.backward()
        optimizer.step()
        return loss

    if args.hip_graph:
        # The whole optimizer step as one HIP graph: at this size the step is a few hundred launches of 5-100 us each and
        # the host cannot keep the GPU fed; captured once, a step is one graph launch.  (Nothing in the MoE layer
        # synchronises with the host or allocates outside torch's allocator, so it captures as it is, second stream included.)
        args.no_kernel_times = True          # events cannot be read out of a replayed graph
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        optimizer.zero_grad(set_to_none=True)
        with torch.cuda.graph(graph):
            static_loss = step()

        def step():
            graph.replay()
            return static_loss

    timer = GemmTimer()
    if not args.no_kernel_times:
        timer.install()
    for _ in range(args.warmup):
        step()
    if not args.no_kernel_times:
        timer.prepare(2 * 60 * args.steps)   # 4 layers x (7 routed + 7 shared-expert launches) per step
    torch.cuda.synchronize()
    if not args.no_kernel_times:
        timer.start()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    timer.enabled = False
    n_params = sum(p.numel() for p in model.parameters())
    log(f"[bench] train_step: {ms:.3f} ms/step, {mbs * seq / ms * 1e3:,.0f} tokens/s, loss {float(loss.detach()):.3f}")
    moe_gemms = None
    if not args.no_kernel_times and timer.records:
        # the expert GEMMs of the four MoE layers: 18 x rows x hidden x FFN FLOP for the routed rows and for the shared expert's
        rows = mbs * seq
        flop = 4 * 18.0 * (rows * cfg.num_experts_per_tok + rows * cfg.num_shared_experts) * cfg.hidden_size * cfg.intermediate_size
        busy = timer.busy_ms() / args.steps
        total = sum(st.elapsed_time(en) for _, _, st, en, _ in timer.records) / args.steps
        moe_gemms = {"busy_ms_per_step": busy, "sum_of_launch_ms_per_step": total, "launches_per_step": len(timer.records) / args.steps,
                     "flop_per_step": flop, "tflops": flop / busy / 1e9,
                     "what": "grouped-GEMM launches of the 4 MoE layers (routed + shared expert); busy = time with at least one of them running"}
        log(f"[bench] MoE expert GEMMs: {busy:.3f} ms/step busy ({total:.3f} ms summed over {len(timer.records) // args.steps} launches), "
            f"{flop / busy / 1e9:.0f} TFLOP/s")
    print(json.dumps({
        "metric": "Llama-MoE train-step tokens/s (fwd + loss + bwd + AdamW, 1 GPU)", "value": mbs * seq / (ms * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "4-layer Llama, MoE feed-forward (hidden 2048, FFN 2048, 8 experts top-2 + 1 shared), "
                               "seq 2048 x mbs 1, vocab 32000, fused AdamW", "tokens": mbs * seq, "parameters": n_params,
                   "shared_expert_on_second_stream": not args.no_shared_stream, "hip_graph": bool(args.hip_graph)},
        "moe_expert_gemms": moe_gemms,
    }), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c5", choices=sorted(WORKLOADS) + ["c2", "train_step"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-times", action="store_true")
    ap.add_argument("--no-shared-stream", action="store_true",
                    help="run the shared expert on the launch stream, after the routed path's kernels instead of beside them")
    ap.add_argument("--hip-graph", action="store_true",
                    help="train_step only: capture the whole optimizer step (forward, loss, backward, AdamW) in one HIP graph and replay it")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="after the timed steps also launch a plain 1 GiB copy kernel three times: the known-size "
                         "reference that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build targets one GPU (the EP=1 MoE hot path); run with --gpus 1")
    if args.workload == "train_step":
        return train_step_bench(args)
    if args.workload == "c2":
        return fp8_bench(args)

    import torch

    from picotron_amd import _lib
    from picotron_amd.expert_parallel.expert_parallel import collect_aux_loss

    _lib.load()  # fail loudly if the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    device = torch.device("cuda:0")
    w = WORKLOADS[args.workload]
    dtype = torch.bfloat16
    moe = build_layer(w, device, dtype, shared_stream=not args.no_shared_stream)
    gx = torch.Generator(device=device).manual_seed(2)
    x = torch.randn(1, w["T"], w["H"], generator=gx, device=device, dtype=torch.float32).to(dtype)
    upstream = torch.randn(1, w["T"], w["H"], generator=gx, device=device, dtype=torch.float32).to(dtype)
    if w["bwd"]:
        x.requires_grad_(True)

    one = torch.ones((), dtype=torch.float32, device=device)

    def step():
        if w["bwd"]:
            moe.zero_grad(set_to_none=True)
            x.grad = None
            out = moe(x)
            aux = collect_aux_loss(moe)
            # backward of loss = <out, g> + aux: d loss / d out = g, d loss / d aux = 1 (the inner product itself is not
            # part of the layer and is not formed)
            if aux is not None:
                torch.autograd.backward([out, aux], [upstream, one])
            else:
                out.backward(upstream)
        else:
            with torch.no_grad():
                moe(x)

    timer = GemmTimer()
    if not args.no_kernel_times:
        timer.install()
    for _ in range(args.warmup):
        step()
    if not args.no_kernel_times:
        timer.prepare(2 * 16 * args.steps)
    torch.cuda.synchronize()
    if not args.no_kernel_times:
        timer.start()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    timer.enabled = False
    if args.traffic_probe:
        traffic_probe(device)
    tokens_per_s = w["T"] / (ms_per_step * 1e-3)
    log(f"[bench] {args.workload}: {ms_per_step:.3f} ms/step, {tokens_per_s:,.0f} tokens/s")

    result = {
        "metric": "MoE layer tokens/s fwd+bwd (1 GPU); grouped-GEMM TFLOPS; FP8 quant GB/s",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w["desc"], "tokens": w["T"], "hidden": w["H"], "ffn": w["I"], "experts": w["E"],
                   "top_k": w["k"], "fp8_dispatch": w["fp8"], "backward": w["bwd"]},
    }

    if not args.no_kernel_times:
        # routed rows that reach the expert GEMMs (kept rows under a capacity limit); the shared expert's
        # launches are timed too but counted with their own row count
        routed_rows = w["T"] * w["k"]
        if w["cap"] > 0:  # count the kept rows from the drop mask, not the routed ones
            from picotron_amd import _ops
            from picotron_amd.expert_parallel.capacity_moe import compute_capacity

            with torch.no_grad():
                idx, _ = moe._route(x.reshape(-1, w["H"]))
                plan = _ops.permute_plan(idx.reshape(-1), w["E"], capacity=compute_capacity(w["T"], w["k"], w["E"], w["cap"]))
                routed_rows = int(plan.kept_counts.sum().item())
            result["config"]["kept_rows"] = routed_rows
        timer.shared_mult = max(w["shared"], 1)
        kt = timer.summary(routed_rows, w["H"], w["I"])
        kt = {k: (t, f) for k, (t, f, _) in kt.items()}
        # time with a grouped GEMM running, per step: the sum of the launch durations, except that launches overlapping
        # on two streams (the shared expert beside the routed path) are counted once
        sum_ms = sum(t for t, _ in kt.values())
        total_ms = timer.busy_ms() / args.steps
        total_flop = sum(f for _, f in kt.values())
        achieved = total_flop / total_ms / 1e9  # TFLOP/s
        result["roofline"] = {
            "bound": "mfma", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": measured_traffic(args.workload)[0],
            "traffic_source": measured_traffic(args.workload)[1],
            "kernel": "ffn_mfma_kernel (grouped SwiGLU GEMMs: %s)" % ", ".join(kt),
            "flop_per_step": total_flop, "gemm_ms_per_step": total_ms, "sum_of_launch_ms_per_step": sum_ms,
            # router, plan, dispatch, combine and their backward passes: what a step spends with no grouped GEMM running
            "step_minus_gemm_ms": result["ms_per_step"] - total_ms,
            "launches": {k: {"ms": t, "tflops": f / t / 1e9} for k, (t, f) in kt.items()},
        }
        log(f"[bench] grouped GEMM: {achieved:.0f} TFLOP/s over {total_ms:.2f} ms/step "
            + " ".join(f"{k}={t:.2f}ms" for k, (t, _) in kt.items()))
        # the ceiling the power limit leaves on this box, and the vendor library's dense GEMMs of the same sizes
        ceiling, n_cus = mfma_ceiling(device)
        dense = hipblaslt_dense(device, w["T"] * w["k"], w["H"], w["I"])
        best = ceiling["bf16_16x16x32"]
        result["roofline"].update({
            "power_capped_mfma_tflops": best,
            "power_capped_mfma": {"tflops": ceiling, "cus": n_cus,
                                  "implied_clock_ghz": MFMA_NOMINAL_CLOCK_GHZ * best / MFMA_BF16_PEAK_TFLOPS,
                                  "what": "picomoe_diag_mfma_loop: MFMA-only loop, 8 wavefronts per CU, random bf16 operands"},
            "frac_of_power_capped_mfma": achieved / best,
            "hipblaslt_dense_tflops": {k: dense[k] for k in ("gate_up", "down")},
            "hipblaslt_dense": {**dense, "what": "torch.nn.functional.linear (hipBLASLt), one dense GEMM over all routed rows "
                                                 "against one expert's weight matrix: x @ [gate_w; up_w].T and act @ down_w.T"},
        })
        log(f"[bench] MFMA-only loop under the power limit: " + ", ".join(f"{k} {v:.0f}" for k, v in ceiling.items() if not isinstance(v, dict))
            + f" TFLOP/s; hipBLASLt dense gate_up {dense['gate_up']:.0f}, down {dense['down']:.0f} TFLOP/s")
        qg, dg, tq, td = fp8_quant_bandwidth(device)
        result["fp8_quant"] = {"GBps": qg, "frac_hbm": qg / HBM_PEAK_GBPS, "us": tq, "dequant_GBps": dg,
                               "dequant_frac_hbm": dg / HBM_PEAK_GBPS, "dequant_us": td,
                               "shape": "16384 x 4096 bf16 (N(0,1), 0.1 % outliers of 50 sigma) -> e4m3 + fp32 scale, 201392128 B per pass"}
        log(f"[bench] fp8 quant {qg:.0f} GB/s ({tq:.1f} us), dequant {dg:.0f} GB/s ({td:.1f} us)")

    if w["fp8"] and not args.no_kernel_times:
        result["fp8_gemm"] = fp8_gemm_variant(moe, step, w, args.steps)

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(w, moe)

    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
