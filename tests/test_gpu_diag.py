"""The diagnostic MFMA loop (``picomoe_diag_mfma_loop``): it launches, finishes and performs the FLOP the library says,
with and without pauses; a pause costs at least its own length."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _time(fn, n=3):
    fn()
    torch.cuda.synchronize()
    st, en = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    st.record()
    for _ in range(n):
        fn()
    en.record()
    torch.cuda.synchronize()
    return st.elapsed_time(en) / n


@pytest.mark.parametrize("shape", [0, 1, 2])
def test_mfma_loop_runs_and_counts_its_flop(gpu, shape):
    from picotron_amd import _lib

    lib = _lib.load()
    n_blocks = torch.cuda.get_device_properties(gpu).multi_processor_count
    data = torch.randn(1 << 20, device=gpu).bfloat16() if shape < 2 else torch.randint(0, 120, (1 << 21,), device=gpu, dtype=torch.uint8)
    nbytes = data.numel() * data.element_size()
    sink = torch.zeros(1, device=gpu)
    iters = 400
    flop = lib.picomoe_diag_mfma_loop_flop(shape, iters, n_blocks)
    per_wave = {0: 64 * 2 * 16 * 16 * 32, 1: 32 * 2 * 32 * 32 * 16, 2: 32 * 2 * 16 * 16 * 128}[shape]
    assert flop == per_wave * 8 * iters * n_blocks
    run = lambda burst, idle: _lib.check(
        lib.picomoe_diag_mfma_loop(_lib.ptr(data), nbytes, shape, iters, burst, idle, n_blocks, _lib.ptr(sink), _lib.stream_ptr()), "diag")
    ms = _time(lambda: run(0, 0))
    rate = flop / ms / 1e9
    peak = 2500.0 if shape < 2 else 5000.0
    print(f"shape {shape}: {ms:.3f} ms, {rate:.0f} TFLOP/s", flush=True)
    assert 0.3 * peak < rate < 1.02 * peak          # the matrix pipes are what runs, and nothing beats the datasheet
    ms_paused = _time(lambda: run(40, 20))           # 10 pauses of 20 us
    assert ms_paused > ms + 0.9 * 10 * 20e-3 * 0.5   # the pauses show (at least half of them: the clock rises meanwhile)
    assert float(sink) == 0.0
    # refused: misaligned operands, unknown shape, a burst length that does not divide the iterations
    bad = lambda *a: lib.picomoe_diag_mfma_loop(*a, _lib.stream_ptr())
    assert bad(_lib.ctypes.c_void_p(data.data_ptr() + 2), nbytes - 2, shape, iters, 0, 0, n_blocks, None) == 1
    assert bad(_lib.ptr(data), nbytes, 7, iters, 0, 0, n_blocks, None) == 1
    assert bad(_lib.ptr(data), nbytes, shape, iters, 33, 5, n_blocks, None) == 1
