"""Timing probes of matrix and vector instruction issue on the GPU (tests/issue_probe.hip, built into
tests/libissueprobe.so): the measurements the fused and distance kernels were shaped by, kept as a
test so that they can be repeated.  Report only: the probes must launch and finish, the rates
are printed (run with `-s` to see the table; the figures the kernels were designed by are recorded
under profiles/) and nothing is asserted about them, since they depend on the clock the box holds
and a parity run must not turn red for that.  The file sorts after the parity tests.

 * a loop of nothing but v_mfma_f32_32x32x2_f32 runs close to the published fp32 matrix peak;
 * vector instructions placed between the matrix instructions, on registers of their own, are not
   hidden behind them: the loop takes longer by about their own issue time;
 * the fused kernel's filter (a tree of v_min3 and two compares per 32 x 32 tile) costs time on top
   of the matrix instructions of its tiles.
"""
import ctypes
import os

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
PEAK_FP32_MATRIX = 157.3e12   # flop/s, published
NOMINAL_CLOCK = 2.4e9         # Hz, the clock the published peak is quoted at
FLOPS_PER_MFMA = 32 * 32 * 2 * 2
CHAIN, FMA, PAIRS, PAIRS_FILTERED = 0, 1, 2, 3


@pytest.fixture(scope="module")
def probe():
    path = os.path.join(HERE, "libissueprobe.so")
    if not os.path.exists(path):
        pytest.fail(f"{path} is missing: build it with `make -C bits-knn-jpdc2024_amd probe`")
    import torch
    lib = ctypes.CDLL(path)
    lib.issue_probe_run.restype = ctypes.c_int
    lib.issue_probe_run.argtypes = [ctypes.c_int] * 5 + [ctypes.c_void_p, ctypes.POINTER(ctypes.c_double),
                                                         ctypes.c_void_p]
    dev = torch.device("cuda:0")
    scratch = torch.zeros(1 << 18, dtype=torch.float32, device=dev)
    units = torch.cuda.get_device_properties(dev).multi_processor_count
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def run(kind, param, workgroups_per_cu, iters):
        """seconds for `iters` loop iterations in every wave (best of 3 launches)"""
        best = None
        for _ in range(3):
            ms = ctypes.c_double(0.0)
            status = lib.issue_probe_run(kind, param, workgroups_per_cu, units, iters, scratch.data_ptr(),
                                         ctypes.byref(ms), stream)
            assert status == 0, (kind, param, status)
            best = ms.value if best is None else min(best, ms.value)
        return best * 1e-3

    run.units = units
    return run


def test_matrix_instructions_alone_reach_the_peak(probe):
    iters = 20000
    print()
    rates = {}
    for waves in (1, 2):
        for chains in (1, 2, 4):
            seconds = probe(CHAIN, chains, waves, iters)
            mfmas = probe.units * 4.0 * waves * iters * chains
            rate = mfmas * FLOPS_PER_MFMA / seconds
            rates[(waves, chains)] = rate / PEAK_FP32_MATRIX
            print(f"matrix instructions only, {waves} wave(s) per SIMD x {chains} chain(s): "
                  f"{rate / 1e12:6.1f} TFLOP/s = {rate / PEAK_FP32_MATRIX:.3f} of the peak, "
                  f"{seconds * NOMINAL_CLOCK / (waves * iters * chains):.1f} cycles per instruction and SIMD at 2.4 GHz")
    assert all(rate > 0 for rate in rates.values())


def test_vector_instructions_are_not_hidden_behind_matrix_instructions(probe):
    iters = 20000
    print()
    seconds = {}
    for v in (0, 2, 4, 8):
        seconds[v] = probe(FMA, v, 2, iters)
        per_pair = seconds[v] * NOMINAL_CLOCK / (2 * iters)
        print(f"two matrix instructions + 2 x {v} independent v_fma_f32 per iteration, 2 waves per SIMD: "
              f"{per_pair:6.1f} cycles per iteration and SIMD at 2.4 GHz (matrix instructions alone: 128)")
    # 16 vector instructions per 128 cycles of matrix instructions: fully hidden they would cost
    # nothing, issued in turn they add 64 cycles
    assert all(value > 0 for value in seconds.values())


def test_the_filter_costs_time_on_top_of_the_matrix_instructions(probe):
    iters = 4000
    print()
    for steps in (4, 8, 16):
        for waves in (2, 3):
            plain = probe(PAIRS, steps, waves, iters)
            filtered = probe(PAIRS_FILTERED, steps, waves, iters)
            to_cycles = NOMINAL_CLOCK / (waves * iters)
            print(f"pairs of tiles of {steps:2d} matrix instructions, {waves} waves per SIMD: "
                  f"{plain * to_cycles:7.1f} cycles per pair and SIMD without the filter, "
                  f"{filtered * to_cycles:7.1f} with it (matrix instructions alone: {128 * steps})")
            assert plain > 0 and filtered > 0
