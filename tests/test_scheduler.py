"""Sampler (pkg/sampler/sampler.go) and the scheduler's bookkeeping: the C++ host code against its oracle
restatement. CPU only; the scheduler loop over a real model is in test_gpu_model.py."""
import numpy as np
import pytest

from oracle import host_logic as hl


@pytest.fixture(scope="module")
def host():
    from vexel_amd.runtime import load_host
    import ctypes as C
    h = load_host()
    h.vh_argmax.argtypes = [C.c_void_p, C.c_int]
    h.vh_sample.argtypes = [C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_float, C.c_float]
    return h


def test_argmax_rules(host):
    """sampler.go:80-91: ties go to the lowest index, NaN never wins, all -inf gives 0."""
    cases = [[1.0, 3.0, 3.0, 2.0], [float("nan"), 1.0, float("nan"), 1.0], [-float("inf")] * 4, [5.0], [-1e30, -3.4e38]]
    wants = [1, 1, 0, 0, 0]
    for c, want in zip(cases, wants):
        a = np.array(c, dtype=np.float32)
        assert hl.sampler_argmax(a) == want
        assert host.vh_argmax(a.ctypes.data, a.size) == want


def test_sampler_known_answers(host):
    """Closed cases: greedy at temperature 0; top_k = 1 and a tiny top_p reduce to the argmax whatever r is; with
    uniform logits and no filter the draw r picks index floor(r * n) (to float32 rounding of the running sum)."""
    rng = np.random.default_rng(1)
    logits = rng.standard_normal(50).astype(np.float32)
    best = int(np.argmax(logits))
    for r in (0.0, 0.3, 0.999):
        assert host.vh_sample(logits.ctypes.data, 50, 0.0, 0, 0.0, r) == best
        assert host.vh_sample(logits.ctypes.data, 50, 0.8, 1, 0.0, r) == best
        assert host.vh_sample(logits.ctypes.data, 50, 0.8, 0, 1e-6, r) == best
    flat = np.zeros(8, dtype=np.float32)
    for r, want in ((0.0, 0), (0.13, 1), (0.51, 4), (0.99, 7)):
        assert host.vh_sample(flat.ctypes.data, 8, 1.0, 0, 0.0, r) == want
        assert hl.sampler_sample(flat, 1.0, 0, 0.0, r) == want


def test_sampler_matches_oracle(host):
    """Random logits, every combination of filters, many draws: the same index as the oracle restatement."""
    rng = np.random.default_rng(2)
    for trial in range(40):
        n = int(rng.integers(2, 300))
        logits = (rng.standard_normal(n) * rng.uniform(0.5, 6)).astype(np.float32)
        if trial % 5 == 0:
            logits[rng.integers(0, n, 3)] = logits.max()          # ties at the top
        for temperature, top_k, top_p in ((1.0, 0, 0.0), (0.7, 40, 0.9), (0.3, 5, 0.0), (1.5, 0, 0.5), (0.9, n + 3, 1.0)):
            for r in rng.uniform(0, 1, 6).astype(np.float32):
                want = hl.sampler_sample(logits, temperature, top_k, top_p, float(r))
                got = host.vh_sample(logits.ctypes.data, n, temperature, top_k, top_p, float(r))
                assert got == want, (trial, temperature, top_k, top_p, float(r))
