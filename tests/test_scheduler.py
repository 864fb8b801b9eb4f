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


# ---------------------------------------------------------------- the oracle's scheduler loop, pinned by hand
class _ScriptedModel:
    """A model whose next token is a closed form of its input, so that a whole schedule can be worked out on paper:
    after a prompt chunk the winner is (sum of the chunk's tokens + start position) mod V, after a decode row
    (token + 2 * position + 1) mod V. Records every call."""
    V = 50

    class _Pool:
        def __init__(self):
            self.live = set()

        def create_sequence(self, i):
            self.live.add(i)

        def has_sequence(self, i):
            return i in self.live

        def delete_sequence(self, i):
            self.live.discard(i)

    def __init__(self):
        self.pool, self.calls = self._Pool(), []

    def _row(self, winner):
        r = np.zeros(self.V, dtype=np.float32)
        r[winner % self.V] = 1.0
        return r

    def prefill_with_paged_kv(self, tokens, seq_id, start):
        self.calls.append(("prefill", seq_id, list(tokens), start))
        return self._row(sum(tokens) + start)

    def decode_batched(self, toks, ids, pos):
        self.calls.append(("decode", list(ids), list(toks), list(pos)))
        return np.stack([self._row(t + 2 * p + 1) for t, p in zip(toks, pos)])


def test_oracle_scheduler_hand_worked_schedule():
    """hl.Scheduler against a schedule worked out by hand from the reference's rules (scheduler.go:245-483,
    sequence.go:116-141,196-219): a prompt is prefilled whole and its sequence decodes in the same step
    (runBatchedPrefill sets StateDecoding, the decode filter then takes it); a decode row feeds the last generated
    token at the sequence's position, then AdvancePosition; an empty prompt decodes from token 1 at position 0;
    the limit is checked after decode rows only, so a request limited to one token still gets two; EOS ends a
    request after the prompt (no decode row in that step) or after a decode row; at most max_batch_size sequences
    run, in ascending id. Every number below is arithmetic on the scripted model's closed forms, not a run of it."""
    m = _ScriptedModel()
    s = hl.Scheduler(m, 2, 4, 13, 0)          # two at a time, four tokens by default, EOS = 13
    s.add_sequence(1, [3, 4, 5])
    s.add_sequence(2, [])
    s.add_sequence(3, [6], 1)
    snap = lambda: {i: (q.state, q.position, list(q.generated)) for i, q in s.seqs.items()}
    # step 0: sequences 1 and 2 run. 1: prompt -> (3+4+5+0) = 12, then the decode row 12 @ 3 -> 12+6+1 = 19.
    #         2: no prompt: token 1 @ 0 -> 2.
    assert s.step() == 3
    assert m.calls == [("prefill", 1, [3, 4, 5], 0), ("decode", [1, 2], [12, 1], [3, 0])]
    assert snap() == {1: (hl.DECODING, 4, [12, 19]), 2: (hl.DECODING, 1, [2]), 3: (hl.PENDING, 0, [])}
    # step 1: 19 @ 4 -> 28; 2 @ 1 -> 5
    assert s.step() == 2
    assert m.calls[-1] == ("decode", [1, 2], [19, 2], [4, 1])
    # step 2: 28 @ 5 -> 39: the fourth token of sequence 1, which finishes; 5 @ 2 -> 10
    assert s.step() == 2
    assert snap() == {1: (hl.FINISHED, 6, [12, 19, 28, 39]), 2: (hl.DECODING, 3, [2, 5, 10]), 3: (hl.PENDING, 0, [])}
    # step 3: sequence 3 gets the free place. Its prompt -> 6, and in the same step 6 @ 1 -> 9: two tokens although
    # its limit is one (the limit is looked at after decode rows only). 2: 10 @ 3 -> 17, its fourth.
    assert s.step() == 3
    assert m.calls[-2:] == [("prefill", 3, [6], 0), ("decode", [2, 3], [10, 6], [3, 1])]
    assert snap()[2] == (hl.FINISHED, 4, [2, 5, 10, 17]) and snap()[3] == (hl.FINISHED, 2, [6, 9])
    # EOS right after the prompt: (20 + 43) mod 50 = 13. No decode row for it in that step.
    s.add_sequence(4, [20, 43])
    s.add_sequence(5, [10])                    # EOS after a decode row: prompt -> 10, then 10 @ 1 -> 13
    n_calls = len(m.calls)
    assert s.step() == 3
    assert m.calls[n_calls:] == [("prefill", 4, [20, 43], 0), ("prefill", 5, [10], 0), ("decode", [5], [10], [1])]
    assert snap()[4] == (hl.FINISHED, 2, [13]) and snap()[5] == (hl.FINISHED, 2, [10, 13])
    # nothing left to run: the finished requests are dropped and their sequences leave the pool
    assert s.step() == 0 and not s.seqs and not m.pool.live


def test_oracle_scheduler_chunked_prompt_positions():
    """prefill_chunk = 4: a 10-token prompt goes in at start positions 0, 4 and 8, one chunk per step, the sequence
    stays in the prefill state in between and does not decode; the step of the last chunk samples from that chunk's
    logits ((8 + 9) + 8 = 25) and runs the first decode row at position 10."""
    m = _ScriptedModel()
    s = hl.Scheduler(m, 2, 3, -1, 4)
    s.add_sequence(7, list(range(10)))
    assert s.step() == 0 and s.seqs[7].state == hl.PREFILL and s.seqs[7].position == 4
    assert s.step() == 0 and s.seqs[7].position == 8
    assert s.step() == 2
    assert m.calls == [("prefill", 7, [0, 1, 2, 3], 0), ("prefill", 7, [4, 5, 6, 7], 4), ("prefill", 7, [8, 9], 8),
                       ("decode", [7], [25], [10])]
    assert (s.seqs[7].state, s.seqs[7].position, s.seqs[7].generated) == (hl.DECODING, 11, [25, 25 + 20 + 1])
    assert s.step() == 1 and s.seqs[7].state == hl.FINISHED and s.seqs[7].generated[-1] == (46 + 22 + 1) % 50
