"""Calls from several host threads at once.  The reference's Projections may be called
from several threads, their products then running one at a time
(src/models/qwen35/gguf_projections.hpp:14-16, the mutex of gguf_projections.cpp:253);
the library does the same under its own mutex, and every caller must get exactly what it
would have got alone - the host-pointer entry points share staging buffers, so a lock
released too early would mix the callers' rows."""
import threading

import numpy as np
import pytest

from gufo_npu_amd import synth

pytestmark = pytest.mark.gpu


def say(*args):
    print(*args, flush=True)


def same_bits(a, b) -> bool:
    return bool(np.array_equal(np.ascontiguousarray(a).view(np.uint8),
                               np.ascontiguousarray(b).view(np.uint8)))


def test_concurrent_callers_get_their_own_results(hip):
    say("threads")
    hidden, ffn, experts, k = 512, 256, 8, 2
    seed = synth.BASE_SEED + 9100
    dense = [hip.Matrix(t, synth.matrix(t, rows, hidden, seed + i), rows, hidden)
             for i, (t, rows) in enumerate([(synth.Q4_K, 768), (synth.Q6_K, 300),
                                            (synth.Q8_0, 128), (synth.F32, 64)])]
    gate = hip.Matrix(synth.Q4_K, synth.kquant_matrix(synth.Q4_K, experts * ffn, hidden, seed + 10),
                      experts * ffn, hidden)
    up = hip.Matrix(synth.Q4_K, synth.kquant_matrix(synth.Q4_K, experts * ffn, hidden, seed + 11),
                    experts * ffn, hidden)
    down = hip.Matrix(synth.Q5_K, synth.kquant_matrix(synth.Q5_K, experts * hidden, ffn, seed + 12),
                      experts * hidden, ffn)

    def work(worker, step):
        """One call of a kind that depends on (worker, step); returns its result arrays."""
        s = seed + 100 * worker + step
        kind = (worker + step) % 4
        if kind == 0:
            tokens = 1 + (step % 4)
            return (hip.gemv([hip.whole(dense[step % 2]), hip.whole(dense[(step + 1) % 2])]
                             if step % 3 == 0 else [hip.whole(dense[step % 4])],
                             synth.activations(tokens, hidden, s), tokens),)
        if kind == 1:
            return hip.route_topk(synth.router_logits(3, 64, s), 6)
        if kind == 2:
            tokens = 1 + (step % 5)
            ids, weights = hip.route_topk(synth.router_logits(tokens, experts, s), k)
            x = synth.activations(tokens, hidden, s + 1) * np.float32(0.05)
            return (hip.moe_ffn(gate, up, down, experts, x, ids, weights),)
        bits = synth.bf16_round(synth.activations(40, hidden, s))
        return (hip.gemm_bf16(dense[step % 3], bits),)

    workers, steps = 6, 24
    alone = [[work(w, s) for s in range(steps)] for w in range(workers)]

    together = [[None] * steps for _ in range(workers)]
    errors = []
    start = threading.Barrier(workers)

    def run(w):
        try:
            start.wait()
            for s in range(steps):
                together[w][s] = work(w, s)
        except Exception as e:  # reported below, in the test's own thread
            errors.append((w, repr(e)))

    threads = [threading.Thread(target=run, args=(w,)) for w in range(workers)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert errors == []
    for w in range(workers):
        for s in range(steps):
            for got, want in zip(together[w][s], alone[w][s]):
                assert same_bits(got, want), (w, s)
    for m in dense + [gate, up, down]:
        m.destroy()
