"""A recorded sequence of products replayed several times (gufo_hip_capture_begin /
_end, gufo_hip_graph_launch: the role of the NPU backend's Chain,
src/npu/gemv.hpp:299-331 of the reference), with fresh inputs and ordinary calls between
the replays: every replay must give what the same calls give when made one by one, bit for
bit.  Covers every kind of device-resident entry point, so that none of them records
anything a replay does not repeat faithfully."""
import numpy as np
import pytest

from gufo_npu_amd import synth

pytestmark = pytest.mark.gpu

EPS = 1e-6


def say(*args):
    print(*args, flush=True)


def same_bits(a, b) -> bool:
    return bool(np.array_equal(np.ascontiguousarray(a).view(np.uint8),
                               np.ascontiguousarray(b).view(np.uint8)))


class Sequence:
    """One layer's worth of calls on device buffers: residual add + norm + [gate | up],
    SwiGLU + down, routing + routed experts, the head with the pick inside, a small
    prefill product."""

    def __init__(self, hip, tokens):
        self.hip, self.tokens = hip, tokens
        hidden, ffn, experts, expert_ffn, vocab = 512, 768, 16, 256, 3000
        self.shape = dict(hidden=hidden, ffn=ffn, experts=experts, k=4, vocab=vocab)
        seed = synth.BASE_SEED + 8800
        make = lambda t, rows, cols, s: hip.Matrix(t, synth.matrix(t, rows, cols, seed + s),
                                                  rows, cols)
        self.gate = make(synth.Q4_K, ffn, hidden, 1)
        self.up = make(synth.Q4_K, ffn, hidden, 2)
        self.down = make(synth.Q6_K, hidden, ffn, 3)
        self.router = make(synth.F32, experts, hidden, 4)
        self.router_gate = make(synth.F32, experts + 1, hidden, 10)
        self.gate_exps = make(synth.Q4_K, experts * expert_ffn, hidden, 5)
        self.up_exps = make(synth.Q4_K, experts * expert_ffn, hidden, 6)
        self.down_exps = make(synth.Q5_K, experts * hidden, expert_ffn, 7)
        self.head = make(synth.Q6_K, vocab, hidden, 8)
        self.prefill = make(synth.Q4_K, 256, hidden, 9)
        norm = (1.0 + 0.1 * np.random.default_rng(seed).standard_normal(hidden))
        self.norm = hip.DeviceBuffer.from_array(norm.astype(np.float32))
        f = lambda n: hip.DeviceBuffer(4 * tokens * n)
        self.h, self.delta, self.h1, self.normed = f(hidden), f(hidden), f(hidden), f(hidden)
        self.gate_up, self.ffn_out = f(2 * ffn), f(hidden)
        self.logits, self.moe_out, self.layer_out = f(experts), f(hidden), f(hidden)
        self.ids, self.weights = hip.DeviceBuffer(4 * tokens * 4), hip.DeviceBuffer(4 * tokens * 4)
        self.token = hip.DeviceBuffer(8 * tokens)
        self.a16 = hip.DeviceBuffer(2 * 64 * hidden)
        self.c = hip.DeviceBuffer(4 * 64 * 256)

    def upload(self, seed):
        hidden = self.shape["hidden"]
        self.h.upload(synth.activations(self.tokens, hidden, seed))
        self.delta.upload(0.5 * synth.activations(self.tokens, hidden, seed + 1))
        self.a16.upload(synth.bf16_round(synth.activations(64, hidden, seed + 2)))

    def enqueue(self):
        hip, n, s = self.hip, self.tokens, self.shape
        hip.gemv_fused_dev([hip.whole(self.gate), hip.whole(self.up)],
                           hip.resnorm_prologue(self.norm, EPS, self.delta, self.h1, self.normed),
                           self.h, n, self.gate_up)
        hip.gemv_fused_dev([hip.whole(self.down)], hip.swiglu_prologue(), self.gate_up, n,
                           self.ffn_out)
        hip.gemv_dev([hip.whole(self.router)], self.normed, n, self.logits)
        hip.route_topk_dev(self.logits, n, s["experts"], s["k"], self.ids, self.weights)
        hip.moe_ffn_dev(self.gate_exps, self.up_exps, self.down_exps, s["experts"], self.normed,
                        n, self.ids, self.weights, s["k"], self.moe_out)
        # the whole mixture layer in one call, over the dense FFN's output as shared expert
        hip.moe_layer_dev(self.router_gate, self.gate_exps, self.up_exps, self.down_exps,
                          s["experts"], s["k"], self.normed, n, self.ffn_out, self.layer_out)
        hip.gemv_argmax_dev([hip.whole(self.head)],
                            hip.resnorm_prologue(self.norm, EPS, self.ffn_out), self.h1, n,
                            self.token)
        hip.gemm_q4k_bf16_dev(self.prefill, self.a16, 64, self.c)

    def results(self):
        n, s = self.tokens, self.shape
        self.hip.synchronize()
        return {
            "h1": self.h1.download((n, s["hidden"]), np.float32),
            "gate_up": self.gate_up.download((n, 2 * s["ffn"]), np.float32),
            "ffn_out": self.ffn_out.download((n, s["hidden"]), np.float32),
            "ids": self.ids.download((n, s["k"]), np.int32),
            "weights": self.weights.download((n, s["k"]), np.float32),
            "moe_out": self.moe_out.download((n, s["hidden"]), np.float32),
            "layer_out": self.layer_out.download((n, s["hidden"]), np.float32),
            "token": self.token.download((n,), np.int64),
            "c": self.c.download((64, 256), np.float32),
        }

    def clear_outputs(self):
        for b in (self.h1, self.normed, self.gate_up, self.ffn_out, self.logits, self.moe_out,
                  self.layer_out,
                  self.ids, self.weights, self.token, self.c):
            b.upload(np.zeros(b.nbytes, dtype=np.uint8))


@pytest.mark.parametrize("tokens", [1, 4])
def test_replays_equal_the_calls_made_one_by_one(hip, tokens):
    seq = Sequence(hip, tokens)
    say("graph, tokens", tokens, ": an ordinary pass (scratch is allocated outside a recording)")
    seq.upload(1)
    seq.enqueue()
    seq.results()
    say("  recording")
    hip.capture_begin()
    seq.enqueue()
    graph = hip.capture_end()
    for replay in range(4):
        say("  replay", replay)
        seq.upload(100 + replay)
        seq.enqueue()                       # the reference result, call by call
        want = seq.results()
        seq.clear_outputs()
        # Ordinary work between the replays, on other buffers.
        other = hip.gemv([hip.whole(seq.head)], synth.activations(2, 512, 7 + replay), 2)
        assert other.shape == (2, 3000)
        graph.launch()
        got = seq.results()
        for name in want:
            assert same_bits(got[name], want[name]), (replay, name)
        assert int(want["token"].min()) >= 0
    graph.destroy()


def test_a_recording_cannot_grow_scratch(hip):
    # A call that needs more library scratch than has been allocated cannot be recorded:
    # the library says so instead of allocating inside the recording.
    cols, rows = 2048, 256
    m = hip.Matrix(synth.Q4_K, synth.matrix(synth.Q4_K, rows, cols, 3), rows, cols)
    tokens = 16384  # 64 MB of fp16 activations: more than any other test's product needs
    a = hip.DeviceBuffer(2 * tokens * cols)
    c = hip.DeviceBuffer(4 * tokens * rows)
    say("recording a call that needs new scratch")
    hip.capture_begin()
    with pytest.raises(hip.LogicError):
        hip.gemm_q4k_bf16_dev(m, a, tokens, c)
    graph = hip.capture_end()
    graph.destroy()
    for b in (a, c):
        b.free()
    m.destroy()
