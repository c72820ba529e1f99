"""The reference's own decoder running on the MI355X backend.

oracle/_ref holds the reference's Decoder (embedding, norms, mixers, residual adds, the
MoE loop: src/models/qwen35/decoder.cpp) compiled from its sources, and a Projections
whose two methods forward to C function pointers.  Handed gufo_model_apply and
gufo_model_apply_expert, the decoder's every matrix product runs on the GPU through
the model-level C-ABI, which is the swap a maintainer of the reference makes:
`Decoder decoder(file, hip_projections)` in place of `Decoder decoder(file,
gguf_projections)`.  The checker is the same decoder over the reference's
GgufProjections in double.

Bars: the greedy token (first maximum of the logits) identical at every step; logits
within rel-L2 1e-4 of the double-precision run after the whole stack of layers.  The
distance of the reference's own fp32 path from the same run is printed beside it."""
import ctypes as C
import time

import numpy as np
import pytest

import gguf_cases
from gufo_npu_amd import model as hip_model

pytestmark = pytest.mark.gpu

TOKENS = [5, 17, 400, 3, 999, 42, 7, 7, 123, 0, 650, 31]


def say(*args):
    print(*args, flush=True)


@pytest.mark.parametrize("name", list(gguf_cases.MODELS))
def test_reference_decoder_over_hip_projections(name, tmp_path, hip, ref_oracle):
    path, spec = gguf_cases.write_model(name, tmp_path)
    say("decoder", name)
    reference = ref_oracle.RefModel(path)
    device = hip_model.Model(path)
    lib = hip_model.load_library()
    exact = ref_oracle.RefDecoder(reference, "double")
    fused = ref_oracle.RefDecoder(reference, "float")
    ours = ref_oracle.RefDecoder(reference, "foreign",
                                 (device.handle, lib.gufo_model_apply,
                                  lib.gufo_model_apply_expert))
    worst, worst_fused = 0.0, 0.0
    for step, token in enumerate(TOKENS):
        say("  step", step, "token", token)
        want = exact.step(token)
        cpu = fused.step(token)
        got = ours.step(token)
        err, err_fused = ref_oracle.rel_l2(got, want), ref_oracle.rel_l2(cpu, want)
        worst, worst_fused = max(worst, err), max(worst_fused, err_fused)
        assert int(np.argmax(got)) == int(np.argmax(want)), (step, err)
        assert err <= 1e-4, (step, err)
    # Every product of every step went through the backend: per layer the input stage,
    # mixer_out, ffn_in and ffn_down, for a mixture layer also the router and two calls
    # per chosen expert, and the head once per step.
    per_layer = 4 + (1 + 2 * spec.experts_used if spec.is_moe else 0)
    assert ours.foreign_calls == len(TOKENS) * (spec.layers * per_layer + 1)
    say(f"  worst rel-L2 vs double: backend {worst:.2e}, reference fp32 path {worst_fused:.2e}")

    # Timing, for the record only: the decoder's host work (mixers, norms) is the
    # reference's in both runs; the products differ.
    for label, decoder in (("reference fp32 projections", fused), ("MI355X projections", ours)):
        decoder.reset()
        start = time.perf_counter()
        for token in TOKENS:
            decoder.step(token)
        elapsed = time.perf_counter() - start
        say(f"  {label}: {len(TOKENS) / elapsed:.0f} steps/s on this toy model")
    for decoder in (exact, fused, ours):
        decoder.close()
    device.close()
    reference.close()


def test_full_size_decode_rate(tmp_path, hip, ref_oracle):
    # The same swap on a model with the 2B decode set's widths (24 layers, hidden 2048,
    # FFN 6144, 151,936-row head; 1.2 GB of synthetic weights): greedy tokens against the
    # reference's fp32 path, and the decode rate of the reference's decoder with its own
    # CPU projections and with the MI355X ones, host mixers and host-pointer copies
    # included.  The rates are printed for the record; only parity is asserted.
    from gufo_npu_amd import gguf_writer
    spec = gguf_writer.dense_2b_like()
    path = tmp_path / "dense_2b_like.gguf"
    say("writing", path)
    gguf_writer.write_model(path, spec)
    say("written")
    reference = ref_oracle.RefModel(path)
    device = hip_model.Model(path)
    say(f"  {device.weight_bytes / 1e9:.2f} GB of projection weights in HBM")
    lib = hip_model.load_library()
    fused = ref_oracle.RefDecoder(reference, "float")
    ours = ref_oracle.RefDecoder(reference, "foreign",
                                 (device.handle, lib.gufo_model_apply,
                                  lib.gufo_model_apply_expert))
    token_cpu = token_gpu = 11
    worst = 0.0
    for step in range(6):
        say("  step", step)
        cpu, got = fused.step(token_cpu), ours.step(token_gpu)
        worst = max(worst, ref_oracle.rel_l2(got, cpu))
        token_cpu, token_gpu = int(np.argmax(cpu)), int(np.argmax(got))
        assert token_cpu == token_gpu, step
    assert worst <= 1e-4
    say(f"  worst rel-L2 between the two paths: {worst:.2e}")
    rates = {}
    for label, decoder in (("reference fp32 projections", fused), ("MI355X projections", ours)):
        decoder.reset()
        token = 11
        steps = 8 if decoder is fused else 32
        start = time.perf_counter()
        for _ in range(steps):
            token = int(np.argmax(decoder.step(token)))
        rates[label] = steps / (time.perf_counter() - start)
        say(f"  {label}: {rates[label]:.1f} tokens/s")
    for decoder in (fused, ours):
        decoder.close()
    device.close()
    reference.close()


def test_foreign_failure_reaches_the_caller(tmp_path, hip, ref_oracle):
    # A status code from the backend surfaces as the exception a Projections consumer
    # expects, and the decoder stays usable: here the backend is handed a null model.
    path, _ = gguf_cases.write_model("tiny_dense", tmp_path)
    reference = ref_oracle.RefModel(path)
    lib = hip_model.load_library()
    broken = ref_oracle.RefDecoder(reference, "foreign",
                                   (C.c_void_p(None), lib.gufo_model_apply,
                                    lib.gufo_model_apply_expert))
    say("decoder over a null model")
    with pytest.raises(RuntimeError):
        broken.step(1)
    broken.close()
    reference.close()
