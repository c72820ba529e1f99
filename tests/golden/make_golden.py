"""Writes the golden fixtures of tests/golden/*.npz from the compiled reference.

Run in the authoring container (needs oracle/_ref, i.e. the reference sources):
    python tests/golden/make_golden.py
Inputs are regenerated from (seed, shape, type) by gufo-npu_amd/configs.py, so the
fixtures hold reference OUTPUTS only:
  * GEMV outputs of the reference's fused AVX2 dots (gguf_dot.hpp) driven over rows
    in MatMul's layout, and of its Dequantize followed by a double-precision sum;
  * Route's ids and weights (moe.cpp) on 64 logit rows with engineered ties;
  * the routed-expert FFN composed as Reference::Ffn composes it (reference.cpp:
    562-606) from those reference pieces: Route, the fused dots, Silu, and the
    weighted sum in slot order in double;
  * for the 151,936-row lm_head: argmax, top-8 and checksums instead of all logits;
  * for the prefill projection: a slice of C in double (64 token rows, every 8th
    output column).
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
import __graft_entry__ as entry  # noqa: E402

entry.load_package()
oracle = entry.load_oracle()
from gufo_npu_amd import configs as cfg  # noqa: E402
from gufo_npu_amd import synth  # noqa: E402

OUT = Path(__file__).resolve().parent
THREADS = 8


def ref_matmul(specs, mats, x):
    parts = [(s.ggml_type, m, 0, s.rows) for s, m in zip(specs, mats)]
    return oracle.matmul(parts, x, threads=THREADS, use_ref=True)


def ref_double(spec, mat, x):
    """Reference Dequantize, then every dot product summed in double."""
    y = np.empty((x.shape[0], spec.rows), np.float64)
    xd = x.astype(np.float64)
    step = 2048
    for r0 in range(0, spec.rows, step):
        r1 = min(spec.rows, r0 + step)
        w = oracle.dequantize(spec.ggml_type, mat[r0:r1], (r1 - r0) * spec.cols, use_ref=True)
        y[:, r0:r1] = xd @ w.reshape(r1 - r0, spec.cols).astype(np.float64).T
    return y


def config1():
    spec = cfg.CONFIG1
    w = spec.build()
    x = synth.activations(1, spec.cols, cfg.CONFIG1_X_SEED)
    np.savez(OUT / "config1_q4k_6144x2048.npz",
             y_reference_avx2=ref_matmul([spec], [w], x),
             y_reference_double=ref_double(spec, w, x).astype(np.float32))


def config2():
    out = {}
    x = synth.activations(1, cfg.HIDDEN2, cfg.CONFIG2_X_SEED)
    act = synth.activations(1, cfg.FFN2, cfg.CONFIG2_ACT_SEED)
    for stage, names in cfg.CONFIG2_STAGES.items():
        specs = [cfg.CONFIG2[n] for n in names]
        mats = [s.build() for s in specs]
        inp = act if stage == "ffn_down" else x
        y = ref_matmul(specs, mats, inp)
        if stage != "lm_head":
            out[stage] = y
            continue
        exact = ref_double(specs[0], mats[0], inp)[0]
        logits = y[0]
        top = np.argsort(-exact, kind="stable")[:8]
        out["lm_head_argmax"] = np.int64(oracle.argmax(logits))
        out["lm_head_argmax_double"] = np.int64(np.argmax(exact))
        out["lm_head_top8_index"] = top.astype(np.int64)
        out["lm_head_top8_value"] = exact[top].astype(np.float32)
        out["lm_head_sum"] = np.float64(exact.sum())
        out["lm_head_abs_sum"] = np.float64(np.abs(exact).sum())
        # every 64th logit, enough to catch a row mapped to the wrong place
        out["lm_head_every64"] = exact[::64].astype(np.float32)
    np.savez(OUT / "config2_decode_set.npz", **out)


def config3():
    out = {}
    gate, up, down = (cfg.CONFIG3[n] for n in ("gate", "up", "down"))
    wg, wu, wd = gate.build(), up.build(), down.build()
    for tokens in (2, 3, 4):
        x = synth.activations(tokens, cfg.HIDDEN3, cfg.CONFIG3_X_SEED + tokens)
        a = synth.activations(tokens, cfg.FFN3, cfg.CONFIG3_ACT_SEED + tokens)
        # every 16th output of [gate | up] keeps the file small
        out[f"gate_up_n{tokens}_every16"] = ref_matmul([gate, up], [wg, wu], x)[:, ::16]
        out[f"down_n{tokens}"] = ref_matmul([down], [wd], a)
    np.savez(OUT / "config3_mtp_verify.npz", **out)


def engineered_logits():
    logits = synth.router_logits(64, cfg.EXPERTS4, cfg.SEED + 180)
    logits[1, :] = 0.0                      # all equal
    logits[2, 40:60] = logits[2, 7]         # a run of ties
    logits[3, ::2] = 1.5                    # half the row tied at the top
    logits[4, 8:] = -900.0                  # probabilities underflow to 0
    logits[5, 200] = logits[5, 3] = logits[5].max() + 1.0  # tie for first place
    logits[6, :] = np.float32(1e-9) * np.arange(cfg.EXPERTS4, dtype=np.float32)
    return logits


def routed_ffn(gate, up, down, wg, wu, wd, logits, x):
    """Reference::Ffn's routed part from reference pieces."""
    lib = oracle.ref()
    tokens = x.shape[0]
    ids, weights = oracle.route(logits, cfg.TOPK4, use_ref=True)
    silu = np.vectorize(lambda v: lib.ref_silu(float(v)), otypes=[np.float32])
    y = np.empty((tokens, cfg.HIDDEN4), np.float32)
    routed = {}
    for e in sorted(set(ids.reshape(-1).tolist())):
        chosen = [(t, s) for t in range(tokens) for s in range(cfg.TOPK4) if ids[t, s] == e]
        xs = np.stack([x[t] for t, _ in chosen])
        gu = oracle.matmul([(gate.ggml_type, wg, e * cfg.FFN4, cfg.FFN4),
                            (up.ggml_type, wu, e * cfg.FFN4, cfg.FFN4)], xs, threads=THREADS,
                           use_ref=True)
        act = (silu(gu[:, :cfg.FFN4]) * gu[:, cfg.FFN4:]).astype(np.float32)
        out = oracle.matmul([(down.ggml_type, wd, e * cfg.HIDDEN4, cfg.HIDDEN4)], act,
                            threads=THREADS, use_ref=True)
        for r, key in enumerate(chosen):
            routed[key] = out[r]
    for t in range(tokens):
        acc = np.zeros(cfg.HIDDEN4, np.float64)
        for s in range(cfg.TOPK4):
            acc += np.float64(weights[t, s]) * routed[(t, s)].astype(np.float64)
        y[t] = acc.astype(np.float32)
    return ids, weights, y


def config4():
    out = {}
    logits = engineered_logits()
    ids, weights = oracle.route(logits, cfg.TOPK4, use_ref=True)
    out["route_ids"] = ids
    out["route_weights"] = weights
    gate, up, down = (cfg.CONFIG4[n] for n in ("gate", "up", "down"))
    wg, wu, wd = gate.build(), up.build(), down.build()
    for tokens in (1, 4):
        lg = synth.router_logits(tokens, cfg.EXPERTS4, cfg.CONFIG4_LOGIT_SEED + tokens)
        x = synth.activations(tokens, cfg.HIDDEN4, cfg.CONFIG4_X_SEED + tokens)
        x = x * np.float32(cfg.CONFIG4_X_SCALE)
        i, w, y = routed_ffn(gate, up, down, wg, wu, wd, lg, x)
        out[f"ids_b{tokens}"] = i
        out[f"weights_b{tokens}"] = w
        out[f"y_b{tokens}"] = y
        counts, offsets, pairs, distinct = oracle.moe_group(i, cfg.EXPERTS4)
        out[f"counts_b{tokens}"] = counts
        out[f"offsets_b{tokens}"] = offsets
        out[f"pairs_b{tokens}"] = pairs
        out[f"distinct_b{tokens}"] = np.int32(distinct)
    np.savez(OUT / "config4_moe.npz", **out)


def config5():
    spec = cfg.CONFIG5
    w = spec.build()
    a = synth.bf16_to_float(synth.bf16_round(
        synth.activations(cfg.CONFIG5_TOKENS, spec.cols, cfg.CONFIG5_A_SEED)))
    tokens = np.arange(0, cfg.CONFIG5_TOKENS, 64)  # 64 token rows spread over the batch
    c = ref_double(spec, w, a[tokens])
    # every 8th output column of those rows keeps the file under 200 KB
    np.savez(OUT / "config5_prefill_slice.npz", tokens=tokens.astype(np.int32),
             c_double_every8=c[:, ::8].astype(np.float32))


if __name__ == "__main__":
    if not oracle.ref_available():
        raise SystemExit("oracle/_ref is not built: the reference sources are needed")
    for step in (config1, config2, config3, config4, config5):
        print(step.__name__, flush=True)
        step()
    for f in sorted(OUT.glob("*.npz")):
        print(f.name, f.stat().st_size)
