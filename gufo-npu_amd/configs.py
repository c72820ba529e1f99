"""The measured workloads: shapes, quantization types and seeds.

One definition serves the bench, the parity tests and the script that writes the
golden fixtures, so all three build identical inputs.  Shapes follow the synthetic
configurations this backend is measured on (Qwen3.5-2B-like decode set,
Qwen3.5-4B-like MTP-verify FFN, Qwen3.6-35B-A3B-like experts, a prefill projection).
"""
from __future__ import annotations

from dataclasses import dataclass

from . import synth

Q4_K, Q5_K, Q6_K = synth.Q4_K, synth.Q5_K, synth.Q6_K
SEED = synth.BASE_SEED


@dataclass(frozen=True)
class MatrixSpec:
    name: str
    ggml_type: int
    rows: int
    cols: int
    seed: int

    @property
    def nbytes(self) -> int:
        return self.rows * synth.row_bytes(self.ggml_type, self.cols)

    def build(self):
        return synth.kquant_matrix(self.ggml_type, self.rows, self.cols, self.seed)


# config 1: one Q4_K GEMV.
CONFIG1 = MatrixSpec("w", Q4_K, 6144, 2048, SEED + 1)
CONFIG1_X_SEED = SEED + 101

# config 2: the decode matvec set at N = 1 (hidden 2048).
HIDDEN2, FFN2, VOCAB2 = 2048, 6144, 151936
CONFIG2 = {
    "q": MatrixSpec("q", Q4_K, 2048, HIDDEN2, SEED + 20),
    "k": MatrixSpec("k", Q4_K, 512, HIDDEN2, SEED + 21),
    "v": MatrixSpec("v", Q4_K, 512, HIDDEN2, SEED + 22),
    "o": MatrixSpec("o", Q4_K, 2048, HIDDEN2, SEED + 23),
    "gate": MatrixSpec("gate", Q4_K, FFN2, HIDDEN2, SEED + 24),
    "up": MatrixSpec("up", Q4_K, FFN2, HIDDEN2, SEED + 25),
    "down": MatrixSpec("down", Q6_K, HIDDEN2, FFN2, SEED + 26),
    "lm_head": MatrixSpec("lm_head", Q6_K, VOCAB2, HIDDEN2, SEED + 29),
}
# Stage -> the matrices that share its input, in output order (the grouping of
# qwen35::Stage, src/models/qwen35/projections.hpp:14-39 of the reference).
CONFIG2_STAGES = {
    "attention_in": ["q", "k", "v"],
    "mixer_out": ["o"],
    "ffn_in": ["gate", "up"],
    "ffn_down": ["down"],
    "lm_head": ["lm_head"],
}
CONFIG2_X_SEED = SEED + 70      # hidden-wide inputs
CONFIG2_ACT_SEED = SEED + 71    # ffn-wide input of ffn_down


def config2_bytes(stages=None) -> int:
    names = [n for s in (stages or CONFIG2_STAGES) for n in CONFIG2_STAGES[s]]
    return sum(CONFIG2[n].nbytes for n in names)


# config 3: MTP speculative-verify FFN (hidden 2560), N = 2, 3, 4.
HIDDEN3, FFN3 = 2560, 9216
CONFIG3 = {
    "gate": MatrixSpec("gate", Q4_K, FFN3, HIDDEN3, SEED + 31),
    "up": MatrixSpec("up", Q4_K, FFN3, HIDDEN3, SEED + 32),
    "down": MatrixSpec("down", Q6_K, HIDDEN3, FFN3, SEED + 33),
}
CONFIG3_X_SEED = SEED + 130     # + tokens
CONFIG3_ACT_SEED = SEED + 140   # + tokens

# config 4: MoE experts (hidden 2048, expert FFN 512, 256 experts, top-8).
EXPERTS4, HIDDEN4, FFN4, TOPK4 = 256, 2048, 512, 8
CONFIG4 = {
    "gate": MatrixSpec("gate_exps", Q4_K, EXPERTS4 * FFN4, HIDDEN4, SEED + 41),
    "up": MatrixSpec("up_exps", Q4_K, EXPERTS4 * FFN4, HIDDEN4, SEED + 42),
    "down": MatrixSpec("down_exps", Q5_K, EXPERTS4 * HIDDEN4, FFN4, SEED + 43),
}
CONFIG4_LOGIT_SEED = SEED + 150  # + tokens
CONFIG4_X_SEED = SEED + 160      # + tokens
# x is scaled so that the SwiGLU stays in a realistic range.
CONFIG4_X_SCALE = 0.02

# config 5: prefill projection, activations 4096 x 2048 bf16.
CONFIG5 = MatrixSpec("w", Q4_K, 6144, 2048, SEED + 51)
CONFIG5_TOKENS = 4096
CONFIG5_A_SEED = SEED + 170
