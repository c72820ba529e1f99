"""Writes tests/golden/gguf/<model>.npz: what the reference's own GgufProjections returns
for every stage of the synthetic model files (tests/gguf_cases.py).

Runs where the reference sources are present: it needs oracle/_ref/libgufo_ref.so, the
reference's GGUF reader, ReadConfig and GgufProjections compiled from its sources by
oracle/Makefile.  The model files are rebuilt from their seeds wherever the tests run;
only the reference's outputs are stored: per call the Precision::kDouble result
("exact") and the Precision::kFloat one ("fused"), TOKENS rows each, and the Config
fields the reference read from the file.

    python tests/golden/make_gguf_golden.py
"""
import sys
import tempfile
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

import __graft_entry__ as entry  # noqa: E402

entry.load_package()
oracle = entry.load_oracle()

import gguf_cases  # noqa: E402


def main() -> None:
    out_dir = ROOT / "tests" / "golden" / "gguf"
    out_dir.mkdir(parents=True, exist_ok=True)
    with tempfile.TemporaryDirectory() as tmp:
        for name in gguf_cases.MODELS:
            path, spec = gguf_cases.write_model(name, Path(tmp))
            model = oracle.RefModel(path)
            config = dict(model.config)
            arrays = {"config_fields": np.array([config[f] for f in oracle.CONFIG_FIELDS],
                                                dtype=np.int32),
                      "rms_eps": np.array([config["rms_eps"]], dtype=np.float32)}
            for stage, layer, expert in gguf_cases.calls(spec):
                x = gguf_cases.call_input(oracle, config, stage, layer, expert)
                outputs = oracle.stage_outputs(config, stage, layer)
                key = gguf_cases.call_key(stage, layer, expert)
                arrays[key + "_exact"] = model.apply(stage, layer, x, outputs, expert, exact=True)
                arrays[key + "_fused"] = model.apply(stage, layer, x, outputs, expert)
            model.close()
            np.savez_compressed(out_dir / f"{name}.npz", **arrays)
            print(f"{name}: {len(arrays) - 2} reference outputs -> {out_dir / (name + '.npz')}")


if __name__ == "__main__":
    main()
