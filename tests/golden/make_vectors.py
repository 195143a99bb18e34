"""Writes the committed fixtures of this directory from the CPU checker (oracle/), not from the
reference: `python tests/golden/make_vectors.py`.

  known_answers.json  values fixed by the reference's own files or by published constants
                      (utils.h:13-18 SplitMix64 finaliser; optim.h:28-43 OneCycle; tests/verify.py:108-127
                      small-update case; bf16 round-to-nearest-even / truncation bit patterns)
  tiny_model.npz      one forward + backward of a 1-block model (d 128, T 128, B 2) on seeded inputs:
                      the inputs' seeds, the logits, the per-position loss, per-tensor gradient norms and 512
                      sampled gradient entries, as the fp32 checker computes them

The tests use them twice: the checker must reproduce them (it cannot drift unnoticed), and the GPU engine
must match them without the checker being rebuilt on the GPU machine."""
import json
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
HERE = Path(__file__).resolve().parent

TINY = dict(depth=1, context=128, batch=2, d_model=128, heads=2)


def tiny_inputs(oracle):
    cfg = oracle.model(TINY["depth"], TINY["context"], TINY["batch"], TINY["d_model"], TINY["heads"])
    w = oracle.init_weights(cfg, seed=42, scale=0.45 / np.sqrt(TINY["d_model"]))
    rng = np.random.default_rng(71)
    x = rng.integers(0, 256, (TINY["batch"], TINY["context"]), dtype=np.uint8)
    y = rng.integers(0, 256, x.shape, dtype=np.uint8)
    return cfg, w, x, y


def main():
    import oracle
    known = {
        "hash_u64": {"0": "0xe220a8397b1dcdaf", "3407": "0x655ec498465366b7"},
        "onecycle_total20": {"0": [0.04, 0.95], "5": [1.0, 0.85], "10": [0.716943001791, 0.878305813044],
                             "19": [4e-6, 0.95]},
        "bf16_round_to_nearest_even": {"0x3f808000": "0x3f80", "0x3f818000": "0x3f82", "0x3f808001": "0x3f81",
                                       "0x7f7fffff": "0x7f80", "0xbf808000": "0xbf80"},
        "bf16_truncate": {"0x3f80ffff": "0x3f80", "0xbf81ffff": "0xbf81"},
        "small_update": {"weight": 0.5, "gradient": 0.01, "learning_rate": 1e-5, "steps": 64,
                         "minimum_change": 5e-4},
    }
    (HERE / "known_answers.json").write_text(json.dumps(known, indent=1) + "\n")

    cfg, w, x, y = tiny_inputs(oracle)
    logits, grad, losses = oracle.model_batch(cfg, w, x, y)
    layout = oracle.Layout(cfg)
    names = [name for name, _, _ in layout.entries]
    norms = np.array([np.linalg.norm(grad[off:off + int(np.prod(shape))].astype(np.float64))
                      for _, off, shape in layout.entries])
    picks = np.random.default_rng(5).choice(grad.size, 512, replace=False).astype(np.int64)
    np.savez_compressed(HERE / "tiny_model.npz", logits=logits.astype(np.float32).reshape(-1, 256),
                        losses=losses.astype(np.float32), gradient_norms=norms, gradient_names=np.array(names),
                        gradient_index=picks, gradient_value=grad[picks].astype(np.float32),
                        parameter_count=np.int64(grad.size))
    print("wrote", HERE / "known_answers.json", HERE / "tiny_model.npz")


if __name__ == "__main__":
    main()
