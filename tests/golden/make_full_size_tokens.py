"""Writes tests/golden/qwen3_4b_synthetic_greedy.json: the greedy tokens of BASELINE config 2 (the full
36-layer Qwen3-4B-shaped model over synthetic LLVQ weights of seed 0, a 512-token prompt, 256 new tokens)
as the CPU oracle runner produces them, with the gap between the two largest logits of every step.

Needs no GPU; takes the oracle about four minutes on 16 host threads and 30 GB of memory (the 252 matrices are
decoded to dense f32 on the CPU first).  Run from the repository root:
    python tests/golden/make_full_size_tokens.py
tests/test_gpu_decoder.py::test_full_size_greedy_tokens_match_the_oracle_fixture compares the device
loop with the file."""
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from llvq_amd import artifact, decoder  # noqa: E402  (host-side model description and synthetic weights only)
from oracle import pyoracle as orc, qwen3_oracle  # noqa: E402

SEED, N_PROMPT, N_NEW = 0, 512, 256


def main():
    cfg = decoder.QWEN3_4B
    t0 = time.time()
    raws = decoder.synthetic_projections(cfg, SEED)
    weights = decoder.synthetic_weights(cfg, SEED)
    dense = []
    for li, layer in enumerate(raws):
        dense.append([orc.read_matrix_raw(artifact.write_matrix_raw(m))[0].decode_matrix() for m in layer])
        print(f"decoded layer {li + 1} of {len(raws)} on the CPU, {time.time() - t0:.0f} s", flush=True)
    ref = qwen3_oracle.Qwen3Oracle(cfg, dense, weights)
    prompt = np.random.default_rng(SEED).integers(0, cfg.vocab_size, size=N_PROMPT)
    ref.reset()
    logits = None
    for i, t in enumerate(prompt):
        logits = ref.forward_token(int(t))
        if i % 16 == 15:
            print(f"prompt position {i + 1} of {N_PROMPT}, {time.time() - t0:.0f} s", flush=True)
    tokens, gaps, tops = [], [], []
    while True:
        order = np.argsort(logits)
        tokens.append(int(np.argmax(logits)))  # first index on ties (model.rs:1041-1073)
        gaps.append(float(logits[order[-1]] - logits[order[-2]]))
        tops.append(float(np.abs(logits).max()))
        if len(tokens) % 16 == 0:
            print(f"token {len(tokens)} of {N_NEW}, {time.time() - t0:.0f} s", flush=True)
        if len(tokens) == N_NEW:
            break
        logits = ref.forward_token(tokens[-1])
    out = {"model": "Qwen3-4B shape, synthetic LLVQ projections and dense weights of seed 0 (llvq_amd.decoder)",
           "prompt_seed": SEED, "prompt_tokens": N_PROMPT, "tokens": tokens, "top_two_gap": gaps, "max_abs_logit": tops}
    path = os.path.join(ROOT, "tests", "golden", "qwen3_4b_synthetic_greedy.json")
    if len(sys.argv) > 1:
        path = sys.argv[1]
    with open(path, "w") as f:
        json.dump(out, f)
    print("wrote", path, flush=True)


if __name__ == "__main__":
    main()
