"""Writes the greedy tokens of the full-size models as the CPU oracle runner produces them, with the gap
between the two largest logits of every step:

  4b   tests/golden/qwen3_4b_synthetic_greedy.json — BASELINE config 2: the 36-layer Qwen3-4B-shaped model
       over synthetic LLVQ weights of seed 0, a 512-token prompt, 256 new tokens.  About four minutes on 16
       host threads and 60 GB of memory (the 252 matrices are decoded to dense weights on the CPU first).
  14b  tests/golden/qwen3_14b_q8kv_synthetic_greedy.json — the 40-layer Qwen3-14B-shaped model of BASELINE
       config 4 with its int8 KV cache, a 96-token prompt, 32 new tokens (the config's 8192-token context
       would take the oracle hours).  About ten minutes and 170 GB.

Needs no GPU.  Run from the repository root:
    python tests/golden/make_full_size_tokens.py 4b|14b [output path]
tests/test_gpu_decoder.py::test_full_size_greedy_tokens_match_the_oracle_fixture compares the device
loop with the files."""
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from llvq_amd import artifact, decoder  # noqa: E402  (host-side model description and synthetic weights only)
from oracle import pyoracle as orc, qwen3_oracle  # noqa: E402

SEED = 0
MODELS = {  # name -> (config, prompt tokens, new tokens, file)
    "4b": (decoder.QWEN3_4B, 512, 256, "qwen3_4b_synthetic_greedy.json"),
    "14b": (decoder.QWEN3_14B, 96, 32, "qwen3_14b_q8kv_synthetic_greedy.json"),
}


def main():
    which = sys.argv[1] if len(sys.argv) > 1 else "4b"
    cfg, N_PROMPT, N_NEW, fname = MODELS[which]
    t0 = time.time()
    raws = decoder.synthetic_projections(cfg, SEED)
    weights = decoder.synthetic_weights(cfg, SEED)
    dense = []
    for li, layer in enumerate(raws):
        dense.append([orc.read_matrix_raw(artifact.write_matrix_raw(m))[0].decode_matrix() for m in layer])
        print(f"decoded layer {li + 1} of {len(raws)} on the CPU, {time.time() - t0:.0f} s", flush=True)
    ref = qwen3_oracle.Qwen3Oracle(cfg, dense, weights, kv_mode=cfg.kv_mode)
    del dense
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
    out = {"model": f"Qwen3-{which.upper()} shape, synthetic LLVQ projections and dense weights of seed 0 (llvq_amd.decoder), "
                    f"KV cache {cfg.kv_mode}",
           "prompt_seed": SEED, "prompt_tokens": N_PROMPT, "tokens": tokens, "top_two_gap": gaps, "max_abs_logit": tops}
    path = sys.argv[2] if len(sys.argv) > 2 else os.path.join(ROOT, "tests", "golden", fname)
    with open(path, "w") as f:
        json.dump(out, f)
    print("wrote", path, flush=True)


if __name__ == "__main__":
    main()
