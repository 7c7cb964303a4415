"""Writes tests/golden/qwen3_14b_widths_q8kv_8192_logits.npz: the CPU oracle runner's logits at the end of an
8192-position context for a model with BASELINE config 4's widths and cache in one piece — hidden 5120,
40 query heads over 8 kv heads of 128, intermediate 17408 (the 17 408-wide down_proj rows), int8 KV cache —
cut to 2 layers and a vocabulary of 2048 so that the oracle can follow.  Rows: the last prompt position
(8186 tokens of seed 41), then six more positions fed the tokens of seed 42.

The prompt goes through the oracle's matrix-form pass (Qwen3Oracle.prefill_rows, which
tests/test_oracle_runner.py holds against the token-by-token form), the six further positions through
forward_token over the cache that pass left.  About 15 minutes on 8 host threads and 25 GB.

Needs no GPU.  Run from the repository root:
    python tests/golden/make_config4_logits.py [output path]
tests/test_gpu_decoder.py::test_config4_widths_and_context_against_the_oracle compares the device loop
with the file."""
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from llvq_amd import artifact, decoder  # noqa: E402  (host-side model description and synthetic weights only)
from oracle import pyoracle as orc, qwen3_oracle  # noqa: E402

CFG = decoder.Qwen3Config(num_hidden_layers=2, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                          head_dim=128, intermediate_size=17408, vocab_size=2048, rope_theta=1e6, rms_norm_eps=1e-6,
                          max_positions=8192, tie_word_embeddings=False, kv_mode="q8")
MODEL_SEED, PROMPT_SEED, MORE_SEED, N_PROMPT, N_MORE = 41, 41, 42, 8186, 6


def main():
    t0 = time.time()
    raws = decoder.synthetic_projections(CFG, MODEL_SEED)
    weights = decoder.synthetic_weights(CFG, MODEL_SEED)
    dense = []
    for li, layer in enumerate(raws):
        dense.append([orc.read_matrix_raw(artifact.write_matrix_raw(m))[0].decode_matrix() for m in layer])
        print(f"decoded layer {li + 1} of {len(raws)} on the CPU, {time.time() - t0:.0f} s", flush=True)
    ref = qwen3_oracle.Qwen3Oracle(CFG, dense, weights, kv_mode=CFG.kv_mode)
    del dense
    tokens = np.random.default_rng(PROMPT_SEED).integers(0, CFG.vocab_size, size=N_PROMPT)
    more = np.random.default_rng(MORE_SEED).integers(0, CFG.vocab_size, size=N_MORE)
    rows = [ref.prefill_rows(tokens, progress=lambda L: print(f"prompt rows through layer {L + 1}, {time.time() - t0:.0f} s", flush=True))]
    for t in more:
        rows.append(ref.forward_token(int(t)))
        print(f"position {ref.pos}, {time.time() - t0:.0f} s", flush=True)
    path = sys.argv[1] if len(sys.argv) > 1 else os.path.join(ROOT, "tests", "golden", "qwen3_14b_widths_q8kv_8192_logits.npz")
    np.savez(path, logits=np.asarray(rows, np.float32), model_seed=MODEL_SEED, prompt_seed=PROMPT_SEED, more_seed=MORE_SEED,
             n_prompt=N_PROMPT)
    print("wrote", path, flush=True)


if __name__ == "__main__":
    main()
