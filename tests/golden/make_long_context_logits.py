"""Writes tests/golden/qwen3_small_q8kv_8192_logits.npz: the CPU oracle runner's logits at the end of an
8192-position context with an int8 KV cache (BASELINE config 4's regime for the attention: heads of 128,
5 query heads per kv head; the model is otherwise small — 2 layers, hidden 256 — so that the oracle can
walk 8192 positions, which takes it about five minutes).  Rows: the last prompt position (8186 tokens of
seed 21), then six more positions fed the tokens of seed 22.

Needs no GPU.  Run from the repository root:
    python tests/golden/make_long_context_logits.py [output path]
tests/test_gpu_decoder.py::test_context_of_8192_positions_int8_cache compares the device loop with the file."""
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from llvq_amd import artifact, decoder  # noqa: E402  (host-side model description and synthetic weights only)
from oracle import pyoracle as orc, qwen3_oracle  # noqa: E402

CFG = decoder.Qwen3Config(num_hidden_layers=2, hidden_size=256, num_attention_heads=10, num_key_value_heads=2,
                          head_dim=128, intermediate_size=384, vocab_size=400, rope_theta=1e6, rms_norm_eps=1e-6,
                          max_positions=8192, tie_word_embeddings=True, kv_mode="q8")
MODEL_SEED, PROMPT_SEED, MORE_SEED, N_PROMPT, N_MORE = 21, 21, 22, 8186, 6


def main():
    t0 = time.time()
    raws = decoder.synthetic_projections(CFG, MODEL_SEED)
    weights = decoder.synthetic_weights(CFG, MODEL_SEED)
    dense = [[orc.read_matrix_raw(artifact.write_matrix_raw(m))[0].decode_matrix() for m in layer] for layer in raws]
    ref = qwen3_oracle.Qwen3Oracle(CFG, dense, weights, kv_mode=CFG.kv_mode)
    tokens = np.random.default_rng(PROMPT_SEED).integers(0, CFG.vocab_size, size=N_PROMPT)
    more = np.random.default_rng(MORE_SEED).integers(0, CFG.vocab_size, size=N_MORE)
    rows = []
    for i, t in enumerate(tokens):
        logits = ref.forward_token(int(t))
        if i % 512 == 511:
            print(f"position {i + 1} of {N_PROMPT}, {time.time() - t0:.0f} s", flush=True)
    rows.append(logits)
    for t in more:
        rows.append(ref.forward_token(int(t)))
    path = sys.argv[1] if len(sys.argv) > 1 else os.path.join(ROOT, "tests", "golden", "qwen3_small_q8kv_8192_logits.npz")
    np.savez(path, logits=np.asarray(rows, np.float32), model_seed=MODEL_SEED, prompt_seed=PROMPT_SEED, more_seed=MORE_SEED,
             n_prompt=N_PROMPT)
    print("wrote", path, flush=True)


if __name__ == "__main__":
    main()
