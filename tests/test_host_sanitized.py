"""The library's host code under AddressSanitizer and UBSan (host only; no GPU): the file readers on
every prefix and on corrupted copies of a sealed file, the shared index decoder on boundaries and
random ranks, the rotation tables on served and awkward widths, the batched launch's work sharing, and the
table behind the last eight slots of the odd-coset walk against an independent lexicographic enumeration.  Reader refusals are pinned case by case elsewhere; this run is about never faulting."""
import os
import subprocess

import numpy as np
import pytest

from llvq_amd import artifact, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "llvq_amd", "csrc")


def test_readers_and_decoder_under_sanitizers(tmp_path):
    exe = tmp_path / "host_fuzz"
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
           "-fno-omit-frame-pointer", "-o", str(exe), os.path.join(ROOT, "tests", "host_fuzz.cpp"),
           os.path.join(CSRC, "artifact.cpp"), os.path.join(CSRC, "codebook.cpp"), os.path.join(CSRC, "rotation.cpp")]
    built = subprocess.run(cmd, capture_output=True, text=True)
    if built.returncode != 0 and "sanitize" in built.stderr and "cannot find" in built.stderr:
        pytest.skip("the sanitizer runtimes are not installed with this g++")
    assert built.returncode == 0, built.stderr[-2000:]

    mats = [synth.make_matrix("model.layers.0.self_attn.q_proj.weight", 16, 104, seed=1),
            synth.make_matrix("model.layers.0.mlp.down_proj.weight", 8, 72, seed=2)]
    mats[1].rotation_seed = 7
    rng = np.random.default_rng(0)
    raws = [artifact.RawTensor("model.norm.weight", [32], data=rng.standard_normal(32).astype(np.float16).view(np.uint16)),
            artifact.RawTensor("model.embed_tokens.weight", [6, 128], bits=8, group=64,
                               packed=rng.integers(0, 256, size=6 * 128, dtype=np.uint8),
                               scales=rng.standard_normal(12).astype(np.float16).view(np.uint16),
                               biases=rng.standard_normal(12).astype(np.float16).view(np.uint16))]
    blobs = [artifact.Blob("config.json", b'{"hidden_size": 32}'), artifact.Blob("tokenizer.json", b"{}")]
    path = tmp_path / "sealed.llvq"
    path.write_bytes(artifact.write_file(mats, version=4, raws=raws, blobs=blobs))

    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", LD_PRELOAD="")
    run = subprocess.run([str(exe), str(path), "12345", "4000"], capture_output=True, text=True, env=env, timeout=600)
    assert run.returncode == 0, (run.stdout[-500:], run.stderr[-3000:])
    assert run.stdout.startswith("ok: 6 records"), run.stdout
