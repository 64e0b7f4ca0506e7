"""The C++ class mako::gen::Sampler (include/gen/sampler.hpp) on the GPU against the oracle: a scripted decode
session must return, step by step, the tokens a reference Sampler with the same seed returns."""
import os
import subprocess
import tempfile

import numpy as np
import pytest

from oracle import pyoracle

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "sampler_class_test")


def build_exe():
    subprocess.run(["g++", "-O2", "-std=c++20", "-I", os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "tests", "cpp", "sampler_class_test.cpp"), "-o", EXE,
                    "-L", os.path.join(ROOT, "mako_amd"), "-lmako_sampler",
                    "-Wl,-rpath," + os.path.join(ROOT, "mako_amd")], check=True)


def expected(oracle, logits, seed, mode, prm):
    """The reference's session semantics restated with the oracle: uniforms come from mt19937_64(seed) in call
    order -- sample() takes one, verify() one plus a second when it redraws."""
    steps = logits.shape[0]
    us = oracle.uniforms(seed, 2 * steps + 2)
    k = 0
    hist, out = [], []
    p = pyoracle.make_params(*prm)
    for i in range(steps):
        if mode == 0:
            t, _ = oracle.sample(logits[i], p, float(us[k]), hist, order_mode=0)
            acc = False
            k += 0 if p.temperature <= 0 else 1
        else:
            draft = int(np.argmax(logits[i]))
            t, acc = oracle.verify(logits[i], p, draft, float(us[k]), float(us[k + 1]), hist, order_mode=0)
            if p.temperature > 0:
                k += 1 if (acc or t == draft) else 2
        hist.append(t)
        out.append((t, int(acc)))
    return out


@pytest.mark.parametrize("mode,prm", [
    (0, (0.8, 40, 0.95, 0.0, 0.3, 0.2, 1.1)),
    (0, (1.0, 0, 0.9, 0.05, 0.0, 0.0, 1.0)),
    (0, (0.0, 0, 1.0, 0.0, 0.3, 0.2, 1.1)),
    (1, (0.9, 20, 0.9, 0.0, 0.0, 0.0, 1.0)),
    (1, (1.3, 0, 0.8, 0.0, 0.5, 0.1, 1.2)),
    (1, (0.0, 0, 1.0, 0.0, 0.0, 0.0, 1.0)),
])
def test_session_matches_reference_stream(oracle, mode, prm):
    if not os.path.exists(EXE):
        build_exe()
    rng = np.random.default_rng(99 + mode)
    v, steps, seed = 5000, 40, 1234567 + mode
    logits = (rng.standard_normal((steps, v)) * 2.5).astype(np.float32)
    with tempfile.NamedTemporaryFile(suffix=".f32") as f:
        logits.tofile(f.name)
        out = subprocess.run([EXE, f.name, str(v), str(steps), str(seed), str(mode)] + [repr(float(x)) if i != 1 else
                             str(int(x)) for i, x in enumerate(prm)], check=True, capture_output=True, text=True,
                             timeout=120).stdout.split("\n")
    assert out[0] == "empty_vocab_throws 1"
    got = [tuple(int(x) for x in line.split()) for line in out[1:] if line]
    assert got == expected(oracle, logits, seed, mode, prm)
