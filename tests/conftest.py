import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.pyoracle import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def manifest():
    with open(os.path.join(GOLDEN, "manifest.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def codec_golden():
    return np.load(os.path.join(GOLDEN, "codec_golden.npz"))


@pytest.fixture(scope="session")
def linear_golden():
    return np.load(os.path.join(GOLDEN, "linear_golden.npz"))


def rel_l2(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


def moe_block_case(manifest, linear_golden, label):
    """One format mix of the MoE-block fixture: the expert matrices redrawn from their seeds (checked against the
    hashes the generator recorded) and the reference's inputs and results. -> dict"""
    import hashlib
    import synth
    mb = manifest["moe_block"]
    case = mb["cases"][label]
    n_expert, n_embd, n_ff = mb["n_expert"], mb["n_embd"], mb["n_ff"]
    types, seeds = case["types"], case["weight_seeds"]
    gate = synth.make_weights(types[0], n_expert * n_ff, n_embd, seed=seeds[0])
    up = synth.make_weights(types[1], n_expert * n_ff, n_embd, seed=seeds[1])
    down = synth.make_weights(types[2], n_expert * n_embd, n_ff, seed=seeds[2])
    for a, h in zip((gate, up, down), case["weights_sha256"]):
        assert hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest() == h, "synthetic weights changed"
    return dict(types=tuple(types), gate=gate, up=up, down=down, n_expert=n_expert, n_embd=n_embd, n_ff=n_ff,
                top_k=mb["top_k"], logits=linear_golden["moe_%s_logits" % label], x=linear_golden["moe_%s_x" % label],
                idx=linear_golden["moe_%s_idx" % label], w=linear_golden["moe_%s_w" % label],
                out=linear_golden["moe_%s_out" % label])
