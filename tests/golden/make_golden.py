#!/usr/bin/env python3
"""Writes the golden fixtures of tests/golden/ from the reference's own C code.

Run in the build container only (it needs oracle/_ref/libref.so, which oracle/Makefile compiles
from the read-only reference checkout):

    make -C oracle && python tests/golden/make_golden.py

The fixtures are data: input block bytes (drawn by gemm_amd.synth from fixed seeds) and the
fp32 bit patterns the reference produced for them. The parity tests read the fixtures and never
need the reference at test time.
"""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from gemm_amd import synth  # noqa: E402
from oracle.pyoracle import Reference  # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))
CODEC_COLS = 512          # 2 super-blocks of 256 / 16 blocks of 32 per row
CODEC_ROWS = 6
SWEEP_ROWS, SWEEP_COLS = 64, 4096
LIN_ROWS, LIN_COLS = 24, 1024


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def canonical_nan(bits):
    """fp32 bit patterns with every NaN replaced by 0x7FC00000: where two NaN scales meet (d and
    dmin of one block), which payload survives depends on the compiler's operand order, not on
    the format, so sweep hashes are taken over canonical NaNs."""
    bits = np.array(bits, dtype=np.uint32, copy=True)
    bits[(bits & 0x7FFFFFFF) > 0x7F800000] = 0x7FC00000
    return bits


def main():
    ref = Reference()
    manifest = {"generator": "tests/golden/make_golden.py", "source": "reference C compiled via oracle/ref_shim.c"}

    # fp16 -> fp32, exhaustive: the full table is 256 KiB, so only its hash is committed
    table = ref.fp16_table()
    manifest["fp16_table_sha256"] = sha(table.view(np.uint32))
    probes = [0x0000, 0x8000, 0x0001, 0x03FF, 0x0400, 0x3C00, 0x7BFF, 0x7C00, 0xFC00, 0x7C01, 0x7E00, 0xFFFF]
    manifest["fp16_probe_bits"] = {"%04x" % h: "%08x" % int(table.view(np.uint32)[h]) for h in probes}

    # codebooks
    manifest["tables_sha256"] = {n: hashlib.sha256(ref.table(n)).hexdigest()
                                 for n in ("iq2xxs_grid", "iq3s_grid", "iq4nl_values", "ksigns", "mxfp4_values",
                                           "iq3xxs_grid", "iq2xs_grid", "iq2s_grid", "iq1s_grid")}

    codec, sweep = {}, {}
    for tid, name in synth.TYPE_NAMES.items():
        # small blocks stored whole: half wild bytes (any fp16 pattern), half config-like
        wild = synth.make_weights(tid, CODEC_ROWS // 2, CODEC_COLS, seed=1000 + tid, wild=True)
        tame = synth.make_weights(tid, CODEC_ROWS // 2, CODEC_COLS, seed=2000 + tid, wild=False)
        src = np.concatenate([wild, tame], axis=0)
        out = np.zeros((CODEC_ROWS, CODEC_COLS), np.uint32)
        for r in range(CODEC_ROWS):
            rc, row = ref.dequant_row(tid, src[r], CODEC_COLS)
            assert rc == 0
            out[r] = row.view(np.uint32)
        codec[name + "_src"] = src
        codec[name + "_f32bits"] = out
        assert ref.row_size(tid, CODEC_COLS) == src.shape[1]
        # a larger seeded sweep, committed as hashes of input and output only
        big = synth.make_weights(tid, SWEEP_ROWS, SWEEP_COLS, seed=3000 + tid, wild=True)
        dec = np.zeros((SWEEP_ROWS, SWEEP_COLS), np.uint32)
        for r in range(SWEEP_ROWS):
            dec[r] = ref.dequant_row(tid, big[r], SWEEP_COLS)[1].view(np.uint32)
        sweep[name] = {"seed": 3000 + tid, "rows": SWEEP_ROWS, "cols": SWEEP_COLS, "wild": True,
                       "input_sha256": sha(big), "output_sha256": sha(canonical_nan(dec))}
    manifest["codec_sweep"] = sweep
    manifest["row_size"] = {str(t): {str(n): ref.row_size(t, n) for n in (0, 1, 31, 32, 33, 255, 256, 257, 4096, 14336)}
                            for t in list(synth.TYPE_NAMES) + [0, 1, 30, 9, 15, 99]}
    # what the model path accepts, and its own row-size function (0 outside that list)
    manifest["tf_row_bytes_4096"] = {str(t): ref.tf_row_bytes(t, 4096) for t in list(range(0, 44)) + [99]}
    rc, _ = ref.dequant_row(99, np.zeros(64, np.uint8), 32)
    manifest["dequant_row_unknown_type_rc"] = rc
    np.savez_compressed(os.path.join(OUT, "codec_golden.npz"), **codec)

    # matvec / prefill / expert slice through the reference's own call sites
    lin = {}
    x = synth.make_activation(LIN_COLS, seed=77)
    X = synth.make_activation(LIN_COLS, seed=78, tokens=5)
    lin["x"], lin["X"] = x, X
    # the types the reference's model path accepts: sixteen block formats and the dense ones
    for tid, name in list(synth.LINEAR_TYPES.items()) + list(synth.DENSE_TYPES.items()):
        W = synth.make_weights(tid, LIN_ROWS, LIN_COLS, seed=4000 + tid)
        lin[name + "_W"] = W
        lin[name + "_y_f32"] = ref.qmatvec(tid, W, x, LIN_COLS)
        lin[name + "_y_f64"] = ref.qmatvec(tid, W, x, LIN_COLS, f64=True)
        lin[name + "_Y_tokmajor"] = ref.gemm_tokenmajor(tid, W, X, LIN_COLS)
        # expert slice: the 24 rows seen as 3 experts of 8 rows
        lin[name + "_y_expert1"] = ref.qmatvec_expert(tid, W, 1, x, 8, LIN_COLS)
    np.savez_compressed(os.path.join(OUT, "linear_golden.npz"), **lin)

    with open(os.path.join(OUT, "manifest.json"), "w") as f:
        json.dump(manifest, f, indent=1, sort_keys=True)
    for fn in ("codec_golden.npz", "linear_golden.npz", "manifest.json"):
        print(fn, os.path.getsize(os.path.join(OUT, fn)), "bytes")


if __name__ == "__main__":
    main()
