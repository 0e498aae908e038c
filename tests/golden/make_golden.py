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
import synth  # noqa: E402
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


def gguf_fixture(ref):
    """A small GGUF file (tests/golden/tiny.gguf) and what the reference's loader reads from it."""
    import ctypes as C
    from tests import gguf_writer as gw
    path = os.path.join(OUT, "tiny.gguf")
    rng = np.random.default_rng(77)
    tensors = [
        ("token_embd.weight", synth.GGML_Q6_K, (256, 40), synth.make_weights(synth.GGML_Q6_K, 40, 256, seed=1)),
        ("blk.0.ffn_gate.weight", synth.GGML_Q4_K, (512, 24), synth.make_weights(synth.GGML_Q4_K, 24, 512, seed=2)),
        ("blk.0.ffn_down_exps.weight", synth.GGML_IQ2_XS, (256, 8, 3), synth.make_weights(synth.GGML_IQ2_XS, 24, 256, seed=3)),
        ("blk.0.attn_norm.weight", synth.GGML_F32, (256,), synth.make_activation(256, seed=4).view(np.uint8)),
        ("output.weight", synth.GGML_Q8_0, (256, 40), synth.make_weights(synth.GGML_Q8_0, 40, 256, seed=5)),
        ("rope_freqs", synth.GGML_F16, (31,), rng.integers(0, 256, 62, dtype=np.uint8)),  # odd size: next start is padded
        ("blk.0.attn_q.weight", synth.GGML_BF16, (256, 16), synth.make_weights(synth.GGML_BF16, 16, 256, seed=6)),
    ]
    kvs = [("general.architecture", gw.STR, "qwen3"), ("qwen3.block_count", gw.U32, 1),
           ("qwen3.embedding_length", gw.U32, 256), ("qwen3.rope.freq_base", gw.F32, 1000000.0),
           ("qwen3.attention.layer_norm_rms_epsilon", gw.F32, 1e-6), ("general.file_type", gw.I32, -3),
           ("some.u8", gw.U8, 200), ("some.i8", gw.I8, -100), ("some.u16", gw.U16, 60000), ("some.i16", gw.I16, -30000),
           ("some.u64", gw.U64, 2 ** 63 + 5), ("some.i64", gw.I64, -2 ** 62), ("some.f64", gw.F64, 2.5), ("some.bool", gw.BOOL, 1),
           ("tokenizer.ggml.tokens", gw.ARR, (gw.STR, ["<s>", "hello", "", "w\u00f6rld"])),
           ("tokenizer.ggml.scores", gw.ARR, (gw.F32, [0.0, -1.5, 2.25])),
           ("tokenizer.ggml.token_type", gw.ARR, (gw.I32, [1, 2, 3, 4, 5]))]
    gw.write(path, kvs, tensors, version=3, alignment=64)
    L = ref.lib
    L.ref_gguf_open.restype = C.c_void_p
    L.ref_gguf_open.argtypes = [C.c_char_p]
    for fn, rt in (("n_tensors", C.c_uint64), ("n_kv", C.c_uint64), ("version", C.c_uint32), ("alignment", C.c_uint32),
                   ("data_offset", C.c_uint64), ("data_size", C.c_uint64)):
        getattr(L, "ref_gguf_" + fn).restype = rt
        getattr(L, "ref_gguf_" + fn).argtypes = [C.c_void_p]
    L.ref_gguf_tensor_name.restype = C.c_char_p
    L.ref_gguf_tensor_name.argtypes = [C.c_void_p, C.c_int]
    L.ref_gguf_tensor_size.restype = C.c_uint64
    L.ref_gguf_tensor_size.argtypes = [C.c_void_p, C.c_int]
    L.ref_gguf_tensor_data.restype = C.c_void_p
    L.ref_gguf_tensor_data.argtypes = [C.c_void_p, C.c_int]
    L.ref_gguf_tensor_info.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
    L.ref_tf_load_tensor.restype = C.c_int64
    L.ref_tf_load_tensor.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p]
    L.ref_gguf_find_key.argtypes = [C.c_void_p, C.c_char_p]
    L.ref_gguf_kv_type.restype = C.c_uint32
    L.ref_gguf_kv_type.argtypes = [C.c_void_p, C.c_int]
    L.ref_gguf_kv_u64.restype = C.c_uint64
    L.ref_gguf_kv_u64.argtypes = [C.c_void_p, C.c_int]
    L.ref_gguf_kv_str.restype = C.c_char_p
    L.ref_gguf_kv_str.argtypes = [C.c_void_p, C.c_int]
    L.ref_gguf_kv_arr_n.restype = C.c_uint64
    L.ref_gguf_kv_arr_n.argtypes = [C.c_void_p, C.c_int]
    L.ref_tf_get_int.argtypes = [C.c_void_p, C.c_char_p, C.c_int]
    L.ref_gguf_close.argtypes = [C.c_void_p]
    ctx = L.ref_gguf_open(path.encode())
    assert ctx
    out = {"file": "tiny.gguf", "file_sha256": hashlib.sha256(open(path, "rb").read()).hexdigest(),
           "version": L.ref_gguf_version(ctx), "alignment": L.ref_gguf_alignment(ctx),
           "data_offset": L.ref_gguf_data_offset(ctx), "data_size": L.ref_gguf_data_size(ctx),
           "n_kv": L.ref_gguf_n_kv(ctx), "tensors": [], "kv": {}}
    for i in range(L.ref_gguf_n_tensors(ctx)):
        info = (C.c_uint64 * 7)()
        L.ref_gguf_tensor_info(ctx, i, info)
        name = L.ref_gguf_tensor_name(ctx, i)
        size = L.ref_gguf_tensor_size(ctx, i)
        raw = C.string_at(L.ref_gguf_tensor_data(ctx, i), size)
        qt = (C.c_int64 * 4)()
        qoff = L.ref_tf_load_tensor(ctx, name, qt)
        out["tensors"].append({"name": name.decode(), "type": info[0], "n_dims": info[1], "dims": list(info[2:6]),
                               "offset": info[6], "size": size, "data_sha256": hashlib.sha256(raw).hexdigest(),
                               "qtensor": {"type": qt[0], "n_rows": qt[1], "n_cols": qt[2], "n_dims": qt[3],
                                           "data_offset": qoff}})
    for key, vtype, _ in kvs + [("general.alignment", gw.U32, 64)]:
        i = L.ref_gguf_find_key(ctx, key.encode())
        assert i >= 0
        e = {"index": i, "type": L.ref_gguf_kv_type(ctx, i)}
        if vtype == gw.STR:
            e["str"] = L.ref_gguf_kv_str(ctx, i).decode()
        elif vtype == gw.ARR:
            e["n"] = L.ref_gguf_kv_arr_n(ctx, i)
        else:
            e["raw_u64"] = L.ref_gguf_kv_u64(ctx, i) & ((1 << (8 * {0: 1, 1: 1, 7: 1, 2: 2, 3: 2, 4: 4, 5: 4, 6: 4, 10: 8, 11: 8, 12: 8}[vtype])) - 1)
        out["kv"][key] = e
    out["tf_get_int"] = {k: L.ref_tf_get_int(ctx, k.encode(), -7) for k in
                         ("qwen3.block_count", "general.file_type", "some.u16", "missing.key")}
    L.ref_gguf_close(ctx)
    return out


MOE_EXPERTS, MOE_TOP, MOE_EMBD, MOE_FF = 16, 4, 512, 256


def heap_top_k(probs, k):
    """The selection of the reference's MoE block (common/transformer.h:4056-4090): one pass over the experts that
    keeps the k largest probabilities in a min-heap (ties keep the earlier expert), then the weights divided by their
    sum, added up in heap order in fp32. -> (expert ids, weights) in the heap's final order."""
    ids, val = [], []

    def swap(a, b):
        ids[a], ids[b] = ids[b], ids[a]
        val[a], val[b] = val[b], val[a]

    for e, p in enumerate(probs):
        if len(ids) < k:
            ids.append(e)
            val.append(p)
            child = len(ids) - 1
            while child > 0 and val[child] < val[(child - 1) // 2]:
                swap(child, (child - 1) // 2)
                child = (child - 1) // 2
        elif p > val[0]:
            ids[0], val[0] = e, p
            node = 0
            while True:
                least = node
                for c in (2 * node + 1, 2 * node + 2):
                    if c < k and val[c] < val[least]:
                        least = c
                if least == node:
                    break
                swap(node, least)
                node = least
    total = np.float32(0.0)
    for v in val:
        total = np.float32(total + v)
    w = np.array(val, np.float32)
    if total > 0:
        w = (w / total).astype(np.float32)
    return np.array(ids, np.int32), w


def moe_block(ref, types, gate, up, down, logits, x):
    """One token through the reference's MoE FFN block (common/transformer.h:4045-4131), composed from its own
    compiled functions: tf_softmax, the selection above, tf_qmatvec_expert for up, gate and down, tf_silu_mul_avx2,
    and the weighted sum (one rounding per element and expert, as its fused multiply-add gives)."""
    idx, w = heap_top_k(ref.softmax(logits), MOE_TOP)
    out = np.zeros(MOE_EMBD, np.float32)
    for e, ew in zip(idx, w):
        u = ref.qmatvec_expert(types[1], up, int(e), x, MOE_FF, MOE_EMBD)
        g = ref.qmatvec_expert(types[0], gate, int(e), x, MOE_FF, MOE_EMBD)
        h = ref.silu_mul(g, u)
        q = ref.qmatvec_expert(types[2], down, int(e), h, MOE_EMBD, MOE_FF)
        out = (np.float64(ew) * q.astype(np.float64) + out.astype(np.float64)).astype(np.float32)
    return idx, w, out


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
    # the MoE FFN block, one token at a time; the expert matrices are drawn from fixed seeds (their hashes are in the
    # manifest), two tokens per format mix
    Q4K, Q6K = synth.GGML_Q4_K, synth.GGML_Q6_K
    moe_manifest = {"n_expert": MOE_EXPERTS, "top_k": MOE_TOP, "n_embd": MOE_EMBD, "n_ff": MOE_FF, "cases": {}}
    for label, types in (("q4k", (Q4K, Q4K, Q4K)), ("q4k_down_q6k", (Q4K, Q4K, Q6K))):
        seeds = (5100 + types[2], 5200 + types[2], 5300 + types[2])
        gate = synth.make_weights(types[0], MOE_EXPERTS * MOE_FF, MOE_EMBD, seed=seeds[0])
        up = synth.make_weights(types[1], MOE_EXPERTS * MOE_FF, MOE_EMBD, seed=seeds[1])
        down = synth.make_weights(types[2], MOE_EXPERTS * MOE_EMBD, MOE_FF, seed=seeds[2])
        logits = synth.make_router_logits(2, MOE_EXPERTS, seed=5400 + types[2])
        xs = synth.make_activation(MOE_EMBD, seed=5500 + types[2], tokens=2)
        res = [moe_block(ref, types, gate, up, down, logits[t], xs[t]) for t in range(2)]
        lin["moe_%s_logits" % label], lin["moe_%s_x" % label] = logits, xs
        lin["moe_%s_idx" % label] = np.stack([r[0] for r in res])
        lin["moe_%s_w" % label] = np.stack([r[1] for r in res])
        lin["moe_%s_out" % label] = np.stack([r[2] for r in res])
        moe_manifest["cases"][label] = {"types": list(types), "weight_seeds": list(seeds),
                                        "weights_sha256": [sha(gate), sha(up), sha(down)]}
    manifest["moe_block"] = moe_manifest
    np.savez_compressed(os.path.join(OUT, "linear_golden.npz"), **lin)

    manifest["gguf_fixture"] = gguf_fixture(ref)

    with open(os.path.join(OUT, "manifest.json"), "w") as f:
        json.dump(manifest, f, indent=1, sort_keys=True)
    for fn in ("codec_golden.npz", "linear_golden.npz", "manifest.json"):
        print(fn, os.path.getsize(os.path.join(OUT, fn)), "bytes")


if __name__ == "__main__":
    main()
