"""Seeded synthetic GGML block data for the benchmark configurations and the parity tests.

Every generator returns a uint8 array [n_rows, row_bytes] holding raw blocks in the on-disk
GGML layout (block structs of common/ggml_dequant.h:30-204, no padding), drawn from
numpy's PCG64 with the given seed. Field distributions follow the benchmark configurations:
fp16 scales uniform in a small positive range (rounded to nearest even), integer fields
uniform over their full range.
"""
import numpy as np

# enum ggml_dtype values (common/gguf_loader.h:45-85)
GGML_F32, GGML_F16, GGML_Q8_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K = 0, 1, 8, 12, 13, 14
GGML_IQ2_XXS, GGML_IQ4_NL, GGML_IQ3_S, GGML_BF16 = 16, 20, 21, 30
GGML_Q4_0, GGML_Q4_1, GGML_Q5_0, GGML_Q5_1, GGML_Q2_K, GGML_Q3_K = 2, 3, 6, 7, 10, 11
GGML_IQ2_XS, GGML_IQ3_XXS, GGML_IQ1_S, GGML_IQ2_S, GGML_IQ4_XS, GGML_IQ1_M = 17, 18, 19, 22, 23, 29
GGML_TQ1_0, GGML_TQ2_0, GGML_MXFP4, GGML_NVFP4, GGML_Q1_0 = 34, 35, 39, 40, 41

# type id -> (elements per block, bytes per block)   (common/ggml_dequant.h:261-294)
BLOCK_GEOMETRY = {
    GGML_Q8_0: (32, 34), GGML_Q4_K: (256, 144), GGML_Q5_K: (256, 176), GGML_Q6_K: (256, 210),
    GGML_IQ2_XXS: (256, 66), GGML_IQ4_NL: (32, 18), GGML_IQ3_S: (256, 110),
    GGML_Q4_0: (32, 18), GGML_Q4_1: (32, 20), GGML_Q5_0: (32, 22), GGML_Q5_1: (32, 24),
    GGML_Q2_K: (256, 84), GGML_Q3_K: (256, 110), GGML_IQ2_XS: (256, 74), GGML_IQ3_XXS: (256, 98),
    GGML_IQ1_S: (256, 50), GGML_IQ2_S: (256, 82), GGML_IQ4_XS: (256, 136), GGML_IQ1_M: (256, 56),
    GGML_TQ1_0: (256, 54), GGML_TQ2_0: (256, 66), GGML_MXFP4: (32, 17), GGML_NVFP4: (64, 36),
    GGML_Q1_0: (128, 18),
}
# every block format with a decoder (the type switch at common/ggml_dequant.h:3177-3265)
TYPE_NAMES = {GGML_Q8_0: "q8_0", GGML_Q4_K: "q4_K", GGML_Q5_K: "q5_K", GGML_Q6_K: "q6_K",
              GGML_IQ2_XXS: "iq2_xxs", GGML_IQ4_NL: "iq4_nl", GGML_IQ3_S: "iq3_s",
              GGML_Q4_0: "q4_0", GGML_Q4_1: "q4_1", GGML_Q5_0: "q5_0", GGML_Q5_1: "q5_1",
              GGML_Q2_K: "q2_K", GGML_Q3_K: "q3_K", GGML_IQ2_XS: "iq2_xs", GGML_IQ3_XXS: "iq3_xxs",
              GGML_IQ1_S: "iq1_s", GGML_IQ2_S: "iq2_s", GGML_IQ4_XS: "iq4_xs", GGML_IQ1_M: "iq1_m",
              GGML_TQ1_0: "tq1_0", GGML_TQ2_0: "tq2_0", GGML_MXFP4: "mxfp4", GGML_NVFP4: "nvfp4",
              GGML_Q1_0: "q1_0"}
# the block formats the reference's model path (matvec, prefill, experts) accepts as weights
# (tf_is_supported_weight_type, common/transformer.h:462-487)
LINEAR_TYPES = {t: TYPE_NAMES[t] for t in (
    GGML_Q8_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_IQ2_XXS, GGML_IQ4_NL, GGML_IQ3_S, GGML_Q4_0,
    GGML_Q2_K, GGML_Q3_K, GGML_IQ2_XS, GGML_IQ3_XXS, GGML_IQ1_S, GGML_IQ2_S, GGML_IQ4_XS, GGML_IQ1_M)}
# dense row formats the model path also takes as weights (one element per "block")
DENSE_TYPES = {GGML_F32: "f32", GGML_F16: "f16", GGML_BF16: "bf16"}
BLOCK_GEOMETRY.update({GGML_F32: (1, 4), GGML_F16: (1, 2), GGML_BF16: (1, 2)})
# offsets of the fp16 scale fields of the formats not spelled out in make_weights
_F16_FIELDS = {
    GGML_IQ4_NL: (0,), GGML_IQ2_XXS: (0,), GGML_IQ3_S: (0,),
    GGML_Q4_0: (0,), GGML_Q4_1: (0, 2), GGML_Q5_0: (0,), GGML_Q5_1: (0, 2), GGML_Q2_K: (80, 82),
    GGML_Q3_K: (108,), GGML_IQ2_XS: (0,), GGML_IQ3_XXS: (0,), GGML_IQ1_S: (0,), GGML_IQ2_S: (0,),
    GGML_IQ4_XS: (0,), GGML_TQ1_0: (52,), GGML_TQ2_0: (64,), GGML_Q1_0: (0,),
}


def row_bytes(type_id, n_cols):
    be, bb = BLOCK_GEOMETRY[type_id]
    return (n_cols + be - 1) // be * bb


def _f16_bytes(rng, shape, lo, hi):
    v = rng.uniform(lo, hi, size=shape).astype(np.float32).astype(np.float16)
    return v.view(np.uint16)


def _put_u16(blocks, off, u16):
    blocks[..., off] = (u16 & 0xFF).astype(np.uint8)
    blocks[..., off + 1] = (u16 >> 8).astype(np.uint8)


def make_weights(type_id, n_rows, n_cols, seed, wild=False):
    """Raw blocks for an [n_rows, n_cols] matrix. wild=True fills EVERY byte with random bits
    (arbitrary fp16 scale patterns including subnormals, infinities and NaNs): used for the
    bit-exact codec tests, never for the matvec tolerance tests."""
    be, bb = BLOCK_GEOMETRY[type_id]
    assert n_cols % be == 0, "n_cols must be a whole number of blocks"
    nb = n_cols // be
    rng = np.random.default_rng(seed)
    if type_id in DENSE_TYPES:  # N(0, 0.02) values (wild: any bit pattern)
        if wild:
            return rng.integers(0, 256, size=(n_rows, nb * bb), dtype=np.uint8)
        v = (rng.standard_normal(size=(n_rows, n_cols)) * 0.02).astype(np.float32)
        if type_id == GGML_F16:
            v = v.astype(np.float16)
        elif type_id == GGML_BF16:
            v = to_bf16_bits(v)
        return np.ascontiguousarray(v).view(np.uint8).reshape(n_rows, nb * bb)
    blocks = rng.integers(0, 256, size=(n_rows, nb, bb), dtype=np.uint8)
    if not wild:
        if type_id == GGML_Q8_0:
            _put_u16(blocks, 0, _f16_bytes(rng, (n_rows, nb), 1e-3, 1e-2))
            q = rng.integers(-127, 128, size=(n_rows, nb, 32), dtype=np.int8)
            blocks[..., 2:34] = q.view(np.uint8)
        elif type_id in (GGML_Q4_K, GGML_Q5_K):
            # 12 uniformly random scale bytes == sixteen independent uniform 6-bit fields
            _put_u16(blocks, 0, _f16_bytes(rng, (n_rows, nb), 1e-3, 2e-2))
            _put_u16(blocks, 2, _f16_bytes(rng, (n_rows, nb), 1e-3, 2e-2))
        elif type_id == GGML_Q6_K:
            sc = rng.integers(-32, 32, size=(n_rows, nb, 16), dtype=np.int8)
            blocks[..., 192:208] = sc.view(np.uint8)
            _put_u16(blocks, 208, _f16_bytes(rng, (n_rows, nb), 1e-3, 1e-2))
        elif type_id == GGML_IQ1_M:
            # the fp16 super-scale is spread over the top nibbles of the four scale words
            d = _f16_bytes(rng, (n_rows, nb), 1e-3, 1e-2).astype(np.uint32)
            for w in range(4):
                hi = blocks[..., 49 + 2 * w].astype(np.uint32)
                blocks[..., 49 + 2 * w] = ((hi & 0x0F) | (((d >> (4 * w)) & 0xF) << 4)).astype(np.uint8)
        elif type_id == GGML_MXFP4:
            # E8M0 exponent byte: scales 2^-10 .. 2^-3
            blocks[..., 0] = rng.integers(118, 126, size=(n_rows, nb), dtype=np.uint8)
        elif type_id == GGML_NVFP4:
            pass  # every scale byte is a finite unsigned E4M3 number
        else:  # one or two fp16 scales at fixed offsets, everything else random bits
            for off in _F16_FIELDS[type_id]:
                _put_u16(blocks, off, _f16_bytes(rng, (n_rows, nb), 1e-3, 1e-2))
    return blocks.reshape(n_rows, nb * bb)


def make_activation(n, seed, tokens=None):
    """fp32 N(0,1) activations: [n] or [tokens, n]."""
    rng = np.random.default_rng(seed)
    shape = (n,) if tokens is None else (tokens, n)
    return rng.standard_normal(size=shape).astype(np.float32)


def to_bf16_bits(x):
    """fp32 -> bf16 bit pattern (uint16), round to nearest even; NaN kept quiet."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    return np.where(nan, (u >> 16) | 0x40, rounded).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def make_router_logits(n_tokens, n_expert, seed):
    """Uniform [0,1) router logits, fp32 [n_tokens, n_expert]."""
    return np.random.default_rng(seed).random(size=(n_tokens, n_expert), dtype=np.float32)
