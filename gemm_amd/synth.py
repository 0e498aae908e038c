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

# type id -> (elements per block, bytes per block)   (common/ggml_dequant.h:261-294)
BLOCK_GEOMETRY = {
    GGML_Q8_0: (32, 34), GGML_Q4_K: (256, 144), GGML_Q5_K: (256, 176), GGML_Q6_K: (256, 210),
    GGML_IQ2_XXS: (256, 66), GGML_IQ4_NL: (32, 18), GGML_IQ3_S: (256, 110),
}
TYPE_NAMES = {GGML_Q8_0: "q8_0", GGML_Q4_K: "q4_K", GGML_Q5_K: "q5_K", GGML_Q6_K: "q6_K",
              GGML_IQ2_XXS: "iq2_xxs", GGML_IQ4_NL: "iq4_nl", GGML_IQ3_S: "iq3_s"}


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
        else:  # IQ4_NL, IQ2_XXS, IQ3_S: fp16 d first, everything else random bits
            _put_u16(blocks, 0, _f16_bytes(rng, (n_rows, nb), 1e-3, 1e-2))
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
