"""Seeded synthetic weight packs in the model-folder stream layout (reference: nslm/model_st.h:10-16,42-43).

A pack is a dict of numpy arrays, slice-major as the reference stacks experts:
  SEED4P4: seeds u16 [S,R,K/8], coefs u16 [S,R,K/8], codes u8 [S,R*K/16] (block g of a slice in nibble g&1 of byte
           g>>1), eb int32 [S]
  SEED4:   seeds u16 [S,R,K/8], nibs u16 [S,R,K/8] (bits 0-3 exponent code, then q0 q1 q2), eb int32 [S]
  Q4/Q8:   words u32 [S,R,K*bits/32], scales / biases BF16 bits u16 [S,R,K/group]
  BF16:    w u16 [S,R,K]
Draws follow the benchmark definition: seeds uniform in [1, 65535], int4 coefficients uniform, exponent codes uniform
in [0, 15]; the affine format draws a BF16 scale ~ U(0.005, 0.02) and a zero point z uniform in [0, 15] stored MLX-style
as bias = bf16(-z * scale) (nslm/affine.h:3-10).
"""
import numpy as np

MF_BF16, MF_SEED4, MF_Q8, MF_Q4, MF_SEED4P4 = 0, 1, 2, 3, 4


def f32_to_bf16_bits(x):
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def bf16_bits_to_f32(h):
    return (np.asarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def round_bf16(x):
    return bf16_bits_to_f32(f32_to_bf16_bits(x))


def seed4p4(rng, S, R, K, eb=-22, code_max=15):
    nb = R * K // 8
    return {
        "fmt": MF_SEED4P4, "S": S, "R": R, "K": K,
        "seeds": rng.integers(1, 65536, size=(S, R, K // 8), dtype=np.uint16),
        "coefs": rng.integers(0, 65536, size=(S, R, K // 8), dtype=np.uint16),
        "codes": _pack_nibbles(rng.integers(0, code_max + 1, size=(S, nb), dtype=np.uint8)),
        "eb": np.full(S, eb, dtype=np.int32) if np.isscalar(eb) else np.asarray(eb, dtype=np.int32),
    }


def seed4(rng, S, R, K, eb=-22):
    return {
        "fmt": MF_SEED4, "S": S, "R": R, "K": K,
        "seeds": rng.integers(1, 65536, size=(S, R, K // 8), dtype=np.uint16),
        "nibs": rng.integers(0, 65536, size=(S, R, K // 8), dtype=np.uint16),
        "eb": np.full(S, eb, dtype=np.int32) if np.isscalar(eb) else np.asarray(eb, dtype=np.int32),
    }


def affine(rng, S, R, K, bits=4, group=64):
    scale = f32_to_bf16_bits(rng.uniform(0.005, 0.02, size=(S, R, K // group)).astype(np.float32))
    z = rng.integers(0, 16 if bits == 4 else 256, size=(S, R, K // group)).astype(np.float32)
    bias = f32_to_bf16_bits(-z * bf16_bits_to_f32(scale))
    per = 32 // bits
    q = rng.integers(0, 1 << bits, size=(S, R, K // per, per), dtype=np.uint32)
    words = np.zeros((S, R, K // per), dtype=np.uint32)
    for i in range(per):
        words |= q[..., i] << np.uint32(bits * i)
    return {"fmt": MF_Q4 if bits == 4 else MF_Q8, "S": S, "R": R, "K": K, "group": group, "words": words,
            "scales": scale, "biases": bias}


def bf16(rng, S, R, K, std=0.02):
    return {"fmt": MF_BF16, "S": S, "R": R, "K": K,
            "w": f32_to_bf16_bits((rng.standard_normal((S, R, K)) * std).astype(np.float32))}


def _pack_nibbles(n):
    """[S, nb] nibbles -> [S, ceil(nb/2)] bytes, block g in nibble g&1 (low first) of byte g>>1."""
    S, nb = n.shape
    if nb & 1:
        n = np.concatenate([n, np.zeros((S, 1), dtype=np.uint8)], axis=1)
    return (n[:, 0::2] | (n[:, 1::2] << 4)).astype(np.uint8)


def unpack_nibbles(codes, nb):
    c = np.asarray(codes, dtype=np.uint8)
    out = np.empty(c.shape[:-1] + (c.shape[-1] * 2,), dtype=np.uint8)
    out[..., 0::2] = c & 15
    out[..., 1::2] = c >> 4
    return out[..., :nb]


def pack_bytes(p):
    """Compressed weight bytes of a pack: the figure effective-GB/s numbers are computed from."""
    n = p["S"] * p["R"] * p["K"]
    f = p["fmt"]
    if f == MF_SEED4P4:
        return n * 36 // 64           # 4.5 B per 8 weights
    if f == MF_SEED4:
        return n // 2                 # 4 B per 8 weights
    if f == MF_Q4:
        return n // 2 + 4 * n // p["group"]
    if f == MF_Q8:
        return n + 4 * n // p["group"]
    return 2 * n
