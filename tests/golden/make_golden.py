"""Writes the golden fixtures under tests/golden/ from the COMPILED C reference (oracle/_ref/libnslm_ref.so, built by
oracle/Makefile from the reference's own sources).  Run in the build container only (the reference tree does not exist
on the GPU box); the .npz files it writes are data: inputs and the reference's outputs.

    python tests/golden/make_golden.py
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from nanoseedlm_amd import packs  # noqa: E402
from oracle import oracle as orc  # noqa: E402


def vp(a):
    return a.ctypes.data_as(C.c_void_p)


def main():
    orc.build()
    ref = orc.ref()
    assert ref is not None, "oracle/_ref/libnslm_ref.so missing: run make -C oracle ref"
    rng = np.random.default_rng(20261125)
    # 1. 2000 random blocks through nslm4_decode_block (P=4) and nslm_decode_block (P=3)
    n = 2000
    seed = rng.integers(1, 65536, n).astype(np.uint16)
    word = rng.integers(0, 65536, n).astype(np.uint16)
    e = rng.integers(-30, -4, n).astype(np.int32)
    p4 = np.zeros((n, 8), dtype=np.uint16)
    p3 = np.zeros((n, 8), dtype=np.uint16)
    for i in range(n):
        ref.nslm4_decode_block(C.c_uint16(seed[i]), C.c_uint16(word[i]), C.c_int(e[i]), vp(p4[i]))
        ref.ref_nslm_decode_block(C.c_uint16(seed[i]), C.c_uint16(word[i]), C.c_int(e[i]), vp(p3[i]))
    np.savez_compressed(os.path.join(HERE, "blocks.npz"), seed=seed, word=word, e=e, p4=p4, p3=p3)
    # 2. a 64 x 512 P=4 matrix: ns_row_f32 rows and cpu_seed4_matvec_mt's y
    rows, kb, bias = 64, 64, -22
    p = packs.seed4p4(rng, 1, rows, kb * 8, eb=bias)
    x = rng.standard_normal(kb * 8).astype(np.float32)
    y = np.zeros(rows, dtype=np.float32)
    ref.ref_matvec(vp(p["seeds"][0]), vp(p["coefs"][0]), vp(p["codes"][0]), bias, vp(x), rows, kb, vp(y), 1)
    rr = np.zeros((rows, kb * 8), dtype=np.float32)
    for r in range(rows):
        ref.ref_row_f32(C.c_int(4), vp(p["seeds"][0]), vp(p["coefs"][0]), vp(p["codes"][0]), C.c_int32(bias), 0, rows,
                        kb * 8, r, 0, vp(rr[r]))
    np.savez_compressed(os.path.join(HERE, "matvec_p4.npz"), rows=rows, kb=kb, bias=bias, seeds=p["seeds"][0],
                        coefs=p["coefs"][0], codes=p["codes"][0], x=x, y_ref=y, rows_ref=rr)
    # 3. the same shape in P=3 and Q4: rows only (the GPU parity tests recompute the products in double)
    p3m = packs.seed4(rng, 1, rows, kb * 8, eb=-20)
    r3 = np.zeros((rows, kb * 8), dtype=np.float32)
    for r in range(rows):
        ref.ref_row_f32(C.c_int(1), vp(p3m["seeds"][0]), vp(p3m["nibs"][0]), None, C.c_int32(-20), 0, rows, kb * 8, r, 0, vp(r3[r]))
    q4 = packs.affine(rng, 1, rows, kb * 8, 4)
    rq = np.zeros((rows, kb * 8), dtype=np.float32)
    for r in range(rows):
        ref.ref_row_f32(C.c_int(3), vp(q4["words"][0]), vp(q4["scales"][0]), vp(q4["biases"][0]), C.c_int32(0), 64, rows, kb * 8, r, 1, vp(rq[r]))
    np.savez_compressed(os.path.join(HERE, "rows_p3_q4.npz"), rows=rows, K=kb * 8, p3_seeds=p3m["seeds"][0], p3_nibs=p3m["nibs"][0],
                        p3_eb=-20, p3_rows=r3, q4_words=q4["words"][0], q4_scales=q4["scales"][0], q4_biases=q4["biases"][0],
                        q4_rows_bf16=packs.f32_to_bf16_bits(rq))
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))


if __name__ == "__main__":
    main()
