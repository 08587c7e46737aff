"""Writes tests/golden/model_folder/ with the reference's own model-folder WRITER (ns_write of nslm/lib_model_st.c, in the
compiled reference oracle/_ref/libnslm_ref.so) and tests/golden/model_folder.json, the list of what was written.  Run in
the build container only; the folder is data (safetensors shards + index), read back by tests/test_model_folder.py.

    python tests/golden/make_folder_golden.py
"""
import ctypes as C
import json
import os
import shutil
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import oracle as orc  # noqa: E402

# (name, encoding, slices, rows, cols); encodings as nslm/model_st.h:31 (= MF_*)
SPECS = [
    ("model.embed_tokens.weight", 2, 1, 96, 128),
    ("model.norm.weight", 0, 1, 1, 64),
    ("model.layers.3.mlp.gate.weight", 0, 1, 4, 64),
    ("model.layers.3.mlp.gate.bias", 0, 1, 1, 4),
    ("model.layers.3.mlp.experts.gate_proj.weight", 4, 4, 64, 256),
    ("model.layers.3.self_attn.q_proj.weight", 5, 1, 64, 256),
    ("model.layers.3.mlp.experts.down_proj.weight", 1, 4, 64, 128),
    ("model.layers.3.self_attn.v_experts.weight", 3, 3, 64, 128),
    ("model.layers.3.mlp.shared_experts.up_proj.weight", 0, 2, 32, 64),
    ("lm_head.weight", 2, 1, 96, 128),
    ("model.layers.3.self_attn.mla.kv_a_x", 2, 1, 64, 128),      # affine, not named *.weight: codes under the bare name
    ("model.layers.3.self_attn.mla.q_lat", 3, 4, 64, 128),
]
SHARD_BYTES = 60000


def pattern(t, s, i):
    """Byte i of stream s of tensor t."""
    return (i * 131 + (i >> 8) * 29 + t * 17 + s * 5) & 255


class NsSpec(C.Structure):
    _fields_ = [("name", C.c_char_p), ("enc", C.c_int), ("slices", C.c_int), ("rows", C.c_int), ("cols", C.c_int)]


FILL = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_uint8), C.c_uint64)


def main():
    orc.build()
    ref = orc.ref()
    assert ref is not None, "oracle/_ref/libnslm_ref.so missing: run make -C oracle ref"
    out = os.path.join(HERE, "model_folder")
    shutil.rmtree(out, ignore_errors=True)
    os.makedirs(out)
    specs = (NsSpec * len(SPECS))(*[NsSpec(n.encode(), e, s, r, c) for n, e, s, r, c in SPECS])

    def fill(ctx, t, s, dst, n):
        for i in range(n):
            dst[i] = pattern(t, s, i)
        return 0
    err = C.create_string_buffer(512)
    ref.ns_write.argtypes = [C.c_char_p, C.POINTER(NsSpec), C.c_int, C.c_uint64, C.c_char_p, FILL, C.c_void_p, C.c_char_p, C.c_int]
    rc = ref.ns_write(out.encode(), specs, len(SPECS), SHARD_BYTES, b'"producer": "make_folder_golden"', FILL(fill), None, err, 512)
    assert rc == 0, err.value
    with open(os.path.join(HERE, "model_folder.json"), "w") as f:
        json.dump({"specs": SPECS, "pattern": "(i * 131 + (i >> 8) * 29 + t * 17 + s * 5) & 255", "shard_bytes": SHARD_BYTES}, f, indent=1)
    print(sorted(os.listdir(out)), sum(os.path.getsize(os.path.join(out, f)) for f in os.listdir(out)), "bytes")


if __name__ == "__main__":
    main()
