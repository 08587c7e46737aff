"""Experts and router loaded from a model folder into the HBM layout: a layer step over the loaded stack is bit-equal to the
same stack filled from the arrays directly, for both seed formats and for streams larger than one staging buffer."""
import json
import struct

import numpy as np
import pytest

from nanoseedlm_amd import packs

pytestmark = pytest.mark.gpu


def write_folder(d, layer_tensors):
    """One safetensors shard + index with the logical tensors' streams under the names of nslm/model_st.h:5-17."""
    ents = []
    for name, arrs in layer_tensors.items():
        for suffix, dtype, a in arrs:
            a = np.ascontiguousarray(a)
            ents.append((name + suffix, dtype, a.shape, a.tobytes()))
    head, off = {}, 0
    for n, dt, shape, data in ents:
        head[n] = {"dtype": dt, "shape": list(shape), "data_offsets": [off, off + len(data)]}
        off += len(data)
    h = json.dumps(head).encode()
    h += b" " * ((-(8 + len(h))) % 16384)
    (d / "model-00001-of-00001.safetensors").write_bytes(struct.pack("<Q", len(h)) + h + b"".join(e[3] for e in ents))
    (d / "model.safetensors.index.json").write_text(json.dumps({"metadata": {}, "weight_map": {e[0]: "model-00001-of-00001.safetensors" for e in ents}}))


def streams(p):
    if p["fmt"] == packs.MF_SEED4P4:
        return [(".seeds", "U16", p["seeds"]), (".coefs", "U16", p["coefs"]), (".exp_bias", "I32", np.asarray(p["eb"], dtype=np.int32)),
                (".codes", "U8", p["codes"])]
    return [(".seeds", "U16", p["seeds"]), (".nibbles", "U16", p["nibs"]), (".exp_bias", "I32", np.asarray(p["eb"], dtype=np.int32))]


@pytest.mark.parametrize("fmt,E,d,ff", [(packs.MF_SEED4P4, 8, 256, 128), (packs.MF_SEED4, 8, 256, 128), (packs.MF_SEED4P4, 16, 2048, 768)])
def test_layer_step_from_a_folder(tmp_path, fmt, E, d, ff):
    from nanoseedlm_amd import backend, folder, moe
    backend.require_gpu()
    rng = np.random.default_rng(E + d)
    mk = packs.seed4p4 if fmt == packs.MF_SEED4P4 else packs.seed4
    k, T = 2, 3
    gate, up, down = mk(rng, E, ff, d, eb=-22), mk(rng, E, ff, d, eb=-21), mk(rng, E, d, ff, eb=-20)
    for p in (gate, up, down):
        p["eb"] = (np.asarray(p["eb"]) + rng.integers(-2, 3, E)).astype(np.int32)      # a different exponent bias per expert
    rw = packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.05).astype(np.float32))
    pre = "model.layers.0.mlp."
    write_folder(tmp_path, {pre + "experts.gate_proj": streams(gate), pre + "experts.up_proj": streams(up), pre + "experts.down_proj": streams(down),
                            pre + "gate": [(".weight", "BF16", rw)]})
    mf = folder.ModelFolder(tmp_path)
    t = mf.find(pre + "experts.gate_proj.weight")
    assert (t.enc, t.slices, t.rows, t.cols) == (fmt, E, ff, d)
    x = moe.DevBuf.from_array(packs.round_bf16(rng.standard_normal((T, d)).astype(np.float32)))
    outs = []
    for how in ("arrays", "folder"):
        st = moe.MoeStack(1, E, k, d, ff, fmt=fmt, router=moe.ROUTE_SOFTMAX, max_rows=8)
        if how == "arrays":
            st.set_layer(0, gate, up, down, rw)
        else:
            for which, nm in enumerate(("gate_proj", "up_proj", "down_proj")):
                mf.load_experts(st, 0, which, pre + "experts." + nm + ".weight")
            mf.load_router(st, 0, pre + "gate.weight")
            with pytest.raises(RuntimeError):
                mf.load_experts(st, 0, 2, pre + "experts.gate_proj.weight")              # [ff][d] is not a down matrix
        st.finalize()
        out = moe.DevBuf(4 * T * d)
        st.step(None, 0, x.ptr, T, out.ptr)
        moe.device_sync()
        outs.append(out.to_array(np.float32, (T, d)))
        st.close()
    mf.close()
    assert np.abs(outs[0]).max() > 0 and np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))


def test_upload_of_a_stream_longer_than_the_staging_buffers(tmp_path):
    """nsf_upload stages through two 8 MiB pinned buffers: a 20 MB stream, from an odd offset, arrives byte for byte."""
    import ctypes as C
    from nanoseedlm_amd import backend, folder, moe
    backend.require_gpu()
    rng = np.random.default_rng(9)
    big = rng.integers(0, 65536, (2560, 4096), dtype=np.uint16)       # 20 MiB of BF16 bit patterns
    write_folder(tmp_path, {"big": [(".weight", "BF16", big)]})
    mf = folder.ModelFolder(tmp_path)
    t = mf.find("big.weight")
    assert t.s[0].len == big.nbytes
    K = backend.host()
    K.nsf_upload.argtypes = [C.c_void_p, C.POINTER(folder.Stream), C.c_uint64, C.c_uint64]
    raw = big.view(np.uint8).reshape(-1)
    for skip, n in ((0, big.nbytes), (12345, 17 * 1024 * 1024 + 77), (big.nbytes - 5, 5)):
        dst = moe.DevBuf(n)
        assert K.nsf_upload(dst.ptr, C.byref(t.s[0]), skip, n) == 0
        assert np.array_equal(dst.to_array(np.uint8, (n,)), raw[skip:skip + n])
        dst.free()
    dst = moe.DevBuf(16)
    assert K.nsf_upload(dst.ptr, C.byref(t.s[0]), big.nbytes - 4, 8) == -1          # past the end of the stream
    mf.close()
