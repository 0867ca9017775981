"""The checkpoint readers (ferrite_amd/st.py) on safetensors files written here: single file and sharded with an index,
EXL3 tensors (format.rs:34-57) and fused / sliced NVFP4 linears (fe-fp4 lib.rs:305-384)."""
import json
import os

import numpy as np
import pytest


def write_safetensors(path, tensors):
    """tensors: name -> (dtype string, shape, bytes)"""
    header, blob = {}, b""
    for name, (dtype, shape, data) in tensors.items():
        header[name] = {"dtype": dtype, "shape": list(shape), "data_offsets": [len(blob), len(blob) + len(data)]}
        blob += data
    header["__metadata__"] = {"format": "pt"}
    h = json.dumps(header).encode()
    h += b" " * (-len(h) % 8)
    with open(path, "wb") as f:
        f.write(len(h).to_bytes(8, "little") + h + blob)


def exl3_entries(base, t, mul1=0x83DCD12D):
    return {
        f"{base}.trellis": ("I16", (t.k // 16, t.n // 16, 16 * t.bits), t.trellis.tobytes()),
        f"{base}.suh": ("F16", (t.k,), t.suh.tobytes()),
        f"{base}.svh": ("F16", (t.n,), t.svh.tobytes()),
        f"{base}.mul1": ("I32", (), np.uint32(mul1).tobytes()),
    }


def test_exl3_load_single_file_and_shards(tmp_path):
    from ferrite_amd import st, synth
    a, b = synth.exl3_tensor(256, 384, 3, 1), synth.exl3_tensor(128, 128, 5, 2)
    one = tmp_path / "one"
    one.mkdir()
    write_safetensors(one / "model.safetensors", {**exl3_entries("m.a", a), **exl3_entries("m.b", b)})
    two = tmp_path / "two"
    two.mkdir()
    write_safetensors(two / "model-00001-of-00002.safetensors", exl3_entries("m.a", a))
    write_safetensors(two / "model-00002-of-00002.safetensors", exl3_entries("m.b", b))
    wm = {k: "model-00001-of-00002.safetensors" for k in exl3_entries("m.a", a)}
    wm.update({k: "model-00002-of-00002.safetensors" for k in exl3_entries("m.b", b)})
    (two / "model.safetensors.index.json").write_text(json.dumps({"weight_map": wm}))
    for folder in (one, two):
        ck = st.Checkpoint(str(folder))
        for base, t in (("m.a", a), ("m.b", b)):
            got = st.load_exl3(ck, base)
            assert (got.k, got.n, got.bits) == (t.k, t.n, t.bits)
            assert np.array_equal(got.trellis, t.trellis) and np.array_equal(got.suh, t.suh) and np.array_equal(got.svh, t.svh)
        with pytest.raises(KeyError):
            st.load_exl3(ck, "m.missing")


def test_exl3_load_rejects_what_the_reference_rejects(tmp_path):
    from ferrite_amd import st, synth
    t = synth.exl3_tensor(128, 128, 4, 3)
    e = exl3_entries("x", t, mul1=0x12345678)
    write_safetensors(tmp_path / "model.safetensors", e)
    with pytest.raises(ValueError, match="mul1"):
        st.load_exl3(st.Checkpoint(str(tmp_path)), "x")
    e = exl3_entries("x", t)
    e["x.trellis"] = ("I16", (8, 8, 72), t.trellis.tobytes() + b"\0" * (8 * 8 * 8 * 2))  # 4.5 bits
    write_safetensors(tmp_path / "model.safetensors", e)
    with pytest.raises(ValueError, match="half-integer"):
        st.load_exl3(st.Checkpoint(str(tmp_path)), "x")
    e = exl3_entries("x", t)
    e["x.svh"] = ("F16", (64,), t.svh[:64].tobytes())
    write_safetensors(tmp_path / "model.safetensors", e)
    with pytest.raises(ValueError, match="svh"):
        st.load_exl3(st.Checkpoint(str(tmp_path)), "x")


def nvfp4_entries(name, h, wscale, in_scale):
    return {
        f"{name}.weight": ("U8", h.codes.shape, h.codes.tobytes()),
        f"{name}.weight_scale": ("F8_E4M3", h.sf.shape, h.sf.tobytes()),
        f"{name}.weight_scale_2": ("F32", (), np.float32(wscale).tobytes()),
        f"{name}.input_scale": ("F32", (), np.float32(in_scale).tobytes()),
    }


def test_nvfp4_load_fused_and_sliced(tmp_path):
    from ferrite_amd import st, synth
    g, u = synth.fp4_linear(256, 512, 1), synth.fp4_linear(384, 512, 2)
    write_safetensors(tmp_path / "model.safetensors", {**nvfp4_entries("l.gate", g, 0.5, 0.02), **nvfp4_entries("l.up", u, 0.25, 0.03)})
    ck = st.Checkpoint(str(tmp_path))
    assert ck.algo("l.gate") == "NVFP4" and ck.algo("l.none") is None
    h = st.load_nvfp4(ck, ["l.gate", "l.up"])
    assert (h.n, h.k) == (640, 512) and h.name == "l.gate+l.up"
    assert np.array_equal(h.codes, np.concatenate([g.codes, u.codes])) and np.array_equal(h.sf, np.concatenate([g.sf, u.sf]))
    # alpha = max(input_scale) * weight_scale_2, g = 1 / max(input_scale) (lib.rs:345-350, 378-383), in f32
    in_scale = np.float32(0.03)
    assert np.array_equal(h.alpha[:256], np.full(256, np.float32(0.5) * in_scale, np.float32))
    assert np.array_equal(h.alpha[256:], np.full(384, np.float32(0.25) * in_scale, np.float32))
    assert h.g == float(np.float32(1.0) / in_scale)
    # a tensor-parallel slice: rows 128..256 of gate, 0..128 and 256..384 of up, K 128..384
    sl = [st.Slice([(128, 256)], (128, 384)), st.Slice([(0, 128), (256, 384)], (128, 384))]
    hs = st.load_nvfp4(ck, ["l.gate", "l.up"], sl)
    assert (hs.n, hs.k) == (384, 256)
    want = np.concatenate([g.codes[128:256, 64:192], u.codes[0:128, 64:192], u.codes[256:384, 64:192]])
    assert np.array_equal(hs.codes, want)
    want = np.concatenate([g.sf[128:256, 8:24], u.sf[0:128, 8:24], u.sf[256:384, 8:24]])
    assert np.array_equal(hs.sf, want)
    with pytest.raises(ValueError, match="slice"):
        st.load_nvfp4(ck, ["l.gate"], [st.Slice([(0, 100)], (0, 512))])
    with pytest.raises(ValueError, match="NVFP4"):
        st.load_nvfp4(ck, ["l.none"])
