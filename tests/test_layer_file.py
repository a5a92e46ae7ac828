"""Host-side layer-file writer (no GPU): the safetensors container of SafeTensorsWriter (src/safetensors.cpp:93-137)
and the tensor set of write_layer_file (src/pipeline.cpp:329-340), checked by parsing the bytes directly, against an
independent loader (the safetensors package) and against the loader's expectations in runtime/src/qtip.cpp:216-276."""
import json
import os
import struct

import numpy as np
import pytest


def _fake_linear(pkg, m, n, seed):
    rng = np.random.default_rng(seed)
    o = pkg.LinearOut(name="x", m=m, n=n)
    o.trellis = rng.integers(0, 65536, (m // 16) * (n // 16) * 32, dtype=np.uint16)
    su = np.where(rng.integers(0, 2, n) > 0, 1.0, -1.0).astype(np.float32)
    o.su_bf16 = (su.view(np.uint32) >> 16).astype(np.uint16)
    o.sv = np.where(rng.integers(0, 2, m) > 0, 1.0, -1.0).astype(np.float32)
    o.wscale = float(np.float32(0.0173))
    return o


def _parse(path):
    raw = open(path, "rb").read()
    hl = struct.unpack("<Q", raw[:8])[0]
    hdr = raw[8:8 + hl].decode()
    return raw, hl, hdr, json.loads(hdr)


def test_container_bytes_exact(pkg, tmp_path):
    """Tiny file whose bytes are written down by hand: sorted keys, compact JSON, space padding, name-ordered data."""
    w = pkg.LayerFileWriter()
    w.add("b", "I16", [2], np.array([1, 2], np.int16))
    w.add("a.rcp", "I64", [], np.array(0, np.int64))
    w.add("Z", "F32", [1, 1], np.array([[1.5]], np.float32))     # upper case sorts before "__metadata__"
    p = str(tmp_path / "t.safetensors")
    nbytes = w.write(p)
    hdr = ('{"Z":{"data_offsets":[0,4],"dtype":"F32","shape":[1,1]},"__metadata__":{"format":"pt"},'
           '"a.rcp":{"data_offsets":[4,12],"dtype":"I64","shape":[]},"b":{"data_offsets":[12,16],"dtype":"I16","shape":[2]}}')
    hdr += " " * (-len(hdr) % 8)
    want = struct.pack("<Q", len(hdr)) + hdr.encode() + struct.pack("<f", 1.5) + struct.pack("<q", 0) + struct.pack("<hh", 1, 2)
    assert open(p, "rb").read() == want
    assert nbytes == len(want)
    assert not os.path.exists(p + ".tmp")
    w.close()


def test_metadata_variants_and_escaping(pkg, tmp_path):
    w = pkg.LayerFileWriter()
    w.add('we"ird\\name\n', "U8", [3], np.array([1, 2, 3], np.uint8))
    p = str(tmp_path / "m.safetensors")
    w.write(p, metadata={})
    _, hl, hdr, js = _parse(p)
    assert "__metadata__" not in js and list(js) == ['we"ird\\name\n'] and hl % 8 == 0
    w.write(p, metadata={"format": "pt", "a": 'q"'})
    _, _, hdr, js = _parse(p)
    assert js["__metadata__"] == {"a": 'q"', "format": "pt"}
    assert hdr.index('"a"') < hdr.index('"format"')


def test_add_checks_and_replace(pkg, tmp_path):
    w = pkg.LayerFileWriter()
    with pytest.raises(pkg.QtipError):
        w.add("x", "F32", [3], np.zeros(2, np.float32))       # byte count does not match shape x dtype
    with pytest.raises(pkg.QtipError):
        w.add("x", "F33", [2], np.zeros(2, np.float32))       # unknown dtype
    with pytest.raises(pkg.QtipError):
        w.add("__metadata__", "U8", [1], np.zeros(1, np.uint8))
    w.add("x", "F32", [2], np.array([1, 2], np.float32))
    w.add("x", "F32", [1], np.array([7], np.float32))         # same name: the later tensor wins
    p = str(tmp_path / "r.safetensors")
    w.write(p)
    raw, hl, _, js = _parse(p)
    assert js["x"] == {"data_offsets": [0, 4], "dtype": "F32", "shape": [1]}
    assert struct.unpack("<f", raw[8 + hl:])[0] == 7.0
    with pytest.raises(pkg.QtipError):
        w.write(str(tmp_path / "no_such_dir" / "r.safetensors"))


def test_qtip_layer_file_loads(pkg, oracle, hyb, tmp_path):
    """A layer with two QTIP linears + norms, read back with the safetensors package and checked against what the
    runtime loader requires (runtime/src/qtip.cpp:244-276): trellis I16 [(m/16)(n/16), 32], SU [n], SV [m] with Wscale
    folded in, tlut F16 [512, 2], rcp = 0, tp_rank = 8."""
    torch = pytest.importorskip("torch")
    st = pytest.importorskip("safetensors.torch")
    w = pkg.LayerFileWriter()
    lins = {"self_attn.o_proj": _fake_linear(pkg, 64, 96, 1), "mlp.down_proj": _fake_linear(pkg, 32, 128, 2)}
    pre = "model.layers.3."
    for name, lo in lins.items():
        w.add_qtip_linear(pre + name + ".", lo)
    ln = (np.ones(64, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    w.add(pre + "input_layernorm.weight", "BF16", [64], ln)
    w.add(pre + "post_attention_layernorm.weight", "BF16", [64], ln)
    p = str(tmp_path / "layer_3.safetensors")
    nbytes = w.write(p)
    assert os.path.getsize(p) == nbytes
    raw, hl, hdr, js = _parse(p)
    names = [k for k in js if k != "__metadata__"]
    assert names == sorted(names) and js["__metadata__"] == {"format": "pt"}
    off = 0
    for k in names:                       # data back to back in name order
        assert js[k]["data_offsets"][0] == off
        off = js[k]["data_offsets"][1]
    assert 8 + hl + off == nbytes
    T = st.load_file(p)
    tl = hyb.tlut.astype(np.float16)
    for name, lo in lins.items():
        b = pre + name + "."
        assert T[b + "trellis"].dtype == torch.int16 and tuple(T[b + "trellis"].shape) == ((lo.m // 16) * (lo.n // 16), 32)
        assert np.array_equal(T[b + "trellis"].numpy().view(np.uint16).reshape(-1), lo.trellis)
        assert T[b + "SU"].dtype == torch.bfloat16
        assert np.array_equal(T[b + "SU"].view(torch.int16).numpy().view(np.uint16), lo.su_bf16)
        assert T[b + "SV"].dtype == torch.float32
        assert np.array_equal(T[b + "SV"].numpy(), lo.sv * np.float32(lo.wscale))
        assert T[b + "tlut"].dtype == torch.float16 and tuple(T[b + "tlut"].shape) == (512, 2)
        assert np.array_equal(T[b + "tlut"].numpy().view(np.uint16), tl.view(np.uint16).reshape(512, 2))
        assert T[b + "rcp"].dtype == torch.int64 and T[b + "rcp"].shape == () and int(T[b + "rcp"]) == 0
        assert int(T[b + "tp_rank"]) == 8
    assert T[pre + "input_layernorm.weight"].dtype == torch.bfloat16


def test_qtip_linear_custom_tlut_and_bad_shapes(pkg, tmp_path):
    w = pkg.LayerFileWriter()
    lo = _fake_linear(pkg, 32, 32, 3)
    tl = np.arange(1024, dtype=np.uint16).reshape(512, 2)
    w.add_qtip_linear("q.", lo, tlut_f16=tl)
    p = str(tmp_path / "c.safetensors")
    w.write(p)
    raw, hl, _, js = _parse(p)
    a, b = js["q.tlut"]["data_offsets"]
    assert np.array_equal(np.frombuffer(raw[8 + hl + a:8 + hl + b], np.uint16), tl.reshape(-1))
    bad = _fake_linear(pkg, 32, 32, 3)
    bad.m = 24
    with pytest.raises(pkg.QtipError):
        w.add_qtip_linear("r.", bad)


def test_nvfp4_layer_file_loads(pkg, tmp_path):
    """An NVFP4 linear in a layer file (src/pipeline.cpp:342-346): weight_packed U8 [m, n/2], weight_scale F8_E4M3
    [m, n/16], weight_global_scale F32 scalar; an independent loader reading the scales as E4M3 numbers reproduces the
    library's dequantizer before its bf16 rounding."""
    torch = pytest.importorskip("torch")
    st = pytest.importorskip("safetensors.torch")
    rng = np.random.default_rng(4)
    wt = (rng.standard_normal((32, 64)) * 0.03).astype(np.float32)
    t = pkg.nvfp4_quantize(wt)
    w = pkg.LayerFileWriter()
    w.add_nvfp4_linear("model.layers.0.mlp.up_proj.", t)
    p = str(tmp_path / "nv.safetensors")
    w.write(p)
    T = st.load_file(p)
    b = "model.layers.0.mlp.up_proj."
    assert T[b + "weight_packed"].dtype == torch.uint8 and tuple(T[b + "weight_packed"].shape) == (32, 32)
    assert T[b + "weight_scale"].dtype == torch.float8_e4m3fn and tuple(T[b + "weight_scale"].shape) == (32, 4)
    assert T[b + "weight_global_scale"].shape == () and float(T[b + "weight_global_scale"]) == t.global_scale
    assert np.array_equal(T[b + "weight_packed"].numpy(), t.packed)
    levels = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6], np.float32)
    codes = np.stack([t.packed & 15, t.packed >> 4], axis=-1).reshape(32, 64)
    sc = T[b + "weight_scale"].float().numpy() * np.float32(t.global_scale)
    full = levels[codes] * np.repeat(sc, 16, axis=1)
    bf = torch.from_numpy(full).bfloat16().float().numpy()
    assert np.array_equal(bf, pkg.nvfp4_dequantize(t))
