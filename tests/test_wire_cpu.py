"""Wire format of the worker contract, host side only (no GPU needed).

The checker for the safetensors codec is the `safetensors` Python package (the
Rust implementation the reference links, behind its Python binding): blobs
written by it must parse, and blobs written here must be byte-identical to its
output and load back through it.  The id codec is checked against the cases
ExpertKey::from_expert_id accepts and rejects (ek-db/src/safetensor/mod.rs:57-73).
"""
import ctypes
import json
import struct

import numpy as np
import pytest
import torch
from safetensors.torch import load as st_load
from safetensors.torch import save as st_save

from ek_hip import _capi as C
from ek_hip import wire


@pytest.mark.parametrize("text,layer,expert", [
    ("ds-tiny/l0-e0", 0, 0),
    ("qwen3-30b/l47-e127", 47, 127),
    ("org/model/l3-e255", 3, 255),       # only "/l" splits; other slashes belong to the model name
    ("m-e1/l2-e9", 2, 9),                # "-e" before "/l" belongs to the model name
    ("m/l+4-e+5", 4, 5),                 # usize::from_str takes a leading plus
])
def test_expert_id_parse(text, layer, expert):
    key = wire.ExpertKey.from_expert_id(text)
    assert (key.layer, key.expert) == (layer, expert)


@pytest.mark.parametrize("text", ["", "model", "m/l1", "m/l1-e", "m/l-e1", "m/lx-e1", "m/l1-ey", "m/l1-e2-e3",
                                  "a/l1-e2/l3-e4", "m/l-1-e2", "m/l1 -e2", "m/l1-e2 "])
def test_expert_id_rejects(text):
    with pytest.raises(C.EKError) as ei:
        wire.ExpertKey.from_expert_id(text)
    assert ei.value.status == C.EK_INVALID_INPUT


def test_expert_id_round_trip():
    for model, layer, expert in [("ds-tiny", 0, 0), ("deepseek-v3", 60, 255), ("a/b", 7, 1023)]:
        text = wire.ExpertKey(model, layer, expert).as_object_key()
        assert text == f"{model}/l{layer}-e{expert}"
        back = wire.ExpertKey.from_expert_id(text)
        assert (back.model, back.layer, back.expert) == (model, layer, expert)
    buf = ctypes.create_string_buffer(4)
    assert C.load().ek_expert_id_format(b"model", 1, 2, buf, 4) == C.EK_INVALID_INPUT


def _rand(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    if dtype == torch.int8:
        return torch.randint(-128, 128, shape, generator=g, dtype=torch.int8)
    if dtype == torch.float8_e4m3fn:
        return torch.randint(0, 256, shape, generator=g, dtype=torch.uint8).view(torch.float8_e4m3fn)
    return torch.randn(shape, generator=g).to(dtype)


def _same(a, b):
    return a.dtype == b.dtype and a.shape == b.shape and \
        torch.equal(a.contiguous().view(torch.uint8), b.contiguous().view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32, torch.int8, torch.float8_e4m3fn])
@pytest.mark.parametrize("shape", [(1, 64), (17, 128), (0, 64), (5,), (2, 3, 4)])
def test_emit_matches_safetensors(dtype, shape):
    t = _rand(shape, dtype, 1)
    mine = wire.emit("data", t)
    theirs = st_save({"data": t})
    assert mine == theirs                       # byte for byte, header padding included
    assert _same(st_load(mine)["data"], t)
    assert _same(wire.find(theirs, "data"), t)


def test_find_in_multi_tensor_blob():
    tensors = {
        "model.layers.3.mlp.experts.7.up_proj.weight": _rand((128, 64), torch.bfloat16, 2),
        "model.layers.3.mlp.experts.7.gate_proj.weight": _rand((128, 64), torch.bfloat16, 3),
        "model.layers.3.mlp.experts.7.down_proj.weight": _rand((64, 128), torch.bfloat16, 4),
        "model.layers.3.mlp.experts.7.down_proj.weight_scale_inv": _rand((1, 1), torch.float32, 5),
    }
    blob = st_save(tensors, metadata={"format": "pt", "note": "a {nested} \"quoted\" [value]"})
    for name, t in tensors.items():
        assert _same(wire.find(blob, name), t)
    # lookup_suffix: "…down_proj.weight_scale_inv" does not end with "down_proj.weight"
    assert _same(wire.find_suffix(blob, ["w2.weight", "down_proj.weight"]),
                 tensors["model.layers.3.mlp.experts.7.down_proj.weight"])
    assert _same(wire.find_suffix(blob, ["w1.weight", "up_proj.weight"]),
                 tensors["model.layers.3.mlp.experts.7.up_proj.weight"])
    with pytest.raises(C.EKError) as ei:
        wire.find(blob, "data")
    assert ei.value.status == C.EK_WEIGHT_NOT_FOUND
    with pytest.raises(C.EKError) as ei:
        wire.find_suffix(blob, ["w9.weight"])
    assert ei.value.status == C.EK_WEIGHT_NOT_FOUND


def _blob(header: dict, data: bytes = b"", pad=True) -> bytes:
    h = json.dumps(header, separators=(",", ":")).encode()
    if pad:
        h += b" " * ((8 - len(h) % 8) % 8)
    return struct.pack("<Q", len(h)) + h + data


@pytest.mark.parametrize("blob", [
    b"",
    b"\x01\x02\x03",
    struct.pack("<Q", 1 << 40) + b"{}",                                                        # header longer than blob
    struct.pack("<Q", 2) + b"[]",                                                              # not an object
    _blob({"data": {"dtype": "BF16", "shape": [2, 4], "data_offsets": [0, 16]}}, b"\0" * 8),   # data truncated
    _blob({"data": {"dtype": "BF16", "shape": [2, 4], "data_offsets": [0, 12]}}, b"\0" * 16),  # size mismatch
    _blob({"data": {"dtype": "BF16", "shape": [2, 4], "data_offsets": [8, 4]}}, b"\0" * 16),   # end < begin
    _blob({"data": {"dtype": "BF16", "shape": [2, -4], "data_offsets": [0, 16]}}, b"\0" * 16),
    _blob({"data": {"dtype": "U64", "shape": [2], "data_offsets": [0, 16]}}, b"\0" * 16),      # dtype outside ek_dtype
    _blob({"data": {"dtype": "BF16", "shape": [1, 1, 1, 1, 8], "data_offsets": [0, 16]}}, b"\0" * 16),
    _blob({"data": {"dtype": "BF16", "shape": [1 << 40, 1 << 40], "data_offsets": [0, 16]}}, b"\0" * 16),
    struct.pack("<Q", 24) + b'{"data":{"dtype":"BF16",',                                       # cut mid-object
])
def test_malformed_blobs_are_rejected(blob):
    view = C.ek_tensor_view()
    st = C.load().ek_safetensors_find(blob, len(blob), b"data", ctypes.byref(view))
    assert st == C.EK_INVALID_INPUT, C.load().ek_last_error()


def test_unpadded_header_and_key_order_are_accepted():
    data = np.arange(8, dtype=np.float32).tobytes()
    blob = _blob({"__metadata__": {"k": "v"},
                  "data": {"data_offsets": [0, 32], "shape": [2, 4], "dtype": "F32"}}, data, pad=False)
    t = wire.find(blob, "data")
    assert t.dtype == torch.float32 and t.tolist() == [[0, 1, 2, 3], [4, 5, 6, 7]]


def test_emit_rejects_small_buffer_and_bad_description():
    lib = C.load()
    shape = (ctypes.c_int64 * 2)(2, 4)
    assert lib.ek_safetensors_size(b"data", 99, 2, shape) == 0
    assert lib.ek_safetensors_size(b"data", C.EK_BF16, 5, shape) == 0
    need = lib.ek_safetensors_size(b"data", C.EK_BF16, 2, shape)
    src = ctypes.create_string_buffer(16)
    out = ctypes.create_string_buffer(need)
    assert lib.ek_safetensors_emit(b"data", C.EK_BF16, 2, shape, src, out, need - 1, None) == C.EK_INVALID_INPUT
    assert lib.ek_safetensors_emit(b"data", C.EK_BF16, 2, shape, src, out, need, None) == C.EK_OK


def test_parser_survives_mutated_blobs():
    """Blobs arrive over the wire: whatever the bytes, the parser answers with a status and a view
    that lies inside the blob (a crash would take the test process down)."""
    lib = C.load()
    rng = np.random.default_rng(20240607)
    good = [st_save({"data": _rand((5, 64), torch.bfloat16, 3)}),
            st_save({"a.w1.weight": _rand((8, 8), torch.float32, 4), "data": _rand((3, 16), torch.int8, 5)},
                    metadata={"k": "v"})]
    ok = bad = 0
    for it in range(6000):
        blob = bytearray(good[it % 2])
        kind = it % 6
        if kind == 0:                                   # truncate anywhere
            del blob[int(rng.integers(0, len(blob))):]
        elif kind == 1:                                 # flip bytes in the header
            hl = struct.unpack("<Q", bytes(blob[:8]))[0]
            for _ in range(int(rng.integers(1, 6))):
                blob[8 + int(rng.integers(0, hl))] = int(rng.integers(0, 256))
        elif kind == 2:                                 # corrupt the length prefix
            blob[:8] = struct.pack("<Q", int(rng.integers(0, 1 << 62)))
        elif kind == 3:                                 # splice digits into numbers
            hl = struct.unpack("<Q", bytes(blob[:8]))[0]
            pos = 8 + int(rng.integers(0, hl))
            blob[pos:pos] = b"9" * int(rng.integers(1, 30))
        elif kind == 4:                                 # random garbage of the same length
            blob = bytearray(rng.integers(0, 256, len(blob), dtype=np.uint8).tobytes())
        else:                                           # drop a slice of the header
            hl = struct.unpack("<Q", bytes(blob[:8]))[0]
            a = 8 + int(rng.integers(0, hl))
            del blob[a:a + int(rng.integers(1, 12))]
        buf = (ctypes.c_char * max(len(blob), 1)).from_buffer(blob if len(blob) else bytearray(1))
        view = C.ek_tensor_view()
        st = lib.ek_safetensors_find(buf, len(blob), b"data", ctypes.byref(view))
        assert st in (C.EK_OK, C.EK_INVALID_INPUT, C.EK_WEIGHT_NOT_FOUND)
        if st == C.EK_OK:
            ok += 1
            base = ctypes.addressof(buf)
            assert base <= view.data and view.data + view.nbytes <= base + len(blob)
            assert 0 <= view.rank <= 4 and view.nbytes >= 0
        else:
            bad += 1
    assert bad > 3000 and ok > 0


def _blob_with_header(header: bytes, payload: bytes) -> bytes:
    return struct.pack("<Q", len(header)) + header + payload


def test_deeply_nested_header_is_refused_not_recursed_into():
    """An unknown key (or a __metadata__) whose value nests a million levels deep must come back
    as EK_INVALID_INPUT: the value skipper recurses once per level, and wire bytes are untrusted
    (an unbounded recursion would overflow the worker thread's stack).  Nesting of a few levels,
    which a real header can hold, still parses."""
    lib = C.load()
    data = bytes(64)
    entry = b'"data":{"dtype":"BF16","shape":[4,8],"data_offsets":[0,64]}'
    view = C.ek_tensor_view()
    for depth, want in ((3, C.EK_OK), (20, C.EK_OK), (64, C.EK_INVALID_INPUT), (1_000_000, C.EK_INVALID_INPUT)):
        for opener, closer in ((b"[", b"]"), (b'{"k":', b"}")):
            nested = opener * depth + b"1" + closer * depth
            # as the __metadata__ value, and as an unknown field inside a tensor's entry
            for head in (b'{"__metadata__":' + nested + b",",
                         b'{"other":{"dtype":"BF16","shape":[0],"data_offsets":[0,0],"extra":' + nested + b"},"):
                key = head[:16]
                blob = _blob_with_header(head + entry + b"}", data)
                st = lib.ek_safetensors_find(blob, len(blob), b"data", ctypes.byref(view))
                assert st == want, (depth, opener, key, st)
                if want == C.EK_OK:
                    assert view.nbytes == 64 and list(view.shape[:2]) == [4, 8]
        # unbalanced: only openers
        blob = _blob_with_header(b'{"x":' + b"[" * depth, data)
        assert lib.ek_safetensors_find(blob, len(blob), b"data", ctypes.byref(view)) == C.EK_INVALID_INPUT


def test_parser_under_the_host_sanitizers(tmp_path):
    """The same kind of mutations, 300 000 of them, through a build of the wire parser's host code
    with AddressSanitizer and UndefinedBehaviorSanitizer (tests/wire_fuzz.cpp; blobs are exact-size
    heap copies): an out-of-bounds read, a signed overflow or a bad shift inside the parser ends the
    run with a report instead of going unnoticed."""
    import os
    import shutil
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    hipcc, clang = "/opt/rocm/bin/hipcc", "/opt/rocm/llvm/bin/clang++"
    lib_dir = os.path.join(root, "expert-kit_amd", "lib")
    if not (os.path.exists(hipcc) and os.path.exists(clang)):
        pytest.skip("no ROCm compiler here")
    assert os.path.exists(os.path.join(lib_dir, "libek_hip.so")), "build the library first"
    san = ["-fsanitize=address", "-fsanitize=undefined", "-fno-sanitize-recover=undefined"]
    host_san = [a for s in san for a in ("-Xarch_host", s)]
    obj, drv, exe = (str(tmp_path / n) for n in ("ek_wire.o", "wire_fuzz.o", "wire_fuzz"))
    src = os.path.join(root, "expert-kit_amd", "csrc")
    run = lambda cmd: subprocess.run(cmd, check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    run([hipcc, "--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-fPIC", *host_san, "-Xclang", "-target-feature",
         "-Xclang", "-packed-fp32-ops", "-I" + src, "-c", os.path.join(src, "ek_wire.hip"), "-o", obj])
    run([clang, "-O1", "-g", "-std=c++17", *san, "-I" + os.path.join(root, "include"), "-c",
         os.path.join(root, "tests", "wire_fuzz.cpp"), "-o", drv])
    # the executable's own (instrumented) parser takes precedence over the library's copy, which
    # only supplies the layer entry points ek_wire.hip refers to
    run([clang, *san[:2], drv, obj, "-L" + lib_dir, "-lek_hip", "-L/opt/rocm/lib", "-lamdhip64",
         "-Wl,-rpath," + lib_dir, "-Wl,-rpath,/opt/rocm/lib", "-o", exe])
    got = subprocess.run([exe, "300000"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert got.returncode == 0, got.stdout[-3000:]
    ok, bad = (int(f.split("=")[1]) for f in got.stdout.split()[-2:])
    assert ok > 1000 and bad > 100000
    shutil.rmtree(tmp_path, ignore_errors=True)
