"""The C-ABI library loads without a GPU, exports every symbol the header
declares, and fails with status codes (never aborts) on the host-checkable
error paths."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ek_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ek_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported(ek):
    lib = ek.load()
    names = declared_symbols()
    assert len(names) >= 16
    for n in names:
        assert hasattr(lib, n), f"{n} declared in ek_hip.h but not exported"
    from ek_hip import _capi
    assert sorted(_capi.PROTOTYPES) == names, "ctypes prototypes out of sync with the header"


def test_backend_name(ek):
    assert ek.load().ek_backend_name() == b"hip"


def test_invalid_cfg_is_reported_not_fatal(ek):
    from ek_hip import _capi as C
    lib = ek.load()
    h = ctypes.c_void_p()
    bad = [
        dict(hidden=100, inter=64),                 # rows are moved 16 bytes at a time
        dict(hidden=0), dict(inter=0),
        dict(act_dtype=C.EK_F32),
        dict(w_dtype=C.EK_F16),                     # neither act dtype nor int8
        dict(n_experts=0), dict(n_experts=5000),
        dict(top_k=0), dict(top_k=99),
        dict(max_tokens=0), dict(max_tokens=1 << 40),
    ]
    base = dict(hidden=128, inter=64, n_experts=8, top_k=2, act_dtype=C.EK_BF16, w_dtype=C.EK_BF16,
                max_tokens=16, device_id=0, flags=0)
    for patch in bad:
        cfg = C.ek_cfg(**{**base, **patch})
        st = lib.ek_layer_create(ctypes.byref(cfg), ctypes.byref(h))
        assert st == C.EK_INVALID_INPUT, (patch, st)
        assert lib.ek_last_error(), patch
        assert not h.value
    assert lib.ek_layer_create(None, ctypes.byref(h)) == C.EK_INVALID_INPUT
    cfg = C.ek_cfg(**base)
    assert lib.ek_layer_create(ctypes.byref(cfg), None) == C.EK_INVALID_INPUT


def test_null_handles(ek):
    from ek_hip import _capi as C
    lib = ek.load()
    assert lib.ek_layer_destroy(None) == C.EK_INVALID_INPUT
    assert lib.ek_layer_forward(None, None, None, None, 0, 0, None, None, 0, None) == C.EK_INVALID_INPUT
    assert lib.ek_layer_pack(None, None, 0, None, None, None, 0, None) == C.EK_INVALID_INPUT
    assert lib.ek_layer_expert_forward(None, 0, None, 0, None, 0, None) == C.EK_INVALID_INPUT
    assert lib.ek_expert_forward(None, None, 0, None, 0, None) == C.EK_INVALID_INPUT
    assert lib.ek_expert_destroy(None) == C.EK_INVALID_INPUT
    assert lib.ek_layer_get_stats(None, None) == C.EK_INVALID_INPUT


def test_no_device_is_an_error_code(ek):
    """Without a GPU, creation returns EK_HIP_ERROR with a message; with one, it works."""
    from ek_hip import _capi as C
    lib = ek.load()
    if lib.ek_device_count() > 0:
        pytest.skip("a GPU is visible")
    with pytest.raises(ek.EKError) as ei:
        ek.HipLayer(128, 64, 8, 2)
    assert ei.value.status == C.EK_HIP_ERROR and "device" in ei.value.message


def test_weight_lookup_suffixes(ek):
    """ExpertWeight::from_safetensor's suffix table (ffn/meta.rs:56-75)."""
    import torch
    t = lambda: torch.zeros(2, 2)
    w = ek.ExpertWeight.from_safetensor({"model.layers.0.mlp.experts.1.up_proj.weight": t(),
                                         "model.layers.0.mlp.experts.1.down_proj.weight": t(),
                                         "model.layers.0.mlp.experts.1.gate_proj.weight": t()})
    assert w.up_w is not None and w.up_scale is None
    ek.ExpertWeight.from_safetensor({"a.w1.weight": t(), "a.w2.weight": t(), "a.w3.weight": t()})
    for missing, text in (("w1", "w1/up_w"), ("w2", "w2/down_w"), ("w3", "w3/gate_w")):
        d = {f"a.{k}.weight": t() for k in ("w1", "w2", "w3") if k != missing}
        with pytest.raises(ek.EKError) as ei:
            ek.ExpertWeight.from_safetensor(d)
        assert ei.value.status == 3 and text in ei.value.message


def test_header_is_plain_c_and_links_from_c(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 on its own, and a C program linked
    against the library must be able to call it (no GPU needed for these entry points)."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    from ek_hip import _capi as C
    src = tmp_path / "abi.c"
    src.write_text(r'''
#include "ek_hip.h"
#include <stdio.h>
#include <string.h>
int main(void) {
    int32_t layer = -1, expert = -1;
    char id[64];
    ek_cfg cfg; ek_weight_desc d; ek_route_out ro; ek_stats st; ek_router_cfg rc; ek_histogram h; ek_tensor_view tv;
    (void)cfg; (void)d; (void)ro; (void)st; (void)rc; (void)h; (void)tv;
    if (strcmp(ek_backend_name(), "hip") != 0) return 1;
    if (ek_expert_id_format("ds-tiny", 3, 17, id, sizeof id) != EK_OK) return 2;
    if (ek_expert_id_parse(id, &layer, &expert) != EK_OK || layer != 3 || expert != 17) return 3;
    if (ek_expert_id_parse("nonsense", &layer, &expert) != EK_INVALID_INPUT) return 4;
    if (strlen(ek_last_error()) == 0) return 5;
    if (ek_layer_forward(NULL, NULL, NULL, NULL, EK_BF16, 0, NULL, NULL, EK_HOST, NULL) != EK_INVALID_INPUT) return 6;
    printf("%s %s\n", ek_backend_name(), id);
    return 0;
}
''')
    inc = os.path.join(ROOT, "include")
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only", "-I", inc, str(src)])
    exe = tmp_path / "abi"
    libdir = os.path.dirname(C.LIB_PATH)
    subprocess.check_call(["gcc", "-std=c99", "-I", inc, str(src), "-o", str(exe), "-L", libdir, "-lek_hip",
                           "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"])
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, (out.returncode, out.stdout, out.stderr)
    assert out.stdout.strip() == "hip ds-tiny/l3-e17"


def test_batcher_rejects_bad_arguments_without_a_gpu(ek):
    from ek_hip import _capi as C
    lib = ek.load()
    out = ctypes.c_void_p()
    assert lib.ek_batcher_create(None, 0, 1, ctypes.byref(out)) == C.EK_INVALID_INPUT
    n = ctypes.c_size_t()
    buf = ctypes.create_string_buffer(8)
    assert lib.ek_batcher_forward(None, b"m/l0-e0", buf, 8, buf, 8, ctypes.byref(n)) == C.EK_INVALID_INPUT
    assert lib.ek_batcher_get_stats(None, None) == C.EK_INVALID_INPUT
    assert lib.ek_batcher_destroy(None) == C.EK_OK
    assert b"NULL" in lib.ek_last_error()
