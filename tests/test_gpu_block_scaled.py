"""Layers that keep fp8 (e4m3fn) or int8 weights with 128x128 block scales as the checkpoint stores them.

The arithmetic is the reference's w8a16_activate (ek-computation/src/ffn/expert_torch.rs:24-53):
W[r,c] = rne_16bit(f32(fp8[r,c]) * scale[r/128, c/128]), here applied in registers by both
kernel families instead of once at load.  Bars: the FFN / layer gates of test_gpu_parity.py
against the oracle fed with weights dequantised that way on the CPU; the fp8 bytes cover all
254 finite encodings, the int8 ones all 256 values.
"""
import pytest
import torch
from safetensors.torch import save as st_save

from test_gpu_parity import check_vs_rounded, ffn_gate, layer_gate

pytestmark = pytest.mark.gpu
F8 = torch.float8_e4m3fn


def fp8_matrix(r, c, g):
    """Shaped like a quantised checkpoint block (a Gaussian scaled so that its tail reaches the
    format's 448), with every finite e4m3fn byte planted at a few random places."""
    w = (torch.randn(r, c, generator=g) * 110).clamp(-448, 448).to(F8).view(torch.uint8).flatten()
    codes = torch.tensor([b for b in range(256) if (b & 0x7f) != 0x7f], dtype=torch.uint8).repeat(3)
    w[torch.randperm(r * c, generator=g)[:codes.numel()]] = codes
    return w.view(r, c).view(F8)


def block_scales(r, c, g):
    return torch.rand((r + 127) // 128, (c + 127) // 128, generator=g) * 3e-4 + 5e-5


def dequant(oracle, w, sc, dt):
    """The oracle's w8a16_activate: its own fp8 widening, its block dequantisation for bf16; the
    fp16 layer's form (same product, rounded to fp16) written out."""
    wf = oracle.fp8_e4m3fn_to_f32(w) if w.dtype == F8 else w.float()
    if dt == torch.bfloat16:
        return oracle.dequant_block(wf, sc)
    full = sc.repeat_interleave(128, 0)[:w.shape[0]].repeat_interleave(128, 1)[:, :w.shape[1]]
    return (wf * full).to(dt)


def int8_matrix(r, c, g):
    return torch.randint(-128, 128, (r, c), generator=g, dtype=torch.int8)


KINDS = {"fp8": dict(w_dtype=F8), "int8": dict(w_dtype=torch.int8, block_scales=True)}


def make_expert(ek, H, I, seed, kind="fp8"):
    g = torch.Generator().manual_seed(seed)
    mat = fp8_matrix if kind == "fp8" else int8_matrix
    return ek.ExpertWeight(up_w=mat(I, H, g), gate_w=mat(I, H, g), down_w=mat(H, I, g),
                           up_scale=block_scales(I, H, g), gate_scale=block_scales(I, H, g),
                           down_scale=block_scales(H, I, g))


def ref_weights(oracle, ew, dt):
    return (dequant(oracle, ew.up_w, ew.up_scale, dt), dequant(oracle, ew.gate_w, ew.gate_scale, dt),
            dequant(oracle, ew.down_w, ew.down_scale, dt))


def test_all_finite_encodings_are_drawn():
    g = torch.Generator().manual_seed(1)
    seen = set(fp8_matrix(64, 64, g).view(torch.uint8).flatten().tolist())
    assert len(seen) == 254 and 0x7f not in seen and 0xff not in seen


@pytest.mark.parametrize("kind", ["fp8", "int8"])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [1, 7, 16, 17, 40, 64, 65, 200])
def test_one_expert_streamed(ek, oracle, cuda, dt, n, kind):
    """A lone per-expert call: the sliced streaming form (n <= 16) and its 64-row form."""
    H, I = 384, 256
    print(f"fp8 expert dt={dt} n={n}", flush=True)
    layer = ek.HipLayer(H, I, 2, 1, act_dtype=dt, max_tokens=256, **KINDS[kind])
    ew = make_expert(ek, H, I, 11, kind)
    layer.set_expert(1, ew)
    x = torch.randn(n, H, generator=torch.Generator().manual_seed(n)).to(dt)
    ref = oracle.ffn(x, *ref_weights(oracle, ew, dt), mode=2)
    got = layer.expert_forward(1, x.to(cuda))
    ffn_gate(got, ref, f"fp8 expert dt={dt} n={n}")
    assert check_vs_rounded(got, ref) > 0.9
    assert torch.equal(layer.expert_forward(1, x).view(torch.int16), got.cpu().view(torch.int16))   # host rows
    layer.close()


@pytest.mark.parametrize("kind", ["fp8", "int8"])
def test_one_expert_tiled(ek, oracle, cuda, kind):
    """A per-expert call long enough to be cut into tiles runs the tile kernel's narrow form (a wave's
    single column block then holds up and gate channels, each with the scale row of its own matrix);
    the same rows through the layer call run the wide form and give the same bits."""
    H, I, n, dt = 384, 256, 1500, torch.bfloat16
    layer = ek.HipLayer(H, I, 2, 1, act_dtype=dt, max_tokens=n, **KINDS[kind])
    ew = make_expert(ek, H, I, 12, kind)
    layer.set_expert(1, ew)
    x = torch.randn(n, H, generator=torch.Generator().manual_seed(n)).to(dt)
    ref = oracle.ffn(x, *ref_weights(oracle, ew, dt), mode=2)
    got = layer.expert_forward(1, x.to(cuda))
    # (fp8: 2.19e-2 on 2 of the 576000 outputs, both y_ref rounded to bf16; int8: 1.27e-2)
    ffn_gate(got, ref, f"{kind} block expert tiled n={n}", plain=kind != "fp8")
    assert check_vs_rounded(got, ref) > 0.9
    routed = layer.forward(x.to(cuda), torch.ones(n, 1, dtype=torch.int32, device=cuda), torch.ones(n, 1, dtype=dt, device=cuda))
    assert torch.equal(routed.view(torch.int16), got.view(torch.int16))
    layer.close()


@pytest.mark.parametrize("kind", ["fp8", "int8"])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,K,H,I", [(24, 8, 2, 384, 256), (300, 6, 2, 512, 384), (700, 4, 1, 256, 640)])
def test_layer_both_kernel_families(ek, oracle, cuda, dt, T, E, K, H, I, kind):
    """Whole layer calls whose segments span the streaming kernel (<= 16 rows) and 32-, 64- and
    128-row tiles; routing skewed so that one expert is hot and one is never used."""
    print(f"fp8 layer dt={dt} T={T} E={E} K={K} H={H} I={I}", flush=True)
    g = torch.Generator().manual_seed(T + E)
    layer = ek.HipLayer(H, I, E, K, act_dtype=dt, max_tokens=T, **KINDS[kind])
    ws = [make_expert(ek, H, I, 100 + e, kind) for e in range(E)]
    for e in range(E - 1):                       # the last expert stays unloaded and unused
        layer.set_expert(e, ws[e])
    p = torch.tensor([8.0] + [1.0] * (E - 3) + [0.05, 0.0])
    ids = torch.stack([torch.multinomial(p, K, generator=g) for _ in range(T)]).to(torch.int32)
    gw = torch.rand(T, K, generator=g) + 0.1
    gw = (gw / gw.sum(-1, keepdim=True)).to(dt)
    x = torch.randn(T, H, generator=g).to(dt)
    wu, wg, wd = zip(*[ref_weights(oracle, w, dt) for w in ws])
    ref, counts, offsets, perm, inv, y3 = oracle.layer_forward(x, ids, gw, list(wu), list(wg), list(wd), mode=2,
                                                             return_y3=True)
    y, rt = layer.forward(x.to(cuda), ids.to(cuda), gw.to(cuda), return_route=True)
    assert torch.equal(rt.perm.cpu(), perm) and torch.equal(rt.counts.cpu(), counts)
    sizes = sorted(set(int(c) for c in counts))
    print("   segment lengths:", sizes, flush=True)
    layer_gate(y, ref, y3, gw, f"fp8 layer T={T}")
    layer.close()


@pytest.mark.parametrize("kind", ["fp8", "int8"])
def test_batch_of_small_calls_and_blob_ingestion(ek, oracle, cuda, kind):
    """Many <= 16-row calls in one launch (the one-wave-per-channel-group streaming form) and
    experts loaded from the bytes ek-db serves (fp8 tensors with weight_scale_inv beside them)."""
    dt, H, I, E = torch.bfloat16, 384, 256, 256
    layer = ek.HipLayer(H, I, E, 1, act_dtype=dt, max_tokens=4096, **KINDS[kind])
    ew = make_expert(ek, H, I, 5, kind)
    blob = st_save({"model.layers.3.mlp.experts.0.up_proj.weight": ew.up_w,
                    "model.layers.3.mlp.experts.0.up_proj.weight_scale_inv": ew.up_scale,
                    "model.layers.3.mlp.experts.0.gate_proj.weight": ew.gate_w,
                    "model.layers.3.mlp.experts.0.gate_proj.weight_scale_inv": ew.gate_scale,
                    "model.layers.3.mlp.experts.0.down_proj.weight": ew.down_w,
                    "model.layers.3.mlp.experts.0.down_proj.weight_scale_inv": ew.down_scale})
    layer.set_expert_safetensors(0, blob)
    x = torch.randn(16 * 200, H, generator=torch.Generator().manual_seed(9)).to(dt)
    outs = torch.cat(layer.experts_forward([0] * 200, list(x.to(cuda).split(16))))
    ref = oracle.ffn(x, *ref_weights(oracle, ew, dt), mode=2)
    # (int8: 2.45e-2 on one of 1.2 million outputs, at 7 sigma, y_ref rounded to bf16; fp8: 1.8e-2)
    ffn_gate(outs, ref, f"{kind} batch of 200 calls", plain=kind != "int8")
    one = layer.expert_forward(0, x[32:48].to(cuda))                    # the same rows alone: same bits
    assert torch.equal(one.view(torch.int16), outs[32:48].view(torch.int16))
    layer.close()


def test_block_scaled_layer_rejects_other_weights(ek):
    with pytest.raises(ek.EKError):
        ek.HipLayer(256, 128, 2, 1, block_scales=True, max_tokens=8)         # needs one-byte weights
    i8 = ek.HipLayer(256, 128, 2, 1, w_dtype=torch.int8, block_scales=True, max_tokens=8)
    with pytest.raises(ek.EKError):
        i8.set_expert(0, make_expert(ek, 256, 128, 3, "fp8"))
    i8.close()
    layer = ek.HipLayer(256, 128, 2, 1, w_dtype=F8, max_tokens=8)
    bf = ek.ExpertWeight.from_rand_linear(256, 128, torch.bfloat16)
    with pytest.raises(ek.EKError) as ei:
        layer.set_expert(0, bf)
    assert ei.value.status == ek.EK_INVALID_INPUT
    ew = make_expert(ek, 256, 128, 3)
    ew.up_scale = None
    with pytest.raises(ek.EKError):
        layer.set_expert(0, ew)
    layer.close()
    with pytest.raises(ek.EKError) as ei:
        ek.HipLayer(16384, 128, 2, 1, w_dtype=F8, max_tokens=8)
    assert ei.value.status == ek.EK_INVALID_INPUT


@pytest.mark.parametrize("kind", ["fp8", "int8", "int8 per channel"])
def test_every_weight_byte_is_converted_exactly(ek, cuda, kind):
    """Reads the kernels' weight conversion back bit for bit.  With one-hot activation rows,
    gate weights of 64 (silu(64) = 64 in fp32 and in 16 bits), an identity down projection and
    unit scales, out[k, j] = 64 * up[j, k] with no rounding anywhere, so every one of the 256
    byte values planted in `up` must come back as the value its format assigns to it -- through
    the streaming kernel (16-row calls, a 128-row call) and through the tile kernel (a layer
    call that routes every token to the expert)."""
    n = 128
    codes = torch.arange(n * n, dtype=torch.int32).remainder(256).reshape(n, n).roll(3, 1).to(torch.uint8)
    if kind == "fp8":
        codes = torch.where((codes & 0x7f) == 0x7f, torch.zeros_like(codes), codes)     # the two NaN encodings
        up = codes.view(F8)
        sign, e, m = (codes >> 7).float(), ((codes >> 3) & 15).float(), (codes & 7).float()
        want = torch.where(e == 0, m / 8 * 2.0 ** -6, (1 + m / 8) * torch.exp2(e - 7)) * (1 - 2 * sign)   # OCP e4m3fn
        mk = lambda v: torch.full((n, n), v).to(F8)
        eye = torch.eye(n).to(F8)
    else:
        up = codes.view(torch.int8)
        want = up.float()
        mk = lambda v: torch.full((n, n), int(v), dtype=torch.int8)
        eye = torch.eye(n).to(torch.int8)
    ones = torch.ones(n) if kind == "int8 per channel" else torch.ones(1, 1)
    ew = ek.ExpertWeight(up_w=up, gate_w=mk(64.0), down_w=eye, up_scale=ones, gate_scale=ones, down_scale=ones)
    layer = ek.HipLayer(n, n, 2, 1, max_tokens=n, **KINDS.get(kind, dict(w_dtype=torch.int8)))
    layer.set_expert(1, ew)
    x = torch.eye(n).to(torch.bfloat16).to(cuda)
    expect = (64 * want.t() + 0.0).to(torch.bfloat16).view(torch.int16)      # exact: at most 8 significant bits;
                                                                             # a sum that starts at +0 turns -0 into +0
    got = {"128-row call": layer.expert_forward(1, x),
           "16-row calls": torch.cat(layer.experts_forward([1] * 8, list(x.split(16)))),
           "layer call": layer.forward(x, torch.ones(n, 1, dtype=torch.int32, device=cuda),
                                       torch.ones(n, 1, dtype=torch.bfloat16, device=cuda))}
    for name, y in got.items():
        bad = (y.cpu().view(torch.int16) != expect).nonzero()
        assert bad.numel() == 0, (name, bad[:5].tolist())
    layer.close()
