"""Parity of a full-size layer call on sampled tokens -- TEST INFRASTRUCTURE ONLY.

The benchmark configurations at full size (256 DeepSeek-V3 experts, 8192 tokens) are beyond what
the scalar oracle recomputes whole in seconds.  Tokens are independent in the reference
(ek-computation/src/controller/executor.rs:283-299 groups pairs, ffn/expert_torch.rs:81-84 works
row by row, qwen3_moe.py:102-104 sums per token), so the oracle recomputes a handful of tokens that
between them sit in the longest segment, in a segment short enough for the weight-streaming
kernel, in segments whose remainder is cut into a 128-, 64- and 32-row tile, plus tokens drawn at
random, and the call's output rows for those tokens are held to it.  Used by the GPU tests,
__graft_entry__.smoke() and the benchmark's pre-timing parity gate; never by the library.
"""
from __future__ import annotations

import torch

from . import oracle


def choose_tokens(ids: torch.Tensor, n_experts: int, n_random: int = 4, seed: int = 5):
    T = ids.shape[0]
    counts = torch.bincount(ids.flatten().long(), minlength=n_experts)
    rem = counts % 128
    classes = [counts == counts.max(), (counts > 0) & (counts <= 16), (counts > 128) & (rem > 64),
               (counts > 128) & (rem > 32) & (rem <= 64), (counts > 128) & (rem > 16) & (rem <= 32)]
    tokens = torch.randint(0, T, (n_random,), generator=torch.Generator().manual_seed(seed)).tolist()
    for c in classes:                     # the last token routed there: it sits in the segment's remainder
        if bool(c.any()):
            e = int(torch.where(c)[0][0])
            tokens.append(int(torch.where((ids == e).any(dim=1))[0][-1]))
    return sorted(set(tokens))


def reference_weights(ew, dt):
    """(up, gate, down) as the reference's backend holds them after load_module's cast
    (ffn/expert_torch.rs:61-78): 16-bit tensors; int8 / fp8 sources dequantised with the oracle."""
    if ew.up_w.dtype == torch.int8 and ew.up_scale.dim() == 1:
        return tuple(oracle.dequant_channel(q.cpu(), s.cpu(), dt) for q, s in
                     ((ew.up_w, ew.up_scale), (ew.gate_w, ew.gate_scale), (ew.down_w, ew.down_scale)))
    if ew.up_scale is not None:           # 128 x 128 block scales (fp8 or int8 bytes)
        def blk(q, s):
            qf = oracle.fp8_e4m3fn_to_f32(q.cpu()) if q.dtype == torch.float8_e4m3fn else q.cpu().float()
            return oracle.dequant_block(qf, s.cpu().float())
        return blk(ew.up_w, ew.up_scale), blk(ew.gate_w, ew.gate_scale), blk(ew.down_w, ew.down_scale)
    return ew.up_w.cpu(), ew.gate_w.cpu(), ew.down_w.cpu()


def check(y_rows: torch.Tensor, x_rows: torch.Tensor, ids_rows: torch.Tensor, gw_rows: torch.Tensor, n_experts: int,
          weights_of, tol: float = 2e-2) -> dict:
    """y_rows: the call's output for the sampled tokens; x_rows / ids_rows / gw_rows: their inputs
    (CPU tensors); weights_of(e) -> the ExpertWeight loaded as expert e.  Returns the plain figures
    against the oracle's reference-rounded form (mode 2) and its fp32-accumulate ideal form (mode 1),
    what the reference's own ops evaluated by libtorch score against the same y_ref on the same
    tokens, and the tensors the tests' gates need."""
    dt = x_rows.dtype
    need = sorted(set(ids_rows.flatten().tolist()))
    wu, wg, wd = [None] * n_experts, [None] * n_experts, [None] * n_experts
    for e in need:
        wu[e], wg[e], wd[e] = reference_weights(weights_of(e), dt)
    ref, _, _, _, _, y3 = oracle.layer_forward(x_rows, ids_rows, gw_rows, wu, wg, wd, mode=2, return_y3=True)
    ideal = oracle.layer_forward(x_rows, ids_rows, gw_rows, wu, wg, wd, mode=1)[0]
    # the reference's own op sequence on libtorch (the library the reference calls), same tokens
    twin, _ = oracle.torch_layer_forward(x_rows, ids_rows, gw_rows, wu, wg, wd)
    y = y_rows.float().cpu()
    rms = float(ref.pow(2).mean().sqrt())
    err = (y - ref).abs()
    err_i = (y - ideal).abs()
    return {"max_err_over_rms": float(err.max()) / rms, "over_frac": float((err > tol * rms).float().mean()),
            "max_err_over_rms_vs_fp32_ideal": float(err_i.max()) / float(ideal.pow(2).mean().sqrt()),
            "over_frac_vs_fp32_ideal": float((err_i > tol * rms).float().mean()),
            "y_ref_rounded_to_output_type": float((ref.to(dt).float() - ref).abs().max()) / rms,
            "reference_ops_on_libtorch_max_err_over_rms": float((twin.float() - ref).abs().max()) / rms,
            "elements": int(err.numel()), "experts_recomputed": len(need), "ref": ref, "y3": y3}
