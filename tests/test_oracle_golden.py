"""The oracle against the only stored known-answer vectors of the reference
(tests/artifacts/aiu_addons/*.pt there, copied as data into tests/golden/)."""
import glob
import os

import pytest
import torch

from oracle import qlinear_oracle as O

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "ref_w-*.pt")))


def test_all_six_fixtures_present():
    assert len(GOLDEN) == 6


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_i8i8_aiu_matches_reference_vectors(path):
    d = torch.load(path, weights_only=True)
    x = d["x"].to(torch.float16)
    qdata = d["qdata"].to(torch.float16)
    out = O.i8i8_aiu(x, d["w_int"], d["bias"], qdata, d["weight_quant_type"], d["activ_quant_type"],
                     d["smoothquant"])
    ref = d["reference_out"]
    assert out.shape == x.shape[:-1] + (d["w_int"].shape[0],)
    # tolerance of the reference's own test (tests/aiu_addons/test_int8_addon.py:75-77)
    assert torch.all((out - ref).abs() < 1e-4)


@pytest.mark.parametrize("path", [p for p in GOLDEN if "per_token" in p])
def test_per_token_vectors_also_pin_the_integer_path(path):
    """The per-token fixture's quantize step (round(x*127/amax), clamp +-127) gives the same
    integers as the deploy quantizer (round(x/(amax/127))) on these inputs, so the stored outputs
    also check  x_int . w_int^T  followed by dequantization with exact integer accumulation."""
    d = torch.load(path, weights_only=True)
    x = d["x"].to(torch.float16).reshape(-1, d["x"].shape[-1])
    w_int = d["w_int"]
    n = w_int.shape[0]
    per_ch = d["weight_quant_type"] == "per_channel"
    w_cv = d["qdata"][: n if per_ch else 1].float()
    q, s, _ = O.quant_act_pertoken_i8(x)
    amax = x.abs().max(dim=-1, keepdim=True)[0]
    q_ref = torch.round(x * (127 / amax)).clamp(-127, 127).to(torch.int8)
    assert torch.equal(q, q_ref)
    acc = O.int_gemm(q, w_int.to(torch.int8))
    y = acc.float() * (amax.float() / 127) * (w_cv / 127) + d["bias"].float()
    ref = d["reference_out"].reshape(-1, n).float()
    # the stored outputs went through fp16 operands and an fp16 F.linear (ulp 0.008 at |y| = 8)
    assert torch.all((y - ref).abs() < 5e-3 + 2e-3 * ref.abs())


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_smoothquant_branch_by_power_of_two_invariance(path):
    """The stored vectors all have SmoothQuant off.  With a power-of-two scale per input channel
    every division and multiplication by it is exact, so feeding x * sq together with sq must give
    the stored outputs again, bit for bit at the quantize step and to the same tolerance at the
    output: a dropped, transposed or doubly applied scale fails this."""
    d = torch.load(path, weights_only=True)
    x = d["x"].to(torch.float16)
    k = x.shape[-1]
    sq = torch.tensor([2.0 ** e for e in [-2, 1, 0, 3, -1, 2, -3, 1, 0, 2][:k]], dtype=torch.float16)
    qdata = torch.cat((d["qdata"].to(torch.float16)[:-1], sq))
    out = O.i8i8_aiu(x * sq, d["w_int"], d["bias"], qdata, d["weight_quant_type"],
                     d["activ_quant_type"], True)
    assert torch.all((out - d["reference_out"]).abs() < 1e-4)
    n = d["w_int"].shape[0]
    i1 = n if d["weight_quant_type"] == "per_channel" else 1
    a_cv, a_cvn = qdata[2 * i1: 2 * i1 + 1], qdata[2 * i1 + 1: 2 * i1 + 2]
    q_plain, _, _ = O.i8i8_aiu_quant_act(x, a_cv, a_cvn, torch.ones(1, dtype=torch.float16),
                                         d["activ_quant_type"])
    q_sq, _, _ = O.i8i8_aiu_quant_act(x * sq, a_cv, a_cvn, sq, d["activ_quant_type"])
    assert torch.equal(q_plain, q_sq)
