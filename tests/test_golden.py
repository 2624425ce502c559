"""Committed golden vectors (tests/golden/sage_small.safetensors, made by make_golden.py):
on the CPU they pin the oracle against drift; on the GPU the HIP path must reproduce the
quantized tensors bit for bit and the attention output within tolerance."""

from pathlib import Path

import pytest
import torch
from safetensors.torch import load_file

from oracle import quant_ref as qr
from oracle.sage_emul_ref import sage_emul_ref
from oracle.sdpa_ref import sdpa_ref

GOLD = Path(__file__).resolve().parent / "golden" / "sage_small.safetensors"


@pytest.fixture(scope="module")
def gold():
    return load_file(str(GOLD))


def test_oracle_reproduces_golden_vectors(gold):
    q, k, v = gold["q"], gold["k"], gold["v"]
    q_i8, q_scale = qr.quant_q_ref(q, 128**-0.5)
    k_i8, k_scale, k_mean = qr.quant_k_ref(k)
    v_fp8, v_scale = qr.quant_v_ref(v)
    assert torch.equal(q_i8, gold["q_i8"]) and torch.equal(q_scale, gold["q_scale"])
    assert torch.equal(k_i8, gold["k_i8"]) and torch.equal(k_scale, gold["k_scale"]) and torch.equal(k_mean, gold["k_mean"])
    assert torch.equal(v_fp8.view(torch.uint8), gold["v_fp8_codes"]) and torch.equal(v_scale, gold["v_scale"])
    # float results: same machine-independent algorithm, allow the last bf16 bit for BLAS differences
    torch.testing.assert_close(sdpa_ref(q, k, v).float(), gold["o_sdpa"].float(), rtol=0, atol=4e-3)
    torch.testing.assert_close(sage_emul_ref(q, k, v).float(), gold["o_emul_exact"].float(), rtol=0, atol=4e-3)
    torch.testing.assert_close(sage_emul_ref(q, k, v, exact_exp2=False).float(), gold["o_emul_pwl"].float(), rtol=0, atol=4e-3)


def test_golden_vectors_are_self_consistent(gold):
    # outliers planted by the generator are visible, shapes are the documented ones
    assert gold["q"].shape == (1, 96, 2, 128) and gold["k"].shape == (1, 130, 1, 128)
    assert gold["q_scale"].shape == (1, 2, 96) and gold["k_scale"].shape == (1, 1, 3)
    assert gold["q_i8"].abs().amax(-1).eq(127).all()
    a, b = gold["o_emul_exact"].double().flatten(), gold["o_sdpa"].double().flatten()
    assert float(a @ b / (a.norm() * b.norm())) > 0.998  # 96 rows only: a loose sanity bound


@pytest.mark.gpu
def test_hip_path_reproduces_golden_vectors(gold, hip_device):
    from ksanadit_amd import sage_ops
    from ksanadit_amd.layout import untile_k, untile_v

    q, k, v = (gold[n].to(hip_device) for n in ("q", "k", "v"))
    ws = sage_ops.workspace_for(q, k)
    for pwl, ref_name in ((False, "o_emul_exact"), (True, "o_emul_pwl")):
        out = sage_ops.sageattn(q, k, v, workspace=ws, pwl_exp2=pwl).cpu()
        ref = gold[ref_name].float()
        diff = (out.float() - ref).abs()
        assert diff.max() <= 2e-2 * ref.abs().max() and (diff > 5e-3 * ref.abs().max()).float().mean() < 2e-3
    Lq, Lk = q.shape[1], k.shape[1]
    assert torch.equal(ws.q_i8.cpu()[:, :, :Lq], gold["q_i8"])
    assert torch.equal(ws.q_scale.cpu()[:, :, :Lq], gold["q_scale"])
    assert torch.equal(untile_k(ws.k_tiles.cpu(), Lk), gold["k_i8"])
    assert torch.equal(ws.k_scale.cpu(), gold["k_scale"])
    assert torch.equal(ws.k_mean.cpu(), gold["k_mean"].float())
    assert torch.equal(untile_v(ws.v_tiles.cpu(), Lk), gold["v_fp8_codes"])
    assert torch.equal(ws.v_scale.cpu(), gold["v_scale"])
