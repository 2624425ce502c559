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


# ------------------------------------------------------------------ norm + RoPE step and the key restrictions
GOLD_PREP = Path(__file__).resolve().parent / "golden" / "sage_prep_small.safetensors"
_EMUL_CASES = {"o_emul": {}, "o_emul_k_lens": {"k_lens": True}, "o_emul_mask": {"block_mask": True},
               "o_emul_causal": {"causal": True}, "o_emul_all": {"causal": True, "block_mask": True, "k_lens": True}}


@pytest.fixture(scope="module")
def gold_prep():
    return load_file(str(GOLD_PREP))


def _emul_kwargs(gold, spec):
    kw = {}
    if spec.get("k_lens"):
        kw["k_lens"] = gold["k_lens"].tolist()
    if spec.get("block_mask"):
        kw["block_mask"] = gold["block_mask"]
    if spec.get("causal"):
        kw["causal"] = True
    return kw


def test_oracle_reproduces_prep_golden_vectors(gold_prep):
    from oracle import prep_ref as pr
    from oracle.sage_emul_ref import sage_emul_from_quant

    g = gold_prep
    table, grid = pr.wan_rope_table(128), g["grid_sizes"].tolist()
    assert torch.equal(pr.inv_rms_ref(g["q_proj"], 1e-6), g["q_inv_rms"])
    assert torch.equal(pr.inv_rms_ref(g["k_proj"], 1e-6), g["k_inv_rms"])
    q = pr.wan_prep_ref(g["q_proj"], g["q_norm_weight"], 1e-6, grid, table, 1)
    k = pr.wan_prep_ref(g["k_proj"], g["k_norm_weight"], 1e-6, grid, table, 1)
    assert torch.equal(q, g["q_prepped"]) and torch.equal(k, g["k_prepped"])
    q_i8, q_scale = qr.quant_q_ref(q, 128**-0.5)
    k_i8, k_scale, k_mean = qr.quant_k_ref(k)
    assert torch.equal(q_i8, g["q_i8"]) and torch.equal(q_scale, g["q_scale"])
    assert torch.equal(k_i8, g["k_i8"]) and torch.equal(k_scale, g["k_scale"]) and torch.equal(k_mean, g["k_mean"])
    v_fp8 = g["v_fp8_codes"].view(torch.float8_e4m3fn)
    for name, spec in _EMUL_CASES.items():
        out = sage_emul_from_quant(g["q_i8"], g["q_scale"], g["k_i8"], g["k_scale"], v_fp8, g["v_scale"], torch.bfloat16,
                                   **_emul_kwargs(g, spec))
        torch.testing.assert_close(out.float(), g[name].float(), rtol=0, atol=4e-3)
    # the restrictions do restrict: batch 1 sees 77 keys, rows 0..127 of batch 0 lose tile 1, causal row 0 is V[0]
    assert not torch.equal(g["o_emul"][1], g["o_emul_k_lens"][1]) and torch.equal(g["o_emul"][0], g["o_emul_k_lens"][0])
    assert not torch.equal(g["o_emul"], g["o_emul_mask"]) and not torch.equal(g["o_emul"], g["o_emul_causal"])
    assert (g["o_emul_all"][1, 128:] == 0).all()  # mask row 1 of batch 1 keeps tile 2 only, k_lens = 77 empties it


@pytest.mark.gpu
def test_hip_path_reproduces_prep_golden_vectors(gold_prep, hip_device):
    from ksanadit_amd import sage_ops
    from ksanadit_amd.layout import untile_k
    from oracle import prep_ref as pr

    g = gold_prep
    dev = hip_device
    B, L, H, D = 2, 130, 1, 128
    prep = sage_ops.WanPrep(g["q_norm_weight"].to(dev), g["k_norm_weight"].to(dev), 1e-6, pr.wan_rope_table(D).to(dev),
                            g["grid_sizes"].tolist())
    qp, kp, v = (g[n].to(dev) for n in ("q_proj", "k_proj", "v"))
    q4, k4 = qp.view(B, L, H, D), kp.view(B, L, H, D)
    ws = sage_ops.workspace_for(q4, k4)
    sage_ops.quant_q(q4, ws, D**-0.5, prep=prep)
    sage_ops.quant_k(k4, ws, True, prep=prep)
    sage_ops.quant_v(v, ws)
    torch.cuda.synchronize()
    assert torch.equal(ws.q_rms.cpu()[:, :L], g["q_inv_rms"]) and torch.equal(ws.k_rms.cpu()[:, :L], g["k_inv_rms"])
    assert torch.equal(ws.q_i8.cpu()[:, :, :L], g["q_i8"]) and torch.equal(ws.q_scale.cpu()[:, :, :L], g["q_scale"])
    assert torch.equal(untile_k(ws.k_tiles.cpu(), L), g["k_i8"]) and torch.equal(ws.k_scale.cpu(), g["k_scale"])
    assert torch.equal(ws.k_mean.cpu(), g["k_mean"].float())
    for name, spec in _EMUL_CASES.items():
        kw = _emul_kwargs(g, spec)
        out = sage_ops.attn_fwd(ws, torch.empty((B, L, H, D), dtype=torch.bfloat16, device=dev), **kw).cpu()
        ref = g[name].float()
        diff = (out.float() - ref).abs()
        assert diff.max() <= 2e-2 * ref.abs().max(), name
        assert (diff > 5e-3 * ref.abs().max()).float().mean() < 2e-3, name
        assert ((ref.abs().sum(-1) == 0) == (out.float().abs().sum(-1) == 0)).all(), name
