#!/usr/bin/env python3
"""Writes tests/golden/sage_prep_small.safetensors: seeded raw projections, what the CPU oracle makes of them
through RMSNorm + 3-axis RoPE + the quantizer, and the emulated attention output under the three key restrictions
(per-batch key counts, a block mask, causal).

The reference holds no fixture for these steps, so the vectors are this repository's own (inputs drawn here, outputs
computed by ``oracle/``; nothing is imported from the reference).  They freeze the oracle's specification: a change of
a summation order or a rounding step shows up as a mismatch with the committed file.
Run from the repository root:  python tests/golden/make_golden_prep.py
"""

import sys
from pathlib import Path

import torch
from safetensors.torch import save_file

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from oracle import prep_ref as pr  # noqa: E402
from oracle import quant_ref as qr  # noqa: E402
from oracle.sage_emul_ref import sage_emul_from_quant  # noqa: E402

OUT = Path(__file__).resolve().parent / "sage_prep_small.safetensors"
GRID = [(2, 5, 13), (1, 9, 11)]  # (frames, rows, columns) per batch entry: 130 and 99 of the 130 positions
EPS = 1e-6


def build():
    g = torch.Generator().manual_seed(20250202)
    B, L, H, D = 2, 130, 1, 128
    qp = (1.5 * torch.randn((B, L, H * D), generator=g)).to(torch.bfloat16)
    kp = (torch.randn((B, L, H * D), generator=g) + 1.0).to(torch.bfloat16)
    v = torch.randn((B, L, H, D), generator=g).to(torch.bfloat16)
    wq = (1.0 + 0.2 * torch.randn(H * D, generator=g)).float()
    wk = (1.0 + 0.2 * torch.randn(H * D, generator=g)).float()
    table = pr.wan_rope_table(D)
    q = pr.wan_prep_ref(qp, wq, EPS, GRID, table, H)
    k = pr.wan_prep_ref(kp, wk, EPS, GRID, table, H)
    sm = D**-0.5
    q_i8, q_scale = qr.quant_q_ref(q, sm)
    k_i8, k_scale, k_mean = qr.quant_k_ref(k)
    v_fp8, v_scale = qr.quant_v_ref(v)
    k_lens = torch.tensor([130, 77], dtype=torch.int32)
    mask = torch.tensor([[[1, 0, 1], [0, 1, 1]], [[1, 1, 0], [0, 0, 1]]], dtype=torch.int8)[:, None]  # [B, 1, 2, 3]
    emul = lambda **kw: sage_emul_from_quant(q_i8, q_scale, k_i8, k_scale, v_fp8, v_scale, torch.bfloat16, **kw).contiguous()  # noqa: E731
    return {
        "q_proj": qp, "k_proj": kp, "v": v, "q_norm_weight": wq, "k_norm_weight": wk,
        "grid_sizes": torch.tensor(GRID, dtype=torch.int32), "k_lens": k_lens, "block_mask": mask,
        "q_inv_rms": pr.inv_rms_ref(qp, EPS), "k_inv_rms": pr.inv_rms_ref(kp, EPS),
        "q_prepped": q.contiguous(), "k_prepped": k.contiguous(),
        "q_i8": q_i8, "q_scale": q_scale, "k_i8": k_i8, "k_scale": k_scale, "k_mean": k_mean,
        "v_fp8_codes": v_fp8.view(torch.uint8), "v_scale": v_scale,
        "o_emul": emul(), "o_emul_k_lens": emul(k_lens=k_lens.tolist()), "o_emul_mask": emul(block_mask=mask),
        "o_emul_causal": emul(causal=True), "o_emul_all": emul(causal=True, block_mask=mask, k_lens=k_lens.tolist()),
    }


def main():
    tensors = build()
    save_file({n: t.contiguous() for n, t in tensors.items()}, str(OUT), metadata={"eps": repr(EPS), "seed": "20250202"})
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes)")


if __name__ == "__main__":
    main()
