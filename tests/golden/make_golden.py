#!/usr/bin/env python3
"""Writes tests/golden/sage_small.safetensors: seeded inputs and what the CPU oracle makes of them.

The reference holds no fixture for this path (its only checks are two tolerances on unseeded
randn, tests/ksana/attention_op_test.py:157-186), so these vectors are this repository's own:
inputs drawn here, outputs computed by ``oracle/`` - nothing is imported from the reference.
Run from the repository root:  python tests/golden/make_golden.py
"""

import sys
from pathlib import Path

import torch
from safetensors.torch import save_file

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from oracle import quant_ref as qr  # noqa: E402
from oracle.sage_emul_ref import sage_emul_ref  # noqa: E402
from oracle.sdpa_ref import sdpa_ref  # noqa: E402

OUT = Path(__file__).resolve().parent / "sage_small.safetensors"


def main():
    g = torch.Generator().manual_seed(20250101)
    B, Lq, Lk, Hq, Hkv, D = 1, 96, 130, 2, 1, 128  # ragged K tail, GQA, rectangular
    q = torch.randn((B, Lq, Hq, D), generator=g)
    k = torch.randn((B, Lk, Hkv, D), generator=g) + 2.0 * torch.randn((1, 1, Hkv, D), generator=g)
    v = torch.randn((B, Lk, Hkv, D), generator=g)
    q[0, 5, 0, 17] *= 20.0  # one outlier each
    k[0, 70, 0, 3] *= 20.0
    q, k, v = q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16)
    sm = D**-0.5
    q_i8, q_scale = qr.quant_q_ref(q, sm)
    k_i8, k_scale, k_mean = qr.quant_k_ref(k)
    v_fp8, v_scale = qr.quant_v_ref(v)
    tensors = {
        "q": q, "k": k, "v": v,
        "q_i8": q_i8, "q_scale": q_scale, "k_i8": k_i8, "k_scale": k_scale, "k_mean": k_mean,
        "v_fp8_codes": v_fp8.view(torch.uint8), "v_scale": v_scale,
        "o_sdpa": sdpa_ref(q, k, v).contiguous(),
        "o_emul_exact": sage_emul_ref(q, k, v, exact_exp2=True).contiguous(),
        "o_emul_pwl": sage_emul_ref(q, k, v, exact_exp2=False).contiguous(),
    }
    save_file({n: t.contiguous() for n, t in tensors.items()}, str(OUT), metadata={"sm_scale": repr(sm), "seed": "20250101"})
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes)")


if __name__ == "__main__":
    main()
