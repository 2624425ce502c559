"""Oracle: where the distance between the quantized scheme and SDPA comes from.  Test infrastructure only.

The attention output of the path is compared with the reference's torch SDPA backend
(ksana/operations/attention/backends/sdpa.py:47-79) within a tolerance; this module splits that distance, on the CPU
and on the same seeded inputs, into the contributions of the three quantizations, switched on one after the other:

    A   INT8 Q and K (Hadamard-transformed, per-row / per-64-key scales), exact softmax, exact V
    B   A + the probabilities rounded to e4m3 (relative to the row maximum, scaled by 2^P_SHIFT)
    C   B + V rounded to per-channel e4m3, result rounded to bf16        = the scheme the kernel implements

each against float64 attention on the bf16 inputs.  ``python -m oracle.error_budget <workload> [heads]`` prints the
table behind the tolerances stated in tests/test_attn_gpu.py; tests/test_error_budget.py checks the structure of the
budget on a reduced size.  ``k_block`` re-quantizes K with a scale per ``k_block`` keys (64 is the path's).
"""

from __future__ import annotations

import sys

import torch

from .quant_ref import BLKK, FP8_MAX, _to_bhld_f32, fwht_ref, quant_k_ref, quant_q_ref, quant_v_ref
from .sage_emul_ref import P_SHIFT

STAGES = ("A", "B", "C")


def _quant_k_blocks(k: torch.Tensor, k_block: int):
    """int8 K and per-key scales with one scale per ``k_block`` keys (same arithmetic as ``quant_k_ref``)."""
    k_i8, k_scale, km = quant_k_ref(k, smooth_k=True)
    L = k.shape[1]
    if k_block == BLKK:
        return k_i8.float(), k_scale.repeat_interleave(BLKK, dim=2)[:, :, :L]
    x = fwht_ref(_to_bhld_f32(k) - km.float()[:, :, None, :])
    B, H, _, D = x.shape
    nb = -(-L // k_block)
    xp = torch.nn.functional.pad(x, (0, 0, 0, nb * k_block - L)).view(B, H, nb, k_block, D)
    amax = xp.abs().amax(dim=(3, 4))
    inv = torch.where(amax > 0, 127.0 / amax, torch.zeros_like(amax))
    codes = torch.round(xp * inv[..., None, None]).clamp(-127, 127).view(B, H, nb * k_block, D)[:, :, :L]
    return codes, (amax / 127.0).repeat_interleave(k_block, dim=2)[:, :, :L]


def error_budget(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, k_block: int = BLKK, rows: int | None = None,
                 chunk: int = 2048) -> dict:
    """``[B, L, H, D]`` half tensors -> per stage: max, 99.9th percentile and mean of ``|O_stage - O_exact|``, the
    worst per-row error relative to that row's largest output, and ``max|O_exact|`` (``ref_max``).  ``rows`` limits
    the query rows looked at (all keys are always used)."""
    B, Lq, H, D = q.shape
    Lk = k.shape[1]
    sm = D**-0.5
    q_i8, q_scale = quant_q_ref(q, sm)
    k_codes, k_scale_key = _quant_k_blocks(k, k_block)
    v_fp8, v_scale = quant_v_ref(v)
    n = Lq if rows is None else min(Lq, rows)
    errs = {s: [] for s in STAGES}
    row_rel = {s: [] for s in STAGES}
    ref_max = 0.0
    for b in range(B):
        for h in range(H):
            qf, kf, vf = q[b, :, h].double(), k[b, :, h].double(), v[b, :, h].double()
            qd = q_i8[b, h].float() * q_scale[b, h][:, None]  # carries sm_scale * log2(e) / 128
            kd = k_codes[b, h] * k_scale_key[b, h][:, None]
            vq = (v_fp8[b, h].float() * v_scale[b, h][None, :]).double()
            for r0 in range(0, n, chunk):
                r1 = min(n, r0 + chunk)
                o_ref = torch.softmax((qf[r0:r1] @ kf.t()) * sm, dim=-1) @ vf
                s_q = qd[r0:r1] @ kd.t()  # log2 domain
                m = s_q.amax(dim=1, keepdim=True)
                p_a = torch.exp2(s_q - m).double()
                p_b = torch.exp2(s_q - m + P_SHIFT).clamp(max=FP8_MAX).to(torch.float8_e4m3fn).double()
                outs = {
                    "A": (p_a @ vf) / p_a.sum(dim=1, keepdim=True),
                    "B": (p_b @ vf) / p_b.sum(dim=1, keepdim=True),
                    "C": ((p_b @ vq) / p_b.sum(dim=1, keepdim=True)).float().to(torch.bfloat16).double(),
                }
                mag = o_ref.abs().amax(dim=1)
                ref_max = max(ref_max, float(mag.max()))
                for s in STAGES:
                    e = (outs[s] - o_ref).abs()
                    errs[s].append(e.flatten().float())
                    row_rel[s].append((e.amax(dim=1) / mag).float())
    res = {"ref_max": ref_max}
    for s in STAGES:
        e, r = torch.cat(errs[s]), torch.cat(row_rel[s])
        kth = max(1, int(0.999 * e.numel()))
        res[s] = {"max_abs": float(e.max()), "p999_abs": float(e.kthvalue(kth).values), "mean_abs": float(e.mean()),
                  "row_rel_max": float(r.max())}
    return res


def main(argv):
    import os

    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    from ksanadit_amd.workloads import make_inputs

    name = argv[1] if len(argv) > 1 else "wan14b_480p"
    heads = int(argv[2]) if len(argv) > 2 else 1
    k_block = int(argv[3]) if len(argv) > 3 else BLKK
    q, k, v = make_inputs(name, heads=heads)
    res = error_budget(q, k, v, k_block=k_block)
    print(f"{name}, {heads} head(s), K scale per {k_block} keys: max|O| = {res['ref_max']:.3f}")
    for s in STAGES:
        r = res[s]
        print(f"  {s}: max_abs {r['max_abs']:.4f} = {r['max_abs'] / res['ref_max']:.3f} max|O|   p99.9 {r['p999_abs']:.4f} = "
              f"{r['p999_abs'] / res['ref_max']:.4f} max|O|   mean {r['mean_abs']:.5f}   worst row rel {r['row_rel_max']:.3f}")


if __name__ == "__main__":
    main(sys.argv)
