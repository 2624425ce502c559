"""Oracle: dequantised emulation of the fused Sage attention kernel.  Test infrastructure only.

Stage (a6.4) of the path: what the third-party kernel called at
ksana/operations/attention/backends/sage_attn.py:75-81 computes, with the operand roles of
the kernel signature visible at sage_sla.py:237-253 (q_int8, k_int8, v_fp8, q_scale, k_scale,
v_scale):

    S  = (Q_i8 . K_i8^T) * q_scale * k_scale        integer dot products, exact
    P  = exp2(S - rowmax(S) + P_SHIFT)              Q already carries sm_scale * log2(e); exp2 either
                                                    exact or with a piecewise-linear mantissa (p_to_e4m3)
    O  = (fp8(P) . V_fp8) * v_scale / rowsum(fp8(P))

It mirrors the kernel's tile-by-tile online softmax in fp32 (or, with ``online=False``, a
full softmax), so it separates "error of the quantised
scheme" from "bug in the kernel": the HIP kernel must agree with this far more tightly than
either agrees with SDPA.  It is an approximation of SDPA by construction and is pinned by
its distance to ``sdpa_ref`` plus exact invariants (see tests/test_oracle.py).
"""

from __future__ import annotations

import torch

from .quant_ref import BLKK, BLKQ, FP8_MAX, e4m3fn_decode_table, quant_k_ref, quant_q_ref, quant_v_ref

# P is scaled by 2**P_SHIFT before the fp8 cast so that small probabilities stay above the
# e4m3 subnormal floor (2**-9); the factor cancels in O = (P V) / rowsum(P).  The online form moves a row's reference
# point (its "running maximum") only when a tile's maximum exceeds it by more than LAZY_MAX octaves, as the kernel
# does: probabilities then reach 2**(P_SHIFT + LAZY_MAX) = 416 < 448.
P_SHIFT = 6.0
LAZY_MAX = 2.7
# The piecewise-linear path keeps 2**8 and follows every new maximum: its code formula fades the subnormal codes
# linearly, which is harmless only far below the true maximum.
P_SHIFT_PWL = 8.0
LAZY_MAX_PWL = 0.0


def p_to_e4m3(x: torch.Tensor, exact_exp2: bool = True) -> torch.Tensor:
    """x = log2 of the (shifted) probability -> the e4m3 value the kernel feeds to the PV MFMA.

    exact (default): round(exp2(x)) to e4m3 (nearest even).
    otherwise: the e4m3 CODE is rne(8*x + 55.5) clamped to [0, 126]; decoding it gives
    2^floor(.) * (1 + m/8): exp2 with a piecewise-linear 3-bit mantissa (codes below 8 are the
    subnormals, so probabilities under 2^-14 of the row maximum fade to zero linearly)."""
    if exact_exp2:
        return torch.exp2(x).clamp(max=FP8_MAX).to(torch.float8_e4m3fn).float()
    code = torch.round(8.0 * x + 55.5).clamp_(0, 126).long()
    return e4m3fn_decode_table().float()[code]


def sage_emul_from_quant(q_i8, q_scale, k_i8, k_scale, v_fp8, v_scale, out_dtype, causal=False, online=True,
                         exact_exp2=True, k_lens=None, block_mask=None, v_mean=None, key_split=None, magic=12582912.0):
    """Logical-layout operands ([B,H,L,D] etc.) -> O [B, Lq, H, D] in ``out_dtype``.

    ``online=True`` walks the keys in tiles of ``BLKK`` like the kernel: the running row max
    decides where each P lands on the e4m3 grid, so the fp8 rounding of P matches the kernel's
    (a full softmax rounds P relative to the FINAL max - same accuracy, different bits).
    ``k_lens``: batch ``b`` uses keys ``[0, k_lens[b])`` of the quantized operands (online form only).
    ``block_mask`` (``[B|1, H|1, ceil(Lq/128), ceil(Lk/64)]``): query rows ``128 i ..`` walk only the key tiles ``j``
    with a non-zero entry ``(i, j)``; rows without any tile give zeros (online form only).
    ``v_mean`` (``[B, Hkv, D]``, optional): the channel mean the V quantizer took off (``quant_v_ref(..., smooth_v=True)``);
    it is added back to every output row that saw at least one key.
    ``key_split`` (``(first_workgroup, runs)``, optional, dense online form only): the kernel cuts the key loop of
    the 256-row query blocks numbered ``first_workgroup`` and up (numbering: ``(b * H + h) * ceil(Lq/256) + block``)
    into ``runs`` equal runs of key tiles, walks each run on its own and merges the partial results; probabilities are
    then rounded relative to the run's own running maximum, which this mirrors.
    ``magic``: the constant the kernel's integer accumulators start from, read as fp32: 1.5 * 2**23 - or 1.5 * 2**24 where
    the kernel multiplies only the lower 64 channels of rows that were zero-extended from head size 64 (after the
    Hadamard transform the upper 64 repeat the lower 64, and at 2**24 the fp32 grid doubles the half product for free).
    The value changes the rounding of the exponent's constant term, nothing else.
    ``causal``: row ``i`` sees keys ``[0, i]`` (for ``Lq != Lk`` too: the triangle sits in the top left corner, as
    torch's ``is_causal`` puts it); in the online form a row sits out the tiles that start after it and sees a prefix
    of the tile that holds its own position.
    """
    B, H, Lq, D = q_i8.shape
    Hkv, Lk = k_i8.shape[1], k_i8.shape[2]
    g = H // Hkv
    out = torch.empty(B, Lq, H, D, dtype=out_dtype)
    qs_row = q_scale.repeat_interleave(BLKQ, dim=2)[:, :, :Lq]  # [B, H, Lq] (BLKQ == 1: already per row)
    ks_col = k_scale.repeat_interleave(BLKK, dim=2)[:, :, :Lk]  # [B, Hkv, Lk]
    if (k_lens is not None or block_mask is not None) and not online:
        raise NotImplementedError("k_lens / block_mask with the full-softmax form")
    if block_mask is not None:
        bm = torch.as_tensor(block_mask) != 0
        while bm.dim() < 4:
            bm = bm.unsqueeze(0)
        bm = bm.expand(B, H, -1, -1)
    for b in range(B):
        lk_b = Lk if k_lens is None else max(0, min(int(k_lens[b]), Lk))
        if lk_b == 0:
            out[b] = 0
            continue
        for h in range(H):
            hk = h // g
            # int8 x int8 sums stay below 2**24, so fp32 matmul is exact here
            s_int = q_i8[b, h].float() @ k_i8[b, hk].float().t()
            s = s_int * (qs_row[b, h][:, None] * ks_col[b, hk][None, :])
            if causal:
                # key <= row, the triangle anchored at the top left corner whatever Lq and Lk (torch's is_causal)
                mask = torch.ones(Lq, Lk, dtype=torch.bool).tril()
                s = s.masked_fill(~mask, float("-inf"))
            vf = v_fp8[b, hk].float()
            if online:
                # Mirrors the kernel's arithmetic operation by operation (fp32, FMAs emulated in
                # float64) so that e4m3 codes agree except at exact rounding ties:
                #   x_f = float(MAGIC + dot)            the int32 accumulator read as fp32
                #   sc  = q_scale * k_scale             one fp32 product per (row, tile)
                #   m   = max(m, fma(x_f_max, sc, -MAGIC * sc))
                #   c   = (SHIFT - m) + (-MAGIC * sc)   fp32, in this order
                #   exponent = fma(x_f, sc, c)          (pwl: fma(x_f, 8 sc, fma(8, c, 55.5)))
                x_f = (s_int + magic).to(torch.float32)  # exact: |dot| < 2**22 (and even where magic is 1.5 * 2**24)
                rows = torch.arange(Lq)[:, None]

                def walk(key_from, key_to):
                    """Online softmax over the tiles of keys [key_from, key_to): (acc, m, l)."""
                    m = torch.full((Lq, 1), float("-inf"))
                    l = torch.zeros(Lq, 1)
                    acc = torch.zeros(Lq, D)
                    for j0 in range(key_from, key_to, BLKK):
                        m, l, acc = step(j0, min(j0 + BLKK, key_to), m, l, acc)
                    return acc, m, l

                def step(j0, j1, m, l, acc):
                    act = None  # rows that take part in this step
                    if block_mask is not None:
                        # rows of a 128-row block that does not ask for this tile sit the step out
                        act = bm[b, h, :, j0 // BLKK].repeat_interleave(128)[:Lq][:, None]
                    allow = None  # keys of this tile each row may see
                    if causal:
                        # key <= row; a row before the tile's first key sits the step out, the rows
                        # on the diagonal see a prefix of the tile
                        allow = torch.arange(j0, j1)[None, :] <= rows
                        act = allow[:, :1] if act is None else (act & allow[:, :1])
                    if act is not None and not bool(act.any()):
                        return m, l, acc
                    sc = (qs_row[b, h][:, None] * k_scale[b, hk, j0 // BLKK]).to(torch.float32)
                    xt = x_f[:, j0:j1]
                    mneg = -(magic * sc)  # fp32
                    # a key the row may not see scores magic - 2**22, below every real dot product
                    xt_max = xt if allow is None else torch.where(allow, xt, torch.tensor(magic - (4194304.0 if magic < 2.0**24 else 8388608.0)))
                    m_tile = (xt_max.amax(dim=1, keepdim=True).double() * sc.double() + mneg.double()).float()  # fma
                    lazy = torch.tensor(LAZY_MAX if exact_exp2 else LAZY_MAX_PWL, dtype=torch.float32)
                    m_new = torch.where(m_tile > m + lazy, m_tile, m)
                    alpha = torch.exp2(m - m_new)  # 1 where the reference point stays, 0 at a row's first tile
                    c = ((P_SHIFT if exact_exp2 else P_SHIFT_PWL) - m_new) + mneg
                    if exact_exp2:
                        e = (xt.double() * sc.double() + c.double()).float()
                        p8 = torch.exp2(e).clamp(max=FP8_MAX).to(torch.float8_e4m3fn).float()
                    else:
                        cp = (8.0 * c.double() + 55.5).float()
                        t = (xt.double() * (8.0 * sc).double() + cp.double()).float()
                        code = torch.round(t).clamp_(0, 126).long()
                        p8 = e4m3fn_decode_table().float()[code]
                    if allow is not None:
                        p8 = torch.where(allow, p8, torch.zeros_like(p8))
                    if act is not None:
                        m_new = torch.where(act, m_new, m)
                        alpha = torch.where(act, alpha, torch.ones_like(alpha))
                        p8 = torch.where(act, p8, torch.zeros_like(p8))
                    l = l * alpha + p8.sum(dim=1, keepdim=True)  # the normaliser sees the rounded P too
                    acc = acc * alpha + p8 @ vf[j0:j1]
                    return m_new, l, acc

                acc, m, l = walk(0, lk_b)
                if key_split is not None:
                    if causal or block_mask is not None:
                        raise NotImplementedError("key_split with causal masking or a block mask")
                    first_wg, runs = key_split
                    n_qwg = (Lq + 255) // 256
                    tiles = (lk_b + BLKK - 1) // BLKK
                    per = (tiles + runs - 1) // runs
                    parts = [walk(r * per * BLKK, min(lk_b, (r + 1) * per * BLKK)) for r in range(runs) if r * per < tiles]
                    m_all = torch.stack([pm for _, pm, _ in parts]).amax(dim=0)
                    acc_s = sum(pa * torch.exp2(pm - m_all) for pa, pm, _ in parts)
                    l_s = sum(pl * torch.exp2(pm - m_all) for _, pm, pl in parts)
                    wg_of_row = (b * H + h) * n_qwg + torch.arange(Lq) // 256
                    cut = (wg_of_row >= first_wg)[:, None]
                    acc, l = torch.where(cut, acc_s, acc), torch.where(cut, l_s, l)
                o = acc / l * v_scale[b, hk][None, :]
                if v_mean is not None:
                    o = o + v_mean[b, hk].float()[None, :]
                o = torch.where(l > 0, o, torch.zeros_like(o))
            else:
                m = s.amax(dim=1, keepdim=True)
                p8 = p_to_e4m3(s - m + (P_SHIFT if exact_exp2 else P_SHIFT_PWL), exact_exp2)
                l = p8.sum(dim=1, keepdim=True)
                o = (p8 @ vf) * v_scale[b, hk][None, :] / l
                if v_mean is not None:
                    o = o + v_mean[b, hk].float()[None, :]
            out[b, :, h, :] = o.to(out_dtype)
    return out


def sage_emul_ref(q, k, v, *, sm_scale=None, smooth_k=True, causal=False, online=True, exact_exp2=True, k_lens=None,
                  block_mask=None, smooth_v=False):
    """[B, L, H, D] half in, same out: quantise with the oracle quantizer, then emulate."""
    D = q.shape[-1]
    sm_scale = D**-0.5 if sm_scale is None else sm_scale
    q_i8, q_scale = quant_q_ref(q, sm_scale)
    k_i8, k_scale, _ = quant_k_ref(k, smooth_k=smooth_k)
    v_fp8, v_scale, *rest = quant_v_ref(v, smooth_v=smooth_v)
    return sage_emul_from_quant(q_i8, q_scale, k_i8, k_scale, v_fp8, v_scale, q.dtype, causal=causal, online=online,
                                exact_exp2=exact_exp2, k_lens=k_lens, block_mask=block_mask,
                                v_mean=rest[0] if rest else None)
