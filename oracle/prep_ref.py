"""Oracle for what the Wan attention block does to Q and K before attention: RMSNorm over the
whole token row, then the 3-axis rotary embedding.  Test infrastructure only.

Restates, with torch CPU ops:
* ``RMSNorm.float_rmsnorm`` - ksana/operations/ops.py:62-72: ``(x.float() * rsqrt(mean(x^2, -1) + eps)
  * weight).type_as(x)``, used by ``norm_q`` / ``norm_k`` of ``WanSelfAttention`` on the ``[B, L, H*D]``
  projections (ksana/models/wan/wan_model.py:81-90,163-165; weights are fp32, ``:82``);
* ``rope_params`` and the three-way frequency table - wan_model.py:51-58,677-684;
* ``apply_default_rope`` for one GPU (``sp_size == 1``) - ksana/utils/rope.py:21-24,43-58,61-128: pairs
  ``(x[2i], x[2i+1])`` as complex128 times ``freqs[axis position, i]``, the first ``22`` pairs (for
  D = 128) turning with the frame index, the next ``21`` with the row, the last ``21`` with the column;
  rows at or beyond ``F*H*W`` pass unchanged; result cast back to the input dtype.

One thing is FROZEN here beyond what the reference states, so that a GPU kernel can be compared
bit for bit: the order of the fp32 sum behind ``mean(x^2)``.  The row is cut into groups of 8
channels; accumulator ``i`` of 64 takes groups ``i, i+64, i+128, ...`` in order, adding the 8
squares of each one after the other; the 64 accumulators are then combined by an adjacent-pair
tree.  ``rsqrt`` is ``1 / sqrt`` with both operations correctly rounded: what ``torch.rsqrt`` computes
on the CPU (``torch.sqrt`` does not always round correctly there, so the two are taken from numpy).  Any other order moves the statistic by ~1e-7 relative, i.e. flips about one bf16
result in 10^5.

Pinned by tests/test_prep_oracle.py: against ``torch.nn.functional.rms_norm`` (the library routine
the reference's default configuration dispatches to), against float64 brute force, against an
independent real-arithmetic form of the rotation, and by the rotation's invariants (pair norms,
position 0, padding rows, angle addition).
"""

from __future__ import annotations

import numpy as np
import torch

ROPE_TABLE_ROWS = 1024  # wan_model.py:679-681


def rope_params(max_seq_len: int, dim: int, theta: float = 10000.0) -> torch.Tensor:
    """complex128 ``[max_seq_len, dim // 2]``: ``exp(i * pos * theta^(-2j/dim))`` (wan_model.py:51-58)."""
    assert dim % 2 == 0
    freqs = torch.outer(
        torch.arange(max_seq_len),
        1.0 / torch.pow(theta, torch.arange(0, dim, 2).to(torch.float64).div(dim)),
    )
    return torch.polar(torch.ones_like(freqs), freqs)


def wan_rope_table(head_dim: int, rows: int = ROPE_TABLE_ROWS) -> torch.Tensor:
    """The model's ``freqs`` buffer: frame, row and column tables side by side (wan_model.py:676-684)."""
    d = head_dim
    return torch.cat(
        [rope_params(rows, d - 4 * (d // 6)), rope_params(rows, 2 * (d // 6)), rope_params(rows, 2 * (d // 6))], dim=1
    )


def rope_split_sizes(half_dim: int) -> list[int]:
    """Pairs per axis (rope.py:21-24): ``[22, 21, 21]`` for ``half_dim == 64``."""
    return [half_dim - 2 * (half_dim // 3), half_dim // 3, half_dim // 3]


def mean_square_ref(x: torch.Tensor) -> torch.Tensor:
    """fp32 ``mean(x^2)`` over the last dim in the frozen order described in the module docstring."""
    n = x.shape[-1]
    assert n % 8 == 0
    sq = x.float() * x.float()  # exact for fp16 / bf16 inputs
    groups = n // 8
    iters = (groups + 63) // 64
    pad = iters * 64 * 8 - n
    if pad:
        sq = torch.cat([sq, torch.zeros(*sq.shape[:-1], pad)], dim=-1)  # adding +0.0 changes nothing
    sq = sq.reshape(*sq.shape[:-1], iters, 64, 8)
    acc = torch.zeros(*sq.shape[:-3], 64)
    for it in range(iters):
        for e in range(8):
            acc = acc + sq[..., it, :, e]
    width = 64
    while width > 1:  # adjacent pairs: (0,1), (2,3), ... then pairs of pairs, ...
        acc = acc.reshape(*acc.shape[:-1], width // 2, 2)
        acc = acc[..., 0] + acc[..., 1]
        width //= 2
    return acc[..., 0] / torch.tensor(float(n), dtype=torch.float32)


def inv_rms_ref(x: torch.Tensor, eps: float) -> torch.Tensor:
    """``rsqrt(mean(x^2) + eps)`` per row, fp32 (ops.py:65-66)."""
    t = (mean_square_ref(x) + torch.tensor(eps, dtype=torch.float32)).numpy()
    return torch.from_numpy((np.float32(1.0) / np.sqrt(t)).astype(np.float32))


def rmsnorm_ref(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``[..., H*D]`` half in, same out (ops.py:62-72)."""
    r = inv_rms_ref(x, eps)[..., None]
    return ((x.float() * r) * weight.float()).type_as(x)


def rope_ref(x: torch.Tensor, grid_sizes, freqs: torch.Tensor) -> torch.Tensor:
    """``[B, L, H, D]`` in, same shape and dtype out (rope.py:61-128, the ``sp_size == 1`` branch)."""
    B, L, H, D = x.shape
    half = D // 2
    parts = freqs.to(torch.complex128).split(rope_split_sizes(half), dim=1)
    out = []
    for b, (f, h, w) in enumerate(torch.as_tensor(grid_sizes).tolist()):
        f, h, w = int(f), int(h), int(w)
        n = f * h * w
        table = torch.cat(
            [
                parts[0][:f].view(f, 1, 1, -1).expand(f, h, w, -1),
                parts[1][:h].view(1, h, 1, -1).expand(f, h, w, -1),
                parts[2][:w].view(1, 1, w, -1).expand(f, h, w, -1),
            ],
            dim=-1,
        ).reshape(n, 1, -1)
        xb = torch.view_as_complex(x[b, :n].to(torch.float64).reshape(n, H, -1, 2))
        xb = torch.view_as_real(xb * table).flatten(2)
        out.append(torch.cat([xb, x[b, n:]]))  # float64 wins the concatenation; the cast below undoes it
    return torch.stack(out, dim=0).type_as(x)


def wan_prep_ref(x: torch.Tensor, weight, eps: float, grid_sizes, freqs, num_heads: int) -> torch.Tensor:
    """``[B, L, H*D]`` projection -> ``[B, L, H, D]`` ready for attention (wan_model.py:163-174).
    ``weight is None`` skips the norm, ``freqs is None`` the rotation."""
    B, L, HD = x.shape
    y = x if weight is None else rmsnorm_ref(x, weight, eps)
    y = y.view(B, L, num_heads, HD // num_heads)
    return y if freqs is None else rope_ref(y, grid_sizes, freqs)


# ---------------------------------------------------------------------------------------------------------------
# The Qwen-Image block's step before attention (ksana/models/qwen/attention.py:340-357):
#   img_q = norm_q(img_q); txt_q = norm_added_q(txt_q)          RMSNorm over the D channels of every head (:269-272)
#   x = apply_rotary_emb_qwen(x, freqs)  (:31-59)                complex64: view_as_complex(x.float()) * freqs
#   joint = cat([txt, img], dim=1)                               text rows first (:355-357)
# ``RMSNorm.float_rmsnorm`` (ops.py:62-72) is the arithmetic restated; the order of the sum of squares over the 128
# channels is frozen here: eight accumulators take 16 consecutive channels each, in channel order, and meet in an
# adjacent-pair tree.  The rotation is written in real arithmetic - four products, one subtraction, one addition, each
# rounded to fp32 - which is bit for bit what torch's complex64 multiplication computes on the CPU (pinned in
# tests/test_prep_oracle.py against ``torch.view_as_complex(...) * freqs``, the reference's own expression).
# ---------------------------------------------------------------------------------------------------------------
def head_mean_square_ref(x: torch.Tensor) -> torch.Tensor:
    """fp32 ``mean(x^2)`` over a last dim of 128 in the frozen order described above."""
    assert x.shape[-1] == 128
    sq = (x.float() * x.float()).reshape(*x.shape[:-1], 8, 16)  # exact for half inputs
    acc = sq[..., 0]
    for e in range(1, 16):
        acc = acc + sq[..., e]
    width = 8
    while width > 1:
        acc = acc.reshape(*acc.shape[:-1], width // 2, 2)
        acc = acc[..., 0] + acc[..., 1]
        width //= 2
    return acc[..., 0] / torch.tensor(128.0, dtype=torch.float32)


def head_rmsnorm_ref(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``[..., 128]`` half in, same out: ``float_rmsnorm`` per head (ops.py:62-72)."""
    t = (head_mean_square_ref(x) + torch.tensor(eps, dtype=torch.float32)).numpy()
    r = torch.from_numpy((np.float32(1.0) / np.sqrt(t)).astype(np.float32))[..., None]
    return ((x.float() * r) * weight.float()).type_as(x)


def qwen_rope_ref(x: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """``apply_rotary_emb_qwen`` (qwen/attention.py:31-59, one GPU): ``x`` ``[B, L, H, D]``, ``freqs`` complex64
    ``[>= L, D/2]``; same shape and dtype out."""
    L = x.shape[1]
    f = torch.view_as_real(freqs[:L].to(torch.complex64))  # [L, D/2, 2]
    c, s = f[..., 0][None, :, None, :], f[..., 1][None, :, None, :]
    xf = x.float().reshape(*x.shape[:-1], -1, 2)
    a, b = xf[..., 0], xf[..., 1]
    re = a * c - b * s
    im = a * s + b * c
    return torch.stack([re, im], dim=-1).flatten(3).type_as(x)


def qwen_prep_ref(x: torch.Tensor, txt_len: int, weight_img, weight_txt, eps: float, img_freqs, txt_freqs) -> torch.Tensor:
    """The joint ``[B, L, H, D]`` projection (text rows first) -> normed and rotated, ready for attention.
    ``None`` weights / tables skip that step for their segment."""
    txt, img = x[:, :txt_len], x[:, txt_len:]
    if weight_txt is not None:
        txt = head_rmsnorm_ref(txt, weight_txt, eps)
    if weight_img is not None:
        img = head_rmsnorm_ref(img, weight_img, eps)
    if txt_freqs is not None and txt.shape[1]:
        txt = qwen_rope_ref(txt, txt_freqs)
    if img_freqs is not None and img.shape[1]:
        img = qwen_rope_ref(img, img_freqs)
    return torch.cat([txt, img], dim=1)


def qwen_rope_table(rows: int, axes_dim=(16, 56, 56), theta: float = 10000.0, offset: int = 0) -> torch.Tensor:
    """A complex64 ``[rows, 64]`` table of the shape ``QwenEmbedRope`` produces (qwen/attention.py:62-96): per axis
    ``exp(i * pos * theta^(-2j/dim))`` in fp32, the three axes side by side; here every axis simply counts the row."""
    parts = []
    for dim in axes_dim:
        fr = torch.outer(torch.arange(offset, offset + rows).float(), 1.0 / torch.pow(theta, torch.arange(0, dim, 2).float().div(dim)))
        parts.append(torch.polar(torch.ones_like(fr), fr))
    return torch.cat(parts, dim=1)


# ---------------------------------------------------------------------------------------------------------------
# The Wan block with ``rope_func == "comfy"`` (wan_model.py:169-171): ``EmbedND`` (ksana/utils/rope.py:151-177) hands
# over one fp32 2x2 rotation matrix per (position, pair) and ``apply_comfyui_rope`` (rope.py:180-212) applies it as
#   x_out = freqs_cis[..., 0] * x_[..., 0];  x_out.addcmul_(freqs_cis[..., 1], x_[..., 1])
# i.e. out[2i+e] = m[e][0] * x[2i] + m[e][1] * x[2i+1] in fp32.  torch evaluates the first product on its own and
# fuses the second into the sum (one rounding for ``m[e][1] * x[2i+1] + first``); that is restated here with float64,
# which holds the product of two fp32 values exactly (pinned against the two torch calls in tests/test_prep_oracle.py).
# Positions past the table get the identity matrix (rope.py:133-148): unchanged rows.
# ---------------------------------------------------------------------------------------------------------------
def comfy_rope_matrices(ids: torch.Tensor, axes_dim=(44, 42, 42), theta: float = 10000.0) -> torch.Tensor:
    """``EmbedND.forward`` without its broadcast dims: ``ids`` ``[L, n_axes]`` positions -> fp32 ``[L, sum(axes)/2, 2, 2]``
    (``_comfy_rope``, rope.py:151-162: float64 frequencies, fp32 angles, ``[[cos, -sin], [sin, cos]]``)."""
    parts = []
    for a, dim in enumerate(axes_dim):
        scale = torch.linspace(0, (dim - 2) / dim, steps=dim // 2, dtype=torch.float64)
        omega = 1.0 / (theta**scale)
        out = torch.einsum("...n,d->...nd", ids[..., a].to(torch.float32), omega)
        out = torch.stack([torch.cos(out), -torch.sin(out), torch.sin(out), torch.cos(out)], dim=-1)
        parts.append(out.reshape(*out.shape[:-1], 2, 2).to(torch.float32))
    return torch.cat(parts, dim=-3)


def comfy_rope_ref(x: torch.Tensor, matrices: torch.Tensor) -> torch.Tensor:
    """``apply_comfyui_rope`` for one GPU: ``x`` ``[B, L, H, D]`` half, ``matrices`` fp32 ``[rows, D/2, 2, 2]``; rows of
    ``x`` at or past ``rows`` stay as they are."""
    B, L, H, D = x.shape
    n = min(L, matrices.shape[0])
    m = matrices[:n].to(torch.float32)[None, :, None]  # [1, n, 1, D/2, 2, 2]
    xf = x[:, :n].float().reshape(B, n, H, D // 2, 2)
    x0, x1 = xf[..., 0:1], xf[..., 1:2]  # [B, n, H, D/2, 1]
    first = m[..., 0] * x0  # fp32 product, rounded
    fused = (m[..., 1].double() * x1.double() + first.double()).float()  # exact product, one rounding of the sum
    return torch.cat([fused.reshape(B, n, H, D).type_as(x), x[:, n:]], dim=1)


def wan_comfy_prep_ref(x: torch.Tensor, weight, eps: float, matrices, num_heads: int) -> torch.Tensor:
    """``[B, L, H*D]`` projection -> normed over the token row, viewed ``[B, L, H, D]``, rotated with the matrices."""
    B, L, HD = x.shape
    y = x if weight is None else rmsnorm_ref(x, weight, eps)
    y = y.view(B, L, num_heads, HD // num_heads)
    return y if matrices is None else comfy_rope_ref(y, matrices)
