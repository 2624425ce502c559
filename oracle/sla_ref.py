"""Oracle: the block map and the linear branch of the sparse-linear ("SLA") backend.  Test infrastructure only.

Restates, on the CPU, what ksana/operations/attention/backends/sage_sla.py computes around its block-sparse
attention call:

* ``block_means_ref``    the pooling of ``compress_kernel`` / ``mean_pool`` (sage_sla.py:43-75): per block of rows the
  fp32 sum divided by the number of rows that exist, rounded to the tensor's dtype.  The reference's kernel leaves
  the order of the sum to the compiler; it is frozen here (row ``r`` of a block goes to slot ``r % 32``, a slot adds
  its rows in increasing order, the 32 slots meet in an adjacent-pair tree) so that the HIP kernel can be compared bit
  for bit.  Against the reference's own order the result can differ by one unit in the last place of the half type:
  **parity unpinned** at that level (no fixture of the reference observes pooled values).
* ``block_map_ref``      ``get_block_map`` (sage_sla.py:78-90): k is centred with its mean over the sequence *as a
  tensor of k's dtype*, q and the centred k are pooled (128 query rows, 64 keys off Hopper, sage_sla.py:189), the
  pooled blocks are multiplied (a matmul in the tensors' dtype) and every query block keeps the ``int(topk * nk)``
  key blocks with the largest products.  Which of two equal products is kept is left open by ``torch.topk``; the
  function also returns the gap between the last kept and the first dropped product so that tests can use inputs on
  which the choice is unambiguous.
* ``linear_branch_ref``  the linear-attention branch (sage_sla.py:135-139, 273-282): softmax over the channels as the
  feature map of q and k (rounded to the dtype), ``(phi(q) (phi(k)^T v)) / (1e-5 + phi(q) . sum_j phi(k_j))``.

Pinned in tests/test_sla_oracle.py by a scalar replay of the summation order, float64 brute force on tiny inputs, an
explicit L x L formulation of the linear branch, and invariants (offset of k, rows of the map).
"""

from __future__ import annotations

import torch

from .quant_ref import k_mean_ref

SLOTS = 32


def block_means_ref(x: torch.Tensor, rows: int, centre: torch.Tensor | None = None) -> torch.Tensor:
    """``x``: ``[B, H, L, D]`` half tensor -> ``[B, H, ceil(L / rows), D]`` of the same dtype.  ``centre``
    (``[B, H, D]``, optional): every ``x - centre`` is rounded to ``x.dtype`` before it is summed."""
    assert rows % SLOTS == 0
    B, H, L, D = x.shape
    nblk = -(-L // rows)
    xf = x.float()
    if centre is not None:
        xf = (xf - centre.float()[:, :, None, :]).to(x.dtype).float()
    pad = nblk * rows - L
    if pad:
        xf = torch.nn.functional.pad(xf, (0, 0, 0, pad))
    # [B, H, nblk, rows / 32, 32, D]: row r = i * 32 + slot
    g = xf.view(B, H, nblk, rows // SLOTS, SLOTS, D)
    acc = g[:, :, :, 0]
    for i in range(1, rows // SLOTS):
        acc = acc + g[:, :, :, i]
    n = SLOTS
    while n > 1:  # adjacent-pair tree over the slots
        acc = acc.view(B, H, nblk, n // 2, 2, D)
        acc = acc[:, :, :, :, 0] + acc[:, :, :, :, 1]
        n //= 2
    total = acc.view(B, H, nblk, D)
    counts = torch.full((nblk,), float(rows))
    counts[-1] = float(rows - pad)
    return (total / counts.view(1, 1, nblk, 1)).to(x.dtype)


def block_map_ref(q: torch.Tensor, k: torch.Tensor, topk_ratio: float, blk_q: int = 128, blk_k: int = 64):
    """``q``, ``k``: ``[B, L, H, D]`` half tensors.  Returns ``(block_map int8 [B, H, nq, nk], kept, gap)`` with
    ``gap[b, h, i]`` = smallest kept product minus largest dropped product (fp32) of query block ``i``."""
    qh, kh = q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3)
    km = k_mean_ref(k)  # [B, H, D] in k's dtype: torch.mean of a half tensor, summation order frozen
    pooled_q = block_means_ref(qh, blk_q)
    pooled_k = block_means_ref(kh, blk_k, centre=km)
    score = (pooled_q.float() @ pooled_k.float().transpose(-1, -2)).to(q.dtype)  # a matmul in the tensors' dtype
    nk = score.shape[-1]
    kept = min(nk, int(topk_ratio * nk))
    order = score.float().sort(dim=-1, descending=True, stable=True)
    block_map = torch.zeros_like(score, dtype=torch.int8)
    block_map.scatter_(-1, order.indices[..., :kept], 1)
    if kept < nk:
        gap = order.values[..., kept - 1] - order.values[..., kept]
    else:
        gap = torch.full(score.shape[:-1], float("inf"))
    return block_map, kept, gap


def linear_branch_ref(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """``[B, L, H, D]`` half tensors -> the linear branch ``[B, H, L, D]`` in their dtype (before ``proj_l``).  Every
    intermediate the reference holds as a tensor of the working dtype is rounded to it here as well."""
    dt = q.dtype
    qh, kh, vh = (t.permute(0, 2, 1, 3).float() for t in (q, k, v))
    fq = torch.softmax(qh, dim=-1).to(dt).float()  # feature maps, sage_sla.py:135-139
    fk = torch.softmax(kh, dim=-1).to(dt).float()
    kv = (fk.transpose(-1, -2) @ vh).to(dt).float()  # calc_linear, sage_sla.py:276-279
    ksum = fk.sum(dim=-2, keepdim=True).to(dt).float()
    num = (fq @ kv).to(dt).float()
    den = (fq * ksum).to(dt).float().sum(dim=-1, keepdim=True).to(dt).float()
    return (num / (1e-5 + den).to(dt).float()).to(dt)
