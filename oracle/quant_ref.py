"""Oracle: the Sage quantizer, specified in PyTorch on the CPU.  Test infrastructure only.

Stage order, block sizes and tensor roles follow the only in-repo evidence of the pipeline,
ksana/operations/attention/backends/sage_sla.py:196-228:

* ``km = k.mean(dim=-2, keepdim=True)`` in the tensor dtype            (sage_sla.py:198)
* ``get_vanilla_qk_quant(q, k, km, 128, 64)`` -> int8 Q/K + fp32 scales (sage_sla.py:202-204)
* V -> fp8 e4m3fn with one fp32 scale per (b, h, d)                     (sage_sla.py:222-228)
* softmax scale ``1/sqrt(D)`` handed to the kernel separately           (sage_sla.py:206)

The arithmetic inside those third-party calls is not in the reference, so every choice the
call sites leave open is frozen HERE, and the HIP kernels reproduce it bit for bit:

1. K mean.  fp32 accumulation in a fixed order: the sequence is cut into chunks of
   ``MEAN_CHUNK`` rows (zero padded); inside a chunk row ``i`` belongs to slot ``i % 32``
   and each slot is summed sequentially in increasing row order; the 32 slot sums are
   reduced by an adjacent-pair binary tree (5 levels); chunk sums are added sequentially in
   increasing chunk order; the total is divided by ``float32(L)`` (IEEE division) and
   rounded to the input dtype (round to nearest even), as ``torch.mean`` of a half tensor
   returns the half dtype.
2. K smoothing: ``float32(k) - float32(km)``, one IEEE subtraction.
3. Outlier spreading: every 128-channel row of Q and of smoothed K goes through an
   UNNORMALISED fast Walsh-Hadamard transform (``fwht_ref``: butterflies of stride
   1, 2, 4, ..., 64 in that order, ``(a, b) -> (a + b, a - b)``, natural ordering).  The
   transform is orthogonal up to the factor 128, so ``Q K^T`` is unchanged once Q absorbs
   ``2**-7``; a single x20 outlier entry is spread over all 128 channels instead of
   dictating the int8 step of its whole block.  (Per-block int8 without this stage reaches
   only cos-sim 0.97 against SDPA on the outlier workload; with it 0.9994.)
4. Q is then multiplied by ``c = (float32(sm_scale) * float32(log2 e)) * 2**-7`` (one fp32
   product and an exact power-of-two scaling), so the attention kernel exponentiates with
   ``exp2`` directly.
5. int8: ``amax = max|x|`` over a block, ``scale = amax / 127``, ``inv = 127 / amax`` (IEEE
   divisions; both 0 when ``amax == 0``), ``x_i8 = rne(x * inv)`` with the product EXACT (not first rounded to
   fp32: what a fused multiply-add onto ``1.5 * 2**23`` leaves in its low byte) and ``rne`` = round-half-to-even;
   ``|x * inv| <= 127 (1 + 2**-24)`` by construction, so no clamp is needed (one is kept here as a guard).  A K block is ``BLKK`` = 64 key rows
   (sage_sla.py:204; a ragged last block uses its valid rows only).  A Q block is ONE query
   row (``BLKQ`` = 1): per-token scales cost nothing in the attention kernel, where a lane
   owns one query column, and keep a Q outlier from degrading 127 other rows.
6. V: ``amax[b,h,d] = max_l |v|``, ``v_scale = amax / 448``, ``inv = 448 / amax`` (0 when
   ``amax == 0``), ``v_fp8 = e4m3fn(clamp(float32(v) * inv, -448, 448))`` with round to
   nearest even (torch's cast; the clamp is there because the cast does not saturate).

All results are returned in the LOGICAL layout ``[B, H, L, D]``; how the kernels tile them
in HBM is the product's business (``ksanadit_amd.layout``).
"""

from __future__ import annotations

import torch

BLKQ = 1
BLKK = 64
MEAN_CHUNK = 256
MEAN_SLOTS = 32
LOG2E = 1.4426950408889634
FP8_MAX = 448.0


def _to_bhld_f32(x: torch.Tensor) -> torch.Tensor:
    """[B, L, H, D] half -> [B, H, L, D] fp32 (exact widening)."""
    return x.permute(0, 2, 1, 3).to(torch.float32).contiguous()


def pad_head_dim(x: torch.Tensor, to: int = 128) -> torch.Tensor:
    """Head size 64 (rule 7 of the specification): every row of Q, K and V is extended to 128 channels with zeros and
    rules 1-6 apply to the extended rows unchanged.  The transform of an extended row is the 64-point transform of the
    row twice in a row, so ``(H q') . (H k') = 128 q . k`` as for head size 128; the extended channels of V quantize to
    zero with scale zero, and the output keeps the first 64 channels."""
    d = x.shape[-1]
    assert d <= to
    return x if d == to else torch.nn.functional.pad(x, (0, to - d))


def q_premul(sm_scale: float, D: int = 128) -> torch.Tensor:
    """``c`` of rule 4, as a 0-d fp32 tensor (``2**-7`` is ``1/D`` for the head size 128)."""
    c = torch.tensor(sm_scale, dtype=torch.float32) * torch.tensor(LOG2E, dtype=torch.float32)
    return c * torch.tensor(1.0 / D, dtype=torch.float32)


def fwht_ref(x: torch.Tensor) -> torch.Tensor:
    """Unnormalised Walsh-Hadamard transform of the last axis (rule 3), fp32, fixed order."""
    shape = x.shape
    D = shape[-1]
    assert D & (D - 1) == 0, "length must be a power of two"
    x = x.to(torch.float32)
    s = 1
    while s < D:
        y = x.reshape(-1, D // (2 * s), 2, s)
        a, b = y[:, :, 0, :], y[:, :, 1, :]
        x = torch.stack([a + b, a - b], dim=2).reshape(shape)
        s *= 2
    return x


def k_mean_sum_ref(k: torch.Tensor) -> torch.Tensor:
    """fp32 column sums of K in the frozen order of rule 1.  k: [B, L, H, D] -> [B, H, D]."""
    kf = _to_bhld_f32(k)
    B, H, L, D = kf.shape
    nch = (L + MEAN_CHUNK - 1) // MEAN_CHUNK
    pad = nch * MEAN_CHUNK - L
    if pad:
        kf = torch.cat([kf, kf.new_zeros(B, H, pad, D)], dim=2)
    x = kf.view(B, H, nch, MEAN_CHUNK // MEAN_SLOTS, MEAN_SLOTS, D)
    acc = x[:, :, :, 0].clone()
    for i in range(1, MEAN_CHUNK // MEAN_SLOTS):
        acc = acc + x[:, :, :, i]
    while acc.shape[3] > 1:
        acc = acc[:, :, :, 0::2] + acc[:, :, :, 1::2]
    part = acc[:, :, :, 0]  # [B, H, nch, D]
    tot = part[:, :, 0].clone()
    for c in range(1, nch):
        tot = tot + part[:, :, c]
    return tot


def k_mean_ref(k: torch.Tensor) -> torch.Tensor:
    """``km`` of sage_sla.py:198 under rule 1.  k: [B, L, H, D] half -> [B, H, D] same dtype."""
    L = k.shape[1]
    tot = k_mean_sum_ref(k)
    return (tot / torch.tensor(float(L), dtype=torch.float32)).to(k.dtype)


def _block_int8(x: torch.Tensor, blk: int):
    """x: [B, H, L, D] fp32 -> (int8 [B, H, L, D], scale fp32 [B, H, ceil(L/blk)]) (rule 5)."""
    B, H, L, D = x.shape
    nb = (L + blk - 1) // blk
    pad = nb * blk - L
    xp = torch.cat([x, x.new_zeros(B, H, pad, D)], dim=2) if pad else x
    xb = xp.view(B, H, nb, blk * D)
    amax = xb.abs().amax(dim=-1)  # zero padding cannot raise a max of absolute values
    nz = amax > 0
    safe = torch.where(nz, amax, torch.ones_like(amax))
    # tensor / tensor on purpose: `scalar / tensor` is reciprocal-then-multiply in torch (two roundings)
    qmax = torch.full_like(amax, 127.0)
    scale = torch.where(nz, amax / qmax, torch.zeros_like(amax))
    inv = torch.where(nz, qmax / safe, torch.zeros_like(amax))
    # float64 holds the product of two fp32 values exactly (48 significant bits); torch.round is half-to-even
    y = torch.round(xb.double() * inv.unsqueeze(-1).double()).clamp_(-127.0, 127.0)
    xi = y.to(torch.int8).view(B, H, nb * blk, D)[:, :, :L].contiguous()
    return xi, scale


def quant_q_ref(q: torch.Tensor, sm_scale: float):
    """q: [B, L, H, D] half -> (q_i8 [B, H, L, D] int8, q_scale [B, H, L] fp32)."""
    x = fwht_ref(_to_bhld_f32(q)) * q_premul(sm_scale, q.shape[-1])
    return _block_int8(x, BLKQ)


def quant_k_ref(k: torch.Tensor, smooth_k: bool = True):
    """k: [B, L, H, D] half -> (k_i8 [B,H,L,D], k_scale [B,H,ceil(L/64)], km [B,H,D] half)."""
    km = k_mean_ref(k) if smooth_k else torch.zeros(k.shape[0], k.shape[2], k.shape[3], dtype=k.dtype)
    x = fwht_ref(_to_bhld_f32(k) - km.to(torch.float32)[:, :, None, :])
    xi, scale = _block_int8(x, BLKK)
    return xi, scale, km


def quant_v_ref(v: torch.Tensor, smooth_v: bool = False):
    """v: [B, L, H, D] half -> (v_fp8 [B, H, L, D] float8_e4m3fn, v_scale [B, H, D] fp32), and with ``smooth_v`` a
    third result, the channel mean [B, H, D] in v's dtype that was taken off before scaling.

    ``smooth_v`` is the V counterpart of the K smoothing: the mean over the sequence (same summation order and rounding
    as ``k_mean_ref``) is subtracted in fp32, the centred values are quantized, and the attention adds the mean back to
    its output - rows of P sum to one, so ``P (V - m) + m == P V``.  A channel whose values sit far from zero then
    spends its eight e4m3 steps per octave on the deviations instead of on the offset."""
    x = _to_bhld_f32(v)
    vm = None
    if smooth_v:
        vm = k_mean_ref(v)
        x = x - vm.to(torch.float32)[:, :, None, :]
    amax = x.abs().amax(dim=2)  # [B, H, D]
    nz = amax > 0
    safe = torch.where(nz, amax, torch.ones_like(amax))
    fmax = torch.full_like(amax, FP8_MAX)
    scale = torch.where(nz, amax / fmax, torch.zeros_like(amax))
    inv = torch.where(nz, fmax / safe, torch.zeros_like(amax))
    y = (x * inv[:, :, None, :]).clamp_(-FP8_MAX, FP8_MAX)
    codes = y.to(torch.float8_e4m3fn)
    return (codes, scale, vm) if smooth_v else (codes, scale)


def e4m3fn_decode_table() -> torch.Tensor:
    """All 256 e4m3fn codes decoded from the format definition (1-4-3, bias 7, no inf,
    S.1111.111 = NaN).  Independent of torch's cast; used to pin it."""
    out = torch.empty(256, dtype=torch.float64)
    for code in range(256):
        s = -1.0 if code & 0x80 else 1.0
        e = (code >> 3) & 0xF
        m = code & 0x7
        if e == 0xF and m == 0x7:
            val = float("nan")
        elif e == 0:
            val = s * (m / 8.0) * 2.0**-6
        else:
            val = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
        out[code] = val
    return out
