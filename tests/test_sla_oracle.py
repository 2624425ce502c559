"""Pins of oracle/sla_ref.py (block means, block map and linear branch of the sparse-linear backend,
ksana/operations/attention/backends/sage_sla.py:43-90, 273-282) by independent formulations; CPU only."""

import pytest
import torch

from oracle.quant_ref import k_mean_ref
from oracle.sla_ref import block_map_ref, block_means_ref, linear_branch_ref


def _rand(shape, seed, dtype=torch.bfloat16, scale=1.0):
    return (torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("L,rows", [(64, 64), (130, 64), (300, 128), (33, 32)])
def test_block_means_against_a_scalar_replay_of_the_order(L, rows, dtype):
    x = _rand((1, 2, L, 4), 10 + L, dtype, 3.0)
    centre = _rand((1, 2, 4), 11, torch.float32)
    for cen in (None, centre):
        got = block_means_ref(x, rows, cen)
        nblk = -(-L // rows)
        assert got.shape == (1, 2, nblk, 4) and got.dtype == dtype
        f32 = lambda t: torch.tensor(t, dtype=torch.float32)
        for h in range(2):
            for blk in range(nblk):
                for d in range(4):
                    slots = []
                    for s in range(32):  # slot s adds rows s, s + 32, ... of the block in order
                        acc = None
                        for i in range(rows // 32):
                            r = blk * rows + i * 32 + s
                            val = f32(0.0)
                            if r < L:
                                val = x[0, h, r, d].float()
                                if cen is not None:
                                    val = (val - cen[0, h, d]).to(dtype).float()
                            acc = val if acc is None else acc + val
                        slots.append(acc)
                    while len(slots) > 1:  # adjacent pairs
                        slots = [slots[2 * i] + slots[2 * i + 1] for i in range(len(slots) // 2)]
                    n = min(rows, L - blk * rows)
                    want = (slots[0] / f32(float(n))).to(dtype)
                    assert got[0, h, blk, d] == want


def test_block_means_closed_forms_and_float64():
    x = torch.full((1, 1, 200, 8), 1.5, dtype=torch.bfloat16)
    assert (block_means_ref(x, 128) == 1.5).all()  # a constant comes back, also from the short last block (72 rows)
    x = _rand((2, 3, 500, 16), 5, torch.bfloat16, 2.0)
    got = block_means_ref(x, 64).double()
    xd = torch.nn.functional.pad(x.double(), (0, 0, 0, 12)).view(2, 3, 8, 64, 16)
    want = xd.sum(dim=3) / torch.tensor([64.0] * 7 + [52.0], dtype=torch.float64).view(1, 1, 8, 1)
    assert (got - want).abs().max() <= 2.0**-8 * want.abs().max() + 1e-6  # one rounding to bf16
    # centring: the differences are rounded to the dtype before they are pooled (the reference pools a half tensor)
    c = _rand((2, 3, 16), 6, torch.float32)
    got = block_means_ref(x, 64, c)
    manual = block_means_ref((x.float() - c[:, :, None, :]).to(torch.bfloat16), 64)
    assert torch.equal(got, manual)


def test_block_map_against_float64_brute_force():
    B, H, Lq, Lk, D = 1, 2, 512, 768, 16
    q = _rand((B, Lq, H, D), 21, scale=2.0)
    k = _rand((B, Lk, H, D), 22, scale=2.0) + 1.5
    bmap, kept, gap = block_map_ref(q, k, 0.25)
    nq, nk = Lq // 128, Lk // 64
    assert bmap.shape == (B, H, nq, nk) and bmap.dtype == torch.int8 and kept == int(0.25 * nk) == 3
    assert (bmap.sum(dim=-1) == kept).all()
    # an offset of k cancels in the centring
    assert torch.equal(bmap, block_map_ref(q, (k.float() + 4.0).to(k.dtype), 0.25)[0]) or gap.min() < 0.05
    # brute force in float64 without any intermediate rounding: the same blocks wherever the cut is clear
    qd, kd = q.double().permute(0, 2, 1, 3), k.double().permute(0, 2, 1, 3)
    kd = kd - kd.mean(dim=2, keepdim=True)
    for h in range(H):
        pq = torch.stack([qd[0, h, i * 128 : (i + 1) * 128].mean(dim=0) for i in range(nq)])
        pk = torch.stack([kd[0, h, j * 64 : (j + 1) * 64].mean(dim=0) for j in range(nk)])
        score = pq @ pk.t()
        for i in range(nq):
            if gap[0, h, i] > 0.05 * score[i].abs().max():
                want = set(score[i].topk(kept).indices.tolist())
                assert set(torch.nonzero(bmap[0, h, i]).flatten().tolist()) == want
    assert (gap > 0.05 * 0.01).any()  # the check above was not vacuous
    # topk 1.0 keeps everything, a tiny ratio keeps nothing (int(ratio * nk) == 0, as in the reference)
    assert (block_map_ref(q, k, 1.0)[0] == 1).all() and (block_map_ref(q, k, 0.01)[0] == 0).all()


def test_block_map_uses_the_frozen_k_mean_and_ragged_blocks():
    q = _rand((1, 200, 1, 8), 31)
    k = _rand((1, 150, 1, 8), 32) + 2.0
    bmap, kept, _ = block_map_ref(q, k, 0.67)
    assert bmap.shape == (1, 1, 2, 3) and kept == 2  # ceil(200/128) x ceil(150/64)
    km = k_mean_ref(k)
    pooled_k = block_means_ref(k.permute(0, 2, 1, 3), 64, centre=km)
    assert pooled_k.shape == (1, 1, 3, 8)
    # the last key block has 22 rows: its mean is over 22, not 64
    tail = ((k[0, 128:, 0].float() - km[0, 0].float()).to(torch.bfloat16).double().mean(dim=0))
    assert (pooled_k[0, 0, 2].double() - tail).abs().max() <= 2.0**-7 * tail.abs().max() + 1e-3


def test_linear_branch_against_the_explicit_quadratic_form():
    """(phi(q) (phi(k)^T v)) / (1e-5 + phi(q) . sum phi(k)) is attention with weights phi(q_i) . phi(k_j): computed
    here row by row in float64, L x L weights and all."""
    B, L, H, D = 1, 40, 2, 8
    q, k, v = _rand((B, L, H, D), 41, scale=1.5), _rand((B, L, H, D), 42, scale=1.5), _rand((B, L, H, D), 43)
    got = linear_branch_ref(q, k, v)
    assert got.shape == (B, H, L, D) and got.dtype == q.dtype
    for h in range(H):
        fq = torch.softmax(q[0, :, h].double(), dim=-1)
        fk = torch.softmax(k[0, :, h].double(), dim=-1)
        w = fq @ fk.t()  # [L, L], all positive
        want = (w @ v[0, :, h].double()) / (1e-5 + w.sum(dim=1, keepdim=True))
        err = (got[0, h].double() - want).abs().max()
        assert err <= 0.03 * want.abs().max() + 1e-3  # a handful of bf16 roundings
    # rows of the feature maps sum to one: a constant v comes back (up to the 1e-5 in the denominator and rounding)
    ones = linear_branch_ref(q, k, torch.full_like(v, 2.0))
    assert (ones.float() - 2.0).abs().max() <= 0.03
    # and the result is linear in v
    twice = linear_branch_ref(q, k, (2 * v.float()).to(v.dtype))
    assert (twice.float() - 2 * got.float()).abs().max() <= 0.03 * got.float().abs().max() + 1e-3
