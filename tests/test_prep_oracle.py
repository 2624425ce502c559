"""Pins for oracle/prep_ref.py (RMSNorm over the token row + Wan 3-axis RoPE) without the reference:
library routines of the torch installed here, float64 brute force, an independent real-arithmetic
form of the rotation, and the invariants of both operations."""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import prep_ref as pr


def _half(shape, seed, dtype=torch.bfloat16, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(shape, generator=g)).to(dtype)


# ------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("n", [128, 1536, 5120, 3072])
def test_mean_square_frozen_order_is_a_mean_square(n):
    x = _half((37, n), n)
    ms = pr.mean_square_ref(x)
    exact = x.double().pow(2).mean(-1)
    assert ms.dtype == torch.float32
    assert ((ms.double() - exact).abs() / exact).max() < 2e-6
    # a row of equal values has that value squared as its mean square, exactly, when n is a power of two times ...
    c = torch.full((1, n), 0.5, dtype=torch.bfloat16)
    assert abs(pr.mean_square_ref(c).item() - 0.25) < 1e-7


def test_mean_square_order_matters_and_is_the_stated_one():
    """Scalar replay of the stated order on one row: groups of 8, accumulator i takes groups i, i+64, ...;
    adjacent-pair tree.  A dropped group, a transposed index or a linear combine fails this."""
    import numpy as np

    x = _half((1, 1536), 5)
    sq = (x.float() * x.float()).numpy()[0]
    acc = [np.float32(0.0)] * 64
    groups = len(sq) // 8
    for gidx in range(groups):
        i = gidx % 64
        for e in range(8):
            acc[i] = np.float32(acc[i] + sq[gidx * 8 + e])
    while len(acc) > 1:
        acc = [np.float32(acc[2 * j] + acc[2 * j + 1]) for j in range(len(acc) // 2)]
    want = np.float32(acc[0] / np.float32(len(sq)))
    assert pr.mean_square_ref(x).item() == float(want)
    linear = np.float32(0.0)
    for v in sq:
        linear = np.float32(linear + v)
    assert float(np.float32(linear / np.float32(len(sq)))) != float(want)  # the order is observable


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rmsnorm_against_library_routine_and_float64(dtype):
    """ops.py:74-81 sends the default configuration to torch's own rms_norm: the restatement must agree with
    it to the last bit except where the summation order moves the statistic by an fp32 ulp."""
    x = _half((256, 5120), 3, dtype, scale=1.7)
    w = (1.0 + 0.2 * torch.randn(5120, generator=torch.Generator().manual_seed(4))).float()
    mine = pr.rmsnorm_ref(x, w, 1e-6)
    lib = F.rms_norm(x, (5120,), w, 1e-6).type_as(x)
    assert mine.dtype == x.dtype and mine.shape == x.shape
    diff = mine != lib
    assert diff.float().mean() < 1e-4
    ulp = 2.0**-7 if dtype == torch.bfloat16 else 2.0**-10  # spacing relative to the value, at most
    assert ((mine.float() - lib.float()).abs() <= 1.01 * ulp * lib.float().abs().clamp(min=1e-3)).all()
    exact = x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True) + 1e-6) * w.double()
    assert ((mine.double() - exact).abs() <= 0.51 * ulp * exact.abs().clamp(min=2.0**-14) + 1e-7).all()


def test_inv_rms_is_the_references_rsqrt():
    """ops.py:66 calls torch.rsqrt: on the CPU that is 1/sqrt with both steps correctly rounded, which is how the
    oracle (and the kernel) compute it."""
    x = _half((512, 1536), 21, scale=0.8)
    ms = pr.mean_square_ref(x)
    want = torch.rsqrt(ms + torch.tensor(1e-6, dtype=torch.float32))
    assert torch.equal(pr.inv_rms_ref(x, 1e-6), want)
    exact = 1.0 / torch.sqrt(ms.double() + float(torch.tensor(1e-6, dtype=torch.float32)))
    assert ((want.double() - exact).abs() / exact).max() < 1.2e-7


def test_rmsnorm_invariants():
    x = _half((8, 1536), 9)
    w = torch.ones(1536)
    y = pr.rmsnorm_ref(x, w, 0.0)
    # unit weight, zero eps: the output row has mean square 1 (up to the bf16 rounding of each element)
    assert ((y.double().pow(2).mean(-1) - 1.0).abs() < 5e-3).all()
    # scaling the input by a power of two changes nothing when eps is zero
    assert torch.equal(pr.rmsnorm_ref((x.float() * 4).to(torch.bfloat16), w, 0.0), y)
    # the weight multiplies after the normalisation, channel by channel
    w2 = torch.full((1536,), 2.0)
    assert torch.equal(pr.rmsnorm_ref(x, w2, 0.0).float(), 2.0 * y.float())
    # eps dominates a zero row: zeros stay zeros, no NaN
    z = torch.zeros(1, 1536, dtype=torch.bfloat16)
    assert (pr.rmsnorm_ref(z, w, 1e-6) == 0).all()


# ------------------------------------------------------------------ RoPE
def test_rope_table_values():
    t = pr.wan_rope_table(128)
    assert t.shape == (1024, 64) and t.dtype == torch.complex128
    assert pr.rope_split_sizes(64) == [22, 21, 21]
    # position 0 never turns; column 0 of each axis turns by one radian per step (theta^0 == 1)
    assert torch.equal(t[0], torch.ones(64, dtype=torch.complex128))
    for col in (0, 22, 43):
        assert abs(t[5, col].real.item() - math.cos(5.0)) < 1e-12 and abs(t[5, col].imag.item() - math.sin(5.0)) < 1e-12
    # the slowest pair of the frame axis: theta^(-(2*21)/44)
    ang = 7.0 * 10000.0 ** (-42.0 / 44.0)
    assert abs(t[7, 21].real.item() - math.cos(ang)) < 1e-12 and abs(t[7, 21].imag.item() - math.sin(ang)) < 1e-12


def _rope_real_arithmetic(x, grid, table):
    """Independent form: explicit cos/sin per (position, pair) in float64, python loops over positions."""
    B, L, H, D = x.shape
    out = x.clone()
    for b, (f, h, w) in enumerate(grid):
        for pos in range(f * h * w):
            fi, hi, wi = pos // (h * w), (pos // w) % h, pos % w
            for i in range(D // 2):
                row = fi if i < 22 else (hi if i < 43 else wi)
                c, s = table[row, i].real.item(), table[row, i].imag.item()
                a = x[b, pos, :, 2 * i].double()
                bb = x[b, pos, :, 2 * i + 1].double()
                out[b, pos, :, 2 * i] = (a * c - bb * s).float().to(x.dtype)
                out[b, pos, :, 2 * i + 1] = (a * s + bb * c).float().to(x.dtype)
    return out


def test_rope_matches_independent_real_form_and_invariants():
    table = pr.wan_rope_table(128)
    grid = [(2, 3, 4), (1, 2, 5)]
    x = _half((2, 30, 2, 128), 12)
    y = pr.rope_ref(x, grid, table)
    assert y.shape == x.shape and y.dtype == x.dtype
    assert torch.equal(y, _rope_real_arithmetic(x, grid, table))
    # rows at or beyond F*H*W pass through untouched (rope.py:124-125)
    assert torch.equal(y[0, 24:], x[0, 24:]) and torch.equal(y[1, 10:], x[1, 10:])
    # position 0 is the identity, every rotation keeps the pair's length (to bf16 rounding)
    assert torch.equal(y[:, 0], x[:, 0])
    n_in = x.double().reshape(2, 30, 2, 64, 2).norm(dim=-1)
    n_out = y.double().reshape(2, 30, 2, 64, 2).norm(dim=-1)
    assert ((n_in - n_out).abs() <= 2.0**-7 * n_in + 1e-6).all()
    # a pair on the frame axis at frame f, column j is turned by f * theta_j: check one by hand
    f_idx, j = 1, 3
    pos = f_idx * 12  # grid (2,3,4): frame 1 starts at position 12
    ang = f_idx * 10000.0 ** (-2.0 * j / 44.0)
    a, b = x[0, pos, 0, 2 * j].double().item(), x[0, pos, 0, 2 * j + 1].double().item()
    want = torch.tensor([a * math.cos(ang) - b * math.sin(ang), a * math.sin(ang) + b * math.cos(ang)]).float().to(torch.bfloat16)
    assert torch.equal(y[0, pos, 0, 2 * j : 2 * j + 2], want)
    # the dot product of a rotated q and k depends on the positions only through their difference
    q = _half((1, 24, 1, 128), 13).float()
    qq = pr.rope_ref(q.double(), [(2, 3, 4)], table)
    s1 = (qq[0, 5, 0] * qq[0, 9, 0]).sum()
    shifted = torch.roll(q, shifts=1, dims=1)  # same vectors one position later along the column axis
    ss = pr.rope_ref(shifted.double(), [(2, 3, 4)], table)
    # positions 5 -> 6 and 9 -> 10 stay in their rows (w = 1 -> 2, 1 -> 2): the difference vector is unchanged
    s2 = (ss[0, 6, 0] * ss[0, 10, 0]).sum()
    assert abs(s1.item() - s2.item()) < 1e-9


def test_wan_prep_composes_norm_then_rope():
    table = pr.wan_rope_table(128)
    x = _half((1, 12, 256), 14)
    w = (1.0 + 0.1 * torch.randn(256, generator=torch.Generator().manual_seed(15))).float()
    out = pr.wan_prep_ref(x, w, 1e-6, [(1, 3, 4)], table, num_heads=2)
    assert out.shape == (1, 12, 2, 128)
    assert torch.equal(out, pr.rope_ref(pr.rmsnorm_ref(x, w, 1e-6).view(1, 12, 2, 128), [(1, 3, 4)], table))
    assert torch.equal(pr.wan_prep_ref(x, None, 0.0, None, None, 2), x.view(1, 12, 2, 128))


# ----------------------------------------------------------------------------- the Qwen-Image block (qwen/attention.py:340-357)
def test_qwen_head_norm_against_scalar_replay_library_routine_and_float64():
    x = _half((1, 5, 3, 128), 21) * 2.0
    w = (1.0 + 0.2 * torch.randn(128, generator=torch.Generator().manual_seed(22))).float()
    got = pr.head_rmsnorm_ref(x, w, 1e-6)
    assert got.shape == x.shape and got.dtype == x.dtype
    # scalar replay of the frozen order: 8 accumulators x 16 channels in order, adjacent-pair tree
    ms = pr.head_mean_square_ref(x)
    f32 = lambda v: torch.tensor(v, dtype=torch.float32)
    for t in range(5):
        for h in range(3):
            accs = []
            for c in range(8):
                a = None
                for e in range(16):
                    v = x[0, t, h, 16 * c + e].float()
                    a = v * v if a is None else a + v * v
                accs.append(a)
            while len(accs) > 1:
                accs = [accs[2 * i] + accs[2 * i + 1] for i in range(len(accs) // 2)]
            assert ms[0, t, h] == accs[0] / f32(128.0)
    # the library routine behind torch.nn.RMSNorm (another summation order): equal except for rare last-place flips
    lib = torch.nn.functional.rms_norm(x.float(), (128,), w, 1e-6).type_as(x)
    assert (got != lib).float().mean() <= 1e-3
    assert (got.float() - lib.float()).abs().max() <= 2.0**-7 * lib.float().abs().max()
    # float64 brute force
    xd = x.double()
    want = xd / torch.sqrt((xd * xd).mean(dim=-1, keepdim=True) + 1e-6) * w.double()
    assert (got.double() - want).abs().max() <= 2.0**-8 * want.abs().max() + 1e-6


def test_qwen_rope_is_torchs_complex64_product_and_a_rotation():
    x = _half((2, 40, 3, 128), 23) * 1.5
    table = pr.qwen_rope_table(64, offset=-7)  # negative positions occur in the model's tables too (scale_rope)
    y = pr.qwen_rope_ref(x, table)
    # the reference's own expression (qwen/attention.py:37,57-59)
    xr = torch.view_as_complex(x.float().reshape(*x.shape[:-1], -1, 2))
    want = torch.view_as_real(xr * table[:40].unsqueeze(1)).flatten(3).type_as(x)
    assert torch.equal(y, want)
    # a rotation: pair lengths survive (to bf16 rounding); the row with angle 0 is the identity
    n_in = x.double().reshape(2, 40, 3, 64, 2).norm(dim=-1)
    n_out = y.double().reshape(2, 40, 3, 64, 2).norm(dim=-1)
    assert ((n_in - n_out).abs() <= 2.0**-7 * n_in + 1e-6).all()
    assert torch.equal(y[:, 7], x[:, 7])  # position -7 + 7 = 0
    # one pair by hand: axis 0 has dim 16, pair j turns by pos * theta^(-2j/16)
    pos, j = 5, 3
    ang = (pos - 7) * 10000.0 ** (-2.0 * j / 16.0)
    a, b = x[1, pos, 2, 2 * j].double().item(), x[1, pos, 2, 2 * j + 1].double().item()
    hand = torch.tensor([a * math.cos(ang) - b * math.sin(ang), a * math.sin(ang) + b * math.cos(ang)])
    assert (y[1, pos, 2, 2 * j : 2 * j + 2].double() - hand).abs().max() <= 2.0**-7 * hand.abs().max() + 1e-6


def test_qwen_prep_composes_the_two_streams():
    g = torch.Generator().manual_seed(24)
    x = _half((1, 30, 2, 128), 25)
    w_img, w_txt = (1.0 + 0.1 * torch.randn(128, generator=g)).float(), (1.0 + 0.1 * torch.randn(128, generator=g)).float()
    f_img, f_txt = pr.qwen_rope_table(20), pr.qwen_rope_table(10, offset=100)
    out = pr.qwen_prep_ref(x, 10, w_img, w_txt, 1e-6, f_img, f_txt)
    txt = pr.qwen_rope_ref(pr.head_rmsnorm_ref(x[:, :10], w_txt, 1e-6), f_txt)
    img = pr.qwen_rope_ref(pr.head_rmsnorm_ref(x[:, 10:], w_img, 1e-6), f_img)
    assert torch.equal(out, torch.cat([txt, img], dim=1))
    assert torch.equal(pr.qwen_prep_ref(x, 10, None, None, 0.0, None, None), x)
    assert torch.equal(pr.qwen_prep_ref(x, 0, w_img, None, 1e-6, None, None), pr.head_rmsnorm_ref(x, w_img, 1e-6))


# ----------------------------------------------------------------------------- the ComfyUI form of the Wan rotation (utils/rope.py:151-212)
def _comfy_ids(f, h, w):
    ids = torch.zeros(f, h, w, 3)
    ids[..., 0] += torch.arange(f).view(f, 1, 1)
    ids[..., 1] += torch.arange(h).view(1, h, 1)
    ids[..., 2] += torch.arange(w).view(1, 1, w)
    return ids.reshape(-1, 3)


@pytest.mark.parametrize("L,dtype", [(1, torch.bfloat16), (37, torch.bfloat16), (64, torch.float16), (100, torch.bfloat16)])
def test_comfy_rope_is_torchs_mul_then_addcmul(L, dtype):
    g = torch.Generator().manual_seed(L)
    x = (2.0 * torch.randn((2, L, 3, 128), generator=g)).to(dtype)
    m = pr.comfy_rope_matrices(_comfy_ids(5, 4, 5)[:L] * 7.0)  # [L, 64, 2, 2]
    # the reference's own two calls (rope.py:209-212) on its broadcast layout [1, L, 1, D/2, 2, 2]
    freqs_cis = m[None, :, None]
    x_ = x.to(dtype=freqs_cis.dtype).reshape(*x.shape[:-1], -1, 1, 2)
    want = freqs_cis[..., 0] * x_[..., 0]
    want.addcmul_(freqs_cis[..., 1], x_[..., 1])
    want = want.reshape(*x.shape).type_as(x)
    assert torch.equal(pr.comfy_rope_ref(x, m), want)


def test_comfy_rope_agrees_with_the_default_rotation_and_pads_with_identity():
    f, h, w = 3, 4, 5
    n = f * h * w
    x = _half((1, n + 6, 2, 128), 31)
    m = pr.comfy_rope_matrices(_comfy_ids(f, h, w))
    y = pr.comfy_rope_ref(x, m)
    assert torch.equal(y[:, n:], x[:, n:])  # past the table: identity (rope.py:133-148)
    # same angles as the complex128 table of the default path (44/42/42 channels per axis = 22/21/21 pairs), so
    # the two rotations agree to fp32-angle accuracy, well inside a bf16 step for these small positions
    ref = pr.rope_ref(x, [(f, h, w)], pr.wan_rope_table(128))
    assert (y.float() - ref.float()).abs().max() <= 2.0**-7 * ref.float().abs().max()
    assert (y != ref).float().mean() <= 0.02
    # a rotation: pair norms survive; position (0, 0, 0) is the identity
    n_in = x.double().reshape(1, n + 6, 2, 64, 2).norm(dim=-1)
    n_out = y.double().reshape(1, n + 6, 2, 64, 2).norm(dim=-1)
    assert ((n_in - n_out).abs() <= 2.0**-7 * n_in + 1e-6).all()
    assert torch.equal(y[:, 0], x[:, 0])
