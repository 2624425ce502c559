"""Pins the CPU oracle itself (no GPU): every oracle function is checked against something that
is NOT a retyping of its own formula - a float64 brute force, a scalar pure-Python second
implementation that replays the specified order element by element, hand-computed blocks, the
fp8 format definition, and invariants the mathematics fixes."""

import math

from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import quant_ref as qr
from oracle.sage_emul_ref import sage_emul_from_quant, sage_emul_ref
from oracle.sdpa_ref import attention_bruteforce_f64, sdpa_ref, sdpa_ref_fp32

f32 = np.float32


def _rand(shape, seed, dtype=torch.bfloat16, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)


# ------------------------------------------------------------------ sdpa_ref
@pytest.mark.parametrize("B,Lq,Lk,H,Hkv,D", [(1, 17, 17, 2, 2, 16), (2, 33, 20, 4, 2, 32), (1, 8, 50, 3, 3, 128)])
def test_sdpa_ref_matches_f64_bruteforce(B, Lq, Lk, H, Hkv, D):
    q, k, v = _rand((B, Lq, H, D), 1, torch.float32), _rand((B, Lk, Hkv, D), 2, torch.float32), _rand((B, Lk, Hkv, D), 3, torch.float32)
    ref = attention_bruteforce_f64(q, k, v)
    out = sdpa_ref(q, k, v)
    assert out.shape == q.shape
    torch.testing.assert_close(out.double(), ref, rtol=1e-5, atol=1e-5)
    out_scaled = sdpa_ref(q, k, v, scale=0.3)
    torch.testing.assert_close(out_scaled.double(), attention_bruteforce_f64(q, k, v, scale=0.3), rtol=1e-5, atol=1e-5)


def test_sdpa_ref_causal_and_half():
    q, k, v = (_rand((1, 24, 2, 32), s, torch.float32) for s in (4, 5, 6))
    torch.testing.assert_close(sdpa_ref(q, k, v, causal=True).double(), attention_bruteforce_f64(q, k, v, causal=True), rtol=1e-5, atol=1e-5)
    qb, kb, vb = (t.to(torch.bfloat16) for t in (q, k, v))
    out = sdpa_ref(qb, kb, vb)
    assert out.dtype == torch.bfloat16
    assert (out.double() - attention_bruteforce_f64(qb, kb, vb)).abs().max() < 2e-2
    torch.testing.assert_close(sdpa_ref_fp32(qb, kb, vb).double(), attention_bruteforce_f64(qb, kb, vb), rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------ K mean
def _scalar_mean_sum(col):
    """Replay rule 1 for ONE column with numpy float32 scalars."""
    L = len(col)
    nch = (L + qr.MEAN_CHUNK - 1) // qr.MEAN_CHUNK
    tot = None
    for c in range(nch):
        slots = []
        for s in range(qr.MEAN_SLOTS):
            acc = None
            for i in range(qr.MEAN_CHUNK // qr.MEAN_SLOTS):
                r = c * qr.MEAN_CHUNK + i * qr.MEAN_SLOTS + s
                x = f32(col[r]) if r < L else f32(0.0)
                acc = x if acc is None else f32(acc + x)
            slots.append(acc)
        while len(slots) > 1:
            slots = [f32(slots[i] + slots[i + 1]) for i in range(0, len(slots), 2)]
        tot = slots[0] if tot is None else f32(tot + slots[0])
    return tot


@pytest.mark.parametrize("L", [1, 31, 256, 257, 700])
def test_k_mean_matches_scalar_replay(L):
    k = _rand((1, L, 2, 4), 10 + L, std=3.0) + 5.0
    tot = qr.k_mean_sum_ref(k)
    km = qr.k_mean_ref(k)
    for h in range(2):
        for d in range(4):
            col = k[0, :, h, d].float().numpy()
            s = _scalar_mean_sum(col)
            assert tot[0, h, d].item() == float(s), (h, d)
            mean = f32(s / f32(L))
            expect = torch.tensor(float(mean)).to(torch.bfloat16)
            assert km[0, h, d].item() == expect.item()


def test_k_mean_close_to_f64_and_constant_columns():
    k = _rand((2, 5000, 3, 8), 77, std=2.0) + 3.0
    km = qr.k_mean_ref(k).double()
    exact = k.double().mean(dim=1)
    assert (km - exact).abs().max() <= exact.abs().max() * 2**-8  # one bf16 rounding
    tot = qr.k_mean_sum_ref(k).double()
    assert ((tot - k.double().sum(dim=1)).abs() / k.double().abs().sum(dim=1)).max() < 1e-6
    const = torch.full((1, 777, 1, 4), 1.5, dtype=torch.bfloat16)
    assert torch.equal(qr.k_mean_ref(const), torch.full((1, 1, 4), 1.5, dtype=torch.bfloat16))
    assert qr.k_mean_ref(k.to(torch.float16)).dtype == torch.float16


# ------------------------------------------------------------------ int8 block quantizer
def _scalar_block_int8(x2d, blk):
    """Independent scalar implementation of rule 5 on a [L, D] float32 numpy array."""
    L, D = x2d.shape
    nb = (L + blk - 1) // blk
    out = np.zeros((L, D), dtype=np.int8)
    scales = np.zeros(nb, dtype=np.float32)
    for b in range(nb):
        rows = range(b * blk, min(L, (b + 1) * blk))
        amax = f32(0.0)
        for r in rows:
            for d in range(D):
                a = f32(abs(x2d[r, d]))
                if a > amax:
                    amax = a
        if amax == 0:
            continue
        scales[b] = f32(amax / f32(127.0))
        inv = f32(f32(127.0) / amax)
        for r in rows:
            for d in range(D):
                # the exact product (rationals), rounded once, half to even (Python's round of a Fraction)
                n = round(Fraction(float(x2d[r, d])) * Fraction(float(inv)))
                assert -127 <= n <= 127  # |x| <= amax and inv = fl(127 / amax): never beyond 127 (1 + 2^-24)
                out[r, d] = n
    return out, scales


# ------------------------------------------------------------------ Walsh-Hadamard stage
def _sylvester(n):
    return np.array([[(-1) ** bin(i & j).count("1") for j in range(n)] for i in range(n)], dtype=np.float64)


def _scalar_fwht(row):
    """Replay rule 3 on one row with float32 scalars: strides 1, 2, 4, ... in that order."""
    x = [f32(v) for v in row]
    n, s = len(x), 1
    while s < n:
        for base in range(0, n, 2 * s):
            for i in range(base, base + s):
                a, b = x[i], x[i + s]
                x[i], x[i + s] = f32(a + b), f32(a - b)
        s *= 2
    return np.array(x, dtype=np.float32)


def test_fwht_is_the_hadamard_matrix_in_natural_order():
    g = torch.Generator().manual_seed(8)
    xi = torch.randint(-50, 50, (5, 128), generator=g).float()  # integers: every butterfly is exact
    assert np.array_equal(qr.fwht_ref(xi).double().numpy(), xi.double().numpy() @ _sylvester(128))
    x = _rand((3, 7, 128), 12, torch.float32, std=3.0)
    y = qr.fwht_ref(x)
    np.testing.assert_allclose(y.double().numpy(), x.double().numpy() @ _sylvester(128), rtol=0, atol=2e-4)
    for r in range(3):
        assert np.array_equal(y[0, r].numpy(), _scalar_fwht(x[0, r].numpy()))
    # orthogonal up to the factor D: dot products are preserved, applying it twice gives D * x
    a, b = _rand((128,), 1, torch.float32), _rand((128,), 2, torch.float32)
    assert abs(float(qr.fwht_ref(a) @ qr.fwht_ref(b)) / 128 - float(a @ b)) < 1e-4
    torch.testing.assert_close(qr.fwht_ref(qr.fwht_ref(x)) / 128, x, rtol=1e-5, atol=1e-5)
    # a lone outlier is spread evenly: |y| == |x_d| on every channel
    e = torch.zeros(128)
    e[37] = 20.0
    assert (qr.fwht_ref(e).abs() == 20.0).all()


# ------------------------------------------------------------------ int8 block quantizer
@pytest.mark.parametrize("L", [5, 128, 130])
def test_quant_q_matches_scalar_implementation(L):
    D, sm = 8, 8**-0.5
    q = _rand((1, L, 2, D), 20 + L, std=2.0)
    qi, qs = qr.quant_q_ref(q, sm)
    assert qi.shape == (1, 2, L, D) and qs.shape == (1, 2, L)  # one scale per query row
    c = f32(f32(f32(sm) * f32(qr.LOG2E)) * f32(1.0 / D))
    assert float(c) == qr.q_premul(sm, D).item()
    for h in range(2):
        rows = q[0, :, h].float().numpy()
        x = np.stack([_scalar_fwht(r) * c for r in rows]).astype(np.float32)
        ei, es = _scalar_block_int8(x, 1)
        assert np.array_equal(qi[0, h].numpy(), ei)
        assert np.array_equal(qs[0, h].numpy(), es)


@pytest.mark.parametrize("L", [3, 64, 65, 200])
def test_quant_k_matches_scalar_implementation(L):
    D = 8
    k = _rand((1, L, 2, D), 30 + L, std=1.0) + _rand((1, 1, 2, D), 99, std=2.0)
    ki, ks, km = qr.quant_k_ref(k)
    assert torch.equal(km, qr.k_mean_ref(k))
    for h in range(2):
        sm = (k[0, :, h].float().numpy() - km[0, h].float().numpy()[None, :]).astype(np.float32)
        x = np.stack([_scalar_fwht(r) for r in sm])
        ei, es = _scalar_block_int8(x, qr.BLKK)
        assert np.array_equal(ki[0, h].numpy(), ei)
        assert np.array_equal(ks[0, h].numpy(), es)
    ki0, ks0, km0 = qr.quant_k_ref(k, smooth_k=False)
    assert torch.count_nonzero(km0) == 0
    ei, es = _scalar_block_int8(np.stack([_scalar_fwht(r) for r in k[0, :, 0].float().numpy()]), qr.BLKK)
    assert np.array_equal(ki0[0, 0].numpy(), ei)


def test_quant_hand_computed_blocks():
    D = 4  # H4 rows: [1,1,1,1], [1,-1,1,-1], [1,1,-1,-1], [1,-1,-1,1]
    # a row of equal values v transforms to (4v, 0, 0, 0): one entry 127, scale 4v/127
    x = torch.full((1, 64, 1, D), 2.0, dtype=torch.bfloat16)
    xi, xs, _ = qr.quant_k_ref(x, smooth_k=False)
    assert (xi[..., 0] == 127).all() and (xi[..., 1:] == 0).all() and xs.item() == float(f32(8.0) / f32(127.0))
    # smoothing removes a constant column entirely -> zero block: zeros and scale 0
    xi, xs, km = qr.quant_k_ref(x, smooth_k=True)
    assert (xi == 0).all() and xs.item() == 0.0 and (km == 2.0).all()
    # exact ties after the transform.  rows (a,b,c,d) -> (a+b+c+d, a-b+c-d, a+b-c-d, a-b-c+d)
    # (64, 63, 0, 0) -> (127, 1, 127, 1); (1, 0.5, 0, 0) -> (1.5, 0.5, 1.5, 0.5); (-2, -0.5, 0, 0) -> (-2.5,-1.5,-2.5,-1.5)
    x = torch.tensor([[64.0, 63.0, 0, 0], [1.0, 0.5, 0, 0], [-2.0, -0.5, 0, 0]], dtype=torch.bfloat16).view(1, 3, 1, 4)
    xi, xs, _ = qr.quant_k_ref(x, smooth_k=False)
    assert xs.item() == 1.0  # amax 127 -> inv 1: values are rounded as they stand, half to even
    assert xi[0, 0].tolist() == [[127, 1, 127, 1], [2, 0, 2, 0], [-2, -2, -2, -2]]
    # a x20 outlier entry no longer dictates the step of its block: it is spread over the channels
    x = torch.ones((1, 128, 1, D), dtype=torch.bfloat16)
    x[0, 3, 0, 1] = -20.0
    xi, xs, _ = qr.quant_k_ref(x, smooth_k=False)
    # row 3 = (1,-20,1,1) -> (-17, 21, -21, 21); other rows -> (4,0,0,0); block amax 21
    inv = f32(f32(127.0) / f32(21.0))
    assert xi[0, 0, 3].tolist() == [round(Fraction(v) * Fraction(float(inv))) for v in (-17, 21, -21, 21)]
    assert xi[0, 0, 0].tolist() == [round(Fraction(4) * Fraction(float(inv))), 0, 0, 0]
    assert xs[0, 0].tolist() == [float(f32(21.0) / f32(127.0)), float(f32(4.0) / f32(127.0))]
    # ragged tail: last block's scale comes from its valid rows only
    x = torch.ones((1, 70, 1, D), dtype=torch.bfloat16)
    x[0, 64:, 0, :] = 0.25
    xi, xs, _ = qr.quant_k_ref(x, smooth_k=False)
    assert xs.shape == (1, 1, 2) and (xi[0, 0, 64:, 0] == 127).all() and xs[0, 0, 1].item() == float(f32(1.0) / f32(127.0))
    # Q: one scale per row, carries sm_scale * log2(e) / D
    q = torch.tensor([[3.0, 3.0, 3.0, 3.0], [0.0, 0.0, 0.0, 0.0], [1.0, 0.0, 0.0, 0.0]], dtype=torch.bfloat16).view(1, 3, 1, 4)
    qi, qs = qr.quant_q_ref(q, 0.25)
    c = f32(f32(f32(0.25) * f32(qr.LOG2E)) * f32(0.25))
    assert qs[0, 0].tolist() == [float(f32(f32(12.0) * c) / f32(127.0)), 0.0, float(f32(f32(1.0) * c) / f32(127.0))]
    assert qi[0, 0].tolist() == [[127, 0, 0, 0], [0, 0, 0, 0], [127, 127, 127, 127]]


def test_quant_invariants_on_workload_like_data():
    g = torch.Generator().manual_seed(5)
    k = torch.randn((1, 1000, 2, 128), generator=g) + 2.0 * torch.randn((1, 1, 2, 128), generator=g)
    mask = torch.rand(k.shape, generator=g) < 1e-3
    k = torch.where(mask, k * 20, k).to(torch.bfloat16)
    ki, ks, km = qr.quant_k_ref(k)
    x = qr.fwht_ref(k.permute(0, 2, 1, 3).float() - km.float()[:, :, None])
    s_row = ks.repeat_interleave(qr.BLKK, dim=2)[:, :, :1000, None]
    err = (x - ki.float() * s_row).abs()
    assert (err <= s_row * 0.5 * (1 + 1e-5)).all()
    blocks = torch.cat([ki, ki.new_zeros(1, 2, 24, 128)], 2).view(1, 2, 16, -1)
    assert (blocks.abs().amax(-1) == 127).all()
    qi, qs = qr.quant_q_ref(k, 128**-0.5)
    assert (qi.abs().amax(-1) == 127).all() and qs.shape == (1, 2, 1000)
    # the int8 dot products reproduce q.(k - km) * sm_scale * log2(e)
    s_int = qi[0, 0].float() @ ki[0, 0].float().t()
    s = s_int * qs[0, 0][:, None] * s_row[0, 0, :, 0][None, :]
    exact = (k[0, :, 0].double() @ (k[0, :, 0].double() - km[0, 0].double()).t()) * (128**-0.5 * qr.LOG2E)
    assert (s.double() - exact).abs().max() < 0.02 * exact.abs().max()


# ------------------------------------------------------------------ fp8 V
def test_e4m3fn_cast_matches_format_definition():
    table = qr.e4m3fn_decode_table()
    codes = torch.arange(256, dtype=torch.uint8)
    decoded = codes.view(torch.float8_e4m3fn).double()
    finite = ~torch.isnan(table)
    assert torch.equal(decoded[finite], table[finite]) and torch.isnan(decoded[~finite]).all()
    assert table[finite].max() == 448.0 and table[1] == 2.0**-9
    # round trip of every finite code is exact, so the cast is the identity on the grid
    vals = table[finite].float()
    back = vals.to(torch.float8_e4m3fn).float()
    assert torch.equal(back, vals)
    # nearest-even between grid points: brute force against the table
    g = torch.Generator().manual_seed(3)
    x = (torch.rand(4000, generator=g) * 2 - 1) * 448.0
    x = torch.cat([x, x * 1e-2, x * 1e-4])
    got = x.to(torch.float8_e4m3fn).double()
    grid = table[finite]
    dist = (x.double()[:, None] - grid[None, :]).abs()
    best = dist.min(dim=1).values
    assert torch.allclose((got - x.double()).abs(), best, rtol=0, atol=0)


def test_quant_v_properties():
    v = _rand((1, 333, 2, 16), 44, std=1.5)
    v8, vs = qr.quant_v_ref(v)
    assert v8.dtype == torch.float8_e4m3fn and v8.shape == (1, 2, 333, 16) and vs.shape == (1, 2, 16)
    amax = v.float().abs().amax(dim=1)
    assert torch.equal(vs, amax / torch.full_like(amax, 448.0))
    assert (v8.float().abs().amax(dim=2) == 448.0).all()  # the channel max lands on +-448 exactly
    deq = v8.float() * vs[:, :, None, :]
    x = v.permute(0, 2, 1, 3).float()
    assert ((deq - x).abs() <= x.abs() * 2**-4 + vs[:, :, None, :] * 2**-9).all()  # 3 mantissa bits
    # scalar second implementation on one channel
    table = qr.e4m3fn_decode_table()
    grid = table[~torch.isnan(table)].numpy()
    col = v[0, :, 1, 5].float().numpy()
    a = f32(np.abs(col).max())
    inv = f32(f32(448.0) / a)
    for r in range(0, 333, 7):
        y = float(f32(col[r] * inv))
        y = max(-448.0, min(448.0, y))
        d = np.abs(grid - y)
        assert abs(float(v8[0, 1, r, 5].float()) - y) == d.min()
    z = torch.zeros((1, 5, 1, 4), dtype=torch.bfloat16)
    z8, zs = qr.quant_v_ref(z)
    assert (z8.float() == 0).all() and (zs == 0).all()


def test_quant_v_smoothing_centres_before_scaling_and_attention_adds_the_mean_back():
    """smooth_v: the channel mean is the K-mean function (pinned above) applied to V; the codes are those of the
    plain quantizer fed with the centred values; a constant added to a channel moves the attention output by that
    constant and nothing else, where without smoothing it costs the channel its resolution."""
    v = (_rand((2, 200, 2, 128), 71, std=1.0).float() + torch.linspace(-6, 6, 128)).to(torch.bfloat16)
    v8, vs, vm = qr.quant_v_ref(v, smooth_v=True)
    assert vm.dtype == v.dtype and torch.equal(vm, qr.k_mean_ref(v))
    centred = v.float() - vm.float()[:, None]  # [B, L, H, D], exact in fp32 here
    amax = centred.abs().amax(dim=1)
    assert torch.equal(vs, amax / torch.full_like(amax, 448.0))
    inv = torch.full_like(amax, 448.0) / amax
    want = (centred * inv[:, None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).permute(0, 2, 1, 3)
    assert torch.equal(v8.view(torch.uint8), want.contiguous().view(torch.uint8))
    assert (v8.float().abs().amax(dim=2) == 448.0).all()
    # dequantised + mean reproduces V to e4m3 precision of the DEVIATION, not of the value
    deq = v8.float() * vs[:, :, None, :] + vm.float()[:, :, None, :]
    x = v.permute(0, 2, 1, 3).float()
    dev = (x - vm.float()[:, :, None, :]).abs()
    assert ((deq - x).abs() <= dev * 2**-4 + vs[:, :, None, :] * 2**-9 + 1e-6).all()
    # plain call unchanged: two results, no centring
    plain8, plain_s = qr.quant_v_ref(v)
    assert torch.equal(plain_s, v.float().abs().amax(dim=1) / 448.0)
    # attention: offsetting V by a per-channel constant offsets O by it
    q, k = _rand((2, 200, 2, 128), 72), _rand((2, 200, 2, 128), 73)
    base = _rand((2, 200, 2, 128), 74)
    off = torch.linspace(-8, 8, 128)
    shifted = (base.float() + off).to(torch.bfloat16)
    ref = sdpa_ref(q.float(), k.float(), shifted.float())
    smooth = sage_emul_ref(q, k, shifted, smooth_v=True).float()
    plain = sage_emul_ref(q, k, shifted).float()
    err_s, err_p = (smooth - ref).abs().max().item(), (plain - ref).abs().max().item()
    assert err_s < 0.06 and err_p > 2 * err_s, (err_s, err_p)
    cs, cp = _cos(smooth - off, ref - off), _cos(plain - off, ref - off)
    assert cs > 0.99 and (1 - cp) > 4 * (1 - cs), (cs, cp)
    # V == const: the centred values are zero, the scale is zero, the output is the constant
    c = torch.full((1, 70, 1, 128), 3.0, dtype=torch.bfloat16)
    o = sage_emul_ref(_rand((1, 70, 1, 128), 75), _rand((1, 70, 1, 128), 76), c, smooth_v=True)
    assert (o.float() == 3.0).all()


def test_sdpa_ref_k_lens_equals_cutting_the_batch_entries():
    """flash_attn.py:131-139 builds batch b from key[b, :k_lens[b]]: the masked oracle must equal attention on the
    cut tensors, entry by entry (an independent formulation: slicing instead of masking)."""
    B, Lq, Lk, H, D = 3, 17, 40, 2, 16
    q, k, v = _rand((B, Lq, H, D), 11).float(), _rand((B, Lk, H, D), 12).float(), _rand((B, Lk, H, D), 13).float()
    lens = [40, 7, 0]
    out = sdpa_ref(q, k, v, k_lens=lens)
    for b, n in enumerate(lens):
        if n == 0:
            assert (out[b] == 0).all()
        else:
            cut = attention_bruteforce_f64(q[b : b + 1], k[b : b + 1, :n], v[b : b + 1, :n])
            assert (out[b : b + 1].double() - cut).abs().max() < 1e-5
    # lengths beyond Lk and below zero are clamped; GQA goes through the same mask
    assert torch.equal(sdpa_ref(q, k, v, k_lens=[99, 7, -4]), out)
    kk, vv = k[:, :, :1], v[:, :, :1]
    o_g = sdpa_ref(q, kk, vv, k_lens=lens)
    assert (o_g[1:2].double() - attention_bruteforce_f64(q[1:2], kk[1:2, :7], vv[1:2, :7])).abs().max() < 1e-5


def test_sdpa_ref_block_mask_equals_attention_over_the_allowed_keys():
    """mask_id of the reference's block-sparse call (radial_sage_attn.py:150-176): 128 query rows x 64 keys per
    entry.  Independent formulation: gather the allowed keys of each query block and run dense attention on them."""
    B, Lq, Lk, H, D = 2, 300, 200, 2, 16
    q, k, v = _rand((B, Lq, H, D), 31).float(), _rand((B, Lk, H, D), 32).float(), _rand((B, Lk, H, D), 33).float()
    g = torch.Generator().manual_seed(34)
    mask = torch.rand((B, H, 3, 4), generator=g) < 0.5
    mask[0, 0, 1] = False  # a query block that sees nothing
    out = sdpa_ref(q, k, v, block_mask=mask)
    for b in range(B):
        for h in range(H):
            for i in range(3):
                rows = slice(128 * i, min(128 * (i + 1), Lq))
                cols = torch.cat([torch.arange(64 * j, min(64 * (j + 1), Lk)) for j in range(4) if mask[b, h, i, j]]
                                 or [torch.zeros(0, dtype=torch.long)])
                if len(cols) == 0:
                    assert (out[b, rows, h] == 0).all()
                    continue
                want = attention_bruteforce_f64(q[b : b + 1, rows, h : h + 1], k[b : b + 1, cols, h : h + 1], v[b : b + 1, cols, h : h + 1])
                assert (out[b : b + 1, rows, h : h + 1].double() - want).abs().max() < 1e-5
    # all-ones mask is dense attention; a [nq, nk] mask broadcasts over batch and heads
    assert torch.allclose(sdpa_ref(q, k, v, block_mask=torch.ones(3, 4)), sdpa_ref(q, k, v), atol=1e-6)
    # with k_lens the two restrictions intersect
    both = sdpa_ref(q, k, v, block_mask=mask, k_lens=[70, 200])
    cut = sdpa_ref(q[:1], k[:1, :70], v[:1, :70], block_mask=mask[:1, :, :, :2])
    assert torch.allclose(both[:1], cut, atol=1e-6)


def test_sage_emul_block_mask_equals_emulating_the_allowed_tiles():
    """On the same quantized operands: walking only the allowed key tiles == emulating with the other tiles removed."""
    B, L, H, D = 1, 256, 1, 128
    q, k, v = _rand((B, L, H, D), 41), _rand((B, L, H, D), 42), _rand((B, L, H, D), 43)
    q_i8, q_s = qr.quant_q_ref(q, D**-0.5)
    k_i8, k_s, _ = qr.quant_k_ref(k)
    v_f8, v_s = qr.quant_v_ref(v)
    mask = torch.tensor([[1, 0, 1, 1], [0, 0, 1, 0]])
    out = sage_emul_from_quant(q_i8, q_s, k_i8, k_s, v_f8, v_s, torch.bfloat16, block_mask=mask)
    for i in range(2):
        tiles = [j for j in range(4) if mask[i, j]]
        cols = torch.cat([torch.arange(64 * j, 64 * (j + 1)) for j in tiles])
        rows = slice(128 * i, 128 * (i + 1))
        cut = sage_emul_from_quant(q_i8[:, :, rows], q_s[:, :, rows], k_i8[:, :, cols], k_s[:, :, tiles], v_f8[:, :, cols], v_s,
                                   torch.bfloat16)
        assert torch.equal(out[:, rows], cut)


def test_sage_emul_k_lens_equals_emulating_the_cut_operands():
    """On the SAME quantized operands, limiting the keys equals dropping the other keys' rows."""
    B, L, H, D = 2, 200, 1, 128
    q, k, v = _rand((B, L, H, D), 21), _rand((B, L, H, D), 22), _rand((B, L, H, D), 23)
    q_i8, q_s = qr.quant_q_ref(q, D**-0.5)
    k_i8, k_s, _ = qr.quant_k_ref(k)
    v_f8, v_s = qr.quant_v_ref(v)
    lens = [130, 64]
    out = sage_emul_from_quant(q_i8, q_s, k_i8, k_s, v_f8, v_s, torch.bfloat16, k_lens=lens)
    for b, n in enumerate(lens):
        cut = sage_emul_from_quant(q_i8[b : b + 1], q_s[b : b + 1], k_i8[b : b + 1, :, :n], k_s[b : b + 1, :, : (n + 63) // 64],
                                   v_f8[b : b + 1, :, :n], v_s[b : b + 1], torch.bfloat16)
        assert torch.equal(out[b : b + 1], cut)


def test_sdpa_ref_causal_with_k_lens_and_block_mask_row_by_row():
    """Causal masking on top of the other two restrictions.  Independent formulation: row i alone, attending to
    the keys it may see, gathered by hand."""
    B, L, H, D = 2, 150, 2, 16
    q, k, v = (_rand((B, L, H, D), s).float() for s in (51, 52, 53))
    lens = [150, 90]
    mask = torch.tensor([[0, 1, 1], [1, 1, 0]])  # [ceil(150/128), ceil(150/64)]: rows 0..63 see nothing
    plain = sdpa_ref(q, k, v, causal=True)
    with_len = sdpa_ref(q, k, v, causal=True, k_lens=lens)
    with_mask = sdpa_ref(q, k, v, causal=True, block_mask=mask)
    for b in range(B):
        for i in (0, 1, 63, 64, 65, 100, 127, 128, 149):
            row = slice(i, i + 1)
            want = attention_bruteforce_f64(q[b : b + 1, row], k[b : b + 1, : i + 1], v[b : b + 1, : i + 1])
            assert (plain[b : b + 1, row].double() - want).abs().max() < 1e-5
            n = min(i + 1, lens[b])
            want = attention_bruteforce_f64(q[b : b + 1, row], k[b : b + 1, :n], v[b : b + 1, :n])
            assert (with_len[b : b + 1, row].double() - want).abs().max() < 1e-5
            cols = torch.tensor([c for c in range(i + 1) if mask[i // 128, c // 64]], dtype=torch.long)
            if len(cols) == 0:
                assert (with_mask[b, i] == 0).all()
            else:
                want = attention_bruteforce_f64(q[b : b + 1, row], k[b : b + 1, cols], v[b : b + 1, cols])
                assert (with_mask[b : b + 1, row].double() - want).abs().max() < 1e-5
    assert (with_mask[:, :64] == 0).all() and (with_mask[:, 64:] != 0).any()


def test_sage_emul_causal_equals_emulating_each_row_on_its_prefix():
    """On the same quantized operands: row i under causal masking == that row alone with the key count cut to
    i + 1 (the k_lens form, pinned above by cutting the operands)."""
    B, L, H, D = 1, 200, 1, 128
    q, k, v = _rand((B, L, H, D), 61), _rand((B, L, H, D), 62), _rand((B, L, H, D), 63)
    q_i8, q_s = qr.quant_q_ref(q, D**-0.5)
    k_i8, k_s, _ = qr.quant_k_ref(k)
    v_f8, v_s = qr.quant_v_ref(v)
    for exact in (True, False):
        out = sage_emul_from_quant(q_i8, q_s, k_i8, k_s, v_f8, v_s, torch.bfloat16, causal=True, exact_exp2=exact)
        for i in (0, 1, 31, 32, 63, 64, 65, 127, 128, 191, 192, 199):
            row = slice(i, i + 1)
            one = sage_emul_from_quant(q_i8[:, :, row], q_s[:, :, row], k_i8, k_s, v_f8, v_s, torch.bfloat16, k_lens=[i + 1],
                                       exact_exp2=exact)
            assert torch.equal(out[:, row], one), i
    # with a block mask the two restrictions intersect: rows 128.. lose tile 2 and with it their own position
    mask = torch.tensor([[1, 1, 1, 1], [1, 1, 0, 1]])
    both = sage_emul_from_quant(q_i8, q_s, k_i8, k_s, v_f8, v_s, torch.bfloat16, causal=True, block_mask=mask)
    ref = sage_emul_from_quant(q_i8, q_s, k_i8, k_s, v_f8, v_s, torch.bfloat16, causal=True)
    assert torch.equal(both[:, :128], ref[:, :128])
    cut = sage_emul_from_quant(q_i8[:, :, 128:192], q_s[:, :, 128:192], k_i8[:, :, :128], k_s[:, :, :2], v_f8[:, :, :128], v_s,
                               torch.bfloat16)
    assert torch.equal(both[:, 128:192], cut)  # rows 128..191: tiles 0 and 1 whole, tile 2 masked, tile 3 in the future
    assert _cos(sdpa_ref(q, k, v, causal=True), ref) > 0.999


def test_sage_emul_key_split_merges_runs_of_keys():
    """key_split: the query blocks from a given number on walk their keys in equal runs of tiles and merge.  Pinned
    by (a) one run == no split, bit for bit; (b) only the blocks from that number on change; (c) an independent
    merge: each run emulated alone on the cut operands, combined with the exact softmax mass of its keys from a
    float64 computation on the same quantized operands."""
    B, Lq, Lk, H, D = 1, 300, 1100, 2, 128
    q, k, v = _rand((B, Lq, H, D), 81), _rand((B, Lk, H, D), 82), _rand((B, Lk, H, D), 83)
    q_i8, q_s = qr.quant_q_ref(q, D**-0.5)
    k_i8, k_s, _ = qr.quant_k_ref(k)
    v_f8, v_s = qr.quant_v_ref(v)
    emul = lambda **kw: sage_emul_from_quant(q_i8, q_s, k_i8, k_s, v_f8, v_s, torch.bfloat16, **kw)  # noqa: E731
    plain = emul()
    assert torch.equal(emul(key_split=(0, 1)), plain)
    runs = 3
    cut = emul(key_split=(1, runs))  # blocks: head 0 -> 0, 1; head 1 -> 2, 3; block 0 stays whole
    assert torch.equal(cut[:, :256, 0], plain[:, :256, 0])
    assert not torch.equal(cut[:, 256:, 0], plain[:, 256:, 0]) and not torch.equal(cut[:, :, 1], plain[:, :, 1])
    assert _cos(cut, plain) > 0.9995  # same attention, P rounded relative to other maxima
    # independent merge for head 1: tiles 18 -> runs of 6 tiles = 384 keys
    per = 6 * 64
    s = (q_i8[0, 1].double() * q_s[0, 1].double()[:, None]) @ (k_i8[0, 1].double() * k_s[0, 1].double().repeat_interleave(64)[:Lk, None]).t()
    mass = torch.stack([torch.exp2(s[:, r * per : (r + 1) * per] - s.amax(dim=1, keepdim=True)).sum(dim=1) for r in range(runs)])
    weight = mass / mass.sum(dim=0, keepdim=True)  # [runs, Lq]
    want = torch.zeros(Lq, D, dtype=torch.float64)
    for r in range(runs):
        lo, hi = r * per, min(Lk, (r + 1) * per)
        alone = sage_emul_from_quant(q_i8[:, 1:2], q_s[:, 1:2], k_i8[:, 1:2, lo:hi], k_s[:, 1:2, lo // 64 : (hi + 63) // 64],
                                     v_f8[:, 1:2, lo:hi], v_s[:, 1:2], torch.float32)
        want += weight[r][:, None] * alone[0, :, 0].double()
    got = cut[0, :, 1].double()
    assert (got - want).abs().max() < 6e-3 * want.abs().max() + 2e-3  # bf16 output, row sums from rounded P
    # with per-batch key counts the runs are cut from the keys that count
    lens = [700]
    a = emul(key_split=(0, 2), k_lens=lens)
    b = sage_emul_from_quant(q_i8, q_s, k_i8[:, :, :700], k_s[:, :, :11], v_f8[:, :, :700], v_s, torch.bfloat16, key_split=(0, 2))
    assert torch.equal(a, b)


# ------------------------------------------------------------------ emulation of the fused kernel
def _cos(a, b):
    a, b = a.double().flatten(), b.double().flatten()
    return float((a @ b) / (a.norm() * b.norm()))


def test_sage_emul_close_to_sdpa_and_invariants():
    B, L, H, D = 1, 300, 2, 128
    q, v = _rand((B, L, H, D), 1), _rand((B, L, H, D), 3)
    k = (_rand((B, L, H, D), 2).float() + 2.0 * _rand((1, 1, H, D), 4).float()).to(torch.bfloat16)
    ref = sdpa_ref(q, k, v)
    out = sage_emul_ref(q, k, v)
    assert out.shape == ref.shape and out.dtype == ref.dtype
    # the scheme's own error is ~3.5 % rms of |O| (two e4m3 roundings per product): cos-sim clears
    # 0.999 at every length, while the ABSOLUTE error shrinks with |O| ~ 1/sqrt(L) - at L = 300 it
    # is still above the 2e-2 that holds from the shortest measured workload (L = 1560) on.
    assert _cos(out, ref) > 0.999 and (out.float() - ref.float()).abs().max() < 4e-2
    # smoothing matters: without it the same data is visibly worse, never better by much
    rough = sage_emul_ref(q, k, v, smooth_k=False)
    assert (rough.float() - ref.float()).abs().mean() > (out.float() - ref.float()).abs().mean()
    # rows of P sum to one: V == 1 gives O == 1 up to bf16/fp8 rounding of the normaliser
    ones = torch.ones_like(v)
    o1 = sage_emul_ref(q, k, ones).float()
    assert (o1 - 1.0).abs().max() < 0.04
    # permuting the keys inside a 64-key scale block permutes nothing in the output
    perm = torch.cat([torch.randperm(64, generator=torch.Generator().manual_seed(9)) + 64 * i for i in range(4)] + [torch.arange(256, 300)])
    o_perm = sage_emul_ref(q, k[:, perm], v[:, perm])
    assert (o_perm.float() - out.float()).abs().max() < 4e-2
    # GQA and rectangular shapes
    kk, vv = k[:, :100, :1], v[:, :100, :1]
    o_r = sage_emul_ref(q, kk, vv)
    assert _cos(o_r, sdpa_ref(q, kk, vv)) > 0.999


def test_sage_emul_meets_stated_tolerance_on_plumbing_workload():
    """cos-sim >= 0.999 and max-abs <= 2e-2 against the SDPA oracle on the CPU-plumbing workload
    (two of its 40 heads, full length 1560)."""
    from ksanadit_amd.workloads import make_inputs

    q, k, v = make_inputs("cpu_plumbing", heads=2)
    ref = sdpa_ref(q, k, v)
    out = sage_emul_ref(q, k, v)
    assert _cos(out, ref) >= 0.999
    assert (out.float() - ref.float()).abs().max() <= 2e-2
    # the piecewise-linear exp2 keeps the cosine bar; its worst element is ~2x further out
    fast = sage_emul_ref(q, k, v, exact_exp2=False)
    assert _cos(fast, ref) >= 0.999
    assert (fast.float() - ref.float()).abs().max() <= 4e-2


def test_sage_emul_survives_outliers():
    """0.1 % entries x20 in Q and K (the headline workload's distribution, shortened): the
    Hadamard stage plus per-token Q scales keep cos-sim >= 0.999."""
    from ksanadit_amd.workloads import make_inputs

    q, k, v = make_inputs("wan14b_480p", heads=1, seq=2048)
    ref, out = sdpa_ref(q, k, v), sage_emul_ref(q, k, v)
    assert _cos(out, ref) >= 0.999


def test_head_size_64_rows_extended_with_zeros_keep_the_products():
    """Rule 7: a 64-channel row extended with zeros transforms into the 64-point transform written twice, so the
    product of two transformed rows is still 128 times the product of the rows (exact on small integers), the extended
    K mean is zero there and the extended V channels quantize to zero codes with scale zero."""
    g = torch.Generator().manual_seed(64)
    q = torch.randint(-8, 9, (1, 5, 2, 64), generator=g).to(torch.bfloat16)
    k = torch.randint(-8, 9, (1, 7, 2, 64), generator=g).to(torch.bfloat16)
    qp, kp = qr.pad_head_dim(q), qr.pad_head_dim(k)
    assert qp.shape[-1] == 128 and torch.equal(qp[..., :64], q) and torch.count_nonzero(qp[..., 64:]) == 0
    hq, hk = qr.fwht_ref(qp.float()), qr.fwht_ref(kp.float())
    h64 = qr.fwht_ref(q.float())
    assert torch.equal(hq, torch.cat([h64, h64], dim=-1))
    exact = torch.einsum("blhd,bmhd->bhlm", q.double(), k.double())
    got = torch.einsum("blhd,bmhd->bhlm", hq.double(), hk.double())
    assert torch.equal(got, 128.0 * exact)
    _, _, km = qr.quant_k_ref(kp)
    assert torch.count_nonzero(km[..., 64:]) == 0
    v = torch.randn((1, 7, 2, 64), generator=g).to(torch.bfloat16)
    v8, vs = qr.quant_v_ref(qr.pad_head_dim(v))
    assert torch.count_nonzero(v8.view(torch.uint8)[..., 64:]) == 0 and torch.count_nonzero(vs[..., 64:]) == 0
    assert torch.equal(qr.pad_head_dim(qp), qp)
