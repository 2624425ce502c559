"""The quantizer with the block's RMSNorm + RoPE folded in (through the C ABI) against
oracle/prep_ref.py followed by oracle/quant_ref.py: every integer and every scale bit for bit."""

import pytest
import torch

from ksanadit_amd import sage_ops
from ksanadit_amd.layout import untile_k
from ksanadit_amd.sage_ops import QwenPrep, WanPrep
from oracle import prep_ref as pr
from oracle import quant_ref as qr
from oracle.sdpa_ref import sdpa_ref

pytestmark = pytest.mark.gpu


def _proj(B, L, H, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    x = 1.5 * torch.randn((B, L, H * 128), generator=g) + 0.7 * torch.randn((1, 1, H * 128), generator=g)
    w = 1.0 + 0.2 * torch.randn(H * 128, generator=g)
    return x.to(dtype), w.float()


def _check_q(ws, ref4d, sm_scale, Lq):
    q_i8, q_scale = qr.quant_q_ref(ref4d, sm_scale)
    assert torch.equal(ws.q_i8.cpu()[:, :, :Lq], q_i8)
    assert torch.equal(ws.q_scale.cpu()[:, :, :Lq], q_scale)


def _check_k(ws, ref4d, Lk):
    k_i8, k_scale, k_mean = qr.quant_k_ref(ref4d)
    assert torch.equal(ws.k_mean.cpu(), k_mean), "k_mean differs"
    assert torch.equal(ws.k_scale.cpu(), k_scale), "k_scale differs"
    assert torch.equal(untile_k(ws.k_tiles.cpu(), Lk), k_i8), "k_int8 differs"


@pytest.mark.parametrize(
    "B,L,H,grids,dtype,norm,rope",
    [
        (1, 24, 2, [(2, 3, 4)], torch.bfloat16, True, True),
        (1, 300, 12, [(3, 9, 11)], torch.bfloat16, True, True),      # 297 of 300 rows rotate, 3 pass through
        (2, 130, 3, [(2, 5, 13), (1, 7, 9)], torch.bfloat16, True, True),
        (1, 200, 40, [(2, 10, 10)], torch.bfloat16, True, True),     # the 14B row: 5120 channels
        (1, 96, 4, [(1, 8, 12)], torch.float16, True, True),
        (1, 96, 4, [(1, 8, 12)], torch.bfloat16, True, False),       # cross-attention: norm only
        (1, 96, 4, [(4, 4, 6)], torch.bfloat16, False, True),        # rotation only
    ],
)
def test_quantizer_with_prep_is_bit_exact(hip_device, B, L, H, grids, dtype, norm, rope):
    print(f"case B={B} L={L} H={H} grids={grids} dtype={dtype} norm={norm} rope={rope}", flush=True)
    qp, wq = _proj(B, L, H, seed=L + H, dtype=dtype)
    kp, wk = _proj(B, L, H, seed=L + H + 1, dtype=dtype)
    table = pr.wan_rope_table(128)
    prep = WanPrep(q_norm_weight=wq if norm else None, k_norm_weight=wk if norm else None, eps=1e-6,
                   freqs=table if rope else None, grid_sizes=grids if rope else None)
    q4 = qp.view(B, L, H, 128).to(hip_device)
    k4 = kp.view(B, L, H, 128).to(hip_device)
    ws = sage_ops.workspace_for(q4, k4)
    ws.blob.fill_(0x7F)
    sage_ops.quant_q(q4, ws, 128**-0.5, prep=prep)
    sage_ops.quant_k(k4, ws, prep=prep)
    torch.cuda.synchronize()
    if norm:
        assert torch.equal(ws.q_rms.cpu(), pr.inv_rms_ref(qp, 1e-6))
        assert torch.equal(ws.k_rms.cpu(), pr.inv_rms_ref(kp, 1e-6))
    q_ref = pr.wan_prep_ref(qp, wq if norm else None, 1e-6, grids, table if rope else None, H)
    k_ref = pr.wan_prep_ref(kp, wk if norm else None, 1e-6, grids, table if rope else None, H)
    _check_q(ws, q_ref, 128**-0.5, L)
    _check_k(ws, k_ref, L)


@pytest.mark.parametrize("kind", ["wan", "qwen"])
def test_prep_k_stays_exact_when_a_wait_runs_out(hip_device, kind, quant_settings):
    """K with the norm / rotation step folded in always takes the one-read kernel; a workgroup whose bounded wait
    runs out recomputes the head's mean from the input, norm and rotation included, in the specified order.  A
    negative bound sends every workgroup but a head's last arriver down that path whatever the timing."""
    quant_settings(wait_ticks=-1)
    if kind == "wan":
        B, L, H, grids = 1, 1500, 4, [(5, 10, 30)]
        kp, wk = _proj(B, L, H, seed=5)
        table = pr.wan_rope_table(128)
        prep = WanPrep(q_norm_weight=None, k_norm_weight=wk, eps=1e-6, freqs=table, grid_sizes=grids)
        k4 = kp.view(B, L, H, 128).to(hip_device)
        k_ref = pr.wan_prep_ref(kp, wk, 1e-6, grids, table, H)
    else:
        B, H, txt, img = 2, 3, 100, 1100
        L = txt + img
        g = torch.Generator().manual_seed(17)
        k = torch.randn((B, L, H, 128), generator=g).bfloat16()
        w_img = (1.0 + 0.1 * torch.randn(128, generator=g)).float()
        w_txt = (1.0 + 0.1 * torch.randn(128, generator=g)).float()
        f_img, f_txt = pr.qwen_rope_table(img, offset=-3), pr.qwen_rope_table(txt, offset=2000)
        prep = QwenPrep(txt_len=txt, eps=1e-6, k_norm_weight=w_img, k_norm_weight_txt=w_txt, img_freqs=f_img, txt_freqs=f_txt)
        k4 = k.to(hip_device)
        k_ref = pr.qwen_prep_ref(k, txt, w_img, w_txt, 1e-6, f_img, f_txt)
    ws = sage_ops.workspace_for(k4, k4)
    ws.blob.fill_(0x7F)
    sage_ops.quant_k(k4, ws, prep=prep)
    torch.cuda.synchronize()
    assert sage_ops.quant_status(ws)[0] == 1, "no workgroup took the recompute path"
    _check_k(ws, k_ref, L)
    assert not sage_ops.one_read_state()["demoted"], "a test-mode bound must not switch the one-read kernels off"


@pytest.mark.parametrize("Lq,Lk,Hq,Hkv,grids", [(300, 300, 12, 12, [(3, 9, 11)]), (200, 520, 4, 4, None), (520, 70, 8, 4, None),
                                                (1000, 1000, 40, 40, [(4, 10, 25)])])
def test_q_and_k_in_one_call_give_the_bits_of_two(hip_device, Lq, Lk, Hq, Hkv, grids):
    """``quant_qk``: q's whole-row kernel brings k's row statistic along (k longer than q, shorter, with fewer
    heads); every workspace area ends up as the two separate calls leave it."""
    B = 2 if grids is None else 1
    qp, wq = _proj(B, Lq, Hq, seed=Lq + Hq)
    kp, wk = _proj(B, Lk, Hkv, seed=Lk + Hkv + 1)
    table = pr.wan_rope_table(128)
    prep = WanPrep(q_norm_weight=wq, k_norm_weight=wk, eps=1e-6, freqs=table if grids else None, grid_sizes=grids)
    q4 = qp.view(B, Lq, Hq, 128).to(hip_device)
    k4 = kp.view(B, Lk, Hkv, 128).to(hip_device)
    two, one = sage_ops.workspace_for(q4, k4), sage_ops.workspace_for(q4, k4)
    two.blob.fill_(0x7F), one.blob.fill_(0x3C)
    sage_ops.quant_q(q4, two, 128**-0.5, prep=prep)
    sage_ops.quant_k(k4, two, prep=prep)
    sage_ops.quant_qk(q4, k4, one, 128**-0.5, prep=prep)
    torch.cuda.synchronize()
    assert sage_ops.quant_status(one)[0] == 0
    for area in ("q_rms", "k_rms", "q_i8", "q_scale", "k_tiles", "k_scale", "k_mean"):
        assert torch.equal(getattr(one, area).cpu(), getattr(two, area).cpu()), area
    assert torch.equal(one.k_rms.cpu(), pr.inv_rms_ref(kp, 1e-6))


def test_wan_block_path_equals_attention_on_prepared_tensors(hip_device):
    """norm + RoPE on the fly, then attention == attention fed with the oracle's normed and rotated q, k."""
    B, L, H = 1, 448, 6
    grids = [(2, 14, 16)]
    qp, wq = _proj(B, L, H, 1)
    kp, wk = _proj(B, L, H, 2)
    vp, _ = _proj(B, L, H, 3)
    table = pr.wan_rope_table(128)
    prep = WanPrep(wq, wk, 1e-6, table, grids)
    fused = sage_ops.wan_self_attention(qp.to(hip_device), kp.to(hip_device), vp.to(hip_device), H, prep).cpu()
    q_ref = pr.wan_prep_ref(qp, wq, 1e-6, grids, table, H)
    k_ref = pr.wan_prep_ref(kp, wk, 1e-6, grids, table, H)
    v4 = vp.view(B, L, H, 128)
    plain = sage_ops.sageattn(q_ref.to(hip_device), k_ref.to(hip_device), v4.to(hip_device)).cpu()
    assert torch.equal(fused, plain)
    ref = sdpa_ref(q_ref, k_ref, v4)
    a, b = fused.double().flatten(), ref.double().flatten()
    assert float((a @ b) / (a.norm() * b.norm())) >= 0.999


def test_prep_at_model_row_width_and_length(hip_device):
    """Wan-14B rows (40 heads) over 4096 tokens of a 4 x 32 x 32 grid: still every bit."""
    B, L, H = 1, 4096, 40
    grids = [(4, 32, 32)]
    qp, wq = _proj(B, L, H, 11)
    kp, wk = _proj(B, L, H, 12)
    table = pr.wan_rope_table(128)
    prep = WanPrep(wq, wk, 1e-6, table, grids)
    q4, k4 = qp.view(B, L, H, 128).to(hip_device), kp.view(B, L, H, 128).to(hip_device)
    ws = sage_ops.workspace_for(q4, k4)
    sage_ops.quant_q(q4, ws, 128**-0.5, prep=prep)
    sage_ops.quant_k(k4, ws, prep=prep)
    torch.cuda.synchronize()
    assert torch.equal(ws.q_rms.cpu(), pr.inv_rms_ref(qp, 1e-6))
    _check_q(ws, pr.wan_prep_ref(qp, wq, 1e-6, grids, table, H), 128**-0.5, L)
    _check_k(ws, pr.wan_prep_ref(kp, wk, 1e-6, grids, table, H), L)


def _comfy_matrices(f, h, w):
    ids = torch.zeros(f, h, w, 3)
    ids[..., 0] += torch.arange(f).view(f, 1, 1)
    ids[..., 1] += torch.arange(h).view(1, h, 1)
    ids[..., 2] += torch.arange(w).view(1, 1, w)
    return pr.comfy_rope_matrices(ids.reshape(-1, 3))


@pytest.mark.parametrize(
    "B,L,H,grid,dtype,norm",
    [
        (1, 24, 2, (2, 3, 4), torch.bfloat16, True),
        (2, 300, 12, (3, 9, 11), torch.bfloat16, True),     # 297 rows rotate, 3 pass through (identity padding)
        (1, 200, 40, (2, 10, 10), torch.bfloat16, True),    # the 14B row: 5120 channels
        (1, 96, 4, (1, 8, 12), torch.float16, True),
        (1, 96, 4, (4, 4, 6), torch.bfloat16, False),
    ],
)
def test_quantizer_with_comfy_rope_is_bit_exact(hip_device, B, L, H, grid, dtype, norm):
    """The Wan block with rope_func == "comfy" (wan_model.py:169-171, utils/rope.py:180-212): token-row RMSNorm, then
    the 2x2-matrix rotation, on the way into the quantizer."""
    print(f"case comfy B={B} L={L} H={H} grid={grid} {dtype} norm={norm}", flush=True)
    qp, wq = _proj(B, L, H, seed=L + H + 7, dtype=dtype)
    kp, wk = _proj(B, L, H, seed=L + H + 8, dtype=dtype)
    m = _comfy_matrices(*grid)
    # the module's layout, broadcast dims included (EmbedND.forward: [1, L_true, 1, D/2, 2, 2])
    prep = WanPrep(q_norm_weight=wq if norm else None, k_norm_weight=wk if norm else None, eps=1e-6,
                   comfy_freqs=m[None, :, None])
    q4 = qp.view(B, L, H, 128).to(hip_device)
    k4 = kp.view(B, L, H, 128).to(hip_device)
    ws = sage_ops.workspace_for(q4, k4)
    ws.blob.fill_(0x7F)
    sage_ops.quant_q(q4, ws, 128**-0.5, prep=prep)
    sage_ops.quant_k(k4, ws, prep=prep)
    torch.cuda.synchronize()
    assert sage_ops.quant_status(ws)[0] == 0
    _check_q(ws, pr.wan_comfy_prep_ref(qp, wq if norm else None, 1e-6, m, H), 128**-0.5, L)
    _check_k(ws, pr.wan_comfy_prep_ref(kp, wk if norm else None, 1e-6, m, H), L)
    with pytest.raises(ValueError, match="either"):
        WanPrep(comfy_freqs=m, freqs=pr.wan_rope_table(128), grid_sizes=[grid]).to_c(hip_device)
    with pytest.raises(ValueError, match="comfy_freqs must be"):
        WanPrep(comfy_freqs=m[:, :32]).to_c(hip_device)


@pytest.mark.parametrize(
    "B,txt,img,H,dtype,norm,rope",
    [
        (1, 7, 50, 2, torch.bfloat16, True, True),
        (2, 256, 4096, 4, torch.bfloat16, True, True),   # the Qwen-Image 1024 x 1024 joint sequence, CFG pair
        (2, 33, 300, 3, torch.float16, True, True),
        (1, 0, 130, 2, torch.bfloat16, True, True),      # no text rows at all
        (1, 64, 64, 2, torch.bfloat16, True, False),
        (1, 64, 64, 2, torch.bfloat16, False, True),
    ],
)
def test_quantizer_with_qwen_prep_is_bit_exact(hip_device, B, txt, img, H, dtype, norm, rope):
    """Per-head RMSNorm (text and image weights) + apply_rotary_emb_qwen on the way into the quantizer
    (qwen/attention.py:340-357) against the oracle's restatement followed by the plain quantizer oracle."""
    print(f"case qwen prep B={B} txt={txt} img={img} H={H} {dtype} norm={norm} rope={rope}", flush=True)
    L = txt + img
    g = torch.Generator().manual_seed(txt * 7 + img)
    q = (1.5 * torch.randn((B, L, H, 128), generator=g)).to(dtype)
    k = (1.5 * torch.randn((B, L, H, 128), generator=g) + 0.7 * torch.randn((1, 1, H, 128), generator=g)).to(dtype)
    q[:, :txt] *= 3.0  # text tokens of another scale, as in the measured workload
    w = [(1.0 + 0.2 * torch.randn(128, generator=g)).float() for _ in range(4)]
    f_img, f_txt = pr.qwen_rope_table(img + 5, offset=-3), pr.qwen_rope_table(max(txt, 1), offset=2000)
    prep = QwenPrep(txt_len=txt, q_norm_weight=w[0] if norm else None, k_norm_weight=w[1] if norm else None,
                    q_norm_weight_txt=w[2] if norm else None, k_norm_weight_txt=w[3] if norm else None, eps=1e-6,
                    img_freqs=f_img if rope else None, txt_freqs=f_txt if rope else None)
    qd, kd = q.to(hip_device), k.to(hip_device)
    ws = sage_ops.workspace_for(qd, kd)
    ws.blob.fill_(0x7F)
    sage_ops.quant_q(qd, ws, 128**-0.5, prep=prep)
    sage_ops.quant_k(kd, ws, prep=prep)
    torch.cuda.synchronize()
    assert sage_ops.quant_status(ws)[0] == 0
    q_ref = pr.qwen_prep_ref(q, txt, w[0] if norm else None, w[2] if norm else None, 1e-6, f_img if rope else None, f_txt if rope else None)
    k_ref = pr.qwen_prep_ref(k, txt, w[1] if norm else None, w[3] if norm else None, 1e-6, f_img if rope else None, f_txt if rope else None)
    _check_q(ws, q_ref, 128**-0.5, L)
    _check_k(ws, k_ref, L)


def test_qwen_block_path_equals_attention_on_prepared_tensors(hip_device):
    B, txt, img, H = 2, 40, 500, 3
    L = txt + img
    g = torch.Generator().manual_seed(99)
    q, k, v = ((1.5 * torch.randn((B, L, H, 128), generator=g)).to(torch.bfloat16) for _ in range(3))
    w = [(1.0 + 0.2 * torch.randn(128, generator=g)).float() for _ in range(4)]
    f_img, f_txt = pr.qwen_rope_table(img), pr.qwen_rope_table(txt, offset=3000)
    prep = QwenPrep(txt, w[0], w[1], w[2], w[3], 1e-6, f_img, f_txt)
    fused = sage_ops.sageattn(q.to(hip_device), k.to(hip_device), v.to(hip_device), prep=prep).cpu()
    q_ref = pr.qwen_prep_ref(q, txt, w[0], w[2], 1e-6, f_img, f_txt)
    k_ref = pr.qwen_prep_ref(k, txt, w[1], w[3], 1e-6, f_img, f_txt)
    plain = sage_ops.sageattn(q_ref.to(hip_device), k_ref.to(hip_device), v.to(hip_device)).cpu()
    assert torch.equal(fused, plain)
    a, b = fused.double().flatten(), sdpa_ref(q_ref, k_ref, v).double().flatten()
    assert float((a @ b) / (a.norm() * b.norm())) >= 0.999
    with pytest.raises(ValueError, match="rows"):
        sage_ops.sageattn(q.to(hip_device), k.to(hip_device), v.to(hip_device),
                          prep=QwenPrep(txt, w[0], w[1], w[2], w[3], 1e-6, f_img[:100], f_txt))


def test_prep_argument_errors(hip_device):
    qp, wq = _proj(1, 64, 2, 5)
    q4 = qp.view(1, 64, 2, 128).to(hip_device)
    ws = sage_ops.workspace_for(q4, q4)
    table = pr.wan_rope_table(128)
    with pytest.raises(ValueError, match="exceeds"):
        sage_ops.quant_q(q4, ws, 0.1, prep=WanPrep(wq, wq, 1e-6, table, [(2, 8, 8)]))  # 128 positions > 64 rows
    with pytest.raises(ValueError, match="outside"):
        sage_ops.quant_q(q4, ws, 0.1, prep=WanPrep(wq, wq, 1e-6, table[:4], [(8, 2, 2)]))  # frame 8 > 4 table rows
    with pytest.raises(ValueError, match="H stride"):
        wide = torch.zeros(1, 64, 2, 256, dtype=torch.bfloat16, device=hip_device)[..., :128]  # heads not adjacent
        sage_ops.quant_q(wide, ws, 0.1, prep=WanPrep(wq, wq, 1e-6, None, None))
    with pytest.raises(ValueError, match="grid_sizes"):
        WanPrep(wq, wq, 1e-6, table, None).to_c(hip_device)
