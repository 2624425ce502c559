"""Bit-exact parity of the HIP quantizer (through the C ABI) with the CPU oracle."""

import pytest
import torch

from ksanadit_amd import sage_ops
from ksanadit_amd.layout import untile_k, untile_v
from ksanadit_amd.workloads import make_inputs
from oracle import quant_ref as qr

pytestmark = pytest.mark.gpu


def _run_quant(q, k, v, dev, sm_scale=None, smooth_k=True, expect_status=(0, 0)):
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    ws = sage_ops.workspace_for(qd, kd)
    ws.blob.fill_(0xA5)  # stale bytes must not leak into any output the attention kernel reads
    sm_scale = q.shape[-1] ** -0.5 if sm_scale is None else sm_scale
    sage_ops.quant_q(qd, ws, sm_scale)
    sage_ops.quant_k(kd, ws, smooth_k)
    sage_ops.quant_v(vd, ws)
    torch.cuda.synchronize()
    if expect_status is not None:
        assert sage_ops.quant_status(ws) == expect_status, "a quantizer workgroup gave up waiting for its head (or did not, where the test makes it)"
    return ws


def _check_against_oracle(q, k, v, dev, sm_scale=None, smooth_k=True, expect_status=(0, 0)):
    ws = _run_quant(q, k, v, dev, sm_scale, smooth_k, expect_status)
    _compare_with_oracle(ws, q, k, v, sm_scale, smooth_k)
    return ws


def _compare_with_oracle(ws, q, k, v, sm_scale=None, smooth_k=True):
    Lq, Lk = q.shape[1], k.shape[1]
    sm = q.shape[-1] ** -0.5 if sm_scale is None else sm_scale
    qi, qs = qr.quant_q_ref(q, sm)
    ki, ks, km = qr.quant_k_ref(k, smooth_k=smooth_k)
    v8, vs = qr.quant_v_ref(v)
    got_qi = ws.q_i8.cpu()
    assert torch.equal(got_qi[:, :, :Lq], qi), "q_int8 differs"
    assert torch.count_nonzero(got_qi[:, :, Lq:]) == 0, "q padding rows not zero"
    assert torch.equal(ws.q_scale.cpu()[:, :, :Lq], qs), "q_scale differs"
    assert torch.equal(ws.k_mean.cpu(), km.float()), "k_mean differs"
    k_tiles = ws.k_tiles.cpu()
    assert torch.equal(untile_k(k_tiles, Lk), ki), "k_int8 differs"
    nkb = k_tiles.shape[2]
    if nkb * 64 > Lk:
        full = untile_k(k_tiles, nkb * 64)
        assert torch.count_nonzero(full[:, :, Lk:]) == 0, "k padding rows not zero"
    assert torch.equal(ws.k_scale.cpu(), ks), "k_scale differs"
    assert torch.equal(ws.v_scale.cpu(), vs), "v_scale differs"
    v_tiles = ws.v_tiles.cpu()
    assert torch.equal(untile_v(v_tiles, Lk), v8.view(torch.uint8)), "v_fp8 differs"
    if nkb * 64 > Lk:
        full = untile_v(v_tiles, nkb * 64)
        assert torch.count_nonzero(full[:, :, Lk:]) == 0, "v padding rows not zero"


@pytest.mark.parametrize("B,Lq,Lk,Hq,Hkv,dtype", [(1, 70, 70, 2, 2, torch.bfloat16), (2, 300, 520, 4, 2, torch.float16)])
def test_quantizer_bit_exact_head_size_64(hip_device, B, Lq, Lk, Hq, Hkv, dtype):
    """Head size 64: the kernels read the upper 64 channels as zeros; the oracle quantizes the zero-extended tensors."""
    print(f"case D=64 B={B} Lq={Lq} Lk={Lk} Hq={Hq} Hkv={Hkv} {dtype}", flush=True)
    g = torch.Generator().manual_seed(Lq + Lk)
    q = torch.randn((B, Lq, Hq, 64), generator=g).to(dtype)
    k = (torch.randn((B, Lk, Hkv, 64), generator=g) + 2.0 * torch.randn((1, 1, Hkv, 64), generator=g)).to(dtype)
    v = (1.5 * torch.randn((B, Lk, Hkv, 64), generator=g)).to(dtype)
    ws = _run_quant(q, k, v, hip_device, 64**-0.5, True)
    qi, qs = qr.quant_q_ref(qr.pad_head_dim(q), 64**-0.5)
    ki, ks, km = qr.quant_k_ref(qr.pad_head_dim(k))
    v8, vs = qr.quant_v_ref(qr.pad_head_dim(v))
    assert torch.equal(ws.q_i8.cpu()[:, :, :Lq], qi) and torch.equal(ws.q_scale.cpu()[:, :, :Lq], qs)
    assert torch.equal(ws.k_mean.cpu(), km.float()) and torch.equal(ws.k_scale.cpu(), ks)
    assert torch.equal(untile_k(ws.k_tiles.cpu(), Lk), ki)
    assert torch.equal(ws.v_scale.cpu(), vs) and torch.equal(untile_v(ws.v_tiles.cpu(), Lk), v8.view(torch.uint8))


def _rand_qkv(B, Lq, Lk, Hq, Hkv, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((B, Lq, Hq, 128), generator=g)
    k = torch.randn((B, Lk, Hkv, 128), generator=g) + 2.0 * torch.randn((1, 1, Hkv, 128), generator=g)
    v = torch.randn((B, Lk, Hkv, 128), generator=g) * 1.5
    return q.to(dtype), k.to(dtype), v.to(dtype)


@pytest.mark.parametrize(
    "B,Lq,Lk,Hq,Hkv",
    [(1, 1, 1, 1, 1), (1, 100, 100, 2, 2), (2, 333, 77, 3, 3), (1, 128, 64, 2, 1), (1, 257, 513, 4, 2), (1, 640, 1000, 1, 1)],
)
def test_quantizer_bit_exact_small(hip_device, B, Lq, Lk, Hq, Hkv):
    print(f"case B={B} Lq={Lq} Lk={Lk} Hq={Hq} Hkv={Hkv}", flush=True)
    q, k, v = _rand_qkv(B, Lq, Lk, Hq, Hkv, seed=Lq * 7 + Lk)
    _check_against_oracle(q, k, v, hip_device)


def test_quantizer_bit_exact_fp16_and_options(hip_device):
    q, k, v = _rand_qkv(1, 200, 300, 2, 2, seed=5, dtype=torch.float16)
    _check_against_oracle(q, k, v, hip_device)
    _check_against_oracle(q, k, v, hip_device, smooth_k=False)
    _check_against_oracle(q, k, v, hip_device, sm_scale=0.37)


def test_quantizer_edge_values(hip_device):
    q, k, v = _rand_qkv(1, 130, 130, 2, 2, seed=9)
    q[:, :3] = 0  # all-zero query rows -> scale 0, zeros
    k[:, 64:128, 0] = k[:, 64:65, 0]  # a K block constant along the sequence ...
    k[:, :, 1] = 1.25  # ... and a head that smoothing cancels completely
    v[:, :, 0, 5] = 0  # a zero V channel
    v[:, 7, 1, 9] = 300.0  # a lone huge V entry sets its channel's scale
    q[0, 50, 1, 3] = 2.0**-120  # tiny magnitudes stay finite
    _check_against_oracle(q, k, v, hip_device)
    # exact .5 ties after scaling: a row (64, 63, 0, ...) transforms to +-127 / +-1 entries
    q2 = torch.zeros_like(q)
    q2[..., 0], q2[..., 1] = 64.0, 63.0
    _check_against_oracle(q2, k, v, hip_device, sm_scale=1.0)


def test_quantizer_strided_inputs(hip_device):
    """q/k/v as views into one fused projection output, the way the DiT blocks produce them
    (ksana/models/wan/wan_model.py:163-166): row stride 3*H*D, not contiguous."""
    g = torch.Generator().manual_seed(3)
    fused = torch.randn((2, 150, 3, 2, 128), generator=g).to(torch.bfloat16)
    q, k, v = fused[:, :, 0], fused[:, :, 1], fused[:, :, 2]
    assert not q.is_contiguous()
    _check_against_oracle(q, k, v, hip_device)


@pytest.mark.parametrize(
    "name,heads,seq",
    [("cpu_plumbing", None, None), ("wan5b_720p", 1, None), ("wan14b_480p", 2, None), ("wan14b_720p", 1, None), ("qwen_cfg", 4, None)],
)
def test_quantizer_bit_exact_workloads(hip_device, name, heads, seq):
    """The five measured shapes at full sequence length (heads reduced where the CPU oracle
    would otherwise take minutes; heads are independent in every stage)."""
    print(f"workload {name} heads={heads}", flush=True)
    q, k, v = make_inputs(name, heads=heads, seq=seq)
    _check_against_oracle(q, k, v, hip_device)


def test_quantizer_bit_exact_past_the_one_read_limit(hip_device):
    """K and V are quantized by kernels that read them once as long as the 256-row chunks of one head are at most
    half of the workgroups the chip holds at a time (1024 on an MI355X); beyond that - here 547 chunks per head - the
    two-pass kernels take over.  Same bits either way; Q (no statistic over the sequence) is kept short."""
    Lk = 140000
    print(f"case long Lk={Lk}", flush=True)
    g = torch.Generator().manual_seed(77)
    q = torch.randn((1, 100, 1, 128), generator=g).to(torch.bfloat16)
    k = (torch.randn((1, Lk, 1, 128), generator=g) + 2.0 * torch.randn((1, 1, 1, 128), generator=g)).to(torch.bfloat16)
    v = (torch.randn((1, Lk, 1, 128), generator=g) * 1.5).to(torch.bfloat16)
    _check_against_oracle(q, k, v, hip_device)


def test_quantizers_repeat_bit_for_bit(hip_device):
    """The one-read kernels meet through counters in the workspace: a second run on the same workspace (the
    counters are cleared by each call) and a run on a fresh one give the same bytes."""
    q, k, v = make_inputs("qwen_cfg", heads=3)
    qd, kd, vd = (t.to(hip_device) for t in (q, k, v))
    ws = sage_ops.workspace_for(qd, kd)
    blobs = []
    for rep in range(3):
        if rep == 2:
            ws = sage_ops.workspace_for(qd, kd)
            ws.blob.fill_(0xFF)  # counters that start from garbage would never reach their target
        sage_ops.quant_k(kd, ws)
        sage_ops.quant_v(vd, ws)
        torch.cuda.synchronize()
        assert sage_ops.quant_status(ws) == (0, 0)
        blobs.append([ws.k_tiles.clone(), ws.k_scale.clone(), ws.k_mean.clone(), ws.v_tiles.clone(), ws.v_scale.clone()])
    for other in blobs[1:]:
        for a, b_ in zip(blobs[0], other):
            assert torch.equal(a, b_)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,L,H", [(1, 64, 1), (2, 130, 2), (1, 1000, 3), (1, 257, 1)])
def test_v_smoothing_bit_exact(hip_device, B, L, H, dtype):
    """smooth_v: channel mean (order and rounding of the K mean), abs-max and codes of the centred values, zero
    padding, and a workspace without smoothing reads zeros where the mean would be."""
    print(f"case smooth_v B={B} L={L} H={H} {dtype}", flush=True)
    g = torch.Generator().manual_seed(31 * L + H)
    v = (1.3 * torch.randn((B, L, H, 128), generator=g) + 5.0 * torch.randn((1, 1, H, 128), generator=g)).to(dtype)
    v[:, :, :, 7] = 2.5  # a constant channel: centred values, scale and codes are all zero
    vd = v.to(hip_device)
    ws = sage_ops.workspace_for(vd, vd)
    ws.blob.fill_(0xA5)
    sage_ops.quant_v(vd, ws, smooth_v=True)
    torch.cuda.synchronize()
    v8, vs, vm = qr.quant_v_ref(v, smooth_v=True)
    assert torch.equal(ws.v_mean.cpu(), vm.float()), "v_mean differs"
    assert torch.equal(ws.v_scale.cpu(), vs), "v_scale differs"
    tiles = ws.v_tiles.cpu()
    assert torch.equal(untile_v(tiles, L), v8.view(torch.uint8)), "v_fp8 differs"
    nkb = tiles.shape[2]
    if nkb * 64 > L:
        assert torch.count_nonzero(untile_v(tiles, nkb * 64)[:, :, L:]) == 0, "v padding rows not zero"
    assert (ws.v_scale.cpu()[:, :, 7] == 0).all() and (ws.v_mean.cpu()[:, :, 7] == 2.5).all()
    # without smoothing: the plain codes, and zeros in the mean slot
    sage_ops.quant_v(vd, ws)
    torch.cuda.synchronize()
    p8, ps = qr.quant_v_ref(v)
    assert torch.count_nonzero(ws.v_mean.cpu()) == 0
    assert torch.equal(ws.v_scale.cpu(), ps) and torch.equal(untile_v(ws.v_tiles.cpu(), L), p8.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_one_read_kernels_stay_exact_when_a_wait_runs_out(hip_device, dtype, quant_settings):
    """The one-read kernels wait, bounded, for the last workgroup of their head.  With a negative bound every
    workgroup but a head's last arriver skips the wait, flags it, and takes the head's statistic from the input
    itself, whatever the timing: the same bits as ever (the status words say that it happened)."""
    quant_settings(one_read="kv", wait_ticks=-1)
    q, k, v = _rand_qkv(2, 300, 3000, 4, 2, seed=91, dtype=dtype)  # 12 chunks per head, the last one ragged
    _check_against_oracle(q, k, v, hip_device, expect_status=(1, 1))
    quant_settings(wait_ticks=0)  # give up at the first poll that finds the flag down: which workgroups do depends on timing
    ws = _run_quant(q, k, v, hip_device, expect_status=None)
    _compare_with_oracle(ws, q, k, v)
    assert not sage_ops.one_read_state()["demoted"]  # test-mode bounds switch nothing off
    quant_settings(wait_ticks=200000)
    _check_against_oracle(q, k, v, hip_device)  # and the next call on a fresh workspace reports nothing


def test_an_expired_production_bound_switches_the_one_read_kernels_off(hip_device, quant_settings):
    """A positive bound that expires is reported through a word of host memory; from the next call on the library
    takes the two-pass kernels on this GPU (same bits), until ``configure`` re-arms it."""
    quant_settings(one_read="kv", wait_ticks=1)  # 10 ns: any workgroup that finds its head's flag down twice gives up
    q, k, v = _rand_qkv(1, 200, 4000, 4, 4, seed=92)
    ws = _run_quant(q, k, v, hip_device, expect_status=None)
    _compare_with_oracle(ws, q, k, v)
    if sage_ops.quant_status(ws) == (0, 0):
        pytest.skip("no workgroup had to wait for its head in this run")
    assert sage_ops.one_read_state()["demoted"]
    ws = _run_quant(q, k, v, hip_device, expect_status=(0, 0))  # the two-pass kernels: nothing to wait for
    _compare_with_oracle(ws, q, k, v)
    quant_settings(wait_ticks=200000)
    assert not sage_ops.one_read_state()["demoted"]
    _check_against_oracle(q, k, v, hip_device)
