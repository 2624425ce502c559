"""The entry point that allocates nothing, ``ksana_sage_quant_k_static``, against ``ksana_sage_quant_k``.

Both are called through the C ABI on the same K; the quantized tiles, their scales and the channel means must agree
bit for bit (and with the CPU oracle).  Two calls in a row share the library's device-resident scratch, the second on
a smaller input, so anything the first call left there would show.  This file sorts after the other test files on
purpose: a failure here must not hide theirs.
"""

import ctypes as C

import pytest
import torch

from ksanadit_amd import _capi, sage_ops
from ksanadit_amd.layout import untile_k
from oracle import quant_ref as qr


def _strides(t):
    return _capi.Strides(*t.stride())


def _quant_k(entry, k, ws, smooth_k=1):
    lib = _capi.load()
    fn = getattr(lib, entry)
    rc = fn(k.data_ptr(), _capi.BF16, _strides(k), C.byref(ws.shape), smooth_k, ws.ptr,
            C.c_void_p(torch.cuda.current_stream(k.device).cuda_stream))
    _capi.check(rc, entry)


def _rand_k(B, L, H, seed):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn((B, L, H, 128), generator=g) + 2.0 * torch.randn((1, 1, H, 128), generator=g)
    return k.to(torch.bfloat16)


@pytest.mark.gpu
def test_static_scratch_entry_point_matches_the_workspace_one(hip_device):
    dev = hip_device
    for case, (B, L, H, seed) in enumerate([(2, 1000, 4, 11), (1, 300, 2, 12)]):  # the second call is the smaller one
        print(f"call {case}: B={B} L={L} H={H}", flush=True)
        k = _rand_k(B, L, H, seed)
        kd = k.to(dev)
        ws_a = sage_ops.SageWorkspace.allocate(B, H, H, L, L, 128, dev)
        ws_b = sage_ops.SageWorkspace.allocate(B, H, H, L, L, 128, dev)
        ws_a.blob.fill_(0xA5)
        ws_b.blob.fill_(0x5A)
        part_before = ws_b.blob[ws_b.layout.k_part : ws_b.layout.v_part].clone()
        _quant_k("ksana_sage_quant_k", kd, ws_a)
        _quant_k("ksana_sage_quant_k_static", kd, ws_b)
        torch.cuda.synchronize()
        for name in ("k_tiles", "k_scale", "k_mean"):
            assert torch.equal(getattr(ws_a, name), getattr(ws_b, name)), f"call {case}: {name} differs"
        # the static variant keeps its chunk sums in the library's own memory, not in the caller's workspace
        assert torch.equal(ws_b.blob[ws_b.layout.k_part : ws_b.layout.v_part], part_before)
        ki, ks, km = qr.quant_k_ref(k, smooth_k=True)
        assert torch.equal(untile_k(ws_b.k_tiles.cpu(), L), ki)
        assert torch.equal(ws_b.k_scale.cpu(), ks)
        assert torch.equal(ws_b.k_mean.cpu(), km.float())
    # without smoothing no chunk sum is taken at all
    k = _rand_k(1, 200, 2, 13).to(dev)
    ws_a = sage_ops.SageWorkspace.allocate(1, 2, 2, 200, 200, 128, dev)
    ws_b = sage_ops.SageWorkspace.allocate(1, 2, 2, 200, 200, 128, dev)
    _quant_k("ksana_sage_quant_k", k, ws_a, smooth_k=0)
    _quant_k("ksana_sage_quant_k_static", k, ws_b, smooth_k=0)
    torch.cuda.synchronize()
    for name in ("k_tiles", "k_scale", "k_mean"):
        assert torch.equal(getattr(ws_a, name), getattr(ws_b, name)), name


@pytest.mark.gpu
def test_static_scratch_entry_point_with_the_one_read_kernel(hip_device, quant_settings):
    """With K set to its one-read kernel the workgroups of a head meet through counters that live in the library's
    own array too (behind the chunk sums); the bits are those of the workspace variant, the caller's counters are
    not touched, and a second, smaller call finds the counters cleared."""
    quant_settings(one_read="kv")
    dev = hip_device
    for case, (B, L, H, seed) in enumerate([(2, 2000, 4, 21), (1, 700, 2, 22)]):
        print(f"one-read call {case}: B={B} L={L} H={H}", flush=True)
        k = _rand_k(B, L, H, seed)
        kd = k.to(dev)
        ws_a = sage_ops.SageWorkspace.allocate(B, H, H, L, L, 128, dev)
        ws_b = sage_ops.SageWorkspace.allocate(B, H, H, L, L, 128, dev)
        ws_a.blob.fill_(0xA5)
        ws_b.blob.fill_(0x5A)
        sync_before = ws_b.blob[ws_b.layout.k_sync : ws_b.layout.v_sync].clone()
        _quant_k("ksana_sage_quant_k", kd, ws_a)
        _quant_k("ksana_sage_quant_k_static", kd, ws_b)
        torch.cuda.synchronize()
        assert sage_ops.quant_status(ws_a)[0] == 0
        for name in ("k_tiles", "k_scale", "k_mean"):
            assert torch.equal(getattr(ws_a, name), getattr(ws_b, name)), f"call {case}: {name} differs"
        assert torch.equal(ws_b.blob[ws_b.layout.k_sync : ws_b.layout.v_sync], sync_before)
        ki, ks, km = qr.quant_k_ref(k, smooth_k=True)
        assert torch.equal(untile_k(ws_b.k_tiles.cpu(), L), ki)
        assert torch.equal(ws_b.k_scale.cpu(), ks)
        assert torch.equal(ws_b.k_mean.cpu(), km.float())


def test_static_scratch_entry_point_rejects_what_does_not_fit():
    """16384 chunk sums is the limit; the refusal comes before any device is touched, so it runs without one."""
    lib = _capi.load()
    fake = C.c_void_p(0x1000)
    shape = _capi.Shape(1, 65, 65, 64, 65536, 128)  # 65 heads x 256 chunks = 16640
    st = _capi.Strides(65536 * 65 * 128, 65 * 128, 128, 1)
    assert lib.ksana_sage_quant_k_static(fake, _capi.BF16, st, C.byref(shape), 1, fake, None) == _capi.ENOTSUP
    assert b"16384" in lib.ksana_sage_last_error() and b"ksana_sage_quant_k" in lib.ksana_sage_last_error()
    ok = _capi.Shape(1, 64, 64, 64, 65536, 128)  # exactly 16384: passes the size check, fails on the null tensor
    st = _capi.Strides(65536 * 64 * 128, 64 * 128, 128, 1)
    assert lib.ksana_sage_quant_k_static(None, _capi.BF16, st, C.byref(ok), 1, fake, None) == _capi.EINVAL
    assert b"k is null" in lib.ksana_sage_last_error()
