"""Host-side contract of the attention op and the C ABI; runs without a GPU.

Mirrors the reference's own boundary behaviour: selector errors (backends/base.py:54-73), the op's
argument checks (attention_op.py:41-42, 80-81), config validation (attention_config.py:79-83),
shape/no-NaN checks of tests/ksana/attention_op_test.py:59-79, and the library's argument validation.
"""

import ctypes as C
import re
from pathlib import Path

import pytest
import torch

import ksanadit_amd
from ksanadit_amd import KsanaAttentionBackend, KsanaAttentionConfig, KsanaAttentionOp, _capi, pick_attn_op, sage_ops
from ksanadit_amd.backends import get_attention_backend_impl, get_backend_mapping
from ksanadit_amd.backends.sage_attn import SageAttentionImpl
from ksanadit_amd.backends.sdpa import SDPAImpl
from ksanadit_amd.layout import TILE_BYTES, k_tile_index, v_tile_index
from ksanadit_amd.workloads import HEADLINE, WORKLOADS, make_inputs
from oracle.sdpa_ref import sdpa_ref

ROOT = Path(__file__).resolve().parent.parent
HAS_GPU = torch.cuda.is_available()


# ----------------------------------------------------------------------------- C ABI
def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "ksana_sage_hip.h").read_text()
    declared = set(re.findall(r"\b(ksana_sage_[a-z_0-9]+)\s*\(", header))
    assert declared >= {"ksana_sage_forward", "ksana_sage_attn_fwd", "ksana_sage_quant_q", "ksana_sage_quant_k",
                        "ksana_sage_quant_v", "ksana_sage_workspace_layout", "ksana_sage_last_error", "ksana_sage_abi_version",
                        "ksana_sage_quant_q_prep", "ksana_sage_quant_k_prep", "ksana_sage_forward_prep"}
    lib = C.CDLL(str(_capi.LIB_PATH))
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert set(_capi.EXPORTS) == declared
    version = int(re.search(r"#define KSANA_SAGE_ABI_VERSION (\d+)", header).group(1))
    assert _capi.load().ksana_sage_abi_version() == version == _capi.ABI_VERSION


def test_workspace_layout_headline_shape():
    w = WORKLOADS[HEADLINE]
    shape, lay = _capi.workspace_layout(w.B, w.H, w.H, w.L, w.L, w.D)
    assert (lay.lq_pad, lay.nkb, lay.nch) == (32768, 512, 128)
    offs = [lay.q_i8, lay.q_scale, lay.k_i8, lay.k_scale, lay.k_mean, lay.v_fp8, lay.v_scale, lay.v_inv, lay.k_part, lay.v_part]
    assert offs == sorted(offs) and all(o % 256 == 0 for o in offs) and lay.total_bytes % 256 == 0
    assert lay.q_scale - lay.q_i8 == w.H * 32768 * 128  # int8 Q, padded to 128 rows
    assert lay.k_scale - lay.k_i8 == w.H * 512 * TILE_BYTES
    # three 8-bit tensors, scales, partial sums, and the fixed 34 MB scratch of the key-split workgroups
    assert lay.total_bytes < 3 * w.elements + (52 << 20)
    assert lay.split_ml - lay.split_o == 256 * 256 * 128 * 4


@pytest.mark.parametrize(
    "args,exc",
    [((1, 4, 4, 16, 16, 96), NotImplementedError), ((1, 4, 3, 16, 16, 128), ValueError), ((1, 4, 4, 0, 16, 128), ValueError),
     ((0, 4, 4, 16, 16, 128), ValueError), ((1, 4, 4, 16, 262145, 128), NotImplementedError), ((1, 70000, 70000, 16, 16, 128), ValueError),
     ((1, 4, 4, (1 << 24) + 1, 16, 128), NotImplementedError), ((8, 65535, 65535, 1 << 20, 16, 128), NotImplementedError)],
)
def test_workspace_layout_rejects_bad_shapes(args, exc):
    with pytest.raises(exc):
        _capi.workspace_layout(*args)


def test_a_workspace_for_another_shape_is_refused_before_any_launch():
    """The library takes B/H/L from the workspace's shape and pointers/strides from the tensors: a workspace laid out
    for other extents (say one reused across self- and cross-attention) must never reach it."""
    shape, layout = _capi.workspace_layout(1, 4, 4, 512, 512, 128)
    ws = sage_ops.SageWorkspace(shape, layout, torch.empty(layout.total_bytes, dtype=torch.uint8))
    ws.require("cpu", B=1, Hq=4, Hkv=4, Lq=512, Lk=512, D=128)
    ws.require("cpu", B=1, Lq=512)  # a stage that knows only some extents
    with pytest.raises(ValueError, match="Lk: workspace 512, tensor 77"):
        ws.require("cpu", B=1, Hq=4, Hkv=4, Lq=512, Lk=77, D=128)
    with pytest.raises(ValueError, match="another shape"):
        ws.require("cpu", B=2, Lq=512)
    with pytest.raises(ValueError, match="lives on"):
        ws.require("meta", B=1)
    short = sage_ops.SageWorkspace(shape, layout, torch.empty(layout.total_bytes - 256, dtype=torch.uint8))
    with pytest.raises(ValueError, match="the layout needs"):
        short.require("cpu", B=1)


def test_sage_backends_need_the_architecture_the_library_was_built_for(monkeypatch):
    """On a HIP device of another architecture the selector must move on (no code object would load)."""
    from ksanadit_amd import platform
    from ksanadit_amd.backends.radial_sage_attn import RadialSageAttentionImpl
    from ksanadit_amd.backends.sage_sla import SageSLAAttentionImpl

    monkeypatch.setattr(platform, "gcn_arch", lambda index=0: "gfx942")
    for impl in (SageAttentionImpl, RadialSageAttentionImpl, SageSLAAttentionImpl):
        assert impl.supports(head_size=128, dtype=torch.bfloat16) is False
    monkeypatch.setattr(platform, "gcn_arch", lambda index=0: "gfx950")
    assert SageAttentionImpl.supports(head_size=128, dtype=torch.bfloat16) is True
    assert SageAttentionImpl.supports(head_size=96, dtype=torch.bfloat16) is False


def test_entry_points_validate_before_touching_the_gpu():
    lib = _capi.load()
    shape = _capi.Shape(1, 2, 2, 64, 64, 128)
    st = _capi.Strides(64 * 2 * 128, 2 * 128, 128, 1)
    null = C.c_void_p(0)
    fake = C.c_void_p(0x1000)  # aligned, never dereferenced: every call below fails validation first
    assert lib.ksana_sage_workspace_layout(None, None) == _capi.EINVAL
    assert lib.ksana_sage_quant_q(null, _capi.BF16, st, C.byref(shape), 0.1, fake, null) == _capi.EINVAL
    assert b"q is null" in lib.ksana_sage_last_error()
    assert lib.ksana_sage_quant_k(fake, 7, st, C.byref(shape), 1, fake, null) == _capi.EINVAL  # dtype
    assert lib.ksana_sage_quant_v(C.c_void_p(0x1008), _capi.BF16, st, C.byref(shape), fake, null) == _capi.EINVAL  # alignment
    bad = _capi.Strides(64 * 2 * 128, 2 * 128, 128, 2)
    assert lib.ksana_sage_quant_q(fake, _capi.BF16, bad, C.byref(shape), 0.1, fake, null) == _capi.EINVAL
    assert b"D stride" in lib.ksana_sage_last_error()
    odd = _capi.Strides(64 * 2 * 128, 2 * 128 + 4, 128, 1)
    assert lib.ksana_sage_quant_q(fake, _capi.BF16, odd, C.byref(shape), 0.1, fake, null) == _capi.EINVAL
    assert lib.ksana_sage_quant_q(fake, _capi.BF16, st, C.byref(shape), 0.1, null, null) == _capi.EINVAL  # workspace
    lay = _capi.WsLayout()
    assert lib.ksana_sage_workspace_layout(C.byref(_capi.Shape(1, 2, 2, 64, 64, 64)), C.byref(lay)) == 0  # head size 64
    lay128 = _capi.WsLayout()
    assert lib.ksana_sage_workspace_layout(C.byref(shape), C.byref(lay128)) == 0
    assert lay.total_bytes == lay128.total_bytes  # it runs zero-padded to 128 channels
    assert lib.ksana_sage_workspace_layout(C.byref(_capi.Shape(1, 2, 2, 64, 64, 96)), C.byref(lay)) == _capi.ENOTSUP
    assert b"head size 96" in lib.ksana_sage_last_error()
    long_k = _capi.Shape(1, 2, 2, 64, 131073, 128)  # causal masking keeps its tile list in LDS: Lk <= 131072
    assert lib.ksana_sage_attn_fwd(fake, fake, _capi.BF16, st, C.byref(long_k), null, 1, 0, null) == _capi.ENOTSUP
    assert b"causal" in lib.ksana_sage_last_error()
    assert lib.ksana_sage_attn_fwd_varlen(fake, fake, _capi.BF16, st, C.byref(shape), null, None, C.c_void_p(0x1002), null,
                                          0, 0, null) == _capi.EINVAL  # q_lens alignment
    assert b"q_lens" in lib.ksana_sage_last_error()
    assert lib.ksana_sage_attn_fwd(fake, fake, _capi.BF16, st, C.byref(shape), null, 0, 0x20, null) == _capi.EINVAL  # flags
    both = _capi.FLAG_TILE_SKIP | _capi.FLAG_PWL_EXP2  # the skip's zero point is the exact exponential's
    assert lib.ksana_sage_attn_fwd(fake, fake, _capi.BF16, st, C.byref(shape), null, 0, both, null) == _capi.EINVAL
    assert b"TILE_SKIP" in lib.ksana_sage_last_error()
    assert lib.ksana_sage_attn_fwd(fake, fake, _capi.BF16, st, C.byref(shape), C.c_void_p(0x1002), 0, 0, null) == _capi.EINVAL  # k_lens alignment
    assert lib.ksana_sage_forward(fake, fake, null, fake, _capi.BF16, st, st, st, st, C.byref(shape), null, 0.1, 1, 0, 0, fake, null) == _capi.EINVAL
    # the step-before-attention descriptor is validated on the host as well
    prep = _capi.Prep()
    prep.q_norm_weight, prep.norm_eps = 0x1004, 1e-6  # misaligned weight
    assert lib.ksana_sage_quant_q_prep(fake, _capi.BF16, st, C.byref(shape), C.byref(prep), 0.1, fake, null) == _capi.EINVAL
    assert b"16-byte aligned" in lib.ksana_sage_last_error()
    prep = _capi.Prep()
    prep.rope_freqs, prep.rope_rows = 0x1000, 1024  # rotation without a grid
    assert lib.ksana_sage_quant_k_prep(fake, _capi.BF16, st, C.byref(shape), C.byref(prep), 1, fake, null) == _capi.EINVAL
    grid = (C.c_int32 * 3)(2, 8, 8)  # 128 positions, 64 rows
    prep.grid_sizes = C.cast(grid, C.POINTER(C.c_int32))
    assert lib.ksana_sage_quant_k_prep(fake, _capi.BF16, st, C.byref(shape), C.byref(prep), 1, fake, null) == _capi.EINVAL
    assert b"exceeds" in lib.ksana_sage_last_error()
    with pytest.raises(ValueError):
        _capi.check(_capi.EINVAL, "x")
    with pytest.raises(NotImplementedError):
        _capi.check(_capi.ENOTSUP, "x")
    with pytest.raises(_capi.SageLibraryError):
        _capi.check(_capi.EHIP, "x")


def test_missing_library_is_loud(monkeypatch, tmp_path):
    monkeypatch.setattr(_capi, "_lib", None)
    monkeypatch.setattr(_capi, "LIB_PATH", tmp_path / "libksana_sage_hip.so")
    with pytest.raises(_capi.SageLibraryError, match="ksanadit_amd.build"):
        _capi.load()
    (tmp_path / "libksana_sage_hip.so").write_bytes(b"not an ELF file")
    with pytest.raises(_capi.SageLibraryError, match="cannot load"):
        _capi.load()


def test_tile_index_maps_are_permutations():
    for idx in (k_tile_index(), v_tile_index()):
        assert idx.shape == (64, 128)
        assert torch.equal(idx.flatten().sort().values, torch.arange(TILE_BYTES))
    # a K operand fragment is 16 consecutive channels of one key; a V^T fragment is 4 consecutive keys
    assert (k_tile_index()[5, 16:32] - k_tile_index()[5, 16] == torch.arange(16)).all()
    assert (v_tile_index()[8:12, 7] - v_tile_index()[8, 7] == torch.arange(4)).all()


# ----------------------------------------------------------------------------- selector / op
def test_enum_values_and_supported_list_follow_the_reference():
    assert KsanaAttentionBackend.SAGE_ATTN.value == "sage_attention" and KsanaAttentionBackend.TORCH_SDPA.value == "torch_sdpa"
    assert KsanaAttentionBackend.get_supported_list() == ["sage_attention", "torch_sdpa", "radial_sage_attention", "sage_sla"]
    assert KsanaAttentionBackend.get_supported_list(exclude=[KsanaAttentionBackend.SAGE_ATTN]) == ["torch_sdpa", "radial_sage_attention", "sage_sla"]
    assert KsanaAttentionBackend.support("torch_sdpa") and not KsanaAttentionBackend.support("flash_attention")
    assert KsanaAttentionBackend.support(KsanaAttentionBackend.FLASH_ATTN) and not KsanaAttentionBackend.support(3)
    mapping = get_backend_mapping()
    assert mapping[KsanaAttentionBackend.SAGE_ATTN] is SageAttentionImpl and mapping[KsanaAttentionBackend.TORCH_SDPA] is SDPAImpl


def test_radial_config_and_backend_contract_without_gpu():
    """attention_config.py:86-104 and radial_sage_attn.py:32-59 (constructor checks)."""
    from ksanadit_amd.backends.radial_sage_attn import RadialSageAttentionImpl
    from ksanadit_amd.config import KsanaRadialSageAttentionConfig

    cfg = KsanaRadialSageAttentionConfig()
    assert cfg.backend is KsanaAttentionBackend.RADIAL_SAGE_ATTN and cfg.block_size == 128 and cfg.decay_factor == 0.02
    assert cfg.dense_attention_config.backend is KsanaAttentionBackend.SAGE_ATTN
    for bad in ({"block_size": 32}, {"decay_factor": 0.0}, {"decay_factor": 1.0}):
        with pytest.raises(ValueError):
            KsanaRadialSageAttentionConfig(**bad)
    assert get_backend_mapping()[KsanaAttentionBackend.RADIAL_SAGE_ATTN] is RadialSageAttentionImpl
    assert RadialSageAttentionImpl.type() is KsanaAttentionBackend.RADIAL_SAGE_ATTN
    if not torch.cuda.is_available():
        assert RadialSageAttentionImpl.supports(head_size=128) is False
        with pytest.raises(RuntimeError):
            RadialSageAttentionImpl(cfg, 2, 128, False, 0.1)


def test_sla_host_logic_without_gpu():
    """Config and the torch halves of the sparse-linear backend (sage_sla.py:83-90, 273-282): the top-k cut over pooled
    blocks and the linear branch, here on CPU tensors with the oracle's pooling in place of the HIP kernel."""
    from ksanadit_amd.backends.sage_sla import SageSLAAttentionImpl, block_map_from_pooled, linear_branch
    from ksanadit_amd.config import KsanaSageSLAConfig
    from oracle.sla_ref import block_map_ref, block_means_ref, linear_branch_ref

    cfg = KsanaSageSLAConfig(topk=0.25)
    assert cfg.backend is KsanaAttentionBackend.SAGE_SLA
    for bad in (0.0, 1.0):
        with pytest.raises(ValueError):
            KsanaSageSLAConfig(topk=bad)
    assert get_backend_mapping()[KsanaAttentionBackend.SAGE_SLA] is SageSLAAttentionImpl
    g = torch.Generator().manual_seed(3)
    # key blocks sit at distinct levels along a direction the queries lean towards: a clear top-k cut in every row
    direction = torch.nn.functional.normalize(torch.randn(16, generator=g), dim=0)
    level = torch.randperm(16, generator=g).float().repeat_interleave(64)
    q = (torch.randn((1, 512, 2, 16), generator=g) + 2.0 * direction).to(torch.bfloat16)
    k = (torch.randn((1, 1024, 2, 16), generator=g) + 3.0 + 0.6 * level[None, :, None, None] * direction).to(torch.bfloat16)
    want, kept, gap = block_map_ref(q, k, 0.25)
    from oracle.quant_ref import k_mean_ref
    pooled_q = block_means_ref(q.permute(0, 2, 1, 3), 128)
    pooled_k = block_means_ref(k.permute(0, 2, 1, 3), 64, centre=k_mean_ref(k))
    bmap, got_kept = block_map_from_pooled(pooled_q, pooled_k, 0.25)
    assert bmap.shape == (1, 2, 4, 16) and bmap.dtype == torch.int8 and got_kept == kept == 4
    assert (bmap.sum(dim=-1) == 4).all()
    assert float(gap.min()) > 0.1 and torch.equal(bmap, want)  # no row's cut hangs on a tie
    v = torch.randn((1, 512, 2, 16), generator=g).to(torch.bfloat16)
    o = linear_branch(*(t.transpose(1, 2) for t in (q, k[:, :512], v)))
    ref = linear_branch_ref(q, k[:, :512], v)
    assert o.shape == (1, 2, 512, 16) and (o.float() - ref.float()).abs().max() <= 0.03 * ref.float().abs().max()


def test_config_and_selector_errors():
    with pytest.raises(ValueError):  # attention_config.py:79-83
        KsanaAttentionConfig(backend="no_such_backend")
    with pytest.raises(ValueError):
        KsanaAttentionConfig(backend="flash_attention")  # known to the reference, not built here
    with pytest.raises(ValueError):  # attention_op.py:41-42
        KsanaAttentionOp(4, 128)
    cfg = KsanaAttentionConfig(backend=KsanaAttentionBackend.FLASH_ATTN)  # enum members pass the config check ...
    with pytest.raises(ValueError):  # ... and fail in the registry (base.py:62-63)
        get_attention_backend_impl(cfg, head_size=128, dtype=torch.bfloat16)
    frozen = KsanaAttentionConfig(backend="torch_sdpa")
    with pytest.raises(Exception):
        frozen.backend = "sage_attention"


def test_no_backend_available_raises_runtime_error(monkeypatch):
    from ksanadit_amd.backends.base import get_backend_mapping

    for impl in get_backend_mapping().values():
        monkeypatch.setattr(impl, "supports", staticmethod(lambda **_: False))
    with pytest.raises(RuntimeError, match="No compatible attention"):
        get_attention_backend_impl(KsanaAttentionConfig(backend="torch_sdpa"), head_size=128, dtype=torch.float16)


@pytest.mark.skipif(HAS_GPU, reason="describes the GPU-less host")
def test_sage_request_on_a_host_without_gpu():
    """supports() is False, the walk moves on to SDPA, and constructing SDPA under a Sage config
    trips check_config - exactly what the reference does without its package (base.py:59-69,102-106)."""
    assert SageAttentionImpl.supports(head_size=128, dtype=torch.bfloat16) is False
    cfg = KsanaAttentionConfig(backend=KsanaAttentionBackend.SAGE_ATTN)
    assert get_attention_backend_impl(cfg, head_size=128, dtype=torch.bfloat16) is SDPAImpl
    op = pick_attn_op(cfg)(num_heads=2, head_size=128)
    q = torch.zeros(1, 8, 2, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="does not match implementation"):
        op(q, q, q)
    with pytest.raises(RuntimeError):
        SageAttentionImpl(cfg, 2, 128, False, 128**-0.5)
    with pytest.raises(RuntimeError, match="no CPU path"):
        sage_ops.sageattn(q, q, q)


def test_sdpa_backend_on_cpu_matches_oracle_and_reference_checks():
    B, L, H, D = 2, 32, 64, 128  # the reference's test shape, attention_op_test.py:24
    torch.manual_seed(0)
    q, k, v = (torch.randn(B, L, H, D, dtype=torch.float16) for _ in range(3))
    attn = pick_attn_op(KsanaAttentionConfig(backend=KsanaAttentionBackend.TORCH_SDPA))(num_heads=H, head_size=D, causal=False)
    assert attn.backend_type is None
    out = attn(q, k, v, k_lens=None, window_size=(-1, -1), block_id=3, dense_only=True)  # model kwargs are tolerated
    assert attn.backend_type == KsanaAttentionBackend.TORCH_SDPA
    assert out.shape == q.shape and not torch.isnan(out).any()
    assert torch.equal(out, sdpa_ref(q, k, v))
    assert attn.softmax_scale == D**-0.5
    # dtype change rebuilds the impl (attention_op.py:53-55); fp32 works on SDPA
    first = attn._attn_impl
    out32 = attn(q.float(), k.float(), v.float())
    assert out32.dtype == torch.float32 and attn._attn_impl is not first
    # per-call scale override and GQA (sdpa.py:52-75)
    kk, vv = k[:, :, :8], v[:, :, :8]
    assert torch.equal(attn(q, kk, vv, softmax_scale=0.2), sdpa_ref(q, kk, vv, scale=0.2))
    for bad in (q[0], q.unsqueeze(0)):
        with pytest.raises(ValueError, match=r"\[B, L, H, D\]"):
            attn(bad, k, v)


def test_cpu_plumbing_workload_through_the_op():
    """configs[0]: the CPU-runnable case goes through this package's SDPA backend."""
    q, k, v = make_inputs("cpu_plumbing", heads=2)
    assert q.shape == (1, 1560, 2, 128) and q.dtype == torch.bfloat16
    attn = pick_attn_op(KsanaAttentionConfig(backend="torch_sdpa"))(num_heads=2, head_size=128)
    out = attn(q, k, v)
    assert out.shape == q.shape and torch.isfinite(out.float()).all()
    assert torch.equal(out, sdpa_ref(q, k, v))


def test_workload_table():
    w = WORKLOADS[HEADLINE]
    assert (w.B, w.H, w.L, w.D) == (1, 40, 32760, 128) and abs(w.flops - 21.98e12) < 0.01e12
    assert [WORKLOADS[n].L for n in ("cpu_plumbing", "wan5b_720p", "wan14b_720p", "qwen_cfg")] == [1560, 27280, 75600, 4352]
    q1, k1, _ = make_inputs("qwen_cfg", heads=1, seq=600)
    q2, k2, _ = make_inputs("qwen_cfg", heads=1, seq=600)
    assert torch.equal(q1, q2) and torch.equal(k1, k2)  # seeded
    assert q1[:, :256].float().std() > 2.0 * q1[:, 256:].float().std()  # text tokens first, N(0, 3)
    qo, ko, _ = make_inputs("wan14b_480p", heads=1, seq=4096)
    assert qo.float().abs().max() > 20 and ko.float().abs().max() > 20  # x20 outliers present
    assert ksanadit_amd.DEFAULT_ATTENTION_BACKEND == KsanaAttentionBackend.SAGE_ATTN


def test_prep_operands_are_converted_once_per_source_tensor():
    """Norm weights and rotary tables that are not in the kernels' dtype (or not on the device) are converted on first
    use and the result is reused until the source tensor is written to."""
    from ksanadit_amd import sage_ops

    w = torch.randn(128, dtype=torch.bfloat16)
    a = sage_ops._prep_operand(w, "cpu", torch.float32)
    assert a.dtype == torch.float32 and torch.equal(a, w.float())
    assert sage_ops._prep_operand(w, "cpu", torch.float32) is a
    w.mul_(2.0)
    b = sage_ops._prep_operand(w, "cpu", torch.float32)
    assert b is not a and torch.equal(b, w.float())
    ready = torch.randn(128)
    assert sage_ops._prep_operand(ready, "cpu", torch.float32) is ready  # nothing to convert: passed through
    table = torch.polar(torch.ones(8, 64), torch.randn(8, 64))  # complex64
    t128 = sage_ops._prep_operand(table, "cpu", torch.complex128)
    assert t128.dtype == torch.complex128 and sage_ops._prep_operand(table, "cpu", torch.complex128) is t128


def test_one_read_settings_and_the_occupancy_cache_without_gpu():
    """``ksana_sage_configure`` validates and stores its settings without touching a device; the launchers' cache of
    resident-workgroup counts keeps one entry per kernel instantiation (two instantiations of one template have the same
    function-pointer type, so the type cannot be the key)."""
    lib = _capi.load()
    assert lib.ksana_sage_selftest() == 0, lib.ksana_sage_last_error()
    before = sage_ops.one_read_state()
    try:
        assert lib.ksana_sage_configure(b"kx", _capi.KEEP) == _capi.EINVAL and b"letters k and v" in lib.ksana_sage_last_error()
        sage_ops.configure(one_read="k", wait_ticks=-1)
        assert sage_ops.one_read_state() == {"k": True, "v": False, "wait_ticks": -1, "demoted": False}
        sage_ops.configure(one_read="")
        assert sage_ops.one_read_state() == {"k": False, "v": False, "wait_ticks": -1, "demoted": False}
        sage_ops.configure(wait_ticks=123)
        assert sage_ops.one_read_state()["wait_ticks"] == 123 and not sage_ops.one_read_state()["k"]
    finally:
        sage_ops.configure(one_read=("k" if before["k"] else "") + ("v" if before["v"] else ""), wait_ticks=before["wait_ticks"])
    assert sage_ops.one_read_state() == before


def test_the_documented_binding_checks_the_current_abi():
    """INTEGRATION.md's reference-side stub switches itself off when the library's ABI number differs from the one it
    was written against: that number must be the header's."""
    root = Path(__file__).resolve().parent.parent
    header = (root / "include" / "ksana_sage_hip.h").read_text()
    abi = int(re.search(r"#define KSANA_SAGE_ABI_VERSION (\d+)", header).group(1))
    doc = (root / "INTEGRATION.md").read_text()
    assert int(re.search(r"_KSANA_SAGE_ABI = (\d+)", doc).group(1)) == abi == _capi.ABI_VERSION


def test_argument_validation_under_the_host_address_sanitizer():
    """``host_args_check`` drives the C ABI's validation paths from C++ with AddressSanitizer on the host pass of every
    source: shapes, strides, the prep descriptor and its host-resident grid sizes are read under the sanitizer, and no
    call reaches a device.  Built by ``__graft_entry__.build()``; rebuilt here when a source is newer (about a minute)."""
    from ksanadit_amd import build_host_check as hc
    from ksanadit_amd.build import CSRC

    sources = list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h")) + list(CSRC.glob("*.cpp")) + \
        [Path(__file__).resolve().parent.parent / "include" / "ksana_sage_hip.h"]
    if not hc.EXE_PATH.exists() or hc.EXE_PATH.stat().st_mtime < max(f.stat().st_mtime for f in sources):
        hc.build_host_check(verbose=False)
    r = hc.run_host_check()
    assert r.returncode == 0, r.stdout + r.stderr
    assert "0 failed" in r.stdout and "AddressSanitizer" not in r.stderr
