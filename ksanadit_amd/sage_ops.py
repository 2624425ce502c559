"""Python face of the HIP library: the functions a backend (or a test) calls.

``sageattn`` has the signature of the third-party function the reference's backend calls
(``sageattn(q, k, v, tensor_layout="NHD", is_causal=...)``,
ksana/operations/attention/backends/sage_attn.py:75-81); the stage functions expose the quantized
operands so they can be compared bit for bit with a specification.

Everything runs on the tensors' HIP device, on torch's current stream, without synchronising.
Scratch comes from torch's caching allocator, so it is stream-ordered and recycled across the
thousands of calls of one generation.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import torch
from torch.utils.weak import WeakTensorKeyDictionary

from . import _capi
from .layout import TILE_BYTES
from .logger import log

_DTYPES = {torch.bfloat16: _capi.BF16, torch.float16: _capi.FP16}


def _strides(t: torch.Tensor):
    return _capi.Strides(*t.stride())


_copy_warned = False


def _usable(t: torch.Tensor) -> torch.Tensor:
    """The kernels read 16 bytes at a time along D: fix up layouts that do not allow it.  The fix-up is a full
    copy of the tensor (one more read and write of it ahead of an HBM-bound stage), so the first one is logged."""
    global _copy_warned
    s = t.stride()
    ok = s[3] == 1 and all(x % 8 == 0 and x > 0 for x, n in zip(s[:3], t.shape[:3]) if n > 1)
    if ok and t.data_ptr() % 16 == 0:
        return t
    if not _copy_warned:
        _copy_warned = True
        log.warning("Sage HIP path: copying a tensor of shape %s, strides %s (the kernels need a unit D stride, other "
                    "strides multiples of 8 and a 16-byte aligned base); further copies are not logged",
                    tuple(t.shape), tuple(s))
    return t.contiguous()


_prep_cache = WeakTensorKeyDictionary()  # source tensor -> {(device, dtype): (version, converted)}
_prep_move_warned = False


def _prep_operand(t: torch.Tensor, device, dtype) -> torch.Tensor:
    """A weight or table of the step before attention as the kernels read it: on ``device``, ``dtype``, contiguous.
    A conversion is remembered per source tensor (and redone once that tensor has been written to), so a caller that
    keeps its weights in another dtype - or on the host - pays for it once, not in every attention call; a transfer
    from another device is logged the first time."""
    global _prep_move_warned
    device = torch.device(device)
    if t.device == device and t.dtype == dtype and t.is_contiguous():
        return t
    key = (device, dtype)
    hit = _prep_cache.get(t, {}).get(key)
    if hit is not None and hit[0] == t._version:
        return hit[1]
    if t.device != device and not _prep_move_warned:
        _prep_move_warned = True
        log.warning("Sage HIP path: a norm weight / rotary table lives on %s, the tensors on %s; it is copied over once "
                    "per tensor (keep them on the device to avoid even that)", t.device, device)
    conv = t.detach().to(device=device, dtype=dtype).contiguous()
    _prep_cache.setdefault(t, {})[key] = (t._version, conv)
    return conv


def _stream_ptr(device) -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _require_hip(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError(
                "the Sage HIP backend needs tensors on a HIP device; there is no CPU path "
                f"(got device {t.device})"
            )
    if len({t.device for t in tensors}) != 1 or len({t.dtype for t in tensors}) != 1:
        raise ValueError("q, k, v must share one device and one dtype")
    if tensors[0].dtype not in _DTYPES:
        raise ValueError(f"dtype {tensors[0].dtype} not supported by the kernels (bf16 / fp16 only)")


@dataclass
class SageWorkspace:
    """One scratch blob plus typed views of its sub-buffers (see include/ksana_sage_hip.h)."""

    shape: _capi.Shape
    layout: _capi.WsLayout
    blob: torch.Tensor

    @classmethod
    def allocate(cls, B, Hq, Hkv, Lq, Lk, D, device) -> "SageWorkspace":
        shape, layout = _capi.workspace_layout(B, Hq, Hkv, Lq, Lk, D)
        blob = torch.empty(layout.total_bytes, dtype=torch.uint8, device=device)
        if blob.data_ptr() % 256:
            raise RuntimeError("allocator returned a workspace that is not 256-byte aligned")
        return cls(shape, layout, blob)

    @property
    def ptr(self) -> C.c_void_p:
        return C.c_void_p(self.blob.data_ptr())

    def require(self, device, *, B=None, Hq=None, Hkv=None, Lq=None, Lk=None, D=None) -> None:
        """Refuse a workspace laid out for other extents than the tensors about to be handed to the library: it
        takes B/H/L from the workspace's shape but pointers and strides from the tensors, so a mismatch would read
        and write out of bounds.  ``None`` extents are not checked (a stage that sees only q knows nothing of Lk)."""
        s = self.shape
        want = {"B": B, "Hq": Hq, "Hkv": Hkv, "Lq": Lq, "Lk": Lk, "D": D}
        bad = {n: (getattr(s, n), x) for n, x in want.items() if x is not None and getattr(s, n) != x}
        if bad:
            detail = ", ".join(f"{n}: workspace {a}, tensor {b}" for n, (a, b) in bad.items())
            raise ValueError(f"workspace was laid out for another shape ({detail})")
        if self.blob.device != torch.device(device):
            raise ValueError(f"workspace lives on {self.blob.device}, the tensors on {device}")
        if self.blob.dtype != torch.uint8 or self.blob.numel() < self.layout.total_bytes:
            raise ValueError(f"workspace blob holds {self.blob.numel() * self.blob.element_size()} bytes, "
                             f"the layout needs {self.layout.total_bytes}")

    def _view(self, off: int, nbytes: int, dtype, shape):
        return self.blob[off : off + nbytes].view(dtype).view(shape)

    @property
    def q_i8(self):
        s, l = self.shape, self.layout
        return self._view(l.q_i8, s.B * s.Hq * l.lq_pad * PAD_D, torch.int8, (s.B, s.Hq, l.lq_pad, PAD_D))

    @property
    def q_scale(self):
        s, l = self.shape, self.layout
        return self._view(l.q_scale, s.B * s.Hq * l.lq_pad * 4, torch.float32, (s.B, s.Hq, l.lq_pad))

    @property
    def k_tiles(self):
        s, l = self.shape, self.layout
        return self._view(l.k_i8, s.B * s.Hkv * l.nkb * TILE_BYTES, torch.int8, (s.B, s.Hkv, l.nkb, TILE_BYTES))

    @property
    def k_scale(self):
        s, l = self.shape, self.layout
        return self._view(l.k_scale, s.B * s.Hkv * l.nkb * 4, torch.float32, (s.B, s.Hkv, l.nkb))

    @property
    def k_mean(self):
        s, l = self.shape, self.layout
        return self._view(l.k_mean, s.B * s.Hkv * PAD_D * 4, torch.float32, (s.B, s.Hkv, PAD_D))

    @property
    def v_tiles(self):
        s, l = self.shape, self.layout
        return self._view(l.v_fp8, s.B * s.Hkv * l.nkb * TILE_BYTES, torch.uint8, (s.B, s.Hkv, l.nkb, TILE_BYTES))

    @property
    def v_scale(self):
        s, l = self.shape, self.layout
        return self._view(l.v_scale, s.B * s.Hkv * PAD_D * 4, torch.float32, (s.B, s.Hkv, PAD_D))


    @property
    def v_mean(self):
        """Channel means the V quantizer took off (zeros unless it ran with ``smooth_v``)."""
        s, l = self.shape, self.layout
        return self._view(l.v_mean, s.B * s.Hkv * PAD_D * 4, torch.float32, (s.B, s.Hkv, PAD_D))

    @property
    def q_rms(self):
        s, l = self.shape, self.layout
        return self._view(l.q_rms, s.B * s.Lq * 4, torch.float32, (s.B, s.Lq))

    @property
    def k_rms(self):
        s, l = self.shape, self.layout
        return self._view(l.k_rms, s.B * s.Lk * 4, torch.float32, (s.B, s.Lk))


@dataclass
class WanPrep:
    """What ``WanSelfAttention.forward`` does to the q and k projections before attention
    (ksana/models/wan/wan_model.py:163-174), handed to the quantizer to apply while it reads them:
    RMSNorm over the whole token row with fp32 weights (``norm_q.weight`` / ``norm_k.weight``; ``None`` skips it),
    then ``apply_default_rope(x, grid_sizes, freqs)`` (ksana/utils/rope.py:61-128; ``freqs=None`` skips it, as in
    the cross-attention block).  ``freqs`` is the model's complex128 buffer ``[1024, D/2]``, ``grid_sizes`` one
    ``(frames, height, width)`` per batch entry.

    With ``rope_func == "comfy"`` (wan_model.py:169-171) the block rotates with ``apply_comfyui_rope``
    (ksana/utils/rope.py:180-212) instead: pass its ``freqs_cis`` as ``comfy_freqs`` - fp32 2x2 matrices,
    ``[1, rows, 1, D/2, 2, 2]`` or ``[rows, D/2, 2, 2]`` - and leave ``freqs`` / ``grid_sizes`` unset; token rows past
    the table are left unrotated (the identity padding of rope.py:133-148)."""

    q_norm_weight: torch.Tensor | None = None
    k_norm_weight: torch.Tensor | None = None
    eps: float = 1e-6
    freqs: torch.Tensor | None = None
    grid_sizes: object = None
    comfy_freqs: torch.Tensor | None = None

    def to_c(self, device):
        """The C struct plus the objects that must outlive the call."""
        keep = []

        def weight(w):
            if w is None:
                return None
            w = _prep_operand(w, device, torch.float32)
            keep.append(w)
            return w.data_ptr()

        c = _capi.Prep()
        c.q_norm_weight, c.k_norm_weight = weight(self.q_norm_weight), weight(self.k_norm_weight)
        c.norm_eps = float(self.eps)
        if self.comfy_freqs is not None:
            if self.freqs is not None:
                raise ValueError("give either freqs (default rope) or comfy_freqs, not both")
            m = self.comfy_freqs
            if m.dim() == 6 and m.shape[0] == 1 and m.shape[2] == 1:
                m = m[0, :, 0]
            if m.dim() != 4 or tuple(m.shape[1:]) != (64, 2, 2) or m.is_complex():
                raise ValueError(f"comfy_freqs must be [1, rows, 1, 64, 2, 2] or [rows, 64, 2, 2], got {tuple(self.comfy_freqs.shape)}")
            m = _prep_operand(m, device, torch.float32)
            keep.append(m)
            c.kind = _capi.PREP_WAN_COMFY
            c.rope_matrices, c.rope_rows = m.data_ptr(), m.shape[0]
        if self.freqs is not None:
            if self.freqs.dim() != 2 or not self.freqs.is_complex():
                raise ValueError("freqs must be a complex [rows, D/2] tensor")
            if self.grid_sizes is None:
                raise ValueError("freqs given without grid_sizes")
            fr = _prep_operand(self.freqs, device, torch.complex128)
            grid = torch.as_tensor(self.grid_sizes).to(device="cpu", dtype=torch.int32).contiguous()
            if grid.dim() != 2 or grid.shape[1] != 3:
                raise ValueError(f"grid_sizes must be [B, 3], got {tuple(grid.shape)}")
            keep += [fr, grid]
            c.rope_freqs, c.rope_rows = fr.data_ptr(), fr.shape[0]
            c.grid_sizes = C.cast(grid.data_ptr(), C.POINTER(C.c_int32))
        return c, keep


@dataclass
class QwenPrep:
    """What ``QwenDoubleStreamAttention.forward`` does to q and k before its joint attention call
    (ksana/models/qwen/attention.py:340-357), handed to the quantizer to apply while it reads them.  q and k are the
    raw projections of the text tokens followed by those of the image tokens (the concatenation the block performs
    anyway, here done before instead of after): RMSNorm over the ``D`` channels of every head - ``norm_q`` /
    ``norm_k`` weights (``[D]``) for the image rows, ``norm_added_q`` / ``norm_added_k`` for the first ``txt_len`` rows -
    then ``apply_rotary_emb_qwen`` with the complex64 tables ``img_freqs`` ``[L - txt_len, D/2]`` and ``txt_freqs``
    ``[txt_len, D/2]``.  ``None`` weights skip the norm of that segment, ``None`` tables its rotation."""

    txt_len: int
    q_norm_weight: torch.Tensor | None = None
    k_norm_weight: torch.Tensor | None = None
    q_norm_weight_txt: torch.Tensor | None = None
    k_norm_weight_txt: torch.Tensor | None = None
    eps: float = 1e-6
    img_freqs: torch.Tensor | None = None
    txt_freqs: torch.Tensor | None = None

    def to_c(self, device):
        keep = []

        def weight(w):
            if w is None:
                return None
            w = _prep_operand(w, device, torch.float32)
            if w.numel() != 128:
                raise ValueError("Qwen norm weights are per head channel: 128 values")
            keep.append(w)
            return w.data_ptr()

        def table(t, rows):
            if t is None:
                return None
            if t.dim() != 2 or not t.is_complex() or t.shape[1] != 64:
                raise ValueError("rotary tables must be complex [rows, 64]")
            if t.shape[0] < rows:
                raise ValueError(f"rotary table has {t.shape[0]} rows, the segment {rows}")
            t = torch.view_as_real(_prep_operand(t, device, torch.complex64))
            keep.append(t)
            return t.data_ptr()

        c = _capi.Prep()
        c.kind = _capi.PREP_QWEN
        c.txt_len = int(self.txt_len)
        c.norm_eps = float(self.eps)
        c.q_norm_weight, c.k_norm_weight = weight(self.q_norm_weight), weight(self.k_norm_weight)
        c.q_norm_weight_txt, c.k_norm_weight_txt = weight(self.q_norm_weight_txt), weight(self.k_norm_weight_txt)
        c.rope_freqs_txt = table(self.txt_freqs, self.txt_len)
        c.rope_freqs_img = table(self.img_freqs, 0)  # its length is checked against L by the caller
        return c, keep


def _as_heads(x: torch.Tensor, num_heads: int | None) -> torch.Tensor:
    """``[B, L, H*D]`` projection -> ``[B, L, H, D]`` view (4-D tensors pass through)."""
    if x.dim() == 4:
        return x
    if x.dim() != 3 or num_heads is None or x.shape[-1] % num_heads:
        raise ValueError("a projection must be [B, L, H*D] with num_heads given, or already [B, L, H, D]")
    return x.view(x.shape[0], x.shape[1], num_heads, x.shape[-1] // num_heads)


def workspace_for(q: torch.Tensor, k: torch.Tensor) -> SageWorkspace:
    B, Lq, Hq, D = q.shape
    _, Lk, Hkv, _ = k.shape
    return SageWorkspace.allocate(B, Hq, Hkv, Lq, Lk, D, q.device)


def _check_qwen_rows(prep, L: int) -> None:
    """The tables of a ``QwenPrep`` must cover their segments: the kernels index them by row without a bound."""
    if not isinstance(prep, QwenPrep):
        return
    if prep.img_freqs is not None and prep.img_freqs.shape[0] < L - prep.txt_len:
        raise ValueError(f"img_freqs has {prep.img_freqs.shape[0]} rows, the image segment {L - prep.txt_len}")
    if prep.txt_freqs is not None and prep.txt_freqs.shape[0] < min(prep.txt_len, L):
        raise ValueError(f"txt_freqs has {prep.txt_freqs.shape[0]} rows, the text segment {min(prep.txt_len, L)}")


def quant_q(q: torch.Tensor, ws: SageWorkspace, sm_scale: float, prep: "WanPrep | QwenPrep | None" = None) -> None:
    _require_hip(q)
    ws.require(q.device, B=q.shape[0], Lq=q.shape[1], Hq=q.shape[2], D=q.shape[3])
    q = _usable(q)
    lib = _capi.load()
    if prep is None:
        rc = lib.ksana_sage_quant_q(q.data_ptr(), _DTYPES[q.dtype], _strides(q), C.byref(ws.shape), sm_scale, ws.ptr,
                                    _stream_ptr(q.device))
    else:
        _check_qwen_rows(prep, q.shape[1])
        c_prep, _keep = prep.to_c(q.device)
        rc = lib.ksana_sage_quant_q_prep(q.data_ptr(), _DTYPES[q.dtype], _strides(q), C.byref(ws.shape),
                                         C.byref(c_prep), sm_scale, ws.ptr, _stream_ptr(q.device))
    _capi.check(rc, "ksana_sage_quant_q")


def quant_k(k: torch.Tensor, ws: SageWorkspace, smooth_k: bool = True, prep: "WanPrep | QwenPrep | None" = None) -> None:
    _require_hip(k)
    ws.require(k.device, B=k.shape[0], Lk=k.shape[1], Hkv=k.shape[2], D=k.shape[3])
    k = _usable(k)
    lib = _capi.load()
    if prep is None:
        rc = lib.ksana_sage_quant_k(k.data_ptr(), _DTYPES[k.dtype], _strides(k), C.byref(ws.shape), int(smooth_k),
                                    ws.ptr, _stream_ptr(k.device))
    else:
        _check_qwen_rows(prep, k.shape[1])
        c_prep, _keep = prep.to_c(k.device)
        rc = lib.ksana_sage_quant_k_prep(k.data_ptr(), _DTYPES[k.dtype], _strides(k), C.byref(ws.shape),
                                         C.byref(c_prep), int(smooth_k), ws.ptr, _stream_ptr(k.device))
    _capi.check(rc, "ksana_sage_quant_k")


def quant_qk(q: torch.Tensor, k: torch.Tensor, ws: SageWorkspace, sm_scale: float, smooth_k: bool = True,
             prep: "WanPrep | QwenPrep | None" = None) -> None:
    """``quant_q`` and ``quant_k`` as one call: the same bits in the same workspace areas.  With a ``prep`` whose norm
    runs over the whole token row, q's kernel takes whole rows anyway and brings k's row statistic along, which saves
    k a pass over its input (``ksana_sage_quant_qk_prep``)."""
    if prep is None:
        quant_q(q, ws, sm_scale)
        quant_k(k, ws, smooth_k)
        return
    _require_hip(q)
    _require_hip(k)
    ws.require(q.device, B=q.shape[0], Lq=q.shape[1], Hq=q.shape[2], D=q.shape[3])
    ws.require(k.device, B=k.shape[0], Lk=k.shape[1], Hkv=k.shape[2], D=k.shape[3])
    if k.dtype != q.dtype:
        raise ValueError("q and k must have the same dtype")
    q, k = _usable(q), _usable(k)
    _check_qwen_rows(prep, q.shape[1])
    _check_qwen_rows(prep, k.shape[1])
    c_prep, _keep = prep.to_c(q.device)
    rc = _capi.load().ksana_sage_quant_qk_prep(q.data_ptr(), k.data_ptr(), _DTYPES[q.dtype], _strides(q), _strides(k),
                                               C.byref(ws.shape), C.byref(c_prep), sm_scale, int(smooth_k), ws.ptr,
                                               _stream_ptr(q.device))
    _capi.check(rc, "ksana_sage_quant_qk_prep")


def quant_v(v: torch.Tensor, ws: SageWorkspace, smooth_v: bool = False) -> None:
    """``smooth_v``: take the channel means off before scaling; the attention adds them back to its output."""
    _require_hip(v)
    ws.require(v.device, B=v.shape[0], Lk=v.shape[1], Hkv=v.shape[2], D=v.shape[3])
    v = _usable(v)
    lib = _capi.load()
    rc = lib.ksana_sage_quant_v_smooth(v.data_ptr(), _DTYPES[v.dtype], _strides(v), C.byref(ws.shape), int(smooth_v),
                                       ws.ptr, _stream_ptr(v.device))
    _capi.check(rc, "ksana_sage_quant_v")


def block_means(x: torch.Tensor, rows: int, centre: torch.Tensor | None = None) -> torch.Tensor:
    """``[B, L, H, D]`` -> ``[B, H, ceil(L / rows), D]`` in ``x.dtype``: the mean of every run of ``rows`` positions (the
    last may be shorter), fp32 sum / count; with ``centre`` (fp32 ``[B, H, D]``) of ``x - centre`` rounded to ``x.dtype``
    first.  The pooling of the reference's ``mean_pool`` (sage_sla.py:43-75) on the layout the blocks hand over."""
    _require_hip(x)
    if x.dim() != 4 or x.shape[3] != 128:
        raise ValueError("block_means expects [B, L, H, 128]")
    x = _usable(x)
    B, L, H, D = x.shape
    if centre is not None:
        if centre.shape != (B, H, D) or centre.dtype != torch.float32 or centre.device != x.device:
            raise ValueError(f"centre must be float32 [{B}, {H}, {D}] on {x.device}")
        centre = centre.contiguous()
    out = torch.empty((B, H, -(-L // rows), D), dtype=x.dtype, device=x.device)
    rc = _capi.load().ksana_sage_block_means(x.data_ptr(), _DTYPES[x.dtype], _strides(x), B, H, L, rows,
                                             None if centre is None else centre.data_ptr(), out.data_ptr(),
                                             _stream_ptr(x.device))
    _capi.check(rc, "ksana_sage_block_means")
    return out


def quant_qk_pooled(q: torch.Tensor, k: torch.Tensor, ws: SageWorkspace, sm_scale: float) -> tuple[torch.Tensor, torch.Tensor]:
    """``quant_q`` + ``quant_k`` (with K smoothing) that hand back the block averages the sparse-linear backend builds
    its block map from: ``block_means(q, 128)`` and ``block_means(k, 64, centre=ws.k_mean)``, bit for bit, without the
    two extra passes over q and k (the quantizers' workgroups are those blocks).  ``[B, L, H, 128]`` tensors."""
    _require_hip(q, k)
    if q.dim() != 4 or k.dim() != 4 or q.shape[3] != 128 or k.shape[3] != 128 or q.dtype != k.dtype:
        raise ValueError("quant_qk_pooled expects [B, L, H, 128] tensors of one dtype")
    ws.require(q.device, B=q.shape[0], Lq=q.shape[1], Hq=q.shape[2], D=q.shape[3])
    ws.require(k.device, B=k.shape[0], Lk=k.shape[1], Hkv=k.shape[2], D=k.shape[3])
    q, k = _usable(q), _usable(k)
    B, Lq, Hq, D = q.shape
    pooled_q = torch.empty((B, Hq, -(-Lq // MASK_BLKQ), D), dtype=q.dtype, device=q.device)
    pooled_k = torch.empty((B, k.shape[2], -(-k.shape[1] // MASK_BLKK), D), dtype=k.dtype, device=k.device)
    rc = _capi.load().ksana_sage_quant_qk_pooled(q.data_ptr(), k.data_ptr(), _DTYPES[q.dtype], _strides(q), _strides(k),
                                                 C.byref(ws.shape), sm_scale, pooled_q.data_ptr(), pooled_k.data_ptr(),
                                                 ws.ptr, _stream_ptr(q.device))
    _capi.check(rc, "ksana_sage_quant_qk_pooled")
    return pooled_q, pooled_k


def sla_block_map(pooled_q: torch.Tensor, pooled_k: torch.Tensor, keep: int) -> torch.Tensor:
    """int8 ``[B, H, nq, nk]``: per query block ones at the ``keep`` key blocks with the largest
    ``pooled_q @ pooled_k^T`` (a tensor of the blocks' dtype); the second half of ``get_block_map`` (sage_sla.py:83-90).
    ``pooled_*``: ``[B, H, n, 128]`` block averages on a HIP device, at most 1024 key blocks."""
    _require_hip(pooled_q, pooled_k)
    if pooled_q.dim() != 4 or pooled_k.dim() != 4 or pooled_q.shape[:2] != pooled_k.shape[:2] or pooled_q.shape[3] != 128 \
            or pooled_k.shape[3] != 128:
        raise ValueError("pooled blocks must be [B, H, n, 128] with equal B, H")
    pooled_q, pooled_k = pooled_q.contiguous(), pooled_k.contiguous()
    B, H, nq, _ = pooled_q.shape
    nk = pooled_k.shape[2]
    block_map = torch.empty((B, H, nq, nk), dtype=torch.int8, device=pooled_q.device)
    rc = _capi.load().ksana_sage_sla_block_map(pooled_q.data_ptr(), pooled_k.data_ptr(), _DTYPES[pooled_q.dtype], B, H, nq, nk,
                                               int(keep), block_map.data_ptr(), _stream_ptr(pooled_q.device))
    _capi.check(rc, "ksana_sage_sla_block_map")
    return block_map


def sla_linear(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, proj_weight: torch.Tensor | None = None,
               proj_bias: torch.Tensor | None = None, add: torch.Tensor | None = None,
               out: torch.Tensor | None = None) -> torch.Tensor:
    """The linear-attention branch of the sparse-linear backend on ``[B, L, H, 128]`` tensors (sage_sla.py:135-139,
    273-287): ``(phi(q) (phi(k)^T v)) / (1e-5 + phi(q) . sum phi(k))`` with ``phi`` = softmax over the channels, then
    (optionally) the block's linear layer ``proj_weight`` ``[128, 128]`` / ``proj_bias`` ``[128]`` applied to it and
    ``add`` (same shape as q; the sparse branch's result) added - all inside two passes over the inputs.  Returns
    ``[B, L, H, 128]`` in q's dtype; ``out`` may be ``add`` itself."""
    _require_hip(q, k, v)
    if q.dim() != 4 or q.shape[3] != 128 or k.shape != q.shape or v.shape != q.shape:
        raise ValueError("sla_linear expects q, k, v of one shape [B, L, H, 128]")
    q, k, v = _usable(q), _usable(k), _usable(v)
    B, L, H, D = q.shape
    if out is None:
        out = torch.empty((B, L, H, D), dtype=q.dtype, device=q.device)
    if out.shape != q.shape or out.dtype != q.dtype or out.device != q.device or _usable(out) is not out:
        raise ValueError("out must have q's shape, dtype and device, with a unit channel stride")
    if add is not None:
        if add.shape != q.shape or add.dtype != q.dtype or add.device != q.device:
            raise ValueError("add must have q's shape, dtype and device")
        if add is not out:
            add = _usable(add)
    w = b = None
    if proj_weight is not None:
        if tuple(proj_weight.shape) != (D, D):
            raise ValueError(f"proj_weight must be [{D}, {D}]")
        # the layer runs in the tensors' dtype under autocast: the weight is rounded to it first
        w = _prep_operand(_prep_operand(proj_weight, q.device, q.dtype), q.device, torch.float32)
        if proj_bias is not None:
            if proj_bias.numel() != D:
                raise ValueError(f"proj_bias must hold {D} values")
            b = _prep_operand(_prep_operand(proj_bias, q.device, q.dtype), q.device, torch.float32)
    elif proj_bias is not None:
        raise ValueError("proj_bias given without proj_weight")
    lib = _capi.load()
    nbytes = C.c_uint64(0)
    _capi.check(lib.ksana_sage_sla_workspace_bytes(B, H, L, C.byref(nbytes)), "ksana_sage_sla_workspace_bytes")
    scratch = torch.empty(nbytes.value, dtype=torch.uint8, device=q.device)
    rc = lib.ksana_sage_sla_linear(q.data_ptr(), k.data_ptr(), v.data_ptr(), _DTYPES[q.dtype], _strides(q), _strides(k),
                                   _strides(v), B, H, L, None if w is None else w.data_ptr(),
                                   None if b is None else b.data_ptr(), None if add is None else add.data_ptr(),
                                   None if add is None else _strides(add), out.data_ptr(), _strides(out),
                                   scratch.data_ptr(), _stream_ptr(q.device))
    _capi.check(rc, "ksana_sage_sla_linear")
    return out


def quant_status(ws: SageWorkspace) -> tuple[int, int]:
    """``(k_status, v_status)`` of the last K / V quantization on ``ws``: 0, or 1 when a workgroup gave up waiting for
    the others of its head and recomputed the head's statistic from the input (same bits, a slow call; see
    ``ksana_sage_quant_status``).  Synchronises the current stream; for tests."""
    ks, vs = C.c_int(-1), C.c_int(-1)
    rc = _capi.load().ksana_sage_quant_status(ws.ptr, C.byref(ws.shape), _stream_ptr(ws.blob.device), C.byref(ks),
                                              C.byref(vs))
    _capi.check(rc, "ksana_sage_quant_status")
    return ks.value, vs.value


def configure(one_read: str | None = None, wait_ticks: int | None = None) -> None:
    """Process-wide settings of the one-read K / V quantizers (``ksana_sage_configure``): ``one_read`` is a string of
    the letters ``k`` and ``v`` (the stages that read their input once when the shape allows), ``wait_ticks`` the bound
    on a workgroup's wait for its head's statistic in 10 ns ticks (0 / negative: test modes, see the header).
    ``None`` leaves a setting as it is.  Every call re-arms the one-read kernels on all GPUs."""
    rc = _capi.load().ksana_sage_configure(None if one_read is None else one_read.encode(),
                                           _capi.KEEP if wait_ticks is None else int(wait_ticks))
    _capi.check(rc, "ksana_sage_configure")


def one_read_state() -> dict:
    """``{"k": bool, "v": bool, "wait_ticks": int, "demoted": bool}``: the settings above, and whether the library has
    switched the one-read kernels off on the current GPU because a wait ran into its bound there."""
    k, v, t, d = C.c_int(0), C.c_int(0), C.c_int64(0), C.c_int(0)
    _capi.check(_capi.load().ksana_sage_one_read_state(C.byref(k), C.byref(v), C.byref(t), C.byref(d)),
                "ksana_sage_one_read_state")
    return {"k": bool(k.value), "v": bool(v.value), "wait_ticks": t.value, "demoted": bool(d.value)}


_demotion_logged = False


def _log_demotion_once() -> None:
    """Debug aid of the op path: say once that the library fell back to its two-pass quantizers on this GPU."""
    global _demotion_logged
    if _demotion_logged or not log.isEnabledFor(10):  # logging.DEBUG
        return
    if one_read_state()["demoted"]:
        _demotion_logged = True
        log.debug("Sage HIP path: a one-read quantizer workgroup waited longer than %d ticks for its head on this GPU "
                  "(the GPU is probably shared); the two-pass quantizers are used from now on (same bits, about "
                  "15 %% slower) until sage_ops.configure() is called", one_read_state()["wait_ticks"])


def _k_lens_arg(k_lens, batch: int, device: torch.device, name: str = "k_lens"):
    """``k_lens`` / ``q_lens`` as the int32 device array the library reads (kept alive by the caller's reference)."""
    if k_lens is None:
        return None
    k_lens = torch.as_tensor(k_lens)
    if k_lens.dim() != 1 or k_lens.numel() != batch:
        raise ValueError(f"{name} must hold one length per batch entry ({batch}), got shape {tuple(k_lens.shape)}")
    return k_lens.to(device=device, dtype=torch.int32).contiguous()


PAD_D = 128  # channels per row of the quantized operands: head size 64 runs zero-padded to 128
MASK_BLKQ, MASK_BLKK = 128, 64  # query rows / keys per block-mask entry


def _block_mask_arg(block_mask, B: int, H: int, Lq: int, Lk: int, device):
    """``block_mask`` as the int8 device array the library reads, plus its two leading strides.
    Accepts ``[nq, nk]``, ``[H, nq, nk]`` or ``[B, H, nq, nk]`` (size-1 or expanded leading dims broadcast)."""
    if block_mask is None:
        return None, None
    m = torch.as_tensor(block_mask)
    nq, nk = -(-Lq // MASK_BLKQ), -(-Lk // MASK_BLKK)
    while m.dim() < 4:
        m = m.unsqueeze(0)
    if m.dim() != 4 or m.shape[2:] != (nq, nk) or m.shape[0] not in (1, B) or m.shape[1] not in (1, H):
        raise ValueError(f"block_mask must be [.., {nq}, {nk}] with leading dims (1|{B}, 1|{H}), got {tuple(m.shape)}")
    lead_b = 1 if (m.shape[0] == 1 or m.stride(0) == 0) else B
    lead_h = 1 if (m.shape[1] == 1 or m.stride(1) == 0) else H
    m = m[:lead_b, :lead_h].to(device=device, dtype=torch.int8).contiguous()
    strides = (C.c_int64 * 2)(m.stride(0) if lead_b > 1 else 0, m.stride(1) if lead_h > 1 else 0)
    return m, strides


def key_split_plan(ws: SageWorkspace):
    """``(first_workgroup, runs)`` of the cut the dense, non-causal attention call makes for this workspace's shape on
    the current device, or ``None`` when it makes none (see ``ksana_sage_attn_key_split``)."""
    first, runs = C.c_int(0), C.c_int(0)
    _capi.check(_capi.load().ksana_sage_attn_key_split(C.byref(ws.shape), C.byref(first), C.byref(runs)),
                "ksana_sage_attn_key_split")
    return (first.value, runs.value) if runs.value else None


def attn_fwd(ws: SageWorkspace, out: torch.Tensor, causal: bool = False, pwl_exp2: bool = False,
             k_lens=None, block_mask=None, q_lens=None, wg_waves: int | None = None, tile_skip: bool = False) -> torch.Tensor:
    """Attention on the quantized operands in ``ws``.  ``k_lens`` (optional, one int per batch entry): batch ``b``
    attends to keys ``[0, k_lens[b])`` only, the meaning the reference's callers give it (wan_model.py:182-189,
    flash_attn.py:131-139); a batch entry without keys yields zeros.  ``block_mask`` (optional, int8/bool
    ``[B, H, ceil(Lq/128), ceil(Lk/64)]``, leading dims may broadcast): block ``(i, j)`` non-zero lets query rows
    ``128 i ..`` attend to keys ``64 j ..`` - the ``mask_id`` of the reference's block-sparse call
    (radial_sage_attn.py:170-176).  ``q_lens`` (optional, one int per batch entry): only the first ``q_lens[b]`` query
    rows of batch ``b`` are computed, the rest of the output is zeros (flash_attn.py:120-124 packs exactly those rows).
    ``wg_waves`` (4 or 8; default: the library's choice) forces the workgroup shape - for measurements and tests.
    ``tile_skip=True``: a wave leaves out the exponentials of a key tile whose probabilities would all round to the zero
    code (scores more than 17 octaves under every row's reference point): the same bits, faster where attention is
    peaked, ~7 % slower where no tile qualifies - off by default."""
    _require_hip(out)
    if out.dim() != 4:
        raise ValueError("out must be [B, Lq, H, D]")
    ws.require(out.device, B=out.shape[0], Lq=out.shape[1], Hq=out.shape[2], D=out.shape[3])
    lib = _capi.load()
    if wg_waves not in (None, 4, 8):
        raise ValueError("wg_waves must be 4 or 8")
    if tile_skip and pwl_exp2:
        raise ValueError("tile_skip goes with the exact exponential only")
    flags = (_capi.FLAG_PWL_EXP2 if pwl_exp2 else 0) | {None: 0, 4: _capi.FLAG_WG_4_WAVES, 8: _capi.FLAG_WG_8_WAVES}[wg_waves]
    flags |= _capi.FLAG_TILE_SKIP if tile_skip else 0
    kl = _k_lens_arg(k_lens, out.shape[0], out.device)
    ql = _k_lens_arg(q_lens, out.shape[0], out.device, "q_lens")
    s = ws.shape
    mask, mask_st = _block_mask_arg(block_mask, s.B, s.Hq, s.Lq, s.Lk, out.device)
    rc = lib.ksana_sage_attn_fwd_varlen(ws.ptr, out.data_ptr(), _DTYPES[out.dtype], _strides(out), C.byref(ws.shape),
                                        None if mask is None else mask.data_ptr(), mask_st,
                                        None if ql is None else ql.data_ptr(),
                                        None if kl is None else kl.data_ptr(), int(causal), flags,
                                        _stream_ptr(out.device))
    _capi.check(rc, "ksana_sage_attn_fwd")
    return out


def sageattn(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    tensor_layout: str = "NHD",
    is_causal: bool = False,
    sm_scale: float | None = None,
    smooth_k: bool = True,
    workspace: SageWorkspace | None = None,
    pwl_exp2: bool = False,
    k_lens=None,
    prep: WanPrep | None = None,
    block_mask=None,
    out_dtype: torch.dtype | None = None,
    smooth_v: bool = False,
    q_lens=None,
    tile_skip: bool = False,
) -> torch.Tensor:
    """Quantized attention, ``[B, L, H, D]`` ("NHD") or ``[B, H, L, D]`` ("HND") in and out.

    ``k_lens`` (optional, one int per batch entry) limits batch ``b`` to its first ``k_lens[b]`` keys.
    ``q_lens`` (optional, likewise): only the first ``q_lens[b]`` query rows of batch ``b`` are computed; the others
    come out as zeros.
    ``prep`` (optional, "NHD" only): q and k are the raw projections and the block's RMSNorm + RoPE are applied
    while they are read (see ``WanPrep``).
    ``block_mask`` (optional): block-sparse attention, see ``attn_fwd`` (not together with ``prep``).
    ``smooth_v``: quantize V with its channel means taken off and add them back to the output - the ``smooth_v``
    option of the library behind the reference's call (off there, off by default here); worth its extra read of V
    when V's channels sit far from zero.
    ``out_dtype`` (optional, fp16 or bf16): write the result in this dtype instead of q's - the cast the Wan block
    applies before its output projection when the projection's weights want another dtype
    (ksana/models/wan/wan_model.py:197-204), done in the kernel's epilogue from the fp32 accumulators.

    ``pwl_exp2=True`` computes the e4m3 code of every probability directly (exp2 with a
    piecewise-linear mantissa, no transcendental): about 1.2x faster, slightly less accurate.
    ``tile_skip=True`` (exact exponential only): see ``attn_fwd``; same bits, faster on sharply peaked attention."""
    if tile_skip and pwl_exp2:
        raise ValueError("tile_skip goes with the exact exponential only")
    if tensor_layout not in ("NHD", "HND"):
        raise ValueError(f"tensor_layout {tensor_layout!r} unknown")
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("sageattn expects 4-D tensors")
    if tensor_layout == "HND":
        if prep is not None:
            raise ValueError("prep needs the NHD layout (a token row must be contiguous)")
        q, k, v = (t.transpose(1, 2) for t in (q, k, v))
    _require_hip(q, k, v)
    if k.shape != v.shape or q.shape[0] != k.shape[0] or q.shape[3] != k.shape[3]:
        raise ValueError(f"incompatible shapes q{tuple(q.shape)} k{tuple(k.shape)} v{tuple(v.shape)}")
    q, k, v = _usable(q), _usable(k), _usable(v)
    B, Lq, Hq, D = q.shape
    if q.numel() == 0:  # nothing to attend from: same empty result SDPA gives
        out = torch.empty((B, Lq, Hq, D), dtype=q.dtype, device=q.device)
        return out.transpose(1, 2) if tensor_layout == "HND" else out
    sm_scale = D**-0.5 if sm_scale is None else float(sm_scale)
    ws = workspace_for(q, k) if workspace is None else workspace
    ws.require(q.device, B=B, Hq=Hq, Hkv=k.shape[2], Lq=Lq, Lk=k.shape[1], D=D)
    lib = _capi.load()
    _log_demotion_once()
    kl = _k_lens_arg(k_lens, B, q.device)
    flags = (_capi.FLAG_PWL_EXP2 if pwl_exp2 else 0) | (_capi.FLAG_SMOOTH_V if smooth_v else 0)
    flags |= _capi.FLAG_TILE_SKIP if tile_skip else 0
    if prep is not None:
        _check_qwen_rows(prep, Lq)
        _check_qwen_rows(prep, k.shape[1])
    result_dtype = q.dtype if out_dtype is None else out_dtype
    if result_dtype not in _DTYPES:
        raise ValueError(f"out_dtype must be float16 or bfloat16, got {out_dtype}")
    out = torch.empty((B, Lq, Hq, D), dtype=result_dtype, device=q.device)
    if q_lens is not None or result_dtype != q.dtype:
        # the one-call entry points take neither q_lens nor a result dtype of their own: quantize (the quantized
        # operands carry no dtype), then the attention entry point that takes both
        quant_qk(q, k, ws, sm_scale, smooth_k, prep=prep)
        quant_v(v, ws, smooth_v)
        attn_fwd(ws, out, causal=is_causal, pwl_exp2=pwl_exp2, k_lens=kl, block_mask=block_mask, q_lens=q_lens)
        return out.transpose(1, 2) if tensor_layout == "HND" else out
    if block_mask is not None:
        if prep is not None:
            raise ValueError("block_mask and prep cannot be combined in one call; quantize with prep, then attn_fwd")
        mask, mask_st = _block_mask_arg(block_mask, B, Hq, Lq, k.shape[1], q.device)
        rc = lib.ksana_sage_forward_masked(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), _DTYPES[q.dtype],
            _strides(q), _strides(k), _strides(v), _strides(out), C.byref(ws.shape), mask.data_ptr(), mask_st,
            None if kl is None else kl.data_ptr(), sm_scale, int(smooth_k), int(is_causal), flags, ws.ptr,
            _stream_ptr(q.device),
        )
        _capi.check(rc, "ksana_sage_forward_masked")
        return out.transpose(1, 2) if tensor_layout == "HND" else out
    c_prep, _keep = (None, None) if prep is None else prep.to_c(q.device)
    rc = lib.ksana_sage_forward_prep(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), _DTYPES[q.dtype],
        _strides(q), _strides(k), _strides(v), _strides(out), C.byref(ws.shape),
        None if c_prep is None else C.byref(c_prep), None if kl is None else kl.data_ptr(), sm_scale, int(smooth_k),
        int(is_causal), flags, ws.ptr, _stream_ptr(q.device),
    )
    _capi.check(rc, "ksana_sage_forward_prep" if prep is not None else "ksana_sage_forward")
    return out.transpose(1, 2) if tensor_layout == "HND" else out


def wan_self_attention(q_proj: torch.Tensor, k_proj: torch.Tensor, v_proj: torch.Tensor, num_heads: int,
                       prep: WanPrep, **kwargs) -> torch.Tensor:
    """The attention part of ``WanSelfAttention.forward`` from the three projections ``[B, L, H*D]`` on:
    norm_q / norm_k, RoPE, attention (ksana/models/wan/wan_model.py:163-190) -> ``[B, L, H, D]``.
    The normed and rotated q and k are never written to memory."""
    q, k, v = (_as_heads(t, num_heads) for t in (q_proj, k_proj, v_proj))
    return sageattn(q, k, v, tensor_layout="NHD", prep=prep, **kwargs)


def block_sparse_sage2_attn(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask_id: torch.Tensor,
                            tensor_layout: str = "NHD", **kwargs) -> torch.Tensor:
    """Same call shape as the reference's ``block_sparse_sage2_attn_cuda(q, k, v, mask_id=..., tensor_layout="NHD")``
    (ksana/operations/attention/backends/radial_sage_attn/radial_sage_attn.py:24,170-176): ``mask_id`` is
    ``[B, H, ceil(Lq/128), ceil(Lk/64)]``, non-zero = attend."""
    return sageattn(q, k, v, tensor_layout=tensor_layout, block_mask=mask_id, **kwargs)
