"""The radial block-mask generator against masks produced by the reference's own generator
(tests/golden/radial_masks.npz, written by tests/golden/make_radial_mask_golden.py), bit for bit."""

from pathlib import Path

import numpy as np
import torch

from ksanadit_amd.backends.radial_mask import kernel_block_mask, radial_block_mask

GOLD = Path(__file__).resolve().parent / "golden" / "radial_masks.npz"


def _cases():
    z = np.load(GOLD, allow_pickle=False)
    idx = 0
    while f"case{idx}_params" in z:
        s, vtn, nf, bs = (int(x) for x in z[f"case{idx}_params"])
        decay = float(z[f"case{idx}_decay"][0])
        shape = tuple(int(x) for x in z[f"case{idx}_shape"])
        bits = np.unpackbits(z[f"case{idx}_bits"])[: shape[0] * shape[1]].reshape(shape).astype(bool)
        yield (s, vtn, nf, bs, decay), torch.from_numpy(bits)
        idx += 1


def test_generator_reproduces_reference_masks():
    n = 0
    for (s, vtn, nf, bs, decay), want in _cases():
        got = radial_block_mask(s, vtn, nf, bs, decay)
        assert got.shape == want.shape, (s, vtn, nf, bs, decay)
        assert torch.equal(got, want), (s, vtn, nf, bs, decay, int((got != want).sum()))
        n += 1
    assert n >= 8


def test_pattern_properties():
    m = radial_block_mask(4096, 4096, 16, 64, 0.3)
    tpf_blocks = 4096 // 16 // 64
    assert m[:, :tpf_blocks].all()  # the first frame is seen by everyone
    assert torch.diagonal(m).all()  # a block sees itself
    wide = radial_block_mask(4096, 4096, 16, 64, 0.9)
    assert (wide | ~m).all()  # a larger decay factor never removes a block
    assert 0.3 < m.float().mean() < 0.9
    # text tokens behind the video are dense in both directions
    t = radial_block_mask(2048, 1920, 5, 128, 0.5)
    assert t[15].all() and t[:, 15].all()


def test_kernel_mask_shapes_and_clipping():
    m = radial_block_mask(2048, 1920, 5, 128, 0.5)
    k = kernel_block_mask(m, 128, 2048)
    assert k.shape == (16, 32) and k.dtype == torch.int8
    assert torch.equal(k[:, 0::2].bool(), m) and torch.equal(k[:, 1::2].bool(), m)
    m64 = radial_block_mask(2048, 1920, 5, 64, 0.02)
    k64 = kernel_block_mask(m64, 64, 2048)
    assert k64.shape == (16, 32)
    assert torch.equal(k64.bool(), m64.view(16, 2, 32).any(dim=1))
    # a sequence that is not a whole number of blocks: the ragged end is dense
    r = radial_block_mask(32760, 32760, 21, 128, 0.2)  # the reference raises here; this generator clips
    kr = kernel_block_mask(r, 128, 32760)
    assert r.shape == (255, 255) and kr.shape == (256, 512)
    assert kr[255].all() and kr[:, 510:].all()
