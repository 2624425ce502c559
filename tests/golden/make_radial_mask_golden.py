"""Writes tests/golden/radial_masks.npz: block masks produced by the reference's own radial mask generator
(ksana/operations/attention/backends/radial_sage_attn/attn_mask.py, loaded as a stand-alone module: it imports
only torch and tqdm) for a handful of small configurations.  Nothing else in the reference's tests or fixtures
observes these masks, so this is the only way to pin ksanadit_amd/backends/radial_mask.py bit for bit.

Run in the build container only (the reference tree does not travel):
    python tests/golden/make_radial_mask_golden.py
"""

import importlib.util
import sys
from pathlib import Path

import numpy as np
import torch

REF = Path("/root/reference/ksana/operations/attention/backends/radial_sage_attn/attn_mask.py")
OUT = Path(__file__).resolve().parent / "radial_masks.npz"

# (seq_len, video_token_num, num_frame, block_size, decay_factor)
CASES = [
    (1536, 1536, 6, 128, 0.2),
    (1536, 1536, 6, 64, 0.2),
    (2048, 1920, 5, 128, 0.5),   # 128 text tokens behind the video tokens
    (2048, 1920, 5, 64, 0.02),
    (3328, 3120, 8, 128, 0.1),   # 390 tokens per frame: frames do not start on block boundaries
    (3328, 3120, 8, 64, 0.9),
    (4096, 4096, 16, 64, 0.3),
    (8192, 7800, 5, 128, 0.05),  # 1560 tokens per frame as in the 480p model, 5 frames
]


def main() -> int:
    spec = importlib.util.spec_from_file_location("ref_attn_mask", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    out = {}
    for idx, (s, vtn, nf, bs, decay) in enumerate(CASES):
        mm = mod.MaskMap(video_token_num=vtn, num_frame=nf, block_size=bs, device="cpu")
        try:
            mask = mm.query_log_mask(s, "radial", block_size=bs, decay_factor=decay)
        except RuntimeError as exc:  # the generator itself rejects some shapes (a frame's padded blocks overrun the mask)
            print(f"case {idx} {(s, vtn, nf, bs, decay)}: reference raised {exc}", file=sys.stderr)
            raise
        out[f"case{idx}_params"] = np.array([s, vtn, nf, bs], dtype=np.int64)
        out[f"case{idx}_decay"] = np.array([decay], dtype=np.float64)
        out[f"case{idx}_shape"] = np.array(mask.shape, dtype=np.int64)
        out[f"case{idx}_bits"] = np.packbits(mask.to(torch.uint8).numpy().reshape(-1))
        print(f"case {idx}: {tuple(mask.shape)} density {mask.float().mean():.4f}", file=sys.stderr)
    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes)", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
