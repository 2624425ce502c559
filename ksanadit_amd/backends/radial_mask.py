"""Block masks of the radial ("log-sparse") attention pattern, host side.

Behaviour follows ksana/operations/attention/backends/radial_sage_attn/attn_mask.py (which credits
mit-han-lab/radial-attention): tokens are laid out frame after frame; a query frame ``i`` sees key frame ``j``

* completely when ``j == 0`` (attention sink, attn_mask.py:84-85);
* otherwise through a band ``|c - r| <= width(i, j)`` of in-frame token distances (attn_mask.py:55-64, 87-88):
  the whole frame at distance 0, half of it at distance 1, then ``2^bitlen(tokens per frame) / 2^bitlen(dist)
  * decay_factor`` but never less than one block;
* and, once that band has shrunk below one block, only for every ``split``-th frame distance
  (attn_mask.py:37-52).

The token-level pattern of each frame pair is reduced to blocks by the rule of ``shrink_mask_strict``
(attn_mask.py:21-34): a block is kept when more than 60 % of its non-empty columns are more than one third
full.  Everything at or beyond ``video_token_num`` (text tokens) is dense (attn_mask.py:78-79, 119-131).

The result is compared bit for bit with masks the reference's generator produced
(tests/golden/radial_masks.npz).  One difference on purpose: a frame whose padded block range runs past the
end of the mask is clipped here; the reference raises a shape error on such inputs.
"""

from __future__ import annotations

import torch


def _band_width(dist: int, tokens_per_frame: int, decay_factor: float, block_size: int) -> float:
    if dist < 1:
        return tokens_per_frame
    if dist == 1:
        return tokens_per_frame // 2
    return max(2 ** tokens_per_frame.bit_length() / 2 ** dist.bit_length() * decay_factor, block_size)


def _frame_distance_kept(dist: int, tokens_per_frame: int, block_size: int) -> bool:
    """False for the frame distances the pattern drops entirely once its band is narrower than a block."""
    reach = 2 ** tokens_per_frame.bit_length() / 2 ** dist.bit_length()
    if reach >= block_size:
        return True
    return dist % int(block_size / reach) == 0


def _blocks_of_frame_pair(token_mask: torch.Tensor, row_off: int, col_off: int, block_size: int) -> torch.Tensor:
    """Token pattern of one frame pair, placed at its offset inside the first block, reduced to blocks."""
    n = token_mask.shape[0]
    nblk = (n - 1) // block_size + 1
    padded = torch.zeros((row_off + nblk * block_size, col_off + nblk * block_size), dtype=torch.bool)
    padded[row_off : row_off + n, col_off : col_off + n] = token_mask
    # the reference cuts the padded pattern to nblk x nblk whole blocks before it counts
    tiles = padded[: nblk * block_size, : nblk * block_size].view(nblk, block_size, nblk, block_size)
    fill = tiles.sum(dim=1) / block_size  # [row block, col block, column]: share of the block's rows that are set
    touched = fill > 0
    well_filled = fill > 1 / 3
    share = well_filled.sum(dim=-1) / (touched.sum(dim=-1) + 1e-9)
    return share > 0.6


def radial_block_mask(seq_len: int, video_token_num: int, num_frame: int, block_size: int = 128,
                      decay_factor: float = 0.5) -> torch.Tensor:
    """bool ``[seq_len // block_size, seq_len // block_size]`` (what ``MaskMap.query_log_mask`` returns,
    attn_mask.py:119-131): video blocks follow the radial pattern, everything else is dense."""
    nb = seq_len // block_size
    tpf = video_token_num // num_frame
    border = video_token_num // block_size
    pattern = torch.zeros((nb, nb), dtype=torch.bool)
    pattern[border:] = True
    pattern[:, border:] = True
    r = torch.arange(tpf).view(-1, 1)
    c = torch.arange(tpf).view(1, -1)
    gap = (c - r).abs()
    for i in range(num_frame):
        for j in range(num_frame):
            if j == 0:
                tokens = torch.ones((tpf, tpf), dtype=torch.bool)
            elif _frame_distance_kept(abs(i - j), tpf, block_size):
                tokens = gap <= _band_width(abs(i - j), tpf, decay_factor, block_size)
            else:
                continue  # an empty pattern sets no block
            blocks = _blocks_of_frame_pair(tokens, (i * tpf) % block_size, (j * tpf) % block_size, block_size)
            r0, c0 = (i * tpf) // block_size, (j * tpf) // block_size
            rows, cols = min(blocks.shape[0], nb - r0), min(blocks.shape[1], nb - c0)
            if rows > 0 and cols > 0:
                pattern[r0 : r0 + rows, c0 : c0 + cols] |= blocks[:rows, :cols]
    out = torch.ones((nb, nb), dtype=torch.bool)
    out[:border, :border] = pattern[:border, :border]
    return out


def kernel_block_mask(mask: torch.Tensor, block_size: int, seq_len: int) -> torch.Tensor:
    """``[seq/bs, seq/bs]`` -> int8 ``[ceil(seq/128), ceil(seq/64)]`` for the attention kernel: 128 query rows per
    mask row, 64 keys per column (radial_sage_attn.py:150-157).  Blocks the source mask does not cover (a ragged
    end of the sequence) are dense, like the text region."""
    if block_size == 128:
        m = torch.repeat_interleave(mask, 2, dim=1)
    elif block_size == 64:
        rows = mask.shape[0] // 2
        m = mask[: 2 * rows].view(rows, 2, mask.shape[1]).max(dim=1).values
        if mask.shape[0] % 2:
            m = torch.cat([m, mask[-1:]], dim=0)
    else:
        raise ValueError(f"block_size must be 64 or 128, got {block_size}")
    nq, nk = -(-seq_len // 128), -(-seq_len // 64)
    out = torch.ones((nq, nk), dtype=torch.bool)
    out[: min(nq, m.shape[0]), : min(nk, m.shape[1])] = m[:nq, :nk]
    return out.to(torch.int8)
