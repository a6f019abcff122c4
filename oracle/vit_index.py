"""ORACLE (test infrastructure, never on the product path): integer routines of the Qwen2.5-VL encoder.

A numpy restatement, step for step, of the reference's index code:

* `get_window_index`      follows eric/models/qwen2_5_vl.py:357-386 (pad with -100, reshape into windows,
                          boolean compaction) and the `unique_consecutive` at :431-436;
* `rot_pos_ids`           follows rot_pos_emb, :325-351 (position ids in 2x2-block-major order);
* `full_cu_seqlens`       follows :445-448 (one segment per frame);
* `rope_angles`           follows Qwen2_5_VisionRotaryEmbedding :236-259 and :352-354.

Pinned by tests/test_oracle_index.py: hand-worked values for two grids ((1,32,32): 16 windows of 64; and
(8,24,42): 288 segments of 16 to 64), the independent closed form, permutation/monotonicity invariants on every even grid up to
28x28 with t <= 3, the committed fixtures in tests/golden/index_*.json (written from the installed
third-party `transformers.vision_utils`, which carries the same algorithm), and, when `transformers`
is importable, a live comparison against it.
"""

from __future__ import annotations

import numpy as np


def get_window_index(grid_thw, window_size: int = 112, spatial_merge_size: int = 2, patch_size: int = 14):
    """Returns (window_index int64 [U], cu_window_seqlens int32 after unique_consecutive)."""
    grid_thw = np.asarray(grid_thw, dtype=np.int64).reshape(-1, 3)
    window_index = []
    cu_window_seqlens = [0]
    window_index_id = 0
    win = window_size // spatial_merge_size // patch_size
    unit = spatial_merge_size * spatial_merge_size
    for grid_t, grid_h, grid_w in grid_thw:
        llm_h, llm_w = int(grid_h) // spatial_merge_size, int(grid_w) // spatial_merge_size
        index = np.arange(grid_t * llm_h * llm_w, dtype=np.int64).reshape(grid_t, llm_h, llm_w)
        pad_h = win - llm_h % win
        pad_w = win - llm_w % win
        nwh = (llm_h + pad_h) // win
        nww = (llm_w + pad_w) // win
        padded = np.pad(index, ((0, 0), (0, pad_h), (0, pad_w)), constant_values=-100)
        padded = padded.reshape(grid_t, nwh, win, nww, win).transpose(0, 1, 3, 2, 4)
        padded = padded.reshape(grid_t, nwh * nww, win, win)
        seqlens = (padded != -100).sum(axis=(2, 3)).reshape(-1)
        flat = padded.reshape(-1)
        window_index.append(flat[flat != -100] + window_index_id)
        cu = np.cumsum(seqlens) * unit + cu_window_seqlens[-1]
        cu_window_seqlens.extend(int(v) for v in cu)
        window_index_id += int(grid_t * llm_h * llm_w)
    window_index = np.concatenate(window_index) if window_index else np.zeros(0, np.int64)
    cu = np.asarray(cu_window_seqlens, dtype=np.int32)
    # torch.unique_consecutive
    keep = np.ones(cu.shape[0], dtype=bool)
    keep[1:] = cu[1:] != cu[:-1]
    return window_index.astype(np.int64), cu[keep]


def rot_pos_ids(grid_thw, spatial_merge_size: int = 2) -> np.ndarray:
    """int64 [L, 2]: (h, w) position of every patch row, in the 2x2-block-major input order."""
    grid_thw = np.asarray(grid_thw, dtype=np.int64).reshape(-1, 3)
    m = spatial_merge_size
    out = []
    for t, h, w in grid_thw:
        t, h, w = int(t), int(h), int(w)
        hpos = np.broadcast_to(np.arange(h)[:, None], (h, w))
        wpos = np.broadcast_to(np.arange(w)[None, :], (h, w))
        hpos = hpos.reshape(h // m, m, w // m, m).transpose(0, 2, 1, 3).reshape(-1)
        wpos = wpos.reshape(h // m, m, w // m, m).transpose(0, 2, 1, 3).reshape(-1)
        out.append(np.tile(np.stack([hpos, wpos], axis=-1), (t, 1)))
    return np.concatenate(out, axis=0).astype(np.int64) if out else np.zeros((0, 2), np.int64)


def full_cu_seqlens(grid_thw) -> np.ndarray:
    """int32 [sum(t)+1]: repeat_interleave(h*w, t).cumsum() with a leading 0."""
    grid_thw = np.asarray(grid_thw, dtype=np.int64).reshape(-1, 3)
    lens = np.repeat(grid_thw[:, 1] * grid_thw[:, 2], grid_thw[:, 0])
    return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)


def window_index_closed_form(grid_thw, win: int = 4, merge: int = 2):
    """Independent derivation used only to pin `get_window_index`: enumerate non-empty windows in
    (item, frame, window row, window col) order and their units row-major."""
    grid_thw = np.asarray(grid_thw, dtype=np.int64).reshape(-1, 3)
    idx, cu, base, run = [], [0], 0, 0
    for t, h, w in grid_thw:
        gh, gw = int(h) // merge, int(w) // merge
        for f in range(int(t)):
            for wr in range(0, gh, win):
                for wc in range(0, gw, win):
                    rows = range(wr, min(wr + win, gh))
                    cols = range(wc, min(wc + win, gw))
                    for r in rows:
                        for c in cols:
                            idx.append(base + f * gh * gw + r * gw + c)
                    run += len(rows) * len(cols) * merge * merge
                    cu.append(run)
        base += int(t) * gh * gw
    return np.asarray(idx, np.int64), np.asarray(cu, np.int32)
