"""Pins oracle/vit_index.py (CPU only).

Checks, each chosen so that a plausible mistake fails it:
  * committed fixtures from transformers.vision_utils (same algorithm as qwen2_5_vl.py:357-386,436);
  * the worked values recorded for grid (1,32,32) and (8,24,42);
  * an independent closed-form enumeration on every even grid up to 28x28, t <= 3 (brute force);
  * invariants: permutation, strictly increasing cu, argsort o gather = identity;
  * a live comparison with transformers.vision_utils when it is importable.
"""

import hashlib
import json

import numpy as np
import pytest

from oracle import vit_index as vi


def _sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


@pytest.fixture(scope="module")
def golden(golden_dir):
    return json.loads((golden_dir / "index_golden.json").read_text())


def test_golden_fixtures(golden):
    assert len(golden) >= 7
    for name, rec in golden.items():
        grids = rec["grids"]
        wi, cu = vi.get_window_index(grids)
        assert wi.dtype == np.int64 and wi.shape[0] == rec["window_index_len"], name
        assert _sha(wi) == rec["window_index_sha256_int64"], name
        if "window_index" in rec:
            assert wi.tolist() == rec["window_index"], name
        else:
            assert wi[:64].tolist() == rec["window_index_head"], name
        assert cu.tolist() == rec["cu_window_seqlens"], name
        assert vi.full_cu_seqlens(grids).tolist() == rec["cu_seqlens"], name
        pos = vi.rot_pos_ids(grids)
        assert list(pos.shape) == rec["pos_ids_shape"], name
        assert _sha(pos) == rec["pos_ids_sha256_int64"], name
        if "pos_ids" in rec:
            assert pos.tolist() == rec["pos_ids"], name


def test_worked_values():
    wi, cu = vi.get_window_index([(1, 32, 32)])
    assert cu.tolist() == list(range(0, 1025, 64))
    assert wi[:20].tolist() == [0, 1, 2, 3, 16, 17, 18, 19, 32, 33, 34, 35, 48, 49, 50, 51, 4, 5, 6, 7]
    wi, cu = vi.get_window_index([(8, 24, 42)] * 2)
    lens = np.diff(cu)
    assert len(lens) == 288 and lens.min() == 16 and lens.max() == 64 and cu[-1] == 16128
    assert vi.full_cu_seqlens([(8, 24, 42)] * 2).tolist() == list(range(0, 16129, 1008))
    pos = vi.rot_pos_ids([(1, 4, 4)])
    assert pos.tolist() == [[0, 0], [0, 1], [1, 0], [1, 1], [0, 2], [0, 3], [1, 2], [1, 3],
                            [2, 0], [2, 1], [3, 0], [3, 1], [2, 2], [2, 3], [3, 2], [3, 3]]


def test_brute_force_against_closed_form():
    for t in (1, 2, 3):
        for h in range(2, 30, 2):
            for w in range(2, 30, 2):
                grids = [(t, h, w), (1, w, h)]
                wi, cu = vi.get_window_index(grids)
                wi2, cu2 = vi.window_index_closed_form(grids)
                assert np.array_equal(wi, wi2), grids
                assert np.array_equal(cu, cu2), grids


def test_invariants():
    rng = np.random.default_rng(0)
    for _ in range(25):
        n = int(rng.integers(1, 5))
        grids = [(int(rng.integers(1, 4)), int(rng.integers(1, 40)) * 2, int(rng.integers(1, 40)) * 2) for _ in range(n)]
        wi, cu = vi.get_window_index(grids)
        U = sum(t * (h // 2) * (w // 2) for t, h, w in grids)
        assert np.array_equal(np.sort(wi), np.arange(U))
        d = np.diff(cu)
        assert cu[0] == 0 and cu[-1] == 4 * U and (d > 0).all() and (d % 4 == 0).all() and d.max() <= 64
        x = rng.standard_normal(U)
        assert np.array_equal(x[wi][np.argsort(wi)], x)
        pos = vi.rot_pos_ids(grids)
        assert pos.shape == (4 * U, 2)
        # every (h, w) of every frame appears exactly once per frame
        off = 0
        for t, h, w in grids:
            for _f in range(t):
                fr = pos[off : off + h * w]
                assert len({(int(a), int(b)) for a, b in fr}) == h * w
                assert fr[:, 0].max() == h - 1 and fr[:, 1].max() == w - 1
                off += h * w


def test_live_transformers_cross_check():
    vu = pytest.importorskip("transformers.vision_utils")
    import torch

    rng = np.random.default_rng(1)
    for _ in range(12):
        n = int(rng.integers(1, 4))
        grids = [(int(rng.integers(1, 4)), int(rng.integers(1, 31)) * 2, int(rng.integers(1, 31)) * 2) for _ in range(n)]
        g = torch.tensor(grids, dtype=torch.int64)
        wi_t, cu_t = vu.get_vision_window_index(g, spatial_merge_size=2, window_size=112, patch_size=14)
        wi, cu = vi.get_window_index(grids)
        assert wi.tolist() == wi_t.tolist() and cu.tolist() == cu_t.tolist()
        assert vi.rot_pos_ids(grids).tolist() == vu.get_vision_position_ids(g, 2).tolist()
        assert vi.full_cu_seqlens(grids).tolist() == vu.get_vision_cu_seqlens(g).tolist()
