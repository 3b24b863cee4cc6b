"""The item lists of the chunk kernels (fm_pf_group / fm_pf_rows, finchmoe_amd/csrc/fm_prefill.hip)
against what the launcher sizes: every item list within its allocation and a workgroup's share
of the rounds within the 64 items it keeps one per lane — restated here in Python over random
routings.  (The split of the decode launch is walked by tests/test_host_bounds.py on the functions
the kernel itself calls.)  No GPU."""
import itertools

import pytest

FM_NW, FM_WAVE = 8, 64


def _items(counts, tm):
    """fm_pf_group: every expert's positions cut into items of at most tm."""
    items, off = [], 0
    for e, c in enumerate(counts):
        for s in range((c + tm - 1) // tm):
            items.append((e, off + s * tm, min(tm, c - s * tm)))
        off += c
    return items


def _pfr_grid(max_items, n_cu):
    need = (max_items + 31) // 32
    return max(need, n_cu)


@pytest.mark.parametrize("seed", range(6))
def test_chunk_items_fit_their_lists_and_a_share_its_lanes(seed):
    """What the launcher sizes on the host — the two item lists in the workspace
    (fm_prefill_affine_ws_bytes) and the grid of a row-tile launch (pfr_grid) — against what
    fm_pf_group writes and a workgroup of fm_pf_rows keeps per lane (the items of its share, one
    per lane of a wave: at most 64), for uniform, skewed and degenerate routings."""
    import numpy as np
    rng = np.random.default_rng(seed)
    for trial in range(60):
        E = int(rng.choice([1, 7, 64, 256, 1024]))
        M = int(rng.choice([32, 33, 100, 512, 2048, 8192]))
        K = int(rng.integers(1, 9))
        n = M * K
        kind = trial % 4
        if kind == 0:
            idx = rng.integers(0, E, n)
        elif kind == 1:                                   # everything on one expert
            idx = np.full(n, int(rng.integers(0, E)))
        elif kind == 2:                                   # Zipf-like
            p = (np.arange(E) + 1.0) ** -1.1
            idx = rng.choice(E, n, p=p / p.sum())
        else:                                             # some indices outside the store: skipped
            idx = rng.integers(-3, E + 3, n)
        counts = np.bincount(idx[(idx >= 0) & (idx < E)], minlength=E)
        for tm, rows_per_task, out_rows in ((16, 16, 512), (8, 16, 512), (16, 32, 2048)):
            items = _items(counts, tm)
            assert len(items) <= E + n // tm + 1                      # the list in the workspace
            assert sum(c for _, _, c in items) == counts.sum()
            rpi = out_rows // rows_per_task // 8                      # rounds per item
            for n_cu in (256, 64):
                grid = _pfr_grid(E + n // tm, n_cu)
                RT = len(items) * rpi
                for share in (0, grid // 2, grid - 1, int(rng.integers(0, grid))):
                    r0, r1 = RT * share // grid, RT * (share + 1) // grid
                    if r0 >= r1:
                        continue
                    it0, it_last = r0 // rpi, (r1 - 1) // rpi
                    assert it_last < len(items)
                    assert it_last - it0 < 64, (E, M, K, tm, n_cu, share)
