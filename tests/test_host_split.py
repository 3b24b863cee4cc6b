"""The work split of the decode launch that sums the experts in LDS (fm_moe_fused_rows,
finchmoe_amd/csrc/fm_decode.hip): what the launcher checks on the host (launch_fused_rows) must
be enough for what the kernel computes from the same numbers (Fm2Stream::run) — every gate/up
unit and every down row block handed out exactly once, at most two gate/up segments per
workgroup, segment tables and the per-part LDS area within their fixed sizes, 32-bit products
that do not overflow.  Both pieces of arithmetic are restated here in Python, line by line, and
run over a grid of shapes (layers or positions 1..96, K 1..8, three widths, several CU counts);
a change to either place in the HIP source has to be mirrored here.  No GPU."""
import itertools

import pytest

FM_NW, FM_WAVE = 8, 64
FM2_MAX_SEG, FM2_PART_BYTES = 12, 12288


def launcher(n_groups, K, hidden, inter, n_cu):
    """launch_fused_rows: the grid, or None when it answers FM_ERR_UNSUPPORTED."""
    lpr_up = hidden // 128
    rps_up, rps_dn = FM_WAVE // lpr_up, FM_WAVE // (lpr_up // 4)
    gu_segu, dn_rbs = (inter // rps_up) * K, hidden // rps_dn
    up_units, rb_total = n_groups * gu_segu, n_groups * dn_rbs
    wgs = n_cu
    small = min(up_units, rb_total * K)
    if small < FM_NW * wgs:
        wgs = (small + FM_NW - 1) // FM_NW
    wgs = max(wgs, 1)
    s_total = 2 * up_units + rb_total * K
    up_share = (s_total // wgs + 1) // 2 + 1
    if up_share > gu_segu or s_total * wgs >= 1 << 31:
        return None
    if wgs >= n_groups:
        n_dn = 1
        part_rbs = (dn_rbs + wgs // n_groups - 1) // (wgs // n_groups)
    else:
        rb_share = (rb_total + wgs - 1) // wgs
        n_dn = (rb_share - 1) // dn_rbs + 2
        part_rbs = min(rb_share, dn_rbs)
    if 2 + n_dn > FM2_MAX_SEG or part_rbs * K * rps_dn * 4 > FM2_PART_BYTES:
        return None
    return wgs


def kernel_split(n_groups, K, hidden, inter, G):
    """Fm2Stream::run: per workgroup (gate/up unit range, down row-block range, n_up, n_dn,
    largest number of row blocks it holds of one layer)."""
    lpr_up = hidden // 128
    rps_up, rps_dn = FM_WAVE // lpr_up, FM_WAVE // (lpr_up // 4)
    gu_upp, dn_upp = inter // rps_up, hidden // rps_dn
    L = n_groups
    gu_segu, dn_segu = gu_upp * K, dn_upp * K
    gu_total, rb_total = n_groups * K * gu_upp, L * dn_upp
    s_total = 2 * gu_total + rb_total * K
    assert s_total * G < 1 << 31          # the kernel's products are 32-bit

    def dn_start(gg):
        if gg >= G:
            return rb_total
        if G < L:
            return rb_total * gg // G
        l = gg * L // G
        g_lo, g_hi = (l * G + L - 1) // L, ((l + 1) * G + L - 1) // L
        return l * dn_upp + dn_upp * (gg - g_lo) // (g_hi - g_lo)

    def gu_start(gg, dn0):
        t, d = s_total * gg // G, dn0 * K
        u = (t - d) // 2 if t > d else 0
        return min(u, gu_total)

    out = []
    for g in range(G):
        rb0, rb1 = dn_start(g), dn_start(g + 1)
        u0, u1 = gu_start(g, rb0), gu_start(g + 1, rb1)
        d0, d1 = rb0 * K, rb1 * K
        n_up = (u1 - 1) // gu_segu + 1 - u0 // gu_segu if u1 > u0 else 0
        n_dn = (d1 - 1) // dn_segu + 1 - d0 // dn_segu if d1 > d0 else 0
        worst = 0
        for s in range(d0 // dn_segu, d0 // dn_segu + n_dn):       # row blocks of layer s in this share
            lo, hi = max(s * dn_upp, rb0), min((s + 1) * dn_upp, rb1)
            worst = max(worst, hi - lo)
        out.append((u0, u1, rb0, rb1, n_up, n_dn, worst))
    return out, gu_total, rb_total, rps_dn


SHAPES = [(2048, 512), (1024, 256), (512, 128), (4096, 1024)]


@pytest.mark.parametrize("hidden,inter", SHAPES)
def test_launcher_bounds_cover_the_kernels_split(hidden, inter):
    if hidden // 128 > 16:
        # 32 lanes per gate row: the launcher never picks this kernel (launch_decode_t)
        assert hidden == 4096
        return
    accepted = 0
    for n_groups, K, n_cu in itertools.product(list(range(1, 49)) + [64, 80, 96, 512], range(1, 9), (256, 64, 304, 8)):
        G = launcher(n_groups, K, hidden, inter, n_cu)
        if G is None:
            continue
        accepted += 1
        shares, gu_total, rb_total, rps_dn = kernel_split(n_groups, K, hidden, inter, G)
        what = (n_groups, K, n_cu, G)
        # every gate/up unit and every row block exactly once, in order
        assert shares[0][0] == 0 and shares[0][2] == 0, what
        assert shares[-1][1] == gu_total and shares[-1][3] == rb_total, what
        for a, b in zip(shares, shares[1:]):
            assert a[1] == b[0] and a[3] == b[2], what
        for u0, u1, rb0, rb1, n_up, n_dn, worst in shares:
            assert u1 >= u0 and rb1 >= rb0, what
            assert n_up <= 2, what                                  # both images are prebuilt, no third
            assert n_up + n_dn <= FM2_MAX_SEG, what                 # the segment table
            assert worst * K * rps_dn * 4 <= FM2_PART_BYTES, what   # partial vectors of a part in LDS
            if G >= n_groups:
                assert n_dn <= 1, what                              # a workgroup's rows lie in one layer
    assert accepted > 500


def test_the_benchmark_shapes_take_this_launch():
    # the 40-layer step and single layers on a 256-CU chip, K = 8
    assert launcher(40, 8, 2048, 512, 256) == 256
    assert launcher(1, 8, 2048, 512, 256) == 128


# ---- chunks of many positions: items and shares of the row-tile kernels (fm_prefill.hip) ----
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
