// fm_index.h — the index arithmetic of the kernels' memory accesses, in functions that compile
// both into the kernels (hipcc) and into a plain host program (g++).
//
// A kernel forms a global address as   base pointer + f(workgroup, wave, lane, unit).
// Everything to the right of the plus sign lives here: how a launch is split over the workgroups,
// which tensor / expert / row step a unit is, which bytes of it a lane touches, and where results
// go.  The kernels call these functions; tests/host_bounds/ walks the same functions over every
// (workgroup, unit, lane, load) of a launch with the launcher's own grid and checks every offset
// against the size of the buffer it indexes — on the host, under the address and undefined-
// behaviour sanitizers, before a shape runs on the GPU for the first time.
//
// Nothing here touches memory; all functions are pure.
#pragma once

#include <stddef.h>
#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define FM_HD __host__ __device__ __forceinline__
#else
#define FM_HD static inline
#endif
#define FM_HDC FM_HD constexpr      // also usable in constant expressions (kernels' LDS layouts)

#ifndef FM_WAVE
#define FM_WAVE 64
#endif
#ifndef FM_CPL
#define FM_CPL 128   // columns per lane of the GEMV lane map
#endif
#ifndef FM_MAX_K
#define FM_MAX_K 8
#endif
#define FM_IDX_MAX_BATCH 8

// bytes of packed codes a lane owns (128 columns) at a code width
FM_HD int fm_lane_bytes(int bits) { return bits == 3 ? 48 : (bits == 8 ? 128 : 64); }

// ---------------------------------------------------------------------------------------------
// shares of a sequence of `total` work units over G workgroups
// ---------------------------------------------------------------------------------------------
struct FmRange {
    long lo, hi;
};
FM_HD FmRange fm_share(long total, unsigned int b, unsigned int G) {
    FmRange r;
    r.lo = total * (long)b / (long)G;
    r.hi = total * ((long)b + 1) / (long)G;
    return r;
}
// Workgroups are dealt out to the eight XCDs in turn and every XCD has an L2 of its own: when the
// grid is a multiple of 8, workgroup b takes share (b % 8) * (G / 8) + b / 8, so that neighbouring
// shares run behind one L2.  A bijection on [0, G).
FM_HD unsigned int fm_xcd_share(unsigned int b, unsigned int G) {
    return G % 8u == 0u ? (b % 8u) * (G / 8u) + b / 8u : b;
}

// ---------------------------------------------------------------------------------------------
// lane map of a wave step ("unit") of the GEMV kernels: LPR lanes share a row
// (lane = 4*chunk + row-in-quad), the step covers 64/LPR consecutive rows
// ---------------------------------------------------------------------------------------------
struct FmUnitLane {
    uint32_t woff;      // this lane's code bytes inside a unit whose rows are row_bytes apart
    uint32_t soff;      // its scale / bias dword inside the unit's [rows][sb_row_bytes]
    int row_in_step;
    int ch;             // 128-column chunk
};
FM_HD FmUnitLane fm_unit_lane(int lane, int lpr, int lane_bytes, int row_bytes, int sb_row_bytes) {
    FmUnitLane u;
    const int j = lane & 3;
    u.ch = (lane >> 2) % lpr;
    const int rq = lane / (4 * lpr);
    u.row_in_step = 4 * rq + j;
    u.woff = (uint32_t)(u.row_in_step * row_bytes + u.ch * lane_bytes);
    u.soff = (uint32_t)(u.row_in_step * sb_row_bytes + u.ch * 4);
    return u;
}

// ---------------------------------------------------------------------------------------------
// stream probe (fm_probe.hip): which 4 KB slots a wave reads
// ---------------------------------------------------------------------------------------------
// (waves per workgroup and slots per wave's ring: the decode kernels' twelve and two)
#define FM_PROBE_WAVES 12
#define FM_PROBE_RING 2
struct FmProbeWalk {
    size_t next, end, step;
};
FM_HD FmProbeWalk fm_probe_walk(int pattern, size_t n_slots, unsigned int b, unsigned int G, int wave,
                                int waves_per_wg) {
    FmProbeWalk w;
    const size_t gw = (size_t)b * waves_per_wg + wave, nw = (size_t)G * waves_per_wg;
    if (pattern == 0) {
        w.next = gw, w.end = n_slots, w.step = nw;
    } else if (pattern == 1) {
        w.next = n_slots * b / G + wave, w.end = n_slots * (b + 1) / G, w.step = (size_t)waves_per_wg;
    } else if (pattern == 2) {
        w.next = n_slots * gw / nw, w.end = n_slots * (gw + 1) / nw, w.step = 1;
    } else if (pattern == 6) {
        // as 1, with neighbouring shares on one XCD
        const unsigned int sh = fm_xcd_share(b, G);
        w.next = n_slots * sh / G + wave, w.end = n_slots * (sh + 1) / G, w.step = (size_t)waves_per_wg;
    } else {
        // groups of `gs` workgroups share a contiguous region, its slots dealt out to the group's
        // waves in turn (3: four consecutive workgroups, 4: eight consecutive workgroups — they sit
        // on different XCDs —, 5 / 7: eight / four workgroups of one XCD, b % 8 equal)
        const unsigned int gs = pattern == 3 || pattern == 7 ? 4u : 8u;
        unsigned int grp, member;
        if ((pattern == 5 || pattern == 7) && G % (8u * gs) == 0u) {
            const unsigned int xcd = b % 8u, k = b / 8u;        // k-th workgroup of its XCD
            grp = xcd * (G / (8u * gs)) + k / gs, member = k % gs;
        } else {
            grp = b / gs, member = b % gs;
        }
        const unsigned int n_grp = (G + gs - 1u) / gs;
        const unsigned int members = grp + 1u < n_grp || G % gs == 0u ? gs : G % gs;
        w.next = n_slots * grp / n_grp + (size_t)member * waves_per_wg + wave;
        w.end = n_slots * (grp + 1u) / n_grp;
        w.step = (size_t)members * waves_per_wg;
    }
    return w;
}

// ---------------------------------------------------------------------------------------------
// row-tile products of a chunk (fm_pf_rows): a task = 32 weight rows of an item (gate/up: 16
// gate rows and the same 16 rows of up; down: 32 rows) over the whole K dimension, a slab = 256
// columns of them = one slot of a wave's ring, a round = eight consecutive tasks of an item
// ---------------------------------------------------------------------------------------------
// code bytes of a row inside a slab
FM_HD int fm_pfr_slab_row_bytes(int bits) { return 8 * bits * 4; }
// the rounds [lo, hi) of workgroup b out of RT (neighbouring shares behind one L2)
FM_HD FmRange fm_pfr_rounds(long RT, unsigned int b, unsigned int G) { return fm_share(RT, fm_xcd_share(b, G), G); }
// one workgroup per CU, more when a share could span more than the 64 items whose experts a
// workgroup keeps one per lane
FM_HD int fm_pfr_grid(int max_items, int n_cu) {
    const int need = (max_items + 31) / 32;
    return need > n_cu ? need : n_cu;
}
// 16-byte piece q (= 64 j + lane, the slot keeps the rows back to back) of a slot copy: its offset
// in the expert's blob from (the task's first row, the slab's first byte).  first_w / second_w:
// offsets of the gate and up (or down, unused) code matrices in the blob
FM_HD uint32_t fm_pfr_piece_off(int gu, int bits, int q, uint32_t first_w, uint32_t second_w, int row_bytes) {
    const int rp = fm_pfr_slab_row_bytes(bits) / 16, rr = q / rp, pc = q - rr * rp;
    const uint32_t mat = gu ? (rr < 16 ? first_w : second_w) : first_w;
    return mat + (uint32_t)((gu ? (rr & 15) : rr) * row_bytes + 16 * pc);
}
// scales (biases) fetched with the slot, 8 bytes per row and slab: the dword of lane `lane`
FM_HD uint32_t fm_pfr_sb_off(int gu, int lane, uint32_t first, uint32_t second, int sb_bytes) {
    const int rr = lane >> 1;
    return (gu ? (rr < 16 ? first : second) : first) + (uint32_t)((gu ? (rr & 15) : rr) * sb_bytes + 4 * (lane & 1));
}

// ---------------------------------------------------------------------------------------------
// dense GEMV, streaming form (fm_dense_stream): all wave steps of all tensors of a launch form
// one sequence; unit_first[i] = first unit of tensor i (unit_first[n..] = total)
// ---------------------------------------------------------------------------------------------
struct FmDensePlan {
    int ok;             // 0: the streaming kernel does not take this launch
    int lpr, ns, rps;   // lanes per row and slab, column slabs, rows per unit
    int units;          // wave steps of the launch
    int wgs;            // workgroups (grid.x)
    int nw;             // waves per workgroup
    int unit_first[FM_IDX_MAX_BATCH + 1];
};
// waves of a streaming workgroup and slices per wave's ring (fm_dense_stream): three waves per
// SIMD where the registers allow it (the 8-bit form and the two-slab form need more than a third
// of a SIMD's file)
#define FM_DENSE_NW(bits, ns) (((bits) == 8 || (ns) == 2) ? 8 : 12)
#define FM_DENSE_RING 2
FM_HD FmDensePlan fm_dense_stream_plan(const int *out_dims, int n, int in_dim, int bits, int n_cu) {
    FmDensePlan p;
    p.ok = 0;
    p.units = p.wgs = 0;
    p.nw = 8;
    const int lpr_full = in_dim / FM_CPL;
    p.ns = lpr_full == 32 ? 2 : 1;
    p.lpr = lpr_full / p.ns;
    p.rps = p.lpr > 0 ? FM_WAVE / p.lpr : 0;
    for (int i = 0; i <= FM_IDX_MAX_BATCH; i++) p.unit_first[i] = 0;
    if (in_dim % FM_CPL || !(p.lpr == 4 || p.lpr == 8 || p.lpr == 16) || (p.ns == 2 && bits != 4)) return p;
    if (n < 1 || n > FM_IDX_MAX_BATCH) return p;
    int units = 0;
    for (int i = 0; i < n; i++) {
        if (out_dims[i] < 1 || out_dims[i] % p.rps) return p;
        p.unit_first[i] = units;
        units += out_dims[i] / p.rps;
    }
    for (int i = n; i <= FM_IDX_MAX_BATCH; i++) p.unit_first[i] = units;
    p.units = units;
    // worth it only when every wave of the chip gets a unit
    if ((long)units < 8L * n_cu) return p;
    long wgs = n_cu;
    p.nw = FM_DENSE_NW(bits, p.ns);
    if (units < p.nw * wgs) wgs = (units + p.nw - 1) / p.nw;
    p.wgs = (int)wgs;
    p.ok = 1;
    return p;
}
// tensor of unit u: the last i < n with unit_first[i] <= u
FM_HD int fm_dense_unit_tensor(const int *unit_first, int n, long u) {
    int t = 0;
#if defined(__HIPCC__)
#pragma unroll
#endif
    for (int i = 1; i < FM_IDX_MAX_BATCH; i++)
        if (i < n && u >= unit_first[i]) t = i;
    return t;
}
// two column slabs (in_dim 4096): byte offset of the 16 bytes lane `lane` copies for row i of the
// unit and slab kn, and of its scale / bias dword
FM_HD size_t fm_dense_slab_woff(int i, int kn, int lane, int row_bytes, int slab_row_bytes) {
    return (size_t)i * row_bytes + (size_t)kn * slab_row_bytes + (size_t)lane * 16;
}
FM_HD uint32_t fm_dense_slab_sboff(int kn, int lane, int sb_row_bytes, int slab_sb) {
    return (uint32_t)((lane >> 4) * sb_row_bytes + kn * slab_sb + (lane & 15) * 4);
}
// riders: wave gw of the launch takes row gw of the raw-BF16 tensors; rider_first[r] = first row
// of rider r, rider_first[n_riders] = all rows.  Returns the rider (or -1) and the row in it.
FM_HD int fm_dense_rider_of(const int *rider_first, int n_riders, int gw, int *row) {
    if (n_riders < 1 || gw >= rider_first[n_riders]) return -1;
    const int r = n_riders > 1 && gw >= rider_first[1] ? 1 : 0;
    *row = gw - (r ? rider_first[1] : 0);
    return r;
}

// ---------------------------------------------------------------------------------------------
// dense GEMV, plain form (fm_dense_gemv / _mixed): one workgroup of four waves per row tile
// ---------------------------------------------------------------------------------------------
// rows per workgroup: grown from four wave steps until the launch fits two workgroups per CU
// (or the tile is eight steps deep)
FM_HD int fm_gemv_rows_per_item(long total_rows, int M, int lpr, int n_cu) {
    const int min_rows = 4 * (FM_WAVE / lpr);
    int rpi = min_rows;
    while (rpi * 2 <= 8 * min_rows && (total_rows * M + rpi - 1) / rpi > 2L * n_cu) rpi *= 2;
    return rpi;
}
struct FmGemvWave {
    int row0;           // first row of this wave
    int steps;          // wave steps it runs (0: none)
};
FM_HD FmGemvWave fm_gemv_wave(int chunk, int wave, int rows_per_item, int lpr, int out_dim) {
    FmGemvWave w;
    const int rps = FM_WAVE / lpr, rows_per_wave = rows_per_item >> 2;
    w.row0 = chunk * rows_per_item + wave * rows_per_wave;
    w.steps = 0;
    if (w.row0 >= out_dim) return w;
    w.steps = rows_per_wave / rps;
    const int left = (out_dim - w.row0 + rps - 1) / rps;
    if (left < w.steps) w.steps = left;
    return w;
}
// rows past the end (out_dim not a multiple of the wave step) re-read the last row
FM_HD int fm_gemv_row_clamp(int row, int out_dim) { return row < out_dim - 1 ? row : out_dim - 1; }

// ---------------------------------------------------------------------------------------------
// dense tensor against M positions on the matrix cores (fm_pf_dense_prep, fm_pf_gemm)
// ---------------------------------------------------------------------------------------------
#define FM_PF_TM 16      // positions per item
// geometry of a slab (four groups = 256 columns of 32 rows) in a ring slot
struct FmPfSlab {
    int cb;             // code bytes of a row inside the slab: 96 / 128
    int rp;             // 16-byte pieces per row: 6 / 8
    int rs;             // piece slots per row in LDS (one stays empty): 7 / 9
    int pieces;         // piece slots of a tile-matrix: 224 / 288
    int nq;             // LDS-direct loads for the codes
    int lds_code;       // 3584 / 4608
    int slot;           // + scales 256 + biases 256
    int ring;
    int lds_bytes;
};
FM_HDC FmPfSlab fm_pf_slab(int bits) {
    FmPfSlab s{};
    s.cb = 8 * bits * 4;
    s.rp = s.cb / 16;
    s.rs = s.rp + 1;
    s.pieces = 32 * s.rs;
    s.nq = (s.pieces + 63) / 64;
    s.lds_code = s.pieces * 16;
    s.slot = s.lds_code + 512;
    const int red = 2 * 2 * 8 * 8 * 64 * 4;
    s.ring = (160 * 1024 - red) / (8 * s.slot);
    s.lds_bytes = 8 * s.ring * s.slot + red;
    return s;
}
// piece q = 64 j + lane of a slot copy: byte offset inside the tile-matrix's rows (valid: the lane
// copies in load j)
FM_HD uint32_t fm_pf_piece_off(const FmPfSlab &g, int j, int lane, int row_bytes, int slab, int *valid) {
    const int q = 64 * j + lane;
    const int row = q / g.rs, piece = q - row * g.rs;
    *valid = q < g.pieces && piece < g.rp;
    return (uint32_t)(row * row_bytes + g.cb * slab + 16 * piece);
}
// scales / biases of the slab: 8 bytes per row, one dword per lane
FM_HD uint32_t fm_pf_sb_off(int lane, int sb_bytes, int slab) {
    const int sb_slab = (2 * 4 * slab) & ~3;
    return (uint32_t)((lane >> 1) * sb_bytes + sb_slab + 4 * (lane & 1));
}
struct FmPfDenseGrid {
    int items, n_steps, grid;
};
// teams: the 512-column form (256 rows per step), otherwise 64 rows per step
FM_HD FmPfDenseGrid fm_pf_dense_grid(int M, int d_rows, int teams, int n_cu) {
    FmPfDenseGrid g;
    g.items = (M + FM_PF_TM - 1) / FM_PF_TM;
    g.n_steps = teams ? d_rows / 256 : d_rows / 64;
    const long steps = (long)g.items * g.n_steps;
    g.grid = steps < n_cu ? (int)steps : n_cu;
    return g;
}
// first row of tile-matrix `mat` of step s (of team `team` in the 512-column form)
FM_HD size_t fm_pf_dense_row(int s, int mat, int team, int teams) {
    return (size_t)s * (teams ? 256u : 64u) + 64u * (size_t)team + (mat ? 32u : 0u);
}
// workspace carve-up of one dense launch (bytes from the workspace start)
struct FmPfDenseWs {
    size_t items, n_items, xop, xsums, total;
};
FM_HD size_t fm_align256(size_t v) { return (v + 255) & ~(size_t)255; }
FM_HD FmPfDenseWs fm_pf_dense_ws(int M, int in_dim) {
    FmPfDenseWs w;
    size_t o = 0;
    w.items = o;   o += fm_align256(((size_t)M / FM_PF_TM + 1) * 16);
    w.n_items = o; o += 256;
    w.xop = o;     o += fm_align256((size_t)M * (in_dim / 64) * 16 * 16);
    w.xsums = o;   o += fm_align256((size_t)M * (in_dim / 64) * 8);
    w.total = o;
    return w;
}
// operand registers of X: uint4 index of (position m, group g, k step k, half h, piece p)
FM_HD size_t fm_pf_xop_index(size_t m, int ng, int g, int k, int h, int p) {
    return ((m * ng + g) * 4 + k) * 4 + 2 * h + p;
}
// prepare task -> (position, group, half)
struct FmPfPrepTask {
    int m, g, h;
};
FM_HD FmPfPrepTask fm_pf_prep_task(int task, int ng) {
    FmPfPrepTask t;
    t.h = task & 1;
    t.g = (task >> 1) % ng;
    t.m = task / (2 * ng);
    return t;
}

// ---------------------------------------------------------------------------------------------
// routed-expert decode, streaming phases (fm_gate_up_swiglu_lds, fm_down_lds, fm_moe_fused):
// both phases split their units over the workgroups in proportion; a gate/up segment is a layer's
// K experts, a down segment one pair
// ---------------------------------------------------------------------------------------------
struct Fm1Split {
    long gu_segu, dn_segu;                      // units per segment
    long gu_wg0, gu_wg1, dn_wg0, dn_wg1;        // this workgroup's unit ranges
    int gu_s0, dn_s0, n_up, n_dn;               // first segment and segment count of each phase
};
FM_HD Fm1Split fm1_split(long gu_total, long dn_total, long gu_segu, long dn_segu, unsigned int b,
                         unsigned int G) {
    Fm1Split s;
    s.gu_segu = gu_segu, s.dn_segu = dn_segu;
    const FmRange gu = fm_share(gu_total, b, G), dn = fm_share(dn_total, b, G);
    s.gu_wg0 = gu.lo, s.gu_wg1 = gu.hi, s.dn_wg0 = dn.lo, s.dn_wg1 = dn.hi;
    s.gu_s0 = (int)(s.gu_wg0 / gu_segu);
    s.dn_s0 = (int)(s.dn_wg0 / dn_segu);
    s.n_up = s.gu_wg1 > s.gu_wg0 ? (int)((s.gu_wg1 - 1) / gu_segu) + 1 - s.gu_s0 : 0;
    s.n_dn = s.dn_wg1 > s.dn_wg0 ? (int)((s.dn_wg1 - 1) / dn_segu) + 1 - s.dn_s0 : 0;
    return s;
}
// segment number q of the workgroup's sequence (gate/up first) -> segment of its phase
FM_HD int fm1_seg(const Fm1Split &s, int q) {
    return s.gu_s0 + q + (q < s.n_up ? 0 : s.dn_s0 - s.gu_s0 - s.n_up);
}
// this workgroup's part of it: first unit inside the segment and count
FM_HD void fm1_part(const Fm1Split &s, int q, int gu, uint32_t *first, uint32_t *n) {
    const long seg = fm1_seg(s, q);
    const long segu = gu ? s.gu_segu : s.dn_segu, w0 = gu ? s.gu_wg0 : s.dn_wg0, w1 = gu ? s.gu_wg1 : s.dn_wg1;
    const long lo = seg * segu > w0 ? seg * segu : w0;
    const long hi = (seg + 1) * segu < w1 ? (seg + 1) * segu : w1;
    *first = (uint32_t)(lo - seg * segu);
    *n = (uint32_t)(hi - lo);
}
// workgroups of a streaming launch: one per CU, fewer when there are not enough units to give
// every wave `per_wave` of them
FM_HD long fm_stream_wgs(long units, int n_cu, int per_wave, int n_waves = 8) {
    long wgs = (long)n_cu;
    const long need = (long)n_waves * per_wave;
    if (units < need * wgs) wgs = (units + need - 1) / need;
    if (wgs < 1) wgs = 1;
    return wgs;
}
// workgroups of the one-launch form with dependency counters (fm_moe_fused)
FM_HD long fm1_fused_wgs(long up_units, long down_units, int n_cu) {
    long wgs = (long)n_cu;
    const long small = up_units < down_units ? up_units : down_units;
    if (small < 8 * wgs) wgs = (small + 7) / 8;
    if (wgs < 1) wgs = 1;
    return wgs;
}

// ---------------------------------------------------------------------------------------------
// u / d for u < 2^31 without the division sequence: with l = ceil(log2 d),
// mul = ceil(2^(31 + l) / d) fits 32 bits and floor(u * mul / 2^(31 + l)) is exact.
struct FmDiv {
    uint32_t mul, shift, d;
};
FM_HD FmDiv fm_div_make(uint32_t d) {
    FmDiv r;
    r.mul = 0u, r.shift = 0u, r.d = d;
    if (d > 1u) {
        uint32_t l = 0;
        while ((1ull << l) < d) l++;
        r.mul = (uint32_t)(((1ull << (31 + l)) + d - 1) / d);
        r.shift = l - 1;
    }
    return r;
}
FM_HD uint32_t fm_div(const FmDiv &v, uint32_t u) {
#if defined(__HIP_DEVICE_COMPILE__)
    return v.d == 1u ? u : __umulhi(u, v.mul) >> v.shift;
#else
    return v.d == 1u ? u : (uint32_t)(((uint64_t)u * v.mul) >> 32) >> v.shift;
#endif
}
// ---------------------------------------------------------------------------------------------
// routed-expert decode, the launch that sums the experts in LDS (fm_moe_fused_rows)
// ---------------------------------------------------------------------------------------------
#define FM2_MAX_SEG 12          // segments of one workgroup's shares
#define FM2_PART_BYTES 12288    // partial vectors of a part
// The launcher works these out on the host and hands them to the kernel by value: the divisions a
// workgroup needs for its split are then multiplications (seventeen division sequences on eight
// waves were 1.4 us in front of the first load).
struct Fm2Dims {
    uint32_t K, G, L;           // slots, workgroups, layer groups
    uint32_t gu_upp, dn_upp;    // gate/up units per pair, down row blocks per layer
    uint32_t gu_segu, dn_segu;  // units per segment: a layer's K experts
    uint32_t gu_total, rb_total, s_total;
    uint32_t wq;                // G / L: a layer has wq or wq + 1 workgroups (G >= L)
    uint32_t gu_wt, dn_wt;      // what a gate/up unit and a (row block, slot) weigh in the balance
    FmDiv by_G, by_L, by_K, by_gu_upp, by_gu_segu, by_dn_segu, by_wq, by_wq1, by_gu_wt;
};
// gu_upp gate/up units per pair, dn_upp down row blocks per layer; a gate/up unit streams gu_wt
// and a down unit dn_wt of some common measure of bytes (affine experts: two slices and one)
FM_HD Fm2Dims fm2_dims_units(int n_pairs, int K, int G, uint32_t gu_upp, uint32_t dn_upp, uint32_t gu_wt,
                             uint32_t dn_wt) {
    Fm2Dims d;
    d.K = (uint32_t)K, d.G = (uint32_t)G, d.L = (uint32_t)(n_pairs / K);
    d.gu_upp = gu_upp;
    d.dn_upp = dn_upp;
    d.gu_wt = gu_wt, d.dn_wt = dn_wt;
    d.gu_segu = d.gu_upp * d.K;
    d.dn_segu = d.dn_upp * d.K;
    d.gu_total = (uint32_t)n_pairs * d.gu_upp;
    d.rb_total = d.L * d.dn_upp;
    d.s_total = gu_wt * d.gu_total + dn_wt * d.rb_total * d.K;
    d.wq = d.L ? d.G / d.L : 0u;
    d.by_G = fm_div_make(d.G), d.by_L = fm_div_make(d.L ? d.L : 1u), d.by_K = fm_div_make(d.K);
    d.by_gu_upp = fm_div_make(d.gu_upp ? d.gu_upp : 1u);
    d.by_gu_segu = fm_div_make(d.gu_segu ? d.gu_segu : 1u), d.by_dn_segu = fm_div_make(d.dn_segu ? d.dn_segu : 1u);
    d.by_wq = fm_div_make(d.wq ? d.wq : 1u), d.by_wq1 = fm_div_make(d.wq + 1u);
    d.by_gu_wt = fm_div_make(gu_wt ? gu_wt : 1u);
    return d;
}
FM_HD Fm2Dims fm2_dims(int n_pairs, int K, int G, int inter, int hidden, int lpr_up) {
    const int rps_up = FM_WAVE / lpr_up, rps_dn = FM_WAVE / (lpr_up / 4);
    return fm2_dims_units(n_pairs, K, G, (uint32_t)(inter / rps_up), (uint32_t)(hidden / rps_dn), 2u, 1u);
}
// first down row block of workgroup gg: a workgroup's row blocks lie in ONE layer whenever there
// are at least as many workgroups as layers
FM_HD uint32_t fm2_dn_start(const Fm2Dims &d, uint32_t gg) {
    if (gg >= d.G) return d.rb_total;
    if (d.G < d.L) return fm_div(d.by_G, d.rb_total * gg);
    const uint32_t l = fm_div(d.by_G, gg * d.L);
    const uint32_t g_lo = fm_div(d.by_L, l * d.G + d.L - 1u), g_hi = fm_div(d.by_L, (l + 1u) * d.G + d.L - 1u);
    // the layer's workgroups: wq or wq + 1 of them
    const uint32_t n = g_hi - g_lo, v = d.dn_upp * (gg - g_lo);
    return l * d.dn_upp + (n == d.wq ? fm_div(d.by_wq, v) : fm_div(d.by_wq1, v));
}
// first gate/up unit of workgroup gg (dn0 = its first down row block): sized so that gate/up +
// down slices are the same for every workgroup
FM_HD uint32_t fm2_gu_start(const Fm2Dims &d, uint32_t gg, uint32_t dn0) {
    const uint32_t t = fm_div(d.by_G, d.s_total * gg), dd = dn0 * d.K * d.dn_wt;
    const uint32_t u = t > dd ? fm_div(d.by_gu_wt, t - dd) : 0u;
    return u > d.gu_total ? d.gu_total : u;
}
struct Fm2Split {
    uint32_t gu_wg0, gu_wg1, dn_wg0, dn_wg1;    // unit ranges (down: row block * K)
    int gu_s0, dn_s0, n_up, n_dn;               // first segment and segment count of each phase
};
FM_HD Fm2Split fm2_split(const Fm2Dims &d, uint32_t g) {
    Fm2Split s;
    const uint32_t dn_rb0 = fm2_dn_start(d, g), dn_rb1 = fm2_dn_start(d, g + 1u);
    s.gu_wg0 = fm2_gu_start(d, g, dn_rb0);
    s.gu_wg1 = fm2_gu_start(d, g + 1u, dn_rb1);
    s.dn_wg0 = dn_rb0 * d.K;
    s.dn_wg1 = dn_rb1 * d.K;
    s.gu_s0 = (int)fm_div(d.by_gu_segu, s.gu_wg0);
    s.dn_s0 = (int)fm_div(d.by_dn_segu, s.dn_wg0);
    s.n_up = s.gu_wg1 > s.gu_wg0 ? (int)fm_div(d.by_gu_segu, s.gu_wg1 - 1u) + 1 - s.gu_s0 : 0;
    s.n_dn = s.dn_wg1 > s.dn_wg0 ? (int)fm_div(d.by_dn_segu, s.dn_wg1 - 1u) + 1 - s.dn_s0 : 0;
    return s;
}
// segment qq of the workgroup's sequence (gate/up segments first): layer group, first unit inside
// the segment, unit count
struct Fm2Part {
    uint32_t seg, first, n;
    int gu;
};
FM_HD Fm2Part fm2_part(const Fm2Dims &d, const Fm2Split &s, int qq) {
    Fm2Part p;
    p.gu = qq < s.n_up;
    p.seg = (uint32_t)(p.gu ? s.gu_s0 + qq : s.dn_s0 + (qq - s.n_up));
    const uint32_t segu = p.gu ? d.gu_segu : d.dn_segu, w0 = p.gu ? s.gu_wg0 : s.dn_wg0,
                   w1 = p.gu ? s.gu_wg1 : s.dn_wg1;
    const uint32_t lo = p.seg * segu > w0 ? p.seg * segu : w0;
    const uint32_t hi = (p.seg + 1u) * segu < w1 ? (p.seg + 1u) * segu : w1;
    p.first = lo - p.seg * segu;
    p.n = hi > lo ? hi - lo : 0u;
    return p;
}
// claimed unit ul of a gate/up part: slot pn of the layer and row step rsn of its expert
FM_HD void fm2_gu_unit(uint32_t first, uint32_t ul, const FmDiv &by_gu_upp, uint32_t *pn, uint32_t *rsn) {
    const uint32_t uq = first + ul;
    *pn = fm_div(by_gu_upp, uq);
    *rsn = uq - *pn * by_gu_upp.d;
}
// claimed unit ul of a down part of nrb row blocks starting at row block rb_first (expert by
// expert: unit ul = row block ul % nrb of slot ul / nrb); inv = 1 / nrb in fp32
FM_HD void fm2_dn_unit(uint32_t rb_first, uint32_t nrb, float inv, uint32_t ul, uint32_t *pn, uint32_t *rsn) {
    *pn = (uint32_t)(((float)ul + 0.5f) * inv);
    *rsn = rb_first + (ul - *pn * nrb);
}
// The layer tail behind the experts in the same launch keeps three small tables in the part of
// LDS the partial vectors leave free: the shared expert's results for the workgroup's rows, the
// shared expert's activations, and the per-wave sums of the norm.  nrb = row blocks of the
// workgroup's (one) down part.
struct Fm2TailLds {
    int ok;
    uint32_t so, act, red, word;     // byte offsets inside the partial-vector area
};
// (the routing at the launch's start uses the area before any of this: n softmax values from its
// first byte, and indices / weights / params in its last FM2_ROUTE_WORDS bytes, which stay until
// the segment tables are built)
#define FM2_ROUTE_WORDS 128
FM_HD int fm2_route_fits(int n) { return n >= 1 && (size_t)n * 4 + FM2_ROUTE_WORDS <= FM2_PART_BYTES; }
FM_HD Fm2TailLds fm2_tail_lds(int nrb, int K, int rps_dn, int shared_inter, int hidden) {
    Fm2TailLds t;
    t.so = (uint32_t)(nrb * K * rps_dn * 4);                 // behind the partial vectors
    t.act = (t.so + (uint32_t)(nrb * rps_dn * 4) + 15u) & ~15u;
    t.red = t.act + (uint32_t)shared_inter * 4u;
    t.word = t.red + (uint32_t)(hidden / rps_dn) * 4u;
    t.ok = nrb >= 1 && nrb <= 8 && shared_inter <= 512 && t.word + 16u <= FM2_PART_BYTES - FM2_ROUTE_WORDS;
    return t;
}
// the launcher's decision: workgroups, and whether the shape fits the kernel's fixed tables
struct Fm2Plan {
    int ok, wgs;
};
FM_HD Fm2Plan fm2_plan_units(int n_pairs, int K, long gu_upp, long dn_rbs, int rps_dn, long gu_wt, long dn_wt,
                             int n_cu) {
    Fm2Plan p;
    p.ok = 0;
    p.wgs = 0;
    if (K < 1 || gu_upp < 1 || dn_rbs < 1 || gu_wt < 1 || dn_wt < 1) return p;
    const int n_groups = n_pairs / K;
    const long gu_segu = gu_upp * K;
    const long up_units = (long)n_groups * gu_segu, rb_total = (long)n_groups * dn_rbs;
    long wgs = n_cu;
    const long small = up_units < rb_total * K ? up_units : rb_total * K;
    if (small < 8 * wgs) wgs = (small + 7) / 8;
    if (wgs < 1) wgs = 1;
    p.wgs = (int)wgs;
    // at most two gate/up segments, and the down segments and the row blocks of one part within
    // the fixed tables
    const long s_total = gu_wt * up_units + dn_wt * rb_total * K;
    const long up_share = (s_total / wgs + 1) / gu_wt + 1;              // upper bound, in units
    if (up_share > gu_segu || s_total * wgs >= (1L << 31)) return p;
    long n_dn, part_rbs;
    if (wgs >= n_groups) {
        n_dn = 1;
        part_rbs = (dn_rbs + wgs / n_groups - 1) / (wgs / n_groups);
    } else {
        const long rb_share = (rb_total + wgs - 1) / wgs;
        n_dn = (rb_share - 1) / dn_rbs + 2;
        part_rbs = rb_share < dn_rbs ? rb_share : dn_rbs;
    }
    if (2 + n_dn > FM2_MAX_SEG) return p;
    if (part_rbs * K * rps_dn * 4 > FM2_PART_BYTES) return p;
    p.ok = 1;
    return p;
}
FM_HD Fm2Plan fm2_plan(int n_pairs, int K, int inter, int hidden, int lpr_up, int n_cu) {
    const int rps_up = FM_WAVE / lpr_up, rps_dn = FM_WAVE / (lpr_up / 4);
    return fm2_plan_units(n_pairs, K, inter / rps_up, hidden / rps_dn, rps_dn, 2, 1, n_cu);
}

// ---------------------------------------------------------------------------------------------
// GGUF experts, streaming kernels (fm_gguf_stream)
// ---------------------------------------------------------------------------------------------
struct FmGgPlan {
    int ok, lpr, rps, upp, wgs;
    long total;
    int slot_data;      // bytes of a slice = the rows of a wave step as they lie in memory
    int row_bytes;
    int n_img, n_pair;  // images / pair entries a workgroup keeps
    int wide;           // Q6_K rows of 2048 values: a lane owns two 64-value pieces, 1024 values apart
    int ring;           // slices per wave's ring
    int nw;             // waves per workgroup
};
// waves of a streaming workgroup and slices per wave's ring (fm_gguf_stream): three waves per SIMD
// with two slices in flight each read faster than two waves with rings of three to five; the
// slices of the wide Q6_K rows (6720 B) leave room for two waves per SIMD
#define FM_GG_NW(wide) ((wide) ? 8 : 12)
#define FM_GG_RING 2
// q6: Q6_K (a lane owns 64 values) else Q4_K (128); gu: gate and up rows of a unit
FM_HD FmGgPlan fm_gg_plan(int n_pairs, int K, int in_dim, int rows, int q6, int gu, int n_cu) {
    FmGgPlan p;
    p.ok = 0;
    p.wgs = 0, p.total = 0;
    const int per_lane = q6 ? 64 : 128;
    p.wide = q6 && !gu && in_dim == 2048;
    p.nw = FM_GG_NW(p.wide);
    p.lpr = p.wide ? 16 : in_dim / per_lane;
    p.rps = p.lpr > 0 ? FM_WAVE / p.lpr : 0;
    p.upp = p.rps > 0 ? rows / p.rps : 0;
    p.row_bytes = q6 ? (in_dim / 256) * 210 : (p.lpr / 2) * 144;
    p.slot_data = p.rps * p.row_bytes;
    p.ring = FM_GG_RING;
    p.n_img = gu ? 2 : 3;
    p.n_pair = gu ? FM_MAX_K + 1 : 3;
    if (in_dim % per_lane || !(p.lpr == 4 || p.lpr == 8 || p.lpr == 16)) return p;
    if (rows % p.rps) return p;
    p.total = (long)n_pairs * p.upp;
    if (p.total >= (1L << 31)) return p;
    // a workgroup holds the images of 2 layers (gate/up) or 3 pairs (down): keep its share of the
    // units within that span
    const long upv = gu ? (long)p.upp * K : p.upp, max_share = upv * (p.n_img - 1);
    long wgs = n_cu;
    if (p.total < p.nw * wgs) wgs = (p.total + p.nw - 1) / p.nw;
    if ((p.total + wgs - 1) / wgs > max_share) wgs = (p.total + max_share - 1) / max_share;
    while (wgs < p.total && (p.total + wgs - 1) / wgs > max_share) wgs++;
    p.wgs = (int)wgs;
    p.ok = 1;
    return p;
}

// The GGUF experts as one launch (fm_gguf_fused_rows): the split of fm_moe_fused_rows with a
// gate/up unit = the gate and the up slice of a wave step (Q4_K) and a down unit = the slice of
// one row block of one expert (Q6_K or Q4_K), weighed by their bytes.  LDS: eight rings (three
// gate/up slots or ring_dn down slots each, whichever is larger) | two gate/up images or K down
// images | segment tables | partial vectors.
// groups (layers of a step: layer_stride != 0; positions of a chunk: 0) up to which a call without
// per-expert vectors takes the one launch; beyond, the three streaming launches are faster
FM_HD int fm_gg_one_launch_max(int layer_stride) { return layer_stride != 0 ? 13 : 8; }
#define FM_GG2_RING_UP 3
#define FM_GG2_SEG_BYTES 192
struct FmGg2Plan {
    int ok, wgs;
    int lpr_up, lpr_dn, rps_up, rps_dn, ring_dn;
    uint32_t gu_upp, dn_upp, gu_wt, dn_wt;
    uint32_t slot_up, slot_dn;        // bytes of a slice (without the 16-byte trailer)
    uint32_t ring_bytes, img_up, img_dn, img_bytes, lds_bytes;
};
FM_HD uint32_t fm_gcd(uint32_t a, uint32_t b) {
    while (b) {
        const uint32_t t = a % b;
        a = b;
        b = t;
    }
    return a;
}
FM_HD FmGg2Plan fm_gg2_plan(int n_pairs, int K, int hidden, int inter, int down_q6, int n_cu) {
    FmGg2Plan p;
    p.ok = 0, p.wgs = 0;
    p.lpr_up = hidden / 128;
    p.lpr_dn = inter / (down_q6 ? 64 : 128);
    p.rps_up = p.rps_dn = 0;
    p.ring_dn = down_q6 ? 4 : 3;
    p.gu_upp = p.dn_upp = p.gu_wt = p.dn_wt = 0u;
    p.slot_up = p.slot_dn = p.ring_bytes = p.img_up = p.img_dn = p.img_bytes = p.lds_bytes = 0u;
    if (K < 1 || K > FM_MAX_K || n_pairs < K || n_pairs % K) return p;
    if (hidden % 256 || inter % 256) return p;
    if (!(p.lpr_up == 4 || p.lpr_up == 8 || p.lpr_up == 16)) return p;
    if (!(p.lpr_dn == 4 || p.lpr_dn == 8 || p.lpr_dn == 16)) return p;
    p.rps_up = FM_WAVE / p.lpr_up, p.rps_dn = FM_WAVE / p.lpr_dn;
    if (inter % p.rps_up || hidden % p.rps_dn) return p;
    p.gu_upp = (uint32_t)(inter / p.rps_up);
    p.dn_upp = (uint32_t)(hidden / p.rps_dn);
    p.slot_up = (uint32_t)(p.rps_up * (p.lpr_up / 2) * 144);
    p.slot_dn = (uint32_t)(down_q6 ? p.rps_dn * (p.lpr_dn / 4) * 210 : p.rps_dn * (p.lpr_dn / 2) * 144);
    const uint32_t r_up = FM_GG2_RING_UP * (p.slot_up + 16u), r_dn = (uint32_t)p.ring_dn * (p.slot_dn + 16u);
    p.ring_bytes = r_up > r_dn ? r_up : r_dn;
    const uint32_t nreg_dn = down_q6 ? 32u : 64u;
    p.img_up = 16u * (4u * p.lpr_up) * 16u + (uint32_t)p.lpr_up * 16u;
    p.img_dn = (nreg_dn / 4u) * (4u * p.lpr_dn) * 16u + (uint32_t)p.lpr_dn * 16u;
    p.img_bytes = 2u * p.img_up > FM_MAX_K * p.img_dn ? 2u * p.img_up : FM_MAX_K * p.img_dn;
    p.lds_bytes = 8u * p.ring_bytes + p.img_bytes + FM2_MAX_SEG * FM_GG2_SEG_BYTES + FM2_PART_BYTES;
    if (p.lds_bytes > 160u * 1024u) return p;
    // weights of the balance: bytes over their greatest common divisor, halved while the
    // kernel's 32-bit products would not hold them (the balance then is approximate)
    const uint32_t gdiv = fm_gcd(2u * p.slot_up, p.slot_dn);
    p.gu_wt = 2u * p.slot_up / gdiv, p.dn_wt = p.slot_dn / gdiv;
    for (;;) {
        const Fm2Plan q = fm2_plan_units(n_pairs, K, p.gu_upp, p.dn_upp, p.rps_dn, p.gu_wt, p.dn_wt, n_cu);
        p.wgs = q.wgs;
        if (q.ok) break;
        const long s_total = (long)p.gu_wt * n_pairs * p.gu_upp + (long)p.dn_wt * n_pairs * p.dn_upp;
        if (s_total * (q.wgs > 0 ? q.wgs : 1) < (1L << 31) || (p.gu_wt <= 2u && p.dn_wt <= 1u)) return p;
        p.gu_wt = (p.gu_wt + 1u) / 2u, p.dn_wt = (p.dn_wt + 1u) / 2u;
    }
    p.ok = 1;
    return p;
}
