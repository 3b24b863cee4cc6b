// bounds_main.cpp — host-side walk of the kernels' memory accesses.
//
// The kernels of finchmoe_amd/csrc form every global address as  base + f(workgroup, wave, lane,
// unit)  with f taken from fm_index.h.  This program includes the same header, takes the grid the
// launcher would take, enumerates every (workgroup, unit, lane, load instruction) of a launch and
// checks each byte range against the size of the buffer it indexes — the sizes bench.py and the
// GPU tests allocate.  For the streaming kernels it also checks that the ranges tile the weights
// exactly once (a wrong split shows up as a gap or an overlap even when it stays in bounds).
// LDS offsets (ring slots, segment tables, partial vectors, images) are checked against the
// kernels' LDS sizes.  Built with -fsanitize=address,undefined by tests/test_host_bounds.py; no
// GPU, no HIP.
//
// What is NOT shared with the kernels and therefore restated here: the order in which a
// workgroup's waves claim units (irrelevant for bounds: every unit of a share is claimed exactly
// once, by fm_claim_unit's counter), the LDS-direct load helpers' fixed per-lane pattern
// (lane * 16 + 1024 * j for codes, lane * 4 for scales and biases: fm_ring.h), the activation
// staging patterns (fm_mfma.h), which index inside one input vector, and — for the chunk's
// row-tile kernels — fm_pf_group's counting sort and item cut, and which (group, position) a thread
// stages.
#include "../../finchmoe_amd/csrc/fm_index.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

static int g_fail = 0;
static std::string g_case;

#define CHECK(cond, ...)                                                  \
    do {                                                                  \
        if (!(cond)) {                                                    \
            if (g_fail < 20) {                                            \
                std::fprintf(stderr, "FAIL [%s] %s: ", g_case.c_str(), #cond); \
                std::fprintf(stderr, __VA_ARGS__);                        \
                std::fprintf(stderr, "\n");                               \
            }                                                             \
            g_fail++;                                                     \
        }                                                                 \
    } while (0)

// a buffer of `size` bytes; touch() checks a range; with `cover` every byte counts how often a
// read touched it (for the once-only tiling check; granularity = `gran` bytes)
struct Region {
    std::string name;
    size_t size = 0;
    size_t gran = 0;
    std::vector<uint8_t> count;
    size_t lo = (size_t)-1, hi = 0;
    unsigned long touches = 0;
    Region(const char *n, size_t sz, size_t g = 0) : name(n), size(sz), gran(g) {
        if (gran) count.assign((size + gran - 1) / gran, 0);
    }
    void touch(size_t off, size_t len, const char *what) {
        touches++;
        if (off > size || len > size - off) {
            CHECK(false, "%s: %s offset %zu + %zu outside %zu bytes", name.c_str(), what, off, len, size);
            return;
        }
        if (off < lo) lo = off;
        if (off + len > hi) hi = off + len;
        if (gran) {
            CHECK(off % gran == 0 && len % gran == 0, "%s: %s range %zu+%zu not on the %zu-byte grid", name.c_str(),
                  what, off, len, gran);
            for (size_t i = off / gran; i < (off + len) / gran; i++)
                if (count[i] < 255) count[i]++;
        }
    }
    // every grid cell of [a, b) touched exactly once
    void expect_once(size_t a, size_t b) {
        size_t bad = 0, first_bad = 0;
        for (size_t i = a / gran; i < b / gran; i++)
            if (count[i] != 1) {
                if (!bad) first_bad = i;
                bad++;
            }
        CHECK(bad == 0, "%s: %zu cells of [%zu, %zu) not read exactly once (first at byte %zu, count %d)",
              name.c_str(), bad, a, b, first_bad * gran, (int)count[first_bad]);
    }
    void expect_untouched(size_t a, size_t b) {
        for (size_t i = a / gran; i < b / gran; i++)
            if (count[i] != 0) {
                CHECK(false, "%s: byte %zu read although outside the operands", name.c_str(), i * gran);
                return;
            }
    }
};

static const int N_CU = 256;

// the LDS-direct copy of one GEMV unit (fm_dma_issue): NQ loads of 64 lanes x 16 bytes for the
// codes, one load of 64 x 4 bytes each for scales and biases
static void unit_dma(Region &W, size_t w0, Region &S, size_t s0, Region &B, size_t b0, int bits) {
    const int nq = fm_lane_bytes(bits) / 16;
    for (int lane = 0; lane < 64; lane++) {
        for (int j = 0; j < nq; j++) W.touch(w0 + (size_t)lane * 16 + 1024 * (size_t)j, 16, "unit codes");
        S.touch(s0 + (size_t)lane * 4, 4, "unit scales");
        B.touch(b0 + (size_t)lane * 4, 4, "unit biases");
    }
}

// ------------------------------------------------------------------------------------ probe
static void walk_probe(size_t nbytes, int pattern) {
    g_case = "stream_probe pattern " + std::to_string(pattern) + " bytes " + std::to_string(nbytes);
    const size_t n_slots = nbytes / 4096;
    Region buf("probe buffer", nbytes, 4096);
    const int G = N_CU, ring = FM_PROBE_RING, slot = 4096;
    CHECK((size_t)FM_PROBE_WAVES * ring * slot <= 160 * 1024, "LDS");
    for (int b = 0; b < G; b++)
        for (int wave = 0; wave < FM_PROBE_WAVES; wave++) {
            FmProbeWalk w = fm_probe_walk(pattern, n_slots, b, G, wave, FM_PROBE_WAVES);
            for (size_t s = w.next; s < w.end; s += w.step) buf.touch(s * 4096, 4096, "slot");
            // ring in LDS: wave * ring * slot + wpos * slot + 1024 j + 16 lane + 16
            CHECK((size_t)wave * ring * slot + (ring - 1) * slot + 3 * 1024 + 63 * 16 + 16 <= (size_t)FM_PROBE_WAVES * ring * slot, "ring");
        }
    buf.expect_once(0, n_slots * 4096);
    std::printf("ok  %-58s %zu slots\n", g_case.c_str(), n_slots);
}

// ------------------------------------------------------------------------------------ dense
struct DenseT {
    int out_dim, bits;      // bits 16: raw bf16
};

static void walk_dense_batch(const char *name, const std::vector<DenseT> &ts, int in_dim, int M,
                             const std::vector<int> &rider_rows) {
    g_case = std::string("dense ") + name;
    const int n = (int)ts.size(), bits = ts[0].bits;
    const int row_bytes = in_dim * bits / 8, sb_row = (in_dim / 64) * 2;
    std::vector<Region> W, S, B, O;
    int out_dims[8];
    long total_rows = 0;
    for (int i = 0; i < n; i++) {
        out_dims[i] = ts[i].out_dim;
        total_rows += ts[i].out_dim;
        W.emplace_back("W", (size_t)ts[i].out_dim * in_dim * ts[i].bits / 8, 16);
        S.emplace_back("S", (size_t)ts[i].out_dim * sb_row, 4);
        B.emplace_back("B", (size_t)ts[i].out_dim * sb_row, 4);
        O.emplace_back("out", (size_t)M * ts[i].out_dim * 4, 4);
    }
    Region X("x", (size_t)M * in_dim * 4);
    bool same = true;
    for (auto &t : ts) same = same && t.bits == bits;
    const FmDensePlan plan = same ? fm_dense_stream_plan(out_dims, n, in_dim, bits, N_CU) : FmDensePlan{};
    if (same && plan.ok) {
        const int lpr = plan.lpr, ns = plan.ns, rps = plan.rps;
        const int slab_row = lpr * fm_lane_bytes(bits), slab_sb = 4 * lpr;
        CHECK(ns == 1 || (slab_row == 1024 && rps == fm_lane_bytes(bits) / 16), "one load per row and slab");
        const int ring = FM_DENSE_RING;
        const size_t slot_bytes = 64 * (size_t)fm_lane_bytes(bits) + 512 + 16;
        const size_t lds = (size_t)plan.nw * ring * slot_bytes + (bits == 8 ? 0 : (size_t)ns * (16 * 4 * lpr * 16 + lpr * 16));
        CHECK(lds + 16 <= 160 * 1024, "LDS %zu", lds);
        int riders_first[3] = {0, 0, 0};
        int n_riders = (int)rider_rows.size();
        for (int i = 0; i < n_riders; i++) riders_first[i + 1] = riders_first[i] + rider_rows[i];
        for (int i = n_riders; i < 2; i++) riders_first[i + 1] = riders_first[n_riders];
        if (n_riders > 0 && riders_first[n_riders] > plan.nw * plan.wgs) n_riders = 0;
        std::vector<Region> RW, RO;
        for (int i = 0; i < n_riders; i++) {
            RW.emplace_back("rider W", (size_t)rider_rows[i] * in_dim * 2, 2);
            RO.emplace_back("rider out", (size_t)M * rider_rows[i] * 4, 4);
        }
        for (int m = 0; m < M; m++)
            for (int b = 0; b < plan.wgs; b++) {
                const FmRange wg = fm_share(plan.units, b, plan.wgs);
                CHECK(wg.hi - wg.lo >= 8, "share of %ld units", wg.hi - wg.lo);
                for (long u = wg.lo; u < wg.hi; u++) {
                    const int t = fm_dense_unit_tensor(plan.unit_first, n, u);
                    const int row0 = (int)(u - plan.unit_first[t]) * rps;
                    CHECK(row0 >= 0 && row0 + rps <= ts[t].out_dim, "unit %ld row0 %d", u, row0);
                    if (m == 0) {
                        if (ns == 1) {
                            unit_dma(W[t], (size_t)row0 * row_bytes, S[t], (size_t)row0 * sb_row, B[t],
                                     (size_t)row0 * sb_row, bits);
                        } else {
                            for (int kn = 0; kn < ns; kn++)
                                for (int lane = 0; lane < 64; lane++) {
                                    for (int i = 0; i < rps; i++)
                                        W[t].touch((size_t)row0 * row_bytes + fm_dense_slab_woff(i, kn, lane, row_bytes, slab_row), 16,
                                                   "slab codes");
                                    const uint32_t so = fm_dense_slab_sboff(kn, lane, sb_row, slab_sb);
                                    S[t].touch((size_t)row0 * sb_row + so, 4, "slab scales");
                                    B[t].touch((size_t)row0 * sb_row + so, 4, "slab biases");
                                }
                        }
                    }
                    for (int lane = 0; lane < 64; lane++) {
                        const FmUnitLane ul = fm_unit_lane(lane, lpr, fm_lane_bytes(bits), slab_row, slab_sb);
                        // the lane's reads back out of the slot
                        CHECK(ul.woff + (uint32_t)fm_lane_bytes(bits) <= 64u * fm_lane_bytes(bits), "woff");
                        CHECK(ul.soff + 4 <= 256, "soff");
                        if (ul.ch == 0) O[t].touch(((size_t)m * ts[t].out_dim + row0 + ul.row_in_step) * 4, 4, "out");
                    }
                }
                for (int wave = 0; wave < plan.nw && n_riders; wave++) {
                    int row = 0;
                    const int r = fm_dense_rider_of(riders_first, n_riders, b * plan.nw + wave, &row);
                    if (r < 0) continue;
                    if (m == 0) RW[r].touch((size_t)row * in_dim * 2, (size_t)in_dim * 2, "rider row");
                    RO[r].touch(((size_t)m * rider_rows[r] + row) * 4, 4, "rider out");
                }
            }
        for (int i = 0; i < n; i++) {
            W[i].expect_once(0, W[i].size);
            S[i].expect_once(0, S[i].size);
            B[i].expect_once(0, B[i].size);
            O[i].expect_once(0, O[i].size);
        }
        for (int i = 0; i < n_riders; i++) RW[i].expect_once(0, RW[i].size), RO[i].expect_once(0, RO[i].size);
        std::printf("ok  %-58s stream: %d units over %d workgroups, ns %d\n", g_case.c_str(), plan.units, plan.wgs, ns);
        return;
    }
    // plain kernel (also the launch of tensors of different widths): a workgroup per row tile
    const int lpr = in_dim / FM_CPL;
    const int rpi = fm_gemv_rows_per_item(total_rows, same ? M : 1, lpr, N_CU);
    const int rps = FM_WAVE / lpr;
    for (int t = 0; t < n; t++) {
        const int tb = ts[t].bits, bpl = fm_lane_bytes(tb), rb = in_dim * tb / 8;
        const int items = (ts[t].out_dim + rpi - 1) / rpi;
        for (int m = 0; m < M; m++)
            for (int chunk = 0; chunk < items; chunk++)
                for (int wave = 0; wave < 4; wave++) {
                    const FmGemvWave gw = fm_gemv_wave(chunk, wave, rpi, lpr, ts[t].out_dim);
                    for (int it = 0; it < gw.steps; it++)
                        for (int lane = 0; lane < 64; lane++) {
                            const int c = lane % lpr, r = lane / lpr;
                            const int row = gw.row0 + it * rps + r;
                            const size_t ro = (size_t)fm_gemv_row_clamp(row, ts[t].out_dim);
                            // (clamped rows re-read the last row: no once-only check on W here)
                            Region w1("W", W[t].size), s1("S", S[t].size);
                            w1.touch(ro * rb + (size_t)c * bpl, bpl, "row slice");
                            s1.touch(ro * sb_row + (size_t)c * 4, 4, "row scale");
                            X.touch(((size_t)m * in_dim + (size_t)c * FM_CPL) * 4, FM_CPL * 4, "x chunk");
                            if (c == 0 && row <= ts[t].out_dim - 1) O[t].touch(((size_t)m * ts[t].out_dim + row) * 4, 4, "out");
                        }
                }
        O[t].expect_once(0, O[t].size);
    }
    std::printf("ok  %-58s plain kernel: %d rows per workgroup\n", g_case.c_str(), rpi);
}

// --------------------------------------------------------------------- dense against M positions
static void walk_pf_dense(int out_dim, int in_dim, int bits, int M) {
    g_case = "prefill dense " + std::to_string(out_dim) + "x" + std::to_string(in_dim) + " " + std::to_string(bits) +
             "-bit M=" + std::to_string(M);
    const bool teams = in_dim == 512;
    const FmPfSlab sl = fm_pf_slab(bits);
    CHECK(sl.ring >= 2 && sl.lds_bytes <= 160 * 1024, "LDS %d ring %d", sl.lds_bytes, sl.ring);
    const int row_bytes = in_dim * bits / 8, sb_bytes = (in_dim / 64) * 2, ng = in_dim / 64;
    const FmPfDenseWs ws = fm_pf_dense_ws(M, in_dim);
    Region WS("workspace", ws.total);
    Region Wt("W", (size_t)out_dim * row_bytes, 16), St("S", (size_t)out_dim * sb_bytes, 4), Bt("B", (size_t)out_dim * sb_bytes, 4);
    Region X("X", (size_t)M * in_dim * 4, 4), Out("out", (size_t)M * out_dim * 4);
    Region Xop("xop", (size_t)M * ng * 16 * 16, 16), Xs("xsums", (size_t)M * ng * 8, 8);
    // carve-up: every part inside the workspace, in order, not overlapping
    CHECK(ws.items + ((size_t)(M + 15) / 16) * 16 <= ws.n_items, "items part");
    CHECK(ws.n_items + 4 <= ws.xop && ws.xop + Xop.size <= ws.xsums && ws.xsums + Xs.size <= ws.total, "carve-up");
    // ---- fm_pf_dense_prep: block 0 writes the items, blocks 1.. prepare X
    const int n_items = (M + FM_PF_TM - 1) / FM_PF_TM;
    const int prep_tasks = M * ng * 2, prep_blocks = (prep_tasks + 1023) / 1024;
    for (int t = 0; t < prep_blocks * 1024; t++) {
        const FmPfPrepTask pt = fm_pf_prep_task(t, ng);
        if (pt.m >= M) continue;
        X.touch(((size_t)pt.m * in_dim + 64 * pt.g + 32 * pt.h) * 4, 32 * 4, "prep x");
        for (int k = 0; k < 4; k++)
            for (int p = 0; p < 2; p++) Xop.touch(fm_pf_xop_index(pt.m, ng, pt.g, k, pt.h, p) * 16, 16, "prep xop");
        if (pt.h == 0) Xs.touch(((size_t)pt.m * ng + pt.g) * 8, 8, "prep xsums");
    }
    X.expect_once(0, X.size);
    Xop.expect_once(0, Xop.size);
    Xs.expect_once(0, Xs.size);
    // ---- fm_pf_gemm
    const FmPfDenseGrid gr = fm_pf_dense_grid(M, out_dim, teams, N_CU);
    CHECK(gr.items == n_items, "items");
    const int passes = teams ? 1 : in_dim / 2048;
    const long T = (long)n_items * gr.n_steps;
    std::vector<uint8_t> seen(T, 0);
    for (int pass = 0; pass < passes; pass++) {
        Region Wp("W (pass)", Wt.size, 16);
        for (int b = 0; b < gr.grid; b++) {
            const FmRange tr = fm_share(T, fm_xcd_share(b, gr.grid), gr.grid);
            for (long t = tr.lo; t < tr.hi; t++) {
                const int it = (int)(t / gr.n_steps), s = (int)(t - (long)it * gr.n_steps);
                CHECK(it < n_items, "item %d", it);
                if (pass == 0) seen[t]++;
                const int start = it * FM_PF_TM, count = M - start < FM_PF_TM ? M - start : FM_PF_TM;
                for (int wave = 0; wave < 8; wave++) {
                    const int slab = teams ? (wave & 1) : wave + 8 * pass, team = teams ? (wave >> 1) : 0;
                    CHECK(4 * slab + 3 < ng, "slab %d of %d groups", slab, ng);
                    for (int mat = 0; mat < 2; mat++) {
                        const size_t row0 = fm_pf_dense_row(s, mat, team, teams);
                        CHECK(row0 + 32 <= (size_t)out_dim, "tile rows %zu", row0);
                        for (int lane = 0; lane < 64; lane++) {
                            for (int j = 0; j < sl.nq; j++) {
                                int valid;
                                const uint32_t co = fm_pf_piece_off(sl, j, lane, row_bytes, slab, &valid);
                                if (!valid) continue;
                                Wp.touch(row0 * row_bytes + co, 16, "slab piece");
                                CHECK((size_t)64 * 16 * j + 16 * lane + 16 <= (size_t)sl.lds_code, "piece slot in LDS");
                            }
                            const uint32_t so = fm_pf_sb_off(lane, sb_bytes, slab);
                            St.touch(row0 * sb_bytes + so, 4, "slab scales");
                            Bt.touch(row0 * sb_bytes + so, 4, "slab biases");
                        }
                    }
                    // operand registers of the item's positions (rows past the item read position 0)
                    for (int lane = 0; lane < 64; lane++) {
                        const int n = lane & 31, hh = lane >> 5, pos = n & 15, piece = n < 16 ? 0 : 1;
                        const size_t m = pos < count ? (size_t)(start + pos) : 0;
                        for (int gi = 0; gi < 4; gi++) {
                            for (int k = 0; k < 4; k++) {
                                Region xo("xop", Xop.size);
                                xo.touch(fm_pf_xop_index(m, ng, 4 * slab + gi, k, hh, piece) * 16, 16, "xop read");
                            }
                            Region xs("xsums", Xs.size);
                            xs.touch((m * ng + 4 * slab + gi) * 8, 8, "xsums read");
                        }
                        // results
                        if (!teams) {
                            const int my_pos = 8 * (wave >> 2) + 4 * hh + (wave & 3);
                            if (my_pos < count) {
                                Out.touch(((size_t)(start + my_pos) * out_dim + 64 * s + n) * 4, 4, "out");
                                Out.touch(((size_t)(start + my_pos) * out_dim + 64 * s + n + 32) * 4, 4, "out");
                            }
                        } else {
                            const int j = wave & 1, row = 256 * s + 64 * team + 32 * j + n;
                            for (int i = 0; i < 8; i++) {
                                const int tok = 8 * (i / 4) + 4 * hh + (i % 4);
                                if (tok < count) Out.touch(((size_t)(start + tok) * out_dim + row) * 4, 4, "out");
                            }
                        }
                    }
                }
            }
        }
        // a pass reads the pass's columns of every row once for every item
        (void)Wp;
    }
    for (long t = 0; t < T; t++) CHECK(seen[t] == 1, "step %ld taken %d times", t, (int)seen[t]);
    CHECK(Out.lo == 0 && Out.hi == Out.size, "output range %zu..%zu of %zu", Out.lo, Out.hi, Out.size);
    std::printf("ok  %-58s %d items x %d steps over %d workgroups, %d passes\n", g_case.c_str(), n_items, gr.n_steps,
                gr.grid, passes);
}

// ------------------------------------------------------------------------- affine expert geometry
struct Geom {
    int hidden, inter, bits;
    size_t gate_w, gate_s, gate_b, up_w, up_s, up_b, down_w, down_s, down_b, expert_size;
};
static Geom geom(int hidden, int inter, int bits) {
    Geom g{};
    g.hidden = hidden, g.inter = inter, g.bits = bits;
    const size_t gu_w = (size_t)inter * hidden * bits / 8, gu_s = (size_t)inter * (hidden / 64) * 2;
    const size_t d_w = (size_t)hidden * inter * bits / 8, d_s = (size_t)hidden * (inter / 64) * 2;
    size_t o = 0;
    g.gate_w = o; o += gu_w; g.gate_s = o; o += gu_s; g.gate_b = o; o += gu_s;
    g.up_w = o;   o += gu_w; g.up_s = o;   o += gu_s; g.up_b = o;   o += gu_s;
    g.down_w = o; o += d_w;  g.down_s = o; o += d_s;  g.down_b = o; o += d_s;
    g.expert_size = o;
    return g;
}

struct ChunkItem { int expert, start, count; };
struct ChunkLists {
    int n;
    std::vector<int> idx, cnt, off, sorted;
    // fm_pf_group: every expert's positions cut into items of at most tm
    std::vector<ChunkItem> items(int tm) const {
        std::vector<ChunkItem> v;
        for (int e = 0; e < (int)cnt.size(); e++)
            for (int s0 = 0; s0 < cnt[e]; s0 += tm) v.push_back({e, off[e] + s0, cnt[e] - s0 < tm ? cnt[e] - s0 : tm});
        return v;
    }
};
// routing of a chunk (K distinct experts per position, low indices preferred) and its counting sort
static ChunkLists chunk_lists(int M, int K, int E, unsigned seed) {
    ChunkLists c;
    const int n = M * K;
    c.n = n;
    c.idx.assign((size_t)n, 0);
    uint64_t st = 0x9E3779B97F4A7C15ull * (seed + 1);
    auto rnd = [&]() { st = st * 6364136223846793005ull + 1442695040888963407ull; return (double)(st >> 11) / 9007199254740992.0; };
    for (int m = 0; m < M; m++)
        for (int k = 0; k < K; k++) {
            for (;;) {
                const double u = rnd();
                const int e = (int)(E * u * u * u);
                bool dup = false;
                for (int j = 0; j < k; j++) dup = dup || c.idx[(size_t)m * K + j] == e;
                if (!dup && e < E) { c.idx[(size_t)m * K + k] = e; break; }
            }
        }
    c.cnt.assign(E, 0), c.off.assign(E + 1, 0);
    for (int p = 0; p < n; p++) c.cnt[c.idx[p]]++;
    for (int e = 0; e < E; e++) c.off[e + 1] = c.off[e] + c.cnt[e];
    c.sorted.assign((size_t)n, 0);
    std::vector<int> cur(c.off.begin(), c.off.end() - 1);
    for (int p = 0; p < n; p++) c.sorted[cur[c.idx[p]]++] = p;
    return c;
}

// fm_pf_group + fm_pf_rows (the grouped products of a chunk, config 3): M positions x K slots on E
// experts, routing skewed like the benchmark's.  The items and the sorted pair list are built by
// fm_pf_group's rule (restated: a counting sort); the workgroups' rounds, the per-lane pieces of a
// slot copy and the scale / bias offsets come from fm_index.h, as in the kernel.  Checked: the shares
// tile the rounds, a share's items fit its lane table, every item reads its expert's matrices
// exactly once, every load stays inside the blob / X / act / sorted list, every output element is
// written exactly once, the LDS of both kernels fits.
static void walk_pf_rows(int M, int K, int E, int bits, bool x_bf16, unsigned seed) {
    g_case = "chunk rows " + std::to_string(M) + " positions x " + std::to_string(K) + " on " + std::to_string(E) +
             " experts, " + std::to_string(bits) + "-bit, " + (x_bf16 ? "bf16" : "fp32") + " positions";
    const int hidden = 2048, inter = 512, n = M * K;
    const Geom g = geom(hidden, inter, bits);
    const ChunkLists cl = chunk_lists(M, K, E, seed);
    const std::vector<int> &sorted = cl.sorted;
    typedef ChunkItem Item;
    for (int mode = 0; mode < 2; mode++) {
        const bool gu = mode == 0;
        const int tm = gu ? (x_bf16 ? 16 : 8) : 16;
        const std::vector<Item> items = cl.items(tm);
        const int n_items = (int)items.size();
        CHECK(n_items <= E + n / tm + 1, "%d items in a list of %d", n_items, E + n / tm + 1);
        const int in_dim = gu ? hidden : inter, out_rows = gu ? inter : hidden;
        const int row_bytes = in_dim * bits / 8, sb_bytes = (in_dim / 64) * 2;
        const int S = in_dim / 256, CB = fm_pfr_slab_row_bytes(bits), NQ = 32 * (CB / 16) / 64;
        const int RPI = out_rows / (gu ? 16 : 32) / 8, TPI = RPI * 8;
        CHECK(S * CB == row_bytes, "slabs of %d bytes in a row of %d", CB, row_bytes);
        CHECK(NQ * 1024 == 32 * CB, "a slot copy is whole load instructions");
        // LDS: rings | image | bias / offset operands (PfRows)
        const int QK = gu ? 1 : 2, slot = 32 * CB + (gu ? 0 : 512), img = S * 4 * 2 * QK * 1024, side = S * 1024;
        int ring = (160 * 1024 - 2048 - img - side) / (8 * slot);
        if (ring > 4) ring = 4;
        CHECK(ring >= 2 && 8 * ring * slot + img + side + 2048 <= 160 * 1024, "LDS: ring of %d", ring);
        for (int j = 0; j < NQ; j++) CHECK(1024 * j + 63 * 16 + 16 <= 32 * CB, "codes of a slot");
        const long RT = (long)n_items * RPI;
        const int G = fm_pfr_grid(E + n / tm, N_CU);
        std::vector<uint8_t> round_owner((size_t)RT, 0);
        Region X("X", (size_t)M * hidden * (x_bf16 ? 2 : 4)), act("act", (size_t)n * inter * 4, 4);
        Region eo("expert_out", (size_t)n * hidden * 4, 4), srt("sorted", (size_t)n * 4);
        for (int b = 0; b < G; b++) {
            const FmRange rr = fm_pfr_rounds(RT, (unsigned)b, (unsigned)G);
            CHECK(rr.lo >= 0 && rr.hi <= RT && rr.lo <= rr.hi, "rounds [%ld, %ld) of %ld", rr.lo, rr.hi, RT);
            if (rr.lo >= rr.hi) continue;
            for (long r = rr.lo; r < rr.hi; r++) round_owner[(size_t)r]++;
            const int it0 = (int)(rr.lo / RPI), it_last = (int)((rr.hi - 1) / RPI);
            CHECK(it_last - it0 < 64 && it_last < n_items, "workgroup %d: items %d..%d of %d", b, it0, it_last, n_items);
            // staging of every item of the share: its pair ids, then 64 activations per (group, position)
            for (int it = it0; it <= it_last && it < n_items; it++) {
                const Item &I = items[it];
                for (int pos = 0; pos < I.count; pos++) {
                    srt.touch((size_t)(I.start + pos) * 4, 4, "pair id");
                    if (I.start + pos >= n) continue;
                    const int pair = sorted[I.start + pos];
                    for (int sg = 0; sg < S * 4; sg++) {
                        if (gu) X.touch(((size_t)(pair / K) * hidden + 64 * (size_t)sg) * (x_bf16 ? 2 : 4), 64 * (x_bf16 ? 2 : 4), "X row");
                        else act.touch(((size_t)(I.start + pos) * inter + 64 * (size_t)sg) * 4, 256, "act row");
                    }
                }
            }
        }
        size_t bad = 0;
        for (long r = 0; r < RT; r++) bad += round_owner[(size_t)r] != 1;
        CHECK(bad == 0, "%zu of %ld rounds not owned by exactly one workgroup", bad, RT);
        // every item: its tasks' loads tile the expert's matrices; outputs once
        if (!gu) act = Region("act", (size_t)n * inter * 4);      // (read above; the output of the other mode)
        Region out = gu ? Region("act", (size_t)n * inter * 4, 4) : Region("expert_out", (size_t)n * hidden * 4, 4);
        for (int it = 0; it < n_items; it++) {
            const Item &I = items[it];
            CHECK(I.expert >= 0 && I.expert < E && I.count >= 1 && I.count <= tm && I.start + I.count <= n, "item %d", it);
            Region blob("expert blob", g.expert_size, 4);
            for (int t = 0; t < TPI; t++) {
                const size_t r0 = (size_t)t * (gu ? 16 : 32);
                for (int s0 = 0; s0 < S; s0++) {
                    for (int q = 0; q < 64 * NQ; q++)
                        blob.touch(r0 * row_bytes + (size_t)s0 * CB +
                                       fm_pfr_piece_off(gu, bits, q, (uint32_t)(gu ? g.gate_w : g.down_w), (uint32_t)g.up_w, row_bytes),
                                   16, "codes");
                    if (!gu)
                        for (int lane = 0; lane < 64; lane++) {
                            blob.touch(r0 * sb_bytes + (size_t)s0 * 8 + fm_pfr_sb_off(0, lane, (uint32_t)g.down_s, 0u, sb_bytes), 4, "scales");
                            blob.touch(r0 * sb_bytes + (size_t)s0 * 8 + fm_pfr_sb_off(0, lane, (uint32_t)g.down_b, 0u, sb_bytes), 4, "biases");
                        }
                }
                if (gu)          // a task's scales and biases: four contiguous KB, 16 bytes per lane
                    for (int lane = 0; lane < 64; lane++) {
                        const size_t sc_lane = (size_t)(lane & 15) * sb_bytes + 16 * (size_t)(lane >> 4);
                        for (size_t m0 : {g.gate_s, g.gate_b, g.up_s, g.up_b}) blob.touch(r0 * sb_bytes + m0 + sc_lane, 16, "scales of a task");
                    }
                for (int tok = 0; tok < I.count; tok++)
                    for (int nn = 0; nn < 16; nn++) {
                        if (gu) out.touch(((size_t)(I.start + tok) * inter + r0 + nn) * 4, 4, "act");
                        else {
                            const size_t pair = (size_t)sorted[I.start + tok];
                            out.touch((pair * hidden + r0 + nn) * 4, 4, "expert_out");
                            out.touch((pair * hidden + r0 + nn + 16) * 4, 4, "expert_out");
                        }
                    }
            }
            if (gu) {
                blob.expect_once(g.gate_w, g.up_w + (g.up_s - g.up_w) + 2 * (g.up_b - g.up_s));      // gate and up: codes, scales, biases
                blob.expect_untouched(g.down_w, g.expert_size);
            } else {
                blob.expect_once(g.down_w, g.expert_size);
                blob.expect_untouched(0, g.down_w);
            }
        }
        out.expect_once(0, out.size);
        std::printf("ok  %-58s %s: %d items, %ld rounds over %d workgroups\n", g_case.c_str(), gu ? "gate/up" : "down", n_items, RT, G);
    }
}

// fm_gq_gate_up / fm_gq_down (the grouped products of a chunk on a GGUF store, config 4's chunk
// variant): the kernels' loops restated — a workgroup's share of the (item, eight tiles) units, the
// staging of an item, a wave's tile, the blocks of its rows and the first block of its next tile
// requested ahead (which may belong to the next item's expert).  Checked: every block read lies in
// the expert's slab, every tile of every item is multiplied exactly once, the ahead-requests stay
// inside the store, outputs are written exactly once, the images fit the LDS the launcher asks for.
static void walk_gq(int M, int K, int E, int hidden, int inter, unsigned seed) {
    g_case = "gguf chunk grouped " + std::to_string(M) + " positions x " + std::to_string(K) + " on " + std::to_string(E) +
             " experts, " + std::to_string(hidden) + "x" + std::to_string(inter);
    const ChunkLists cl = chunk_lists(M, K, E, seed);
    const int n = cl.n;
    for (int mode = 0; mode < 2; mode++) {
        const bool gu = mode == 0;
        const int tm = gu ? (hidden <= 2048 ? 16 : 8) : 16;
        const std::vector<ChunkItem> items = cl.items(tm);
        const int n_items = (int)items.size();
        CHECK(n_items <= E + n / tm + 1, "%d items in a list of %d", n_items, E + n / tm + 1);
        const int in_dim = gu ? hidden : inter, rows = gu ? inter : hidden;
        const int NB = in_dim / 256, blk = gu ? 144 : 210, NW = 8;
        const size_t row_bytes = (size_t)NB * blk, slab = (size_t)rows * row_bytes;
        const int tiles = rows / 16, per_item = (tiles + NW - 1) / NW;
        const size_t lds = gu ? (size_t)(hidden / 32) * ((tm == 16 ? 2048 : 1024) + 64)
                              : (size_t)(inter / 16) * 1024 + (size_t)(inter / 256) * 1536;
        CHECK(lds <= 160 * 1024 - 1024, "LDS %zu", lds);
        const int G = gu ? N_CU : 2 * N_CU;
        const long total = (long)n_items * per_item;
        Region X("X", (size_t)M * hidden * 4), act_in("act", (size_t)n * inter * 4), srt("sorted", (size_t)n * 4);
        Region out = gu ? Region("act", (size_t)n * inter * 4, 4) : Region("expert_out", (size_t)n * hidden * 4, 4);
        // per (item, tile): how often it was multiplied
        std::vector<uint8_t> done((size_t)n_items * tiles, 0);
        Region store("expert slabs", (size_t)E * slab);       // gate (and, at the same offsets, up) or down
        auto block = [&](size_t row_off, int b, const char *what) {     // a lane's words of block b of a row
            store.touch(row_off + (size_t)b * blk, (size_t)blk, what);
        };
        for (int bq = 0; bq < G; bq++) {
            const FmRange sh = fm_share(total, (unsigned)bq, (unsigned)G);
            int cur_item = -1;
            ChunkItem item{0, 0, 0}, item_next{0, 0, 0};
            for (long u = sh.lo; u < sh.hi; u++) {
                const int it = (int)(u / per_item), part = (int)(u - (long)it * per_item);
                CHECK(it < n_items, "unit %ld -> item %d of %d", u, it, n_items);
                if (it >= n_items) break;
                if (it != cur_item) {
                    cur_item = it;
                    item = items[it];
                    item_next = items[it + 1 < n_items ? it + 1 : it];
                    for (int p = 0; p < item.count; p++) {
                        srt.touch((size_t)(item.start + p) * 4, 4, "pair id");
                        if (gu) X.touch((size_t)(cl.sorted[item.start + p] / K) * hidden * 4, (size_t)hidden * 4, "X row");
                        else act_in.touch((size_t)(item.start + p) * inter * 4, (size_t)inter * 4, "act row");
                    }
                }
                for (int wave = 0; wave < NW; wave++) {
                    const int tile = part * NW + wave;
                    if (tile >= tiles) continue;
                    done[(size_t)it * tiles + tile]++;
                    for (int nn = 0; nn < 16; nn++) {
                        const size_t row_off = ((size_t)item.expert * rows + (size_t)tile * 16 + nn) * row_bytes;
                        for (int b = 0; b < NB; b++) block(row_off, b, "block of the tile's row");
                        for (int pos = 0; pos < item.count; pos++) {
                            if (gu) out.touch(((size_t)(item.start + pos) * inter + (size_t)tile * 16 + nn) * 4, 4, "act");
                            else out.touch(((size_t)cl.sorted[item.start + pos] * hidden + (size_t)tile * 16 + nn) * 4, 4, "expert_out");
                        }
                    }
                    // the first block of the wave's tile of the next unit, requested ahead
                    if (u + 1 < sh.hi) {
                        const int it2 = (int)((u + 1) / per_item), tile2 = (int)(u + 1 - (long)it2 * per_item) * NW + wave;
                        if (tile2 < tiles) {
                            CHECK(it2 == cur_item || it2 == cur_item + 1, "next unit's item %d after %d", it2, cur_item);
                            CHECK(it2 < n_items, "next unit's item %d of %d", it2, n_items);
                            const int e2 = it2 == cur_item ? item.expert : item_next.expert;
                            if (it2 < n_items) CHECK(e2 == items[it2].expert, "expert of the item ahead");
                            for (int nn = 0; nn < 16; nn++)
                                block(((size_t)e2 * rows + (size_t)tile2 * 16 + nn) * row_bytes, 0, "block requested ahead");
                        }
                    }
                }
            }
        }
        size_t bad = 0;
        for (uint8_t d : done) bad += d != 1;
        CHECK(bad == 0, "%zu (item, tile) combinations not multiplied exactly once", bad);
        out.expect_once(0, out.size);
        std::printf("ok  %-58s %s: %d items, %ld units over %d workgroups\n", g_case.c_str(), gu ? "gate/up" : "down", n_items, total, G);
    }
}

// fm_moe_fused_rows: n_groups layer groups (layers of a step / positions of a chunk) x K slots.
// Every pair gets an expert blob of its own here, so "read exactly once" is checked per pair.
static void walk_fused_rows(int n_groups, int K, int hidden, int inter, int bits) {
    g_case = "fused rows " + std::to_string(n_groups) + " groups x " + std::to_string(K) + ", " + std::to_string(bits) + "-bit";
    const Geom g = geom(hidden, inter, bits);
    const int lpr_up = hidden / FM_CPL, lpr_dn = lpr_up / 4, n_pairs = n_groups * K;
    CHECK(inter / FM_CPL == lpr_dn, "widths");
    const int rps_up = FM_WAVE / lpr_up, rps_dn = FM_WAVE / lpr_dn;
    const Fm2Plan plan = fm2_plan(n_pairs, K, inter, hidden, lpr_up, N_CU);
    if (!plan.ok) {
        std::printf("--  %-58s not taken by this launch form\n", g_case.c_str());
        return;
    }
    const int G = plan.wgs;
    const Fm2Dims dm = fm2_dims(n_pairs, K, G, inter, hidden, lpr_up);
    const uint32_t gu_wstep = rps_up * (hidden * bits / 8), gu_sstep = rps_up * (hidden / 64) * 2;
    const uint32_t dn_wstep = rps_dn * (inter * bits / 8), dn_sstep = rps_dn * (inter / 64) * 2;
    // LDS: rings | two gate/up images | segment tables | partial vectors
    const int ring = 2, n_waves = 12;          // fm_decode.hip: FM_NW, FmDma::RING
    const size_t slot = 64 * (size_t)fm_lane_bytes(bits) + 512 + 16;
    const size_t img_up = (size_t)16 * 4 * lpr_up * 16 + lpr_up * 16, img_dn = (size_t)16 * 4 * lpr_dn * 16 + lpr_dn * 16;
    const size_t seg_bytes = 8 * 8 + 8 * 4 + 6 * 4;
    const size_t lds = (size_t)n_waves * ring * slot + 2 * img_up + FM2_MAX_SEG * seg_bytes + FM2_PART_BYTES;
    CHECK(lds <= 160 * 1024, "LDS %zu", lds);
    CHECK((size_t)FM_MAX_K * img_dn <= 2 * img_up, "down images in the gate/up images");
    std::vector<Region> blob;
    blob.reserve(n_pairs);
    for (int p = 0; p < n_pairs; p++) blob.emplace_back("expert blob", g.expert_size, 4);
    Region act("act", (size_t)n_pairs * inter * 4, 4), out("out", (size_t)n_groups * hidden * 4, 4);
    Region X("x", (size_t)n_groups * hidden * 4), idx("idx", (size_t)n_pairs * 4);
    int max_seq = 0;
    size_t max_bytes = 0, min_bytes = (size_t)-1;
    for (int gi = 0; gi <= G; gi++) {
        // the prepared divisions against plain ones
        const uint32_t ug = (uint32_t)gi;
        uint32_t dn_ref;
        if (ug >= dm.G) dn_ref = dm.rb_total;
        else if (dm.G < dm.L) dn_ref = dm.rb_total * ug / dm.G;
        else {
            const uint32_t l = ug * dm.L / dm.G;
            const uint32_t g_lo = (l * dm.G + dm.L - 1u) / dm.L, g_hi = ((l + 1u) * dm.G + dm.L - 1u) / dm.L;
            CHECK(g_hi - g_lo == dm.wq || g_hi - g_lo == dm.wq + 1u, "layer %u has %u workgroups", l, g_hi - g_lo);
            dn_ref = l * dm.dn_upp + dm.dn_upp * (ug - g_lo) / (g_hi - g_lo);
        }
        CHECK(fm2_dn_start(dm, ug) == dn_ref, "first down row block of workgroup %d", gi);
        const uint32_t t = dm.s_total * ug / dm.G, dd = dn_ref * dm.K * dm.dn_wt;
        CHECK(dm.gu_wt == 2u && dm.dn_wt == 1u, "affine experts: two slices per gate/up unit, one per down unit");
        uint32_t gu_ref = t > dd ? (t - dd) / dm.gu_wt : 0u;
        if (gu_ref > dm.gu_total) gu_ref = dm.gu_total;
        CHECK(fm2_gu_start(dm, ug, dn_ref) == gu_ref, "first gate/up unit of workgroup %d", gi);
    }
    for (int gi = 0; gi < G; gi++) {
        const Fm2Split sp = fm2_split(dm, gi);
        const int n_seq = sp.n_up + sp.n_dn;
        if (n_seq > max_seq) max_seq = n_seq;
        CHECK(sp.n_up <= 2, "workgroup %d: %d gate/up segments", gi, sp.n_up);
        CHECK(n_seq <= FM2_MAX_SEG && n_seq <= 64, "workgroup %d: %d segments", gi, n_seq);
        // the two input vectors loaded up front
        if (sp.n_up > 0) X.touch((size_t)sp.gu_s0 * hidden * 4, (size_t)hidden * 4, "x of the first segment");
        if (sp.n_up > 1) X.touch((size_t)(sp.gu_s0 + 1) * hidden * 4, (size_t)hidden * 4, "x of the second segment");
        size_t bytes = 0;
        for (int qq = 0; qq < n_seq; qq++) {
            const Fm2Part pt = fm2_part(dm, sp, qq);
            CHECK(pt.seg < (uint32_t)n_groups, "segment %u", pt.seg);
            for (int k = 0; k < K; k++) idx.touch(((size_t)pt.seg * K + k) * 4, 4, "idx");
            if (pt.gu) {
                for (uint32_t ul = 0; ul < pt.n; ul++) {
                    uint32_t pn, rsn;
                    fm2_gu_unit(pt.first, ul, dm.by_gu_upp, &pn, &rsn);
                    CHECK(pn < (uint32_t)K && rsn < dm.gu_upp, "gate/up unit %u -> slot %u step %u", ul, pn, rsn);
                    if (pn >= (uint32_t)K) continue;
                    Region &bl = blob[pt.seg * K + pn];
                    for (int second = 0; second < 2; second++)
                        unit_dma(bl, (size_t)rsn * gu_wstep + (second ? g.up_w : g.gate_w), bl,
                                 (size_t)rsn * gu_sstep + (second ? g.up_s : g.gate_s), bl,
                                 (size_t)rsn * gu_sstep + (second ? g.up_b : g.gate_b), bits);
                    bytes += 2 * (64 * (size_t)fm_lane_bytes(bits) + 512);
                    for (int lane = 0; lane < 64; lane++) {
                        const FmUnitLane ulr = fm_unit_lane(lane, lpr_up, fm_lane_bytes(bits), hidden * bits / 8, (hidden / 64) * 2);
                        if (ulr.ch == 0)
                            act.touch((((size_t)pt.seg * dm.gu_segu + pt.first) * rps_up + ulr.row_in_step + (size_t)ul * rps_up) * 4, 4, "act");
                    }
                }
            } else {
                CHECK(pt.first % K == 0 && pt.n % K == 0, "down part %u + %u not whole row blocks", pt.first, pt.n);
                const uint32_t rb_first = pt.first / K, nrb = pt.n / K;
                const float inv = 1.0f / (float)(nrb ? nrb : 1u);
                CHECK((size_t)nrb * K * rps_dn * 4 <= FM2_PART_BYTES, "partial vectors of %u row blocks", nrb);
                for (uint32_t ul = 0; ul < pt.n; ul++) {
                    uint32_t pn, rsn;
                    fm2_dn_unit(rb_first, nrb, inv, ul, &pn, &rsn);
                    CHECK(pn == ul / nrb && rsn == rb_first + ul % nrb, "down unit %u -> slot %u block %u", ul, pn, rsn);
                    CHECK(pn < (uint32_t)K && rsn < dm.dn_upp, "down unit %u -> slot %u block %u", ul, pn, rsn);
                    if (pn >= (uint32_t)K) continue;
                    Region &bl = blob[pt.seg * K + pn];
                    unit_dma(bl, (size_t)rsn * dn_wstep + g.down_w, bl, (size_t)rsn * dn_sstep + g.down_s, bl,
                             (size_t)rsn * dn_sstep + g.down_b, bits);
                    bytes += 64 * (size_t)fm_lane_bytes(bits) + 512;
                    const uint32_t rbi = ul - pn * nrb;
                    for (int ris = 0; ris < rps_dn; ris++)
                        CHECK(4u * ((rbi * K + pn) * rps_dn + ris) + 4 <= FM2_PART_BYTES, "partial slot");
                }
                // activations of the layer's K experts, and the part's rows of out
                Region a1("act", act.size);
                a1.touch((size_t)pt.seg * K * inter * 4, (size_t)K * inter * 4, "act of the layer");
                const int rows = (int)nrb * rps_dn;
                out.touch(((size_t)pt.seg * hidden + (size_t)rb_first * rps_dn) * 4, (size_t)rows * 4, "out rows");
            }
        }
        if (bytes > max_bytes) max_bytes = bytes;
        if (bytes < min_bytes) min_bytes = bytes;
    }
    for (int p = 0; p < n_pairs; p++) blob[p].expect_once(0, g.expert_size);
    act.expect_once(0, act.size);
    out.expect_once(0, out.size);
    std::printf("ok  %-58s %d workgroups, <= %d segments, bytes per workgroup %zu..%zu\n", g_case.c_str(), G, max_seq,
                min_bytes, max_bytes);
}

// the same split over a grid of shapes, unit bookkeeping only (no byte maps): every gate/up unit
// and every (row block, slot) of the down phase handed out exactly once, tables within their sizes
static void sweep_fused_rows() {
    g_case = "fused rows, sweep of shapes";
    int taken = 0;
    for (int lpr_up : {4, 8, 16})
        for (int n_groups : {1, 2, 3, 5, 8, 13, 31, 40, 41, 47, 64, 100})
            for (int K : {1, 2, 5, 8})
                for (int n_cu : {256, 240, 104, 30}) {
                    const int hidden = 128 * lpr_up, inter = hidden / 4;     // the kernel covers inter = hidden / 4
                    const int n_pairs = n_groups * K;
                    const Fm2Plan plan = fm2_plan(n_pairs, K, inter, hidden, lpr_up, n_cu);
                    if (!plan.ok) continue;
                    taken++;
                    const int rps_dn = FM_WAVE / (lpr_up / 4);
                    const Fm2Dims dm = fm2_dims(n_pairs, K, plan.wgs, inter, hidden, lpr_up);
                    std::vector<uint8_t> gu(dm.gu_total, 0), dn((size_t)dm.rb_total * K, 0);
                    for (int b = 0; b < plan.wgs; b++) {
                        const Fm2Split sp = fm2_split(dm, b);
                        CHECK(sp.n_up <= 2 && sp.n_up + sp.n_dn <= FM2_MAX_SEG, "%d groups K %d lpr %d cu %d: segments %d + %d",
                              n_groups, K, lpr_up, n_cu, sp.n_up, sp.n_dn);
                        for (int qq = 0; qq < sp.n_up + sp.n_dn; qq++) {
                            const Fm2Part pt = fm2_part(dm, sp, qq);
                            if (pt.gu) {
                                for (uint32_t ul = 0; ul < pt.n; ul++) {
                                    const size_t u = (size_t)pt.seg * dm.gu_segu + pt.first + ul;
                                    CHECK(pt.first + ul < dm.gu_segu && u < gu.size(), "gate/up unit");
                                    if (u < gu.size()) gu[u]++;
                                }
                            } else {
                                const uint32_t rb_first = pt.first / K, nrb = pt.n / K;
                                CHECK(pt.first % K == 0 && pt.n % K == 0 && (size_t)nrb * K * rps_dn * 4 <= FM2_PART_BYTES,
                                      "%d groups K %d lpr %d cu %d: part of %u row blocks", n_groups, K, lpr_up, n_cu, nrb);
                                const float inv = 1.0f / (float)(nrb ? nrb : 1u);
                                for (uint32_t ul = 0; ul < pt.n; ul++) {
                                    uint32_t pn, rsn;
                                    fm2_dn_unit(rb_first, nrb, inv, ul, &pn, &rsn);
                                    CHECK(pn < (uint32_t)K && rsn < dm.dn_upp, "down unit");
                                    const size_t u = ((size_t)pt.seg * dm.dn_upp + rsn) * K + pn;
                                    if (pn < (uint32_t)K && rsn < dm.dn_upp) dn[u]++;
                                }
                            }
                        }
                    }
                    size_t bad = 0;
                    for (uint8_t c : gu) bad += c != 1;
                    for (uint8_t c : dn) bad += c != 1;
                    CHECK(bad == 0, "%d groups K %d lpr %d cu %d: %zu units not handed out exactly once", n_groups, K, lpr_up, n_cu, bad);
                }
    std::printf("ok  %-58s %d shapes taken by this launch form\n", g_case.c_str(), taken);
}

// the streaming phases with per-phase proportional shares: fm_gate_up_swiglu_lds / fm_down_lds as
// separate launches (per_wave 2) and fm_moe_fused (both phases in one grid)
static void walk_phases(int n_groups, int K, int hidden, int inter, int bits, bool fused) {
    g_case = std::string(fused ? "fused (counters) " : "split phases ") + std::to_string(n_groups) + " groups x " +
             std::to_string(K) + ", " + std::to_string(bits) + "-bit";
    const Geom g = geom(hidden, inter, bits);
    const int lpr_up = hidden / FM_CPL, lpr_dn = inter / FM_CPL, n_pairs = n_groups * K;
    const int rps_up = FM_WAVE / lpr_up, rps_dn = FM_WAVE / lpr_dn;
    const long gu_upp = inter / rps_up, dn_upp = hidden / rps_dn;
    const long gu_total = (long)n_pairs * gu_upp, dn_total = (long)n_pairs * dn_upp;
    const uint32_t gu_wstep = rps_up * (hidden * bits / 8), gu_sstep = rps_up * (hidden / 64) * 2;
    const uint32_t dn_wstep = rps_dn * (inter * bits / 8), dn_sstep = rps_dn * (inter / 64) * 2;
    std::vector<Region> blob;
    blob.reserve(n_pairs);
    for (int p = 0; p < n_pairs; p++) blob.emplace_back("expert blob", g.expert_size, 4);
    Region act("act", (size_t)n_pairs * inter * 4, 4), eo("expert_out", (size_t)n_pairs * hidden * 4, 4);
    for (int phase = 0; phase < 2; phase++) {
        const bool up = phase == 0;
        const long G = fused ? fm1_fused_wgs(gu_total, dn_total, N_CU) : fm_stream_wgs(up ? gu_total : dn_total, N_CU, 2, 12);
        for (long b = 0; b < G; b++) {
            const Fm1Split sp = fm1_split(fused || up ? gu_total : 0, fused || !up ? dn_total : 0, gu_upp * K, dn_upp, (unsigned)b, (unsigned)G);
            const int q0 = up ? 0 : sp.n_up, q1 = up ? sp.n_up : sp.n_up + sp.n_dn;
            for (int q = q0; q < q1; q++) {
                const int seg = fm1_seg(sp, q);
                uint32_t first, n;
                fm1_part(sp, q, up, &first, &n);
                CHECK(seg >= 0 && seg < (up ? n_groups : n_pairs), "segment %d", seg);
                for (uint32_t ul = 0; ul < n; ul++) {
                    const uint32_t uq = first + ul;
                    const uint32_t pn = up ? uq / (uint32_t)gu_upp : 0u, rsn = uq - pn * (uint32_t)gu_upp;
                    CHECK(pn < (uint32_t)K && rsn < (uint32_t)(up ? gu_upp : dn_upp), "unit %u -> slot %u step %u", ul, pn, rsn);
                    if (pn >= (uint32_t)K) continue;
                    Region &bl = blob[up ? seg * K + pn : seg];
                    if (up) {
                        for (int second = 0; second < 2; second++)
                            unit_dma(bl, (size_t)rsn * gu_wstep + (second ? g.up_w : g.gate_w), bl,
                                     (size_t)rsn * gu_sstep + (second ? g.up_s : g.gate_s), bl,
                                     (size_t)rsn * gu_sstep + (second ? g.up_b : g.gate_b), bits);
                        for (int ris = 0; ris < rps_up; ris++)
                            act.touch((((size_t)seg * gu_upp * K + first) * rps_up + ris + (size_t)ul * rps_up) * 4, 4, "act");
                    } else {
                        unit_dma(bl, (size_t)rsn * dn_wstep + g.down_w, bl, (size_t)rsn * dn_sstep + g.down_s, bl,
                                 (size_t)rsn * dn_sstep + g.down_b, bits);
                        for (int ris = 0; ris < rps_dn; ris++)
                            eo.touch((((size_t)seg * dn_upp + first) * rps_dn + ris + (size_t)ul * rps_dn) * 4, 4, "expert_out");
                    }
                }
            }
        }
    }
    for (int p = 0; p < n_pairs; p++) blob[p].expect_once(0, g.expert_size);
    act.expect_once(0, act.size);
    eo.expect_once(0, eo.size);
    std::printf("ok  %-58s\n", g_case.c_str());
}

// ----------------------------------------------------------------------------- GGUF streaming
static void walk_gguf_stream(int n_groups, int K, int hidden, int inter, bool gu, int down_q6 = 1,
                             const char *label = nullptr) {
    const bool q6 = !gu && down_q6;
    g_case = label ? std::string("gguf dense ") + label
                   : std::string("gguf stream ") + (gu ? "gate/up Q4_K " : "down Q6_K ") + std::to_string(n_groups) + " groups x " + std::to_string(K);
    const int n_pairs = n_groups * K, in_dim = gu ? hidden : inter, rows = gu ? inter : hidden;
    const FmGgPlan pl = fm_gg_plan(n_pairs, K, in_dim, rows, q6, gu, N_CU);
    if (!pl.ok) {
        std::printf("--  %-58s not taken by the streaming kernel\n", g_case.c_str());
        return;
    }
    const size_t slab = (size_t)rows * pl.row_bytes;       // one expert's rows of one matrix
    CHECK((size_t)pl.upp * pl.slot_data == slab, "slices tile the expert");
    const int ring = pl.ring, nreg = q6 ? 32 : 64, img_lpr = pl.wide ? 2 * pl.lpr : pl.lpr;
    CHECK(ring == FM_GG_RING, "ring of %d slices", ring);
    CHECK(pl.row_bytes == (q6 ? (in_dim / 256) * 210 : (in_dim / 256) * 144), "row of %d bytes", pl.row_bytes);
    const size_t img = (size_t)(nreg / 4) * 4 * img_lpr * 16 + img_lpr * 16;
    if (q6) {   // every column of the row is some lane's: chunk c (and c + 16 where a lane owns two), value v
        std::vector<uint8_t> seen((size_t)in_dim, 0);
        for (int lane = 0; lane < 64; lane++) {
            const int j = lane & 3, ch = (lane >> 2) % pl.lpr, ris = 4 * (lane / (4 * pl.lpr)) + j;
            CHECK(ris < pl.rps, "row in step %d", ris);
            if (ris != 0) continue;
            for (int pass = 0; pass < (pl.wide ? 2 : 1); pass++) {
                const int c = ch + 16 * pass;
                CHECK(4 * c + 3 < 4 * img_lpr, "image entry of chunk %d", c);
                // bytes of the lane's piece inside its row: ql [64 hf + 32 sd, +32) and qh [128 + 32 hf, +32) of block c / 4
                const int hf = (c >> 1) & 1, sd = c & 1, blk = (c >> 2) * 210;
                CHECK(blk + 210 <= pl.row_bytes && blk + 64 * hf + 32 * sd + 36 <= pl.row_bytes + 2, "piece of chunk %d", c);
                for (int v = 0; v < 64; v++) {
                    const int col = 128 * (c >> 1) + 32 * (c & 1) + (v < 32 ? v : v + 32);
                    CHECK(col < in_dim, "column %d", col);
                    if (col < in_dim) seen[col]++;
                }
            }
        }
        for (int c = 0; c < in_dim; c++) CHECK(seen[c] == 1, "column %d owned %d times", c, (int)seen[c]);
    }
    const size_t lds = (size_t)pl.nw * ring * (pl.slot_data + 16) + pl.n_img * img + pl.n_pair * 32 + 16;
    CHECK(lds <= 160 * 1024, "LDS %zu", lds);
    std::vector<Region> m0, m1;
    for (int p = 0; p < n_pairs; p++) {
        m0.emplace_back(gu ? "gate rows" : "down rows", slab, 2);
        if (gu) m1.emplace_back("up rows", slab, 2);
    }
    Region outv(gu ? "act" : "expert_out", (size_t)n_pairs * rows * 4, 4);
    const FmDiv by_upp = fm_div_make(pl.upp), by_k = fm_div_make(K);
    for (int b = 0; b < pl.wgs; b++) {
        const FmRange wg = fm_share(pl.total, b, pl.wgs);
        if (wg.hi == wg.lo) continue;
        const uint32_t pair0 = fm_div(by_upp, (uint32_t)wg.lo), pair_last = fm_div(by_upp, (uint32_t)wg.hi - 1u);
        CHECK(pair0 == wg.lo / pl.upp && pair_last == (wg.hi - 1) / pl.upp, "division by multiply-shift");
        CHECK(pair_last - pair0 < (uint32_t)pl.n_pair, "workgroup %d touches %u pairs", b, pair_last - pair0 + 1);
        const uint32_t vid0 = gu ? fm_div(by_k, pair0) : pair0, vid1 = gu ? fm_div(by_k, pair_last) : pair_last;
        CHECK(vid1 - vid0 < (uint32_t)pl.n_img, "workgroup %d needs %u images", b, vid1 - vid0 + 1);
        for (long u = wg.lo; u < wg.hi; u++) {
            const uint32_t pair = fm_div(by_upp, (uint32_t)u), step = (uint32_t)u - pair * by_upp.d;
            CHECK(pair == u / pl.upp && pair < (uint32_t)n_pairs && step < (uint32_t)pl.upp, "unit %ld", u);
            for (int kn = 0; kn < (gu ? 2 : 1); kn++) {
                Region &r = kn ? m1[pair] : m0[pair];
                for (int lane = 0; lane < 64; lane++)
                    for (int i = 0; i * 1024 < pl.slot_data; i++)
                        if (i * 1024 + lane * 16 < pl.slot_data) {
                            // the last load of a slice may be partial in bytes as well: 16 bytes per
                            // lane must still end inside the slice
                            CHECK(i * 1024 + lane * 16 + 16 <= pl.slot_data, "load %d lane %d runs over the slice", i, lane);
                            r.touch((size_t)step * pl.slot_data + (size_t)i * 1024 + (size_t)lane * 16, 16, "slice");
                        }
            }
            for (int ris = 0; ris < pl.rps; ris++) outv.touch(((size_t)pair * rows + step * pl.rps + ris) * 4, 4, "result");
        }
    }
    for (int p = 0; p < n_pairs; p++) {
        m0[p].expect_once(0, slab);
        if (gu) m1[p].expect_once(0, slab);
    }
    outv.expect_once(0, outv.size);
    std::printf("ok  %-58s %ld units over %d workgroups\n", g_case.c_str(), pl.total, pl.wgs);
}


// fm_gguf_fused_rows: the GGUF experts as one launch.  Every pair gets slabs of its own here, so
// "read exactly once" is checked per pair and matrix.
static void walk_gguf_fused(int n_groups, int K, int hidden, int inter, int down_q6) {
    g_case = std::string("gguf fused rows ") + (down_q6 ? "Q6_K" : "Q4_K") + " down, " + std::to_string(n_groups) + " groups x " +
             std::to_string(K) + ", " + std::to_string(hidden) + "x" + std::to_string(inter);
    const int n_pairs = n_groups * K;
    const FmGg2Plan pl = fm_gg2_plan(n_pairs, K, hidden, inter, down_q6, N_CU);
    if (!pl.ok) {
        std::printf("--  %-58s not taken by this launch form\n", g_case.c_str());
        return;
    }
    const int G = pl.wgs;
    CHECK(G >= 1 && G <= N_CU, "%d workgroups", G);
    const Fm2Dims dm = fm2_dims_units(n_pairs, K, G, pl.gu_upp, pl.dn_upp, pl.gu_wt, pl.dn_wt);
    CHECK((uint64_t)dm.s_total * (uint64_t)G < (1ull << 31), "32-bit products");
    const size_t gu_row = (size_t)(hidden / 256) * 144, dn_row = (size_t)(inter / 256) * (down_q6 ? 210 : 144);
    const size_t gu_slab = (size_t)inter * gu_row, dn_slab = (size_t)hidden * dn_row;
    CHECK((size_t)pl.gu_upp * pl.slot_up == gu_slab && (size_t)pl.dn_upp * pl.slot_dn == dn_slab, "slices tile the expert");
    // LDS: rings | images | segment tables | partial vectors
    CHECK(FM_GG2_RING_UP * (pl.slot_up + 16) <= pl.ring_bytes && (uint32_t)pl.ring_dn * (pl.slot_dn + 16) <= pl.ring_bytes,
          "ring slots inside a wave's ring");
    CHECK(2 * pl.img_up <= pl.img_bytes && FM_MAX_K * pl.img_dn <= pl.img_bytes, "images");
    CHECK(pl.lds_bytes == 8 * pl.ring_bytes + pl.img_bytes + FM2_MAX_SEG * FM_GG2_SEG_BYTES + FM2_PART_BYTES &&
              pl.lds_bytes <= 160 * 1024, "LDS %u", pl.lds_bytes);
    {   // the image writes of the down phase: thread t, item t + 512 i
        const int nreg = down_q6 ? 32 : 64, per = pl.lpr_dn * nreg, ne = 4 * pl.lpr_dn, grp = down_q6 ? 8 : 16;
        CHECK(FM_MAX_K * per % 512 == 0 && per % 64 == 0, "whole waves per image");
        std::vector<uint8_t> cols((size_t)inter, 0);
        for (int it = 0; it < per; it++) {
            const int ch = it / nreg, r = it % nreg, lo = 32 * (r >> 4) + 4 * ((r & 15) >> 1) + (r & 1);
            for (int d = 0; d < 3; d += 2) {
                const int v = lo + d;
                const int col = down_q6 ? 128 * (ch >> 1) + 32 * (ch & 1) + (v < 32 ? v : v + 32) : 128 * ch + v;
                CHECK(col >= 0 && col < inter, "image column %d", col);
                if (col >= 0 && col < inter) cols[col]++;
            }
            const size_t dst = (size_t)((((r >> 2) * ne + 4 * ch) * 4 + (r & 3)) * 4);
            CHECK(dst + 48 + 4 <= (size_t)(nreg / 4) * ne * 16, "image register of chunk %d", ch);
            const size_t sum = (size_t)(nreg / 4) * ne * 16 + ch * 16 + (r / grp) * 4;
            CHECK(sum + 4 <= pl.img_dn, "image sums");
        }
        for (int c = 0; c < inter; c++) CHECK(cols[c] == 1, "activation column %d polled %d times", c, (int)cols[c]);
    }
    std::vector<Region> gate, up, down;
    for (int p = 0; p < n_pairs; p++) {
        gate.emplace_back("gate rows", gu_slab, 16);
        up.emplace_back("up rows", gu_slab, 16);
        down.emplace_back("down rows", dn_slab, 16);
    }
    Region act("act", (size_t)n_pairs * inter * 4, 4), out("out", (size_t)n_groups * hidden * 4, 4);
    Region X("x", (size_t)n_groups * hidden * 4), idx("idx", (size_t)n_pairs * 4);
    auto slice = [&](Region &r, size_t off, uint32_t data) {
        for (int lane = 0; lane < 64; lane++)
            for (uint32_t i = 0; i * 1024 < data; i++)
                if (i * 1024 + lane * 16 < data) {
                    CHECK(i * 1024 + lane * 16 + 16 <= data, "load %u lane %d runs over the slice", i, lane);
                    r.touch(off + (size_t)i * 1024 + (size_t)lane * 16, 16, "slice");
                }
    };
    for (int gi = 0; gi <= G; gi++) {     // the prepared divisions against plain ones
        const uint32_t ug = (uint32_t)gi;
        uint32_t dn_ref;
        if (ug >= dm.G) dn_ref = dm.rb_total;
        else if (dm.G < dm.L) dn_ref = dm.rb_total * ug / dm.G;
        else {
            const uint32_t l = ug * dm.L / dm.G;
            const uint32_t g_lo = (l * dm.G + dm.L - 1u) / dm.L, g_hi = ((l + 1u) * dm.G + dm.L - 1u) / dm.L;
            dn_ref = l * dm.dn_upp + dm.dn_upp * (ug - g_lo) / (g_hi - g_lo);
        }
        CHECK(fm2_dn_start(dm, ug) == dn_ref, "first down row block of workgroup %d", gi);
        const uint32_t t = (uint32_t)((uint64_t)dm.s_total * ug / dm.G), dd = dn_ref * dm.K * dm.dn_wt;
        uint32_t gu_ref = t > dd ? (t - dd) / dm.gu_wt : 0u;
        if (gu_ref > dm.gu_total) gu_ref = dm.gu_total;
        CHECK(fm2_gu_start(dm, ug, dn_ref) == gu_ref, "first gate/up unit of workgroup %d", gi);
    }
    int max_seq = 0;
    size_t max_bytes = 0, min_bytes = (size_t)-1;
    uint32_t gu_prev = 0;
    for (int gi = 0; gi < G; gi++) {
        const Fm2Split sp = fm2_split(dm, gi);
        CHECK(sp.gu_wg0 == gu_prev && sp.gu_wg1 >= sp.gu_wg0, "gate/up shares of workgroup %d follow on", gi);
        gu_prev = sp.gu_wg1;
        const int n_seq = sp.n_up + sp.n_dn;
        if (n_seq > max_seq) max_seq = n_seq;
        CHECK(sp.n_up <= 2, "workgroup %d: %d gate/up segments", gi, sp.n_up);
        CHECK(n_seq <= FM2_MAX_SEG && n_seq <= 64, "workgroup %d: %d segments", gi, n_seq);
        for (int v = 0; v < sp.n_up && v < 2; v++)
            X.touch((size_t)(sp.gu_s0 + v) * hidden * 4, (size_t)hidden * 4, "x of a gate/up segment");
        size_t bytes = 0;
        for (int qq = 0; qq < n_seq; qq++) {
            const Fm2Part pt = fm2_part(dm, sp, qq);
            CHECK(pt.seg < (uint32_t)n_groups, "segment %u", pt.seg);
            for (int k = 0; k < K; k++) idx.touch(((size_t)pt.seg * K + k) * 4, 4, "idx");
            if (pt.gu) {
                for (uint32_t ul = 0; ul < pt.n; ul++) {
                    uint32_t pn, rsn;
                    fm2_gu_unit(pt.first, ul, dm.by_gu_upp, &pn, &rsn);
                    CHECK(pn < (uint32_t)K && rsn < dm.gu_upp, "gate/up unit %u -> slot %u step %u", ul, pn, rsn);
                    CHECK(ul < (1u << 28), "unit number in the tag");
                    if (pn >= (uint32_t)K) continue;
                    slice(gate[pt.seg * K + pn], (size_t)rsn * pl.slot_up, pl.slot_up);
                    slice(up[pt.seg * K + pn], (size_t)rsn * pl.slot_up, pl.slot_up);
                    bytes += 2 * (size_t)pl.slot_up;
                    for (int lane = 0; lane < 64; lane++) {
                        const int j = lane & 3, ch = (lane >> 2) % pl.lpr_up, ris = 4 * (lane / (4 * pl.lpr_up)) + j;
                        CHECK(ris < pl.rps_up, "row in step %d", ris);
                        if (ch == 0)
                            act.touch((((size_t)pt.seg * dm.gu_segu + pt.first) * pl.rps_up + ris + (size_t)ul * pl.rps_up) * 4, 4, "act");
                    }
                }
            } else {
                CHECK(pt.first % K == 0 && pt.n % K == 0, "down part %u + %u not whole row blocks", pt.first, pt.n);
                const uint32_t rb_first = pt.first / K, nrb = pt.n / K;
                const float inv = 1.0f / (float)(nrb ? nrb : 1u);
                CHECK((size_t)nrb * K * pl.rps_dn * 4 <= FM2_PART_BYTES, "partial vectors of %u row blocks", nrb);
                for (uint32_t ul = 0; ul < pt.n; ul++) {
                    uint32_t pn, rsn;
                    fm2_dn_unit(rb_first, nrb, inv, ul, &pn, &rsn);
                    CHECK(pn == ul / nrb && rsn == rb_first + ul % nrb, "down unit %u -> slot %u block %u", ul, pn, rsn);
                    CHECK(pn < (uint32_t)K && rsn < dm.dn_upp, "down unit %u -> slot %u block %u", ul, pn, rsn);
                    if (pn >= (uint32_t)K) continue;
                    slice(down[pt.seg * K + pn], (size_t)rsn * pl.slot_dn, pl.slot_dn);
                    bytes += pl.slot_dn;
                    const uint32_t rbi = ul - pn * nrb;
                    for (int lane = 0; lane < 64; lane++) {
                        const int j = lane & 3, ris = 4 * (lane / (4 * pl.lpr_dn)) + j;
                        CHECK(ris < pl.rps_dn, "row in step %d", ris);
                        CHECK(4u * ((rbi * K + pn) * pl.rps_dn + ris) + 4 <= FM2_PART_BYTES, "partial slot");
                    }
                }
                Region a1("act", act.size);
                a1.touch((size_t)pt.seg * K * inter * 4, (size_t)K * inter * 4, "act of the layer");
                out.touch(((size_t)pt.seg * hidden + (size_t)rb_first * pl.rps_dn) * 4, (size_t)nrb * pl.rps_dn * 4, "out rows");
            }
        }
        if (bytes > max_bytes) max_bytes = bytes;
        if (bytes < min_bytes) min_bytes = bytes;
    }
    CHECK(gu_prev == dm.gu_total, "gate/up units handed out: %u of %u", gu_prev, dm.gu_total);
    for (int p = 0; p < n_pairs; p++) {
        gate[p].expect_once(0, gu_slab);
        up[p].expect_once(0, gu_slab);
        down[p].expect_once(0, dn_slab);
    }
    act.expect_once(0, act.size);
    out.expect_once(0, out.size);
    std::printf("ok  %-58s %d workgroups, <= %d segments, weights %u:%u, bytes per workgroup %zu..%zu\n", g_case.c_str(), G,
                max_seq, pl.gu_wt, pl.dn_wt, min_bytes, max_bytes);
}

int main() {
    // ---- the probes of bench.py --workload stream_probe (2 GiB) and of the decode profile (440 MB)
    for (int pattern = 0; pattern < 8; pattern++) {
        walk_probe((size_t)2 << 30, pattern);
        walk_probe(440401920, pattern);
        walk_probe(4096 * 3 + 100, pattern);
    }
    // ---- config 1 (bench.py --workload gdn): qkv + z in one launch, out_proj on its own
    walk_dense_batch("gdn in_proj qkv+z 4-bit", {{8192, 4}, {4096, 4}}, 2048, 1, {});
    walk_dense_batch("gdn in_proj qkv+z with riders b, a", {{8192, 4}, {4096, 4}}, 2048, 1, {32, 32});
    walk_dense_batch("gdn out_proj 2048x4096 4-bit", {{2048, 4}}, 4096, 1, {});
    walk_dense_batch("8192x4096 4-bit (two column slabs)", {{8192, 4}}, 4096, 1, {});
    walk_dense_batch("lm_head 248320x2048 8-bit", {{248320, 8}}, 2048, 1, {});
    walk_dense_batch("routing batch, mixed widths", {{256, 8}, {1, 8}, {512, 4}, {512, 4}}, 2048, 1, {});
    walk_dense_batch("3-bit 12288x2048", {{12288, 3}}, 2048, 1, {});
    walk_dense_batch("ragged 4-bit 1000x1024 x 3 positions", {{1000, 4}}, 1024, 3, {});
    walk_dense_batch("qkv+z per position, 5 positions", {{8192, 4}, {4096, 4}}, 2048, 5, {});
    // ---- config 1 against M positions (bench.py --workload gdn_prefill)
    for (int M : {16, 100, 512, 513}) {
        walk_pf_dense(8192, 2048, 4, M);
        walk_pf_dense(4096, 2048, 4, M);
        walk_pf_dense(2048, 4096, 4, M);
        walk_pf_dense(2048, 512, 4, M);
    }
    walk_pf_dense(2048, 2048, 3, 512);
    walk_pf_dense(512, 512, 3, 64);
    // ---- config 3: chunks of 32 positions and more on 256 experts (bench.py --workload prefill, the tests)
    walk_pf_rows(512, 8, 256, 3, true, 1);
    walk_pf_rows(512, 8, 256, 3, false, 2);
    walk_pf_rows(512, 8, 256, 4, true, 3);
    walk_pf_rows(2048, 8, 256, 3, true, 4);
    walk_pf_rows(32, 8, 256, 3, true, 5);
    walk_pf_rows(200, 5, 12, 4, false, 6);
    walk_pf_rows(8192, 1, 3, 3, true, 7);
    // ---- config 4's chunk variant: grouped products on a GGUF store (bench.py --workload gguf_chunk, the tests)
    walk_gq(512, 8, 256, 2048, 512, 11);
    walk_gq(64, 8, 256, 2048, 512, 12);
    walk_gq(97, 4, 12, 1024, 256, 13);
    walk_gq(36, 4, 12, 4096, 256, 14);
    walk_gq(2048, 8, 256, 2048, 512, 15);
    // ---- routed experts: the decode step (config 2, and its 4-bit form), one layer per call
    // (config 0), chunks below 32 positions (config 3 at chunk 8)
    for (int bits : {3, 4}) {
        walk_fused_rows(40, 8, 2048, 512, bits);
        walk_fused_rows(1, 8, 2048, 512, bits);
        walk_fused_rows(8, 8, 2048, 512, bits);
        walk_fused_rows(31, 8, 2048, 512, bits);
        walk_fused_rows(3, 5, 2048, 512, bits);
        walk_fused_rows(40, 8, 1024, 256, bits);
        walk_phases(40, 8, 2048, 512, bits, false);
        walk_phases(40, 8, 2048, 512, bits, true);
        walk_phases(1, 8, 2048, 512, bits, false);
        walk_phases(1, 8, 2048, 512, bits, true);
    }
    sweep_fused_rows();
    {   // the one-layer launch with the layer tail along: its three tables beside the partial vectors
        g_case = "fused rows + tail, LDS tables";
        for (int K : {1, 5, 8})
            for (int lpr_up : {4, 8, 16}) {
                const int hidden = 128 * lpr_up, inter = hidden / 4, rps_dn = FM_WAVE / (lpr_up / 4);
                const Fm2Plan plan = fm2_plan(K, K, inter, hidden, lpr_up, N_CU);
                if (!plan.ok) continue;
                const int dn_rbs = hidden / rps_dn;
                if (plan.wgs > dn_rbs) continue;                  // (the launcher refuses these)
                const int nrb = (dn_rbs + plan.wgs - 1) / plan.wgs;
                const Fm2TailLds t = fm2_tail_lds(nrb, K, rps_dn, inter, hidden);
                if (!t.ok) continue;
                CHECK(t.so >= (uint32_t)(nrb * K * rps_dn * 4), "shared results over the partial vectors");
                CHECK(t.act >= t.so + (uint32_t)(nrb * rps_dn * 4) && t.act % 16 == 0, "activations over the shared results");
                CHECK(t.red >= t.act + (uint32_t)inter * 4, "sums over the activations");
                CHECK(t.word >= t.red + (uint32_t)(hidden / rps_dn) * 4 && t.word + 4 <= FM2_PART_BYTES, "word outside the area");
                // every workgroup owns at least one row block, at most nrb
                const Fm2Dims dm = fm2_dims(K, K, plan.wgs, inter, hidden, lpr_up);
                for (int b = 0; b < plan.wgs; b++) {
                    const Fm2Split sp = fm2_split(dm, b);
                    const uint32_t n = (sp.dn_wg1 - sp.dn_wg0) / K;
                    CHECK(sp.n_dn == 1 && n >= 1 && n <= (uint32_t)nrb, "workgroup %d owns %u row blocks (at most %d)", b, n, nrb);
                    CHECK((sp.dn_wg0 / K + n) * rps_dn <= (uint32_t)hidden, "rows past the layer");
                }
            }
        std::printf("ok  %-58s\n", g_case.c_str());
    }
    walk_fused_rows(64, 8, 2048, 512, 3);
    walk_fused_rows(300, 8, 2048, 512, 3);
    // ---- config 4: GGUF step, one layer, chunk of 8 positions
    for (int groups : {40, 1, 8}) {
        walk_gguf_stream(groups, 8, 2048, 512, true);
        walk_gguf_stream(groups, 8, 2048, 512, false);
    }
    // ---- the GGUF experts as one launch: the step, one layer, the tests' shapes
    for (int groups : {40, 1, 2, 3, 8, 31, 64})
        walk_gguf_fused(groups, 8, 2048, 512, 1);
    walk_gguf_fused(3, 5, 2048, 512, 1);
    walk_gguf_fused(2, 8, 1024, 256, 1);
    walk_gguf_fused(40, 8, 1024, 256, 1);
    walk_gguf_fused(3, 8, 1024, 512, 0);
    walk_gguf_fused(1, 2, 2048, 2048, 0);
    walk_gguf_fused(1, 4, 512, 1024, 1);
    walk_gguf_fused(300, 8, 2048, 512, 1);
    // ---- one dense GGUF tensor as the streaming kernel's single "expert" (rows = hidden, columns =
    // inter in the down phase's names): the vocabulary projection at Q4_K, and smaller shapes
    walk_gguf_stream(1, 1, 248320, 2048, false, 0, "Q4_K 248320x2048");
    walk_gguf_stream(1, 1, 248320, 1024, false, 1, "Q6_K 248320x1024");
    walk_gguf_stream(1, 1, 4096, 2048, false, 0, "Q4_K 4096x2048");
    walk_gguf_stream(1, 1, 4096, 1024, false, 1, "Q6_K 4096x1024");
    walk_gguf_stream(1, 1, 1024, 2048, false, 1, "Q6_K 1024x2048 (two chunks per lane)");
    walk_gguf_stream(1, 1, 248320, 2048, false, 1, "Q6_K 248320x2048 (two chunks per lane)");
    walk_gguf_stream(2, 4, 512, 2048, false, 1, nullptr);
    if (g_fail) {
        std::fprintf(stderr, "%d checks failed\n", g_fail);
        return 1;
    }
    std::printf("all address ranges inside their buffers\n");
    return 0;
}
