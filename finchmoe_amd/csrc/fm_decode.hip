// fm_decode.hip — routed-expert decode for affine-packed experts:
//   kernel 1  gate GEMV + up GEMV + SwiGLU for every (layer, slot) pair
//   kernel 2  down GEMV per pair -> per-expert output vectors
//   kernel 3  router-weighted sum of the K vectors of a layer, in slot order
// Replaces the four dispatches per expert of gpu_encode_experts_batched
// (finchmoe/infer.m:4337-4378: dequant_matvec_3bit x3 + swiglu_fused) and the
// weighted sum of moe_combine_residual (finchmoe/shaders.metal:2213-2228).
//
// Work decomposition.  A pair p = (layer l, slot k) selects expert idx[l][k].
// A 256-thread workgroup (4 waves) takes `rows_per_item` consecutive output
// rows of one pair.  Inside a wave, LPR = in_dim/128 adjacent lanes share a
// row (each owns 128 columns, see fm_unpack.h), so one wave step covers
// 64/LPR rows, read as one contiguous run of memory:
//   gate/up (in 2048): 16 lanes x 48 B = one 768-byte row, 4 rows per step
//   down    (in 512):   4 lanes x 48 B = one 192-byte row, 16 rows per step
// The scales (and biases) of those rows are contiguous too — [rows][groups]
// 16-bit, two groups per lane = one dword per lane.
#include "fm_mfma.h"

namespace {

struct DecodeArgs {
    const uint8_t *const *layer_ptrs;   // [n_layers] device pointers to layer blobs
    FmExpertGeom g;
    int layer0;
    int layer_stride;   // 1: pair group l is layer layer0+l; 0: all groups use layer0 (positions of a chunk)
    int K;
    const float *x;          // [nl][hidden]
    const int32_t *idx;      // [nl][K]
    const float *w;          // [nl][K]
    float *act;              // [nl][K][inter]   scratch
    float *expert_out;       // [nl][K][hidden]
    float *out;              // [nl][hidden]
    int rows_per_item;
    int items_per_pair;
    int flags;
};

// ---------------------------------------------------------------- kernel 1
template <int BITS, int LPR, bool FP16>
__global__ __launch_bounds__(256) void fm_gate_up_swiglu(DecodeArgs a) {
    constexpr int RPS = FM_WAVE / LPR;   // rows per wave step
    constexpr int BPL = FmLaneBytes<BITS>::value;
    const int item = blockIdx.x;
    const int pair = item / a.items_per_pair;
    const int chunk = item - pair * a.items_per_pair;
    const int l = pair / a.K;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = lane % LPR, r = lane / LPR;
    const int rows_per_wave = a.rows_per_item >> 2;
    const int row0 = chunk * a.rows_per_item + wave * rows_per_wave;
    float *act = a.act + (size_t)pair * a.g.inter;

    const int e = a.idx[pair];
    if ((unsigned)e >= (unsigned)a.g.n_experts) {   // treated as weight 0
        for (int i = lane; i < rows_per_wave; i += FM_WAVE) act[row0 + i] = 0.0f;
        return;
    }
    const uint8_t *blob = a.layer_ptrs[a.layer0 + l * a.layer_stride] + (size_t)e * a.g.expert_size;
    const int row_bytes = a.g.hidden * BITS / 8;
    const int sb_row_bytes = (a.g.hidden / 64) * 2;

    // issue the first weight loads before the activation loads
    size_t woff = (size_t)(row0 + r) * row_bytes + (size_t)c * BPL;
    size_t soff = (size_t)(row0 + r) * sb_row_bytes + (size_t)c * 4;
    const size_t wstep = (size_t)RPS * row_bytes, sstep = (size_t)RPS * sb_row_bytes;
    FmRowSlice<BITS> gcur, ucur, gnext, unext;
    fm_load_slice<BITS>(gcur, blob + a.g.gate_w + woff, blob + a.g.gate_s + soff,
                        blob + a.g.gate_b + soff);
    fm_load_slice<BITS>(ucur, blob + a.g.up_w + woff, blob + a.g.up_s + soff,
                        blob + a.g.up_b + soff);

    float xs[FM_CPL], xsum0, xsum1;
    fm_load_x<BITS>(a.x + (size_t)l * a.g.hidden + c * FM_CPL, xs, xsum0, xsum1);

    const int steps = rows_per_wave / RPS;
    for (int it = 0; it < steps; it++) {
        if (it + 1 < steps) {
            woff += wstep;
            soff += sstep;
            fm_load_slice<BITS>(gnext, blob + a.g.gate_w + woff, blob + a.g.gate_s + soff,
                                blob + a.g.gate_b + soff);
            fm_load_slice<BITS>(unext, blob + a.g.up_w + woff, blob + a.g.up_s + soff,
                                blob + a.g.up_b + soff);
        }
        float gv = fm_group_sum<LPR>(fm_lane_dot<BITS, FP16>(gcur, xs, xsum0, xsum1));
        float uv = fm_group_sum<LPR>(fm_lane_dot<BITS, FP16>(ucur, xs, xsum0, xsum1));
        if (c == 0) act[row0 + it * RPS + r] = fm_silu_mul(gv, uv);
        gcur = gnext;
        ucur = unext;
    }
}

// ---------------------------------------------------------------- kernel 3
// out[l][j] = sum_k w[l][k] * expert_out[l][k][j], k in slot order
// (finchmoe/shaders.metal:2213-2228).  GUARD adds the CPU path's finite check
// and renormalisation (finchmoe/infer.m:10190-10204); it needs the whole
// vector of each expert, so one workgroup covers a layer.
template <bool GUARD>
__global__ __launch_bounds__(256) void fm_combine(DecodeArgs a) {
    __shared__ float red[4];
    const int l = blockIdx.x;
    const int H = a.g.hidden, K = a.K;
    const float *eo = a.expert_out + (size_t)l * K * H;
    float wk[FM_MAX_K];
    float total = 0.0f;
#pragma unroll
    for (int k = 0; k < FM_MAX_K; k++) {
        float w = 0.0f;
        if (k < K) {
            w = a.w[l * K + k];
            if ((unsigned)a.idx[l * K + k] >= (unsigned)a.g.n_experts) w = 0.0f;
            if constexpr (GUARD) {
                float part = 0.0f;
                for (int j = threadIdx.x; j < H; j += blockDim.x) {
                    float v = eo[(size_t)k * H + j];
                    part = fmaf(v, v, part);
                }
                part = fm_group_sum<64>(part);
                __syncthreads();
                if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = part;
                __syncthreads();
                float er = red[0] + red[1] + red[2] + red[3];
                bool keep = isfinite(er) && er < 1e20f;
                if (keep) total += w; else w = 0.0f;
            }
        }
        wk[k] = w;
    }
    float rn = 1.0f;
    if constexpr (GUARD) {
        if (total > 0.0f && total < 0.99f) rn = 1.0f / total;
    }
    float *out = a.out + (size_t)l * H;
    const int j0 = GUARD ? 0 : blockIdx.y * blockDim.x;
    const int j1 = GUARD ? H : min(H, j0 + (int)blockDim.x);
    for (int j = j0 + threadIdx.x; j < j1; j += blockDim.x) {
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < FM_MAX_K; k++)
            if (k < K && wk[k] != 0.0f) acc += wk[k] * eo[(size_t)k * H + j];
        if constexpr (GUARD) acc *= rn;
        out[j] = (a.flags & FM_ACCUMULATE) ? out[j] + acc : acc;
    }
}

// ---------------------------------------------------------------- kernel 2
template <int BITS, int LPR, bool FP16>
__global__ __launch_bounds__(256) void fm_down(DecodeArgs a) {
    constexpr int RPS = FM_WAVE / LPR;
    constexpr int BPL = FmLaneBytes<BITS>::value;
    const int item = blockIdx.x;
    const int pair = item / a.items_per_pair;
    const int chunk = item - pair * a.items_per_pair;
    const int l = pair / a.K;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = lane % LPR, r = lane / LPR;
    const int rows_per_wave = a.rows_per_item >> 2;
    const int row0 = chunk * a.rows_per_item + wave * rows_per_wave;
    float *eo = a.expert_out + (size_t)pair * a.g.hidden;

    const int e = a.idx[pair];
    if ((unsigned)e >= (unsigned)a.g.n_experts) {
        for (int i = lane; i < rows_per_wave; i += FM_WAVE) eo[row0 + i] = 0.0f;
    } else {
        const uint8_t *blob = a.layer_ptrs[a.layer0 + l * a.layer_stride] + (size_t)e * a.g.expert_size;
        const int row_bytes = a.g.inter * BITS / 8;
        const int sb_row_bytes = (a.g.inter / 64) * 2;
        size_t woff = (size_t)(row0 + r) * row_bytes + (size_t)c * BPL;
        size_t soff = (size_t)(row0 + r) * sb_row_bytes + (size_t)c * 4;
        const size_t wstep = (size_t)RPS * row_bytes, sstep = (size_t)RPS * sb_row_bytes;
        FmRowSlice<BITS> cur, next;
        fm_load_slice<BITS>(cur, blob + a.g.down_w + woff, blob + a.g.down_s + soff,
                            blob + a.g.down_b + soff);
        float xs[FM_CPL], xsum0, xsum1;
        fm_load_x<BITS>(a.act + (size_t)pair * a.g.inter + c * FM_CPL, xs, xsum0, xsum1);
        const int steps = rows_per_wave / RPS;
        for (int it = 0; it < steps; it++) {
            if (it + 1 < steps) {
                woff += wstep;
                soff += sstep;
                fm_load_slice<BITS>(next, blob + a.g.down_w + woff, blob + a.g.down_s + soff,
                                    blob + a.g.down_b + soff);
            }
            float v = fm_group_sum<LPR>(fm_lane_dot<BITS, FP16>(cur, xs, xsum0, xsum1));
            if (c == 0) eo[row0 + it * RPS + r] = v;
            cur = next;
        }
    }

}

// ======================================================================
// Matrix-core path (fm_mfma.h): persistent workgroups over a static partition.
//
// All row steps of all pairs form one sequence of "units" (a unit = one wave
// step = 64/LPR rows of one pair).  The launch has a fixed number of
// workgroups; workgroup g takes the contiguous unit range [U*g/G, U*(g+1)/G),
// its four waves interleave over it, each with the next unit's loads in
// flight — so a wave streams tens of kilobytes back to back instead of a few
// rows, and every wave ends after its own share (no queue, no spinning).
// A range is cut into segments that share an input vector (a layer for
// gate/up, a pair for down); per segment the workgroup builds the activation
// registers once in LDS (fm_build_act_lds) and every wave copies its own.
// ======================================================================
template <int BITS, int LPR>
__device__ __forceinline__ void fm_unit_lane_offsets(int lane, int row_bytes, int sb_row_bytes,
                                                     size_t &woff, size_t &soff, int &row_in_step,
                                                     int &ch) {
    const int j = lane & 3;
    ch = (lane >> 2) % LPR;
    const int rq = lane / (4 * LPR);
    row_in_step = 4 * rq + j;
    woff = (size_t)row_in_step * row_bytes + (size_t)ch * FmLaneBytes<BITS>::value;
    soff = (size_t)row_in_step * sb_row_bytes + (size_t)ch * 4;
}

__device__ __forceinline__ const uint8_t *fm_pair_blob(const DecodeArgs &a, int p) {
    int e = a.idx[p];
    if ((unsigned)e >= (unsigned)a.g.n_experts) return nullptr;   // treated as weight 0
    return a.layer_ptrs[a.layer0 + (p / a.K) * a.layer_stride] + (size_t)e * a.g.expert_size;
}

// A pointer every lane of the wave agrees on, moved to scalar registers so the
// loads can use the scalar-base + 32-bit lane offset addressing form.
__device__ __forceinline__ const uint8_t *fm_uniform(const uint8_t *p) {
    uintptr_t v = (uintptr_t)p;
    uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const uint8_t *)(((uintptr_t)hi << 32) | lo);
}

// gate + up + SwiGLU.  a.items_per_pair carries the number of pairs.
//
// Pipeline: the wave walks "half steps" — gate rows of a unit, then up rows of
// the same unit — through a ring of three register slices: while slice k is
// being multiplied, the loads of the next two half steps are in flight (a full
// unit, ~6.6 KB per wave).  The loop is unrolled by three units so the ring
// rotates without register copies.
template <int BITS, int LPR, bool FP16>
__global__ __launch_bounds__(256)
void fm_gate_up_swiglu_mfma(DecodeArgs a) {
    constexpr int RPS = FM_WAVE / LPR;
    __shared__ FmActLds<LPR> lds;
    __shared__ const uint8_t *lds_blob[FM_MAX_K];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_pairs = a.items_per_pair;
    const int upp = a.g.inter / RPS;        // units per pair (>= 4)
    const long upl = (long)upp * a.K;       // units per layer
    const long total = (long)n_pairs * upp;
    const long wg0 = total * blockIdx.x / gridDim.x, wg1 = total * (blockIdx.x + 1) / gridDim.x;
    const int row_bytes = a.g.hidden * BITS / 8, sb_row_bytes = (a.g.hidden / 64) * 2;
    size_t woff_, soff_;
    int ris, ch;
    fm_unit_lane_offsets<BITS, LPR>(lane, row_bytes, sb_row_bytes, woff_, soff_, ris, ch);
    const uint32_t woff = (uint32_t)woff_, soff = (uint32_t)soff_;
    const uint32_t wstep = (uint32_t)(RPS * row_bytes), sstep = (uint32_t)(RPS * sb_row_bytes);
    FmBuildSlot<BITS> bslot;
    bslot.init();

    for (long seg0 = wg0; seg0 < wg1;) {
        const int l = (int)(seg0 / upl);
        long seg1 = (long)(l + 1) * upl;
        if (seg1 > wg1) seg1 = wg1;
        __syncthreads();                          // previous segment's readers are done
        if (threadIdx.x < a.K) lds_blob[threadIdx.x] = fm_pair_blob(a, l * a.K + threadIdx.x);
        __syncthreads();
        // loader: half step (pair pn, row step rsn, matrix hn) of this wave
        long u = seg0 + wave;          // unit being computed
        long un = u;                   // unit being loaded
        int pn = (int)(u / upp) - l * a.K, rsn = (int)(u % upp), hn = 0;
        const uint8_t *blob_n = un < seg1 ? fm_uniform(lds_blob[pn]) : nullptr;
        const uint8_t *blob_c = blob_n;            // blob of the unit being computed
        const uint8_t *blob_q[2] = {blob_n, blob_n};   // blobs of the units in flight
        auto load_half = [&](FmRowSlice<BITS> &t) {
            if (un < seg1) {
                if (blob_n) {
                    const uint8_t *b = blob_n + (size_t)rsn * wstep;
                    const uint8_t *sb = blob_n + (size_t)rsn * sstep;
                    if (hn == 0)
                        fm_load_slice<BITS>(t, b + a.g.gate_w + woff, sb + a.g.gate_s + soff,
                                            sb + a.g.gate_b + soff);
                    else
                        fm_load_slice<BITS>(t, b + a.g.up_w + woff, sb + a.g.up_s + soff,
                                            sb + a.g.up_b + soff);
                }
                if (hn == 1) {
                    un += 4;
                    rsn += 4;
                    if (rsn >= upp) {
                        rsn -= upp;
                        pn++;
                        if (un < seg1) blob_n = fm_uniform(lds_blob[pn]);
                    }
                }
                hn ^= 1;
            }
        };
        FmRowSlice<BITS> r0, r1, r2;
        load_half(r0);                            // one unit in flight during the build
        load_half(r1);
        blob_q[0] = blob_n;                       // blob of unit u+4 (after the two loads)
        fm_build_act_lds<BITS, LPR>(a.x + (size_t)l * a.g.hidden, bslot, lds);
        __syncthreads();
        FmActRegs ar;
        fm_read_act_lds<LPR>(lds, lane, ar);
        float gv = 0.0f;
        // one half step: start the load two half steps ahead, multiply the current slice
        auto gate_step = [&](FmRowSlice<BITS> &cur, FmRowSlice<BITS> &tgt) {
            load_half(tgt);
            if (blob_c) gv = fm_chunk_sum<LPR>(fm_lane_dot_mfma<BITS, FP16>(cur, ar));
        };
        auto up_step = [&](FmRowSlice<BITS> &cur, FmRowSlice<BITS> &tgt) {
            // the load issued here is the up half of unit u+4... its blob is blob_q[0]
            load_half(tgt);
            float v = 0.0f;
            if (blob_c) {
                float uv = fm_chunk_sum<LPR>(fm_lane_dot_mfma<BITS, FP16>(cur, ar));
                v = fm_silu_mul(gv, uv);
            }
            // unit u = (pair, row step): act is [pair][inter], rows are contiguous
            if (ch == 0) a.act[(size_t)u * RPS + ris] = v;
            u += 4;
            blob_c = blob_q[0];
            blob_q[0] = blob_n;
        };
        while (u < seg1) {
            gate_step(r0, r2);
            up_step(r1, r0);
            if (u >= seg1) break;
            gate_step(r2, r1);
            up_step(r0, r2);
            if (u >= seg1) break;
            gate_step(r1, r0);
            up_step(r2, r1);
        }
        seg0 = seg1;
    }
}

// down projection -> per-expert output vectors.  Ring of three slices: two units
// of loads in flight ahead of the one being multiplied.
template <int BITS, int LPR, bool FP16>
__global__ __launch_bounds__(256)
void fm_down_mfma(DecodeArgs a) {
    constexpr int RPS = FM_WAVE / LPR;
    __shared__ FmActLds<LPR> lds;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_pairs = a.items_per_pair;
    const int upp = a.g.hidden / RPS;
    const long total = (long)n_pairs * upp;
    const long wg0 = total * blockIdx.x / gridDim.x, wg1 = total * (blockIdx.x + 1) / gridDim.x;
    const int row_bytes = a.g.inter * BITS / 8, sb_row_bytes = (a.g.inter / 64) * 2;
    size_t woff_, soff_;
    int ris, ch;
    fm_unit_lane_offsets<BITS, LPR>(lane, row_bytes, sb_row_bytes, woff_, soff_, ris, ch);
    const uint32_t woff = (uint32_t)woff_, soff = (uint32_t)soff_;
    const uint32_t wstep = (uint32_t)(RPS * row_bytes), sstep = (uint32_t)(RPS * sb_row_bytes);
    FmBuildSlot<BITS> bslot;
    bslot.init();

    for (long seg0 = wg0; seg0 < wg1;) {
        const int p = (int)(seg0 / upp);
        long seg1 = (long)(p + 1) * upp;
        if (seg1 > wg1) seg1 = wg1;
        const uint8_t *blob = fm_pair_blob(a, p);
        long u = seg0 + wave;
        int rsn = (int)(u - (long)p * upp);
        long un = u;
        auto load_next = [&](FmRowSlice<BITS> &ds) {
            if (un < seg1) {
                const uint8_t *b = blob + (size_t)rsn * wstep;
                const uint8_t *sb = blob + (size_t)rsn * sstep;
                fm_load_slice<BITS>(ds, b + a.g.down_w + woff, sb + a.g.down_s + soff,
                                    sb + a.g.down_b + soff);
                un += 4;
                rsn += 4;
            }
        };
        __syncthreads();
        if (blob) {
            FmRowSlice<BITS> r0, r1, r2;
            load_next(r0);
            load_next(r1);
            fm_build_act_lds<BITS, LPR>(a.act + (size_t)p * a.g.inter, bslot, lds);
            __syncthreads();
            FmActRegs ar;
            fm_read_act_lds<LPR>(lds, lane, ar);
            auto step = [&](FmRowSlice<BITS> &cur, FmRowSlice<BITS> &tgt) {
                load_next(tgt);
                float v = fm_chunk_sum<LPR>(fm_lane_dot_mfma<BITS, FP16>(cur, ar));
                if (ch == 0) a.expert_out[(size_t)u * RPS + ris] = v;
                u += 4;
            };
            while (u < seg1) {
                step(r0, r2);
                if (u >= seg1) break;
                step(r1, r0);
                if (u >= seg1) break;
                step(r2, r1);
            }
        } else {
            for (; u < seg1; u += 4)
                if (ch == 0) a.expert_out[(size_t)u * RPS + ris] = 0.0f;
        }
        seg0 = seg1;
    }
}

template <int BITS, bool FP16>
int launch_decode_t(const DecodeArgs &a, int n_pairs, int rpi_up, int rpi_down, int n_cu,
                    hipStream_t st, hipEvent_t *kev) {
    DecodeArgs a1 = a, a2 = a;
    a1.rows_per_item = rpi_up;
    a1.items_per_pair = a.g.inter / rpi_up;
    a2.rows_per_item = rpi_down;
    a2.items_per_pair = a.g.hidden / rpi_down;
    dim3 b(256);
    const int lpr_up = a.g.hidden / FM_CPL, lpr_down = a.g.inter / FM_CPL;
    // matrix-core path: one wave per SIMD slot that the register budget allows,
    // fewer when there are not enough units to give every wave two
    const bool mfma_up = lpr_up >= 4 && lpr_up <= 16, mfma_down = lpr_down <= 16;
    // two workgroups per CU (register budget); fewer when the launch has too few
    // units to give every wave two
    auto stream_grid = [&](long units) {
        long wgs = (long)n_cu * 2;
        if (units < 8 * wgs) wgs = (units + 7) / 8;
        if (wgs < 1) wgs = 1;
        return dim3((unsigned)wgs);
    };
    if (kev) (void)hipEventRecord(kev[0], st);
    if (mfma_up) {
        DecodeArgs am = a;
        am.items_per_pair = n_pairs;
        dim3 g = stream_grid((long)n_pairs * (a.g.inter / (FM_WAVE / lpr_up)));
#define FM_UPM(L) hipLaunchKernelGGL((fm_gate_up_swiglu_mfma<BITS, L, FP16>), g, b, 0, st, am)
        switch (lpr_up) {
            case 4: FM_UPM(4); break;
            case 8: FM_UPM(8); break;
            default: FM_UPM(16); break;
        }
#undef FM_UPM
    } else {
#define FM_UP(L) \
    hipLaunchKernelGGL((fm_gate_up_swiglu<BITS, L, FP16>), dim3(n_pairs * a1.items_per_pair), b, 0, st, a1)
        switch (lpr_up) {
            case 32: FM_UP(32); break;
            default: return FM_ERR_UNSUPPORTED;
        }
#undef FM_UP
    }
    if (kev) (void)hipEventRecord(kev[1], st);
    if (mfma_down) {
        DecodeArgs am = a;
        am.items_per_pair = n_pairs;
        dim3 g = stream_grid((long)n_pairs * (a.g.hidden / (FM_WAVE / lpr_down)));
#define FM_DOWNM(L) hipLaunchKernelGGL((fm_down_mfma<BITS, L, FP16>), g, b, 0, st, am)
        switch (lpr_down) {
            case 1: FM_DOWNM(1); break;
            case 2: FM_DOWNM(2); break;
            case 4: FM_DOWNM(4); break;
            case 8: FM_DOWNM(8); break;
            default: FM_DOWNM(16); break;
        }
#undef FM_DOWNM
    } else {
        return FM_ERR_UNSUPPORTED;
    }
    (void)a2;
    const int n_groups = n_pairs / a.K;
    if (a.flags & FM_GUARD)
        hipLaunchKernelGGL(fm_combine<true>, dim3(n_groups), b, 0, st, a);
    else
        hipLaunchKernelGGL(fm_combine<false>, dim3(n_groups, (a.g.hidden + 255) / 256), b, 0, st, a);
    if (kev) (void)hipEventRecord(kev[2], st);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

// rows per workgroup: min_rows * 2^j dividing `rows`, as large as possible (at
// most `cap`) while the launch still has at least `want` workgroups
int pick_rows_per_item(int rows, int n_pairs, int min_rows, int cap, int want) {
    int rpi = min_rows;
    while (rpi * 2 <= cap && rows % (rpi * 2) == 0 && (rows / (rpi * 2)) * n_pairs >= want)
        rpi *= 2;
    return rpi;
}

}  // namespace

// Enqueue both kernels for n_layers x K pairs (n_layers groups of K slots: the
// layers of a decode step, or with layer_stride 0 the positions of a chunk).  Shapes are validated by the
// caller (fm_api.cpp): hidden, inter multiples of 128 with a supported
// lanes-per-row, every layer resident.
extern "C" int fm_launch_decode_affine(const uint8_t *const *d_layer_ptrs,
                                       const FmExpertGeom *g, int layer0, int layer_stride,
                                       int n_layers, const float *d_x, const int32_t *d_idx,
                                       const float *d_w, int K, float *d_act,
                                       float *d_expert_out, float *d_out,
                                       unsigned int *d_counters, int flags, int n_cu,
                                       hipStream_t st, hipEvent_t *kev) {
    DecodeArgs a;
    a.layer_ptrs = d_layer_ptrs;
    a.g = *g;
    a.layer0 = layer0;
    a.layer_stride = layer_stride;
    a.K = K;
    a.x = d_x;
    a.idx = d_idx;
    a.w = d_w;
    a.act = d_act;
    a.expert_out = d_expert_out;
    a.out = d_out;
    (void)d_counters;
    a.flags = flags;
    a.rows_per_item = a.items_per_pair = 0;
    const int n_pairs = n_layers * K;
    const int lpr_up = g->hidden / FM_CPL, lpr_down = g->inter / FM_CPL;
    if (lpr_up < 1 || lpr_down < 1) return FM_ERR_UNSUPPORTED;
    // a wave step covers 64/LPR rows and a workgroup has 4 waves
    const int min_up = 4 * (FM_WAVE / lpr_up), min_down = 4 * (FM_WAVE / lpr_down);
    if (g->inter % min_up || g->hidden % min_down) return FM_ERR_UNSUPPORTED;
    const int want = 4 * n_cu;
    const int rpi_up = pick_rows_per_item(g->inter, n_pairs, min_up, 64, want);
    const int rpi_down = pick_rows_per_item(g->hidden, n_pairs, min_down, 256, want);
    if (g->bits == 3) {
        return g->scale_fp16 ? launch_decode_t<3, true>(a, n_pairs, rpi_up, rpi_down, n_cu, st, kev)
                             : launch_decode_t<3, false>(a, n_pairs, rpi_up, rpi_down, n_cu, st, kev);
    }
    if (g->bits == 4) {
        return g->scale_fp16 ? launch_decode_t<4, true>(a, n_pairs, rpi_up, rpi_down, n_cu, st, kev)
                             : launch_decode_t<4, false>(a, n_pairs, rpi_up, rpi_down, n_cu, st, kev);
    }
    return FM_ERR_UNSUPPORTED;
}
