// fm_dense.hip — dense affine-quantized GEMV: n tensors sharing one input
// vector, optionally over M positions.  Replaces dequant_matvec_4bit_v3 /
// _8bit / _3bit driven through BatchMatvecSpec (finchmoe/infer.m:3401-3411,
// 3528-3652; finchmoe/shaders.metal:374-463) and the M-position clone
// dequant_matvec_4bit_prefill (shaders.metal:2460-2529), whose grid is
// position x row tile exactly as here.
//
// Same lane mapping as the expert kernels: a lane owns 128 columns, LPR =
// in_dim/128 lanes share a row, a wave step covers 64/LPR rows that are
// contiguous in memory.
#include "fm_unpack.h"

#define FM_MAX_BATCH 8

struct FmDenseSpec {
    const uint8_t *W, *S, *B;
    float *out;
    int out_dim;
    int first_item;   // first workgroup of this tensor
};

struct FmDenseArgs {
    FmDenseSpec spec[FM_MAX_BATCH];
    int n;
    int in_dim;
    int rows_per_item;
    const float *x;      // [M][in_dim]
    size_t out_stride;   // elements between positions in every out (= out_dim of that tensor if 0)
};

namespace {

template <int BITS, int LPR, bool FP16>
__global__ __launch_bounds__(256) void fm_dense_gemv(FmDenseArgs a) {
    constexpr int RPS = FM_WAVE / LPR;
    constexpr int BPL = FmLaneBytes<BITS>::value;
    int t = 0;
#pragma unroll
    for (int i = 1; i < FM_MAX_BATCH; i++)
        if (i < a.n && (int)blockIdx.x >= a.spec[i].first_item) t = i;
    const FmDenseSpec sp = a.spec[t];
    const int chunk = blockIdx.x - sp.first_item;
    const int m = blockIdx.y;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = lane % LPR, r = lane / LPR;
    const int rows_per_wave = a.rows_per_item >> 2;
    const int row0 = chunk * a.rows_per_item + wave * rows_per_wave;
    if (row0 >= sp.out_dim) return;
    int steps = rows_per_wave / RPS;
    {   // the last workgroup of a tensor may be short
        int left = (sp.out_dim - row0 + RPS - 1) / RPS;
        if (left < steps) steps = left;
    }
    const int row_bytes = a.in_dim * BITS / 8;
    const int sb_row_bytes = (a.in_dim / 64) * 2;
    const int last_row = sp.out_dim - 1;
    // rows past the end (only when out_dim is not a multiple of 64/LPR) re-read
    // the last row and are not stored
    auto rowc = [&](int row) { return row < last_row ? row : last_row; };
    int row = row0 + r;
    FmRowSlice<BITS> cur, next;
    {
        size_t ro = (size_t)rowc(row);
        fm_load_slice<BITS>(cur, sp.W + ro * row_bytes + (size_t)c * BPL,
                            sp.S + ro * sb_row_bytes + (size_t)c * 4,
                            sp.B + ro * sb_row_bytes + (size_t)c * 4);
    }
    float xs[FM_CPL], xsum0, xsum1;
    fm_load_x<BITS>(a.x + (size_t)m * a.in_dim + c * FM_CPL, xs, xsum0, xsum1);
    float *out = sp.out + (size_t)m * sp.out_dim;
    for (int it = 0; it < steps; it++) {
        if (it + 1 < steps) {
            size_t ro = (size_t)rowc(row + RPS);
            fm_load_slice<BITS>(next, sp.W + ro * row_bytes + (size_t)c * BPL,
                                sp.S + ro * sb_row_bytes + (size_t)c * 4,
                                sp.B + ro * sb_row_bytes + (size_t)c * 4);
        }
        float v = fm_group_sum<LPR>(fm_lane_dot<BITS, FP16>(cur, xs, xsum0, xsum1));
        if (c == 0 && row <= last_row) out[row] = v;
        row += RPS;
        cur = next;
    }
}

template <int BITS, bool FP16>
int launch_dense_t(const FmDenseArgs &a, int total_items, int M, hipStream_t st) {
    dim3 grid(total_items, M), b(256);
#define FM_D(L) hipLaunchKernelGGL((fm_dense_gemv<BITS, L, FP16>), grid, b, 0, st, a)
    switch (a.in_dim / FM_CPL) {
        case 1: FM_D(1); break;
        case 2: FM_D(2); break;
        case 4: FM_D(4); break;
        case 8: FM_D(8); break;
        case 16: FM_D(16); break;
        case 32: FM_D(32); break;
        case 64: FM_D(64); break;
        default: return FM_ERR_UNSUPPORTED;
    }
#undef FM_D
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

}  // namespace

// specs[i].first_item is filled here.  in_dim must be 128 * 2^j, j <= 6.
extern "C" int fm_launch_dense(FmDenseSpec *specs, int n, int in_dim, int bits, int scale_fp16,
                               const float *d_x, int M, int n_cu, hipStream_t st) {
    if (n < 1 || n > FM_MAX_BATCH || M < 1) return FM_ERR_ARG;
    const int lpr = in_dim / FM_CPL;
    if (lpr < 1 || lpr > 64 || (lpr & (lpr - 1)) || in_dim % FM_CPL) return FM_ERR_UNSUPPORTED;
    const int min_rows = 4 * (FM_WAVE / lpr);
    long total_rows = 0;
    for (int i = 0; i < n; i++) total_rows += specs[i].out_dim;
    // Rows per workgroup: the register budget keeps two workgroups per CU resident, and a
    // launch that needs a second round of workgroups pays its start-up latencies twice —
    // so grow the tile until the launch fits in one round (or the tile is 8 steps deep).
    int rpi = min_rows;
    while (rpi * 2 <= 8 * min_rows && (total_rows * M + rpi - 1) / rpi > 2L * n_cu) rpi *= 2;
    FmDenseArgs a;
    a.n = n;
    a.in_dim = in_dim;
    a.rows_per_item = rpi;
    a.x = d_x;
    a.out_stride = 0;
    int items = 0;
    for (int i = 0; i < n; i++) {
        specs[i].first_item = items;
        items += (specs[i].out_dim + rpi - 1) / rpi;
        a.spec[i] = specs[i];
    }
    for (int i = n; i < FM_MAX_BATCH; i++) a.spec[i] = a.spec[0];
    switch (bits) {
        case 3: return scale_fp16 ? launch_dense_t<3, true>(a, items, M, st)
                                  : launch_dense_t<3, false>(a, items, M, st);
        case 4: return scale_fp16 ? launch_dense_t<4, true>(a, items, M, st)
                                  : launch_dense_t<4, false>(a, items, M, st);
        case 8: return scale_fp16 ? launch_dense_t<8, true>(a, items, M, st)
                                  : launch_dense_t<8, false>(a, items, M, st);
        default: return FM_ERR_UNSUPPORTED;
    }
}
