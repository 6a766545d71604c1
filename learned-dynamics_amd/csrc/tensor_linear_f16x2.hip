// fp32-class GEMM on the fp16 matrix cores with two-piece operand splitting ("f16x2").
//
// Every fp32 operand is scaled by a per-row power of two (exact) and split into two fp16
// pieces, v = hi + lo with hi = RNE16(v) and lo = RNE16(v - hi): 11 + 11 significand bits, so
// |v - hi - lo| <= 2^-22 |v|.  A product is assembled from three piece products
//     a*b ~= a_lo*b_hi + a_hi*b_lo + a_hi*b_hi            (dropped: a_lo*b_lo <= 2^-22 |a||b|)
// accumulated in fp32 by v_mfma_f32_32x32x16_f16: half the matrix work of a three-piece bf16
// split, at an error of a few fp32 ulps per product (the rounding of an fp32 dot product of
// length K is of the same size).  The power-of-two scales put the largest element of an x row
// (a W row) into [2^14, 2^15), which removes fp16's narrow exponent range from the picture:
// an element e of a row with scaled maximum M carries an error of max(2^-22 |e|, 2^-25), i.e.
// the result is normwise as accurate as the fp32 dot product whenever M >= 1, and the scales
// are undone exactly in the epilogue.  The row maxima of x come from the kernel that produced
// x (this kernel's own epilogue can emit them for its output) or from row_absmax_kernel.
//
// Kernel shape (row streaming): a workgroup of WAVES waves owns a tile of 32 WAVES rows x 32 NI
// columns; wave w owns rows [32 w, 32 w + 32) of the tile and ALL its columns.
//   * x never touches LDS: a lane loads the 16 consecutive floats of ITS row that it will feed to
//     the matrix core (lane = row + 32 g holds k = 32 c + 16 g .. + 16 of chunk c: 64 contiguous
//     bytes, four 16-byte loads), two chunks ahead, and splits them in registers.  Every row is
//     loaded and split exactly once per tile, nothing about x is tied to a barrier, and the LDS
//     carries only W.
//   * W planes (already fp16) go global -> registers -> LDS, double buffered, K chunk 32 (rows of
//     64 B padded to 80 B: conflict free for 16-byte reads), one barrier per chunk.
//   * the k order inside a chunk is a permutation (MFMA step s takes k = 16 g + 8 s .. + 8 from
//     lane group g); W is read from LDS with the same permutation, so the products pair up.
//   * loads are never predicated (rows past the end are clamped to the last row, whose
//     accumulators are simply not written): a loop body without branches lets every load stay in
//     flight until the chunk that needs it.  W (L2 resident, needed one chunk later) is requested
//     before x (HBM, needed two chunks later), because loads return in order.
//   * the epilogue runs once per tile with nothing to overlap it, so its instruction count is
//     what matters: one row pointer, row scale and bounds check per accumulator row, column
//     offsets as immediates, activation and accumulate chosen at compile time.
// v_mfma_f32_32x32x16_f16 layout: A[m][k]: lane = m + 32*(k/8), 8 consecutive k per lane;
// B[k][n] likewise; D[m][n]: n = lane%32, m = 8*(q/4) + 4*(lane/32) + q%4 for register q.
#include "common.hpp"
#include "f16x2.hpp"
#include <type_traits>

namespace mg {
namespace {

__device__ __forceinline__ float activate(float v, int act) {
    if (act == 1) return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    if (act == 2) return v > 0.f ? v : 0.1f * v;
    return v;
}

template <int ACT>
__device__ __forceinline__ float activate_c(float v) {
    // SiLU through the hardware exp2 and reciprocal (about 1 ulp each): far inside the fp32 tolerance
    if constexpr (ACT == 1) return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    if constexpr (ACT == 2) return v > 0.f ? v : 0.1f * v;
    return v;
}

// one wave per output row: row maximum -> scale -> hi / lo planes (O_pad rows, zero filled) + 1/scale per row
__global__ void __launch_bounds__(256) pack_weight_f16x2_kernel(const float* __restrict__ W, long so, long si, int I,
                                                                int O, int O_pad, _Float16* __restrict__ planes,
                                                                float* __restrict__ inv_scale) {
    const int lane = threadIdx.x & 63;
    const long total = (long)O_pad * I;
    for (long o = ((long)blockIdx.x * blockDim.x + threadIdx.x) >> 6; o < O_pad; o += ((long)gridDim.x * blockDim.x) >> 6) {
        float amax = 0.f;
        if (o < O)
            for (int i = lane; i < I; i += 64) amax = fmaxf(amax, fabsf(W[o * so + (long)i * si]));
        for (int d = 1; d < 64; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
        float inv;
        const float s = pow2_scale(amax, &inv);
        for (int i = lane; i < I; i += 64) {
            const float v = o < O ? W[o * so + (long)i * si] * s : 0.f;
            const _Float16 h = (_Float16)v;
            planes[o * I + i] = h;
            planes[total + o * I + i] = (_Float16)(v - (float)h);
        }
        if (lane == 0) inv_scale[o] = inv;
    }
}

// out[r] = max_i |x[r, i]|; a wave per row, 16-byte loads when the row length allows
__global__ void __launch_bounds__(256) row_absmax_kernel(const float* __restrict__ x, long R, int I,
                                                         float* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    const long wave = ((long)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const long n_waves = ((long)gridDim.x * blockDim.x) >> 6;
    for (long r = wave; r < R; r += n_waves) {
        const float* row = x + r * I;
        float m = 0.f;
        if ((I & 3) == 0) {
            for (int i = lane * 4; i < I; i += 256) {
                const float4 v = *reinterpret_cast<const float4*>(row + i);
                m = fmaxf(fmaxf(m, fmaxf(fabsf(v.x), fabsf(v.y))), fmaxf(fabsf(v.z), fabsf(v.w)));
            }
        } else {
            for (int i = lane; i < I; i += 64) m = fmaxf(m, fabsf(row[i]));
        }
        for (int d = 1; d < 64; d <<= 1) m = fmaxf(m, __shfl_xor(m, d));
        if (lane == 0) out[r] = m;
    }
}


// x (rows, K, T) in the reference's tensor layout (channel, then components) -> xt (rows * T, K_pad): one plain
// GEMM row per (row, component), channels zero-padded to K_pad, and the maximum of |xt| per output row.
// A thread writes four consecutive channels of one output row; the K_pad / 4 threads of a row are neighbours.
__global__ void __launch_bounds__(256) components_to_rows_kernel(const float* __restrict__ x, long rows, int K, int T,
                                                                 int K_pad, float* __restrict__ xt,
                                                                 float* __restrict__ rowmax) {
    const int per_row = K_pad / 4;                            // 8, 16, ...: a power of two <= 64
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long out_row = idx / per_row;
    const int k0 = (int)(idx - out_row * per_row) * 4;
    const bool live = out_row < rows * T;
    const long r = live ? out_row / T : 0;
    const int t = live ? (int)(out_row - r * T) : 0;
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) v[j] = (live && k0 + j < K) ? x[(r * K + k0 + j) * T + t] : 0.f;
    if (live) *reinterpret_cast<float4*>(xt + out_row * K_pad + k0) = make_float4(v[0], v[1], v[2], v[3]);
    float mx = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    for (int d = 1; d < per_row; d <<= 1) mx = fmaxf(mx, __shfl_xor(mx, d));
    if (live && k0 == 0) rowmax[out_row] = mx;
}

template <int WAVES, int NI>
__global__ void __launch_bounds__(64 * WAVES)
linear_rows_f16x2_kernel(const _Float16* __restrict__ Wp, const float* __restrict__ w_inv, const float* __restrict__ X,
                         const float* __restrict__ xmax, int xmax_parts, long xmax_stride, long xmax_div, long R, int I,
                         int O, int O_pad, const float* __restrict__ bias, int act, int accumulate,
                         float* __restrict__ Y, float* __restrict__ ymax, int tiles_n, long tiles_total, int out_T,
                         float bound_mul, float bound_add) {
    constexpr int TM = 32 * WAVES, TN = 32 * NI, THREADS = 64 * WAVES;
    constexpr int kPlaneW = TN * kRowW, kBufW = 2 * kPlaneW;
    constexpr int kPieces = 8 * TN;                          // 16-byte pieces of W per chunk (2 planes x TN rows x 4)
    constexpr int kPer = (kPieces + THREADS - 1) / THREADS;  // per thread
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kBufW];
    __shared__ float inv_sx[TM];

    const long bid = blockIdx.x;
    const long per_xcd = (tiles_total + 7) / 8;
    const long logical = (bid % 8) * per_xcd + bid / 8;
    if (logical >= tiles_total) return;
    const long tile_m = logical / tiles_n;
    const int tile_n = (int)(logical - tile_m * tiles_n);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, g = lane >> 5;
    const long r0 = tile_m * TM;
    const int n0 = tile_n * TN;
    const long plane_elems = (long)O_pad * I;

    floatx16 acc[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ni++)
#pragma unroll
        for (int q = 0; q < 16; q++) acc[ni][q] = 0.f;

    // this lane's row of x (clamped past the end: those accumulators are never written)
    const long my_row = r0 + wave * 32 + m;
    const long ld_row = my_row < R ? my_row : R - 1;
    const float* xrow = X + ld_row * I + 16 * g;
    float sx;
    {
        float amax = 0.f;
        const float* xm = xmax + (ld_row / xmax_div) * xmax_stride;
        for (int p = 0; p < xmax_parts; p++) amax = fmaxf(amax, xm[p]);
        amax = fmaf(amax, bound_mul, bound_add);             // the caller's bound of |x| is bound_mul * xmax + bound_add
        float inv;
        sx = pow2_scale(amax, &inv);
        if (g == 0) inv_sx[wave * 32 + m] = inv;
    }
    const _Float16* wsrc[kPer];
    int wdst[kPer];
#pragma unroll
    for (int j = 0; j < kPer; j++) {
        int q = tid + THREADS * j;
        if (q >= kPieces) q = kPieces - 1;                    // surplus threads repeat the last piece
        const int plane = q / (4 * TN), row = (q % (4 * TN)) >> 2, piece = q & 3;
        wsrc[j] = Wp + plane * plane_elems + (long)(n0 + row) * I + 8 * piece;
        wdst[j] = plane * kPlaneW + row * kRowW + piece * 16;
    }
    const int k_last = I - kCK;

    struct ARegs { float4 v[4]; };
    struct WRegs { halfx8 v[kPer]; };
    auto load_a = [&](ARegs& a, int k0) {
        k0 = k0 < I ? k0 : k_last;                            // surplus loads of the last trips are never used
#pragma unroll
        for (int j = 0; j < 4; j++) a.v[j] = *reinterpret_cast<const float4*>(xrow + k0 + 4 * j);
    };
    auto load_w = [&](WRegs& w, int k0) {
        k0 = k0 < I ? k0 : k_last;
#pragma unroll
        for (int j = 0; j < kPer; j++) w.v[j] = *reinterpret_cast<const halfx8*>(wsrc[j] + k0);
    };
    auto store_w = [&](const WRegs& w, unsigned char* buf) {
#pragma unroll
        for (int j = 0; j < kPer; j++) *reinterpret_cast<halfx8*>(buf + wdst[j]) = w.v[j];
    };
    const int b_off = m * kRowW + 32 * g;
    auto compute = [&](const ARegs& a, const unsigned char* buf, float scale) {
        halfx8 ah[2], al[2];
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const HalfSplit4 p0 = split(a.v[2 * s], scale), p1 = split(a.v[2 * s + 1], scale);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                ah[s][i] = p0.hi[i]; ah[s][4 + i] = p1.hi[i];
                al[s][i] = p0.lo[i]; al[s][4 + i] = p1.lo[i];
            }
        }
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
            for (int ni = 0; ni < NI; ni++) {
                const halfx8 bh = *reinterpret_cast<const halfx8*>(buf + b_off + ni * 32 * kRowW + 16 * s);
                const halfx8 bl = *reinterpret_cast<const halfx8*>(buf + kPlaneW + b_off + ni * 32 * kRowW + 16 * s);
                // small terms first
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[s], bh, acc[ni], 0, 0, 0);
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[s], bl, acc[ni], 0, 0, 0);
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[s], bh, acc[ni], 0, 0, 0);
            }
    };

    unsigned char* buf0 = lds;
    unsigned char* buf1 = lds + kBufW;
    ARegs a0, a1;
    WRegs w;
    load_w(w, 0);
    load_a(a0, 0);
    store_w(w, buf0);
    load_w(w, kCK);
    load_a(a1, kCK);
    __syncthreads();
    // chunks in pairs (even chunk: a0 / buf0, odd chunk: a1 / buf1); with an odd chunk count the
    // surplus chunk (a clamped reload of the last one) is scaled by zero instead of being branched
    // around, which keeps the loop body straight-line
    for (int k0 = 0; k0 < I; k0 += 2 * kCK) {
        compute(a0, buf0, sx);
        store_w(w, buf1);
        __builtin_amdgcn_sched_barrier(0);     // keep this issue order: the compiler would hoist the loads
        load_w(w, k0 + 2 * kCK);
        __builtin_amdgcn_sched_barrier(0);
        load_a(a0, k0 + 2 * kCK);
        __syncthreads();
        compute(a1, buf1, k0 + kCK < I ? sx : 0.f);
        store_w(w, buf0);
        __builtin_amdgcn_sched_barrier(0);
        load_w(w, k0 + 3 * kCK);
        __builtin_amdgcn_sched_barrier(0);
        load_a(a1, k0 + 3 * kCK);
        __syncthreads();
    }

    const bool full_cols = n0 + TN <= O;
    // ---- fast path, plain rows: y (rows, O)
    auto epilogue_rows = [&](auto act_tag, auto acc_tag) {
        constexpr int kAct = decltype(act_tag)::value;
        constexpr bool kAccumulate = decltype(acc_tag)::value;
        float bv[NI], iw[NI];
#pragma unroll
        for (int ni = 0; ni < NI; ni++) {
            bv[ni] = bias ? bias[n0 + ni * 32 + m] : 0.f;
            iw[ni] = w_inv[n0 + ni * 32 + m];
        }
#pragma unroll
        for (int q = 0; q < 16; q++) {
            const int rl = wave * 32 + 8 * (q / 4) + 4 * g + (q % 4);
            const long r = r0 + rl;
            if (r < R) {
                float* yrow = Y + r * O + n0 + m;
                const float isx = inv_sx[rl];
                float mx = 0.f;
#pragma unroll
                for (int ni = 0; ni < NI; ni++) {
                    float v = activate_c<kAct>(acc[ni][q] * isx * iw[ni] + bv[ni]);
                    if constexpr (kAccumulate) v += yrow[ni * 32];
                    yrow[ni * 32] = v;
                    mx = fmaxf(mx, fabsf(v));
                }
                if (ymax) {
#pragma unroll
                    for (int d = 1; d < 32; d <<= 1) mx = fmaxf(mx, __shfl_xor(mx, d));
                    if (m == 0) ymax[r * tiles_n + tile_n] = mx;
                }
            }
        }
    };
    // ---- fast path, rows are (row, comp) pairs and y is stored (row, chan, comp): no bias, no activation
    auto epilogue_comps = [&](auto t_tag) {
        constexpr int T = decltype(t_tag)::value;
        float iw[NI];
#pragma unroll
        for (int ni = 0; ni < NI; ni++) iw[ni] = w_inv[n0 + ni * 32 + m];
#pragma unroll
        for (int q = 0; q < 16; q++) {
            const int rl = wave * 32 + 8 * (q / 4) + 4 * g + (q % 4);
            const long r = r0 + rl;
            if (r < R) {
                const long row = r / T;
                float* yp = Y + (row * O + n0 + m) * T + (r - row * T);
                const float isx = inv_sx[rl];
#pragma unroll
                for (int ni = 0; ni < NI; ni++) {
                    float v = acc[ni][q] * isx * iw[ni];
                    if (accumulate) v += yp[ni * 32 * T];
                    yp[ni * 32 * T] = v;
                }
            }
        }
    };
    if (full_cols && out_T == 1) {
        if (accumulate) {
            if (act == 1) epilogue_rows(std::integral_constant<int, 1>{}, std::true_type{});
            else if (act == 2) epilogue_rows(std::integral_constant<int, 2>{}, std::true_type{});
            else epilogue_rows(std::integral_constant<int, 0>{}, std::true_type{});
        } else {
            if (act == 1) epilogue_rows(std::integral_constant<int, 1>{}, std::false_type{});
            else if (act == 2) epilogue_rows(std::integral_constant<int, 2>{}, std::false_type{});
            else epilogue_rows(std::integral_constant<int, 0>{}, std::false_type{});
        }
        return;
    }
    if (full_cols && act == 0 && bias == nullptr && out_T == 3) { epilogue_comps(std::integral_constant<int, 3>{}); return; }
    if (full_cols && act == 0 && bias == nullptr && out_T == 9) { epilogue_comps(std::integral_constant<int, 9>{}); return; }

    // ---- general path: partial column tiles, or components with bias / activation
    float rmax[16];
#pragma unroll
    for (int q = 0; q < 16; q++) rmax[q] = 0.f;
#pragma unroll
    for (int ni = 0; ni < NI; ni++) {
        const int n = n0 + ni * 32 + m;
        if (n >= O) continue;
        const float bv = bias ? bias[n] : 0.f;
        const float iw = w_inv[n];
#pragma unroll
        for (int q = 0; q < 16; q++) {
            const int rl = wave * 32 + 8 * (q / 4) + 4 * g + (q % 4);
            const long r = r0 + rl;
            if (r < R) {
                const long row = r / out_T;
                const long addr = (row * O + n) * out_T + (r - row * out_T);
                float v = activate(acc[ni][q] * inv_sx[rl] * iw + bv, act);
                if (accumulate) v += Y[addr];
                Y[addr] = v;
                rmax[q] = fmaxf(rmax[q], fabsf(v));
            }
        }
    }
    if (ymax) {
#pragma unroll
        for (int q = 0; q < 16; q++) {
            float mx = rmax[q];
#pragma unroll
            for (int d = 1; d < 32; d <<= 1) mx = fmaxf(mx, __shfl_xor(mx, d));
            const long r = r0 + wave * 32 + 8 * (q / 4) + 4 * g + (q % 4);
            if (m == 0 && r < R) ymax[r * tiles_n + tile_n] = mx;
        }
    }
}

// Few rows, few columns, long K (the output linears of one small system: 18 432 rows, K = 1280, 16 columns): the
// row-streaming kernel above gives such a problem a handful of workgroups that each walk 40 chunks one barrier at a
// time, about 1.3 us per chunk of load and LDS latency with nothing to overlap it.  Here a workgroup owns a tile of
// 32 rows x 32 NI columns and its WAVES waves split K: wave w takes chunks w, w + WAVES, ... with private
// accumulators, reads its W fragments straight from the packed planes (L2 resident; no LDS, no barrier in the loop),
// and the partial tiles are summed through LDS in wave order, so the result does not depend on timing.
template <int WAVES, int NI>
__global__ void __launch_bounds__(64 * WAVES)
linear_rows_splitk_f16x2_kernel(const _Float16* __restrict__ Wp, const float* __restrict__ w_inv,
                                const float* __restrict__ X, const float* __restrict__ xmax, int xmax_parts,
                                long xmax_stride, long xmax_div, long R, int I, int O, int O_pad,
                                const float* __restrict__ bias, int act, int accumulate, float* __restrict__ Y,
                                float* __restrict__ ymax, int tiles_n, int out_T, float bound_mul, float bound_add) {
    constexpr int TN = 32 * NI, THREADS = 64 * WAVES;
    constexpr int kPitch = TN + 1;                            // floats per row of a partial tile
    __shared__ float partial[WAVES][32 * kPitch];
    __shared__ float inv_sx[32];

    const long tile_m = blockIdx.x / tiles_n;
    const int tile_n = (int)(blockIdx.x - tile_m * tiles_n);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, g = lane >> 5;
    const long r0 = tile_m * 32;
    const int n0 = tile_n * TN;
    const long plane_elems = (long)O_pad * I;

    const long my_row = r0 + m;
    const long ld_row = my_row < R ? my_row : R - 1;
    const float* xrow = X + ld_row * I + 16 * g;
    float sx;
    {
        float amax = 0.f;
        const float* xm = xmax + (ld_row / xmax_div) * xmax_stride;
        for (int p = 0; p < xmax_parts; p++) amax = fmaxf(amax, xm[p]);
        amax = fmaf(amax, bound_mul, bound_add);
        float inv;
        sx = pow2_scale(amax, &inv);
        if (wave == 0 && g == 0) inv_sx[m] = inv;
    }
    // lane's fragment of W for MFMA step s, column block ni: row n0 + 32 ni + m, k = k0 + 16 g + 8 s .. + 8
    const _Float16* wrow = Wp + (long)(n0 + m) * I + 16 * g;

    floatx16 acc[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ni++)
#pragma unroll
        for (int q = 0; q < 16; q++) acc[ni][q] = 0.f;

    struct Chunk {
        float4 a[4];
        halfx8 wh[NI][2], wl[NI][2];
    };
    auto load = [&](Chunk& c, int k0) {
#pragma unroll
        for (int ni = 0; ni < NI; ni++)
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++) {
                c.wh[ni][s2] = *reinterpret_cast<const halfx8*>(wrow + (long)ni * 32 * I + k0 + 8 * s2);
                c.wl[ni][s2] = *reinterpret_cast<const halfx8*>(wrow + plane_elems + (long)ni * 32 * I + k0 + 8 * s2);
            }
#pragma unroll
        for (int j = 0; j < 4; j++) c.a[j] = *reinterpret_cast<const float4*>(xrow + k0 + 4 * j);
    };
    auto compute = [&](const Chunk& c) {
#pragma unroll
        for (int s2 = 0; s2 < 2; s2++) {
            const HalfSplit4 p0 = split(c.a[2 * s2], sx), p1 = split(c.a[2 * s2 + 1], sx);
            halfx8 ah, al;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                ah[i] = p0.hi[i]; ah[4 + i] = p1.hi[i];
                al[i] = p0.lo[i]; al[4 + i] = p1.lo[i];
            }
#pragma unroll
            for (int ni = 0; ni < NI; ni++) {
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, c.wh[ni][s2], acc[ni], 0, 0, 0);
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, c.wl[ni][s2], acc[ni], 0, 0, 0);
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, c.wh[ni][s2], acc[ni], 0, 0, 0);
            }
        }
    };
    // this wave's chunks, the next one requested before the current one is consumed
    const int chunks = I / kCK;
    Chunk cur, nxt;
    if (wave < chunks) load(cur, wave * kCK);
    for (int c = wave; c < chunks; c += WAVES) {
        const bool more = c + WAVES < chunks;
        if (more) load(nxt, (c + WAVES) * kCK);
        compute(cur);
        if (more) cur = nxt;
    }
    // partial tiles -> LDS; accumulator register q of block ni is row 8 (q / 4) + 4 g + q % 4, column 32 ni + m
#pragma unroll
    for (int ni = 0; ni < NI; ni++)
#pragma unroll
        for (int q = 0; q < 16; q++)
            partial[wave][(8 * (q / 4) + 4 * g + (q % 4)) * kPitch + 32 * ni + m] = acc[ni][q];
    __syncthreads();
    // a thread finishes the elements e = tid, tid + THREADS, ...: row e / TN, column e % TN (the TN / 1 lanes of a
    // row are neighbours, so its maximum is a shuffle away)
    constexpr int kPer = 32 * TN / THREADS;
    static_assert(32 * TN % THREADS == 0 && THREADS % TN == 0, "whole rows per pass");
#pragma unroll
    for (int j = 0; j < kPer; j++) {
        const int e = tid + THREADS * j;
        const int rl = e / TN, col = e - rl * TN;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) sum += partial[w][rl * kPitch + col];
        const long r = r0 + rl;
        const int n = n0 + col;
        float v = 0.f;
        if (r < R && n < O) {
            const long row = r / out_T;
            const long addr = (row * O + n) * out_T + (r - row * out_T);
            v = activate(sum * inv_sx[rl] * w_inv[n] + (bias ? bias[n] : 0.f), act);
            if (accumulate) v += Y[addr];
            Y[addr] = v;
        }
        if (ymax) {
            float mx = fabsf(v);
#pragma unroll
            for (int d = 1; d < TN; d <<= 1) mx = fmaxf(mx, __shfl_xor(mx, d));
            if (col == 0 && r < R) ymax[r * tiles_n + tile_n] = mx;
        }
    }
}

inline int o_pad_of(int dim_out) { return (dim_out + 255) / 256 * 256; }

// the split-K kernel's domain: one column tile of at most 64 columns (the packed planes are zero filled up to a
// multiple of 256 rows, so a partly used tile reads zeros), at least 16 chunks of K, and few rows.  Measured
// against the row-streaming kernel for K = 512 .. 2048: 11 - 19 us against 13 - 67 us up to 6144 rows; from
// about 12 000 rows on the row-streaming kernel (which reads W once per 256 rows and keeps more of x in flight)
// is level or ahead, except at 16 columns or fewer, where its 32-column tile is half empty (31 against 48 us at
// 18 432 rows, K = 1280).
inline bool use_splitk(long R, int I, int O) {
    return O <= 64 && I >= 512 && (R <= 8192 || (O <= 16 && R <= 32768));
}

struct Shape {
    int ni;      // 32-column blocks per tile
    int waves;   // waves per workgroup (32 rows each)
};
inline Shape choose_shape(long R, int I, int O) {
    Shape s;
    s.ni = O <= 32 ? 1 : (O <= 64 ? 2 : (O <= 128 ? 4 : 8));
    // column tiles that divide O: a partly filled tile takes the slow, bounds-checked epilogue (O = 384 with
    // 256-column tiles ran 4 times slower than with 128-column tiles)
    if (O % 32 == 0)
        while (s.ni > 1 && O % (32 * s.ni) != 0 && ceil_div(O, 16 * s.ni) <= 64) s.ni >>= 1;
    const long tiles_m = ceil_div(R, 256);
    if (tiles_m * ceil_div(O, 32 * s.ni) >= 1024 || O % 32 != 0) {
        s.waves = 8;                                       // many tiles: the widest tile, one 8-wave workgroup per CU
        return s;
    }
    // Few tiles (node-sized problems, the edges of one small system).  The chip takes 256 workgroups of 8 waves at
    // a time, and a workgroup's time was measured (33 392 rows, K = 256 .. 768, all tile widths) as about
    // 5 us + chunks x (1 + ni / 4) us: among the column tiles that divide O take the one with the least
    // (rounds of 256 workgroups) x (time per workgroup); ties go to the wider tile, which re-reads x less often.
    const long chunks = ceil_div(I, 32);
    long best = -1;
    for (int ni = s.ni; ni >= 1; ni >>= 1) {
        if (O % (32 * ni) != 0 || ceil_div(O, 32 * ni) > 64) continue;   // at most 64 column tiles (row maxima per tile)
        const long cost = ceil_div(tiles_m * (O / (32 * ni)), 256) * (20 + chunks * (4 + ni));
        if (best < 0 || cost < best) { best = cost; s.ni = ni; }
    }
    // fewer than two chips' worth of 8-wave workgroups: 4-wave workgroups (128 rows) double their number; not with
    // 256-column tiles, whose 4-wave variant keeps one wave per SIMD
    s.waves = (tiles_m * ceil_div(O, 32 * s.ni) >= 512 || (s.ni == 8 && tiles_m >= 32)) ? 8 : 4;
    return s;
}

template <int WAVES, int NI>
int launch(const _Float16* planes, const float* w_inv, const float* x, const float* xmax, int parts, long stride,
           long div, long rows, int I, int O, int O_pad, const float* bias, int act, int accumulate, float* y,
           float* ymax, int out_T, float bound_mul, float bound_add, hipStream_t st) {
    const long tiles_m = ceil_div(rows, 32 * WAVES);
    const int tiles_n = (int)ceil_div(O, 32 * NI);
    const long total = tiles_m * tiles_n;
    const long grid = ceil_div(total, 8) * 8;
    MG_REQUIRE(grid <= 0x7fffffffL, "mg_tensor_linear_f16x2: grid too large (rows=%ld dim_out=%d)", rows, O);
    hipLaunchKernelGGL((linear_rows_f16x2_kernel<WAVES, NI>), dim3((unsigned)grid), dim3(64 * WAVES), 0, st, planes,
                       w_inv, x, xmax, parts, stride, div, rows, I, O, O_pad, bias, act, accumulate, y, ymax, tiles_n,
                       total, out_T, bound_mul, bound_add);
    return check_launch("mg_tensor_linear_f16x2");
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_linear_f16x2_packed_weight_bytes(int dim_in, int dim_out, size_t* bytes) {
    MG_REQUIRE(bytes != nullptr && dim_in >= 0 && dim_out >= 0, "mg_linear_f16x2_packed_weight_bytes: bad argument");
    const size_t o_pad = (size_t)o_pad_of(dim_out);
    *bytes = 2 * o_pad * (size_t)dim_in * sizeof(_Float16) + o_pad * sizeof(float);
    return MG_OK;
}

int mg_linear_f16x2_pack_weight(const float* W, long w_stride_o, long w_stride_i, int dim_in, int dim_out,
                                void* packed, mg_stream_t stream) {
    MG_REQUIRE(dim_in >= 0 && dim_out >= 0, "mg_linear_f16x2_pack_weight: negative size");
    if (dim_in == 0 || dim_out == 0) return MG_OK;
    MG_REQUIRE(W && packed && aligned16(packed), "mg_linear_f16x2_pack_weight: null or unaligned pointer");
    MG_REQUIRE(dim_in % 8 == 0, "mg_linear_f16x2_pack_weight: dim_in must be a multiple of 8");
    const int O_pad = o_pad_of(dim_out);
    _Float16* planes = static_cast<_Float16*>(packed);
    float* inv = reinterpret_cast<float*>(planes + 2L * O_pad * dim_in);
    hipLaunchKernelGGL(pack_weight_f16x2_kernel, dim3((unsigned)ceil_div(O_pad, 4)), dim3(256), 0, (hipStream_t)stream,
                       W, w_stride_o, w_stride_i, dim_in, dim_out, O_pad, planes, inv);
    return check_launch("mg_linear_f16x2_pack_weight");
}

int mg_row_absmax(const float* x, long rows, int dim, float* out, mg_stream_t stream) {
    MG_REQUIRE(rows >= 0 && dim >= 0, "mg_row_absmax: negative size");
    if (rows == 0) return MG_OK;
    MG_REQUIRE(out && (x || dim == 0), "mg_row_absmax: null pointer");
    MG_REQUIRE(dim % 4 != 0 || aligned16(x), "mg_row_absmax: x must be 16-byte aligned");
    long blocks = ceil_div(rows, 4);
    if (blocks > 256L * 32) blocks = 256L * 32;
    hipLaunchKernelGGL(row_absmax_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, x, rows, dim, out);
    return check_launch("mg_row_absmax");
}

int mg_components_to_rows(const float* x, long rows, int dim, int comps, int dim_pad, float* xt, float* rowmax,
                          mg_stream_t stream) {
    MG_REQUIRE(rows >= 0 && dim > 0 && comps > 0, "mg_components_to_rows: bad size");
    MG_REQUIRE(dim_pad >= dim && dim_pad % 32 == 0 && dim_pad <= 256 && (dim_pad & (dim_pad - 1)) == 0,
               "mg_components_to_rows: dim_pad must be a power of two in 32..256, at least dim (got %d for %d)", dim_pad, dim);
    if (rows == 0) return MG_OK;
    MG_REQUIRE(x && xt && rowmax && aligned16(xt), "mg_components_to_rows: null or unaligned pointer");
    const long threads = rows * comps * (dim_pad / 4);
    hipLaunchKernelGGL(components_to_rows_kernel, dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0,
                       (hipStream_t)stream, x, rows, dim, comps, dim_pad, xt, rowmax);
    return check_launch("mg_components_to_rows");
}

int mg_tensor_linear_f16x2_rowmax_parts(long rows, int dim_in, int dim_out) {
    if (use_splitk(rows, dim_in, dim_out)) return 1;
    return (int)ceil_div(dim_out, 32 * choose_shape(rows, dim_in, dim_out).ni);
}

int mg_tensor_linear_f16x2(const void* packed_W, const float* x, const float* x_rowmax, int x_rowmax_parts,
                           long x_rowmax_stride, long x_rows_per_bound, long rows, int dim_in, int dim_out,
                           const float* bias, int act, int accumulate, int out_comps, float* y, float* y_rowmax,
                           mg_stream_t stream) {
    return mg_tensor_linear_f16x2_scaled_bound(packed_W, x, x_rowmax, x_rowmax_parts, x_rowmax_stride, x_rows_per_bound,
                                               rows, dim_in, dim_out, bias, act, accumulate, out_comps, y, y_rowmax, 1.0f,
                                               0.0f, stream);
}

int mg_tensor_linear_f16x2_scaled_bound(const void* packed_W, const float* x, const float* x_rowmax, int x_rowmax_parts,
                                        long x_rowmax_stride, long x_rows_per_bound, long rows, int dim_in, int dim_out,
                                        const float* bias, int act, int accumulate, int out_comps, float* y,
                                        float* y_rowmax, float bound_mul, float bound_add, mg_stream_t stream) {
    MG_REQUIRE(bound_mul >= 0.f && bound_add >= 0.f && bound_mul == bound_mul && bound_add == bound_add,
               "mg_tensor_linear_f16x2: the bound's factor and offset must be non-negative numbers");
    MG_REQUIRE(rows >= 0 && dim_in > 0 && dim_out >= 0, "mg_tensor_linear_f16x2: bad size");
    MG_REQUIRE(dim_in % 32 == 0, "mg_tensor_linear_f16x2: dim_in must be a multiple of 32");
    MG_REQUIRE(act >= 0 && act <= 2, "mg_tensor_linear_f16x2: unknown activation %d", act);
    MG_REQUIRE(out_comps == 1 || out_comps == 3 || out_comps == 9, "mg_tensor_linear_f16x2: out_comps must be 1, 3 or 9");
    MG_REQUIRE(x_rowmax_parts >= 1 && x_rowmax_parts <= 64, "mg_tensor_linear_f16x2: x_rowmax_parts must be in 1..64");
    MG_REQUIRE(x_rowmax_stride == 0 || x_rowmax_stride >= x_rowmax_parts,
               "mg_tensor_linear_f16x2: x_rowmax_stride must be 0 (one bound for all rows) or >= x_rowmax_parts");
    MG_REQUIRE(x_rows_per_bound >= 1, "mg_tensor_linear_f16x2: x_rows_per_bound must be positive");
    MG_REQUIRE(y_rowmax == nullptr || out_comps == 1, "mg_tensor_linear_f16x2: y_rowmax needs out_comps == 1");
    if (rows == 0 || dim_out == 0) return MG_OK;
    MG_REQUIRE(packed_W && x && y && x_rowmax && aligned16(x) && aligned16(packed_W),
               "mg_tensor_linear_f16x2: null or unaligned pointer");
    const int O_pad = o_pad_of(dim_out);
    const _Float16* planes = static_cast<const _Float16*>(packed_W);
    const float* w_inv = reinterpret_cast<const float*>(planes + 2L * O_pad * dim_in);
    hipStream_t st = (hipStream_t)stream;
    if (use_splitk(rows, dim_in, dim_out)) {
        const long tiles = ceil_div(rows, 32);
        MG_REQUIRE(tiles <= 0x7fffffffL, "mg_tensor_linear_f16x2: grid too large (rows=%ld)", rows);
        if (dim_out <= 32)
            hipLaunchKernelGGL((linear_rows_splitk_f16x2_kernel<8, 1>), dim3((unsigned)tiles), dim3(512), 0, st, planes,
                               w_inv, x, x_rowmax, x_rowmax_parts, x_rowmax_stride, x_rows_per_bound, rows, dim_in,
                               dim_out, O_pad, bias, act, accumulate, y, y_rowmax, 1, out_comps, bound_mul, bound_add);
        else
            hipLaunchKernelGGL((linear_rows_splitk_f16x2_kernel<8, 2>), dim3((unsigned)tiles), dim3(512), 0, st, planes,
                               w_inv, x, x_rowmax, x_rowmax_parts, x_rowmax_stride, x_rows_per_bound, rows, dim_in,
                               dim_out, O_pad, bias, act, accumulate, y, y_rowmax, 1, out_comps, bound_mul, bound_add);
        return check_launch("mg_tensor_linear_f16x2");
    }
    const Shape sh = choose_shape(rows, dim_in, dim_out);
#define MG_F16X2_LAUNCH(WV, N)                                                                                       \
    return launch<WV, N>(planes, w_inv, x, x_rowmax, x_rowmax_parts, x_rowmax_stride, x_rows_per_bound, rows, dim_in, \
                         dim_out, O_pad, bias, act, accumulate, y, y_rowmax, out_comps, bound_mul, bound_add, st)
    if (sh.waves == 8) {
        if (sh.ni == 1) MG_F16X2_LAUNCH(8, 1);
        if (sh.ni == 2) MG_F16X2_LAUNCH(8, 2);
        if (sh.ni == 4) MG_F16X2_LAUNCH(8, 4);
        MG_F16X2_LAUNCH(8, 8);
    }
    if (sh.ni == 1) MG_F16X2_LAUNCH(4, 1);
    if (sh.ni == 2) MG_F16X2_LAUNCH(4, 2);
    if (sh.ni == 4) MG_F16X2_LAUNCH(4, 4);
    MG_F16X2_LAUNCH(4, 8);
#undef MG_F16X2_LAUNCH
}

}  // extern "C"
