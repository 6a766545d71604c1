// TensorProds in one kernel: y = lin_o(prod(lin_l(x_l), lin_r(x_r)))   (managan/tensor_products.py:109-121)
//     u[b, k, :] = sum_i W_l[k, i] x_l[b, i, :]      w[b, k, :] = sum_j W_r[k, j] x_r[b, j, :]
//     p[b, k, :] = u[b, k, :] (x) w[b, k, :]         (TensorProdBare: trailing indices contracted)
//     y[b, o, :] = sum_k W_o[o, k] p[b, k, :]
// Three chained GEMMs with an elementwise product between them, all on the fp32 matrix instruction
// v_mfma_f32_16x16x4_f32 (exact fp32 products, fp32 accumulation) and without any intermediate leaving
// the registers: every GEMM is computed transposed (channels x rows), so that an accumulator tile, whose
// lanes hold one row each and whose four registers hold four consecutive channels, is already laid out
// as the B operand of the next GEMM (lane = row, lane group and register = reduction index).  The weights
// are staged once per workgroup in LDS in A-operand order (one conflict-free 16-byte read per lane gives
// four reduction steps); x is read straight from global memory, every lane a contiguous run of its row.
// A wave owns 16 rows; a workgroup is four waves and walks over many 64-row tiles with the weights staged once,
// requesting the next tile's operands while it computes on the current one.
#include "common.hpp"

namespace mg {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

#include "ant16_coupling.inc"

constexpr int comps(int rank) { return rank == 0 ? 1 : (rank == 1 ? 3 : 9); }
// position of a non-chiral product type in the label order 000 110 220 011 101 121 211 022 202 112 222
constexpr int label_of(int l, int r, int o) {
    constexpr int code[11] = {0, 110, 220, 11, 101, 121, 211, 22, 202, 112, 222};
    for (int k = 0; k < 11; k++)
        if (code[k] == 100 * l + 10 * r + o) return k;
    return -1;
}

constexpr int kOT = 4;      // 16-channel output tiles per workgroup (64 output channels per grid row)

constexpr int kHoistPer = 16;   // operands of rank <= 1 live in registers: at most 16 channels per lane group (dim <= 64)

// One 16-channel tile of lin(x)^T for this wave's 16 rows: acc[c] += W-tile . x^T over all input channels.
// per: input channels per lane group (lane group g takes channels g * per ... g * per + per - 1, the same on the
// A side).  This lane's A values of steps 4 k ... 4 k + 3 are the four floats at wa + k * wstride: either the
// staged copy in LDS ([steps / 4][64 lanes][4]: wa = tile + 4 lane, wstride = 256) or W itself in global memory
// (wa = &W[16 t + m][g per], wstride = 4).
// Operand kept in registers: xv[s * C + c] = component c of channel g * per + s of this lane's row.
template <int C>
__device__ __forceinline__ void linear_tile_regs(const float* __restrict__ wa, int wstride, const float (&xv)[kHoistPer * C],
                                                 int per, floatx4 (&acc)[C]) {
#pragma unroll
    for (int s0 = 0; s0 < kHoistPer; s0 += 4) {
        if (s0 < per) {
            const floatx4 a = *reinterpret_cast<const floatx4*>(wa + (s0 >> 2) * wstride);
#pragma unroll
            for (int s = 0; s < 4; s++)
#pragma unroll
                for (int c = 0; c < C; c++)
                    acc[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s], xv[(s0 + s) * C + c], acc[c], 0, 0, 0);
        }
    }
}

template <int C>
__device__ __forceinline__ void load_run(const float* __restrict__ xp, int per, float (&xv)[kHoistPer * C]) {
#pragma unroll
    for (int s0 = 0; s0 < kHoistPer; s0 += 4)
#pragma unroll
        for (int q = 0; q < C; q++) {
            floatx4 v = floatx4{0.f, 0.f, 0.f, 0.f};
            if (s0 < per) v = *reinterpret_cast<const floatx4*>(xp + s0 * C + 4 * q);
            xv[s0 * C + 4 * q] = v[0]; xv[s0 * C + 4 * q + 1] = v[1]; xv[s0 * C + 4 * q + 2] = v[2]; xv[s0 * C + 4 * q + 3] = v[3];
        }
}

// Operand streamed from global memory (rank-2 operands: too many values to keep): four steps per trip, the
// next trip's values requested before this trip's matrix instructions are issued.
template <int C>
__device__ __forceinline__ void linear_tile_stream(const float* __restrict__ wa, int wstride, const float* __restrict__ xp,
                                                   int per, floatx4 (&acc)[C]) {
    floatx4 nxt[C];
#pragma unroll
    for (int q = 0; q < C; q++) nxt[q] = *reinterpret_cast<const floatx4*>(xp + 4 * q);
    for (int s0 = 0; s0 < per; s0 += 4) {
        const floatx4 a = *reinterpret_cast<const floatx4*>(wa + (s0 >> 2) * wstride);
        float xv[4 * C];
#pragma unroll
        for (int q = 0; q < C; q++) { xv[4 * q] = nxt[q][0]; xv[4 * q + 1] = nxt[q][1]; xv[4 * q + 2] = nxt[q][2]; xv[4 * q + 3] = nxt[q][3]; }
        const int sn = s0 + 4 < per ? s0 + 4 : s0;
#pragma unroll
        for (int q = 0; q < C; q++) nxt[q] = *reinterpret_cast<const floatx4*>(xp + sn * C + 4 * q);
#pragma unroll
        for (int s = 0; s < 4; s++)
#pragma unroll
            for (int c = 0; c < C; c++) acc[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s], xv[s * C + c], acc[c], 0, 0, 0);
    }
}

// Weights into LDS in A-operand order, 16 bytes at a time: entry (tile, step group s4, lane (m, g)) holds
// W[row0 + 16 tile_row + m][col(tile, g, s4) ... + 3].
__device__ __forceinline__ void stage_inner(const float* __restrict__ W, long ld, int rank, int dim, float* __restrict__ dst, int tid) {
    const int per = dim >> 2, q4 = per >> 2;                      // lane group g takes columns g per ... ; q4 step groups
    for (int e = tid; e < (rank * dim) >> 2; e += 256) {
        const int ln = e & 63, rest = e >> 6;                     // rest = t * q4 + s4
        const int t = rest / q4, s4 = rest - t * q4;
        *reinterpret_cast<floatx4*>(dst + 4 * e) =
            *reinterpret_cast<const floatx4*>(W + (long)(16 * t + (ln & 15)) * ld + (ln >> 4) * per + 4 * s4);
    }
}

// SPLIT = false: a wave owns 16 rows of a 64-row tile and runs over every inner tile; a workgroup (four waves)
// walks over tiles gridDim.x apart, with the weights staged once.
// SPLIT = true (few rows): the four waves of a workgroup share 16 rows and split the inner tiles; their partial
// outputs are exchanged through LDS so that wave w ends up with output tile w, which it stores.
template <int L, int R, int O, bool SPLIT>
__global__ void __launch_bounds__(256)
tensor_prods_kernel(const float* __restrict__ W_l, long ldl, const float* __restrict__ W_r, long ldr,
                    const float* __restrict__ W_o, long ldo, const float* __restrict__ x_l, const float* __restrict__ x_r,
                    long rows, int dim_l, int dim_r, int rank, int dim_o, float* __restrict__ y) {
    constexpr int CL = comps(L), CR = comps(R), CO = comps(O);
    constexpr int LAB = label_of(L, R, O);
    constexpr bool HOIST_L = CL <= 3, HOIST_R = CR <= 3;       // rank-2 operands are streamed
    static_assert(LAB >= 0, "not a TensorProdBare product");
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = lane & 15, g = lane >> 4;
    const int RT = rank >> 4;                                    // 16-channel tiles of the inner dimension
    const int per_l = dim_l >> 2, per_r = dim_r >> 2;            // input channels per lane group
    const int o_base = blockIdx.y * (16 * kOT);
    const int n_ot = (dim_o - o_base) / 16 < kOT ? (dim_o - o_base) / 16 : kOT;
    float* wl = smem;                                            // [RT][per_l / 4][64][4]
    float* wr = wl + rank * dim_l;                               // [RT][per_r / 4][64][4]
    float* wo = wr + rank * dim_r;                               // [n_ot][RT][64][4]

    const long rows_per_block = SPLIT ? 16 : 64;
    const long n_tiles = (rows + rows_per_block - 1) / rows_per_block;
    long tile = blockIdx.x;
    long r0 = SPLIT ? tile * 16 : (tile * 4 + wave) * 16;
    float xlv[HOIST_L ? kHoistPer * CL : 1], xrv[HOIST_R ? kHoistPer * CR : 1];
    // the first tile's operands are requested before the weights are staged
    {
        const long row = r0 + m < rows ? r0 + m : rows - 1;      // rows past the end repeat the last one, never stored
        if constexpr (HOIST_L) load_run<CL>(x_l + (row * dim_l + (long)g * per_l) * CL, per_l, xlv);
        if constexpr (HOIST_R) load_run<CR>(x_r + (row * dim_r + (long)g * per_r) * CR, per_r, xrv);
    }
    if constexpr (!SPLIT) {
        stage_inner(W_l, ldl, rank, dim_l, wl, tid);
        stage_inner(W_r, ldr, rank, dim_r, wr, tid);
        // second GEMM: lane (m, g), steps 0..3 of (output tile ot, inner tile t) <- W_o[o_base + 16 ot + m][16 t + 4 g ...]
        for (int e = tid; e < n_ot * 4 * rank; e += 256) {
            const int ln = e & 63, rest = e >> 6;                // rest = ot * RT + t
            const int ot = rest / RT, t = rest - ot * RT;
            *reinterpret_cast<floatx4*>(wo + 4 * e) =
                *reinterpret_cast<const floatx4*>(W_o + (long)(o_base + 16 * ot + (ln & 15)) * ldo + 16 * t + 4 * (ln >> 4));
        }
        __syncthreads();
    }

    for (; tile < n_tiles; tile += gridDim.x) {
        r0 = SPLIT ? tile * 16 : (tile * 4 + wave) * 16;
        const long row = r0 + m < rows ? r0 + m : rows - 1;
        const float* xl_run = x_l + (row * dim_l + (long)g * per_l) * CL;
        const float* xr_run = x_r + (row * dim_r + (long)g * per_r) * CR;
        // operands of the next tile of this workgroup, requested now and consumed in the next trip
        float xln[HOIST_L ? kHoistPer * CL : 1], xrn[HOIST_R ? kHoistPer * CR : 1];
        const long tile_n = tile + gridDim.x;
        if (!SPLIT && tile_n < n_tiles) {
            const long rn = (tile_n * 4 + wave) * 16 + m;
            const long row_n = rn < rows ? rn : rows - 1;
            if constexpr (HOIST_L) load_run<CL>(x_l + (row_n * dim_l + (long)g * per_l) * CL, per_l, xln);
            if constexpr (HOIST_R) load_run<CR>(x_r + (row_n * dim_r + (long)g * per_r) * CR, per_r, xrn);
        }

        floatx4 yacc[kOT][CO];
#pragma unroll
        for (int ot = 0; ot < kOT; ot++)
#pragma unroll
            for (int c = 0; c < CO; c++) yacc[ot][c] = floatx4{0.f, 0.f, 0.f, 0.f};

        if (r0 < rows) {
            for (int t = SPLIT ? wave : 0; t < RT; t += SPLIT ? 4 : 1) {
                floatx4 u[CL], w[CR];
#pragma unroll
                for (int c = 0; c < CL; c++) u[c] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < CR; c++) w[c] = floatx4{0.f, 0.f, 0.f, 0.f};
                // a wave of the split variant meets every weight once: it reads them from global memory
                const float* al = SPLIT ? W_l + (long)(16 * t + m) * ldl + g * per_l : wl + t * 16 * dim_l + 4 * lane;
                const float* ar = SPLIT ? W_r + (long)(16 * t + m) * ldr + g * per_r : wr + t * 16 * dim_r + 4 * lane;
                constexpr int wstride = SPLIT ? 4 : 256;
                floatx4 ao[kOT];
#pragma unroll
                for (int ot = 0; ot < kOT; ot++) {
                    ao[ot] = floatx4{0.f, 0.f, 0.f, 0.f};
                    if (ot < n_ot)
                        ao[ot] = SPLIT ? *reinterpret_cast<const floatx4*>(W_o + (long)(o_base + 16 * ot + m) * ldo + 16 * t + 4 * g)
                                       : *reinterpret_cast<const floatx4*>(wo + (((ot * RT + t) * 64) + lane) * 4);
                }
                if constexpr (HOIST_L) linear_tile_regs<CL>(al, wstride, xlv, per_l, u);
                else linear_tile_stream<CL>(al, wstride, xl_run, per_l, u);
                if constexpr (HOIST_R) linear_tile_regs<CR>(ar, wstride, xrv, per_r, w);
                else linear_tile_stream<CR>(ar, wstride, xr_run, per_r, w);
#pragma unroll
                for (int c = 0; c < CO; c++) {
                    floatx4 p = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int k = 0; k < 9; k++) {
                        if (k < kCoupling[0][LAB][c][0]) {       // folded at compile time: c and k are unrolled
                            const int e = kCoupling[0][LAB][c][1 + k];
                            if (e & 256) p -= u[e & 15] * w[(e >> 4) & 15];
                            else p += u[e & 15] * w[(e >> 4) & 15];
                        }
                    }
#pragma unroll
                    for (int s = 0; s < 4; s++)
#pragma unroll
                        for (int ot = 0; ot < kOT; ot++)
                            if (ot < n_ot)
                                yacc[ot][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(ao[ot][s], p[s], yacc[ot][c], 0, 0, 0);
                }
            }
        }

        if constexpr (SPLIT) {
            // every wave parks its partials of the output tiles it does not own in LDS; the owner of tile ot
            // (wave ot) adds the three it receives.
            float* xch = smem;                                   // [4 tiles][4 senders][CO][4][64]
#pragma unroll
            for (int ot = 0; ot < kOT; ot++)
                if (ot != wave && ot < n_ot)
#pragma unroll
                    for (int c = 0; c < CO; c++)
#pragma unroll
                        for (int q = 0; q < 4; q++) xch[(((ot * 4 + wave) * CO + c) * 4 + q) * 64 + lane] = yacc[ot][c][q];
            __syncthreads();
#pragma unroll
            for (int ot = 0; ot < kOT; ot++)
                if (ot == wave && ot < n_ot)
#pragma unroll
                    for (int sender = 0; sender < 4; sender++)
                        if (sender != ot)
#pragma unroll
                            for (int c = 0; c < CO; c++)
#pragma unroll
                                for (int q = 0; q < 4; q++)
                                    yacc[ot][c][q] += xch[(((ot * 4 + sender) * CO + c) * 4 + q) * 64 + lane];
        }

        // lane (row m, group g) holds channels o_base + 16 ot + 4 g + q (register q) of every component:
        // 4 * CO consecutive floats of y per output tile
        if (r0 + m < rows) {
#pragma unroll
            for (int ot = 0; ot < kOT; ot++) {
                if (ot >= n_ot) break;
                if (SPLIT && ot != wave) continue;
                float* yp = y + ((r0 + m) * dim_o + o_base + 16 * ot + 4 * g) * CO;
                float out[4 * CO];
#pragma unroll
                for (int q = 0; q < 4; q++)
#pragma unroll
                    for (int c = 0; c < CO; c++) out[q * CO + c] = yacc[ot][c][q];
#pragma unroll
                for (int v = 0; v < CO; v++)
                    *reinterpret_cast<floatx4*>(yp + 4 * v) = floatx4{out[4 * v], out[4 * v + 1], out[4 * v + 2], out[4 * v + 3]};
            }
        }
        if (!SPLIT && tile_n < n_tiles) {
            if constexpr (HOIST_L) {
#pragma unroll
                for (int k = 0; k < kHoistPer * CL; k++) xlv[k] = xln[k];
            }
            if constexpr (HOIST_R) {
#pragma unroll
                for (int k = 0; k < kHoistPer * CR; k++) xrv[k] = xrn[k];
            }
        }
    }
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_tensor_prods_supported(int inds_l, int inds_r, int inds_o, int dim_l, int dim_r, int rank, int dim_o) {
    if (inds_l < 0 || inds_l > 2 || inds_r < 0 || inds_r > 2 || inds_o < 0 || inds_o > 2) return 0;
    if (label_of(inds_l, inds_r, inds_o) < 0) return 0;
    if (dim_l <= 0 || dim_r <= 0 || rank <= 0 || dim_o <= 0) return 0;
    if (dim_l % 16 || dim_r % 16 || rank % 16 || dim_o % 16) return 0;
    // operands of rank <= 1 are kept in registers, 16 channels per lane group
    if ((inds_l <= 1 && dim_l > 4 * kHoistPer) || (inds_r <= 1 && dim_r > 4 * kHoistPer)) return 0;
    const int ow = dim_o < 16 * kOT ? dim_o : 16 * kOT;
    const size_t lds = sizeof(float) * ((size_t)rank * dim_l + (size_t)rank * dim_r + (size_t)rank * ow);
    return lds <= 64 * 1024 ? 1 : 0;
}

int mg_tensor_prods(int inds_l, int inds_r, int inds_o, const float* W_l, long ldl, const float* W_r, long ldr,
                    const float* W_o, long ldo, const float* x_l, const float* x_r, long rows, int dim_l, int dim_r,
                    int rank, int dim_o, float* y, mg_stream_t stream) {
    MG_REQUIRE(rows >= 0, "mg_tensor_prods: negative size");
    if (!mg_tensor_prods_supported(inds_l, inds_r, inds_o, dim_l, dim_r, rank, dim_o))
        return fail(MG_ERR_UNSUPPORTED, "mg_tensor_prods: needs a TensorProdBare product of ranks <= 2, channel counts that "
                    "are multiples of 16 and weights that fit 64 KB of LDS (got ranks %d %d %d, channels %d %d %d %d)",
                    inds_l, inds_r, inds_o, dim_l, dim_r, rank, dim_o);
    if (rows == 0) return MG_OK;
    MG_REQUIRE(W_l && W_r && W_o && x_l && x_r && y, "mg_tensor_prods: null pointer");
    MG_REQUIRE(ldl >= dim_l && ldr >= dim_r && ldo >= rank, "mg_tensor_prods: weight row stride shorter than a row");
    MG_REQUIRE(((reinterpret_cast<uintptr_t>(x_l) | reinterpret_cast<uintptr_t>(x_r) | reinterpret_cast<uintptr_t>(y)) & 15) == 0,
               "mg_tensor_prods: x_l, x_r and y must be 16-byte aligned");
    MG_REQUIRE(ceil_div(rows, 64) <= 0x7fffffffL, "mg_tensor_prods: too many rows");
    MG_REQUIRE(ldl % 4 == 0 && ldr % 4 == 0 && ldo % 4 == 0 &&
               ((reinterpret_cast<uintptr_t>(W_l) | reinterpret_cast<uintptr_t>(W_r) | reinterpret_cast<uintptr_t>(W_o)) & 15) == 0,
               "mg_tensor_prods: weights must be 16-byte aligned with row strides that are multiples of 4");
    const int ow = dim_o < 16 * kOT ? dim_o : 16 * kOT;
    size_t lds = sizeof(float) * ((size_t)rank * dim_l + (size_t)rank * dim_r + (size_t)rank * ow);
    // few rows: one workgroup per 16 rows, its waves splitting the inner dimension, so that the chip fills
    const bool split = ceil_div(rows, 64) < 512 && rank >= 64;
    const size_t xch = sizeof(float) * 16 * (inds_o == 0 ? 1 : (inds_o == 1 ? 3 : 9)) * 4 * 64;   // the exchange buffer of the split variant
    if (split) lds = xch;                                        // that variant does not stage the weights
    hipStream_t st = (hipStream_t)stream;
    // the split variant takes one workgroup per 16 rows; the other
    // one runs as many workgroups as fit the chip at once and lets each walk over its share of the 64-row tiles
#define MG_TP_LAUNCH(L_, R_, O_, S_)                                                                                \
    do {                                                                                                            \
        const void* fn = reinterpret_cast<const void*>(tensor_prods_kernel<L_, R_, O_, S_>);                        \
        if (lds > 48 * 1024) MG_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        long gx = ceil_div(rows, S_ ? 16 : 64);                                                                     \
        if (!S_) {                                                                                                  \
            int device = 0, cus = 0, per_cu = 1;                                                                    \
            MG_HIP(hipGetDevice(&device));                                                                          \
            MG_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));                     \
            MG_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, 256, lds));                            \
            const long resident = (long)(per_cu > 0 ? per_cu : 1) * (cus > 0 ? cus : 1);                            \
            if (gx > resident) gx = resident;                                                                       \
        }                                                                                                           \
        const dim3 grid((unsigned)gx, (unsigned)ceil_div(dim_o, 16 * kOT));                                         \
        hipLaunchKernelGGL((tensor_prods_kernel<L_, R_, O_, S_>), grid, dim3(256), lds, st, W_l, ldl, W_r, ldr, W_o, ldo, \
                           x_l, x_r, rows, dim_l, dim_r, rank, dim_o, y);                                           \
    } while (0)
#define MG_TP_CASE(L_, R_, O_)                                                                                      \
    if (inds_l == L_ && inds_r == R_ && inds_o == O_) {                                                             \
        if (split) MG_TP_LAUNCH(L_, R_, O_, true);                                                                  \
        else MG_TP_LAUNCH(L_, R_, O_, false);                                                                       \
        return check_launch("mg_tensor_prods");                                                                     \
    }
    MG_TP_CASE(0, 0, 0) MG_TP_CASE(1, 1, 0) MG_TP_CASE(2, 2, 0) MG_TP_CASE(0, 1, 1) MG_TP_CASE(1, 0, 1) MG_TP_CASE(1, 2, 1)
    MG_TP_CASE(2, 1, 1) MG_TP_CASE(0, 2, 2) MG_TP_CASE(2, 0, 2) MG_TP_CASE(1, 1, 2) MG_TP_CASE(2, 2, 2)
#undef MG_TP_CASE
#undef MG_TP_LAUNCH
    return fail(MG_ERR_UNSUPPORTED, "mg_tensor_prods: unsupported product");
}

}  // extern "C"
