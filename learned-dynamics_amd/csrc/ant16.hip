// Ant16: y_o[b, o, :] = sum over product types (l r o) of sum_{i < dim_l, j < dim_r}
//            P_lro[o, i, j] * (left_lro[b, i, :] (x) x_r[b, j, :])     (the 13 Cartesian products)
// (managan/codegen_tensor_products.py:19-34; kernels extensions/codegen_tensops/codegen_tensops_kern.cu:1341-1448).
//
// One dense contraction per product type with K = dim_l * dim_r, M = (row, output component),
// N = output channel, whose A operand is never stored: every lane builds its A value
//     A[(b, c), (i, j)] = component c of left[b, i, :] (x) x[b, j, :]
// from a few LDS reads right before the fp32 matrix instruction (v_mfma_f32_32x32x2_f32: exact
// fp32 products), and P is read in place.  A workgroup owns the rows of one tile (32, 10 or 3 rows
// for output rank 0, 1, 2: 32 = rows x components, rounded down to whole rows) and up to four
// 32-channel column blocks; its four waves split the contraction over the left channels, so an
// A value is built once and meets every column block; operands of the tile are staged in LDS per
// product type and the partial accumulators are summed through LDS.
// Every product component is a short signed dot product  sum_t l[lb + t ls] * r[rb + t rs]  whose
// offsets depend only on the lane's output component, so one generic inner loop serves all 13 types.
#include "common.hpp"

namespace mg {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

struct Term {
    const float* P;      // (dim_o, dim_l, dim_r)
    const float* left;   // (rows, dim_l, 3^rank_l)
    int label;           // index into kLabels
};
constexpr int kMaxTerms = 4;
struct Terms {
    int n;
    Term t[kMaxTerms];
};

// label order: 000 110 220 011 101 121 211 022 202 112 222 111 212
__constant__ const int kRankL[13] = {0, 1, 2, 0, 1, 1, 2, 0, 2, 1, 2, 1, 2};
__constant__ const int kRankR[13] = {0, 1, 2, 1, 0, 2, 1, 2, 0, 1, 2, 1, 1};
constexpr int h_rank_l[13] = {0, 1, 2, 0, 1, 1, 2, 0, 2, 1, 2, 1, 2};
constexpr int h_rank_r[13] = {0, 1, 2, 1, 0, 2, 1, 2, 0, 1, 2, 1, 1};
constexpr int h_rank_o[13] = {0, 0, 0, 1, 1, 1, 1, 2, 2, 2, 2, 1, 2};

struct Dot {
    int lb, ls, rb, rs, nt;
    bool cross;          // two terms, the second one negative
};

// component c of the product of type `label`: the signed dot product it reduces to
__device__ __forceinline__ Dot dot_of(int label, int c) {
    const int i = c / 3, j = c - 3 * i;                  // rank-2 output component (i, j)
    const int j1 = (j + 1) % 3, j2 = (j + 2) % 3;
    const int c1 = (c + 1) % 3, c2 = (c + 2) % 3;        // rank-1 output component c
    switch (label) {
        case 0: return {0, 0, 0, 0, 1, false};                       // 000: l r
        case 1: return {0, 1, 0, 1, 3, false};                       // 110: sum_x l_x r_x
        case 2: return {0, 1, 0, 1, 9, false};                       // 220: sum_xy l_xy r_xy
        case 3: return {0, 0, c, 0, 1, false};                       // 011: l r_c
        case 4: return {c, 0, 0, 0, 1, false};                       // 101: l_c r
        case 5: return {0, 1, 3 * c, 1, 3, false};                   // 121: sum_x l_x r_cx
        case 6: return {3 * c, 1, 0, 1, 3, false};                   // 211: sum_y l_cy r_y
        case 7: return {0, 0, c, 0, 1, false};                       // 022: l r_c
        case 8: return {c, 0, 0, 0, 1, false};                       // 202: l_c r
        case 9: return {i, 0, j, 0, 1, false};                       // 112: l_i r_j
        case 10: return {3 * i, 1, 3 * j, 1, 3, false};              // 222: sum_y l_iy r_jy
        case 11: return {c1, c2 - c1, c2, c1 - c2, 2, true};         // 111: l_c1 r_c2 - l_c2 r_c1
        default: return {3 * i + j1, j2 - j1, j2, j1 - j2, 2, true}; // 212: l_ij1 r_j2 - l_ij2 r_j1
    }
}

constexpr int kMaxNT = 4;   // 32-channel column blocks per workgroup (dim_o <= 128 per grid row)

template <int RANK_O>
__global__ void __launch_bounds__(256)
ant16_kernel(Terms terms, const float* __restrict__ x_0, const float* __restrict__ x_1, const float* __restrict__ x_2,
             long rows, int dim_0, int dim_1, int dim_2, int dim_l, int dim_o, int accumulate,
             float* __restrict__ y) {
    constexpr int CO = RANK_O == 0 ? 1 : (RANK_O == 1 ? 3 : 9);
    constexpr int BPT = 32 / CO;                         // rows per tile
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, kk = lane >> 5;
    const long b0 = (long)blockIdx.x * BPT;
    const int o_base = blockIdx.y * (32 * kMaxNT);
    const int nt = (dim_o - o_base + 31) / 32 < kMaxNT ? (dim_o - o_base + 31) / 32 : kMaxNT;   // column blocks here
    // this lane's A row: (row b0 + bl, component co)
    const int bl = m / CO, co = m - bl * CO;
    const bool row_ok = bl < BPT && b0 + bl < rows;

    // The four waves share the tile's rows and all its column blocks and split the contraction:
    // wave w takes the left channels i = w, w + 4, ...; an A value is built once and meets every
    // column block; the partial accumulators are summed through LDS at the end.
    floatx16 acc[kMaxNT];
#pragma unroll
    for (int t = 0; t < kMaxNT; t++)
#pragma unroll
        for (int q = 0; q < 16; q++) acc[t][q] = 0.f;

    for (int ti = 0; ti < terms.n; ti++) {
        const int label = terms.t[ti].label;
        const int rl = kRankL[label], rr = kRankR[label];
        const int CL = rl == 0 ? 1 : (rl == 1 ? 3 : 9), CR = rr == 0 ? 1 : (rr == 1 ? 3 : 9);
        const float* xr = rr == 0 ? x_0 : (rr == 1 ? x_1 : x_2);
        const int dim_r = rr == 0 ? dim_0 : (rr == 1 ? dim_1 : dim_2);
        const int lrow = dim_l * CL, xrow = dim_r * CR;  // floats per row of left / x
        float* ls = smem;                                // [BPT][dim_l][CL]
        float* xs = smem + BPT * lrow;                   // [BPT][dim_r][CR]
        __syncthreads();                                 // the previous type's tiles are consumed
        for (int t = tid; t < BPT * lrow; t += 256) {
            const int b = t / lrow;
            ls[t] = b0 + b < rows ? terms.t[ti].left[(b0 + b) * lrow + (t - b * lrow)] : 0.f;
        }
        for (int t = tid; t < BPT * xrow; t += 256) {
            const int b = t / xrow;
            xs[t] = b0 + b < rows ? xr[(b0 + b) * xrow + (t - b * xrow)] : 0.f;
        }
        __syncthreads();
        const Dot d = dot_of(label, co);
        const float* lrow_p = ls + (row_ok ? bl : 0) * lrow + d.lb;
        const float* xrow_p = xs + (row_ok ? bl : 0) * xrow + d.rb;
        // this lane's B columns (clamped for loads; columns past dim_o are never written)
        const float* Pn[kMaxNT];
#pragma unroll
        for (int t = 0; t < kMaxNT; t++) {
            int o = o_base + t * 32 + m;
            if (o >= dim_o) o = dim_o - 1;
            Pn[t] = terms.t[ti].P + (long)o * dim_l * dim_r;
        }
        for (int i = wave; i < dim_l; i += 4) {
            float lv[9];
#pragma unroll
            for (int t = 0; t < 9; t++) lv[t] = t < d.nt ? lrow_p[i * CL + t * d.ls] : 0.f;
            if (d.cross) lv[1] = -lv[1];
            // four K-steps per trip: all B values are requested before the first is consumed, so
            // the load latency is paid once per trip instead of once per matrix instruction
            for (int j0 = 0; j0 < dim_r; j0 += 8) {
                float bval[4][kMaxNT], aval[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int j = j0 + 2 * u + kk;
                    const bool j_ok = j < dim_r;
                    const int jc = j_ok ? j : dim_r - 1;
                    const long poff = (long)i * dim_r + jc;
#pragma unroll
                    for (int t = 0; t < kMaxNT; t++) bval[u][t] = (t < nt && j_ok) ? Pn[t][poff] : 0.f;
                    const float* rp = xrow_p + jc * CR;
                    float a = 0.f;
#pragma unroll
                    for (int t = 0; t < 9; t++)
                        if (t < d.nt) a = fmaf(lv[t], rp[t * d.rs], a);
                    aval[u] = (row_ok && j_ok) ? a : 0.f;
                }
#pragma unroll
                for (int u = 0; u < 4; u++)
#pragma unroll
                    for (int t = 0; t < kMaxNT; t++)
                        if (t < nt) acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(aval[u], bval[u][t], acc[t], 0, 0, 0);
            }
        }
    }
    // sum the four partial tiles: waves 1..3 park theirs in LDS (64 floats per (block, register): no conflicts)
    __syncthreads();
    float* red = smem;                                   // [3][kMaxNT][16][64]
    if (wave > 0) {
#pragma unroll
        for (int t = 0; t < kMaxNT; t++)
            if (t < nt)
#pragma unroll
                for (int q = 0; q < 16; q++) red[(((wave - 1) * kMaxNT + t) * 16 + q) * 64 + lane] = acc[t][q];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int t = 0; t < kMaxNT; t++) {
        if (t >= nt) break;
        const int o = o_base + t * 32 + m;
#pragma unroll
        for (int q = 0; q < 16; q++) {
            float v = acc[t][q];
#pragma unroll
            for (int w = 0; w < 3; w++) v += red[((w * kMaxNT + t) * 16 + q) * 64 + lane];
            const int mr = 8 * (q / 4) + 4 * kk + (q % 4);     // accumulator row -> (row, component)
            const int b = mr / CO, c = mr - b * CO;
            if (o < dim_o && b < BPT && b0 + b < rows) {
                float* p = y + ((b0 + b) * dim_o + o) * CO + c;
                *p = accumulate ? *p + v : v;
            }
        }
    }
}

__global__ void __launch_bounds__(256) fill_zero_kernel(float* __restrict__ y, long n) {
    for (long t = (long)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (long)gridDim.x * blockDim.x) y[t] = 0.f;
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_ant16_fwd(int rank_o, int n_terms, const int* labels, const float* const* P, const float* const* left,
                 const float* x_0, const float* x_1, const float* x_2, long rows, int dim_0, int dim_1, int dim_2,
                 int dim_l, int accumulate, float* y, mg_stream_t stream) {
    MG_REQUIRE(rank_o >= 0 && rank_o <= 2, "mg_ant16_fwd: rank_o must be 0, 1 or 2");
    MG_REQUIRE(n_terms >= 1 && n_terms <= kMaxTerms, "mg_ant16_fwd: between 1 and %d product types per call", kMaxTerms);
    MG_REQUIRE(rows >= 0 && dim_0 >= 0 && dim_1 >= 0 && dim_2 >= 0 && dim_l >= 0, "mg_ant16_fwd: negative size");
    MG_REQUIRE(labels && P && left, "mg_ant16_fwd: null table");
    const int dim_o = rank_o == 0 ? dim_0 : (rank_o == 1 ? dim_1 : dim_2);
    if (rows == 0 || dim_o == 0) return MG_OK;
    MG_REQUIRE(y != nullptr, "mg_ant16_fwd: null output");
    Terms terms{};
    const int CO = rank_o == 0 ? 1 : (rank_o == 1 ? 3 : 9);
    const int BPT = 32 / CO;
    size_t lds_floats = 0;
    for (int t = 0; t < n_terms; t++) {
        const int lab = labels[t];
        MG_REQUIRE(lab >= 0 && lab < 13, "mg_ant16_fwd: unknown product type %d", lab);
        MG_REQUIRE(h_rank_o[lab] == rank_o, "mg_ant16_fwd: product type %d does not have output rank %d", lab, rank_o);
        const int rr = h_rank_r[lab], rl = h_rank_l[lab];
        const int dim_r = rr == 0 ? dim_0 : (rr == 1 ? dim_1 : dim_2);
        if (dim_r == 0 || dim_l == 0) continue;            // an empty contraction adds nothing
        MG_REQUIRE(P[t] && left[t], "mg_ant16_fwd: null operand of term %d", t);
        MG_REQUIRE((rr == 0 ? x_0 : (rr == 1 ? x_1 : x_2)) != nullptr, "mg_ant16_fwd: null x of rank %d", rr);
        terms.t[terms.n].P = P[t];
        terms.t[terms.n].left = left[t];
        terms.t[terms.n].label = lab;
        terms.n++;
        const size_t CL = rl == 0 ? 1 : (rl == 1 ? 3 : 9), CR = rr == 0 ? 1 : (rr == 1 ? 3 : 9);
        const size_t need = (size_t)BPT * ((size_t)dim_l * CL + (size_t)dim_r * CR);
        if (need > lds_floats) lds_floats = need;
    }
    if (lds_floats < 3 * kMaxNT * 16 * 64) lds_floats = 3 * kMaxNT * 16 * 64;   // the final reduction reuses the tiles' space
    const size_t lds_bytes = lds_floats * sizeof(float);
    MG_REQUIRE(lds_bytes <= 160 * 1024, "mg_ant16_fwd: a tile of operands needs %zu bytes of LDS (limit 163840): "
               "channel counts too wide", lds_bytes);
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)ceil_div(rows, BPT), (unsigned)ceil_div(dim_o, 128));
    MG_REQUIRE(ceil_div(rows, BPT) <= 0x7fffffffL, "mg_ant16_fwd: too many rows");
    if (terms.n == 0) {
        if (!accumulate) {   // a kernel, not a memset node: callers may capture this launch into a graph
            const long total = rows * dim_o * CO;
            long blocks = ceil_div(total, 256);
            if (blocks > 4096) blocks = 4096;
            hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, st, y, total);
            return check_launch("mg_ant16_fwd");
        }
        return MG_OK;
    }
#define MG_ANT16_LAUNCH(R)                                                                                          \
    do {                                                                                                            \
        if (lds_bytes > 48 * 1024)                                                                                  \
            MG_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(ant16_kernel<R>),                              \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));                \
        hipLaunchKernelGGL(ant16_kernel<R>, grid, dim3(256), lds_bytes, st, terms, x_0, x_1, x_2, rows, dim_0,      \
                           dim_1, dim_2, dim_l, dim_o, accumulate, y);                                              \
    } while (0)
    if (rank_o == 0) MG_ANT16_LAUNCH(0);
    else if (rank_o == 1) MG_ANT16_LAUNCH(1);
    else MG_ANT16_LAUNCH(2);
#undef MG_ANT16_LAUNCH
    return check_launch("mg_ant16_fwd");
}

}  // extern "C"
