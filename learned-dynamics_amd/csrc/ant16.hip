// Ant16: y_o[b, o, :] = sum over product types (l r o) of sum_{i < dim_l, j < dim_r}
//            P_lro[o, i, j] * (left_lro[b, i, :] (x) x_r[b, j, :])     (the 13 Cartesian products)
// (managan/codegen_tensor_products.py:19-34; kernels extensions/codegen_tensops/codegen_tensops_kern.cu:1341-1448)
// and its three gradients (codegen_tensops.cpp:669-821, 892-1070, 1142-1325, 1374-1517).
//
// The forward and the gradients for x and left are one dense contraction per product type over two
// of the three channel axes of P, between two per-row operands U and V:
//     forward   (mode 0)  y[b, o, O]  = sum_{i, j} P[o, i, j] * C_O(left[b, i, :], x[b, j, :])       U = left, V = x
//     grad x    (mode 1)  dx[b, j, X] = sum_{i, o} P[o, i, j] * C_X(left[b, i, :], dy[b, o, :])      U = left, V = dy
//     grad left (mode 2)  dl[b, i, L] = sum_{j, o} P[o, i, j] * C_L(x[b, j, :],    dy[b, o, :])      U = x,    V = dy
// with K = dim_u * dim_v, M = (row, output component), N = the remaining channel axis of P.  The A
// operand is never stored: every lane builds its value
//     A[(b, c), (u, v)] = C_c(U[b, u, :], V[b, v, :]) = sum_t sign_t U[b, u, a_t] V[b, v, b_t]
// (at most nine terms, listed per mode, type and component in the generated ant16_coupling.inc) from a
// few LDS reads right before the fp32 matrix instruction (v_mfma_f32_32x32x2_f32: exact fp32 products),
// and P is read in place through the strides of its (u, v, n) axes.  A workgroup owns the rows of one
// tile (32, 10 or 3 rows for output rank 0, 1, 2: 32 = rows x components, rounded down to whole rows)
// and up to four 32-channel column blocks; its four waves split the contraction over u, so an A value
// is built once and meets every column block; operands of the tile are staged in LDS per product type
// and the partial accumulators are summed through LDS.
//
// The weight gradient dP[o, i, j] = sum_{b, O} dy[b, o, O] * C_O(left[b, i, :], x[b, j, :]) is a
// contraction over rows: M = o, N = (i, j), K = (row, component); the rows are split over workgroups,
// each writes its partial tile to its own plane of a workspace, and a second kernel adds the planes in
// order (no atomics: the result does not depend on the order in which workgroups finish).
#include "common.hpp"

namespace mg {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

#include "ant16_coupling.inc"

struct Term {
    const float* P;      // (dim_o, dim_l, dim_r)
    const float* U;      // (rows, dim_u, cu)
    const float* V;      // (rows, dim_v, cv)
    long su, sv, sn;     // strides of P along u, v and the output channel
    int label;           // index into the label order below
    int dim_u, dim_v, cu, cv;
    int max_terms;       // most terms of any output component of this mode and type
};
constexpr int kMaxTerms = 6;
struct Terms {
    int n;
    Term t[kMaxTerms];
};

// label order: 000 110 220 011 101 121 211 022 202 112 222 111 212
constexpr int h_rank_l[13] = {0, 1, 2, 0, 1, 1, 2, 0, 2, 1, 2, 1, 2};
constexpr int h_rank_r[13] = {0, 1, 2, 1, 0, 2, 1, 2, 0, 1, 2, 1, 1};
constexpr int h_rank_o[13] = {0, 0, 0, 1, 1, 1, 1, 2, 2, 2, 2, 1, 2};
constexpr int comps(int rank) { return rank == 0 ? 1 : (rank == 1 ? 3 : 9); }

constexpr int kMaxNT = 4;   // 32-channel column blocks per workgroup (128 output channels per grid row)

template <int RANK_N>
__global__ void __launch_bounds__(256)
ant16_kernel(Terms terms, int mode, long rows, int dim_n, int accumulate, float* __restrict__ y) {
    constexpr int CO = comps(RANK_N);
    constexpr int BPT = 32 / CO;                         // rows per tile
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, kk = lane >> 5;
    const long b0 = (long)blockIdx.x * BPT;
    const int n_base = blockIdx.y * (32 * kMaxNT);
    const int nt = (dim_n - n_base + 31) / 32 < kMaxNT ? (dim_n - n_base + 31) / 32 : kMaxNT;   // column blocks here
    // this lane's A row: (row b0 + bl, component co)
    const int bl = m / CO, co = m - bl * CO;
    const bool row_ok = bl < BPT && b0 + bl < rows;

    // The four waves share the tile's rows and all its column blocks and split the contraction:
    // wave w takes u = w, w + 4, ...; an A value is built once and meets every column block;
    // the partial accumulators are summed through LDS at the end.
    floatx16 acc[kMaxNT];
#pragma unroll
    for (int t = 0; t < kMaxNT; t++)
#pragma unroll
        for (int q = 0; q < 16; q++) acc[t][q] = 0.f;

    for (int ti = 0; ti < terms.n; ti++) {
        const Term& T = terms.t[ti];
        const int urow = T.dim_u * T.cu, vrow = T.dim_v * T.cv;   // floats per row of U / V
        float* us = smem;                                // [BPT][dim_u][cu]
        float* vs = smem + BPT * urow;                   // [BPT][dim_v][cv]
        __syncthreads();                                 // the previous type's tiles are consumed
        for (int t = tid; t < BPT * urow; t += 256) {
            const int b = t / urow;
            us[t] = b0 + b < rows ? T.U[(b0 + b) * urow + (t - b * urow)] : 0.f;
        }
        for (int t = tid; t < BPT * vrow; t += 256) {
            const int b = t / vrow;
            vs[t] = b0 + b < rows ? T.V[(b0 + b) * vrow + (t - b * vrow)] : 0.f;
        }
        __syncthreads();
        // the terms of this lane's component
        const unsigned short* cp = &kCoupling[mode][T.label][co < CO ? co : 0][0];
        const int my_terms = cp[0];
        int ua[9], vb[9];
        float sg[9];
#pragma unroll
        for (int t = 0; t < 9; t++) {
            const int e = t < my_terms ? cp[1 + t] : 0;
            ua[t] = e & 15;
            vb[t] = (e >> 4) & 15;
            sg[t] = t < my_terms ? ((e & 256) ? -1.f : 1.f) : 0.f;
        }
        const float* urow_p = us + (row_ok ? bl : 0) * urow;
        const float* vrow_p = vs + (row_ok ? bl : 0) * vrow;
        // this lane's B columns (clamped for loads; columns past dim_n are never written)
        const float* Pn[kMaxNT];
#pragma unroll
        for (int t = 0; t < kMaxNT; t++) {
            int n = n_base + t * 32 + m;
            if (n >= dim_n) n = dim_n - 1;
            Pn[t] = T.P + (long)n * T.sn;
        }
        const int cu = T.cu, cv = T.cv, dim_v = T.dim_v, max_terms = T.max_terms;
        const long su = T.su, sv = T.sv;
        for (int u = wave; u < T.dim_u; u += 4) {
            float uv[9];
#pragma unroll
            for (int t = 0; t < 9; t++) uv[t] = t < max_terms ? sg[t] * urow_p[u * cu + ua[t]] : 0.f;
            // four K-steps per trip: all B values are requested before the first is consumed, so
            // the load latency is paid once per trip instead of once per matrix instruction
            for (int v0 = 0; v0 < dim_v; v0 += 8) {
                float bval[4][kMaxNT], aval[4];
#pragma unroll
                for (int s = 0; s < 4; s++) {
                    const int v = v0 + 2 * s + kk;
                    const bool v_ok = v < dim_v;
                    const int vc = v_ok ? v : dim_v - 1;
                    const long poff = (long)u * su + (long)vc * sv;
#pragma unroll
                    for (int t = 0; t < kMaxNT; t++) bval[s][t] = (t < nt && v_ok) ? Pn[t][poff] : 0.f;
                    const float* rp = vrow_p + vc * cv;
                    float a = 0.f;
#pragma unroll
                    for (int t = 0; t < 9; t++)
                        if (t < max_terms) a = fmaf(uv[t], rp[vb[t]], a);
                    aval[s] = (row_ok && v_ok) ? a : 0.f;
                }
#pragma unroll
                for (int s = 0; s < 4; s++)
#pragma unroll
                    for (int t = 0; t < kMaxNT; t++)
                        if (t < nt) acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(aval[s], bval[s][t], acc[t], 0, 0, 0);
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
        const int n = n_base + t * 32 + m;
#pragma unroll
        for (int q = 0; q < 16; q++) {
            float v = acc[t][q];
#pragma unroll
            for (int w = 0; w < 3; w++) v += red[((w * kMaxNT + t) * 16 + q) * 64 + lane];
            const int mr = 8 * (q / 4) + 4 * kk + (q % 4);     // accumulator row -> (row, component)
            const int b = mr / CO, c = mr - b * CO;
            if (n < dim_n && b < BPT && b0 + b < rows) {
                float* p = y + ((b0 + b) * dim_n + n) * CO + c;
                *p = accumulate ? *p + v : v;
            }
        }
    }
}

__global__ void __launch_bounds__(256) fill_zero_kernel(float* __restrict__ y, long n) {
    for (long t = (long)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (long)gridDim.x * blockDim.x) y[t] = 0.f;
}

int launch_fill_zero(float* y, long n, hipStream_t st, const char* what) {
    long blocks = ceil_div(n, 256);
    if (blocks > 4096) blocks = 4096;
    if (blocks < 1) return MG_OK;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, st, y, n);
    return check_launch(what);
}

// Shared by the forward and the two per-row gradients.  U[t] / V[t] are the row operands of term t
// (left / x, left / dy or x / dy by mode); the output has rank rank_n and dim_n channels.
int launch_contraction(const char* what, int mode, int rank_n, int n_terms, const int* labels, const float* const* P,
                       const float* const* U, const float* const* V, long rows, const int dims[3], int dim_l,
                       int accumulate, float* y, hipStream_t st) {
    MG_REQUIRE(rank_n >= 0 && rank_n <= 2, "%s: the output rank must be 0, 1 or 2", what);
    MG_REQUIRE(n_terms >= 1 && n_terms <= kMaxTerms, "%s: between 1 and %d product types per call", what, kMaxTerms);
    MG_REQUIRE(rows >= 0 && dims[0] >= 0 && dims[1] >= 0 && dims[2] >= 0 && dim_l >= 0, "%s: negative size", what);
    MG_REQUIRE(labels && P && U && V, "%s: null table", what);
    const int dim_n = mode == 2 ? dim_l : dims[rank_n];
    if (rows == 0 || dim_n == 0) return MG_OK;
    MG_REQUIRE(y != nullptr, "%s: null output", what);
    Terms terms{};
    const int CO = comps(rank_n);
    const int BPT = 32 / CO;
    size_t lds_floats = 0;
    for (int t = 0; t < n_terms; t++) {
        const int lab = labels[t];
        MG_REQUIRE(lab >= 0 && lab < 13, "%s: unknown product type %d", what, lab);
        const int rl = h_rank_l[lab], rr = h_rank_r[lab], ro = h_rank_o[lab];
        const int rank_here = mode == 0 ? ro : (mode == 1 ? rr : rl);
        MG_REQUIRE(rank_here == rank_n, "%s: product type %d does not produce rank %d here", what, lab, rank_n);
        const int dim_r = dims[rr], dim_o = dims[ro];
        if (dim_r == 0 || dim_l == 0 || dim_o == 0) continue;   // an empty contraction adds nothing
        MG_REQUIRE(P[t] && U[t] && V[t], "%s: null operand of term %d", what, t);
        Term& T = terms.t[terms.n++];
        T.P = P[t];
        T.U = U[t];
        T.V = V[t];
        T.label = lab;
        T.max_terms = kCouplingMaxTerms[mode][lab];
        const long lr = (long)dim_l * dim_r;
        if (mode == 0)      { T.dim_u = dim_l; T.cu = comps(rl); T.dim_v = dim_r; T.cv = comps(rr); T.su = dim_r; T.sv = 1;  T.sn = lr; }
        else if (mode == 1) { T.dim_u = dim_l; T.cu = comps(rl); T.dim_v = dim_o; T.cv = comps(ro); T.su = dim_r; T.sv = lr; T.sn = 1; }
        else                { T.dim_u = dim_r; T.cu = comps(rr); T.dim_v = dim_o; T.cv = comps(ro); T.su = 1;     T.sv = lr; T.sn = dim_r; }
        const size_t need = (size_t)BPT * ((size_t)T.dim_u * T.cu + (size_t)T.dim_v * T.cv);
        if (need > lds_floats) lds_floats = need;
    }
    if (lds_floats < 3 * kMaxNT * 16 * 64) lds_floats = 3 * kMaxNT * 16 * 64;   // the final reduction reuses the tiles' space
    const size_t lds_bytes = lds_floats * sizeof(float);
    MG_REQUIRE(lds_bytes <= 160 * 1024, "%s: a tile of operands needs %zu bytes of LDS (limit 163840): "
               "channel counts too wide", what, lds_bytes);
    MG_REQUIRE(ceil_div(rows, BPT) <= 0x7fffffffL, "%s: too many rows", what);
    const dim3 grid((unsigned)ceil_div(rows, BPT), (unsigned)ceil_div(dim_n, 32 * kMaxNT));
    if (terms.n == 0)   // a kernel, not a memset node: callers may capture this launch into a graph
        return accumulate ? MG_OK : launch_fill_zero(y, rows * dim_n * CO, st, what);
#define MG_ANT16_LAUNCH(R)                                                                                          \
    do {                                                                                                            \
        if (lds_bytes > 48 * 1024)                                                                                  \
            MG_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(ant16_kernel<R>),                              \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));                \
        hipLaunchKernelGGL(ant16_kernel<R>, grid, dim3(256), lds_bytes, st, terms, mode, rows, dim_n, accumulate, y); \
    } while (0)
    if (rank_n == 0) MG_ANT16_LAUNCH(0);
    else if (rank_n == 1) MG_ANT16_LAUNCH(1);
    else MG_ANT16_LAUNCH(2);
#undef MG_ANT16_LAUNCH
    return check_launch(what);
}

// ---------------------------------------------------------------------------------------------------
// weight gradient

constexpr int kWgRows = 4;          // rows staged per step

__global__ void __launch_bounds__(256)
ant16_wgrad_kernel(const float* __restrict__ left, const float* __restrict__ x, const float* __restrict__ dy, int label,
                   long rows, int dim_l, int dim_r, int dim_o, int cl, int cr, int co, int max_terms,
                   long rows_per_block, float* __restrict__ part) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    __shared__ unsigned short coupling[9][10];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, kk = lane >> 5;
    const long pairs = (long)dim_l * dim_r;
    const long n = (long)blockIdx.x * 128 + wave * 32 + m;        // this lane's B column: the pair (i, j)
    const bool n_ok = n < pairs;
    const int i = n_ok ? (int)(n / dim_r) : 0, j = n_ok ? (int)(n - (long)i * dim_r) : 0;
    const int o_base = blockIdx.y * (32 * kMaxNT);
    const int ow = dim_o - o_base < 32 * kMaxNT ? dim_o - o_base : 32 * kMaxNT;   // output channels of this workgroup
    const int nt = (ow + 31) / 32;
    const int lrow = dim_l * cl, xrow = dim_r * cr, yrow = ow * co;
    float* ls = smem;                         // [kWgRows][dim_l][cl]
    float* xs = ls + kWgRows * lrow;          // [kWgRows][dim_r][cr]
    float* ys = xs + kWgRows * xrow;          // [kWgRows][ow][co]
    if (tid < 90) coupling[tid / 10][tid % 10] = kCoupling[0][label][tid / 10][tid % 10];
    const long r_lo = (long)blockIdx.z * rows_per_block;
    const long r_hi = r_lo + rows_per_block < rows ? r_lo + rows_per_block : rows;
    floatx16 acc[kMaxNT];
#pragma unroll
    for (int t = 0; t < kMaxNT; t++)
#pragma unroll
        for (int q = 0; q < 16; q++) acc[t][q] = 0.f;

    for (long r0 = r_lo; r0 < r_hi; r0 += kWgRows) {
        __syncthreads();
        for (int t = tid; t < kWgRows * lrow; t += 256) {
            const int b = t / lrow;
            ls[t] = r0 + b < r_hi ? left[(r0 + b) * lrow + (t - b * lrow)] : 0.f;
        }
        for (int t = tid; t < kWgRows * xrow; t += 256) {
            const int b = t / xrow;
            xs[t] = r0 + b < r_hi ? x[(r0 + b) * xrow + (t - b * xrow)] : 0.f;
        }
        for (int t = tid; t < kWgRows * yrow; t += 256) {
            const int b = t / yrow;
            ys[t] = r0 + b < r_hi ? dy[((r0 + b) * dim_o + o_base) * co + (t - b * yrow)] : 0.f;
        }
        __syncthreads();
        for (int b = 0; b < kWgRows; b++) {
            const float* lp = ls + b * lrow + i * cl;
            const float* xp = xs + b * xrow + j * cr;
            const float* yp = ys + b * yrow;
            for (int c0 = 0; c0 < co; c0 += 2) {
                const int c = c0 + kk;
                const bool c_ok = c < co;
                const unsigned short* cp = coupling[c_ok ? c : 0];
                float bv = 0.f;
                for (int t = 0; t < max_terms; t++) {
                    const int e = cp[1 + t];
                    const float s = t < cp[0] ? ((e & 256) ? -1.f : 1.f) : 0.f;
                    bv = fmaf(s * lp[e & 15], xp[(e >> 4) & 15], bv);
                }
                bv = (c_ok && n_ok) ? bv : 0.f;
#pragma unroll
                for (int t = 0; t < kMaxNT; t++) {
                    if (t >= nt) break;
                    const int ol = t * 32 + m;                      // A row: output channel o_base + ol
                    const float av = (c_ok && ol < ow) ? yp[ol * co + c] : 0.f;
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[t], 0, 0, 0);
                }
            }
        }
    }
    float* plane = part + (long)blockIdx.z * dim_o * pairs;
#pragma unroll
    for (int t = 0; t < kMaxNT; t++) {
        if (t >= nt) break;
#pragma unroll
        for (int q = 0; q < 16; q++) {
            const int o = o_base + t * 32 + 8 * (q / 4) + 4 * kk + (q % 4);
            if (o < dim_o && n_ok) plane[(long)o * pairs + n] = acc[t][q];
        }
    }
}

// dP[k] = part[0][k] + part[1][k] + ... in this order
__global__ void __launch_bounds__(256) planes_sum_kernel(const float* __restrict__ part, long n, int splits,
                                                         float* __restrict__ out) {
    for (long k = (long)blockIdx.x * blockDim.x + threadIdx.x; k < n; k += (long)gridDim.x * blockDim.x) {
        float s = 0.f;
        int z = 0;
        for (; z + 8 <= splits; z += 8) {                  // eight loads in flight, added in slice order
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = part[(long)(z + u) * n + k];
#pragma unroll
            for (int u = 0; u < 8; u++) s += v[u];
        }
        for (; z < splits; z++) s += part[(long)z * n + k];
        out[k] = s;
    }
}

// rows per slice and number of slices (the same on the sizing and the launching side)
void wgrad_split(long rows, int dim_o, int dim_l, int dim_r, long* rows_per_block, long* splits) {
    const long tiles = ceil_div((long)dim_l * dim_r, 128) * ceil_div(dim_o, 32 * kMaxNT);
    long s = ceil_div(1024, tiles > 0 ? tiles : 1);     // aim at ~4 workgroups per CU
    const long max_splits = ceil_div(rows, 64);
    if (s > max_splits) s = max_splits;
    if (s < 1) s = 1;
    if (s > 65535) s = 65535;
    long rpb = ceil_div(rows, s);
    rpb = ceil_div(rpb, kWgRows) * kWgRows;
    *rows_per_block = rpb;
    *splits = rows > 0 ? ceil_div(rows, rpb) : 0;
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_ant16_fwd(int rank_o, int n_terms, const int* labels, const float* const* P, const float* const* left,
                 const float* x_0, const float* x_1, const float* x_2, long rows, int dim_0, int dim_1, int dim_2,
                 int dim_l, int accumulate, float* y, mg_stream_t stream) {
    MG_REQUIRE(n_terms >= 1 && n_terms <= kMaxTerms && labels, "mg_ant16_fwd: between 1 and %d product types per call", kMaxTerms);
    const float* xs[3] = {x_0, x_1, x_2};
    const float* V[kMaxTerms];
    for (int t = 0; t < n_terms; t++) {
        MG_REQUIRE(labels[t] >= 0 && labels[t] < 13, "mg_ant16_fwd: unknown product type %d", labels[t]);
        V[t] = xs[h_rank_r[labels[t]]];
    }
    const int dims[3] = {dim_0, dim_1, dim_2};
    return launch_contraction("mg_ant16_fwd", 0, rank_o, n_terms, labels, P, left, V, rows, dims, dim_l, accumulate, y,
                              (hipStream_t)stream);
}

int mg_ant16_grad_x(int rank_r, int n_terms, const int* labels, const float* const* P, const float* const* left,
                    const float* dy_0, const float* dy_1, const float* dy_2, long rows, int dim_0, int dim_1, int dim_2,
                    int dim_l, int accumulate, float* dx, mg_stream_t stream) {
    MG_REQUIRE(n_terms >= 1 && n_terms <= kMaxTerms && labels, "mg_ant16_grad_x: between 1 and %d product types per call", kMaxTerms);
    const float* dys[3] = {dy_0, dy_1, dy_2};
    const float* V[kMaxTerms];
    for (int t = 0; t < n_terms; t++) {
        MG_REQUIRE(labels[t] >= 0 && labels[t] < 13, "mg_ant16_grad_x: unknown product type %d", labels[t]);
        V[t] = dys[h_rank_o[labels[t]]];
    }
    const int dims[3] = {dim_0, dim_1, dim_2};
    return launch_contraction("mg_ant16_grad_x", 1, rank_r, n_terms, labels, P, left, V, rows, dims, dim_l, accumulate, dx,
                              (hipStream_t)stream);
}

int mg_ant16_grad_left(int label, const float* P, const float* x, const float* dy, long rows, int dim_0, int dim_1,
                       int dim_2, int dim_l, float* dleft, mg_stream_t stream) {
    MG_REQUIRE(label >= 0 && label < 13, "mg_ant16_grad_left: unknown product type %d", label);
    const int dims[3] = {dim_0, dim_1, dim_2};
    return launch_contraction("mg_ant16_grad_left", 2, h_rank_l[label], 1, &label, &P, &x, &dy, rows, dims, dim_l, 0, dleft,
                              (hipStream_t)stream);
}

int mg_ant16_grad_weight_workspace_bytes(long rows, int dim_o, int dim_l, int dim_r, size_t* bytes) {
    MG_REQUIRE(bytes != nullptr && rows >= 0 && dim_o >= 0 && dim_l >= 0 && dim_r >= 0,
               "mg_ant16_grad_weight_workspace_bytes: bad argument");
    long rpb, splits;
    wgrad_split(rows, dim_o, dim_l, dim_r, &rpb, &splits);
    *bytes = (size_t)splits * (size_t)dim_o * (size_t)dim_l * (size_t)dim_r * sizeof(float) + 16;
    return MG_OK;
}

int mg_ant16_grad_weight(int label, const float* left, const float* x, const float* dy, long rows, int dim_0, int dim_1,
                         int dim_2, int dim_l, void* workspace, float* dP, mg_stream_t stream) {
    MG_REQUIRE(label >= 0 && label < 13, "mg_ant16_grad_weight: unknown product type %d", label);
    MG_REQUIRE(rows >= 0 && dim_0 >= 0 && dim_1 >= 0 && dim_2 >= 0 && dim_l >= 0, "mg_ant16_grad_weight: negative size");
    const int dims[3] = {dim_0, dim_1, dim_2};
    const int rl = h_rank_l[label], rr = h_rank_r[label], ro = h_rank_o[label];
    const int dim_r = dims[rr], dim_o = dims[ro];
    const long total = (long)dim_o * dim_l * dim_r;
    if (total == 0) return MG_OK;
    MG_REQUIRE(dP != nullptr, "mg_ant16_grad_weight: dP is null");
    hipStream_t st = (hipStream_t)stream;
    if (rows == 0) return launch_fill_zero(dP, total, st, "mg_ant16_grad_weight");
    MG_REQUIRE(left && x && dy && workspace, "mg_ant16_grad_weight: null pointer");
    long rpb, splits;
    wgrad_split(rows, dim_o, dim_l, dim_r, &rpb, &splits);
    const int cl = comps(rl), cr = comps(rr), co = comps(ro);
    const int ow = dim_o < 32 * kMaxNT ? dim_o : 32 * kMaxNT;
    const size_t lds_bytes = sizeof(float) * kWgRows * ((size_t)dim_l * cl + (size_t)dim_r * cr + (size_t)ow * co);
    MG_REQUIRE(lds_bytes <= 150 * 1024, "mg_ant16_grad_weight: a tile of operands needs %zu bytes of LDS: channel counts "
               "too wide", lds_bytes);
    const long gx = ceil_div((long)dim_l * dim_r, 128);
    MG_REQUIRE(gx <= 0x7fffffffL, "mg_ant16_grad_weight: P too large");
    float* part = reinterpret_cast<float*>((reinterpret_cast<uintptr_t>(workspace) + 15) & ~uintptr_t(15));
    if (lds_bytes > 48 * 1024)
        MG_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(ant16_wgrad_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    hipLaunchKernelGGL(ant16_wgrad_kernel, dim3((unsigned)gx, (unsigned)ceil_div(dim_o, 32 * kMaxNT), (unsigned)splits),
                       dim3(256), lds_bytes, st, left, x, dy, label, rows, dim_l, dim_r, dim_o, cl, cr, co,
                       kCouplingMaxTerms[0][label], rpb, part);
    const long blocks = ceil_div(total, 256) < 1024 ? ceil_div(total, 256) : 1024;
    hipLaunchKernelGGL(planes_sum_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const float*)part, total, (int)splits, dP);
    return check_launch("mg_ant16_grad_weight");
}

}  // extern "C"
