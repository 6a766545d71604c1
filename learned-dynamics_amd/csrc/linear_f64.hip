// y = act(x W^T + b) in float64 arithmetic: the weights are the float32 parameters, widened exactly; inputs,
// products, sums, activation and outputs are double.  Not a hot path: it is what decides whether an approximation of
// a float32 MLP (the PaiNN filter taken from a grid over the edge length) stays below a stated error, which cannot be
// measured through float32 GEMMs whose own rounding is of that size.
//
// Shape: a workgroup of 256 threads owns a 64 x 64 output tile, a thread 4 x 4 outputs; x and W go through LDS in
// chunks of 16 along the reduction, transposed so that a thread reads its 4 + 4 operands of a step as two 32-byte
// runs (rows padded by one double pair against bank conflicts).  Sums run in index order of the reduction: the result
// does not depend on the launch shape.
#include "common.hpp"

namespace {

constexpr int TILE = 64, KC = 16, PAD = 2;

__device__ __forceinline__ double act_f64(double z, int act) {
    if (act == 1) return z / (1.0 + exp(-z));            // SiLU
    if (act == 2) return z >= 0.0 ? z : 0.1 * z;         // LeakyReLU(0.1), as the per-edge MLPs of the rank-0/1/2 layers
    return z;
}

__global__ __launch_bounds__(256) void linear_f64_kernel(const float* __restrict__ W, const float* __restrict__ bias,
                                                         const double* __restrict__ x, long rows, int dim_in,
                                                         int dim_out, int act, double* __restrict__ y) {
    __shared__ double xs[KC][TILE + PAD];
    __shared__ double ws[KC][TILE + PAD];
    const int tid = threadIdx.x;
    const long row0 = (long)blockIdx.x * TILE;
    const int col0 = blockIdx.y * TILE;
    const int tr = (tid / 16) * 4, tc = (tid % 16) * 4;
    double acc[4][4] = {};
    for (int k0 = 0; k0 < dim_in; k0 += KC) {
        // 64 rows x 16 k of each operand: thread -> (row = tid / 4, four consecutive k)
        const int lr = tid / 4, lk = (tid % 4) * 4;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int k = k0 + lk + q;
            const long r = row0 + lr;
            const int c = col0 + lr;
            xs[lk + q][lr] = (r < rows && k < dim_in) ? x[r * dim_in + k] : 0.0;
            ws[lk + q][lr] = (c < dim_out && k < dim_in) ? (double)W[(long)c * dim_in + k] : 0.0;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < KC; ++k) {
            double a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = xs[k][tr + i]; b[i] = ws[k][tc + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fma(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const long r = row0 + tr + i;
        if (r >= rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = col0 + tc + j;
            if (c < dim_out) y[r * dim_out + c] = act_f64(acc[i][j] + (bias ? (double)bias[c] : 0.0), act);
        }
    }
}

}  // namespace

extern "C" int mg_linear_f64(const float* W, const float* bias, const double* x, long rows, int dim_in, int dim_out,
                             int act, double* y, mg_stream_t stream) {
    MG_REQUIRE(rows >= 0 && dim_in > 0 && dim_out > 0, "mg_linear_f64: bad size");
    MG_REQUIRE(act >= 0 && act <= 2, "mg_linear_f64: unknown activation %d", act);
    if (rows == 0) return MG_OK;
    MG_REQUIRE(W && x && y, "mg_linear_f64: null pointer");
    const long row_tiles = mg::ceil_div(rows, TILE);
    MG_REQUIRE(row_tiles < (1L << 31), "mg_linear_f64: too many rows");
    dim3 grid((unsigned)row_tiles, (unsigned)mg::ceil_div(dim_out, TILE));
    MG_REQUIRE(grid.y < 65536, "mg_linear_f64: dim_out too large");
    hipLaunchKernelGGL(linear_f64_kernel, grid, dim3(256), 0, (hipStream_t)stream, W, bias, x, rows, dim_in, dim_out, act,
                       y);
    return mg::check_launch("mg_linear_f64");
}
