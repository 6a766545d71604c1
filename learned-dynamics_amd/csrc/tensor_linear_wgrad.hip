// Weight gradient of the channel-mixing linear:
//   dW[o, i] = sum_{r, t} dy[r, o, t] x[r, i, t]
// A GEMM whose reduction dimension (rows x components) is the long one, so the
// rows are split over workgroups (split-K); each workgroup reduces its slice
// for one 64x64 tile of dW in registers and writes it to its own plane of a
// workspace; a second kernel adds the planes in slice order.  No atomics: the
// result does not depend on the order in which workgroups finish.
// Training-side helper: not on the inference hot path and not tuned.
#include "common.hpp"

namespace mg {
namespace {

constexpr int kTile = 64;      // dW tile edge
constexpr int kRowsPerStep = 4;

__global__ void __launch_bounds__(256) zero_f32_kernel(float* __restrict__ p, long n) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) p[i] = 0.f;
}

template <int T>
__global__ void __launch_bounds__(256) wgrad_kernel(const float* __restrict__ dy, const float* __restrict__ x, long R,
                                                    int I, int O, long rows_per_block, float* __restrict__ part) {
    __shared__ float dys[kRowsPerStep * T][kTile + 1];
    __shared__ float xs[kRowsPerStep * T][kTile + 1];
    const int o0 = blockIdx.x * kTile, i0 = blockIdx.y * kTile;
    const long r_lo = (long)blockIdx.z * rows_per_block;
    const long r_hi = r_lo + rows_per_block < R ? r_lo + rows_per_block : R;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;   // tx -> i, ty -> o
    float acc[4][4] = {};
    for (long r = r_lo; r < r_hi; r += kRowsPerStep) {
        __syncthreads();
        for (int idx = threadIdx.x; idx < kRowsPerStep * kTile * T; idx += 256) {
            const int rr = idx / (kTile * T), rem = idx % (kTile * T), c = rem / T, t = rem % T;
            const bool row_ok = r + rr < r_hi;
            dys[rr * T + t][c] = (row_ok && o0 + c < O) ? dy[((r + rr) * O + o0 + c) * T + t] : 0.f;
            xs[rr * T + t][c] = (row_ok && i0 + c < I) ? x[((r + rr) * I + i0 + c) * T + t] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < kRowsPerStep * T; k++) {
            float a[4], b[4];
#pragma unroll
            for (int q = 0; q < 4; q++) { a[q] = dys[k][ty + 16 * q]; b[q] = xs[k][tx + 16 * q]; }
#pragma unroll
            for (int p = 0; p < 4; p++)
#pragma unroll
                for (int q = 0; q < 4; q++) acc[p][q] += a[p] * b[q];
        }
    }
#pragma unroll
    for (int p = 0; p < 4; p++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int o = o0 + ty + 16 * p, i = i0 + tx + 16 * q;
            if (o < O && i < I) part[((long)blockIdx.z * O + o) * I + i] = acc[p][q];
        }
}

// dW[k] = part[0][k] + part[1][k] + ... in this order
__global__ void __launch_bounds__(256) wgrad_reduce_kernel(const float* __restrict__ part, long n, int splits,
                                                           float* __restrict__ dW) {
    for (long k = (long)blockIdx.x * blockDim.x + threadIdx.x; k < n; k += (long)gridDim.x * blockDim.x) {
        float s = 0.f;
        for (int z = 0; z < splits; z++) s += part[(long)z * n + k];
        dW[k] = s;
    }
}

// rows per slice and number of slices for a problem (the same on the sizing and the launching side)
void wgrad_split(long rows, int dim_in, int dim_out, long* rows_per_block, long* splits) {
    const int gx = (int)ceil_div(dim_out, kTile), gy = (int)ceil_div(dim_in, kTile);
    long s = ceil_div(1024, (long)gx * gy);             // aim at ~4 workgroups per CU
    const long max_splits = ceil_div(rows, 64);
    if (s > max_splits) s = max_splits;
    if (s < 1) s = 1;
    if (s > 65535) s = 65535;
    long rpb = ceil_div(rows, s);
    rpb = ceil_div(rpb, kRowsPerStep) * kRowsPerStep;
    *rows_per_block = rpb;
    *splits = rows > 0 ? ceil_div(rows, rpb) : 0;
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_tensor_linear_wgrad_workspace_bytes(long rows, int dim_in, int dim_out, size_t* bytes) {
    MG_REQUIRE(bytes != nullptr && rows >= 0 && dim_in >= 0 && dim_out >= 0, "mg_tensor_linear_wgrad_workspace_bytes: bad argument");
    long rpb, splits;
    wgrad_split(rows, dim_in, dim_out, &rpb, &splits);
    *bytes = (size_t)splits * (size_t)dim_in * (size_t)dim_out * sizeof(float) + 16;
    return MG_OK;
}

int mg_tensor_linear_wgrad(int inds, const float* dy, const float* x, long rows, int dim_in, int dim_out,
                           void* workspace, float* dW, mg_stream_t stream) {
    if (inds < 0 || inds > 2)
        return fail(MG_ERR_UNSUPPORTED, "tensor_linear currently only supports a number of indices up to 2.");
    MG_REQUIRE(rows >= 0 && dim_in >= 0 && dim_out >= 0, "mg_tensor_linear_wgrad: negative size");
    const long n = (long)dim_in * dim_out;
    if (n == 0) return MG_OK;
    MG_REQUIRE(dW != nullptr, "mg_tensor_linear_wgrad: dW is null");
    hipStream_t st = (hipStream_t)stream;
    const unsigned nblocks = (unsigned)(ceil_div(n, 256) < 1024 ? ceil_div(n, 256) : 1024);
    if (rows == 0) {
        hipLaunchKernelGGL(zero_f32_kernel, dim3(nblocks), dim3(256), 0, st, dW, n);
        return check_launch("mg_tensor_linear_wgrad");
    }
    MG_REQUIRE(dy && x && workspace, "mg_tensor_linear_wgrad: null pointer");
    long rpb, splits;
    wgrad_split(rows, dim_in, dim_out, &rpb, &splits);
    float* part = reinterpret_cast<float*>((reinterpret_cast<uintptr_t>(workspace) + 15) & ~uintptr_t(15));
    const int gx = (int)ceil_div(dim_out, kTile), gy = (int)ceil_div(dim_in, kTile);
    dim3 grid(gx, gy, (unsigned)splits), block(256);
    switch (inds) {
        case 0: hipLaunchKernelGGL(wgrad_kernel<1>, grid, block, 0, st, dy, x, rows, dim_in, dim_out, rpb, part); break;
        case 1: hipLaunchKernelGGL(wgrad_kernel<3>, grid, block, 0, st, dy, x, rows, dim_in, dim_out, rpb, part); break;
        default: hipLaunchKernelGGL(wgrad_kernel<9>, grid, block, 0, st, dy, x, rows, dim_in, dim_out, rpb, part); break;
    }
    hipLaunchKernelGGL(wgrad_reduce_kernel, dim3(nblocks), dim3(256), 0, st, (const float*)part, n, (int)splits, dW);
    return check_launch("mg_tensor_linear_wgrad");
}

}  // extern "C"
