// TensGroupNorm (managan/tensor_products.py:215-232) on bf16 storage in the component-major layout of the bf16 stack:
// y (batch * nodes, T, chan), T = 1, 3 or 9 components,
//     out = gamma[c] * y / sqrt(eps + m2[b, g]) (+ res),   m2[b, g] = mean over (nodes, channels of group g) of sum_t y^2
// Statistics in fp32 per chunk of nodes and in double across chunks, in a fixed order (no atomics); three launches
// (statistics, scales, apply) that read y twice and write out once, all in 16-byte pieces along the channel axis.
// The same sequence written with tensor-library calls took a dozen launches with fp32 temporaries of the tensor's size.
#include "common.hpp"

namespace mg {
namespace {

constexpr int kGnNodesPerChunk = 32; // nodes per workgroup of the statistics pass (a thread then sums 32 values per column)
constexpr int kGnMaxChunks = 4096;
constexpr int kGnMaxWidth = 4608;   // T * chan floats of LDS per workgroup (9 x 512)

__device__ __forceinline__ float bf16_bits_to_float(unsigned short h) { return __builtin_bit_cast(float, (unsigned)h << 16); }

// partial[(b * chunks + chunk) * groups + g] = sum over the chunk's nodes, all components and the group's channels of y^2
__global__ void __launch_bounds__(256) gn_stats_bf16_kernel(const unsigned short* __restrict__ y, int N, int T, int chan,
                                                            int groups, int chunks, double* __restrict__ partial) {
    __shared__ float col[kGnMaxWidth];
    const int chunk = blockIdx.x, b = blockIdx.y;
    const int W = T * chan, cg = chan / groups;
    const int per = (N + chunks - 1) / chunks;
    const int n_lo = chunk * per, n_hi = n_lo + per < N ? n_lo + per : N;
    for (int p = threadIdx.x; p < W; p += blockDim.x) {
        float acc = 0.f;
        const unsigned short* col_p = y + ((long)b * N + n_lo) * W + p;
        for (int i = n_lo; i < n_hi; i++, col_p += W) {
            const float v = bf16_bits_to_float(*col_p);
            acc += v * v;
        }
        col[p] = acc;
    }
    __syncthreads();
    if ((int)threadIdx.x < groups) {
        const int g = threadIdx.x;
        double s = 0.0;
        for (int t = 0; t < T; t++)
            for (int c = g * cg; c < (g + 1) * cg; c++) s += col[t * chan + c];
        partial[((long)b * chunks + chunk) * groups + g] = s;
    }
}

// scale[b * groups + g] = 1 / sqrt(eps + total / (N * cg)); one workgroup per (box, group) folds the chunks in a fixed order
__global__ void __launch_bounds__(256) gn_scales_kernel(const double* __restrict__ partial, int groups, int chunks,
                                                        double count, float eps, float* __restrict__ scale) {
    __shared__ double fold[256];
    const int bg = blockIdx.x, b = bg / groups, g = bg - b * groups;
    double s = 0.0;
    for (int k = threadIdx.x; k < chunks; k += blockDim.x) s += partial[((long)b * chunks + k) * groups + g];
    fold[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) fold[threadIdx.x] += fold[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) scale[bg] = (float)(1.0 / sqrt((double)eps + fold[0] / count));
}

// eight consecutive channels per thread
__global__ void __launch_bounds__(256) gn_apply_bf16_kernel(const unsigned short* __restrict__ y,
                                                            const unsigned short* __restrict__ res,
                                                            const float* __restrict__ scale, const float* __restrict__ gamma,
                                                            long rows, int N, int T, int chan, int groups,
                                                            unsigned short* __restrict__ out) {
    typedef unsigned short ushort8 __attribute__((ext_vector_type(8)));
    const long W = (long)T * chan;
    const long vecs = rows * W / 8;
    const int cg = chan / groups;
    for (long v = (long)blockIdx.x * blockDim.x + threadIdx.x; v < vecs; v += (long)gridDim.x * blockDim.x) {
        const long e0 = 8 * v;
        const long row = e0 / W;
        const int c0 = (int)((e0 - row * W) % chan);
        const int b = (int)(row / N);
        const ushort8 in = *reinterpret_cast<const ushort8*>(y + e0);
        ushort8 r8 = {0, 0, 0, 0, 0, 0, 0, 0};
        if (res) r8 = *reinterpret_cast<const ushort8*>(res + e0);
        ushort8 o;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int c = c0 + k;
            float val = bf16_bits_to_float(in[k]) * scale[b * groups + c / cg] * gamma[c];
            if (res) val += bf16_bits_to_float(r8[k]);
            o[k] = __builtin_bit_cast(unsigned short, (__bf16)val);
        }
        *reinterpret_cast<ushort8*>(out + e0) = o;
    }
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_tens_group_norm_bf16_scratch_bytes(int batch, int groups, size_t* bytes) {
    MG_REQUIRE(bytes && batch >= 0 && groups >= 1, "mg_tens_group_norm_bf16_scratch_bytes: bad argument");
    *bytes = (size_t)batch * groups * (kGnMaxChunks * sizeof(double) + sizeof(float)) + 16;
    return MG_OK;
}

int mg_tens_group_norm_bf16(const void* y, const void* res, int batch, int nodes, int comps, int chan, int groups, float eps,
                            const float* gamma, void* scratch, void* out, mg_stream_t stream) {
    MG_REQUIRE(batch >= 0 && nodes >= 0 && comps >= 1 && chan >= 1 && groups >= 1, "mg_tens_group_norm_bf16: bad size");
    MG_REQUIRE(chan % groups == 0, "mg_tens_group_norm_bf16: groups must divide chan");
    MG_REQUIRE(chan % 8 == 0, "mg_tens_group_norm_bf16: chan must be a multiple of 8 (16-byte pieces along the channel axis)");
    MG_REQUIRE(comps * chan <= kGnMaxWidth, "mg_tens_group_norm_bf16: comps * chan must be at most %d", kGnMaxWidth);
    MG_REQUIRE(groups <= 256, "mg_tens_group_norm_bf16: at most 256 groups");
    if (batch == 0 || nodes == 0) return MG_OK;
    MG_REQUIRE(y && gamma && scratch && out && aligned16(y) && aligned16(out) && (!res || aligned16(res)) &&
                   (reinterpret_cast<uintptr_t>(scratch) & 7u) == 0,
               "mg_tens_group_norm_bf16: null or unaligned pointer");
    hipStream_t st = (hipStream_t)stream;
    double* partial = static_cast<double*>(scratch);
    float* scale = reinterpret_cast<float*>(partial + (size_t)batch * groups * kGnMaxChunks);
    long chunks = ceil_div(nodes, kGnNodesPerChunk);
    if (chunks > kGnMaxChunks) chunks = kGnMaxChunks;
    const long rows = (long)batch * nodes;
    gn_stats_bf16_kernel<<<dim3((unsigned)chunks, (unsigned)batch), dim3(256), 0, st>>>(
        static_cast<const unsigned short*>(y), nodes, comps, chan, groups, (int)chunks, partial);
    if (int code = check_launch("gn_stats_bf16_kernel")) return code;
    const int n_bg = batch * groups;
    gn_scales_kernel<<<dim3((unsigned)n_bg), dim3(256), 0, st>>>(partial, groups, (int)chunks,
                                                                 (double)nodes * (chan / groups), eps, scale);
    if (int code = check_launch("gn_scales_kernel")) return code;
    const long vecs = rows * comps * chan / 8;
    long blocks = ceil_div(vecs, 256);
    if (blocks > 256L * 32) blocks = 256L * 32;
    gn_apply_bf16_kernel<<<dim3((unsigned)blocks), dim3(256), 0, st>>>(
        static_cast<const unsigned short*>(y), static_cast<const unsigned short*>(res), scale, gamma, rows, nodes, comps, chan,
        groups, static_cast<unsigned short*>(out));
    return check_launch("gn_apply_bf16_kernel");
}

}  // extern "C"
