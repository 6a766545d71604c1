// Gather node rows to edges and sum edge rows back to nodes over a CSR
// (src-sorted) edge list.  Both are pure HBM streaming.
//
// segment sum: all edges of one node are consecutive, and each edge carries
// `feat` contiguous floats, so the data of a node is ONE contiguous
// [n_edges x feat] matrix and the result is its column sum.  A wave owns one
// (node, column chunk); the chunk width is a power of two (<= 64 lanes x VEC
// floats), and when the chunk is narrower than the wave the spare lanes take
// further edges of the same node and are folded together with xor-shuffles at
// the end.  Every input byte is read exactly once with unit-stride 16-byte (or
// 4-byte) accesses; there are no atomics and the summation order is fixed.
#include "common.hpp"

namespace mg {
namespace {

constexpr int kMaxChunks = 24;

struct Chunks {
    int n;
    int start[kMaxChunks];   // first float of the chunk
    int lanes[kMaxChunks];   // lanes per edge (power of two <= 64)
};

// split feat/VEC units into power-of-two pieces of at most 64 lanes
inline Chunks make_chunks(int feat, int vec) {
    Chunks c{};
    int units = feat / vec, pos = 0;
    while (units > 0 && c.n < kMaxChunks) {
        int p = 64;
        while (p > units) p >>= 1;
        c.start[c.n] = pos * vec;
        c.lanes[c.n] = p;
        c.n++;
        pos += p;
        units -= p;
    }
    return c;
}

template <int VEC>
struct Acc;
template <>
struct Acc<4> {
    float4 v;
    __device__ void zero() { v = make_float4(0.f, 0.f, 0.f, 0.f); }
    __device__ void add(const float* p) {
        const float4 t = *reinterpret_cast<const float4*>(p);
        v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
    }
    __device__ void fold(int d) {
        v.x += __shfl_xor(v.x, d); v.y += __shfl_xor(v.y, d);
        v.z += __shfl_xor(v.z, d); v.w += __shfl_xor(v.w, d);
    }
    __device__ void merge(const Acc& o) { v.x += o.v.x; v.y += o.v.y; v.z += o.v.z; v.w += o.v.w; }
    __device__ void store(float* p) const { *reinterpret_cast<float4*>(p) = v; }
};
template <>
struct Acc<1> {
    float v;
    __device__ void zero() { v = 0.f; }
    __device__ void add(const float* p) { v += *p; }
    __device__ void fold(int d) { v += __shfl_xor(v, d); }
    __device__ void merge(const Acc& o) { v += o.v; }
    __device__ void store(float* p) const { *p = v; }
};

// PERM: edge e of the CSR order is row perm[e] of x (an index that is not sorted, summed in its sorted order without
// first copying the rows into that order)
template <int VEC, bool PERM>
__global__ void __launch_bounds__(256) segment_sum_kernel(const float* __restrict__ x, const int* __restrict__ perm,
                                                          const int* __restrict__ row_ptr,
                                                          long n_rows, int feat, Chunks ch, float* __restrict__ out) {
    const int lane = threadIdx.x & (kWave - 1);
    const long wave_global = ((long)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    const long n_waves = ((long)gridDim.x * blockDim.x) / kWave;
    const long items = n_rows * ch.n;
    for (long item = wave_global; item < items; item += n_waves) {
        const long row = item / ch.n;
        const int c = (int)(item - row * ch.n);
        const int L = ch.lanes[c];                 // lanes per edge
        const int col = ch.start[c] + (lane & (L - 1)) * VEC;
        const int sub = lane / L, per_iter = kWave / L;
        const long lo = row_ptr[row], hi = row_ptr[row + 1];
        Acc<VEC> a0, a1, a2, a3;
        a0.zero();
        a1.zero();
        a2.zero();
        a3.zero();
        long e = lo + sub;
        for (; e + 3 * per_iter < hi; e += 4 * per_iter) {   // four independent loads in flight
            const long r0 = PERM ? perm[e] : e, r1 = PERM ? perm[e + per_iter] : e + per_iter;
            const long r2 = PERM ? perm[e + 2 * per_iter] : e + 2 * per_iter;
            const long r3 = PERM ? perm[e + 3 * per_iter] : e + 3 * per_iter;
            a0.add(x + r0 * feat + col);
            a1.add(x + r1 * feat + col);
            a2.add(x + r2 * feat + col);
            a3.add(x + r3 * feat + col);
        }
        for (; e < hi; e += per_iter) a0.add(x + (PERM ? (long)perm[e] : e) * feat + col);
        a0.merge(a1);
        a2.merge(a3);
        a0.merge(a2);
        for (int d = L; d < kWave; d <<= 1) a0.fold(d);
        if (sub == 0) a0.store(out + row * feat + col);
    }
}

// bf16 storage, fp32 accumulation: a lane owns 4 consecutive channels (8-byte loads), L lanes cover
// one edge row, the other 64/L lane groups take further edges and are folded at the end.
// out[row] = scale * sum over the row's edges.
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(256) segment_sum_bf16_kernel(const __bf16* __restrict__ x,
                                                               const int* __restrict__ row_ptr, long n_rows, int feat,
                                                               int L, int chunks, float scale,
                                                               __bf16* __restrict__ out) {
    const int lane = threadIdx.x & (kWave - 1);
    const long wave_global = ((long)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    const long n_waves = ((long)gridDim.x * blockDim.x) / kWave;
    const long items = n_rows * chunks;
    const int sub = lane / L, per_iter = kWave / L;
    for (long item = wave_global; item < items; item += n_waves) {
        const long row = item / chunks;
        const int c = (int)(item - row * chunks);
        const int col = c * 256 + (lane & (L - 1)) * 4;
        const bool active = col < feat;
        const long lo = row_ptr[row], hi = row_ptr[row + 1];
        float a[4] = {0.f, 0.f, 0.f, 0.f};
        if (active) {
            for (long e = lo + sub; e < hi; e += per_iter) {
                const bf16x4 v = *reinterpret_cast<const bf16x4*>(x + e * feat + col);
#pragma unroll
                for (int k = 0; k < 4; k++) a[k] += (float)v[k];
            }
        }
        for (int d = L; d < kWave; d <<= 1) {
#pragma unroll
            for (int k = 0; k < 4; k++) a[k] += __shfl_xor(a[k], d, kWave);
        }
        if (active && sub == 0) {
            bf16x4 o;
#pragma unroll
            for (int k = 0; k < 4; k++) o[k] = (__bf16)(a[k] * scale);
            *reinterpret_cast<bf16x4*>(out + row * feat + col) = o;
        }
    }
}

template <int VEC>
__global__ void __launch_bounds__(256) gather_kernel(const float* __restrict__ x, const void* __restrict__ index,
                                                     int is64, long n_edges, long n_rows, int feat,
                                                     float* __restrict__ out) {
    const long units = (long)(feat / VEC);
    const long total = n_edges * units;
    for (long t = (long)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (long)gridDim.x * blockDim.x) {
        const long e = t / units;
        const long u = t - e * units;
        long r = is64 ? static_cast<const long long*>(index)[e] : (long)static_cast<const int*>(index)[e];
        if (r < 0 || r >= n_rows) r = 0;   // callers validate; never read out of bounds
        if (VEC == 4)
            reinterpret_cast<float4*>(out)[t] = reinterpret_cast<const float4*>(x + r * feat)[u];
        else
            out[t] = x[r * feat + u];
    }
}

// row_ptr[r] = number of entries with index < r, for a sorted index
__global__ void __launch_bounds__(256) row_ptr_kernel(const void* __restrict__ index, int is64, long n_edges,
                                                      int n_rows, int* __restrict__ row_ptr) {
    auto at = [&](long e) -> long {
        return is64 ? (long)static_cast<const long long*>(index)[e] : (long)static_cast<const int*>(index)[e];
    };
    auto clampi = [&](long v) -> long { return v < -1 ? -1 : (v > n_rows - 1 ? n_rows - 1 : v); };
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (n_edges == 0) {
        if (e <= n_rows) row_ptr[e] = 0;
        return;
    }
    if (e >= n_edges) return;
    const long cur = clampi(at(e));
    const long prev = e == 0 ? -1 : clampi(at(e - 1));
    for (long r = prev + 1; r <= cur; r++) row_ptr[r] = (int)e;
    if (e == n_edges - 1)
        for (long r = cur + 1; r <= n_rows; r++) row_ptr[r] = (int)n_edges;
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_segment_row_ptr(const void* index, int index_is_int64, long n_edges, int n_rows, int* row_ptr,
                       mg_stream_t stream) {
    MG_REQUIRE(n_edges >= 0 && n_rows >= 0, "mg_segment_row_ptr: negative size");
    MG_REQUIRE(n_edges < 0x7fffffffL, "mg_segment_row_ptr: edge count does not fit int32");
    MG_REQUIRE(row_ptr != nullptr && (n_edges == 0 || index != nullptr), "mg_segment_row_ptr: null pointer");
    const long threads = n_edges > 0 ? n_edges : (long)n_rows + 1;
    hipLaunchKernelGGL(row_ptr_kernel, dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0, (hipStream_t)stream, index,
                       index_is_int64, n_edges, n_rows, row_ptr);
    return check_launch("mg_segment_row_ptr");
}

int mg_segment_sum_csr(const float* x_edge, const int* row_ptr, int n_rows, int feat, float* out,
                       mg_stream_t stream) {
    return mg_segment_sum_csr_perm(x_edge, nullptr, row_ptr, n_rows, feat, out, stream);
}

int mg_segment_sum_csr_perm(const float* x_edge, const int* perm, const int* row_ptr, int n_rows, int feat, float* out,
                            mg_stream_t stream) {
    MG_REQUIRE(n_rows >= 0 && feat >= 0, "mg_segment_sum_csr: negative size");
    if (n_rows == 0 || feat == 0) return MG_OK;
    MG_REQUIRE(row_ptr && out, "mg_segment_sum_csr: null pointer");
    const bool vec = (feat % 4 == 0) && aligned16(x_edge) && aligned16(out);
    const Chunks ch = make_chunks(feat, vec ? 4 : 1);
    int covered = 0;
    for (int k = 0; k < ch.n; k++) covered += ch.lanes[k] * (vec ? 4 : 1);
    MG_REQUIRE(covered == feat, "mg_segment_sum_csr: feat=%d is too wide", feat);
    const long items = (long)n_rows * ch.n;
    long blocks = ceil_div(items, 4);
    if (blocks > 256L * 64) blocks = 256L * 64;   // grid-stride beyond 64 workgroups per CU
    const dim3 grid((unsigned)blocks), block(256);
    hipStream_t st = (hipStream_t)stream;
    if (vec && perm)
        hipLaunchKernelGGL((segment_sum_kernel<4, true>), grid, block, 0, st, x_edge, perm, row_ptr, (long)n_rows, feat, ch, out);
    else if (vec)
        hipLaunchKernelGGL((segment_sum_kernel<4, false>), grid, block, 0, st, x_edge, perm, row_ptr, (long)n_rows, feat, ch, out);
    else if (perm)
        hipLaunchKernelGGL((segment_sum_kernel<1, true>), grid, block, 0, st, x_edge, perm, row_ptr, (long)n_rows, feat, ch, out);
    else
        hipLaunchKernelGGL((segment_sum_kernel<1, false>), grid, block, 0, st, x_edge, perm, row_ptr, (long)n_rows, feat, ch, out);
    return check_launch("mg_segment_sum_csr");
}

int mg_segment_sum_csr_bf16(const void* x_edge, const int* row_ptr, int n_rows, int feat, float scale, void* out,
                            mg_stream_t stream) {
    MG_REQUIRE(n_rows >= 0 && feat >= 0, "mg_segment_sum_csr_bf16: negative size");
    if (n_rows == 0 || feat == 0) return MG_OK;
    MG_REQUIRE(feat % 4 == 0, "mg_segment_sum_csr_bf16: feat must be a multiple of 4 (got %d)", feat);
    MG_REQUIRE(row_ptr && out, "mg_segment_sum_csr_bf16: null pointer");
    MG_REQUIRE((reinterpret_cast<uintptr_t>(x_edge) & 7u) == 0 && (reinterpret_cast<uintptr_t>(out) & 7u) == 0,
               "mg_segment_sum_csr_bf16: pointers must be 8-byte aligned");
    const int chunks = (int)ceil_div(feat, 256);
    int L = 1;
    while (L < 64 && L * 4 < (feat < 256 ? feat : 256)) L <<= 1;
    const long items = (long)n_rows * chunks;
    long blocks = ceil_div(items, 4);
    if (blocks > 256L * 64) blocks = 256L * 64;
    hipLaunchKernelGGL(segment_sum_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       static_cast<const __bf16*>(x_edge), row_ptr, (long)n_rows, feat, L, chunks, scale,
                       static_cast<__bf16*>(out));
    return check_launch("mg_segment_sum_csr_bf16");
}

int mg_gather_rows(const float* x, const void* index, int index_is_int64, long n_edges, int n_rows, int feat,
                   float* out, mg_stream_t stream) {
    MG_REQUIRE(n_edges >= 0 && n_rows >= 0 && feat >= 0, "mg_gather_rows: negative size");
    if (n_edges == 0 || feat == 0) return MG_OK;
    MG_REQUIRE(n_rows > 0, "mg_gather_rows: gather from an empty tensor");
    MG_REQUIRE(x && index && out, "mg_gather_rows: null pointer");
    const bool vec = (feat % 4 == 0) && aligned16(x) && aligned16(out);
    const long total = n_edges * (feat / (vec ? 4 : 1));
    long blocks = ceil_div(total, 256);
    if (blocks > 256L * 256) blocks = 256L * 256;
    if (vec)
        hipLaunchKernelGGL(gather_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, x, index,
                           index_is_int64, n_edges, (long)n_rows, feat, out);
    else
        hipLaunchKernelGGL(gather_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, x, index,
                           index_is_int64, n_edges, (long)n_rows, feat, out);
    return check_launch("mg_gather_rows");
}

}  // extern "C"
