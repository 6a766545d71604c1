// The 13 Cartesian products on node rows in component-major layout (node, comp, chan), for the
// self-interaction block (archs/diffuser_atoms15.py:59-95) of the bf16-storage configuration.
//
// Inputs  l0/r0 (N, chan), l1/r1 (N, 3, chan), l2/r2 (N, 9, chan)
// Outputs P0 (N, 3, chan)      labels 000, 110, 220
//         P1 (N, 3, 5, chan)   labels 011, 101, 121, 211, 111 per vector component
//         P2 (N, 9, 5, chan)   labels 022, 202, 112, 222, 212 per rank-2 component (xy -> 3x+y)
// i.e. the layout the edge kernel uses for its per-node sums, so the output linears of a rank are
// one GEMM with K = 3*chan or 5*chan.  A lane owns one (node, channel): every access of a wave is
// unit stride.  Bound by HBM: 26 values in, 63 out per (node, channel).
#include "common.hpp"
#include "rank2_linear.hpp"

namespace mg {
namespace {

template <typename T>
__global__ void __launch_bounds__(256) node_products_kernel(long n_nodes, int chan, const T* __restrict__ l0,
                                                            const T* __restrict__ l1, const T* __restrict__ l2,
                                                            const T* __restrict__ r0, const T* __restrict__ r1,
                                                            const T* __restrict__ r2, T* __restrict__ P0,
                                                            T* __restrict__ P1, T* __restrict__ P2,
                                                            float* __restrict__ node_max) {
    const long total = n_nodes * chan;
    for (long t = (long)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (long)gridDim.x * blockDim.x) {
        const long node = t / chan;
        const int c = (int)(t - node * chan);
        const float a = (float)l0[t], b = (float)r0[t];
        float u[3], v[3], L[9], R[9];
#pragma unroll
        for (int x = 0; x < 3; x++) {
            u[x] = (float)l1[(node * 3 + x) * chan + c];
            v[x] = (float)r1[(node * 3 + x) * chan + c];
        }
#pragma unroll
        for (int k = 0; k < 9; k++) {
            L[k] = (float)l2[(node * 9 + k) * chan + c];
            R[k] = (float)r2[(node * 9 + k) * chan + c];
        }
        float dot = 0.f, ddot = 0.f;
#pragma unroll
        for (int x = 0; x < 3; x++) dot += u[x] * v[x];
#pragma unroll
        for (int k = 0; k < 9; k++) ddot += L[k] * R[k];
        T* p0 = P0 + (node * 3) * chan + c;
        p0[0] = (T)(a * b);
        p0[chan] = (T)dot;
        p0[2 * chan] = (T)ddot;
        float mx = fmaxf(fabsf(a * b), fmaxf(fabsf(dot), fabsf(ddot)));

        const float cr[3] = {u[1] * v[2] - u[2] * v[1], u[2] * v[0] - u[0] * v[2], u[0] * v[1] - u[1] * v[0]};
#pragma unroll
        for (int x = 0; x < 3; x++) {
            T* p1 = P1 + ((node * 3 + x) * 5) * chan + c;
            p1[0] = (T)(a * v[x]);                                                      // 011
            p1[chan] = (T)(u[x] * b);                                                   // 101
            p1[2 * chan] = (T)(u[0] * R[3 * x] + u[1] * R[3 * x + 1] + u[2] * R[3 * x + 2]);   // 121: sum_k l_k r_{x k}
            p1[3 * chan] = (T)(L[3 * x] * v[0] + L[3 * x + 1] * v[1] + L[3 * x + 2] * v[2]);   // 211
            p1[4 * chan] = (T)cr[x];                                                    // 111
            mx = fmaxf(mx, fmaxf(fmaxf(fabsf(a * v[x]), fabsf(u[x] * b)), fabsf(cr[x])));
            mx = fmaxf(mx, fabsf(u[0] * R[3 * x] + u[1] * R[3 * x + 1] + u[2] * R[3 * x + 2]));
            mx = fmaxf(mx, fabsf(L[3 * x] * v[0] + L[3 * x + 1] * v[1] + L[3 * x + 2] * v[2]));
        }
#pragma unroll
        for (int x = 0; x < 3; x++) {
            // 212: row x of L crossed with v
            const float rc[3] = {L[3 * x + 1] * v[2] - L[3 * x + 2] * v[1], L[3 * x + 2] * v[0] - L[3 * x] * v[2],
                                 L[3 * x] * v[1] - L[3 * x + 1] * v[0]};
#pragma unroll
            for (int z = 0; z < 3; z++) {
                const int k = 3 * x + z;
                T* p2 = P2 + ((node * 9 + k) * 5) * chan + c;
                p2[0] = (T)(a * R[k]);                                                  // 022
                p2[chan] = (T)(L[k] * b);                                               // 202
                p2[2 * chan] = (T)(u[x] * v[z]);                                        // 112
                p2[3 * chan] = (T)(L[3 * x] * R[3 * z] + L[3 * x + 1] * R[3 * z + 1] + L[3 * x + 2] * R[3 * z + 2]);  // 222
                p2[4 * chan] = (T)rc[z];                                                // 212
                mx = fmaxf(mx, fmaxf(fmaxf(fabsf(a * R[k]), fabsf(L[k] * b)), fmaxf(fabsf(u[x] * v[z]), fabsf(rc[z]))));
                mx = fmaxf(mx, fabsf(L[3 * x] * R[3 * z] + L[3 * x + 1] * R[3 * z + 1] + L[3 * x + 2] * R[3 * z + 2]));
            }
        }
        if (node_max) {
            // chan is a multiple of 64 here, so a wave lies inside one node: one partial maximum
            // per (node, 64-channel chunk), a row bound for the GEMMs that read P0 / P1 / P2
            for (int d = 1; d < kWave; d <<= 1) mx = fmaxf(mx, __shfl_xor(mx, d));
            if ((threadIdx.x & (kWave - 1)) == 0) node_max[node * (chan / kWave) + c / kWave] = mx;
        }
    }
}

// The five rank-2 products of a node (labels 022, 202, 112, 222, 212) and the rank-2 output linear of SelfTensProds
// in one pass: a wave owns (node, 64-channel chunk), a lane one channel; the 45 product values stay in registers
// and go through rank2_linear_of_node_sums.  Reads the 26 operand rows of a node once (unit stride), writes
// (node, dim_d, 9); the products themselves are never stored.  For chan = 64, 128 or 256 and dim_d <= 16.
// (A persistent variant whose workgroups walk over the nodes with the next node's operands already requested was
// measured at 65 536 nodes, 256 channels: 0.61 ms against 0.57 ms; the kernel is bound by the matrix instructions,
// 0.31 ms of pipe time at 9 of 16 rows used, and what each wave does around them, not by the latency of its loads.)
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(5, 8)))
node_rank2_linear_kernel(long n_nodes, int chan, const float* __restrict__ l0,
                                                                const float* __restrict__ l1, const float* __restrict__ l2,
                                                                const float* __restrict__ r0, const float* __restrict__ r1,
                                                                const float* __restrict__ r2,
                                                                const float* __restrict__ y2_packed, int dim_d,
                                                                float* __restrict__ out, float* __restrict__ P0,
                                                                float* __restrict__ P1, float* __restrict__ node_max,
                                                                const float* __restrict__ x_d,
                                                                const float* __restrict__ L2t,
                                                                const float* __restrict__ R2t, int dim_in2) {
    __shared__ __attribute__((aligned(16))) float tr_buf[4][16 * kTrPitch];
    __shared__ float part[4][16 * 16];
    __shared__ float xd_buf[4][16 * 9];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int chunks = chan / kWave;
    const long items = n_nodes * chunks;
    long item = (long)blockIdx.x * 4 + wave;
    const bool valid = item < items;                           // uniform over the wave
    item = valid ? item : items - 1;
    const long node = item / chunks;
    const int chunk = (int)(item - node * chunks);
    const int c = chunk * kWave + lane;
    float s2[45];
    if (valid) {
        const float a = l0[node * chan + c], b = r0[node * chan + c];
        float u[3], v[3], L[9], R[9];
#pragma unroll
        for (int x = 0; x < 3; x++) {
            u[x] = l1[(node * 3 + x) * chan + c];
            v[x] = r1[(node * 3 + x) * chan + c];
        }
        if (x_d) {
            // the rank-2 operands are formed here: l2[k] = sum_i L2[c, i] x_d[node, i, k] (dim_in2 <= 16 input
            // channels; the node's 9 dim_in2 values go through LDS and are read back as broadcasts, the weights come
            // transposed, (dim_in2, chan), one coalesced row per input channel).  Two GEMMs that would each write
            // (node, 9, chan) and this kernel's read of both are not needed.
            float* xd = xd_buf[wave];
            const float* src = x_d + node * (long)(dim_in2 * 9);
            for (int t = lane; t < dim_in2 * 9; t += kWave) xd[t] = src[t];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int k = 0; k < 9; k++) { L[k] = 0.f; R[k] = 0.f; }
            for (int i = 0; i < dim_in2; i++) {
                const float wl = L2t[(long)i * chan + c], wr = R2t[(long)i * chan + c];
#pragma unroll
                for (int k = 0; k < 9; k++) {
                    const float xv = xd[i * 9 + k];
                    L[k] = fmaf(wl, xv, L[k]);
                    R[k] = fmaf(wr, xv, R[k]);
                }
            }
        } else {
#pragma unroll
            for (int k = 0; k < 9; k++) {
                L[k] = l2[(node * 9 + k) * chan + c];
                R[k] = r2[(node * 9 + k) * chan + c];
            }
        }
        if (P0) {
            // the scalar and vector products as well, stored in the layout of mg_bee_node_products with their
            // maximum per (node, chunk): the operands are in registers once, and the two GEMMs that follow read
            // 18 chan floats per node instead of gathering 26 chan through their operand loads
            float dot = 0.f, ddot = 0.f;
#pragma unroll
            for (int x = 0; x < 3; x++) dot += u[x] * v[x];
#pragma unroll
            for (int k = 0; k < 9; k++) ddot += L[k] * R[k];
            float* p0 = P0 + (node * 3) * chan + c;
            __builtin_nontemporal_store(a * b, p0);
            __builtin_nontemporal_store(dot, p0 + chan);
            __builtin_nontemporal_store(ddot, p0 + 2 * chan);
            float mx = fmaxf(fabsf(a * b), fmaxf(fabsf(dot), fabsf(ddot)));
            const float cr[3] = {u[1] * v[2] - u[2] * v[1], u[2] * v[0] - u[0] * v[2], u[0] * v[1] - u[1] * v[0]};
#pragma unroll
            for (int x = 0; x < 3; x++) {
                float* p1 = P1 + ((node * 3 + x) * 5) * chan + c;
                const float q[5] = {a * v[x], u[x] * b, u[0] * R[3 * x] + u[1] * R[3 * x + 1] + u[2] * R[3 * x + 2],
                                    L[3 * x] * v[0] + L[3 * x + 1] * v[1] + L[3 * x + 2] * v[2], cr[x]};   // 011 101 121 211 111
#pragma unroll
                for (int t = 0; t < 5; t++) {
                    __builtin_nontemporal_store(q[t], p1 + t * chan);
                    mx = fmaxf(mx, fabsf(q[t]));
                }
            }
            if (node_max) {
                for (int d = 1; d < kWave; d <<= 1) mx = fmaxf(mx, __shfl_xor(mx, d));
                if (lane == 0) node_max[node * chunks + chunk] = mx;
            }
        }
#pragma unroll
        for (int x = 0; x < 3; x++) {
            // 212: row x of L crossed with v
            const float rc[3] = {L[3 * x + 1] * v[2] - L[3 * x + 2] * v[1], L[3 * x + 2] * v[0] - L[3 * x] * v[2],
                                 L[3 * x] * v[1] - L[3 * x + 1] * v[0]};
#pragma unroll
            for (int z = 0; z < 3; z++) {
                const int k = 3 * x + z;
                s2[k * 5 + 0] = a * R[k];                                                                       // 022
                s2[k * 5 + 1] = L[k] * b;                                                                       // 202
                s2[k * 5 + 2] = u[x] * v[z];                                                                    // 112
                s2[k * 5 + 3] = L[3 * x] * R[3 * z] + L[3 * x + 1] * R[3 * z + 1] + L[3 * x + 2] * R[3 * z + 2];  // 222
                s2[k * 5 + 4] = rc[z];                                                                          // 212
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < 45; k++) s2[k] = 0.f;
    }
    rank2_linear_of_node_sums(s2, tr_buf, part, chunk, chunks, valid, y2_packed, dim_d, out + node * (long)dim_d * 9);
}

template <typename T>
int launch(const char* what, long n_nodes, int chan, const void* l0, const void* l1, const void* l2, const void* r0,
           const void* r1, const void* r2, void* P0, void* P1, void* P2, float* node_max, mg_stream_t stream) {
    MG_REQUIRE(n_nodes >= 0 && chan >= 0, "%s: negative size", what);
    MG_REQUIRE(node_max == nullptr || chan % kWave == 0, "%s: node_max needs chan to be a multiple of 64", what);
    if (n_nodes == 0 || chan == 0) return MG_OK;
    MG_REQUIRE(l0 && l1 && l2 && r0 && r1 && r2 && P0 && P1 && P2, "%s: null pointer", what);
    long blocks = ceil_div(n_nodes * chan, 256);
    if (blocks > 256L * 32) blocks = 256L * 32;
    hipLaunchKernelGGL(node_products_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, n_nodes,
                       chan, static_cast<const T*>(l0), static_cast<const T*>(l1), static_cast<const T*>(l2),
                       static_cast<const T*>(r0), static_cast<const T*>(r1), static_cast<const T*>(r2),
                       static_cast<T*>(P0), static_cast<T*>(P1), static_cast<T*>(P2), node_max);
    return check_launch(what);
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_bee_node_products(long n_nodes, int chan, const float* l0, const float* l1, const float* l2, const float* r0,
                         const float* r1, const float* r2, float* P0, float* P1, float* P2, float* node_max,
                         mg_stream_t stream) {
    return launch<float>("mg_bee_node_products", n_nodes, chan, l0, l1, l2, r0, r1, r2, P0, P1, P2, node_max, stream);
}

int mg_bee_node_products_rank2(long n_nodes, int chan, const float* l0, const float* l1, const float* l2,
                               const float* r0, const float* r1, const float* r2, const float* packed_Y2, int dim_d,
                               float* out_d, float* P0, float* P1, float* node_max, const float* x_d,
                               const float* L2t, const float* R2t, int dim_in2, mg_stream_t stream) {
    MG_REQUIRE((P0 == nullptr) == (P1 == nullptr) && (node_max == nullptr || P0 != nullptr),
               "mg_bee_node_products_rank2: P0 and P1 go together, node_max with them");
    MG_REQUIRE(x_d == nullptr || (L2t && R2t && dim_in2 >= 1 && dim_in2 <= 16),
               "mg_bee_node_products_rank2: x_d needs both transposed weights and 1 .. 16 input channels");

    MG_REQUIRE(n_nodes >= 0, "mg_bee_node_products_rank2: negative size");
    MG_REQUIRE(rank2_fusable(chan, dim_d), "mg_bee_node_products_rank2: needs chan = 64, 128 or 256 and dim_d <= 16");
    if (n_nodes == 0) return MG_OK;
    MG_REQUIRE(l0 && l1 && r0 && r1 && packed_Y2 && out_d && aligned16(packed_Y2),
               "mg_bee_node_products_rank2: null or unaligned pointer");
    MG_REQUIRE(x_d != nullptr || (l2 && r2), "mg_bee_node_products_rank2: l2 and r2, or x_d and the weights");
    const long blocks = ceil_div(n_nodes * (chan / kWave), 4);
    MG_REQUIRE(blocks < (1L << 31), "mg_bee_node_products_rank2: too many nodes for one launch");
    hipLaunchKernelGGL(node_rank2_linear_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, n_nodes,
                       chan, l0, l1, l2, r0, r1, r2, packed_Y2, dim_d, out_d, P0, P1, node_max, x_d, L2t, R2t, dim_in2);
    return check_launch("mg_bee_node_products_rank2");
}

int mg_bee_node_products_bf16(long n_nodes, int chan, const void* l0, const void* l1, const void* l2, const void* r0,
                              const void* r1, const void* r2, void* P0, void* P1, void* P2, mg_stream_t stream) {
    return launch<__bf16>("mg_bee_node_products_bf16", n_nodes, chan, l0, l1, l2, r0, r1, r2, P0, P1, P2, nullptr, stream);
}

}  // extern "C"
