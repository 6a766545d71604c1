// The bias-free output linear of the rank-2 channel applied to a node's rank-2 sums (or products) while they are
// still in registers, shared by the edge kernel of Messages and the node kernel of SelfTensProds
// (archs/diffuser_atoms15.py:82-94, 244-252):
//     out[o][comp i] = sum over (label, channel) of s2[i][label][channel] Y2[o][label chan + channel],  o < dim_d <= 16.
// A workgroup is four waves, a wave holds one 64-channel chunk of one node (lane = channel, registers = the 45
// (comp, label) values), and the 4 / chunks nodes of a workgroup are whole.  The fp32 matrix core
// (v_mfma_f32_16x16x4_f32: rows = the 9 components) wants lane (i, kk) to hold comp i at k = kk: one label at a time
// the wave's 9 x 64 values go through its own LDS rows, and step t of the label multiplies channels 16 kk + t (read
// four steps at a time); 80 matrix instructions per wave.  The waves' partial 9 x 16 results are added through LDS
// by the first wave of each node.  y2_packed: [chunk][label][tq][lane = 16 kk + j][tr] = Y2[j][label chan + 64 chunk
// + 16 kk + 4 tq + tr], zero for j >= dim_d (pack_rank2_weight_kernel).
#pragma once
#include "common.hpp"

namespace mg {

constexpr int kTrPitch = 68;   // floats per LDS row of a wave's transposition buffer (16-byte aligned rows)
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Called by all four waves of the workgroup (it holds two barriers); valid = false: a wave without an item, whose s2
// must be zeros.  out: this wave's node, (dim_d, 9); accumulate: the result is added to what out holds.
__device__ __forceinline__ void rank2_linear_of_node_sums(const float (&s2)[45], float (&tr_buf)[4][16 * kTrPitch],
                                                          float (&part)[4][16 * 16], int chunk, int chunks, bool valid,
                                                          const float* __restrict__ y2_packed, int dim_d,
                                                          float* __restrict__ out, bool accumulate = false) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    float* tr = tr_buf[wave];
    const int ci = lane & 15, kk = lane >> 4;
    // rows 9 .. 15 of the matrix operand are rows of zeros, written once
#pragma unroll
    for (int k = 9; k < 16; k++) tr[k * kTrPitch + lane] = 0.f;
    const float* a_src = tr + ci * kTrPitch + 16 * kk;
    const float4* yb = reinterpret_cast<const float4*>(y2_packed) + (long)chunk * 5 * 4 * 64 + lane;
    floatx4 d0 = {0.f, 0.f, 0.f, 0.f}, d1 = d0, d2 = d0, d3 = d0;   // four chains: a matrix instruction does not wait for the last one
    float4 b[4];
#pragma unroll
    for (int tq = 0; tq < 4; tq++) b[tq] = yb[tq * 64];
#pragma unroll
    for (int lab = 0; lab < 5; lab++) {
#pragma unroll
        for (int k = 0; k < 9; k++) tr[k * kTrPitch + lane] = s2[k * 5 + lab];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        float4 a[4];
#pragma unroll
        for (int tq = 0; tq < 4; tq++) a[tq] = *reinterpret_cast<const float4*>(a_src + 4 * tq);
        float4 bn[4];
        if (lab < 4) {
#pragma unroll
            for (int tq = 0; tq < 4; tq++) bn[tq] = yb[((lab + 1) * 4 + tq) * 64];
        }
#pragma unroll
        for (int tq = 0; tq < 4; tq++) {
            d0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[tq].x, b[tq].x, d0, 0, 0, 0);
            d1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[tq].y, b[tq].y, d1, 0, 0, 0);
            d2 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[tq].z, b[tq].z, d2, 0, 0, 0);
            d3 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[tq].w, b[tq].w, d3, 0, 0, 0);
        }
        if (lab < 4) {
#pragma unroll
            for (int tq = 0; tq < 4; tq++) b[tq] = bn[tq];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();                        // the rows are rewritten by the next label
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    // accumulator register q of lane l: comp 4 (l / 16) + q, output l % 16
#pragma unroll
    for (int q = 0; q < 4; q++) part[wave][(4 * kk + q) * 16 + ci] = (d0[q] + d1[q]) + (d2[q] + d3[q]);
    __syncthreads();
    if (chunk == 0 && valid) {                                  // the first wave of a node adds up its chunks
        for (int idx = lane; idx < dim_d * 9; idx += kWave) {
            const int j = idx / 9, i = idx - 9 * j;
            float sum = 0.f;
            for (int wv = 0; wv < chunks; wv++) sum += part[wave + wv][i * 16 + j];
            out[idx] = accumulate ? out[idx] + sum : sum;
        }
    }
    __syncthreads();                                            // before the workgroup's next use of part
}

inline bool rank2_fusable(int chan, int dim_d) {
    const int chunks = chan / 64;
    return chan > 0 && chan % 64 == 0 && (chunks == 1 || chunks == 2 || chunks == 4) && dim_d >= 1 && dim_d <= 16;
}

}  // namespace mg
