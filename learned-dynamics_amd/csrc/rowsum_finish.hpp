// Finishing pass of the GEMMs that sum the rows of each segment in their epilogue: every block of 32 rows left
// two partial rows (slot A: the run that starts at the block's first row, slot B: a later run that ends at its
// last row); runs strictly inside a block were written to `out` directly.
#pragma once
#include "common.hpp"

namespace mg {
namespace {

// out[s] = scale * (slots of the blocks the rows of segment s lie in, in block order); segments strictly inside
// one block were written by the kernel above, empty segments get zero.  One thread per four columns.
__global__ void __launch_bounds__(256)
rowsum_finish_kernel(const int* __restrict__ row_ptr, long n_out, long n_blocks, int O, const float* __restrict__ slots,
                     float scale, float* __restrict__ out) {
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const int quads = O / 4;
    if (idx >= n_out * quads) return;
    const long s_id = idx / quads;
    const int x = (int)(idx - s_id * quads) * 4;
    const long lo = row_ptr[s_id], hi = row_ptr[s_id + 1];
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (hi > lo) {
        const long b_lo = lo / 32, b_hi = (hi - 1) / 32;
        if (b_lo == b_hi && lo > 32 * b_lo && hi - 1 < 32 * b_lo + 31) return;   // written directly
        for (long b = b_lo; b <= b_hi; b++) {
            const float* slot = 32 * b >= lo ? slots + b * O : slots + (n_blocks + b) * O;
            const float4 t = *reinterpret_cast<const float4*>(slot + x);
            s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
        }
    }
    *reinterpret_cast<float4*>(out + s_id * O + x) = make_float4(scale * s.x, scale * s.y, scale * s.z, scale * s.w);
}

}  // namespace
}  // namespace mg
