// Weight gradient of the channel-mixing linear:
//   dW[o, i] = sum_{r, t} dy[r, o, t] x[r, i, t]
// A GEMM whose reduction dimension (rows x components) is the long one, so the
// rows are split over workgroups (split-K); each workgroup reduces its slice
// for one 64x64 tile of dW in registers and writes it to its own plane of a
// workspace; a second kernel adds the planes in slice order.  No atomics: the
// result does not depend on the order in which workgroups finish.
// Plain rows (no tensor components) go through the matrix cores.  mg_tensor_linear_wgrad uses the fp32 ones:
// v_mfma_f32_32x32x2_f32 takes dy and x exactly as they lie in memory (for the reduction index r, lanes 0..31 supply
// 32 consecutive columns of row r and lanes 32..63 those of row r + 1), products and sums are fp32, nothing is
// rounded to a shorter format.  mg_tensor_linear_wgrad_f16x2 uses the fp16 ones with two-piece operands (three times
// the rate at an error of a few fp32 ulps of sum |dy| |x|) and also sums the columns of dy, the bias gradient.
// Training-side helper: not on the inference hot path.
#include "common.hpp"
#include "f16x2.hpp"

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

// Plain rows on the matrix cores.  A workgroup of 4 waves owns a 128 x 128 tile of dW over its slice of the rows;
// wave w owns the 64 x 64 quarter (w / 2, w % 2) as 2 x 2 accumulators of 32 x 32.  Columns past the matrix and rows
// past the slice are read from a clamped address and replaced by zero.
constexpr int kMTile = 128;
constexpr int kMRows = 8;       // rows per trip of the loop: 4 matrix steps of 2 rows

__global__ void __launch_bounds__(256) wgrad_mfma_kernel(const float* __restrict__ dy, const float* __restrict__ x,
                                                         long R, int I, int O, long rows_per_block,
                                                         float* __restrict__ part) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = lane & 31, kk = lane >> 5;
    const int o_base = blockIdx.x * kMTile + (wave >> 1) * 64, i_base = blockIdx.y * kMTile + (wave & 1) * 64;
    const long r_lo = (long)blockIdx.z * rows_per_block;
    const long r_hi = r_lo + rows_per_block < R ? r_lo + rows_per_block : R;
    // this lane's two columns of dy and of x (clamped; `live` says whether the column exists)
    int oc[2], ic[2];
    bool o_live[2], i_live[2];
#pragma unroll
    for (int p = 0; p < 2; p++) {
        const int o = o_base + 32 * p + m, i = i_base + 32 * p + m;
        o_live[p] = o < O; i_live[p] = i < I;
        oc[p] = o_live[p] ? o : O - 1;
        ic[p] = i_live[p] ? i : I - 1;
    }
    floatx16 acc[2][2];
#pragma unroll
    for (int p = 0; p < 2; p++)
#pragma unroll
        for (int q = 0; q < 2; q++)
#pragma unroll
            for (int k = 0; k < 16; k++) acc[p][q][k] = 0.f;

    // the operands of the next trip are requested before the matrix instructions of this one
    float a[2][kMRows / 2][2], b[2][kMRows / 2][2];
    auto fetch = [&](float (&aa)[kMRows / 2][2], float (&bb)[kMRows / 2][2], long r) {
#pragma unroll
        for (int s = 0; s < kMRows / 2; s++) {
            const long row = r + 2 * s + kk;
            const bool row_live = row < r_hi;
            const long rc = row_live ? row : r_hi - 1;
#pragma unroll
            for (int p = 0; p < 2; p++) {
                const float va = dy[rc * O + oc[p]], vb = x[rc * I + ic[p]];
                aa[s][p] = (row_live && o_live[p]) ? va : 0.f;
                bb[s][p] = (row_live && i_live[p]) ? vb : 0.f;
            }
        }
    };
    auto multiply = [&](const float (&aa)[kMRows / 2][2], const float (&bb)[kMRows / 2][2]) {
#pragma unroll
        for (int s = 0; s < kMRows / 2; s++)
#pragma unroll
            for (int p = 0; p < 2; p++)
#pragma unroll
                for (int q = 0; q < 2; q++)
                    acc[p][q] = __builtin_amdgcn_mfma_f32_32x32x2f32(aa[s][p], bb[s][q], acc[p][q], 0, 0, 0);
    };
    fetch(a[0], b[0], r_lo);
    for (long r = r_lo; r < r_hi; r += 2 * kMRows) {
        fetch(a[1], b[1], r + kMRows);                 // (past the slice: clamped addresses, zeros)
        multiply(a[0], b[0]);
        fetch(a[0], b[0], r + 2 * kMRows);
        multiply(a[1], b[1]);
    }
    // D[o][i]: i = lane % 32, o = 8 (k / 4) + 4 (lane / 32) + k % 4 for register k
    float* plane = part + (long)blockIdx.z * O * I;
#pragma unroll
    for (int p = 0; p < 2; p++)
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const int i = i_base + 32 * q + m;
#pragma unroll
            for (int k = 0; k < 16; k++) {
                const int o = o_base + 32 * p + 8 * (k / 4) + 4 * kk + (k % 4);
                if (o < O && i < I) plane[(long)o * I + i] = acc[p][q][k];
            }
        }
}

// The same with the operands staged through LDS, for dimensions that are multiples of 4: a lane of the kernel above
// loads one float per matrix operand, and the vector memory front end spends as long on such a load as on a 16-byte
// one (about a cycle per lane), four times the matrix time of the tile.  Here the workgroup loads 16 rows x 128
// columns of dy and of x with 16-byte loads into LDS (rows padded to 160 floats: the two rows that the two halves of a
// wave read lie 32 banks apart) and the lanes pick their operands out of LDS; the next 16 rows are on their way while
// the current ones are multiplied.
constexpr int kSRows = 16, kSPitch = 160;
__global__ void __launch_bounds__(256) wgrad_mfma_lds_kernel(const float* __restrict__ dy, const float* __restrict__ x,
                                                             long R, int I, int O, long rows_per_block,
                                                             float* __restrict__ part) {
    __shared__ __attribute__((aligned(16))) float dys[2][kSRows * kSPitch];
    __shared__ __attribute__((aligned(16))) float xs[2][kSRows * kSPitch];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = lane & 31, kk = lane >> 5;
    const int o_tile = blockIdx.x * kMTile, i_tile = blockIdx.y * kMTile;
    const int o_wave = (wave >> 1) * 64, i_wave = (wave & 1) * 64;
    const long r_lo = (long)blockIdx.z * rows_per_block;
    const long r_hi = r_lo + rows_per_block < R ? r_lo + rows_per_block : R;

    // staging: thread -> two 16-byte pieces per operand (piece = row * 32 + column quad)
    int st_row[2], st_col[2];
    bool o_ok[2], i_ok[2];
    const float* dy_src[2];
    const float* x_src[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int piece = threadIdx.x + 256 * u;
        st_row[u] = piece >> 5;
        st_col[u] = (piece & 31) * 4;
        o_ok[u] = o_tile + st_col[u] < O;
        i_ok[u] = i_tile + st_col[u] < I;
        dy_src[u] = dy + (o_ok[u] ? o_tile + st_col[u] : 0);
        x_src[u] = x + (i_ok[u] ? i_tile + st_col[u] : 0);
    }
    float4 ra[2], rb[2];
    auto fetch = [&](long r) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const long row = r + st_row[u];
            const long rc = row < r_hi ? row : r_hi - 1;            // (clamped: replaced by zeros when stored)
            ra[u] = *reinterpret_cast<const float4*>(dy_src[u] + rc * O);
            rb[u] = *reinterpret_cast<const float4*>(x_src[u] + rc * I);
        }
    };
    auto store = [&](long r, int buf) {
        const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const bool row_ok = r + st_row[u] < r_hi;
            *reinterpret_cast<float4*>(&dys[buf][st_row[u] * kSPitch + st_col[u]]) = (row_ok && o_ok[u]) ? ra[u] : zero;
            *reinterpret_cast<float4*>(&xs[buf][st_row[u] * kSPitch + st_col[u]]) = (row_ok && i_ok[u]) ? rb[u] : zero;
        }
    };

    floatx16 acc[2][2];
#pragma unroll
    for (int p = 0; p < 2; p++)
#pragma unroll
        for (int q = 0; q < 2; q++)
#pragma unroll
            for (int k = 0; k < 16; k++) acc[p][q][k] = 0.f;

    fetch(r_lo);
    store(r_lo, 0);
    __syncthreads();
    int buf = 0;
    for (long r = r_lo; r < r_hi; r += kSRows) {
        const bool more = r + kSRows < r_hi;                          // uniform
        if (more) fetch(r + kSRows);
        const float* a_lds = &dys[buf][kk * kSPitch + o_wave + m];
        const float* b_lds = &xs[buf][kk * kSPitch + i_wave + m];
#pragma unroll
        for (int s = 0; s < kSRows / 2; s++) {
            float a[2], b[2];
#pragma unroll
            for (int p = 0; p < 2; p++) {
                a[p] = a_lds[2 * s * kSPitch + 32 * p];
                b[p] = b_lds[2 * s * kSPitch + 32 * p];
            }
#pragma unroll
            for (int p = 0; p < 2; p++)
#pragma unroll
                for (int q = 0; q < 2; q++)
                    acc[p][q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[p], b[q], acc[p][q], 0, 0, 0);
        }
        if (more) store(r + kSRows, buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
    // D[o][i]: i = lane % 32, o = 8 (k / 4) + 4 (lane / 32) + k % 4 for register k
    float* plane = part + (long)blockIdx.z * O * I;
#pragma unroll
    for (int p = 0; p < 2; p++)
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const int i = i_tile + i_wave + 32 * q + m;
#pragma unroll
            for (int k = 0; k < 16; k++) {
                const int o = o_tile + o_wave + 32 * p + 8 * (k / 4) + 4 * kk + (k % 4);
                if (o < O && i < I) plane[(long)o * I + i] = acc[p][q][k];
            }
        }
}

// Plain rows on the fp16 matrix cores with two-piece operands: dy and x are scaled by one power of two each (taken
// from an upper bound of their magnitudes, so that nothing overflows fp16; an entry 2^17 times smaller than the bound
// still keeps 22 bits) and split into hi + lo fp16 pieces; dy^T x takes three v_mfma_f32_32x32x16_f16 per step
// (lo hi, hi lo, hi hi; the lo lo term is below fp32 rounding), accumulated in fp32 and unscaled on the way out.
//
// The matrix instruction wants, per lane, 8 consecutive values along the reduction index, which here is the row
// index: both operands are transposed on their way into LDS.  A stage is 32 rows x 128 columns of each operand.
// Waves 0-1 stage dy, waves 2-3 stage x: a thread loads 8 rows x 4 columns (eight 16-byte loads), splits the 32
// values and writes, for each of its 4 columns, the 8 row-consecutive halves of each piece with one 16-byte store.
// Column c of the tile lives in LDS row 32 (c % 4) + c / 4, so that the 32 column quads of a wave write 32
// consecutive LDS rows (as the matrix lanes read 32 consecutive rows); the epilogue undoes the permutation.  Two
// stage buffers: while one is multiplied the next stage is split into the other and the loads of the one after are
// in flight.
constexpr int kFTile = 128;                        // dW tile edge
constexpr int kFRows = 32;                         // rows per stage: two matrix steps of 16
constexpr int kFRowW = 64;                         // bytes per LDS row: 32 halves in four 16-byte pieces, piece k of
                                                   // row R at position k ^ ((R >> 2) & 3): 16 consecutive rows
                                                   // touch every bank once, in writes and in reads
constexpr int kFPlane = kFTile * kFRowW;           // bytes of one piece of one operand
constexpr int kFBuf = 4 * kFPlane;                 // one stage: two operands x two pieces
constexpr int kFParts = 1024;                      // partial maxima per operand
constexpr int kFRun = 4096;                        // rows per accumulation run (a multiple of kFRows)

// parts[b] = max |x| over the b-th share of n floats (n % 4 == 0, x 16-byte aligned)
__global__ void __launch_bounds__(256) absmax_parts_kernel(const float* __restrict__ x, long n,
                                                           float* __restrict__ parts) {
    float m = 0.f;
    const long n4 = n >> 2, stride = (long)gridDim.x * 256;
    const float4* x4 = reinterpret_cast<const float4*>(x);
    long k = (long)blockIdx.x * 256 + threadIdx.x;
    for (; k + 3 * stride < n4; k += 4 * stride) {
        const float4 a = x4[k], b = x4[k + stride], c = x4[k + 2 * stride], d = x4[k + 3 * stride];
        m = fmaxf(m, fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w))));
        m = fmaxf(m, fmaxf(fmaxf(fabsf(b.x), fabsf(b.y)), fmaxf(fabsf(b.z), fabsf(b.w))));
        m = fmaxf(m, fmaxf(fmaxf(fabsf(c.x), fabsf(c.y)), fmaxf(fabsf(c.z), fabsf(c.w))));
        m = fmaxf(m, fmaxf(fmaxf(fabsf(d.x), fabsf(d.y)), fmaxf(fabsf(d.z), fabsf(d.w))));
    }
    for (; k < n4; k += stride) {
        const float4 a = x4[k];
        m = fmaxf(m, fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w))));
    }
    for (int d = 1; d < 64; d <<= 1) m = fmaxf(m, __shfl_xor(m, d));
    __shared__ float wave_max[4];
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) parts[blockIdx.x] = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
}
// the same for an array of any length and alignment (bounds handed in by the caller)
__global__ void __launch_bounds__(256) absmax_parts_scalar_kernel(const float* __restrict__ x, long n,
                                                                  float* __restrict__ parts) {
    float m = 0.f;
    for (long k = (long)blockIdx.x * 256 + threadIdx.x; k < n; k += (long)gridDim.x * 256) m = fmaxf(m, fabsf(x[k]));
    for (int d = 1; d < 64; d <<= 1) m = fmaxf(m, __shfl_xor(m, d));
    __shared__ float wave_max[4];
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) parts[blockIdx.x] = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
}

__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) wgrad_f16x2_kernel(const float* __restrict__ dy, const float* __restrict__ x,
                                                          const float* __restrict__ dy_parts, int n_dy_parts,
                                                          const float* __restrict__ x_parts, int n_x_parts,
                                                          long R, int I, int O, long rows_per_block,
                                                          float* __restrict__ part, float* __restrict__ colsum_part) {
    // [stage buffer][operand: dy, x][piece: hi, lo][LDS row][64 bytes]
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kFBuf];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int m = lane & 31, g = lane >> 5;
    const int o_tile = blockIdx.x * kFTile, i_tile = blockIdx.y * kFTile;
    const long r_lo = (long)blockIdx.z * rows_per_block;
    const long r_hi = r_lo + rows_per_block < R ? r_lo + rows_per_block : R;

    float scale = 0.f, unscale = 0.f;                      // (set by set_scales below)
    // staging role of this thread: operand (wave-uniform), 8 rows from row 8 * octet, columns 4 cq .. 4 cq + 3.
    // A stage is the 32 rows from `first`; the last stage of a slice starts at r_hi - 32, inside the matrix
    // (rows >= 32), and the rows it shares with the stage before, or with the slice before, are scaled by zero, as
    // are the columns past the matrix (read from column 0): every load is unconditional and in bounds, and its
    // address is a uniform row address plus a constant lane offset.
    const bool stage_x = wave >= 2;
    const int st = threadIdx.x & 127, octet = st >> 5, cq = st & 31;
    const int dim = stage_x ? I : O, tile0 = stage_x ? i_tile : o_tile;
    const bool col_ok = tile0 + 4 * cq < dim;
    const float* operand = stage_x ? x : dy;                                       // (uniform)
    const unsigned lane_off = (unsigned)(8 * octet * dim + (col_ok ? tile0 + 4 * cq : 0));
    // LDS rows cq + 32 j: their swizzle term ((row >> 2) & 3) does not depend on j
    unsigned char* st_dst = lds + (stage_x ? 2 * kFPlane : 0) + cq * kFRowW + 16 * (octet ^ ((cq >> 2) & 3));
    float4 v[8];
    auto first_row = [&](long r) { return r + kFRows <= r_hi ? r : r_hi - kFRows; };
    auto fetch = [&](long r) {
        const float* rows = operand + first_row(r) * dim;                          // (uniform)
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = *reinterpret_cast<const float4*>(rows + u * dim + lane_off);
    };
    // column sums of dy over the slice (the bias gradient), by the workgroups of the first column of tiles
    const bool sum_cols = colsum_part != nullptr && blockIdx.y == 0 && !stage_x;   // (uniform)
    float4 colsum = make_float4(0.f, 0.f, 0.f, 0.f);
    auto store = [&](long r, int buf_off) {
        const int first_live = (int)(r - first_row(r)) - 8 * octet;                // rows u >= first_live count
        halfx8 hi[4], lo[4];
        if (sum_cols) {
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const float w = (u >= first_live && r < r_hi) ? 1.f : 0.f;
                colsum.x += w * v[u].x; colsum.y += w * v[u].y; colsum.z += w * v[u].z; colsum.w += w * v[u].w;
            }
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const HalfSplit4 p = split(v[u], u >= first_live ? scale : 0.f);
#pragma unroll
            for (int j = 0; j < 4; j++) { hi[j][u] = p.hi[j]; lo[j][u] = p.lo[j]; }
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            *reinterpret_cast<halfx8*>(st_dst + buf_off + 32 * j * kFRowW) = hi[j];
            *reinterpret_cast<halfx8*>(st_dst + buf_off + kFPlane + 32 * j * kFRowW) = lo[j];
        }
    };

    // the two scales, from the partial maxima
    auto set_scales = [&]() {
    // (16-byte loads, four of them requested before the first is used: up to 64 values per thread and array)
    auto absmax_of = [&](const float* __restrict__ p, int n) {
        float mx = 0.f;
        const int n4 = (reinterpret_cast<uintptr_t>(p) & 15) == 0 ? n / 4 : 0;
        const float4* p4 = reinterpret_cast<const float4*>(p);
        auto fold = [&](const float4 t) {
            mx = fmaxf(fmaxf(mx, fmaxf(fabsf(t.x), fabsf(t.y))), fmaxf(fabsf(t.z), fabsf(t.w)));
        };
        int k = threadIdx.x;
        for (; k + 3 * 256 < n4; k += 4 * 256) {
            const float4 t0 = p4[k], t1 = p4[k + 256], t2 = p4[k + 512], t3 = p4[k + 768];
            fold(t0); fold(t1); fold(t2); fold(t3);
        }
        for (; k < n4; k += 256) fold(p4[k]);
        for (int j = 4 * n4 + threadIdx.x; j < n; j += 256) mx = fmaxf(mx, fabsf(p[j]));
        return mx;
    };
    float ma = absmax_of(dy_parts, n_dy_parts), mb = absmax_of(x_parts, n_x_parts);
    for (int d = 1; d < 64; d <<= 1) { ma = fmaxf(ma, __shfl_xor(ma, d)); mb = fmaxf(mb, __shfl_xor(mb, d)); }
    float* wave_max = reinterpret_cast<float*>(lds);
    if (lane == 0) { wave_max[wave] = ma; wave_max[4 + wave] = mb; }
    __syncthreads();
    ma = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
    mb = fmaxf(fmaxf(wave_max[4], wave_max[5]), fmaxf(wave_max[6], wave_max[7]));
    __syncthreads();
    float inv_a, inv_b;
    const float scale_a = pow2_scale(ma, &inv_a), scale_b = pow2_scale(mb, &inv_b);
    scale = col_ok ? (stage_x ? scale_b : scale_a) : 0.f;
    unscale = inv_a * inv_b;
    };

    floatx16 acc[2][2];
#pragma unroll
    for (int p = 0; p < 2; p++)
#pragma unroll
        for (int q = 0; q < 2; q++)
#pragma unroll
            for (int k = 0; k < 16; k++) acc[p][q][k] = 0.f;

    // matrix lanes: LDS rows 64 (wave / 2) + 32 p + m of dy, 64 (wave % 2) + 32 q + m of x; 16-byte piece 2 step + g,
    // swizzled with (row >> 2) & 3 = (m >> 2) & 3
    const int sw = (m >> 2) & 3;
    const unsigned char* a_lds = lds + ((wave >> 1) * 64 + m) * kFRowW;
    const unsigned char* b_lds = lds + 2 * kFPlane + ((wave & 1) * 64 + m) * kFRowW;
    auto multiply = [&](int buf_off) {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const int piece = buf_off + 16 * ((2 * s + g) ^ sw);
            halfx8 ah[2], al[2], bh[2], bl[2];
#pragma unroll
            for (int p = 0; p < 2; p++) {
                ah[p] = *reinterpret_cast<const halfx8*>(a_lds + piece + 32 * p * kFRowW);
                al[p] = *reinterpret_cast<const halfx8*>(a_lds + piece + kFPlane + 32 * p * kFRowW);
                bh[p] = *reinterpret_cast<const halfx8*>(b_lds + piece + 32 * p * kFRowW);
                bl[p] = *reinterpret_cast<const halfx8*>(b_lds + piece + kFPlane + 32 * p * kFRowW);
            }
#pragma unroll
            for (int p = 0; p < 2; p++)
#pragma unroll
                for (int q = 0; q < 2; q++) {
                    // small terms first
                    acc[p][q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[p], bh[q], acc[p][q], 0, 0, 0);
                    acc[p][q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[p], bl[q], acc[p][q], 0, 0, 0);
                    acc[p][q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[p], bh[q], acc[p][q], 0, 0, 0);
                }
        }
    };

    // a stage is multiplied out of one buffer while the next one is split into the other and the loads of the one
    // after that are on their way
    // (stages past the slice are fetched and stored like the others, scaled by zero and never multiplied: the loop
    // body has no branch, and the splitting of one stage can be issued between the matrix instructions of another)
    fetch(r_lo);
    set_scales();                                          // (the first stage is on its way meanwhile)
    store(r_lo, 0);
    fetch(r_lo + kFRows);
    __syncthreads();
    // The matrix instructions accumulate runs of kFRun rows; the runs are added in a second set of registers: the
    // rounding error of an fp32 sum grows with its length, and a slice of 50 000 rows in one chain was 1.7 times
    // less accurate than the same sum in chunks.
    floatx16 total[2][2];
#pragma unroll
    for (int p = 0; p < 2; p++)
#pragma unroll
        for (int q = 0; q < 2; q++)
#pragma unroll
            for (int k = 0; k < 16; k++) total[p][q][k] = 0.f;
    int buf_off = 0;
    for (long r = r_lo; r < r_hi;) {
        const long run_hi = r + kFRun < r_hi ? r + kFRun : r_hi;
        for (; r < run_hi; r += kFRows) {
            multiply(buf_off);
            buf_off ^= kFBuf;
            store(r + kFRows, buf_off);
            fetch(r + 2 * kFRows);
#pragma unroll
            for (int k = 0; k < 24; k++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     // one matrix instruction,
                __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);     // seven vector instructions in its shadow
            }
            __syncthreads();
        }
#pragma unroll
        for (int p = 0; p < 2; p++)
#pragma unroll
            for (int q = 0; q < 2; q++)
#pragma unroll
                for (int k = 0; k < 16; k++) { total[p][q][k] += acc[p][q][k]; acc[p][q][k] = 0.f; }
    }
    if (colsum_part != nullptr && blockIdx.y == 0) {                              // (uniform)
        // the four row groups of a column quad, added in a fixed order
        float4* sums = reinterpret_cast<float4*>(lds);                             // [octet][cq]; the stage buffers are done with
        if (!stage_x) sums[octet * 32 + cq] = colsum;
        __syncthreads();
        if (threadIdx.x < 32) {
            const float4 s0 = sums[cq], s1 = sums[32 + cq], s2 = sums[64 + cq], s3 = sums[96 + cq];
            const int o = o_tile + 4 * cq;
            if (o < O)
                *reinterpret_cast<float4*>(colsum_part + (long)blockIdx.z * O + o) =
                    make_float4((s0.x + s1.x) + (s2.x + s3.x), (s0.y + s1.y) + (s2.y + s3.y),
                                (s0.z + s1.z) + (s2.z + s3.z), (s0.w + s1.w) + (s2.w + s3.w));
        }
    }
    // D[row][col]: col = lane % 32, row = 8 (k / 4) + 4 (lane / 32) + k % 4 for register k; LDS row 32 j + c / 4 of
    // an operand is column 4 (c / 4) + j of the tile
    float* plane = part + (long)blockIdx.z * O * I;
#pragma unroll
    for (int p = 0; p < 2; p++)
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const int i = i_tile + 4 * m + 2 * (wave & 1) + q;
#pragma unroll
            for (int k = 0; k < 16; k++) {
                const int o = o_tile + 4 * (8 * (k / 4) + 4 * g + (k % 4)) + 2 * (wave >> 1) + p;
                if (o < O && i < I) plane[(long)o * I + i] = total[p][q][k] * unscale;
            }
        }
}

// dW[k] = part[0][k] + part[1][k] + ... in this order
__global__ void __launch_bounds__(256) wgrad_reduce_kernel(const float* __restrict__ part, long n, int splits,
                                                           float* __restrict__ dW) {
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
        dW[k] = s;
    }
}

// the same for two sets of planes in one launch (the weight gradient and the column sums)
__global__ void __launch_bounds__(256) wgrad_reduce2_kernel(const float* __restrict__ part_a, long n_a,
                                                            float* __restrict__ out_a,
                                                            const float* __restrict__ part_b, long n_b,
                                                            float* __restrict__ out_b, int splits) {
    for (long k = (long)blockIdx.x * blockDim.x + threadIdx.x; k < n_a + n_b; k += (long)gridDim.x * blockDim.x) {
        const bool first = k < n_a;
        const float* src = first ? part_a + k : part_b + (k - n_a);
        const long stride = first ? n_a : n_b;
        float s = 0.f;
        int z = 0;
        for (; z + 8 <= splits; z += 8) {                  // eight loads in flight, added in slice order
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = src[(long)(z + u) * stride];
#pragma unroll
            for (int u = 0; u < 8; u++) s += v[u];
        }
        for (; z < splits; z++) s += src[(long)z * stride];
        if (first) out_a[k] = s; else out_b[k - n_a] = s;
    }
}

// rows per slice and number of slices for a problem (the same on the sizing and the launching side)
// resident_groups = 0: aim at ~4 workgroups per CU; otherwise the number of workgroups the chip holds at once, which
// the grid then does not exceed (a second, partly filled round would cost a whole slice's time)
void wgrad_split(long rows, int dim_in, int dim_out, int tile, long* rows_per_block, long* splits,
                 long resident_groups = 0) {
    const int gx = (int)ceil_div(dim_out, tile), gy = (int)ceil_div(dim_in, tile);
    long s = resident_groups > 0 ? resident_groups / ((long)gx * gy) : ceil_div(1024, (long)gx * gy);
    const long max_splits = ceil_div(rows, 64);
    if (s > max_splits) s = max_splits;
    if (s < 1) s = 1;
    if (s > 65535) s = 65535;
    long rpb = ceil_div(rows, s);
    rpb = ceil_div(rpb, 32) * 32;                      // (a multiple of every kernel's rows per trip)
    *rows_per_block = rpb;
    *splits = rows > 0 ? ceil_div(rows, rpb) : 0;
}
// plain rows take the matrix-core kernel and its 128 x 128 tiles
inline int wgrad_tile(int inds) { return inds == 0 ? kMTile : kTile; }

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_tensor_linear_wgrad_workspace_bytes(long rows, int dim_in, int dim_out, size_t* bytes) {
    MG_REQUIRE(bytes != nullptr && rows >= 0 && dim_in >= 0 && dim_out >= 0, "mg_tensor_linear_wgrad_workspace_bytes: bad argument");
    // (the number of tensor indices is not known here: room for either kernel's slices)
    long rpb, s_plain, s_comp;
    wgrad_split(rows, dim_in, dim_out, kMTile, &rpb, &s_plain);
    wgrad_split(rows, dim_in, dim_out, kTile, &rpb, &s_comp);
    const long splits = s_plain > s_comp ? s_plain : s_comp;
    // (+ the partial maxima and the column sums of the split-fp16 variant)
    *bytes = (size_t)splits * ((size_t)dim_in + 1) * (size_t)dim_out * sizeof(float) + 16 + 2 * kFParts * sizeof(float);
    return MG_OK;
}

int mg_tensor_linear_wgrad_f16x2_supported(long rows, int dim_in, int dim_out) {
    return rows >= 4096 && dim_in >= 4 && dim_out >= 4 && dim_in % 4 == 0 && dim_out % 4 == 0;
}

int mg_tensor_linear_wgrad_f16x2(const float* dy, const float* x, const float* dy_bound, long n_dy_bound,
                                 const float* x_bound, long n_x_bound, long rows, int dim_in, int dim_out,
                                 void* workspace, float* dW, float* db, mg_stream_t stream) {
    MG_REQUIRE(mg_tensor_linear_wgrad_f16x2_supported(rows, dim_in, dim_out),
               "mg_tensor_linear_wgrad_f16x2: needs rows >= 4096 and dims that are multiples of 4");
    MG_REQUIRE(dy && x && workspace && dW, "mg_tensor_linear_wgrad_f16x2: null pointer");
    MG_REQUIRE(aligned16(dy) && aligned16(x), "mg_tensor_linear_wgrad_f16x2: dy and x must be 16-byte aligned");
    MG_REQUIRE((dy_bound == nullptr || n_dy_bound > 0) && (x_bound == nullptr || n_x_bound > 0),
               "mg_tensor_linear_wgrad_f16x2: empty bound array");
    hipStream_t st = (hipStream_t)stream;
    const long n = (long)dim_in * dim_out;
    long rpb, splits;
    // two workgroups per CU fit; with node-sized operands one per CU is faster (longer slices, half the partial
    // results to write and add up: 4096 x 512 x 512 29 against 35 us, 12288 x 128 x 384 26 against 30 us;
    // 101000 x 512 x 512 281 against 238 us)
    wgrad_split(rows, dim_in, dim_out, kFTile, &rpb, &splits, rows < 65536 ? 256 : 512);
    float* part = reinterpret_cast<float*>((reinterpret_cast<uintptr_t>(workspace) + 15) & ~uintptr_t(15));
    float* maxima = part + splits * n;                       // [dy: kFParts][x: kFParts]
    float* colsum_part = db ? maxima + 2 * kFParts : nullptr; // [slice][dim_out]
    constexpr long kDirectBounds = 16384;                    // a bound array this short is read by every workgroup itself
    auto bound_parts = [&](const float* data, long count, const float* bound, long n_bound, float* parts) -> int {
        // partial maxima of the caller's bounds, or of the data itself
        if (bound && n_bound <= kDirectBounds) return (int)n_bound;
        const float* from = bound ? bound : data;
        const long len = bound ? n_bound : count;
        const int blocks = (int)(ceil_div(len, 4096) < kFParts ? ceil_div(len, 4096) : kFParts);
        if (bound)
            hipLaunchKernelGGL(absmax_parts_scalar_kernel, dim3(blocks), dim3(256), 0, st, from, len, parts);
        else
            hipLaunchKernelGGL(absmax_parts_kernel, dim3(blocks), dim3(256), 0, st, from, len, parts);
        return blocks;
    };
    const int na = bound_parts(dy, rows * dim_out, dy_bound, n_dy_bound, maxima);
    const int nb = bound_parts(x, rows * dim_in, x_bound, n_x_bound, maxima + kFParts);
    const float* dy_parts = (dy_bound && n_dy_bound <= kDirectBounds) ? dy_bound : maxima;
    const float* x_parts = (x_bound && n_x_bound <= kDirectBounds) ? x_bound : maxima + kFParts;
    dim3 grid((unsigned)ceil_div(dim_out, kFTile), (unsigned)ceil_div(dim_in, kFTile), (unsigned)splits), block(256);
    hipLaunchKernelGGL(wgrad_f16x2_kernel, grid, block, 0, st, dy, x, dy_parts, na, x_parts, nb, rows, dim_in, dim_out,
                       rpb, part, colsum_part);
    const long n_sum = n + (db ? dim_out : 0);
    const unsigned nblocks = (unsigned)(ceil_div(n_sum, 256) < 1024 ? ceil_div(n_sum, 256) : 1024);
    hipLaunchKernelGGL(wgrad_reduce2_kernel, dim3(nblocks), dim3(256), 0, st, (const float*)part, n, dW,
                       (const float*)colsum_part, (long)(db ? dim_out : 0), db, (int)splits);
    return check_launch("mg_tensor_linear_wgrad_f16x2");
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
    const int tile = wgrad_tile(inds);
    wgrad_split(rows, dim_in, dim_out, tile, &rpb, &splits);
    float* part = reinterpret_cast<float*>((reinterpret_cast<uintptr_t>(workspace) + 15) & ~uintptr_t(15));
    const int gx = (int)ceil_div(dim_out, tile), gy = (int)ceil_div(dim_in, tile);
    dim3 grid(gx, gy, (unsigned)splits), block(256);
    switch (inds) {
        case 0:
            if (dim_in % 4 == 0 && dim_out % 4 == 0 && aligned16(dy) && aligned16(x))
                hipLaunchKernelGGL(wgrad_mfma_lds_kernel, grid, block, 0, st, dy, x, rows, dim_in, dim_out, rpb, part);
            else
                hipLaunchKernelGGL(wgrad_mfma_kernel, grid, block, 0, st, dy, x, rows, dim_in, dim_out, rpb, part);
            break;
        case 1: hipLaunchKernelGGL(wgrad_kernel<3>, grid, block, 0, st, dy, x, rows, dim_in, dim_out, rpb, part); break;
        default: hipLaunchKernelGGL(wgrad_kernel<9>, grid, block, 0, st, dy, x, rows, dim_in, dim_out, rpb, part); break;
    }
    hipLaunchKernelGGL(wgrad_reduce_kernel, dim3(nblocks), dim3(256), 0, st, (const float*)part, n, (int)splits, dW);
    return check_launch("mg_tensor_linear_wgrad");
}

}  // extern "C"
