// Two kernels that end a per-edge GEMM with a sum over the edges of each node, so that the per-edge
// result is never stored: the PaiNN message (below) and a plain linear layer whose rows are only
// needed summed per segment (linear_rowsum_f16x2_kernel, further down).
//
// PaiNN message with the last layer of the filter MLP folded in: the per-edge filter
//     W(e) = h(e) W3^T + b3            (h: (edges, hidden) output of the MLP's second layer, W3: (4n, hidden))
// is produced tile by tile on the matrix cores and consumed in the same kernel by
//     P = W(e) * A(j),  m_v = v(j) P0 + (v(j) x u) P1 + u (x) P2,  m_a = P3,   out(i) = res(i) + sum_e m(e)
// (archs/meanflow_painn8.py:77-100), so the (edges, 4n) filter never exists in memory.
//
// * The GEMM is the split-fp16 row-streaming kernel (three MFMAs per product, fp32 accumulate,
//   per-row power-of-two scales) with the operands swapped: W is the FIRST matrix operand, so an
//   accumulator register holds one EDGE (lane % 32) and four consecutive filter columns.  A lane
//   then owns its edge's neighbour index and direction, and gathers A(j) / v(j) as 16-byte pieces.
// * The rows of W3 are packed in the order (channel block of 64, k = 0..3, channel in block): one
//   256-column tile holds all four filter blocks of 64 channels, i.e. everything the message of
//   those channels needs.
// * Edges are sorted by receiving node.  A wave reduces its 32 edges through its slice of LDS
//   (free once the main loop is over): lanes take one output column each and walk the 32 rows,
//   flushing at the row boundaries of the graph.  A run of edges that starts at the first row of
//   the wave's block goes to partial slot A of the block, a run that starts later and ends at the
//   block's last row to slot B, a run strictly inside the block is a whole node and is written
//   directly (plus the residual).  A second small kernel adds the slots of every node in block
//   order: fixed summation order, no atomics.
#include "common.hpp"
#include "f16x2.hpp"
#include "rowsum_finish.hpp"

namespace mg {
namespace {

constexpr int kFW = 8;                       // waves per workgroup
constexpr int kFTM = 32 * kFW;               // edges per tile
constexpr int kFTN = 256;                    // filter columns per tile: 4 blocks x 64 channels
constexpr int kFNI = kFTN / 32;

__device__ __forceinline__ float4 ldf4(const float* p) { return *reinterpret_cast<const float4*>(p); }

template <int ACT>
__device__ __forceinline__ float activate_c(float v) {
    // 1: SiLU through the hardware exp2 and reciprocal (about 1 ulp each); 2: LeakyReLU(0.1)
    if constexpr (ACT == 1) return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    if constexpr (ACT == 2) return v > 0.f ? v : 0.1f * v;
    return v;
}

constexpr int kFThreads = 64 * kFW;
constexpr int kFPlaneW = kFTN * kRowW, kFBufW = 2 * kFPlaneW;   // bytes of one W plane / of both planes of a chunk
constexpr int kFSlice = 2 * kFBufW / kFW / 4;                    // floats of LDS per wave once the main loop is over
constexpr int kFRed = 68;                                        // floats per row of a slice: 64 + 4 (spreads 16-byte writes over the banks)
static_assert(kFSlice >= 32 * kFRed, "a reduction pass needs 32 rows x 64 columns per wave");

// Source of the second operand: the 16 values x[row][k0 + 16 g ..] of this lane's row for chunk k0, from memory
struct RowFromMemory {
    static constexpr bool kAhead = true;      // requested two chunks before use (HBM latency)
    const float* xrow;       // this lane's row of x, offset by 16 (lane / 32)
    int I;
    __device__ __forceinline__ void operator()(float4 (&v)[4], int k0) const {
        k0 = k0 < I ? k0 : I - kCK;                       // surplus requests of the last trips are never used
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = *reinterpret_cast<const float4*>(xrow + k0 + 4 * j);
    }
};

// acc[ni][q] += sum_k W[n0 + 32 ni + i][k] x[row][k] for the wave's 32 rows (row = lane % 32) and the tile's 256
// columns, i = 8 (q / 4) + 4 (lane / 32) + q % 4: the split-fp16 row-streaming main loop with W as the first
// matrix operand.  a_src(v, k0) delivers the lane's 16 values of x for chunk k0 (two chunks ahead of their use);
// lds: 2 * kFBufW bytes; all waves of the workgroup call it together, and the W buffers are free again when it
// returns.
template <typename ASrc>
__device__ __forceinline__ void wfirst_gemm_tile(floatx16 (&acc)[kFNI], const _Float16* __restrict__ Wp,
                                                 long plane_elems, int n0, const ASrc& a_src, int I,
                                                 float sx, unsigned char* lds) {
    constexpr int THREADS = kFThreads, kPlaneW = kFPlaneW, kBufW = kFBufW;
    constexpr int kPer = 8 * kFTN / THREADS;                 // 16-byte pieces of W per thread and chunk
    const int tid = threadIdx.x;
    const int m = tid & 31, g = (tid >> 5) & 1;
    const _Float16* wsrc[kPer];
    int wdst[kPer];
#pragma unroll
    for (int j = 0; j < kPer; j++) {
        const int q = tid + THREADS * j;
        const int plane = q / (4 * kFTN), row = (q % (4 * kFTN)) >> 2, piece = q & 3;
        wsrc[j] = Wp + plane * plane_elems + (long)(n0 + row) * I + 8 * piece;
        wdst[j] = plane * kPlaneW + row * kRowW + piece * 16;
    }
    const int k_last = I - kCK;

    struct ARegs { float4 v[4]; };
    struct WRegs { halfx8 v[kPer]; };
    auto load_a = [&](ARegs& a, int k0) { a_src(a.v, k0); };
    auto load_w = [&](WRegs& w, int k0) {
        k0 = k0 < I ? k0 : k_last;
#pragma unroll
        for (int j = 0; j < kPer; j++) w.v[j] = *reinterpret_cast<const halfx8*>(wsrc[j] + k0);
    };
    auto store_w = [&](const WRegs& w, unsigned char* buf) {
#pragma unroll
        for (int j = 0; j < kPer; j++) *reinterpret_cast<halfx8*>(buf + wdst[j]) = w.v[j];
    };
    const int b_off = m * kRowW + 32 * g;
    auto compute = [&](const ARegs& a, const unsigned char* buf, float scale) {
        halfx8 ah[2], al[2];
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const HalfSplit4 p0 = split(a.v[2 * s], scale), p1 = split(a.v[2 * s + 1], scale);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                ah[s][i] = p0.hi[i]; ah[s][4 + i] = p1.hi[i];
                al[s][i] = p0.lo[i]; al[s][4 + i] = p1.lo[i];
            }
        }
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
            for (int ni = 0; ni < kFNI; ni++) {
                const halfx8 bh = *reinterpret_cast<const halfx8*>(buf + b_off + ni * 32 * kRowW + 16 * s);
                const halfx8 bl = *reinterpret_cast<const halfx8*>(buf + kPlaneW + b_off + ni * 32 * kRowW + 16 * s);
                // W first: D[i][j] with i the filter column in the block and j the edge
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bh, al[s], acc[ni], 0, 0, 0);
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bl, ah[s], acc[ni], 0, 0, 0);
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bh, ah[s], acc[ni], 0, 0, 0);
            }
    };

    unsigned char* buf0 = lds;
    unsigned char* buf1 = lds + kBufW;
    WRegs w;
    if constexpr (ASrc::kAhead) {
        ARegs a0, a1;
        load_w(w, 0);
        load_a(a0, 0);
        store_w(w, buf0);
        load_w(w, kCK);
        load_a(a1, kCK);
        __syncthreads();
        for (int k0 = 0; k0 < I; k0 += 2 * kCK) {
            compute(a0, buf0, sx);
            store_w(w, buf1);
            __builtin_amdgcn_sched_barrier(0);
            load_w(w, k0 + 2 * kCK);
            __builtin_amdgcn_sched_barrier(0);
            load_a(a0, k0 + 2 * kCK);
            __syncthreads();
            compute(a1, buf1, k0 + kCK < I ? sx : 0.f);
            store_w(w, buf0);
            __builtin_amdgcn_sched_barrier(0);
            load_w(w, k0 + 3 * kCK);
            __builtin_amdgcn_sched_barrier(0);
            load_a(a1, k0 + 3 * kCK);
            __syncthreads();
        }
    } else {
        ARegs a;
        load_w(w, 0);
        store_w(w, buf0);
        load_w(w, kCK);
        __syncthreads();
        for (int k0 = 0; k0 < I; k0 += 2 * kCK) {
            load_a(a, k0);
            compute(a, buf0, sx);
            store_w(w, buf1);
            __builtin_amdgcn_sched_barrier(0);
            load_w(w, k0 + 2 * kCK);
            __syncthreads();
            load_a(a, k0 + kCK);
            compute(a, buf1, k0 + kCK < I ? sx : 0.f);
            store_w(w, buf0);
            __builtin_amdgcn_sched_barrier(0);
            load_w(w, k0 + 3 * kCK);
            __syncthreads();
        }
    }
}

__global__ void __launch_bounds__(64 * kFW)
painn_filter_message_kernel(const _Float16* __restrict__ Wp, const float* __restrict__ w_inv,
                            const float* __restrict__ bias, const float* __restrict__ X,
                            const float* __restrict__ xmax, int xmax_parts, long xmax_stride, long R, int I,
                            const int* __restrict__ src, const int* __restrict__ dst, const float* __restrict__ r_ij,
                            const float* __restrict__ actv, const float* __restrict__ x_v, int n, float epsilon,
                            const float* __restrict__ res_a, const float* __restrict__ res_v,
                            float* __restrict__ slots, long n_blocks, float* __restrict__ out_a,
                            float* __restrict__ out_v, int tiles_n, long tiles_total) {
    constexpr int kSlice = kFSlice, kRed = kFRed;
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kFBufW];
    __shared__ __attribute__((aligned(16))) float wb[2 * kFTN];   // the tile's 1 / weight scale, then its bias

    const long bid = blockIdx.x;
    const long per_xcd = (tiles_total + 7) / 8;
    const long logical = (bid % 8) * per_xcd + bid / 8;
    if (logical >= tiles_total) return;
    const long tile_m = logical / tiles_n;
    const int tile_n = (int)(logical - tile_m * tiles_n);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, g = lane >> 5;
    const long r0 = tile_m * kFTM;
    const int n0 = tile_n * kFTN;
    const long plane_elems = (long)tiles_n * kFTN * I;

    floatx16 acc[kFNI];
#pragma unroll
    for (int ni = 0; ni < kFNI; ni++)
#pragma unroll
        for (int q = 0; q < 16; q++) acc[ni][q] = 0.f;

    const long block = r0 / 32 + wave;                       // this wave's block of 32 edges
    const long my_row = block * 32 + m;
    const long ld_row = my_row < R ? my_row : R - 1;
    const float* xrow = X + ld_row * I + 16 * g;
    float sx, isx;
    {
        float amax = 0.f;
        const float* xm = xmax + ld_row * xmax_stride;
        for (int p = 0; p < xmax_parts; p++) amax = fmaxf(amax, xm[p]);
        sx = pow2_scale(amax, &isx);
    }
    // the edge this lane owns in the epilogue
    const int my_src = src[ld_row];
    const long my_j = dst[ld_row];
    float ux = r_ij[3 * ld_row], uy = r_ij[3 * ld_row + 1], uz = r_ij[3 * ld_row + 2];

    if (tid < kFTN) {
        wb[tid] = w_inv[n0 + tid];
        wb[kFTN + tid] = bias[n0 + tid];
    }
    wfirst_gemm_tile(acc, Wp, plane_elems, n0, RowFromMemory{xrow, I}, I, sx, lds);
    // every wave is past its last read of the W buffers: LDS is now eight private slices

    const bool valid = my_row < R;
    {
        const float inv = 1.0f / sqrtf(epsilon + (ux * ux + uy * uy + uz * uz));
        ux *= inv; uy *= inv; uz *= inv;
    }
    // runs of equal receiving node among the wave's rows: bit r set = row r starts a run
    const long rows_left = R - block * 32;
    const int nv = rows_left >= 32 ? 32 : (rows_left > 0 ? (int)rows_left : 0);
    const int prev_src = __shfl_up(my_src, 1);
    const unsigned starts = (unsigned)__ballot(g == 0 && (m == 0 || my_src != prev_src));
    const int runs = __popc(starts);
    const int second = runs >= 2 ? __ffs(starts & ~1u) - 1 : 32;      // first row of the second run
    float* slice = reinterpret_cast<float*>(lds) + wave * kSlice;
    const int cb = 64 * tile_n;                               // first channel of this tile
    const long row4n = 4L * n;
    const float* arow = actv + my_j * row4n;
    const float* vrow = x_v + my_j * 3L * n;
    float* slot_a = slots + block * row4n;
    float* slot_b = slots + (n_blocks + block) * row4n;
    const float keep = valid ? 1.f : 0.f;                     // rows past the end add nothing

    // gathered operands of one group: 4 consecutive channels, all four filter blocks
    struct Gather { float4 a[4], v[3]; };
    auto gather = [&](Gather& t, int gidx) {
        const int c = cb + 32 * (gidx >> 2) + 8 * (gidx & 3) + 4 * g;
#pragma unroll
        for (int k = 0; k < 4; k++) t.a[k] = ldf4(arow + k * n + c);
#pragma unroll
        for (int k = 0; k < 3; k++) t.v[k] = ldf4(vrow + 3 * c + 4 * k);
    };
    auto flush = [&](float sum, int run_start, int r, long off_v, long off_a, bool is_v) {
        // the run [run_start, r] of this wave's rows is complete; the same branch for every lane
        const long off_slot = is_v ? off_v : 3L * n + off_a;
        if (run_start == 0) {
            slot_a[off_slot] = sum;
        } else if (r == 31) {
            slot_b[off_slot] = sum;
        } else {
            const long node = __shfl(my_src, r);
            if (is_v) {
                const long at = node * 3L * n + off_v;
                out_v[at] = (res_v ? res_v[at] : 0.f) + sum;
            } else {
                const long at = node * n + off_a;
                out_a[at] = (res_a ? res_a[at] : 0.f) + sum;
            }
        }
    };

    Gather cur, nxt;
    gather(cur, 0);
#pragma unroll
    for (int gidx = 0; gidx < 8; gidx++) {
        // the next group's gathers fly during this group's arithmetic and the reduction
        gather(nxt, gidx < 7 ? gidx + 1 : 7);
        __builtin_amdgcn_sched_barrier(0);
        const int h = gidx >> 2, qq = gidx & 3, gi = gidx & 1;
        const int cl = 32 * h + 8 * qq + 4 * g;               // channel in the tile's block of 64
        float4 p[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const float4 iw = *reinterpret_cast<const float4*>(wb + 64 * k + cl);
            const float4 bv = *reinterpret_cast<const float4*>(wb + 256 + 64 * k + cl);
            const float4 a = cur.a[k];
            const floatx16& t = acc[2 * k + h];
            p[k].x = (t[4 * qq + 0] * isx * iw.x + bv.x) * a.x;
            p[k].y = (t[4 * qq + 1] * isx * iw.y + bv.y) * a.y;
            p[k].z = (t[4 * qq + 2] * isx * iw.z + bv.z) * a.z;
            p[k].w = (t[4 * qq + 3] * isx * iw.w + bv.w) * a.w;
        }
        const float4 v0 = cur.v[0], v1 = cur.v[1], v2 = cur.v[2];
        const float vv[12] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w, v2.x, v2.y, v2.z, v2.w};
        const float q0[4] = {p[0].x, p[0].y, p[0].z, p[0].w}, q1[4] = {p[1].x, p[1].y, p[1].z, p[1].w};
        const float q2[4] = {p[2].x, p[2].y, p[2].z, p[2].w};
        float o[12];
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const float x = vv[3 * t], y = vv[3 * t + 1], z = vv[3 * t + 2];
            const float cx = y * uz - z * uy, cy = z * ux - x * uz, cz = x * uy - y * ux;   // v x u
            o[3 * t + 0] = x * q0[t] + cx * q1[t] + ux * q2[t];
            o[3 * t + 1] = y * q0[t] + cy * q1[t] + uy * q2[t];
            o[3 * t + 2] = z * q0[t] + cz * q1[t] + uz * q2[t];
        }
        // row m of the slice: 64 floats = [g][gi][12 of m_v, 4 of m_a]
        float* wr = slice + m * kRed + g * 32 + gi * 16;
        *reinterpret_cast<float4*>(wr) = make_float4(o[0] * keep, o[1] * keep, o[2] * keep, o[3] * keep);
        *reinterpret_cast<float4*>(wr + 4) = make_float4(o[4] * keep, o[5] * keep, o[6] * keep, o[7] * keep);
        *reinterpret_cast<float4*>(wr + 8) = make_float4(o[8] * keep, o[9] * keep, o[10] * keep, o[11] * keep);
        *reinterpret_cast<float4*>(wr + 12) = make_float4(p[3].x * keep, p[3].y * keep, p[3].z * keep, p[3].w * keep);
        cur = nxt;
        if (gi == 0) continue;
        // ---- two groups are in the slice: reduce its 64 columns over the rows
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // lane = output column: which element of the node's outputs it is
        const int cg = lane >> 5, cgi = (lane >> 4) & 1, k16 = lane & 15;
        const int cch = cb + 32 * h + 8 * ((qq & 2) + cgi) + 4 * cg;
        const bool is_v = k16 < 12;
        const long off_v = 3L * cch + k16;                    // in the (n, 3) vector part
        const long off_a = cch + (k16 - 12);                  // in the (n) scalar part
        if (nv > 0) {
            if (runs <= 2) {
                // the usual case: all rows in flight at once, one or two sums, no branches in the loop
                float val[32];
#pragma unroll
                for (int r = 0; r < 32; r++) val[r] = slice[r * kRed + lane];
                float s0 = 0.f, s1 = 0.f;
#pragma unroll
                for (int r = 0; r < 32; r++) {
                    s0 += r < second ? val[r] : 0.f;
                    s1 += r < second ? 0.f : val[r];
                }
                flush(s0, 0, second - 1, off_v, off_a, is_v);
                if (runs == 2) flush(s1, second, nv - 1, off_v, off_a, is_v);
            } else {
                float sum = 0.f;
                int run_start = 0;
                for (int r = 0; r < nv; r++) {
                    sum += slice[r * kRed + lane];
                    if ((r == nv - 1) || ((starts >> (r + 1)) & 1u)) {
                        flush(sum, run_start, r, off_v, off_a, is_v);
                        sum = 0.f;
                        run_start = r + 1;
                    }
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

// y = act(x W^T + bias) for rows sorted by segment (seg[row] ascending), reduced over the rows of each segment
// in the epilogue: out[s] = scale * sum_{rows of s} y[row].  Same tile, same slots A / B per block of 32 rows
// and same finishing pass as the message kernel above; y itself is written only when STORE_Y is set
// (coalesced, from the LDS slice the reduction reads anyway).
template <int ACT, bool STORE_Y>
__global__ void __launch_bounds__(64 * kFW)
linear_rowsum_f16x2_kernel(const _Float16* __restrict__ Wp, const float* __restrict__ w_inv,
                           const float* __restrict__ bias, const float* __restrict__ X,
                           const float* __restrict__ xmax, int xmax_parts, long xmax_stride, long R, int I, int O,
                           const int* __restrict__ seg, float* __restrict__ slots, long n_blocks, float scale,
                           float* __restrict__ Y, float* __restrict__ out, int tiles_n, long tiles_total,
                           float bound_mul, float bound_add) {
    constexpr int kSlice = kFSlice, kRed = kFRed;
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kFBufW];
    __shared__ __attribute__((aligned(16))) float wb[2 * kFTN];   // the tile's 1 / weight scale, then its bias

    const long bid = blockIdx.x;
    const long per_xcd = (tiles_total + 7) / 8;
    const long logical = (bid % 8) * per_xcd + bid / 8;
    if (logical >= tiles_total) return;
    const long tile_m = logical / tiles_n;
    const int tile_n = (int)(logical - tile_m * tiles_n);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, g = lane >> 5;
    const int n0 = tile_n * kFTN;
    const long plane_elems = (long)O * I;

    floatx16 acc[kFNI];
#pragma unroll
    for (int ni = 0; ni < kFNI; ni++)
#pragma unroll
        for (int q = 0; q < 16; q++) acc[ni][q] = 0.f;

    const long block = tile_m * kFW + wave;                  // this wave's block of 32 rows
    const long my_row = block * 32 + m;
    const long ld_row = my_row < R ? my_row : R - 1;
    const float* xrow = X + ld_row * I + 16 * g;
    float sx, isx;
    {
        float amax = 0.f;
        const float* xm = xmax + ld_row * xmax_stride;
        for (int p = 0; p < xmax_parts; p++) amax = fmaxf(amax, xm[p]);
        amax = fmaf(amax, bound_mul, bound_add);             // the caller's bound of |x| is bound_mul * xmax + bound_add
        sx = pow2_scale(amax, &isx);
    }
    const int my_seg = seg[ld_row];
    if (tid < kFTN) {
        wb[tid] = w_inv[n0 + tid];
        wb[kFTN + tid] = bias ? bias[n0 + tid] : 0.f;
    }
    wfirst_gemm_tile(acc, Wp, plane_elems, n0, RowFromMemory{xrow, I}, I, sx, lds);

    const float keep = my_row < R ? 1.f : 0.f;               // rows past the end add nothing
    const long rows_left = R - block * 32;
    const int nv = rows_left >= 32 ? 32 : (rows_left > 0 ? (int)rows_left : 0);
    const int prev_seg = __shfl_up(my_seg, 1);
    const unsigned starts = (unsigned)__ballot(g == 0 && (m == 0 || my_seg != prev_seg));
    const int runs = __popc(starts);
    const int second = runs >= 2 ? __ffs(starts & ~1u) - 1 : 32;
    float* slice = reinterpret_cast<float*>(lds) + wave * kSlice;
    float* slot_a = slots + block * O;
    float* slot_b = slots + (n_blocks + block) * O;

#pragma unroll
    for (int pass = 0; pass < 4; pass++) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int ni = 2 * pass + h;
#pragma unroll
            for (int qq = 0; qq < 4; qq++) {
                const int cl = 32 * ni + 8 * qq + 4 * g;      // column in the tile
                const float4 iw = *reinterpret_cast<const float4*>(wb + cl);
                const float4 bv = *reinterpret_cast<const float4*>(wb + kFTN + cl);
                float4 v;
                v.x = keep * activate_c<ACT>(acc[ni][4 * qq + 0] * isx * iw.x + bv.x);
                v.y = keep * activate_c<ACT>(acc[ni][4 * qq + 1] * isx * iw.y + bv.y);
                v.z = keep * activate_c<ACT>(acc[ni][4 * qq + 2] * isx * iw.z + bv.z);
                v.w = keep * activate_c<ACT>(acc[ni][4 * qq + 3] * isx * iw.w + bv.w);
                *reinterpret_cast<float4*>(slice + m * kRed + 32 * h + 8 * qq + 4 * g) = v;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int col = n0 + 64 * pass + lane;                // lane = output column of this pass
        auto flush = [&](float sum, int run_start, int r) {
            if (run_start == 0) {
                slot_a[col] = sum;
            } else if (r == 31) {
                slot_b[col] = sum;
            } else {
                const long s_id = __shfl(my_seg, r);          // a whole segment inside the block
                out[s_id * O + col] = scale * sum;
            }
        };
        if (nv > 0) {
            float val[32];
#pragma unroll
            for (int r = 0; r < 32; r++) val[r] = slice[r * kRed + lane];
            if constexpr (STORE_Y) {
                float* yp = Y + block * 32 * O + col;
#pragma unroll
                for (int r = 0; r < 32; r++)
                    if (r < nv) yp[(long)r * O] = val[r];
            }
            if (runs <= 2) {
                float s0 = 0.f, s1 = 0.f;
#pragma unroll
                for (int r = 0; r < 32; r++) {
                    s0 += r < second ? val[r] : 0.f;
                    s1 += r < second ? 0.f : val[r];
                }
                flush(s0, 0, second - 1);
                if (runs == 2) flush(s1, second, nv - 1);
            } else {
                float sum = 0.f;
                int run_start = 0;
                for (int r = 0; r < nv; r++) {
                    sum += slice[r * kRed + lane];
                    if ((r == nv - 1) || ((starts >> (r + 1)) & 1u)) {
                        flush(sum, run_start, r);
                        sum = 0.f;
                        run_start = r + 1;
                    }
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

// ---------------------------------------------------------------------------------------------------------
// First two layers of the PaiNN filter MLP from the edge vectors (archs/meanflow_painn8.py:25-35 feeding
// :38-51): y = SiLU(W2 SiLU(W1 enc(|r|) + b1) + b2), y (edges, hidden), with the first layer's output never
// stored.  The first layer has K = 16, exactly one matrix-core step: for every 32-column chunk of its output
// the generator below runs three split-fp16 MFMAs (W1 block x encodings) and lands the chunk in registers in
// the accumulator layout, which IS the operand layout the second layer's main loop wants (lane = edge, 16 of
// the chunk's 32 channels per lane half) up to a fixed permutation of the channels inside a chunk; the caller
// packs W2 with its input channels in that order (position 16 g + p of a chunk holds channel
// 8 (p / 4) + 4 g + p % 4).
constexpr int kHidMax = 512;

struct HiddenFromDistance {
    static constexpr bool kAhead = false;     // built right before use: LDS and matrix-core latency only
    const _Float16* w1h;     // LDS: W1 (hidden, 16) hi / lo halves, each row scaled by a power of two
    const _Float16* w1l;
    const float* w1inv;      // LDS: 1 / (row scale * 2^14)
    const float* b1;         // LDS
    halfx8 eh, el;           // this lane's 8 encodings k = 8 g .. 8 g + 7, times 2^14, as hi + lo
    int I, m, g;
    __device__ __forceinline__ void operator()(float4 (&v)[4], int k0) const {
        k0 = k0 < I ? k0 : I - kCK;
        const halfx8 ah = *reinterpret_cast<const halfx8*>(w1h + (k0 + m) * 16 + 8 * g);
        const halfx8 al = *reinterpret_cast<const halfx8*>(w1l + (k0 + m) * 16 + 8 * g);
        floatx16 d;
#pragma unroll
        for (int q = 0; q < 16; q++) d[q] = 0.f;
        d = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, el, d, 0, 0, 0);
        d = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, eh, d, 0, 0, 0);
        d = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, eh, d, 0, 0, 0);
#pragma unroll
        for (int qq = 0; qq < 4; qq++) {
            const float4 iw = *reinterpret_cast<const float4*>(w1inv + k0 + 8 * qq + 4 * g);
            const float4 bv = *reinterpret_cast<const float4*>(b1 + k0 + 8 * qq + 4 * g);
            v[qq].x = activate_c<1>(d[4 * qq + 0] * iw.x + bv.x);
            v[qq].y = activate_c<1>(d[4 * qq + 1] * iw.y + bv.y);
            v[qq].z = activate_c<1>(d[4 * qq + 2] * iw.z + bv.z);
            v[qq].w = activate_c<1>(d[4 * qq + 3] * iw.w + bv.w);
        }
    }
};

__global__ void __launch_bounds__(64 * kFW)
painn_filter_hidden_kernel(const _Float16* __restrict__ Wp, const float* __restrict__ w_inv,
                           const float* __restrict__ bias2, const float* __restrict__ r_ij, long R, float base,
                           const float* __restrict__ W1, long so, long si, const float* __restrict__ b1g, int hidden,
                           const float* __restrict__ h1_bound, float* __restrict__ Y, int tiles_n, long tiles_total) {
    constexpr int kSlice = kFSlice, kRed = kFRed;
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kFBufW];
    __shared__ __attribute__((aligned(16))) float wb[2 * kFTN];
    __shared__ __attribute__((aligned(16))) _Float16 w1h[kHidMax * 16];
    __shared__ __attribute__((aligned(16))) _Float16 w1l[kHidMax * 16];
    __shared__ __attribute__((aligned(16))) float w1inv[kHidMax];
    __shared__ __attribute__((aligned(16))) float b1s[kHidMax];

    const long bid = blockIdx.x;
    const long per_xcd = (tiles_total + 7) / 8;
    const long logical = (bid % 8) * per_xcd + bid / 8;
    if (logical >= tiles_total) return;
    const long tile_m = logical / tiles_n;
    const int tile_n = (int)(logical - tile_m * tiles_n);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, g = lane >> 5;
    const int n0 = tile_n * kFTN;
    const int I = hidden, O = hidden;
    const long plane_elems = (long)O * I;

    // first-layer weights: one row per thread, split into fp16 hi + lo under a per-row power-of-two scale
    for (int t = tid; t < hidden; t += kFThreads) {
        float wrow[16];
        float amax = 0.f;
#pragma unroll
        for (int k = 0; k < 16; k++) {
            wrow[k] = W1[t * so + k * si];
            amax = fmaxf(amax, fabsf(wrow[k]));
        }
        float inv;
        const float sc = pow2_scale(amax, &inv);
#pragma unroll
        for (int k = 0; k < 16; k++) {
            const float sv = wrow[k] * sc;
            const _Float16 h = (_Float16)sv;
            w1h[t * 16 + k] = h;
            w1l[t * 16 + k] = (_Float16)(sv - (float)h);
        }
        w1inv[t] = inv * (1.0f / 16384.0f);                  // the encodings are scaled by 2^14
        b1s[t] = b1g ? b1g[t] : 0.f;
    }
    if (tid < kFTN) {
        wb[tid] = w_inv[n0 + tid];
        wb[kFTN + tid] = bias2 ? bias2[n0 + tid] : 0.f;
    }

    floatx16 acc[kFNI];
#pragma unroll
    for (int ni = 0; ni < kFNI; ni++)
#pragma unroll
        for (int q = 0; q < 16; q++) acc[ni][q] = 0.f;

    const long block = tile_m * kFW + wave;
    const long my_row = block * 32 + m;
    const long ld_row = my_row < R ? my_row : R - 1;
    float sx, isx;
    sx = pow2_scale(h1_bound[0], &isx);

    // the lane's half of the 16 radial encodings of its edge (archs/meanflow_painn8.py:25-35 with n = 16:
    // entries 0..7 are cos, 8..15 sin of (pi / rmax) (1 + f / 2) d, f = entry % 8)
    HiddenFromDistance gen;
    {
        const float x = r_ij[3 * ld_row], y = r_ij[3 * ld_row + 1], z = r_ij[3 * ld_row + 2];
        const float dist = sqrtf(x * x + y * y + z * z);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float phase = (base * (float)(1 + i / 2)) * dist;
            const float e = (g == 0 ? cosf(phase) : sinf(phase)) * 16384.0f;
            const _Float16 h = (_Float16)e;
            gen.eh[i] = h;
            gen.el[i] = (_Float16)(e - (float)h);
        }
    }
    gen.w1h = w1h; gen.w1l = w1l; gen.w1inv = w1inv; gen.b1 = b1s; gen.I = I; gen.m = m; gen.g = g;
    __syncthreads();                                         // the first-layer tables are in LDS
    wfirst_gemm_tile(acc, Wp, plane_elems, n0, gen, I, sx, lds);

    // y = SiLU(acc / scales + b2), written through the wave's LDS slice so that every store instruction covers
    // whole 256-byte row segments
    float* slice = reinterpret_cast<float*>(lds) + wave * kSlice;
    const long rows_left = R - block * 32;
    const int nv = rows_left >= 32 ? 32 : (rows_left > 0 ? (int)rows_left : 0);
#pragma unroll
    for (int pass = 0; pass < 4; pass++) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int ni = 2 * pass + h;
#pragma unroll
            for (int qq = 0; qq < 4; qq++) {
                const int cl = 32 * ni + 8 * qq + 4 * g;
                const float4 iw = *reinterpret_cast<const float4*>(wb + cl);
                const float4 bv = *reinterpret_cast<const float4*>(wb + kFTN + cl);
                float4 v;
                v.x = activate_c<1>(acc[ni][4 * qq + 0] * isx * iw.x + bv.x);
                v.y = activate_c<1>(acc[ni][4 * qq + 1] * isx * iw.y + bv.y);
                v.z = activate_c<1>(acc[ni][4 * qq + 2] * isx * iw.z + bv.z);
                v.w = activate_c<1>(acc[ni][4 * qq + 3] * isx * iw.w + bv.w);
                *reinterpret_cast<float4*>(slice + m * kRed + 32 * h + 8 * qq + 4 * g) = v;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        float* yp = Y + block * 32 * O + n0 + 64 * pass + lane;
#pragma unroll
        for (int r = 0; r < 32; r++)
            if (r < nv) yp[(long)r * O] = slice[r * kRed + lane];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

// out(node) = res(node) + the partial sums of the blocks its edges lie in, in block order.  Nodes whose
// edges lie strictly inside one block were written by the kernel above and are skipped; nodes without
// edges get the residual.  One thread per four consecutive floats of the node's 4n outputs.
__global__ void __launch_bounds__(256)
painn_message_finish_kernel(const int* __restrict__ row_ptr, long n_nodes, long n_blocks, int n,
                            const float* __restrict__ slots, const float* __restrict__ res_a,
                            const float* __restrict__ res_v, float* __restrict__ out_a, float* __restrict__ out_v) {
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_nodes * n) return;
    const long node = idx / n;
    const int x = (int)(idx - node * n) * 4;                  // offset in the node's [3n of v | n of a]
    const long lo = row_ptr[node], hi = row_ptr[node + 1];
    const bool is_v = x < 3 * n;
    const float* res = is_v ? res_v : res_a;
    float* out = is_v ? out_v + node * 3L * n + x : out_a + node * (long)n + (x - 3 * n);
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (res) s = ldf4(is_v ? res + node * 3L * n + x : res + node * (long)n + (x - 3 * n));
    if (hi > lo) {
        const long b_lo = lo / 32, b_hi = (hi - 1) / 32;
        if (b_lo == b_hi && lo > 32 * b_lo && hi - 1 < 32 * b_lo + 31) return;   // written directly
        const long row4n = 4L * n;
        for (long b = b_lo; b <= b_hi; b++) {
            const float* slot = 32 * b >= lo ? slots + b * row4n : slots + (n_blocks + b) * row4n;
            const float4 t = ldf4(slot + x);
            s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
        }
    }
    *reinterpret_cast<float4*>(out) = s;
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_painn_filter_message_workspace_bytes(long n_edges, int n, size_t* bytes) {
    MG_REQUIRE(bytes != nullptr && n_edges >= 0 && n >= 0, "mg_painn_filter_message_workspace_bytes: bad argument");
    // slots A and B of every block of 32 edges, 4n floats each (never zero bytes: callers allocate it)
    *bytes = (size_t)(2L * (ceil_div(n_edges, 32) + 1) * 4L * n) * sizeof(float);
    return MG_OK;
}

int mg_painn_filter_message(const void* packed_W3, const float* bias3, const float* h, const float* h_rowmax,
                            int h_rowmax_parts, long h_rowmax_stride, int hidden, const int* row_ptr,
                            const int* src, const int* dst, const float* r_ij, const float* actv, const float* x_v,
                            long n_nodes, long n_edges, int n, float epsilon, const float* res_a,
                            const float* res_v, void* workspace, float* out_a, float* out_v, mg_stream_t stream) {
    MG_REQUIRE(n >= 64 && n % 64 == 0, "mg_painn_filter_message: n must be a multiple of 64 (got %d)", n);
    MG_REQUIRE(hidden >= 64 && hidden % 32 == 0, "mg_painn_filter_message: hidden must be a multiple of 32, at least 64 (got %d)", hidden);
    MG_REQUIRE(n_nodes >= 0 && n_edges >= 0, "mg_painn_filter_message: negative size");
    MG_REQUIRE(n_edges < (1L << 31) && n_nodes < (1L << 31), "mg_painn_filter_message: int32 indices");
    MG_REQUIRE(h_rowmax_parts >= 1 && h_rowmax_parts <= 64, "mg_painn_filter_message: 1..64 bound parts");
    if (n_nodes == 0) return MG_OK;
    MG_REQUIRE(packed_W3 && bias3 && row_ptr && actv && x_v && out_a && out_v, "mg_painn_filter_message: null operand");
    MG_REQUIRE(aligned16(packed_W3) && aligned16(bias3) && aligned16(actv) && aligned16(x_v) && aligned16(out_a) &&
                   aligned16(out_v) && (!res_a || aligned16(res_a)) && (!res_v || aligned16(res_v)),
               "mg_painn_filter_message: operands must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const long n_blocks = ceil_div(n_edges, 32);
    if (n_edges > 0) {
        MG_REQUIRE(h && h_rowmax && src && dst && r_ij && workspace, "mg_painn_filter_message: null edge operand");
        MG_REQUIRE(aligned16(h) && aligned16(workspace), "mg_painn_filter_message: h and workspace must be 16-byte aligned");
        const int tiles_n = n / 64;
        const long tiles_total = ceil_div(n_edges, kFTM) * tiles_n;
        const long O_pad = (long)tiles_n * kFTN;                       // = 4n: already a multiple of 256
        const _Float16* planes = static_cast<const _Float16*>(packed_W3);
        const float* w_inv = reinterpret_cast<const float*>(planes + 2 * O_pad * hidden);
        const long grid = 8 * ceil_div(tiles_total, 8);
        MG_REQUIRE(grid < (1L << 31), "mg_painn_filter_message: too many tiles");
        painn_filter_message_kernel<<<dim3((unsigned)grid), dim3(64 * kFW), 0, s>>>(
            planes, w_inv, bias3, h, h_rowmax, h_rowmax_parts, h_rowmax_stride, n_edges, hidden, src, dst, r_ij, actv,
            x_v, n, epsilon, res_a, res_v, static_cast<float*>(workspace), n_blocks, out_a, out_v, tiles_n, tiles_total);
        if (int st = check_launch("painn_filter_message_kernel")) return st;
    }
    const long threads = n_nodes * n;
    painn_message_finish_kernel<<<dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0, s>>>(
        row_ptr, n_nodes, n_blocks, n, static_cast<const float*>(workspace), res_a, res_v, out_a, out_v);
    return check_launch("painn_message_finish_kernel");
}

int mg_tensor_linear_f16x2_rowsum_workspace_bytes(long rows, int dim_out, size_t* bytes) {
    MG_REQUIRE(bytes != nullptr && rows >= 0 && dim_out >= 0, "mg_tensor_linear_f16x2_rowsum_workspace_bytes: bad argument");
    *bytes = (size_t)(2L * (ceil_div(rows, 32) + 1) * dim_out) * sizeof(float);
    return MG_OK;
}

int mg_tensor_linear_f16x2_rowsum(const void* packed_W, const float* x, const float* x_rowmax, int x_rowmax_parts,
                                  long x_rowmax_stride, long rows, int dim_in, int dim_out, const float* bias, int act,
                                  const int* row_ptr, const int* seg, long n_out, float scale, void* workspace,
                                  float* y, float* out, mg_stream_t stream) {
    return mg_tensor_linear_f16x2_rowsum_scaled_bound(packed_W, x, x_rowmax, x_rowmax_parts, x_rowmax_stride, rows, dim_in,
                                                      dim_out, bias, act, row_ptr, seg, n_out, scale, workspace, y, out,
                                                      1.0f, 0.0f, stream);
}

int mg_tensor_linear_f16x2_rowsum_scaled_bound(const void* packed_W, const float* x, const float* x_rowmax,
                                               int x_rowmax_parts, long x_rowmax_stride, long rows, int dim_in,
                                               int dim_out, const float* bias, int act, const int* row_ptr,
                                               const int* seg, long n_out, float scale, void* workspace, float* y,
                                               float* out, float bound_mul, float bound_add, mg_stream_t stream) {
    MG_REQUIRE(bound_mul >= 0.f && bound_add >= 0.f && bound_mul == bound_mul && bound_add == bound_add,
               "mg_tensor_linear_f16x2_rowsum: the bound's factor and offset must be non-negative numbers");
    MG_REQUIRE(dim_out >= 256 && dim_out % 256 == 0, "mg_tensor_linear_f16x2_rowsum: dim_out must be a multiple of 256 (got %d)", dim_out);
    MG_REQUIRE(dim_in >= 64 && dim_in % 32 == 0, "mg_tensor_linear_f16x2_rowsum: dim_in must be a multiple of 32, at least 64 (got %d)", dim_in);
    MG_REQUIRE(rows >= 0 && n_out >= 0 && rows < (1L << 31) && n_out < (1L << 31), "mg_tensor_linear_f16x2_rowsum: bad size");
    MG_REQUIRE(act >= 0 && act <= 2, "mg_tensor_linear_f16x2_rowsum: unknown activation %d", act);
    MG_REQUIRE(x_rowmax_parts >= 1 && x_rowmax_parts <= 64, "mg_tensor_linear_f16x2_rowsum: 1..64 bound parts");
    if (n_out == 0) return MG_OK;
    MG_REQUIRE(packed_W && row_ptr && out && aligned16(packed_W) && aligned16(out) && (!bias || aligned16(bias)),
               "mg_tensor_linear_f16x2_rowsum: null or unaligned operand");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const long n_blocks = ceil_div(rows, 32);
    if (rows > 0) {
        MG_REQUIRE(x && x_rowmax && seg && workspace && aligned16(x) && aligned16(workspace) && (!y || aligned16(y)),
                   "mg_tensor_linear_f16x2_rowsum: null or unaligned row operand");
        const int tiles_n = dim_out / kFTN;
        const long tiles_total = ceil_div(rows, kFTM) * tiles_n;
        const _Float16* planes = static_cast<const _Float16*>(packed_W);
        const float* w_inv = reinterpret_cast<const float*>(planes + 2L * dim_out * dim_in);
        const long grid = 8 * ceil_div(tiles_total, 8);
        MG_REQUIRE(grid < (1L << 31), "mg_tensor_linear_f16x2_rowsum: too many tiles");
        float* slots = static_cast<float*>(workspace);
#define MG_ROWSUM_LAUNCH(A, S)                                                                                       \
    linear_rowsum_f16x2_kernel<A, S><<<dim3((unsigned)grid), dim3(64 * kFW), 0, s>>>(                                \
        planes, w_inv, bias, x, x_rowmax, x_rowmax_parts, x_rowmax_stride, rows, dim_in, dim_out, seg, slots, n_blocks, \
        scale, y, out, tiles_n, tiles_total, bound_mul, bound_add)
        if (y) {
            if (act == 1) MG_ROWSUM_LAUNCH(1, true);
            else if (act == 2) MG_ROWSUM_LAUNCH(2, true);
            else MG_ROWSUM_LAUNCH(0, true);
        } else {
            if (act == 1) MG_ROWSUM_LAUNCH(1, false);
            else if (act == 2) MG_ROWSUM_LAUNCH(2, false);
            else MG_ROWSUM_LAUNCH(0, false);
        }
#undef MG_ROWSUM_LAUNCH
        if (int st = check_launch("linear_rowsum_f16x2_kernel")) return st;
    }
    const long threads = n_out * (dim_out / 4);
    rowsum_finish_kernel<<<dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0, s>>>(
        row_ptr, n_out, n_blocks, dim_out, static_cast<const float*>(workspace), scale, out);
    return check_launch("rowsum_finish_kernel");
}

int mg_painn_filter_hidden(const float* r_ij, long n_edges, float rmax, const float* W1, long w1_stride_o,
                           long w1_stride_i, const float* b1, const void* packed_W2, const float* b2, int hidden,
                           const float* h1_bound, float* y, mg_stream_t stream) {
    MG_REQUIRE(hidden >= 256 && hidden % 256 == 0 && hidden <= kHidMax,
               "mg_painn_filter_hidden: hidden must be 256 or 512 (got %d)", hidden);
    MG_REQUIRE(n_edges >= 0 && n_edges < (1L << 31), "mg_painn_filter_hidden: bad size");
    MG_REQUIRE(rmax > 0.f, "mg_painn_filter_hidden: rmax must be positive");
    if (n_edges == 0) return MG_OK;
    MG_REQUIRE(r_ij && W1 && packed_W2 && h1_bound && y && aligned16(packed_W2) && aligned16(y),
               "mg_painn_filter_hidden: null or unaligned pointer");
    const int tiles_n = hidden / kFTN;
    const long tiles_total = ceil_div(n_edges, kFTM) * tiles_n;
    const _Float16* planes = static_cast<const _Float16*>(packed_W2);
    const float* w_inv = reinterpret_cast<const float*>(planes + 2L * hidden * hidden);
    const long grid = 8 * ceil_div(tiles_total, 8);
    MG_REQUIRE(grid < (1L << 31), "mg_painn_filter_hidden: too many tiles");
    const float base = (float)(3.14159265358979323846 / (double)rmax);
    painn_filter_hidden_kernel<<<dim3((unsigned)grid), dim3(64 * kFW), 0, static_cast<hipStream_t>(stream)>>>(
        planes, w_inv, b2, r_ij, n_edges, base, W1, w1_stride_o, w1_stride_i, b1, hidden, h1_bound, y, tiles_n,
        tiles_total);
    return check_launch("painn_filter_hidden_kernel");
}

}  // extern "C"
