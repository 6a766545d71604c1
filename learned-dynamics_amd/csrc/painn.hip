// PaiNN message passing (edge side), fused gather-product-scatter over CSR rows.
//
// For edge e = (i <- j) with filter W(e) in R^{4n} (output of the radial MLP),
// node activations A(j) in R^{4n}, node vectors v(j) in R^{n x 3} and unit-ish
// direction u = r / sqrt(eps + |r|^2):
//     P     = W(e) * A(j)                                  (elementwise, 4 blocks of n)
//     m_v   = v(j) * P0 + (v(j) x u) * P1 + u (x) P2       (n x 3)
//     m_a   = P3                                           (n)
//     out_v(i) = res_v(i) + sum_j m_v,   out_a(i) = res_a(i) + sum_j m_a
// Nothing per-edge is written to HBM: the only streamed operand is the filter
// (16n bytes per edge); A(j) and v(j) are gathers of node-sized arrays that live
// in L2 / Infinity Cache.  One wave owns (node, channel chunk); a lane owns four
// consecutive channels and moves them with 16-byte accesses; when the chunk is
// narrower than the wave the spare lanes take the next edges of the same node and
// are folded with xor-shuffles.  Rows are summed in edge order: no atomics.
#include "common.hpp"

namespace mg {
namespace {

__device__ __forceinline__ float activate_fast(float v, int act) {
    // SiLU with the hardware exp2 / reciprocal (about 1 ulp each), as in the GEMM epilogues
    if (act == 1) return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    if (act == 2) return v > 0.f ? v : 0.1f * v;
    return v;
}

constexpr int kMaxChunks = 16;
struct Chunks {
    int n;
    int start[kMaxChunks];   // first channel of the chunk
    int lanes[kMaxChunks];   // lanes per edge, power of two <= 64
};

inline Chunks make_chunks(int units, int unit_width) {
    Chunks c{};
    int pos = 0;
    while (units > 0 && c.n < kMaxChunks) {
        int p = 64;
        while (p > units) p >>= 1;
        c.start[c.n] = pos * unit_width;
        c.lanes[c.n] = p;
        c.n++;
        pos += p;
        units -= p;
    }
    return c;
}

__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
// streamed-once data: keep it from displacing the gathered node rows in L2
typedef float float4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 ld4_stream(const float* p) {
    const float4v t = __builtin_nontemporal_load(reinterpret_cast<const float4v*>(p));
    return make_float4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ void st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ float4 mul4(float4 a, float4 b) { return make_float4(a.x * b.x, a.y * b.y, a.z * b.z, a.w * b.w); }

struct EdgeAcc {
    float v[12];   // 4 channels x 3 components, channel-major (as in memory)
    float a[4];
    __device__ void zero() {
#pragma unroll
        for (int k = 0; k < 12; k++) v[k] = 0.f;
#pragma unroll
        for (int k = 0; k < 4; k++) a[k] = 0.f;
    }
};

// operands of one edge for 4 consecutive channels starting at c
struct EdgeLoads {
    float4 f[4], a[4], v[3];
    __device__ __forceinline__ void load(const float* __restrict__ filt_row, const float* __restrict__ actv_row,
                                         const float* __restrict__ xv_row, int n, int c) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            f[k] = ld4_stream(filt_row + k * n + c);
            a[k] = ld4(actv_row + k * n + c);
        }
#pragma unroll
        for (int k = 0; k < 3; k++) v[k] = ld4(xv_row + 3 * c + 4 * k);
    }
    // the filter from a periodic table of its values at d = k h (k = 0 .. mask): 4-point Lagrange interpolation
    // between the rows i - 1 .. i + 2 with weights w (error at most 0.0234 h^4 max |fourth derivative|)
    __device__ __forceinline__ void load_table(const float* __restrict__ tab, int i, int mask, const float (&w)[4],
                                               const float* __restrict__ actv_row, const float* __restrict__ xv_row,
                                               int n, int c) {
        const long row_f = 4L * n;
        const float* r0 = tab + (long)((i - 1) & mask) * row_f + c;
        const float* r1 = tab + (long)(i & mask) * row_f + c;
        const float* r2 = tab + (long)((i + 1) & mask) * row_f + c;
        const float* r3 = tab + (long)((i + 2) & mask) * row_f + c;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const float4 t0 = ld4(r0 + k * n), t1 = ld4(r1 + k * n), t2 = ld4(r2 + k * n), t3 = ld4(r3 + k * n);
            f[k] = make_float4(w[0] * t0.x + w[1] * t1.x + w[2] * t2.x + w[3] * t3.x,
                               w[0] * t0.y + w[1] * t1.y + w[2] * t2.y + w[3] * t3.y,
                               w[0] * t0.z + w[1] * t1.z + w[2] * t2.z + w[3] * t3.z,
                               w[0] * t0.w + w[1] * t1.w + w[2] * t2.w + w[3] * t3.w);
            a[k] = ld4(actv_row + k * n + c);
        }
#pragma unroll
        for (int k = 0; k < 3; k++) v[k] = ld4(xv_row + 3 * c + 4 * k);
    }
    __device__ __forceinline__ void accumulate(EdgeAcc& acc, float ux, float uy, float uz) const {
        accumulate_products(acc, mul4(f[0], a[0]), mul4(f[1], a[1]), mul4(f[2], a[2]), mul4(f[3], a[3]), ux, uy, uz);
    }
    // p0 .. p3: filter x activation of the four blocks for this lane's 4 channels
    __device__ __forceinline__ void accumulate_products(EdgeAcc& acc, float4 p0, float4 p1, float4 p2, float4 p3, float ux,
                                                        float uy, float uz) const {
        const float vv[12] = {v[0].x, v[0].y, v[0].z, v[0].w, v[1].x, v[1].y, v[1].z, v[1].w,
                              v[2].x, v[2].y, v[2].z, v[2].w};
        const float q0[4] = {p0.x, p0.y, p0.z, p0.w}, q1[4] = {p1.x, p1.y, p1.z, p1.w};
        const float q2[4] = {p2.x, p2.y, p2.z, p2.w}, q3[4] = {p3.x, p3.y, p3.z, p3.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const float x = vv[3 * k], y = vv[3 * k + 1], z = vv[3 * k + 2];
            const float cx = y * uz - z * uy, cy = z * ux - x * uz, cz = x * uy - y * ux;   // v x u
            // three fused multiply-adds straight into the running sum (a separate add per component would be
            // a twentieth of the loop's vector instructions)
            acc.v[3 * k + 0] = fmaf(ux, q2[k], fmaf(cx, q1[k], fmaf(x, q0[k], acc.v[3 * k + 0])));
            acc.v[3 * k + 1] = fmaf(uy, q2[k], fmaf(cy, q1[k], fmaf(y, q0[k], acc.v[3 * k + 1])));
            acc.v[3 * k + 2] = fmaf(uz, q2[k], fmaf(cz, q1[k], fmaf(z, q0[k], acc.v[3 * k + 2])));
            acc.a[k] += q3[k];
        }
    }
};

// register budget of 5 waves per SIMD (102 VGPRs): room to keep a whole step's loads in flight
// TABLE: `filt` is a table of the filter over one period of the distance (rows d = k / inv_h, k = 0 .. tab_mask)
// instead of one row per edge
template <bool TABLE>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(TABLE ? 3 : 4, TABLE ? 4 : 5))) painn_message_kernel(
    const int* __restrict__ row_ptr, const int* __restrict__ dst, const int* __restrict__ node_order, long n_nodes,
    const float* __restrict__ r_ij,
    const float* __restrict__ filt, const float* __restrict__ actv, const float* __restrict__ x_v, int n,
    float epsilon, const float* __restrict__ res_a, const float* __restrict__ res_v, float* __restrict__ out_a,
    float* __restrict__ out_v, Chunks ch, int tab_mask, float inv_h) {
    const int lane = threadIdx.x & (kWave - 1);
    // Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  Give every XCD
    // one contiguous range of nodes: neighbouring nodes share most of their neighbours, so the
    // gathers of actv / x_v rows are then served by that XCD's L2 instead of the fabric.
    const long items = n_nodes * ch.n;
    const long per_xcd = (items + 7) / 8;
    const int xcd = blockIdx.x & 7;
    const long waves_per_xcd = (long)(gridDim.x >> 3) * (blockDim.x / kWave);
    const long wave_local = (long)(blockIdx.x >> 3) * (blockDim.x / kWave) + threadIdx.x / kWave;
    const long row_f = 4L * n;
    for (long item_local = wave_local; item_local < per_xcd; item_local += waves_per_xcd) {
        const long item = xcd * per_xcd + item_local;
        if (item >= items) break;
        const long slot = item / ch.n;
        const int ci = (int)(item - slot * ch.n);
        // optional processing order (results do not depend on it)
        const long node = node_order ? node_order[slot] : slot;
        const int L = ch.lanes[ci];
        const int c = ch.start[ci] + (lane & (L - 1)) * 4;
        const int sub = lane / L, per_iter = kWave / L;
        const long lo = row_ptr[node], hi = row_ptr[node + 1];
        EdgeAcc acc;
        acc.zero();
        // The edge header (dst, r_ij) of the next step is fetched one step ahead of its use, so
        // the eleven 16-byte operand loads of a step can all be issued at once.
        long e = lo + sub;
        long j = 0;
        float rx = 0.f, ry = 0.f, rz = 0.f;
        if (e < hi) { j = dst[e]; rx = r_ij[3 * e]; ry = r_ij[3 * e + 1]; rz = r_ij[3 * e + 2]; }
        while (e < hi) {
            EdgeLoads ld;
            const float r2 = rx * rx + ry * ry + rz * rz;
            if constexpr (TABLE) {
                const float u = sqrtf(r2) * inv_h;
                const float fl = floorf(u);
                const float t = u - fl;
                const float tp = t + 1.0f, tm = t - 1.0f, tq = t - 2.0f;
                const float w[4] = {-(1.0f / 6.0f) * t * tm * tq, 0.5f * tp * tm * tq, -0.5f * tp * t * tq,
                                    (1.0f / 6.0f) * tp * t * tm};
                ld.load_table(filt, (int)fl, tab_mask, w, actv + j * row_f, x_v + j * 3L * n, n, c);
            } else {
                ld.load(filt + e * row_f, actv + j * row_f, x_v + j * 3L * n, n, c);
            }
            const long e_next = e + per_iter;
            long j_next = 0;
            float nx = 0.f, ny = 0.f, nz = 0.f;
            if (e_next < hi) { j_next = dst[e_next]; nx = r_ij[3 * e_next]; ny = r_ij[3 * e_next + 1]; nz = r_ij[3 * e_next + 2]; }
            const float inv = 1.0f / sqrtf(epsilon + r2);
            ld.accumulate(acc, rx * inv, ry * inv, rz * inv);
            e = e_next; j = j_next; rx = nx; ry = ny; rz = nz;
        }
        for (int d = L; d < kWave; d <<= 1) {
#pragma unroll
            for (int k = 0; k < 12; k++) acc.v[k] += __shfl_xor(acc.v[k], d);
#pragma unroll
            for (int k = 0; k < 4; k++) acc.a[k] += __shfl_xor(acc.a[k], d);
        }
        if (sub == 0) {
            float* oa = out_a + node * n + c;
            float* ov = out_v + (node * n + c) * 3;
            if (res_a) {
                const float4 r = ld4(res_a + node * n + c);
                acc.a[0] += r.x; acc.a[1] += r.y; acc.a[2] += r.z; acc.a[3] += r.w;
            }
            if (res_v) {
                const float* rv = res_v + (node * n + c) * 3;
                const float4 ra = ld4(rv), rb = ld4(rv + 4), rc = ld4(rv + 8);
                const float rr[12] = {ra.x, ra.y, ra.z, ra.w, rb.x, rb.y, rb.z, rb.w, rc.x, rc.y, rc.z, rc.w};
#pragma unroll
                for (int k = 0; k < 12; k++) acc.v[k] += rr[k];
            }
            st4(oa, make_float4(acc.a[0], acc.a[1], acc.a[2], acc.a[3]));
            st4(ov, make_float4(acc.v[0], acc.v[1], acc.v[2], acc.v[3]));
            st4(ov + 4, make_float4(acc.v[4], acc.v[5], acc.v[6], acc.v[7]));
            st4(ov + 8, make_float4(acc.v[8], acc.v[9], acc.v[10], acc.v[11]));
        }
    }
}

// The table variant with the grid in LDS.  A workgroup owns one slice of 16 channels (its 4 x 16 filter columns of
// every grid row: rows x 64 floats, at most 512 rows) and walks over nodes; the 4 lanes of an edge hold 4 channels
// each, so a wave takes 16 edges of its node per step and only the node rows (actv, x_v) come through the vector
// caches: 3.5 KB per edge instead of 11.5 KB.  actv is expected slice-major, (node, n / 16, 4, 16), so that a
// slice's 64 values are two whole cache lines; x_v (node, n, 3) already has a slice's 48 values contiguous.
//
// What an edge contributes besides its node rows depends on the edge alone, not on the channel: the first of its four
// grid rows, the four interpolation weights and the direction.  A pass over the edges writes them once as a 32-byte
// record (painn_edge_records_kernel); the 8 slices x 4 lanes that work on an edge read the record instead of
// repeating the square root, floor, weight polynomials and reciprocal square root (a fifth of the loop's vector
// instructions before).  The grid in LDS carries three extra rows (copies of rows 0..2) behind the last one, so the
// four rows of an edge are always consecutive: one address per edge, the rest are immediates.
// LDS rows are padded to 68 floats so that the rows different edges read start in different banks.
constexpr int kSliceChan = 16, kSliceCols = 4 * kSliceChan, kSliceRowF = kSliceCols + 4, kSliceMaxRows = 512;
constexpr int kSliceExtraRows = 3;

// rec[2e] = (float offset of the first grid row in LDS as int bits, w0, w1, w2), rec[2e+1] = (w3, ux, uy, uz):
// grid rows i-1 .. i+2 with i = floor(|r| / h), 4-point Lagrange weights at t = |r| / h - i, u = r / sqrt(eps + |r|^2)
__global__ void __launch_bounds__(256) painn_edge_records_kernel(const float* __restrict__ r_ij, long E, int mask,
                                                                 float inv_h, float epsilon, float4* __restrict__ rec) {
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    const float rx = r_ij[3 * e], ry = r_ij[3 * e + 1], rz = r_ij[3 * e + 2];
    const float r2 = rx * rx + ry * ry + rz * rz;
    const float u = sqrtf(r2) * inv_h;
    const float fl = floorf(u);
    const float t = u - fl;
    const float tp = t + 1.0f, tm = t - 1.0f, tq = t - 2.0f;
    const float w0 = -(1.0f / 6.0f) * t * tm * tq, w1 = 0.5f * tp * tm * tq, w2 = -0.5f * tp * t * tq,
                w3 = (1.0f / 6.0f) * tp * t * tm;
    const int first = ((int)fl - 1) & mask;                   // 0 .. rows - 1; rows first .. first + 3 exist in LDS
    const float inv = 1.0f / sqrtf(epsilon + r2);
    rec[2 * e] = make_float4(__int_as_float(first * kSliceRowF), w0, w1, w2);
    rec[2 * e + 1] = make_float4(w3, rx * inv, ry * inv, rz * inv);
}

// Sum of 16 per-lane values over the 16 lanes that share (lane & 3), leaving value s of the 16 in the lane with
// (lane >> 2) == s: each step pairs the registers, exchanges the halves two lanes do not keep and adds, so the whole
// reduction is 15 additions instead of 16 x 4.  Lane halves (xor 32) and odd / even rows of 16 lanes (xor 16) are
// exchanged by the swap instructions, lanes 8 and 4 apart by LDS-crossbar swizzles.
__device__ __forceinline__ void swap_add32(float& a, const float b) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    a = __uint_as_float(r[0]) + __uint_as_float(r[1]);        // lanes 0..31: a over both halves; 32..63: b
}
__device__ __forceinline__ void swap_add16(float& a, const float b) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    a = __uint_as_float(r[0]) + __uint_as_float(r[1]);        // even rows of 16 lanes: a; odd rows: b
}
template <int XOR>
__device__ __forceinline__ void swizzle_add(float& a, const float b, bool upper) {
    const float keep = upper ? b : a, send = upper ? a : b;
    constexpr int pattern = (XOR << 10) | 0x1f;               // lane' = lane ^ XOR inside each group of 32
    a = keep + __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(send), pattern));
}

__global__ void __launch_bounds__(1024) painn_table_message_lds_kernel(
    const int* __restrict__ row_ptr, const int* __restrict__ dst, const int* __restrict__ node_order, long n_nodes,
    const float4* __restrict__ rec, const float* __restrict__ table, int tab_rows, const float* __restrict__ actv_s,
    const float* __restrict__ x_v, int n, const float* __restrict__ res_a, const float* __restrict__ res_v,
    float* __restrict__ out_a, float* __restrict__ out_v) {
    extern __shared__ float tab[];                            // (tab_rows + 3) x kSliceRowF
    const int n_slices = n / kSliceChan;
    // consecutive workgroup ids go to consecutive XCDs: with 8 slices every XCD works on one slice, and its L2 only
    // ever holds that slice's columns of the node rows
    const int slice = blockIdx.x % n_slices;
    const int group = blockIdx.x / n_slices, groups = gridDim.x / n_slices;
    for (int q = threadIdx.x; q < (tab_rows + kSliceExtraRows) * (kSliceCols / 4); q += blockDim.x) {
        const int row = q / (kSliceCols / 4), piece = q % (kSliceCols / 4), k = piece / 4, c4 = piece % 4;
        st4(tab + row * kSliceRowF + 4 * piece,
            ld4(table + (long)(row & (tab_rows - 1)) * 4 * n + k * n + slice * kSliceChan + 4 * c4));
    }
    __syncthreads();
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave, waves = blockDim.x / kWave;
    const int l4 = lane & 3, sub = lane >> 2;                 // 4 channels of edge `sub` of the step
    constexpr int kPerIter = kWave / 4;
    // 32-bit element offsets (the host checks that they fit) keep the address arithmetic short
    const unsigned a_stride = (unsigned)n_slices * kSliceCols, v_stride = 3u * (unsigned)n;
    const float* a_base = actv_s + slice * kSliceCols + 4 * l4;
    const float* v_base = x_v + (slice * kSliceChan + 4 * l4) * 3;
    const float* tab_l = tab + 4 * l4;
    // after the reduction a lane holds ONE of its channel quad's 16 sums: the vector sums 0..11 (channel-major, as in
    // memory), then the 4 scalar sums
    const bool is_a = sub >= 12;
    const long o_lane = slice * kSliceChan + 4 * l4;
    for (long slot = (long)group * waves + wave; slot < n_nodes; slot += (long)groups * waves) {
        const long node = node_order ? node_order[slot] : slot;
        const int lo = row_ptr[node], hi = row_ptr[node + 1];
        float acc[16];
#pragma unroll
        for (int k = 0; k < 16; k++) acc[k] = 0.f;
        int e = lo + sub;
        unsigned j = 0;
        float4 ra = make_float4(0.f, 0.f, 0.f, 0.f), rb = ra;
        if (e < hi) { j = (unsigned)dst[e]; ra = rec[2 * (long)e]; rb = rec[2 * (long)e + 1]; }
        while (e < hi) {
            const float* a_row = a_base + j * a_stride;
            const float* v_row = v_base + j * v_stride;
            float4 a[4], v[3];
#pragma unroll
            for (int k = 0; k < 4; k++) a[k] = ld4(a_row + k * kSliceChan);
#pragma unroll
            for (int k = 0; k < 3; k++) v[k] = ld4(v_row + 4 * k);
            e += kPerIter;
            unsigned j_next = 0;
            float4 na = ra, nb = rb;
            if (e < hi) { j_next = (unsigned)dst[e]; na = rec[2 * (long)e]; nb = rec[2 * (long)e + 1]; }
            const float* tp = tab_l + __float_as_int(ra.x);
            const float w0 = ra.y, w1 = ra.z, w2 = ra.w, w3 = rb.x, ux = rb.y, uy = rb.z, uz = rb.w;
            float p[4][4];                                    // filter x activation: block k, channel c
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const float4 t0 = ld4(tp + k * kSliceChan), t1 = ld4(tp + kSliceRowF + k * kSliceChan),
                             t2 = ld4(tp + 2 * kSliceRowF + k * kSliceChan), t3 = ld4(tp + 3 * kSliceRowF + k * kSliceChan);
                p[k][0] = (w0 * t0.x + w1 * t1.x + w2 * t2.x + w3 * t3.x) * a[k].x;
                p[k][1] = (w0 * t0.y + w1 * t1.y + w2 * t2.y + w3 * t3.y) * a[k].y;
                p[k][2] = (w0 * t0.z + w1 * t1.z + w2 * t2.z + w3 * t3.z) * a[k].z;
                p[k][3] = (w0 * t0.w + w1 * t1.w + w2 * t2.w + w3 * t3.w) * a[k].w;
            }
            const float vv[12] = {v[0].x, v[0].y, v[0].z, v[0].w, v[1].x, v[1].y, v[1].z, v[1].w,
                                  v[2].x, v[2].y, v[2].z, v[2].w};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const float x = vv[3 * c], y = vv[3 * c + 1], z = vv[3 * c + 2];
                const float cx = y * uz - z * uy, cy = z * ux - x * uz, cz = x * uy - y * ux;   // v x u
                acc[3 * c + 0] = fmaf(ux, p[2][c], fmaf(cx, p[1][c], fmaf(x, p[0][c], acc[3 * c + 0])));
                acc[3 * c + 1] = fmaf(uy, p[2][c], fmaf(cy, p[1][c], fmaf(y, p[0][c], acc[3 * c + 1])));
                acc[3 * c + 2] = fmaf(uz, p[2][c], fmaf(cz, p[1][c], fmaf(z, p[0][c], acc[3 * c + 2])));
                acc[12 + c] += p[3][c];
            }
            j = j_next; ra = na; rb = nb;
        }
        // 16 sums over the 16 edge slots of the wave: value index sub = bit2 + 2 bit3 + 4 bit4 + 8 bit5 of the lane id
#pragma unroll
        for (int k = 0; k < 8; k++) swap_add32(acc[k], acc[k + 8]);          // registers 0..7: value k + 8 bit5
#pragma unroll
        for (int k = 0; k < 4; k++) swap_add16(acc[k], acc[k + 4]);          // registers 0..3: value k + 4 bit4 + 8 bit5
#pragma unroll
        for (int k = 0; k < 2; k++) swizzle_add<8>(acc[k], acc[k + 2], (lane & 8) != 0);
        swizzle_add<4>(acc[0], acc[1], (lane & 4) != 0);
        const long o = node * n + o_lane;
        float sum = acc[0];
        float* outp = is_a ? out_a + o + (sub - 12) : out_v + o * 3 + sub;
        const float* resp = is_a ? (res_a ? res_a + o + (sub - 12) : nullptr) : (res_v ? res_v + o * 3 + sub : nullptr);
        if (resp) sum += *resp;
        *outp = sum;
    }
}

// fallback for channel counts that are not a multiple of 4 or unaligned operands:
// one lane per channel, one wave per (node, 64-channel chunk)
__global__ void __launch_bounds__(256) painn_message_scalar_kernel(
    const int* __restrict__ row_ptr, const int* __restrict__ dst, long n_nodes, const float* __restrict__ r_ij,
    const float* __restrict__ filt, const float* __restrict__ actv, const float* __restrict__ x_v, int n,
    float epsilon, const float* __restrict__ res_a, const float* __restrict__ res_v, float* __restrict__ out_a,
    float* __restrict__ out_v) {
    const int lane = threadIdx.x & (kWave - 1);
    const long wave_global = ((long)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    const long n_waves = ((long)gridDim.x * blockDim.x) / kWave;
    const int chunks = (n + kWave - 1) / kWave;
    const long items = n_nodes * chunks;
    const long row_f = 4L * n;
    for (long item = wave_global; item < items; item += n_waves) {
        const long node = item / chunks;
        const int c = (int)(item - node * chunks) * kWave + lane;
        if (c >= n) continue;
        float ax = 0.f, ay = 0.f, az = 0.f, aa = 0.f;
        for (long e = row_ptr[node]; e < row_ptr[node + 1]; e++) {
            const long j = dst[e];
            const float rx = r_ij[3 * e], ry = r_ij[3 * e + 1], rz = r_ij[3 * e + 2];
            const float inv = 1.0f / sqrtf(epsilon + (rx * rx + ry * ry + rz * rz));
            const float ux = rx * inv, uy = ry * inv, uz = rz * inv;
            const float* f = filt + e * row_f;
            const float* a = actv + j * row_f;
            const float p0 = f[c] * a[c], p1 = f[n + c] * a[n + c], p2 = f[2 * n + c] * a[2 * n + c];
            const float p3 = f[3 * n + c] * a[3 * n + c];
            const float* v = x_v + (j * n + c) * 3;
            const float x = v[0], y = v[1], z = v[2];
            ax += x * p0 + (y * uz - z * uy) * p1 + ux * p2;
            ay += y * p0 + (z * ux - x * uz) * p1 + uy * p2;
            az += z * p0 + (x * uy - y * ux) * p1 + uz * p2;
            aa += p3;
        }
        const long o = node * n + c;
        if (res_a) aa += res_a[o];
        if (res_v) { ax += res_v[3 * o]; ay += res_v[3 * o + 1]; az += res_v[3 * o + 2]; }
        out_a[o] = aa;
        out_v[3 * o] = ax; out_v[3 * o + 1] = ay; out_v[3 * o + 2] = az;
    }
}

// out[e, m] = cos(k_m d) for m < hn, sin(k_{m-hn} d) for hn <= m < n, k_m = (pi/rmax)(1 + m/2), hn = (n+1)/2
__global__ void __launch_bounds__(256) radial_encode_painn_kernel(const float* __restrict__ r_ij, long E, int n,
                                                                  float base, float* __restrict__ out) {
    const long total = E * n;
    const int hn = (n + 1) / 2;
    for (long t = (long)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (long)gridDim.x * blockDim.x) {
        const long e = t / n;
        const int m = (int)(t - e * n);
        const float x = r_ij[3 * e], y = r_ij[3 * e + 1], z = r_ij[3 * e + 2];
        const float d = sqrtf(x * x + y * y + z * z);
        const int f = m < hn ? m : m - hn;
        const float phase = (base * (float)(1 + f / 2)) * d;
        out[t] = m < hn ? cosf(phase) : sinf(phase);
    }
}

// First layer of the radial MLP fused with the encoding:
//   y[e, o] = act(b[o] + sum_m W[o, m] * enc[e, m]),  enc = radial_encode(r_ij[e])  (N_ENC >= n columns, zero padded)
// The layer has K = n <= 32 and dim_out in the hundreds, so it is bound by writing y: a GEMM tile
// machine buys nothing.  A workgroup takes 64 edges: their encodings go to LDS (one cos/sin per
// entry), then every lane keeps the weights of four consecutive output channels in registers and
// walks the 64 rows: the encoding row is an LDS broadcast, the output one 16-byte store per lane
// (a wave writes 1 KB contiguous).
template <int N_ENC>
__global__ void __launch_bounds__(256) painn_radial_linear_kernel(const float* __restrict__ r_ij, long E, int n,
                                                                  float base, const float* __restrict__ W, long so,
                                                                  long si, const float* __restrict__ bias, int O,
                                                                  int act, float* __restrict__ Y) {
    constexpr int kRows = 64;
    __shared__ __attribute__((aligned(16))) float enc[kRows * N_ENC];
    const int tid = threadIdx.x;
    const int groups = O / 4;               // lanes per output row; divides 256
    const int g = tid % groups, sub = tid / groups;
    const int rows_per_pass = 256 / groups;
    const int hn = (n + 1) / 2;

    float w[4][N_ENC], b[4];
#pragma unroll
    for (int c = 0; c < 4; c++) {
        b[c] = bias ? bias[4 * g + c] : 0.f;
#pragma unroll
        for (int m = 0; m < N_ENC; m++) w[c][m] = m < n ? W[(long)(4 * g + c) * so + (long)m * si] : 0.f;
    }

    const long tiles = (E + kRows - 1) / kRows;
    for (long tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const long e0 = tile * kRows;
        __syncthreads();                    // the previous tile's rows are consumed
#pragma unroll
        for (int i = 0; i < kRows * N_ENC / 256; i++) {
            const int idx = tid + 256 * i;
            const int row = idx / N_ENC, m = idx % N_ENC;
            const long e = e0 + row;
            float v = 0.f;
            if (e < E && m < n) {
                const float x = r_ij[3 * e], y = r_ij[3 * e + 1], z = r_ij[3 * e + 2];
                const float d = sqrtf(x * x + y * y + z * z);
                const int f = m < hn ? m : m - hn;
                const float phase = (base * (float)(1 + f / 2)) * d;
                v = m < hn ? cosf(phase) : sinf(phase);
            }
            enc[idx] = v;
        }
        __syncthreads();
        for (int row = sub; row < kRows; row += rows_per_pass) {
            const long e = e0 + row;
            if (e >= E) break;
            float acc[4] = {b[0], b[1], b[2], b[3]};
#pragma unroll
            for (int m4 = 0; m4 < N_ENC / 4; m4++) {
                const float4 ev = *reinterpret_cast<const float4*>(enc + row * N_ENC + 4 * m4);
                const float evs[4] = {ev.x, ev.y, ev.z, ev.w};
#pragma unroll
                for (int k = 0; k < 4; k++)
#pragma unroll
                    for (int c = 0; c < 4; c++) acc[c] = fmaf(w[c][4 * m4 + k], evs[k], acc[c]);
            }
            typedef float floatx4 __attribute__((ext_vector_type(4)));
            floatx4 out;
            out.x = activate_fast(acc[0], act);
            out.y = activate_fast(acc[1], act);
            out.z = activate_fast(acc[2], act);
            out.w = activate_fast(acc[3], act);
            __builtin_nontemporal_store(out, reinterpret_cast<floatx4*>(Y + e * O + 4 * g));
        }
    }
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_painn_radial_encode(const float* r_ij, long n_edges, int n, float rmax, float* out, mg_stream_t stream) {
    MG_REQUIRE(n_edges >= 0 && n >= 0, "mg_painn_radial_encode: negative size");
    MG_REQUIRE(rmax > 0.f, "mg_painn_radial_encode: rmax must be positive");
    const long total = n_edges * n;
    if (total == 0) return MG_OK;
    MG_REQUIRE(r_ij && out, "mg_painn_radial_encode: null pointer");
    const float base = (float)(3.14159265358979323846 / (double)rmax);
    long blocks = ceil_div(total, 256);
    if (blocks > 256L * 64) blocks = 256L * 64;
    hipLaunchKernelGGL(radial_encode_painn_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, r_ij,
                       n_edges, n, base, out);
    return check_launch("mg_painn_radial_encode");
}

int mg_painn_radial_linear(const float* r_ij, long n_edges, int n, float rmax, const float* W, long w_stride_o,
                           long w_stride_i, const float* bias, int dim_out, int act, float* y, mg_stream_t stream) {
    MG_REQUIRE(n_edges >= 0 && n >= 0 && dim_out >= 0, "mg_painn_radial_linear: negative size");
    MG_REQUIRE(rmax > 0.f, "mg_painn_radial_linear: rmax must be positive");
    MG_REQUIRE(act >= 0 && act <= 2, "mg_painn_radial_linear: unknown activation %d", act);
    MG_REQUIRE(n <= 32, "mg_painn_radial_linear: at most 32 radial functions (got %d)", n);
    const int groups = dim_out / 4;
    MG_REQUIRE(dim_out % 4 == 0 && groups >= 1 && groups <= 256 && 256 % groups == 0,
               "mg_painn_radial_linear: dim_out must be 4 * a power of two, at most 1024 (got %d)", dim_out);
    if (n_edges == 0) return MG_OK;
    MG_REQUIRE(r_ij && W && y && aligned16(y), "mg_painn_radial_linear: null or unaligned pointer");
    const float base = (float)(3.14159265358979323846 / (double)rmax);
    long blocks = ceil_div(n_edges, 64);
    if (blocks > 256L * 8) blocks = 256L * 8;
    if (n <= 16)
        hipLaunchKernelGGL(painn_radial_linear_kernel<16>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                           r_ij, n_edges, n, base, W, w_stride_o, w_stride_i, bias, dim_out, act, y);
    else
        hipLaunchKernelGGL(painn_radial_linear_kernel<32>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                           r_ij, n_edges, n, base, W, w_stride_o, w_stride_i, bias, dim_out, act, y);
    return check_launch("mg_painn_radial_linear");
}

int mg_painn_message(const int* row_ptr, const int* dst, const int* node_order, int n_nodes, long n_edges,
                     const float* r_ij,
                     const float* filt, const float* actv, const float* x_v, int n, float epsilon,
                     const float* res_a, const float* res_v, float* out_a, float* out_v, mg_stream_t stream) {
    MG_REQUIRE(n_nodes >= 0 && n_edges >= 0 && n >= 0, "mg_painn_message: negative size");
    if (n_nodes == 0 || n == 0) return MG_OK;
    MG_REQUIRE(row_ptr && out_a && out_v && actv && x_v, "mg_painn_message: null pointer");
    MG_REQUIRE(n_edges == 0 || (dst && r_ij && filt), "mg_painn_message: null edge operand");
    hipStream_t st = (hipStream_t)stream;
    const bool vec = (n % 4 == 0) && aligned16(filt) && aligned16(actv) && aligned16(x_v) && aligned16(out_a) &&
                     aligned16(out_v) && (!res_a || aligned16(res_a)) && (!res_v || aligned16(res_v));
    if (vec) {
        const Chunks ch = make_chunks(n / 4, 4);
        int covered = 0;
        for (int k = 0; k < ch.n; k++) covered += ch.lanes[k] * 4;
        if (covered == n) {
            long blocks = ceil_div((long)n_nodes * ch.n, 4);
            if (blocks > 256L * 32) blocks = 256L * 32;
            blocks = ceil_div(blocks, 8) * 8;   // the XCD-aware item order needs a multiple of 8
            hipLaunchKernelGGL(painn_message_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, st, row_ptr, dst,
                               node_order, (long)n_nodes, r_ij, filt, actv, x_v, n, epsilon, res_a, res_v, out_a, out_v, ch,
                               0, 0.f);
            return check_launch("mg_painn_message");
        }
    }
    long blocks = ceil_div((long)n_nodes * ceil_div(n, kWave), 4);
    if (blocks > 256L * 64) blocks = 256L * 64;
    hipLaunchKernelGGL(painn_message_scalar_kernel, dim3((unsigned)blocks), dim3(256), 0, st, row_ptr, dst,
                       (long)n_nodes, r_ij, filt, actv, x_v, n, epsilon, res_a, res_v, out_a, out_v);
    return check_launch("mg_painn_message");
}

int mg_painn_table_message(const int* row_ptr, const int* dst, const int* node_order, int n_nodes, long n_edges,
                           const float* r_ij, const float* table, int table_rows, float period, const float* actv,
                           const float* x_v, int n, float epsilon, const float* res_a, const float* res_v, float* out_a,
                           float* out_v, mg_stream_t stream) {
    MG_REQUIRE(n_nodes >= 0 && n_edges >= 0 && n >= 0, "mg_painn_table_message: negative size");
    if (n_nodes == 0 || n == 0) return MG_OK;
    MG_REQUIRE(row_ptr && out_a && out_v && actv && x_v && table, "mg_painn_table_message: null pointer");
    MG_REQUIRE(n_edges == 0 || (dst && r_ij), "mg_painn_table_message: null edge operand");
    MG_REQUIRE(table_rows >= 4 && (table_rows & (table_rows - 1)) == 0,
               "mg_painn_table_message: table_rows must be a power of two >= 4 (got %d)", table_rows);
    MG_REQUIRE(period > 0.f, "mg_painn_table_message: period must be positive");
    MG_REQUIRE(n % 4 == 0 && aligned16(table) && aligned16(actv) && aligned16(x_v) && aligned16(out_a) && aligned16(out_v) &&
                   (!res_a || aligned16(res_a)) && (!res_v || aligned16(res_v)),
               "mg_painn_table_message: n must be a multiple of 4 and the operands 16-byte aligned");
    const Chunks ch = make_chunks(n / 4, 4);
    int covered = 0;
    for (int k = 0; k < ch.n; k++) covered += ch.lanes[k] * 4;
    MG_REQUIRE(covered == n, "mg_painn_table_message: unsupported channel count %d", n);
    long blocks = ceil_div((long)n_nodes * ch.n, 4);
    if (blocks > 256L * 32) blocks = 256L * 32;
    blocks = ceil_div(blocks, 8) * 8;
    hipLaunchKernelGGL(painn_message_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, row_ptr, dst,
                       node_order, (long)n_nodes, r_ij, table, actv, x_v, n, epsilon, res_a, res_v, out_a, out_v, ch,
                       table_rows - 1, (float)table_rows / period);
    return check_launch("mg_painn_table_message");
}

int mg_painn_edge_records(const float* r_ij, long n_edges, int table_rows, float period, float epsilon,
                           float* records, mg_stream_t stream) {
    MG_REQUIRE(n_edges >= 0, "mg_painn_edge_records: negative size");
    if (n_edges == 0) return MG_OK;
    MG_REQUIRE(r_ij && records && aligned16(records), "mg_painn_edge_records: null or unaligned pointer");
    MG_REQUIRE(table_rows >= 4 && table_rows <= kSliceMaxRows && (table_rows & (table_rows - 1)) == 0,
               "mg_painn_edge_records: table_rows must be a power of two in 4..%d (got %d)", kSliceMaxRows, table_rows);
    MG_REQUIRE(period > 0.f, "mg_painn_edge_records: period must be positive");
    hipLaunchKernelGGL(painn_edge_records_kernel, dim3((unsigned)ceil_div(n_edges, 256)), dim3(256), 0,
                       (hipStream_t)stream, r_ij, n_edges, table_rows - 1, (float)table_rows / period, epsilon,
                       reinterpret_cast<float4*>(records));
    return check_launch("mg_painn_edge_records");
}

int mg_painn_table_message_sliced(const int* row_ptr, const int* dst, const int* node_order, int n_nodes, long n_edges,
                                  const float* records, const float* table, int table_rows, const float* actv_sliced,
                                  const float* x_v, int n, const float* res_a, const float* res_v, float* out_a,
                                  float* out_v, mg_stream_t stream) {
    MG_REQUIRE(n_nodes >= 0 && n_edges >= 0 && n >= 0, "mg_painn_table_message_sliced: negative size");
    if (n_nodes == 0 || n == 0) return MG_OK;
    MG_REQUIRE(row_ptr && out_a && out_v && actv_sliced && x_v && table, "mg_painn_table_message_sliced: null pointer");
    MG_REQUIRE(n_edges == 0 || (dst && records), "mg_painn_table_message_sliced: null edge operand");
    MG_REQUIRE(table_rows >= 4 && table_rows <= kSliceMaxRows && (table_rows & (table_rows - 1)) == 0,
               "mg_painn_table_message_sliced: table_rows must be a power of two in 4..%d (got %d)", kSliceMaxRows, table_rows);
    MG_REQUIRE(n % kSliceChan == 0 && aligned16(table) && aligned16(actv_sliced) && aligned16(x_v) && aligned16(out_a) &&
                   aligned16(out_v) && (!res_a || aligned16(res_a)) && (!res_v || aligned16(res_v)) &&
                   (!records || aligned16(records)),
               "mg_painn_table_message_sliced: n must be a multiple of %d and the operands 16-byte aligned", kSliceChan);
    MG_REQUIRE((long)n_nodes * 4 * n < (1L << 32), "mg_painn_table_message_sliced: n_nodes * 4 n must be below 2^32");
    MG_REQUIRE(n_edges < (1L << 31), "mg_painn_table_message_sliced: n_edges must be below 2^31");
    const int n_slices = n / kSliceChan;
    const size_t lds_bytes = (size_t)(table_rows + kSliceExtraRows) * kSliceRowF * sizeof(float);
    // more than 64 KB of dynamic LDS has to be asked for (per device, so on every call)
    MG_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(painn_table_message_lds_kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize,
                               (kSliceMaxRows + kSliceExtraRows) * kSliceRowF * (int)sizeof(float)));
    long groups = ceil_div(256, n_slices);                    // one workgroup per CU
    const long max_groups = ceil_div(n_nodes, 16);
    if (groups > max_groups) groups = max_groups;
    hipLaunchKernelGGL(painn_table_message_lds_kernel, dim3((unsigned)(groups * n_slices)), dim3(1024), lds_bytes,
                       (hipStream_t)stream, row_ptr, dst, node_order, (long)n_nodes,
                       reinterpret_cast<const float4*>(records), table, table_rows, actv_sliced, x_v, n, res_a, res_v,
                       out_a, out_v);
    return check_launch("mg_painn_table_message_sliced");
}

}  // extern "C"
