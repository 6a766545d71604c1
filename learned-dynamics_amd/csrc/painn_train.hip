// Training-side helper of the PaiNN message (archs/meanflow_painn8.py:94-100): the elementwise middle of
// Message.forward, between the two MLPs / the gathers and the sums over edges, as one pass and its adjoint as
// another.  With p = dist * actv (E, 4n), v the gathered vectors (E, n, 3) and d the edge directions (E, 3):
//   m[e, c, :] = v[e, c, :] p[e, c] + (v[e, c, :] x d[e]) p[e, n + c] + d[e] p[e, 2n + c]
//   a[e, c]    = p[e, 3n + c]
// Written out in tensor arithmetic this is a dozen kernels that each stream an (E, 3n) or (E, 4n) array through
// HBM, and twice as many in the backward pass; here every input is read once and every output written once.
// A thread owns 4 consecutive channels of one edge (16-byte loads and stores throughout); the n / 4 threads of an
// edge are neighbours in a wave, which is what the gradient of d, a sum over channels, is reduced over.
// actv and v may be given per node with an index (`node`, the edge's destination): the rows are then read through the
// caches instead of from a gathered per-edge copy; their gradients are still written per edge (the caller sums them
// over the edges of a node).
// Not on the inference hot path (that one never materialises dist, actv or v per edge).
#include "common.hpp"

namespace mg {
namespace {

struct Vec3 { float x, y, z; };
__device__ __forceinline__ Vec3 cross(Vec3 a, Vec3 b) {
    return {a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x};
}
__device__ __forceinline__ float dot(Vec3 a, Vec3 b) { return a.x * b.x + a.y * b.y + a.z * b.z; }

__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ void st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ float4 mul4(float4 a, float4 b) { return make_float4(a.x * b.x, a.y * b.y, a.z * b.z, a.w * b.w); }

// 4 channels x 3 components, as they lie in memory: (c, k) at 3 c + k
struct Vec3x4 {
    float f[12];
    __device__ __forceinline__ Vec3 get(int j) const { return {f[3 * j], f[3 * j + 1], f[3 * j + 2]}; }
    __device__ __forceinline__ void set(int j, Vec3 v) { f[3 * j] = v.x; f[3 * j + 1] = v.y; f[3 * j + 2] = v.z; }
};
__device__ __forceinline__ Vec3x4 ld12(const float* p) {
    Vec3x4 r;
    const float4 a = ld4(p), b = ld4(p + 4), c = ld4(p + 8);
    r.f[0] = a.x; r.f[1] = a.y; r.f[2] = a.z; r.f[3] = a.w;
    r.f[4] = b.x; r.f[5] = b.y; r.f[6] = b.z; r.f[7] = b.w;
    r.f[8] = c.x; r.f[9] = c.y; r.f[10] = c.z; r.f[11] = c.w;
    return r;
}
__device__ __forceinline__ void st12(float* p, const Vec3x4& r) {
    st4(p, make_float4(r.f[0], r.f[1], r.f[2], r.f[3]));
    st4(p + 4, make_float4(r.f[4], r.f[5], r.f[6], r.f[7]));
    st4(p + 8, make_float4(r.f[8], r.f[9], r.f[10], r.f[11]));
}
__device__ __forceinline__ float at(const float4& v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }

__global__ void __launch_bounds__(256) painn_combine_fwd_kernel(const float* __restrict__ dist,
                                                                const float* __restrict__ actv,
                                                                const float* __restrict__ v,
                                                                const float* __restrict__ dir,
                                                                const int* __restrict__ node, long n_rows, long E,
                                                                int n, int terms, float* __restrict__ m,
                                                                float* __restrict__ a) {
    const int tpe = n >> 2;                                       // threads per edge
    const long t = (long)blockIdx.x * 256 + threadIdx.x;
    const long e = t / tpe;
    if (e >= E) return;
    const int c = (int)(t - e * tpe) * 4;
    // row of actv and v that this edge reads (an index outside the rows is clamped: never an access out of bounds)
    const long en = node ? min(max((long)node[e], 0L), n_rows - 1) : e;
    const float* de = dist + e * 4 * n + c;
    const float* ae = actv + en * 4 * n + c;
    const float4 p0 = mul4(ld4(de), ld4(ae)), p1 = mul4(ld4(de + n), ld4(ae + n));
    const float4 p2 = mul4(ld4(de + 2 * n), ld4(ae + 2 * n)), p3 = mul4(ld4(de + 3 * n), ld4(ae + 3 * n));
    const Vec3x4 vv = ld12(v + (en * n + c) * 3);
    const Vec3 d = {dir[3 * e], dir[3 * e + 1], dir[3 * e + 2]};
    // terms (bit k: the term with p[k n + c] takes part): all four for the message itself; subsets when a gradient of
    // a gradient puts another tensor in the place of v (bits 0, 1: the terms that contain v) or of d (bits 1, 2)
    const float k0 = (terms & 1) ? 1.f : 0.f, k1 = (terms & 2) ? 1.f : 0.f, k2 = (terms & 4) ? 1.f : 0.f;
    const float k3 = (terms & 8) ? 1.f : 0.f;
    Vec3x4 out;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const Vec3 x = vv.get(j), xd = cross(x, d);
        const float s0 = at(p0, j) * k0, s1 = at(p1, j) * k1, s2 = at(p2, j) * k2;
        out.set(j, {x.x * s0 + xd.x * s1 + d.x * s2, x.y * s0 + xd.y * s1 + d.y * s2, x.z * s0 + xd.z * s1 + d.z * s2});
    }
    st12(m + (e * n + c) * 3, out);
    st4(a + e * n + c, make_float4(p3.x * k3, p3.y * k3, p3.z * k3, p3.w * k3));
}

// 4-point Lagrange weights on the grid rows i - 1 .. i + 2 at the fraction t (the grid kernels further down use them too)
__device__ __forceinline__ void lagrange4(float t, float (&w)[4]) {
    const float tp = t + 1.0f, tm = t - 1.0f, tq = t - 2.0f;
    w[0] = -(1.0f / 6.0f) * t * tm * tq;
    w[1] = 0.5f * tp * tm * tq;
    w[2] = -0.5f * tp * t * tq;
    w[3] = (1.0f / 6.0f) * tp * t * tm;
}
__device__ __forceinline__ float4 fma4(float w, float4 a, float4 acc) {
    return make_float4(fmaf(w, a.x, acc.x), fmaf(w, a.y, acc.y), fmaf(w, a.z, acc.z), fmaf(w, a.w, acc.w));
}

// The same pass with the sums over the edges of a source node inside: a group of n / 4 threads owns an output row r
// and walks its edges (positions row_ptr[r] .. row_ptr[r + 1] - 1 of the edge arrays, which are sorted by that row),
// adds their m and a in that order and writes out_v[r], out_a[r] once: no per-edge m and a and no segment sums after.
__global__ void __launch_bounds__(256) painn_combine_fwd_rows_kernel(
    const float* __restrict__ dist, const float* __restrict__ actv, const float* __restrict__ v,
    const float* __restrict__ dir, const int* __restrict__ node, long n_rows, const int* __restrict__ row_ptr,
    long n_out_rows, long E, int n, int terms, float* __restrict__ out_v, float* __restrict__ out_a) {
    const int tpe = n >> 2;
    const long t = (long)blockIdx.x * 256 + threadIdx.x;
    const long r = t / tpe;
    if (r >= n_out_rows) return;
    const int c = (int)(t - r * tpe) * 4;
    const float k0 = (terms & 1) ? 1.f : 0.f, k1 = (terms & 2) ? 1.f : 0.f, k2 = (terms & 4) ? 1.f : 0.f;
    const float k3 = (terms & 8) ? 1.f : 0.f;
    Vec3x4 acc_m;
#pragma unroll
    for (int q = 0; q < 12; q++) acc_m.f[q] = 0.f;
    float4 acc_a = make_float4(0.f, 0.f, 0.f, 0.f);
    const long lo = max((long)row_ptr[r], 0L), hi = min((long)row_ptr[r + 1], E);
    for (long e = lo; e < hi; e++) {
        const long en = node ? min(max((long)node[e], 0L), n_rows - 1) : e;
        const float* de = dist + e * 4 * n + c;
        const float* ae = actv + en * 4 * n + c;
        const float4 p0 = mul4(ld4(de), ld4(ae)), p1 = mul4(ld4(de + n), ld4(ae + n));
        const float4 p2 = mul4(ld4(de + 2 * n), ld4(ae + 2 * n)), p3 = mul4(ld4(de + 3 * n), ld4(ae + 3 * n));
        const Vec3x4 vv = ld12(v + (en * n + c) * 3);
        const Vec3 d = {dir[3 * e], dir[3 * e + 1], dir[3 * e + 2]};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const Vec3 x = vv.get(j), xd = cross(x, d);
            const float s0 = at(p0, j) * k0, s1 = at(p1, j) * k1, s2 = at(p2, j) * k2;
            acc_m.f[3 * j] += x.x * s0 + xd.x * s1 + d.x * s2;
            acc_m.f[3 * j + 1] += x.y * s0 + xd.y * s1 + d.y * s2;
            acc_m.f[3 * j + 2] += x.z * s0 + xd.z * s1 + d.z * s2;
        }
        acc_a.x += p3.x * k3; acc_a.y += p3.y * k3; acc_a.z += p3.z * k3; acc_a.w += p3.w * k3;
    }
    st12(out_v + (r * n + c) * 3, acc_m);
    st4(out_a + r * n + c, acc_a);
}

// Adjoint: with p = dist actv and dp its gradient,
//   dp[c] = dm[c] . v[c],  dp[n + c] = dm[c] . (v[c] x d),  dp[2n + c] = dm[c] . d,  dp[3n + c] = da[c]
//   d_dist = dp actv,  d_actv = dp dist,  dv[c] = dm[c] p[c] + (d x dm[c]) p[n + c]
//   d_dir = sum_c (dm[c] x v[c]) p[n + c] + dm[c] p[2n + c]
// GRID: dist is a (mask + 1, 4n) grid of the filter over one period of the edge length and edge e interpolates its row
// at len[e] (the arithmetic of table_interp_kernel, order 0): the per-edge filter is never stored.
template <bool GRID>
__global__ void __launch_bounds__(256) painn_combine_bwd_kernel(
    const float* __restrict__ dist, const float* __restrict__ actv, const float* __restrict__ v,
    const float* __restrict__ dir, const int* __restrict__ node, long n_rows, const float* __restrict__ dm,
    const float* __restrict__ da, const int* __restrict__ grad_row, long n_grad_rows, long E, int n, int terms,
    float* __restrict__ d_dist, float* __restrict__ d_actv, float* __restrict__ dv, float* __restrict__ d_dir,
    const float* __restrict__ len, int mask, float inv_h) {
    const int tpe = n >> 2;                                       // a power of two <= 64
    const long t = (long)blockIdx.x * 256 + threadIdx.x;
    const long e_raw = t / tpe;
    const bool live = e_raw < E;                                  // (dead threads still take part in the shuffles)
    const long e = live ? e_raw : E - 1;
    const int c = (int)(t - e_raw * tpe) * 4;
    // row of actv and v that this edge reads (an index outside the rows is clamped: never an access out of bounds)
    const long en = node ? min(max((long)node[e], 0L), n_rows - 1) : e;
    const float* ae = actv + en * 4 * n + c;
    float4 dk[4], ak[4];
#pragma unroll
    for (int k = 0; k < 4; k++) ak[k] = ld4(ae + k * n);
    if constexpr (GRID) {
        const float u = len[e] * inv_h, fl = floorf(u);
        float w[4];
        lagrange4(u - fl, w);
        const int i = (int)fl;
#pragma unroll
        for (int k = 0; k < 4; k++) dk[k] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float* row = dist + (long)((i - 1 + j) & mask) * 4 * n + c;
#pragma unroll
            for (int k = 0; k < 4; k++) dk[k] = fma4(w[j], ld4(row + k * n), dk[k]);
        }
    } else {
        const float* de = dist + e * 4 * n + c;
#pragma unroll
        for (int k = 0; k < 4; k++) dk[k] = ld4(de + k * n);
    }
    // row of dm and da: the edge itself, or (the outputs were summed over the edges of a source node) that node
    const long eg = grad_row ? min(max((long)grad_row[e], 0L), n_grad_rows - 1) : e;
    const Vec3x4 vv = ld12(v + (en * n + c) * 3), g = ld12(dm + (eg * n + c) * 3);
    const float4 ga = ld4(da + eg * n + c);
    const Vec3 d = {dir[3 * e], dir[3 * e + 1], dir[3 * e + 2]};
    const float k0 = (terms & 1) ? 1.f : 0.f, k1 = (terms & 2) ? 1.f : 0.f, k2 = (terms & 4) ? 1.f : 0.f;
    const float k3 = (terms & 8) ? 1.f : 0.f;
    float dp[3][4];
    Vec3x4 gv;
    Vec3 gd = {0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const Vec3 x = vv.get(j), gm = g.get(j);
        const float p0 = at(dk[0], j) * at(ak[0], j) * k0, p1 = at(dk[1], j) * at(ak[1], j) * k1;
        const float p2 = at(dk[2], j) * at(ak[2], j) * k2;
        dp[0][j] = dot(gm, x) * k0;
        dp[1][j] = dot(gm, cross(x, d)) * k1;
        dp[2][j] = dot(gm, d) * k2;
        const Vec3 dg = cross(d, gm), gx = cross(gm, x);
        gv.set(j, {gm.x * p0 + dg.x * p1, gm.y * p0 + dg.y * p1, gm.z * p0 + dg.z * p1});
        gd.x += gx.x * p1 + gm.x * p2;
        gd.y += gx.y * p1 + gm.y * p2;
        gd.z += gx.z * p1 + gm.z * p2;
    }
    for (int s = 1; s < tpe; s <<= 1) {
        gd.x += __shfl_xor(gd.x, s);
        gd.y += __shfl_xor(gd.y, s);
        gd.z += __shfl_xor(gd.z, s);
    }
    if (!live) return;
    // (an output that the caller does not want is a null pointer: uniform branches)
    const float4 ga3 = make_float4(ga.x * k3, ga.y * k3, ga.z * k3, ga.w * k3);
    if (d_dist) {
        float* dde = d_dist + e * 4 * n + c;
#pragma unroll
        for (int k = 0; k < 3; k++) st4(dde + k * n, mul4(make_float4(dp[k][0], dp[k][1], dp[k][2], dp[k][3]), ak[k]));
        st4(dde + 3 * n, mul4(ga3, ak[3]));
    }
    if (d_actv) {
        float* dae = d_actv + e * 4 * n + c;
#pragma unroll
        for (int k = 0; k < 3; k++) st4(dae + k * n, mul4(make_float4(dp[k][0], dp[k][1], dp[k][2], dp[k][3]), dk[k]));
        st4(dae + 3 * n, mul4(ga3, dk[3]));
    }
    if (dv) st12(dv + (e * n + c) * 3, gv);
    if (d_dir && c == 0) { d_dir[3 * e] = gd.x; d_dir[3 * e + 1] = gd.y; d_dir[3 * e + 2] = gd.z; }
}

// The same adjoint with the gradients of actv and v summed inside the kernel.  actv and v hold one row per node and
// every edge reads the row of its destination; a group of n / 4 threads owns one such row r and walks the edges that
// read it (edge ids order[row_ptr[r]] .. order[row_ptr[r + 1] - 1], or the positions themselves when order is null:
// edges sorted by that row), keeps the row's actv and v in registers, adds the edges' contributions to d_actv[r] and
// dv[r] in that order (the same on every run) and writes them once: no per-edge copies of the two gradients and no
// segment sums after the kernel.  d_dist and d_dir stay per edge.  GRID as above.
template <bool GRID>
__global__ void __launch_bounds__(256) painn_combine_bwd_rows_kernel(
    const float* __restrict__ dist, const float* __restrict__ actv, const float* __restrict__ v,
    const float* __restrict__ dir, const int* __restrict__ row_ptr, const int* __restrict__ order, long n_rows,
    const float* __restrict__ dm, const float* __restrict__ da, const int* __restrict__ grad_row, long n_grad_rows,
    long E, int n, int terms, float* __restrict__ d_dist, float* __restrict__ d_actv, float* __restrict__ dv,
    float* __restrict__ d_dir, const float* __restrict__ len, int mask, float inv_h) {
    const int tpe = n >> 2;                                       // a power of two <= 64: a group never straddles waves
    const long t = (long)blockIdx.x * 256 + threadIdx.x;
    const long r_raw = t / tpe;
    const bool live = r_raw < n_rows;
    const long r = live ? r_raw : n_rows - 1;
    const int c = (int)(t - r_raw * tpe) * 4;
    const float* ae = actv + r * 4 * n + c;
    float4 ak[4], acc_a[4];
#pragma unroll
    for (int k = 0; k < 4; k++) { ak[k] = ld4(ae + k * n); acc_a[k] = make_float4(0.f, 0.f, 0.f, 0.f); }
    const Vec3x4 vv = ld12(v + (r * n + c) * 3);
    Vec3x4 acc_v;
#pragma unroll
    for (int q = 0; q < 12; q++) acc_v.f[q] = 0.f;
    const float k0 = (terms & 1) ? 1.f : 0.f, k1 = (terms & 2) ? 1.f : 0.f, k2 = (terms & 4) ? 1.f : 0.f;
    const float k3 = (terms & 8) ? 1.f : 0.f;
    // (the threads of a group share r, so they make the same trips and the shuffles below stay inside live lanes)
    const int lo = max(row_ptr[r], 0), hi = live ? min(row_ptr[r + 1], (int)min(E, 0x7fffffffL)) : lo;
    for (int pos = lo; pos < hi; pos++) {
        long e = order ? (long)order[pos] : (long)pos;
        e = min(max(e, 0L), E - 1);                               // (never an access out of bounds)
        float4 dk[4];
        if constexpr (GRID) {
            const float u = len[e] * inv_h, fl = floorf(u);
            float w[4];
            lagrange4(u - fl, w);
            const int i = (int)fl;
#pragma unroll
            for (int k = 0; k < 4; k++) dk[k] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float* row = dist + (long)((i - 1 + j) & mask) * 4 * n + c;
#pragma unroll
                for (int k = 0; k < 4; k++) dk[k] = fma4(w[j], ld4(row + k * n), dk[k]);
            }
        } else {
            const float* de = dist + e * 4 * n + c;
#pragma unroll
            for (int k = 0; k < 4; k++) dk[k] = ld4(de + k * n);
        }
        const long eg = grad_row ? min(max((long)grad_row[e], 0L), n_grad_rows - 1) : e;
        const Vec3x4 g = ld12(dm + (eg * n + c) * 3);
        const float4 ga = ld4(da + eg * n + c);
        const Vec3 d = {dir[3 * e], dir[3 * e + 1], dir[3 * e + 2]};
        float dp[3][4];
        Vec3 gd = {0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const Vec3 x = vv.get(j), gm = g.get(j);
            const float p0 = at(dk[0], j) * at(ak[0], j) * k0, p1 = at(dk[1], j) * at(ak[1], j) * k1;
            const float p2 = at(dk[2], j) * at(ak[2], j) * k2;
            dp[0][j] = dot(gm, x) * k0;
            dp[1][j] = dot(gm, cross(x, d)) * k1;
            dp[2][j] = dot(gm, d) * k2;
            const Vec3 dg = cross(d, gm), gx = cross(gm, x);
            acc_v.f[3 * j] += gm.x * p0 + dg.x * p1;
            acc_v.f[3 * j + 1] += gm.y * p0 + dg.y * p1;
            acc_v.f[3 * j + 2] += gm.z * p0 + dg.z * p1;
            gd.x += gx.x * p1 + gm.x * p2;
            gd.y += gx.y * p1 + gm.y * p2;
            gd.z += gx.z * p1 + gm.z * p2;
        }
        const float4 ga3 = make_float4(ga.x * k3, ga.y * k3, ga.z * k3, ga.w * k3);
        float4 dpk[4];
#pragma unroll
        for (int k = 0; k < 3; k++) dpk[k] = make_float4(dp[k][0], dp[k][1], dp[k][2], dp[k][3]);
        dpk[3] = ga3;
        if (d_dist) {
            float* dde = d_dist + e * 4 * n + c;
#pragma unroll
            for (int k = 0; k < 4; k++) st4(dde + k * n, mul4(dpk[k], ak[k]));
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            acc_a[k].x = fmaf(dpk[k].x, dk[k].x, acc_a[k].x);
            acc_a[k].y = fmaf(dpk[k].y, dk[k].y, acc_a[k].y);
            acc_a[k].z = fmaf(dpk[k].z, dk[k].z, acc_a[k].z);
            acc_a[k].w = fmaf(dpk[k].w, dk[k].w, acc_a[k].w);
        }
        if (d_dir) {                                              // (uniform)
            for (int sh = 1; sh < tpe; sh <<= 1) {
                gd.x += __shfl_xor(gd.x, sh);
                gd.y += __shfl_xor(gd.y, sh);
                gd.z += __shfl_xor(gd.z, sh);
            }
            if (c == 0) { d_dir[3 * e] = gd.x; d_dir[3 * e + 1] = gd.y; d_dir[3 * e + 2] = gd.z; }
        }
    }
    if (!live) return;
    if (d_actv) {
        float* dae = d_actv + r * 4 * n + c;
#pragma unroll
        for (int k = 0; k < 4; k++) st4(dae + k * n, acc_a[k]);
    }
    if (dv) st12(dv + (r * n + c) * 3, acc_v);
}

// ---------------------------------------------------------------------------------------------------------------
// The filter from its grid, for training.  The filter MLP sees an edge only through its length d, so inference
// evaluates it on a grid over one period of d and interpolates (painn.hip); training can do the same: the forward
// pass interpolates the (rows, cols) grid at every edge, and the backward pass sends each edge's gradient row to the
// four grid rows it read, after which the MLP is differentiated on the grid's few hundred rows instead of on every
// edge.  Interpolation as in painn.hip: u = d * inv_h, i = floor(u), t = u - i, 4-point Lagrange weights on the rows
// i - 1 .. i + 2 (mod rows; rows is a power of two).
//
// The sum over edges has to come out the same on every run: the edges are taken in the order of a stable sort by
// grid row (perm, bucket_ptr from the host side), each grid row's edges are cut into `splits` consecutive pieces,
// a workgroup sums one piece (its thread groups take the piece's edges round robin, each in order, and are added in
// group order), and the pieces and the four taps are added in a fixed order by a second kernel.
__device__ __forceinline__ void lagrange4_derivative(float t, float (&w)[4]) {
    const float tp = t + 1.0f, tm = t - 1.0f, tq = t - 2.0f;
    w[0] = -(1.0f / 6.0f) * (tm * tq + t * tq + t * tm);
    w[1] = 0.5f * (tm * tq + tp * tq + tp * tm);
    w[2] = -0.5f * (t * tq + tp * tq + tp * t);
    w[3] = (1.0f / 6.0f) * (t * tm + tp * tm + tp * t);
}
// the order-th derivative of the four weights with respect to t (order 0 .. 3; the weights are cubics)
__device__ __forceinline__ void lagrange4_order(float t, int order, float (&w)[4]) {
    if (order == 0) { lagrange4(t, w); return; }
    if (order == 1) { lagrange4_derivative(t, w); return; }
    if (order == 2) {
        w[0] = 1.0f - t; w[1] = 3.0f * t - 2.0f; w[2] = 1.0f - 3.0f * t; w[3] = t;
        return;
    }
    w[0] = -1.0f; w[1] = 3.0f; w[2] = -3.0f; w[3] = 1.0f;
}

// bucket[e] = i_e & mask, the grid row an edge is sorted by (computed here so that it is the kernels' own i_e)
__global__ void __launch_bounds__(256) table_bucket_kernel(const float* __restrict__ d, long E, int mask, float inv_h,
                                                           int* __restrict__ bucket) {
    const long e = (long)blockIdx.x * 256 + threadIdx.x;
    if (e < E) bucket[e] = (int)floorf(d[e] * inv_h) & mask;
}

// out[e, :] = sum_j w_j(t_e) table[(i_e - 1 + j) & mask, :]; a thread owns 4 columns of one edge
// (order > 0: the order-th derivative with respect to d, weights differentiated and scaled by inv_h^order)
__global__ void __launch_bounds__(256) table_interp_kernel(const float* __restrict__ table, const float* __restrict__ d,
                                                           long E, int cols, int mask, float inv_h, int order,
                                                           float scale, float* __restrict__ out) {
    const int tpe = cols >> 2;
    const long t = (long)blockIdx.x * 256 + threadIdx.x;
    const long e = t / tpe;
    if (e >= E) return;
    const int c = (int)(t - e * tpe) * 4;
    const float u = d[e] * inv_h, fl = floorf(u);
    float w[4];
    lagrange4_order(u - fl, order, w);
    const int i = (int)fl;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int j = 0; j < 4; j++) acc = fma4(w[j] * scale, ld4(table + (long)((i - 1 + j) & mask) * cols + c), acc);
    st4(out + e * cols + c, acc);
}

// part[((row * splits + s) * 4 + j) * cols + c] = sum over the edges e of piece s of grid row `row` of w_j(t_e) g[e, c]
__global__ void __launch_bounds__(256) table_scatter_kernel(const float* __restrict__ g, const float* __restrict__ d,
                                                            const int* __restrict__ perm,
                                                            const int* __restrict__ bucket_ptr, int cols, float inv_h,
                                                            int order, float scale, int splits,
                                                            float* __restrict__ part) {
    __shared__ float4 fold[256 * 4];
    const int tpe = cols >> 2;                                    // threads per edge: a power of two <= 256
    const int groups = 256 / tpe, group = threadIdx.x / tpe;
    const int c = (threadIdx.x - group * tpe) * 4;
    const int row = blockIdx.x, s = blockIdx.y;
    const long lo = bucket_ptr[row], hi = bucket_ptr[row + 1];
    const long len = hi - lo;
    const long p_lo = lo + len * s / splits, p_hi = lo + len * (s + 1) / splits;
    float4 acc[4];
#pragma unroll
    for (int j = 0; j < 4; j++) acc[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    long p = p_lo + group;
    for (; p + 3 * groups < p_hi; p += 4 * groups) {              // four edges in flight, added in order
        long e[4];
        float u[4];
        float4 ge[4];
#pragma unroll
        for (int q = 0; q < 4; q++) e[q] = perm[p + q * groups];
#pragma unroll
        for (int q = 0; q < 4; q++) { u[q] = d[e[q]] * inv_h; ge[q] = ld4(g + e[q] * cols + c); }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            float w[4];
            lagrange4_order(u[q] - floorf(u[q]), order, w);
#pragma unroll
            for (int j = 0; j < 4; j++) acc[j] = fma4(w[j] * scale, ge[q], acc[j]);
        }
    }
    for (; p < p_hi; p += groups) {
        const long e = perm[p];
        const float u = d[e] * inv_h;
        float w[4];
        lagrange4_order(u - floorf(u), order, w);
        const float4 ge = ld4(g + e * cols + c);
#pragma unroll
        for (int j = 0; j < 4; j++) acc[j] = fma4(w[j] * scale, ge, acc[j]);
    }
    // thread groups added in group order
#pragma unroll
    for (int j = 0; j < 4; j++) fold[threadIdx.x * 4 + j] = acc[j];
    __syncthreads();
    if (group == 0) {
        for (int k = 1; k < groups; k++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float4 o = fold[(k * tpe + threadIdx.x) * 4 + j];
                acc[j].x += o.x; acc[j].y += o.y; acc[j].z += o.z; acc[j].w += o.w;
            }
        float* dst = part + ((long)(row * splits + s) * 4) * cols + c;
#pragma unroll
        for (int j = 0; j < 4; j++) st4(dst + (long)j * cols, acc[j]);
    }
}

// d_table[m, :] = sum_j sum_s part[(m + 1 - j) & mask][s][j][:], taps and pieces in this order
__global__ void __launch_bounds__(256) table_scatter_finish_kernel(const float* __restrict__ part, int rows, int cols,
                                                                   int splits, float* __restrict__ d_table) {
    const int tpe = cols >> 2;
    const long t = (long)blockIdx.x * 256 + threadIdx.x;
    const long m = t / tpe;
    if (m >= rows) return;
    const int c = (int)(t - m * tpe) * 4;
    const int mask = rows - 1;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int j = 0; j < 4; j++) {
        const long row = (m + 1 - j) & mask;
        const float* src = part + ((row * splits) * 4 + j) * (long)cols + c;
        int s = 0;
        for (; s + 8 <= splits; s += 8) {                      // eight loads in flight, added in piece order
            float4 v[8];
#pragma unroll
            for (int q = 0; q < 8; q++) v[q] = ld4(src + (long)(s + q) * 4 * cols);
#pragma unroll
            for (int q = 0; q < 8; q++) { acc.x += v[q].x; acc.y += v[q].y; acc.z += v[q].z; acc.w += v[q].w; }
        }
        for (; s < splits; s++) {
            const float4 v = ld4(src + (long)s * 4 * cols);
            acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
        }
    }
    st4(d_table + m * cols + c, acc);
}

// dd[e] = inv_h * sum_c g[e, c] sum_j w_j'(t_e) table[(i_e - 1 + j) & mask, c]: a wave per edge
__global__ void __launch_bounds__(256) table_interp_grad_length_kernel(const float* __restrict__ g,
                                                                       const float* __restrict__ table,
                                                                       const float* __restrict__ d, long E, int cols,
                                                                       int mask, float inv_h, int order, float scale,
                                                                       float* __restrict__ dd) {
    const int lane = threadIdx.x & 63;
    const long wave = ((long)blockIdx.x * 256 + threadIdx.x) >> 6, n_waves = ((long)gridDim.x * 256) >> 6;
    for (long e = wave; e < E; e += n_waves) {
        const float u = d[e] * inv_h, fl = floorf(u);
        float w[4];
        lagrange4_order(u - fl, order + 1, w);
        const int i = (int)fl;
        float s = 0.f;
        for (int c = lane * 4; c < cols; c += 256) {
            float4 tv = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int j = 0; j < 4; j++) tv = fma4(w[j], ld4(table + (long)((i - 1 + j) & mask) * cols + c), tv);
            const float4 ge = ld4(g + e * cols + c);
            s += ge.x * tv.x + ge.y * tv.y + ge.z * tv.z + ge.w * tv.w;
        }
        for (int k = 1; k < 64; k <<= 1) s += __shfl_xor(s, k);
        if (lane == 0) dd[e] = s * scale * inv_h;
    }
}

// pieces per grid row: 16 for 512 rows, fewer for finer grids (whose rows hold fewer edges): the partial sums stay
// within 64 MB for 512 columns
inline int table_splits(int rows) { const int s = 8192 / rows; return s < 1 ? 1 : (s > 16 ? 16 : s); }
inline bool table_shape_ok(int rows, int cols) {
    return rows >= 4 && (rows & (rows - 1)) == 0 && cols >= 4 && cols <= 1024 && (cols & (cols - 1)) == 0;
}

// ---------------------------------------------------------------------------------------------------------------
// The edge filters of the rank-0/1/2 Messages layer (archs/diffuser_atoms15.py:240-243) for its training path:
//   phi_v[e, c, i] = enc[e, c] rh[e, i],   phi_d[e, c, i, j] = (enc[e, c] rh[e, j]) rh[e, i]
// and the adjoint: d_enc[e, c] = sum_i g_v[e,c,i] rh[e,i] + sum_ij g_d[e,c,i,j] rh[e,i] rh[e,j],
//   d_rh[e, k] = sum_c enc[e,c] (g_v[e,c,k] + sum_j (g_d[e,c,k,j] + g_d[e,c,j,k]) rh[e,j]).
// As broadcasting tensor arithmetic these are two passes forward and a dozen (products and reductions over the
// broadcast axes) backward over (E, C, 9) arrays.  One workgroup per edge; the channel sum of d_rh is reduced in LDS
// in a fixed order.
__global__ void __launch_bounds__(256) edge_filters_fwd_kernel(const float* __restrict__ enc, const float* __restrict__ rh,
                                                               int C, float* __restrict__ phi_v, float* __restrict__ phi_d) {
    const long e = blockIdx.x;
    const float r[3] = {rh[3 * e], rh[3 * e + 1], rh[3 * e + 2]};
    for (int c = threadIdx.x; c < C; c += 256) {
        const float v = enc[e * C + c];
        float* pv = phi_v + (e * C + c) * 3;
        float* pd = phi_d + (e * C + c) * 9;
#pragma unroll
        for (int i = 0; i < 3; i++) pv[i] = v * r[i];
#pragma unroll
        for (int i = 0; i < 3; i++)
#pragma unroll
            for (int j = 0; j < 3; j++) pd[3 * i + j] = (v * r[j]) * r[i];
    }
}

__global__ void __launch_bounds__(256) edge_filters_bwd_kernel(const float* __restrict__ enc, const float* __restrict__ rh,
                                                               const float* __restrict__ g_v, const float* __restrict__ g_d,
                                                               int C, float* __restrict__ d_enc, float* __restrict__ d_rh) {
    __shared__ float part[4][3];
    const long e = blockIdx.x;
    const float r[3] = {rh[3 * e], rh[3 * e + 1], rh[3 * e + 2]};
    float acc[3] = {0.f, 0.f, 0.f};
    for (int c = threadIdx.x; c < C; c += 256) {
        const float v = enc[e * C + c];
        const float* gv = g_v + (e * C + c) * 3;
        const float* gd = g_d + (e * C + c) * 9;
        float g9[9], g3[3];
#pragma unroll
        for (int k = 0; k < 9; k++) g9[k] = gd[k];
#pragma unroll
        for (int k = 0; k < 3; k++) g3[k] = gv[k];
        float de = 0.f;
#pragma unroll
        for (int i = 0; i < 3; i++) {
            de += g3[i] * r[i];
            float row = 0.f, sym = 0.f;
#pragma unroll
            for (int j = 0; j < 3; j++) { row += g9[3 * i + j] * r[j]; sym += (g9[3 * i + j] + g9[3 * j + i]) * r[j]; }
            de += row * r[i];
            acc[i] += v * (g3[i] + sym);
        }
        d_enc[e * C + c] = de;
    }
#pragma unroll
    for (int k = 0; k < 3; k++)
        for (int s = 1; s < 64; s <<= 1) acc[k] += __shfl_xor(acc[k], s);
    if ((threadIdx.x & 63) == 0)
        for (int k = 0; k < 3; k++) part[threadIdx.x >> 6][k] = acc[k];
    __syncthreads();
    if (threadIdx.x < 3) d_rh[3 * e + threadIdx.x] = (part[0][threadIdx.x] + part[1][threadIdx.x]) + (part[2][threadIdx.x] + part[3][threadIdx.x]);
}

inline bool combine_shape_ok(int n) { return n >= 4 && n <= 256 && (n & (n - 1)) == 0; }


// k-th derivative of SiLU(z) = z sigma(z), k = 0..4, times an optional factor.  With s = sigma(z), p = s (1 - s) and
// u = 1 - 2 s the derivatives of sigma are d1 = p, d2 = p u, d3 = p (u^2 - 2 p), d4 = p u (u^2 - 8 p), and
// SiLU^(k) = k d(k-1) + z d(k).  Differentiating an MLP k times needs SiLU^(k) of the same pre-activations;
// autograd's own formula for the derivative of SiLU's derivative is a chain of seven elementwise launches.
__device__ __forceinline__ float silu_derivative(float z, int order) {
    const float s = 1.0f / (1.0f + expf(-z));
    if (order == 0) return z * s;
    const float p = s * (1.0f - s), u = 1.0f - 2.0f * s;
    if (order == 1) return s + z * p;
    if (order == 2) return p * (2.0f + z * u);
    const float q = u * u - 2.0f * p;
    if (order == 3) return p * (3.0f * u + z * q);
    return p * (4.0f * q + z * u * (u * u - 8.0f * p));
}

__global__ void __launch_bounds__(256) silu_order_kernel(const float* __restrict__ z, const float* __restrict__ mul,
                                                         long n, int order, float* __restrict__ out) {
    const long n4 = n / 4;
    for (long k = (long)blockIdx.x * blockDim.x + threadIdx.x; k < n4; k += (long)gridDim.x * blockDim.x) {
        const float4 v = reinterpret_cast<const float4*>(z)[k];
        float4 r = make_float4(silu_derivative(v.x, order), silu_derivative(v.y, order), silu_derivative(v.z, order),
                               silu_derivative(v.w, order));
        if (mul) {
            const float4 m = reinterpret_cast<const float4*>(mul)[k];
            r.x *= m.x; r.y *= m.y; r.z *= m.z; r.w *= m.w;
        }
        reinterpret_cast<float4*>(out)[k] = r;
    }
    if (blockIdx.x == 0 && threadIdx.x < n - 4 * n4) {
        const long k = 4 * n4 + threadIdx.x;
        out[k] = silu_derivative(z[k], order) * (mul ? mul[k] : 1.0f);
    }
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_painn_combine_supported(int n) { return combine_shape_ok(n) ? 1 : 0; }

int mg_painn_combine_fwd(const float* dist, const float* actv, const float* v, const float* dir, const int* node,
                         long n_rows, long E, int n, int terms, float* m, float* a, mg_stream_t stream) {
    MG_REQUIRE(E >= 0 && combine_shape_ok(n), "mg_painn_combine_fwd: n must be a power of two in 4..256");
    MG_REQUIRE(terms >= 0 && terms <= 15, "mg_painn_combine_fwd: terms is a mask of four bits");
    if (E == 0) return MG_OK;
    MG_REQUIRE(dist && actv && v && dir && m && a, "mg_painn_combine_fwd: null pointer");
    MG_REQUIRE(node == nullptr || n_rows > 0, "mg_painn_combine_fwd: an index needs n_rows > 0");
    MG_REQUIRE(aligned16(dist) && aligned16(actv) && aligned16(v) && aligned16(m) && aligned16(a),
               "mg_painn_combine_fwd: arrays must be 16-byte aligned");
    const long threads = E * (n / 4);
    MG_REQUIRE(ceil_div(threads, 256) < (1L << 31), "mg_painn_combine_fwd: too many edges");
    hipLaunchKernelGGL(painn_combine_fwd_kernel, dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0,
                       (hipStream_t)stream, dist, actv, v, dir, node, n_rows, E, n, terms, m, a);
    return check_launch("mg_painn_combine_fwd");
}

int mg_painn_combine_fwd_rows(const float* dist, const float* actv, const float* v, const float* dir, const int* node,
                              long n_rows, const int* row_ptr, long n_out_rows, long E, int n, int terms, float* out_v,
                              float* out_a, mg_stream_t stream) {
    MG_REQUIRE(E >= 0 && n_out_rows >= 0 && combine_shape_ok(n), "mg_painn_combine_fwd_rows: n must be a power of two in 4..256");
    MG_REQUIRE(terms >= 0 && terms <= 15, "mg_painn_combine_fwd_rows: terms is a mask of four bits");
    if (n_out_rows == 0) return MG_OK;
    MG_REQUIRE(row_ptr && out_v && out_a && (E == 0 || (dist && actv && v && dir)), "mg_painn_combine_fwd_rows: null pointer");
    MG_REQUIRE(node == nullptr || n_rows > 0, "mg_painn_combine_fwd_rows: an index needs n_rows > 0");
    MG_REQUIRE(aligned16(dist) && aligned16(actv) && aligned16(v) && aligned16(out_v) && aligned16(out_a),
               "mg_painn_combine_fwd_rows: arrays must be 16-byte aligned");
    const long threads = n_out_rows * (n / 4);
    MG_REQUIRE(ceil_div(threads, 256) < (1L << 31), "mg_painn_combine_fwd_rows: too many rows");
    hipLaunchKernelGGL(painn_combine_fwd_rows_kernel, dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0,
                       (hipStream_t)stream, dist, actv, v, dir, node, n_rows, row_ptr, n_out_rows, E, n, terms, out_v, out_a);
    return check_launch("mg_painn_combine_fwd_rows");
}

int mg_painn_combine_bwd(const float* dist, const float* actv, const float* v, const float* dir, const int* node,
                         long n_rows, const float* dm, const float* da, const int* grad_row, long n_grad_rows, long E,
                         int n, int terms, float* d_dist, float* d_actv, float* dv, float* d_dir, mg_stream_t stream) {
    MG_REQUIRE(E >= 0 && combine_shape_ok(n), "mg_painn_combine_bwd: n must be a power of two in 4..256");
    MG_REQUIRE(terms >= 0 && terms <= 15, "mg_painn_combine_bwd: terms is a mask of four bits");
    if (E == 0) return MG_OK;
    MG_REQUIRE(dist && actv && v && dir && dm && da, "mg_painn_combine_bwd: null pointer");
    if (!d_dist && !d_actv && !dv && !d_dir) return MG_OK;       // (any of the four outputs may be left out)
    MG_REQUIRE((node == nullptr || n_rows > 0) && (grad_row == nullptr || n_grad_rows > 0),
               "mg_painn_combine_bwd: an index needs a positive row count");
    MG_REQUIRE(aligned16(dist) && aligned16(actv) && aligned16(v) && aligned16(dm) && aligned16(da) &&
                   aligned16(d_dist) && aligned16(d_actv) && aligned16(dv),
               "mg_painn_combine_bwd: arrays must be 16-byte aligned");     // (a null pointer counts as aligned)
    const long threads = E * (n / 4);
    MG_REQUIRE(ceil_div(threads, 256) < (1L << 31), "mg_painn_combine_bwd: too many edges");
    hipLaunchKernelGGL(painn_combine_bwd_kernel<false>, dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0,
                       (hipStream_t)stream, dist, actv, v, dir, node, n_rows, dm, da, grad_row, n_grad_rows, E, n, terms, d_dist,
                       d_actv, dv, d_dir, nullptr, 0, 0.f);
    return check_launch("mg_painn_combine_bwd");
}

int mg_painn_combine_bwd_grid(const float* table, int table_rows, float period, const float* len, const float* actv,
                              const float* v, const float* dir, const int* node, long n_rows, const float* dm,
                              const float* da, const int* grad_row, long n_grad_rows, long E, int n, int terms,
                              float* d_dist, float* d_actv, float* dv, float* d_dir, mg_stream_t stream) {
    MG_REQUIRE(E >= 0 && combine_shape_ok(n), "mg_painn_combine_bwd_grid: n must be a power of two in 4..256");
    MG_REQUIRE(table_shape_ok(table_rows, 4 * n) && period > 0.f,
               "mg_painn_combine_bwd_grid: grid rows must be a power of two, period positive");
    MG_REQUIRE(terms >= 0 && terms <= 15, "mg_painn_combine_bwd_grid: terms is a mask of four bits");
    if (E == 0) return MG_OK;
    MG_REQUIRE(table && len && actv && v && dir && dm && da, "mg_painn_combine_bwd_grid: null pointer");
    if (!d_dist && !d_actv && !dv && !d_dir) return MG_OK;       // (any of the four outputs may be left out)
    MG_REQUIRE((node == nullptr || n_rows > 0) && (grad_row == nullptr || n_grad_rows > 0),
               "mg_painn_combine_bwd_grid: an index needs a positive row count");
    MG_REQUIRE(aligned16(table) && aligned16(actv) && aligned16(v) && aligned16(dm) && aligned16(da) &&
                   aligned16(d_dist) && aligned16(d_actv) && aligned16(dv),
               "mg_painn_combine_bwd_grid: arrays must be 16-byte aligned");
    const long threads = E * (n / 4);
    MG_REQUIRE(ceil_div(threads, 256) < (1L << 31), "mg_painn_combine_bwd_grid: too many edges");
    hipLaunchKernelGGL(painn_combine_bwd_kernel<true>, dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0,
                       (hipStream_t)stream, table, actv, v, dir, node, n_rows, dm, da, grad_row, n_grad_rows, E, n, terms,
                       d_dist, d_actv, dv, d_dir, len, table_rows - 1, (float)table_rows / period);
    return check_launch("mg_painn_combine_bwd_grid");
}

int mg_painn_combine_bwd_rows(const float* dist, const float* table, int table_rows, float period, const float* len,
                              const float* actv, const float* v, const float* dir, const int* row_ptr, const int* order,
                              long n_rows, const float* dm, const float* da, const int* grad_row, long n_grad_rows,
                              long E, int n, int terms, float* d_dist, float* d_actv, float* dv, float* d_dir,
                              mg_stream_t stream) {
    MG_REQUIRE(E >= 0 && n_rows >= 0 && combine_shape_ok(n), "mg_painn_combine_bwd_rows: n must be a power of two in 4..256");
    MG_REQUIRE(terms >= 0 && terms <= 15, "mg_painn_combine_bwd_rows: terms is a mask of four bits");
    MG_REQUIRE(E == 0 || (dist != nullptr) != (table != nullptr),       // (without edges neither is read)
               "mg_painn_combine_bwd_rows: give dist or table, not both");
    MG_REQUIRE(table == nullptr || (table_shape_ok(table_rows, 4 * n) && period > 0.f && (len != nullptr || E == 0)),
               "mg_painn_combine_bwd_rows: grid rows must be a power of two, period positive, len given");
    if (n_rows == 0) return MG_OK;
    if (!d_dist && !d_actv && !dv && !d_dir) return MG_OK;       // (any of the four outputs may be left out)
    MG_REQUIRE(actv && v && row_ptr && (E == 0 || (dir && dm && da)), "mg_painn_combine_bwd_rows: null pointer");
    MG_REQUIRE(grad_row == nullptr || n_grad_rows > 0, "mg_painn_combine_bwd_rows: an index needs a positive row count");
    MG_REQUIRE(aligned16(dist) && aligned16(table) && aligned16(actv) && aligned16(v) && aligned16(dm) && aligned16(da) &&
                   aligned16(d_dist) && aligned16(d_actv) && aligned16(dv),
               "mg_painn_combine_bwd_rows: arrays must be 16-byte aligned");
    const long threads = n_rows * (n / 4);
    MG_REQUIRE(ceil_div(threads, 256) < (1L << 31), "mg_painn_combine_bwd_rows: too many rows");
    const dim3 grid((unsigned)ceil_div(threads, 256)), block(256);
    if (table)
        hipLaunchKernelGGL(painn_combine_bwd_rows_kernel<true>, grid, block, 0, (hipStream_t)stream, table, actv, v, dir,
                           row_ptr, order, n_rows, dm, da, grad_row, n_grad_rows, E, n, terms, d_dist, d_actv, dv, d_dir, len,
                           table_rows - 1, (float)table_rows / period);
    else
        hipLaunchKernelGGL(painn_combine_bwd_rows_kernel<false>, grid, block, 0, (hipStream_t)stream, dist, actv, v, dir,
                           row_ptr, order, n_rows, dm, da, grad_row, n_grad_rows, E, n, terms, d_dist, d_actv, dv, d_dir,
                           nullptr, 0, 0.f);
    return check_launch("mg_painn_combine_bwd_rows");
}

int mg_painn_table_interp_supported(int table_rows, int cols) { return table_shape_ok(table_rows, cols) ? 1 : 0; }

inline float int_power(float x, int k) { float p = 1.f; for (int i = 0; i < k; i++) p *= x; return p; }

int mg_painn_table_interp_fwd(const float* table, int table_rows, int cols, float period, const float* d, long E,
                              int order, float* out, mg_stream_t stream) {
    MG_REQUIRE(E >= 0 && table_shape_ok(table_rows, cols) && period > 0.f && order >= 0 && order <= 3,
               "mg_painn_table_interp_fwd: rows and cols must be powers of two (cols <= 1024), period positive, order 0..3");
    if (E == 0) return MG_OK;
    MG_REQUIRE(table && d && out && aligned16(table) && aligned16(out), "mg_painn_table_interp_fwd: null or unaligned pointer");
    const long threads = E * (cols / 4);
    MG_REQUIRE(ceil_div(threads, 256) < (1L << 31), "mg_painn_table_interp_fwd: too many edges");
    hipLaunchKernelGGL(table_interp_kernel, dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0, (hipStream_t)stream,
                       table, d, E, cols, table_rows - 1, (float)table_rows / period, order,
                       int_power((float)table_rows / period, order), out);
    return check_launch("mg_painn_table_interp_fwd");
}

int mg_painn_table_buckets(const float* d, long E, int table_rows, float period, int* bucket, mg_stream_t stream) {
    MG_REQUIRE(E >= 0 && table_rows >= 4 && (table_rows & (table_rows - 1)) == 0 && period > 0.f,
               "mg_painn_table_buckets: rows must be a power of two, period positive");
    if (E == 0) return MG_OK;
    MG_REQUIRE(d && bucket, "mg_painn_table_buckets: null pointer");
    hipLaunchKernelGGL(table_bucket_kernel, dim3((unsigned)ceil_div(E, 256)), dim3(256), 0, (hipStream_t)stream, d, E,
                       table_rows - 1, (float)table_rows / period, bucket);
    return check_launch("mg_painn_table_buckets");
}

int mg_painn_table_interp_bwd_workspace_bytes(int table_rows, int cols, size_t* bytes) {
    MG_REQUIRE(bytes != nullptr && table_shape_ok(table_rows, cols), "mg_painn_table_interp_bwd_workspace_bytes: bad argument");
    *bytes = (size_t)table_rows * table_splits(table_rows) * 4 * (size_t)cols * sizeof(float) + 16;
    return MG_OK;
}

int mg_painn_table_interp_bwd(const float* g, const float* table, int table_rows, int cols, float period, const float* d,
                              const int* perm, const int* bucket_ptr, long E, int order, void* workspace,
                              float* d_table, float* dd, mg_stream_t stream) {
    MG_REQUIRE(E >= 0 && table_shape_ok(table_rows, cols) && period > 0.f && order >= 0 && order <= 3,
               "mg_painn_table_interp_bwd: rows and cols must be powers of two (cols <= 1024), period positive, order 0..3");
    MG_REQUIRE(dd == nullptr || order < 3, "mg_painn_table_interp_bwd: the third derivative has no length gradient");
    MG_REQUIRE(d_table && workspace && bucket_ptr && aligned16(d_table), "mg_painn_table_interp_bwd: null or unaligned pointer");
    MG_REQUIRE(E == 0 || (g && d && perm && aligned16(g)), "mg_painn_table_interp_bwd: null or unaligned pointer");
    hipStream_t st = (hipStream_t)stream;
    const float inv_h = (float)table_rows / period;
    float* part = reinterpret_cast<float*>((reinterpret_cast<uintptr_t>(workspace) + 15) & ~uintptr_t(15));
    const float scale = int_power(inv_h, order);
    const int splits = table_splits(table_rows);
    hipLaunchKernelGGL(table_scatter_kernel, dim3((unsigned)table_rows, (unsigned)splits), dim3(256), 0, st, g, d, perm,
                       bucket_ptr, cols, inv_h, order, scale, splits, part);
    const long threads = (long)table_rows * (cols / 4);
    hipLaunchKernelGGL(table_scatter_finish_kernel, dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0, st,
                       (const float*)part, table_rows, cols, splits, d_table);
    if (dd && E > 0) {
        MG_REQUIRE(table && aligned16(table), "mg_painn_table_interp_bwd: the length gradient needs the table");
        long blocks = ceil_div(E, 4);
        if (blocks > 256L * 32) blocks = 256L * 32;
        hipLaunchKernelGGL(table_interp_grad_length_kernel, dim3((unsigned)blocks), dim3(256), 0, st, g, table, d, E, cols,
                           table_rows - 1, inv_h, order, scale, dd);
    }
    return check_launch("mg_painn_table_interp_bwd");
}

int mg_bee_edge_filters_fwd(const float* enc, const float* rh, long E, int chan, float* phi_v, float* phi_d,
                            mg_stream_t stream) {
    MG_REQUIRE(E >= 0 && chan >= 0 && E < (1L << 31), "mg_bee_edge_filters_fwd: bad size");
    if (E == 0 || chan == 0) return MG_OK;
    MG_REQUIRE(enc && rh && phi_v && phi_d, "mg_bee_edge_filters_fwd: null pointer");
    hipLaunchKernelGGL(edge_filters_fwd_kernel, dim3((unsigned)E), dim3(256), 0, (hipStream_t)stream, enc, rh, chan, phi_v,
                       phi_d);
    return check_launch("mg_bee_edge_filters_fwd");
}

int mg_bee_edge_filters_bwd(const float* enc, const float* rh, const float* g_v, const float* g_d, long E, int chan,
                            float* d_enc, float* d_rh, mg_stream_t stream) {
    MG_REQUIRE(E >= 0 && chan >= 0 && E < (1L << 31), "mg_bee_edge_filters_bwd: bad size");
    if (E == 0) return MG_OK;
    MG_REQUIRE(rh && d_rh && (chan == 0 || (enc && g_v && g_d && d_enc)), "mg_bee_edge_filters_bwd: null pointer");
    hipLaunchKernelGGL(edge_filters_bwd_kernel, dim3((unsigned)E), dim3(256), 0, (hipStream_t)stream, enc, rh, g_v, g_d,
                       chan, d_enc, d_rh);
    return check_launch("mg_bee_edge_filters_bwd");
}

int mg_silu_order(const float* z, const float* mul, long n, int order, float* out, mg_stream_t stream) {
    MG_REQUIRE(n >= 0 && order >= 0 && order <= 4, "mg_silu_order: order must be in 0..4 (got %d)", order);
    if (n == 0) return MG_OK;
    MG_REQUIRE(z && out && aligned16(z) && aligned16(out) && (mul == nullptr || aligned16(mul)),
               "mg_silu_order: null or unaligned pointer");
    long blocks = ceil_div(ceil_div(n, 4), 256);
    if (blocks > 256L * 16) blocks = 256L * 16;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(silu_order_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, z, mul, n, order, out);
    return check_launch("mg_silu_order");
}

}  // extern "C"
