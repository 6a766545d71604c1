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
                                                                int n, float* __restrict__ m, float* __restrict__ a) {
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
    Vec3x4 out;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const Vec3 x = vv.get(j), xd = cross(x, d);
        const float s0 = at(p0, j), s1 = at(p1, j), s2 = at(p2, j);
        out.set(j, {x.x * s0 + xd.x * s1 + d.x * s2, x.y * s0 + xd.y * s1 + d.y * s2, x.z * s0 + xd.z * s1 + d.z * s2});
    }
    st12(m + (e * n + c) * 3, out);
    st4(a + e * n + c, p3);
}

// Adjoint: with p = dist actv and dp its gradient,
//   dp[c] = dm[c] . v[c],  dp[n + c] = dm[c] . (v[c] x d),  dp[2n + c] = dm[c] . d,  dp[3n + c] = da[c]
//   d_dist = dp actv,  d_actv = dp dist,  dv[c] = dm[c] p[c] + (d x dm[c]) p[n + c]
//   d_dir = sum_c (dm[c] x v[c]) p[n + c] + dm[c] p[2n + c]
__global__ void __launch_bounds__(256) painn_combine_bwd_kernel(
    const float* __restrict__ dist, const float* __restrict__ actv, const float* __restrict__ v,
    const float* __restrict__ dir, const int* __restrict__ node, long n_rows, const float* __restrict__ dm,
    const float* __restrict__ da, long E, int n,
    float* __restrict__ d_dist, float* __restrict__ d_actv, float* __restrict__ dv, float* __restrict__ d_dir) {
    const int tpe = n >> 2;                                       // a power of two <= 64
    const long t = (long)blockIdx.x * 256 + threadIdx.x;
    const long e_raw = t / tpe;
    const bool live = e_raw < E;                                  // (dead threads still take part in the shuffles)
    const long e = live ? e_raw : E - 1;
    const int c = (int)(t - e_raw * tpe) * 4;
    // row of actv and v that this edge reads (an index outside the rows is clamped: never an access out of bounds)
    const long en = node ? min(max((long)node[e], 0L), n_rows - 1) : e;
    const float* de = dist + e * 4 * n + c;
    const float* ae = actv + en * 4 * n + c;
    float4 dk[4], ak[4];
#pragma unroll
    for (int k = 0; k < 4; k++) { dk[k] = ld4(de + k * n); ak[k] = ld4(ae + k * n); }
    const Vec3x4 vv = ld12(v + (en * n + c) * 3), g = ld12(dm + (e * n + c) * 3);
    const float4 ga = ld4(da + e * n + c);
    const Vec3 d = {dir[3 * e], dir[3 * e + 1], dir[3 * e + 2]};
    float dp[3][4];
    Vec3x4 gv;
    Vec3 gd = {0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const Vec3 x = vv.get(j), gm = g.get(j);
        const float p0 = at(dk[0], j) * at(ak[0], j), p1 = at(dk[1], j) * at(ak[1], j), p2 = at(dk[2], j) * at(ak[2], j);
        dp[0][j] = dot(gm, x);
        dp[1][j] = dot(gm, cross(x, d));
        dp[2][j] = dot(gm, d);
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
    float* dde = d_dist + e * 4 * n + c;
    float* dae = d_actv + e * 4 * n + c;
#pragma unroll
    for (int k = 0; k < 3; k++) {
        const float4 gp = make_float4(dp[k][0], dp[k][1], dp[k][2], dp[k][3]);
        st4(dde + k * n, mul4(gp, ak[k]));
        st4(dae + k * n, mul4(gp, dk[k]));
    }
    st4(dde + 3 * n, mul4(ga, ak[3]));
    st4(dae + 3 * n, mul4(ga, dk[3]));
    st12(dv + (e * n + c) * 3, gv);
    if (c == 0) { d_dir[3 * e] = gd.x; d_dir[3 * e + 1] = gd.y; d_dir[3 * e + 2] = gd.z; }
}

inline bool combine_shape_ok(int n) { return n >= 4 && n <= 256 && (n & (n - 1)) == 0; }

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_painn_combine_supported(int n) { return combine_shape_ok(n) ? 1 : 0; }

int mg_painn_combine_fwd(const float* dist, const float* actv, const float* v, const float* dir, const int* node,
                         long n_rows, long E, int n, float* m, float* a, mg_stream_t stream) {
    MG_REQUIRE(E >= 0 && combine_shape_ok(n), "mg_painn_combine_fwd: n must be a power of two in 4..256");
    if (E == 0) return MG_OK;
    MG_REQUIRE(dist && actv && v && dir && m && a, "mg_painn_combine_fwd: null pointer");
    MG_REQUIRE(node == nullptr || n_rows > 0, "mg_painn_combine_fwd: an index needs n_rows > 0");
    MG_REQUIRE(aligned16(dist) && aligned16(actv) && aligned16(v) && aligned16(m) && aligned16(a),
               "mg_painn_combine_fwd: arrays must be 16-byte aligned");
    const long threads = E * (n / 4);
    MG_REQUIRE(ceil_div(threads, 256) < (1L << 31), "mg_painn_combine_fwd: too many edges");
    hipLaunchKernelGGL(painn_combine_fwd_kernel, dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0,
                       (hipStream_t)stream, dist, actv, v, dir, node, n_rows, E, n, m, a);
    return check_launch("mg_painn_combine_fwd");
}

int mg_painn_combine_bwd(const float* dist, const float* actv, const float* v, const float* dir, const int* node,
                         long n_rows, const float* dm, const float* da, long E, int n, float* d_dist, float* d_actv,
                         float* dv, float* d_dir, mg_stream_t stream) {
    MG_REQUIRE(E >= 0 && combine_shape_ok(n), "mg_painn_combine_bwd: n must be a power of two in 4..256");
    if (E == 0) return MG_OK;
    MG_REQUIRE(dist && actv && v && dir && dm && da && d_dist && d_actv && dv && d_dir,
               "mg_painn_combine_bwd: null pointer");
    MG_REQUIRE(node == nullptr || n_rows > 0, "mg_painn_combine_bwd: an index needs n_rows > 0");
    MG_REQUIRE(aligned16(dist) && aligned16(actv) && aligned16(v) && aligned16(dm) && aligned16(da) &&
                   aligned16(d_dist) && aligned16(d_actv) && aligned16(dv),
               "mg_painn_combine_bwd: arrays must be 16-byte aligned");
    const long threads = E * (n / 4);
    MG_REQUIRE(ceil_div(threads, 256) < (1L << 31), "mg_painn_combine_bwd: too many edges");
    hipLaunchKernelGGL(painn_combine_bwd_kernel, dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0,
                       (hipStream_t)stream, dist, actv, v, dir, node, n_rows, dm, da, E, n, d_dist, d_actv, dv, d_dir);
    return check_launch("mg_painn_combine_bwd");
}

}  // extern "C"
