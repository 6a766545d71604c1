// Edge sums of DisplacementTensors.forward (archs/diffuser_atoms15.py:216-225): with phi (E, C) the radial MLP's
// output per edge and u = tens_sigmoid(1, r_ij * scale) = s r / sqrt(1 + |s r|^2),
//     A_a[i, c]       = sum over the edges e of node i of phi[e, c]
//     A_v[i, c, x]    = sum_e phi[e, c] u_x
//     A_d[i, c, x, y] = sum_e phi[e, c] u_x u_y
// The reference materialises phi (x) u and phi (x) u (x) u per edge (E x C x 13 floats) before its scatter sums;
// here one wave owns (node, 64 channels), a lane one channel: phi is streamed once with 256-byte wave accesses,
// the 13 sums live in registers (6 for the symmetric rank-2 part) and are written once per node.  Edges are
// summed in order: no atomics.
#include "common.hpp"

namespace mg {
namespace {

__global__ void __launch_bounds__(256) displacement_sums_kernel(const int* __restrict__ row_ptr, long n_nodes,
                                                                const float* __restrict__ r_ij,
                                                                const float* __restrict__ phi, int C, float scale,
                                                                float* __restrict__ out_a, float* __restrict__ out_v,
                                                                float* __restrict__ out_d) {
    const int lane = threadIdx.x & (kWave - 1);
    const long wave = ((long)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    const long waves = ((long)gridDim.x * blockDim.x) / kWave;
    const int chunks = (C + kWave - 1) / kWave;
    for (long item = wave; item < n_nodes * chunks; item += waves) {
        const long node = item / chunks;
        const int c = (int)(item - node * chunks) * kWave + lane;
        const bool live = c < C;
        const long lo = row_ptr[node], hi = row_ptr[node + 1];
        float a = 0.f, vx = 0.f, vy = 0.f, vz = 0.f, dxx = 0.f, dxy = 0.f, dxz = 0.f, dyy = 0.f, dyz = 0.f, dzz = 0.f;
        for (long e = lo; e < hi; e++) {
            const float rx = scale * r_ij[3 * e], ry = scale * r_ij[3 * e + 1], rz = scale * r_ij[3 * e + 2];
            const float inv = 1.0f / sqrtf(1.0f + (rx * rx + ry * ry + rz * rz));
            const float ux = rx * inv, uy = ry * inv, uz = rz * inv;
            const float p = live ? phi[e * C + c] : 0.f;
            const float px = p * ux, py = p * uy, pz = p * uz;
            a += p;
            vx += px; vy += py; vz += pz;
            dxx += px * ux; dxy += px * uy; dxz += px * uz;
            dyy += py * uy; dyz += py * uz; dzz += pz * uz;
        }
        if (!live) continue;
        const long o = node * C + c;
        out_a[o] = a;
        out_v[3 * o] = vx; out_v[3 * o + 1] = vy; out_v[3 * o + 2] = vz;
        float* d = out_d + 9 * o;
        d[0] = dxx; d[1] = dxy; d[2] = dxz;
        d[3] = dxy; d[4] = dyy; d[5] = dyz;
        d[6] = dxz; d[7] = dyz; d[8] = dzz;
    }
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" int mg_displacement_sums(const int* row_ptr, long n_nodes, long n_edges, const float* r_ij, const float* phi,
                                    int chan, float scale, float* out_a, float* out_v, float* out_d, mg_stream_t stream) {
    MG_REQUIRE(n_nodes >= 0 && n_edges >= 0 && chan >= 0, "mg_displacement_sums: negative size");
    if (n_nodes == 0 || chan == 0) return MG_OK;
    MG_REQUIRE(row_ptr && out_a && out_v && out_d, "mg_displacement_sums: null pointer");
    MG_REQUIRE(n_edges == 0 || (r_ij && phi), "mg_displacement_sums: null edge operand");
    long blocks = ceil_div(n_nodes * ceil_div(chan, kWave), 4);
    if (blocks > 256L * 32) blocks = 256L * 32;
    displacement_sums_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(row_ptr, n_nodes, r_ij, phi, chan,
                                                                                             scale, out_a, out_v, out_d);
    return check_launch("mg_displacement_sums");
}
