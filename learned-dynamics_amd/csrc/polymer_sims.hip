// Langevin dynamics of bead chains with harmonic bonds and a soft r^-12-like repulsion: the data generator
// `repel5_sim` (extensions/polymer_sims_cuda/polymer_sims_kern.cu:72-164).
//
// One workgroup integrates one chain for all the steps of a call: every bead's position and velocity live in its
// thread's registers, the chain's positions are mirrored in two LDS buffers (structure of arrays) that alternate
// per step, so one barrier per step orders the position update against the n^2 force sweep.  The reference
// launches 256-thread blocks over the flattened (chain, bead) index and synchronises only inside a block, so a
// chain that straddles two blocks reads positions of either step; here every force is computed from the
// positions of one step.  The force on bead i is summed in the reference's order: bond to i - 1, bond to i + 1,
// then k = i + 2, ..., i + n - 2 (mod n).
//
// Noise: the reference draws from per-thread XORWOW states seeded from the wall clock.  Here the three normals
// of bead b at kick s are Box-Muller transforms of Philox4x32-10 with counter (b, s, 0, 0) and the 64-bit seed as
// key: a pure function of (seed, bead, kick), independent of the launch shape.
#include "common.hpp"

namespace mg {
namespace {

constexpr float kRepelScale = 20.0f, kBondK = 20.0f, kBondR0 = 0.8f, kLjEpsilon = 0.2f;
constexpr int kMaxBeads = 2048;      // two LDS buffers of 3 n floats within the 64 KB a launch gets by default

struct Philox {
    uint32_t c[4];
};

__device__ __forceinline__ Philox philox4x32_10(uint32_t c0, uint32_t c1, uint32_t k0, uint32_t k1) {
    uint32_t c[4] = {c0, c1, 0u, 0u};
#pragma unroll
    for (int round = 0; round < 10; round++) {
        const uint32_t hi0 = __umulhi(0xD2511F53u, c[0]), lo0 = 0xD2511F53u * c[0];
        const uint32_t hi1 = __umulhi(0xCD9E8D57u, c[2]), lo1 = 0xCD9E8D57u * c[2];
        const uint32_t n0 = hi1 ^ c[1] ^ k0, n1 = lo1, n2 = hi0 ^ c[3] ^ k1, n3 = lo0;
        c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return Philox{{c[0], c[1], c[2], c[3]}};
}

__device__ __forceinline__ float unit_open(uint32_t r) { return ((float)(r >> 8) + 0.5f) * 0x1p-24f; }   // (0, 1)

__device__ __forceinline__ float3 normal3(uint32_t bead, uint32_t kick, uint32_t k0, uint32_t k1) {
    const Philox p = philox4x32_10(bead, kick, k0, k1);
    const float r0 = sqrtf(-2.0f * logf(unit_open(p.c[0]))), a0 = 6.28318530717958647692f * unit_open(p.c[1]);
    const float r1 = sqrtf(-2.0f * logf(unit_open(p.c[2]))), a1 = 6.28318530717958647692f * unit_open(p.c[3]);
    return make_float3(r0 * cosf(a0), r0 * sinf(a0), r1 * cosf(a1));
}

__device__ __forceinline__ void add_bond(float3& f, float dx, float dy, float dz) {
    const float factor = 1.0f - kBondR0 / sqrtf(dx * dx + dy * dy + dz * dz);
    const float s = -kBondK * factor;
    f.x += s * dx; f.y += s * dy; f.z += s * dz;
}

__device__ __forceinline__ void add_repel(float3& f, float dx, float dy, float dz) {
    const float q = dx * dx + dy * dy + dz * dz + kLjEpsilon;
    const float q2 = q * q;
    const float s = kRepelScale * __builtin_amdgcn_rcpf(q2 * q2 * q2);   // 1 ulp; an IEEE division costs ten instructions
    f.x += s * dx; f.y += s * dy; f.z += s * dz;
}

// force on bead i of a chain of n beads whose positions are px, py, pz (LDS)
__device__ __forceinline__ float3 chain_force(int i, int n, const float* px, const float* py, const float* pz) {
    const float xi = px[i], yi = py[i], zi = pz[i];
    float3 f = make_float3(0.f, 0.f, 0.f);
    if (i > 0) add_bond(f, xi - px[i - 1], yi - py[i - 1], zi - pz[i - 1]);
    if (i < n - 1) add_bond(f, xi - px[i + 1], yi - py[i + 1], zi - pz[i + 1]);
    int k = i + 2;
    k = k >= n ? k - n : k;
#pragma unroll 4
    for (int j = 3; j < n; j++) {                            // every bead but i - 1, i, i + 1 (cyclically)
        add_repel(f, xi - px[k], yi - py[k], zi - pz[k]);
        k = k + 1 == n ? 0 : k + 1;
    }
    return f;
}

// BPT beads per thread: bead i = threadIdx.x + t * blockDim.x
template <int BPT>
__global__ void __launch_bounds__(1024) repel5_sim_kernel(float* __restrict__ x, float* __restrict__ v,
                                                          const float* __restrict__ drag, float T, float dt, int drifts,
                                                          int n, uint32_t key0, uint32_t key1, uint32_t kick0) {
    extern __shared__ float lds[];                            // 2 buffers x 3 coordinates x n
    const int chain = blockIdx.x;
    float* xg = x + (long)chain * n * 3;
    float* vg = v + (long)chain * n * 3;
    float3 xi[BPT], vi[BPT];
    float drag_i[BPT], noise_i[BPT];
    bool live[BPT];
#pragma unroll
    for (int t = 0; t < BPT; t++) {
        const int i = threadIdx.x + t * blockDim.x;
        live[t] = i < n;
        const int ii = live[t] ? i : n - 1;
        xi[t] = make_float3(xg[3 * ii], xg[3 * ii + 1], xg[3 * ii + 2]);
        vi[t] = make_float3(vg[3 * ii], vg[3 * ii + 1], vg[3 * ii + 2]);
        drag_i[t] = drag[ii];
        noise_i[t] = sqrtf(2.0f * drag_i[t] * T * dt);
    }
    auto publish = [&](int buf) {
        float* p = lds + buf * 3 * n;
#pragma unroll
        for (int t = 0; t < BPT; t++) {
            const int i = threadIdx.x + t * blockDim.x;
            if (live[t]) { p[i] = xi[t].x; p[n + i] = xi[t].y; p[2 * n + i] = xi[t].z; }
        }
        __syncthreads();
    };
    // velocity update from the positions in buffer `buf`: v += w (dt (a - drag v) + c noise xi)
    auto kick = [&](int buf, uint32_t kick_index, float w, float c) {
        const float* p = lds + buf * 3 * n;
#pragma unroll
        for (int t = 0; t < BPT; t++) {
            const int i = threadIdx.x + t * blockDim.x;
            if (!live[t]) continue;
            const float3 a = chain_force(i, n, p, p + n, p + 2 * n);
            const float3 g = normal3((uint32_t)(chain * n + i), kick_index, key0, key1);
            const float cn = c * noise_i[t];
            vi[t].x += w * (dt * (a.x - drag_i[t] * vi[t].x) + cn * g.x);
            vi[t].y += w * (dt * (a.y - drag_i[t] * vi[t].y) + cn * g.y);
            vi[t].z += w * (dt * (a.z - drag_i[t] * vi[t].z) + cn * g.z);
        }
    };
    auto drift = [&]() {
#pragma unroll
        for (int t = 0; t < BPT; t++) { xi[t].x += dt * vi[t].x; xi[t].y += dt * vi[t].y; xi[t].z += dt * vi[t].z; }
    };

    const float half_noise = 0.70710678118654752440f;         // sqrt(0.5): the half kicks' share of the noise
    publish(0);
    kick(0, kick0, 0.5f, half_noise);
    for (int s = 1; s < drifts; s++) {
        drift();
        publish(s & 1);
        kick(s & 1, kick0 + (uint32_t)s, 1.0f, 1.0f);
    }
    drift();
    publish(drifts & 1);
    kick(drifts & 1, kick0 + (uint32_t)drifts, 0.5f, half_noise);

#pragma unroll
    for (int t = 0; t < BPT; t++) {
        const int i = threadIdx.x + t * blockDim.x;
        if (!live[t]) continue;
        xg[3 * i] = xi[t].x; xg[3 * i + 1] = xi[t].y; xg[3 * i + 2] = xi[t].z;
        vg[3 * i] = vi[t].x; vg[3 * i + 1] = vi[t].y; vg[3 * i + 2] = vi[t].z;
    }
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" int mg_repel5_sim(float* x, float* v, const float* drag, float T, float dt, int nsteps, int batch_size,
                             int n, unsigned long long seed, unsigned int first_kick, mg_stream_t stream) {
    MG_REQUIRE(batch_size >= 0 && n >= 0, "mg_repel5_sim: negative size");
    if (batch_size == 0 || n == 0) return MG_OK;
    MG_REQUIRE(x && v && drag, "mg_repel5_sim: null operand");
    MG_REQUIRE(n <= kMaxBeads, "mg_repel5_sim: at most %d beads per chain (got %d)", kMaxBeads, n);
    MG_REQUIRE((long)batch_size * n < (1L << 32), "mg_repel5_sim: more than 2^32 beads");
    MG_REQUIRE(T >= 0.f, "mg_repel5_sim: negative temperature");
    const int drifts = nsteps > 1 ? nsteps : 1;               // the reference moves positions max(nsteps, 1) times
    MG_REQUIRE((unsigned long long)first_kick + (unsigned long long)drifts < (1ull << 32),
               "mg_repel5_sim: kick index would wrap");
    const int bpt = n <= 1024 ? 1 : 2;
    const int threads = (int)ceil_div(ceil_div(n, bpt), kWave) * kWave;
    const size_t lds_bytes = (size_t)2 * 3 * n * sizeof(float);
    const uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
    hipStream_t st = (hipStream_t)stream;
    if (bpt == 1)
        repel5_sim_kernel<1><<<dim3(batch_size), dim3(threads), lds_bytes, st>>>(x, v, drag, T, dt, drifts, n, k0, k1, first_kick);
    else
        repel5_sim_kernel<2><<<dim3(batch_size), dim3(threads), lds_bytes, st>>>(x, v, drag, T, dt, drifts, n, k0, k1, first_kick);
    return check_launch("repel5_sim_kernel");
}
