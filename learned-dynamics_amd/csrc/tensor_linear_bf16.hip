// Linear layers for the bf16-storage configuration: activations live in HBM as bf16,
// products are accumulated in fp32 on the bf16 matrix cores.
//
//   y[r, o] = act(bias[o] + sum_i W[o, i] * x[r, i])       x bf16 (rows, dim_in), y bf16 or fp32
//
// The weight keeps 16 significand bits: it is given as the first two planes (hi, mid) of the
// pre-split format of mg_linear_pack_weight, and every x piece meets both (two MFMAs per k-step),
// so the only rounding beyond fp32 accumulation is the bf16 storage of the activations themselves.
// These layers are bound by HBM traffic (2 bytes per element in and out), not by the MFMAs.
//
// Tile 128x128 per workgroup, 4 waves (2x2) of 64x64, K slab 32, LDS double buffer
// (2 x 30 KB -> two workgroups per CU), one barrier per slab.  Tiles go HBM -> registers -> LDS
// as 16-byte pieces; LDS rows are 80 bytes (5 quads, odd: ds_read_b128 of 8 consecutive rows
// covers all banks).  v_mfma_f32_32x32x16_bf16: A[m][k] lane = m + 32*(k/8), 8 k per lane.
#include "common.hpp"
#include <type_traits>

namespace mg {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kBK = 32;
constexpr int kRowB = 80;
constexpr int kPlane = 128 * kRowB;
constexpr int kBuf = 3 * kPlane;            // x, W hi, W mid

__device__ __forceinline__ float activate(float v, int act) {
    if (act == 1) return v * __frcp_rn(1.0f + __expf(-v));
    if (act == 2) return v > 0.f ? v : 0.1f * v;
    return v;
}

struct Stage {
    bf16x8 x[2];
    bf16x8 w[2][2];
};

template <typename YT>
__global__ void __launch_bounds__(256)
linear_rows_bf16_kernel(const __bf16* __restrict__ Wp, long plane_elems, const __bf16* __restrict__ X, long R, int I,
                        int O, const float* __restrict__ bias, int act, int accumulate, YT* __restrict__ Y,
                        int tiles_n, long tiles_total, int out_T) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kBuf];

    const long bid = blockIdx.x;
    const long per_xcd = (tiles_total + 7) / 8;
    const long logical = (bid % 8) * per_xcd + bid / 8;
    if (logical >= tiles_total) return;
    const long tile_m = logical / tiles_n;
    const int tile_n = (int)(logical - tile_m * tiles_n);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave >> 1, wave_n = wave & 1;
    const long r0 = tile_m * 128;
    const int n0 = tile_n * 128;
    const int kgroup = lane >> 5;

    floatx16 acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; mi++)
#pragma unroll
        for (int ni = 0; ni < 2; ni++)
#pragma unroll
            for (int q = 0; q < 16; q++) acc[mi][ni][q] = 0.f;

    // a 128 x 32 bf16 tile is 512 pieces of 16 bytes: thread -> rows (tid>>2) and (tid>>2)+64, piece tid&3
    const int sr = tid >> 2, sc = (tid & 3) * 8;
    const int k_last = I - kBK;
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

    auto load_stage = [&](Stage& g, int k0) {
        k0 = k0 < I ? k0 : k_last;                     // surplus loads of the last trips are never used
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const long r = r0 + sr + 64 * h;
            g.x[h] = r < R ? *reinterpret_cast<const bf16x8*>(X + r * I + k0 + sc) : zero;
#pragma unroll
            for (int p = 0; p < 2; p++)
                g.w[p][h] = *reinterpret_cast<const bf16x8*>(Wp + p * plane_elems + (long)(n0 + sr + 64 * h) * I + k0 + sc);
        }
    };
    auto store_stage = [&](const Stage& g, unsigned char* buf) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int off = (sr + 64 * h) * kRowB + sc * 2;
            *reinterpret_cast<bf16x8*>(buf + off) = g.x[h];
            *reinterpret_cast<bf16x8*>(buf + kPlane + off) = g.w[0][h];
            *reinterpret_cast<bf16x8*>(buf + 2 * kPlane + off) = g.w[1][h];
        }
    };

    int a_off[2], b_off[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        a_off[i] = ((wave_m * 2 + i) * 32 + (lane & 31)) * kRowB + kgroup * 16;
        b_off[i] = kPlane + ((wave_n * 2 + i) * 32 + (lane & 31)) * kRowB + kgroup * 16;
    }
    auto compute = [&](const unsigned char* buf) {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            bf16x8 a[2], b[2][2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                a[i] = *reinterpret_cast<const bf16x8*>(buf + a_off[i] + s * 32);
#pragma unroll
                for (int p = 0; p < 2; p++) b[i][p] = *reinterpret_cast<const bf16x8*>(buf + p * kPlane + b_off[i] + s * 32);
            }
#pragma unroll
            for (int p = 1; p >= 0; p--)     // small terms first
#pragma unroll
                for (int mi = 0; mi < 2; mi++)
#pragma unroll
                    for (int ni = 0; ni < 2; ni++)
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mi], b[ni][p], acc[mi][ni], 0, 0, 0);
        }
    };

    unsigned char* buf0 = lds;
    unsigned char* buf1 = lds + kBuf;
    Stage ga, gb;
    load_stage(ga, 0);
    load_stage(gb, kBK);
    store_stage(ga, buf0);
    load_stage(ga, 2 * kBK);
    // slabs in pairs (even slab in buf0, odd slab in buf1); an odd slab count runs one surplus slab
    // on clamped (valid) addresses whose products are discarded by the k0 < I test
    for (int k0 = 0; k0 < I; k0 += 2 * kBK) {
        __syncthreads();
        compute(buf0);
        store_stage(gb, buf1);
        load_stage(gb, k0 + 3 * kBK);
        __syncthreads();
        if (k0 + kBK < I) compute(buf1);
        store_stage(ga, buf0);
        load_stage(ga, k0 + 4 * kBK);
    }

    auto epilogue = [&](auto plain) {
        constexpr bool kPlain = decltype(plain)::value;
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            const int n = n0 + (wave_n * 2 + ni) * 32 + (lane & 31);
            if (n >= O) continue;
            const float bv = bias ? bias[n] : 0.f;
#pragma unroll
            for (int mi = 0; mi < 2; mi++) {
#pragma unroll
                for (int q = 0; q < 16; q++) {
                    const long r = r0 + (wave_m * 2 + mi) * 32 + 8 * (q / 4) + 4 * kgroup + (q % 4);
                    if (r < R) {
                        long addr;
                        if constexpr (kPlain) {
                            addr = r * O + n;
                        } else {
                            const long row = r / out_T;
                            addr = (row * O + n) * out_T + (r - row * out_T);
                        }
                        float v = activate(acc[mi][ni][q] + bv, act);
                        if (accumulate) v += (float)Y[addr];
                        Y[addr] = (YT)v;
                    }
                }
            }
        }
    };
    if (out_T == 1) epilogue(std::true_type{});
    else epilogue(std::false_type{});
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_tensor_linear_bf16(const void* packed_W, const void* x, long rows, int dim_in, int dim_out, const float* bias,
                          int act, int accumulate, int out_comps, int y_is_bf16, void* y, mg_stream_t stream) {
    MG_REQUIRE(rows >= 0 && dim_in > 0 && dim_out >= 0, "mg_tensor_linear_bf16: bad size");
    MG_REQUIRE(dim_in % 32 == 0, "mg_tensor_linear_bf16: dim_in must be a multiple of 32 (got %d)", dim_in);
    MG_REQUIRE(act >= 0 && act <= 2, "mg_tensor_linear_bf16: unknown activation %d", act);
    MG_REQUIRE(out_comps == 1 || out_comps == 3 || out_comps == 9, "mg_tensor_linear_bf16: out_comps must be 1, 3 or 9");
    if (rows == 0 || dim_out == 0) return MG_OK;
    MG_REQUIRE(packed_W && x && y && aligned16(x) && aligned16(packed_W), "mg_tensor_linear_bf16: null or unaligned pointer");
    const long tiles_m = ceil_div(rows, 128);
    const int tiles_n = (int)ceil_div(dim_out, 128);
    const long total = tiles_m * tiles_n;
    const long grid = ceil_div(total, 8) * 8;
    MG_REQUIRE(grid <= 0x7fffffffL, "mg_tensor_linear_bf16: grid too large (rows=%ld dim_out=%d)", rows, dim_out);
    const long plane_elems = (long)tiles_n * 128 * dim_in;
    hipStream_t st = (hipStream_t)stream;
    if (y_is_bf16)
        hipLaunchKernelGGL(linear_rows_bf16_kernel<__bf16>, dim3((unsigned)grid), dim3(256), 0, st,
                           static_cast<const __bf16*>(packed_W), plane_elems, static_cast<const __bf16*>(x), rows, dim_in,
                           dim_out, bias, act, accumulate, static_cast<__bf16*>(y), tiles_n, total, out_comps);
    else
        hipLaunchKernelGGL(linear_rows_bf16_kernel<float>, dim3((unsigned)grid), dim3(256), 0, st,
                           static_cast<const __bf16*>(packed_W), plane_elems, static_cast<const __bf16*>(x), rows, dim_in,
                           dim_out, bias, act, accumulate, static_cast<float*>(y), tiles_n, total, out_comps);
    return check_launch("mg_tensor_linear_bf16");
}

}  // extern "C"
