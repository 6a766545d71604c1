// fp32-accurate GEMM on the bf16 matrix cores ("bf16x3" operand splitting).
//
// Each fp32 operand is split exactly into three bf16 pieces, x = hi + mid + lo
// (8 + 8 + 8 significand bits, each piece the RNE rounding of the remainder), and
// the product is assembled from the six piece products whose weight is >= 2^-24:
//     a*b ~= ah*bh + ah*bm + am*bh + ah*bl + al*bh + am*bm
// accumulated in fp32 inside v_mfma_f32_32x32x16_bf16.  The dropped terms
// (am*bl, al*bm, al*bl) are below 2^-24 |a||b|, i.e. at the level of fp32 rounding
// of the individual products, so the result is as accurate as an fp32 FMA chain.
// Six bf16 MFMAs cost 6/16 of one fp32 MFMA of the same shape: ~2.7x the fp32
// matrix rate.  Used for the wide per-edge MLP layers (T = 1, K % 32 == 0).
//
// Tile 128x128 per workgroup, 4 waves (2x2) of 64x64, K slab 32.  x and W tiles are
// read from HBM as fp32 (16-byte loads, one 128-byte line per row and slab), split
// in registers, and stored to LDS as three bf16 planes with 80-byte rows (5 quads,
// odd: 8 consecutive rows of a ds_read_b128 cover all banks).  A lane's MFMA
// operand is 8 consecutive k of one row: one ds_read_b128 per piece.
// v_mfma_f32_32x32x16_bf16 layout: A[m][k]: lane = m + 32*(k/8), 8 k per lane;
// B[k][n] likewise; D as for the fp32 32x32 shapes.
#include "common.hpp"
#include <type_traits>

namespace mg {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

constexpr int kBK = 32;
constexpr int kRowB = 80;                 // bytes per LDS row of one plane (32 bf16 + pad)
constexpr int kPlane = 128 * kRowB;       // bytes per plane

__device__ __forceinline__ float activate(float v, int act) {
    // SiLU with the hardware exp2 / reciprocal (about 1 ulp each): far inside the fp32 tolerance
    if (act == 1) return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    if (act == 2) return v > 0.f ? v : 0.1f * v;
    return v;
}

struct Split4 {
    bf16x4 hi, mid, lo;
};

__device__ __forceinline__ Split4 split(float4 v) {
    Split4 s;
    const float in[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const __bf16 h = (__bf16)in[k];
        const float r1 = in[k] - (float)h;
        const __bf16 m = (__bf16)r1;
        const float r2 = r1 - (float)m;
        s.hi[k] = h;
        s.mid[k] = m;
        s.lo[k] = (__bf16)r2;
    }
    return s;
}

// W -> three bf16 planes (dim_out rounded up to 128 rows, zero filled), each row-major (rows, dim_in)
__global__ void __launch_bounds__(256) pack_weight_kernel(const float* __restrict__ W, long so, long si, int I, int O,
                                                          int O_pad, __bf16* __restrict__ packed) {
    const long total = (long)O_pad * I;
    for (long t = (long)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (long)gridDim.x * blockDim.x) {
        const int o = (int)(t / I), i = (int)(t - (long)o * I);
        const float v = o < O ? W[(long)o * so + (long)i * si] : 0.f;
        const __bf16 h = (__bf16)v;
        const float r1 = v - (float)h;
        const __bf16 m = (__bf16)r1;
        packed[t] = h;
        packed[total + t] = m;
        packed[2 * total + t] = (__bf16)(r1 - (float)m);
    }
}

template <bool PACKED>
__global__ void __launch_bounds__(256)
linear_rows_bf16x3_kernel(const float* __restrict__ W, long so, const float* __restrict__ X, long R, int I, int O,
                          const float* __restrict__ bias, int act, int accumulate, float* __restrict__ Y, int tiles_n,
                          long tiles_total, int out_T) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[6 * kPlane];
    unsigned char* xs = lds;                  // planes 0..2: x hi, mid, lo
    unsigned char* ws = lds + 3 * kPlane;     // planes 3..5: W hi, mid, lo

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

    float4 xv[4], wv[PACKED ? 1 : 4];
    bf16x8 wp[PACKED ? 6 : 1];     // packed W: 2 rows x 3 planes of 8 bf16 per thread and slab
    Split4 sx[4];
    const int ld_r = tid >> 3, ld_c = (tid & 7) * 4;
    // packed W: 128 rows x 64 B per plane and slab = 512 16-byte pieces -> 2 per thread
    const int pw_r = tid >> 2, pw_c = (tid & 3) * 8;    // + 64 rows for the second piece
    const __bf16* Wp = reinterpret_cast<const __bf16*>(W);
    const long plane_elems = (long)((O + 127) / 128) * 128 * I;

    auto load_x = [&](int k0) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int r = ld_r + 32 * j;
            xv[j] = (r0 + r < R) ? *reinterpret_cast<const float4*>(X + (r0 + r) * I + k0 + ld_c)
                                 : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto load_w = [&](int k0) {
        if constexpr (!PACKED) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int n = n0 + ld_r + 32 * j;
                wv[j] = (n < O) ? *reinterpret_cast<const float4*>(W + (long)n * so + k0 + ld_c)
                                : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
        if constexpr (PACKED) {
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int p = 0; p < 3; p++)
                    wp[h * 3 + p] = *reinterpret_cast<const bf16x8*>(Wp + p * plane_elems +
                                                                     (long)(n0 + pw_r + 64 * h) * I + k0 + pw_c);
        }
    };
    auto split_tile = [&]() {
#pragma unroll
        for (int j = 0; j < 4; j++) sx[j] = split(xv[j]);
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int off = (ld_r + 32 * j) * kRowB + ld_c * 2;
            *reinterpret_cast<bf16x4*>(xs + off) = sx[j].hi;
            *reinterpret_cast<bf16x4*>(xs + kPlane + off) = sx[j].mid;
            *reinterpret_cast<bf16x4*>(xs + 2 * kPlane + off) = sx[j].lo;
            if constexpr (!PACKED) {
                const Split4 sw = split(wv[j]);
                *reinterpret_cast<bf16x4*>(ws + off) = sw.hi;
                *reinterpret_cast<bf16x4*>(ws + kPlane + off) = sw.mid;
                *reinterpret_cast<bf16x4*>(ws + 2 * kPlane + off) = sw.lo;
            }
        }
        if constexpr (PACKED) {
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int p = 0; p < 3; p++)
                    *reinterpret_cast<bf16x8*>(ws + p * kPlane + (pw_r + 64 * h) * kRowB + pw_c * 2) = wp[h * 3 + p];
        }
    };

    int a_off[2], b_off[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        a_off[i] = ((wave_m * 2 + i) * 32 + (lane & 31)) * kRowB + kgroup * 16;
        b_off[i] = ((wave_n * 2 + i) * 32 + (lane & 31)) * kRowB + kgroup * 16;
    }

    // Software pipeline.  W (L2 resident, short latency) is fetched one slab ahead at the top of
    // the MFMA phase.  x comes from HBM: its loads for slab k+2 are issued at the END of the MFMA
    // phase of slab k, right after slab k+1 has been split out of the same registers, which gives
    // them a whole slab (store + MFMA phase) to land.
    // The slab index of the prefetches is clamped to the last slab instead of being guarded:
    // the loop body is then branch free (the final trips re-load and re-split the last slab,
    // which nobody reads).
    const int k_last = I - kBK;
    load_x(0);
    load_w(0);
    split_tile();
    load_x(kBK < I ? kBK : k_last);
    for (int k0 = 0; k0 < I; k0 += kBK) {
        __syncthreads();
        store_tile();
        __syncthreads();
        load_w(k0 + kBK < I ? k0 + kBK : k_last);
#pragma unroll
        for (int s = 0; s < 2; s++) {
            bf16x8 a[2][3], b[2][3];
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int p = 0; p < 3; p++) {
                    a[i][p] = *reinterpret_cast<const bf16x8*>(xs + p * kPlane + a_off[i] + s * 32);
                    b[i][p] = *reinterpret_cast<const bf16x8*>(ws + p * kPlane + b_off[i] + s * 32);
                }
            // small terms first; the six products of one output tile are issued as three rounds over
            // the four independent accumulators so that no MFMA waits for the previous one
#pragma unroll
            for (int t = 0; t < 6; t++) {
                constexpr int pa[6] = {2, 0, 1, 1, 0, 0};   // lo*hi, hi*lo, mid*mid, mid*hi, hi*mid, hi*hi
                constexpr int pb[6] = {0, 2, 1, 0, 1, 0};
#pragma unroll
                for (int mi = 0; mi < 2; mi++)
#pragma unroll
                    for (int ni = 0; ni < 2; ni++)
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mi][pa[t]], b[ni][pb[t]], acc[mi][ni],
                                                                              0, 0, 0);
            }
        }
        split_tile();
        load_x(k0 + 2 * kBK < I ? k0 + 2 * kBK : k_last);
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
                        } else {   // rows are (row, comp) pairs, output stored (row, chan, comp)
                            const long row = r / out_T;
                            addr = (row * O + n) * out_T + (r - row * out_T);
                        }
                        float v = activate(acc[mi][ni][q] + bv, act);
                        if (accumulate) v += Y[addr];
                        Y[addr] = v;
                    }
                }
            }
        }
    };
    if (out_T == 1) epilogue(std::true_type{});
    else epilogue(std::false_type{});
}


// ---------------------------------------------------------------------------
// Pipelined variant for pre-split weights (the one the MLP layers use).
// K slab 16, LDS double buffered (2 x 36 KB -> two workgroups per CU), ONE barrier
// per slab.  In slab k a wave (a) reads its operands of slab k from buffer k&1 and
// runs the 24 MFMAs, (b) splits the x registers of slab k+1 and stores them, with
// the W pieces of slab k+1, into the other buffer, (c) issues the HBM loads of slab
// k+3.  Work (b) and (c) sits in the same instruction stream as the MFMAs, so the
// matrix pipe stays busy while one wave does its own data movement; two register
// sets alternate (the loop is unrolled by two) so a load has two slabs to land.
constexpr int kBKp = 16;
constexpr int kRowP = 48;                   // bytes per LDS row of one plane (16 bf16 + pad, 3 quads)
constexpr int kPlaneP = 128 * kRowP;
constexpr int kBufP = 6 * kPlaneP;          // x hi/mid/lo, W hi/mid/lo

struct StageRegs {
    float4 x[2];       // 2 rows x 4 consecutive k (fp32)
    bf16x8 w[3];       // one 16-byte piece of each W plane
};

__global__ void __launch_bounds__(256)
linear_rows_bf16x3_pipelined_kernel(const __bf16* __restrict__ Wp, const float* __restrict__ X, long R, int I, int O,
                                    const float* __restrict__ bias, int act, int accumulate, float* __restrict__ Y,
                                    int tiles_n, long tiles_total, int out_T) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kBufP];

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
    const long plane_elems = (long)((O + 127) / 128) * 128 * I;

    floatx16 acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; mi++)
#pragma unroll
        for (int ni = 0; ni < 2; ni++)
#pragma unroll
            for (int q = 0; q < 16; q++) acc[mi][ni][q] = 0.f;

    // x tile of a slab: 128 rows x 16 floats = 512 float4: thread -> rows (tid>>2) and (tid>>2)+64, k = (tid&3)*4
    const int xr = tid >> 2, xc = (tid & 3) * 4;
    // W tile: 3 planes x 128 rows x 32 B = 768 pieces of 16 B: thread -> plane p, row (tid>>1), half (tid&1)
    const int wr = tid >> 1, wc = (tid & 1) * 8;
    const int k_last = I - kBKp;

    auto load_stage = [&](StageRegs& g, int k0) {
        k0 = k0 < I ? k0 : k_last;                   // clamped: the surplus loads of the last trips are never used
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const long r = r0 + xr + 64 * h;
            g.x[h] = r < R ? *reinterpret_cast<const float4*>(X + r * I + k0 + xc) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int p = 0; p < 3; p++)
            g.w[p] = *reinterpret_cast<const bf16x8*>(Wp + p * plane_elems + (long)(n0 + wr) * I + k0 + wc);
    };
    auto store_stage = [&](const StageRegs& g, unsigned char* buf) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const Split4 sx = split(g.x[h]);
            const int off = (xr + 64 * h) * kRowP + xc * 2;
            *reinterpret_cast<bf16x4*>(buf + off) = sx.hi;
            *reinterpret_cast<bf16x4*>(buf + kPlaneP + off) = sx.mid;
            *reinterpret_cast<bf16x4*>(buf + 2 * kPlaneP + off) = sx.lo;
        }
#pragma unroll
        for (int p = 0; p < 3; p++)
            *reinterpret_cast<bf16x8*>(buf + (3 + p) * kPlaneP + wr * kRowP + wc * 2) = g.w[p];
    };

    int a_off[2], b_off[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        a_off[i] = ((wave_m * 2 + i) * 32 + (lane & 31)) * kRowP + kgroup * 16;
        b_off[i] = 3 * kPlaneP + ((wave_n * 2 + i) * 32 + (lane & 31)) * kRowP + kgroup * 16;
    }
    auto compute = [&](const unsigned char* buf) {
        bf16x8 a[2][3], b[2][3];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int p = 0; p < 3; p++) {
                a[i][p] = *reinterpret_cast<const bf16x8*>(buf + p * kPlaneP + a_off[i]);
                b[i][p] = *reinterpret_cast<const bf16x8*>(buf + p * kPlaneP + b_off[i]);
            }
#pragma unroll
        for (int t = 0; t < 6; t++) {
            constexpr int pa[6] = {2, 0, 1, 1, 0, 0};   // lo*hi, hi*lo, mid*mid, mid*hi, hi*mid, hi*hi
            constexpr int pb[6] = {0, 2, 1, 0, 1, 0};
#pragma unroll
            for (int mi = 0; mi < 2; mi++)
#pragma unroll
                for (int ni = 0; ni < 2; ni++)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mi][pa[t]], b[ni][pb[t]], acc[mi][ni], 0, 0, 0);
        }
    };

    unsigned char* buf0 = lds;
    unsigned char* buf1 = lds + kBufP;
    StageRegs ga, gb;
    // prologue: slab 0 -> buf0 (via ga), slab 1 in gb, slab 2 in ga
    load_stage(ga, 0);
    load_stage(gb, kBKp);
    store_stage(ga, buf0);
    load_stage(ga, 2 * kBKp);
    // I is a multiple of 32: the loop handles slabs in pairs (even slab in buf0, odd slab in buf1)
    for (int k0 = 0; k0 < I; k0 += 2 * kBKp) {
        __syncthreads();                  // buf0 complete; everyone is done reading buf1
        compute(buf0);                    // slab k
        store_stage(gb, buf1);            // slab k+1
        load_stage(gb, k0 + 3 * kBKp);
        __syncthreads();                  // buf1 complete; everyone is done reading buf0
        compute(buf1);                    // slab k+1
        store_stage(ga, buf0);            // slab k+2
        load_stage(ga, k0 + 4 * kBKp);
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
                        if (accumulate) v += Y[addr];
                        Y[addr] = v;
                    }
                }
            }
        }
    };
    if (out_T == 1) epilogue(std::true_type{});
    else epilogue(std::false_type{});
}


// ---------------------------------------------------------------------------
// Wide variant: 256x256 tile per workgroup, 8 waves (4x2) of 64x128, same K slab
// and double buffering.  Per MFMA it needs 3/4 of the LDS reads and half of the
// split/stage work and barriers of the 128x128 kernel; LDS 2 x 72 KB -> one
// workgroup (two waves per SIMD) per CU.  Requires dim_out % 256 == 0.
constexpr int kPlaneQ = 256 * kRowP;
constexpr int kBufQ = 6 * kPlaneQ;

__global__ void __launch_bounds__(512)
linear_rows_bf16x3_wide_kernel(const __bf16* __restrict__ Wp, const float* __restrict__ X, long R, int I, int O,
                               const float* __restrict__ bias, int act, int accumulate, float* __restrict__ Y,
                               int tiles_n, long tiles_total, int out_T) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kBufQ];

    const long bid = blockIdx.x;
    const long per_xcd = (tiles_total + 7) / 8;
    const long logical = (bid % 8) * per_xcd + bid / 8;
    if (logical >= tiles_total) return;
    const long tile_m = logical / tiles_n;
    const int tile_n = (int)(logical - tile_m * tiles_n);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave >> 1, wave_n = wave & 1;
    const long r0 = tile_m * 256;
    const int n0 = tile_n * 256;
    const int kgroup = lane >> 5;
    const long plane_elems = (long)O * I;      // O is a multiple of 256 here

    floatx16 acc[2][4];
#pragma unroll
    for (int mi = 0; mi < 2; mi++)
#pragma unroll
        for (int ni = 0; ni < 4; ni++)
#pragma unroll
            for (int q = 0; q < 16; q++) acc[mi][ni][q] = 0.f;

    // x tile of a slab: 256 rows x 16 floats = 1024 float4: thread -> rows (tid>>2) and (tid>>2)+128, k = (tid&3)*4
    const int xr = tid >> 2, xc = (tid & 3) * 4;
    // W tile: 3 planes x 256 rows x 32 B = 1536 pieces of 16 B: thread -> row (tid>>1), half (tid&1), every plane
    const int wr = tid >> 1, wc = (tid & 1) * 8;
    const int k_last = I - kBKp;

    auto load_stage = [&](StageRegs& g, int k0) {
        k0 = k0 < I ? k0 : k_last;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const long r = r0 + xr + 128 * h;
            g.x[h] = r < R ? *reinterpret_cast<const float4*>(X + r * I + k0 + xc) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int p = 0; p < 3; p++)
            g.w[p] = *reinterpret_cast<const bf16x8*>(Wp + p * plane_elems + (long)(n0 + wr) * I + k0 + wc);
    };
    auto store_stage = [&](const StageRegs& g, unsigned char* buf) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const Split4 sx = split(g.x[h]);
            const int off = (xr + 128 * h) * kRowP + xc * 2;
            *reinterpret_cast<bf16x4*>(buf + off) = sx.hi;
            *reinterpret_cast<bf16x4*>(buf + kPlaneQ + off) = sx.mid;
            *reinterpret_cast<bf16x4*>(buf + 2 * kPlaneQ + off) = sx.lo;
        }
#pragma unroll
        for (int p = 0; p < 3; p++)
            *reinterpret_cast<bf16x8*>(buf + (3 + p) * kPlaneQ + wr * kRowP + wc * 2) = g.w[p];
    };

    int a_off[2], b_off[4];
#pragma unroll
    for (int i = 0; i < 2; i++) a_off[i] = ((wave_m * 2 + i) * 32 + (lane & 31)) * kRowP + kgroup * 16;
#pragma unroll
    for (int i = 0; i < 4; i++) b_off[i] = 3 * kPlaneQ + ((wave_n * 4 + i) * 32 + (lane & 31)) * kRowP + kgroup * 16;

    auto compute = [&](const unsigned char* buf) {
        bf16x8 a[2][3];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int p = 0; p < 3; p++) a[i][p] = *reinterpret_cast<const bf16x8*>(buf + p * kPlaneQ + a_off[i]);
#pragma unroll
        for (int nh = 0; nh < 2; nh++) {
            bf16x8 b[2][3];
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int p = 0; p < 3; p++)
                    b[i][p] = *reinterpret_cast<const bf16x8*>(buf + p * kPlaneQ + b_off[nh * 2 + i]);
#pragma unroll
            for (int t = 0; t < 6; t++) {
                constexpr int pa[6] = {2, 0, 1, 1, 0, 0};   // lo*hi, hi*lo, mid*mid, mid*hi, hi*mid, hi*hi
                constexpr int pb[6] = {0, 2, 1, 0, 1, 0};
#pragma unroll
                for (int mi = 0; mi < 2; mi++)
#pragma unroll
                    for (int nj = 0; nj < 2; nj++)
                        acc[mi][nh * 2 + nj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mi][pa[t]], b[nj][pb[t]],
                                                                                       acc[mi][nh * 2 + nj], 0, 0, 0);
            }
        }
    };

    unsigned char* buf0 = lds;
    unsigned char* buf1 = lds + kBufQ;
    // Waves w and w+4 share a SIMD.  The upper four stage the next slab before their
    // MFMAs, the lower four after: while one wave of a SIMD splits and stores, the
    // other keeps the matrix pipe busy.
    const bool store_first = __builtin_amdgcn_readfirstlane(wave) >= 4;
    StageRegs ga, gb;
    load_stage(ga, 0);
    load_stage(gb, kBKp);
    store_stage(ga, buf0);
    load_stage(ga, 2 * kBKp);
    for (int k0 = 0; k0 < I; k0 += 2 * kBKp) {
        __syncthreads();
        if (store_first) {
            store_stage(gb, buf1);
            load_stage(gb, k0 + 3 * kBKp);
        }
        compute(buf0);
        if (!store_first) {
            store_stage(gb, buf1);
            load_stage(gb, k0 + 3 * kBKp);
        }
        __syncthreads();
        if (store_first) {
            store_stage(ga, buf0);
            load_stage(ga, k0 + 4 * kBKp);
        }
        compute(buf1);
        if (!store_first) {
            store_stage(ga, buf0);
            load_stage(ga, k0 + 4 * kBKp);
        }
    }

    auto epilogue = [&](auto plain) {
        constexpr bool kPlain = decltype(plain)::value;
#pragma unroll
        for (int ni = 0; ni < 4; ni++) {
            const int n = n0 + (wave_n * 4 + ni) * 32 + (lane & 31);
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
                        if (accumulate) v += Y[addr];
                        Y[addr] = v;
                    }
                }
            }
        }
    };
    if (out_T == 1) epilogue(std::true_type{});
    else epilogue(std::false_type{});
}

}  // namespace

// requires: dim_in % 32 == 0, x and W 16-byte aligned, W rows contiguous (stride_i == 1), so % 4 == 0
int launch_rows_bf16x3(const float* W, long so, const float* X, long R, int I, int O, const float* bias, int act,
                       int accumulate, float* Y, hipStream_t st, int out_T) {
    const long tiles_m = ceil_div(R, 128);
    const int tiles_n = (int)ceil_div(O, 128);
    const long total = tiles_m * tiles_n;
    const long grid = ceil_div(total, 8) * 8;
    MG_REQUIRE(grid <= 0x7fffffffL, "mg_tensor_linear: grid too large (rows=%ld dim_out=%d)", R, O);
    hipLaunchKernelGGL(linear_rows_bf16x3_kernel<false>, dim3((unsigned)grid), dim3(256), 0, st, W, so, X, R, I, O,
                       bias, act, accumulate, Y, tiles_n, total, out_T);
    return check_launch("mg_tensor_linear(bf16x3)");
}

size_t packed_weight_bytes(int dim_in, int dim_out) {
    return (size_t)3 * ((dim_out + 127) / 128) * 128 * (size_t)dim_in * sizeof(__bf16);
}

int pack_weight(const float* W, long so, long si, int I, int O, void* packed, hipStream_t st) {
    const int O_pad = (O + 127) / 128 * 128;
    const long total = (long)O_pad * I;
    long blocks = ceil_div(total, 256);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(pack_weight_kernel, dim3((unsigned)blocks), dim3(256), 0, st, W, so, si, I, O, O_pad,
                       static_cast<__bf16*>(packed));
    return check_launch("mg_linear_pack_weight");
}

int launch_rows_bf16x3_packed(const void* packed, const float* X, long R, int I, int O, const float* bias, int act,
                              int accumulate, float* Y, hipStream_t st, int out_T) {
    if (O % 256 == 0 && ceil_div(R, 256) * (O / 256) >= 1024) {
        const long tiles_m = ceil_div(R, 256);
        const int tiles_n = O / 256;
        const long total = tiles_m * tiles_n;
        const long grid = ceil_div(total, 8) * 8;
        MG_REQUIRE(grid <= 0x7fffffffL, "mg_tensor_linear_packed: grid too large (rows=%ld dim_out=%d)", R, O);
        hipLaunchKernelGGL(linear_rows_bf16x3_wide_kernel, dim3((unsigned)grid), dim3(512), 0, st,
                           static_cast<const __bf16*>(packed), X, R, I, O, bias, act, accumulate, Y, tiles_n, total,
                           out_T);
        return check_launch("mg_tensor_linear_packed");
    }
    const long tiles_m = ceil_div(R, 128);
    const int tiles_n = (int)ceil_div(O, 128);
    const long total = tiles_m * tiles_n;
    const long grid = ceil_div(total, 8) * 8;
    MG_REQUIRE(grid <= 0x7fffffffL, "mg_tensor_linear_packed: grid too large (rows=%ld dim_out=%d)", R, O);
    hipLaunchKernelGGL(linear_rows_bf16x3_pipelined_kernel, dim3((unsigned)grid), dim3(256), 0, st,
                       static_cast<const __bf16*>(packed), X, R, I, O, bias, act, accumulate, Y, tiles_n, total, out_T);
    return check_launch("mg_tensor_linear_packed");
}

}  // namespace mg

using namespace mg;

extern "C" {

int mg_linear_packed_weight_bytes(int dim_in, int dim_out, size_t* bytes) {
    MG_REQUIRE(bytes != nullptr && dim_in >= 0 && dim_out >= 0, "mg_linear_packed_weight_bytes: bad argument");
    *bytes = packed_weight_bytes(dim_in, dim_out);
    return MG_OK;
}

int mg_linear_pack_weight(const float* W, long w_stride_o, long w_stride_i, int dim_in, int dim_out, void* packed,
                          mg_stream_t stream) {
    MG_REQUIRE(dim_in >= 0 && dim_out >= 0, "mg_linear_pack_weight: negative size");
    if (dim_in == 0 || dim_out == 0) return MG_OK;
    MG_REQUIRE(W && packed && aligned16(packed), "mg_linear_pack_weight: null or unaligned pointer");
    return pack_weight(W, w_stride_o, w_stride_i, dim_in, dim_out, packed, (hipStream_t)stream);
}

int mg_tensor_linear_packed(const void* packed_W, const float* x, long rows, int dim_in, int dim_out,
                            const float* bias, int act, int accumulate, int out_comps, float* y,
                            mg_stream_t stream) {
    MG_REQUIRE(rows >= 0 && dim_in > 0 && dim_out >= 0, "mg_tensor_linear_packed: bad size");
    MG_REQUIRE(dim_in % 32 == 0, "mg_tensor_linear_packed: dim_in must be a multiple of 32");
    MG_REQUIRE(act >= 0 && act <= 2, "mg_tensor_linear_packed: unknown activation %d", act);
    MG_REQUIRE(out_comps == 1 || out_comps == 3 || out_comps == 9, "mg_tensor_linear_packed: out_comps must be 1, 3 or 9");
    if (rows == 0 || dim_out == 0) return MG_OK;
    MG_REQUIRE(packed_W && x && y && aligned16(x) && aligned16(packed_W), "mg_tensor_linear_packed: null or unaligned pointer");
    return launch_rows_bf16x3_packed(packed_W, x, rows, dim_in, dim_out, bias, act, accumulate, y, (hipStream_t)stream,
                                     out_comps);
}

}  // extern "C"
