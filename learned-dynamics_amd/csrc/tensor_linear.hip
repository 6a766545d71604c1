// Per-irrep channel-mixing linear on the matrix cores (fp32 MFMA, gfx950).
//
//   y[r, o, t] = act( sum_i W[o, i] x[r, i, t] + bias[o] ),   t < T = 3^inds
//
// GEMM view: M = the flattened (r, t) index, N = o, K = i.  x keeps its HBM
// layout (r, i, t) all the way into LDS: for a k-slab [k0, k0+BK) the data of
// one row r is one contiguous run of BK*T floats, so HBM is read with
// unit-stride 16-byte accesses; the (r,t) <-> MFMA-row mapping is pure LDS
// address arithmetic.  The LDS row stride RS is chosen with RS = T (mod 32), so
// the 32 consecutive flattened rows a half-wave reads for one k land in 32
// different banks.
//
// v_mfma_f32_32x32x2_f32 operand layout (wave64):
//   A[m][k]: lane = m + 32k  (m < 32, k < 2)      B[k][n]: lane = n + 32k
//   D[m][n]: n = lane % 32,  m = 8*(reg/4) + 4*(lane/32) + reg%4,  reg < 16
#include "common.hpp"
#include <atomic>

namespace mg {
// defined in tensor_linear_bf16x3.hip
int launch_rows_bf16x3(const float* W, long so, const float* X, long R, int I, int O, const float* bias, int act,
                       int accumulate, float* Y, hipStream_t st, int out_T);

namespace {

std::atomic<int> g_linear_mode{2};   // 0: fp32 MFMA everywhere; 1: bf16x3 split for the wide T=1 GEMMs; 2 (default): host side uses the f16x2 entry point where it can, bf16x3 here

typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kBK = 16;

constexpr int lds_row_stride(int T) {
    // smallest stride >= BK*T with stride % 32 == T % 32; for T == 1 any odd stride does
    if (T == 1) return kBK + 1;
    int s = kBK * T;
    while (s % 32 != T % 32) s++;
    return s;
}

__device__ __forceinline__ float activate(float v, int act) {
    // SiLU with the hardware exp2 / reciprocal (about 1 ulp each): far inside the fp32 tolerance
    if (act == 1) return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    if (act == 2) return v > 0.f ? v : 0.1f * v;      // LeakyReLU(0.1)
    return v;
}

template <int T, int WAVES_M, int WAVES_N, int WM, int WN>
struct Cfg {
    static constexpr int NT = 64 * WAVES_M * WAVES_N;
    static constexpr int BM = 32 * WAVES_M * WM;   // flattened (r,t) rows per workgroup
    static constexpr int BN = 32 * WAVES_N * WN;
    static constexpr int RB = BM / T;              // x rows per workgroup
    static_assert(BM % T == 0, "tile must hold whole rows");
    static constexpr int RS = lds_row_stride(T);
    static constexpr int RSW = kBK + 1;
    static constexpr int XV4 = RB * (kBK * T / 4);              // float4 loads per x tile
    static constexpr int XV4_PER = (XV4 + NT - 1) / NT;
    static constexpr int XS = RB * kBK * T;                     // scalar loads per x tile
    static constexpr int XS_PER = (XS + NT - 1) / NT;
    static constexpr int WS = BN * kBK;
    static constexpr int WS_PER = (WS + NT - 1) / NT;
};

template <int T, int WAVES_M, int WAVES_N, int WM, int WN, bool XVEC, bool SOA_OUT>
__global__ void __launch_bounds__(64 * WAVES_M * WAVES_N)
linear_kernel(const float* __restrict__ W, long so, long si, const float* __restrict__ X, long R, int I, int O,
              const float* __restrict__ bias, int act, int accumulate, float* __restrict__ Y, int out_T) {
    using C = Cfg<T, WAVES_M, WAVES_N, WM, WN>;
    __shared__ float xs[C::RB * C::RS];
    __shared__ float ws[C::BN * C::RSW];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const long r0 = (long)blockIdx.x * C::RB;
    const int n0 = blockIdx.y * C::BN;
    const long row_floats = (long)I * T;

    float16v acc[WM][WN];
#pragma unroll
    for (int mi = 0; mi < WM; mi++)
#pragma unroll
        for (int ni = 0; ni < WN; ni++)
#pragma unroll
            for (int q = 0; q < 16; q++) acc[mi][ni][q] = 0.f;

    // LDS read bases (without the k term)
    int a_base[WM];
#pragma unroll
    for (int mi = 0; mi < WM; mi++) {
        const int m = (wave_m * WM + mi) * 32 + (lane & 31);
        a_base[mi] = (m / T) * C::RS + (m % T);
    }
    int b_base[WN];
#pragma unroll
    for (int ni = 0; ni < WN; ni++) b_base[ni] = ((wave_n * WN + ni) * 32 + (lane & 31)) * C::RSW;
    const int khalf = lane >> 5;

    // register staging of the next k-slab
    // (the scalar x path is the fallback for odd sizes: it goes HBM -> LDS without staging)
    float4 xv[XVEC ? C::XV4_PER : 1];
    float wsc[C::WS_PER];

    auto load_tile = [&](int k0) {
        if constexpr (XVEC) {
#pragma unroll
            for (int j = 0; j < C::XV4_PER; j++) {
                const int idx = tid + j * C::NT;
                const int r = idx / (kBK * T / 4), c4 = idx % (kBK * T / 4);
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (idx < C::XV4 && r0 + r < R)
                    v = *reinterpret_cast<const float4*>(X + (r0 + r) * row_floats + (long)k0 * T + c4 * 4);
                xv[j] = v;
            }
        }
#pragma unroll
        for (int j = 0; j < C::WS_PER; j++) {
            const int idx = tid + j * C::NT;
            const int n = idx / kBK, k = idx % kBK;
            float v = 0.f;
            if (idx < C::WS && n0 + n < O && k0 + k < I) v = W[(long)(n0 + n) * so + (long)(k0 + k) * si];
            wsc[j] = v;
        }
    };
    auto store_tile = [&](int k0) {
        if constexpr (XVEC) {
#pragma unroll
            for (int j = 0; j < C::XV4_PER; j++) {
                const int idx = tid + j * C::NT;
                if (idx < C::XV4) {
                    const int r = idx / (kBK * T / 4), c4 = idx % (kBK * T / 4);
                    float* p = xs + r * C::RS + c4 * 4;
                    p[0] = xv[j].x; p[1] = xv[j].y; p[2] = xv[j].z; p[3] = xv[j].w;
                }
            }
        } else {
            const int valid = (I - k0 < kBK ? I - k0 : kBK) * T;
            for (int idx = tid; idx < C::XS; idx += C::NT) {
                const int r = idx / (kBK * T), c = idx % (kBK * T);
                float v = 0.f;
                if (r0 + r < R && c < valid) v = X[(r0 + r) * row_floats + (long)k0 * T + c];
                xs[r * C::RS + c] = v;
            }
        }
#pragma unroll
        for (int j = 0; j < C::WS_PER; j++) {
            const int idx = tid + j * C::NT;
            if (idx < C::WS) ws[(idx / kBK) * C::RSW + idx % kBK] = wsc[j];
        }
    };

    load_tile(0);
    for (int k0 = 0; k0 < I; k0 += kBK) {
        __syncthreads();          // everyone finished reading the previous slab
        store_tile(k0);
        __syncthreads();
        if (k0 + kBK < I) load_tile(k0 + kBK);   // in flight during the MFMA loop
#pragma unroll
        for (int kk = 0; kk < kBK / 2; kk++) {
            const int k = 2 * kk + khalf;
            float a[WM], b[WN];
#pragma unroll
            for (int mi = 0; mi < WM; mi++) a[mi] = xs[a_base[mi] + k * T];
#pragma unroll
            for (int ni = 0; ni < WN; ni++) b[ni] = ws[b_base[ni] + k];
#pragma unroll
            for (int mi = 0; mi < WM; mi++)
#pragma unroll
                for (int ni = 0; ni < WN; ni++)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[mi], b[ni], acc[mi][ni], 0, 0, 0);
        }
    }

    // epilogue
#pragma unroll
    for (int ni = 0; ni < WN; ni++) {
        const int n = n0 + (wave_n * WN + ni) * 32 + (lane & 31);
        if (n >= O) continue;
        const float bv = bias ? bias[n] : 0.f;
#pragma unroll
        for (int mi = 0; mi < WM; mi++) {
#pragma unroll
            for (int q = 0; q < 16; q++) {
                const int m = (wave_m * WM + mi) * 32 + 8 * (q / 4) + 4 * khalf + (q % 4);
                const long r = r0 + m / T;
                if (r < R) {
                    // SOA_OUT: component-major output (row, comp, chan) instead of (row, chan, comp)
                    // T == 1 with out_T > 1: rows are (row, comp) pairs, output stored (row, chan, comp)
                    long addr = SOA_OUT ? (r * T + (m % T)) * O + n : (r * O + n) * T + (m % T);
                    if (T == 1 && out_T > 1) addr = ((r / out_T) * O + n) * out_T + r % out_T;
                    float v = acc[mi][ni][q] + bv;
                    v = activate(v, act);
                    if (accumulate) v += Y[addr];
                    Y[addr] = v;
                }
            }
        }
    }
}

template <int T, int WAVES_M, int WAVES_N, int WM, int WN>
int launch_cfg(const float* W, long so, long si, const float* X, long R, int I, int O, const float* bias, int act,
               int accumulate, float* Y, hipStream_t st, bool soa_out = false, int out_T = 1) {
    using C = Cfg<T, WAVES_M, WAVES_N, WM, WN>;
    const long gx = ceil_div(R, C::RB);
    const long gy = ceil_div(O, C::BN);
    MG_REQUIRE(gx <= 0x7fffffffL && gy <= 65535, "mg_tensor_linear: grid too large (rows=%ld dim_out=%d)", R, O);
    const bool xvec = I > 0 && aligned16(X) && (I % kBK == 0) && (((long)I * T) % 4 == 0);
    dim3 grid((unsigned)gx, (unsigned)gy), block(C::NT);
    if (xvec && soa_out)
        hipLaunchKernelGGL((linear_kernel<T, WAVES_M, WAVES_N, WM, WN, true, true>), grid, block, 0, st, W, so, si, X,
                           R, I, O, bias, act, accumulate, Y, out_T);
    else if (xvec)
        hipLaunchKernelGGL((linear_kernel<T, WAVES_M, WAVES_N, WM, WN, true, false>), grid, block, 0, st, W, so, si, X,
                           R, I, O, bias, act, accumulate, Y, out_T);
    else if (soa_out)
        hipLaunchKernelGGL((linear_kernel<T, WAVES_M, WAVES_N, WM, WN, false, true>), grid, block, 0, st, W, so, si, X,
                           R, I, O, bias, act, accumulate, Y, out_T);
    else
        hipLaunchKernelGGL((linear_kernel<T, WAVES_M, WAVES_N, WM, WN, false, false>), grid, block, 0, st, W, so, si,
                           X, R, I, O, bias, act, accumulate, Y, out_T);
    return check_launch("mg_tensor_linear");
}


// ---------------------------------------------------------------------------
// T == 1 (plain rows x dim_in @ W^T): the MLP GEMMs that dominate a PaiNN layer.
// 128x128 output tile, 4 waves (2x2, 64x64 each), BK = 32.
//  * K order is permuted inside a slab: lanes 0-31 own k = 0..15 and lanes 32-63
//    own k = 16..31 of the slab for BOTH operands, so MFMA step s multiplies
//    A[m][16h+s] B[16h+s][n] (h = lane/32) and every lane fetches its 16 k values
//    with four ds_read_b128 instead of 16 ds_read_b32.  Any pairing of k values
//    into steps is a valid reordering of the K sum.
//  * LDS rows are padded to 36 floats (9 quads, odd) so that b128 reads of 8
//    consecutive rows and b128 writes of one row hit 32 distinct banks.
//  * HBM side: a row of a slab is 128 B = one cache line, read by 8 lanes.
//  * Workgroup ids are remapped so that the N-tiles of one M-tile run back to
//    back on the SAME XCD (ids are dealt round-robin to the 8 XCDs, each with its
//    own L2): x is then fetched from HBM once and re-read from that L2.
constexpr int kBK1 = 32;
constexpr int kRS1 = kBK1 + 4;

template <bool WVEC>
__global__ void __launch_bounds__(256)
linear_rows_kernel(const float* __restrict__ W, long so, long si, const float* __restrict__ X, long R, int I, int O,
                   const float* __restrict__ bias, int act, int accumulate, float* __restrict__ Y, int tiles_n,
                   long tiles_total, int out_T) {
    __shared__ __attribute__((aligned(16))) float xs[128 * kRS1];
    __shared__ __attribute__((aligned(16))) float ws[128 * kRS1];

    // XCD-aware tile order
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
    const int khalf = lane >> 5;

    float16v acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; mi++)
#pragma unroll
        for (int ni = 0; ni < 2; ni++)
#pragma unroll
            for (int q = 0; q < 16; q++) acc[mi][ni][q] = 0.f;

    float4 xv[4], wv[4];
    const int ld_r = tid >> 3, ld_c = (tid & 7) * 4;   // + 32 rows per j

    auto load_tile = [&](int k0) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int r = ld_r + 32 * j;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (r0 + r < R) v = *reinterpret_cast<const float4*>(X + (r0 + r) * I + k0 + ld_c);
            xv[j] = v;
            float4 w = make_float4(0.f, 0.f, 0.f, 0.f);
            const int n = n0 + r;
            if (n < O) {
                if constexpr (WVEC) {
                    w = *reinterpret_cast<const float4*>(W + (long)n * so + k0 + ld_c);
                } else {
                    const float* wp = W + (long)n * so + (long)(k0 + ld_c) * si;
                    w = make_float4(wp[0], wp[si], wp[2 * si], wp[3 * si]);
                }
            }
            wv[j] = w;
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int r = ld_r + 32 * j;
            *reinterpret_cast<float4*>(xs + r * kRS1 + ld_c) = xv[j];
            *reinterpret_cast<float4*>(ws + r * kRS1 + ld_c) = wv[j];
        }
    };

    const float* a_ptr[2];
    const float* b_ptr[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        a_ptr[i] = xs + ((wave_m * 2 + i) * 32 + (lane & 31)) * kRS1 + khalf * 16;
        b_ptr[i] = ws + ((wave_n * 2 + i) * 32 + (lane & 31)) * kRS1 + khalf * 16;
    }

    load_tile(0);
    for (int k0 = 0; k0 < I; k0 += kBK1) {
        __syncthreads();
        store_tile();
        __syncthreads();
        if (k0 + kBK1 < I) load_tile(k0 + kBK1);
#pragma unroll
        for (int half = 0; half < 2; half++) {
            float4 a[2][2], b[2][2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                a[i][0] = *reinterpret_cast<const float4*>(a_ptr[i] + half * 8);
                a[i][1] = *reinterpret_cast<const float4*>(a_ptr[i] + half * 8 + 4);
                b[i][0] = *reinterpret_cast<const float4*>(b_ptr[i] + half * 8);
                b[i][1] = *reinterpret_cast<const float4*>(b_ptr[i] + half * 8 + 4);
            }
#pragma unroll
            for (int s = 0; s < 8; s++) {
                float av[2], bv[2];
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    const float4 aa = a[i][s >> 2], bb = b[i][s >> 2];
                    av[i] = (s & 3) == 0 ? aa.x : (s & 3) == 1 ? aa.y : (s & 3) == 2 ? aa.z : aa.w;
                    bv[i] = (s & 3) == 0 ? bb.x : (s & 3) == 1 ? bb.y : (s & 3) == 2 ? bb.z : bb.w;
                }
#pragma unroll
                for (int mi = 0; mi < 2; mi++)
#pragma unroll
                    for (int ni = 0; ni < 2; ni++)
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[mi], bv[ni], acc[mi][ni], 0, 0, 0);
            }
        }
    }

#pragma unroll
    for (int ni = 0; ni < 2; ni++) {
        const int n = n0 + (wave_n * 2 + ni) * 32 + (lane & 31);
        if (n >= O) continue;
        const float bv = bias ? bias[n] : 0.f;
#pragma unroll
        for (int mi = 0; mi < 2; mi++) {
#pragma unroll
            for (int q = 0; q < 16; q++) {
                const long r = r0 + (wave_m * 2 + mi) * 32 + 8 * (q / 4) + 4 * khalf + (q % 4);
                if (r < R) {
                    // out_T > 1: the rows are (row, comp) pairs and the output is stored (row, chan, comp)
                    const long addr = out_T == 1 ? r * O + n : ((r / out_T) * O + n) * out_T + r % out_T;
                    float v = activate(acc[mi][ni][q] + bv, act);
                    if (accumulate) v += Y[addr];
                    Y[addr] = v;
                }
            }
        }
    }
}

int launch_rows(const float* W, long so, long si, const float* X, long R, int I, int O, const float* bias, int act,
                int accumulate, float* Y, hipStream_t st, int out_T = 1) {
    const long tiles_m = ceil_div(R, 128);
    const int tiles_n = (int)ceil_div(O, 128);
    const long total = tiles_m * tiles_n;
    const long grid = ceil_div(total, 8) * 8;
    MG_REQUIRE(grid <= 0x7fffffffL, "mg_tensor_linear: grid too large (rows=%ld dim_out=%d)", R, O);
    const bool wvec = si == 1 && so % 4 == 0 && aligned16(W);
    if (wvec)
        hipLaunchKernelGGL(linear_rows_kernel<true>, dim3((unsigned)grid), dim3(256), 0, st, W, so, si, X, R, I, O, bias,
                           act, accumulate, Y, tiles_n, total, out_T);
    else
        hipLaunchKernelGGL(linear_rows_kernel<false>, dim3((unsigned)grid), dim3(256), 0, st, W, so, si, X, R, I, O,
                           bias, act, accumulate, Y, tiles_n, total, out_T);
    return check_launch("mg_tensor_linear");
}


// A handful of output channels (readouts: n -> 1 vectors).  The matrix tiles above are 32 columns wide, so a one-column
// output uses 1/32 of them, and the launch is bound by the latency of its few workgroups' loop over dim_in.  Here a
// group of lanes takes one row of x, (dim_in, T) with T = 1, 3 or 9 components per channel: a lane reads 4 channels
// = T 16-byte pieces at a time, so which component and channel an element belongs to is fixed at compile time, forms
// OC x T partial sums and the group adds them up with lane shuffles.  y_comp_major: y (row, comp, chan) instead of
// (row, chan, comp).
template <int T, int OC>
__global__ void __launch_bounds__(256) linear_few_outputs_kernel(const float* __restrict__ W, long so, long si,
                                                                 const float* __restrict__ X, long R, int I, int O,
                                                                 const float* __restrict__ bias, int act, int accumulate,
                                                                 int y_comp_major, int lanes_per_row,
                                                                 float* __restrict__ Y) {
    const int lane = threadIdx.x & 63;
    const long wave = ((long)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int rows_per_wave = 64 / lanes_per_row;
    const int sub = lane & (lanes_per_row - 1);
    const long row = wave * rows_per_wave + lane / lanes_per_row;
    const long ld_row = row < R ? row : R - 1;                  // (surplus groups repeat the last row and store nothing)
    const float* xrow = X + ld_row * (long)I * T;
    float sum[OC][T];
#pragma unroll
    for (int o = 0; o < OC; o++)
#pragma unroll
        for (int t = 0; t < T; t++) sum[o][t] = 0.f;
    for (int p = sub; p < I / 4; p += lanes_per_row) {
        float4 v[T];
#pragma unroll
        for (int k = 0; k < T; k++) v[k] = *reinterpret_cast<const float4*>(xrow + 4L * T * p + 4 * k);
        float e[4 * T];
#pragma unroll
        for (int k = 0; k < T; k++) { e[4 * k] = v[k].x; e[4 * k + 1] = v[k].y; e[4 * k + 2] = v[k].z; e[4 * k + 3] = v[k].w; }
#pragma unroll
        for (int o = 0; o < OC; o++) {
            const float* wrow = W + (long)(o < O ? o : 0) * so + 4L * p * si;
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const float w = wrow[c * si];
#pragma unroll
                for (int t = 0; t < T; t++) sum[o][t] = fmaf(w, e[c * T + t], sum[o][t]);
            }
        }
    }
#pragma unroll
    for (int o = 0; o < OC; o++)
#pragma unroll
        for (int t = 0; t < T; t++)
            for (int d = 1; d < lanes_per_row; d <<= 1) sum[o][t] += __shfl_xor(sum[o][t], d);
    if (sub != 0 || row >= R) return;
#pragma unroll
    for (int o = 0; o < OC; o++) {
        if (o >= O) break;
        const float bv = bias ? bias[o] : 0.f;
#pragma unroll
        for (int t = 0; t < T; t++) {
            float* dst = Y + (y_comp_major ? (row * T + t) * O + o : (row * O + o) * T + t);
            float v = activate(sum[o][t] + bv, act);
            if (accumulate) v += *dst;
            *dst = v;
        }
    }
}

template <int T>
int launch_few_outputs(const float* W, long so, long si, const float* X, long R, int I, int O, const float* bias, int act,
                       int accumulate, int y_comp_major, float* Y, hipStream_t st) {
    int lanes = 1;
    while (lanes < 64 && lanes < I / 4) lanes <<= 1;
    const long waves = ceil_div(R, 64 / lanes);
    const long grid = ceil_div(waves, 4);
    MG_REQUIRE(grid <= 0x7fffffffL, "mg_tensor_linear: grid too large (rows=%ld)", R);
    if (O == 1)
        hipLaunchKernelGGL((linear_few_outputs_kernel<T, 1>), dim3((unsigned)grid), dim3(256), 0, st, W, so, si, X, R, I, O,
                           bias, act, accumulate, y_comp_major, lanes, Y);
    else
        hipLaunchKernelGGL((linear_few_outputs_kernel<T, 4>), dim3((unsigned)grid), dim3(256), 0, st, W, so, si, X, R, I, O,
                           bias, act, accumulate, y_comp_major, lanes, Y);
    return check_launch("mg_tensor_linear");
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_tensor_linear_layout(int inds, const float* W, long w_stride_o, long w_stride_i, const float* x, long rows,
                            int dim_in, int dim_out, const float* bias, int act, int accumulate, int x_layout,
                            int y_layout, float* y, mg_stream_t stream) {
    if (inds < 0 || inds > 2)
        return fail(MG_ERR_UNSUPPORTED,
                    "tensor_linear currently only supports a number of indices up to 2.");
    MG_REQUIRE(rows >= 0 && dim_in >= 0 && dim_out >= 0, "mg_tensor_linear: negative size");
    MG_REQUIRE(act >= 0 && act <= 2, "mg_tensor_linear: unknown activation %d", act);
    MG_REQUIRE((x_layout == 0 || x_layout == 1) && (y_layout == 0 || y_layout == 1),
               "mg_tensor_linear: layouts are 0 (row, chan, comp) or 1 (row, comp, chan)");
    if (rows == 0 || dim_out == 0) return MG_OK;
    MG_REQUIRE(y != nullptr && (dim_in == 0 || (W != nullptr && x != nullptr)), "mg_tensor_linear: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const float* b = bias;
    const long so = w_stride_o, si = w_stride_i;
    const int T = inds == 0 ? 1 : (inds == 1 ? 3 : 9);
    if (dim_out <= 4 && dim_in >= 16 && dim_in % 4 == 0 && aligned16(x) && (x_layout == 0 || inds == 0)) {
        // a readout: too few output channels for a 32-column matrix tile
        const int ycm = (inds > 0 && y_layout == 1) ? 1 : 0;
        if (inds == 0) return launch_few_outputs<1>(W, so, si, x, rows, dim_in, dim_out, b, act, accumulate, ycm, y, st);
        if (inds == 1) return launch_few_outputs<3>(W, so, si, x, rows, dim_in, dim_out, b, act, accumulate, ycm, y, st);
        return launch_few_outputs<9>(W, so, si, x, rows, dim_in, dim_out, b, act, accumulate, ycm, y, st);
    }
    if (inds == 0 || x_layout == 1) {
        // component-major input: every (row, comp) pair is an independent row of a plain GEMM
        const long R = rows * T;
        const int out_T = (y_layout == 1) ? 1 : T;
        if (dim_in % kBK1 == 0 && aligned16(x) && (dim_out > 64 || out_T > 1)) {
            if (g_linear_mode.load() >= 1 && si == 1 && so % 4 == 0 && aligned16(W) && dim_in >= 64 && R >= 1024)
                return launch_rows_bf16x3(W, so, x, R, dim_in, dim_out, b, act, accumulate, y, st, out_T);
            return launch_rows(W, so, si, x, R, dim_in, dim_out, b, act, accumulate, y, st, out_T);
        }
        if (dim_out <= 32) return launch_cfg<1, 4, 1, 2, 1>(W, so, si, x, R, dim_in, dim_out, b, act, accumulate, y, st, false, out_T);
        if (dim_out <= 64) return launch_cfg<1, 2, 2, 2, 1>(W, so, si, x, R, dim_in, dim_out, b, act, accumulate, y, st, false, out_T);
        return launch_cfg<1, 2, 2, 2, 2>(W, so, si, x, R, dim_in, dim_out, b, act, accumulate, y, st, false, out_T);
    }
    const bool soa = y_layout == 1;
    // column tile of 128, 64 or 32: the widest one that still gives the chip two workgroups per CU (a node-sized problem
    // on 128-column tiles runs on a quarter of the CUs and takes twice as long)
    auto tile_cols = [&](int rows_per_group) {
        const long row_groups = ceil_div(rows, rows_per_group);
        int cols = dim_out <= 32 ? 32 : (dim_out <= 64 ? 64 : 128);
        while (cols > 32 && row_groups * ceil_div(dim_out, cols) < 512) cols >>= 1;
        return cols;
    };
    if (inds == 1) {
        const int cols = tile_cols(64);
        if (cols == 32) return launch_cfg<3, 2, 1, 3, 1>(W, so, si, x, rows, dim_in, dim_out, b, act, accumulate, y, st, soa);
        if (cols == 64) return launch_cfg<3, 2, 2, 3, 1>(W, so, si, x, rows, dim_in, dim_out, b, act, accumulate, y, st, soa);
        return launch_cfg<3, 2, 2, 3, 2>(W, so, si, x, rows, dim_in, dim_out, b, act, accumulate, y, st, soa);
    }
    const int cols = tile_cols(32);
    if (cols == 32) return launch_cfg<9, 3, 1, 3, 1>(W, so, si, x, rows, dim_in, dim_out, b, act, accumulate, y, st, soa);
    if (cols == 64) return launch_cfg<9, 3, 1, 3, 2>(W, so, si, x, rows, dim_in, dim_out, b, act, accumulate, y, st, soa);
    return launch_cfg<9, 3, 2, 3, 2>(W, so, si, x, rows, dim_in, dim_out, b, act, accumulate, y, st, soa);
}

int mg_set_linear_mode(int mode) {
    MG_REQUIRE(mode >= 0 && mode <= 2, "mg_set_linear_mode: mode must be 0 (fp32 MFMA), 1 (bf16x3 split) or 2 (f16x2 split)");
    g_linear_mode.store(mode);
    return MG_OK;
}

int mg_get_linear_mode(void) { return g_linear_mode.load(); }

int mg_tensor_linear(int inds, const float* W, long w_stride_o, long w_stride_i, const float* x, long rows,
                     int dim_in, int dim_out, const float* bias, int act, int accumulate, float* y,
                     mg_stream_t stream) {
    return mg_tensor_linear_layout(inds, W, w_stride_o, w_stride_i, x, rows, dim_in, dim_out, bias, act, accumulate, 0,
                                   0, y, stream);
}

}  // extern "C"
