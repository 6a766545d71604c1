// SelfTensProds after its six input linears (archs/diffuser_atoms15.py:82-94): the Cartesian products of
// l_k = L_k x_k and r_k = R_k x_k and the output linears Y_lab, in one kernel per output rank:
//     y_o[node, :, comp] = sum over the product types `lab` of output rank o of  Y_lab p_lab[node, comp, :]
// The products are never stored.  The kernel is the split-fp16 row-streaming GEMM (rows = (node, comp),
// K = (product type, channel), three fp16 MFMAs per product, fp32 accumulate) whose A operand is built in
// registers: every product component is a short signed sum of elementwise products of one component row of
// l and one of r,
//     p_lab[node, comp, c] = sum_t (+/-) l[node, lb + t ls, c] r[node, rb + t rs, c]        (1, 2, 3 or 9 terms),
// so a lane that owns a GEMM row loads 16 consecutive channels of the rows it needs (64 contiguous bytes
// each, component-major operands, L2 resident: a node's 13 + 13 rows serve all its components and all
// product types) and multiplies them.  Row scales come from per-node bounds of |l| and |r|.
// The weight planes go through LDS exactly as in the plain kernel.
#include "common.hpp"
#include "f16x2.hpp"

namespace mg {
namespace {

// product types in the order 000 110 220 011 101 121 211 022 202 112 222 111 212
__constant__ const int kPRankL[13] = {0, 1, 2, 0, 1, 1, 2, 0, 2, 1, 2, 1, 2};
__constant__ const int kPRankR[13] = {0, 1, 2, 1, 0, 2, 1, 2, 0, 1, 2, 1, 1};

struct SignedDot {
    int lb, ls, rb, rs, nt;
    bool cross;          // two terms, the second one negative
};

// component c of the product of type `label` as a signed dot product over component rows of l and r
__device__ __forceinline__ SignedDot signed_dot(int label, int c) {
    const int i = c / 3, j = c - 3 * i;                  // rank-2 output component (i, j)
    const int j1 = (j + 1) % 3, j2 = (j + 2) % 3;
    const int c1 = (c + 1) % 3, c2 = (c + 2) % 3;        // rank-1 output component c
    switch (label) {
        case 0: return {0, 0, 0, 0, 1, false};                       // 000: l r
        case 1: return {0, 1, 0, 1, 3, false};                       // 110: sum_x l_x r_x
        case 2: return {0, 1, 0, 1, 9, false};                       // 220: sum_xy l_xy r_xy
        case 3: return {0, 0, c, 0, 1, false};                       // 011: l r_c
        case 4: return {c, 0, 0, 0, 1, false};                       // 101: l_c r
        case 5: return {0, 1, 3 * c, 1, 3, false};                   // 121: sum_x l_x r_cx
        case 6: return {3 * c, 1, 0, 1, 3, false};                   // 211: sum_y l_cy r_y
        case 7: return {0, 0, c, 0, 1, false};                       // 022: l r_c
        case 8: return {c, 0, 0, 0, 1, false};                       // 202: l_c r
        case 9: return {i, 0, j, 0, 1, false};                       // 112: l_i r_j
        case 10: return {3 * i, 1, 3 * j, 1, 3, false};              // 222: sum_y l_iy r_jy
        case 11: return {c1, c2 - c1, c2, c1 - c2, 2, true};         // 111: l_c1 r_c2 - l_c2 r_c1
        default: return {3 * i + j1, j2 - j1, j2, j1 - j2, 2, true}; // 212: l_ij1 r_j2 - l_ij2 r_j1
    }
}

struct Operands {
    const float* l[3];   // (nodes, 3^k, chan)
    const float* r[3];
    int labels[5];
    int n_labels;
};

template <int WAVES, int NI, int T>
__global__ void __launch_bounds__(64 * WAVES)
products_linear_kernel(const _Float16* __restrict__ Wp, const float* __restrict__ w_inv, Operands ops,
                       const float* __restrict__ node_bound, long n_nodes, int chan, int O, int O_pad,
                       float* __restrict__ Y, int tiles_n, long tiles_total) {
    constexpr int TM = 32 * WAVES, TN = 32 * NI, THREADS = 64 * WAVES;
    constexpr int kPlaneW = TN * kRowW, kBufW = 2 * kPlaneW;
    constexpr int kPieces = 8 * TN;
    constexpr int kPer = (kPieces + THREADS - 1) / THREADS;
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kBufW];
    __shared__ float inv_sx[TM];

    const long bid = blockIdx.x;
    const long per_xcd = (tiles_total + 7) / 8;
    const long logical = (bid % 8) * per_xcd + bid / 8;
    if (logical >= tiles_total) return;
    const long tile_m = logical / tiles_n;
    const int tile_n = (int)(logical - tile_m * tiles_n);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, g = lane >> 5;
    const long R = n_nodes * T;
    const int I = ops.n_labels * chan;
    const long r0 = tile_m * TM;
    const int n0 = tile_n * TN;
    const long plane_elems = (long)O_pad * I;

    floatx16 acc[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ni++)
#pragma unroll
        for (int q = 0; q < 16; q++) acc[ni][q] = 0.f;

    // this lane's GEMM row: (node, output component); rows past the end shadow the last one
    const long my_row = r0 + wave * 32 + m;
    const long ld_row = my_row < R ? my_row : R - 1;
    const long node = ld_row / T;
    const int co = (int)(ld_row - node * T);
    float sx;
    {
        float inv;
        sx = pow2_scale(node_bound[node], &inv);
        if (g == 0) inv_sx[wave * 32 + m] = inv;
    }
    const _Float16* wsrc[kPer];
    int wdst[kPer];
#pragma unroll
    for (int j = 0; j < kPer; j++) {
        int q = tid + THREADS * j;
        if (q >= kPieces) q = kPieces - 1;
        const int plane = q / (4 * TN), row = (q % (4 * TN)) >> 2, piece = q & 3;
        wsrc[j] = Wp + plane * plane_elems + (long)(n0 + row) * I + 8 * piece;
        wdst[j] = plane * kPlaneW + row * kRowW + piece * 16;
    }
    const int k_last = I - kCK;

    struct ARegs { float4 v[4]; };
    struct WRegs { halfx8 v[kPer]; };
    // the 16 values of this lane's row for chunk k0: product type k0 / chan, channels k0 % chan + 16 g ..
    auto build_a = [&](ARegs& a, int k0) {
        k0 = k0 < I ? k0 : k_last;
        const int li = k0 / chan;
        const int c0 = k0 - li * chan + 16 * g;
        const int label = ops.labels[li];
        const int rl = kPRankL[label], rr = kPRankR[label];
        const int CL = rl == 0 ? 1 : (rl == 1 ? 3 : 9), CR = rr == 0 ? 1 : (rr == 1 ? 3 : 9);
        const SignedDot d = signed_dot(label, co);
        const float* lp = (rl == 0 ? ops.l[0] : (rl == 1 ? ops.l[1] : ops.l[2])) + (node * CL + d.lb) * chan + c0;
        const float* rp = (rr == 0 ? ops.r[0] : (rr == 1 ? ops.r[1] : ops.r[2])) + (node * CR + d.rb) * chan + c0;
        const long lstep = (long)d.ls * chan, rstep = (long)d.rs * chan;
#pragma unroll
        for (int j = 0; j < 4; j++) a.v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        // one term at a time: the latency of these L1 / L2 reads is hidden by the other waves of the CU (the
        // kernel keeps few registers), which measured faster than requesting all terms of a component at once.
        // The trip count depends on the product type only, so it is the same for every lane.
        for (int t = 0; t < d.nt; t++) {
            const float sgn = (d.cross && t == 1) ? -1.f : 1.f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float4 x = *reinterpret_cast<const float4*>(lp + t * lstep + 4 * j);
                const float4 y = *reinterpret_cast<const float4*>(rp + t * rstep + 4 * j);
                a.v[j].x += sgn * x.x * y.x;
                a.v[j].y += sgn * x.y * y.y;
                a.v[j].z += sgn * x.z * y.z;
                a.v[j].w += sgn * x.w * y.w;
            }
        }
    };
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
            for (int ni = 0; ni < NI; ni++) {
                const halfx8 bh = *reinterpret_cast<const halfx8*>(buf + b_off + ni * 32 * kRowW + 16 * s);
                const halfx8 bl = *reinterpret_cast<const halfx8*>(buf + kPlaneW + b_off + ni * 32 * kRowW + 16 * s);
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[s], bh, acc[ni], 0, 0, 0);
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[s], bl, acc[ni], 0, 0, 0);
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[s], bh, acc[ni], 0, 0, 0);
            }
    };

    unsigned char* buf0 = lds;
    unsigned char* buf1 = lds + kBufW;
    ARegs a0, a1;
    WRegs w;
    load_w(w, 0);
    build_a(a0, 0);
    store_w(w, buf0);
    load_w(w, kCK);
    __syncthreads();
    // chan is a multiple of 32, so I / 32 chunks; they are taken in pairs and a surplus last chunk is scaled by zero
    for (int k0 = 0; k0 < I; k0 += 2 * kCK) {
        build_a(a1, k0 + kCK);                 // operands of the next chunk are requested before this chunk's MFMAs
        compute(a0, buf0, sx);
        store_w(w, buf1);
        load_w(w, k0 + 2 * kCK);
        __syncthreads();
        build_a(a0, k0 + 2 * kCK);
        compute(a1, buf1, k0 + kCK < I ? sx : 0.f);
        store_w(w, buf0);
        load_w(w, k0 + 3 * kCK);
        __syncthreads();
    }

    // y (node, O, T): the reference's layout; one row pointer, scale and bounds check per accumulator row
    float iw[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ni++) {
        const int n = n0 + ni * 32 + m;
        iw[ni] = n < O ? w_inv[n] : 0.f;
    }
#pragma unroll
    for (int q = 0; q < 16; q++) {
        const int rl = wave * 32 + 8 * (q / 4) + 4 * g + (q % 4);
        const long r = r0 + rl;
        if (r < R) {
            const long nd = r / T;
            float* yp = Y + (nd * O + n0 + m) * T + (r - nd * T);
            const float isx = inv_sx[rl];
#pragma unroll
            for (int ni = 0; ni < NI; ni++)
                if (n0 + ni * 32 + m < O) yp[ni * 32 * T] = acc[ni][q] * isx * iw[ni];
        }
    }
}

// Rank-2 output (nine GEMM rows per node): the 13 + 13 component rows of the tile's nodes are staged in LDS once
// per block of 32 channels and serve all five product types and all nine components from there; reading the
// operands through L1 instead costs one cache lookup per lane and 16 bytes, which bounded the kernel above.
// K is ordered (channel block of 32, product type, channel in block); the caller packs W with its columns in
// that order.
template <int NI>
__global__ void __launch_bounds__(256)
products_linear_staged_kernel(const _Float16* __restrict__ Wp, const float* __restrict__ w_inv, Operands ops,
                              const float* __restrict__ node_bound, long n_nodes, int chan, int O, int O_pad,
                              float* __restrict__ Y, int tiles_n, long tiles_total) {
    constexpr int T = 9, WAVES = 4, TM = 32 * WAVES, TN = 32 * NI, THREADS = 64 * WAVES;
    constexpr int NN = TM / T + 2;                           // nodes a tile of TM rows can touch
    constexpr int kRowF = 36;                                // floats per staged row: 32 channels + 4 (bank spread)
    constexpr int kPlaneW = TN * kRowW, kBufW = 2 * kPlaneW;
    constexpr int kPieces = 8 * TN;
    constexpr int kPer = (kPieces + THREADS - 1) / THREADS;
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kBufW];
    __shared__ __attribute__((aligned(16))) float stage[26 * NN * kRowF];
    __shared__ float inv_sx[TM];

    const long bid = blockIdx.x;
    const long per_xcd = (tiles_total + 7) / 8;
    const long logical = (bid % 8) * per_xcd + bid / 8;
    if (logical >= tiles_total) return;
    const long tile_m = logical / tiles_n;
    const int tile_n = (int)(logical - tile_m * tiles_n);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, g = lane >> 5;
    const long R = n_nodes * T;
    const int NL = ops.n_labels;
    const int I = NL * chan;
    const long r0 = tile_m * TM;
    const int n0 = tile_n * TN;
    const long plane_elems = (long)O_pad * I;
    const long node_lo = r0 / T;

    floatx16 acc[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ni++)
#pragma unroll
        for (int q = 0; q < 16; q++) acc[ni][q] = 0.f;

    const long my_row = r0 + wave * 32 + m;
    const long ld_row = my_row < R ? my_row : R - 1;
    const long node = ld_row / T;
    const int co = (int)(ld_row - node * T);
    const int nl = (int)(node - node_lo);                    // 0 .. NN-1
    float sx;
    {
        float inv;
        sx = pow2_scale(node_bound[node], &inv);
        if (g == 0) inv_sx[wave * 32 + m] = inv;
    }
    const _Float16* wsrc[kPer];
    int wdst[kPer];
#pragma unroll
    for (int j = 0; j < kPer; j++) {
        int q = tid + THREADS * j;
        if (q >= kPieces) q = kPieces - 1;
        const int plane = q / (4 * TN), row = (q % (4 * TN)) >> 2, piece = q & 3;
        wsrc[j] = Wp + plane * plane_elems + (long)(n0 + row) * I + 8 * piece;
        wdst[j] = plane * kPlaneW + row * kRowW + piece * 16;
    }
    const int k_last = I - kCK;
    struct ARegs { float4 v[4]; };
    struct WRegs { halfx8 v[kPer]; };

    // staged row index: 0 l_0, 1..3 l_1, 4..12 l_2, 13 r_0, 14..16 r_1, 17..25 r_2
    constexpr int kStagePieces = 26 * NN * 8, kStagePer = (kStagePieces + THREADS - 1) / THREADS;
    auto stage_block = [&](int cb) {
        // all loads of the block are requested before the first LDS store: one round trip, not kStagePer.
        // (Requesting the next block a whole block early, to hide that round trip too, measured slower: the
        // weight loads of every chunk then queue behind it.)
        float4 v[kStagePer];
        int dst[kStagePer];
#pragma unroll
        for (int u = 0; u < kStagePer; u++) {
            int idx = tid + THREADS * u;
            idx = idx < kStagePieces ? idx : kStagePieces - 1;       // surplus threads repeat the last piece
            const int rr = idx / (NN * 8), rem = idx - rr * (NN * 8);
            const int nd = rem >> 3, piece = rem & 7;
            long ng = node_lo + nd;
            ng = ng < n_nodes ? ng : n_nodes - 1;
            const int side = rr >= 13, k = side ? rr - 13 : rr;      // k: 0, 1..3, 4..12
            const int rank = k == 0 ? 0 : (k < 4 ? 1 : 2);
            const int comp = k == 0 ? 0 : (k < 4 ? k - 1 : k - 4);
            const int C = rank == 0 ? 1 : (rank == 1 ? 3 : 9);
            const float* base = side ? ops.r[rank] : ops.l[rank];
            v[u] = *reinterpret_cast<const float4*>(base + (ng * C + comp) * chan + cb * 32 + 4 * piece);
            dst[u] = (rr * NN + nd) * kRowF + 4 * piece;
        }
#pragma unroll
        for (int u = 0; u < kStagePer; u++) *reinterpret_cast<float4*>(stage + dst[u]) = v[u];
    };
    auto build_a = [&](ARegs& a, int li) {
        const int label = ops.labels[li];
        const int rl = kPRankL[label], rr = kPRankR[label];
        const SignedDot d = signed_dot(label, co);
        const int lrow = (rl == 0 ? 0 : (rl == 1 ? 1 : 4)) + d.lb;
        const int rrow = 13 + (rr == 0 ? 0 : (rr == 1 ? 1 : 4)) + d.rb;
        const float* lp = stage + (lrow * NN + nl) * kRowF + 16 * g;
        const float* rp = stage + (rrow * NN + nl) * kRowF + 16 * g;
        const int lstep = d.ls * NN * kRowF, rstep = d.rs * NN * kRowF;
#pragma unroll
        for (int j = 0; j < 4; j++) a.v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int t = 0; t < d.nt; t++) {                  // trip count fixed by the product type: uniform
            const float sgn = (d.cross && t == 1) ? -1.f : 1.f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float4 x = *reinterpret_cast<const float4*>(lp + t * lstep + 4 * j);
                const float4 y = *reinterpret_cast<const float4*>(rp + t * rstep + 4 * j);
                a.v[j].x += sgn * x.x * y.x;
                a.v[j].y += sgn * x.y * y.y;
                a.v[j].z += sgn * x.z * y.z;
                a.v[j].w += sgn * x.w * y.w;
            }
        }
    };
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
    auto compute = [&](const ARegs& a, const unsigned char* buf) {
        halfx8 ah[2], al[2];
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const HalfSplit4 p0 = split(a.v[2 * s], sx), p1 = split(a.v[2 * s + 1], sx);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                ah[s][i] = p0.hi[i]; ah[s][4 + i] = p1.hi[i];
                al[s][i] = p0.lo[i]; al[s][4 + i] = p1.lo[i];
            }
        }
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
            for (int ni = 0; ni < NI; ni++) {
                const halfx8 bh = *reinterpret_cast<const halfx8*>(buf + b_off + ni * 32 * kRowW + 16 * s);
                const halfx8 bl = *reinterpret_cast<const halfx8*>(buf + kPlaneW + b_off + ni * 32 * kRowW + 16 * s);
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[s], bh, acc[ni], 0, 0, 0);
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[s], bl, acc[ni], 0, 0, 0);
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[s], bh, acc[ni], 0, 0, 0);
            }
    };

    WRegs w;
    load_w(w, 0);
    stage_block(0);
    store_w(w, lds);
    load_w(w, kCK);
    __syncthreads();
    const int n_chunks = I / kCK;
    int li = 0, cb = 0;
    for (int ch = 0; ch < n_chunks; ch++) {
        ARegs a;
        build_a(a, li);
        compute(a, lds + (ch & 1) * kBufW);
        store_w(w, lds + ((ch + 1) & 1) * kBufW);         // chunk ch + 1 (a clamped reload past the end, never used)
        load_w(w, (ch + 2) * kCK);
        if (++li == NL) {
            li = 0;
            cb++;
            __syncthreads();                               // every wave has built its last operand of this block
            if (ch + 1 < n_chunks) stage_block(cb);
        }
        __syncthreads();
    }

    float iw[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ni++) {
        const int n = n0 + ni * 32 + m;
        iw[ni] = n < O ? w_inv[n] : 0.f;
    }
#pragma unroll
    for (int q = 0; q < 16; q++) {
        const int rl = wave * 32 + 8 * (q / 4) + 4 * g + (q % 4);
        const long r = r0 + rl;
        if (r < R) {
            const long nd = r / T;
            float* yp = Y + (nd * O + n0 + m) * T + (r - nd * T);
            const float isx = inv_sx[rl];
#pragma unroll
            for (int ni = 0; ni < NI; ni++)
                if (n0 + ni * 32 + m < O) yp[ni * 32 * T] = acc[ni][q] * isx * iw[ni];
        }
    }
}

template <int WAVES, int NI, int T>
int launch(const _Float16* planes, const float* w_inv, const Operands& ops, const float* bound, long n_nodes, int chan,
           int O, int O_pad, float* y, hipStream_t st) {
    const long tiles_m = ceil_div(n_nodes * T, 32 * WAVES);
    const int tiles_n = (int)ceil_div(O, 32 * NI);
    const long total = tiles_m * tiles_n;
    const long grid = ceil_div(total, 8) * 8;
    MG_REQUIRE(grid <= 0x7fffffffL, "mg_bee_products_linear: grid too large");
    hipLaunchKernelGGL((products_linear_kernel<WAVES, NI, T>), dim3((unsigned)grid), dim3(64 * WAVES), 0, st, planes,
                       w_inv, ops, bound, n_nodes, chan, O, O_pad, y, tiles_n, total);
    return check_launch("mg_bee_products_linear");
}

template <int T>
int dispatch(const _Float16* planes, const float* w_inv, const Operands& ops, const float* bound, long n_nodes,
             int chan, int O, int O_pad, float* y, hipStream_t st) {
    // few rows: narrow column tiles, so that the chip sees a hundred workgroups and more instead of a handful (a
    // workgroup walks the whole reduction dimension: with 2048 nodes and 256 outputs the 256-column tile gave 8
    // workgroups 24 chunks each and took 270 us; the operands re-read by the column tiles come from L2)
    const long rows = n_nodes * T;
    if (O <= 32 || (O % 32 == 0 && ceil_div(rows, 128) * ceil_div(O, 64) < 256))
        return launch<4, 1, T>(planes, w_inv, ops, bound, n_nodes, chan, O, O_pad, y, st);
    if (O <= 64 || (O % 64 == 0 && ceil_div(rows, 256) * ceil_div(O, 128) < 256))
        return launch<4, 2, T>(planes, w_inv, ops, bound, n_nodes, chan, O, O_pad, y, st);
    if (O <= 128) return launch<8, 4, T>(planes, w_inv, ops, bound, n_nodes, chan, O, O_pad, y, st);
    return launch<8, 8, T>(planes, w_inv, ops, bound, n_nodes, chan, O, O_pad, y, st);
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_bee_products_linear(int rank_o, const float* l_0, const float* l_1, const float* l_2, const float* r_0,
                           const float* r_1, const float* r_2, const float* node_bound, long n_nodes, int chan,
                           const void* packed_W, int k_order, int dim_out, float* y, mg_stream_t stream) {
    MG_REQUIRE(k_order == 0 || (k_order == 1 && rank_o == 2 && dim_out <= 64),
               "mg_bee_products_linear: k_order 1 (channel blocks outermost) is for rank_o == 2 with dim_out <= 64");
    MG_REQUIRE(rank_o >= 0 && rank_o <= 2, "mg_bee_products_linear: rank_o must be 0, 1 or 2");
    MG_REQUIRE(chan >= 32 && chan % 32 == 0, "mg_bee_products_linear: chan must be a multiple of 32 (got %d)", chan);
    MG_REQUIRE(n_nodes >= 0 && dim_out >= 0, "mg_bee_products_linear: negative size");
    if (n_nodes == 0 || dim_out == 0) return MG_OK;
    MG_REQUIRE(l_0 && l_1 && l_2 && r_0 && r_1 && r_2 && node_bound && packed_W && y, "mg_bee_products_linear: null pointer");
    MG_REQUIRE(aligned16(l_0) && aligned16(l_1) && aligned16(l_2) && aligned16(r_0) && aligned16(r_1) && aligned16(r_2) &&
                   aligned16(packed_W),
               "mg_bee_products_linear: operands must be 16-byte aligned");
    Operands ops{};
    ops.l[0] = l_0; ops.l[1] = l_1; ops.l[2] = l_2;
    ops.r[0] = r_0; ops.r[1] = r_1; ops.r[2] = r_2;
    static const int by_rank[3][5] = {{0, 1, 2, 0, 0}, {3, 4, 5, 6, 11}, {7, 8, 9, 10, 12}};
    ops.n_labels = rank_o == 0 ? 3 : 5;
    for (int k = 0; k < 5; k++) ops.labels[k] = by_rank[rank_o][k];
    const int dim_in = ops.n_labels * chan;
    const int O_pad = (dim_out + 255) / 256 * 256;
    const _Float16* planes = static_cast<const _Float16*>(packed_W);
    const float* w_inv = reinterpret_cast<const float*>(planes + 2L * O_pad * dim_in);
    hipStream_t st = (hipStream_t)stream;
    if (k_order == 1) {
        const long tiles_m = ceil_div(n_nodes * 9, 128);
        const int ni = dim_out <= 32 ? 1 : 2;
        const int tiles_n = (int)ceil_div(dim_out, 32 * ni);
        const long total = tiles_m * tiles_n;
        const long grid = ceil_div(total, 8) * 8;
        MG_REQUIRE(grid <= 0x7fffffffL, "mg_bee_products_linear: grid too large");
        if (ni == 1)
            hipLaunchKernelGGL((products_linear_staged_kernel<1>), dim3((unsigned)grid), dim3(256), 0, st, planes, w_inv,
                               ops, node_bound, n_nodes, chan, dim_out, O_pad, y, tiles_n, total);
        else
            hipLaunchKernelGGL((products_linear_staged_kernel<2>), dim3((unsigned)grid), dim3(256), 0, st, planes, w_inv,
                               ops, node_bound, n_nodes, chan, dim_out, O_pad, y, tiles_n, total);
        return check_launch("mg_bee_products_linear");
    }
    if (rank_o == 0) return dispatch<1>(planes, w_inv, ops, node_bound, n_nodes, chan, dim_out, O_pad, y, st);
    if (rank_o == 1) return dispatch<3>(planes, w_inv, ops, node_bound, n_nodes, chan, dim_out, O_pad, y, st);
    return dispatch<9>(planes, w_inv, ops, node_bound, n_nodes, chan, dim_out, O_pad, y, st);
}

}  // extern "C"
