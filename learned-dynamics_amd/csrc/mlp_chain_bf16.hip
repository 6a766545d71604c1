// The per-edge chain of the rank-0/1/2 messages on bf16 storage (archs/diffuser_atoms15.py:98-110, 244-246),
// for the two sums over edges that the node-side layers need:
//     psi = Y P0                      (edges, 128)      -> sum over the edges of each node of bf16(psi)
//     h1  = act(W1 psi + b1)          (edges, 256)
//     h2  = act(W2 h1 + b2)           (edges, 256)      -> sum over the edges of each node of bf16(h2)
// in ONE kernel: psi, h1 and h2 never leave the registers.  With W as the first matrix operand an accumulator
// register holds (edge = lane % 32, four consecutive channels), and that is also the layout the matrix core
// wants for its second operand (16 of a 32-channel chunk's channels per lane half), up to a fixed permutation of
// the channels inside a chunk which the caller applies to the input channels of W1 and W2 before packing.  So
// the bf16-rounded outputs of one layer (rounded exactly where the separate kernels round them when they store)
// are the operands of the next without any data movement.  Weights stream through LDS as in the plain kernel
// (two bf16 planes, 16 significand bits); x = P0 is the only tensor read from HBM, the sums the only output.
// Widths are fixed (128 -> 256 -> 256) by the register budget: 64 + 128 accumulators and 64 operand registers.
#include "common.hpp"
#include "rowsum_finish.hpp"

namespace mg {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kCK = 32;      // k per chunk (two MFMA steps)
constexpr int kRowW = 80;    // bytes per LDS row of one W plane (64 + 16 pad)
constexpr int kRB = 1;       // blocks of 32 rows per wave.  With 2 every W fragment read from LDS would feed two matrix
                             // instructions, but 256 accumulators leave one wave per SIMD and nothing to hide the
                             // loads and barriers behind: measured 4.7 ms against 2.0 ms at 2.26 M rows
constexpr int kWaves = 8 / kRB, kThreads = 64 * kWaves;      // 256 rows per workgroup
constexpr int kD = 128, kH = 256;
constexpr int kLdsBytes = 2 * 2 * kH * kRowW;               // two buffers of two planes of 256 rows
constexpr int kRed = 68;                                     // floats per row of a reduction slice

template <int ACT>
__device__ __forceinline__ float activate_c(float v) {
    if constexpr (ACT == 1) return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    if constexpr (ACT == 2) return v > 0.f ? v : 0.1f * v;
    return v;
}

// Streams the two planes of W (rows n0 .. n0 + 32 NI of a (w_rows, I) packed matrix) through LDS chunk by chunk.
template <int NI>
struct WStream {
    static constexpr int TN = 32 * NI, kPlaneW = TN * kRowW, kBufW = 2 * kPlaneW;
    static constexpr int kPer = 8 * TN / kThreads;           // 16-byte pieces per thread and chunk
    static_assert(TN % 128 == 0, "a thread's pieces must differ by whole planes and rows only");
    const __bf16* src;                                        // piece j: + plane(j) plane_elems + row(j) I
    long plane_elems;
    int dst, I;
    bf16x8 regs[kPer];
    static constexpr int plane_of(int j) { return (kThreads * j) / (4 * TN); }
    static constexpr int row_of(int j) { return ((kThreads * j) % (4 * TN)) / 4; }
    __device__ __forceinline__ void init(const __bf16* Wp, long plane_elems_, int I_) {
        I = I_;
        plane_elems = plane_elems_;
        const int tid = threadIdx.x;
        src = Wp + (long)(tid >> 2) * I + 8 * (tid & 3);
        dst = (tid >> 2) * kRowW + (tid & 3) * 16;
    }
    __device__ __forceinline__ void load(int k0) {
        k0 = k0 < I ? k0 : I - kCK;                           // surplus requests past the end are never used
#pragma unroll
        for (int j = 0; j < kPer; j++)
            regs[j] = *reinterpret_cast<const bf16x8*>(src + plane_of(j) * plane_elems + (long)row_of(j) * I + k0);
    }
    __device__ __forceinline__ void store(unsigned char* buf) const {
#pragma unroll
        for (int j = 0; j < kPer; j++)
            *reinterpret_cast<bf16x8*>(buf + dst + plane_of(j) * kPlaneW + row_of(j) * kRowW) = regs[j];
    }
    // acc[rb][ni] += W chunk (from buf) x the lane's 16 operand values of the chunk (two 8-value steps)
    template <typename XOf>
    __device__ __forceinline__ void multiply(floatx16 (&acc)[kRB][NI], const unsigned char* buf, XOf x_of) const {
        const int lane = threadIdx.x & 63;
        const int b_off = (lane & 31) * kRowW + 32 * (lane >> 5);
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
            for (int ni = 0; ni < NI; ni++) {
                const bf16x8 wh = *reinterpret_cast<const bf16x8*>(buf + b_off + ni * 32 * kRowW + 16 * s);
                const bf16x8 wm = *reinterpret_cast<const bf16x8*>(buf + kPlaneW + b_off + ni * 32 * kRowW + 16 * s);
#pragma unroll
                for (int rb = 0; rb < kRB; rb++) {
                    acc[rb][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wm, x_of(rb, s), acc[rb][ni], 0, 0, 0);   // small term first
                    acc[rb][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wh, x_of(rb, s), acc[rb][ni], 0, 0, 0);
                }
            }
    }
};

// act(acc + bias) of a layer with 32 NI channels, rounded to bf16: chunk c, step s -> the lane's eight operand
// values for the next layer (accumulator registers 8 s .. 8 s + 7 of block c).  BIAS = false: no bias.
template <int ACT, bool BIAS, int NI>
__device__ __forceinline__ void to_operands(const floatx16 (&acc)[kRB][NI], const float* __restrict__ bias,
                                            bf16x8 (&ops)[kRB][NI][2]) {
    const int g = (threadIdx.x >> 5) & 1;
#pragma unroll
    for (int c = 0; c < NI; c++) {
        float4 b[4];
#pragma unroll
        for (int qq = 0; qq < 4; qq++)
            b[qq] = BIAS ? *reinterpret_cast<const float4*>(bias + 32 * c + 8 * qq + 4 * g) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int rb = 0; rb < kRB; rb++)
#pragma unroll
            for (int q = 0; q < 16; q++) {
                const float v = activate_c<ACT>(acc[rb][c][q] + (&b[q / 4].x)[q % 4]);
                ops[rb][c][q / 8][q % 8] = (__bf16)v;
            }
        __builtin_amdgcn_sched_barrier(0);                    // one block at a time: the registers are nearly all taken
    }
}

// layer whose operands are in registers: K = 32 NCH
template <int NI, int NCH>
__device__ __forceinline__ void layer_from_registers(floatx16 (&acc)[kRB][NI], const __bf16* Wp, long plane_elems,
                                                     const bf16x8 (&ops)[kRB][NCH][2], unsigned char* lds) {
    WStream<NI> w;
    w.init(Wp, plane_elems, 32 * NCH);
    w.load(0);
    __syncthreads();                                          // the previous layer is done with the W buffers
    w.store(lds);
    w.load(kCK);
    __syncthreads();
#pragma unroll
    for (int c = 0; c < NCH; c++) {
        w.multiply(acc, lds + (c & 1) * WStream<NI>::kBufW, [&](int rb, int s) { return ops[rb][c][s]; });
        w.store(lds + ((c + 1) & 1) * WStream<NI>::kBufW);
        w.load((c + 2) * kCK);
        __syncthreads();
    }
}

struct SegmentRuns {
    int my_seg, nv, runs, second;
    unsigned starts;
};

// sum over the rows of each segment of the bf16-rounded act(acc + bias): two partial slots per block of 32 rows,
// runs strictly inside a block written to `out` directly (fp32 accumulation, scale applied there)
template <int ACT, bool BIAS, int NI>
__device__ __forceinline__ void row_sums(const floatx16 (&acc)[NI], const float* __restrict__ bias, bool row_live,
                                         const SegmentRuns& sr, float* slice, float* __restrict__ slots, long block,
                                         long n_blocks, float* __restrict__ out, float scale) {
    constexpr int O = 32 * NI;
    const int lane = threadIdx.x & 63, m = lane & 31, g = lane >> 5;
#pragma unroll
    for (int pass = 0; pass < NI / 2; pass++) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int ni = 2 * pass + h;
#pragma unroll
            for (int qq = 0; qq < 4; qq++) {
                const float4 b = BIAS ? *reinterpret_cast<const float4*>(bias + 32 * ni + 8 * qq + 4 * g)
                                      : make_float4(0.f, 0.f, 0.f, 0.f);
                float4 v;
                float* vp = &v.x;
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const float x = activate_c<ACT>(acc[ni][4 * qq + t] + (&b.x)[t]);
                    vp[t] = row_live ? (float)(__bf16)x : 0.f;
                }
                *reinterpret_cast<float4*>(slice + m * kRed + 32 * h + 8 * qq + 4 * g) = v;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int col = 64 * pass + lane;
        auto flush = [&](float sum, int run_start, int r) {
            if (run_start == 0) {
                slots[block * O + col] = sum;
            } else if (r == 31) {
                slots[(n_blocks + block) * O + col] = sum;
            } else {
                const long s_id = __shfl(sr.my_seg, r);
                out[s_id * O + col] = scale * sum;
            }
        };
        if (sr.nv > 0) {
            if (sr.runs <= 2) {
                float s0 = 0.f, s1 = 0.f;
#pragma unroll
                for (int r = 0; r < 32; r++) {
                    const float val = slice[r * kRed + lane];
                    s0 += r < sr.second ? val : 0.f;
                    s1 += r < sr.second ? 0.f : val;
                }
                flush(s0, 0, sr.second - 1);
                if (sr.runs == 2) flush(s1, sr.second, sr.nv - 1);
            } else {
                float sum = 0.f;
                int run_start = 0;
                for (int r = 0; r < sr.nv; r++) {
                    sum += slice[r * kRed + lane];
                    if ((r == sr.nv - 1) || ((sr.starts >> (r + 1)) & 1u)) {
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

template <int ACT>
__global__ void __launch_bounds__(kThreads)
mlp_chain_bf16_kernel(const __bf16* __restrict__ X, long R, int I, const __bf16* __restrict__ Wa, long plane_a,
                      const __bf16* __restrict__ Wb, long plane_b, const float* __restrict__ bias_b,
                      const __bf16* __restrict__ Wc, long plane_c, const float* __restrict__ bias_c,
                      const int* __restrict__ seg, float* __restrict__ slots_x, float* __restrict__ slots_h,
                      long n_blocks, float* __restrict__ out_x, float* __restrict__ out_h, long tiles_total) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[kLdsBytes];
    static_assert(kLdsBytes / kWaves / 4 >= 32 * kRed, "a reduction pass needs 32 rows x 64 columns per wave");

    const long bid = blockIdx.x;
    const long per_xcd = (tiles_total + 7) / 8;
    const long tile = (bid % 8) * per_xcd + bid / 8;
    if (tile >= tiles_total) return;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, g = lane >> 5;
    const long block0 = (tile * kWaves + wave) * kRB;         // this wave's first block of 32 rows
    long ld_row[kRB];
    bool row_live[kRB];
    SegmentRuns sr[kRB];
#pragma unroll
    for (int rb = 0; rb < kRB; rb++) {
        const long my_row = (block0 + rb) * 32 + m;
        ld_row[rb] = my_row < R ? my_row : R - 1;
        row_live[rb] = my_row < R;
        sr[rb].my_seg = seg[ld_row[rb]];
        const long rows_left = R - (block0 + rb) * 32;
        sr[rb].nv = rows_left >= 32 ? 32 : (rows_left > 0 ? (int)rows_left : 0);
        const int prev = __shfl_up(sr[rb].my_seg, 1);
        sr[rb].starts = (unsigned)__ballot(g == 0 && (m == 0 || sr[rb].my_seg != prev));
        sr[rb].runs = __popc(sr[rb].starts);
        sr[rb].second = sr[rb].runs >= 2 ? __ffs(sr[rb].starts & ~1u) - 1 : 32;
    }
    float* slice = reinterpret_cast<float*>(lds) + wave * (kLdsBytes / kWaves / 4);

    // ---- layer A: psi = Y x, x from memory (the lane's 16 bf16 of its row per chunk, two chunks ahead)
    floatx16 acc_a[kRB][kD / 32];
#pragma unroll
    for (int rb = 0; rb < kRB; rb++)
#pragma unroll
        for (int ni = 0; ni < kD / 32; ni++)
#pragma unroll
            for (int q = 0; q < 16; q++) acc_a[rb][ni][q] = 0.f;
    {
        using WS = WStream<kD / 32>;
        WS w;
        w.init(Wa, plane_a, I);
        const int k_last = I - kCK;
        auto load_x = [&](bf16x8 (&x)[kRB][2], int k0) {
            k0 = k0 < I ? k0 : k_last;
#pragma unroll
            for (int rb = 0; rb < kRB; rb++) {
                const __bf16* xrow = X + ld_row[rb] * I + 16 * g + k0;
                x[rb][0] = *reinterpret_cast<const bf16x8*>(xrow);
                x[rb][1] = *reinterpret_cast<const bf16x8*>(xrow + 8);
            }
        };
        const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
        bf16x8 x0[kRB][2], x1[kRB][2];
        w.load(0);
        load_x(x0, 0);
        w.store(lds);
        w.load(kCK);
        load_x(x1, kCK);
        __syncthreads();
        for (int k0 = 0; k0 < I; k0 += 2 * kCK) {
            w.multiply(acc_a, lds, [&](int rb, int s) { return x0[rb][s]; });
            w.store(lds + WS::kBufW);
            __builtin_amdgcn_sched_barrier(0);
            w.load(k0 + 2 * kCK);
            __builtin_amdgcn_sched_barrier(0);
            load_x(x0, k0 + 2 * kCK);
            __syncthreads();
            if (k0 + kCK >= I) {                              // a surplus odd chunk contributes nothing
#pragma unroll
                for (int rb = 0; rb < kRB; rb++) { x1[rb][0] = zero; x1[rb][1] = zero; }
            }
            w.multiply(acc_a, lds + WS::kBufW, [&](int rb, int s) { return x1[rb][s]; });
            w.store(lds);
            __builtin_amdgcn_sched_barrier(0);
            w.load(k0 + 3 * kCK);
            __builtin_amdgcn_sched_barrier(0);
            load_x(x1, k0 + 3 * kCK);
            __syncthreads();
        }
    }
    // sums of bf16(psi) per node, and psi as the operands of layer B
    bf16x8 ops_a[kRB][kD / 32][2];
#pragma unroll
    for (int rb = 0; rb < kRB; rb++)
        row_sums<0, false>(acc_a[rb], nullptr, row_live[rb], sr[rb], slice, slots_x, block0 + rb, n_blocks, out_x, 1.0f);
    to_operands<0, false>(acc_a, nullptr, ops_a);

    // ---- layer B: h1 = act(W1 psi + b1)
    floatx16 acc_b[kRB][kH / 32];
#pragma unroll
    for (int rb = 0; rb < kRB; rb++)
#pragma unroll
        for (int ni = 0; ni < kH / 32; ni++)
#pragma unroll
            for (int q = 0; q < 16; q++) acc_b[rb][ni][q] = 0.f;
    layer_from_registers<kH / 32, kD / 32>(acc_b, Wb, plane_b, ops_a, lds);
    bf16x8 ops_b[kRB][kH / 32][2];
    to_operands<ACT, true>(acc_b, bias_b, ops_b);

    // ---- layer C: h2 = act(W2 h1 + b2), only its sums per node leave the kernel
#pragma unroll
    for (int rb = 0; rb < kRB; rb++)
#pragma unroll
        for (int ni = 0; ni < kH / 32; ni++)
#pragma unroll
            for (int q = 0; q < 16; q++) acc_b[rb][ni][q] = 0.f;
    layer_from_registers<kH / 32, kH / 32>(acc_b, Wc, plane_c, ops_b, lds);
#pragma unroll
    for (int rb = 0; rb < kRB; rb++)
        row_sums<ACT, true>(acc_b[rb], bias_c, row_live[rb], sr[rb], slice, slots_h, block0 + rb, n_blocks, out_h, 1.0f);
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_mlp_chain_bf16_workspace_bytes(long rows, size_t* bytes) {
    MG_REQUIRE(bytes != nullptr && rows >= 0, "mg_mlp_chain_bf16_workspace_bytes: bad argument");
    *bytes = (size_t)(2L * (ceil_div(rows, 32) + 1) * (kD + kH)) * sizeof(float);
    return MG_OK;
}

int mg_mlp_chain_bf16(const void* x, long rows, int dim_in, const void* packed_Y, const void* packed_W1,
                      const float* b1, const void* packed_W2, const float* b2, int act, const int* row_ptr,
                      const int* seg, long n_out, void* workspace, float* sum_psi, float* sum_h2, mg_stream_t stream) {
    MG_REQUIRE(dim_in >= 32 && dim_in % 32 == 0, "mg_mlp_chain_bf16: dim_in must be a multiple of 32 (got %d)", dim_in);
    MG_REQUIRE(rows >= 0 && n_out >= 0 && rows < (1L << 31) && n_out < (1L << 31), "mg_mlp_chain_bf16: bad size");
    MG_REQUIRE(act >= 0 && act <= 2, "mg_mlp_chain_bf16: unknown activation %d", act);
    if (n_out == 0) return MG_OK;
    MG_REQUIRE(packed_Y && packed_W1 && packed_W2 && row_ptr && sum_psi && sum_h2 && workspace && aligned16(packed_Y) &&
                   aligned16(packed_W1) && aligned16(packed_W2) && aligned16(workspace) && aligned16(sum_psi) &&
                   aligned16(sum_h2),
               "mg_mlp_chain_bf16: null or unaligned operand");
    hipStream_t st = (hipStream_t)stream;
    const long n_blocks = ceil_div(rows, 32);
    float* slots_x = static_cast<float*>(workspace);
    float* slots_h = slots_x + 2L * (n_blocks + 1) * kD;
    if (rows > 0) {
        MG_REQUIRE(x && seg && aligned16(x), "mg_mlp_chain_bf16: null or unaligned row operand");
        const long tiles = ceil_div(rows, 32 * kWaves);
        const long grid = ceil_div(tiles, 8) * 8;
        MG_REQUIRE(grid <= 0x7fffffffL, "mg_mlp_chain_bf16: grid too large");
        // packed weights: planes of ceil(dim_out / 128) * 128 rows
        const long plane_a = (long)kD * dim_in, plane_b = (long)kH * kD, plane_c = (long)kH * kH;
#define MG_CHAIN_LAUNCH(A)                                                                                          \
    hipLaunchKernelGGL((mlp_chain_bf16_kernel<A>), dim3((unsigned)grid), dim3(kThreads), 0, st,                        \
                       static_cast<const __bf16*>(x), rows, dim_in, static_cast<const __bf16*>(packed_Y), plane_a,    \
                       static_cast<const __bf16*>(packed_W1), plane_b, b1, static_cast<const __bf16*>(packed_W2),     \
                       plane_c, b2, seg, slots_x, slots_h, n_blocks, sum_psi, sum_h2, tiles)
        if (act == 1) MG_CHAIN_LAUNCH(1);
        else if (act == 2) MG_CHAIN_LAUNCH(2);
        else MG_CHAIN_LAUNCH(0);
#undef MG_CHAIN_LAUNCH
        if (int code = check_launch("mlp_chain_bf16_kernel")) return code;
    }
    rowsum_finish_kernel<<<dim3((unsigned)ceil_div(n_out * (kD / 4), 256)), dim3(256), 0, st>>>(
        row_ptr, n_out, n_blocks, kD, slots_x, 1.0f, sum_psi);
    if (int code = check_launch("rowsum_finish_kernel")) return code;
    rowsum_finish_kernel<<<dim3((unsigned)ceil_div(n_out * (kH / 4), 256)), dim3(256), 0, st>>>(
        row_ptr, n_out, n_blocks, kH, slots_h, 1.0f, sum_h2);
    return check_launch("rowsum_finish_kernel");
}

}  // extern "C"
