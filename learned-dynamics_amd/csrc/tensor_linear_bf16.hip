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
// Row-streaming shape: a workgroup of WAVES waves owns 32 WAVES rows x 32 NI columns; wave w owns
// rows [32 w, 32 w + 32) and all columns of the tile.
//   * x never touches LDS: lane = row + 32 g loads the 16 consecutive bf16 of ITS row that it
//     feeds to the matrix core (k = 32 c + 16 g .. + 16 of chunk c, two 16-byte loads that ARE
//     the MFMA operands), two chunks ahead.  No load is predicated (rows past the end are
//     clamped and never written), so loads stay in flight across the loop.
//   * the two W planes go global -> registers -> LDS, double buffered, chunk of 32 k (80-byte rows:
//     conflict free for 16-byte reads), one barrier per chunk; W is requested before x because
//     loads return in order and W (L2 resident) is needed first.
//   * W is the FIRST matrix operand and x the second, so a lane ends up with its own row of x and
//     four consecutive output channels per accumulator quad: the epilogue writes 8-byte (bf16) or
//     16-byte (fp32) vectors, one row pointer and one bounds check per lane.
// v_mfma_f32_32x32x16_bf16: A[i][k]: lane = i + 32*(k/8), 8 k per lane; B[k][j] likewise;
// D[i][j]: j = lane%32, i = 8*(q/4) + 4*(lane/32) + q%4 for register q.
#include "common.hpp"
#include "rowsum_finish.hpp"
#include <type_traits>

namespace mg {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

constexpr int kCK = 32;      // k per chunk (two MFMA steps)
constexpr int kRowW = 80;    // bytes per LDS row of one W plane (64 + 16 pad)

template <int ACT>
__device__ __forceinline__ float activate_c(float v) {
    // SiLU through the hardware exp2 and reciprocal (about 1 ulp each)
    if constexpr (ACT == 1) return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    if constexpr (ACT == 2) return v > 0.f ? v : 0.1f * v;
    return v;
}

__device__ __forceinline__ floatx4 load4(const float* p) { return *reinterpret_cast<const floatx4*>(p); }
__device__ __forceinline__ floatx4 load4(const __bf16* p) {
    const bf16x4 t = *reinterpret_cast<const bf16x4*>(p);
    return floatx4{(float)t[0], (float)t[1], (float)t[2], (float)t[3]};
}
__device__ __forceinline__ void store4(float* p, floatx4 v) { *reinterpret_cast<floatx4*>(p) = v; }
__device__ __forceinline__ void store4(__bf16* p, floatx4 v) {
    *reinterpret_cast<bf16x4*>(p) = bf16x4{(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
}

// Sum of the output rows per segment in the epilogue (rows sorted by segment): seg[row] ascending, two partial
// slots per block of 32 rows, runs inside a block written to `out` directly, as in the fp32 kernels that do this.
struct RowSum {
    const int* seg;
    float* slots;
    long n_blocks;
    float* out;      // (segments, O) float32
    float scale;
    int store_y;     // also write the rows themselves
};

template <int WAVES, int NI, typename YT, bool ROWSUM = false>
__global__ void __launch_bounds__(64 * WAVES)
linear_rows_bf16_kernel(const __bf16* __restrict__ Wp, long plane_elems, int w_rows, const __bf16* __restrict__ X,
                        long R, int I, int O, const float* __restrict__ bias, int act, int accumulate,
                        YT* __restrict__ Y, int tiles_n, long tiles_total, int out_T, RowSum rs = RowSum{}) {
    constexpr int TM = 32 * WAVES, TN = 32 * NI, THREADS = 64 * WAVES;
    constexpr int kPlaneW = TN * kRowW, kBufW = 2 * kPlaneW;
    constexpr int kPieces = 8 * TN;                          // 16-byte pieces of W per chunk (2 planes x TN rows x 4)
    constexpr int kPer = (kPieces + THREADS - 1) / THREADS;
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kBufW];

    const long bid = blockIdx.x;
    const long per_xcd = (tiles_total + 7) / 8;
    const long logical = (bid % 8) * per_xcd + bid / 8;
    if (logical >= tiles_total) return;
    const long tile_m = logical / tiles_n;
    const int tile_n = (int)(logical - tile_m * tiles_n);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, g = lane >> 5;
    const long r0 = tile_m * TM;
    const int n0 = tile_n * TN;

    floatx16 acc[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ni++)
#pragma unroll
        for (int q = 0; q < 16; q++) acc[ni][q] = 0.f;

    const long my_row = r0 + wave * 32 + m;
    const long ld_row = my_row < R ? my_row : R - 1;       // clamped: such rows are never written
    const __bf16* xrow = X + ld_row * I + 16 * g;
    const __bf16* wsrc[kPer];
    int wdst[kPer];
#pragma unroll
    for (int j = 0; j < kPer; j++) {
        int q = tid + THREADS * j;
        if (q >= kPieces) q = kPieces - 1;                   // surplus threads repeat the last piece
        const int plane = q / (4 * TN), row = (q % (4 * TN)) >> 2, piece = q & 3;
        int wrow = n0 + row;
        if (wrow >= w_rows) wrow = w_rows - 1;               // columns past dim_out are never written
        wsrc[j] = Wp + plane * plane_elems + (long)wrow * I + 8 * piece;
        wdst[j] = plane * kPlaneW + row * kRowW + piece * 16;
    }
    const int k_last = I - kCK;

    struct ARegs { bf16x8 v[2]; };
    struct WRegs { bf16x8 v[kPer]; };
    auto load_a = [&](ARegs& a, int k0) {
        k0 = k0 < I ? k0 : k_last;                           // surplus loads of the last trips are never used
#pragma unroll
        for (int s = 0; s < 2; s++) a.v[s] = *reinterpret_cast<const bf16x8*>(xrow + k0 + 8 * s);
    };
    auto load_w = [&](WRegs& w, int k0) {
        k0 = k0 < I ? k0 : k_last;
#pragma unroll
        for (int j = 0; j < kPer; j++) w.v[j] = *reinterpret_cast<const bf16x8*>(wsrc[j] + k0);
    };
    auto store_w = [&](const WRegs& w, unsigned char* buf) {
#pragma unroll
        for (int j = 0; j < kPer; j++) *reinterpret_cast<bf16x8*>(buf + wdst[j]) = w.v[j];
    };
    const int b_off = m * kRowW + 32 * g;
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    auto compute = [&](const ARegs& a, const unsigned char* buf, bool live) {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const bf16x8 xs = live ? a.v[s] : zero;          // a surplus odd chunk contributes nothing
#pragma unroll
            for (int ni = 0; ni < NI; ni++) {
                const bf16x8 wh = *reinterpret_cast<const bf16x8*>(buf + b_off + ni * 32 * kRowW + 16 * s);
                const bf16x8 wm = *reinterpret_cast<const bf16x8*>(buf + kPlaneW + b_off + ni * 32 * kRowW + 16 * s);
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wm, xs, acc[ni], 0, 0, 0);   // small term first
                acc[ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wh, xs, acc[ni], 0, 0, 0);
            }
        }
    };

    unsigned char* buf0 = lds;
    unsigned char* buf1 = lds + kBufW;
    ARegs a0, a1;
    WRegs w;
    load_w(w, 0);
    load_a(a0, 0);
    store_w(w, buf0);
    load_w(w, kCK);
    load_a(a1, kCK);
    __syncthreads();
    for (int k0 = 0; k0 < I; k0 += 2 * kCK) {
        compute(a0, buf0, true);
        store_w(w, buf1);
        __builtin_amdgcn_sched_barrier(0);     // keep this issue order: the compiler would hoist the loads
        load_w(w, k0 + 2 * kCK);
        __builtin_amdgcn_sched_barrier(0);
        load_a(a0, k0 + 2 * kCK);
        __syncthreads();
        compute(a1, buf1, k0 + kCK < I);
        store_w(w, buf0);
        __builtin_amdgcn_sched_barrier(0);
        load_w(w, k0 + 3 * kCK);
        __builtin_amdgcn_sched_barrier(0);
        load_a(a1, k0 + 3 * kCK);
        __syncthreads();
    }

    // lane (m, g) holds row my_row and, for accumulator quad qq of block ni, the four channels
    // n0 + 32 ni + 8 qq + 4 g .. + 4
    //
    // bf16 output, full tile: the rows are first transposed through the wave's own slice of the
    // (now idle) W buffers, so that the stores to HBM are 16 bytes per lane and whole 64..256-byte
    // row segments per instruction instead of 8-byte pieces scattered over 32 rows (the output is
    // half of this kernel's traffic).  A wave touches only its own slice and its LDS operations
    // execute in order, so no barrier is needed.
    constexpr int kRegion = 2 * kBufW / WAVES;                              // bytes of LDS per wave
    constexpr int kColsFit = (kRegion - 512) / 64;                          // 32 rows x (2 cols + 16) bytes
    constexpr int kPassCols = kColsFit >= 128 ? 128 : (kColsFit >= 64 ? 64 : (kColsFit >= 32 ? 32 : 0));
    if constexpr (std::is_same<YT, __bf16>::value && kPassCols > 0) {
        if (ROWSUM || (out_T == 1 && n0 + TN <= O && (O & 7) == 0 && !accumulate)) {
            constexpr int kCols = kPassCols < TN ? kPassCols : TN;          // columns per pass
            static_assert(!ROWSUM || kCols % 64 == 0, "the row sums take whole groups of 64 columns per pass");
            // ROWSUM: runs of equal segment among the wave's rows (bit r set = row r starts a run)
            const long block = r0 / 32 + wave;
            int my_seg = 0, nv = 0, runs = 1, second = 32;
            unsigned starts = 1u;
            if constexpr (ROWSUM) {
                my_seg = rs.seg[ld_row];
                const long rows_left = R - block * 32;
                nv = rows_left >= 32 ? 32 : (rows_left > 0 ? (int)rows_left : 0);
                const int prev_seg = __shfl_up(my_seg, 1);
                starts = (unsigned)__ballot(g == 0 && (m == 0 || my_seg != prev_seg));
                runs = __popc(starts);
                second = runs >= 2 ? __ffs(starts & ~1u) - 1 : 32;
            }
            constexpr int kRowBytes = 2 * kCols + 16;
            constexpr int kPieces = 32 * kCols / 8;                         // 16-byte pieces per pass
            unsigned char* slice = lds + wave * kRegion;
            const float* brow = bias ? bias + n0 + 4 * g : nullptr;
            auto epilogue = [&](auto act_tag) {
                constexpr int kAct = decltype(act_tag)::value;
#pragma unroll
                for (int pass = 0; pass < TN / kCols; pass++) {
#pragma unroll
                    for (int nl = 0; nl < kCols / 32; nl++) {
                        const int ni = pass * (kCols / 32) + nl;
#pragma unroll
                        for (int qq = 0; qq < 4; qq++) {
                            floatx4 v = {acc[ni][4 * qq], acc[ni][4 * qq + 1], acc[ni][4 * qq + 2], acc[ni][4 * qq + 3]};
                            if (brow) v += load4(brow + 32 * ni + 8 * qq);
#pragma unroll
                            for (int i = 0; i < 4; i++) v[i] = activate_c<kAct>(v[i]);
                            if constexpr (ROWSUM) {
                                if (my_row >= R) v = floatx4{0.f, 0.f, 0.f, 0.f};      // rows past the end add nothing
                            }
                            store4(reinterpret_cast<__bf16*>(slice + m * kRowBytes) + 32 * nl + 8 * qq + 4 * g, v);
                        }
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    if (!ROWSUM || rs.store_y) {
#pragma unroll
                        for (int it = 0; it < (kPieces + 63) / 64; it++) {
                            const int piece = it * 64 + lane;
                            const int row = piece / (kCols / 8), c8 = piece % (kCols / 8);
                            const long r = r0 + wave * 32 + row;
                            if (piece < kPieces && r < R) {
                                const bf16x8 t = *reinterpret_cast<const bf16x8*>(slice + row * kRowBytes + c8 * 16);
                                *reinterpret_cast<bf16x8*>(Y + r * O + n0 + pass * kCols + c8 * 8) = t;
                            }
                        }
                    }
                    if constexpr (ROWSUM) {
                        // lanes take one column (two with 128-column passes) and add the bf16 values of the rows
                        // in fp32, split at the run boundaries
                        if (nv > 0) {
#pragma unroll
                            for (int cc = 0; cc < (kCols + 63) / 64; cc++) {
                                const int cl = cc * 64 + lane;                       // column in this pass
                                if (cl < kCols) {
                                    const int col = n0 + pass * kCols + cl;
                                    const __bf16* colp = reinterpret_cast<const __bf16*>(slice) + cl;
                                    auto flush = [&](float sum, int run_start, int r) {
                                        if (run_start == 0) {
                                            rs.slots[block * O + col] = sum;
                                        } else if (r == 31) {
                                            rs.slots[(rs.n_blocks + block) * O + col] = sum;
                                        } else {
                                            const long s_id = __shfl(my_seg, r);
                                            rs.out[s_id * O + col] = rs.scale * sum;
                                        }
                                    };
                                    if (runs <= 2) {
                                        float s0 = 0.f, s1 = 0.f;
#pragma unroll
                                        for (int r = 0; r < 32; r++) {
                                            const float val = (float)colp[r * (kRowBytes / 2)];
                                            s0 += r < second ? val : 0.f;
                                            s1 += r < second ? 0.f : val;
                                        }
                                        flush(s0, 0, second - 1);
                                        if (runs == 2) flush(s1, second, nv - 1);
                                    } else {
                                        float sum = 0.f;
                                        int run_start = 0;
                                        for (int r = 0; r < nv; r++) {
                                            sum += (float)colp[r * (kRowBytes / 2)];
                                            if ((r == nv - 1) || ((starts >> (r + 1)) & 1u)) {
                                                flush(sum, run_start, r);
                                                sum = 0.f;
                                                run_start = r + 1;
                                            }
                                        }
                                    }
                                }
                            }
                        }
                    }
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                }
            };
            if (act == 1) epilogue(std::integral_constant<int, 1>{});
            else if (act == 2) epilogue(std::integral_constant<int, 2>{});
            else epilogue(std::integral_constant<int, 0>{});
            return;
        }
    }
    if (my_row >= R) return;
    if (out_T == 1 && n0 + TN <= O && (O & 3) == 0) {
        YT* yrow = Y + my_row * O + n0 + 4 * g;
        const float* brow = bias ? bias + n0 + 4 * g : nullptr;
        auto epilogue = [&](auto act_tag) {
            constexpr int kAct = decltype(act_tag)::value;
#pragma unroll
            for (int ni = 0; ni < NI; ni++)
#pragma unroll
                for (int qq = 0; qq < 4; qq++) {
                    const int c = 32 * ni + 8 * qq;
                    floatx4 v = {acc[ni][4 * qq], acc[ni][4 * qq + 1], acc[ni][4 * qq + 2], acc[ni][4 * qq + 3]};
                    if (brow) v += load4(brow + c);
#pragma unroll
                    for (int i = 0; i < 4; i++) v[i] = activate_c<kAct>(v[i]);
                    if (accumulate) v += load4(yrow + c);
                    store4(yrow + c, v);
                }
        };
        if (act == 1) epilogue(std::integral_constant<int, 1>{});
        else if (act == 2) epilogue(std::integral_constant<int, 2>{});
        else epilogue(std::integral_constant<int, 0>{});
        return;
    }
    // general path: partial column tiles, or rows that are (row, comp) pairs with y stored (row, chan, comp)
    const long row = my_row / out_T;
    const long comp = my_row - row * out_T;
#pragma unroll
    for (int ni = 0; ni < NI; ni++)
#pragma unroll
        for (int q = 0; q < 16; q++) {
            const int n = n0 + 32 * ni + 8 * (q / 4) + 4 * g + (q % 4);
            if (n < O) {
                const long addr = (row * O + n) * out_T + comp;
                float v = acc[ni][q] + (bias ? bias[n] : 0.f);
                v = act == 1 ? activate_c<1>(v) : (act == 2 ? activate_c<2>(v) : v);
                if (accumulate) v += (float)Y[addr];
                Y[addr] = (YT)v;
            }
        }
}

struct Shape {
    int ni, waves;
};
inline Shape choose_shape(long R, int O) {
    Shape s;
    s.ni = O <= 32 ? 1 : (O <= 64 ? 2 : (O <= 128 ? 4 : 8));
    const long tiles = ceil_div(R, 256) * ceil_div(O, 32 * s.ni);
    s.waves = tiles >= 512 ? 8 : 4;
    return s;
}

template <int WAVES, int NI, typename YT>
int launch(const __bf16* Wp, long plane_elems, int w_rows, const __bf16* x, long rows, int I, int O, const float* bias,
           int act, int accumulate, YT* y, int out_T, hipStream_t st) {
    const long tiles_m = ceil_div(rows, 32 * WAVES);
    const int tiles_n = (int)ceil_div(O, 32 * NI);
    const long total = tiles_m * tiles_n;
    const long grid = ceil_div(total, 8) * 8;
    MG_REQUIRE(grid <= 0x7fffffffL, "mg_tensor_linear_bf16: grid too large (rows=%ld dim_out=%d)", rows, O);
    hipLaunchKernelGGL((linear_rows_bf16_kernel<WAVES, NI, YT>), dim3((unsigned)grid), dim3(64 * WAVES), 0, st, Wp,
                       plane_elems, w_rows, x, rows, I, O, bias, act, accumulate, y, tiles_n, total, out_T);
    return check_launch("mg_tensor_linear_bf16");
}

template <typename YT>
int dispatch(const __bf16* Wp, long plane_elems, int w_rows, const __bf16* x, long rows, int I, int O,
             const float* bias, int act, int accumulate, YT* y, int out_T, hipStream_t st) {
    const Shape sh = choose_shape(rows, O);
#define MG_BF16_LAUNCH(WV, N) \
    return launch<WV, N, YT>(Wp, plane_elems, w_rows, x, rows, I, O, bias, act, accumulate, y, out_T, st)
    if (sh.waves == 8) {
        if (sh.ni == 1) MG_BF16_LAUNCH(8, 1);
        if (sh.ni == 2) MG_BF16_LAUNCH(8, 2);
        if (sh.ni == 4) MG_BF16_LAUNCH(8, 4);
        MG_BF16_LAUNCH(8, 8);
    }
    if (sh.ni == 1) MG_BF16_LAUNCH(4, 1);
    if (sh.ni == 2) MG_BF16_LAUNCH(4, 2);
    if (sh.ni == 4) MG_BF16_LAUNCH(4, 4);
    MG_BF16_LAUNCH(4, 8);
#undef MG_BF16_LAUNCH
}

template <int NI>
int launch_rowsum(const __bf16* Wp, long plane_elems, int w_rows, const __bf16* x, long rows, int I, int O,
                  const float* bias, int act, __bf16* y, const RowSum& rs, hipStream_t st) {
    const long tiles_m = ceil_div(rows, 256);
    const int tiles_n = O / (32 * NI);
    const long total = tiles_m * tiles_n;
    const long grid = ceil_div(total, 8) * 8;
    MG_REQUIRE(grid <= 0x7fffffffL, "mg_tensor_linear_bf16_rowsum: grid too large");
    hipLaunchKernelGGL((linear_rows_bf16_kernel<8, NI, __bf16, true>), dim3((unsigned)grid), dim3(512), 0, st, Wp,
                       plane_elems, w_rows, x, rows, I, O, bias, act, 0, y, tiles_n, total, 1, rs);
    return check_launch("mg_tensor_linear_bf16_rowsum");
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_tensor_linear_bf16_rowsum_workspace_bytes(long rows, int dim_out, size_t* bytes) {
    MG_REQUIRE(bytes != nullptr && rows >= 0 && dim_out >= 0, "mg_tensor_linear_bf16_rowsum_workspace_bytes: bad argument");
    *bytes = (size_t)(2L * (ceil_div(rows, 32) + 1) * dim_out) * sizeof(float);
    return MG_OK;
}

int mg_tensor_linear_bf16_rowsum(const void* packed_W, const void* x, long rows, int dim_in, int dim_out,
                                 const float* bias, int act, const int* row_ptr, const int* seg, long n_out, float scale,
                                 void* workspace, void* y, float* out, mg_stream_t stream) {
    MG_REQUIRE(dim_out >= 128 && dim_out % 128 == 0, "mg_tensor_linear_bf16_rowsum: dim_out must be a multiple of 128 (got %d)", dim_out);
    MG_REQUIRE(dim_in > 0 && dim_in % 32 == 0, "mg_tensor_linear_bf16_rowsum: dim_in must be a multiple of 32 (got %d)", dim_in);
    MG_REQUIRE(rows >= 0 && n_out >= 0 && rows < (1L << 31) && n_out < (1L << 31), "mg_tensor_linear_bf16_rowsum: bad size");
    MG_REQUIRE(act >= 0 && act <= 2, "mg_tensor_linear_bf16_rowsum: unknown activation %d", act);
    if (n_out == 0) return MG_OK;
    MG_REQUIRE(packed_W && row_ptr && out && aligned16(packed_W) && aligned16(out) && (!bias || aligned16(bias)),
               "mg_tensor_linear_bf16_rowsum: null or unaligned operand");
    hipStream_t st = (hipStream_t)stream;
    const long n_blocks = ceil_div(rows, 32);
    if (rows > 0) {
        MG_REQUIRE(x && seg && workspace && aligned16(x) && aligned16(workspace) && (!y || aligned16(y)),
                   "mg_tensor_linear_bf16_rowsum: null or unaligned row operand");
        const int w_rows = (int)ceil_div(dim_out, 128) * 128;
        const long plane_elems = (long)w_rows * dim_in;
        RowSum rs{seg, static_cast<float*>(workspace), n_blocks, out, scale, y != nullptr};
        const int st_code = dim_out % 256 == 0
            ? launch_rowsum<8>(static_cast<const __bf16*>(packed_W), plane_elems, w_rows, static_cast<const __bf16*>(x),
                               rows, dim_in, dim_out, bias, act, static_cast<__bf16*>(y), rs, st)
            : launch_rowsum<4>(static_cast<const __bf16*>(packed_W), plane_elems, w_rows, static_cast<const __bf16*>(x),
                               rows, dim_in, dim_out, bias, act, static_cast<__bf16*>(y), rs, st);
        if (st_code) return st_code;
    }
    const long threads = n_out * (dim_out / 4);
    rowsum_finish_kernel<<<dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0, st>>>(
        row_ptr, n_out, n_blocks, dim_out, static_cast<const float*>(workspace), scale, out);
    return check_launch("rowsum_finish_kernel");
}

int mg_tensor_linear_bf16(const void* packed_W, const void* x, long rows, int dim_in, int dim_out, const float* bias,
                          int act, int accumulate, int out_comps, int y_is_bf16, void* y, mg_stream_t stream) {
    MG_REQUIRE(rows >= 0 && dim_in > 0 && dim_out >= 0, "mg_tensor_linear_bf16: bad size");
    MG_REQUIRE(dim_in % 32 == 0, "mg_tensor_linear_bf16: dim_in must be a multiple of 32 (got %d)", dim_in);
    MG_REQUIRE(act >= 0 && act <= 2, "mg_tensor_linear_bf16: unknown activation %d", act);
    MG_REQUIRE(out_comps == 1 || out_comps == 3 || out_comps == 9, "mg_tensor_linear_bf16: out_comps must be 1, 3 or 9");
    if (rows == 0 || dim_out == 0) return MG_OK;
    MG_REQUIRE(packed_W && x && y && aligned16(x) && aligned16(packed_W) && aligned16(y),
               "mg_tensor_linear_bf16: null or unaligned pointer");
    MG_REQUIRE(bias == nullptr || aligned16(bias), "mg_tensor_linear_bf16: bias must be 16-byte aligned");
    const int w_rows = (int)ceil_div(dim_out, 128) * 128;       // rows per plane in the packed format
    const long plane_elems = (long)w_rows * dim_in;
    hipStream_t st = (hipStream_t)stream;
    if (y_is_bf16)
        return dispatch<__bf16>(static_cast<const __bf16*>(packed_W), plane_elems, w_rows, static_cast<const __bf16*>(x),
                                rows, dim_in, dim_out, bias, act, accumulate, static_cast<__bf16*>(y), out_comps, st);
    return dispatch<float>(static_cast<const __bf16*>(packed_W), plane_elems, w_rows, static_cast<const __bf16*>(x), rows,
                           dim_in, dim_out, bias, act, accumulate, static_cast<float*>(y), out_comps, st);
}

}  // extern "C"
