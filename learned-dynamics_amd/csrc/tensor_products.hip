// Cartesian tensor products between rank-0/1/2 features, elementwise over
// (row, chan).  HBM-bound: 167 flop against 356 bytes per element for the full
// 13-product set, so all the work is in moving operands with unit-stride
// accesses (see elementwise.hpp).
//
// Index convention: contracted indices trail both operands; kept left indices
// come first in the output, then kept right indices; a rank-2 operand is the
// full 3x3 tensor stored row-major (xy -> 3x+y).
#include "common.hpp"
#include "elementwise.hpp"

namespace mg {
namespace {

// ---- forward primitives (label lro = ranks of left, right, output) ----------
__device__ __forceinline__ float dot3(const float* a, const float* b) {
    return a[0] * b[0] + a[1] * b[1] + a[2] * b[2];
}
__device__ __forceinline__ void cross3(const float* a, const float* b, float* o) {
    o[0] = a[1] * b[2] - a[2] * b[1];
    o[1] = a[2] * b[0] - a[0] * b[2];
    o[2] = a[0] * b[1] - a[1] * b[0];
}
__device__ __forceinline__ float p110(const float* l, const float* r) { return dot3(l, r); }
__device__ __forceinline__ float p220(const float* l, const float* r) {
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < 9; k++) s += l[k] * r[k];
    return s;
}
__device__ __forceinline__ void p011(float l, const float* r, float* y) {
#pragma unroll
    for (int x = 0; x < 3; x++) y[x] = l * r[x];
}
__device__ __forceinline__ void p101(const float* l, float r, float* y) {
#pragma unroll
    for (int x = 0; x < 3; x++) y[x] = l[x] * r;
}
// y_y = sum_x l_x r_yx
__device__ __forceinline__ void p121(const float* l, const float* r, float* y) {
#pragma unroll
    for (int j = 0; j < 3; j++) y[j] = dot3(l, r + 3 * j);
}
// y_x = sum_y l_xy r_y
__device__ __forceinline__ void p211(const float* l, const float* r, float* y) {
#pragma unroll
    for (int i = 0; i < 3; i++) y[i] = dot3(l + 3 * i, r);
}
__device__ __forceinline__ void p022(float l, const float* r, float* y) {
#pragma unroll
    for (int k = 0; k < 9; k++) y[k] = l * r[k];
}
__device__ __forceinline__ void p202(const float* l, float r, float* y) {
#pragma unroll
    for (int k = 0; k < 9; k++) y[k] = l[k] * r;
}
__device__ __forceinline__ void p112(const float* l, const float* r, float* y) {
#pragma unroll
    for (int i = 0; i < 3; i++)
#pragma unroll
        for (int j = 0; j < 3; j++) y[3 * i + j] = l[i] * r[j];
}
// y_xz = sum_y l_xy r_zy
__device__ __forceinline__ void p222(const float* l, const float* r, float* y) {
#pragma unroll
    for (int i = 0; i < 3; i++)
#pragma unroll
        for (int j = 0; j < 3; j++) y[3 * i + j] = dot3(l + 3 * i, r + 3 * j);
}
__device__ __forceinline__ void p111(const float* l, const float* r, float* y) { cross3(l, r, y); }
// y_xw = sum_yz eps_yzw l_xy r_z : row x of the result is l[x,:] cross r
__device__ __forceinline__ void p212(const float* l, const float* r, float* y) {
#pragma unroll
    for (int i = 0; i < 3; i++) cross3(l + 3 * i, r, y + 3 * i);
}

// ---- programs -----------------------------------------------------------------
struct BeeFwd {
    static constexpr int NIN = 6, NOUT = 13;
    static constexpr int in_T[NIN] = {1, 3, 9, 1, 3, 9};
    static constexpr int out_T[NOUT] = {1, 1, 1, 3, 3, 3, 3, 9, 9, 9, 9, 3, 9};
    static __device__ __forceinline__ void compute(const float* in, float* o) {
        const float l0 = in[0], *l1 = in + 1, *l2 = in + 4;
        const float r0 = in[13], *r1 = in + 14, *r2 = in + 17;
        o[0] = l0 * r0;
        o[1] = p110(l1, r1);
        o[2] = p220(l2, r2);
        p011(l0, r1, o + 3);
        p101(l1, r0, o + 6);
        p121(l1, r2, o + 9);
        p211(l2, r1, o + 12);
        p022(l0, r2, o + 15);
        p202(l2, r0, o + 24);
        p112(l1, r1, o + 33);
        p222(l2, r2, o + 42);
        p111(l1, r1, o + 51);
        p212(l2, r1, o + 54);
    }
};

// dy packed in the forward output order:
// 000@0 110@1 220@2 011@3 101@6 121@9 211@12 022@15 202@24 112@33 222@42 111@51 212@54
template <int SIDE>
struct BeeBwd {
    static constexpr int NIN = 16, NOUT = 3;
    static constexpr int in_T[NIN] = {1, 3, 9, 1, 1, 1, 3, 3, 3, 3, 9, 9, 9, 9, 3, 9};
    static constexpr int out_T[NOUT] = {1, 3, 9};
    static __device__ __forceinline__ void compute(const float* in, float* o) {
        const float o0 = in[0], *o1 = in + 1, *o2 = in + 4;  // the other side's operands
        const float* dy = in + 13;
        float* d0 = o;
        float* d1 = o + 1;
        float* d2 = o + 4;
        if constexpr (SIDE == 0) {
            // gradients of the LEFT operands; o* are the right operands r
            d0[0] = dy[0] * o0 + dot3(dy + 3, o1) + p220(dy + 15, o2);
            float c[3];
            cross3(o1, dy + 51, c);  // 111: dl = r x dy
#pragma unroll
            for (int x = 0; x < 3; x++) {
                float s = dy[1] * o1[x] + dy[6 + x] * o0 + c[x];
#pragma unroll
                for (int y = 0; y < 3; y++) s += dy[9 + y] * o2[3 * y + x];   // 121
                s += dot3(dy + 33 + 3 * x, o1);                               // 112
                d1[x] = s;
            }
#pragma unroll
            for (int x = 0; x < 3; x++) {
                float c2[3];
                cross3(o1, dy + 54 + 3 * x, c2);  // 212: dl2[x,:] = r1 x dy212[x,:]
#pragma unroll
                for (int y = 0; y < 3; y++) {
                    float s = dy[2] * o2[3 * x + y] + dy[12 + x] * o1[y] + dy[24 + 3 * x + y] * o0 + c2[y];
#pragma unroll
                    for (int z = 0; z < 3; z++) s += dy[42 + 3 * x + z] * o2[3 * z + y];  // 222
                    d2[3 * x + y] = s;
                }
            }
        } else {
            // gradients of the RIGHT operands; o* are the left operands l
            d0[0] = dy[0] * o0 + dot3(dy + 6, o1) + p220(dy + 24, o2);
            float c[3];
            cross3(dy + 51, o1, c);  // 111: dr = dy x l
            float c212[3] = {0.f, 0.f, 0.f};
#pragma unroll
            for (int x = 0; x < 3; x++) {
                float t[3];
                cross3(dy + 54 + 3 * x, o2 + 3 * x, t);  // 212: sum_x dy212[x,:] x l2[x,:]
                c212[0] += t[0]; c212[1] += t[1]; c212[2] += t[2];
            }
#pragma unroll
            for (int y = 0; y < 3; y++) {
                float s = dy[1] * o1[y] + dy[3 + y] * o0 + c[y] + c212[y];
#pragma unroll
                for (int x = 0; x < 3; x++) {
                    s += dy[12 + x] * o2[3 * x + y];   // 211
                    s += dy[33 + 3 * x + y] * o1[x];   // 112
                }
                d1[y] = s;
            }
#pragma unroll
            for (int z = 0; z < 3; z++)
#pragma unroll
                for (int y = 0; y < 3; y++) {
                    // r2 component [z,y]
                    float s = dy[2] * o2[3 * z + y] + dy[9 + z] * o1[y] + dy[15 + 3 * z + y] * o0;
#pragma unroll
                    for (int x = 0; x < 3; x++) s += dy[42 + 3 * x + z] * o2[3 * x + y];  // 222
                    d2[3 * z + y] = s;
                }
        }
    }
};

struct Cow0Fwd {
    static constexpr int NIN = 4, NOUT = 2;
    static constexpr int in_T[NIN] = {1, 3, 1, 3};
    static constexpr int out_T[NOUT] = {1, 1};
    static __device__ __forceinline__ void compute(const float* in, float* o) {
        o[0] = in[0] * in[4];
        o[1] = p110(in + 1, in + 5);
    }
};
struct Cow1Fwd {
    static constexpr int NIN = 4, NOUT = 3;
    static constexpr int in_T[NIN] = {1, 3, 1, 3};
    static constexpr int out_T[NOUT] = {3, 3, 3};
    static __device__ __forceinline__ void compute(const float* in, float* o) {
        p011(in[0], in + 5, o);
        p101(in + 1, in[4], o + 3);
        p111(in + 1, in + 5, o + 6);
    }
};
// in: o_0, o_1, dy_000, dy_110 -> d_0, d_1 (the two products are symmetric in l and r)
struct Cow0Bwd {
    static constexpr int NIN = 4, NOUT = 2;
    static constexpr int in_T[NIN] = {1, 3, 1, 1};
    static constexpr int out_T[NOUT] = {1, 3};
    static __device__ __forceinline__ void compute(const float* in, float* o) {
        o[0] = in[4] * in[0];
#pragma unroll
        for (int x = 0; x < 3; x++) o[1 + x] = in[5] * in[1 + x];
    }
};
// in: o_0, o_1, dy_011, dy_101, dy_111 -> d_0, d_1
template <int SIDE>
struct Cow1Bwd {
    static constexpr int NIN = 5, NOUT = 2;
    static constexpr int in_T[NIN] = {1, 3, 3, 3, 3};
    static constexpr int out_T[NOUT] = {1, 3};
    static __device__ __forceinline__ void compute(const float* in, float* o) {
        const float o0 = in[0], *o1 = in + 1, *dy011 = in + 4, *dy101 = in + 7, *dy111 = in + 10;
        float c[3];
        if constexpr (SIDE == 0) {  // dl: o = r
            o[0] = dot3(dy011, o1);
            cross3(o1, dy111, c);
#pragma unroll
            for (int x = 0; x < 3; x++) o[1 + x] = dy101[x] * o0 + c[x];
        } else {                    // dr: o = l
            o[0] = dot3(dy101, o1);
            cross3(dy111, o1, c);
#pragma unroll
            for (int x = 0; x < 3; x++) o[1 + x] = dy011[x] * o0 + c[x];
        }
    }
};

constexpr int pow3(int k) { return k == 0 ? 1 : (k == 1 ? 3 : 9); }

template <int L, int R, int O>
struct Bare {
    static constexpr int NIN = 2, NOUT = 1;
    static constexpr int in_T[NIN] = {pow3(L), pow3(R)};
    static constexpr int out_T[NOUT] = {pow3(O)};
    static __device__ __forceinline__ void compute(const float* in, float* o) {
        const float* l = in;
        const float* r = in + pow3(L);
        if constexpr (L == 0 && R == 0 && O == 0) o[0] = l[0] * r[0];
        else if constexpr (L == 1 && R == 1 && O == 0) o[0] = p110(l, r);
        else if constexpr (L == 2 && R == 2 && O == 0) o[0] = p220(l, r);
        else if constexpr (L == 0 && R == 1 && O == 1) p011(l[0], r, o);
        else if constexpr (L == 1 && R == 0 && O == 1) p101(l, r[0], o);
        else if constexpr (L == 1 && R == 2 && O == 1) p121(l, r, o);
        else if constexpr (L == 2 && R == 1 && O == 1) p211(l, r, o);
        else if constexpr (L == 0 && R == 2 && O == 2) p022(l[0], r, o);
        else if constexpr (L == 2 && R == 0 && O == 2) p202(l, r[0], o);
        else if constexpr (L == 1 && R == 1 && O == 2) p112(l, r, o);
        else if constexpr (L == 2 && R == 2 && O == 2) p222(l, r, o);
    }
};

// a (scalar), v_l, v_r (vectors) -> v_l.v_r, a v_r, v_l (x) v_r
struct AvdTrio {
    static constexpr int NIN = 3, NOUT = 3;
    static constexpr int in_T[NIN] = {1, 3, 3};
    static constexpr int out_T[NOUT] = {1, 3, 9};
    static __device__ __forceinline__ void compute(const float* in, float* o) {
        o[0] = p110(in + 1, in + 4);
        p011(in[0], in + 4, o + 1);
        p112(in + 1, in + 4, o + 4);
    }
};

// in_index / in_rows (or null): row indirection per input (ew::Args), for `chan` channels per row
template <class F>
int launch(const float* const* in, float* const* out, long n, hipStream_t stream, const char* name,
           const int* const* in_index = nullptr, const long* in_rows = nullptr, int chan = 0) {
    ew::Args<F::NIN, F::NOUT> a;
    a.in_vec = 0;
    a.out_vec = 0;
    a.chan = 0;
    for (int k = 0; k < F::NIN; k++) {
        MG_REQUIRE(in[k] != nullptr, "%s: input %d is null", name, k);
        a.in[k] = in[k];
        if (aligned16(in[k])) a.in_vec |= 1u << k;
        a.in_index[k] = in_index ? in_index[k] : nullptr;
        a.in_rows[k] = in_index && in_index[k] ? in_rows[k] : 0;
        if (a.in_index[k]) {
            MG_REQUIRE(chan > 0 && chan % ew::kTile == 0, "%s: indexed operands need a channel count that is a multiple of %d",
                       name, ew::kTile);
            MG_REQUIRE(a.in_rows[k] > 0, "%s: indexed input %d has no rows", name, k);
            a.chan = chan;
        }
    }
    for (int k = 0; k < F::NOUT; k++) {
        MG_REQUIRE(out[k] != nullptr, "%s: output %d is null", name, k);
        a.out[k] = out[k];
        if (aligned16(out[k])) a.out_vec |= 1u << k;
    }
    const long blocks = ceil_div(n, ew::kTile);
    MG_REQUIRE(blocks <= 0x7fffffffL, "%s: rows*chan = %ld too large", name, n);
    hipLaunchKernelGGL(ew::kernel<F>, dim3((unsigned)blocks), dim3(ew::kTile), 0, stream, a, n);
    return check_launch(name);
}

int check_sizes(long rows, int chan, const char* name) {
    MG_REQUIRE(rows >= 0 && chan >= 0, "%s: negative size (rows=%ld chan=%d)", name, rows, chan);
    return MG_OK;
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_bee_fwd(const float* l_0, const float* l_1, const float* l_2, const float* r_0,
               const float* r_1, const float* r_2, long rows, int chan, float* const y[13],
               mg_stream_t stream) {
    if (int s = check_sizes(rows, chan, "mg_bee_fwd")) return s;
    if (rows == 0 || chan == 0) return MG_OK;
    MG_REQUIRE(y != nullptr, "mg_bee_fwd: y is null");
    const float* in[6] = {l_0, l_1, l_2, r_0, r_1, r_2};
    return launch<BeeFwd>(in, y, rows * chan, (hipStream_t)stream, "mg_bee_fwd");
}

int mg_bee_bwd(int side, const float* o_0, const float* o_1, const float* o_2,
               const float* const dy[13], long rows, int chan, float* d_0, float* d_1, float* d_2,
               mg_stream_t stream) {
    if (int s = check_sizes(rows, chan, "mg_bee_bwd")) return s;
    MG_REQUIRE(side == 0 || side == 1, "mg_bee_bwd: side must be 0 (left) or 1 (right)");
    if (rows == 0 || chan == 0) return MG_OK;
    MG_REQUIRE(dy != nullptr, "mg_bee_bwd: dy is null");
    const float* in[16] = {o_0, o_1, o_2};
    for (int k = 0; k < 13; k++) in[3 + k] = dy[k];
    float* out[3] = {d_0, d_1, d_2};
    if (side == 0) return launch<BeeBwd<0>>(in, out, rows * chan, (hipStream_t)stream, "mg_bee_bwd(left)");
    return launch<BeeBwd<1>>(in, out, rows * chan, (hipStream_t)stream, "mg_bee_bwd(right)");
}

int mg_bee_indexed_supported(int chan) { return chan > 0 && chan % ew::kTile == 0; }

int mg_bee_fwd_indexed(const float* l_0, const float* l_1, const float* l_2, const int* l_index, long l_rows,
                       const float* r_0, const float* r_1, const float* r_2, long rows, int chan, float* const y[13],
                       mg_stream_t stream) {
    if (int s = check_sizes(rows, chan, "mg_bee_fwd_indexed")) return s;
    if (rows == 0 || chan == 0) return MG_OK;
    MG_REQUIRE(y != nullptr && l_index != nullptr, "mg_bee_fwd_indexed: null pointer");
    const float* in[6] = {l_0, l_1, l_2, r_0, r_1, r_2};
    const int* index[6] = {l_index, l_index, l_index, nullptr, nullptr, nullptr};
    const long n_rows[6] = {l_rows, l_rows, l_rows, 0, 0, 0};
    return launch<BeeFwd>(in, y, rows * chan, (hipStream_t)stream, "mg_bee_fwd_indexed", index, n_rows, chan);
}

int mg_bee_bwd_indexed(int side, const float* o_0, const float* o_1, const float* o_2, const int* o_index, long o_rows,
                       const float* const dy[13], const int* dy_index, long dy_rows, unsigned dy_indexed, long rows,
                       int chan, float* d_0, float* d_1, float* d_2, mg_stream_t stream) {
    if (int s = check_sizes(rows, chan, "mg_bee_bwd_indexed")) return s;
    MG_REQUIRE(side == 0 || side == 1, "mg_bee_bwd_indexed: side must be 0 (left) or 1 (right)");
    if (rows == 0 || chan == 0) return MG_OK;
    MG_REQUIRE(dy != nullptr, "mg_bee_bwd_indexed: dy is null");
    MG_REQUIRE(dy_indexed == 0 || dy_index != nullptr, "mg_bee_bwd_indexed: dy_indexed without an index");
    const float* in[16] = {o_0, o_1, o_2};
    const int* index[16] = {o_index, o_index, o_index};
    long n_rows[16] = {o_rows, o_rows, o_rows};
    for (int k = 0; k < 13; k++) {
        in[3 + k] = dy[k];
        const bool indexed = (dy_indexed >> k) & 1u;
        index[3 + k] = indexed ? dy_index : nullptr;
        n_rows[3 + k] = indexed ? dy_rows : 0;
    }
    float* out[3] = {d_0, d_1, d_2};
    hipStream_t st = (hipStream_t)stream;
    if (side == 0) return launch<BeeBwd<0>>(in, out, rows * chan, st, "mg_bee_bwd_indexed(left)", index, n_rows, chan);
    return launch<BeeBwd<1>>(in, out, rows * chan, st, "mg_bee_bwd_indexed(right)", index, n_rows, chan);
}

int mg_cow_o0_fwd(const float* l_0, const float* l_1, const float* r_0, const float* r_1, long rows,
                  int chan, float* y_000, float* y_110, mg_stream_t stream) {
    if (int s = check_sizes(rows, chan, "mg_cow_o0_fwd")) return s;
    if (rows == 0 || chan == 0) return MG_OK;
    const float* in[4] = {l_0, l_1, r_0, r_1};
    float* out[2] = {y_000, y_110};
    return launch<Cow0Fwd>(in, out, rows * chan, (hipStream_t)stream, "mg_cow_o0_fwd");
}

int mg_cow_o1_fwd(const float* l_0, const float* l_1, const float* r_0, const float* r_1, long rows,
                  int chan, float* y_011, float* y_101, float* y_111, mg_stream_t stream) {
    if (int s = check_sizes(rows, chan, "mg_cow_o1_fwd")) return s;
    if (rows == 0 || chan == 0) return MG_OK;
    const float* in[4] = {l_0, l_1, r_0, r_1};
    float* out[3] = {y_011, y_101, y_111};
    return launch<Cow1Fwd>(in, out, rows * chan, (hipStream_t)stream, "mg_cow_o1_fwd");
}

int mg_cow_o0_bwd(int side, const float* o_0, const float* o_1, const float* dy_000,
                  const float* dy_110, long rows, int chan, float* d_0, float* d_1,
                  mg_stream_t stream) {
    if (int s = check_sizes(rows, chan, "mg_cow_o0_bwd")) return s;
    MG_REQUIRE(side == 0 || side == 1, "mg_cow_o0_bwd: side must be 0 (left) or 1 (right)");
    if (rows == 0 || chan == 0) return MG_OK;
    const float* in[4] = {o_0, o_1, dy_000, dy_110};
    float* out[2] = {d_0, d_1};
    return launch<Cow0Bwd>(in, out, rows * chan, (hipStream_t)stream, "mg_cow_o0_bwd");
}

int mg_cow_o1_bwd(int side, const float* o_0, const float* o_1, const float* dy_011,
                  const float* dy_101, const float* dy_111, long rows, int chan, float* d_0,
                  float* d_1, mg_stream_t stream) {
    if (int s = check_sizes(rows, chan, "mg_cow_o1_bwd")) return s;
    MG_REQUIRE(side == 0 || side == 1, "mg_cow_o1_bwd: side must be 0 (left) or 1 (right)");
    if (rows == 0 || chan == 0) return MG_OK;
    const float* in[5] = {o_0, o_1, dy_011, dy_101, dy_111};
    float* out[2] = {d_0, d_1};
    if (side == 0) return launch<Cow1Bwd<0>>(in, out, rows * chan, (hipStream_t)stream, "mg_cow_o1_bwd(left)");
    return launch<Cow1Bwd<1>>(in, out, rows * chan, (hipStream_t)stream, "mg_cow_o1_bwd(right)");
}

int mg_tensor_prod_bare(int inds_l, int inds_r, int inds_o, const float* x_l, const float* x_r,
                        long rows, int chan, float* y, mg_stream_t stream) {
    if (int s = check_sizes(rows, chan, "mg_tensor_prod_bare")) return s;
    if (inds_l < 0 || inds_r < 0 || inds_o < 0 || inds_l > 2 || inds_r > 2 || inds_o > 2)
        return fail(MG_ERR_UNSUPPORTED, "mg_tensor_prod_bare: ranks (%d,%d,%d) above 2 are not supported",
                    inds_l, inds_r, inds_o);
    const int twice = inds_l + inds_r - inds_o;
    MG_REQUIRE(twice % 2 == 0, "parity mismatch");
    const int contracts = twice / 2;
    MG_REQUIRE(contracts >= 0 && contracts <= (inds_l < inds_r ? inds_l : inds_r),
               "%d contractions is out of range for %d, %d index tensors", contracts, inds_l, inds_r);
    if (rows == 0 || chan == 0) return MG_OK;
    const float* in[2] = {x_l, x_r};
    float* out[1] = {y};
    const long n = rows * chan;
    hipStream_t st = (hipStream_t)stream;
    const int key = inds_l * 100 + inds_r * 10 + inds_o;
    switch (key) {
        case 0:   return launch<Bare<0, 0, 0>>(in, out, n, st, "tensor_prod_bare(000)");
        case 110: return launch<Bare<1, 1, 0>>(in, out, n, st, "tensor_prod_bare(110)");
        case 220: return launch<Bare<2, 2, 0>>(in, out, n, st, "tensor_prod_bare(220)");
        case 11:  return launch<Bare<0, 1, 1>>(in, out, n, st, "tensor_prod_bare(011)");
        case 101: return launch<Bare<1, 0, 1>>(in, out, n, st, "tensor_prod_bare(101)");
        case 121: return launch<Bare<1, 2, 1>>(in, out, n, st, "tensor_prod_bare(121)");
        case 211: return launch<Bare<2, 1, 1>>(in, out, n, st, "tensor_prod_bare(211)");
        case 22:  return launch<Bare<0, 2, 2>>(in, out, n, st, "tensor_prod_bare(022)");
        case 202: return launch<Bare<2, 0, 2>>(in, out, n, st, "tensor_prod_bare(202)");
        case 112: return launch<Bare<1, 1, 2>>(in, out, n, st, "tensor_prod_bare(112)");
        case 222: return launch<Bare<2, 2, 2>>(in, out, n, st, "tensor_prod_bare(222)");
    }
    return fail(MG_ERR_UNSUPPORTED, "mg_tensor_prod_bare: no product for ranks (%d,%d,%d)", inds_l, inds_r, inds_o);
}

int mg_tensor_prods_avd(const float* a, const float* v_l, const float* v_r, long rows, int chan,
                        float* y_110, float* y_011, float* y_112, mg_stream_t stream) {
    if (int s = check_sizes(rows, chan, "mg_tensor_prods_avd")) return s;
    if (rows == 0 || chan == 0) return MG_OK;
    const float* in[3] = {a, v_l, v_r};
    float* out[3] = {y_110, y_011, y_112};
    return launch<AvdTrio>(in, out, rows * chan, (hipStream_t)stream, "mg_tensor_prods_avd");
}

}  // extern "C"
