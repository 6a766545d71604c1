// Tiled elementwise engine for per-(row,chan) tensor programs.
//
// Every operand is a dense array of n elements with T in {1,3,9} float
// components per element (component index fastest).  A workgroup of 256 lanes
// owns 256 consecutive elements.  Operands with T > 1 are moved between HBM
// and registers THROUGH LDS: the tile of an operand is one contiguous span of
// 256*T floats, so the HBM side is read/written with unit-stride dword (or
// 16-byte) accesses and the stride-T access happens in LDS, where an odd
// stride is bank-conflict free.  A lane reading its own 9 floats straight from
// HBM would touch 18 cache lines per wave instruction; this way each line is
// touched once.
//
// A program F provides
//   static constexpr int NIN, NOUT; static constexpr int in_T[NIN], out_T[NOUT];
//   static __device__ void compute(const float* in, float* out);   // packed registers
// Operands are processed in groups that fit the LDS budget of kBudget floats
// per element.
#pragma once
#include <hip/hip_runtime.h>
#include <type_traits>

namespace mg {
namespace ew {

constexpr int kTile = 256;    // elements per workgroup == lanes per workgroup
constexpr int kBudget = 27;   // LDS floats per element (27.6 KB per workgroup)

template <int N>
struct Plan {
    int off[N + 1];   // packed register offset of operand k
    int grp[N];       // LDS group of operand k (-1: T == 1, direct)
    int lds_off[N];   // float offset (per element) inside the group
    int ngroups;
    int lds_floats;   // largest group, floats per element
};

template <int N>
constexpr Plan<N> make_plan(const int (&T)[N]) {
    Plan<N> p{};
    int acc = 0, g = 0, used = 0, peak = 0;
    bool any = false;
    for (int k = 0; k < N; k++) {
        p.off[k] = acc;
        acc += T[k];
        if (T[k] == 1) {
            p.grp[k] = -1;
            p.lds_off[k] = 0;
        } else {
            if (used + T[k] > kBudget) { g++; used = 0; }
            p.grp[k] = g;
            p.lds_off[k] = used;
            used += T[k];
            if (used > peak) peak = used;
            any = true;
        }
    }
    p.off[N] = acc;
    p.ngroups = any ? g + 1 : 0;
    p.lds_floats = peak;
    return p;
}

template <int NIN, int NOUT>
struct Args {
    const float* in[NIN];
    float* out[NOUT];
    unsigned in_vec;   // bit k: operand k is 16-byte aligned
    unsigned out_vec;
    // Row indirection of inputs (all null / zero: none).  The elements are (row, channel) pairs, `chan` channels per
    // row, chan a multiple of kTile, so that a workgroup's elements lie in one row; input k with in_index[k] != null
    // holds in_rows[k] rows and the workgroup's row r reads its row in_index[k][r] (clamped into the operand): a gather
    // folded into the kernel.
    const int* in_index[NIN];
    long in_rows[NIN];
    int chan;
};

// span copy HBM -> LDS, `count` floats, both sides unit stride
__device__ inline void span_to_lds(const float* __restrict__ g, float* __restrict__ l, int count,
                                   bool vec, int tid) {
    if (vec) {
        const float4* g4 = reinterpret_cast<const float4*>(g);
        float4* l4 = reinterpret_cast<float4*>(l);
        for (int i = tid; i < count / 4; i += kTile) l4[i] = g4[i];
    } else {
        for (int i = tid; i < count; i += kTile) l[i] = g[i];
    }
}

__device__ inline void span_from_lds(float* __restrict__ g, const float* __restrict__ l, int count,
                                     bool vec, int tid) {
    if (vec) {
        float4* g4 = reinterpret_cast<float4*>(g);
        const float4* l4 = reinterpret_cast<const float4*>(l);
        for (int i = tid; i < count / 4; i += kTile) g4[i] = l4[i];
    } else {
        for (int i = tid; i < count; i += kTile) g[i] = l[i];
    }
}

template <int I, int N, class Fn>
__device__ __forceinline__ void static_for(Fn&& fn) {
    if constexpr (I < N) {
        fn(std::integral_constant<int, I>{});
        static_for<I + 1, N>(fn);
    }
}

template <class F>
__global__ void __launch_bounds__(kTile) kernel(Args<F::NIN, F::NOUT> a, long n) {
    constexpr Plan<F::NIN> pin = make_plan<F::NIN>(F::in_T);
    constexpr Plan<F::NOUT> pout = make_plan<F::NOUT>(F::out_T);
    constexpr int kLds = (pin.lds_floats > pout.lds_floats ? pin.lds_floats : pout.lds_floats);
    __shared__ __attribute__((aligned(16))) float lds[(kLds > 0 ? kLds : 1) * kTile];

    const int tid = threadIdx.x;
    const long base = (long)blockIdx.x * kTile;
    const long left = n - base;
    const int nvalid = left < kTile ? (int)left : kTile;
    const bool full = nvalid == kTile;
    const bool active = tid < nvalid;

    float in[pin.off[F::NIN]];
    float out[pout.off[F::NOUT]];

    // first element of this workgroup in input k (another row of the operand when the input is indexed)
    const long tile_row = a.chan > 0 ? base / a.chan : 0;
    const long tile_col = a.chan > 0 ? base - tile_row * a.chan : 0;
    auto in_base = [&](int k) -> long {
        if (a.in_index[k] == nullptr) return base;
        long r = a.in_index[k][tile_row];
        r = r < 0 ? 0 : (r >= a.in_rows[k] ? a.in_rows[k] - 1 : r);
        return r * a.chan + tile_col;
    };

    static_for<0, F::NIN>([&](auto K) {
        constexpr int k = decltype(K)::value;
        if constexpr (pin.grp[k] < 0) in[pin.off[k]] = active ? a.in[k][in_base(k) + tid] : 0.0f;
    });
    static_for<0, pin.ngroups>([&](auto G) {
        constexpr int g = decltype(G)::value;
        if constexpr (g > 0) __syncthreads();
        static_for<0, F::NIN>([&](auto K) {
            constexpr int k = decltype(K)::value;
            if constexpr (pin.grp[k] == g) {
                constexpr int T = F::in_T[k];
                span_to_lds(a.in[k] + in_base(k) * T, lds + pin.lds_off[k] * kTile, nvalid * T,
                            full && ((a.in_vec >> k) & 1u), tid);
            }
        });
        __syncthreads();
        static_for<0, F::NIN>([&](auto K) {
            constexpr int k = decltype(K)::value;
            if constexpr (pin.grp[k] == g) {
                constexpr int T = F::in_T[k];
                static_for<0, T>([&](auto C) {
                    constexpr int c = decltype(C)::value;
                    in[pin.off[k] + c] = active ? lds[pin.lds_off[k] * kTile + tid * T + c] : 0.0f;
                });
            }
        });
    });

    F::compute(in, out);

    static_for<0, F::NOUT>([&](auto K) {
        constexpr int k = decltype(K)::value;
        if constexpr (pout.grp[k] < 0) {
            if (active) a.out[k][base + tid] = out[pout.off[k]];
        }
    });
    static_for<0, pout.ngroups>([&](auto G) {
        constexpr int g = decltype(G)::value;
        __syncthreads();  // earlier users of the LDS buffer are done
        static_for<0, F::NOUT>([&](auto K) {
            constexpr int k = decltype(K)::value;
            if constexpr (pout.grp[k] == g) {
                constexpr int T = F::out_T[k];
                static_for<0, T>([&](auto C) {
                    constexpr int c = decltype(C)::value;
                    lds[pout.lds_off[k] * kTile + tid * T + c] = out[pout.off[k] + c];
                });
            }
        });
        __syncthreads();
        static_for<0, F::NOUT>([&](auto K) {
            constexpr int k = decltype(K)::value;
            if constexpr (pout.grp[k] == g) {
                constexpr int T = F::out_T[k];
                span_from_lds(a.out[k] + base * T, lds + pout.lds_off[k] * kTile, nvalid * T,
                              full && ((a.out_vec >> k) & 1u), tid);
            }
        });
    });
}

}  // namespace ew
}  // namespace mg
