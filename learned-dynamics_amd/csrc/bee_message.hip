// Rank-0/1/2 ("a/v/d") message passing with the 13 Cartesian products, fused
// over CSR rows.
//
// For edge e = (i <- j): phi_a = lin_enc(radial_encode_8(r_ij)) (chan),
// rh = s / sqrt(1 + |s|^2) with s = r_ij * 7 / r0, phi_v = phi_a (x) rh,
// phi_d = phi_a (x) rh (x) rh; left operands are the node features
// l_k = (L_k x_k)[j]; the 13 products p_lab = prod_lab(l, phi) follow.
// Because every right operand is phi_a[c] times a per-edge geometric factor, each
// product is phi_a[c] * g_lab(l[c], rh): nothing of size E x chan x 3 x 3 exists.
//
// What leaves the kernel:
//   P0 (E, 3, chan)      the three scalar products per edge (they feed a per-edge
//                        MLP, which does not commute with the sum over edges)
//   S1 (N, 3, 5, chan)   sum over the edges of node i of the five vector products
//   S2 (N, 9, 5, chan)   ... of the five rank-2 products
// The bias-free output linears Y_lab commute with the sum over edges, so they are
// applied to S1/S2 on N rows afterwards; the (comp, label, chan) order makes
// each of those one plain GEMM with K = 5*chan.
//
// With Y2F the rank-2 sums do not leave the kernel either: the four waves of a workgroup hold the sums of
// 4 / chunks whole nodes, the bias-free output linear of the rank-2 channel (K = 5 chan, dim_d <= 16 outputs) is
// applied to them on the fp32 matrix cores (v_mfma_f32_16x16x4_f32: rows = the 9 components, 80 steps per wave),
// the waves' partial results are summed through LDS, and (node, dim_d, 9) is stored instead of (node, 9, 5, chan):
// 45 chan floats per node less to write, the same again less to read, and one GEMM launch less.
//
// Node features are read in component-major layout (node, comp, chan): the 13
// gathers of a wave are 13 unit-stride 256-byte reads.  A lane owns one channel
// and keeps its 60 running sums in registers; rows are summed in edge order.
#include "common.hpp"
#include "rank2_linear.hpp"
#include <type_traits>

namespace mg {
namespace {

struct Jacobi8 {
    double a[8][9];   // coefficient of z^j in the i-th shifted Jacobi(1,0) polynomial
};

// binomial coefficients as doubles (exact for the sizes used here)
double binom(int n, int k) {
    if (k < 0 || k > n) return 0.0;
    double r = 1.0;
    for (int i = 1; i <= k; i++) r = r * (n - k + i) / i;
    return r;
}

// P_n^{(1,0)}(2x-1) = sum_s C(n+1, n-s) C(n, s) (x-1)^s x^(n-s)
Jacobi8 jacobi_table() {
    Jacobi8 t{};
    for (int n = 0; n < 8; n++)
        for (int s = 0; s <= n; s++) {
            const double w = binom(n + 1, n - s) * binom(n, s);
            for (int k = 0; k <= s; k++)
                t.a[n][k + n - s] += w * binom(s, k) * (((s - k) & 1) ? -1.0 : 1.0);
        }
    return t;
}

// enc (E,8): radial_encode_8; rhat (E,3): tens_sigmoid(1, r * 7 / r0).
// The polynomial is evaluated in fp64: its monomial form has alternating
// coefficients up to ~1e5, so an fp32 evaluation carries ~1e-3 of rounding noise.
__global__ void __launch_bounds__(256) bee_geometry_kernel(const float* __restrict__ r_ij, long E, float r0,
                                                           float scale, Jacobi8 jac, float* __restrict__ enc,
                                                           float* __restrict__ rhat) {
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    const float x = r_ij[3 * e], y = r_ij[3 * e + 1], z = r_ij[3 * e + 2];
    const float d = sqrtf(x * x + y * y + z * z);
    const float zz = d / r0;
    const double zd = (double)zz;
    const float cut = fmaxf(1.0f - zz, 0.0f);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        double acc = jac.a[i][8];
#pragma unroll
        for (int j = 7; j >= 0; j--) acc = acc * zd + jac.a[i][j];
        enc[8 * e + i] = (float)(acc * (double)cut);
    }
    const float sx = x * scale, sy = y * scale, sz = z * scale;
    const float inv = 1.0f / sqrtf(1.0f + (sx * sx + sy * sy + sz * sz));
    rhat[3 * e] = sx * inv;
    rhat[3 * e + 1] = sy * inv;
    rhat[3 * e + 2] = sz * inv;
}

__device__ __forceinline__ void cross3(const float* a, const float* b, float* o) {
    o[0] = a[1] * b[2] - a[2] * b[1];
    o[1] = a[2] * b[0] - a[0] * b[2];
    o[2] = a[0] * b[1] - a[1] * b[0];
}

// max over the wave of non-negative values, valid in lane 63: six cross-lane VALU moves (shifts within
// rows of 16 lanes, then row broadcasts), no LDS traffic
__device__ __forceinline__ float wave_max_nonneg_last_lane(float v) {
    auto step = [](float x, auto ctrl, auto row_mask) {
        const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(x), decltype(ctrl)::value,
                                                      decltype(row_mask)::value, 0xf, false);
        return fmaxf(x, __int_as_float(moved));
    };
    v = step(v, std::integral_constant<int, 0x111>{}, std::integral_constant<int, 0xf>{});   // row_shr:1
    v = step(v, std::integral_constant<int, 0x112>{}, std::integral_constant<int, 0xf>{});   // row_shr:2
    v = step(v, std::integral_constant<int, 0x114>{}, std::integral_constant<int, 0xf>{});   // row_shr:4
    v = step(v, std::integral_constant<int, 0x118>{}, std::integral_constant<int, 0xf>{});   // row_shr:8
    v = step(v, std::integral_constant<int, 0x142>{}, std::integral_constant<int, 0xa>{});   // row_bcast:15
    v = step(v, std::integral_constant<int, 0x143>{}, std::integral_constant<int, 0xc>{});   // row_bcast:31
    return v;
}

__device__ __forceinline__ long uniform(long v) {
    // the value is the same in every lane: keep it in scalar registers
    const int lo = __builtin_amdgcn_readfirstlane((int)(v & 0xffffffffL));
    const int hi = __builtin_amdgcn_readfirstlane((int)(v >> 32));
    return ((long)hi << 32) | (unsigned)lo;
}

// Gathers of node rows go through buffer loads: the row's byte offset is uniform (scalar offset operand), the lane's
// channel offset a constant vector register, so a gather needs no vector address arithmetic at all (with global
// loads every one of the 13 gathers of an edge built its own 64-bit per-lane address: a tenth of the loop).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t node_rows(const void* base, long bytes) {
    const unsigned n = bytes > 0xffffffffL ? 0xffffffffu : (unsigned)bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)n, 0x00020000);
}
__device__ __forceinline__ float gather_row(__amdgpu_buffer_rsrc_t r, unsigned lane_bytes, unsigned row_bytes, float) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)lane_bytes, (int)row_bytes, 0));
}
__device__ __forceinline__ __bf16 gather_row(__amdgpu_buffer_rsrc_t r, unsigned lane_bytes, unsigned row_bytes, __bf16) {
    return __builtin_bit_cast(__bf16, __builtin_amdgcn_raw_buffer_load_b16(r, (int)lane_bytes, (int)row_bytes, 0));
}

// T: storage type of the node features and of the outputs (float, or __bf16 with fp32 arithmetic)
// PIPE: keep one edge of operands in flight ahead of the one being consumed (pays on long rows)
// Y2F: the rank-2 output linear is applied here (float storage, chan % 64 == 0, 1, 2 or 4 chunks, dim_d <= 16):
// y2_packed as written by pack_rank2_weight_kernel, out_d (nodes, dim_d, 9); S2 is not touched
template <typename T, bool PIPE, bool Y2F>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 4)))
bee_message_kernel(const int* __restrict__ row_ptr, const int* __restrict__ dst, const int* __restrict__ order,
                   long n_nodes, const float* __restrict__ rhat, const float* __restrict__ enc,
                   const T* __restrict__ La, const T* __restrict__ Lv, const T* __restrict__ Ld, int chan,
                   const float* __restrict__ enc_W, const float* __restrict__ enc_b, T* __restrict__ P0,
                   T* __restrict__ S1, T* __restrict__ S2, float* __restrict__ node_max,
                   float* __restrict__ edge_max, const float* __restrict__ y2_packed, int dim_d,
                   float* __restrict__ out_d, int out_d_accumulate) {
    static_assert(!Y2F || std::is_same<T, float>::value, "the fused output linear is for float storage");
    const int lane = threadIdx.x & (kWave - 1);
    const int chunks = (chan + kWave - 1) / kWave;
    const long items = n_nodes * chunks;
    const long a_bytes = n_nodes * chan * (long)sizeof(T);
    const __amdgpu_buffer_rsrc_t rs_a = node_rows(La, a_bytes), rs_v = node_rows(Lv, 3 * a_bytes), rs_d = node_rows(Ld, 9 * a_bytes);
    // Workgroup ids go round-robin over the 8 XCDs and an XCD starts its workgroups in id order as slots free up:
    // XCD x takes the x-th eighth of the items and workgroup (id >> 3) of it the four items 4 (id >> 3) .. + 3, one
    // per wave.  The waves in flight on an XCD are then a window of consecutive nodes of the processing order (cell
    // order) that slides forward, and the gathers of neighbouring atoms, which ask for the same rows, come close
    // enough in time to meet in the L2.  A persistent grid whose waves stride over the items put a different
    // system's nodes into flight at every trip: 2.66 ms against 2.37 ms at 32 x 2048 atoms, 256 channels, and 5.26
    // against 4.44 ms at 65536 atoms with 90 neighbours, 128 channels.  (Giving each XCD one 64-channel chunk, so
    // that its L2 sees a quarter of each row, was measured with both grids and is slower by 5 %.)
    // Y2F: a workgroup's four items must be whole nodes, and its four waves must make the same trips (barriers)
    const long per_xcd = Y2F ? (((items + 7) / 8 + 3) & ~3L) : (items + 7) / 8;
    const int xcd = blockIdx.x & 7;
    const long waves_per_xcd = (long)(gridDim.x >> 3) * (blockDim.x / kWave);
    const long wave_local = (long)(blockIdx.x >> 3) * (blockDim.x / kWave) + threadIdx.x / kWave;

    for (long item_local = wave_local; item_local < per_xcd; item_local += waves_per_xcd) {
        long item = uniform(xcd * per_xcd + item_local);
        const bool valid = item < items;                       // uniform over the wave
        if constexpr (Y2F) {
            item = valid ? item : items - 1;                   // a wave without an item still meets the barriers
        } else {
            if (!valid) break;
        }
        const long k_node = item / chunks;
        const int chunk = (int)(item - k_node * chunks);
        const int c = chunk * kWave + lane;
        const bool active = c < chan;
        const int cc = active ? c : chan - 1;   // inactive lanes shadow a valid channel, stores are masked
        const long node = order ? (long)order[k_node] : k_node;
        const long lo = valid ? row_ptr[node] : 0, hi = valid ? row_ptr[node + 1] : 0;

        float w[8];
#pragma unroll
        for (int m = 0; m < 8; m++) w[m] = enc_W[cc * 8 + m];
        const float bias = enc_b[cc];

        float s1[15], s2[45];
#pragma unroll
        for (int k = 0; k < 15; k++) s1[k] = 0.f;
#pragma unroll
        for (int k = 0; k < 45; k++) s2[k] = 0.f;

        // Software pipeline: the 13 gathered rows, the encoding and the direction of edge e + 1 are
        // requested before edge e is consumed (the gathers are L2 / fabric latency, and a wave has
        // nothing else to do while it waits), and dst of edge e + 2 one step earlier still.  The
        // look-ahead indices are clamped to the row, so no load is predicated.
        struct EdgeOps {
            T l0, l1[3], l2[9];
            float en[8], rh[3];
        };
        const unsigned lane_off = (unsigned)cc;   // rows are addressed as (uniform base) + 32-bit lane offset
        const unsigned lane_bytes = lane_off * (unsigned)sizeof(T);
        const unsigned row_bytes = (unsigned)chan * (unsigned)sizeof(T);
        auto fetch = [&](EdgeOps& o, long e, long j) {
            const unsigned jr = (unsigned)__builtin_amdgcn_readfirstlane((int)j) * row_bytes;   // byte offset of La[j]
            o.l0 = gather_row(rs_a, lane_bytes, jr, T{});
#pragma unroll
            for (int t = 0; t < 3; t++) o.l1[t] = gather_row(rs_v, lane_bytes, 3u * jr + (unsigned)t * row_bytes, T{});
#pragma unroll
            for (int k = 0; k < 9; k++) o.l2[k] = gather_row(rs_d, lane_bytes, 9u * jr + (unsigned)k * row_bytes, T{});
#pragma unroll
            for (int m = 0; m < 8; m++) o.en[m] = enc[8 * e + m];
#pragma unroll
            for (int t = 0; t < 3; t++) o.rh[t] = rhat[3 * e + t];
        };
        const long last = hi - 1;
        EdgeOps nxt;
        long j_next = 0;
        if (PIPE && lo < hi) {
            fetch(nxt, lo, dst[lo]);
            j_next = dst[lo + 1 < hi ? lo + 1 : last];
        }
        for (long e = lo; e < hi; e++) {
            EdgeOps cur;
            if constexpr (PIPE) {
                cur = nxt;
                const long e1 = e + 1 < hi ? e + 1 : last;
                fetch(nxt, e1, j_next);
                j_next = dst[e + 2 < hi ? e + 2 : last];
            } else {
                fetch(cur, e, dst[e]);
            }
            float en[8], rh[3];
#pragma unroll
            for (int m = 0; m < 8; m++) en[m] = cur.en[m];
#pragma unroll
            for (int t = 0; t < 3; t++) rh[t] = cur.rh[t];
            const float l0 = (float)cur.l0;
            float l1[3], l2[9];
#pragma unroll
            for (int t = 0; t < 3; t++) l1[t] = (float)cur.l1[t];
#pragma unroll
            for (int k = 0; k < 9; k++) l2[k] = (float)cur.l2[k];
            float phi = bias;
#pragma unroll
            for (int m = 0; m < 8; m++) phi += w[m] * en[m];

            // geometric pieces
            float t_[3];   // L rh
#pragma unroll
            for (int x = 0; x < 3; x++) t_[x] = l2[3 * x] * rh[0] + l2[3 * x + 1] * rh[1] + l2[3 * x + 2] * rh[2];
            const float dot1 = l1[0] * rh[0] + l1[1] * rh[1] + l1[2] * rh[2];          // l1 . rh
            const float quad = t_[0] * rh[0] + t_[1] * rh[1] + t_[2] * rh[2];           // rh^T L rh
            float cr[3];
            cross3(l1, rh, cr);
            const float pl0 = phi * l0;
            const float pd1 = phi * dot1;

            if (active) {
                T* p = P0 + (e * 3) * chan;
                // outputs are written once and not read back here: streaming stores leave the L2 to the gathered rows
                __builtin_nontemporal_store((T)pl0, p + lane_off);                       // 000
                __builtin_nontemporal_store((T)pd1, p + chan + lane_off);                // 110
                __builtin_nontemporal_store((T)(phi * quad), p + 2 * chan + lane_off);   // 220
            }
            if (edge_max) {
                // largest |P0| entry of this (edge, 64-channel chunk): a row bound for the per-edge GEMM
                float mx = fmaxf(fmaxf(fabsf(pl0), fabsf(pd1)), fabsf(phi * quad));
                mx = wave_max_nonneg_last_lane(active ? mx : 0.f);
                if (lane == kWave - 1) edge_max[e * chunks + chunk] = mx;
            }
            // vector sums, label order 011, 101, 121, 211, 111
#pragma unroll
            for (int x = 0; x < 3; x++) {
                s1[x * 5 + 0] += pl0 * rh[x];
                s1[x * 5 + 1] += phi * l1[x];
                s1[x * 5 + 2] += pd1 * rh[x];
                s1[x * 5 + 3] += phi * t_[x];
                s1[x * 5 + 4] += phi * cr[x];
            }
            // rank-2 sums, label order 022, 202, 112, 222, 212 ; component xy -> 3x+y
#pragma unroll
            for (int x = 0; x < 3; x++) {
                float rowx[3];
                cross3(l2 + 3 * x, rh, rowx);   // L[x,:] x rh
                const float pl1x = phi * l1[x];
                const float ptx = phi * t_[x];
#pragma unroll
                for (int y = 0; y < 3; y++) {
                    const int k = 3 * x + y;
                    s2[k * 5 + 0] += pl0 * (rh[y] * rh[x]);
                    s2[k * 5 + 1] += phi * l2[k];
                    s2[k * 5 + 2] += pl1x * rh[y];
                    s2[k * 5 + 3] += ptx * rh[y];
                    s2[k * 5 + 4] += phi * rowx[y];
                }
            }
        }
        if (active && valid) {
            T* o1 = S1 + node * 15 * chan;
#pragma unroll
            for (int k = 0; k < 15; k++) __builtin_nontemporal_store((T)s1[k], o1 + k * chan + lane_off);
            if constexpr (!Y2F) {
                T* o2 = S2 + node * 45 * chan;
#pragma unroll
                for (int k = 0; k < 45; k++) __builtin_nontemporal_store((T)s2[k], o2 + k * chan + lane_off);
            }
        }
        if (node_max) {
            // largest |sum| of this (node, 64-channel chunk): a row bound for the GEMMs that read S1 / S2
            float mx = 0.f;
#pragma unroll
            for (int k = 0; k < 15; k++) mx = fmaxf(mx, fabsf(s1[k]));
#pragma unroll
            for (int k = 0; k < 45; k++) mx = fmaxf(mx, fabsf(s2[k]));
            mx = wave_max_nonneg_last_lane(active ? mx : 0.f);
            if (lane == kWave - 1 && valid) node_max[node * chunks + chunk] = mx;
        }
        if constexpr (Y2F) {
            __shared__ __attribute__((aligned(16))) float tr_buf[4][16 * kTrPitch];
            __shared__ float part[4][16 * 16];
            rank2_linear_of_node_sums(s2, tr_buf, part, chunk, chunks, valid, y2_packed, dim_d,
                                      out_d + node * (long)dim_d * 9, out_d_accumulate != 0);
        }
    }
}

// Y2 (dim_d, 5 chan), row stride ld -> [chunk][label][tq][lane = 16 kk + j][tr] = Y2[j][label chan + 64 chunk + 16 kk + 4 tq + tr]
// (zero for j >= dim_d): what lane (kk, j) of the fused kernel multiplies in steps 4 tq .. 4 tq + 3 of a label
__global__ void __launch_bounds__(256) pack_rank2_weight_kernel(const float* __restrict__ Y2, long ld, int chan,
                                                                int dim_d, float* __restrict__ packed) {
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)(chan / 64) * 5 * 4 * 64 * 4;
    if (idx >= total) return;
    const int tr = (int)(idx & 3), lane = (int)((idx >> 2) & 63), tq = (int)((idx >> 8) & 3);
    const long rest = idx >> 10;                              // chunk * 5 + label
    const int label = (int)(rest % 5), chunk = (int)(rest / 5);
    const int j = lane & 15, kk = lane >> 4;
    packed[idx] = j < dim_d ? Y2[j * ld + (long)label * chan + 64 * chunk + 16 * kk + 4 * tq + tr] : 0.f;
}

}  // namespace
}  // namespace mg

using namespace mg;

template <typename T>
static int launch_bee_message(const char* what, const int* row_ptr, const int* dst, const int* node_order, int n_nodes,
                              long n_edges, const float* rhat, const float* enc, const T* La, const T* Lv, const T* Ld,
                              int chan, const float* enc_W, const float* enc_b, T* P0, T* S1, T* S2,
                              float* node_max, float* edge_max, mg_stream_t stream, const float* y2_packed = nullptr,
                              int dim_d = 0, float* out_d = nullptr, int out_d_accumulate = 0) {
    MG_REQUIRE(n_nodes >= 0 && n_edges >= 0 && chan >= 0, "%s: negative size", what);
    if (n_nodes == 0 || chan == 0) return MG_OK;
    const bool fused = y2_packed != nullptr;
    MG_REQUIRE(row_ptr && La && Lv && Ld && enc_W && enc_b && S1 && (fused ? out_d != nullptr : S2 != nullptr),
               "%s: null pointer", what);
    MG_REQUIRE(n_edges == 0 || (dst && rhat && enc && P0), "%s: null edge operand", what);
    MG_REQUIRE((long)n_nodes * 9 * chan * (long)sizeof(T) < (1L << 32),
               "%s: the rank-2 node rows must stay below 4 GiB (32-bit row offsets)", what);
    const long items = (long)n_nodes * ceil_div(chan, kWave);
    // one item per wave, four per workgroup, an eighth of the items per XCD (the kernel's loop then makes one trip)
    const long blocks = 8 * ceil_div(ceil_div(items, 8), 4);
    MG_REQUIRE(blocks < (1L << 31), "%s: too many (node, channel chunk) items for one launch", what);
    // rows of a few edges do not repay the pipeline's start-up (one extra set of loads per row), unless the system
    // is so small that the chip is not filled and a row's chain of load latencies is all there is to the time
    const bool pipe = n_edges >= 8L * n_nodes || items <= 16384;
#define MG_BEE_LAUNCH(PIPE, Y2F)                                                                                      \
    hipLaunchKernelGGL((bee_message_kernel<T, PIPE, Y2F>), dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, \
                       row_ptr, dst, node_order, (long)n_nodes, rhat, enc, La, Lv, Ld, chan, enc_W, enc_b, P0, S1, S2, \
                       node_max, edge_max, y2_packed, dim_d, out_d, out_d_accumulate)
    if constexpr (std::is_same<T, float>::value) {
        if (fused) {
            MG_REQUIRE(rank2_fusable(chan, dim_d), "%s: the fused rank-2 linear needs chan = 64, 128 or 256 and dim_d <= 16", what);
            MG_REQUIRE(aligned16(y2_packed), "%s: packed weight must be 16-byte aligned", what);
            if (pipe) MG_BEE_LAUNCH(true, true);
            else MG_BEE_LAUNCH(false, true);
            return check_launch(what);
        }
    }
    if (pipe) MG_BEE_LAUNCH(true, false);
    else MG_BEE_LAUNCH(false, false);
#undef MG_BEE_LAUNCH
    return check_launch(what);
}

extern "C" {

int mg_bee_edge_geometry(const float* r_ij, long n_edges, float r0, float* enc, float* rhat, mg_stream_t stream) {
    MG_REQUIRE(n_edges >= 0, "mg_bee_edge_geometry: negative size");
    MG_REQUIRE(r0 > 0.f, "mg_bee_edge_geometry: r0 must be positive");
    if (n_edges == 0) return MG_OK;
    MG_REQUIRE(r_ij && enc && rhat, "mg_bee_edge_geometry: null pointer");
    static const Jacobi8 table = jacobi_table();
    const float scale = (float)(7.0 / (double)r0);
    hipLaunchKernelGGL(bee_geometry_kernel, dim3((unsigned)ceil_div(n_edges, 256)), dim3(256), 0, (hipStream_t)stream,
                       r_ij, n_edges, r0, scale, table, enc, rhat);
    return check_launch("mg_bee_edge_geometry");
}

int mg_bee_message(const int* row_ptr, const int* dst, const int* node_order, int n_nodes, long n_edges,
                   const float* rhat, const float* enc, const float* La, const float* Lv, const float* Ld, int chan,
                   const float* enc_W, const float* enc_b, float* P0, float* S1, float* S2, float* node_max,
                   float* edge_max, mg_stream_t stream) {
    return launch_bee_message<float>("mg_bee_message", row_ptr, dst, node_order, n_nodes, n_edges, rhat, enc, La, Lv,
                                     Ld, chan, enc_W, enc_b, P0, S1, S2, node_max, edge_max, stream);
}

int mg_bee_message_rank2_supported(int chan, int dim_d) { return rank2_fusable(chan, dim_d) ? 1 : 0; }

int mg_bee_rank2_weight_bytes(int chan, size_t* bytes) {
    MG_REQUIRE(bytes != nullptr && chan >= 0, "mg_bee_rank2_weight_bytes: bad argument");
    *bytes = (size_t)ceil_div(chan, 64) * 5 * 4 * 64 * 4 * sizeof(float);
    return MG_OK;
}

int mg_bee_pack_rank2_weight(const float* Y2, long ld, int chan, int dim_d, float* packed, mg_stream_t stream) {
    MG_REQUIRE(rank2_fusable(chan, dim_d), "mg_bee_pack_rank2_weight: needs chan = 64, 128 or 256 and dim_d <= 16");
    MG_REQUIRE(Y2 && packed && ld >= 5L * chan, "mg_bee_pack_rank2_weight: null pointer or short rows");
    const long total = (long)(chan / 64) * 5 * 4 * 64 * 4;
    hipLaunchKernelGGL(pack_rank2_weight_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, (hipStream_t)stream,
                       Y2, ld, chan, dim_d, packed);
    return check_launch("mg_bee_pack_rank2_weight");
}

int mg_bee_message_rank2(const int* row_ptr, const int* dst, const int* node_order, int n_nodes, long n_edges,
                         const float* rhat, const float* enc, const float* La, const float* Lv, const float* Ld, int chan,
                         const float* enc_W, const float* enc_b, const float* packed_Y2, int dim_d, float* P0, float* S1,
                         float* out_d, int accumulate, float* node_max, float* edge_max, mg_stream_t stream) {
    MG_REQUIRE(packed_Y2 != nullptr, "mg_bee_message_rank2: null weight");
    return launch_bee_message<float>("mg_bee_message_rank2", row_ptr, dst, node_order, n_nodes, n_edges, rhat, enc, La,
                                     Lv, Ld, chan, enc_W, enc_b, P0, S1, nullptr, node_max, edge_max, stream, packed_Y2,
                                     dim_d, out_d, accumulate);
}

int mg_bee_message_bf16(const int* row_ptr, const int* dst, const int* node_order, int n_nodes, long n_edges,
                        const float* rhat, const float* enc, const void* La, const void* Lv, const void* Ld, int chan,
                        const float* enc_W, const float* enc_b, void* P0, void* S1, void* S2, mg_stream_t stream) {
    return launch_bee_message<__bf16>("mg_bee_message_bf16", row_ptr, dst, node_order, n_nodes, n_edges, rhat, enc,
                                      static_cast<const __bf16*>(La), static_cast<const __bf16*>(Lv),
                                      static_cast<const __bf16*>(Ld), chan, enc_W, enc_b, static_cast<__bf16*>(P0),
                                      static_cast<__bf16*>(S1), static_cast<__bf16*>(S2), nullptr, nullptr, stream);
}

}  // extern "C"
