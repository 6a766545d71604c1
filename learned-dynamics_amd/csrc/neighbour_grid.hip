// Periodic cell-list radius graph for gfx950.
//
// Pipeline (all on the caller's stream, no allocation, no host sync):
//   bin      wrap each atom into the box, cell id, histogram of cell sizes
//   scan     exclusive prefix of the histogram -> cell_start
//   place    atoms into cell order (slot from the histogram atomics)
//   order    rank atoms inside their cell by index so the cell-ordered array,
//            and with it every output row, is deterministic
//   pairs<0> one workgroup per home cell: the 27 window cells are staged in LDS
//            once, each wave takes home atoms and sweeps the staged candidates
//            64 at a time, counting hits with ballot/popcount -> degree
//   scan     degrees -> CSR row_ptr (+ per-box edge counts, statistics)
//   pairs<1> same sweep, hits compacted with ballot + prefix popcount and written
//            at row_ptr[i] + running offset (exact-size rows, no atomics per edge)
//
// fp32 recipe (this file is compiled with -ffp-contract=off):
//   w    = remainderf(x - box/2, box) + box/2                 (IEEE remainder)
//   cell = (int)(((float)ndiv * w) / box) % ndiv              (correctly rounded divide)
//   d    = remainder(w_i - w_j, box) per axis, evaluated as one conditional
//          +-box (|w_i - w_j| <= box, so the quotient is -1, 0 or 1 and the
//          result is exact; ties at +-box/2 keep their sign like round-to-even)
//   d2   = fma(dz,dz, fma(dy,dy, dx*dx)) <= cutoff*cutoff, i != j
//   only the periodic 3x3x3 cell window is searched, with ndiv = ceil(box/cutoff):
//   when box/cutoff is not an integer the cells are narrower than the cutoff and
//   pairs two cells apart are not listed.
#include "common.hpp"
#include <mutex>

namespace mg {
namespace {

// Built-in workspace of mg_neighbour_edges_static, for callers that cannot allocate one.  One copy per GPU, held
// from the moment the library is loaded until the process ends.  Host code never passes `scratch` itself anywhere:
// the name is a host-side handle, the device address comes from hipGetSymbolAddress (scratch_of_current_device).
constexpr size_t kScratchBytes = size_t(32) << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {nullptr};
std::mutex g_scratch_mutex;

// Device address of this GPU's copy of `scratch`; looked up once per device, with that device current.
int scratch_of_current_device(void** out) {
    int dev = -1;
    MG_HIP(hipGetDevice(&dev));
    MG_REQUIRE(dev >= 0 && dev < kMaxDevices, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        MG_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        MG_REQUIRE(p != nullptr, "hipGetSymbolAddress returned a null address for the built-in workspace");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return MG_OK;
}

constexpr int kCandCapDense = 1024;   // candidates staged in LDS per home cell (16 KB), 4-wave workgroups
constexpr int kCandCapSparse = 256;   // sparse boxes: 1-wave workgroups, 4 KB
constexpr int kScanThreads = 256;
constexpr int kScanItems = 8;       // per thread
constexpr int kScanTile = kScanThreads * kScanItems;

struct Grid {
    int nx, ny, nz, ncells;   // per box
    float bx, by, bz;
    float r0sq;
    int batch, nodes;
};

struct Workspace {
    float4* wrapped;    // A: (w.x, w.y, w.z, bits of box-local index)
    float4* sorted;     // A: same records in cell order
    int* cell_of;       // A: global cell id (batch offset included)
    int* slot;          // A
    int* placed;        // A: atom ids in cell order before ranking
    int* degree;        // A
    int* cell_count;    // C
    int* cell_start;    // C + 1
    int* block_sums;    // scan scratch
    int* block_max;     // scan scratch
    unsigned long long* masks;   // A x mask_words: hit bits of the count pass, reused by the fill pass
    int mask_words;     // 64-candidate groups kept per atom (= LDS tile size / 64)
    size_t bytes;
};

inline size_t align_up(size_t v) { return (v + 255) & ~size_t(255); }

Workspace carve(void* base, long A, long C, int mask_words) {
    Workspace w{};
    size_t off = 0;
    auto take = [&](size_t bytes) {
        void* p = base ? static_cast<char*>(base) + off : nullptr;
        off += align_up(bytes);
        return p;
    };
    const long scan_blocks = ceil_div((A > C ? A : C) + 1, kScanTile) + 1;
    w.wrapped = static_cast<float4*>(take(sizeof(float4) * A));
    w.sorted = static_cast<float4*>(take(sizeof(float4) * A));
    w.cell_of = static_cast<int*>(take(sizeof(int) * A));
    w.slot = static_cast<int*>(take(sizeof(int) * A));
    w.placed = static_cast<int*>(take(sizeof(int) * A));
    w.degree = static_cast<int*>(take(sizeof(int) * A));
    w.cell_count = static_cast<int*>(take(sizeof(int) * C));
    w.cell_start = static_cast<int*>(take(sizeof(int) * (C + 1)));
    w.block_sums = static_cast<int*>(take(sizeof(int) * scan_blocks));
    w.block_max = static_cast<int*>(take(sizeof(int) * scan_blocks));
    w.masks = static_cast<unsigned long long*>(take(sizeof(unsigned long long) * A * mask_words));
    w.mask_words = mask_words;
    w.bytes = off;
    return w;
}

int make_grid(float cutoff, float bx, float by, float bz, int batch, int nodes, Grid* g) {
    MG_REQUIRE(cutoff > 0.f && bx > 0.f && by > 0.f && bz > 0.f, "cutoff and box must be positive");
    MG_REQUIRE(batch >= 0 && nodes >= 0, "negative batch or nodes");
    int nd[3];
    mg_neighbour_ndiv(cutoff, bx, by, bz, nd);
    if (nd[0] < 3 || nd[1] < 3 || nd[2] < 3)
        return fail(MG_ERR_BOX_TOO_SMALL, "box dimension must be greater than 3*cutoff");
    const long ncells = (long)nd[0] * nd[1] * nd[2];
    MG_REQUIRE(ncells * (batch > 0 ? batch : 1) < 0x7fffffffL, "too many cells (%ld per box)", ncells);
    MG_REQUIRE((long)batch * nodes < 0x7fffffffL, "batch*nodes does not fit int32");
    g->nx = nd[0]; g->ny = nd[1]; g->nz = nd[2]; g->ncells = (int)ncells;
    g->bx = bx; g->by = by; g->bz = bz;
    g->r0sq = cutoff * cutoff;
    g->batch = batch; g->nodes = nodes;
    return MG_OK;
}

// ---------------------------------------------------------------- device math
__device__ __forceinline__ float wrap_into_box(float x, float box) {
    const float half = 0.5f * box;
    return remainderf(x - half, box) + half;
}

__device__ __forceinline__ int cell_coord(float w, float box, int ndiv) {
    const float scaled = (float)ndiv * w;
    const float q = __fdiv_rn(scaled, box);
    int c = ((int)q) % ndiv;
    return c < 0 ? 0 : c;   // only reachable with non-finite input
}

// remainder(d, box) for d = a - b with a, b in [0, box]
__device__ __forceinline__ float wrap_delta(float d, float box, float half) {
    if (d > half) d -= box;
    else if (d < -half) d += box;
    return d;
}

// ------------------------------------------------------------------- kernels
// Clearing is done by a kernel, not a memset node, so that the sequence behaves
// the same when a caller records it into a HIP graph.
__global__ void __launch_bounds__(256) zero3_kernel(int* __restrict__ a, long na, int* __restrict__ b, long nb,
                                                    int* __restrict__ c, long nc) {
    const long stride = (long)gridDim.x * blockDim.x;
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    for (long i = t; i < na; i += stride) a[i] = 0;
    for (long i = t; i < nb; i += stride) b[i] = 0;
    for (long i = t; i < nc; i += stride) c[i] = 0;
}

__global__ void __launch_bounds__(256) bin_kernel(const float* __restrict__ x, Grid g, Workspace w) {
    const long A = (long)g.batch * g.nodes;
    const long a = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (a >= A) return;
    const int b = (int)(a / g.nodes);
    const int i = (int)(a - (long)b * g.nodes);
    const float wx = wrap_into_box(x[3 * a + 0], g.bx);
    const float wy = wrap_into_box(x[3 * a + 1], g.by);
    const float wz = wrap_into_box(x[3 * a + 2], g.bz);
    const int cx = cell_coord(wx, g.bx, g.nx);
    const int cy = cell_coord(wy, g.by, g.ny);
    const int cz = cell_coord(wz, g.bz, g.nz);
    const int cell = ((b * g.nx + cx) * g.ny + cy) * g.nz + cz;
    w.wrapped[a] = make_float4(wx, wy, wz, __int_as_float(i));
    w.cell_of[a] = cell;
    w.slot[a] = atomicAdd(&w.cell_count[cell], 1);
}

__global__ void __launch_bounds__(256) place_kernel(Grid g, Workspace w) {
    const long A = (long)g.batch * g.nodes;
    const long a = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (a >= A) return;
    w.placed[w.cell_start[w.cell_of[a]] + w.slot[a]] = (int)a;
}

// position p holds atom a of cell c; its final place is its rank by atom id inside c
__global__ void __launch_bounds__(256) order_kernel(Grid g, Workspace w) {
    const long A = (long)g.batch * g.nodes;
    const long p = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= A) return;
    const int a = w.placed[p];
    const int c = w.cell_of[a];
    const int lo = w.cell_start[c], hi = w.cell_start[c + 1];
    int rank = 0;
    for (int q = lo; q < hi; q++) rank += (w.placed[q] < a) ? 1 : 0;
    w.sorted[lo + rank] = w.wrapped[a];
}

// --- three-kernel exclusive scan of n ints: out[0..n] (out[n] = total) -------
__device__ __forceinline__ int wave_incl_scan(int v, int lane) {
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        int t = __shfl_up(v, d);
        if (lane >= d) v += t;
    }
    return v;
}

// block-wide exclusive scan of one value per thread (256 threads); returns the
// exclusive prefix and leaves the block total in *total
__device__ __forceinline__ int block_excl_scan(int v, int* total, int* lds /* >= 8 ints */) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int incl = wave_incl_scan(v, lane);
    if (lane == kWave - 1) lds[wave] = incl;
    __syncthreads();
    int off = 0, tot = 0;
    const int nw = blockDim.x / kWave;
    for (int k = 0; k < nw; k++) {
        const int s = lds[k];
        if (k < wave) off += s;
        tot += s;
    }
    __syncthreads();
    *total = tot;
    return off + incl - v;
}

__global__ void __launch_bounds__(kScanThreads) scan_sums_kernel(const int* __restrict__ in, long n,
                                                                 int* block_sums, int* block_max) {
    __shared__ int lds[8];
    const long base = (long)blockIdx.x * kScanTile + (long)threadIdx.x * kScanItems;
    int s = 0, m = 0;
#pragma unroll
    for (int k = 0; k < kScanItems; k++) {
        const int v = (base + k < n) ? in[base + k] : 0;
        s += v;
        m = v > m ? v : m;
    }
    int total;
    block_excl_scan(s, &total, lds);
    // block max through the same LDS words
    for (int d = kWave / 2; d > 0; d >>= 1) { int t = __shfl_xor(m, d); m = t > m ? t : m; }
    if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        int mm = 0;
        for (int k = 0; k < kScanThreads / kWave; k++) mm = lds[k] > mm ? lds[k] : mm;
        block_sums[blockIdx.x] = total;
        block_max[blockIdx.x] = mm;
    }
}

// single workgroup: block_sums -> exclusive offsets in place; total and max out
__global__ void __launch_bounds__(kScanThreads) scan_top_kernel(int* block_sums, const int* block_max,
                                                                int nblocks, int* out_total /* may be null */,
                                                                int* out_max /* may be null */,
                                                                int* out_overflow /* may be null */) {
    __shared__ int lds[8];
    long long carry = 0;
    int mx = 0;
    for (int base = 0; base < nblocks; base += kScanThreads) {
        const int k = base + threadIdx.x;
        const int v = k < nblocks ? block_sums[k] : 0;
        const int m = k < nblocks ? block_max[k] : 0;
        mx = m > mx ? m : mx;
        int total;
        const int ex = block_excl_scan(v, &total, lds);
        if (k < nblocks) block_sums[k] = (int)(carry + ex);
        carry += total;
    }
    for (int d = kWave / 2; d > 0; d >>= 1) { int t = __shfl_xor(mx, d); mx = t > mx ? t : mx; }
    if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = mx;
    __syncthreads();
    if (threadIdx.x == 0) {
        int mm = 0;
        for (int k = 0; k < kScanThreads / kWave; k++) mm = lds[k] > mm ? lds[k] : mm;
        if (out_total) *out_total = carry > 0x7fffffffLL ? 0x7fffffff : (int)carry;
        if (out_max) *out_max = mm;
        if (out_overflow) *out_overflow = carry > 0x7fffffffLL ? 1 : 0;
    }
}

// whole scan in one workgroup (n small): out[0..n], optional total / max.  Each lane scans a
// contiguous chunk serially, the chunk totals are scanned across the workgroup once.
__global__ void __launch_bounds__(kScanThreads) scan_small_kernel(const int* __restrict__ in, int n,
                                                                  int* __restrict__ out, int* out_total, int* out_max) {
    __shared__ int lds[8];
    const int chunk = (n + kScanThreads) / kScanThreads;          // covers indices 0..n
    const int lo = threadIdx.x * chunk;
    const int hi = lo + chunk < n ? lo + chunk : n;
    int sum = 0, mx = 0;
    for (int k = lo; k < hi; k++) {
        const int v = in[k];
        sum += v;
        mx = v > mx ? v : mx;
    }
    int total;
    int run = block_excl_scan(sum, &total, lds);
    for (int k = lo; k < lo + chunk && k <= n; k++) {
        out[k] = run;
        if (k < n) run += in[k];
    }
    for (int d = kWave / 2; d > 0; d >>= 1) { int t = __shfl_xor(mx, d); mx = t > mx ? t : mx; }
    if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = mx;
    __syncthreads();
    if (threadIdx.x == 0) {
        int mm = 0;
        for (int k = 0; k < kScanThreads / kWave; k++) mm = lds[k] > mm ? lds[k] : mm;
        if (out_total) *out_total = total;
        if (out_max) *out_max = mm;
    }
}

// nodes > 0: also edge_counts[b] = out[(b+1)*nodes] (inclusive prefix of edges per box)
__global__ void __launch_bounds__(kScanThreads) scan_apply_kernel(const int* __restrict__ in, long n,
                                                                  const int* __restrict__ block_offsets,
                                                                  int* __restrict__ out, int nodes,
                                                                  int* __restrict__ edge_counts) {
    __shared__ int lds[8];
    const long base = (long)blockIdx.x * kScanTile + (long)threadIdx.x * kScanItems;
    int v[kScanItems];
    int s = 0;
#pragma unroll
    for (int k = 0; k < kScanItems; k++) {
        v[k] = (base + k < n) ? in[base + k] : 0;
        s += v[k];
    }
    int total;
    int run = block_excl_scan(s, &total, lds) + block_offsets[blockIdx.x];
#pragma unroll
    for (int k = 0; k < kScanItems; k++) {
        if (base + k <= n) {
            out[base + k] = run;   // index n receives the grand total
            if (nodes > 0 && base + k > 0) {
                const unsigned idx = (unsigned)(base + k), q = idx / (unsigned)nodes;   // n < 2^31: 32-bit divide
                if (q * (unsigned)nodes == idx) edge_counts[q - 1] = run;
            }
        }
        run += v[k];
    }
}


// One workgroup per home cell.  FILL = false: degrees (+ hit masks).  FILL = true: src/dst.
//
// The count pass keeps, per home atom, one 64-bit ballot per group of 64 window
// candidates; the fill pass replays those masks and never touches the geometry
// again (it stages only the candidates' atom ids).  Windows larger than the LDS
// tile (kCandCap candidates) fall back to recomputing in the fill pass.
//
// Minimum image: a wrapped coordinate lies in [0, box] with BOTH ends possible
// (remainderf(x - box/2, box) + box/2 gives exactly box for x = box, -box, 3 box, ...
// and for x within half an ulp below box), and such an atom sits in cell 0 because
// the cell index is taken modulo ndiv.  So cell 0 holds coordinates near 0 and
// coordinates equal (or within rounding of) box; every other cell c holds
// coordinates within rounding of [c, c+1) box/ndiv.  In an axis with at least 5
// cells whose window (home - 1 .. home + 1) contains neither cell 0 nor, from the
// other side, wraps around the box (home cell 2 .. ndiv-2), |w_i - w_j| < 2/5 box
// < box/2 for every window candidate, remainder(w_i - w_j, box) is the plain
// difference and the conditional +-box is skipped (same bits, 40 % fewer
// instructions per pair).  Home cell 1 keeps the wrap: its window contains cell 0.
template <bool FILL, int kCandCap>
__global__ void __launch_bounds__(256) pairs_kernel(Grid g, Workspace w, const int* __restrict__ row_ptr,
                                                    int* __restrict__ src, int* __restrict__ dst, int capacity) {
    constexpr int kWords = kCandCap / kWave;
    __shared__ float4 cand[FILL ? 1 : kCandCap];      // count pass: wrapped positions + atom id
    __shared__ int cand_idx[FILL ? kCandCap : 1];     // fill pass: atom ids only
    __shared__ int range_start[27];
    __shared__ int range_prefix[28];

    const int cell = blockIdx.x;              // global cell id
    const int home_lo = w.cell_start[cell];
    const int home_n = w.cell_start[cell + 1] - home_lo;
    if (home_n == 0) return;                  // uniform over the workgroup

    const int b = cell / g.ncells;
    const int c = cell - b * g.ncells;
    const int cx = c / (g.ny * g.nz), cy = (c / g.nz) % g.ny, cz = c % g.nz;

    if (threadIdx.x < 27) {
        const int t = threadIdx.x;
        const int dx = t / 9 - 1, dy = (t / 3) % 3 - 1, dz = t % 3 - 1;
        const int nx = (cx + dx + g.nx) % g.nx;
        const int ny = (cy + dy + g.ny) % g.ny;
        const int nz = (cz + dz + g.nz) % g.nz;
        const int nc = ((b * g.nx + nx) * g.ny + ny) * g.nz + nz;
        range_start[t] = w.cell_start[nc];
        range_prefix[t + 1] = w.cell_start[nc + 1] - w.cell_start[nc];
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int acc = 0;
        range_prefix[0] = 0;
        for (int t = 0; t < 27; t++) { acc += range_prefix[t + 1]; range_prefix[t + 1] = acc; }
    }
    __syncthreads();
    const int M = range_prefix[27];
    const bool masks_ok = M <= kCandCap;      // uniform: the count pass stored every ballot of this cell

    // candidate k of the concatenated window -> address in the cell-ordered array
    auto locate = [&](int k) {
        int lo = 0, hi = 26;   // last range with prefix <= k
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (range_prefix[mid] <= k) lo = mid; else hi = mid - 1;
        }
        return range_start[lo] + (k - range_prefix[lo]);
    };

    const int staged = M < kCandCap ? M : kCandCap;
    for (int k = threadIdx.x; k < staged; k += blockDim.x) {
        const float4 v = w.sorted[locate(k)];
        if (FILL) cand_idx[k] = __float_as_int(v.w);
        else cand[k] = v;
    }
    __syncthreads();

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave, nwaves = blockDim.x / kWave;
    const float hx = 0.5f * g.bx, hy = 0.5f * g.by, hz = 0.5f * g.bz;
    const bool wrap_x = g.nx < 5 || cx <= 1 || cx == g.nx - 1;
    const bool wrap_y = g.ny < 5 || cy <= 1 || cy == g.ny - 1;
    const bool wrap_z = g.nz < 5 || cz <= 1 || cz == g.nz - 1;
    const unsigned long long lt_mask = (1ull << lane) - 1ull;
    const int node_base = b * g.nodes;

    auto test_pair = [&](const float4& self, const float4& o) {
        float dx = self.x - o.x, dy = self.y - o.y, dz = self.z - o.z;
        if (wrap_x) dx = wrap_delta(dx, g.bx, hx);
        if (wrap_y) dy = wrap_delta(dy, g.by, hy);
        if (wrap_z) dz = wrap_delta(dz, g.bz, hz);
        const float d2 = __fmaf_rn(dz, dz, __fmaf_rn(dy, dy, dx * dx));
        return d2 <= g.r0sq;
    };

    for (int h = wave; h < home_n; h += nwaves) {
        const float4 self = w.sorted[home_lo + h];
        const int self_idx = __float_as_int(self.w);
        const int row = node_base + self_idx;
        unsigned long long* my_masks = w.masks + (long)row * kWords;
        int running = 0;
        const int words = (M + kWave - 1) / kWave;     // <= kWords when masks_ok
        if (!FILL) {
            unsigned long long keep = 0;               // lane i keeps the ballot of candidate group i
            for (int k0 = 0; k0 < M; k0 += kWave) {
                const int k = k0 + lane;
                bool hit = false;
                if (k < M) {
                    const float4 o = k < kCandCap ? cand[k] : w.sorted[locate(k)];
                    hit = (__float_as_int(o.w) != self_idx) && test_pair(self, o);
                }
                const unsigned long long mask = __ballot(hit);
                if (lane == k0 / kWave) keep = mask;
                running += __popcll(mask);
            }
            if (masks_ok && lane < words) my_masks[lane] = keep;   // one unit-stride store per atom
            if (lane == 0) w.degree[row] = running;
        } else {
            const int out_base = row_ptr[row];
            unsigned long long keep = 0;
            if (masks_ok && lane < words) keep = my_masks[lane];
            for (int k0 = 0; k0 < M; k0 += kWave) {
                const int k = k0 + lane;
                unsigned long long mask;
                int other_idx = 0;
                if (masks_ok) {
                    const int it = k0 / kWave;
                    const unsigned lo = __shfl((unsigned)(keep & 0xffffffffull), it);
                    const unsigned hi = __shfl((unsigned)(keep >> 32), it);
                    mask = ((unsigned long long)hi << 32) | lo;
                    if (k < M) other_idx = cand_idx[k];
                } else {
                    bool hit = false;
                    if (k < M) {
                        const float4 o = w.sorted[locate(k)];
                        other_idx = __float_as_int(o.w);
                        hit = (other_idx != self_idx) && test_pair(self, o);
                    }
                    mask = __ballot(hit);
                }
                if ((mask >> lane) & 1ull) {
                    const int pos = out_base + running + __popcll(mask & lt_mask);
                    if (pos < capacity) {      // src / dst hold `capacity` edges: the rest is dropped, never written
                        src[pos] = row;
                        dst[pos] = node_base + other_idx;
                    }
                }
                running += __popcll(mask);
            }
        }
    }
}

// order[k] = global id of the k-th atom in cell order (cells x-major, atoms by id inside a cell)
__global__ void __launch_bounds__(256) cell_order_kernel(Grid g, Workspace w, int* __restrict__ order) {
    const long A = (long)g.batch * g.nodes;
    const long k = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= A) return;
    order[k] = (int)(k / g.nodes) * g.nodes + __float_as_int(w.sorted[k].w);
}

__global__ void __launch_bounds__(256) wrap_cells_kernel(const float* __restrict__ x, Grid g,
                                                         float* __restrict__ wrapped, int* __restrict__ cell) {
    const long A = (long)g.batch * g.nodes;
    const long a = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (a >= A) return;
    const float wx = wrap_into_box(x[3 * a + 0], g.bx);
    const float wy = wrap_into_box(x[3 * a + 1], g.by);
    const float wz = wrap_into_box(x[3 * a + 2], g.bz);
    wrapped[3 * a + 0] = wx; wrapped[3 * a + 1] = wy; wrapped[3 * a + 2] = wz;
    cell[a] = (cell_coord(wx, g.bx, g.nx) * g.ny + cell_coord(wy, g.by, g.ny)) * g.nz + cell_coord(wz, g.bz, g.nz);
}

__global__ void __launch_bounds__(256) pad_kernel(const int* __restrict__ row_ptr, const int* __restrict__ dst,
                                                  long A, int nodes, int nmax, int* __restrict__ neighbours,
                                                  int* __restrict__ counts) {
    // one wave per node
    const long a = ((long)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    const int lane = threadIdx.x & (kWave - 1);
    if (a >= A) return;
    const int lo = row_ptr[a], n = row_ptr[a + 1] - lo;
    const int node_base = (int)(a / nodes) * nodes;
    if (lane == 0) counts[a] = n;
    for (int k = lane; k < n && k < nmax; k += kWave) neighbours[a * nmax + k] = dst[lo + k] - node_base;
}

__global__ void __launch_bounds__(256) padded_read_kernel(const int* __restrict__ counts,
                                                          const int* __restrict__ neighbours,
                                                          const float* __restrict__ x, long A, int nodes, int nmax,
                                                          int chan, float* __restrict__ edge) {
    // flat over (node, slot, chan)
    const long total = A * nmax * chan;
    for (long t = (long)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (long)gridDim.x * blockDim.x) {
        const int c = (int)(t % chan);
        const long as = t / chan;
        const int j = (int)(as % nmax);
        const long a = as / nmax;
        float v = 0.f;
        if (j < counts[a]) {
            const long nb = (a / nodes) * nodes + neighbours[a * nmax + j];
            v = x[nb * chan + c];
        }
        edge[t] = v;
    }
}

__global__ void __launch_bounds__(256) padded_reduce_kernel(const int* __restrict__ counts,
                                                            const float* __restrict__ edge, long A, int nmax,
                                                            int chan, float* __restrict__ out) {
    const long total = A * chan;
    for (long t = (long)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (long)gridDim.x * blockDim.x) {
        const int c = (int)(t % chan);
        const long a = t / chan;
        const int n = counts[a] < nmax ? counts[a] : nmax;
        float s = 0.f;
        for (int j = 0; j < n; j++) s += edge[(a * nmax + j) * chan + c];
        out[t] = s;
    }
}

// torch's float `%` (floor-mod): fmod, then move a result of the wrong sign by one period
__device__ __forceinline__ float floor_mod(float a, float b) {
    float m = fmodf(a, b);
    if (m != 0.f && ((b < 0.f) != (m < 0.f))) m += b;
    return m;
}

__global__ void __launch_bounds__(256) edge_vectors_kernel(const float* __restrict__ x, const int* __restrict__ src,
                                                           const int* __restrict__ dst, long E, float bx, float by,
                                                           float bz, float* __restrict__ r_ij,
                                                           int8_t* __restrict__ shift) {
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    const long i = src[e], j = dst[e];
    const float box[3] = {bx, by, bz};
#pragma unroll
    for (int d = 0; d < 3; d++) {
        const float raw = x[3 * j + d] - x[3 * i + d];
        const float half = 0.5f * box[d];
        const float r = floor_mod(raw + half, box[d]) - half;
        r_ij[3 * e + d] = r;
        if (shift) shift[3 * e + d] = (int8_t)rintf(__fdiv_rn(raw - r, box[d]));
    }
}

int run_scan(const int* in, long n, int* out, Workspace& w, int* out_total, int* out_max, int* out_overflow,
             hipStream_t st, int nodes = 0, int* edge_counts = nullptr) {
    if (n <= 16384 && nodes == 0 && out_overflow == nullptr) {
        hipLaunchKernelGGL(scan_small_kernel, dim3(1), dim3(kScanThreads), 0, st, in, (int)n, out, out_total, out_max);
        return check_launch("neighbour scan");
    }
    const int nblocks = (int)ceil_div(n + 1, kScanTile);
    hipLaunchKernelGGL(scan_sums_kernel, dim3(nblocks), dim3(kScanThreads), 0, st, in, n, w.block_sums, w.block_max);
    hipLaunchKernelGGL(scan_top_kernel, dim3(1), dim3(kScanThreads), 0, st, w.block_sums, w.block_max, nblocks,
                       out_total, out_max, out_overflow);
    hipLaunchKernelGGL(scan_apply_kernel, dim3(nblocks), dim3(kScanThreads), 0, st, in, n, w.block_sums, out, nodes,
                       edge_counts);
    return check_launch("neighbour scan");
}

int pairs_block_size(const Grid& g);
int mask_words(const Grid& g) { return (pairs_block_size(g) == 64 ? kCandCapSparse : kCandCapDense) / kWave; }

int pairs_block_size(const Grid& g) {
    // sparse boxes: one wave per cell is plenty
    const double mean_occ = (double)g.nodes / (double)g.ncells;
    return mean_occ <= 4.0 ? 64 : 256;
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_neighbour_ndiv(float cutoff, float box_x, float box_y, float box_z, int ndiv[3]) {
    ndiv[0] = (int)ceilf(box_x / cutoff);
    ndiv[1] = (int)ceilf(box_y / cutoff);
    ndiv[2] = (int)ceilf(box_z / cutoff);
    return MG_OK;
}

int mg_neighbour_workspace_bytes(int batch, int nodes, float cutoff, float box_x, float box_y, float box_z,
                                 size_t* bytes) {
    MG_REQUIRE(bytes != nullptr, "bytes is null");
    Grid g;
    if (int s = make_grid(cutoff, box_x, box_y, box_z, batch, nodes, &g)) return s;
    const long A = (long)batch * nodes, C = (long)batch * g.ncells;
    *bytes = carve(nullptr, A, C, mask_words(g)).bytes + 256;
    return MG_OK;
}

int mg_neighbour_count(const float* x, int batch, int nodes, float cutoff, float box_x, float box_y,
                       float box_z, void* workspace, size_t workspace_bytes, int* row_ptr,
                       int* edge_counts, int* stats, mg_stream_t stream) {
    Grid g;
    if (int s = make_grid(cutoff, box_x, box_y, box_z, batch, nodes, &g)) return s;
    MG_REQUIRE(row_ptr && stats && workspace, "mg_neighbour_count: null pointer");
    MG_REQUIRE(batch == 0 || edge_counts, "mg_neighbour_count: edge_counts is null");
    const long A = (long)batch * nodes, C = (long)batch * g.ncells;
    void* base = reinterpret_cast<void*>((reinterpret_cast<uintptr_t>(workspace) + 255) & ~uintptr_t(255));
    Workspace w = carve(base, A, C, mask_words(g));
    if (w.bytes + 256 > workspace_bytes)
        return fail(MG_ERR_WORKSPACE, "mg_neighbour_count: workspace has %zu bytes, %zu needed", workspace_bytes,
                    w.bytes + 256);
    hipStream_t st = (hipStream_t)stream;
    if (A == 0) {
        hipLaunchKernelGGL(zero3_kernel, dim3(1), dim3(256), 0, st, stats, 4L, row_ptr, 1L, edge_counts, (long)batch);
        return check_launch("mg_neighbour_count");
    }
    MG_REQUIRE(x != nullptr, "mg_neighbour_count: x is null");
    hipLaunchKernelGGL(zero3_kernel, dim3((unsigned)(ceil_div(C, 256) < 1024 ? ceil_div(C, 256) : 1024)), dim3(256), 0,
                       st, stats, 4L, row_ptr, 1L, w.cell_count, C);
    const unsigned ablocks = (unsigned)ceil_div(A, 256);
    hipLaunchKernelGGL(bin_kernel, dim3(ablocks), dim3(256), 0, st, x, g, w);
    if (int s = run_scan(w.cell_count, C, w.cell_start, w, nullptr, stats + 1, nullptr, st)) return s;
    hipLaunchKernelGGL(place_kernel, dim3(ablocks), dim3(256), 0, st, g, w);
    hipLaunchKernelGGL(order_kernel, dim3(ablocks), dim3(256), 0, st, g, w);
    if (pairs_block_size(g) == 64)
        hipLaunchKernelGGL((pairs_kernel<false, kCandCapSparse>), dim3((unsigned)C), dim3(64), 0, st, g, w,
                           (const int*)nullptr, (int*)nullptr, (int*)nullptr, 0);
    else
        hipLaunchKernelGGL((pairs_kernel<false, kCandCapDense>), dim3((unsigned)C), dim3(256), 0, st, g, w,
                           (const int*)nullptr, (int*)nullptr, (int*)nullptr, 0);
    if (int s = run_scan(w.degree, A, row_ptr, w, stats + 0, stats + 2, stats + 3, st, nodes, edge_counts)) return s;
    return check_launch("mg_neighbour_count");
}

int mg_neighbour_fill(const void* workspace, size_t workspace_bytes, int batch, int nodes, float cutoff,
                      float box_x, float box_y, float box_z, const int* row_ptr, int n_edges, int* src,
                      int* dst, mg_stream_t stream) {
    Grid g;
    if (int s = make_grid(cutoff, box_x, box_y, box_z, batch, nodes, &g)) return s;
    MG_REQUIRE(n_edges >= 0, "mg_neighbour_fill: negative n_edges");
    const long A = (long)batch * nodes, C = (long)batch * g.ncells;
    if (A == 0 || n_edges == 0) return MG_OK;
    MG_REQUIRE(workspace && row_ptr && src && dst, "mg_neighbour_fill: null pointer");
    void* base = reinterpret_cast<void*>((reinterpret_cast<uintptr_t>(workspace) + 255) & ~uintptr_t(255));
    Workspace w = carve(base, A, C, mask_words(g));
    if (w.bytes + 256 > workspace_bytes)
        return fail(MG_ERR_WORKSPACE, "mg_neighbour_fill: workspace has %zu bytes, %zu needed", workspace_bytes,
                    w.bytes + 256);
    if (pairs_block_size(g) == 64)
        hipLaunchKernelGGL((pairs_kernel<true, kCandCapSparse>), dim3((unsigned)C), dim3(64), 0, (hipStream_t)stream,
                           g, w, row_ptr, src, dst, n_edges);
    else
        hipLaunchKernelGGL((pairs_kernel<true, kCandCapDense>), dim3((unsigned)C), dim3(256), 0, (hipStream_t)stream,
                           g, w, row_ptr, src, dst, n_edges);
    return check_launch("mg_neighbour_fill");
}

int mg_neighbour_edges(const float* x, int batch, int nodes, float cutoff, float box_x, float box_y, float box_z,
                       void* workspace, size_t workspace_bytes, int* row_ptr, int* edge_counts, int* stats,
                       int capacity, int* src, int* dst, mg_stream_t stream) {
    MG_REQUIRE(capacity >= 0, "mg_neighbour_edges: negative capacity");
    MG_REQUIRE(capacity == 0 || (src && dst), "mg_neighbour_edges: src / dst is null");
    if (int s = mg_neighbour_count(x, batch, nodes, cutoff, box_x, box_y, box_z, workspace, workspace_bytes, row_ptr,
                                   edge_counts, stats, stream))
        return s;
    return mg_neighbour_fill(workspace, workspace_bytes, batch, nodes, cutoff, box_x, box_y, box_z, row_ptr, capacity,
                             src, dst, stream);
}

int mg_neighbour_edges_static(const float* x, int batch, int nodes, float cutoff, float box_x, float box_y,
                              float box_z, int* row_ptr, int* edge_counts, int* stats, int capacity, int* src,
                              int* dst, mg_stream_t stream) {
    size_t need = 0;
    if (int s = mg_neighbour_workspace_bytes(batch, nodes, cutoff, box_x, box_y, box_z, &need)) return s;
    if (need > kScratchBytes)
        return fail(MG_ERR_WORKSPACE,
                    "mg_neighbour_edges_static: this search needs %zu bytes of workspace, the built-in one holds %zu "
                    "(about %ld atoms in total); use mg_neighbour_edges with a workspace of your own",
                    need, kScratchBytes, (long)(kScratchBytes / 180));
    void* ws = nullptr;
    if (int s = scratch_of_current_device(&ws)) return s;
    // every array of the workspace that must start at zero (the cell histogram) is cleared by a kernel inside
    // mg_neighbour_count; everything else is written before it is read, so what the previous call left is harmless
    return mg_neighbour_edges(x, batch, nodes, cutoff, box_x, box_y, box_z, ws, kScratchBytes, row_ptr, edge_counts,
                              stats, capacity, src, dst, stream);
}

int mg_neighbour_cell_order(const void* workspace, size_t workspace_bytes, int batch, int nodes, float cutoff,
                            float box_x, float box_y, float box_z, int* order, mg_stream_t stream) {
    Grid g;
    if (int s = make_grid(cutoff, box_x, box_y, box_z, batch, nodes, &g)) return s;
    const long A = (long)batch * nodes, C = (long)batch * g.ncells;
    if (A == 0) return MG_OK;
    MG_REQUIRE(workspace && order, "mg_neighbour_cell_order: null pointer");
    void* base = reinterpret_cast<void*>((reinterpret_cast<uintptr_t>(workspace) + 255) & ~uintptr_t(255));
    Workspace w = carve(base, A, C, mask_words(g));
    if (w.bytes + 256 > workspace_bytes)
        return fail(MG_ERR_WORKSPACE, "mg_neighbour_cell_order: workspace has %zu bytes, %zu needed", workspace_bytes,
                    w.bytes + 256);
    hipLaunchKernelGGL(cell_order_kernel, dim3((unsigned)ceil_div(A, 256)), dim3(256), 0, (hipStream_t)stream, g, w,
                       order);
    return check_launch("mg_neighbour_cell_order");
}

int mg_neighbour_wrap_cells(const float* x, int batch, int nodes, float cutoff, float box_x, float box_y,
                            float box_z, float* wrapped, int* cell, mg_stream_t stream) {
    Grid g;
    if (int s = make_grid(cutoff, box_x, box_y, box_z, batch, nodes, &g)) return s;
    const long A = (long)batch * nodes;
    if (A == 0) return MG_OK;
    MG_REQUIRE(x && wrapped && cell, "mg_neighbour_wrap_cells: null pointer");
    hipLaunchKernelGGL(wrap_cells_kernel, dim3((unsigned)ceil_div(A, 256)), dim3(256), 0, (hipStream_t)stream, x, g,
                       wrapped, cell);
    return check_launch("mg_neighbour_wrap_cells");
}

int mg_neighbour_pad(const int* row_ptr, const int* dst, int batch, int nodes, int neighboursmax,
                     int* neighbours, int* counts, mg_stream_t stream) {
    MG_REQUIRE(batch >= 0 && nodes >= 0 && neighboursmax >= 0, "mg_neighbour_pad: negative size");
    const long A = (long)batch * nodes;
    if (A == 0) return MG_OK;
    MG_REQUIRE(row_ptr && counts && (neighboursmax == 0 || neighbours), "mg_neighbour_pad: null pointer");
    hipLaunchKernelGGL(pad_kernel, dim3((unsigned)ceil_div(A * kWave, 256)), dim3(256), 0, (hipStream_t)stream,
                       row_ptr, dst, A, nodes, neighboursmax, neighbours, counts);
    return check_launch("mg_neighbour_pad");
}

int mg_padded_edges_read(const int* counts, const int* neighbours, const float* x, int batch, int nodes,
                         int neighboursmax, int chan, float* edge_data, mg_stream_t stream) {
    MG_REQUIRE(batch >= 0 && nodes >= 0 && neighboursmax >= 0 && chan >= 0, "mg_padded_edges_read: negative size");
    const long A = (long)batch * nodes, total = A * neighboursmax * chan;
    if (total == 0) return MG_OK;
    MG_REQUIRE(counts && neighbours && x && edge_data, "mg_padded_edges_read: null pointer");
    const long blocks = ceil_div(total, 256);
    hipLaunchKernelGGL(padded_read_kernel, dim3((unsigned)(blocks < 65536 * 16 ? blocks : 65536 * 16)), dim3(256), 0,
                       (hipStream_t)stream, counts, neighbours, x, A, nodes, neighboursmax, chan, edge_data);
    return check_launch("mg_padded_edges_read");
}

int mg_padded_edges_reduce(const int* counts, const float* edge_data, int batch, int nodes, int neighboursmax,
                           int chan, float* out, mg_stream_t stream) {
    MG_REQUIRE(batch >= 0 && nodes >= 0 && neighboursmax >= 0 && chan >= 0, "mg_padded_edges_reduce: negative size");
    const long A = (long)batch * nodes, total = A * chan;
    if (total == 0) return MG_OK;
    MG_REQUIRE(counts && out && (neighboursmax == 0 || edge_data), "mg_padded_edges_reduce: null pointer");
    const long blocks = ceil_div(total, 256);
    hipLaunchKernelGGL(padded_reduce_kernel, dim3((unsigned)(blocks < 65536 * 16 ? blocks : 65536 * 16)), dim3(256),
                       0, (hipStream_t)stream, counts, edge_data, A, neighboursmax, chan, out);
    return check_launch("mg_padded_edges_reduce");
}

int mg_edge_vectors(const float* x, const int* src, const int* dst, long n_edges, float box_x, float box_y,
                    float box_z, float* r_ij, int8_t* shift, mg_stream_t stream) {
    MG_REQUIRE(n_edges >= 0, "mg_edge_vectors: negative n_edges");
    if (n_edges == 0) return MG_OK;
    MG_REQUIRE(x && src && dst && r_ij, "mg_edge_vectors: null pointer");
    MG_REQUIRE(box_x > 0.f && box_y > 0.f && box_z > 0.f, "mg_edge_vectors: box must be positive");
    hipLaunchKernelGGL(edge_vectors_kernel, dim3((unsigned)ceil_div(n_edges, 256)), dim3(256), 0,
                       (hipStream_t)stream, x, src, dst, n_edges, box_x, box_y, box_z, r_ij, shift);
    return check_launch("mg_edge_vectors");
}

}  // extern "C"
