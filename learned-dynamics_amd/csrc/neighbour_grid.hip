// Periodic cell-list radius graph for gfx950.
//
// Pipeline (all on the caller's stream, no allocation, no host sync):
//   bin      wrap each atom into the box, cell id
//   sort     up to 16 workgroups per box, each sorting a slab of the box's cells:
//            counting sort by cell in LDS (histogram, scan, placement, rank by
//            atom id inside the cell, so that the cell-ordered array, and with it
//            every output row, is deterministic) -> cell_start.
//            Boxes of more than 16384 atoms or 4096 cells take four kernels instead
//            (histogram with global atomics, scan, place, order)
//   count    one workgroup per home cell: the 27 window cells are staged in LDS
//            once, each wave takes home atoms and sweeps the staged candidates
//            64 at a time, counting hits with ballot/popcount -> degree; the hits
//            themselves go, in window order, into the atom's row of a scratch
//            array (hit rows of a fixed capacity)
//   scan     degrees -> CSR row_ptr (+ per-box edge counts, statistics)
//   fill     copies the hit rows to row_ptr[i] (exact-size rows, no atomics per
//            edge, no geometry); a row with more hits than a hit row holds is
//            swept again by one wave
//
// fp32 recipe (this file is compiled with -ffp-contract=off):
//   w    = remainderf(x - box/2, box) + box/2                 (IEEE remainder)
//   cell = (int)(((float)ndiv * w) / box) % ndiv              (correctly rounded divide)
//   d    = remainder(w_i - w_j, box) per axis, evaluated as fma(-rint(t / box), box, t)
//          (|w_i - w_j| <= box, so the multiple is -1, 0 or 1 and the result is exact;
//          see count_kernel for why quotients within rounding of 1/2 do not matter)
//   d2   = fma(dz,dz, fma(dy,dy, dx*dx)) <= cutoff*cutoff, i != j
//   only the periodic 3x3x3 cell window is searched, with ndiv = ceil(box/cutoff):
//   when box/cutoff is not an integer the cells are narrower than the cutoff and
//   pairs two cells apart are not listed.
#include "common.hpp"
#include <mutex>
#include <type_traits>

namespace mg {
namespace {

// Built-in workspace of mg_neighbour_edges_static, for callers that cannot allocate one.  One copy per GPU, held
// from the moment the library is loaded until the process ends.  Host code never passes `scratch` itself anywhere:
// the name is a host-side handle, the device address comes from hipGetSymbolAddress (scratch_of_current_device).
constexpr size_t kScratchBytes = size_t(64) << 20;
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
constexpr int kCandCapSparse = 512;   // sparse boxes: 1-wave workgroups, 8 KB
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
    int* block_sums;    // scan scratch (cell histogram)
    int* block_max;     // scan scratch
    int* deg_sums;      // sums / maxima of the degrees per tile of kScanTile rows
    int* deg_max;
    int* box_max;       // batch: largest cell occupancy of each box (per-box sort)
    void* hits;         // A x hit_cap: neighbours found by the count pass (box-local atom ids, window order);
                        // 16-bit entries when a box has at most 65536 atoms, else 32-bit
    int hit_cap;        // entries per hit row; rows with more hits are recomputed by the fill pass
    int hit_bytes;      // 2 or 4
    size_t bytes;
};

inline size_t align_up(size_t v) { return (v + 255) & ~size_t(255); }

Workspace carve(void* base, long A, long C, int hit_cap, int hit_bytes) {
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
    w.deg_sums = static_cast<int*>(take(sizeof(int) * scan_blocks));
    w.deg_max = static_cast<int*>(take(sizeof(int) * scan_blocks));
    w.box_max = static_cast<int*>(take(sizeof(int) * (A > 0 ? A : 1)));   // (batch <= A)
    w.hits = take((size_t)hit_bytes * A * hit_cap);
    w.hit_cap = hit_cap;
    w.hit_bytes = hit_bytes;
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
    MG_REQUIRE((long)nd[0] * (batch > 0 ? batch : 1) <= 65535 && nd[1] <= 65535,
               "batch * cells along x (%ld) and cells along y (%d) must not exceed 65535", (long)nd[0] * batch, nd[1]);
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

__device__ __forceinline__ int wave_incl_scan(int v, int lane) {
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        int t = __shfl_up(v, d);
        if (lane >= d) v += t;
    }
    return v;
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

// HIST: also the histogram of cell sizes and each atom's slot in its cell (boxes too large for the per-box sort)
template <bool HIST>
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
    if (HIST) w.slot[a] = atomicAdd(&w.cell_count[cell], 1);
}

// Counting sort of a box by cell, entirely in LDS: histogram (LDS atomics), scan, placement, rank by atom id inside
// the cell.  A box is shared by gridDim.x workgroups: each takes a contiguous range of the box's cells (a slab),
// reads the cell of every atom of the box, counts the atoms of the slabs before its own (its place in the
// cell-ordered array) and sorts the atoms of its own slab.  Replaces the histogram / scan / place / order kernels
// for boxes of at most kSortNodes atoms and kSortCells cells.  Writes cell_start (global positions), sorted,
// box_max[b * slabs + slab].
constexpr int kSortThreads = 1024, kSortNodes = 16384, kSortCells = 4096;   // 2^14 atoms: 14 key bits
constexpr int kSortSlabsMax = 16;
__global__ void __launch_bounds__(kSortThreads) sort_box_kernel(Grid g, Workspace w) {
    constexpr int kPer = kSortNodes / kSortThreads, kCellsPer = kSortCells / kSortThreads;
    // cell sizes, then exclusive starts (start[cells of the slab] = its atoms), then a spare bin per lane
    __shared__ int start[kSortCells + 1 + kWave];
    // keys (cell << 14 | atom) in cell order: a key of a later cell compares greater than any key of this cell, so the
    // rank loop may read past the end of its cell without a bounds check (the array ends in 8 keys of INT_MAX)
    __shared__ int placed[kSortNodes + 8 + 1];   // (+ a spare word that takes the writes for atoms of other slabs)
    __shared__ int wave_sum[kSortThreads / kWave], wave_max[kSortThreads / kWave], wave_before[kSortThreads / kWave];
    const int slab = blockIdx.x, slabs = gridDim.x;
    const int b = blockIdx.y, tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    const long base = (long)b * g.nodes;
    const int cell_base = b * g.ncells;
    const int c_lo = (int)((long)slab * g.ncells / slabs), c_hi = (int)((long)(slab + 1) * g.ncells / slabs);
    const int ncs = c_hi - c_lo;              // cells of this slab
    for (int c = tid; c <= ncs + kWave; c += kSortThreads) start[c] = 0;
    __syncthreads();
    int cl[kPer], sl[kPer];                   // cell within the slab (-1: another slab's atom), slot within the cell
    int n_before = 0;
    // Straight-line code, so that the 16 loads (and then the 16 LDS atomics) of a thread are in flight together:
    // an index past the box reads the box's last atom and is discarded, an atom of another slab counts into a
    // spare bin of its lane.
    const int* cells = w.cell_of + base;
    const int last = g.nodes - 1;
#pragma unroll
    for (int j = 0; j < kPer; j++) {
        const int i = tid + kSortThreads * j;
        const int c = cells[i < g.nodes ? i : last] - cell_base;
        cl[j] = i < g.nodes ? c : g.ncells;
    }
#pragma unroll
    for (int j = 0; j < kPer; j++) {
        const int c = cl[j];
        n_before += c < c_lo ? 1 : 0;
        const bool own = c >= c_lo && c < c_hi;
        cl[j] = own ? c - c_lo : -1;
        sl[j] = atomicAdd(&start[own ? c - c_lo : ncs + 1 + lane], 1);
    }
    for (int d = kWave / 2; d > 0; d >>= 1) n_before += __shfl_xor(n_before, d);
    if (lane == 0) wave_before[wave] = n_before;
    __syncthreads();
    // exclusive scan of the cell sizes: a thread owns kCellsPer consecutive cells
    int cnt[kCellsPer], sum = 0, mx = 0;
#pragma unroll
    for (int k = 0; k < kCellsPer; k++) {
        const int c = tid * kCellsPer + k;
        cnt[k] = c < ncs ? start[c] : 0;
        sum += cnt[k];
        mx = cnt[k] > mx ? cnt[k] : mx;
    }
    const int incl = wave_incl_scan(sum, lane);
    for (int d = kWave / 2; d > 0; d >>= 1) { const int t = __shfl_xor(mx, d); mx = t > mx ? t : mx; }
    if (lane == kWave - 1) wave_sum[wave] = incl;
    if (lane == 0) wave_max[wave] = mx;
    int before = 0;                           // atoms of this box in the slabs before this one
    for (int k = 0; k < kSortThreads / kWave; k++) before += wave_before[k];
    __syncthreads();
    int run = incl - sum;
    for (int k = 0; k < wave; k++) run += wave_sum[k];
    int mine = 0;                             // atoms of this slab
    for (int k = 0; k < kSortThreads / kWave; k++) mine += wave_sum[k];
#pragma unroll
    for (int k = 0; k < kCellsPer; k++) {
        const int c = tid * kCellsPer + k;
        if (c < ncs) {
            start[c] = run;
            w.cell_start[cell_base + c_lo + c] = (int)base + before + run;
        }
        run += cnt[k];
    }
    if (tid == 0) {
        start[ncs] = mine;
        int m = 0;
        for (int k = 0; k < kSortThreads / kWave; k++) m = wave_max[k] > m ? wave_max[k] : m;
        w.box_max[b * slabs + slab] = m;
        if (b == g.batch - 1 && slab == slabs - 1) w.cell_start[(long)g.batch * g.ncells] = g.batch * g.nodes;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kPer; j++) {
        const int i = tid + kSortThreads * j;
        const bool own = cl[j] >= 0;
        const int first = start[own ? cl[j] : 0];
        placed[own ? first + sl[j] : kSortNodes + 8] = (cl[j] << 14) | i;
    }
    if (tid < 8) placed[mine + tid] = 0x7fffffff;
    __syncthreads();
    // position p of the slab holds atom (key & 16383) of cell (key >> 14); its final place is its rank by atom id
    // inside the cell.  Going by position keeps every lane busy (a slab has about gridDim.x times fewer atoms than
    // the box), and the atom's record is requested before the ranking, not after it.
    for (int p = tid; p < mine; p += kSortThreads) {
        const int key = placed[p];
        const int c = key >> 14;
        const float4 rec = w.wrapped[base + (key & (kSortNodes - 1))];
        const int lo = start[c], hi = start[c + 1];
        int rank = 0;
        for (int q0 = lo; q0 < hi; q0 += 8) {          // 8 independent LDS reads per trip, one wait
            int v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = placed[q0 + u];
#pragma unroll
            for (int u = 0; u < 8; u++) rank += v[u] < key ? 1 : 0;
        }
        w.sorted[base + before + lo + rank] = rec;
    }
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

// --- two-kernel exclusive scan of n ints: out[0..n] (out[n] = total) -------

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

// whole scan in one workgroup (n small): out[0..n], optional total / max.  Each lane scans a
// contiguous chunk serially, the chunk totals are scanned across the workgroup once.
constexpr int kScanSmallThreads = 1024;
__global__ void __launch_bounds__(kScanSmallThreads) scan_small_kernel(const int* __restrict__ in, int n,
                                                                       int* __restrict__ out, int* out_total, int* out_max) {
    __shared__ int lds[16];
    const int chunk = (n + kScanSmallThreads) / kScanSmallThreads;          // covers indices 0..n
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
        for (int k = 0; k < kScanSmallThreads / kWave; k++) mm = lds[k] > mm ? lds[k] : mm;
        if (out_total) *out_total = total;
        if (out_max) *out_max = mm;
    }
}

// nodes > 0: also edge_counts[b] = out[(b+1)*nodes] (inclusive prefix of edges per box)
// Every workgroup adds up the sums of the workgroups before it (at most a few thousand values: one strided pass)
// instead of waiting for a third kernel to scan them; workgroup 0 also reduces all of them to the totals.
__global__ void __launch_bounds__(kScanThreads) scan_apply_kernel(const int* __restrict__ in, long n,
                                                                  const int* __restrict__ block_sums,
                                                                  const int* __restrict__ block_max, int nblocks,
                                                                  int* __restrict__ out, int nodes,
                                                                  int* __restrict__ edge_counts, int* out_total,
                                                                  int* out_max, int* out_overflow,
                                                                  const int* __restrict__ box_max, int n_box,
                                                                  int* out_box_max) {
    __shared__ int lds[8];
    __shared__ long long before_lds[kScanThreads / kWave];
    __shared__ int max_lds[kScanThreads / kWave];
    long long before = 0, all = 0;
    int mx = 0;
    const bool totals = blockIdx.x == 0;
    const int upto = totals ? nblocks : (int)blockIdx.x;
    for (int k = threadIdx.x; k < upto; k += kScanThreads) {
        const int v = block_sums[k];
        all += v;
        if (k < (int)blockIdx.x) before += v;
        if (totals) { const int m = block_max[k]; mx = m > mx ? m : mx; }
    }
    for (int d = kWave / 2; d > 0; d >>= 1) {
        before += __shfl_xor(before, d);
        all += __shfl_xor(all, d);
        const int t = __shfl_xor(mx, d);
        mx = t > mx ? t : mx;
    }
    if ((threadIdx.x & (kWave - 1)) == 0) {
        before_lds[threadIdx.x / kWave] = totals ? all : before;
        max_lds[threadIdx.x / kWave] = mx;
    }
    __syncthreads();
    long long sum_w = 0;
    int max_w = 0;
    for (int k = 0; k < kScanThreads / kWave; k++) {
        sum_w += before_lds[k];
        max_w = max_lds[k] > max_w ? max_lds[k] : max_w;
    }
    const int block_offset = totals ? 0 : (int)sum_w;         // (an overflowing total is flagged by workgroup 0)
    if (totals && box_max != nullptr && threadIdx.x < kWave) {
        // largest cell occupancy over the boxes (the per-box sort leaves one value per box)
        int m = 0;
        for (int k = threadIdx.x; k < n_box; k += kWave) m = box_max[k] > m ? box_max[k] : m;
        for (int d = kWave / 2; d > 0; d >>= 1) { const int t = __shfl_xor(m, d); m = t > m ? t : m; }
        if (threadIdx.x == 0) *out_box_max = m;
    }
    if (totals && threadIdx.x == 0) {
        if (out_total) *out_total = sum_w > 0x7fffffffLL ? 0x7fffffff : (int)sum_w;
        if (out_max) *out_max = max_w;
        if (out_overflow) *out_overflow = sum_w > 0x7fffffffLL ? 1 : 0;
    }
    const long base = (long)blockIdx.x * kScanTile + (long)threadIdx.x * kScanItems;
    int v[kScanItems];
    int s = 0;
#pragma unroll
    for (int k = 0; k < kScanItems; k++) {
        v[k] = (base + k < n) ? in[base + k] : 0;
        s += v[k];
    }
    int total;
    int run = block_excl_scan(s, &total, lds) + block_offset;
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


// One workgroup per home cell.  The count pass stages the 27 window cells in LDS once (wrapped positions
// + atom ids), each wave takes home atoms and sweeps the staged candidates 64 at a time; the hits of a
// group go straight into the atom's hit row, behind the hits of the groups before it, so a hit row lists
// the neighbours in window order.  The fill pass is a copy of the hit rows to their places in the edge
// list and never touches the geometry again.  Windows larger than the LDS tile (kCandCap candidates) read
// their tail from global memory.
//
// The hot loop is straight-line code:
//   * the tile is padded to a multiple of 64 with candidates at +infinity (their distance test fails),
//     so no lane checks whether its candidate exists;
//   * a hit row is addressed through a buffer descriptor that covers exactly that row: entries past its
//     capacity are dropped by the bounds check of the store, the count goes on, and the fill pass finds
//     such rows by their degree;
//   * minimum image without compares: remainder(t, box) = t - rint(t / box) box, evaluated as
//     fma(-rint(t * (1 / box)), box, t).  For |t| <= box the multiple is -1, 0 or 1 and the fma is
//     exact, so the result is the IEEE remainder bit for bit unless t / box is within rounding of
//     +-1/2, where the other representative may be chosen; there |result| is about box / 2, which
//     exceeds the cutoff (the grid has at least 3 cells per axis, so box > 2 cutoff): such a pair is
//     listed by neither choice.
//   * a wrapped coordinate lies in [0, box] with BOTH ends possible (remainderf(x - box/2, box) +
//     box/2 gives exactly box for x = box, -box, 3 box, ... and for x within half an ulp below box),
//     and such an atom sits in cell 0 because the cell index is taken modulo ndiv.  Only a home cell
//     whose window holds neither cell 0 nor cell ndiv - 1 on any axis (coordinates 2 .. ndiv - 3,
//     ndiv >= 5) skips the minimum image altogether: there |w_i - w_j| < 2/5 box.
struct Window {
    int M;            // candidates in the 27 cells
    int self_base;    // the home cell's atoms are candidates self_base .. self_base + home_n - 1
    int home_lo, home_n;
};

// First wave: lane t < 27 looks cell t of the window up, a shuffle scan gives the prefix of the lengths.
// Returns false (uniformly) when the home cell is empty.
__device__ __forceinline__ bool window_ranges(const Grid& g, const Workspace& w, int b, int cx, int cy, int cz,
                                              int* range_start, int* range_prefix, Window* win) {
    if (threadIdx.x < kWave) {
        const int lane = threadIdx.x;
        const int t = lane < 27 ? lane : 26;
        const int dx = t / 9 - 1, dy = (t / 3) % 3 - 1, dz = t % 3 - 1;      // divisions by constants: multiplies
        int nx = cx + dx, ny = cy + dy, nz = cz + dz;                        // periodic neighbours without a division
        nx = nx < 0 ? nx + g.nx : (nx >= g.nx ? nx - g.nx : nx);
        ny = ny < 0 ? ny + g.ny : (ny >= g.ny ? ny - g.ny : ny);
        nz = nz < 0 ? nz + g.nz : (nz >= g.nz ? nz - g.nz : nz);
        const int nc = ((b * g.nx + nx) * g.ny + ny) * g.nz + nz;
        const int start = w.cell_start[nc];
        const int len = lane < 27 ? w.cell_start[nc + 1] - start : 0;
        int incl = len;
#pragma unroll
        for (int d = 1; d < 32; d <<= 1) {
            const int up = __shfl_up(incl, d);
            if (lane >= d) incl += up;
        }
        if (lane < 27) {
            range_start[lane] = start;
            range_prefix[lane + 1] = incl;
        }
        if (lane == 0) range_prefix[0] = 0;
    }
    __syncthreads();
    win->M = range_prefix[27];
    win->self_base = range_prefix[13];
    win->home_lo = range_start[13];
    win->home_n = range_prefix[14] - range_prefix[13];
    return win->home_n > 0;
}

// candidate k of the concatenated window -> address in the cell-ordered array
__device__ __forceinline__ int locate(const int* range_start, const int* range_prefix, int k) {
    int lo = 0, hi = 26;   // last range with prefix <= k
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (range_prefix[mid] <= k) lo = mid; else hi = mid - 1;
    }
    return range_start[lo] + (k - range_prefix[lo]);
}

// WRAP: bit 0 / 1 / 2 = apply the minimum image along x / y / z
template <int WRAP>
__device__ __forceinline__ bool within_cutoff(const float4& self, const float4& o, const Grid& g, float ibx, float iby,
                                              float ibz) {
    float dx = self.x - o.x, dy = self.y - o.y, dz = self.z - o.z;
    if (WRAP & 1) dx = __fmaf_rn(-rintf(dx * ibx), g.bx, dx);
    if (WRAP & 2) dy = __fmaf_rn(-rintf(dy * iby), g.by, dy);
    if (WRAP & 4) dz = __fmaf_rn(-rintf(dz * ibz), g.bz, dz);
    const float d2 = __fmaf_rn(dz, dz, __fmaf_rn(dy, dy, dx * dx));
    return d2 <= g.r0sq;
}

// hits below this lane in a ballot, plus `add`
__device__ __forceinline__ int hits_below(unsigned long long mask, int add) {
    return (int)__builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32),
                                          __builtin_amdgcn_mbcnt_lo((unsigned)(mask & 0xffffffffull), (unsigned)add));
}

// HitT: unsigned short (boxes of at most 65536 atoms) or int
__device__ __forceinline__ void store_hit(__amdgpu_buffer_rsrc_t row, int id, int entry, unsigned short) {
    __builtin_amdgcn_raw_buffer_store_b16((short)id, row, entry << 1, 0, 0);
}
__device__ __forceinline__ void store_hit(__amdgpu_buffer_rsrc_t row, int id, int entry, int) {
    __builtin_amdgcn_raw_buffer_store_b32(id, row, entry << 2, 0, 0);
}

template <int kCandCap, typename HitT>
__global__ void __launch_bounds__(256) count_kernel(Grid g, Workspace w) {
    __shared__ float4 cand[kCandCap];
    __shared__ int range_start[27];
    __shared__ int range_prefix[28];

    // grid (nz, ny, nx * batch): the cell coordinates come from the workgroup id without a division chain
    const int cz = blockIdx.x, cy = blockIdx.y;
    const int b = blockIdx.z / g.nx, cx = blockIdx.z - b * g.nx;
    Window win;
    if (!window_ranges(g, w, b, cx, cy, cz, range_start, range_prefix, &win)) return;   // uniform
    const int M = win.M;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), nwaves = blockDim.x / kWave;   // (scalar)

    const int staged = M < kCandCap ? M : kCandCap;
    const int padded = (staged + kWave - 1) & ~(kWave - 1);        // <= kCandCap (a multiple of 64)
    const float inf = __int_as_float(0x7f800000);
    for (int k = threadIdx.x; k < padded; k += blockDim.x)
        cand[k] = k < staged ? w.sorted[locate(range_start, range_prefix, k)] : make_float4(inf, inf, inf, __int_as_float(-1));
    __syncthreads();

    // an axis needs the minimum image unless the window stays clear of cells 0 and ndiv - 1 (see above)
    const int wrap = ((g.nx < 5 || cx < 2 || cx > g.nx - 3) ? 1 : 0) | ((g.ny < 5 || cy < 2 || cy > g.ny - 3) ? 2 : 0) |
                     ((g.nz < 5 || cz < 2 || cz > g.nz - 3) ? 4 : 0);
    const float ibx = 1.0f / g.bx, iby = 1.0f / g.by, ibz = 1.0f / g.bz;
    const int node_base = b * g.nodes;
    const int row_bytes = w.hit_cap * (int)sizeof(HitT);
    HitT* const hits = static_cast<HitT*>(w.hits);

    const int self_base = __builtin_amdgcn_readfirstlane(win.self_base), home_n = __builtin_amdgcn_readfirstlane(win.home_n);
    for (int h = wave; h < home_n; h += nwaves) {
        const int k_self = self_base + h;              // uniform
        float4 self;
        if (k_self < kCandCap) self = cand[k_self];
        else self = w.sorted[win.home_lo + h];
        const int row = node_base + __builtin_amdgcn_readfirstlane(__float_as_int(self.w));
        // descriptor of this atom's hit row alone: a store past the row's capacity is dropped
        const __amdgpu_buffer_rsrc_t hit_row =
            __builtin_amdgcn_make_buffer_rsrc(hits + (long)row * w.hit_cap, 0, row_bytes, 0x00020000);
        // the home atom is itself a candidate and passes the distance test: its bit is taken out of the ballot of
        // its group with scalar instructions (no lane compares ids)
        const int self_group = k_self & ~(kWave - 1);
        const unsigned long long self_clear = ~(1ull << (k_self & (kWave - 1)));
        int running = 0;
        auto sweep = [&](auto wrap_tag) {
            constexpr int kWrap = decltype(wrap_tag)::value;
            for (int k0 = 0; k0 < padded; k0 += kWave) {
                const float4 o = cand[k0 + lane];
                unsigned long long mask = __ballot(within_cutoff<kWrap>(self, o, g, ibx, iby, ibz));
                if (k0 == self_group) mask &= self_clear;
                // (box-local atom ids: the fill pass adds the box's first row)
                if (__builtin_amdgcn_inverse_ballot_w64(mask))
                    store_hit(hit_row, __float_as_int(o.w), hits_below(mask, running), HitT{});
                running += __popcll(mask);
            }
        };
        switch (wrap) {                                // uniform over the workgroup
            case 0: sweep(std::integral_constant<int, 0>{}); break;
            case 1: sweep(std::integral_constant<int, 1>{}); break;
            case 2: sweep(std::integral_constant<int, 2>{}); break;
            case 3: sweep(std::integral_constant<int, 3>{}); break;
            case 4: sweep(std::integral_constant<int, 4>{}); break;
            case 5: sweep(std::integral_constant<int, 5>{}); break;
            case 6: sweep(std::integral_constant<int, 6>{}); break;
            default: sweep(std::integral_constant<int, 7>{}); break;
        }
        // candidates beyond the tile: from global memory
        for (int k0 = kCandCap; k0 < M; k0 += kWave) {
            const int k = k0 + lane;
            bool hit = false;
            int other = 0;
            if (k < M) {
                const float4 o = w.sorted[locate(range_start, range_prefix, k)];
                other = __float_as_int(o.w);
                hit = k != k_self && within_cutoff<7>(self, o, g, ibx, iby, ibz);
            }
            const unsigned long long mask = __ballot(hit);
            if (hit) store_hit(hit_row, other, hits_below(mask, running), HitT{});
            running += __popcll(mask);
        }
        if (lane == 0) w.degree[row] = running;
    }
}

// Fill pass, slow path: one wave sweeps the window of atom `row` again (candidates from global memory, all axes with
// the minimum image) and writes its hits at out_pos, in window order.  For rows whose hit row was too short.
__device__ void refill_row(const Grid& g, const Workspace& w, int row, int out_pos, int capacity,
                           int* __restrict__ src, int* __restrict__ dst) {
    const int lane = threadIdx.x & (kWave - 1);
    const int b = row / g.nodes;
    const int id_self = row - b * g.nodes;
    const int node_base = b * g.nodes;
    const float4 self = w.wrapped[row];
    int c = w.cell_of[row] - b * g.ncells;
    const int cz = c % g.nz;
    c /= g.nz;
    const int cy = c % g.ny, cx = c / g.ny;
    const int t = lane < 27 ? lane : 26;
    const int dx = t / 9 - 1, dy = (t / 3) % 3 - 1, dz = t % 3 - 1;
    int nx = cx + dx, ny = cy + dy, nz = cz + dz;
    nx = nx < 0 ? nx + g.nx : (nx >= g.nx ? nx - g.nx : nx);
    ny = ny < 0 ? ny + g.ny : (ny >= g.ny ? ny - g.ny : ny);
    nz = nz < 0 ? nz + g.nz : (nz >= g.nz ? nz - g.nz : nz);
    const int nc = ((b * g.nx + nx) * g.ny + ny) * g.nz + nz;
    const int start = w.cell_start[nc];
    const int len = lane < 27 ? w.cell_start[nc + 1] - start : 0;
    const int incl = wave_incl_scan(len, lane);
    const int excl = incl - len;                       // lane t < 27: candidates before cell t of the window
    const int M = __shfl(incl, 26);
    const float ibx = 1.0f / g.bx, iby = 1.0f / g.by, ibz = 1.0f / g.bz;
    int cnt = 0;
    for (int k0 = 0; k0 < M; k0 += kWave) {
        const int k = k0 + lane;
        int lo = 0, hi = 26;                           // last cell of the window with excl <= k (5 halvings of 27)
#pragma unroll
        for (int it = 0; it < 5; it++) {
            const int mid = (lo + hi + 1) >> 1;
            const int pm = __shfl(excl, mid);
            if (pm <= k) lo = mid; else hi = mid - 1;
        }
        const int st = __shfl(start, lo), ex = __shfl(excl, lo);
        bool hit = false;
        int other = 0;
        if (k < M) {
            const float4 o = w.sorted[st + (k - ex)];
            other = __float_as_int(o.w);
            hit = other != id_self && within_cutoff<7>(self, o, g, ibx, iby, ibz);
        }
        const unsigned long long mask = __ballot(hit);
        const int pos = out_pos + hits_below(mask, cnt);
        if (hit && pos >= 0 && pos < capacity) {
            src[pos] = row;
            dst[pos] = node_base + other;
        }
        cnt += __popcll(mask);
    }
}

// Fill pass: a workgroup takes kFillRows consecutive rows, whose edges are one contiguous range of the edge list; a
// thread takes every 256th edge of the range, finds its row among the staged row starts and copies one entry of
// that row's hits.  Edges beyond the capacity are dropped.
constexpr int kFillRows = 64;
template <typename HitT>
__global__ void __launch_bounds__(256) fill_kernel(Grid g, Workspace w, const int* __restrict__ row_ptr,
                                                   int* __restrict__ src, int* __restrict__ dst, int capacity) {
    __shared__ int rp[kFillRows + 1];
    __shared__ int first_row[kFillRows];      // first row of the box that the row belongs to
    const long A = (long)g.batch * g.nodes;
    const long r0 = (long)blockIdx.x * kFillRows;
    const int nrows = A - r0 < kFillRows ? (int)(A - r0) : kFillRows;
    if ((int)threadIdx.x <= nrows) rp[threadIdx.x] = row_ptr[r0 + threadIdx.x];
    if ((int)threadIdx.x < nrows) first_row[threadIdx.x] = (int)((r0 + threadIdx.x) / g.nodes) * g.nodes;
    __syncthreads();
    const int cap = w.hit_cap;
    const HitT* __restrict__ hits = static_cast<const HitT*>(w.hits);
    const int e_hi = rp[nrows];
    for (int e = rp[0] + (int)threadIdx.x; e < e_hi; e += 256) {
        int lo = 0, hi = nrows - 1;                    // last row with rp <= e (6 halvings of 64)
#pragma unroll
        for (int it = 0; it < 6; it++) {
            const int mid = (lo + hi + 1) >> 1;
            if (rp[mid] <= e) lo = mid; else hi = mid - 1;
        }
        const int idx = e - rp[lo], deg = rp[lo + 1] - rp[lo];
        if (deg <= cap && idx >= 0 && idx < deg && e >= 0 && e < capacity) {
            src[e] = (int)(r0 + lo);
            dst[e] = first_row[lo] + (int)hits[(r0 + lo) * cap + idx];
        }
    }
    // rows with more hits than a hit row holds: a wave each
    const int wave = threadIdx.x / kWave;
    for (int r = wave; r < nrows; r += 256 / kWave)
        if (rp[r + 1] - rp[r] > cap) refill_row(g, w, (int)(r0 + r), rp[r], capacity, src, dst);
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
        hipLaunchKernelGGL(scan_small_kernel, dim3(1), dim3(kScanSmallThreads), 0, st, in, (int)n, out, out_total, out_max);
        return check_launch("neighbour scan");
    }
    const int nblocks = (int)ceil_div(n + 1, kScanTile);
    hipLaunchKernelGGL(scan_sums_kernel, dim3(nblocks), dim3(kScanThreads), 0, st, in, n, w.block_sums, w.block_max);
    hipLaunchKernelGGL(scan_apply_kernel, dim3(nblocks), dim3(kScanThreads), 0, st, in, n, w.block_sums, w.block_max,
                       nblocks, out, nodes, edge_counts, out_total, out_max, out_overflow, (const int*)nullptr, 0,
                       (int*)nullptr);
    return check_launch("neighbour scan");
}

// The graph truncated at `capacity` edges: row pointers and per-box counts above the capacity are lowered to it, so
// that every kernel that walks the edges through row_ptr stays inside edge arrays of that many entries.  stats[0]
// keeps the true count; bit 1 of stats[3] says that edges were dropped.
__global__ void __launch_bounds__(256) clamp_row_ptr_kernel(int* __restrict__ row_ptr, long n_ptr,
                                                            int* __restrict__ edge_counts, int batch, int capacity,
                                                            int* __restrict__ stats) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_ptr && row_ptr[i] > capacity) row_ptr[i] = capacity;
    if (i < batch && edge_counts[i] > capacity) edge_counts[i] = capacity;
    if (i == 0 && stats[0] > capacity) stats[3] |= 2;
}

int pairs_block_size(const Grid& g);
// workgroups that share the sort of one box: one per 1024 atoms (box_max has batch * nodes entries, so slabs <= nodes)
int sort_slabs(const Grid& g) {
    const int s = g.nodes / 1024;
    return s < 1 ? 1 : (s > kSortSlabsMax ? kSortSlabsMax : s);
}
// one workgroup per cell, laid out so that the kernels read the cell coordinates off the workgroup id
dim3 cell_grid(const Grid& g) { return dim3((unsigned)g.nz, (unsigned)g.ny, (unsigned)(g.nx * g.batch)); }
// Hit rows.  An entry is a box-local atom id: 16 bits when a box has at most 65536 atoms.  The host knows the mean
// density only, and a row that is too short costs a second sweep of the atom's window in the fill pass, so a row has
// kHitCapMax entries (enough for any density short of a dense liquid with a long cutoff: 512 bytes of address space
// per atom, of which a search touches what its neighbour counts need) whenever the workspace is as large as
// mg_neighbour_workspace_bytes says; a smaller workspace (the library's built-in one) gets the longest rows that
// fit, down to kHitCapMin entries.  Count, fill and cell-order calls derive the same layout from the same
// (batch, nodes, box, workspace size).
constexpr int kHitCapMax = 256, kHitCapMin = 32;
int hit_entry_bytes(const Grid& g) { return g.nodes <= 65536 ? 2 : 4; }

// Workspace layout for a buffer of `workspace_bytes` (0: the preferred size).  Returns false when not even the
// shortest rows fit; *needed is then the smallest size that works.
bool layout(const Grid& g, void* base, size_t workspace_bytes, Workspace* w, size_t* needed) {
    const long A = (long)g.batch * g.nodes, C = (long)g.batch * g.ncells;
    const int eb = hit_entry_bytes(g);
    int cap = kHitCapMax;
    if (workspace_bytes != 0 && A > 0) {
        const size_t fixed = carve(nullptr, A, C, 0, eb).bytes + 512;      // alignment of the base and of the rows
        const size_t room = workspace_bytes > fixed ? workspace_bytes - fixed : 0;
        long fit = (long)(room / ((size_t)eb * (size_t)A));
        fit &= ~7L;                                     // rows stay 16-byte aligned
        if (fit < kHitCapMin) {
            if (needed) *needed = carve(nullptr, A, C, kHitCapMin, eb).bytes + 256;
            return false;
        }
        cap = fit < kHitCapMax ? (int)fit : kHitCapMax;
    }
    *w = carve(base, A, C, cap, eb);
    if (workspace_bytes != 0 && w->bytes + 256 > workspace_bytes) {     // (A == 0: the fixed arrays alone)
        if (needed) *needed = w->bytes + 256;
        return false;
    }
    return true;
}

int pairs_block_size(const Grid& g) {
    // sparse boxes: one wave per cell and a tile of 256 candidates are plenty (10 % faster than four waves at 1.2
    // atoms per cell).  Only the mean is known here: 16384 atoms clumped in a ball inside a box of 8000 cells (2 per
    // cell on average, 22 where they are) overflow that tile and take 0.30 ms with one wave against 0.18 ms with four,
    // hence the low threshold.
    const double mean_occ = (double)g.nodes / (double)g.ncells;
    return mean_occ <= 2.0 ? 64 : 256;
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
    Workspace w;
    layout(g, nullptr, 0, &w, nullptr);
    *bytes = w.bytes + 256;
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
    Workspace w;
    size_t needed = 0;
    if (workspace_bytes == 0 || !layout(g, base, workspace_bytes, &w, &needed))
        return fail(MG_ERR_WORKSPACE, "mg_neighbour_count: workspace has %zu bytes, at least %zu needed", workspace_bytes,
                    needed);
    hipStream_t st = (hipStream_t)stream;
    if (A == 0) {
        hipLaunchKernelGGL(zero3_kernel, dim3(1), dim3(256), 0, st, stats, 4L, row_ptr, 1L, edge_counts, (long)batch);
        return check_launch("mg_neighbour_count");
    }
    MG_REQUIRE(x != nullptr, "mg_neighbour_count: x is null");
    const unsigned ablocks = (unsigned)ceil_div(A, 256);
    const int deg_tiles = (int)ceil_div(A + 1, kScanTile);
    const bool per_box_sort = nodes <= kSortNodes && g.ncells <= kSortCells;
    if (per_box_sort) {
        // six launches in all: bin, per-box sort, count, two for the scan of the degrees, fill
        hipLaunchKernelGGL(bin_kernel<false>, dim3(ablocks), dim3(256), 0, st, x, g, w);
        hipLaunchKernelGGL(sort_box_kernel, dim3((unsigned)sort_slabs(g), (unsigned)batch), dim3(kSortThreads), 0, st, g, w);
    } else {
        hipLaunchKernelGGL(zero3_kernel, dim3((unsigned)(ceil_div(C, 256) < 1024 ? ceil_div(C, 256) : 1024)), dim3(256),
                           0, st, (int*)nullptr, 0L, row_ptr, 1L, w.cell_count, C);    // (every word of stats is stored below)
        hipLaunchKernelGGL(bin_kernel<true>, dim3(ablocks), dim3(256), 0, st, x, g, w);
        if (int s = run_scan(w.cell_count, C, w.cell_start, w, nullptr, stats + 1, nullptr, st)) return s;
        hipLaunchKernelGGL(place_kernel, dim3(ablocks), dim3(256), 0, st, g, w);
        hipLaunchKernelGGL(order_kernel, dim3(ablocks), dim3(256), 0, st, g, w);
    }
    const bool narrow = w.hit_bytes == 2;
    if (pairs_block_size(g) == 64) {
        if (narrow) hipLaunchKernelGGL((count_kernel<kCandCapSparse, unsigned short>), cell_grid(g), dim3(64), 0, st, g, w);
        else hipLaunchKernelGGL((count_kernel<kCandCapSparse, int>), cell_grid(g), dim3(64), 0, st, g, w);
    } else {
        if (narrow) hipLaunchKernelGGL((count_kernel<kCandCapDense, unsigned short>), cell_grid(g), dim3(256), 0, st, g, w);
        else hipLaunchKernelGGL((count_kernel<kCandCapDense, int>), cell_grid(g), dim3(256), 0, st, g, w);
    }
    hipLaunchKernelGGL(scan_sums_kernel, dim3((unsigned)deg_tiles), dim3(kScanThreads), 0, st, (const int*)w.degree, A,
                       w.deg_sums, w.deg_max);
    hipLaunchKernelGGL(scan_apply_kernel, dim3((unsigned)deg_tiles), dim3(kScanThreads), 0, st, (const int*)w.degree, A,
                       (const int*)w.deg_sums, (const int*)w.deg_max, deg_tiles, row_ptr, nodes, edge_counts, stats + 0,
                       stats + 2, stats + 3, per_box_sort ? (const int*)w.box_max : (const int*)nullptr, batch * sort_slabs(g), stats + 1);
    return check_launch("mg_neighbour_count");
}

int mg_neighbour_fill(const void* workspace, size_t workspace_bytes, int batch, int nodes, float cutoff,
                      float box_x, float box_y, float box_z, const int* row_ptr, int n_edges, int* src,
                      int* dst, mg_stream_t stream) {
    Grid g;
    if (int s = make_grid(cutoff, box_x, box_y, box_z, batch, nodes, &g)) return s;
    MG_REQUIRE(n_edges >= 0, "mg_neighbour_fill: negative n_edges");
    const long A = (long)batch * nodes;
    if (A == 0 || n_edges == 0) return MG_OK;
    MG_REQUIRE(workspace && row_ptr && src && dst, "mg_neighbour_fill: null pointer");
    void* base = reinterpret_cast<void*>((reinterpret_cast<uintptr_t>(workspace) + 255) & ~uintptr_t(255));
    Workspace w;
    size_t needed = 0;
    if (workspace_bytes == 0 || !layout(g, base, workspace_bytes, &w, &needed))
        return fail(MG_ERR_WORKSPACE, "mg_neighbour_fill: workspace has %zu bytes, at least %zu needed", workspace_bytes,
                    needed);
    if (w.hit_bytes == 2)
        hipLaunchKernelGGL(fill_kernel<unsigned short>, dim3((unsigned)ceil_div(A, kFillRows)), dim3(256), 0,
                           (hipStream_t)stream, g, w, row_ptr, src, dst, n_edges);
    else
        hipLaunchKernelGGL(fill_kernel<int>, dim3((unsigned)ceil_div(A, kFillRows)), dim3(256), 0, (hipStream_t)stream, g,
                           w, row_ptr, src, dst, n_edges);
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
    if (int s = mg_neighbour_fill(workspace, workspace_bytes, batch, nodes, cutoff, box_x, box_y, box_z, row_ptr,
                                  capacity, src, dst, stream))
        return s;
    const long n_ptr = (long)batch * nodes + 1;
    if (n_ptr == 1) return MG_OK;
    // after the fill pass (which places edges by the exact row_ptr): the caller's view is the graph cut at capacity
    hipLaunchKernelGGL(clamp_row_ptr_kernel, dim3((unsigned)ceil_div(n_ptr, 256)), dim3(256), 0, (hipStream_t)stream,
                       row_ptr, n_ptr, edge_counts, batch, capacity, stats);
    return check_launch("mg_neighbour_edges");
}

int mg_neighbour_edges_static(const float* x, int batch, int nodes, float cutoff, float box_x, float box_y,
                              float box_z, int* row_ptr, int* edge_counts, int* stats, int capacity, int* src,
                              int* dst, mg_stream_t stream) {
    Grid g;
    if (int s = make_grid(cutoff, box_x, box_y, box_z, batch, nodes, &g)) return s;
    Workspace probe;
    size_t need = 0;
    if (!layout(g, nullptr, kScratchBytes, &probe, &need))
        return fail(MG_ERR_WORKSPACE,
                    "mg_neighbour_edges_static: this search needs at least %zu bytes of workspace (%zu per atom), the "
                    "built-in one holds %zu; use mg_neighbour_edges with a workspace of your own",
                    need, need / (size_t)((long)batch * nodes > 0 ? (long)batch * nodes : 1), kScratchBytes);
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
    const long A = (long)batch * nodes;
    if (A == 0) return MG_OK;
    MG_REQUIRE(workspace && order, "mg_neighbour_cell_order: null pointer");
    void* base = reinterpret_cast<void*>((reinterpret_cast<uintptr_t>(workspace) + 255) & ~uintptr_t(255));
    Workspace w;
    size_t needed = 0;
    if (workspace_bytes == 0 || !layout(g, base, workspace_bytes, &w, &needed))
        return fail(MG_ERR_WORKSPACE, "mg_neighbour_cell_order: workspace has %zu bytes, at least %zu needed",
                    workspace_bytes, needed);
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
