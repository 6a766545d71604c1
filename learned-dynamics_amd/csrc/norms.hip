// Node-level pieces of the layers that call the hot path: group norms over the
// atoms of a box, the tensor squash, the elementwise parts of the PaiNN update, and
// the remaining radial encodings.  All HBM-bound streaming over node-sized (or, for
// the encodings, edge-sized) arrays; the norms need one box-wide reduction each.
//
// Reductions are deterministic: workgroup partials in a caller-provided scratch
// array (fp64), folded in a fixed order by the apply kernel.
#include "common.hpp"

namespace mg {
namespace {

constexpr int kChunks = 64;   // partial sums per (box, group)

__device__ __forceinline__ double block_sum(double v, double* lds) {
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) v += __shfl_xor(v, d);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) lds[wave] = v;
    __syncthreads();
    double t = 0.0;
    for (int k = 0; k < (int)(blockDim.x / kWave); k++) t += lds[k];
    return t;
}

// x element (box b, node i, channel c, comp t) at x[((b*N + i)*x_stride + c)*T + t]; optional elementwise
// multiplier mul at the same index pattern with mul_stride.  partial[(b*G + g)*kChunks + chunk][0..1] =
// (sum, sum of squares) over that chunk's nodes, the group's channels and all components.
// A group's channels and components of one node are cg*T consecutive floats, so an element is addressed by its
// node and its offset in that run; both advance by constants from one trip to the next (no division per element).
__global__ void __launch_bounds__(256) group_stats_kernel(const float* __restrict__ x, long x_stride,
                                                          const float* __restrict__ mul, long mul_stride, int N,
                                                          int chan, int groups, int T, double* __restrict__ partial) {
    __shared__ double lds[8];
    const int bg = blockIdx.x, chunk = blockIdx.y;
    const int b = bg / groups, g = bg - b * groups;
    const int cg = chan / groups;
    const int per = (N + kChunks - 1) / kChunks;
    const int n_lo = chunk * per, n_hi = n_lo + per < N ? n_lo + per : N;
    const int run = cg * T;
    const int step_i = (int)blockDim.x / run, step_r = (int)blockDim.x % run;
    int i = n_lo + (int)threadIdx.x / run, r = (int)threadIdx.x % run;
    const float* xg = x + (long)g * cg * T;
    const float* mul_g = mul ? mul + (long)g * cg * T : nullptr;
    const long x_row = x_stride * T, m_row = mul_stride * T;
    double s = 0.0, ss = 0.0;
    // four trips' loads are requested before the first is used (a trip alone waits out the memory latency); a trip
    // past the end re-reads the chunk's last node and counts as zero
    constexpr int kAhead = 4;
    while (i < n_hi) {
        float v[kAhead], m[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; u++) {
            const bool live = i < n_hi;
            const long row = (long)b * N + (live ? i : n_hi - 1);
            v[u] = xg[row * x_row + r];
            m[u] = mul_g ? mul_g[row * m_row + r] : 1.0f;
            if (!live) m[u] = 0.f;
            i += step_i;
            r += step_r;
            if (r >= run) { r -= run; i++; }
        }
#pragma unroll
        for (int u = 0; u < kAhead; u++) {
            const float w = v[u] * m[u];
            s += w;
            ss += (double)w * w;
        }
    }
    const double ts = block_sum(s, lds);
    const double tss = block_sum(ss, lds);
    if (threadIdx.x == 0) {
        partial[((long)bg * kChunks + chunk) * 2] = ts;
        partial[((long)bg * kChunks + chunk) * 2 + 1] = tss;
    }
}

// fold the kChunks partials of every (box, group) in a fixed order and derive what the apply kernel uses:
// partial[bg*kChunks*2 + {0,1}] <- totals, + 2 <- the mean that is subtracted (0 for the tensor norm),
// + 3 <- the denominator sqrt(eps + variance or mean square); both rounded to float as the apply kernel takes them
__global__ void group_finalize_kernel(double* __restrict__ partial, int n_bg, double count, int mode, float eps) {
    const int bg = blockIdx.x * blockDim.x + threadIdx.x;
    if (bg >= n_bg) return;
    double* p = partial + (long)bg * kChunks * 2;
    double s = 0.0, ss = 0.0;
    for (int k = 0; k < kChunks; k++) { s += p[2 * k]; ss += p[2 * k + 1]; }
    p[0] = s;
    p[1] = ss;
    if (mode == 0) {
        p[2] = 0.0;
        p[3] = (double)sqrtf(eps + (float)(ss / count));          // mean over nodes, group channels of sum_comp v^2
    } else {
        const double mean = s / count;
        double var = ss / count - mean * mean;
        var = var > 0.0 ? var : 0.0;
        p[2] = (double)(float)mean;
        p[3] = (double)sqrtf(eps + (float)var);
    }
}

// mode 0 (TensGroupNorm): y = gamma[c] * v / sqrt(eps + mean(sum_comp v^2))
// mode 1 (ScalGroupNorm, T = 1): y = beta[c] + gamma[c] * (v - mean) / sqrt(eps + var)
// then y += add (optional, add_stride) and y += res (optional, same layout as out).
// A thread keeps one (channel, component) position k = c*T + comp of the rows of box blockIdx.z and walks over
// nodes: channel, group, gamma, beta and the group's statistics are fixed per thread, consecutive threads touch
// consecutive floats.
__global__ void __launch_bounds__(256) group_apply_kernel(const float* __restrict__ x, long x_stride,
                                                          const float* __restrict__ mul, long mul_stride,
                                                          const double* __restrict__ partial, int N, int chan,
                                                          int groups, int T, int mode,
                                                          const float* __restrict__ gamma, const float* __restrict__ beta,
                                                          const float* __restrict__ add, long add_stride,
                                                          const float* __restrict__ res, float* __restrict__ out) {
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    const int CT = chan * T;
    if (k >= CT) return;
    const int b = blockIdx.z;
    const int c = k / T, g = c / (chan / groups);
    const double* p = partial + ((long)(b * groups + g) * kChunks) * 2;
    const float mean = (float)p[2], denom = (float)p[3];
    const float ga = gamma[c], be = mode == 0 ? 0.f : beta[c];
    const long x_row = x_stride * T, m_row = mul_stride * T, a_row = add_stride * T;
    for (int i = blockIdx.y; i < N; i += gridDim.y) {
        const long row = (long)b * N + i;
        float v = x[row * x_row + k];
        if (mul) v *= mul[row * m_row + k];
        float y = mode == 0 ? ga * (v / denom) : be + ga * ((v - mean) / denom);
        if (add) y += add[row * a_row + k];
        if (res) y += res[row * CT + k];
        out[row * CT + k] = y;
    }
}

// x / sqrt(1 + sum_comp x^2) per (row, chan)
__global__ void __launch_bounds__(256) tens_sigmoid_kernel(const float* __restrict__ x, long n, int T,
                                                           float* __restrict__ out) {
    for (long e = (long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (long)gridDim.x * blockDim.x) {
        float v[9], q = 0.f;
        for (int t = 0; t < T; t++) { v[t] = x[e * T + t]; q += v[t] * v[t]; }
        const float inv = 1.0f / sqrtf(1.0f + q);
        for (int t = 0; t < T; t++) out[e * T + t] = v[t] * inv;
    }
}

// PaiNN Update, first elementwise stage: lrv = [lin_l | lin_r | lin_v](x_v), stored (rows, 3n, 3) or, COMP_MAJOR,
// (rows, 3, 3n) (what the GEMM stores at full rate, and what a wave reads here with unit stride)
//   ip[r,c] = sum_x l[c,x] r[c,x];  cat[r] = [x_a[r] | |r[c]|]   (rows, 2n)
// One workgroup row per node row: blockIdx.x = r, the channel from blockIdx.y and the thread.
template <bool COMP_MAJOR>
__device__ __forceinline__ float lrv_at(const float* __restrict__ row, int n, int j, int x) {
    return COMP_MAJOR ? row[x * 3 * n + j] : row[j * 3 + x];
}

// cat_rowmax (rows; or null): max |cat[r, :]|, the row bound of the MLP that reads cat; written when one workgroup
// covers a row (n <= 256: gridDim.y == 1)
template <bool COMP_MAJOR>
__global__ void __launch_bounds__(256) painn_update_pre_kernel(const float* __restrict__ lrv, const float* __restrict__ x_a,
                                                               int n, float* __restrict__ ip, float* __restrict__ cat,
                                                               float* __restrict__ cat_rowmax) {
    __shared__ float wave_max[4];
    const long r = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    float mx = 0.f;
    if (c < n) {
        const float* row = lrv + r * 9 * n;
        float l[3], rr[3];
#pragma unroll
        for (int x = 0; x < 3; x++) { l[x] = lrv_at<COMP_MAJOR>(row, n, c, x); rr[x] = lrv_at<COMP_MAJOR>(row, n, n + c, x); }
        ip[r * n + c] = l[0] * rr[0] + l[1] * rr[1] + l[2] * rr[2];
        const float a = x_a[r * n + c], nr = sqrtf(rr[0] * rr[0] + rr[1] * rr[1] + rr[2] * rr[2]);
        cat[r * 2 * n + c] = a;
        cat[r * 2 * n + n + c] = nr;
        mx = fmaxf(fabsf(a), nr);
    }
    if (cat_rowmax) {                                         // uniform over the workgroup
        for (int d = 1; d < kWave; d <<= 1) mx = fmaxf(mx, __shfl_xor(mx, d));
        if ((threadIdx.x & (kWave - 1)) == 0) wave_max[threadIdx.x / kWave] = mx;
        __syncthreads();
        if (threadIdx.x == 0) {
            for (int w = 1; w < (int)(blockDim.x / kWave); w++) mx = fmaxf(mx, wave_max[w]);
            cat_rowmax[r] = mx;
        }
    }
}

// PaiNN Update, vector output: v = lin_v(x_v) * y[0:n]; out = res_v + v / sqrt(1 + |v|^2), out (rows, n, 3)
template <bool COMP_MAJOR>
__global__ void __launch_bounds__(256) painn_update_vec_kernel(const float* __restrict__ lrv, const float* __restrict__ y,
                                                               const float* __restrict__ res_v, int n,
                                                               float* __restrict__ out_v) {
    const long r = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= n) return;
    const float* row = lrv + r * 9 * n;
    const float s = y[r * 3 * n + c];
    const float a = lrv_at<COMP_MAJOR>(row, n, 2 * n + c, 0) * s, b = lrv_at<COMP_MAJOR>(row, n, 2 * n + c, 1) * s,
                d = lrv_at<COMP_MAJOR>(row, n, 2 * n + c, 2) * s;
    const float inv = 1.0f / sqrtf(1.0f + (a * a + b * b + d * d));
    float o0 = a * inv, o1 = b * inv, o2 = d * inv;
    const long t = r * n + c;
    if (res_v) { o0 += res_v[3 * t]; o1 += res_v[3 * t + 1]; o2 += res_v[3 * t + 2]; }
    out_v[3 * t] = o0; out_v[3 * t + 1] = o1; out_v[3 * t + 2] = o2;
}

// kinds: 1 sq_radial_encode of normed_sq_dist (archs/diffuser_atoms14.py:32-48)
//        2 radial_encode_edge (archs/diffuser_atoms5.py:25-30)
__global__ void __launch_bounds__(256) radial_encode_kernel(int kind, const float* __restrict__ r_ij, long E, int n,
                                                            float rmax, float c0, float c1, float* __restrict__ out) {
    const long total = E * n;
    for (long t = (long)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (long)gridDim.x * blockDim.x) {
        const long e = t / n;
        const int m = (int)(t - e * n);
        const float x = r_ij[3 * e], y = r_ij[3 * e + 1], z = r_ij[3 * e + 2];
        const float sq = x * x + y * y + z * z;
        if (kind == 1) {
            const float q = sq / (rmax * rmax);
            const float h = sqrtf(1.0f + q);
            const float coeff = c0 * expf(c1 * (float)m);        // (pi / sqrt 2) exp(n^-0.7 m)
            out[t] = sinf(coeff * h) * (0.70710678118654752f - h);
        } else {
            const float q = sq / rmax;                             // divided by rmax, not rmax^2, as in the reference
            const float cut = fmaxf(1.0f - q, 0.0f);
            out[t] = cosf((c0 * (float)m) * sqrtf(q)) * cut;      // c0 = pi
        }
    }
}

long grid_for(long total) {
    long b = ceil_div(total, 256);
    return b > 256L * 32 ? 256L * 32 : (b < 1 ? 1 : b);
}

}  // namespace
}  // namespace mg

using namespace mg;

extern "C" {

int mg_group_norm_scratch_bytes(int batch, int groups, size_t* bytes) {
    MG_REQUIRE(bytes && batch >= 0 && groups >= 0, "mg_group_norm_scratch_bytes: bad argument");
    *bytes = (size_t)batch * groups * kChunks * 2 * sizeof(double);
    return MG_OK;
}

int mg_group_norm(int mode, const float* x, long x_stride, const float* mul, long mul_stride, int batch, int nodes,
                  int chan, int groups, int comps, float eps, const float* gamma, const float* beta, const float* add,
                  long add_stride, const float* res, void* scratch, float* out, mg_stream_t stream) {
    MG_REQUIRE(mode == 0 || mode == 1, "mg_group_norm: mode must be 0 (tensor) or 1 (scalar)");
    MG_REQUIRE(batch >= 0 && nodes >= 0 && chan >= 0 && groups > 0 && chan % groups == 0, "mg_group_norm: bad sizes");
    MG_REQUIRE(comps == 1 || comps == 3 || comps == 9, "mg_group_norm: comps must be 1, 3 or 9");
    MG_REQUIRE(mode == 0 || comps == 1, "mg_group_norm: the scalar norm takes comps == 1");
    const long total = (long)batch * nodes * chan * comps;
    if (total == 0) return MG_OK;
    MG_REQUIRE(x && gamma && out && scratch && (mode == 0 || beta), "mg_group_norm: null pointer");
    MG_REQUIRE(batch <= 65535 && (long)chan * comps <= 0x7fffffffL, "mg_group_norm: more than 65535 boxes");
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(group_stats_kernel, dim3((unsigned)(batch * groups), kChunks), dim3(256), 0, st, x, x_stride, mul,
                       mul_stride, nodes, chan, groups, comps, static_cast<double*>(scratch));
    hipLaunchKernelGGL(group_finalize_kernel, dim3((unsigned)ceil_div((long)batch * groups, 64)), dim3(64), 0, st,
                       static_cast<double*>(scratch), batch * groups, (double)nodes * (chan / groups), mode, eps);
    const int CT = chan * comps;
    const int threads = CT >= 256 ? 256 : (int)ceil_div(CT, kWave) * kWave;
    const long kx = ceil_div(CT, threads);
    long ny = ceil_div(8192L, kx * batch);                      // about 8192 workgroups, each thread a few nodes
    ny = ny > nodes ? nodes : (ny < 1 ? 1 : ny);
    hipLaunchKernelGGL(group_apply_kernel, dim3((unsigned)kx, (unsigned)ny, (unsigned)batch), dim3(threads), 0, st, x,
                       x_stride, mul, mul_stride, static_cast<const double*>(scratch), nodes, chan, groups, comps, mode,
                       gamma, beta, add, add_stride, res, out);
    return check_launch("mg_group_norm");
}

int mg_tens_sigmoid(int inds, const float* x, long rows_times_chan, float* out, mg_stream_t stream) {
    MG_REQUIRE(inds >= 0 && inds <= 2 && rows_times_chan >= 0, "mg_tens_sigmoid: bad argument");
    if (rows_times_chan == 0) return MG_OK;
    MG_REQUIRE(x && out, "mg_tens_sigmoid: null pointer");
    const int T = inds == 0 ? 1 : (inds == 1 ? 3 : 9);
    hipLaunchKernelGGL(tens_sigmoid_kernel, dim3((unsigned)grid_for(rows_times_chan)), dim3(256), 0,
                       (hipStream_t)stream, x, rows_times_chan, T, out);
    return check_launch("mg_tens_sigmoid");
}

int mg_painn_update_pre(const float* lrv, int lrv_comp_major, const float* x_a, long rows, int n, float* ip, float* cat,
                        float* cat_rowmax, mg_stream_t stream) {
    MG_REQUIRE(cat_rowmax == nullptr || n <= 256, "mg_painn_update_pre: row maxima are emitted for n <= 256");
    MG_REQUIRE(rows >= 0 && n >= 0, "mg_painn_update_pre: negative size");
    if (rows * n == 0) return MG_OK;
    MG_REQUIRE(lrv && x_a && ip && cat, "mg_painn_update_pre: null pointer");
    MG_REQUIRE(rows <= 0x7fffffffL, "mg_painn_update_pre: more than 2^31 - 1 rows");
    const int threads = n >= 256 ? 256 : (int)ceil_div(n, kWave) * kWave;
    const dim3 grid((unsigned)rows, (unsigned)ceil_div(n, threads));
    if (lrv_comp_major)
        hipLaunchKernelGGL(painn_update_pre_kernel<true>, grid, dim3(threads), 0, (hipStream_t)stream, lrv, x_a, n, ip, cat,
                           cat_rowmax);
    else
        hipLaunchKernelGGL(painn_update_pre_kernel<false>, grid, dim3(threads), 0, (hipStream_t)stream, lrv, x_a, n, ip, cat,
                           cat_rowmax);
    return check_launch("mg_painn_update_pre");
}

int mg_painn_update_vec(const float* lrv, int lrv_comp_major, const float* y, const float* res_v, long rows, int n,
                        float* out_v, mg_stream_t stream) {
    MG_REQUIRE(rows >= 0 && n >= 0, "mg_painn_update_vec: negative size");
    if (rows * n == 0) return MG_OK;
    MG_REQUIRE(lrv && y && out_v, "mg_painn_update_vec: null pointer");
    MG_REQUIRE(rows <= 0x7fffffffL, "mg_painn_update_vec: more than 2^31 - 1 rows");
    const int threads = n >= 256 ? 256 : (int)ceil_div(n, kWave) * kWave;
    const dim3 grid((unsigned)rows, (unsigned)ceil_div(n, threads));
    if (lrv_comp_major)
        hipLaunchKernelGGL(painn_update_vec_kernel<true>, grid, dim3(threads), 0, (hipStream_t)stream, lrv, y, res_v, n, out_v);
    else
        hipLaunchKernelGGL(painn_update_vec_kernel<false>, grid, dim3(threads), 0, (hipStream_t)stream, lrv, y, res_v, n, out_v);
    return check_launch("mg_painn_update_vec");
}

int mg_radial_encode(int kind, const float* r_ij, long n_edges, int n, float rmax, float* out, mg_stream_t stream) {
    MG_REQUIRE(kind == 1 || kind == 2, "mg_radial_encode: kind must be 1 (sq_radial_encode) or 2 (radial_encode_edge)");
    MG_REQUIRE(n_edges >= 0 && n >= 0 && rmax > 0.f, "mg_radial_encode: bad argument");
    if (n_edges * n == 0) return MG_OK;
    MG_REQUIRE(r_ij && out, "mg_radial_encode: null pointer");
    float c0, c1 = 0.f;
    if (kind == 1) {
        c0 = (float)(3.14159265358979323846 * 0.70710678118654752440);
        c1 = (float)pow((double)n, -0.7);
    } else {
        c0 = (float)3.14159265358979323846;
    }
    hipLaunchKernelGGL(radial_encode_kernel, dim3((unsigned)grid_for(n_edges * n)), dim3(256), 0, (hipStream_t)stream,
                       kind, r_ij, n_edges, n, rmax, c0, c1, out);
    return check_launch("mg_radial_encode");
}

}  // extern "C"
