/*
 * TEST INFRASTRUCTURE ONLY — CPU restatement of the reference's periodic
 * cell-list radius graph.  Nothing in the product path may call this file;
 * it exists so tests and the benchmark's cpu_baseline leg have an independent
 * answer to compare the HIP kernels with.
 *
 * Follows (file:line relative to the reference checkout):
 *   extensions/neighbour_grid/neighbour_grid.cpp:59-103   ndiv = ceilf(box/cutoff), ndiv >= 3
 *   extensions/neighbour_grid/neighbour_grid_kern.cu:39-48   0-centred IEEE-remainder wrap,
 *                                                            minimum-image delta
 *   extensions/neighbour_grid/neighbour_grid_kern.cu:57-93   wrap + cell assignment
 *   extensions/neighbour_grid/neighbour_grid_kern.cu:95-150  3x3x3 window scan, d2 <= r0^2, i != j
 *   extensions/neighbour_grid/neighbour_grid_kern.cu:334-352 flat (src,dst) rows ordered by (b,i)
 *   extensions/neighbour_grid/neighbour_grid.cpp:170-195     edgeCounts = inclusive cumsum per box
 *
 * fp32 policy: every operation is a single correctly rounded fp32 operation,
 * compiled with -ffp-contract=off, except the squared distance which is the
 * explicit contraction fmaf(dz,dz, fmaf(dy,dy, dx*dx)) — what nvcc's default
 * -fmad=true makes of `a.x*b.x + a.y*b.y + a.z*b.z`.  (Assumption: only a run
 * of the reference on CUDA hardware could confirm it for pairs within an ulp
 * of the cutoff; "parity unpinned" for exactly those pairs.)
 *
 * Modes:
 *   0  cell list as the reference walks it (cells, then 27-window scan)
 *   1  O(N^2) all pairs, keeping the reference's cell-adjacency predicate
 *      (reproduces the under-resolved grid when box/cutoff is not an integer)
 *   2  O(N^2) all pairs, plain minimum-image radius graph (textbook); equals
 *      modes 0/1 whenever box/cutoff is an integer in every dimension
 * Rows are emitted with dst ascending (the reference's intra-row order is
 * unspecified: slots come from atomicAdd).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct { float x, y, z; } vec3;

static inline float wrap0(float r, float box) { return remainderf(r, box); }

static inline float dist2(vec3 a, vec3 b, vec3 box) {
    float dx = wrap0(a.x - b.x, box.x);
    float dy = wrap0(a.y - b.y, box.y);
    float dz = wrap0(a.z - b.z, box.z);
    return fmaf(dz, dz, fmaf(dy, dy, dx * dx));
}

static inline vec3 wrap_into_box(vec3 p, vec3 box) {
    vec3 h = {0.5f * box.x, 0.5f * box.y, 0.5f * box.z};
    vec3 w;
    w.x = wrap0(p.x - h.x, box.x) + h.x;
    w.y = wrap0(p.y - h.y, box.y) + h.y;
    w.z = wrap0(p.z - h.z, box.z) + h.z;
    return w;
}

static inline int cell_coord(float w, float box, int ndiv) {
    float scaled = (float)ndiv * w;
    float q = scaled / box;
    return ((int)q) % ndiv;
}

static int cmp_int(const void* a, const void* b) {
    int x = *(const int*)a, y = *(const int*)b;
    return (x > y) - (x < y);
}

/* in-window test: is cell c2 within the periodic 3x3x3 window of c1 (per axis) */
static inline int axis_adjacent(int c1, int c2, int ndiv) {
    int d = c2 - c1;
    if (d < 0) d += ndiv;
    return d == 0 || d == 1 || d == ndiv - 1;
}

int nbr_oracle_ndiv(float cutoff, float bx, float by, float bz, int* ndiv) {
    ndiv[0] = (int)ceilf(bx / cutoff);
    ndiv[1] = (int)ceilf(by / cutoff);
    ndiv[2] = (int)ceilf(bz / cutoff);
    return (ndiv[0] >= 3 && ndiv[1] >= 3 && ndiv[2] >= 3) ? 0 : -1;
}

/* Wrapped positions and linear cell ids (cell id excludes the batch offset). */
void nbr_oracle_wrap_cells(const float* x, int batch, int nodes, float cutoff,
                           float bx, float by, float bz, float* wrapped, int* cell) {
    int ndiv[3];
    nbr_oracle_ndiv(cutoff, bx, by, bz, ndiv);
    vec3 box = {bx, by, bz};
    for (long i = 0; i < (long)batch * nodes; i++) {
        vec3 p = {x[3 * i], x[3 * i + 1], x[3 * i + 2]};
        vec3 w = wrap_into_box(p, box);
        wrapped[3 * i] = w.x; wrapped[3 * i + 1] = w.y; wrapped[3 * i + 2] = w.z;
        int cx = cell_coord(w.x, bx, ndiv[0]);
        int cy = cell_coord(w.y, by, ndiv[1]);
        int cz = cell_coord(w.z, bz, ndiv[2]);
        cell[i] = (cx * ndiv[1] + cy) * ndiv[2] + cz;
    }
}

/*
 * Returns the number of directed edges E (>= 0), or -1 if ndiv < 3, -2 on
 * allocation failure.  When src/dst are non-NULL, at most `capacity` edges are
 * written (E is still the full count).  counts (batch*nodes) and
 * edge_counts (batch, inclusive cumsum) may be NULL.
 * stats[0] = max atoms in one cell, stats[1] = max degree,
 * stats[2] = pairs with |d2 - r0sq| <= 2 ulp (borderline census), may be NULL.
 */
long nbr_oracle_edges(const float* x, int batch, int nodes, float cutoff,
                      float bx, float by, float bz, int mode,
                      int* src, int* dst, long capacity,
                      int* counts, int* edge_counts, long* stats) {
    int ndiv[3];
    if (nbr_oracle_ndiv(cutoff, bx, by, bz, ndiv) != 0) return -1;
    const vec3 box = {bx, by, bz};
    const float r0sq = cutoff * cutoff;
    const long total = (long)batch * nodes;
    const int ncells = ndiv[0] * ndiv[1] * ndiv[2];

    float* wrapped = (float*)malloc(sizeof(float) * 3 * (total > 0 ? total : 1));
    int* cell = (int*)malloc(sizeof(int) * (total > 0 ? total : 1));
    int* row = (int*)malloc(sizeof(int) * (nodes > 0 ? nodes : 1));
    int* cell_start = (int*)malloc(sizeof(int) * (ncells + 1));
    int* cell_items = (int*)malloc(sizeof(int) * (nodes > 0 ? nodes : 1));
    if (!wrapped || !cell || !row || !cell_start || !cell_items) {
        free(wrapped); free(cell); free(row); free(cell_start); free(cell_items);
        return -2;
    }
    nbr_oracle_wrap_cells(x, batch, nodes, cutoff, bx, by, bz, wrapped, cell);

    long E = 0, max_occ = 0, max_deg = 0, borderline = 0;
    const float lo = nextafterf(nextafterf(r0sq, 0.0f), 0.0f);
    const float hi = nextafterf(nextafterf(r0sq, INFINITY), INFINITY);

    for (int b = 0; b < batch; b++) {
        const float* wb = wrapped + 3 * (long)b * nodes;
        const int* cb = cell + (long)b * nodes;
        /* counting sort of this box's atoms by cell (ascending index inside a cell) */
        memset(cell_start, 0, sizeof(int) * (ncells + 1));
        for (int i = 0; i < nodes; i++) cell_start[cb[i] + 1]++;
        for (int c = 0; c < ncells; c++) {
            if (cell_start[c + 1] > max_occ) max_occ = cell_start[c + 1];
            cell_start[c + 1] += cell_start[c];
        }
        {
            int* fill = (int*)calloc(ncells, sizeof(int));
            if (!fill) { free(wrapped); free(cell); free(row); free(cell_start); free(cell_items); return -2; }
            for (int i = 0; i < nodes; i++) cell_items[cell_start[cb[i]] + fill[cb[i]]++] = i;
            free(fill);
        }
        for (int i = 0; i < nodes; i++) {
            vec3 pi = {wb[3 * i], wb[3 * i + 1], wb[3 * i + 2]};
            int ci = cb[i];
            int cx = ci / (ndiv[1] * ndiv[2]), cy = (ci / ndiv[2]) % ndiv[1], cz = ci % ndiv[2];
            int deg = 0;
            if (mode == 0) {
                for (int dx = -1; dx <= 1; dx++)
                for (int dy = -1; dy <= 1; dy++)
                for (int dz = -1; dz <= 1; dz++) {
                    int nx = (cx + dx + ndiv[0]) % ndiv[0];
                    int ny = (cy + dy + ndiv[1]) % ndiv[1];
                    int nz = (cz + dz + ndiv[2]) % ndiv[2];
                    int c = (nx * ndiv[1] + ny) * ndiv[2] + nz;
                    for (int k = cell_start[c]; k < cell_start[c + 1]; k++) {
                        int j = cell_items[k];
                        vec3 pj = {wb[3 * j], wb[3 * j + 1], wb[3 * j + 2]};
                        float d2 = dist2(pi, pj, box);
                        if (j != i && d2 >= lo && d2 <= hi) borderline++;
                        if (j != i && d2 <= r0sq) row[deg++] = j;
                    }
                }
                qsort(row, deg, sizeof(int), cmp_int);
            } else {
                for (int j = 0; j < nodes; j++) {
                    if (j == i) continue;
                    if (mode == 1) {
                        int cj = cb[j];
                        int jx = cj / (ndiv[1] * ndiv[2]), jy = (cj / ndiv[2]) % ndiv[1], jz = cj % ndiv[2];
                        if (!(axis_adjacent(cx, jx, ndiv[0]) && axis_adjacent(cy, jy, ndiv[1]) &&
                              axis_adjacent(cz, jz, ndiv[2]))) continue;
                    }
                    vec3 pj = {wb[3 * j], wb[3 * j + 1], wb[3 * j + 2]};
                    float d2 = dist2(pi, pj, box);
                    if (d2 >= lo && d2 <= hi) borderline++;
                    if (d2 <= r0sq) row[deg++] = j;
                }
            }
            if (counts) counts[(long)b * nodes + i] = deg;
            if (deg > max_deg) max_deg = deg;
            if (src && dst) {
                for (int k = 0; k < deg && E + k < capacity; k++) {
                    src[E + k] = b * nodes + i;
                    dst[E + k] = b * nodes + row[k];
                }
            }
            E += deg;
        }
        if (edge_counts) edge_counts[b] = (int)E;
    }
    if (stats) { stats[0] = max_occ; stats[1] = max_deg; stats[2] = borderline; }
    free(wrapped); free(cell); free(row); free(cell_start); free(cell_items);
    return E;
}

/* Exposed so tests can check the branch-based wrap used on the GPU against libm. */
float nbr_oracle_remainderf(float a, float b) { return remainderf(a, b); }
