/*
 * CPU restatement of the Accel-GCN SpMM hot path in plain C.
 *
 * TEST INFRASTRUCTURE ONLY: linked or loaded by tests/, by the smoke check and
 * by the cpu_baseline leg of the benchmark, always as the checker and never as
 * the thing shipped or measured.  The product library does not link it.
 *
 * Functions and the reference lines they follow (paths relative to upstream):
 *   oracle_partition_walk     block_level_partition.py:7-21 (tables), :48-103 (walk)
 *   oracle_degree_sort        not in the reference; order evidenced by
 *                             block_level_partition.py:31,38 and the golden
 *                             .block4 files (ascending); stable tie-break is
 *                             this build's definition
 *   oracle_spmm_block4        spmm_accel.cu:16-102: the kernel's own
 *                             decomposition (12 slices of <= 32 non-zeros per
 *                             block, slice partials added into the output row)
 *   oracle_spmm_csr_f32/_f64  the quantity the kernel is checked against
 *                             upstream (main.cu:143-155 uses cuSPARSE CSR SpMM,
 *                             alpha=1 beta=0); here a plain row loop, fp32 in
 *                             CSR order, or fp64 accumulation
 *
 * Pinned by: the 16 golden .block4 files (partition), scipy's csr @ dense and a
 * brute-force dense product on small inputs (SpMM), closed forms (ones -> row
 * degree, identity -> X), and oracle_spmm_block4 == oracle_spmm_csr on the
 * metadata produced by oracle_partition_walk.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define DEG_BOUND 384
#define SLICES 12
#define SLICE_NZ 32

static void slice_rule(int d, int *w_nz, int *rows)
{
    /* degrees 1..191 use split factors 1,2,3,4,6; 192..384 fall back to one
     * row per block with 32-non-zero slices (block_level_partition.py:56-63) */
    static const int f[5] = {1, 2, 3, 4, 6};
    if (d >= DEG_BOUND / 2) { *w_nz = SLICE_NZ; *rows = 1; return; }
    for (int i = 0; i < 5; i++)
        if (f[i] * SLICE_NZ >= d) { *w_nz = (d + f[i] - 1) / f[i]; *rows = SLICES / f[i]; return; }
}

/* Returns the number of blocks; writes at most cap quadruples to out (out may
 * be NULL to count only). */
int64_t oracle_partition_walk(const int32_t *indptr, int64_t n_rows, int32_t *out, int64_t cap)
{
    int64_t nb = 0, row = 0;
    int64_t loc = 0;
    while (row < n_rows) {
        int64_t d = (int64_t)indptr[row + 1] - indptr[row];
        if (d <= 0) { row++; continue; }
        if (d <= DEG_BOUND) {
            int w = SLICE_NZ, r = 1;
            slice_rule((int)d, &w, &r);
            int taken = 1;
            while (taken < r && row + taken < n_rows &&
                   (int64_t)indptr[row + taken + 1] - indptr[row + taken] == d)
                taken++;
            if (out && nb < cap) {
                int32_t *q = out + 4 * nb;
                q[0] = (int32_t)d; q[1] = (int32_t)row; q[2] = (int32_t)loc; q[3] = (w << 16) + taken;
            }
            nb++;
            row += taken;
            loc += (int64_t)taken * d;
        } else {
            for (int64_t done = 0; done < d; done += DEG_BOUND) {
                int64_t seg = d - done < DEG_BOUND ? d - done : DEG_BOUND;
                if (out && nb < cap) {
                    int32_t *q = out + 4 * nb;
                    q[0] = (int32_t)d; q[1] = (int32_t)row; q[2] = (int32_t)(loc + done); q[3] = (int32_t)seg;
                }
                nb++;
            }
            loc += d;
            row++;
        }
    }
    return nb;
}

/* perm[new_row] = old_row; ascending degree, ties by old row id (counting sort). */
int oracle_degree_sort(const int32_t *indptr, int64_t n_rows, int32_t *perm)
{
    int64_t maxd = 0;
    for (int64_t r = 0; r < n_rows; r++) {
        int64_t d = (int64_t)indptr[r + 1] - indptr[r];
        if (d < 0) return -1;
        if (d > maxd) maxd = d;
    }
    int64_t *start = (int64_t *)calloc((size_t)maxd + 2, sizeof(int64_t));
    if (!start) return -2;
    for (int64_t r = 0; r < n_rows; r++) start[indptr[r + 1] - indptr[r] + 1]++;
    for (int64_t d = 0; d <= maxd; d++) start[d + 1] += start[d];
    for (int64_t r = 0; r < n_rows; r++) perm[start[indptr[r + 1] - indptr[r]]++] = (int32_t)r;
    free(start);
    return 0;
}

/* Y = A X, fp32 accumulation in CSR order (the order scipy's csr_matvecs uses). */
void oracle_spmm_csr_f32(const int32_t *indptr, const int32_t *idx, const float *val,
                         int64_t n_rows, const float *X, float *Y, int64_t N)
{
    for (int64_t r = 0; r < n_rows; r++) {
        float *y = Y + r * N;
        for (int64_t j = 0; j < N; j++) y[j] = 0.0f;
        for (int64_t p = indptr[r]; p < indptr[r + 1]; p++) {
            const float a = val[p];
            const float *x = X + (int64_t)idx[p] * N;
            for (int64_t j = 0; j < N; j++) y[j] += a * x[j];
        }
    }
}

/* Same product accumulated in fp64: Y64 = A X, and S = |A| |X| for error scaling
 * (either output may be NULL). */
void oracle_spmm_csr_f64(const int32_t *indptr, const int32_t *idx, const float *val,
                         int64_t n_rows, const float *X, double *Y64, double *S, int64_t N)
{
    double *acc = (double *)malloc(sizeof(double) * (size_t)N * 2);
    double *sab = acc + N;
    for (int64_t r = 0; r < n_rows; r++) {
        for (int64_t j = 0; j < N; j++) { acc[j] = 0.0; sab[j] = 0.0; }
        for (int64_t p = indptr[r]; p < indptr[r + 1]; p++) {
            const double a = val[p];
            const double aa = a < 0 ? -a : a;
            const float *x = X + (int64_t)idx[p] * N;
            for (int64_t j = 0; j < N; j++) {
                const double xv = x[j];
                acc[j] += a * xv;
                sab[j] += aa * (xv < 0 ? -xv : xv);
            }
        }
        if (Y64) memcpy(Y64 + r * N, acc, sizeof(double) * (size_t)N);
        if (S) memcpy(S + r * N, sab, sizeof(double) * (size_t)N);
    }
    free(acc);
}

/* The reference kernel's decomposition, one block4 entry at a time
 * (spmm_accel.cu:21-28 decode, :34 slices per row, :47-48 slice -> row/offset,
 * :56-78 slice loop, :82-99 slice partial added to the output row).  Y must be
 * zero on entry, as upstream requires.  Rows are in the CSR's own order. */
void oracle_spmm_block4(const int32_t *block4, int64_t n_blocks, const int32_t *idx,
                        const float *val, const float *X, float *Y, int64_t N)
{
    float *part = (float *)malloc(sizeof(float) * (size_t)N);
    for (int64_t b = 0; b < n_blocks; b++) {
        const int32_t *q = block4 + 4 * b;
        const int deg = q[0], row0 = q[1], loc0 = q[2], info = q[3];
        const int n_rows = deg <= DEG_BOUND ? (info & 65535) : 1;
        const int w_nz = deg <= DEG_BOUND ? (info >> 16) : SLICE_NZ;
        const int row_nz = deg <= DEG_BOUND ? deg : info;
        const int per_row = (row_nz + w_nz - 1) / w_nz;
        for (int s = 0; s < SLICES; s++) {
            const int r = s / per_row, off = (s % per_row) * w_nz;
            if (r >= n_rows) break;
            for (int64_t j = 0; j < N; j++) part[j] = 0.0f;
            for (int i = 0; i < w_nz && i + off < row_nz; i++) {
                const int64_t p = (int64_t)loc0 + (int64_t)r * row_nz + i + off;
                const float a = val[p];
                const float *x = X + (int64_t)idx[p] * N;
                for (int64_t j = 0; j < N; j++) part[j] += a * x[j];
            }
            float *y = Y + ((int64_t)row0 + r) * N;
            for (int64_t j = 0; j < N; j++) y[j] += part[j];
        }
    }
    free(part);
}
