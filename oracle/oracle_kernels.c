/*
 * CPU oracle kernels for the Plexus GCN hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * Plain-C restatement of the operators the reference calls on its hot path, used as the
 * large-size arbiter (fp64 accumulation) where the torch CPU operators are too slow or
 * where two fp32 summation orders have to be judged.  Never linked into the product
 * library; only tests, the smoke check and the benchmark's cpu_baseline leg load it.
 *
 * The reference holds no golden vectors for this path; these routines are pinned against
 * dense matmul, scipy and torch CPU operators in tests/test_oracle.py.
 *
 *   orc_csr_spmm_*      : Y = A.H, A in CSR          (plexus/gcn_conv.py:188, :265)
 *   orc_gemm_*          : C = op(A).op(B)            (plexus/gcn_conv.py:211,237,256 ->
 *                                                     plexus/utils/matmul_tuning.py:95)
 *   orc_softmax_xent    : loss and d(loss)/d(logits) (plexus/cross_entropy.py:35-101,111-114)
 *   orc_gcn_norm_csr    : D^-1/2 A D^-1/2            (plexus/utils/dataset.py:101)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* Y[M x D] = A[M x K] . H[K x D]; fp32 storage, accumulation in `double` per output element. */
void orc_csr_spmm_f32_acc64(int64_t M, const int64_t *rowptr, const int64_t *col, const float *val,
                            const float *H, int64_t ldh, int64_t D, float *Y, int64_t ldy)
{
#pragma omp parallel
    {
        double *acc = (double *)malloc(sizeof(double) * (size_t)D);
#pragma omp for schedule(dynamic, 64)
        for (int64_t r = 0; r < M; ++r) {
            for (int64_t d = 0; d < D; ++d) acc[d] = 0.0;
            for (int64_t j = rowptr[r]; j < rowptr[r + 1]; ++j) {
                const double v = (double)val[j];
                const float *h = H + col[j] * ldh;
                for (int64_t d = 0; d < D; ++d) acc[d] += v * (double)h[d];
            }
            for (int64_t d = 0; d < D; ++d) Y[r * ldy + d] = (float)acc[d];
        }
        free(acc);
    }
}

/* Same product with fp32 accumulation in storage order (the textbook CSR row loop). */
void orc_csr_spmm_f32(int64_t M, const int64_t *rowptr, const int64_t *col, const float *val,
                      const float *H, int64_t ldh, int64_t D, float *Y, int64_t ldy)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (int64_t r = 0; r < M; ++r) {
        float *y = Y + r * ldy;
        for (int64_t d = 0; d < D; ++d) y[d] = 0.0f;
        for (int64_t j = rowptr[r]; j < rowptr[r + 1]; ++j) {
            const float v = val[j];
            const float *h = H + col[j] * ldh;
            for (int64_t d = 0; d < D; ++d) y[d] += v * h[d];
        }
    }
}

/* fp64 in, fp64 out. */
void orc_csr_spmm_f64(int64_t M, const int64_t *rowptr, const int64_t *col, const double *val,
                      const double *H, int64_t ldh, int64_t D, double *Y, int64_t ldy)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (int64_t r = 0; r < M; ++r) {
        double *y = Y + r * ldy;
        for (int64_t d = 0; d < D; ++d) y[d] = 0.0;
        for (int64_t j = rowptr[r]; j < rowptr[r + 1]; ++j) {
            const double v = val[j];
            const double *h = H + col[j] * ldh;
            for (int64_t d = 0; d < D; ++d) y[d] += v * h[d];
        }
    }
}

/*
 * C[M x N] = op(A) . op(B), fp32 storage, fp64 accumulation.
 *   ta == 0: A is [M x K] (lda),  ta == 1: A is stored [K x M] and used transposed
 *   tb == 0: B is [K x N] (ldb),  tb == 1: B is stored [N x K] and used transposed
 */
void orc_gemm_f32_acc64(int ta, int tb, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                        const float *B, int64_t ldb, float *C, int64_t ldc)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; ++i) {
        for (int64_t j = 0; j < N; ++j) {
            double s = 0.0;
            for (int64_t k = 0; k < K; ++k) {
                const double a = ta ? (double)A[k * lda + i] : (double)A[i * lda + k];
                const double b = tb ? (double)B[j * ldb + k] : (double)B[k * ldb + j];
                s += a * b;
            }
            C[i * ldc + j] = (float)s;
        }
    }
}

/*
 * Row-softmax cross-entropy as the reference computes it at one rank:
 *   classes >= num_classes get probability 0; rows >= num_nodes or with label < 0 get a zero
 *   softmax row; labels outside [0, C) give an all-zero one-hot row; loss_i = -log(max(p_iy, 1e-9));
 *   loss = sum_i loss_i / num_nodes; dlogits = (softmax - onehot) / num_nodes * gscale.
 * A row whose softmax is zeroed but whose label is valid contributes -log(1e-9).
 * Returns the loss; dlogits may be NULL.
 */
double orc_softmax_xent(int64_t M, int64_t C, const float *logits, int64_t ld, const int64_t *labels,
                        int64_t num_nodes, int64_t num_classes, double gscale, float *dlogits, int64_t ldd)
{
    double total = 0.0;
    const int64_t cv = num_classes < C ? num_classes : C;
#pragma omp parallel for schedule(static) reduction(+ : total)
    for (int64_t i = 0; i < M; ++i) {
        const float *x = logits + i * ld;
        const int64_t y = labels[i];
        const int invalid_node = (i >= num_nodes) || (y < 0);
        const int label_ok = (y >= 0) && (y < C);
        double mx = -INFINITY;
        for (int64_t c = 0; c < cv; ++c)
            if ((double)x[c] > mx) mx = (double)x[c];
        double den = 0.0;
        for (int64_t c = 0; c < cv; ++c) den += exp((double)x[c] - mx);
        for (int64_t c = 0; c < C; ++c) {
            double p = (c < cv && !invalid_node) ? exp((double)x[c] - mx) / den : 0.0;
            const double t = (label_ok && c == y) ? 1.0 : 0.0;
            if (t != 0.0) total += -log(p > 1e-9 ? p : 1e-9);
            if (dlogits) dlogits[i * ldd + c] = (float)((p - t) / (double)num_nodes * gscale);
        }
    }
    return total / (double)num_nodes;
}

/* out_j = val_j / sqrt(d_row d_col) with d_i = sum of row i; 0 where a degree is 0. */
void orc_gcn_norm_csr(int64_t M, const int64_t *rowptr, const int64_t *col, const float *val, float *out)
{
    double *dinv = (double *)malloc(sizeof(double) * (size_t)(M > 0 ? M : 1));
    for (int64_t r = 0; r < M; ++r) {
        double d = 0.0;
        for (int64_t j = rowptr[r]; j < rowptr[r + 1]; ++j) d += (double)val[j];
        dinv[r] = d > 0.0 ? 1.0 / sqrt(d) : 0.0;
    }
    for (int64_t r = 0; r < M; ++r)
        for (int64_t j = rowptr[r]; j < rowptr[r + 1]; ++j)
            out[j] = (float)(dinv[r] * (double)val[j] * dinv[col[j]]);
    free(dinv);
}
