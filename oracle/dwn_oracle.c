/* CPU restatement of the RandomLayer + DWN layer pass in plain C.
 *
 * TEST INFRASTRUCTURE: linked only by tests/, the smoke check and the CPU-baseline
 * leg of the benchmark.  Nothing in the shipped library calls it.
 *
 * It follows the reference loop for loop:
 *   forward  - difflut/layers/random_layer.py:284-340 (gather, per-node loop) and
 *              difflut/nodes/dwn_node.py:137-165 (threshold >= 0.5, LSB-first address, lookup)
 *   backward - difflut/nodes/dwn_node.py:167-229 (EFDFunctionCPU.backward: table-entry
 *              gradient by direct accumulation; input gradient as a 2^k-term sum
 *              accumulated in double and stored as float), then the adjoint of the
 *              gather (sum over every (node, slot) that reads an input).
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC (see oracle/Makefile).
 */
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline unsigned node_address(const float *xrow, const int32_t *idx, int k) {
    unsigned addr = 0;
    for (int i = 0; i < k; ++i)
        if (xrow[idx[i]] >= 0.5f) addr |= 1u << i; /* dwn_node.py:186-188 */
    return addr;
}

/* x [B,I], idx [N,k] (int32), luts [N,O,L], y [B,N,O] */
void oracle_dwn_layer_forward(const float *x, const int32_t *idx, const float *luts, float *y,
                              int B, int I, int N, int k, int O) {
    const int L = 1 << k;
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; ++b)
        for (int n = 0; n < N; ++n) {
            unsigned addr = node_address(x + (size_t)b * I, idx + (size_t)n * k, k);
            for (int d = 0; d < O; ++d)
                y[((size_t)b * N + n) * O + d] = luts[((size_t)n * O + d) * L + addr];
        }
}

/* gx [B,I] and gl [N,O,L] are overwritten.  Threads split the batch; every thread
 * keeps a private double table-gradient copy; the copies are summed in thread order. */
void oracle_dwn_layer_backward(const float *x, const int32_t *idx, const float *luts,
                               const float *gy, double alpha, double beta, float *gx, float *gl,
                               int B, int I, int N, int k, int O) {
    const int L = 1 << k;
    double bp[33];
    for (int h = 0; h <= k; ++h) bp[h] = pow(beta, (double)h); /* beta**hamming_dist, :223 */
    const size_t T = (size_t)N * O * L;
    const int nthreads = omp_get_max_threads();
    double *glp_all = (double *)calloc(T * (size_t)nthreads, sizeof(double));
#pragma omp parallel num_threads(nthreads)
    {
        double *row = (double *)malloc(sizeof(double) * (size_t)I);
        double *glp = glp_all + T * (size_t)omp_get_thread_num();
#pragma omp for schedule(static)
        for (int b = 0; b < B; ++b) {
            for (int i = 0; i < I; ++i) row[i] = 0.0;
            for (int n = 0; n < N; ++n) {
                const int32_t *ix = idx + (size_t)n * k;
                const float *lut = luts + (size_t)n * O * L;
                const float *g = gy + ((size_t)b * N + n) * O;
                unsigned addr = node_address(x + (size_t)b * I, ix, k);
                for (int d = 0; d < O; ++d) glp[((size_t)n * O + d) * L + addr] += g[d]; /* :190-192 */
                for (int l = 0; l < k; ++l) { /* :195-227 */
                    unsigned mask = ((1u << k) - 1u) & ~(1u << l);
                    unsigned am = addr & mask;
                    double total = 0.0;
                    for (unsigned kk = 0; kk < (unsigned)L; ++kk) {
                        int h = __builtin_popcount(am ^ (kk & mask));
                        double sgn = ((kk >> l) & 1u) ? 1.0 : -1.0;
                        for (int d = 0; d < O; ++d)
                            total += alpha * sgn * (double)lut[d * L + kk] * bp[h] * (double)g[d];
                    }
                    row[ix[l]] += (double)(float)total; /* stored as float, then gathered back */
                }
            }
            for (int i = 0; i < I; ++i) gx[(size_t)b * I + i] = (float)row[i];
        }
        free(row);
    }
    for (size_t t = 0; t < T; ++t) { /* fixed thread order: run-to-run identical */
        double s = 0.0;
        for (int th = 0; th < nthreads; ++th) s += glp_all[T * (size_t)th + t];
        gl[t] = (float)s;
    }
    free(glp_all);
}
