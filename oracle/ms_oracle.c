/* CPU oracle for the MeshSlice sliced 2-D GEMM, plain C (TEST INFRASTRUCTURE ONLY).
 *
 * A second, loop-level restatement of the reference's sliced bodies, independent of the numpy
 * oracle: every mesh device (i,j) walks the positions of the gathered slice it would receive,
 * peer by peer, exactly as the reshape -> dynamic_slice -> all_gather -> einsum -> psum_scatter
 * -> dynamic_update sequence of the reference lays them out, and accumulates in double.
 *
 *   ms_oracle_meshflow_os  follows TensorParallel.py:153-172 (without the K==1 double count)
 *   ms_oracle_meshflow_ls  follows TensorParallel.py:174-193
 *   ms_oracle_meshflow_rs  follows TensorParallel.py:195-214
 *   ms_oracle_bf16_round   round-to-nearest-even fp32 -> bf16 -> fp32
 *
 * Only tests, the smoke test and the benchmark's CPU-baseline leg may load this library.
 * Parity status: pinned against exact rational arithmetic on the reference's arange fixtures
 * and against the numpy oracle (tests/test_oracle_c.py).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define API __attribute__((visibility("default")))

/* Global index of position p (0 <= p < L/S) of slice k of a length-L axis that is sharded over
 * `parts` peers, each peer's shard viewed as (len/(S*B), S, B) and its slice-k part gathered in
 * peer order.  Derived per peer, not from a closed form. */
static long gathered_to_global(long p, long L, int parts, int S, int B, int k)
{
    long shard_len = L / parts;            /* elements per peer */
    long per_peer = shard_len / S;         /* slice-k elements contributed by one peer */
    long peer = p / per_peer;
    long lp = p % per_peer;                /* position inside the peer's (q, 1, b) block */
    long q = lp / B, b = lp % B;
    long local = (q * S + k) * B + b;      /* index inside the peer's un-sliced shard */
    return peer * shard_len + local;
}

/* Y[M,N] = X[M,Kd] @ W[Kd,N] computed the MeshFlow_OS way on an R x C mesh with S slices. */
API int ms_oracle_meshflow_os(const float *X, const float *W, long M, long Kd, long N,
                              int R, int C, int S, int B, double *Y)
{
    if (M % R || N % C || Kd % ((long)C * S * B) || Kd % ((long)R * S * B)) return -1;
    long m = M / R, n = N / C, ks = Kd / S;
    for (int i = 0; i < R; i++)
        for (int j = 0; j < C; j++)
            for (long r = 0; r < m; r++) {
                double *yrow = Y + (i * m + r) * N + j * n;
                for (long c = 0; c < n; c++) yrow[c] = 0.0;
                for (int k = 0; k < S; k++)
                    for (long p = 0; p < ks; p++) {
                        long gx = gathered_to_global(p, Kd, C, S, B, k); /* X gathered over col */
                        long gw = gathered_to_global(p, Kd, R, S, B, k); /* W gathered over row */
                        double x = X[(i * m + r) * Kd + gx];
                        const float *wrow = W + gw * N + j * n;
                        for (long c = 0; c < n; c++) yrow[c] += x * (double)wrow[c];
                    }
            }
    return 0;
}

/* Y[M,O] = X[M,I] @ W[O,I]^T the MeshFlow_LS way; Y sharded P(row,col) in natural order. */
API int ms_oracle_meshflow_ls(const float *X, const float *W, long M, long I, long O,
                              int R, int C, int S, int B, double *Y)
{
    if (M % R || I % C || O % ((long)R * S * B) || O % ((long)C * S * B)) return -1;
    long m = M / R, ic = I / C, os = O / S, nb = O / ((long)S * B); /* blocks per gathered slice */
    double *part = (double *)malloc(sizeof(double) * (size_t)os);
    if (!part) return -2;
    for (int i = 0; i < R; i++)
        for (long r = 0; r < m; r++)
            for (int k = 0; k < S; k++) {
                /* psum over the C devices of mesh row i of their partial chunks */
                memset(part, 0, sizeof(double) * (size_t)os);
                for (int jj = 0; jj < C; jj++)
                    for (long p = 0; p < os; p++) {
                        long gw = gathered_to_global(p, O, R, S, B, k);
                        const float *xr = X + (i * m + r) * I + jj * ic;
                        const float *wr = W + gw * I + jj * ic;
                        double s = 0.0;
                        for (long t = 0; t < ic; t++) s += (double)xr[t] * (double)wr[t];
                        part[p] += s;
                    }
                /* scatter: device j keeps blocks [j*nb/C, (j+1)*nb/C); written at slice slot k
                 * of its (m, O/(S*B*C), S, B) output view */
                for (int j = 0; j < C; j++)
                    for (long u = j * (nb / C); u < (j + 1) * (nb / C); u++)
                        for (int b = 0; b < B; b++) {
                            long local = ((u - j * (nb / C)) * S + k) * B + b;
                            Y[(i * m + r) * O + j * (O / C) + local] = part[u * B + b];
                        }
            }
    free(part);
    return 0;
}

/* Y[N,O] = X[I,N]^T @ W[I,O] the MeshFlow_RS way. */
API int ms_oracle_meshflow_rs(const float *X, const float *W, long I, long N, long O,
                              int R, int C, int S, int B, double *Y)
{
    if (I % R || O % C || N % ((long)C * S * B) || N % ((long)R * S * B)) return -1;
    long ir = I / R, oc = O / C, ns = N / S, nb = N / ((long)S * B);
    double *part = (double *)malloc(sizeof(double) * (size_t)oc);
    if (!part) return -2;
    for (int j = 0; j < C; j++)
        for (int k = 0; k < S; k++)
            for (long p = 0; p < ns; p++) {
                long gx = gathered_to_global(p, N, C, S, B, k);
                memset(part, 0, sizeof(double) * (size_t)oc);
                for (int ii = 0; ii < R; ii++)            /* psum over mesh column j */
                    for (long t = 0; t < ir; t++) {
                        double x = X[(ii * ir + t) * N + gx];
                        const float *wr = W + (ii * ir + t) * O + j * oc;
                        for (long c = 0; c < oc; c++) part[c] += x * (double)wr[c];
                    }
                long u = p / B, b = p % B;
                int i = (int)(u / (nb / R));               /* the device row that keeps block u */
                long local = ((u - i * (nb / R)) * S + k) * B + b;
                double *yr = Y + (i * (N / R) + local) * O + j * oc;
                for (long c = 0; c < oc; c++) yr[c] = part[c];
            }
    free(part);
    return 0;
}

API void ms_oracle_bf16_round(const float *in, float *out, long n)
{
    for (long t = 0; t < n; t++) {
        uint32_t u;
        memcpy(&u, in + t, 4);
        if ((u & 0x7fffffffu) > 0x7f800000u) { out[t] = in[t]; continue; } /* NaN */
        u += 0x7fffu + ((u >> 16) & 1u);
        u &= 0xffff0000u;
        memcpy(out + t, &u, 4);
    }
}
