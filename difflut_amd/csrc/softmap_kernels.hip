// LearnableLayer soft connectivity on gfx950:  m = x * softmax(W / tau)^T  and its adjoint.
// S = softmax(W / tau) is never written to memory: a pre-pass stores, per row of W, the row
// maximum and the reciprocal of sum_i exp((W - max)/tau); every product kernel rebuilds the
// entries of S it needs while it loads its W tile.
//
//   forward   m[b,o]  = sum_i x[b,i] S[o,i]
//   backward  gx[b,i] = sum_o gm[b,o] S[o,i]
//             gW[o,i] = S[o,i] (G[o,i] - r[o]) / tau,  G = gm^T x,  r[o] = sum_b gm[b,o] m[b,o]
//             (r is the row sum of G*S written through the saved forward output, so the M x I
//              matrix G never needs a second pass)
#include "dl_common.h"

#define SM_T 64   // output tile edge
#define SM_K 16   // reduction step

// one wavefront per row of W
__global__ __launch_bounds__(256) void softmap_rowstats(const float *__restrict__ W, float inv_tau, float *__restrict__ stats,
                                                         int M, int I) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= M) return;
    const float *w = W + (size_t)row * I;
    float mx = -INFINITY;
    for (int i = lane; i < I; i += 64) mx = fmaxf(mx, w[i]);
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    float sum = 0.0f;
    for (int i = lane; i < I; i += 64) sum += expf((w[i] - mx) * inv_tau);
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if (lane == 0) { stats[2 * row] = mx; stats[2 * row + 1] = 1.0f / sum; }
}

__global__ __launch_bounds__(256) void softmap_rowdot(const float *__restrict__ gm, const float *__restrict__ m,
                                                       float *__restrict__ r, int B, int M) {
    const int o = blockIdx.x * 256 + threadIdx.x;
    if (o >= M) return;
    float acc = 0.0f;
    for (int b = 0; b < B; ++b) acc += gm[(size_t)b * M + o] * m[(size_t)b * M + o];
    r[o] = acc;
}

// 64x64 tile, 256 threads, 4x4 outputs per thread; As[k][m], Bs[k][n] in LDS.
struct TileAcc {
    float c[4][4];
    __device__ void clear() {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) c[i][j] = 0.0f;
    }
    __device__ void step(const float (*As)[SM_T + 4], const float (*Bs)[SM_T + 4], int ty, int tx) {
#pragma unroll
        for (int kk = 0; kk < SM_K; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = As[kk][ty * 4 + i]; b[i] = Bs[kk][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) c[i][j] += a[i] * b[j];
        }
    }
};

// MODE 0: forward   rows=b cols=o red=i   A = x[b,i]     Bop = S[o,i]
// MODE 1: gx        rows=b cols=i red=o   A = gm[b,o]    Bop = S[o,i]
// MODE 2: gW        rows=o cols=i red=b   A = gm[b,o]    Bop = x[b,i]   epilogue S (C - r)/tau
template <int MODE>
__global__ __launch_bounds__(256) void softmap_gemm(const float *__restrict__ x, const float *__restrict__ W,
                                                     const float *__restrict__ stats, const float *__restrict__ gm,
                                                     const float *__restrict__ r, float inv_tau, float *__restrict__ out,
                                                     int B, int I, int M) {
    __shared__ float As[SM_K][SM_T + 4];
    __shared__ float Bs[SM_K][SM_T + 4];
    const int R = MODE == 2 ? M : B;            // rows of the output
    const int C = MODE == 0 ? M : I;            // columns of the output
    const int KD = MODE == 0 ? I : (MODE == 1 ? M : B);  // reduction length
    const int r0 = blockIdx.y * SM_T, c0 = blockIdx.x * SM_T;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    TileAcc acc;
    acc.clear();
    for (int k0 = 0; k0 < KD; k0 += SM_K) {
        // ---- A tile: As[kk][rr]
        if (MODE == 0 || MODE == 1) {  // A[row][k] with k contiguous
            const float *A = MODE == 0 ? x : gm;
            const int lda = MODE == 0 ? I : M;
            const int kk = threadIdx.x & 15;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int rr = (threadIdx.x >> 4) + 16 * p;
                const int row = r0 + rr, k = k0 + kk;
                As[kk][rr] = (row < R && k < KD) ? A[(size_t)row * lda + k] : 0.0f;
            }
        } else {  // A(o,b) = gm[b,o], o contiguous
            const int rr = threadIdx.x & 63;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int kk = (threadIdx.x >> 6) + 4 * p;
                const int row = r0 + rr, k = k0 + kk;
                As[kk][rr] = (row < R && k < KD) ? gm[(size_t)k * M + row] : 0.0f;
            }
        }
        // ---- B tile: Bs[kk][cc]
        if (MODE == 0) {  // S[o=col][i=k], k contiguous in W
            const int kk = threadIdx.x & 15;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int cc = (threadIdx.x >> 4) + 16 * p;
                const int col = c0 + cc, k = k0 + kk;
                float v = 0.0f;
                if (col < C && k < KD) v = expf((W[(size_t)col * I + k] - stats[2 * col]) * inv_tau) * stats[2 * col + 1];
                Bs[kk][cc] = v;
            }
        } else if (MODE == 1) {  // S[o=k][i=col], col contiguous in W
            const int cc = threadIdx.x & 63;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int kk = (threadIdx.x >> 6) + 4 * p;
                const int col = c0 + cc, k = k0 + kk;
                float v = 0.0f;
                if (col < C && k < KD) v = expf((W[(size_t)k * I + col] - stats[2 * k]) * inv_tau) * stats[2 * k + 1];
                Bs[kk][cc] = v;
            }
        } else {  // x[b=k][i=col]
            const int cc = threadIdx.x & 63;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int kk = (threadIdx.x >> 6) + 4 * p;
                const int col = c0 + cc, k = k0 + kk;
                Bs[kk][cc] = (col < C && k < KD) ? x[(size_t)k * I + col] : 0.0f;
            }
        }
        __syncthreads();
        acc.step(As, Bs, ty, tx);
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = r0 + ty * 4 + i;
        if (row >= R) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = c0 + tx * 4 + j;
            if (col >= C) continue;
            float v = acc.c[i][j];
            if (MODE == 2) {
                const float s = expf((W[(size_t)row * I + col] - stats[2 * row]) * inv_tau) * stats[2 * row + 1];
                v = s * (v - r[row]) * inv_tau;
            }
            out[(size_t)row * C + col] = v;
        }
    }
}

// ---------------------------------------------------------------------------------
static int softmap_check(int B, int I, int M, int precision) {
    if (B <= 0 || I <= 0 || M <= 0) return DL_ERR_SHAPE;
    if (precision != 0 && precision != 1) return DL_ERR_UNSUPPORTED;
    return DL_OK;
}

extern "C" size_t dl_soft_map_workspace_bytes(int B, int I, int M, int precision) {
    (void)B; (void)I; (void)precision;
    return dl_align256((size_t)M * sizeof(float));
}

extern "C" int dl_soft_map_fwd(const float *x, const float *W, float tau, float *m, float *stats, void *ws,
                               size_t ws_bytes, int B, int I, int M, int precision, void *stream) {
    (void)ws; (void)ws_bytes;
    if (!x || !W || !m || !stats) return DL_ERR_NULL;
    int rc = softmap_check(B, I, M, precision);
    if (rc) return rc;
    if (!(tau > 0.0f)) return DL_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    const float inv_tau = 1.0f / tau;
    DL_TIMED("softmap_rowstats", s, (softmap_rowstats<<<dl_ceil_div(M, 4), 256, 0, s>>>(W, inv_tau, stats, M, I)));
    DL_TIMED("softmap_gemm_fwd", s, (softmap_gemm<0><<<dim3(dl_ceil_div(M, SM_T), dl_ceil_div(B, SM_T)), 256, 0, s>>>(x, W, stats, nullptr, nullptr, inv_tau,
                                                                                   m, B, I, M)));
    return dl_launch_status();
}

extern "C" int dl_soft_map_bwd(const float *x, const float *W, float tau, const float *m, const float *stats,
                               const float *gm, float *gx, float *gW, void *ws, size_t ws_bytes, int B, int I, int M,
                               int precision, void *stream) {
    if (!x || !W || !m || !stats || !gm || !gx || !gW || !ws) return DL_ERR_NULL;
    int rc = softmap_check(B, I, M, precision);
    if (rc) return rc;
    if (!(tau > 0.0f)) return DL_ERR_SHAPE;
    if (ws_bytes < dl_soft_map_workspace_bytes(B, I, M, precision)) return DL_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    const float inv_tau = 1.0f / tau;
    float *r = (float *)ws;
    DL_TIMED("softmap_rowdot", s, (softmap_rowdot<<<dl_ceil_div(M, 256), 256, 0, s>>>(gm, m, r, B, M)));
    DL_TIMED("softmap_gemm_gx", s, (softmap_gemm<1><<<dim3(dl_ceil_div(I, SM_T), dl_ceil_div(B, SM_T)), 256, 0, s>>>(x, W, stats, gm, nullptr, inv_tau, gx,
                                                                                   B, I, M)));
    DL_TIMED("softmap_gemm_gw", s, (softmap_gemm<2><<<dim3(dl_ceil_div(I, SM_T), dl_ceil_div(M, SM_T)), 256, 0, s>>>(x, W, stats, gm, r, inv_tau, gW, B, I,
                                                                                   M)));
    return dl_launch_status();
}
