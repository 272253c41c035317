// LearnableLayer soft connectivity on gfx950:  m = x * softmax(W / tau)^T  and its adjoint, on the
// matrix cores (v_mfma_f32_32x32x2_f32: fp32 operands, fp32 accumulation).
// S = softmax(W / tau) is never written to memory: a pre-pass stores, per row of W, the row
// maximum and the reciprocal of sum_i exp((W - max)/tau); every product kernel rebuilds the
// entries of S it needs while it stages its W tile in LDS.
//
//   forward   m[b,o]  = sum_i x[b,i] S[o,i]
//   backward  gx[b,i] = sum_o gm[b,o] S[o,i]      (reduction over M = N*k: split into chunks,
//                                                   partial products reduced in fixed order)
//             gW[o,i] = S[o,i] (G[o,i] - r[o]) / tau,  G = gm^T x,  r[o] = sum_b gm[b,o] m[b,o]
//             (r is the row sum of G*S written through the saved forward output, so the M x I
//              matrix G never needs a second pass)
//
// One product kernel, three operand modes.  Block = 256 threads = 2x2 wavefronts, output tile
// 128 x 128, each wavefront 64 x 64 = 2x2 MFMA tiles (4 x 16 accumulator registers), reduction
// staged through LDS 32 deep as As[k][row], Bs[k][col] (k-major, so an MFMA operand read is 64
// consecutive floats).  The next stage's global loads are issued before the current stage's
// MFMAs.
#include "dl_common.h"

typedef float floatx16 __attribute__((ext_vector_type(16)));

#define SM_T 128   // output tile edge
#define SM_K 32    // reduction depth per LDS stage
#define SM_LD 132  // LDS row stride in floats (multiple of 4: float4 stores stay aligned)

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

// r[o] = sum_b gm[b,o] m[b,o]
__global__ __launch_bounds__(256) void softmap_rowdot(const float *__restrict__ gm, const float *__restrict__ m,
                                                       float *__restrict__ r, int B, int M) {
    const int o = blockIdx.x * 256 + threadIdx.x;
    if (o >= M) return;
    float acc = 0.0f;
    for (int b = 0; b < B; ++b) acc += gm[(size_t)b * M + o] * m[(size_t)b * M + o];
    r[o] = acc;
}

// out[e] = sum over chunks of part[chunk][e], fixed order
__global__ __launch_bounds__(256) void softmap_reduce_chunks(const float *__restrict__ part, float *__restrict__ out,
                                                              long long total, int chunks) {
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    float acc = 0.0f;
    for (int c = 0; c < chunks; ++c) acc += part[(size_t)c * total + e];
    out[e] = acc;
}

__device__ __forceinline__ float softmap_s(float w, float mx, float rs, float inv_tau) {
    return expf((w - mx) * inv_tau) * rs;
}

// MODE 0: forward   rows=b cols=o red=i   A = x[b,i]  (red contiguous)   B = S[o,i] (red contiguous)
// MODE 1: gx        rows=b cols=i red=o   A = gm[b,o] (red contiguous)   B = S[o,i] (col contiguous)
// MODE 2: gW        rows=o cols=i red=b   A = gm[b,o] (row contiguous)   B = x[b,i] (col contiguous)
//                   epilogue S[o,i] (C - r[o]) / tau
// blockIdx.z selects a chunk of the reduction (MODE 1); out then points at [chunks][R][C] partials.
template <int MODE>
__global__ __launch_bounds__(256) void softmap_mfma(const float *__restrict__ x, const float *__restrict__ W,
                                                     const float *__restrict__ stats, const float *__restrict__ gm,
                                                     const float *__restrict__ r, float inv_tau, float *__restrict__ out,
                                                     int B, int I, int M, int red_chunk) {
    __shared__ __align__(16) float As[SM_K][SM_LD];
    __shared__ __align__(16) float Bs[SM_K][SM_LD];
    const int R = MODE == 2 ? M : B;                      // rows of the output
    const int C = MODE == 0 ? M : I;                      // columns of the output
    const int KD = MODE == 0 ? I : (MODE == 1 ? M : B);   // reduction length
    const int r0 = blockIdx.y * SM_T, c0 = blockIdx.x * SM_T;
    const int k_begin = blockIdx.z * red_chunk;
    const int k_end = min(KD, k_begin + red_chunk);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;  // wavefront's corner inside the tile
    constexpr bool A_RED_CONTIG = MODE != 2;
    constexpr bool B_RED_CONTIG = MODE == 0;
    // staging registers: 4 float4 per operand per thread (128 x 32 floats / 256 threads)
    float4 pa[4], pb[4];
    float bmx[4], brs[4];  // row statistics that go with pb (B operand built from W)

    auto in_a = [&](int row, int k) -> float {  // scalar fallback for ragged edges
        if (row >= R || k >= k_end) return 0.0f;
        if (MODE == 0) return x[(size_t)row * I + k];
        if (MODE == 1) return gm[(size_t)row * M + k];
        return gm[(size_t)k * M + row];
    };
    auto in_b = [&](int k, int col) -> float {
        if (col >= C || k >= k_end) return 0.0f;
        if (MODE == 0) return softmap_s(W[(size_t)col * I + k], stats[2 * col], stats[2 * col + 1], inv_tau);
        if (MODE == 1) return softmap_s(W[(size_t)k * I + col], stats[2 * k], stats[2 * k + 1], inv_tau);
        return x[(size_t)k * I + col];
    };
    // thread -> piece of the tile.  red-contiguous operand: float4 runs along k (8 per 32-deep row),
    // 32 rows per pass; row/col-contiguous operand: float4 runs along the row/col axis (32 per k), 8 k per pass
    const int a_q = A_RED_CONTIG ? (tid & 7) : (tid & 31), a_o = A_RED_CONTIG ? (tid >> 3) : (tid >> 5);
    const int b_q = B_RED_CONTIG ? (tid & 7) : (tid & 31), b_o = B_RED_CONTIG ? (tid >> 3) : (tid >> 5);
    const int lda = MODE == 0 ? I : M;
    const bool a_vec = (lda % 4 == 0), b_vec = (I % 4 == 0);

    auto fetch = [&](int k0) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            if (A_RED_CONTIG) {
                const int row = r0 + a_o + 32 * p, k = k0 + a_q * 4;
                const float *A = MODE == 0 ? x : gm;
                if (a_vec && row < R && k + 3 < k_end) pa[p] = *reinterpret_cast<const float4 *>(A + (size_t)row * lda + k);
                else pa[p] = make_float4(in_a(row, k), in_a(row, k + 1), in_a(row, k + 2), in_a(row, k + 3));
            } else {
                const int k = k0 + a_o + 8 * p, row = r0 + a_q * 4;
                if (a_vec && k < k_end && row + 3 < R) pa[p] = *reinterpret_cast<const float4 *>(gm + (size_t)k * M + row);
                else pa[p] = make_float4(in_a(row, k), in_a(row + 1, k), in_a(row + 2, k), in_a(row + 3, k));
            }
            if (B_RED_CONTIG) {
                const int col = c0 + b_o + 32 * p, k = k0 + b_q * 4;
                if (b_vec && col < C && k + 3 < k_end) {
                    pb[p] = *reinterpret_cast<const float4 *>(W + (size_t)col * I + k);
                    bmx[p] = stats[2 * col]; brs[p] = stats[2 * col + 1];
                } else {
                    pb[p] = make_float4(in_b(k, col), in_b(k + 1, col), in_b(k + 2, col), in_b(k + 3, col));
                    bmx[p] = 0.0f; brs[p] = -1.0f;  // already transformed
                }
            } else {
                const int k = k0 + b_o + 8 * p, col = c0 + b_q * 4;
                const float *Bsrc = MODE == 1 ? W : x;
                if (b_vec && k < k_end && col + 3 < C) {
                    pb[p] = *reinterpret_cast<const float4 *>(Bsrc + (size_t)k * I + col);
                    if (MODE == 1) { bmx[p] = stats[2 * k]; brs[p] = stats[2 * k + 1]; }
                } else {
                    pb[p] = make_float4(in_b(k, col), in_b(k, col + 1), in_b(k, col + 2), in_b(k, col + 3));
                    bmx[p] = 0.0f; brs[p] = -1.0f;
                }
            }
        }
    };
    auto commit = [&]() {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            if (A_RED_CONTIG) {
                const int rr = a_o + 32 * p, kk = a_q * 4;
                As[kk][rr] = pa[p].x; As[kk + 1][rr] = pa[p].y; As[kk + 2][rr] = pa[p].z; As[kk + 3][rr] = pa[p].w;
            } else {
                *reinterpret_cast<float4 *>(&As[a_o + 8 * p][a_q * 4]) = pa[p];
            }
            float4 v = pb[p];
            if (MODE != 2 && brs[p] >= 0.0f) {  // W values -> softmax entries
                v.x = softmap_s(v.x, bmx[p], brs[p], inv_tau); v.y = softmap_s(v.y, bmx[p], brs[p], inv_tau);
                v.z = softmap_s(v.z, bmx[p], brs[p], inv_tau); v.w = softmap_s(v.w, bmx[p], brs[p], inv_tau);
            }
            if (B_RED_CONTIG) {
                const int cc = b_o + 32 * p, kk = b_q * 4;
                Bs[kk][cc] = v.x; Bs[kk + 1][cc] = v.y; Bs[kk + 2][cc] = v.z; Bs[kk + 3][cc] = v.w;
            } else {
                *reinterpret_cast<float4 *>(&Bs[b_o + 8 * p][b_q * 4]) = v;
            }
        }
    };

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    if (k_begin < k_end) fetch(k_begin);
    for (int k0 = k_begin; k0 < k_end; k0 += SM_K) {
        __syncthreads();  // previous stage fully consumed
        commit();
        __syncthreads();
        if (k0 + SM_K < k_end) fetch(k0 + SM_K);
        const int kh = lane >> 5, l32 = lane & 31;
#pragma unroll
        for (int k2 = 0; k2 < SM_K; k2 += 2) {
            const float a0 = As[k2 + kh][wm + l32], a1 = As[k2 + kh][wm + 32 + l32];
            const float b0 = Bs[k2 + kh][wn + l32], b1 = Bs[k2 + kh][wn + 32 + l32];
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
        }
    }
    // accumulator layout of a 32x32 tile: register v of lane l holds row 8*(v/4) + 4*(l/32) + v%4, column l%32
    float *dst = out + (size_t)blockIdx.z * R * C;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = c0 + wn + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = r0 + wm + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row < R && col < C) {
                    float val = acc[i][j][v];
                    if (MODE == 2) {
                        const float sv = softmap_s(W[(size_t)row * I + col], stats[2 * row], stats[2 * row + 1], inv_tau);
                        val = sv * (val - r[row]) * inv_tau;
                    }
                    dst[(size_t)row * C + col] = val;
                }
            }
        }
}

// ---------------------------------------------------------------------------------
static int softmap_check(int B, int I, int M, int precision) {
    if (B <= 0 || I <= 0 || M <= 0) return DL_ERR_SHAPE;
    if (precision != 0) return DL_ERR_UNSUPPORTED;  // bf16 operands: not built yet
    return DL_OK;
}

// the gx product reduces over M; it is cut into chunks so that the grid fills the chip
static inline int softmap_gx_chunks(int B, int I, int M) {
    const int tiles = dl_ceil_div(I, SM_T) * dl_ceil_div(B, SM_T);
    int chunks = dl_ceil_div(1024, tiles);
    const int max_chunks = dl_ceil_div(M, 4 * SM_K);
    if (chunks > max_chunks) chunks = max_chunks;
    return chunks < 1 ? 1 : chunks;
}

extern "C" size_t dl_soft_map_workspace_bytes(int B, int I, int M, int precision) {
    (void)precision;
    if (B <= 0 || I <= 0 || M <= 0) return 256;
    return dl_align256((size_t)M * sizeof(float)) +
           dl_align256((size_t)softmap_gx_chunks(B, I, M) * B * I * sizeof(float));
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
    DL_TIMED("softmap_mfma_fwd", s,
             (softmap_mfma<0><<<dim3(dl_ceil_div(M, SM_T), dl_ceil_div(B, SM_T), 1), 256, 0, s>>>(
                 x, W, stats, nullptr, nullptr, inv_tau, m, B, I, M, I)));
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
    float *part = (float *)((char *)ws + dl_align256((size_t)M * sizeof(float)));
    const int chunks = softmap_gx_chunks(B, I, M);
    int red_chunk = dl_ceil_div(M, chunks);
    red_chunk = dl_ceil_div(red_chunk, SM_K) * SM_K;  // whole stages, so float4 loads stay aligned
    DL_TIMED("softmap_rowdot", s, (softmap_rowdot<<<dl_ceil_div(M, 256), 256, 0, s>>>(gm, m, r, B, M)));
    DL_TIMED("softmap_mfma_gx", s,
             (softmap_mfma<1><<<dim3(dl_ceil_div(I, SM_T), dl_ceil_div(B, SM_T), dl_ceil_div(M, red_chunk)), 256, 0, s>>>(
                 x, W, stats, gm, nullptr, inv_tau, chunks > 1 ? part : gx, B, I, M, red_chunk)));
    if (chunks > 1)
        DL_TIMED("softmap_reduce_chunks", s,
                 (softmap_reduce_chunks<<<dl_ceil_div((long long)B * I, 256), 256, 0, s>>>(part, gx, (long long)B * I,
                                                                                         dl_ceil_div(M, red_chunk))));
    DL_TIMED("softmap_mfma_gw", s,
             (softmap_mfma<2><<<dim3(dl_ceil_div(I, SM_T), dl_ceil_div(M, SM_T), 1), 256, 0, s>>>(
                 x, W, stats, gm, r, inv_tau, gW, B, I, M, B)));
    return dl_launch_status();
}
