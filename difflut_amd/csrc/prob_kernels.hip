// RandomLayer + Probabilistic nodes on gfx950.
//   y[b,n,d] = sum_a sigmoid(w[n,a,d]/T) * prod_j (x_j a_j + (1-x_j)(1-a_j)),  x_j = x[b, idx[n,j]]
// i.e. the multilinear interpolation of the node's sigmoid table at the point x.
//
// k <= 6: a thread owns one node; its 2^k table entries live in registers (all of them are
// touched by every evaluation, in a fixed order, so no dynamic indexing is needed), the rows of
// x are staged in LDS and shared by the block's 256 nodes, writes of y are coalesced.
//   forward : folds the table along x_0, x_1, ... (2^k - 1 lerps)
//   backward: the same fold run backwards gives dy/dx_j and dy/dtable in O(2^k):
//             table-gradient partials are kept in registers over the block's rows and written
//             once per block to a partial buffer that a second kernel reduces in fixed order
//             (and scales by sigmoid'(w/T)/T); input-gradient terms go to a [B,N,k] buffer
//             that the CSR gather of the mapping sums in fixed order.
// k > 6: one-thread-per-element kernels with atomics.
#include "dl_common.h"

__device__ __forceinline__ float dl_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }

#define PROB_NODES 256  // nodes (= threads) per block
#define PROB_ROWS 16    // batch rows per block in the forward


// Row staging shared by the forward and backward kernels: the block's next row of x is fetched
// into registers (up to PROB_PRE float4 per thread, i.e. rows of up to 4096 floats) while the
// current one is being used from LDS, so only one barrier pair per row sits on the critical path.
// Wider or unaligned rows are staged directly.
#define PROB_PRE 4
struct ProbRowStage {
    float4 pre[PROB_PRE];
    bool vec;
    __device__ void init(const float *x, int I) { vec = (I % 4 == 0) && I <= 4 * PROB_NODES * PROB_PRE && (((size_t)x & 15) == 0); }
    __device__ void fetch(const float *x, int I, int b) {
        if (!vec) return;
        const float4 *row = reinterpret_cast<const float4 *>(x + (size_t)b * I);
#pragma unroll
        for (int u = 0; u < PROB_PRE; ++u) {
            const int q = u * PROB_NODES + threadIdx.x;
            if (q * 4 < I) pre[u] = row[q];
        }
    }
    // call between two __syncthreads(): the first guards the previous row's readers
    __device__ void commit(float *xrow, const float *x, int I, int b) {
        if (vec) {
#pragma unroll
            for (int u = 0; u < PROB_PRE; ++u) {
                const int q = u * PROB_NODES + threadIdx.x;
                if (q * 4 < I) reinterpret_cast<float4 *>(xrow)[q] = pre[u];
            }
        } else {
            for (int i = threadIdx.x; i < I; i += PROB_NODES) xrow[i] = x[(size_t)b * I + i];
        }
    }
};

// ---------------------------------------------------------------------------------
template <int K>
__global__ __launch_bounds__(PROB_NODES) void prob_fwd_kernel(const float *__restrict__ x, const int *__restrict__ idx32,
                                                               const float *__restrict__ raw, float inv_t,
                                                               float *__restrict__ y, int B, int I, int N, int O,
                                                               int rows_per_block) {
    extern __shared__ __align__(16) float xrow[];  // I floats
    constexpr int L = 1 << K;
    const int n = blockIdx.x * PROB_NODES + threadIdx.x;
    const bool live = n < N;
    int src[K];
#pragma unroll
    for (int j = 0; j < K; ++j) src[j] = live ? idx32[(size_t)n * K + j] : 0;
    const int b0 = blockIdx.y * rows_per_block;
    const int b1 = min(B, b0 + rows_per_block);
    for (int d = 0; d < O; ++d) {
        float tab[L];
#pragma unroll
        for (int a = 0; a < L; ++a) tab[a] = live ? dl_sigmoid(raw[((size_t)n * L + a) * O + d] * inv_t) : 0.0f;
        ProbRowStage stage;
        stage.init(x, I);
        if (b0 < b1) stage.fetch(x, I, b0);
        for (int b = b0; b < b1; ++b) {
            __syncthreads();
            stage.commit(xrow, x, I, b);
            __syncthreads();
            if (b + 1 < b1) stage.fetch(x, I, b + 1);
            float v[L];
#pragma unroll
            for (int a = 0; a < L; ++a) v[a] = tab[a];
#pragma unroll
            for (int j = 0; j < K; ++j) {  // fold bit j: entries a and a + 2^j with bit j clear
                const float xj = xrow[src[j]];
#pragma unroll
                for (int a = 0; a < (L >> (j + 1)); ++a) v[a] = v[2 * a] + xj * (v[2 * a + 1] - v[2 * a]);
            }
            if (live) y[((size_t)b * N + n) * O + d] = v[0];
        }
    }
}

// ---------------------------------------------------------------------------------
// Backward main kernel.  gm [B,N,k] receives dL/d(mapped input); gpart [chunks][N*L*O] the
// per-block sums of gy * p_a (before the sigmoid-derivative factor).
template <int K>
__global__ __launch_bounds__(PROB_NODES) void prob_bwd_kernel(const float *__restrict__ x, const int *__restrict__ idx32,
                                                               const float *__restrict__ raw, float inv_t,
                                                               const float *__restrict__ gy, float *__restrict__ gm,
                                                               float *__restrict__ gpart, int B, int I, int N, int O,
                                                               int rows_per_block, int want_gm) {
    extern __shared__ __align__(16) float xrow[];
    constexpr int L = 1 << K;
    const int n = blockIdx.x * PROB_NODES + threadIdx.x;
    const bool live = n < N;
    int src[K];
#pragma unroll
    for (int j = 0; j < K; ++j) src[j] = live ? idx32[(size_t)n * K + j] : 0;
    const int b0 = blockIdx.y * rows_per_block;
    const int b1 = min(B, b0 + rows_per_block);
    for (int d = 0; d < O; ++d) {
        float tab[L], gt[L];
#pragma unroll
        for (int a = 0; a < L; ++a) {
            tab[a] = live ? dl_sigmoid(raw[((size_t)n * L + a) * O + d] * inv_t) : 0.0f;
            gt[a] = 0.0f;
        }
        ProbRowStage stage;
        stage.init(x, I);
        if (b0 < b1) stage.fetch(x, I, b0);
        for (int b = b0; b < b1; ++b) {
            __syncthreads();
            stage.commit(xrow, x, I, b);
            __syncthreads();
            if (b + 1 < b1) stage.fetch(x, I, b + 1);
            float xs[K];
#pragma unroll
            for (int j = 0; j < K; ++j) xs[j] = xrow[src[j]];
            const float g = live ? gy[((size_t)b * N + n) * O + d] : 0.0f;
            // p[a] = prod_j (a_j ? x_j : 1 - x_j), built by doubling: after step j, p[0 .. 2^(j+1)) is
            // the product over inputs 0..j
            float p[L];
            p[0] = 1.0f;
#pragma unroll
            for (int j = 0; j < K; ++j) {
#pragma unroll
                for (int a = (1 << j) - 1; a >= 0; --a) {
                    p[a + (1 << j)] = p[a] * xs[j];
                    p[a] = p[a] * (1.0f - xs[j]);
                }
            }
#pragma unroll
            for (int a = 0; a < L; ++a) gt[a] += g * p[a];
            if (want_gm) {
                // dy/dx_j = sum_a tab[a] (2 a_j - 1) prod_{m != j} q_m: fold the table along every input but j
#pragma unroll
                for (int j = 0; j < K; ++j) {
                    float v[L / 2 > 0 ? L / 2 : 1];
#pragma unroll
                    for (int a = 0; a < L / 2; ++a) {
                        const int lo = (a & ((1 << j) - 1)) | ((a >> j) << (j + 1));
                        v[a] = tab[lo | (1 << j)] - tab[lo];
                    }
                    int m = 0;
#pragma unroll
                    for (int jj = 0; jj < K; ++jj) {
                        if (jj == j) continue;
#pragma unroll
                        for (int a = 0; a < (L >> (m + 2)); ++a) v[a] = v[2 * a] + xs[jj] * (v[2 * a + 1] - v[2 * a]);
                        ++m;
                    }
                    if (live) {
                        float *dst = gm + ((size_t)b * N + n) * K + j;
                        if (d == 0) *dst = g * v[0]; else *dst += g * v[0];
                    }
                }
            }
        }
        if (live) {
            float *dst = gpart + (size_t)blockIdx.y * N * L * O + (size_t)n * L * O + d;
#pragma unroll
            for (int a = 0; a < L; ++a) dst[(size_t)a * O] = gt[a];
        }
    }
}

// graw[e] = sigmoid'(w/T)/T * sum over chunks of gpart[chunk][e]
__global__ __launch_bounds__(256) void prob_reduce_weights(const float *__restrict__ gpart, const float *__restrict__ raw,
                                                            float inv_t, float *__restrict__ graw, long long total,
                                                            int chunks) {
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    float acc = 0.0f;
    for (int c = 0; c < chunks; ++c) acc += gpart[(size_t)c * total + e];
    const float s = dl_sigmoid(raw[e] * inv_t);
    graw[e] = acc * s * (1.0f - s) * inv_t;
}

// ---------------------------------------------------------------------------------
// Generic kernels, any k up to DL_MAX_K.
__global__ __launch_bounds__(256) void prob_generic_fwd(const float *__restrict__ x, const int *__restrict__ idx32,
                                                         const float *__restrict__ raw, float inv_t, float *__restrict__ y,
                                                         int B, int I, int N, int K, int O) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long NO = (long long)N * O;
    if (gid >= (long long)B * NO) return;
    const int b = (int)(gid / NO);
    const int n = (int)((gid % NO) / O), d = (int)((gid % NO) % O);
    float xs[DL_MAX_K];
    for (int j = 0; j < K; ++j) xs[j] = x[(size_t)b * I + idx32[(size_t)n * K + j]];
    const int L = 1 << K;
    float acc = 0.0f;
    for (int a = 0; a < L; ++a) {
        float p = 1.0f;
        for (int j = 0; j < K; ++j) p *= ((a >> j) & 1) ? xs[j] : 1.0f - xs[j];
        acc += dl_sigmoid(raw[((size_t)n * L + a) * O + d] * inv_t) * p;
    }
    y[gid] = acc;
}

__global__ __launch_bounds__(256) void prob_generic_bwd(const float *__restrict__ x, const int *__restrict__ idx32,
                                                         const float *__restrict__ raw, float inv_t,
                                                         const float *__restrict__ gy, float *__restrict__ gx,
                                                         float *__restrict__ graw, int B, int I, int N, int K, int O) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (long long)B * N) return;
    const int b = (int)(gid / N), n = (int)(gid % N);
    float xs[DL_MAX_K], gxs[DL_MAX_K];
    for (int j = 0; j < K; ++j) { xs[j] = x[(size_t)b * I + idx32[(size_t)n * K + j]]; gxs[j] = 0.0f; }
    const int L = 1 << K;
    for (int d = 0; d < O; ++d) {
        const float g = gy[((size_t)b * N + n) * O + d];
        for (int a = 0; a < L; ++a) {
            const size_t w = ((size_t)n * L + a) * O + d;
            const float s = dl_sigmoid(raw[w] * inv_t);
            float p = 1.0f;
            for (int j = 0; j < K; ++j) p *= ((a >> j) & 1) ? xs[j] : 1.0f - xs[j];
            atomicAdd(&graw[w], g * p * s * (1.0f - s) * inv_t);
            if (gx) {
                for (int j = 0; j < K; ++j) {
                    float q = 1.0f;
                    for (int m = 0; m < K; ++m)
                        if (m != j) q *= ((a >> m) & 1) ? xs[m] : 1.0f - xs[m];
                    gxs[j] += g * s * (((a >> j) & 1) ? q : -q);
                }
            }
        }
    }
    if (gx)
        for (int j = 0; j < K; ++j) atomicAdd(&gx[(size_t)b * I + idx32[(size_t)n * K + j]], gxs[j]);
}

__global__ __launch_bounds__(256) void prob_eval_kernel(const float *__restrict__ x, const int *__restrict__ idx32,
                                                         const float *__restrict__ raw, float inv_t, float *__restrict__ y,
                                                         int B, int I, int N, int K, int O) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long NO = (long long)N * O;
    if (gid >= (long long)B * NO) return;
    const int b = (int)(gid / NO);
    const int n = (int)((gid % NO) / O), d = (int)((gid % NO) % O);
    float s = 0.0f;
    for (int j = 0; j < K; ++j) s += x[(size_t)b * I + idx32[(size_t)n * K + j]] * (float)(1 << j);
    long long a = (long long)s;
    const int L = 1 << K;
    a = a < 0 ? 0 : (a > L - 1 ? L - 1 : a);
    y[gid] = dl_sigmoid(raw[((size_t)n * L + a) * O + d] * inv_t) >= 0.5f ? 1.0f : 0.0f;
}

__global__ __launch_bounds__(256) void prob_fill_zero(float *p, long long n) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0.0f;
}

// gather of the mapping adjoint: one block per batch row; the row of gm [N*k] is staged in LDS when it
// fits (coalesced read), then every input sums its CSR entries from LDS in fixed order.
__global__ __launch_bounds__(256) void prob_gather_bwd(const float *__restrict__ gm, const int *__restrict__ inv_ptr,
                                                        const int *__restrict__ inv_pos, float *__restrict__ gx, int I,
                                                        long long NK, int staged) {
    extern __shared__ __align__(16) float grow[];
    const int b = blockIdx.x;
    const float *row = gm + (size_t)b * NK;
    if (staged) {
        for (long long p = threadIdx.x; p < NK; p += 256) grow[p] = row[p];
        __syncthreads();
    }
    for (int i = threadIdx.x; i < I; i += 256) {
        float acc = 0.0f;
        for (int e = inv_ptr[i]; e < inv_ptr[i + 1]; ++e) acc += staged ? grow[inv_pos[e]] : row[inv_pos[e]];
        gx[(size_t)b * I + i] = acc;
    }
}

// ---------------------------------------------------------------------------------
static int prob_check(int B, int I, int N, int k, int O) {
    if (B <= 0 || I <= 0 || N <= 0 || k <= 0 || O <= 0) return DL_ERR_SHAPE;
    if (k > DL_MAX_K) return DL_ERR_UNSUPPORTED;
    return DL_OK;
}
static inline bool prob_fast(int I, int k) { return k <= DL_MAX_FAST_K && (size_t)I * sizeof(float) <= 64 * 1024; }
static inline float prob_inv_t(float t) { return 1.0f / (t > 1e-6f ? t : 1e-6f); }  // temperature.clamp(min=1e-6)
static inline int prob_bwd_rows(int B) {  // rows per block: at most 64 partial buffers
    int r = (B + 63) / 64;
    return r < 16 ? 16 : r;
}

extern "C" size_t dl_prob_bwd_workspace_bytes(int B, int I, int N, int k, int O) {
    if (!prob_fast(I, k)) return 256;
    const int chunks = dl_ceil_div(B, prob_bwd_rows(B));
    return dl_align256((size_t)B * N * k * sizeof(float)) +
           dl_align256((size_t)chunks * N * ((size_t)1 << k) * O * sizeof(float));
}

#define PROB_DISPATCH(K, CALL) \
    switch (K) {               \
        case 1: CALL(1); break; case 2: CALL(2); break; case 3: CALL(3); break; \
        case 4: CALL(4); break; case 5: CALL(5); break; default: CALL(6); break; \
    }

extern "C" int dl_prob_layer_fwd(const float *x, const int32_t *idx32, const float *raw_w, float temperature, float *y,
                                 int B, int I, int N, int k, int O, void *stream) {
    if (!x || !idx32 || !raw_w || !y) return DL_ERR_NULL;
    int rc = prob_check(B, I, N, k, O);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    const float inv_t = prob_inv_t(temperature);
    if (!prob_fast(I, k)) {
        DL_TIMED("prob_generic_fwd", s, (prob_generic_fwd<<<dl_ceil_div((long long)B * N * O, 256), 256, 0, s>>>(x, idx32, raw_w, inv_t, y, B, I, N, k, O)));
        return dl_launch_status();
    }
    dim3 grid(dl_ceil_div(N, PROB_NODES), dl_ceil_div(B, PROB_ROWS));
    const size_t lds = (size_t)I * sizeof(float);
#define CALL(KK) \
    DL_TIMED("prob_fwd_kernel", s, (prob_fwd_kernel<KK><<<grid, PROB_NODES, lds, s>>>(x, idx32, raw_w, inv_t, y, B, I, N, O, PROB_ROWS)))
    PROB_DISPATCH(k, CALL)
#undef CALL
    return dl_launch_status();
}

extern "C" int dl_prob_layer_bwd(const float *x, const int32_t *idx32, const int32_t *inv_ptr, const int32_t *inv_pos,
                                 const float *raw_w, float temperature, const float *gy, float *gx, float *graw,
                                 void *ws, size_t ws_bytes, int B, int I, int N, int k, int O, void *stream) {
    if (!x || !idx32 || !raw_w || !gy || !graw) return DL_ERR_NULL;
    if (gx && (!inv_ptr || !inv_pos)) return DL_ERR_NULL;
    int rc = prob_check(B, I, N, k, O);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    const float inv_t = prob_inv_t(temperature);
    const long long WT = (long long)N * ((long long)1 << k) * O;
    if (!prob_fast(I, k)) {
        DL_TIMED("prob_fill_zero", s, (prob_fill_zero<<<dl_ceil_div(WT, 256), 256, 0, s>>>(graw, WT)));
        if (gx) prob_fill_zero<<<dl_ceil_div((long long)B * I, 256), 256, 0, s>>>(gx, (long long)B * I);
        DL_TIMED("prob_generic_bwd", s, (prob_generic_bwd<<<dl_ceil_div((long long)B * N, 256), 256, 0, s>>>(x, idx32, raw_w, inv_t, gy, gx, graw, B, I, N,
                                                                          k, O)));
        return dl_launch_status();
    }
    if (!ws) return DL_ERR_NULL;
    if (ws_bytes < dl_prob_bwd_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    const int rows = prob_bwd_rows(B);
    const int chunks = dl_ceil_div(B, rows);
    float *gm = (float *)ws;
    float *gpart = (float *)((char *)ws + dl_align256((size_t)B * N * k * sizeof(float)));
    dim3 grid(dl_ceil_div(N, PROB_NODES), chunks);
    const size_t lds = (size_t)I * sizeof(float);
#define CALL(KK)                                                                                                     \
    DL_TIMED("prob_bwd_kernel", s,                                                                                   \
             (prob_bwd_kernel<KK><<<grid, PROB_NODES, lds, s>>>(x, idx32, raw_w, inv_t, gy, gm, gpart, B, I, N, O, rows, \
                                                                gx != nullptr)))
    PROB_DISPATCH(k, CALL)
#undef CALL
    DL_TIMED("prob_reduce_weights", s,
             (prob_reduce_weights<<<dl_ceil_div(WT, 256), 256, 0, s>>>(gpart, raw_w, inv_t, graw, WT, chunks)));
    const int staged = (size_t)N * k * sizeof(float) <= 64 * 1024;
    const size_t gbytes = staged ? (size_t)N * k * sizeof(float) : 0;
    if (gx)
        DL_TIMED("prob_gather_bwd", s,
                 (prob_gather_bwd<<<B, 256, gbytes, s>>>(gm, inv_ptr, inv_pos, gx, I, (long long)N * k, staged)));
    return dl_launch_status();
}

extern "C" int dl_prob_layer_eval(const float *x, const int32_t *idx32, const float *raw_w, float temperature, float *y,
                                  int B, int I, int N, int k, int O, void *stream) {
    if (!x || !idx32 || !raw_w || !y) return DL_ERR_NULL;
    int rc = prob_check(B, I, N, k, O);
    if (rc) return rc;
    DL_TIMED("prob_eval_kernel", (hipStream_t)stream, (prob_eval_kernel<<<dl_ceil_div((long long)B * N * O, 256), 256, 0, (hipStream_t)stream>>>(
        x, idx32, raw_w, prob_inv_t(temperature), y, B, I, N, k, O)));
    return dl_launch_status();
}
