// RandomLayer + DWN nodes, generic kernels: any k up to DL_MAX_K, one thread per element, x read
// directly, atomics for the table gradient.  Used when tables do not fit a wavefront (k > 6) and
// for the eval-mode forward; the fast path for k <= 6 is in dwn_kernels.hip.
#include "dl_common.h"
#include "dwn_generic.h"

// Generic kernels (any k up to DL_MAX_K): one thread per element, x read directly.
__device__ __forceinline__ unsigned dwn_addr_generic(const float *xrow, const int *ix, int K) {
    unsigned a = 0;
    for (int j = 0; j < K; ++j) a |= (xrow[ix[j]] >= 0.5f ? 1u : 0u) << j;
    return a;
}

__global__ __launch_bounds__(256) void dwn_generic_fwd(const float *__restrict__ x, const int *__restrict__ idx32,
                                                        const float *__restrict__ luts, float *__restrict__ y,
                                                        int B, int I, int N, int K, int O) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long NO = (long long)N * O;
    if (gid >= (long long)B * NO) return;
    const int b = (int)(gid / NO);
    const long long c = gid % NO;
    const int n = (int)(c / O);
    const unsigned a = dwn_addr_generic(x + (size_t)b * I, idx32 + (size_t)n * K, K);
    y[gid] = luts[(c << K) + a];
}

__global__ __launch_bounds__(256) void dwn_generic_bwd_gx(const float *__restrict__ x, const int *__restrict__ idx32,
                                                           const int *__restrict__ inv_ptr, const int *__restrict__ inv_pos,
                                                           const float *__restrict__ luts, const float *__restrict__ gy,
                                                           float alpha, float beta, const float *__restrict__ scale,
                                                           float *__restrict__ gx, int B, int I, int N, int K, int O,
                                                           const float *__restrict__ alpha_n, const float *__restrict__ beta_n) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (long long)B * I) return;
    const int b = (int)(gid / I), i = (int)(gid % I);
    const int L = 1 << K;
    double bp[DL_MAX_K + 1];
    bp[0] = 1.0;
    for (int h = 1; h <= K; ++h) bp[h] = scale ? 1.0 / (double)(h + 1) : bp[h - 1] * (double)beta;
    float acc = 0.0f;
    for (int e = inv_ptr[i]; e < inv_ptr[i + 1]; ++e) {
        const int p = inv_pos[e];
        const int n = p / K, j = p - n * K;
        const unsigned a = dwn_addr_generic(x + (size_t)b * I, idx32 + (size_t)n * K, K);
        const unsigned keep = ~(1u << j);
        if (beta_n)  // the node's own beta
            for (int h = 1; h <= K; ++h) bp[h] = bp[h - 1] * (double)beta_n[n];
        const double al = scale ? (double)scale[n] : (alpha_n ? (double)alpha_n[n] : (double)alpha);
        for (int d = 0; d < O; ++d) {
            const float *lut = luts + (((size_t)n * O + d) << K);
            double s = 0.0;
            for (int kap = 0; kap < L; ++kap) {
                const double w = bp[__popc((a ^ (unsigned)kap) & keep)];
                s += (((unsigned)kap >> j) & 1u) ? (double)lut[kap] * w : -(double)lut[kap] * w;
            }
            acc += gy[((size_t)b * N + n) * O + d] * (float)(al * s);
        }
    }
    gx[gid] = acc;
}

// The EFD weights alpha * beta^h are a product over the inputs, so the 2^k-term sum per (row, entry) above factors: with
// the table smoothed along every input once, S[a] = alpha / (1 - beta) * sum_kappa lut[kappa] beta^popc(a ^ kappa), the
// gradient term of slot j at address a is S[a | bit j] - S[a & ~bit j] (the S form of the k <= 6 path).  One block per
// table: the table in LDS as doubles, k butterfly passes (v <- v + beta * v[a ^ bit m]), one rounding to float.
// Amplifies rounding by (1 + |beta|)^k / (1 - beta): used for |beta| <= 1/2 only.
__global__ __launch_bounds__(256) void dwn_generic_smooth(const float *__restrict__ luts, float *__restrict__ S, float alpha,
                                                           float beta, const float *__restrict__ alpha_n,
                                                           const float *__restrict__ beta_n, int K, int O) {
    extern __shared__ double tab[];
    const int L = 1 << K;
    const size_t c = blockIdx.x;
    const double al = alpha_n ? (double)alpha_n[c / O] : (double)alpha, be = beta_n ? (double)beta_n[c / O] : (double)beta;
    for (int a = threadIdx.x; a < L; a += 256) tab[a] = (double)luts[c * L + a];
    __syncthreads();
    for (int m = 0; m < K; ++m) {
        for (int a = threadIdx.x; a < L; a += 256) {
            if (a & (1 << m)) continue;  // this thread updates the pair (a, a | bit m)
            const double lo = tab[a], hi = tab[a | (1 << m)];
            tab[a] = lo + be * hi;
            tab[a | (1 << m)] = hi + be * lo;
        }
        __syncthreads();
    }
    for (int a = threadIdx.x; a < L; a += 256) S[c * L + a] = (float)(al / (1.0 - be) * tab[a]);
}

// the input gradient from the smoothed tables: per (row, input) the entries of the input in CSR order
__global__ __launch_bounds__(256) void dwn_generic_bwd_gx_smooth(const float *__restrict__ x, const int *__restrict__ idx32,
                                                                  const int *__restrict__ inv_ptr,
                                                                  const int *__restrict__ inv_pos, const float *__restrict__ S,
                                                                  const float *__restrict__ gy, float *__restrict__ gx, int B,
                                                                  int I, int N, int K, int O) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (long long)B * I) return;
    const int b = (int)(gid / I), i = (int)(gid % I);
    float acc = 0.0f;
    for (int e = inv_ptr[i]; e < inv_ptr[i + 1]; ++e) {
        const int p = inv_pos[e];
        const int n = p / K, j = p - n * K;
        const unsigned a = dwn_addr_generic(x + (size_t)b * I, idx32 + (size_t)n * K, K);
        for (int d = 0; d < O; ++d) {
            const float *row = S + (((size_t)n * O + d) << K);
            acc += gy[((size_t)b * N + n) * O + d] * (row[a | (1u << j)] - row[a & ~(1u << j)]);
        }
    }
    gx[gid] = acc;
}

__global__ __launch_bounds__(256) void dwn_generic_bwd_luts(const float *__restrict__ x, const int *__restrict__ idx32,
                                                             const float *__restrict__ gy, const float *__restrict__ scale,
                                                             float *__restrict__ gluts, int B, int I, int N, int K, int O) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long NO = (long long)N * O;
    if (gid >= (long long)B * NO) return;
    const int b = (int)(gid / NO);
    const long long c = gid % NO;
    const int n = (int)(c / O);
    const unsigned a = dwn_addr_generic(x + (size_t)b * I, idx32 + (size_t)n * K, K);
    atomicAdd(&gluts[(c << K) + a], scale ? gy[gid] * scale[n] : gy[gid]);
}

// Eval: address = floor(sum_j x_j 2^j), no thresholding of x; table value binarised at 0.5.
// `skip_if_set` (nullable): a device flag; when it reads non-zero another kernel produces y and this one returns.
__global__ __launch_bounds__(256) void dwn_eval_fwd(const float *__restrict__ x, const int *__restrict__ idx32,
                                                     const float *__restrict__ luts, float *__restrict__ y,
                                                     int B, int I, int N, int K, int O,
                                                     const int *__restrict__ skip_if_set) {
    if (skip_if_set && *skip_if_set != 0) return;
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long NO = (long long)N * O;
    if (gid >= (long long)B * NO) return;
    const int b = (int)(gid / NO);
    const long long c = gid % NO;
    const int n = (int)(c / O);
    const float *xrow = x + (size_t)b * I;
    const int *ix = idx32 + (size_t)n * K;
    float s = 0.0f;
    for (int j = 0; j < K; ++j) s += xrow[ix[j]] * (float)(1 << j);
    long long a = (long long)s;  // truncation, as tensor.long()
    a = a < 0 ? 0 : (a > (1 << K) - 1 ? (1 << K) - 1 : a);
    y[gid] = luts[(c << K) + a] >= 0.5f ? 1.0f : 0.0f;
}

__global__ __launch_bounds__(256) void dwn_generic_zero(float *p, long long n) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0.0f;
}

// The forward with the row of x staged in the LDS by persistent blocks of 1024 threads (the thread-per-element kernel
// above reads x at random from memory: 1.62 ms at 4096 x 16384 -> 8192 nodes of 8 inputs).  Indices are read per row
// (coalesced, from the L2); what stays random is one table entry per element.
#define DWN_GENERIC_LDS_FLOATS 32768
__global__ __launch_bounds__(1024) void dwn_generic_fwd_lds(const float *__restrict__ x, const int *__restrict__ idx32,
                                                             const float *__restrict__ luts, float *__restrict__ y, int B,
                                                             int I, long long NO, int K, int O) {
    extern __shared__ float dwn_generic_row[];
    float *row = dwn_generic_row;
    const bool vec = (I & 3) == 0 && (((uintptr_t)x) & 15) == 0;
    for (int b = blockIdx.x; b < B; b += gridDim.x) {
        const float *xrow = x + (size_t)b * I;
        __syncthreads();  // the readers of the row before are done
        if (vec) {
            for (int i = threadIdx.x * 4; i < I; i += 4096)
                *reinterpret_cast<float4 *>(row + i) = *reinterpret_cast<const float4 *>(xrow + i);
        } else {
            for (int i = threadIdx.x; i < I; i += 1024) row[i] = xrow[i];
        }
        __syncthreads();
        for (long long c = threadIdx.x; c < NO; c += 1024) {
            const unsigned a = dwn_addr_generic(row, idx32 + (size_t)(c / O) * K, K);
            __builtin_nontemporal_store(luts[(c << K) + a], y + (size_t)b * NO + c);
        }
    }
}

int dwn_generic_forward(const float *x, const int *idx32, const float *luts, float *y, int B, int I, int N, int k, int O,
                        hipStream_t s) {
    const long long NO = (long long)N * O;
    if (I <= DWN_GENERIC_LDS_FLOATS && NO >= 1024) {
        const size_t lds = (size_t)I * sizeof(float);
        if (lds > 64 * 1024) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&dwn_generic_fwd_lds),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
        }
        const int per_cu = lds + 1024 <= 80 * 1024 ? 2 : 1;
        dwn_generic_fwd_lds<<<B < 256 * per_cu ? B : 256 * per_cu, 1024, lds, s>>>(x, idx32, luts, y, B, I, NO, k, O);
        return dl_launch_status();
    }
    dwn_generic_fwd<<<dl_ceil_div((long long)B * N * O, 256), 256, 0, s>>>(x, idx32, luts, y, B, I, N, k, O);
    return dl_launch_status();
}

size_t dwn_generic_smooth_bytes(int N, int k, int O) { return ((size_t)N * O << k) * sizeof(float); }

int dwn_generic_backward(const float *x, const int *idx32, const int *inv_ptr, const int *inv_pos, const float *luts,
                         const float *gy, float alpha, float beta, const float *scale, float *gx, float *gluts, int B, int I,
                         int N, int k, int O, hipStream_t s, const float *alpha_n, const float *beta_n, float beta_abs_max,
                         void *ws, size_t ws_bytes) {
    const long long NO = (long long)N * O;
    dwn_generic_zero<<<dl_ceil_div(NO << k, 256), 256, 0, s>>>(gluts, NO << k);
    dwn_generic_bwd_luts<<<dl_ceil_div((long long)B * NO, 256), 256, 0, s>>>(x, idx32, gy, scale, gluts, B, I, N, k, O);
    // EFD weights with every |beta| <= 1/2 and room for the smoothed tables: two loads per (row, entry, output)
    // instead of a 2^k-term sum
    if (gx && !scale && beta_abs_max <= 0.5f && k <= 12 && ws && ws_bytes >= dwn_generic_smooth_bytes(N, k, O)) {  // 2^k doubles of LDS
        float *S = (float *)ws;
        dwn_generic_smooth<<<(unsigned)NO, 256, sizeof(double) << k, s>>>(luts, S, alpha, beta, alpha_n, beta_n, k, O);
        dwn_generic_bwd_gx_smooth<<<dl_ceil_div((long long)B * I, 256), 256, 0, s>>>(x, idx32, inv_ptr, inv_pos, S, gy, gx, B,
                                                                                   I, N, k, O);
        return dl_launch_status();
    }
    if (gx)
        dwn_generic_bwd_gx<<<dl_ceil_div((long long)B * I, 256), 256, 0, s>>>(x, idx32, inv_ptr, inv_pos, luts, gy, alpha,
                                                                            beta, scale, gx, B, I, N, k, O, alpha_n, beta_n);
    return dl_launch_status();
}

extern "C" int dl_dwn_layer_eval(const float *x, const int32_t *idx32, const float *luts, float *y, int B, int I, int N,
                                 int k, int O, void *stream) {
    if (!x || !idx32 || !luts || !y) return DL_ERR_NULL;
    if (B <= 0 || I <= 0 || N <= 0 || k <= 0 || O <= 0) return DL_ERR_SHAPE;
    if (k > DL_MAX_K) return DL_ERR_UNSUPPORTED;
    return dwn_generic_eval(x, idx32, luts, y, B, I, N, k, O, nullptr, (hipStream_t)stream);
}

// The same eval forward for k <= 6 with the row of x staged in the LDS (64 random 4-byte reads of a row in memory cost
// the texture addresser 64 cycles per wavefront instruction; dwn_eval_fwd takes 1.03 ms at 4096 x 16384 -> 8192, this
// one a fraction).  Persistent blocks of 1024 threads; a thread owns up to QC columns of a window of columns, whose input
// indices and whose table, binarised into a 64-bit mask, it keeps in registers over all its rows: per row nothing is
// read from memory but the row of x, and y leaves coalesced.
#define DWN_EVAL_LDS_FLOATS 32768
template <int K, int QC>
__global__ __launch_bounds__(1024) void dwn_eval_fwd_lds(const float *__restrict__ x, const int *__restrict__ idx32,
                                                          const float *__restrict__ luts, float *__restrict__ y, int B,
                                                          int I, long long NO, int O, long long c_begin, long long c_end,
                                                          const int *__restrict__ skip_if_set) {
    if (skip_if_set && *skip_if_set != 0) return;
    extern __shared__ float dwn_eval_row[];
    float *row = dwn_eval_row;
    constexpr int L = 1 << K;
    int ix[QC][K];
    unsigned long long mask[QC];
#pragma unroll
    for (int q = 0; q < QC; ++q) {
        const long long c = c_begin + threadIdx.x + 1024LL * q;
        mask[q] = 0ull;
#pragma unroll
        for (int j = 0; j < K; ++j) ix[q][j] = 0;
        if (c < c_end) {
            const long long n = c / O;
#pragma unroll
            for (int j = 0; j < K; ++j) ix[q][j] = idx32[n * K + j];
            for (int a = 0; a < L; ++a) mask[q] |= (luts[(c << K) + a] >= 0.5f ? 1ull : 0ull) << a;
        }
    }
    const bool vec = (I & 3) == 0 && (((uintptr_t)x) & 15) == 0;
    for (int b = blockIdx.x; b < B; b += gridDim.x) {
        const float *xrow = x + (size_t)b * I;
        __syncthreads();  // the readers of the row before are done
        if (vec) {
            for (int i = threadIdx.x * 4; i < I; i += 4096)
                *reinterpret_cast<float4 *>(row + i) = *reinterpret_cast<const float4 *>(xrow + i);
        } else {
            for (int i = threadIdx.x; i < I; i += 1024) row[i] = xrow[i];
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < QC; ++q) {
            const long long c = c_begin + threadIdx.x + 1024LL * q;
            if (c >= c_end) break;
            float sum = 0.0f;
#pragma unroll
            for (int j = 0; j < K; ++j) sum += row[ix[q][j]] * (float)(1 << j);  // the order of dwn_eval_fwd's loop
            long long a = (long long)sum;  // truncation, as tensor.long()
            a = a < 0 ? 0 : (a > L - 1 ? L - 1 : a);
            __builtin_nontemporal_store(((mask[q] >> a) & 1ull) ? 1.0f : 0.0f, y + (size_t)b * NO + c);
        }
    }
}

int dwn_generic_eval(const float *x, const int *idx32, const float *luts, float *y, int B, int I, int N, int k, int O,
                     const int *skip_if_set, hipStream_t s) {
    const long long NO = (long long)N * O;
    if (k <= 6 && I <= DWN_EVAL_LDS_FLOATS && NO >= 1024) {
        const size_t lds = (size_t)I * sizeof(float);
        const int blocks = B < 256 ? B : 256;  // one block of 1024 threads per CU (registers)
        for (long long c0 = 0; c0 < NO; c0 += 8192) {  // windows of 8192 columns: eight per thread
            const long long c1 = c0 + 8192 < NO ? c0 + 8192 : NO;
#define DWN_EVAL_LDS(K_)                                                                                               \
    do {                                                                                                               \
        if (lds > 64 * 1024) {                                                                                         \
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&dwn_eval_fwd_lds<K_, 8>),          \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);            \
            if (e != hipSuccess) return (int)e;                                                                        \
        }                                                                                                              \
        DL_TIMED("dwn_eval_generic", s, (dwn_eval_fwd_lds<K_, 8><<<blocks, 1024, lds, s>>>(x, idx32, luts, y, B, I, NO, O, c0, c1, \
                                                                                       skip_if_set)));                 \
    } while (0)
            switch (k) {
                case 1: DWN_EVAL_LDS(1); break;
                case 2: DWN_EVAL_LDS(2); break;
                case 3: DWN_EVAL_LDS(3); break;
                case 4: DWN_EVAL_LDS(4); break;
                case 5: DWN_EVAL_LDS(5); break;
                default: DWN_EVAL_LDS(6); break;
            }
#undef DWN_EVAL_LDS
        }
        return dl_launch_status();
    }
    DL_TIMED("dwn_eval_generic", s, (dwn_eval_fwd<<<dl_ceil_div((long long)B * N * O, 256), 256, 0, s>>>(
                                        x, idx32, luts, y, B, I, N, k, O, skip_if_set)));
    return dl_launch_status();
}
