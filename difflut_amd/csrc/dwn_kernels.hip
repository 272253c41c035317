// RandomLayer + DWN nodes on gfx950: forward (threshold, address, lookup) and the
// extended-finite-difference backward, whole layer per call.
//
// Layout idea (k <= 6): a wavefront's 64 lanes are 64 batch rows.  Everything that
// belongs to a node - its k input indices, its 2^k-entry table, its EFD coefficient
// rows - is then wave-uniform: indices and bit-plane words come through scalar loads,
// a table sits one entry per lane in a single VGPR and a lookup is one ds_bpermute.
// The random RandomLayer mapping costs nothing in this layout; what it costs instead
// is one transpose through LDS wherever a tensor crosses the [batch, feature] boundary
// (y out, gy in, gx out).
//
//   forward   pack_planes : x [B,I] fp32 -> planes [B/64][I] u64 (bit r = x[64t+r][i] >= 0.5)
//             lookup_fwd  : planes + idx + luts -> y [B,N*O] (LDS-transposed tiles) and
//                           addrT [N][B] u8, the address of every (node,row), kept for backward
//   backward  efd_table   : luts -> D[n][d][j][a'] = alpha * sum_kappa s(kappa_j) lut[kappa]
//                           beta^popc((a^kappa)&~(1<<j)), a' = address with bit j squeezed out
//             transpose_hist : gy [B,N*O] -> gyT [N*O][B]; per-node 2^k-bin histogram of gy
//                           in LDS, one float atomic per bin per block into gluts
//             bwd_gx      : for every input i the (node,slot) pairs that read it (CSR):
//                           gx[b,i] = sum gyT[c][b] * D[c][j][a'(b)]  - a gather in fixed order
// k > 6 falls back to plain one-thread-per-element kernels further down.
#include "dl_common.h"

typedef unsigned long long u64;

// ---------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dl_fill_zero_kernel(float *p, long long n) {
    long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0.0f;
}
static void dl_fill_zero(float *p, long long n, hipStream_t s) {
    if (n > 0) DL_TIMED("dl_fill_zero", s, (dl_fill_zero_kernel<<<dl_ceil_div(n, 256), 256, 0, s>>>(p, n)));
}

// ---------------------------------------------------------------------------------
// pack_planes: grid (ceil(I / (256*VEC)), B/64 rounded up), 256 threads, thread = VEC inputs.
// Every load of a wavefront is one contiguous 64*VEC*4-byte piece of a row of x.
template <int VEC>
__global__ __launch_bounds__(256) void dwn_pack_planes(const float *__restrict__ x, u64 *__restrict__ planes,
                                                        int B, int I) {
    const int t = blockIdx.y;
    const int i0 = (blockIdx.x * 256 + threadIdx.x) * VEC;
    if (i0 >= I) return;
    const int rows = min(64, B - t * 64);
    const float *base = x + (size_t)t * 64 * I + i0;
    unsigned lo[VEC], hi[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) lo[v] = hi[v] = 0u;
    if (rows == 64) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            unsigned *acc = half ? hi : lo;
#pragma unroll
            for (int r = 0; r < 32; ++r) {
                const float *src = base + (size_t)(r + 32 * half) * I;
                if constexpr (VEC == 4) {
                    const float4 q = *reinterpret_cast<const float4 *>(src);
                    acc[0] |= (q.x >= 0.5f ? 1u : 0u) << r;
                    acc[1] |= (q.y >= 0.5f ? 1u : 0u) << r;
                    acc[2] |= (q.z >= 0.5f ? 1u : 0u) << r;
                    acc[3] |= (q.w >= 0.5f ? 1u : 0u) << r;
                } else {
                    acc[0] |= (src[0] >= 0.5f ? 1u : 0u) << r;
                }
            }
        }
    } else {
        for (int r = 0; r < rows; ++r) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                const unsigned bit = base[(size_t)r * I + v] >= 0.5f ? 1u : 0u;
                if (r < 32) lo[v] |= bit << r; else hi[v] |= bit << (r - 32);
            }
        }
    }
    u64 *out = planes + (size_t)t * I + i0;
#pragma unroll
    for (int v = 0; v < VEC; ++v) out[v] = ((u64)hi[v] << 32) | lo[v];
}

// ---------------------------------------------------------------------------------
// lookup_fwd: grid (ceil(N*O / 128), B/64), 256 threads = 4 wavefronts, lane = batch row.
#define DWN_TC 128
template <int K>
__global__ __launch_bounds__(256) void dwn_lookup_fwd(const u64 *__restrict__ planes, const int *__restrict__ idx32,
                                                       const float *__restrict__ luts, float *__restrict__ y,
                                                       uint8_t *__restrict__ addrT, int B, int I, int N, int O, int BP) {
    __shared__ float tile[64][DWN_TC + 1];
    constexpr int L = 1 << K;
    const int t = blockIdx.y;
    const int c0 = blockIdx.x * DWN_TC;
    const int NO = N * O;
    const int lane = threadIdx.x & 63;
    const int wave = dl_uniform(threadIdx.x >> 6);
    const u64 *pl = planes + (size_t)t * I;
    const int cend = min(DWN_TC, NO - c0);
    for (int cc = wave; cc < cend; cc += 4) {
        const int c = c0 + cc;
        const int n = c / O;
        unsigned addr = 0;
#pragma unroll
        for (int j = 0; j < K; ++j) {
            const int src = idx32[n * K + j];  // wave-uniform: scalar load
            const u64 w = pl[src];             // wave-uniform: scalar load
            const unsigned half = lane < 32 ? (unsigned)w : (unsigned)(w >> 32);
            addr |= ((half >> (lane & 31)) & 1u) << j;
        }
        const float entry = luts[(size_t)c * L + (lane & (L - 1))];  // table, one entry per lane
        tile[lane][cc] = dl_lane_read(entry, (int)addr);
        if (c - n * O == 0) addrT[(size_t)n * BP + t * 64 + lane] = (uint8_t)addr;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < 64 * DWN_TC; e += 256) {
        const int r = e / DWN_TC, cc = e % DWN_TC;
        const int b = t * 64 + r;
        if (b < B && cc < cend) y[(size_t)b * NO + c0 + cc] = tile[r][cc];
    }
}

// ---------------------------------------------------------------------------------
// efd_table: one thread per coefficient.  Double accumulation, one rounding to float.
__global__ __launch_bounds__(256) void dwn_efd_table(const float *__restrict__ luts, float *__restrict__ D,
                                                      int NO, int K, float alpha, float beta) {
    const int Lh = 1 << (K - 1), L = 1 << K;
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (long long)NO * K * Lh) return;
    const int ap = (int)(gid % Lh);
    const int j = (int)((gid / Lh) % K);
    const long long c = gid / ((long long)Lh * K);
    const unsigned a = ((unsigned)ap & ((1u << j) - 1u)) | (((unsigned)ap >> j) << (j + 1));  // bit j = 0
    double bp[DL_MAX_FAST_K + 1];
    bp[0] = 1.0;
#pragma unroll
    for (int h = 1; h <= DL_MAX_FAST_K; ++h) bp[h] = bp[h - 1] * (double)beta;
    const unsigned keep = ~(1u << j);
    const float *lut = luts + c * L;
    double acc = 0.0;
    for (int kap = 0; kap < L; ++kap) {
        const int h = __popc((a ^ (unsigned)kap) & keep);
        double w = 1.0;
#pragma unroll
        for (int q = 1; q <= DL_MAX_FAST_K; ++q) w = (h == q) ? bp[q] : w;
        acc += (((unsigned)kap >> j) & 1u) ? (double)lut[kap] * w : -(double)lut[kap] * w;
    }
    D[gid] = (float)((double)alpha * acc);
}

// ---------------------------------------------------------------------------------
// transpose_hist: grid (ceil(N*O / 128), chunks), block streams `tiles_per_chunk` 64-row tiles.
template <bool WRITE_T>
__global__ __launch_bounds__(256) void dwn_bwd_transpose_hist(const float *__restrict__ gy, const uint8_t *__restrict__ addrT,
                                                               float *__restrict__ gyT, float *__restrict__ gluts,
                                                               int B, int NO, int O, int L, int BP, int BT,
                                                               int tiles_per_chunk) {
    __shared__ float tile[64][DWN_TC + 1];
    __shared__ float hist[DWN_TC * 64];
    const int c0 = blockIdx.x * DWN_TC;
    const int lane = threadIdx.x & 63;
    const int wave = dl_uniform(threadIdx.x >> 6);
    const int cend = min(DWN_TC, NO - c0);
    for (int e = threadIdx.x; e < DWN_TC * 64; e += 256) hist[e] = 0.0f;
    const int t_begin = blockIdx.y * tiles_per_chunk;
    const int t_end = min(BT, t_begin + tiles_per_chunk);
    const bool vec4 = (NO % 4 == 0);
    for (int t = t_begin; t < t_end; ++t) {
        __syncthreads();
        if (vec4) {  // 32 threads x 16 B cover one 128-column row piece; 8 rows per pass
            const int q = threadIdx.x & 31, rr = threadIdx.x >> 5;
#pragma unroll
            for (int r8 = 0; r8 < 64; r8 += 8) {
                const int r = r8 + rr, b = t * 64 + r, cc = q * 4;
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (b < B && cc < cend) v = *reinterpret_cast<const float4 *>(gy + (size_t)b * NO + c0 + cc);
                tile[r][cc] = v.x; tile[r][cc + 1] = v.y; tile[r][cc + 2] = v.z; tile[r][cc + 3] = v.w;
            }
        } else {
            for (int e = threadIdx.x; e < 64 * DWN_TC; e += 256) {
                const int r = e / DWN_TC, cc = e % DWN_TC;
                const int b = t * 64 + r;
                tile[r][cc] = (b < B && cc < cend) ? gy[(size_t)b * NO + c0 + cc] : 0.0f;
            }
        }
        __syncthreads();
        for (int cc = wave; cc < cend; cc += 4) {
            const int c = c0 + cc;
            const int n = c / O;
            const float v = tile[lane][cc];
            if (WRITE_T) gyT[(size_t)c * BP + t * 64 + lane] = v;
            const unsigned a = addrT[(size_t)n * BP + t * 64 + lane];
            atomicAdd(&hist[cc * L + a], v);  // rows past B carry v = 0
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < cend * L; e += 256) atomicAdd(&gluts[(size_t)c0 * L + e], hist[e]);
}

// ---------------------------------------------------------------------------------
// bwd_gx: grid (ceil(I / 128), B/64), lane = batch row, wavefront walks inputs of the slab.
#define DWN_IS 128
template <int K>
__global__ __launch_bounds__(256) void dwn_bwd_gx(const float *__restrict__ gyT, const uint8_t *__restrict__ addrT,
                                                   const float *__restrict__ D, const int *__restrict__ inv_ptr,
                                                   const int *__restrict__ inv_pos, float *__restrict__ gx,
                                                   int B, int I, int O, int BP) {
    __shared__ float tile[DWN_IS][65];
    constexpr int Lh = 1 << (K - 1);
    const int t = blockIdx.y;
    const int i0 = blockIdx.x * DWN_IS;
    const int lane = threadIdx.x & 63;
    const int wave = dl_uniform(threadIdx.x >> 6);
    const int iend = min(DWN_IS, I - i0);
    const size_t col = (size_t)t * 64 + lane;
    for (int ii = wave; ii < iend; ii += 4) {
        const int e0 = inv_ptr[i0 + ii], e1 = inv_ptr[i0 + ii + 1];
        float acc = 0.0f;
        for (int e = e0; e < e1; ++e) {
            const int p = inv_pos[e];
            const int n = p / K, j = p - n * K;
            const unsigned a = addrT[(size_t)n * BP + col];
            const unsigned ap = (a & ((1u << j) - 1u)) | ((a >> (j + 1)) << j);
            for (int d = 0; d < O; ++d) {
                const size_t c = (size_t)n * O + d;
                const float g = gyT[c * BP + col];
                const float coef = D[(c * K + j) * Lh + (lane & (Lh - 1))];
                acc += g * dl_lane_read(coef, (int)ap);
            }
        }
        tile[ii][lane] = acc;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < 64 * DWN_IS; e += 256) {
        const int r = e / DWN_IS, ii = e % DWN_IS;
        const int b = t * 64 + r;
        if (b < B && ii < iend) gx[(size_t)b * I + i0 + ii] = tile[ii][r];
    }
}

// ---------------------------------------------------------------------------------
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
                                                           float alpha, float beta, float *__restrict__ gx,
                                                           int B, int I, int N, int K, int O) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (long long)B * I) return;
    const int b = (int)(gid / I), i = (int)(gid % I);
    const int L = 1 << K;
    double bp[DL_MAX_K + 1];
    bp[0] = 1.0;
    for (int h = 1; h <= K; ++h) bp[h] = bp[h - 1] * (double)beta;
    float acc = 0.0f;
    for (int e = inv_ptr[i]; e < inv_ptr[i + 1]; ++e) {
        const int p = inv_pos[e];
        const int n = p / K, j = p - n * K;
        const unsigned a = dwn_addr_generic(x + (size_t)b * I, idx32 + (size_t)n * K, K);
        const unsigned keep = ~(1u << j);
        for (int d = 0; d < O; ++d) {
            const float *lut = luts + (((size_t)n * O + d) << K);
            double s = 0.0;
            for (int kap = 0; kap < L; ++kap) {
                const double w = bp[__popc((a ^ (unsigned)kap) & keep)];
                s += (((unsigned)kap >> j) & 1u) ? (double)lut[kap] * w : -(double)lut[kap] * w;
            }
            acc += gy[((size_t)b * N + n) * O + d] * (float)((double)alpha * s);
        }
    }
    gx[gid] = acc;
}

__global__ __launch_bounds__(256) void dwn_generic_bwd_luts(const float *__restrict__ x, const int *__restrict__ idx32,
                                                             const float *__restrict__ gy, float *__restrict__ gluts,
                                                             int B, int I, int N, int K, int O) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long NO = (long long)N * O;
    if (gid >= (long long)B * NO) return;
    const int b = (int)(gid / NO);
    const long long c = gid % NO;
    const int n = (int)(c / O);
    const unsigned a = dwn_addr_generic(x + (size_t)b * I, idx32 + (size_t)n * K, K);
    atomicAdd(&gluts[(c << K) + a], gy[gid]);
}

// Eval: address = floor(sum_j x_j 2^j), no thresholding of x; table value binarised at 0.5.
__global__ __launch_bounds__(256) void dwn_eval_fwd(const float *__restrict__ x, const int *__restrict__ idx32,
                                                     const float *__restrict__ luts, float *__restrict__ y,
                                                     int B, int I, int N, int K, int O) {
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

// ---------------------------------------------------------------------------------
// Host side
static inline int dwn_bt(int B) { return (B + 63) / 64; }
static inline size_t dwn_planes_bytes(int B, int I) { return dl_align256((size_t)dwn_bt(B) * I * sizeof(u64)); }
static inline size_t dwn_table_bytes(int N, int k, int O) {
    return dl_align256((size_t)N * O * k * ((size_t)1 << (k - 1)) * sizeof(float));
}
static inline size_t dwn_gyT_bytes(int B, int N, int O) {
    return dl_align256((size_t)N * O * dwn_bt(B) * 64 * sizeof(float));
}

static int dwn_check(int B, int I, int N, int k, int O) {
    if (B <= 0 || I <= 0 || N <= 0 || k <= 0 || O <= 0) return DL_ERR_SHAPE;
    if (k > DL_MAX_K) return DL_ERR_UNSUPPORTED;
    if ((long long)N * O * ((long long)1 << k) > 0x7fffffffLL) return DL_ERR_UNSUPPORTED;
    return DL_OK;
}

extern "C" size_t dl_dwn_saved_bytes(int B, int I, int N, int k, int O) {
    (void)I; (void)O;
    if (k > DL_MAX_FAST_K) return 256;  // nothing is kept; a token allocation keeps callers simple
    return dl_align256((size_t)N * dwn_bt(B) * 64);
}
extern "C" size_t dl_dwn_fwd_workspace_bytes(int B, int I, int N, int k, int O) {
    (void)N; (void)O;
    return k > DL_MAX_FAST_K ? 256 : dwn_planes_bytes(B, I);
}
extern "C" size_t dl_dwn_bwd_workspace_bytes(int B, int I, int N, int k, int O) {
    (void)I;
    return k > DL_MAX_FAST_K ? 256 : dwn_table_bytes(N, k, O) + dwn_gyT_bytes(B, N, O);
}

template <int K>
static void dwn_launch_lookup(const u64 *planes, const int *idx32, const float *luts, float *y, uint8_t *addrT,
                              int B, int I, int N, int O, hipStream_t s) {
    dim3 grid(dl_ceil_div((long long)N * O, DWN_TC), dwn_bt(B));
    DL_TIMED("dwn_lookup_fwd", s, (dwn_lookup_fwd<K><<<grid, 256, 0, s>>>(planes, idx32, luts, y, addrT, B, I, N, O, dwn_bt(B) * 64)));
}

extern "C" int dl_dwn_layer_fwd(const float *x, const int32_t *idx32, const float *luts, float *y, void *saved,
                                void *ws, size_t ws_bytes, int B, int I, int N, int k, int O, void *stream) {
    if (!x || !idx32 || !luts || !y) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (k > DL_MAX_FAST_K) {
        dwn_generic_fwd<<<dl_ceil_div((long long)B * N * O, 256), 256, 0, s>>>(x, idx32, luts, y, B, I, N, k, O);
        return dl_launch_status();
    }
    if (!saved || !ws) return DL_ERR_NULL;
    if (ws_bytes < dl_dwn_fwd_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    u64 *planes = (u64 *)ws;
    const int BT = dwn_bt(B);
    if (I % 4 == 0 && ((uintptr_t)x & 15) == 0)
        DL_TIMED("dwn_pack_planes", s, (dwn_pack_planes<4><<<dim3(dl_ceil_div(I, 1024), BT), 256, 0, s>>>(x, planes, B, I)));
    else
        DL_TIMED("dwn_pack_planes", s, (dwn_pack_planes<1><<<dim3(dl_ceil_div(I, 256), BT), 256, 0, s>>>(x, planes, B, I)));
    uint8_t *addrT = (uint8_t *)saved;
    switch (k) {
        case 1: dwn_launch_lookup<1>(planes, idx32, luts, y, addrT, B, I, N, O, s); break;
        case 2: dwn_launch_lookup<2>(planes, idx32, luts, y, addrT, B, I, N, O, s); break;
        case 3: dwn_launch_lookup<3>(planes, idx32, luts, y, addrT, B, I, N, O, s); break;
        case 4: dwn_launch_lookup<4>(planes, idx32, luts, y, addrT, B, I, N, O, s); break;
        case 5: dwn_launch_lookup<5>(planes, idx32, luts, y, addrT, B, I, N, O, s); break;
        default: dwn_launch_lookup<6>(planes, idx32, luts, y, addrT, B, I, N, O, s); break;
    }
    return dl_launch_status();
}

template <int K>
static void dwn_launch_gx(const float *gyT, const uint8_t *addrT, const float *D, const int *inv_ptr, const int *inv_pos,
                          float *gx, int B, int I, int O, hipStream_t s) {
    dim3 grid(dl_ceil_div(I, DWN_IS), dwn_bt(B));
    DL_TIMED("dwn_bwd_gx", s, (dwn_bwd_gx<K><<<grid, 256, 0, s>>>(gyT, addrT, D, inv_ptr, inv_pos, gx, B, I, O, dwn_bt(B) * 64)));
}

extern "C" int dl_dwn_layer_bwd(const float *x, const void *saved, const int32_t *idx32, const int32_t *inv_ptr,
                                const int32_t *inv_pos, const float *luts, const float *gy, float alpha, float beta,
                                float *gx, float *gluts, void *ws, size_t ws_bytes, int B, int I, int N, int k, int O,
                                void *stream) {
    if (!idx32 || !luts || !gy || !gluts) return DL_ERR_NULL;
    if (gx && (!inv_ptr || !inv_pos)) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    const long long NO = (long long)N * O;
    const int L = 1 << k;
    dl_fill_zero(gluts, NO * L, s);
    if (k > DL_MAX_FAST_K) {
        if (!x) return DL_ERR_NULL;
        dwn_generic_bwd_luts<<<dl_ceil_div((long long)B * NO, 256), 256, 0, s>>>(x, idx32, gy, gluts, B, I, N, k, O);
        if (gx)
            dwn_generic_bwd_gx<<<dl_ceil_div((long long)B * I, 256), 256, 0, s>>>(x, idx32, inv_ptr, inv_pos, luts, gy,
                                                                                alpha, beta, gx, B, I, N, k, O);
        return dl_launch_status();
    }
    if (!saved || !ws) return DL_ERR_NULL;
    if (ws_bytes < dl_dwn_bwd_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    const uint8_t *addrT = (const uint8_t *)saved;
    float *D = (float *)ws;
    float *gyT = (float *)((char *)ws + dwn_table_bytes(N, k, O));
    const int BT = dwn_bt(B), BP = BT * 64;
    // enough blocks to fill 256 CUs several times over, few enough that the per-block
    // histogram flush (one atomic per bin) stays small next to the streaming work
    const int col_tiles = dl_ceil_div(NO, DWN_TC);
    int chunks = dl_ceil_div(1024, col_tiles);
    if (chunks > BT) chunks = BT;
    const int tpc = dl_ceil_div(BT, chunks);
    chunks = dl_ceil_div(BT, tpc);
    if (gx) {
        DL_TIMED("dwn_efd_table", s, (dwn_efd_table<<<dl_ceil_div(NO * k * (L / 2), 256), 256, 0, s>>>(luts, D, (int)NO, k, alpha, beta)));
        DL_TIMED("dwn_bwd_transpose_hist", s, (dwn_bwd_transpose_hist<true><<<dim3(col_tiles, chunks), 256, 0, s>>>(
                                                  gy, addrT, gyT, gluts, B, (int)NO, O, L, BP, BT, tpc)));
        switch (k) {
            case 1: dwn_launch_gx<1>(gyT, addrT, D, inv_ptr, inv_pos, gx, B, I, O, s); break;
            case 2: dwn_launch_gx<2>(gyT, addrT, D, inv_ptr, inv_pos, gx, B, I, O, s); break;
            case 3: dwn_launch_gx<3>(gyT, addrT, D, inv_ptr, inv_pos, gx, B, I, O, s); break;
            case 4: dwn_launch_gx<4>(gyT, addrT, D, inv_ptr, inv_pos, gx, B, I, O, s); break;
            case 5: dwn_launch_gx<5>(gyT, addrT, D, inv_ptr, inv_pos, gx, B, I, O, s); break;
            default: dwn_launch_gx<6>(gyT, addrT, D, inv_ptr, inv_pos, gx, B, I, O, s); break;
        }
    } else {
        DL_TIMED("dwn_bwd_transpose_hist", s, (dwn_bwd_transpose_hist<false><<<dim3(col_tiles, chunks), 256, 0, s>>>(
                                                  gy, addrT, gyT, gluts, B, (int)NO, O, L, BP, BT, tpc)));
    }
    return dl_launch_status();
}

extern "C" int dl_dwn_layer_eval(const float *x, const int32_t *idx32, const float *luts, float *y, int B, int I, int N,
                                 int k, int O, void *stream) {
    if (!x || !idx32 || !luts || !y) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    dwn_eval_fwd<<<dl_ceil_div((long long)B * N * O, 256), 256, 0, (hipStream_t)stream>>>(x, idx32, luts, y, B, I, N, k, O);
    return dl_launch_status();
}
