// Adam update of the layers' parameter banks: one launch for all banks of a model.
//
// The tables of a layer live in one contiguous [N, O, 2^k] tensor; a training step on the deep stack updates four of
// them (7.7 MB of parameters).  torch's fused Adam takes ~46 us for that on an MI355X; this is the same arithmetic as
// torch.optim.Adam (no amsgrad) as one streaming kernel over up to DL_ADAM_MAX_TENSORS tensors, float4 wide.
#include "dl_common.h"

struct AdamTensors {
    float *p[DL_ADAM_MAX_TENSORS];
    const float *g[DL_ADAM_MAX_TENSORS];
    float *m[DL_ADAM_MAX_TENSORS];
    float *v[DL_ADAM_MAX_TENSORS];
    long long first_block[DL_ADAM_MAX_TENSORS + 1];  // blocks [first_block[t], first_block[t + 1]) work on tensor t
    long long n[DL_ADAM_MAX_TENSORS];
    int count;
};

#define ADAM_PER_BLOCK 2048  // elements per block: 256 threads x 2 float4

__device__ __forceinline__ void adam_one(float &p, float g, float &m, float &v, float beta1, float beta2, float step_size,
                                         float inv_bc2_sqrt, float eps, float weight_decay, int maximize) {
    if (maximize) g = -g;
    if (weight_decay != 0.0f) g += weight_decay * p;
    m = m + (1.0f - beta1) * (g - m);                  // exp_avg.lerp_(grad, 1 - beta1)
    v = beta2 * v + (1.0f - beta2) * g * g;            // exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)
    const float denom = sqrtf(v) * inv_bc2_sqrt + eps; // (exp_avg_sq.sqrt() / bias_correction2_sqrt).add_(eps)
    p = p - step_size * (m / denom);                   // param.addcdiv_(exp_avg, denom, value=-step_size)
}

__global__ __launch_bounds__(256) void adam_step_kernel(AdamTensors T, float beta1, float beta2, float step_size,
                                                         float inv_bc2_sqrt, float eps, float weight_decay, int maximize) {
    int t = 0;
    while (t + 1 < T.count && (long long)blockIdx.x >= T.first_block[t + 1]) ++t;
    const long long base = ((long long)blockIdx.x - T.first_block[t]) * ADAM_PER_BLOCK;
    float *__restrict__ p = T.p[t];
    const float *__restrict__ g = T.g[t];
    float *__restrict__ m = T.m[t];
    float *__restrict__ v = T.v[t];
    const long long n = T.n[t];
    const bool vec = ((((uintptr_t)p) | ((uintptr_t)g) | ((uintptr_t)m) | ((uintptr_t)v)) & 15) == 0;
#pragma unroll
    for (int u = 0; u < ADAM_PER_BLOCK / 1024; ++u) {
        const long long e = base + (long long)u * 1024 + threadIdx.x * 4;
        if (e >= n) return;
        if (vec && e + 4 <= n) {
            float4 pp = *reinterpret_cast<float4 *>(p + e), mm = *reinterpret_cast<float4 *>(m + e),
                   vv = *reinterpret_cast<float4 *>(v + e);
            const float4 gg = *reinterpret_cast<const float4 *>(g + e);
            adam_one(pp.x, gg.x, mm.x, vv.x, beta1, beta2, step_size, inv_bc2_sqrt, eps, weight_decay, maximize);
            adam_one(pp.y, gg.y, mm.y, vv.y, beta1, beta2, step_size, inv_bc2_sqrt, eps, weight_decay, maximize);
            adam_one(pp.z, gg.z, mm.z, vv.z, beta1, beta2, step_size, inv_bc2_sqrt, eps, weight_decay, maximize);
            adam_one(pp.w, gg.w, mm.w, vv.w, beta1, beta2, step_size, inv_bc2_sqrt, eps, weight_decay, maximize);
            *reinterpret_cast<float4 *>(p + e) = pp;
            *reinterpret_cast<float4 *>(m + e) = mm;
            *reinterpret_cast<float4 *>(v + e) = vv;
        } else {
            for (int q = 0; q < 4 && e + q < n; ++q)
                adam_one(p[e + q], g[e + q], m[e + q], v[e + q], beta1, beta2, step_size, inv_bc2_sqrt, eps, weight_decay, maximize);
        }
    }
}

extern "C" int dl_adam_step(void *const *params, const void *const *grads, void *const *exp_avg, void *const *exp_avg_sq,
                            const long long *numel, int count, float lr, float beta1, float beta2, float eps,
                            float weight_decay, int step, int maximize, void *stream) {
    if (!params || !grads || !exp_avg || !exp_avg_sq || !numel) return DL_ERR_NULL;
    if (count <= 0 || step <= 0) return DL_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    // bias corrections in double on the host, as torch.optim.Adam computes them in Python floats
    const double bc1 = 1.0 - pow((double)beta1, (double)step), bc2 = 1.0 - pow((double)beta2, (double)step);
    const float step_size = (float)((double)lr / bc1), inv_bc2_sqrt = (float)(1.0 / sqrt(bc2));
    for (int t0 = 0; t0 < count; t0 += DL_ADAM_MAX_TENSORS) {
        AdamTensors T;
        T.count = count - t0 < DL_ADAM_MAX_TENSORS ? count - t0 : DL_ADAM_MAX_TENSORS;
        long long blocks = 0;
        for (int t = 0; t < T.count; ++t) {
            if (!params[t0 + t] || !grads[t0 + t] || !exp_avg[t0 + t] || !exp_avg_sq[t0 + t]) return DL_ERR_NULL;
            if (numel[t0 + t] <= 0) return DL_ERR_SHAPE;
            T.p[t] = (float *)params[t0 + t];
            T.g[t] = (const float *)grads[t0 + t];
            T.m[t] = (float *)exp_avg[t0 + t];
            T.v[t] = (float *)exp_avg_sq[t0 + t];
            T.n[t] = numel[t0 + t];
            T.first_block[t] = blocks;
            blocks += (numel[t0 + t] + ADAM_PER_BLOCK - 1) / ADAM_PER_BLOCK;
        }
        T.first_block[T.count] = blocks;
        if (blocks > 0x7fffffffLL) return DL_ERR_UNSUPPORTED;
        DL_TIMED("adam_step", s, (adam_step_kernel<<<(int)blocks, 256, 0, s>>>(T, beta1, beta2, step_size, inv_bc2_sqrt, eps,
                                                                            weight_decay, maximize)));
    }
    return dl_launch_status();
}

// ---------------------------------------------------------------------------------
// Gradient stabilisation of the layers (base_layer.py:266-339 of the reference): out = (g - mean) * sqrt(target /
// (mean((g - mean)^2) + eps)), the mean taken over the whole tensor ("layerwise") or per row ("batchwise"), the mean
// subtracted only when asked.  Sums are kept in double and added in a fixed order.
//   per row:   one block per row, one launch.
//   layerwise: grad_stab_partials leaves (sum, sum of squares) per block; grad_stab_apply lets every block add the
//              partials in block order and rescale its own piece - two launches instead of torch's seven kernels.
#define GS_THREADS 256
#define GS_PER_BLOCK 4096  // elements per block of the layerwise form

__device__ __forceinline__ void gs_block_sums(double &s, double &q, double *red) {
    // sum over the block in a fixed order: lanes by butterfly, wavefronts in order
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        s += __shfl_xor(s, o);
        q += __shfl_xor(q, o);
    }
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { red[2 * wave] = s; red[2 * wave + 1] = q; }
    __syncthreads();
    s = 0.0; q = 0.0;
    for (int w = 0; w < GS_THREADS / 64; ++w) { s += red[2 * w]; q += red[2 * w + 1]; }
    __syncthreads();
}

__global__ __launch_bounds__(GS_THREADS) void grad_stab_rows(const float *__restrict__ g, float *__restrict__ out, long long cols,
                                                              float target, int subtract_mean, float eps) {
    __shared__ double red[2 * GS_THREADS / 64];
    const float *row = g + (size_t)blockIdx.x * cols;
    float *dst = out + (size_t)blockIdx.x * cols;
    double s = 0.0, q = 0.0;
    for (long long c = threadIdx.x; c < cols; c += GS_THREADS) { const double v = row[c]; s += v; q += v * v; }
    gs_block_sums(s, q, red);
    const double mean = subtract_mean ? s / (double)cols : 0.0;
    const double var = q / (double)cols - (subtract_mean ? mean * mean : 0.0);  // mean((g - mean)^2)
    const float scale = (float)sqrt((double)target / ((var > 0.0 ? var : 0.0) + (double)eps)), m = (float)mean;
    for (long long c = threadIdx.x; c < cols; c += GS_THREADS) dst[c] = (row[c] - m) * scale;
}

__global__ __launch_bounds__(GS_THREADS) void grad_stab_partials(const float *__restrict__ g, double *__restrict__ part, long long n) {
    __shared__ double red[2 * GS_THREADS / 64];
    const long long base = (long long)blockIdx.x * GS_PER_BLOCK;
    double s = 0.0, q = 0.0;
    for (int u = threadIdx.x; u < GS_PER_BLOCK; u += GS_THREADS)
        if (base + u < n) { const double v = g[base + u]; s += v; q += v * v; }
    gs_block_sums(s, q, red);
    if (threadIdx.x == 0) { part[2 * (size_t)blockIdx.x] = s; part[2 * (size_t)blockIdx.x + 1] = q; }
}

__global__ __launch_bounds__(GS_THREADS) void grad_stab_apply(const float *__restrict__ g, float *__restrict__ out,
                                                               const double *__restrict__ part, long long n, int blocks,
                                                               float target, int subtract_mean, float eps) {
    __shared__ double red[2 * GS_THREADS / 64];
    double s = 0.0, q = 0.0;
    for (int b = threadIdx.x; b < blocks; b += GS_THREADS) { s += part[2 * (size_t)b]; q += part[2 * (size_t)b + 1]; }
    gs_block_sums(s, q, red);  // every block adds the partials in the same order: one value for the whole tensor
    const double mean = subtract_mean ? s / (double)n : 0.0;
    const double var = q / (double)n - (subtract_mean ? mean * mean : 0.0);
    const float scale = (float)sqrt((double)target / ((var > 0.0 ? var : 0.0) + (double)eps)), m = (float)mean;
    const long long base = (long long)blockIdx.x * GS_PER_BLOCK;
    for (int u = threadIdx.x; u < GS_PER_BLOCK; u += GS_THREADS)
        if (base + u < n) out[base + u] = (g[base + u] - m) * scale;
}

extern "C" size_t dl_grad_stabilize_workspace_bytes(long long rows, long long cols, int per_row) {
    if (rows <= 0 || cols <= 0 || per_row) return 256;
    return dl_align256((size_t)((rows * cols + GS_PER_BLOCK - 1) / GS_PER_BLOCK) * 2 * sizeof(double));
}

extern "C" int dl_grad_stabilize(const float *g, float *out, long long rows, long long cols, int per_row, float target_std,
                                 int subtract_mean, float eps, void *ws, size_t ws_bytes, void *stream) {
    if (!g || !out) return DL_ERR_NULL;
    if (rows <= 0 || cols <= 0) return DL_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    if (per_row) {
        if (rows > 0x7fffffffLL) return DL_ERR_UNSUPPORTED;
        DL_TIMED("grad_stab_rows", s, (grad_stab_rows<<<(int)rows, GS_THREADS, 0, s>>>(g, out, cols, target_std, subtract_mean, eps)));
        return dl_launch_status();
    }
    const long long n = rows * cols, blocks = (n + GS_PER_BLOCK - 1) / GS_PER_BLOCK;
    if (blocks > 0x7fffffffLL) return DL_ERR_UNSUPPORTED;
    if (!ws) return DL_ERR_NULL;
    if (ws_bytes < dl_grad_stabilize_workspace_bytes(rows, cols, 0)) return DL_ERR_WORKSPACE;
    DL_TIMED("grad_stab_partials", s, (grad_stab_partials<<<(int)blocks, GS_THREADS, 0, s>>>(g, (double *)ws, n)));
    DL_TIMED("grad_stab_apply", s, (grad_stab_apply<<<(int)blocks, GS_THREADS, 0, s>>>(g, out, (const double *)ws, n, (int)blocks,
                                                                                    target_std, subtract_mean, eps)));
    return dl_launch_status();
}
