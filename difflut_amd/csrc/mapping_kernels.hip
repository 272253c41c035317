// RandomLayer index gather and its adjoint, LearnableLayer hard selection, thermometer
// encoding and GroupSum: the streaming pieces either side of the node kernels.
#include "dl_common.h"
#include <algorithm>

// m[b,n,j] = x[b, idx[n,j]]: one block per (row, slab of the flattened [N*k] axis).  The row of
// x is read through the cache (random but inside one 4*I-byte row), writes are coalesced.
template <typename index_t>
__global__ __launch_bounds__(256) void gather_fwd_kernel(const float *__restrict__ x, const index_t *__restrict__ idx,
                                                          float *__restrict__ m, int B, int I, long long NK) {
    for (int b = blockIdx.y; b < B; b += gridDim.y) {  // grid.y is capped at 65535 rows
        const float *xrow = x + (size_t)b * I;
        float *out = m + (size_t)b * NK;
        for (long long p = (long long)blockIdx.x * 1024 + threadIdx.x; p < min(NK, ((long long)blockIdx.x + 1) * 1024);
             p += 256)
            out[p] = xrow[idx[p]];
    }
}

// gx[b,i] = sum over CSR entries of input i of gm[b, pos]; fixed order, no atomics.
__global__ __launch_bounds__(256) void gather_bwd_kernel(const float *__restrict__ gm, const int *__restrict__ inv_ptr,
                                                          const int *__restrict__ inv_pos, float *__restrict__ gx,
                                                          int B, int I, long long NK) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= I) return;
    for (int b = blockIdx.y; b < B; b += gridDim.y) {  // grid.y is capped at 65535 rows
        const float *row = gm + (size_t)b * NK;
        float acc = 0.0f;
        for (int e = inv_ptr[i]; e < inv_ptr[i + 1]; ++e) acc += row[inv_pos[e]];
        gx[(size_t)b * I + i] = acc;
    }
}

// The same two operations with the row that is read at random staged in the LDS: a wavefront's 64 random 4-byte reads
// of a row in memory cost the texture addresser 64 cycles (the kernels above reach 1.25 and 0.95 TB/s at 4096 x 16384
// -> 8192 x 6), from the LDS a few.  Blocks of 1024 threads walk the rows; global reads and writes are all coalesced.
// fwd: the row of x (I floats, at most DL_GATHER_LDS_FLOATS) is staged, m[b][p] = row[idx[p]].
#define DL_GATHER_LDS_FLOATS 32768  // 128 KB of the CU's 160
#define DL_GATHER_BWD_FLOATS 24576  // pieces of the adjoint's rows: 96 KB, six 16-byte loads per thread
template <typename index_t>
__global__ __launch_bounds__(1024) void gather_fwd_lds(const float *__restrict__ x, const index_t *__restrict__ idx,
                                                        float *__restrict__ m, int B, int I, long long NK) {
    extern __shared__ float dl_gather_row[];
    float *row = dl_gather_row;
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
        float *out = m + (size_t)b * NK;
        long long p = threadIdx.x;
        for (; p + 3 * 1024 < NK; p += 4 * 1024) {  // four in flight
            const int i0 = idx[p], i1 = idx[p + 1024], i2 = idx[p + 2048], i3 = idx[p + 3072];
            const float v0 = row[i0], v1 = row[i1], v2 = row[i2], v3 = row[i3];
            __builtin_nontemporal_store(v0, out + p);
            __builtin_nontemporal_store(v1, out + p + 1024);
            __builtin_nontemporal_store(v2, out + p + 2048);
            __builtin_nontemporal_store(v3, out + p + 3072);
        }
        for (; p < NK; p += 1024) __builtin_nontemporal_store(row[idx[p]], out + p);
    }
}
// bwd: the row of gm is staged piece by piece (CH floats); a thread owns inputs tid, tid + T, ... and walks each
// one's CSR list, whose positions ascend: the additions happen in list order, as in gather_bwd_kernel.  NK < 2^31 - 1
// (positions are int32).
template <int QI>
__global__ __launch_bounds__(1024) void gather_bwd_lds(const float *__restrict__ gm, const int *__restrict__ inv_ptr,
                                                        const int *__restrict__ inv_pos, float *__restrict__ gx, int B,
                                                        int I, long long NK, int CH, int i_begin, int i_end) {
    extern __shared__ float dl_gather_row[];
    float *piece = dl_gather_row;
    constexpr int NONE = 0x7fffffff;
    const bool vec = (NK & 3) == 0 && (CH & 3) == 0 && (((uintptr_t)gm) & 15) == 0;
    // positions through a buffer descriptor: one register of offset per load in flight instead of a 64-bit address
    const __amdgpu_buffer_rsrc_t rs_pos = __builtin_amdgcn_make_buffer_rsrc((void *)inv_pos, 0, (int)(NK * 4), DL_BUFFER_WORD3);
    auto position = [&](int e) { return (int)__builtin_amdgcn_raw_buffer_load_b32(rs_pos, e * 4, 0, 0); };
    for (int b = blockIdx.x; b < B; b += gridDim.x) {
        const float *grow = gm + (size_t)b * NK;
        float acc[QI];
        int cur[QI], e1[QI], nxt[QI];  // nxt: the position of the entry at the cursor (NONE: list done)
#pragma unroll
        for (int q = 0; q < QI; ++q) {  // (the list bounds are read again for every row: registers are short at QI = 16)
            const int i = i_begin + threadIdx.x + 1024 * q;
            acc[q] = 0.0f;
            cur[q] = i < i_end ? inv_ptr[i] : 0;
            e1[q] = i < i_end ? inv_ptr[i + 1] : 0;
            nxt[q] = cur[q] < e1[q] ? position(cur[q]) : NONE;
        }
        for (long long base = 0; base < NK; base += CH) {
            const int len = (int)min((long long)CH, NK - base);
            __syncthreads();  // the readers of the piece before are done
            if (vec) {
                for (int i = threadIdx.x * 4; i < len; i += 4096)
                    *reinterpret_cast<float4 *>(piece + i) = *reinterpret_cast<const float4 *>(grow + base + i);
            } else {
                for (int i = threadIdx.x; i < len; i += 1024) piece[i] = grow[base + i];
            }
            __syncthreads();
            // one entry per input and sweep: the loads of the next positions of all my inputs are in flight together
            const long long end = base + len;
            bool moved = true;
            while (moved) {
                moved = false;
#pragma unroll
                for (int q = 0; q < QI; ++q) {
                    if (nxt[q] < end) {
                        if (nxt[q] >= base) acc[q] += piece[nxt[q] - base];  // (before the piece: not ascending as promised)
                        ++cur[q];
                        nxt[q] = cur[q] < e1[q] ? position(cur[q]) : NONE;
                        moved = true;
                    }
                }
            }
        }
#pragma unroll
        for (int q = 0; q < QI; ++q) {
            const int i = i_begin + threadIdx.x + 1024 * q;
            if (i < i_end) __builtin_nontemporal_store(acc[q], gx + (size_t)b * I + i);
        }
    }
}

// The adjoint for short lists: the first FMAX positions of every list of a thread's inputs stay in registers over all
// the block's rows (QI x FMAX of them), so a row costs no index reads at all; used when no list is longer (checked by
// the host through the average: N k <= FMAX I, and by every thread for its own lists - a longer one is finished through
// its cursor, in order).
template <int QI, int FMAX>
__global__ __launch_bounds__(1024) void gather_bwd_lds_short(const float *__restrict__ gm, const int *__restrict__ inv_ptr,
                                                              const int *__restrict__ inv_pos, float *__restrict__ gx, int B,
                                                              int I, long long NK, int CH, int i_begin, int i_end) {
    extern __shared__ float dl_gather_row[];
    float *piece = dl_gather_row;
    constexpr int NONE = 0x7fffffff;
    int pos[QI][FMAX];
    bool longer = false;  // one of my lists has more than FMAX entries
#pragma unroll
    for (int q = 0; q < QI; ++q) {
        const int i = i_begin + threadIdx.x + 1024 * q;
        const int e0 = i < i_end ? inv_ptr[i] : 0, e1 = i < i_end ? inv_ptr[i + 1] : 0;
#pragma unroll
        for (int f = 0; f < FMAX; ++f) pos[q][f] = e0 + f < e1 ? inv_pos[e0 + f] : NONE;
        longer = longer || e1 - e0 > FMAX;
    }
    const bool vec = (NK & 3) == 0 && (CH & 3) == 0 && (((uintptr_t)gm) & 15) == 0;
    for (int b = blockIdx.x; b < B; b += gridDim.x) {
        const float *grow = gm + (size_t)b * NK;
        float acc[QI];
#pragma unroll
        for (int q = 0; q < QI; ++q) acc[q] = 0.0f;
        for (long long base = 0; base < NK; base += CH) {
            const int len = (int)min((long long)CH, NK - base);
            __syncthreads();  // the readers of the piece before are done
            if (vec) {
                for (int i = threadIdx.x * 4; i < len; i += 4096)
                    *reinterpret_cast<float4 *>(piece + i) = *reinterpret_cast<const float4 *>(grow + base + i);
            } else {
                for (int i = threadIdx.x; i < len; i += 1024) piece[i] = grow[base + i];
            }
            __syncthreads();
            const long long end = base + len;
#pragma unroll
            for (int q = 0; q < QI; ++q) {
#pragma unroll
                for (int f = 0; f < FMAX; ++f)
                    if (pos[q][f] >= base && pos[q][f] < end) acc[q] += piece[pos[q][f] - base];
            }
            if (longer) {  // the rest of a long list, in order, after its first FMAX entries (positions ascend)
                for (int q = 0; q < QI; ++q) {
                    const int i = i_begin + threadIdx.x + 1024 * q;
                    if (i >= i_end) break;
                    const int e1 = inv_ptr[i + 1];
                    for (int e = inv_ptr[i] + FMAX; e < e1; ++e) {
                        const long long p = inv_pos[e];
                        if (p >= end) break;
                        if (p >= base) acc[q] += piece[p - base];
                    }
                }
            }
        }
#pragma unroll
        for (int q = 0; q < QI; ++q) {
            const int i = i_begin + threadIdx.x + 1024 * q;
            if (i < i_end) __builtin_nontemporal_store(acc[q], gx + (size_t)b * I + i);
        }
    }
}

// One wavefront per row of W; lowest index wins ties.
__global__ __launch_bounds__(256) void row_argmax_kernel(const float *__restrict__ W, int *__restrict__ sel, int M, int I) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= M) return;
    const float *w = W + (size_t)row * I;
    float best = -INFINITY;
    int arg = 0x7fffffff;
    auto take = [&](float v, int i) {
        if (v > best || (v == best && i < arg) || arg == 0x7fffffff) { best = v; arg = i; }
    };
    if ((I & 3) == 0 && (((uintptr_t)W) & 15) == 0) {  // 16 bytes per lane and load, four loads in flight
        int i = lane * 4;
        for (; i + 768 < I; i += 1024) {
            float4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const float4 *>(w + i + 256 * u);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                take(v[u].x, i + 256 * u); take(v[u].y, i + 256 * u + 1); take(v[u].z, i + 256 * u + 2); take(v[u].w, i + 256 * u + 3);
            }
        }
        for (; i < I; i += 256) {
            const float4 v = *reinterpret_cast<const float4 *>(w + i);
            take(v.x, i); take(v.y, i + 1); take(v.z, i + 2); take(v.w, i + 3);
        }
    } else {
        for (int i = lane; i < I; i += 64) take(w[i], i);
    }
    for (int off = 32; off > 0; off >>= 1) {
        const float ob = __shfl_xor(best, off);
        const int oa = __shfl_xor(arg, off);
        if (oa != 0x7fffffff && (arg == 0x7fffffff || ob > best || (ob == best && oa < arg))) { best = ob; arg = oa; }
    }
    if (lane == 0) sel[row] = arg;
}

__global__ __launch_bounds__(256) void thermometer_kernel(const float *__restrict__ x, const float *__restrict__ thr,
                                                           float *__restrict__ bits, long long total, int FB, int nbits) {
    // four consecutive outputs per thread, one 16-byte store (FB a multiple of four: they stay within a row)
    const long long g4 = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (g4 >= total) return;
    if ((FB & 3) == 0 && (((uintptr_t)bits) & 15) == 0) {
        const long long b = g4 / FB;
        const int fb = (int)(g4 % FB);
        const float *xrow = x + b * (FB / nbits);
        float4 out;
        out.x = xrow[fb / nbits] > thr[fb] ? 1.0f : 0.0f;  // strict compare
        out.y = xrow[(fb + 1) / nbits] > thr[fb + 1] ? 1.0f : 0.0f;
        out.z = xrow[(fb + 2) / nbits] > thr[fb + 2] ? 1.0f : 0.0f;
        out.w = xrow[(fb + 3) / nbits] > thr[fb + 3] ? 1.0f : 0.0f;
        *reinterpret_cast<float4 *>(bits + g4) = out;
        return;
    }
    for (long long gid = g4; gid < min(total, g4 + 4); ++gid) {
        const long long b = gid / FB;
        const int fb = (int)(gid % FB);
        bits[gid] = x[b * (FB / nbits) + fb / nbits] > thr[fb] ? 1.0f : 0.0f;
    }
}

// Thermometer bits as bit-planes for a following DWN layer: word (t, f*nbits + j) holds, in bit r,
// (x[64t + r][f] > thr[f][j]).  Block = (64 features, batch tile t): the x tile is read row-wise
// (coalesced) into LDS; then every thread builds whole output words, one (feature, threshold) pair at a
// time, by walking the 64 rows of its feature in LDS (lanes of one feature read the same word: a
// broadcast; different features sit in different banks).  Consecutive threads hold consecutive words, so
// the stores are contiguous.  Rows past B read as "not greater".
__global__ __launch_bounds__(256) void thermometer_planes_kernel(const float *__restrict__ x, const float *__restrict__ thr,
                                                                  unsigned long long *__restrict__ planes, int B, int F,
                                                                  int nbits) {
    __shared__ float tile[64][65];  // [feature][row]
    const int t = blockIdx.y, f0 = blockIdx.x * 64;
    for (int e = threadIdx.x; e < 4096; e += 256) {
        const int r = e >> 6, c = e & 63;
        const int b = t * 64 + r;
        tile[c][r] = (b < B && f0 + c < F) ? x[(size_t)b * F + f0 + c] : -INFINITY;
    }
    __syncthreads();
    const int words = min(64, F - f0) * nbits;
    const float *th = thr + (size_t)f0 * nbits;
    unsigned long long *out = planes + ((size_t)t * F + f0) * nbits;
    for (int w = threadIdx.x; w < words; w += 256) {
        const float *row = tile[w / nbits];
        const float limit = th[w];
        unsigned lo = 0u, hi = 0u;
#pragma unroll
        for (int r = 0; r < 32; ++r) {
            lo |= (row[r] > limit ? 1u : 0u) << r;  // strict compare, as the encoder
            hi |= (row[r + 32] > limit ? 1u : 0u) << r;
        }
        out[w] = ((unsigned long long)hi << 32) | lo;
    }
}

// One wavefront per (row, group): sum a contiguous run of group_size features.
__global__ __launch_bounds__(256) void group_sum_fwd_kernel(const float *__restrict__ x, float *__restrict__ y, int B,
                                                             int F, int groups, int gsize, float inv_tau) {
    const long long w = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (w >= (long long)B * groups) return;
    const int b = (int)(w / groups), g = (int)(w % groups);
    const float *row = x + (size_t)b * F;
    float acc = 0.0f;
    for (int f = g * gsize + lane; f < min(F, (g + 1) * gsize); f += 64) acc += row[f];
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    if (lane == 0) y[w] = acc * inv_tau;
}

// thread = four consecutive features of one row
__global__ __launch_bounds__(256) void group_sum_bwd_kernel(const float *__restrict__ gy, float *__restrict__ gx,
                                                             long long total, int F, int groups, int gsize,
                                                             float inv_tau) {
    const long long e = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (e >= total) return;
    if ((F & 3) == 0 && (((uintptr_t)gx) & 15) == 0) {
        const long long b = e / F;
        const int f = (int)(e - b * F);
        const float *src = gy + b * groups;
        typedef float f4 __attribute__((ext_vector_type(4)));
        const f4 v = {src[(f + 0) / gsize] * inv_tau, src[(f + 1) / gsize] * inv_tau, src[(f + 2) / gsize] * inv_tau,
                      src[(f + 3) / gsize] * inv_tau};
        __builtin_nontemporal_store(v, reinterpret_cast<f4 *>(gx + e));
        return;
    }
    for (long long i = e; i < min(total, e + 4); ++i) {
        const long long b = i / F;
        gx[i] = gy[b * groups + (int)(i - b * F) / gsize] * inv_tau;
    }
}

// ---------------------------------------------------------------------------------
// Cross-entropy with mean reduction over the batch on [B, C] logits (the loss that follows GroupSum in the
// training configurations): one thread per row computes the row's loss (logsumexp - logit[label]) and the
// gradient of the MEAN loss, (softmax - onehot) / B; a single block then adds the B row losses in a fixed order.
__global__ __launch_bounds__(256) void cross_entropy_rows(const float *__restrict__ logits, const long long *__restrict__ labels,
                                                           float *__restrict__ row_loss, float *__restrict__ glogits, int B,
                                                           int C) {
    const int b = blockIdx.x * 256 + threadIdx.x;
    if (b >= B) return;
    const float *z = logits + (size_t)b * C;
    float m = -INFINITY;
    for (int c = 0; c < C; ++c) m = fmaxf(m, z[c]);
    float sum = 0.0f;
    for (int c = 0; c < C; ++c) sum += expf(z[c] - m);
    const long long label = labels[b];
    const bool ok = label >= 0 && label < C;
    row_loss[b] = ok ? (logf(sum) + m) - z[label] : 0.0f;  // rows with a label outside [0, C) are left out
    const float inv = 1.0f / sum, invB = 1.0f / (float)B;
    float *g = glogits + (size_t)b * C;
    for (int c = 0; c < C; ++c) g[c] = ok ? (expf(z[c] - m) * inv - (c == label ? 1.0f : 0.0f)) * invB : 0.0f;
}
__global__ __launch_bounds__(256) void cross_entropy_mean(const float *__restrict__ row_loss, float *__restrict__ loss, int B) {
    __shared__ float part[256];
    float acc = 0.0f;
    for (int b = threadIdx.x; b < B; b += 256) acc += row_loss[b];
    part[threadIdx.x] = acc;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) part[threadIdx.x] += part[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) *loss = part[0] / (float)B;
}

// ---------------------------------------------------------------------------------
// more than 64 KB of dynamic LDS has to be asked for, once per kernel (any thread may be the first)
static int dl_gather_lds_attr(const void *fn, size_t bytes) {
    if (bytes <= 64 * 1024) return 0;
    return (int)hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

extern "C" int dl_gather_fwd(const float *x, const void *idx, int idx_bits, float *m, int B, int I, int N, int k,
                             void *stream) {
    if (!x || !idx || !m) return DL_ERR_NULL;
    if (B <= 0 || I <= 0 || N <= 0 || k <= 0) return DL_ERR_SHAPE;
    if (idx_bits != 16 && idx_bits != 32) return DL_ERR_UNSUPPORTED;
    const long long NK = (long long)N * k;
    if (I <= DL_GATHER_LDS_FLOATS && NK >= 4096) {  // the row of x through the LDS
        const size_t lds = (size_t)I * sizeof(float);
        const int per_cu = (int)std::max<size_t>(1, std::min<size_t>(2, (160 * 1024) / (lds + 1024)));
        const int blocks = std::min(B, 256 * per_cu);
        hipStream_t s = (hipStream_t)stream;
        if (idx_bits == 16) {
            if (int rc = dl_gather_lds_attr(reinterpret_cast<const void *>(&gather_fwd_lds<int16_t>), lds)) return rc;
            DL_TIMED("gather_fwd", s, (gather_fwd_lds<int16_t><<<blocks, 1024, lds, s>>>(x, (const int16_t *)idx, m, B, I, NK)));
        } else {
            if (int rc = dl_gather_lds_attr(reinterpret_cast<const void *>(&gather_fwd_lds<int32_t>), lds)) return rc;
            DL_TIMED("gather_fwd", s, (gather_fwd_lds<int32_t><<<blocks, 1024, lds, s>>>(x, (const int32_t *)idx, m, B, I, NK)));
        }
        return dl_launch_status();
    }
    dim3 grid(dl_ceil_div(NK, 1024), B < 65535 ? B : 65535);
    if (idx_bits == 16)
        gather_fwd_kernel<int16_t><<<grid, 256, 0, (hipStream_t)stream>>>(x, (const int16_t *)idx, m, B, I, NK);
    else
        gather_fwd_kernel<int32_t><<<grid, 256, 0, (hipStream_t)stream>>>(x, (const int32_t *)idx, m, B, I, NK);
    return dl_launch_status();
}

extern "C" int dl_gather_bwd(const float *gm, const int32_t *inv_ptr, const int32_t *inv_pos, float *gx, int B, int I,
                             int N, int k, void *stream) {
    if (!gm || !inv_ptr || !inv_pos || !gx) return DL_ERR_NULL;
    if (B <= 0 || I <= 0 || N <= 0 || k <= 0) return DL_ERR_SHAPE;
    const long long NK = (long long)N * k;
    if (NK >= 4096 && NK < (1LL << 29)) {  // the row of gm through the LDS, piece by piece (byte offsets of positions: 32-bit)
        const long long pieces = dl_ceil_div(NK, (long long)DL_GATHER_BWD_FLOATS);
        const int CH = (int)((dl_ceil_div(NK, pieces) + 3) / 4 * 4);
        const size_t lds = (size_t)CH * sizeof(float);
        const int per_cu = (int)std::max<size_t>(1, std::min<size_t>(2, (160 * 1024) / (lds + 1024)));
        const int blocks = std::min(B, 256 * per_cu);
        hipStream_t s = (hipStream_t)stream;
        // a thread has at most 16 inputs, so wider layers are taken 16384 inputs at a time (the row of gm is then staged
        // once per such window)
        for (int i0 = 0; i0 < I; i0 += 16384) {
            const int i1 = std::min(I, i0 + 16384), In = i1 - i0;
#define DL_GBWD(QI_)                                                                                                   \
    do {                                                                                                               \
        if (int rc = dl_gather_lds_attr(reinterpret_cast<const void *>(&gather_bwd_lds<QI_>), lds)) return rc;         \
        DL_TIMED("gather_bwd", s,                                                                                      \
                 (gather_bwd_lds<QI_><<<blocks, 1024, lds, s>>>(gm, inv_ptr, inv_pos, gx, B, I, NK, CH, i0, i1)));      \
    } while (0)
            if (In > 4096 && NK <= 3LL * I) {  // short lists: their positions in registers
                if (int rc = dl_gather_lds_attr(reinterpret_cast<const void *>(&gather_bwd_lds_short<16, 3>), lds)) return rc;
                DL_TIMED("gather_bwd", s, (gather_bwd_lds_short<16, 3><<<blocks, 1024, lds, s>>>(gm, inv_ptr, inv_pos, gx, B, I, NK,
                                                                                              CH, i0, i1)));
            } else if (In <= 1024) DL_GBWD(1);
            else if (In <= 4096) DL_GBWD(4);
            else DL_GBWD(16);
#undef DL_GBWD
        }
        return dl_launch_status();
    }
    gather_bwd_kernel<<<dim3(dl_ceil_div(I, 256), B < 65535 ? B : 65535), 256, 0, (hipStream_t)stream>>>(
        gm, inv_ptr, inv_pos, gx, B, I, (long long)N * k);
    return dl_launch_status();
}

extern "C" int dl_row_argmax(const float *W, int32_t *sel, int M, int I, void *stream) {
    if (!W || !sel) return DL_ERR_NULL;
    if (M <= 0 || I <= 0) return DL_ERR_SHAPE;
    row_argmax_kernel<<<dl_ceil_div(M, 4), 256, 0, (hipStream_t)stream>>>(W, sel, M, I);
    return dl_launch_status();
}

extern "C" int dl_hard_select_fwd(const float *x, const int32_t *sel, float *m, int B, int I, int M, void *stream) {
    return dl_gather_fwd(x, sel, 32, m, B, I, M, 1, stream);
}

extern "C" int dl_hard_select_bwd(const float *gm, const int32_t *inv_ptr, const int32_t *inv_pos, float *gx, int B,
                                  int I, int M, void *stream) {
    return dl_gather_bwd(gm, inv_ptr, inv_pos, gx, B, I, M, 1, stream);
}

extern "C" int dl_thermometer_encode(const float *x, const float *thr, float *bits, int B, int F, int nbits,
                                     void *stream) {
    if (!x || !thr || !bits) return DL_ERR_NULL;
    if (B <= 0 || F <= 0 || nbits <= 0) return DL_ERR_SHAPE;
    const long long total = (long long)B * F * nbits;
    thermometer_kernel<<<dl_ceil_div(total, 1024), 256, 0, (hipStream_t)stream>>>(x, thr, bits, total, F * nbits, nbits);
    return dl_launch_status();
}

extern "C" int dl_thermometer_planes(const float *x, const float *thr, void *planes, int B, int F, int nbits,
                                     void *stream) {
    if (!x || !thr || !planes) return DL_ERR_NULL;
    if (B <= 0 || F <= 0 || nbits <= 0) return DL_ERR_SHAPE;
    if (B > 4000000) return DL_ERR_UNSUPPORTED;  // batch tiles ride in grid.y (at most 65535 of them)
    hipStream_t s = (hipStream_t)stream;
    DL_TIMED("thermometer_planes", s,
             (thermometer_planes_kernel<<<dim3(dl_ceil_div(F, 64), dl_ceil_div(B, 64)), 256, 0, s>>>(
                 x, thr, (unsigned long long *)planes, B, F, nbits)));
    return dl_launch_status();
}

extern "C" size_t dl_cross_entropy_workspace_bytes(int B) { return B > 0 ? dl_align256((size_t)B * sizeof(float)) : 256; }
extern "C" int dl_cross_entropy(const float *logits, const long long *labels, float *loss, float *glogits, void *ws,
                                size_t ws_bytes, int B, int C, void *stream) {
    if (!logits || !labels || !loss || !glogits || !ws) return DL_ERR_NULL;
    if (B <= 0 || C <= 0) return DL_ERR_SHAPE;
    if (ws_bytes < dl_cross_entropy_workspace_bytes(B)) return DL_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    DL_TIMED("cross_entropy_rows", s,
             (cross_entropy_rows<<<dl_ceil_div(B, 256), 256, 0, s>>>(logits, labels, (float *)ws, glogits, B, C)));
    DL_TIMED("cross_entropy_mean", s, (cross_entropy_mean<<<1, 256, 0, s>>>((const float *)ws, loss, B)));
    return dl_launch_status();
}

extern "C" int dl_group_sum_fwd(const float *x, float *y, int B, int F, int groups, float tau, void *stream) {
    if (!x || !y) return DL_ERR_NULL;
    if (B <= 0 || F <= 0 || groups <= 0 || !(tau > 0.0f)) return DL_ERR_SHAPE;
    const int gsize = (F + groups - 1) / groups;  // features zero-padded up to groups * gsize
    DL_TIMED("group_sum_fwd", (hipStream_t)stream,
             (group_sum_fwd_kernel<<<dl_ceil_div((long long)B * groups, 4), 256, 0, (hipStream_t)stream>>>(
                 x, y, B, F, groups, gsize, 1.0f / tau)));
    return dl_launch_status();
}

extern "C" int dl_group_sum_bwd(const float *gy, float *gx, int B, int F, int groups, float tau, void *stream) {
    if (!gy || !gx) return DL_ERR_NULL;
    if (B <= 0 || F <= 0 || groups <= 0 || !(tau > 0.0f)) return DL_ERR_SHAPE;
    const int gsize = (F + groups - 1) / groups;
    const long long total = (long long)B * F;
    DL_TIMED("group_sum_bwd", (hipStream_t)stream,
             (group_sum_bwd_kernel<<<dl_ceil_div(total, 1024), 256, 0, (hipStream_t)stream>>>(gy, gx, total, F, groups, gsize,
                                                                                           1.0f / tau)));
    return dl_launch_status();
}

// ---------------------------------------------------------------------------------
// per-kernel timing
#define DL_PROF_MAX 64
static struct {
    int on, count, created;
    hipEvent_t ev[2 * DL_PROF_MAX];
    const char *name[DL_PROF_MAX];
} g_prof;

void dl_prof_begin(const char *kernel_name, hipStream_t s) {
    if (!g_prof.on || g_prof.count >= DL_PROF_MAX) return;
    while (g_prof.created < 2 * (g_prof.count + 1)) {
        if (hipEventCreate(&g_prof.ev[g_prof.created]) != hipSuccess) { g_prof.on = 0; return; }
        ++g_prof.created;
    }
    g_prof.name[g_prof.count] = kernel_name;
    (void)hipEventRecord(g_prof.ev[2 * g_prof.count], s);
}
void dl_prof_end(hipStream_t s) {
    if (!g_prof.on || g_prof.count >= DL_PROF_MAX) return;
    (void)hipEventRecord(g_prof.ev[2 * g_prof.count + 1], s);
    ++g_prof.count;
}

extern "C" int dl_profile_enable(int on) {
    g_prof.on = on ? 1 : 0;
    g_prof.count = 0;
    return DL_OK;
}

extern "C" int dl_profile_read(char *names, size_t names_bytes, float *ms, int max_entries) {
    int n = g_prof.count < max_entries ? g_prof.count : max_entries;
    size_t used = 0;
    if (names && names_bytes) names[0] = 0;
    for (int i = 0; i < n; ++i) {
        float t = 0.0f;
        if (hipEventSynchronize(g_prof.ev[2 * i + 1]) != hipSuccess ||
            hipEventElapsedTime(&t, g_prof.ev[2 * i], g_prof.ev[2 * i + 1]) != hipSuccess)
            t = -1.0f;  // a failed measurement is reported as negative, never as zero
        if (ms) ms[i] = t;
        if (names) {
            const char *nm = g_prof.name[i];
            for (size_t c = 0; nm[c] && used + 2 < names_bytes; ++c) names[used++] = nm[c];
            if (used + 1 < names_bytes) names[used++] = ';';
            names[used] = 0;
        }
    }
    g_prof.count = 0;
    return n;
}

extern "C" int dl_version(void) { return 100; }

extern "C" const char *dl_error_string(int code) {
    switch (code) {
        case DL_OK: return "ok";
        case DL_ERR_NULL: return "a required pointer is null";
        case DL_ERR_SHAPE: return "a size is not positive or sizes are inconsistent";
        case DL_ERR_UNSUPPORTED: return "k, O or an option is outside what the kernels cover";
        case DL_ERR_WORKSPACE: return "workspace is smaller than the matching *_workspace_bytes()";
        case DL_ERR_INDEX: return "an index is outside [0, I)";
        case DL_ERR_SCRATCH: return "the call needs more scratch than the library's static device array holds";
        default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
    }
}
