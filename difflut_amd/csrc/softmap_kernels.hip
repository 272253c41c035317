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
// 128 x 128, each wavefront 64 x 64 = 2x2 MFMA tiles (4 x 16 accumulator registers).  The
// reduction is staged through LDS SM_K deep as As[k][row], Bs[k][col] (k-major, so an MFMA operand
// read is 64 consecutive floats), two stages resident: while the MFMAs read one, the next is
// written piecewise between MFMA groups and the one after that is on its way from memory.
#include <type_traits>

#include "dl_common.h"

typedef float floatx16 __attribute__((ext_vector_type(16)));

#define SM_T 128     // output tile edge
#define SM_K 16      // reduction depth per LDS stage (32 measured 2 % slower in all three modes)
#define SM_LD_V 132  // LDS row stride (floats) of a stage written with float4 stores: multiple of 4
#define SM_LD_T 133  // ... of a stage written transposed, one float at a time: odd, spreads the banks
#define SM_LOG2E 1.4426950408889634f

// exp((w - mx)/tau) / sum, with scale = log2(e)/tau: one subtract, one multiply, the hardware
// exp2 and the normalisation.  Relative error about |w - mx|/tau * 6e-8 plus one ulp of exp2.
// The row sums are built with the same function, so rows of S sum to one to rounding.
__device__ __forceinline__ float softmap_e(float w, float mx, float scale) {
    return __builtin_amdgcn_exp2f((w - mx) * scale);
}
__device__ __forceinline__ float softmap_s(float w, float mx, float rs, float scale) {
    return softmap_e(w, mx, scale) * rs;
}

// one wavefront per row of W; the second sweep of the row comes from cache
__global__ __launch_bounds__(256) void softmap_rowstats(const float *__restrict__ W, float scale, float *__restrict__ stats,
                                                         int M, int I) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= M) return;
    const float *w = W + (size_t)row * I;
    float mx = -INFINITY, sum = 0.0f;
    if (I % 4 == 0) {
        const float4 *w4 = reinterpret_cast<const float4 *>(w);
        const int n4 = I >> 2;
        float m0 = -INFINITY, m1 = -INFINITY;
        int i = lane;
        for (; i + 64 < n4; i += 128) {
            const float4 a = w4[i], b = w4[i + 64];
            m0 = fmaxf(m0, fmaxf(fmaxf(a.x, a.y), fmaxf(a.z, a.w)));
            m1 = fmaxf(m1, fmaxf(fmaxf(b.x, b.y), fmaxf(b.z, b.w)));
        }
        if (i < n4) { const float4 a = w4[i]; m0 = fmaxf(m0, fmaxf(fmaxf(a.x, a.y), fmaxf(a.z, a.w))); }
        mx = fmaxf(m0, m1);
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
        for (i = lane; i < n4; i += 64) {
            const float4 a = w4[i];
            sum += (softmap_e(a.x, mx, scale) + softmap_e(a.y, mx, scale)) +
                   (softmap_e(a.z, mx, scale) + softmap_e(a.w, mx, scale));
        }
    } else {
        for (int i = lane; i < I; i += 64) mx = fmaxf(mx, w[i]);
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
        for (int i = lane; i < I; i += 64) sum += softmap_e(w[i], mx, scale);
    }
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if (lane == 0) { stats[2 * row] = mx; stats[2 * row + 1] = 1.0f / sum; }
}

// r[o] = sum_b gm[b,o] m[b,o]; block = 32 columns x 8 row groups, partial sums joined in LDS in fixed order
__global__ __launch_bounds__(256) void softmap_rowdot(const float *__restrict__ gm, const float *__restrict__ m,
                                                       float *__restrict__ r, int B, int M) {
    __shared__ float part[8][33];
    const int c = threadIdx.x & 31, g = threadIdx.x >> 5;
    const int o = blockIdx.x * 32 + c;
    float acc = 0.0f;
    if (o < M) {
        int b = g;
        for (; b + 24 < B; b += 32) {
            const size_t e = (size_t)b * M + o;
            const float g0 = gm[e], g1 = gm[e + 8 * (size_t)M], g2 = gm[e + 16 * (size_t)M], g3 = gm[e + 24 * (size_t)M];
            const float m0 = m[e], m1 = m[e + 8 * (size_t)M], m2 = m[e + 16 * (size_t)M], m3 = m[e + 24 * (size_t)M];
            acc += g0 * m0; acc += g1 * m1; acc += g2 * m2; acc += g3 * m3;
        }
        for (; b < B; b += 8) acc += gm[(size_t)b * M + o] * m[(size_t)b * M + o];
    }
    part[g][c] = acc;
    __syncthreads();
    if (g == 0 && o < M) {
        float t = part[0][c];
#pragma unroll
        for (int q = 1; q < 8; ++q) t += part[q][c];
        r[o] = t;
    }
}

// out[e] = sum over chunks of part[chunk][e], fixed order; VEC = 4 when total is a multiple of 4
template <int VEC>
__global__ __launch_bounds__(256) void softmap_reduce_chunks(const float *__restrict__ part, float *__restrict__ out,
                                                              long long total, int chunks) {
    const long long e = ((long long)blockIdx.x * 256 + threadIdx.x) * VEC;
    if (e >= total) return;
    if (VEC == 4) {
        float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        int c = 0;
        for (; c + 4 <= chunks; c += 4) {  // four independent loads in flight, added in chunk order
            const float4 p0 = *reinterpret_cast<const float4 *>(part + (size_t)c * total + e);
            const float4 p1 = *reinterpret_cast<const float4 *>(part + (size_t)(c + 1) * total + e);
            const float4 p2 = *reinterpret_cast<const float4 *>(part + (size_t)(c + 2) * total + e);
            const float4 p3 = *reinterpret_cast<const float4 *>(part + (size_t)(c + 3) * total + e);
            acc.x += p0.x; acc.y += p0.y; acc.z += p0.z; acc.w += p0.w;
            acc.x += p1.x; acc.y += p1.y; acc.z += p1.z; acc.w += p1.w;
            acc.x += p2.x; acc.y += p2.y; acc.z += p2.z; acc.w += p2.w;
            acc.x += p3.x; acc.y += p3.y; acc.z += p3.z; acc.w += p3.w;
        }
        for (; c < chunks; ++c) {
            const float4 p = *reinterpret_cast<const float4 *>(part + (size_t)c * total + e);
            acc.x += p.x; acc.y += p.y; acc.z += p.z; acc.w += p.w;
        }
        *reinterpret_cast<float4 *>(out + e) = acc;
    } else {
        float acc = 0.0f;
        for (int c = 0; c < chunks; ++c) acc += part[(size_t)c * total + e];
        out[e] = acc;
    }
}

struct SoftmapArgs {
    const float *x, *W, *stats, *gm, *r;
    float scale, inv_tau;
    float *out;
    int B, I, M;
    int inner_count, outer_count, col_tiles, red_chunk;
    const unsigned short *Eb;  // precision 1: bf16 softmax numerators [M][I]
    const float *rs;           // precision 1: 1 / row sum [M]
    // precision 1: operands rounded to bf16 once, in the layout their product reads
    const unsigned short *xb;   // x [B][I]                      (forward A operand)
    const uint4 *x8;            // x in blocks of 8 batch rows: [ceil(B/8)][I] x 8 bf16   (gW B operand)
    const unsigned short *gms;  // gm[b][o] / sum[o], [B][M]     (gx A operand)
    const uint4 *gm8;           // gm in blocks of 8 batch rows: [ceil(B/8)][M] x 8 bf16  (gW A operand)
};

// MODE 0: forward   rows=b cols=o red=i   A = x[b,i]  (red contiguous)   B = S[o,i] (red contiguous)
// MODE 1: gx        rows=b cols=i red=o   A = gm[b,o] (red contiguous)   B = S[o,i] (col contiguous)
// MODE 2: gW        rows=o cols=i red=b   A = gm[b,o] (row contiguous)   B = x[b,i] (col contiguous)
//                   epilogue S[o,i] (C - r[o]) / tau
// EDGE false: the tile lies inside the matrices, the reduction range is a whole number of stages
// and every float4 is aligned, so the loop body is straight-line code and the compiler can count
// outstanding loads exactly.  EDGE true: every access is predicated (ragged shapes).
template <int MODE, int KC, bool EDGE>
__device__ __forceinline__ void softmap_tile(const SoftmapArgs &g, float *sm_lds, int rt, int ct, int zc) {
    constexpr bool A_RED_CONTIG = MODE != 2;
    constexpr bool B_RED_CONTIG = MODE == 0;
    constexpr int LDA = A_RED_CONTIG ? SM_LD_T : SM_LD_V;
    constexpr int LDB = B_RED_CONTIG ? SM_LD_T : SM_LD_V;
    constexpr int P = KC / 8;  // float4 pieces per operand per thread per stage
    float *const As = sm_lds;                  // [2][KC][LDA]
    float *const Bs = sm_lds + 2 * KC * LDA;   // [2][KC][LDB]
    const float *__restrict__ x = g.x, *__restrict__ W = g.W, *__restrict__ stats = g.stats, *__restrict__ gm = g.gm;
    const int B = g.B, I = g.I, M = g.M;
    const float scale = g.scale;

    const int R = MODE == 2 ? M : B;                      // rows of the output
    const int C = MODE == 0 ? M : I;                      // columns of the output
    const int KD = MODE == 0 ? I : (MODE == 1 ? M : B);   // reduction length
    const int r0 = rt * SM_T, c0 = ct * SM_T;
    const int k_begin = zc * g.red_chunk;
    const int k_end = min(KD, k_begin + g.red_chunk);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;  // wavefront's corner inside the tile
    float4 pa[P], pb[P];
    float bmx[P], brs[P];  // row statistics that go with pb (B operand built from W)

    // thread -> piece of the tile.  red-contiguous operand: float4 runs along k (KC/4 per row),
    // 1024/KC rows per pass; row/col-contiguous operand: float4 runs along the row/col axis (32 per k), 8 k per pass
    constexpr int QR = KC / 4, RP = 1024 / KC;
    const int a_q = A_RED_CONTIG ? (tid % QR) : (tid & 31), a_o = A_RED_CONTIG ? (tid / QR) : (tid >> 5);
    const int b_q = B_RED_CONTIG ? (tid % QR) : (tid & 31), b_o = B_RED_CONTIG ? (tid / QR) : (tid >> 5);
    const int lda = MODE == 0 ? I : M;

    auto in_a = [&](int row, int k) -> float {  // predicated scalar access
        if (row >= R || k >= k_end) return 0.0f;
        if (MODE == 0) return x[(size_t)row * I + k];
        if (MODE == 1) return gm[(size_t)row * M + k];
        return gm[(size_t)k * M + row];
    };
    auto in_b = [&](int k, int col) -> float {
        if (col >= C || k >= k_end) return 0.0f;
        if (MODE == 0) return softmap_s(W[(size_t)col * I + k], stats[2 * col], stats[2 * col + 1], scale);
        if (MODE == 1) return softmap_s(W[(size_t)k * I + col], stats[2 * k], stats[2 * k + 1], scale);
        return x[(size_t)k * I + col];
    };

    if (!EDGE && MODE == 0) {  // the W rows a thread stages do not change from stage to stage
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int col = c0 + b_o + RP * p;
            bmx[p] = stats[2 * col]; brs[p] = stats[2 * col + 1];
        }
    }
    auto fetch = [&](int p, int k0) __attribute__((always_inline)) {
        if (EDGE) {
            if (A_RED_CONTIG) {
                const int row = r0 + a_o + RP * p, k = k0 + a_q * 4;
                pa[p] = make_float4(in_a(row, k), in_a(row, k + 1), in_a(row, k + 2), in_a(row, k + 3));
            } else {
                const int k = k0 + a_o + 8 * p, row = r0 + a_q * 4;
                pa[p] = make_float4(in_a(row, k), in_a(row + 1, k), in_a(row + 2, k), in_a(row + 3, k));
            }
            if (B_RED_CONTIG) {
                const int col = c0 + b_o + RP * p, k = k0 + b_q * 4;
                pb[p] = make_float4(in_b(k, col), in_b(k + 1, col), in_b(k + 2, col), in_b(k + 3, col));
            } else {
                const int k = k0 + b_o + 8 * p, col = c0 + b_q * 4;
                pb[p] = make_float4(in_b(k, col), in_b(k, col + 1), in_b(k, col + 2), in_b(k, col + 3));
            }
        } else {
            if (A_RED_CONTIG) {
                const int row = r0 + a_o + RP * p, k = k0 + a_q * 4;
                pa[p] = *reinterpret_cast<const float4 *>((MODE == 0 ? x : gm) + (size_t)row * lda + k);
            } else {
                const int k = k0 + a_o + 8 * p, row = r0 + a_q * 4;
                pa[p] = *reinterpret_cast<const float4 *>(gm + (size_t)k * M + row);
            }
            if (B_RED_CONTIG) {
                const int col = c0 + b_o + RP * p, k = k0 + b_q * 4;
                pb[p] = *reinterpret_cast<const float4 *>(W + (size_t)col * I + k);
            } else {
                const int k = k0 + b_o + 8 * p, col = c0 + b_q * 4;
                pb[p] = *reinterpret_cast<const float4 *>((MODE == 1 ? W : x) + (size_t)k * I + col);
                if (MODE == 1) { bmx[p] = stats[2 * k]; brs[p] = stats[2 * k + 1]; }
            }
        }
    };
    auto commit = [&](int p, int buf) __attribute__((always_inline)) {
        float *Ab = As + buf * KC * LDA, *Bb = Bs + buf * KC * LDB;
        if (A_RED_CONTIG) {
            float *d = Ab + (a_q * 4) * LDA + a_o + RP * p;
            d[0] = pa[p].x; d[LDA] = pa[p].y; d[2 * LDA] = pa[p].z; d[3 * LDA] = pa[p].w;
        } else {
            const float4 va = make_float4(pa[p].x, pa[p].y, pa[p].z, pa[p].w);  // by value: keeps pa in registers
            *reinterpret_cast<float4 *>(Ab + (a_o + 8 * p) * LDA + a_q * 4) = va;
        }
        float4 v = pb[p];
        if (!EDGE && MODE != 2) {  // W values -> softmax entries (the predicated path did it on load)
            v.x = softmap_s(v.x, bmx[p], brs[p], scale); v.y = softmap_s(v.y, bmx[p], brs[p], scale);
            v.z = softmap_s(v.z, bmx[p], brs[p], scale); v.w = softmap_s(v.w, bmx[p], brs[p], scale);
        }
        if (B_RED_CONTIG) {
            float *d = Bb + (b_q * 4) * LDB + b_o + RP * p;
            d[0] = v.x; d[LDB] = v.y; d[2 * LDB] = v.z; d[3 * LDB] = v.w;
        } else {
            *reinterpret_cast<float4 *>(Bb + (b_o + 8 * p) * LDB + b_q * 4) = v;
        }
    };

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    const int nst = (k_end - k_begin + KC - 1) / KC;
    if (nst > 0) {
#pragma unroll
        for (int p = 0; p < P; ++p) fetch(p, k_begin);
#pragma unroll
        for (int p = 0; p < P; ++p) commit(p, 0);
        if (nst > 1) {
#pragma unroll
            for (int p = 0; p < P; ++p) fetch(p, k_begin + KC);
        }
    }
    __syncthreads();
    const int kh = lane >> 5, l32 = lane & 31;
    // one stage: MFMAs over buffer s&1; between MFMA groups, piece p of stage s+1 goes from
    // registers to the other buffer and piece p of stage s+2 is requested from memory
    auto stage = [&](int s, auto do_commit, auto do_fetch) __attribute__((always_inline)) {
        const int cur = s & 1;
        const float *Ab = As + cur * KC * LDA + kh * LDA + wm + l32;
        const float *Bb = Bs + cur * KC * LDB + kh * LDB + wn + l32;
        float a0 = Ab[0], a1 = Ab[32], b0 = Bb[0], b1 = Bb[32];
#pragma unroll
        for (int p = 0; p < P; ++p) {
#pragma unroll
            for (int k2 = p * 8; k2 < p * 8 + 8; k2 += 2) {
                float na0 = 0.0f, na1 = 0.0f, nb0 = 0.0f, nb1 = 0.0f;
                if (k2 + 2 < KC) {  // operands of the next step are on their way while this step's MFMAs issue
                    na0 = Ab[(k2 + 2) * LDA]; na1 = Ab[(k2 + 2) * LDA + 32];
                    nb0 = Bb[(k2 + 2) * LDB]; nb1 = Bb[(k2 + 2) * LDB + 32];
                }
                acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
                acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
                acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
                acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
                a0 = na0; a1 = na1; b0 = nb0; b1 = nb1;
            }
            // keep the scheduler from sinking the loads to the end of the stage (their data is
            // needed one stage later, not sooner) or hoisting the staging work above the MFMAs
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (decltype(do_commit)::value) commit(p, cur ^ 1);
            if constexpr (decltype(do_fetch)::value) fetch(p, k_begin + (s + 2) * KC);
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
    };
    {
        using T = std::true_type;
        using F = std::false_type;
        int s = 0;
        for (; s + 2 < nst; ++s) stage(s, T{}, T{});
        if (s + 1 < nst) { stage(s, T{}, F{}); ++s; }
        if (s < nst) stage(s, F{}, F{});
    }
    // accumulator layout of a 32x32 tile: register v of lane l holds row 8*(v/4) + 4*(l/32) + v%4, column l%32
    float *dst = g.out + (size_t)zc * R * C;
    float *rowst = reinterpret_cast<float *>(sm_lds);  // MODE 2: per tile row {max, 1/sum, r}, staged once
    if (MODE == 2) {
        if (tid < SM_T) {
            const int row = min(r0 + tid, R - 1);
            rowst[tid * 4] = stats[2 * row];
            rowst[tid * 4 + 1] = stats[2 * row + 1];
            rowst[tid * 4 + 2] = g.r[row];
        }
        __syncthreads();
    }
    if (MODE == 2 && !EDGE) {
        // Interior tiles: a wavefront's 64 x 64 block of G goes through LDS 32 rows at a time, so that a
        // lane owns four consecutive columns of a row: 16-byte loads of W and 16-byte stores of gW in runs
        // of 256 bytes per row (the accumulator layout itself gives 4-byte accesses in runs of 128).
        // Each wavefront uses its own LDS region behind the row statistics; no block barrier is needed.
        constexpr int TS = 68;  // floats per staged row: 64 + 4, keeps 16-byte alignment
        float *stg = rowst + 4 * SM_T + (tid >> 6) * (32 * TS);
        const int rr = lane >> 4, c4 = (lane & 15) * 4;
#pragma clang loop unroll(disable)
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const floatx16 a = i == 0 ? (j == 0 ? acc[0][0] : acc[0][1]) : (j == 0 ? acc[1][0] : acc[1][1]);
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    stg[(8 * (v >> 2) + 4 * (lane >> 5) + (v & 3)) * TS + j * 32 + (lane & 31)] = a[v];
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int it = 0; it < 8; ++it) {
                const int lr = wm + i * 32 + it * 4 + rr;
                const size_t at = (size_t)(r0 + lr) * I + c0 + wn + c4;
                const float4 gv = *reinterpret_cast<const float4 *>(stg + (it * 4 + rr) * TS + c4);
                const float4 wv = *reinterpret_cast<const float4 *>(W + at);
                const float mx = rowst[lr * 4], f = rowst[lr * 4 + 1] * g.inv_tau, rv = rowst[lr * 4 + 2];
                float4 o;
                o.x = softmap_e(wv.x, mx, scale) * f * (gv.x - rv);
                o.y = softmap_e(wv.y, mx, scale) * f * (gv.y - rv);
                o.z = softmap_e(wv.z, mx, scale) * f * (gv.z - rv);
                o.w = softmap_e(wv.w, mx, scale) * f * (gv.w - rv);
                *reinterpret_cast<float4 *>(dst + at) = o;
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    } else if (MODE == 2) {
        // one 32x32 sub-tile per trip of a loop that is kept rolled: unrolled, the scheduler puts all
        // 64 W loads in flight at once and the registers that costs push the staging buffers of
        // the main loop into scratch memory
#pragma clang loop unroll(disable)
        for (int ij = 0; ij < 4; ++ij) {
            const int i = ij >> 1, j = ij & 1;
            const floatx16 a = ij == 0 ? acc[0][0] : ij == 1 ? acc[0][1] : ij == 2 ? acc[1][0] : acc[1][1];
            const int col = c0 + wn + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int lr = wm + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                const int row = r0 + lr;
                if (!EDGE || (row < R && col < C)) {
                    const float sv = softmap_s(W[(size_t)row * I + col], rowst[lr * 4], rowst[lr * 4 + 1], scale);
                    dst[(size_t)row * C + col] = sv * (a[v] - rowst[lr * 4 + 2]) * g.inv_tau;
                }
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int col = c0 + wn + j * 32 + (lane & 31);
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = r0 + wm + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                    if (!EDGE || (row < R && col < C)) dst[(size_t)row * C + col] = acc[i][j][v];
                }
            }
    }
}

// 1-D grid decoded so that blocks which share the large operand tile (W, or the gm column slab in
// MODE 2) sit next to each other on one XCD and find it in that XCD's L2.  MODE 1 also carries a
// chunk of the reduction in the block index; out then points at [chunks][R][C] partial products.
template <int MODE, int KC>
__global__ __launch_bounds__(256, 3) void softmap_mfma(SoftmapArgs g) {
    extern __shared__ __align__(16) float sm_lds[];
    int inner, outer;
    if (!dl_xcd_map(g.inner_count, g.outer_count, inner, outer)) return;
    const int rt = MODE == 2 ? outer : inner;
    const int ct = MODE == 2 ? inner : (MODE == 1 ? outer % g.col_tiles : outer);
    const int zc = MODE == 1 ? outer / g.col_tiles : 0;
    const int R = MODE == 2 ? g.M : g.B, C = MODE == 0 ? g.M : g.I;
    const int KD = MODE == 0 ? g.I : (MODE == 1 ? g.M : g.B);
    const int k_begin = zc * g.red_chunk, k_end = min(KD, k_begin + g.red_chunk);
    const bool inside = (rt + 1) * SM_T <= R && (ct + 1) * SM_T <= C && (k_end - k_begin) % KC == 0 &&
                        g.red_chunk % 4 == 0 && g.I % 4 == 0 && g.M % 4 == 0;
    if (inside) softmap_tile<MODE, KC, false>(g, sm_lds, rt, ct, zc);
    else softmap_tile<MODE, KC, true>(g, sm_lds, rt, ct, zc);
}

template <int MODE, int KC>
static void softmap_launch(const SoftmapArgs &g, hipStream_t s) {
    constexpr int LDA = MODE != 2 ? SM_LD_T : SM_LD_V, LDB = MODE == 0 ? SM_LD_T : SM_LD_V;
    // the gW epilogue re-uses the stages: row statistics (4 floats per tile row) + 32 x 68 floats per wavefront
    constexpr int stage_bytes = 2 * KC * (LDA + LDB) * (int)sizeof(float);
    constexpr int epi_bytes = MODE == 2 ? (4 * SM_T + 4 * 32 * 68) * (int)sizeof(float) : 0;
    constexpr int lds_bytes = stage_bytes > epi_bytes ? stage_bytes : epi_bytes;
    if (lds_bytes > 65536)
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&softmap_mfma<MODE, KC>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    softmap_mfma<MODE, KC><<<dl_xcd_grid(g.inner_count, g.outer_count), 256, lds_bytes, s>>>(g);
}

// ---------------------------------------------------------------------------------
// bf16 operands, fp32 accumulation (v_mfma_f32_32x32x16_bf16), precision = 1.  Same tiling and
// operand modes as the fp32 kernel.  Here the softmax numerators E[o,i] = exp((W - max)/tau) are
// written once, rounded to bf16, by the row-statistics pass (301 MB for the 48000 x 3136 case, kept
// with the statistics for the backward); 1/sum stays a per-row fp32 factor that is applied to the
// forward output, to the gm operand of the gx product and in the gW epilogue.  x and gm are rounded
// to bf16 (nearest even) once per call by a packing pass (softmap_pack_bf16), into the layout the
// staging code copies to LDS unchanged.  A lane feeds the MFMA eight consecutive k of one row, so LDS
// holds a stage row-major, As[row][32 k], unpadded and XOR-swizzled in units of 16 bytes.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
#define SB_K 32   // reduction depth per stage
#define SB_LD 64  // bytes per LDS row: 32 k, no padding
// Rows are unpadded, so two consecutive rows fill the 32 banks exactly; the 16-byte block (8 k) of a row
// sits at position block ^ softmap_swz(row).  Eight consecutive rows then put a given logical block on
// eight different bank groups: the 16-byte stores of a stage (consecutive lanes = the blocks of two
// consecutive rows) and the 16-byte MFMA operand reads (consecutive lanes = consecutive rows, one logical
// block) are both free of bank conflicts.  The second term separates rows 16 apart for the one stage
// that is written transposed, 4 bytes at a time.
__device__ __forceinline__ int softmap_swz(int row) { return ((row >> 1) ^ (row >> 4)) & 3; }

__device__ __forceinline__ unsigned softmap_pk_bf16(float lo, float hi) {
    const floatx2 v = {lo, hi};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ float softmap_bf16_f32(unsigned short h) { return __uint_as_float((unsigned)h << 16); }

// one wavefront per row of W: max, then E = bf16(exp2((w - max) * scale)) and 1 / sum of the rounded E
__global__ __launch_bounds__(256) void softmap_rowstats_bf16(const float *__restrict__ W, float scale, float *__restrict__ mxs,
                                                              float *__restrict__ rss, unsigned short *__restrict__ Eb,
                                                              int M, int I) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= M) return;
    const float *w = W + (size_t)row * I;
    unsigned short *e = Eb + (size_t)row * I;
    float mx = -INFINITY, sum = 0.0f;
    if (I % 4 == 0) {
        const float4 *w4 = reinterpret_cast<const float4 *>(w);
        const int n4 = I >> 2;
        for (int i = lane; i < n4; i += 64) {
            const float4 a = w4[i];
            mx = fmaxf(mx, fmaxf(fmaxf(a.x, a.y), fmaxf(a.z, a.w)));
        }
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
        for (int i = lane; i < n4; i += 64) {
            const float4 a = w4[i];
            const unsigned lo = softmap_pk_bf16(softmap_e(a.x, mx, scale), softmap_e(a.y, mx, scale));
            const unsigned hi = softmap_pk_bf16(softmap_e(a.z, mx, scale), softmap_e(a.w, mx, scale));
            sum += (__uint_as_float(lo << 16) + __uint_as_float(lo & 0xffff0000u)) +
                   (__uint_as_float(hi << 16) + __uint_as_float(hi & 0xffff0000u));
            *reinterpret_cast<uint2 *>(e + 4 * i) = make_uint2(lo, hi);
        }
    } else {
        for (int i = lane; i < I; i += 64) mx = fmaxf(mx, w[i]);
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
        for (int i = lane; i < I; i += 64) {
            const unsigned short h = (unsigned short)(softmap_pk_bf16(softmap_e(w[i], mx, scale), 0.0f) & 0xffffu);
            sum += softmap_bf16_f32(h);
            e[i] = h;
        }
    }
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if (lane == 0) { mxs[row] = mx; rss[row] = 1.0f / sum; }
}

// Row statistics with the row held in registers (rows of up to 256 * NV floats, I a multiple of 4): W is
// read once - the two-sweep kernels above fetch it twice, the second sweep does not stay in cache when
// every wavefront of the chip streams its own 12 KB row.  One wavefront per row; BF16 also writes the bf16
// numerators and sums the rounded values, exactly as softmap_rowstats_bf16 does.
template <int NV, bool BF16>
__global__ __launch_bounds__(256) void softmap_rowstats_regs(const float *__restrict__ W, float scale, float *__restrict__ out_a,
                                                              float *__restrict__ out_b, unsigned short *__restrict__ Eb,
                                                              int M, int I) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= M) return;
    const float4 *w4 = reinterpret_cast<const float4 *>(W + (size_t)row * I);
    const int n4 = I >> 2;
    float4 v[NV];
#pragma unroll
    for (int q = 0; q < NV; ++q) {
        const int i = lane + 64 * q;
        v[q] = i < n4 ? w4[i] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int q = 0; q < NV; ++q) mx = fmaxf(mx, fmaxf(fmaxf(v[q].x, v[q].y), fmaxf(v[q].z, v[q].w)));
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    float sum = 0.0f;
#pragma unroll
    for (int q = 0; q < NV; ++q) {
        const int i = lane + 64 * q;
        // exp2(-inf) = 0: the padding adds nothing
        const float e0 = softmap_e(v[q].x, mx, scale), e1 = softmap_e(v[q].y, mx, scale);
        const float e2 = softmap_e(v[q].z, mx, scale), e3 = softmap_e(v[q].w, mx, scale);
        if (BF16) {
            const unsigned lo = softmap_pk_bf16(e0, e1), hi = softmap_pk_bf16(e2, e3);
            sum += (__uint_as_float(lo << 16) + __uint_as_float(lo & 0xffff0000u)) +
                   (__uint_as_float(hi << 16) + __uint_as_float(hi & 0xffff0000u));
            if (i < n4) *reinterpret_cast<uint2 *>(Eb + (size_t)row * I + 4 * i) = make_uint2(lo, hi);
        } else {
            sum += (e0 + e1) + (e2 + e3);
        }
    }
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if (lane == 0) {
        if (BF16) { out_a[row] = mx; out_b[row] = 1.0f / sum; }
        else { out_a[2 * row] = mx; out_a[2 * row + 1] = 1.0f / sum; }
    }
}

// Operands of the bf16 products, rounded once (nearest even) into the layout the staging code copies:
// row-major bf16 for an operand that is contiguous along the reduction; for one that is contiguous
// along the rows / columns of the product (the reduction runs over its rows) blocks of 8 consecutive
// reduction steps per element, because an MFMA lane wants 8 consecutive k side by side - the
// transposition happens here, through coalesced accesses, and not as bank-conflicting LDS stores.
// src [R][C] fp32 -> rows [R][C] bf16 (optionally scaled per column) and/or blocks [ceil(R/8)][C] x 8 bf16.
__global__ __launch_bounds__(256) void softmap_pack_bf16(const float *__restrict__ src, const float *__restrict__ colscale,
                                                          unsigned short *__restrict__ rows, uint4 *__restrict__ blocks,
                                                          int R, int C) {
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    const int RB = (R + 7) / 8;
    if (e >= (long long)RB * C) return;
    const int c = (int)(e % C);
    const int rb = (int)(e / C);
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = 8 * rb + i < R ? src[(size_t)(8 * rb + i) * C + c] : 0.0f;
    if (blocks)
        blocks[e] = make_uint4(softmap_pk_bf16(v[0], v[1]), softmap_pk_bf16(v[2], v[3]), softmap_pk_bf16(v[4], v[5]),
                               softmap_pk_bf16(v[6], v[7]));
    if (rows) {
        const float f = colscale ? colscale[c] : 1.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (8 * rb + i < R) rows[(size_t)(8 * rb + i) * C + c] = (unsigned short)(softmap_pk_bf16(v[i] * f, 0.0f) & 0xffffu);
    }
}

template <int MODE, bool EDGE>
__device__ __forceinline__ void softmap_tile_bf16(const SoftmapArgs &g, char *lds, int rt, int ct, int zc) {
    constexpr int KC = SB_K;
    constexpr bool A_RED_CONTIG = MODE != 2;
    constexpr int STAGE = SM_T * SB_LD;  // bytes of one operand stage
    char *const As = lds;                // [2][128][SB_LD]
    char *const Bs = lds + 2 * STAGE;
    const float *__restrict__ rs = g.rs;
    const unsigned short *__restrict__ Eb = g.Eb;
    const int B = g.B, I = g.I, M = g.M;
    const int R = MODE == 2 ? M : B, C = MODE == 0 ? M : I;
    const int KD = MODE == 0 ? I : (MODE == 1 ? M : B);
    const int r0 = rt * SM_T, c0 = ct * SM_T;
    const int k_begin = zc * g.red_chunk;
    const int k_end = min(KD, k_begin + g.red_chunk);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;

    // ---- A operand, bf16 in memory (softmap_pack_bf16): two 16-byte pieces per thread and stage.
    // red-contiguous (x rows; gm / sum rows): 8 consecutive k of row a_o + 64 p, copied as they are.
    // row-contiguous (gW: gm in blocks of 8 k): k-block a_q (= my wavefront) of row a_o + 64 p, so a
    // wavefront reads 64 consecutive rows = 1 KB and stores them to 64 consecutive LDS rows.
    uint4 pa[2];
    const int a_q = A_RED_CONTIG ? (tid & 3) : (tid >> 6), a_o = A_RED_CONTIG ? (tid >> 2) : (tid & 63);
    const unsigned short *__restrict__ arow = MODE == 0 ? g.xb : g.gms;
    const int lda = MODE == 0 ? I : M;
    const int kb_end = (k_end + 7) / 8;
    auto fetch_a = [&](int p, int k0) __attribute__((always_inline)) {
        if (A_RED_CONTIG) {
            const int row = r0 + a_o + 64 * p, k = k0 + a_q * 8;
            if (EDGE) {
                unsigned w[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const unsigned lo = (row < R && k + 2 * j < k_end) ? arow[(size_t)row * lda + k + 2 * j] : 0u;
                    const unsigned hi = (row < R && k + 2 * j + 1 < k_end) ? arow[(size_t)row * lda + k + 2 * j + 1] : 0u;
                    w[j] = lo | (hi << 16);
                }
                pa[p] = make_uint4(w[0], w[1], w[2], w[3]);
            } else {
                pa[p] = *reinterpret_cast<const uint4 *>(arow + (size_t)row * lda + k);
            }
        } else {
            const int kb = (k0 >> 3) + a_q, row = r0 + a_o + 64 * p;
            if (EDGE) pa[p] = (kb < kb_end && row < R) ? g.gm8[(size_t)kb * M + row] : make_uint4(0u, 0u, 0u, 0u);
            else pa[p] = g.gm8[(size_t)kb * M + row];
        }
    };
    auto commit_a = [&](int p, int buf) __attribute__((always_inline)) {
        char *Ab = As + buf * STAGE;
        const uint4 v = make_uint4(pa[p].x, pa[p].y, pa[p].z, pa[p].w);
        const int row = a_o + 64 * p;  // both forms: 8 k of one row
        *reinterpret_cast<uint4 *>(Ab + row * SB_LD + ((a_q ^ softmap_swz(row)) << 4)) = v;
    };

    // ---- B operand
    //  MODE 0: E[o, k] bf16, red-contiguous: 8 consecutive k of column (= row of W) b_o + 64 p, copied as
    //          they are, like the A operand
    //  MODE 1: E[k, i] bf16, column-contiguous: rows 2 kp and 2 kp + 1, 8 columns each -> packed pairs
    //  MODE 2: x in blocks of 8 k, column-contiguous: as the A operand of that mode
    uint4 pe[2];
    const int e_q = tid & 15, e_o = tid >> 4;
    const int b_q = tid & 3, b_o = tid >> 2;  // MODE 0
    auto eb = [&](int o, int i) -> unsigned {  // predicated scalar access, bits of E[o,i]
        return (o < M && i < I) ? (unsigned)Eb[(size_t)o * I + i] : 0u;
    };
    auto fetch_b = [&](int p, int k0) __attribute__((always_inline)) {
        if (MODE == 0) {
            const int col = c0 + b_o + 64 * p, k = k0 + b_q * 8;
            if (EDGE) {
                unsigned wv[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const unsigned lo = k + 2 * j < k_end ? eb(col, k + 2 * j) : 0u;
                    const unsigned hi = k + 2 * j + 1 < k_end ? eb(col, k + 2 * j + 1) : 0u;
                    wv[j] = lo | (hi << 16);
                }
                pe[p] = make_uint4(wv[0], wv[1], wv[2], wv[3]);
            } else {
                pe[p] = *reinterpret_cast<const uint4 *>(Eb + (size_t)col * I + k);
            }
        } else if (MODE == 1) {
            const int k = k0 + 2 * e_o + p, col = c0 + e_q * 8;  // p = 0, 1: the two rows of the pair
            if (EDGE) {
                unsigned wv[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const unsigned lo = k < k_end ? eb(k, col + 2 * j) : 0u;
                    const unsigned hi = k < k_end ? eb(k, col + 2 * j + 1) : 0u;
                    wv[j] = lo | (hi << 16);
                }
                pe[p] = make_uint4(wv[0], wv[1], wv[2], wv[3]);
            } else {
                pe[p] = *reinterpret_cast<const uint4 *>(Eb + (size_t)k * I + col);
            }
        } else {
            const int kb = (k0 >> 3) + (tid >> 6), col = c0 + (tid & 63) + 64 * p;
            if (EDGE) pe[p] = (kb < kb_end && col < C) ? g.x8[(size_t)kb * I + col] : make_uint4(0u, 0u, 0u, 0u);
            else pe[p] = g.x8[(size_t)kb * I + col];
        }
    };
    auto commit_b = [&](int p, int buf) __attribute__((always_inline)) {
        char *Bb = Bs + buf * STAGE;
        if (MODE == 0) {
            const int row = b_o + 64 * p;
            *reinterpret_cast<uint4 *>(Bb + row * SB_LD + ((b_q ^ softmap_swz(row)) << 4)) = make_uint4(pe[p].x, pe[p].y, pe[p].z, pe[p].w);
        } else if (MODE == 1) {
            if (p == 1) {
                const unsigned ra[4] = {pe[0].x, pe[0].y, pe[0].z, pe[0].w};
                const unsigned rb[4] = {pe[1].x, pe[1].y, pe[1].z, pe[1].w};
                // The pair (k, k+1) = dword e_o of rows 8 e_q + j, j = 0..7.  Lanes that differ in e_q are 8
                // rows apart, i.e. on the same banks but for the swizzle; to use both halves of the banks in
                // every store, lanes with odd e_q walk their columns in the order j ^ 1.
                const int odd = e_q & 1;
                const unsigned sel_lo = 0x05040100u, sel_hi = 0x07060302u;  // low / high halves of the two rows
#pragma unroll
                for (int st = 0; st < 8; ++st) {
                    const int j = st ^ odd;  // j >> 1 == st >> 1: same source registers for every lane
                    const unsigned a = ra[st >> 1], b = rb[st >> 1];
                    const unsigned v = __builtin_amdgcn_perm(b, a, (j & 1) ? sel_hi : sel_lo);
                    const int row = e_q * 8 + j;
                    *reinterpret_cast<unsigned *>(Bb + row * SB_LD + ((((e_o >> 2) ^ softmap_swz(row)) << 2) | (e_o & 3)) * 4) = v;
                }
            }
        } else {
            const int row = (tid & 63) + 64 * p;
            *reinterpret_cast<uint4 *>(Bb + row * SB_LD + (((tid >> 6) ^ softmap_swz(row)) << 4)) =
                make_uint4(pe[p].x, pe[p].y, pe[p].z, pe[p].w);
        }
    };
    // pieces handled after the first (h = 0) and the second (h = 1) half of a stage's MFMAs
    // (the two rows of a MODE 1 pair travel together in the second half: they are packed in one go)
    auto fetch_half = [&](int h, int k0) __attribute__((always_inline)) {
        fetch_a(h, k0);
        if (MODE != 1) fetch_b(h, k0);
        else if (h == 1) { fetch_b(0, k0); fetch_b(1, k0); }
    };
    auto commit_half = [&](int h, int buf) __attribute__((always_inline)) {
        commit_a(h, buf);
        if (MODE != 1) commit_b(h, buf);
        else if (h == 1) commit_b(1, buf);
    };

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    const int nst = (k_end - k_begin + KC - 1) / KC;
    if (nst > 0) {
        fetch_half(0, k_begin); fetch_half(1, k_begin);
        commit_half(0, 0); commit_half(1, 0);
        if (nst > 1) { fetch_half(0, k_begin + KC); fetch_half(1, k_begin + KC); }
    }
    __syncthreads();
    const int kh = lane >> 5, l32 = lane & 31;
    auto stage = [&](int s, auto do_commit, auto do_fetch) __attribute__((always_inline)) {
        const int cur = s & 1;
        const char *Ab = As + cur * STAGE + (wm + l32) * SB_LD;
        const char *Bb = Bs + cur * STAGE + (wn + l32) * SB_LD;
        // k-block kh + 2 kk of my rows, at its swizzled position; rows 32 apart differ in the swizzle by 2
        const int swa = softmap_swz(wm + l32), swb = softmap_swz(wn + l32);
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            const int blk = kh + 2 * kk;
            const bf16x8 a0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(Ab + ((blk ^ swa) << 4)));
            const bf16x8 a1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(Ab + 32 * SB_LD + ((blk ^ swa ^ 2) << 4)));
            const bf16x8 b0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(Bb + ((blk ^ swb) << 4)));
            const bf16x8 b1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(Bb + 32 * SB_LD + ((blk ^ swb ^ 2) << 4)));
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b1, acc[1][1], 0, 0, 0);
            if constexpr (decltype(do_commit)::value) commit_half(kk, cur ^ 1);
            if constexpr (decltype(do_fetch)::value) fetch_half(kk, k_begin + (s + 2) * KC);
        }
        __syncthreads();
    };
    {
        using T = std::true_type;
        using F = std::false_type;
        int s = 0;
        for (; s + 2 < nst; ++s) stage(s, T{}, T{});
        if (s + 1 < nst) { stage(s, T{}, F{}); ++s; }
        if (s < nst) stage(s, F{}, F{});
    }
    float *dst = g.out + (size_t)zc * R * C;
    if (MODE == 2) {
        float *rowst = reinterpret_cast<float *>(lds);  // per tile row {1/sum, r}
        if (tid < SM_T) {
            const int row = min(r0 + tid, R - 1);
            rowst[tid * 2] = rs[row];
            rowst[tid * 2 + 1] = g.r[row];
        }
        __syncthreads();
        if (!EDGE) {
            // Interior tiles: a wavefront's 64 x 64 block of G goes through LDS 32 rows at a time, so that
            // a lane owns four consecutive columns of a row: 8-byte loads of the numerators, 16-byte stores of
            // gW in runs of 256 bytes per row (the accumulator layout itself gives 2-byte loads and 4-byte
            // stores in runs of 128).  Each wavefront uses its own LDS region; no block barrier is needed.
            constexpr int TS = 68;  // floats per staged row: 64 + 4, keeps 16-byte alignment
            float *stg = reinterpret_cast<float *>(lds) + 2 * SM_T + wave * (32 * TS);
            const int rr = lane >> 4, c4 = (lane & 15) * 4;
#pragma clang loop unroll(disable)
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const floatx16 a = i == 0 ? (j == 0 ? acc[0][0] : acc[0][1]) : (j == 0 ? acc[1][0] : acc[1][1]);
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        stg[(8 * (v >> 2) + 4 * (lane >> 5) + (v & 3)) * TS + j * 32 + (lane & 31)] = a[v];
                }
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int it = 0; it < 8; ++it) {
                    const int lr = wm + i * 32 + it * 4 + rr;
                    const size_t at = (size_t)(r0 + lr) * I + c0 + wn + c4;
                    const float4 gv = *reinterpret_cast<const float4 *>(stg + (it * 4 + rr) * TS + c4);
                    const uint2 e = *reinterpret_cast<const uint2 *>(Eb + at);
                    const float f = rowst[lr * 2] * g.inv_tau, rv = rowst[lr * 2 + 1];
                    float4 o;
                    o.x = __uint_as_float(e.x << 16) * f * (gv.x - rv);
                    o.y = __uint_as_float(e.x & 0xffff0000u) * f * (gv.y - rv);
                    o.z = __uint_as_float(e.y << 16) * f * (gv.z - rv);
                    o.w = __uint_as_float(e.y & 0xffff0000u) * f * (gv.w - rv);
                    *reinterpret_cast<float4 *>(dst + at) = o;
                }
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
        } else {
        // rolled on purpose (see the fp32 kernel): gW = S (G - r) / tau with S = E / sum
#pragma clang loop unroll(disable)
        for (int ij = 0; ij < 4; ++ij) {
            const int i = ij >> 1, j = ij & 1;
            const floatx16 a = ij == 0 ? acc[0][0] : ij == 1 ? acc[0][1] : ij == 2 ? acc[1][0] : acc[1][1];
            const int col = c0 + wn + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int lr = wm + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                const int row = r0 + lr;
                if (row < R && col < C) {
                    const float sv = softmap_bf16_f32(Eb[(size_t)row * I + col]) * rowst[lr * 2];
                    dst[(size_t)row * C + col] = sv * (a[v] - rowst[lr * 2 + 1]) * g.inv_tau;
                }
            }
        }
        }
    } else {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int col = c0 + wn + j * 32 + (lane & 31);
                const float f = MODE == 0 ? rs[min(col, C - 1)] : 1.0f;  // forward: columns are rows of W
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = r0 + wm + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                    if (!EDGE || (row < R && col < C)) dst[(size_t)row * C + col] = acc[i][j][v] * f;
                }
            }
    }
}

template <int MODE>
__global__ __launch_bounds__(256, 3) void softmap_mfma_bf16(SoftmapArgs g) {
    __shared__ __align__(16) char lds[MODE == 2 ? (2 * SM_T + 4 * 32 * 68) * 4 : 4 * SM_T * SB_LD];  // gW: its epilogue's staging
    int inner, outer;
    if (!dl_xcd_map(g.inner_count, g.outer_count, inner, outer)) return;
    const int rt = MODE == 2 ? outer : inner;
    const int ct = MODE == 2 ? inner : (MODE == 1 ? outer % g.col_tiles : outer);
    const int zc = MODE == 1 ? outer / g.col_tiles : 0;
    const int R = MODE == 2 ? g.M : g.B, C = MODE == 0 ? g.M : g.I;
    const int KD = MODE == 0 ? g.I : (MODE == 1 ? g.M : g.B);
    const int k_begin = zc * g.red_chunk, k_end = min(KD, k_begin + g.red_chunk);
    // whole tiles and stages, and rows of the bf16 operands that start on 16-byte boundaries
    const bool inside = (rt + 1) * SM_T <= R && (ct + 1) * SM_T <= C && (k_end - k_begin) % SB_K == 0 &&
                        g.red_chunk % 8 == 0 && g.I % 8 == 0 && g.M % 8 == 0;
    if (inside) softmap_tile_bf16<MODE, false>(g, lds, rt, ct, zc);
    else softmap_tile_bf16<MODE, true>(g, lds, rt, ct, zc);
}

template <int MODE>
static void softmap_launch_bf16(const SoftmapArgs &g, hipStream_t s) {
    softmap_mfma_bf16<MODE><<<dl_xcd_grid(g.inner_count, g.outer_count), 256, 0, s>>>(g);
}

// ---------------------------------------------------------------------------------
static int softmap_check(int B, int I, int M, int precision) {
    if (B <= 0 || I <= 0 || M <= 0) return DL_ERR_SHAPE;
    if (precision != 0 && precision != 1) return DL_ERR_UNSUPPORTED;
    return DL_OK;
}

// The gx product reduces over M.  It is cut into chunks, one block per (output tile, chunk), about
// 4096 blocks in all: measured on the 512 x 3136 x 48000 case the kernel keeps getting faster down
// to chunks of about 1000 (short blocks keep the gm and W slabs of the blocks resident on an XCD
// within its L2), while the fixed-order reduction of the partial products costs 2 us per chunk.
static inline int softmap_gx_chunks(int B, int I, int M, int precision) {
    (void)precision;
    const long long tiles = (long long)dl_ceil_div(I, SM_T) * dl_ceil_div(B, SM_T);
    int chunks = dl_ceil_div(4096, tiles);
    const int max_chunks = dl_ceil_div(M, 256);
    if (chunks > max_chunks) chunks = max_chunks;
    return chunks < 1 ? 1 : chunks;
}

// what the forward leaves for the backward in `stats`: fp32 operands: {max, 1/sum} per row of W;
// bf16 operands: max[M], 1/sum[M] and the bf16 softmax numerators [M][I]
static inline size_t softmap_stats_bytes(int M) { return dl_align256((size_t)2 * M * sizeof(float)); }
extern "C" size_t dl_soft_map_saved_bytes(int B, int I, int M, int precision) {
    (void)B;
    if (I <= 0 || M <= 0) return 256;
    return softmap_stats_bytes(M) + (precision == 1 ? dl_align256((size_t)M * I * sizeof(unsigned short)) : 0);
}

// workspace: r [M], the partial gx products, and for bf16 operands the packed copies of x and gm
static inline size_t softmap_r_bytes(int M) { return dl_align256((size_t)M * sizeof(float)); }
static inline size_t softmap_part_bytes(int B, int I, int M, int precision) {
    return dl_align256((size_t)softmap_gx_chunks(B, I, M, precision) * B * I * sizeof(float));
}
static inline size_t softmap_rows_bytes(int R, int C) { return dl_align256((size_t)R * C * sizeof(unsigned short)); }
static inline size_t softmap_blocks_bytes(int R, int C) { return dl_align256((size_t)((R + 7) / 8) * C * sizeof(uint4)); }
extern "C" size_t dl_soft_map_workspace_bytes(int B, int I, int M, int precision) {
    if (B <= 0 || I <= 0 || M <= 0) return 256;
    size_t bytes = softmap_r_bytes(M) + softmap_part_bytes(B, I, M, precision);
    if (precision == 1)
        bytes += softmap_rows_bytes(B, I) + softmap_blocks_bytes(B, I) + softmap_rows_bytes(B, M) + softmap_blocks_bytes(B, M);
    return bytes;
}
static void softmap_pack(const float *src, const float *colscale, unsigned short *rows, uint4 *blocks, int R, int C,
                         hipStream_t s) {
    const long long total = (long long)((R + 7) / 8) * C;
    DL_TIMED("softmap_pack_bf16", s,
             (softmap_pack_bf16<<<dl_ceil_div(total, 256), 256, 0, s>>>(src, colscale, rows, blocks, R, C)));
}

// rows that fit a wavefront's registers are read once; longer or unaligned rows take the two-sweep kernels
template <bool BF16>
static void softmap_stats_launch(const float *W, float scale, float *a, float *b, unsigned short *Eb, int M, int I,
                                 hipStream_t s) {
    const int grid = dl_ceil_div(M, 4), n4 = I >> 2;
    const bool regs = I % 4 == 0 && n4 <= 1024 && ((uintptr_t)W & 15) == 0;
    const char *name = BF16 ? "softmap_rowstats_bf16" : "softmap_rowstats";
    if (regs && n4 <= 256) DL_TIMED(name, s, (softmap_rowstats_regs<4, BF16><<<grid, 256, 0, s>>>(W, scale, a, b, Eb, M, I)));
    else if (regs && n4 <= 512) DL_TIMED(name, s, (softmap_rowstats_regs<8, BF16><<<grid, 256, 0, s>>>(W, scale, a, b, Eb, M, I)));
    else if (regs) DL_TIMED(name, s, (softmap_rowstats_regs<16, BF16><<<grid, 256, 0, s>>>(W, scale, a, b, Eb, M, I)));
    else if (BF16) DL_TIMED(name, s, (softmap_rowstats_bf16<<<grid, 256, 0, s>>>(W, scale, a, b, Eb, M, I)));
    else DL_TIMED(name, s, (softmap_rowstats<<<grid, 256, 0, s>>>(W, scale, a, M, I)));
}

extern "C" int dl_soft_map_fwd(const float *x, const float *W, float tau, float *m, float *stats, void *ws,
                               size_t ws_bytes, int B, int I, int M, int precision, void *stream) {
    if (!x || !W || !m || !stats) return DL_ERR_NULL;
    int rc = softmap_check(B, I, M, precision);
    if (rc) return rc;
    if (!(tau > 0.0f)) return DL_ERR_SHAPE;
    if (precision == 1 && !ws) return DL_ERR_NULL;
    if (precision == 1 && ws_bytes < dl_soft_map_workspace_bytes(B, I, M, precision)) return DL_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    const float inv_tau = 1.0f / tau, scale = SM_LOG2E / tau;
    SoftmapArgs g{x, W, stats, nullptr, nullptr, scale, inv_tau, m, B, I, M,
                  dl_ceil_div(B, SM_T), dl_ceil_div(M, SM_T), 1, dl_ceil_div(I, 8) * 8, nullptr, nullptr,
                  nullptr, nullptr, nullptr, nullptr};
    if (precision == 1) {
        unsigned short *Eb = (unsigned short *)((char *)stats + softmap_stats_bytes(M));
        softmap_stats_launch<true>(W, scale, stats, stats + M, Eb, M, I, s);
        unsigned short *xb = (unsigned short *)((char *)ws + softmap_r_bytes(M) + softmap_part_bytes(B, I, M, precision));
        softmap_pack(x, nullptr, xb, nullptr, B, I, s);
        g.xb = xb;
        g.Eb = Eb;
        g.rs = stats + M;
        DL_TIMED("softmap_bf16_fwd", s, (softmap_launch_bf16<0>(g, s)));
    } else {
        softmap_stats_launch<false>(W, scale, stats, nullptr, nullptr, M, I, s);
        DL_TIMED("softmap_mfma_fwd", s, (softmap_launch<0, SM_K>(g, s)));
    }
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
    const float inv_tau = 1.0f / tau, scale = SM_LOG2E / tau;
    float *r = (float *)ws;
    float *part = (float *)((char *)ws + softmap_r_bytes(M));
    const int chunks = softmap_gx_chunks(B, I, M, precision);
    int red_chunk = dl_ceil_div(M, chunks);
    red_chunk = dl_ceil_div(red_chunk, 32) * 32;  // whole stages, so float4 loads stay aligned
    const int col_tiles = dl_ceil_div(I, SM_T), used_chunks = dl_ceil_div(M, red_chunk);
    const unsigned short *Eb = precision == 1 ? (const unsigned short *)((const char *)stats + softmap_stats_bytes(M)) : nullptr;
    const float *rs = precision == 1 ? stats + M : nullptr;
    DL_TIMED("softmap_rowdot", s, (softmap_rowdot<<<dl_ceil_div(M, 32), 256, 0, s>>>(gm, m, r, B, M)));
    uint4 *x8 = nullptr, *gm8 = nullptr;
    unsigned short *gms = nullptr;
    if (precision == 1) {
        char *w = (char *)ws + softmap_r_bytes(M) + softmap_part_bytes(B, I, M, precision) + softmap_rows_bytes(B, I);
        x8 = (uint4 *)w; w += softmap_blocks_bytes(B, I);
        gms = (unsigned short *)w; w += softmap_rows_bytes(B, M);
        gm8 = (uint4 *)w;
        softmap_pack(x, nullptr, nullptr, x8, B, I, s);
        softmap_pack(gm, rs, gms, gm8, B, M, s);
    }
    const SoftmapArgs ggx{x, W, stats, gm, nullptr, scale, inv_tau, used_chunks > 1 ? part : gx, B, I, M,
                          dl_ceil_div(B, SM_T), col_tiles * used_chunks, col_tiles, red_chunk, Eb, rs,
                          nullptr, x8, gms, gm8};
    if (precision == 1) DL_TIMED("softmap_bf16_gx", s, (softmap_launch_bf16<1>(ggx, s)));
    else DL_TIMED("softmap_mfma_gx", s, (softmap_launch<1, SM_K>(ggx, s)));
    if (used_chunks > 1) {
        const long long total = (long long)B * I;
        if (total % 4 == 0 && ((uintptr_t)gx & 15) == 0)
            DL_TIMED("softmap_reduce_chunks", s,
                     (softmap_reduce_chunks<4><<<dl_ceil_div(total / 4, 256), 256, 0, s>>>(part, gx, total, used_chunks)));
        else
            DL_TIMED("softmap_reduce_chunks", s,
                     (softmap_reduce_chunks<1><<<dl_ceil_div(total, 256), 256, 0, s>>>(part, gx, total, used_chunks)));
    }
    const SoftmapArgs ggw{x, W, stats, gm, r, scale, inv_tau, gW, B, I, M,
                          col_tiles, dl_ceil_div(M, SM_T), 1, dl_ceil_div(B, 8) * 8, Eb, rs,
                          nullptr, x8, gms, gm8};
    if (precision == 1) DL_TIMED("softmap_bf16_gw", s, (softmap_launch_bf16<2>(ggw, s)));
    else DL_TIMED("softmap_mfma_gw", s, (softmap_launch<2, SM_K>(ggw, s)));
    return dl_launch_status();
}
