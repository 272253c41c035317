// RandomLayer + Probabilistic nodes on gfx950.
//   y[b,n,d] = sum_a sigmoid(w[n,a,d]/T) * prod_j (x_j a_j + (1-x_j)(1-a_j)),  x_j = x[b, idx[n,j]]
// i.e. the multilinear interpolation of the node's sigmoid table at the point x.
//
// k <= 6: tiled kernels with lanes = batch rows (see below); k > 6: one-thread-per-element kernels
// with atomics.
#include "dl_common.h"

__device__ __forceinline__ float dl_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }

typedef float prob_f4 __attribute__((ext_vector_type(4)));
#define PROB_RSRC 0x00020000
#define PROB_HYBRID_EPS 1e-8f

// ---------------------------------------------------------------------------------
// k <= 6 path.  As for the DWN nodes, a wavefront's 64 lanes are 64 batch rows and everything
// that belongs to a node is wave-uniform: its input indices are scalar byte offsets, its sigmoid
// table is read through scalar loads.  Tensors that cross the [batch, feature] boundary are
// re-tiled once: xT [B/64][I][64], gyT [B/64][N*O][64], gmT [B/64][N*O*k][64], so the row of an
// input (or a column's gradient) for a batch tile is 256 contiguous bytes, whatever the mapping.
//   sig_table   : sig[c][a] = sigmoid(raw[n,a,d] / T), c = n*O + d                (tiny)
//   to_tiles    : [B][C] -> [B/64][C][64], rows past B are zero        (x; gy only for k > 5, see bwd_t)
//   fwd_t       : per (column, batch tile): fold the table along x_0, x_1, ... ; y leaves through
//                 an LDS transpose as whole rows
//   bwd_t       : one wavefront per column over a chunk of batch tiles.  The fold is run forward
//                 keeping the differences of every level, then backward: that gives dy/dx_j for
//                 all j and, at the bottom, p_a = dy/dtable_a (the product weights) in about
//                 5 * 2^k operations.  Table-gradient partials stay in registers over the chunk,
//                 are summed across lanes once and written per chunk; gm_j goes to gmT.
//   reduce      : fixed-order sum of the chunk partials, times sigmoid'(w/T)/T
//   gather_t    : gx[b,i] = sum over the CSR entries (n,j) of input i (and d) of gmT: a wavefront
//                 owns 16 inputs, sums each in CSR order in a register, rows leave through LDS.
// The temperature of the layer: one value (inv = 1 / max(T, 1e-6)) or every node's own (t_n, a device array [N],
// probabilistic_node.py:277-282 reads each node's buffer).
struct ProbTemp {
    float inv;
    const float *t_n;
};
__device__ __forceinline__ float prob_inv_t_of(const ProbTemp &T, int n) {
    if (!T.t_n) return T.inv;
    const float t = T.t_n[n];
    return 1.0f / (t > 1e-6f ? t : 1e-6f);
}
__global__ __launch_bounds__(256) void prob_sig_table(const float *__restrict__ raw, ProbTemp T, float *__restrict__ sig,
                                                       int N, int L, int O) {
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    if (e >= (long long)N * L * O) return;
    const int a = (int)(e % L);
    const long long c = e / L;
    const int n = (int)(c / O), d = (int)(c % O);
    sig[e] = dl_sigmoid(raw[((size_t)n * L + a) * O + d] * prob_inv_t_of(T, n));
}

// grid (ceil(C / 64), B/64 rounded up), 256 threads.  With `sig` set the launch carries extra rows of blocks
// (blockIdx.y >= tiles) that build the sigmoid table in the same launch: the two jobs are independent and each is
// too short to fill the machine on its own.
__global__ __launch_bounds__(256) void prob_to_tiles(const float *__restrict__ src, float *__restrict__ dst, int B, int C,
                                                      int tiles = 1 << 30, const float *__restrict__ raw = nullptr,
                                                      ProbTemp T = {1.0f, nullptr}, float *__restrict__ sig = nullptr,
                                                      int N = 0, int L = 1, int O = 1) {
    __shared__ float tile[64][65];  // [column][row]
    if ((int)blockIdx.y >= tiles) {
        const long long e = ((long long)(blockIdx.y - tiles) * gridDim.x + blockIdx.x) * 256 + threadIdx.x;
        if (e < (long long)N * L * O) {
            const int a = (int)(e % L);
            const long long c = e / L;
            const int n = (int)(c / O), d = (int)(c % O);
            sig[e] = dl_sigmoid(raw[((size_t)n * L + a) * O + d] * prob_inv_t_of(T, n));
        }
        return;
    }
    const int t = blockIdx.y, c0 = blockIdx.x * 64;
    if ((C & 3) == 0 && c0 + 64 <= C && (((uintptr_t)src) & 15) == 0) {
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const int e = pass * 256 + threadIdx.x;
            const int r = e >> 4, c = (e & 15) * 4;
            const int b = t * 64 + r;
            prob_f4 v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (b < B) v = *reinterpret_cast<const prob_f4 *>(src + (size_t)b * C + c0 + c);
            tile[c][r] = v.x; tile[c + 1][r] = v.y; tile[c + 2][r] = v.z; tile[c + 3][r] = v.w;
        }
    } else {
        for (int e = threadIdx.x; e < 4096; e += 256) {
            const int r = e >> 6, c = e & 63;
            const int b = t * 64 + r;
            tile[c][r] = (b < B && c0 + c < C) ? src[(size_t)b * C + c0 + c] : 0.0f;
        }
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int e = pass * 256 + threadIdx.x;
        const int c = e >> 4, r = (e & 15) * 4;
        const prob_f4 v = {tile[c][r], tile[c][r + 1], tile[c][r + 2], tile[c][r + 3]};
        if (c0 + c < C) *reinterpret_cast<prob_f4 *>(dst + ((size_t)t * C + c0 + c) * 64 + r) = v;
    }
}

// table of one column as wave-uniform values
template <int K>
__device__ __forceinline__ void prob_load_table(const float *__restrict__ sig, int c, float (&tab)[1 << K]) {
    const float *row = sig + (size_t)c * (1 << K);
#pragma unroll
    for (int a = 0; a < (1 << K); ++a) tab[a] = row[a];
}

#define PROB_TC 128                    // columns per block
#define PROB_FW 8                      // wavefronts per block
#define PROB_WC (PROB_TC / PROB_FW)    // columns per wavefront
template <int K>
__global__ __launch_bounds__(64 * PROB_FW) void prob_fwd_t(const float *__restrict__ xT, const int *__restrict__ idx32,
                                                            const float *__restrict__ sig, float *__restrict__ y,
                                                            int B, int I, int N, int O, int BT) {
    __shared__ float tile[PROB_TC][65];  // [column][row]
    constexpr int L = 1 << K;
    const int NO = N * O;
    int ctile, t;
    if (!dl_xcd_map((NO + PROB_TC - 1) / PROB_TC, BT, ctile, t)) return;
    const int c0 = ctile * PROB_TC;
    const int lane = threadIdx.x & 63;
    const int wave = dl_uniform(threadIdx.x >> 6);
    const int cend = min(PROB_TC, NO - c0);
    const int wbeg = wave * PROB_WC;
    const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc((void *)(xT + (size_t)t * I * 64), 0, I * 256, PROB_RSRC);
    const int lane4 = lane * 4;
    // slot s = (column within my 16) * K + j  ->  lane s % 64 of register s / 64: byte offset of the input's row
    constexpr int NIDX = (PROB_WC * K + 63) / 64;
    int myoff[NIDX];
#pragma unroll
    for (int v = 0; v < NIDX; ++v) {
        const int s = v * 64 + lane;
        const int c = min(c0 + wbeg + min(s / K, PROB_WC - 1), NO - 1);
        myoff[v] = idx32[(size_t)(c / O) * K + s % K] * 256;
    }
    constexpr int CG = 4;  // columns whose input rows are requested together
#pragma unroll
    for (int g = 0; g < PROB_WC; g += CG) {
        if (wbeg + g >= cend) break;  // wave-uniform
        float xs[CG][K];
#pragma unroll
        for (int q = 0; q < CG; ++q)
#pragma unroll
            for (int j = 0; j < K; ++j) {
                const int s = (g + q) * K + j;  // compile-time after unrolling
                const int off = __builtin_amdgcn_readlane(myoff[s / 64], s % 64);
                xs[q][j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs_x, lane4, off, 0));
            }
#pragma unroll
        for (int q = 0; q < CG; ++q) {
            const int cc = wbeg + g + q;
            if (cc >= cend) break;  // wave-uniform
            float tab[L];
            prob_load_table<K>(sig, c0 + cc, tab);
            float v[L / 2 > 0 ? L / 2 : 1];
            {
                const float om = 1.0f - xs[q][0];
#pragma unroll
                for (int a = 0; a < L / 2; ++a) v[a] = fmaf(tab[2 * a + 1], xs[q][0], tab[2 * a] * om);
            }
#pragma unroll
            for (int j = 1; j < K; ++j) {
#pragma unroll
                for (int a = 0; a < (L >> (j + 1)); ++a) v[a] = v[2 * a] + xs[q][j] * (v[2 * a + 1] - v[2 * a]);
            }
            tile[cc][lane] = v[0];
        }
    }
    __syncthreads();
    if (cend == PROB_TC && t * 64 + 64 <= B && (NO & 3) == 0 && (((uintptr_t)y) & 15) == 0) {  // whole tile: 16-byte stores
#pragma unroll
        for (int pass = 0; pass < 64 * PROB_TC / 4 / (64 * PROB_FW); ++pass) {
            const int e = pass * 64 * PROB_FW + threadIdx.x;
            const int r = e / (PROB_TC / 4), c4 = (e % (PROB_TC / 4)) * 4;
            const prob_f4 v = {tile[c4][r], tile[c4 + 1][r], tile[c4 + 2][r], tile[c4 + 3][r]};
            __builtin_nontemporal_store(v, reinterpret_cast<prob_f4 *>(&y[(size_t)(t * 64 + r) * NO + c0 + c4]));
        }
        return;
    }
    for (int e = threadIdx.x; e < 64 * PROB_TC; e += 64 * PROB_FW) {
        const int r = e / PROB_TC, cc = e % PROB_TC;
        const int b = t * 64 + r;
        if (b < B && cc < cend) __builtin_nontemporal_store(tile[cc][r], &y[(size_t)b * NO + c0 + cc]);
    }
}

// one wavefront per (column, chunk of batch tiles); W wavefronts per block.
// HYB (hybrid node): the table is used as given and the input gradient carries the factor
// q / (q + 1e-8), q = x_j (1 - x_j), of that node's backward.
// W = 4: gy arrives tile-major (gyT [B/64][N*O][64], written by prob_to_tiles).  W = 16 (k <= 5, where 16 wavefronts
// of this kernel fit a CU's registers): gy is the row-major gradient itself; the block's 16 columns are 64 contiguous
// bytes of a row, the 64 x 16 piece of a batch tile is fetched one value per thread a tile ahead and turned through
// the LDS (two buffers, one barrier per tile), so the re-tiling pass and its launch are not needed.
template <int K, bool HYB, int W = 4>
__global__ __launch_bounds__(64 * W) void prob_bwd_t(const float *__restrict__ xT, const float *__restrict__ gyT,
                                                     const int *__restrict__ idx32, const float *__restrict__ sig,
                                                     float *__restrict__ gmT, float *__restrict__ gpart, int I, int N,
                                                     int O, int BT, int tiles_per_chunk, int want_gm, int B = 0) {
    constexpr int L = 1 << K;
    constexpr bool GYROW = W == 16;
    __shared__ float gturn[GYROW ? 2 : 1][GYROW ? W : 1][GYROW ? 65 : 1];  // [buffer][column][row]
    const int NO = N * O;
    const int lane = threadIdx.x & 63;
    const int c_raw = blockIdx.x * W + dl_uniform(threadIdx.x >> 6);
    if (!GYROW && c_raw >= NO) return;
    const bool live = c_raw < NO;        // GYROW: wavefronts past the last column still serve the barriers
    const int c = live ? c_raw : NO - 1;
    const int chunk = blockIdx.y;
    const int n = c / O;
    const int lane4 = lane * 4;
    int off[K];
#pragma unroll
    for (int j = 0; j < K; ++j) off[j] = idx32[(size_t)n * K + j] * 256;
    float tab[L];
    prob_load_table<K>(sig, c, tab);
    float acc[L];
#pragma unroll
    for (int a = 0; a < L; ++a) acc[a] = 0.0f;
    const int t0 = chunk * tiles_per_chunk, t1 = min(BT, t0 + tiles_per_chunk);
    float nxs[K], ng = 0.0f;  // operands of the next batch tile, requested one tile ahead
    const int trow = threadIdx.x >> 4, tcol = threadIdx.x & 15;  // GYROW: my value of the 64 x 16 piece
    auto request = [&](int t) {
        const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc((void *)(xT + (size_t)t * I * 64), 0, I * 256, PROB_RSRC);
#pragma unroll
        for (int j = 0; j < K; ++j) nxs[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs_x, lane4, off[j], 0));
        if (GYROW) {
            const int b = t * 64 + trow, cc = blockIdx.x * W + tcol;
            ng = (b < B && cc < NO) ? gyT[(size_t)b * NO + cc] : 0.0f;
        } else {
            ng = gyT[((size_t)t * NO + c) * 64 + lane];
        }
    };
    if (t0 < t1) request(t0);
    for (int t = t0; t < t1; ++t) {
        float xs[K];
#pragma unroll
        for (int j = 0; j < K; ++j) xs[j] = nxs[j];
        float g = ng;
        if (GYROW) {
            const int buf = (t - t0) & 1;
            gturn[buf][tcol][trow] = ng;
            __syncthreads();  // the other buffer is rewritten only after the next barrier: its readers are done by then
            g = gturn[buf][threadIdx.x >> 6][lane];
        }
        if (t + 1 < t1) request(t + 1);
        // forward fold, keeping the differences d_j[a] = lvl_j[2a+1] - lvl_j[2a] of every level
        float diff[L > 1 ? L - 1 : 1];  // level j occupies [L - (L >> j), L - (L >> (j+1)))
        float v[L / 2 > 0 ? L / 2 : 1];
#pragma unroll
        for (int a = 0; a < L / 2; ++a) {
            diff[a] = tab[2 * a + 1] - tab[2 * a];
            v[a] = fmaf(xs[0], diff[a], tab[2 * a]);
        }
        int base = L / 2;
#pragma unroll
        for (int j = 1; j < K; ++j) {
#pragma unroll
            for (int a = 0; a < (L >> (j + 1)); ++a) {
                diff[base + a] = v[2 * a + 1] - v[2 * a];
                v[a] = fmaf(xs[j], diff[base + a], v[2 * a]);
            }
            base += L >> (j + 1);
        }
        // backward: bar_K[0] = 1; dx_j = sum_a bar_{j+1}[a] d_j[a]; bar_j[2a] = bar_{j+1}[a] (1 - x_j), bar_j[2a+1] = bar_{j+1}[a] x_j
        float bar[L];
        bar[0] = 1.0f;
        float dx[K];
#pragma unroll
        for (int j = K - 1; j >= 0; --j) {
            base -= L >> (j + 1);
            const int cnt = L >> (j + 1);
            float sum = 0.0f;
#pragma unroll
            for (int a = 0; a < cnt; ++a) sum = fmaf(bar[a], diff[base + a], sum);
            const float om = 1.0f - xs[j];
            if (HYB) {
                const float q = xs[j] * om;
                sum = sum * q / (q + PROB_HYBRID_EPS);
            }
            dx[j] = sum;
#pragma unroll
            for (int a = cnt - 1; a >= 0; --a) {
                const float w = bar[a];
                bar[2 * a + 1] = w * xs[j];
                bar[2 * a] = w * om;
            }
        }
#pragma unroll
        for (int a = 0; a < L; ++a) acc[a] = fmaf(g, bar[a], acc[a]);
        if (want_gm && live) {
#pragma unroll
            for (int j = 0; j < K; ++j) gmT[(((size_t)t * NO + c) * K + j) * 64 + lane] = g * dx[j];
        }
    }
    // Sum the 64 per-row partials of every table entry with L - 1 + (6 - K) exchanges instead of 6 L:
    // round r pairs the entries (2i, 2i+1); the half of the wavefront with lane bit (5 - r) set keeps
    // the odd one and hands over the even one, so after K rounds a lane holds one entry,
    // a = sum_r ((lane >> (5 - r)) & 1) << r, summed over the lanes that differ in the top K bits.
#pragma unroll
    for (int r = 0; r < K; ++r) {
        const int width = 32 >> r;
        const bool upper = (lane & width) != 0;
#pragma unroll
        for (int i = 0; i < (L >> (r + 1)); ++i) {
            const float keep = upper ? acc[2 * i + 1] : acc[2 * i];
            const float send = upper ? acc[2 * i] : acc[2 * i + 1];
            acc[i] = keep + __shfl_xor(send, width);
        }
    }
    float mine = acc[0];
#pragma unroll
    for (int width = 32 >> K; width > 0; width >>= 1) mine += __shfl_xor(mine, width);
    int a = 0;
#pragma unroll
    for (int r = 0; r < K; ++r) a |= ((lane >> (5 - r)) & 1) << r;
    if (live && (lane & ((64 >> K) - 1)) == 0) gpart[((size_t)chunk * NO + c) * L + a] = mine;
}

// graw[n,a,d] = sigmoid'(w/T)/T * sum over chunks of gpart[chunk][c][a];
// sig == null (hybrid node): the plain sum, kept in the table's own layout [c][a]
struct ProbReduce {  // the table-gradient reduction, also carried as extra blocks of the gather launch
    const float *gpart, *sig;
    ProbTemp T;
    float *graw;
    int N, L, O, chunks;
};
__device__ __forceinline__ void prob_reduce_element(const ProbReduce &R, long long e);
__global__ __launch_bounds__(256) void prob_reduce_weights(ProbReduce R) {
    prob_reduce_element(R, (long long)blockIdx.x * 256 + threadIdx.x);
}
__device__ __forceinline__ void prob_reduce_element(const ProbReduce &R, long long e) {
    const float *gpart = R.gpart, *sig = R.sig;
    float *graw = R.graw;
    const int N = R.N, L = R.L, O = R.O, chunks = R.chunks;
    const long long total = (long long)N * L * O;
    if (e >= total) return;
    float acc = 0.0f;
    for (int ch = 0; ch < chunks; ++ch) acc += gpart[(size_t)ch * total + e];
    if (!sig) {
        graw[e] = acc;
        return;
    }
    const int a = (int)(e % L);
    const long long c = e / L;
    const int n = (int)(c / O), d = (int)(c % O);
    const float s = sig[e];
    graw[((size_t)n * L + a) * O + d] = acc * s * (1.0f - s) * prob_inv_t_of(R.T, n);
}

#define PROB_IS 64  // inputs per block of the gather
#define PROB_WI 16  // inputs per wavefront
#define PROB_EG 8   // entries requested together
// FAST (one output per node): the CSR entries of a wavefront's 16 inputs are held one per lane
// (row offset, local input) and replayed eight at a time with buffer loads whose offset travels
// in an SGPR, the next eight requested before the current ones are summed.
template <bool FAST>
__global__ __launch_bounds__(256) void prob_gather_t(const float *__restrict__ gmT, const int *__restrict__ inv_ptr,
                                                      const int *__restrict__ inv_pos, float *__restrict__ gx, int B,
                                                      int I, int N, int K, int O, int BT, int gather_blocks, ProbReduce R) {
    __shared__ float tile[PROB_IS][65];  // [input][row]
    if ((int)blockIdx.x >= gather_blocks) {  // the blocks appended for the independent table-gradient reduction
        prob_reduce_element(R, (long long)(blockIdx.x - gather_blocks) * 256 + threadIdx.x);
        return;
    }
    int slab, t;
    if (!dl_xcd_map((I + PROB_IS - 1) / PROB_IS, BT, slab, t)) return;
    const int i0 = slab * PROB_IS;
    const int lane = threadIdx.x & 63;
    const int wave = dl_uniform(threadIdx.x >> 6);
    const int iend = min(PROB_IS, I - i0);
    const int wbeg = wave * PROB_WI;
    if (FAST) {
        const __amdgpu_buffer_rsrc_t rs =
            __builtin_amdgcn_make_buffer_rsrc((void *)(gmT + (size_t)t * N * K * 64), 0, N * K * 256, PROB_RSRC);
        const int lane4 = lane * 4;
        const int myptr = inv_ptr[min(i0 + wbeg + min(lane, PROB_WI), I)];
#pragma unroll
        for (int r = 0; r < PROB_WI; ++r) tile[wbeg + r][lane] = 0.0f;  // inputs nobody reads keep 0
        const int ebeg = __builtin_amdgcn_readlane(myptr, 0);
        const int eend = __builtin_amdgcn_readlane(myptr, PROB_WI);
        float acc = 0.0f;
        int cur = -1;
        for (int base = ebeg; base < eend; base += 64) {
            const int e = base + lane;
            const bool valid = e < eend;
            const int p = valid ? inv_pos[e] : 0;
            int ii = 0;  // local input of entry e
#pragma unroll
            for (int l = 1; l <= PROB_WI; ++l) ii += (__builtin_amdgcn_readlane(myptr, l) <= e) ? 1 : 0;
            const int rec = valid ? ((p << 8) | ii) : 0;  // row offset p * 256 in the upper bits
            const int cnt = min(64, eend - base);
            struct Group { int r[PROB_EG]; float g[PROB_EG]; };
            auto request = [&](int s0, Group &G) {
#pragma unroll
                for (int q = 0; q < PROB_EG; ++q) {
                    const int r = __builtin_amdgcn_readlane(rec, s0 + q);
                    G.r[q] = r;
                    G.g[q] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, lane4, r & ~255, 0));
                }
            };
            auto sum_up = [&](const Group &G, int s0) {
#pragma unroll
                for (int q = 0; q < PROB_EG; ++q) {
                    if (s0 + q >= cnt) break;  // wave-uniform
                    const int ri = G.r[q] & 31;
                    if (ri != cur) {
                        if (cur >= 0) tile[wbeg + cur][lane] = acc;
                        acc = 0.0f;
                        cur = ri;
                    }
                    acc += G.g[q];
                }
            };
            const int m = (cnt + PROB_EG - 1) / PROB_EG;
            Group A, Bq;
            request(0, A);
            int gi = 0;
            for (; gi + 2 < m; gi += 2) {
                request((gi + 1) * PROB_EG, Bq);
                sum_up(A, gi * PROB_EG);
                request((gi + 2) * PROB_EG, A);
                sum_up(Bq, (gi + 1) * PROB_EG);
            }
            if (gi + 1 < m) {
                request((gi + 1) * PROB_EG, Bq);
                sum_up(A, gi * PROB_EG);
                sum_up(Bq, (gi + 1) * PROB_EG);
            } else {
                sum_up(A, gi * PROB_EG);
            }
        }
        if (cur >= 0) tile[wbeg + cur][lane] = acc;
    } else {
        const float *slabT = gmT + (size_t)t * N * O * K * 64 + lane;
        for (int r = 0; r < PROB_WI; ++r) {
            const int i = i0 + wbeg + r;
            float acc = 0.0f;
            if (i < I) {
                const int e0 = inv_ptr[i], e1 = inv_ptr[i + 1];  // wave-uniform
                for (int e = e0; e < e1; ++e) {
                    const int p = inv_pos[e];
                    const int n = p / K, j = p - n * K;
                    for (int d = 0; d < O; ++d) acc += slabT[(((size_t)n * O + d) * K + j) * 64];
                }
            }
            tile[wbeg + r][lane] = acc;
        }
    }
    __syncthreads();
    if (iend == PROB_IS && (I & 3) == 0 && ((uintptr_t)gx & 15) == 0) {
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const int e = pass * 256 + threadIdx.x;
            const int r = e / (PROB_IS / 4), i4 = (e % (PROB_IS / 4)) * 4;
            const int b = t * 64 + r;
            const prob_f4 v = {tile[i4][r], tile[i4 + 1][r], tile[i4 + 2][r], tile[i4 + 3][r]};
            if (b < B) *reinterpret_cast<prob_f4 *>(&gx[(size_t)b * I + i0 + i4]) = v;
        }
    } else {
        for (int e = threadIdx.x; e < 64 * PROB_IS; e += 256) {
            const int r = e / PROB_IS, ii = e % PROB_IS;
            const int b = t * 64 + r;
            if (b < B && ii < iend) gx[(size_t)b * I + i0 + ii] = tile[ii][r];
        }
    }
}

// the gather and the reduction of the table-gradient partials do not depend on each other: one launch, the
// reduction as extra blocks behind the gather's
static void prob_launch_gather_and_reduce(const float *gmT, const int *inv_ptr, const int *inv_pos, float *gx, int B, int I,
                                          int N, int k, int O, int BT, const ProbReduce &R, long long WT, hipStream_t s) {
    const int rblocks = dl_ceil_div(WT, 256);
    if (!gx) {
        DL_TIMED("prob_reduce_weights", s, (prob_reduce_weights<<<rblocks, 256, 0, s>>>(R)));
        return;
    }
    const int gblocks = dl_xcd_grid(dl_ceil_div(I, PROB_IS), BT);
    if (O == 1)
        DL_TIMED("prob_gather_t+reduce", s, (prob_gather_t<true><<<gblocks + rblocks, 256, 0, s>>>(gmT, inv_ptr, inv_pos, gx, B, I,
                                                                                               N, k, O, BT, gblocks, R)));
    else
        DL_TIMED("prob_gather_t+reduce", s, (prob_gather_t<false><<<gblocks + rblocks, 256, 0, s>>>(gmT, inv_ptr, inv_pos, gx, B, I,
                                                                                                N, k, O, BT, gblocks, R)));
}

// ---------------------------------------------------------------------------------
// Generic kernels, any k up to DL_MAX_K.
__global__ __launch_bounds__(256) void prob_generic_fwd(const float *__restrict__ x, const int *__restrict__ idx32,
                                                         const float *__restrict__ raw, ProbTemp T, float *__restrict__ y,
                                                         int B, int I, int N, int K, int O) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long NO = (long long)N * O;
    if (gid >= (long long)B * NO) return;
    const int b = (int)(gid / NO);
    const int n = (int)((gid % NO) / O), d = (int)((gid % NO) % O);
    const float inv_t = prob_inv_t_of(T, n);
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

// hybrid: `raw` is the table itself in the layout [n][d][a] and the input gradient carries q / (q + 1e-8)
__global__ __launch_bounds__(256) void prob_generic_bwd(const float *__restrict__ x, const int *__restrict__ idx32,
                                                         const float *__restrict__ raw, ProbTemp T,
                                                         const float *__restrict__ gy, float *__restrict__ gx,
                                                         float *__restrict__ graw, int B, int I, int N, int K, int O,
                                                         int hybrid) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (long long)B * N) return;
    const int b = (int)(gid / N), n = (int)(gid % N);
    const float inv_t = prob_inv_t_of(T, n);
    float xs[DL_MAX_K], gxs[DL_MAX_K];
    for (int j = 0; j < K; ++j) { xs[j] = x[(size_t)b * I + idx32[(size_t)n * K + j]]; gxs[j] = 0.0f; }
    const int L = 1 << K;
    for (int d = 0; d < O; ++d) {
        const float g = gy[((size_t)b * N + n) * O + d];
        for (int a = 0; a < L; ++a) {
            const size_t w = hybrid ? ((size_t)n * O + d) * L + a : ((size_t)n * L + a) * O + d;
            const float s = hybrid ? raw[w] : dl_sigmoid(raw[w] * inv_t);
            float p = 1.0f;
            for (int j = 0; j < K; ++j) p *= ((a >> j) & 1) ? xs[j] : 1.0f - xs[j];
            atomicAdd(&graw[w], hybrid ? g * p : g * p * s * (1.0f - s) * inv_t);
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
        for (int j = 0; j < K; ++j) {
            const float q = xs[j] * (1.0f - xs[j]);
            atomicAdd(&gx[(size_t)b * I + idx32[(size_t)n * K + j]], hybrid ? gxs[j] * q / (q + PROB_HYBRID_EPS) : gxs[j]);
        }
}

__global__ __launch_bounds__(256) void prob_eval_kernel(const float *__restrict__ x, const int *__restrict__ idx32,
                                                         const float *__restrict__ raw, ProbTemp T, float *__restrict__ y,
                                                         int B, int I, int N, int K, int O) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long NO = (long long)N * O;
    if (gid >= (long long)B * NO) return;
    const int b = (int)(gid / NO);
    const int n = (int)((gid % NO) / O), d = (int)((gid % NO) % O);
    const float inv_t = prob_inv_t_of(T, n);
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

// ---------------------------------------------------------------------------------
static int prob_check(int B, int I, int N, int k, int O) {
    if (B <= 0 || I <= 0 || N <= 0 || k <= 0 || O <= 0) return DL_ERR_SHAPE;
    if (k > DL_MAX_K) return DL_ERR_UNSUPPORTED;
    if (B > 4000000) return DL_ERR_UNSUPPORTED;  // batch tiles ride in grid.y (at most 65535 of them, extra rows included)
    return DL_OK;
}
// the tiled path addresses a batch tile of xT with 32-bit byte offsets (input * 256)
static inline bool prob_fast(int I, int N, int k, int O) {
    return k <= DL_MAX_FAST_K && I < (1 << 23) && (long long)N * O * k < (1 << 23);
}
// temperature.clamp(min=1e-6); with a per-node array the kernels take every node's own value
static inline ProbTemp prob_temp(float t, const float *t_n) { return ProbTemp{1.0f / (t > 1e-6f ? t : 1e-6f), t_n}; }
static inline int prob_bt(int B) { return (B + 63) / 64; }
// batch tiles per wavefront of prob_bwd_t: enough (column, chunk) wavefronts to fill the chip
static inline int prob_tiles_per_chunk(int B, int N, int O) {
    const int BT = prob_bt(B);
    int chunks = dl_ceil_div(4096, (long long)N * O);
    if (chunks > BT) chunks = BT;
    if (chunks < 1) chunks = 1;
    return dl_ceil_div(BT, chunks);
}
static inline size_t prob_sig_bytes(int N, int k, int O) { return dl_align256((size_t)N * O * ((size_t)1 << k) * sizeof(float)); }
static inline size_t prob_xT_bytes(int B, int I) { return dl_align256((size_t)prob_bt(B) * I * 64 * sizeof(float)); }

// what the forward leaves for the backward: the sigmoid table and the re-tiled input
extern "C" size_t dl_prob_saved_bytes(int B, int I, int N, int k, int O) {
    if (B <= 0 || I <= 0 || N <= 0 || k <= 0 || O <= 0 || !prob_fast(I, N, k, O)) return 256;
    return prob_sig_bytes(N, k, O) + prob_xT_bytes(B, I);
}
extern "C" size_t dl_prob_bwd_workspace_bytes(int B, int I, int N, int k, int O) {
    if (B <= 0 || I <= 0 || N <= 0 || k <= 0 || O <= 0 || !prob_fast(I, N, k, O)) return 256;
    const size_t BT = prob_bt(B);
    const int chunks = dl_ceil_div(prob_bt(B), prob_tiles_per_chunk(B, N, O));
    return prob_sig_bytes(N, k, O) + prob_xT_bytes(B, I) + dl_align256(BT * N * O * 64 * sizeof(float)) +
           dl_align256(BT * N * O * k * 64 * sizeof(float)) + dl_align256((size_t)chunks * N * O * ((size_t)1 << k) * sizeof(float));
}

#define PROB_DISPATCH(K, CALL) \
    switch (K) {               \
        case 1: CALL(1); break; case 2: CALL(2); break; case 3: CALL(3); break; \
        case 4: CALL(4); break; case 5: CALL(5); break; default: CALL(6); break; \
    }

static int prob_forward(const float *x, const int32_t *idx32, const float *raw_w, ProbTemp inv_t, float *y, void *saved,
                        size_t saved_bytes, int B, int I, int N, int k, int O, void *stream) {
    if (!x || !idx32 || !raw_w || !y) return DL_ERR_NULL;
    int rc = prob_check(B, I, N, k, O);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (!prob_fast(I, N, k, O)) {
        DL_TIMED("prob_generic_fwd", s, (prob_generic_fwd<<<dl_ceil_div((long long)B * N * O, 256), 256, 0, s>>>(x, idx32, raw_w, inv_t, y, B, I, N, k, O)));
        return dl_launch_status();
    }
    if (!saved) return DL_ERR_NULL;
    if (saved_bytes < dl_prob_saved_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    const int BT = prob_bt(B), L = 1 << k;
    float *sig = (float *)saved;
    float *xT = (float *)((char *)saved + prob_sig_bytes(N, k, O));
    {   // x re-tiled and the sigmoid table built in one launch
        const int gx_ = dl_ceil_div(I, 64);
        const int extra = dl_ceil_div(dl_ceil_div((long long)N * L * O, 256), gx_);
        DL_TIMED("prob_to_tiles_x+sig_table", s, (prob_to_tiles<<<dim3(gx_, BT + extra), 256, 0, s>>>(
                                                     x, xT, B, I, BT, raw_w, inv_t, sig, N, L, O)));
    }
    const int grid = dl_xcd_grid(dl_ceil_div((long long)N * O, PROB_TC), BT);
#define CALL(KK) DL_TIMED("prob_fwd_t", s, (prob_fwd_t<KK><<<grid, 64 * PROB_FW, 0, s>>>(xT, idx32, sig, y, B, I, N, O, BT)))
    PROB_DISPATCH(k, CALL)
#undef CALL
    return dl_launch_status();
}

extern "C" int dl_prob_layer_fwd(const float *x, const int32_t *idx32, const float *raw_w, float temperature, float *y,
                                 void *saved, size_t saved_bytes, int B, int I, int N, int k, int O, void *stream) {
    return prob_forward(x, idx32, raw_w, prob_temp(temperature, nullptr), y, saved, saved_bytes, B, I, N, k, O, stream);
}
extern "C" int dl_prob_layer_fwd_nodes(const float *x, const int32_t *idx32, const float *raw_w, const float *temperature_n,
                                       float *y, void *saved, size_t saved_bytes, int B, int I, int N, int k, int O,
                                       void *stream) {
    if (!temperature_n) return DL_ERR_NULL;
    return prob_forward(x, idx32, raw_w, prob_temp(1.0f, temperature_n), y, saved, saved_bytes, B, I, N, k, O, stream);
}

static int prob_backward(const float *x, const void *saved, const int32_t *idx32, const int32_t *inv_ptr,
                         const int32_t *inv_pos, const float *raw_w, ProbTemp inv_t, const float *gy, float *gx, float *graw,
                         void *ws, size_t ws_bytes, int B, int I, int N, int k, int O, void *stream) {
    if (!x || !idx32 || !raw_w || !gy || !graw) return DL_ERR_NULL;
    if (gx && (!inv_ptr || !inv_pos)) return DL_ERR_NULL;
    int rc = prob_check(B, I, N, k, O);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    const long long WT = (long long)N * ((long long)1 << k) * O;
    if (!prob_fast(I, N, k, O)) {
        DL_TIMED("prob_fill_zero", s, (prob_fill_zero<<<dl_ceil_div(WT, 256), 256, 0, s>>>(graw, WT)));
        if (gx) prob_fill_zero<<<dl_ceil_div((long long)B * I, 256), 256, 0, s>>>(gx, (long long)B * I);
        DL_TIMED("prob_generic_bwd", s, (prob_generic_bwd<<<dl_ceil_div((long long)B * N, 256), 256, 0, s>>>(x, idx32, raw_w, inv_t, gy, gx, graw, B, I, N,
                                                                          k, O, 0)));
        return dl_launch_status();
    }
    if (!ws) return DL_ERR_NULL;
    if (ws_bytes < dl_prob_bwd_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    const int BT = prob_bt(B), L = 1 << k, NO = N * O;
    const int tpc = prob_tiles_per_chunk(B, N, O);
    const int chunks = dl_ceil_div(BT, tpc);
    char *w = (char *)ws;
    float *sig = (float *)w; w += prob_sig_bytes(N, k, O);
    float *xT = (float *)w; w += prob_xT_bytes(B, I);
    float *gyT = (float *)w; w += dl_align256((size_t)BT * NO * 64 * sizeof(float));
    float *gmT = (float *)w; w += dl_align256((size_t)BT * NO * k * 64 * sizeof(float));
    float *gpart = (float *)w;
    if (saved) {  // what the forward of the same x, raw_w and temperature left
        sig = (float *)saved;
        xT = (float *)((char *)saved + prob_sig_bytes(N, k, O));
    } else {
        DL_TIMED("prob_sig_table", s, (prob_sig_table<<<dl_ceil_div(WT, 256), 256, 0, s>>>(raw_w, inv_t, sig, N, L, O)));
        DL_TIMED("prob_to_tiles_x", s, (prob_to_tiles<<<dim3(dl_ceil_div(I, 64), BT), 256, 0, s>>>(x, xT, B, I)));
    }
    if (k <= 5) {  // 16 wavefronts per block take gy as it is (see prob_bwd_t)
#define CALL(KK)                                                                                                       \
    DL_TIMED("prob_bwd_t", s,                                                                                          \
             (prob_bwd_t<KK, false, 16><<<dim3(dl_ceil_div(NO, 16), chunks), 1024, 0, s>>>(xT, gy, idx32, sig, gmT, gpart, I, N, \
                                                                                        O, BT, tpc, gx != nullptr, B)))
        switch (k) {
            case 1: CALL(1); break; case 2: CALL(2); break; case 3: CALL(3); break; case 4: CALL(4); break;
            default: CALL(5); break;
        }
#undef CALL
    } else {
        DL_TIMED("prob_to_tiles_gy", s, (prob_to_tiles<<<dim3(dl_ceil_div(NO, 64), BT), 256, 0, s>>>(gy, gyT, B, NO)));
#define CALL(KK)                                                                                                    \
    DL_TIMED("prob_bwd_t", s,                                                                                       \
             (prob_bwd_t<KK, false><<<dim3(dl_ceil_div(NO, 4), chunks), 256, 0, s>>>(xT, gyT, idx32, sig, gmT, gpart, I, N, O, \
                                                                                  BT, tpc, gx != nullptr)))
        PROB_DISPATCH(k, CALL)
#undef CALL
    }
    const ProbReduce R = {gpart, sig, inv_t, graw, N, L, O, chunks};
    prob_launch_gather_and_reduce(gmT, inv_ptr, inv_pos, gx, B, I, N, k, O, BT, R, WT, s);
    return dl_launch_status();
}

extern "C" int dl_prob_layer_bwd(const float *x, const void *saved, const int32_t *idx32, const int32_t *inv_ptr,
                                 const int32_t *inv_pos,
                                 const float *raw_w, float temperature, const float *gy, float *gx, float *graw,
                                 void *ws, size_t ws_bytes, int B, int I, int N, int k, int O, void *stream) {
    return prob_backward(x, saved, idx32, inv_ptr, inv_pos, raw_w, prob_temp(temperature, nullptr), gy, gx, graw, ws, ws_bytes,
                         B, I, N, k, O, stream);
}
extern "C" int dl_prob_layer_bwd_nodes(const float *x, const void *saved, const int32_t *idx32, const int32_t *inv_ptr,
                                       const int32_t *inv_pos, const float *raw_w, const float *temperature_n,
                                       const float *gy, float *gx, float *graw, void *ws, size_t ws_bytes, int B, int I,
                                       int N, int k, int O, void *stream) {
    if (!temperature_n) return DL_ERR_NULL;
    return prob_backward(x, saved, idx32, inv_ptr, inv_pos, raw_w, prob_temp(1.0f, temperature_n), gy, gx, graw, ws, ws_bytes,
                         B, I, N, k, O, stream);
}

// Hybrid nodes: the forward is the DWN lookup; the backward is the probabilistic one on the table as given.
extern "C" size_t dl_hybrid_bwd_workspace_bytes(int B, int I, int N, int k, int O) {
    if (B <= 0 || I <= 0 || N <= 0 || k <= 0 || O <= 0 || !prob_fast(I, N, k, O)) return 256;
    return dl_prob_bwd_workspace_bytes(B, I, N, k, O) - prob_sig_bytes(N, k, O);
}

extern "C" int dl_hybrid_layer_bwd(const float *x, const int32_t *idx32, const int32_t *inv_ptr, const int32_t *inv_pos,
                                   const float *luts, const float *gy, float *gx, float *gluts, void *ws, size_t ws_bytes,
                                   int B, int I, int N, int k, int O, void *stream) {
    if (!x || !idx32 || !luts || !gy || !gluts) return DL_ERR_NULL;
    if (gx && (!inv_ptr || !inv_pos)) return DL_ERR_NULL;
    int rc = prob_check(B, I, N, k, O);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    const long long WT = (long long)N * ((long long)1 << k) * O;
    if (!prob_fast(I, N, k, O)) {
        DL_TIMED("prob_fill_zero", s, (prob_fill_zero<<<dl_ceil_div(WT, 256), 256, 0, s>>>(gluts, WT)));
        if (gx) prob_fill_zero<<<dl_ceil_div((long long)B * I, 256), 256, 0, s>>>(gx, (long long)B * I);
        DL_TIMED("prob_generic_bwd", s, (prob_generic_bwd<<<dl_ceil_div((long long)B * N, 256), 256, 0, s>>>(
                                            x, idx32, luts, ProbTemp{1.0f, nullptr}, gy, gx, gluts, B, I, N, k, O, 1)));
        return dl_launch_status();
    }
    if (!ws) return DL_ERR_NULL;
    if (ws_bytes < dl_hybrid_bwd_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    const int BT = prob_bt(B), L = 1 << k, NO = N * O;
    const int tpc = prob_tiles_per_chunk(B, N, O);
    const int chunks = dl_ceil_div(BT, tpc);
    char *w = (char *)ws;
    float *xT = (float *)w; w += prob_xT_bytes(B, I);
    float *gyT = (float *)w; w += dl_align256((size_t)BT * NO * 64 * sizeof(float));
    float *gmT = (float *)w; w += dl_align256((size_t)BT * NO * k * 64 * sizeof(float));
    float *gpart = (float *)w;
    DL_TIMED("prob_to_tiles_x", s, (prob_to_tiles<<<dim3(dl_ceil_div(I, 64), BT), 256, 0, s>>>(x, xT, B, I)));
    DL_TIMED("prob_to_tiles_gy", s, (prob_to_tiles<<<dim3(dl_ceil_div(NO, 64), BT), 256, 0, s>>>(gy, gyT, B, NO)));
#define CALL(KK)                                                                                                          \
    DL_TIMED("hybrid_bwd_t", s,                                                                                           \
             (prob_bwd_t<KK, true><<<dim3(dl_ceil_div(NO, 4), chunks), 256, 0, s>>>(xT, gyT, idx32, luts, gmT, gpart, I, N, O, \
                                                                                 BT, tpc, gx != nullptr)))
    PROB_DISPATCH(k, CALL)
#undef CALL
    const ProbReduce R = {gpart, nullptr, ProbTemp{1.0f, nullptr}, gluts, N, L, O, chunks};
    prob_launch_gather_and_reduce(gmT, inv_ptr, inv_pos, gx, B, I, N, k, O, BT, R, WT, s);
    return dl_launch_status();
}

// Eval forward with a workspace: the binarised sigmoid table of every node is the table of a DWN layer, so the
// DWN eval path (bit-planes when every input is 0 or 1, the literal float address otherwise) answers.
extern "C" size_t dl_dwn_eval_workspace_bytes(int B, int I, int N, int k, int O);
extern "C" int dl_dwn_layer_eval_ws(const float *x, const int32_t *idx32, const float *luts, float *y, void *ws,
                                    size_t ws_bytes, int B, int I, int N, int k, int O, void *stream);
static inline size_t prob_eval_table_bytes(int N, int k, int O) { return dl_align256((size_t)N * O * ((size_t)1 << k) * 4); }
extern "C" size_t dl_prob_eval_workspace_bytes(int B, int I, int N, int k, int O) {
    if (B <= 0 || I <= 0 || N <= 0 || k <= 0 || O <= 0 || k > DL_MAX_FAST_K) return 256;
    return prob_eval_table_bytes(N, k, O) + dl_dwn_eval_workspace_bytes(B, I, N, k, O);
}
static int prob_eval_ws(const float *x, const int32_t *idx32, const float *raw_w, ProbTemp T, float *y, void *ws,
                        size_t ws_bytes, int B, int I, int N, int k, int O, void *stream) {
    if (!x || !idx32 || !raw_w || !y) return DL_ERR_NULL;
    int rc = prob_check(B, I, N, k, O);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (k > DL_MAX_FAST_K) {
        DL_TIMED("prob_eval_kernel", s, (prob_eval_kernel<<<dl_ceil_div((long long)B * N * O, 256), 256, 0, s>>>(
                                            x, idx32, raw_w, T, y, B, I, N, k, O)));
        return dl_launch_status();
    }
    if (!ws) return DL_ERR_NULL;
    if (ws_bytes < dl_prob_eval_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    float *sig = (float *)ws;
    const int L = 1 << k;
    DL_TIMED("prob_sig_table", s, (prob_sig_table<<<dl_ceil_div((long long)N * L * O, 256), 256, 0, s>>>(
                                      raw_w, T, sig, N, L, O)));
    const size_t tb = prob_eval_table_bytes(N, k, O);
    return dl_dwn_layer_eval_ws(x, idx32, sig, y, (char *)ws + tb, ws_bytes - tb, B, I, N, k, O, stream);
}
extern "C" int dl_prob_layer_eval_ws(const float *x, const int32_t *idx32, const float *raw_w, float temperature, float *y,
                                     void *ws, size_t ws_bytes, int B, int I, int N, int k, int O, void *stream) {
    return prob_eval_ws(x, idx32, raw_w, prob_temp(temperature, nullptr), y, ws, ws_bytes, B, I, N, k, O, stream);
}
extern "C" int dl_prob_layer_eval_ws_nodes(const float *x, const int32_t *idx32, const float *raw_w,
                                           const float *temperature_n, float *y, void *ws, size_t ws_bytes, int B, int I,
                                           int N, int k, int O, void *stream) {
    if (!temperature_n) return DL_ERR_NULL;
    return prob_eval_ws(x, idx32, raw_w, prob_temp(1.0f, temperature_n), y, ws, ws_bytes, B, I, N, k, O, stream);
}

// The same for k <= 6 with the row of x staged in the LDS by persistent blocks of 1024 threads: a thread keeps the input
// indices of its (up to eight) columns and their binarised tables - bit a of a 64-bit mask = (sigmoid(w[a] / T) >= 0.5),
// taken with the expression of prob_eval_kernel - in registers over all its rows.
template <int K>
__global__ __launch_bounds__(1024) void prob_eval_lds(const float *__restrict__ x, const int *__restrict__ idx32,
                                                       const float *__restrict__ raw, ProbTemp T, float *__restrict__ y,
                                                       int B, int I, long long NO, int O, long long c_begin, long long c_end) {
    extern __shared__ float prob_eval_row[];
    float *row = prob_eval_row;
    constexpr int L = 1 << K, QC = 8;
    int ix[QC][K];
    unsigned long long mask[QC];
#pragma unroll
    for (int q = 0; q < QC; ++q) {
        const long long c = c_begin + threadIdx.x + 1024LL * q;
        mask[q] = 0ull;
#pragma unroll
        for (int j = 0; j < K; ++j) ix[q][j] = 0;
        if (c < c_end) {
            const int n = (int)(c / O), d = (int)(c % O);
            const float inv_t = prob_inv_t_of(T, n);
#pragma unroll
            for (int j = 0; j < K; ++j) ix[q][j] = idx32[(size_t)n * K + j];
            for (int a = 0; a < L; ++a)
                mask[q] |= (dl_sigmoid(raw[((size_t)n * L + a) * O + d] * inv_t) >= 0.5f ? 1ull : 0ull) << a;
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
            for (int j = 0; j < K; ++j) sum += row[ix[q][j]] * (float)(1 << j);  // the order of prob_eval_kernel's loop
            long long a = (long long)sum;
            a = a < 0 ? 0 : (a > L - 1 ? L - 1 : a);
            __builtin_nontemporal_store(((mask[q] >> a) & 1ull) ? 1.0f : 0.0f, y + (size_t)b * NO + c);
        }
    }
}

extern "C" int dl_prob_layer_eval(const float *x, const int32_t *idx32, const float *raw_w, float temperature, float *y,
                                  int B, int I, int N, int k, int O, void *stream) {
    if (!x || !idx32 || !raw_w || !y) return DL_ERR_NULL;
    int rc = prob_check(B, I, N, k, O);
    if (rc) return rc;
    const long long NO = (long long)N * O;
    if (k <= 6 && I <= 32768 && NO >= 1024) {
        hipStream_t s = (hipStream_t)stream;
        const size_t lds = (size_t)I * sizeof(float);
        const ProbTemp T = prob_temp(temperature, nullptr);
        for (long long c0 = 0; c0 < NO; c0 += 8192) {  // windows of 8192 columns: eight per thread
            const long long c1 = c0 + 8192 < NO ? c0 + 8192 : NO;
#define CALL(KK)                                                                                                       \
    do {                                                                                                               \
        if (lds > 64 * 1024) {                                                                                         \
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&prob_eval_lds<KK>),               \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);            \
            if (e != hipSuccess) return (int)e;                                                                        \
        }                                                                                                              \
        DL_TIMED("prob_eval_kernel", s,                                                                                \
                 (prob_eval_lds<KK><<<B < 256 ? B : 256, 1024, lds, s>>>(x, idx32, raw_w, T, y, B, I, NO, O, c0, c1))); \
    } while (0)
            PROB_DISPATCH(k, CALL)
#undef CALL
        }
        return dl_launch_status();
    }
    DL_TIMED("prob_eval_kernel", (hipStream_t)stream, (prob_eval_kernel<<<dl_ceil_div((long long)B * N * O, 256), 256, 0, (hipStream_t)stream>>>(
        x, idx32, raw_w, prob_temp(temperature, nullptr), y, B, I, N, k, O)));
    return dl_launch_status();
}
