// RandomLayer + DWN nodes on gfx950: forward (threshold, address, lookup) and the
// extended-finite-difference backward, whole layer per call.
//
// Layout idea (k <= 6): a wavefront's 64 lanes are 64 batch rows.  Everything that
// belongs to a node - its k input indices, its 2^k-entry table, its EFD coefficient
// rows - is then wave-uniform: indices and bit-plane words come through scalar loads,
// a table sits one entry per lane in a single VGPR and a lookup is one ds_bpermute.
// The random RandomLayer mapping costs nothing in this layout (it is scalar addressing);
// what it costs instead is one transpose through LDS wherever a tensor crosses the
// [batch, feature] boundary (y out, gy in, gx out).
//
//   forward   pack_planes : x [B,I] fp32 -> planes [B/64][I] u64 (bit r = x[64t+r][i] >= 0.5)
//             lookup_fwd  : planes + idx + luts -> y [B,N*O] (LDS-transposed tiles) and
//                           addrT [B/64][N][64] u8, the address of every (node,row), kept for backward
//   backward  transpose_hist : gy [B,N*O] -> gyT [B/64][N*O][64]; per-node 2^k-bin histogram of gy
//                           in LDS; blocks of one column tile leave partials per chunk of batch tiles.
//                           The same launch carries the blocks that build the gather's coefficient tables
//                           (efd_table_block): luts -> D[n][d][j][a'] = alpha * sum_kappa s(kappa_j) lut[kappa]
//                           beta^popc((a^kappa)&~(1<<j)), a' = address with bit j squeezed out
//             bwd_gx      : for every input i the (node,slot) pairs that read it (CSR):
//                           gx[b,i] = sum gyT[c][b] * D[c][j][a'(b)]  - a gather in fixed order; its launch
//                           also carries the blocks that add the histogram partials in chunk order (no
//                           floating-point atomics anywhere)
// k > 6 goes to the one-thread-per-element kernels of dwn_generic.hip.
#include "dl_common.h"
#include <algorithm>
#include <mutex>
#include <type_traits>
#include "dwn_generic.h"

typedef unsigned long long u64;

// addr <- 2*addr + (bit `lane` of mask): the 64-bit scalar is used directly as a per-lane carry-in.
__device__ __forceinline__ unsigned dwn_shift_in(unsigned addr, u64 mask) {
    unsigned out;
    u64 carry_out;
    asm("v_addc_co_u32_e64 %0, %1, %2, %2, %3" : "=v"(out), "=s"(carry_out) : "v"(addr), "s"(mask));
    return out;
}

// ---------------------------------------------------------------------------------
// pack_planes: grid (ceil(I / (256*VEC)), 4 * tiles), 256 threads; a thread takes VEC inputs over 16 of the 64 rows
// of a batch tile and writes its 16-bit piece of each plane word (piece p = rows 16p .. 16p + 15 = bits 16p .. of
// the little-endian word).  Four times the threads of a whole-tile-per-thread version, each a quarter as long:
// 6.4 instead of 5.4 TB/s on a 4096 x 16384 input.  Every load of a wavefront is one contiguous 64*VEC*4-byte
// piece of a row of x.  Rows past B give 0 bits.
// CHECK: also clears *all_binary (preset to 1 by the caller) when some value is neither 0 nor 1.
#define DWN_PACK_ROWS 16
static inline int dwn_pack_grid_y(int BT) { return 4 * BT < 65535 ? 4 * BT : 65535; }
template <int VEC, bool CHECK = false>
__global__ __launch_bounds__(256) void dwn_pack_planes(const float *__restrict__ x, u64 *__restrict__ planes,
                                                        int B, int I, int *__restrict__ all_binary = nullptr) {
    constexpr int PIECES = 64 / DWN_PACK_ROWS;
    bool odd = false;  // saw a value other than 0 and 1
    const int i0 = (blockIdx.x * 256 + threadIdx.x) * VEC;
    if (i0 >= I) return;
    const int pieces_total = PIECES * ((B + 63) / 64);
    for (int by = blockIdx.y; by < pieces_total; by += gridDim.y) {  // grid.y is capped at 65535 (pieces of 16 rows)
        const int t = by / PIECES, piece = by % PIECES;
        const int r0 = t * 64 + piece * DWN_PACK_ROWS;
        const int rows = min(DWN_PACK_ROWS, B - r0);  // <= 0 for pieces past the batch
        const float *base = x + (size_t)r0 * I + i0;
        unsigned acc[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] = 0u;
        if (rows == DWN_PACK_ROWS) {
#pragma unroll
            for (int r = 0; r < DWN_PACK_ROWS; ++r) {
                const float *src = base + (size_t)r * I;
                if constexpr (VEC == 4) {
                    typedef float f4v __attribute__((ext_vector_type(4)));
                    const f4v q = __builtin_nontemporal_load(reinterpret_cast<const f4v *>(src));  // x is read once
                    acc[0] |= (q.x >= 0.5f ? 1u : 0u) << r;
                    acc[1] |= (q.y >= 0.5f ? 1u : 0u) << r;
                    acc[2] |= (q.z >= 0.5f ? 1u : 0u) << r;
                    acc[3] |= (q.w >= 0.5f ? 1u : 0u) << r;
                    if (CHECK)
                        odd = odd || !((q.x == 0.0f || q.x == 1.0f) && (q.y == 0.0f || q.y == 1.0f) &&
                                       (q.z == 0.0f || q.z == 1.0f) && (q.w == 0.0f || q.w == 1.0f));
                } else {
                    const float v0 = __builtin_nontemporal_load(src);
                    acc[0] |= (v0 >= 0.5f ? 1u : 0u) << r;
                    if (CHECK) odd = odd || !(v0 == 0.0f || v0 == 1.0f);
                }
            }
        } else {
            for (int r = 0; r < rows; ++r) {
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    const float val = base[(size_t)r * I + v];
                    acc[v] |= (val >= 0.5f ? 1u : 0u) << r;
                    if (CHECK) odd = odd || !(val == 0.0f || val == 1.0f);
                }
            }
        }
        unsigned short *out = reinterpret_cast<unsigned short *>(planes + (size_t)t * I + i0) + piece;
#pragma unroll
        for (int v = 0; v < VEC; ++v) out[v * PIECES] = (unsigned short)acc[v];
    }
    if (CHECK && odd) *all_binary = 0;  // every writer stores the same value
}
__global__ void dwn_set_flag(int *flag, int value) {
    if (threadIdx.x == 0) *flag = value;
}

// ---------------------------------------------------------------------------------
// lookup_fwd: one block per (128-column tile, 64-row batch tile), 512 threads = 8 wavefronts,
// lane = batch row, column = node*O + output.  A wavefront owns 16 consecutive columns.  Their
// k*16 input indices are fetched once (one per lane) and handed out with readlane; the bit-plane
// word of (tile, input) is wave-uniform, so it comes through a scalar load and is used directly
// as a lane mask: one add-with-carry per input shifts the lane's bit into its address
// (addr <- 2*addr + bit), one bpermute per column reads the table entry.  Columns are taken four
// at a time so that the 4*k scalar loads of a group are in flight together.
#define DWN_TC 128
#define DWN_FW 8                      // wavefronts per block
#define DWN_WC (DWN_TC / DWN_FW)      // columns per wavefront
#define DWN_CG 4                      // columns per group
// CHAIN: the variant for chained layers, which can also (or only) emit the columns as bit-planes.
// GSUM: the variant under a GroupSum head.  Instead of y it writes, per row, the sums of the tile's columns
// that fall into each group the tile touches (at most DWN_GS_SLOTS of them):
// partial[(column tile * slots + slot)][row], slot = group - first group of the tile; dwn_group_finish
// adds the tiles of a group in a fixed order.
#define DWN_GS_SLOTS 4
// EVAL: the inference form (DWNNode.forward_eval on inputs that are exactly 0 or 1, where its address
// floor(sum x_j 2^j) is the thresholded one): the output is (table entry >= 0.5) as 0/1, nothing is saved
// for a backward.
template <int K, bool O1, bool CHAIN = false, bool GSUM = false, bool EVAL = false>
__global__ __launch_bounds__(64 * DWN_FW) void dwn_lookup_fwd(const u64 *__restrict__ planes, const int *__restrict__ idx32,
                                                               const float *__restrict__ luts, float *__restrict__ y,
                                                               uint8_t *__restrict__ addrT, u64 *__restrict__ planes_out,
                                                               int B, int I, int N, int O, int BT, int gsize = 1,
                                                               int slots = 1, const int *__restrict__ run_if_set = nullptr) {
    if (EVAL && run_if_set && *run_if_set == 0) return;  // the inputs were not all 0/1: the generic kernel answers
    __shared__ float tile[DWN_TC][65];  // [column][row]
    __shared__ u64 plane_tile[CHAIN ? DWN_TC : 1];  // thresholded outputs of the tile's columns, one bit per row
    __shared__ float gpart[GSUM ? DWN_FW : 1][GSUM ? DWN_GS_SLOTS : 1][64];  // [wavefront][slot][row]
    constexpr int L = 1 << K;
    constexpr int NIDX = (DWN_WC * K + 63) / 64;  // index registers per lane
    const int NO = N * O;
    int ctile, t;
    if (!dl_xcd_map((NO + DWN_TC - 1) / DWN_TC, BT, ctile, t)) return;
    const int c0 = ctile * DWN_TC;
    const int lane = threadIdx.x & 63;
    const int wave = dl_uniform(threadIdx.x >> 6);
    const u64 *pl = planes + (size_t)t * I;
    const __amdgpu_buffer_rsrc_t rs_luts = __builtin_amdgcn_make_buffer_rsrc((void *)luts, 0, NO * L * 4, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_addr =
        __builtin_amdgcn_make_buffer_rsrc((void *)(addrT + (size_t)t * N * 64), 0, N * 64, 0x00020000);
    const int lane4s = (lane & (L - 1)) * 4;
    const int cend = min(DWN_TC, NO - c0);
    const int wbeg = wave * DWN_WC;
    // slot s = (column within my 16) * K + j  ->  lane s % 64 of register s / 64
    int myidx[NIDX];
#pragma unroll
    for (int v = 0; v < NIDX; ++v) {
        const int s = v * 64 + lane;
        const int c = min(c0 + wbeg + min(s / K, DWN_WC - 1), NO - 1);
        myidx[v] = idx32[(O1 ? c : c / O) * K + s % K] * 8;  // byte offset of the input's plane word
    }
    // FULL: all 128 columns of the tile exist (every tile but possibly the last): no clamps, no per-column checks,
    // so the column offsets fold into the instructions
    u64 my_plane = 0;  // CHAIN: lane l keeps the thresholded bits of my wavefront's column l
    auto columns = [&](auto full_tag) {
        constexpr bool FULL = decltype(full_tag)::value;
#pragma unroll
        for (int g = 0; g < DWN_WC; g += DWN_CG) {
            u64 w[DWN_CG][K];
            float entry[DWN_CG];
#pragma unroll
            for (int q = 0; q < DWN_CG; ++q) {
                const int c = FULL ? c0 + wbeg + g + q : min(c0 + wbeg + g + q, NO - 1);
                // table row of column c, one entry per lane; the row offset travels in an SGPR
                entry[q] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs_luts, lane4s, c * (L * 4), 0));
#pragma unroll
                for (int j = 0; j < K; ++j) {
                    constexpr int dummy = 0;
                    (void)dummy;
                    const int s = (g + q) * K + j;  // compile-time after unrolling
                    // wave-uniform unsigned byte offset: a scalar load with the offset in an SGPR,
                    // no scalar address arithmetic
                    const unsigned src = (unsigned)__builtin_amdgcn_readlane(myidx[s / 64], s % 64);
                    w[q][j] = *reinterpret_cast<const u64 *>(reinterpret_cast<const char *>(pl) + src);
                }
            }
#pragma unroll
            for (int q = 0; q < DWN_CG; ++q) {
                const int cc = wbeg + g + q;
                unsigned addr = 0;
#pragma unroll
                for (int j = K - 1; j >= 0; --j) addr = dwn_shift_in(addr, w[q][j]);
                const float v = dl_lane_read(entry[q], (int)addr);
                if (FULL || cc < cend) {
                    tile[cc][lane] = EVAL ? (v >= 0.5f ? 1.0f : 0.0f) : v;
                    if (CHAIN && planes_out) {  // the next layer's view of this column: bit r = (y[64t+r][c] >= 0.5)
                        const u64 m = __ballot(v >= 0.5f);
                        if (lane == g + q) my_plane = m;  // a select, the column number is a constant here
                    }
                    const int c = c0 + cc;
                    const int n = O1 ? c : c / O;
                    if (!EVAL && (O1 || c - n * O == 0))
                        __builtin_amdgcn_raw_buffer_store_b8((uint8_t)addr, rs_addr, lane, n * 64, 0);
                }
            }
        }
    };
    if (CHAIN && c0 + DWN_TC <= NO) {  // (the variant that writes y gains nothing from a second copy of the loop)
        columns(std::true_type{});
    } else if (wbeg < cend) {
        columns(std::false_type{});
    }
    if (CHAIN && planes_out && lane < DWN_WC && wbeg + lane < cend) plane_tile[wbeg + lane] = my_plane;
    __syncthreads();
    if (CHAIN && planes_out && (int)threadIdx.x < cend) {
        const int rows = min(64, B - t * 64);  // rows past B read as 0, like the planes packed from x
        const u64 valid = rows == 64 ? ~0ull : ((1ull << rows) - 1ull);
        planes_out[(size_t)t * NO + c0 + threadIdx.x] = plane_tile[threadIdx.x] & valid;
    }
    if (GSUM) {
        // wavefront w adds columns w, w + 8, ... of the tile for its row (lane), one running sum per slot
        const int b1 = (c0 / gsize + 1) * gsize - c0;  // first column of the tile that belongs to slot 1
        float acc[DWN_GS_SLOTS];
#pragma unroll
        for (int sl = 0; sl < DWN_GS_SLOTS; ++sl) acc[sl] = 0.0f;
        for (int cc = wave; cc < cend; cc += DWN_FW) {
            const int sl = (cc >= b1 ? 1 : 0) + (cc >= b1 + gsize ? 1 : 0) + (cc >= b1 + 2 * gsize ? 1 : 0);  // wave-uniform
            const float v = tile[cc][lane];
#pragma unroll
            for (int q = 0; q < DWN_GS_SLOTS; ++q) acc[q] += (q == sl) ? v : 0.0f;
        }
#pragma unroll
        for (int sl = 0; sl < DWN_GS_SLOTS; ++sl) gpart[wave][sl][lane] = acc[sl];
        __syncthreads();
        if ((int)threadIdx.x < 64 * slots) {
            const int sl = threadIdx.x >> 6;
            float sum = 0.0f;
#pragma unroll
            for (int w = 0; w < DWN_FW; ++w) sum += gpart[w][sl][lane];
            y[((size_t)ctile * slots + sl) * ((size_t)BT * 64) + t * 64 + lane] = sum;  // y = the partial sums here
        }
        return;
    }
    if (CHAIN && !y) return;
    if (cend == DWN_TC && t * 64 + 64 <= B && (NO & 3) == 0 && (((uintptr_t)y) & 15) == 0) {
        // whole tile: 16-byte stores, a wavefront covers two 512-byte row pieces per instruction
        typedef float f4v __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int pass = 0; pass < 64 * DWN_TC / 4 / (64 * DWN_FW); ++pass) {
            const int e = pass * 64 * DWN_FW + threadIdx.x;
            const int r = e / (DWN_TC / 4), c4 = (e % (DWN_TC / 4)) * 4;
            const f4v v = {tile[c4][r], tile[c4 + 1][r], tile[c4 + 2][r], tile[c4 + 3][r]};
            __builtin_nontemporal_store(v, reinterpret_cast<f4v *>(&y[(size_t)(t * 64 + r) * NO + c0 + c4]));
        }
        return;
    }
    for (int e = threadIdx.x; e < 64 * DWN_TC; e += 64 * DWN_FW) {
        const int r = e / DWN_TC, cc = e % DWN_TC;
        const int b = t * 64 + r;
        if (b < B && cc < cend) __builtin_nontemporal_store(tile[cc][r], &y[(size_t)b * NO + c0 + cc]);
    }
}

// gluts[e] = scale * (partial[0][e] + partial[1][e] + ...), four entries per thread, the chunks' loads in flight together.
// `block` = index among the blocks that reduce (the table kernels below append these blocks to their own grid, so that
// the backward needs one launch for both).
struct DwnReduce {
    const float *partial;  // null: nothing to reduce
    float *gluts;
    long long NOL;
    int chunks;
    const float *scale;
    int L, O;
};
// From DWN_SLICED_CHUNKS chunks on (few columns, many batch tiles: a convolutional level, a narrow last layer) a thread
// that added all chunks of its four elements would run alone for tens of microseconds.  Then sixteen lanes share four
// elements: lane slice s adds chunks s, s + 16, ... in order, and the sixteen sums are joined by a butterfly over the
// lanes - another fixed order.
#define DWN_SLICED_CHUNKS 64
__device__ __forceinline__ bool dwn_reduce_sliced(const DwnReduce &r) { return r.chunks >= DWN_SLICED_CHUNKS && r.NOL % 4 == 0; }
__device__ __forceinline__ void dwn_reduce_block(const DwnReduce &r, int block) {
    if (dwn_reduce_sliced(r)) {
        const int lane = threadIdx.x & 63, col = lane & 3, slice = lane >> 2;
        const long long e4 = (((long long)block * 4 + (threadIdx.x >> 6)) * 4 + col) * 4;  // a wavefront: 16 elements
        const bool live = e4 < r.NOL;
        float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live)
            for (int ch = slice; ch < r.chunks; ch += 16) {
                const float4 v = *reinterpret_cast<const float4 *>(r.partial + (size_t)ch * r.NOL + e4);
                sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
            }
#pragma unroll
        for (int off = 4; off < 64; off <<= 1) {
            sum.x += __shfl_xor(sum.x, off); sum.y += __shfl_xor(sum.y, off);
            sum.z += __shfl_xor(sum.z, off); sum.w += __shfl_xor(sum.w, off);
        }
        if (live && slice == 0) {
            const float sc[4] = {r.scale ? r.scale[((e4 + 0) / r.L) / r.O] : 1.0f, r.scale ? r.scale[((e4 + 1) / r.L) / r.O] : 1.0f,
                                 r.scale ? r.scale[((e4 + 2) / r.L) / r.O] : 1.0f, r.scale ? r.scale[((e4 + 3) / r.L) / r.O] : 1.0f};
            r.gluts[e4] = sum.x * sc[0], r.gluts[e4 + 1] = sum.y * sc[1];  // the caller's array: no alignment assumed
            r.gluts[e4 + 2] = sum.z * sc[2], r.gluts[e4 + 3] = sum.w * sc[3];
        }
        return;
    }
    const long long e4 = ((long long)block * 256 + threadIdx.x) * 4;
    if (e4 >= r.NOL) return;
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
    if (r.NOL % 4 == 0) {
        for (int ch0 = 0; ch0 < r.chunks; ch0 += 8) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                v[u] = ch0 + u < r.chunks ? *reinterpret_cast<const float4 *>(r.partial + (size_t)(ch0 + u) * r.NOL + e4)
                                          : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int u = 0; u < 8; ++u) { sum[0] += v[u].x; sum[1] += v[u].y; sum[2] += v[u].z; sum[3] += v[u].w; }
        }
    } else {
        for (int ch = 0; ch < r.chunks; ++ch)
            for (int q = 0; q < 4; ++q)
                if (e4 + q < r.NOL) sum[q] += r.partial[(size_t)ch * r.NOL + e4 + q];
    }
    for (int q = 0; q < 4; ++q)
        if (e4 + q < r.NOL) r.gluts[e4 + q] = sum[q] * (r.scale ? r.scale[((e4 + q) / r.L) / r.O] : 1.0f);
}
static inline int dwn_reduce_blocks(const DwnReduce &r) {
    if (!r.partial) return 0;
    return r.chunks >= DWN_SLICED_CHUNKS && r.NOL % 4 == 0 ? dl_ceil_div(r.NOL, 64) : dl_ceil_div(r.NOL, 1024);
}
__global__ __launch_bounds__(256) void dwn_reduce_partials(DwnReduce r) { dwn_reduce_block(r, blockIdx.x); }

// ---------------------------------------------------------------------------------
// efd_table: one wavefront per table (column), lane = table entry.  Two forms of the EFD coefficients, both in double with one rounding to float:
//   D form: for every input j the table is smoothed along all OTHER inputs
//           (v <- v + beta * v[entry ^ bit]) and differenced along j; lanes whose bit j is clear
//           hold D[c][j][a'] = alpha * (v[a | bit j] - v[a & ~bit j]).          192 floats/table
//   S form: the table smoothed along ALL inputs, scaled by alpha / (1 - beta).    64 floats/table
//           Smoothing along j maps (u0,u1) -> (u0 + beta u1, beta u0 + u1), so the difference of
//           the fully smoothed table across bit j is (1 - beta) times the D-form value:
//           D[c][j][a'] = S[c][a | bit j] - S[c][a & ~bit j].  Cheaper to build, a third of the
//           memory, shared by the k slots of a node - but it amplifies rounding by
//           (1+|beta|)^k / (1-beta), so it is only used for |beta| <= 1/2 (the default is 1/3).
// alpha_n / beta_n (nullable): the nodes' own alpha and beta [N] instead of one value for the layer.
struct DwnTables {
    const float *luts;   // null: no coefficient table wanted
    float *D;
    const float *scale;  // stabilised node: per-node factor (selects dwn_stable_table_block)
    const float *alpha_n, *beta_n;
    float alpha, beta;
    int NO, K, O, sform;
};
static inline int dwn_table_blocks(const DwnTables &t) { return t.luts ? dl_ceil_div(t.NO, 4) : 0; }

// 256 threads = four tables; `block` = index among the blocks that build tables
__device__ __forceinline__ void dwn_efd_table_block(const DwnTables &tb, int block) {
    const int c = block * 4 + (threadIdx.x >> 6);
    const int a = threadIdx.x & 63;
    if (c >= tb.NO) return;
    const int K = tb.K;
    const float alpha = tb.alpha_n ? tb.alpha_n[c / tb.O] : tb.alpha;
    const float beta = tb.beta_n ? tb.beta_n[c / tb.O] : tb.beta;
    const int L = 1 << K, Lh = L >> 1;
    const bool live = a < L;
    const double v0 = live ? (double)tb.luts[(size_t)c * L + a] : 0.0;
    float *__restrict__ D = tb.D;
    if (tb.sform) {
        double v = v0;
        for (int m = 0; m < K; ++m) v += (double)beta * __shfl_xor(v, 1 << m);
        const float sv = (float)((double)alpha / (1.0 - (double)beta) * v);
        if (tb.sform == 2) {
            // the differences a gather would take from the S form, taken here instead (same operands, same rounding)
            // and laid out like the D form: two slots' rows then fill one 64-lane register
            for (int j = 0; j < K; ++j) {
                const float upper = __shfl_xor(sv, 1 << j);
                if (live && !((a >> j) & 1)) {
                    const int ap = (a & ((1 << j) - 1)) | ((a >> (j + 1)) << j);
                    D[((size_t)c * K + j) * Lh + ap] = upper - sv;
                }
            }
            return;
        }
        if (live) D[(size_t)c * L + a] = sv;
        return;
    }
    for (int j = 0; j < K; ++j) {
        double v = v0;
        for (int m = 0; m < K; ++m) {
            const double other = __shfl_xor(v, 1 << m);
            if (m != j) v += (double)beta * other;
        }
        const double upper = __shfl_xor(v, 1 << j);
        if (live && !((a >> j) & 1)) {
            const int ap = (a & ((1 << j) - 1)) | ((a >> (j + 1)) << j);
            D[((size_t)c * K + j) * Lh + ap] = (float)((double)alpha * (upper - v));
        }
    }
}

// stable_table: the D form for the gradient-stabilised node, whose weight of a table entry at
// Hamming distance h (over the other k-1 inputs) is scale[n] / (h + 1) instead of alpha * beta^h.
// That weight is not a product over inputs, so the sums are taken directly, in double: one wavefront
// per table keeps it in LDS and shares out the k * 2^(k-1) outputs (j, a'), one 2^(k-1)-term sum
//   D[c][j][a'] = scale * sum_kappa' (lut[kappa' with bit j set] - lut[kappa' with bit j clear]) / (popc(a' ^ kappa') + 1)
// each.  Called by every thread of the block.
__device__ __forceinline__ void dwn_stable_table_block(const DwnTables &tb, int block) {
    __shared__ double rec[8];
    __shared__ float tab[4][64];
    if (threadIdx.x < 8) rec[threadIdx.x] = 1.0 / (double)(threadIdx.x + 1);
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = block * 4 + w;
    const int K = tb.K, NO = tb.NO;
    const int L = 1 << K, Lh = L >> 1;
    if (c < NO && lane < L) {
        tab[w][lane] = tb.luts[(size_t)c * L + lane];
    }
    __syncthreads();
    if (c >= NO) return;
    const double sc = (double)tb.scale[c / tb.O];
    for (int o = lane; o < K * Lh; o += 64) {
        const int j = o / Lh, ap = o - j * Lh;
        const int low = (1 << j) - 1;
        double acc = 0.0;
        for (int kp = 0; kp < Lh; ++kp) {
            const int lo = (kp & low) | ((kp & ~low) << 1);  // kappa' with a clear bit j put in
            acc += ((double)tab[w][lo | (1 << j)] - (double)tab[w][lo]) * rec[__popc(ap ^ kp)];
        }
        tb.D[((size_t)c * K + j) * Lh + ap] = (float)(sc * acc);
    }
}
__device__ __forceinline__ void dwn_table_block(const DwnTables &tb, int block) {
    if (tb.scale) dwn_stable_table_block(tb, block);
    else dwn_efd_table_block(tb, block);
}

// gluts[c][a] *= scale[c / O]: the stabilised node scales its table gradient as well
__global__ __launch_bounds__(256) void dwn_scale_tables(float *__restrict__ gluts, const float *__restrict__ scale,
                                                         long long total, int L, int O) {
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    if (e < total) gluts[e] *= scale[(e / L) / O];
}

// luts = sigmoid(raw) and its adjoint graw = gluts * luts * (1 - luts), elementwise
__global__ __launch_bounds__(256) void dwn_table_sigmoid(const float *__restrict__ raw, float *__restrict__ luts,
                                                          long long total) {
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    if (e < total) luts[e] = 1.0f / (1.0f + expf(-raw[e]));
}
__global__ __launch_bounds__(256) void dwn_table_sigmoid_bwd(const float *__restrict__ gluts, const float *__restrict__ luts,
                                                              float *__restrict__ graw, long long total) {
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    if (e < total) {
        const float v = luts[e];
        graw[e] = gluts[e] * v * (1.0f - v);
    }
}

// ---------------------------------------------------------------------------------
// transpose_hist: grid (ceil(N*O / 64), chunks); a block streams `tiles_per_chunk` 64-row tiles
// of its 64 columns.  The next tile (gy values and their addresses) is prefetched into registers
// while the current one sits in LDS.  Each wavefront owns 16 of the columns:
//   * lane = batch row: reads a column of the LDS tile and stores 256 contiguous bytes of gyT;
//   * lane = (column, row mod 4): adds gy into the column's 2^k-bin histogram with a plain LDS
//     read-modify-write - the four lanes of a column are one quad, so equal addresses inside a
//     step are merged with quad permutes first and no two lanes of the block ever update the same
//     word at once (float atomics in LDS are far slower than this).
#define DWN_HC 64
// value held by lane (lane ^ X) of the same quad, X = 1..3: a DPP quad permute, no LDS traffic
template <int X>
__device__ __forceinline__ int dwn_quad_xor(int v) {
    constexpr int ctrl = X == 1 ? 0xB1 : (X == 2 ? 0x4E : 0x1B);  // quad_perm [1,0,3,2] / [2,3,0,1] / [3,2,1,0]
    return __builtin_amdgcn_update_dpp(0, v, ctrl, 0xf, 0xf, true);
}
// The four lanes of a quad hold four rows of one column: (address a, value v), lane rank hr = lane & 3.  Lanes with equal
// addresses are merged: `sum` = v plus the values of the partners with the same address (adding 0 for the others keeps
// the order of additions), and the function says whether this lane is the one that adds `sum` to the bin - the
// lowest-ranked lane of its group.  Partner hr ^ 1 ranks lower when hr is odd, partners hr ^ 2 and hr ^ 3 when hr >= 2;
// written on booleans so that the comparisons stay lane masks in scalar registers.
// One lane's addition into its LDS bin: read, add, write.  (The LDS float add instruction, which needs no wait in between,
// measured three times slower here: 196 us instead of 60 for the 4096 x 8192 histogram.)
__device__ __forceinline__ void dwn_bin_add(float *bin, float v) { *bin += v; }
__device__ __forceinline__ bool dwn_quad_merge(unsigned a, float v, int hr, float &sum) {
    const unsigned a1 = (unsigned)dwn_quad_xor<1>((int)a), a2 = (unsigned)dwn_quad_xor<2>((int)a),
                   a3 = (unsigned)dwn_quad_xor<3>((int)a);
    const float v1 = __int_as_float(dwn_quad_xor<1>(__float_as_int(v))), v2 = __int_as_float(dwn_quad_xor<2>(__float_as_int(v))),
                v3 = __int_as_float(dwn_quad_xor<3>(__float_as_int(v)));
    const bool e1 = a1 == a, e2 = a2 == a, e3 = a3 == a;
    sum = v;
    sum += e1 ? v1 : 0.0f;
    sum += e2 ? v2 : 0.0f;
    sum += e3 ? v3 : 0.0f;
    const bool odd = (hr & 1) != 0, upper = (hr & 2) != 0;
    return !((e1 & odd) | ((e2 | e3) & upper));
}
// End of a histogram block: the table gradient in a fixed order of additions.  With one chunk of batch tiles per
// column tile the block's bins are the result.  With several, every block stores its bins as a partial
// ([chunk][column][bin]) and dwn_reduce_partials adds them in chunk order afterwards, so the sums do not depend on the
// order the blocks ran in (no floating-point atomics).  scale (nullable): the stabilised node's per-node factor.
__device__ __forceinline__ void dwn_hist_flush(const float (*hist)[65], int c0, int cend, int L, long long NOL, int chunks,
                                               float *__restrict__ partial, float *__restrict__ gluts,
                                               const float *__restrict__ scale, int O) {
    if (chunks == 1) {
        for (int e = threadIdx.x; e < cend * L; e += 256)
            gluts[(size_t)c0 * L + e] = hist[e / L][e % L] * (scale ? scale[(c0 + e / L) / O] : 1.0f);
        return;
    }
    float *mine = partial + (size_t)blockIdx.y * NOL + (size_t)c0 * L;
    for (int e = threadIdx.x; e < cend * L; e += 256) mine[e] = hist[e / L][e % L];
}

template <bool WRITE_T>
__global__ __launch_bounds__(256) void dwn_bwd_transpose_hist(const float *__restrict__ gy, const uint8_t *__restrict__ addrT,
                                                               float *__restrict__ gyT, float *__restrict__ gluts,
                                                               int B, int NO, int O, int L, int BP, int BT,
                                                               int tiles_per_chunk, float *__restrict__ partial,
                                                               const float *__restrict__ scale, int chunks, DwnTables tb) {
    __shared__ float tile[64][DWN_HC + 1];       // [row][column]
    __shared__ float hist[DWN_HC][65];           // [column][bin]
    __shared__ __align__(16) uint8_t atile[DWN_HC][64 + 4];  // [column][row] addresses
    if ((int)blockIdx.y >= chunks) return dwn_table_block(tb, ((int)blockIdx.y - chunks) * gridDim.x + blockIdx.x);
    const int c0 = blockIdx.x * DWN_HC;
    const int lane = threadIdx.x & 63;
    const int wave = dl_uniform(threadIdx.x >> 6);
    const int cend = min(DWN_HC, NO - c0);
    for (int e = threadIdx.x; e < DWN_HC * 65; e += 256) (&hist[0][0])[e] = 0.0f;
    const int t_begin = blockIdx.y * tiles_per_chunk;
    const int t_end = min(BT, t_begin + tiles_per_chunk);
    const bool vec4 = (NO % 4 == 0) && cend == DWN_HC;
    const int q = threadIdx.x & 15, rr = threadIdx.x >> 4;  // 16 threads x 16 B cover one 64-column row piece
    const int N = NO / O;
    const int wc0 = wave * (DWN_HC / 4);  // my wavefront's first column
    float4 pre[4];
    unsigned apre[DWN_HC / 16];  // addresses of my 16 columns for the tile being fetched: four rows per lane and pass
    auto fetch = [&](int t) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int b = t * 64 + rr + 16 * p;
            pre[p] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (b < B) {
                const float *src = gy + (size_t)b * NO + c0 + q * 4;
                if (vec4) {
                    typedef float f4v __attribute__((ext_vector_type(4)));
                    const f4v g4 = __builtin_nontemporal_load(reinterpret_cast<const f4v *>(src));  // gy is read once
                    pre[p] = make_float4(g4.x, g4.y, g4.z, g4.w);
                } else {
                    if (q * 4 + 0 < cend) pre[p].x = src[0];
                    if (q * 4 + 1 < cend) pre[p].y = src[1];
                    if (q * 4 + 2 < cend) pre[p].z = src[2];
                    if (q * 4 + 3 < cend) pre[p].w = src[3];
                }
            }
        }
#pragma unroll
        for (int p = 0; p < DWN_HC / 16; ++p) {  // pass p: column wc0 + 4p + lane / 16, rows 4 (lane % 16) .. + 3, one 32-bit load
            const int c = min(c0 + wc0 + 4 * p + (lane >> 4), NO - 1);
            apre[p] = *reinterpret_cast<const unsigned *>(addrT + ((size_t)t * N + c / O) * 64 + 4 * (lane & 15));
        }
    };
    if (t_begin < t_end) fetch(t_begin);
    const int hc = wc0 + (lane >> 2), hr = lane & 3;  // histogram role: column and row phase of this lane
    for (int t = t_begin; t < t_end; ++t) {
        __syncthreads();  // previous tile fully consumed (and hist cleared on the first pass)
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            float *dst = &tile[rr + 16 * p][q * 4];
            dst[0] = pre[p].x; dst[1] = pre[p].y; dst[2] = pre[p].z; dst[3] = pre[p].w;
        }
#pragma unroll
        for (int p = 0; p < DWN_HC / 16; ++p)
            *reinterpret_cast<unsigned *>(&atile[wc0 + 4 * p + (lane >> 4)][4 * (lane & 15)]) = apre[p];
        __syncthreads();
        if (t + 1 < t_end) fetch(t + 1);
        if (WRITE_T) {
#pragma unroll
            for (int u = 0; u < DWN_HC / 4; ++u) {
                const int cc = wc0 + u;
                if (cc < cend) gyT[((size_t)t * NO + c0 + cc) * 64 + lane] = tile[lane][cc];
            }
        }
        if (hc < cend) {  // whole quads share hc, so the quad permutes below stay inside active lanes
            for (int r0 = 0; r0 < 64; r0 += 4) {
                const float v = tile[r0 + hr][hc];  // rows past B carry 0
                const unsigned a = atile[hc][r0 + hr];
                float sum;
                if (dwn_quad_merge(a, v, hr, sum)) dwn_bin_add(&hist[hc][a], sum);
            }
        }
    }
    __syncthreads();
    // scale (nullable): the stabilised node multiplies a node's table gradient by its gradient_scale
    dwn_hist_flush(hist, c0, cend, L, (long long)NO * L, chunks, partial, gluts, scale, O);
}

// hist_tiled: the histogram alone, for gy that arrives tile-major ([B/64][N*O][64]).  Nothing has to be
// transposed then: lane = (column, quarter), a quad covers one column, and lane `hr` of the quad loads the
// 16-byte pieces 4m + hr (m = 0..3) of the column's 256 bytes, i.e. rows 16m + 4hr + e, together with the four
// address bytes of the same rows (one 32-bit load per m).  Step (m, e) then adds four rows per column with the
// quad merge of transpose_hist; no LDS tile, no block barrier inside the tile loop.
// GROUPS: gy is the [B][groups] gradient of a GroupSum head instead (column c takes gy[b][c / gsize] * inv_tau);
// the tile-major gradient is then written to gyT (when non-null) for the gather that follows.
template <bool GROUPS = false>
__global__ __launch_bounds__(256) void dwn_bwd_hist_tiled(const float *__restrict__ gy, const uint8_t *__restrict__ addrT,
                                                           float *__restrict__ gluts, int NO, int O, int L, int BT,
                                                           int tiles_per_chunk, float *__restrict__ partial, int chunks, DwnTables tb,
                                                           float *__restrict__ gyT = nullptr, int B = 0, int groups = 0, int gsize = 1,
                                                           float inv_tau = 1.0f) {
    __shared__ float hist[DWN_HC][65];  // [column][bin]
    if ((int)blockIdx.y >= chunks) return dwn_table_block(tb, ((int)blockIdx.y - chunks) * gridDim.x + blockIdx.x);
    const int c0 = blockIdx.x * DWN_HC;
    const int lane = threadIdx.x & 63;
    const int wave = dl_uniform(threadIdx.x >> 6);
    const int cend = min(DWN_HC, NO - c0);
    for (int e = threadIdx.x; e < DWN_HC * 65; e += 256) (&hist[0][0])[e] = 0.0f;
    __syncthreads();
    const int t_begin = blockIdx.y * tiles_per_chunk;
    const int t_end = min(BT, t_begin + tiles_per_chunk);
    const int hc = wave * (DWN_HC / 4) + (lane >> 2), hr = lane & 3;
    const int N = NO / O;
    if (hc < cend && t_begin < t_end) {  // whole quads share hc
        const int c = c0 + hc;
        const float *gcol = gy + (size_t)c * 64 + hr * 4;
        const uint8_t *acol = addrT + (size_t)(c / O) * 64 + hr * 4;
        float4 g[4], gn[4];
        unsigned aw[4], awn[4];
        const int grp = GROUPS ? c / gsize : 0;
        auto fetch = [&](int t, float4 (&gg)[4], unsigned (&aa)[4]) {
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                if (GROUPS) {
                    const int b = t * 64 + m * 16 + hr * 4;  // my four rows of this piece
                    const float *src = gy + (size_t)b * groups + grp;
                    gg[m].x = b + 0 < B ? src[0] * inv_tau : 0.0f;
                    gg[m].y = b + 1 < B ? src[groups] * inv_tau : 0.0f;
                    gg[m].z = b + 2 < B ? src[2 * groups] * inv_tau : 0.0f;
                    gg[m].w = b + 3 < B ? src[3 * groups] * inv_tau : 0.0f;
                    if (gyT) *reinterpret_cast<float4 *>(gyT + ((size_t)t * NO + c) * 64 + hr * 4 + m * 16) = gg[m];
                } else {
                    gg[m] = *reinterpret_cast<const float4 *>(gcol + (size_t)t * NO * 64 + m * 16);
                }
                aa[m] = *reinterpret_cast<const unsigned *>(acol + (size_t)t * N * 64 + m * 16);
            }
        };
        fetch(t_begin, g, aw);
        for (int t = t_begin; t < t_end; ++t) {
            if (t + 1 < t_end) fetch(t + 1, gn, awn);
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const float vs[4] = {g[m].x, g[m].y, g[m].z, g[m].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float v = vs[e];
                    const unsigned a = (aw[m] >> (8 * e)) & 0xffu;
                    float sum;
                    if (dwn_quad_merge(a, v, hr, sum)) dwn_bin_add(&hist[hc][a], sum);
                }
            }
#pragma unroll
            for (int m = 0; m < 4; ++m) { g[m] = gn[m]; aw[m] = awn[m]; }
        }
    }
    __syncthreads();
    dwn_hist_flush(hist, c0, cend, L, (long long)NO * L, chunks, partial, gluts, nullptr, O);
}

// ---------------------------------------------------------------------------------
// bwd_gx: one block per (64-input slab, 64-row batch tile), 256 threads, lane = batch row.  A wavefront
// owns 16 consecutive inputs, i.e. one contiguous run of CSR entries.  The run is read 64 entries
// at a time into registers (one entry per lane: node, slot, local input), then replayed 8 entries
// per step with wave-uniform addressing: the 8 x 3 vector loads of a step are requested together,
// then evaluated.  The entries of one input are consecutive, so its sum is
// kept in a register and written to the LDS tile once, in CSR order (reproducible sums).
#define DWN_WI 16        // inputs per wavefront (slab of 64 inputs per block)
#define DWN_WI_SMALL 4   // for layers with long CSR lists per input: slabs of 16 inputs
#define DWN_EG 8
template <int K, bool O1, bool SFORM, int WI = DWN_WI>
__global__ __launch_bounds__(256) void dwn_bwd_gx(const float *__restrict__ gyT, const uint8_t *__restrict__ addrT,
                                                   const float *__restrict__ D, const int *__restrict__ inv_ptr,
                                                   const int *__restrict__ inv_pos, float *__restrict__ gx,
                                                   int B, int I, int N, int O, int BT, int out_tiled, int gather_blocks,
                                                   DwnReduce red) {
    constexpr int IS = 4 * WI;  // inputs per block
    __shared__ float tile[IS][65];  // [input][row]
    if ((int)blockIdx.x >= gather_blocks) return dwn_reduce_block(red, (int)blockIdx.x - gather_blocks);
    constexpr int Lh = 1 << (K - 1);
    int slab, t;
    if (!dl_xcd_map((I + IS - 1) / IS, BT, slab, t)) return;
    const int i0 = slab * IS;
    const int NO = N * O;
    const int lane = threadIdx.x & 63;
    const int wave = dl_uniform(threadIdx.x >> 6);
    const int iend = min(IS, I - i0);
    const uint8_t *addr_t = addrT + (size_t)t * N * 64 + lane;
    const float *gy_t = gyT + (size_t)t * NO * 64 + lane;
    const int wbeg = wave * WI;
    // CSR pointers of my inputs: lane l (0..WI) holds inv_ptr[first + l], clamped at I
    const int myptr = inv_ptr[min(i0 + wbeg + min(lane, WI), I)];
#pragma unroll
    for (int r = 0; r < WI; ++r) tile[wbeg + r][lane] = 0.0f;  // inputs nobody reads keep 0
    const int ebeg = __builtin_amdgcn_readlane(myptr, 0);
    const int eend = __builtin_amdgcn_readlane(myptr, WI);
    struct Group {
        int rj[DWN_EG], ri[DWN_EG];
        bool live[DWN_EG];
        unsigned a[DWN_EG];
        float g[DWN_EG], coef[DWN_EG];
    };
    float acc = 0.0f;  // running sum of the input `cur`
    int cur = -1;
    // Uniform fan-in: a table of f full permutations (RandomLayer with N*k = f*I) uses every input exactly f times.
    // For f = 3 - the reference's usual ratio - a wavefront whose 16 inputs all have three entries replays its 48
    // entries fully unrolled: which input an entry belongs to and where a sum ends are then known at compile time,
    // so there is no bookkeeping per entry.  Same order of additions as the general loop below.
    constexpr int FAN = 3;
    bool uniform3 = false;
    if (WI == 16 && O1 && SFORM) {
        const int len = __shfl_down(myptr, 1) - myptr;  // lanes 0..15: entries of my input
        uniform3 = __ballot(lane >= WI || len == FAN) == ~0ull;
    }
    if (WI == 16 && O1 && SFORM && uniform3) {
        const int p = lane < WI * FAN ? inv_pos[ebeg + lane] : 0;
        const int n = p / K;
        const int rec = (n << 3) | (p - n * K);
#pragma unroll
        for (int s0 = 0; s0 < WI * FAN; s0 += DWN_EG) {
            int rj[DWN_EG];
            unsigned a[DWN_EG];
            float g[DWN_EG], coef[DWN_EG];
#pragma unroll
            for (int q = 0; q < DWN_EG; ++q) {
                const int r = __builtin_amdgcn_readlane(rec, s0 + q);
                const int rn = r >> 3;
                rj[q] = r & 7;
                a[q] = addr_t[(size_t)rn * 64];
                g[q] = gy_t[(size_t)rn * 64];
                coef[q] = D[(size_t)rn * (2 * Lh) + (lane & (2 * Lh - 1))];
            }
#pragma unroll
            for (int q = 0; q < DWN_EG; ++q) {
                const float hi = dl_lane_read(coef[q], (int)(a[q] | (1u << rj[q])));
                const float lo = dl_lane_read(coef[q], (int)(a[q] & ~(1u << rj[q])));
                const float term = g[q] * (hi - lo);
                constexpr int dummy = 0;
                (void)dummy;
                const int s = s0 + q;  // compile-time after unrolling
                acc = (s % FAN == 0) ? 0.0f + term : acc + term;
                if (s % FAN == FAN - 1) tile[wbeg + s / FAN][lane] = acc;
            }
        }
    } else
    for (int base = ebeg; base < eend; base += 64) {
        const int e = base + lane;
        const bool valid = e < eend;
        const int p = valid ? inv_pos[e] : 0;
        int ii = 0;  // local input of entry e = number of my inputs that end at or before e
#pragma unroll
        for (int l = 1; l <= WI; ++l) ii += (__builtin_amdgcn_readlane(myptr, l) <= e) ? 1 : 0;
        const int n = p / K, j = p - n * K;
        const int rec = valid ? ((n << 8) | (j << 5) | ii) : -1;
        const int cnt = min(64, eend - base);
        auto request = [&](int s0, Group &G) {
#pragma unroll
            for (int q = 0; q < DWN_EG; ++q) {
                const int r = __builtin_amdgcn_readlane(rec, min(s0 + q, 63));
                G.live[q] = r >= 0 && s0 + q < 64;
                const int rr = G.live[q] ? r : 0;
                const int rn = rr >> 8;
                G.rj[q] = (rr >> 5) & 7;
                G.ri[q] = rr & 31;
                G.a[q] = addr_t[(size_t)rn * 64];
                if (O1) {
                    G.g[q] = gy_t[(size_t)rn * 64];
                    if (SFORM)
                        G.coef[q] = D[(size_t)rn * (2 * Lh) + (lane & (2 * Lh - 1))];
                    else
                        G.coef[q] = D[((size_t)rn * K + G.rj[q]) * Lh + (lane & (Lh - 1))];
                } else {
                    G.g[q] = __int_as_float(rn);  // node number; outputs are walked in evaluate()
                }
            }
        };
        auto evaluate = [&](const Group &G) {
#pragma unroll
            for (int q = 0; q < DWN_EG; ++q) {
                if (!G.live[q]) continue;  // wave-uniform
                const int j_ = G.rj[q];
                const unsigned ap = (G.a[q] & ((1u << j_) - 1u)) | ((G.a[q] >> (j_ + 1)) << j_);
                float term;
                if (O1 && SFORM) {
                    const float hi = dl_lane_read(G.coef[q], (int)(G.a[q] | (1u << j_)));
                    const float lo = dl_lane_read(G.coef[q], (int)(G.a[q] & ~(1u << j_)));
                    term = G.g[q] * (hi - lo);
                } else if (O1) {
                    term = G.g[q] * dl_lane_read(G.coef[q], (int)ap);
                } else {
                    const int rn = __float_as_int(G.g[q]);
                    term = 0.0f;
                    for (int d = 0; d < O; ++d) {
                        const size_t c = (size_t)rn * O + d;
                        if (SFORM) {
                            const float coef = D[c * (2 * Lh) + (lane & (2 * Lh - 1))];
                            term += gy_t[c * 64] * (dl_lane_read(coef, (int)(G.a[q] | (1u << j_))) -
                                                    dl_lane_read(coef, (int)(G.a[q] & ~(1u << j_))));
                        } else {
                            const float coef = D[(c * K + j_) * Lh + (lane & (Lh - 1))];
                            term += gy_t[c * 64] * dl_lane_read(coef, (int)ap);
                        }
                    }
                }
                if (G.ri[q] != cur) {
                    if (cur >= 0) tile[wbeg + cur][lane] = acc;
                    acc = 0.0f;
                    cur = G.ri[q];
                }
                acc += term;
            }
        };
        // one group in flight per wavefront: the other resident wavefronts cover its latency, and a
        // second group in registers measured slower (fewer wavefronts fit)
        Group G;
        for (int s0 = 0; s0 < cnt; s0 += DWN_EG) {
            request(s0, G);
            evaluate(G);
        }
    }
    if (cur >= 0) tile[wbeg + cur][lane] = acc;
    if (out_tiled) {
        // gx as [B/64][I][64] for a preceding layer that takes its gy in that form: my 16 inputs, 256 B each
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int r = 0; r < WI; ++r)
            if (wbeg + r < iend)  // streamed past the L2, which holds the rows the gather re-reads
                __builtin_nontemporal_store(tile[wbeg + r][lane], &gx[((size_t)t * I + i0 + wbeg + r) * 64 + lane]);
        return;
    }
    __syncthreads();
    if (IS % 4 == 0 && iend == IS && t * 64 + 64 <= B && (I & 3) == 0 && (((uintptr_t)gx) & 15) == 0) {
        typedef float f4v __attribute__((ext_vector_type(4)));  // whole tile: 16-byte stores
#pragma unroll
        for (int pass = 0; pass < (64 * IS / 4 + 255) / 256; ++pass) {
            const int e = pass * 256 + threadIdx.x;
            if (64 * IS / 4 % 256 != 0 && e >= 64 * IS / 4) break;
            const int r = e / (IS / 4), i4 = (e % (IS / 4)) * 4;
            const f4v v = {tile[i4][r], tile[i4 + 1][r], tile[i4 + 2][r], tile[i4 + 3][r]};
            __builtin_nontemporal_store(v, reinterpret_cast<f4v *>(&gx[(size_t)(t * 64 + r) * I + i0 + i4]));
        }
        return;
    }
    for (int e = threadIdx.x; e < 64 * IS; e += 256) {
        const int r = e / IS, ii = e % IS;
        const int b = t * 64 + r;
        if (b < B && ii < iend) __builtin_nontemporal_store(tile[ii][r], &gx[(size_t)b * I + i0 + ii]);
    }
}

// ---------------------------------------------------------------------------------
// bwd_gx_walk: the input gradient by blocks that keep their slab of 64 inputs and walk batch tiles, in two roles.
// HIST (chained layers): written tile-major, with the table-gradient histogram of the layer IN FRONT folded in.  In a
// chain the input gradient of layer l + 1 is the output gradient of layer l: column i of it, together with the addresses
// layer l saved, is all layer l's histogram needs - and here it sits in the LDS the moment it is complete.  So the
// wavefront that has just summed its inputs' rows of a batch tile adds them into the bins of those columns (the quad
// merge of hist_tiled) before it moves on, and the separate pass that re-reads the [B, I] fp32 gradient for layer l's
// histogram is gone.  Bins have to live across batch tiles, so a block keeps its slab and walks `tiles_per_block` tiles
// of its class (t = cls + ncls i); it ends with its bins as one partial set ([set][column][bin]), the sets are added
// in set order afterwards (dwn_reduce_partials): fixed order, no atomics.
// ROWS (a single big layer): the row-major gradient gx [B, I] through the block's LDS tile, the blocks paced (below).
// The gather itself is dwn_bwd_gx's (O == 1): the unrolled path for WI inputs of FAN entries each per wavefront, with
// the entries' coefficient rows kept in registers over all tiles (S form: one row of 64 per entry, WI = 16 or 4; PACK:
// two D-form rows of 32 per register, WI = 32), the general loop otherwise; same order of additions.
// gx == null (HIST only): the sums are made for the bins of the layer in front and not stored.
// Pacing of the walking gather (ROWS).  Its blocks are independent; left alone they spread over several batch tiles and
// every tile's rows are fetched into an XCD's L2 more than once (measured at the headline shape, 16 inputs per
// wavefront: 692 MiB against 320 compulsory, 55 % L2 misses, 160 us).  So every block starts its tile number i no
// earlier than i * pace after its own start (the 100 MHz clock all CUs share: no memory traffic, no signal between CUs),
// which keeps the blocks of an XCD on one tile as long as the pace is one they can hold.  Too fast a pace and more and
// more blocks fall behind for good (they then run unpaced, as before); too slow costs its own length.  Measured at that
// shape with 32 inputs per wavefront (PACK), step of the layer per pace, given as the rate at which a tile step's bytes
// would move: 4600 GB/s 0.259 ms with 8 % of the sampled tile starts late, 4800 0.255 (14 %), 4900 0.253 (18 %), 5000
// 0.253 (22 %), 5100 0.258 (31 %), 5200 0.267 (54 %), no pacing 0.284.  The pace is therefore steered, per shape, on the
// device: every fourth block adds up how many of its tile starts were late, the first block of the next launch of that
// shape moves the scale by +0.5 % above the band's upper per cent of late starts (+3 % above 40: far off, and the pace
// is then held for DWN_PACE_HOLD launches before it may become faster again) and by -0.25 % below the lower one.
// Timing only: the sums and their order do not depend on it.
#define DWN_PACE_LATE_LO 15  // per cent of late tile starts: the band while the rows come from the Infinity Cache
#define DWN_PACE_LATE_HI 24
#define DWN_PACE_EDGE_LO 1   // and beyond that size
#define DWN_PACE_EDGE_HI 5
#define DWN_PACE_CACHE_MB 260.0
#define DWN_PACE_HOLD 64   // launches the pace is kept after a step back from far off
#define DWN_PACE_LINES 16  // counters of the sampled blocks, spread over as many cache lines
struct DwnPace {
    float scale;  // multiplies the launch's base pace; 0 = not yet set (1)
    int hold;  // launches for which the pace is not made faster again
    int pad[30];
    struct { int late, starts, pad[30]; } seen[DWN_PACE_LINES];  // since the scale was last moved
};
#define DWN_PACE_SLOTS 16
static __device__ DwnPace dwn_pace_state[DWN_PACE_SLOTS];
// the coefficient row of an entry (node n, slot j) as a lane holds it, and what a row gives for an address: the S form
// (one row per node, two lane reads and their difference) or the D form (one row of 2^(k-1) per slot, one lane read at the
// address with bit j taken out) - as in dwn_bwd_gx
template <int K, bool DFORM>
__device__ __forceinline__ float dwn_walk_coef(const float *__restrict__ T, int n, int j, int lane) {
    constexpr int L = 1 << K, Lh = K > 1 ? L >> 1 : 1;
    return DFORM ? T[((size_t)n * K + j) * Lh + (lane & (Lh - 1))] : T[(size_t)n * L + (lane & (L - 1))];
}
template <bool DFORM>
__device__ __forceinline__ float dwn_walk_diff(float coef, unsigned a, int j) {
    if (DFORM) {
        const unsigned ap = (a & ((1u << j) - 1u)) | ((a >> (j + 1)) << j);
        return dl_lane_read(coef, (int)ap);
    }
    return dl_lane_read(coef, (int)(a | (1u << j))) - dl_lane_read(coef, (int)(a & ~(1u << j)));
}
// D-form rows of two entries in one register: lanes 0-31 the even entry's, lanes 32-63 the odd one's
__device__ __forceinline__ float dwn_walk_diff_packed(float coef, unsigned a, int j, int odd) {
    const unsigned low = (1u << j) - 1u;
    const unsigned ap = (a & low) | ((a >> 1) & ~low);  // the address without its bit j
    return __int_as_float(__builtin_amdgcn_ds_bpermute((int)((ap << 2) | (odd ? 128u : 0u)), __float_as_int(coef)));
}
// PACK (with DFORM; with HIST only up to 16 inputs per wavefront): the D-form row of a slot has 2^(K-1) <= 32 values, so the rows of two entries share one
// register (lanes 0-31 and 32-63) and a wavefront keeps 32 inputs' entries in the registers that 16 inputs' S-form rows
// take: half as many blocks cover the inputs, and twice as many inputs are resident on an XCD.
template <int K, int WI, int FAN, bool HIST = true, bool ROWS = false, bool DFORM = false, bool PACK = false>
__global__ __launch_bounds__(256) void dwn_bwd_gx_walk(const float *__restrict__ gyT, const uint8_t *__restrict__ addrT,
                                                        const float *__restrict__ S, const int *__restrict__ inv_ptr,
                                                        const int *__restrict__ inv_pos, float *__restrict__ gx,
                                                        const uint8_t *__restrict__ prev_addrT, float *__restrict__ prev_partial,
                                                        int I, int N, int BT, int slabs, int split, int part,
                                                        int tiles_per_block, int Lp, int gather_blocks, DwnReduce red,
                                                        int B = 0, int pace = 0, int pace_slot = 0) {
    // the fixed-order sum of this layer's own histogram partials rides behind the gather's blocks
    if ((int)blockIdx.x >= gather_blocks) return dwn_reduce_block(red, (int)blockIdx.x - gather_blocks);
    constexpr int IS = 4 * WI;  // inputs per block
    constexpr int L = 1 << K;
    __shared__ float tile[IS][65];             // [input][row]
    __shared__ float hist[HIST ? IS : 1][65];  // [input = column of the layer in front][bin]
    // `split` XCDs share a class of tiles, each with its own part of the slabs (at most as many as stay resident on an
    // XCD): the blocks that read a tile on one XCD then all run at once, and a tile's rows pass through that L2 once.
    const int xcd = blockIdx.x % DL_XCDS, q = blockIdx.x / DL_XCDS;
    const int sub = xcd % split, cls = xcd / split, ncls = DL_XCDS / split;
    const int slab = sub * part + q % part, grp = q / part;
    if (slab >= slabs) return;
    const int i0 = slab * IS;
    const int lane = threadIdx.x & 63;
    const int wave = dl_uniform(threadIdx.x >> 6);
    const int iend = min(IS, I - i0);
    const int wbeg = wave * WI;
    const int myptr = inv_ptr[min(i0 + wbeg + min(lane, WI), I)];
    const int ebeg = __builtin_amdgcn_readlane(myptr, 0);
    const int eend = __builtin_amdgcn_readlane(myptr, WI);
    if (HIST) {
#pragma unroll
        for (int r = 0; r < WI; ++r) hist[wbeg + r][lane] = 0.0f;  // my columns' bins (wave-local rows of the array)
    }
    // histogram role of this lane: column (of my wavefront's WI) and the sixteen rows 16 hr .. 16 hr + 15 of a tile
    const int hcl = lane >> 2, hr = lane & 3;
    const bool hlive = hcl < WI && wbeg + hcl < iend;  // whole quads share the column
    const int hc = wbeg + min(hcl, WI - 1);
    const size_t hcol = (size_t)min(i0 + hc, I - 1) * 64 + hr * 16;  // my sixteen address bytes within a tile of prev_addrT
    // step h of a tile's histogram: row 16 hr + h of my column, the quad's equal addresses merged into one addition
    auto hist_step = [&](const float (&hv)[16], const uint4 &haw, int h) {
        const unsigned w = h < 4 ? haw.x : h < 8 ? haw.y : h < 12 ? haw.z : haw.w;
        const unsigned a = (w >> (8 * (h & 3))) & 0xffu;
        float sum;
        if (dwn_quad_merge(a, hv[h], hr, sum)) dwn_bin_add(&hist[HIST ? hc : 0][a], sum);
    };
    auto store_rows = [&](int t) {
        __syncthreads();
        if (IS % 4 == 0 && iend == IS && t * 64 + 64 <= B && (I & 3) == 0 && (((uintptr_t)gx) & 15) == 0) {
            typedef float f4v __attribute__((ext_vector_type(4)));
#pragma unroll
            for (int pass = 0; pass < (64 * IS / 4 + 255) / 256; ++pass) {
                const int e = pass * 256 + threadIdx.x;
                if (64 * IS / 4 % 256 != 0 && e >= 64 * IS / 4) break;
                const int r = e / (IS / 4), i4 = (e % (IS / 4)) * 4;
                const f4v v = {tile[i4][r], tile[i4 + 1][r], tile[i4 + 2][r], tile[i4 + 3][r]};
                __builtin_nontemporal_store(v, reinterpret_cast<f4v *>(&gx[(size_t)(t * 64 + r) * I + i0 + i4]));
            }
        } else {
            for (int e = threadIdx.x; e < 64 * IS; e += 256) {
                const int r = e / IS, ii = e % IS;
                const int b = t * 64 + r;
                if (b < B && ii < iend) __builtin_nontemporal_store(tile[ii][r], &gx[(size_t)b * I + i0 + ii]);
            }
        }
        __syncthreads();
    };
    // FAN > 0: the host found N K = FAN I, which is what a mapping built from whole permutations of the inputs gives -
    // every input read exactly FAN times; checked per wavefront, anything else takes the general loop.
    bool uniform3 = false;
    constexpr int NREC = FAN > 0 ? (WI * FAN + 63) / 64 : 1;
    int rec3[NREC] = {};  // entry e of the wavefront: lane e % 64 of rec3[e / 64]
    if constexpr (FAN > 0) {
        static_assert(!PACK || (DFORM && (!HIST || WI <= 16) && WI * FAN % 2 == 0),
                      "packed rows: D form; the histogram role covers sixteen columns per wavefront");
        const int len = __shfl_down(myptr, 1) - myptr;  // lanes 0..WI-1: entries of my input
        uniform3 = __ballot(lane >= WI || len == FAN) == ~0ull;
        if (uniform3) {
#pragma unroll
            for (int r = 0; r < NREC; ++r) {
                const int p = r * 64 + lane < WI * FAN ? inv_pos[ebeg + r * 64 + lane] : 0;
                const int n = p / K;
                rec3[r] = (n << 3) | (p - n * K);
            }
        }
    }
    const int tiles_cls = (BT - cls + ncls - 1) / ncls;  // tiles t = cls + ncls i < BT
    const int i_begin = grp * tiles_per_block, i_end = min(tiles_cls, i_begin + tiles_per_block);
    if constexpr (FAN > 0) {
        if (uniform3) {
            // Sixteen inputs of FAN entries each (then every input of the wavefront exists): unrolled.  (Running a tile's
            // histogram one tile late, from registers, between the requests of a group of entries and their use, measured
            // slower: 247 against 238 us per launch over the deep stack - the steps cost issue slots, not latency.)
            // The block keeps its entries over all its tiles, so the coefficient rows of the wavefront's 16 FAN entries
            // stay in registers: one load per entry and block instead of one per entry and tile, and the 256 B x N of
            // coefficient rows no longer share the L2 with the rows of the tiles.
            float coef[FAN > 0 ? (PACK ? WI * FAN / 2 : WI * FAN) : 1];
            if constexpr (PACK) {
                constexpr int Lh = 1 << (K - 1);
#pragma unroll
                for (int e = 0; e < WI * FAN; e += 2) {  // lanes 0-31: entry e, lanes 32-63: entry e + 1
                    const int r0 = __builtin_amdgcn_readlane(rec3[e / 64], e % 64);
                    const int r1 = __builtin_amdgcn_readlane(rec3[(e + 1) / 64], (e + 1) % 64);
                    const int r = lane < 32 ? r0 : r1;
                    coef[e / 2] = S[((size_t)(r >> 3) * K + (r & 7)) * Lh + (lane & (Lh - 1))];
                }
            } else {
#pragma unroll
                for (int e = 0; e < WI * FAN; ++e)
                    coef[e] = dwn_walk_coef<K, DFORM>(S, __builtin_amdgcn_readlane(rec3[e / 64], e % 64) >> 3,
                                                      __builtin_amdgcn_readlane(rec3[e / 64], e % 64) & 7, lane);
            }
            const unsigned long long t_start = __builtin_amdgcn_s_memrealtime();
            int late = 0;
            if (ROWS && pace > 0) {
                const int late_lo = (pace_slot >> 8) & 255, late_hi = (pace_slot >> 16) & 255;
                pace_slot &= 255;
                DwnPace *st = &dwn_pace_state[pace_slot];
                float scale = st->scale;
                if (!(scale > 0.0f)) scale = 1.0f;
                if (blockIdx.x == 0 && threadIdx.x == 0) {  // steer on what the sampled blocks of the last launch saw
                    long long starts = 0, was_late = 0;
                    for (int l = 0; l < DWN_PACE_LINES; ++l) {
                        starts += st->seen[l].starts;
                        was_late += st->seen[l].late;
                        st->seen[l].starts = 0;
                        st->seen[l].late = 0;
                    }
                    if (starts > 0) {
                        if (was_late * 100 > starts * 40) {  // far off: most blocks cannot hold the pace
                            scale *= 1.03f;
                            st->hold = DWN_PACE_HOLD;
                        } else if (was_late * 100 > starts * late_hi) {
                            scale *= 1.005f;
                            st->hold = DWN_PACE_HOLD / 4;
                        } else if (was_late * 100 < starts * late_lo) {
                            if (st->hold > 0) --st->hold;  // stay a while where the last step back led
                            else scale *= 0.9975f;
                        }
                        scale = fminf(fmaxf(scale, 0.6f), 1.6f);
                    }
                    st->scale = scale;
                }
                pace = (int)((float)pace * scale);
            }
            for (int ti = i_begin; ti < i_end; ++ti) {
                if (ROWS && pace > 0 && ti > i_begin) {
                    const unsigned long long due = (unsigned long long)(ti - i_begin) * pace;
                    if (__builtin_amdgcn_s_memrealtime() - t_start >= due) ++late;
                    while (__builtin_amdgcn_s_memrealtime() - t_start < due) __builtin_amdgcn_s_sleep(8);
                }
                const int t = cls + ncls * ti;
                const uint8_t *addr_t = addrT + (size_t)t * N * 64 + lane;
                const float *gy_t = gyT + (size_t)t * N * 64 + lane;
                float *gx_t = gx + ((size_t)t * I + i0 + wbeg) * 64 + lane;
                uint4 haw = {0u, 0u, 0u, 0u};
                if (HIST) haw = *reinterpret_cast<const uint4 *>(prev_addrT + (size_t)t * I * 64 + hcol);
                float acc = 0.0f;
#pragma unroll
                for (int s0 = 0; s0 < WI * FAN; s0 += DWN_EG) {
                    int rj[DWN_EG];
                    unsigned a[DWN_EG];
                    float g[DWN_EG];
#pragma unroll
                    for (int qq = 0; qq < DWN_EG; ++qq) {
                        const int r = __builtin_amdgcn_readlane(rec3[(s0 + qq) / 64], (s0 + qq) % 64);
                        const int rn = r >> 3;
                        rj[qq] = r & 7;
                        a[qq] = addr_t[(size_t)rn * 64];
                        g[qq] = gy_t[(size_t)rn * 64];
                    }
#pragma unroll
                    for (int qq = 0; qq < DWN_EG; ++qq) {
                        const int sidx = s0 + qq;  // compile-time after unrolling
                        const float term = g[qq] * (PACK ? dwn_walk_diff_packed(coef[PACK ? sidx / 2 : 0], a[qq], rj[qq], sidx & 1)
                                                         : dwn_walk_diff<DFORM>(coef[PACK ? 0 : sidx], a[qq], rj[qq]));
                        acc = (sidx % FAN == 0) ? 0.0f + term : acc + term;
                        if (sidx % FAN == FAN - 1) {
                            if (HIST || ROWS) tile[wbeg + sidx / FAN][lane] = acc;
                            // gx as [B/64][I][64], streamed past the L2 (which holds the rows the gather re-reads)
                            if (!ROWS && gx) __builtin_nontemporal_store(acc, gx_t + (size_t)(sidx / FAN) * 64);
                        }
                    }
                }
                if (ROWS) store_rows(t);
                if (HIST) {
                    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    if (hcl < WI) {  // (every lane when WI = 16)
                        float hv[16];
#pragma unroll
                        for (int h = 0; h < 16; ++h) hv[h] = tile[hc][hr * 16 + h];
#pragma unroll
                        for (int h = 0; h < 16; ++h) hist_step(hv, haw, h);
                    }
                    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                    __builtin_amdgcn_wave_barrier();  // the next tile overwrites the rows just read
                }
            }
            if (ROWS && pace > 0 && (blockIdx.x / DL_XCDS) % 4 == 0 && threadIdx.x == 0 && i_end - i_begin > 1) {
                // every fourth slab of every XCD reports
                auto &seen = dwn_pace_state[pace_slot].seen[(blockIdx.x / (4 * DL_XCDS) * DL_XCDS + blockIdx.x % DL_XCDS) % DWN_PACE_LINES];
                atomicAdd(&seen.late, late);
                atomicAdd(&seen.starts, i_end - i_begin - 1);
            }
    }
    }
    if (!(FAN > 0 && uniform3)) {
        for (int ti = i_begin; ti < i_end; ++ti) {
            const int t = cls + ncls * ti;
            const uint8_t *addr_t = addrT + (size_t)t * N * 64 + lane;
            const float *gy_t = gyT + (size_t)t * N * 64 + lane;
            // the addresses of the layer in front for my column and rows: asked for now, used after the gather
            uint4 haw = {0u, 0u, 0u, 0u};
            if (HIST) haw = *reinterpret_cast<const uint4 *>(prev_addrT + (size_t)t * I * 64 + hcol);
#pragma unroll
            for (int r = 0; r < WI; ++r) tile[wbeg + r][lane] = 0.0f;  // inputs nobody reads keep 0
            float acc = 0.0f;
            int cur = -1;
            for (int base = ebeg; base < eend; base += 64) {
                const int e = base + lane;
                const bool valid = e < eend;
                const int p = valid ? inv_pos[e] : 0;
                int ii = 0;  // local input of entry e = number of my inputs that end at or before e
#pragma unroll
                for (int l = 1; l <= WI; ++l) ii += (__builtin_amdgcn_readlane(myptr, l) <= e) ? 1 : 0;
                const int n = p / K, j = p - n * K;
                const int rec = (n << 8) | (j << 5) | ii;
                const int cnt = min(64, eend - base);
                for (int s0 = 0; s0 < cnt; s0 += DWN_EG) {
                    int rj[DWN_EG], ri[DWN_EG];
                    unsigned a[DWN_EG];
                    float g[DWN_EG], coef[DWN_EG];
#pragma unroll
                    for (int qq = 0; qq < DWN_EG; ++qq) {
                        const int r = __builtin_amdgcn_readlane(rec, min(s0 + qq, cnt - 1));
                        const int rn = r >> 8;
                        rj[qq] = (r >> 5) & 7;
                        ri[qq] = r & 31;
                        a[qq] = addr_t[(size_t)rn * 64];
                        g[qq] = gy_t[(size_t)rn * 64];
                        coef[qq] = dwn_walk_coef<K, DFORM>(S, rn, rj[qq], lane);
                    }
#pragma unroll
                    for (int qq = 0; qq < DWN_EG; ++qq) {
                        if (s0 + qq >= cnt) break;  // wave-uniform
                        const float diff = dwn_walk_diff<DFORM>(coef[qq], a[qq], rj[qq]);
                        if (ri[qq] != cur) {
                            if (cur >= 0) tile[wbeg + cur][lane] = acc;
                            acc = 0.0f;
                            cur = ri[qq];
                        }
                        acc += g[qq] * diff;
                    }
                }
            }
            if (cur >= 0) tile[wbeg + cur][lane] = acc;
            if (ROWS) {
                store_rows(t);
            } else {
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                __builtin_amdgcn_wave_barrier();
                // gx as [B/64][I][64]: my inputs, 256 B each, streamed past the L2 (which holds the rows the gather
                // re-reads); gx == null: the sums are only wanted for the bins of the layer in front
                if (gx) {
#pragma unroll
                    for (int r = 0; r < WI; ++r)
                        if (wbeg + r < iend)
                            __builtin_nontemporal_store(tile[wbeg + r][lane], &gx[((size_t)t * I + i0 + wbeg + r) * 64 + lane]);
                }
            }
            // the same rows into the bins of the layer in front (rows past the batch carry 0 and add nothing)
            if (HIST && hlive) {
                float hv[16];
#pragma unroll
                for (int h = 0; h < 16; ++h) hv[h] = tile[hc][hr * 16 + h];
#pragma unroll
                for (int h = 0; h < 16; ++h) hist_step(hv, haw, h);
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();  // the next tile clears the rows just read
        }
    
    }
    if (!HIST) return;
    // my columns' bins as one partial set
    const int set = grp * ncls + cls;
    float *out = prev_partial + ((size_t)set * I + i0 + wbeg) * Lp;
    const int ncols = max(0, min(WI, iend - wbeg));
    for (int e = lane; e < ncols * Lp; e += 64) out[e] = hist[wbeg + e / Lp][e % Lp];
}

// ---------------------------------------------------------------------------------
// Host side
static inline int dwn_bt(int B) { return (B + 63) / 64; }
static inline size_t dwn_planes_bytes(int B, int I) { return dl_align256((size_t)dwn_bt(B) * I * sizeof(u64)); }
// room for either coefficient form: k * 2^(k-1) floats per column (D form) or 2^k (S form, the larger one at k = 1)
static inline size_t dwn_table_bytes(int N, int k, int O) {
    const size_t d_form = (size_t)k << (k - 1), s_form = (size_t)1 << k;
    return dl_align256((size_t)N * O * (d_form > s_form ? d_form : s_form) * sizeof(float));
}
static inline size_t dwn_gyT_bytes(int B, int N, int O) {
    return dl_align256((size_t)N * O * dwn_bt(B) * 64 * sizeof(float));
}
// grid of the histogram kernels: column tiles x chunks of batch tiles.  Enough blocks to fill 256 CUs several times
// over; four blocks fit a CU (LDS), so at most about 1024 of them - all resident at once, no second, mostly empty round.
static inline void dwn_hist_grid(long long NO, int BT, int &col_tiles, int &chunks, int &tpc) {
    col_tiles = dl_ceil_div(NO, DWN_HC);
    chunks = col_tiles >= 1024 ? 1 : 1024 / col_tiles;
    if (chunks > BT) chunks = BT;
    tpc = dl_ceil_div(BT, chunks);
    chunks = dl_ceil_div(BT, tpc);
}
// A big layer's backward with row-major gradients is taken in chunks of about DWN_ROW_CHUNK_BYTES worth of batch tiles,
// histogram and gather of one chunk after the other (whichever gather the layer takes; 8192 -> 8192 nodes with the
// in-order one, B = 8192: 0.592 -> 0.502 ms): the tile-major copy of a chunk's
// gy (and its saved addresses) is then still in the 256 MB Infinity Cache when the gather reads it.  Measured at
// 16384 -> 8192 nodes: the gather takes 109 us for 4096 rows but 284 us for 8192 and 566 us for 16384 in one piece.
// Every chunk leaves its own partial sets of the table gradient; the last chunk's launch adds all of them, in order.
#define DWN_ROW_CHUNK_BYTES 172e6  // gy tile-major + saved addresses of a chunk (the headline's 4096 rows: 168 MB)
static inline int dwn_walk_rows(int BT, int I, int N, int k, int O, int gx_tiled);
static inline int dwn_row_chunks(int BT, int I, int N, int k, int O) {
    (void)I, (void)k;
    int tiles = (int)(DWN_ROW_CHUNK_BYTES / ((double)N * O * 320));
    if (tiles < 32) tiles = 32;  // (the walking gather wants 32 tiles)
    if (2 * BT < 3 * tiles) return 1;
    if (dl_ceil_div((long long)N * O, DWN_HC) > 512) return 1;  // (a chunk's histogram must leave partial sets)
    return (BT + tiles / 2) / tiles;
}
// the tiles of chunk c of n: as even as they come (BT / n each, the first BT % n one more), so that no chunk is tiny
static inline int dwn_row_chunk_tiles(int BT, int n, int c) { return BT / n + (c < BT % n ? 1 : 0); }
static inline int dwn_row_chunk_begin(int BT, int n, int c) { return c * (BT / n) + (c < BT % n ? c : BT % n); }
// chunk partials of the table gradient (none when one chunk covers the batch)
static inline size_t dwn_partial_bytes(int B, int I, int N, int k, int O) {
    int col_tiles, chunks, tpc;
    const int BT = dwn_bt(B), n = dwn_row_chunks(BT, I, N, k, O);
    if (n > 1) {
        size_t sets = 0;
        for (int c = 0; c < n; ++c) {
            dwn_hist_grid((long long)N * O, dwn_row_chunk_tiles(BT, n, c), col_tiles, chunks, tpc);
            sets += chunks;
        }
        return dl_align256(sets * N * O * sizeof(float) << k);
    }
    dwn_hist_grid((long long)N * O, BT, col_tiles, chunks, tpc);
    return chunks > 1 ? dl_align256((size_t)chunks * N * O * sizeof(float) << k) : 0;
}

static int dwn_check(int B, int I, int N, int k, int O) {
    if (B <= 0 || I <= 0 || N <= 0 || k <= 0 || O <= 0) return DL_ERR_SHAPE;
    if (k > DL_MAX_K) return DL_ERR_UNSUPPORTED;
    if (I > (1 << 28)) return DL_ERR_UNSUPPORTED;  // byte offsets into one batch tile's bit-planes are 32-bit
    if ((long long)N * O * ((long long)1 << k) > 0x7fffffffLL) return DL_ERR_UNSUPPORTED;
    // batch tiles, padded row counts and the 1-D grids (column or input tiles x batch tiles rounded up to the 8 XCDs, plus
    // the blocks that ride behind them) are 32-bit: refuse what would overflow them
    if (B > 0x7fffffff - 64) return DL_ERR_UNSUPPORTED;
    const long long bt8 = DL_XCDS * (((long long)B + 63) / 64 + DL_XCDS - 1) / DL_XCDS;
    const long long lookup_blocks = (((long long)N * O + DWN_TC - 1) / DWN_TC) * bt8;
    const long long gather_blocks = (((long long)I + 3) / 4) * bt8 + (((long long)N * O << k) + 1023) / 1024;
    if (lookup_blocks > 0x7fffffffLL || gather_blocks > 0x7fffffffLL) return DL_ERR_UNSUPPORTED;
    return DL_OK;
}
// the fast kernels pack a node number into 23 bits of an entry record and address table rows and
// saved addresses with 32-bit byte offsets (column * 2^k * 4 and node * 64)
static inline bool dwn_fast(int N, int k, int O) {
    return k <= DL_MAX_FAST_K && N < (1 << 23) && (long long)N * O * ((long long)4 << k) < 0x7fffffffLL;
}

extern "C" size_t dl_dwn_saved_bytes(int B, int I, int N, int k, int O) {
    (void)I;
    if (!dwn_fast(N, k, O)) return 256;  // nothing is kept; a token allocation keeps callers simple
    return dl_align256((size_t)N * dwn_bt(B) * 64);
}
extern "C" size_t dl_dwn_fwd_workspace_bytes(int B, int I, int N, int k, int O) {
    return dwn_fast(N, k, O) ? dwn_planes_bytes(B, I) : 256;
}
extern "C" size_t dl_dwn_bwd_workspace_bytes(int B, int I, int N, int k, int O) {
    return dwn_fast(N, k, O) ? dwn_table_bytes(N, k, O) + dwn_gyT_bytes(B, N, O) + dwn_partial_bytes(B, I, N, k, O)
                             : dl_align256(dwn_generic_smooth_bytes(N, k, O));  // k > 6: the smoothed tables
}

template <int K>
static void dwn_launch_lookup(const u64 *planes, const int *idx32, const float *luts, float *y, uint8_t *addrT,
                              u64 *planes_out, int B, int I, int N, int O, hipStream_t s, int gsize = 0, int slots = 0,
                              bool eval = false, const int *run_if_set = nullptr) {
    const int BT = dwn_bt(B);
    const int grid = dl_xcd_grid(dl_ceil_div((long long)N * O, DWN_TC), BT);
    if (eval) {  // addrT is not written
#define DWN_EVAL(O1_, CHAIN_, GSUM_)                                                                                     \
    DL_TIMED("dwn_lookup_eval", s, (dwn_lookup_fwd<K, O1_, CHAIN_, GSUM_, true><<<grid, 64 * DWN_FW, 0, s>>>(            \
                                       planes, idx32, luts, y, addrT, planes_out, B, I, N, O, BT, gsize > 0 ? gsize : 1, \
                                       slots > 0 ? slots : 1, run_if_set)))
        if (gsize > 0 && O == 1) DWN_EVAL(true, false, true);
        else if (gsize > 0) DWN_EVAL(false, false, true);
        else if (O == 1) DWN_EVAL(true, true, false);
        else DWN_EVAL(false, true, false);
#undef DWN_EVAL
        return;
    }
    if (gsize > 0) {  // y holds the per-tile group sums
        if (O == 1)
            DL_TIMED("dwn_lookup_fwd", s, (dwn_lookup_fwd<K, true, false, true><<<grid, 64 * DWN_FW, 0, s>>>(
                                              planes, idx32, luts, y, addrT, nullptr, B, I, N, O, BT, gsize, slots)));
        else
            DL_TIMED("dwn_lookup_fwd", s, (dwn_lookup_fwd<K, false, false, true><<<grid, 64 * DWN_FW, 0, s>>>(
                                              planes, idx32, luts, y, addrT, nullptr, B, I, N, O, BT, gsize, slots)));
        return;
    }
#define DWN_LOOKUP(O1_, CHAIN_)                                                                                        \
    DL_TIMED("dwn_lookup_fwd", s,                                                                                      \
             (dwn_lookup_fwd<K, O1_, CHAIN_><<<grid, 64 * DWN_FW, 0, s>>>(planes, idx32, luts, y, addrT, planes_out, B, I, \
                                                                         N, O, BT)))
    const bool chain = planes_out != nullptr || y == nullptr;
    if (O == 1 && !chain) DWN_LOOKUP(true, false);
    else if (O == 1) DWN_LOOKUP(true, true);
    else if (!chain) DWN_LOOKUP(false, false);
    else DWN_LOOKUP(false, true);
#undef DWN_LOOKUP
}

// forward of the k <= 6 path: x -> bit-planes (scratch) -> y and the saved addresses
static int dwn_forward_fast(const float *x, const int32_t *idx32, const float *luts, float *y, void *saved, u64 *planes,
                            int B, int I, int N, int k, int O, hipStream_t s) {
    const int BT = dwn_bt(B);
    if (I % 4 == 0 && ((uintptr_t)x & 15) == 0)
        DL_TIMED("dwn_pack_planes", s, (dwn_pack_planes<4><<<dim3(dl_ceil_div(I, 1024), dwn_pack_grid_y(BT)), 256, 0, s>>>(x, planes, B, I)));
    else
        DL_TIMED("dwn_pack_planes", s, (dwn_pack_planes<1><<<dim3(dl_ceil_div(I, 256), dwn_pack_grid_y(BT)), 256, 0, s>>>(x, planes, B, I)));
    uint8_t *addrT = (uint8_t *)saved;
    switch (k) {
        case 1: dwn_launch_lookup<1>(planes, idx32, luts, y, addrT, nullptr, B, I, N, O, s); break;
        case 2: dwn_launch_lookup<2>(planes, idx32, luts, y, addrT, nullptr, B, I, N, O, s); break;
        case 3: dwn_launch_lookup<3>(planes, idx32, luts, y, addrT, nullptr, B, I, N, O, s); break;
        case 4: dwn_launch_lookup<4>(planes, idx32, luts, y, addrT, nullptr, B, I, N, O, s); break;
        case 5: dwn_launch_lookup<5>(planes, idx32, luts, y, addrT, nullptr, B, I, N, O, s); break;
        default: dwn_launch_lookup<6>(planes, idx32, luts, y, addrT, nullptr, B, I, N, O, s); break;
    }
    return dl_launch_status();
}

extern "C" int dl_dwn_layer_fwd(const float *x, const int32_t *idx32, const float *luts, float *y, void *saved,
                                void *ws, size_t ws_bytes, int B, int I, int N, int k, int O, void *stream) {
    if (!x || !idx32 || !luts || !y) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (!dwn_fast(N, k, O)) return dwn_generic_forward(x, idx32, luts, y, B, I, N, k, O, s);
    if (!saved || !ws) return DL_ERR_NULL;
    if (ws_bytes < dl_dwn_fwd_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    return dwn_forward_fast(x, idx32, luts, y, saved, (u64 *)ws, B, I, N, k, O, s);
}

// ---- the same forward for callers that cannot allocate a workspace.  The bit-planes go to a device array that
// belongs to the library: every GPU the library runs on holds its own copy of it (DL_DWN_STATIC_SCRATCH_BYTES, until
// the process ends) at its own address, looked up once per device.  `scratch` itself is only the host-side handle
// of the symbol - kernels are always given the looked-up device address.
static __device__ __align__(256) unsigned char scratch[DL_DWN_STATIC_SCRATCH_BYTES];
#define DWN_MAX_DEVICES 64
static void *g_scratch_ptr[DWN_MAX_DEVICES];  // device address of `scratch` on each device, null until looked up
static std::mutex g_scratch_mutex;

static int dwn_scratch_address(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= DWN_MAX_DEVICES) return DL_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));  // the current device's copy
        if (e != hipSuccess) return (int)e;
        if (!p) return DL_ERR_NULL;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return DL_OK;
}

extern "C" int dl_dwn_layer_fwd_static(const float *x, const int32_t *idx32, const float *luts, float *y, void *saved,
                                       int B, int I, int N, int k, int O, void *stream) {
    if (!x || !idx32 || !luts || !y) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (!dwn_fast(N, k, O)) return dwn_generic_forward(x, idx32, luts, y, B, I, N, k, O, s);  // uses no scratch
    if (!saved) return DL_ERR_NULL;
    if (dwn_planes_bytes(B, I) > (size_t)DL_DWN_STATIC_SCRATCH_BYTES) return DL_ERR_SCRATCH;
    void *planes = nullptr;
    rc = dwn_scratch_address(&planes);
    if (rc) return rc;
    // every plane word of the ceil(B/64) tiles is rewritten by the pack kernel, so nothing has to be cleared
    return dwn_forward_fast(x, idx32, luts, y, saved, (u64 *)planes, B, I, N, k, O, s);
}

template <int K>
static void dwn_launch_gx(const float *gyT, const uint8_t *addrT, const float *D, const int *inv_ptr, const int *inv_pos,
                          float *gx, int B, int I, int N, int O, bool sform, int out_tiled, const DwnReduce &red,
                          hipStream_t s) {
    const int BT = dwn_bt(B);
    const int rb = dwn_reduce_blocks(red);  // the fixed-order sum of the histogram partials rides behind the gather's blocks
    // Long CSR lists per input (average N*k/I: ~70 on the first level of a convolutional layer, 15 under a learnable
    // mapping) want fewer inputs per wavefront: more, shorter and evenly filled blocks.  Measured at B = 4096, k = 6:
    // lists of 3 - 16 inputs per wavefront is best (169 vs 221 us); 7.7 - 4 inputs (67 vs 73 us); 15 - 4 (134 vs
    // 179 us); 31 - 4 (368 vs 442 us); 69 with tile-major output - 1 (249 vs 265 vs 375 us).
    if (O == 1 && sform && out_tiled && (long long)N * K >= 32LL * I) {
        const int grid_s = dl_xcd_grid(dl_ceil_div(I, 4), BT);
        DL_TIMED("dwn_bwd_gx", s, (dwn_bwd_gx<K, true, true, 1><<<grid_s + rb, 256, 0, s>>>(gyT, addrT, D, inv_ptr, inv_pos, gx, B,
                                                                                          I, N, O, BT, out_tiled, grid_s, red)));
        return;
    }
    if (O == 1 && sform && (long long)N * K >= 6LL * I) {
        const int grid_s = dl_xcd_grid(dl_ceil_div(I, 4 * DWN_WI_SMALL), BT);
        DL_TIMED("dwn_bwd_gx", s, (dwn_bwd_gx<K, true, true, DWN_WI_SMALL><<<grid_s + rb, 256, 0, s>>>(
                                      gyT, addrT, D, inv_ptr, inv_pos, gx, B, I, N, O, BT, out_tiled, grid_s, red)));
        return;
    }
    const int grid = dl_xcd_grid(dl_ceil_div(I, 4 * DWN_WI), BT);
#define DWN_GX(O1_, S_) \
    DL_TIMED("dwn_bwd_gx", s, (dwn_bwd_gx<K, O1_, S_><<<grid + rb, 256, 0, s>>>(gyT, addrT, D, inv_ptr, inv_pos, gx, B, I, N, O, BT, out_tiled, grid, red)))
    if (O == 1 && sform) DWN_GX(true, true);
    else if (O == 1) DWN_GX(true, false);
    else if (sform) DWN_GX(false, true);
    else DWN_GX(false, false);
#undef DWN_GX
}

// backward of the k <= 6 path; gy row-major [B, N*O] or (gy_tiled) tile-major [B/64][N*O][64];
// gx row-major [B, I] or (gx_tiled) tile-major [B/64][I][64]
// scale == null: EFD weights alpha * beta^h; otherwise the stabilised weights scale[n] / (h + 1),
// which also multiply the table gradient
struct DwnGroupHead {
    int groups, gsize;
    float inv_tau;
};
// The layer in front of this one in a chain (its N_prev * 1 outputs are this layer's I inputs): with its saved addresses
// the gather can fill that layer's table-gradient bins from the input gradient it has just summed (dwn_bwd_gx_walk).
struct DwnFusedPrev {
    const uint8_t *addrT;  // [B/64][I][64], what that layer's forward saved
    float *gluts;          // [I][2^k_prev] out
    int k;
    float *partial;        // [sets][I][2^k_prev] scratch
};
__global__ __launch_bounds__(256) void dwn_build_tables(DwnTables tb) { dwn_table_block(tb, blockIdx.x); }
// one chunk of rows of a backward taken in several (dwn_row_chunks)
struct DwnRowChunk {
    float *partial_base;  // the partial sets of all chunks
    int set_offset;       // where this chunk's sets start
    int total_sets;       // > 0: the last chunk, whose launch adds all sets
    bool first;           // builds the coefficient tables
};
// How the fused gather is laid over the chip.  An XCD keeps DWN_RESIDENT of its blocks at a time; blocks that read the
// same tile through the same L2 should all be among them, or the tile's rows are fetched once per round of blocks.  So
// `split` XCDs (1, 2, 4 or 8) share a class of tiles, each taking `part` <= DWN_RESIDENT of the slabs, and where a part
// is smaller than that, `groups` blocks per slab share the class's tiles (each ends with a partial set of bins that has
// to be written and summed again; at most 128 MB of them).  One round of blocks, every block the same number of tiles.
#define DWN_RESIDENT 128  // 32 CUs x 4 blocks (33 KB of LDS each)
struct DwnFusedSplit {
    int slabs, split, part, groups, tpb, sets;
};
static inline DwnFusedSplit dwn_fused_split(int BT, int I, int k_prev, int IS) {
    DwnFusedSplit f;
    f.slabs = dl_ceil_div(I, IS);
    f.split = 1;
    while (f.split < DL_XCDS && dl_ceil_div(f.slabs, f.split) > DWN_RESIDENT) f.split *= 2;
    f.part = dl_ceil_div(f.slabs, f.split);
    const int ncls = DL_XCDS / f.split, tiles_cls = dl_ceil_div(BT, ncls);
    const long long set_bytes = (long long)I * ((long long)4 << k_prev);
    int by_memory = (int)((128LL << 20) / (set_bytes * ncls > 0 ? set_bytes * ncls : 1));
    f.groups = DWN_RESIDENT / f.part;
    if (f.groups > by_memory) f.groups = by_memory;
    if (f.groups > tiles_cls) f.groups = tiles_cls;
    if (f.groups < 1) f.groups = 1;
    f.tpb = dl_ceil_div(tiles_cls, f.groups);
    f.groups = dl_ceil_div(tiles_cls, f.tpb);
    f.sets = f.groups * ncls;
    return f;
}
// inputs per wavefront of the fused gather: the rule of dwn_launch_gx; 0 = lists too long for it (not fused)
static inline int dwn_fused_wi(int I, int N, int K) {
    if ((long long)N * K >= 32LL * I) return 0;
    return (long long)N * K >= 6LL * I ? DWN_WI_SMALL : DWN_WI;
}
// Inputs that are all read six times (equal widths at k = 6) take the packed rows: two D-form rows per register, so a
// wavefront keeps 16 inputs' 96 entries instead of 4 inputs' 24, and a quarter as many blocks cover the inputs (an
// 8000-input layer then fits one XCD's resident blocks, and a tile is read through one L2 instead of four).
static inline bool dwn_fused_pack(int I, int N, int K) {
    return dwn_fused_wi(I, N, K) == DWN_WI_SMALL && (long long)N * K == 6LL * I;
}
static inline size_t dwn_fused_partial_bytes(int B, int I, int N, int k, int k_prev) {
    const int wi = dwn_fused_pack(I, N, k) ? DWN_WI : dwn_fused_wi(I, N, k);
    if (!wi) return 0;
    const DwnFusedSplit f = dwn_fused_split(dwn_bt(B), I, k_prev, 4 * wi);
    return dl_align256((size_t)f.sets * I * ((size_t)4 << k_prev));
}
// When the row-major input gradient is taken by the walking, paced gather instead of one block per (slab, tile): one
// output per node, every input read three times on the host's count (N k = 3 I; wavefronts check their own inputs), and
// a layer big enough that the rows of a tile crowd an XCD's L2.  Forward + backward of the layer, in-order gather ->
// walking gather with 16 inputs per wavefront -> with 32 (PACK, when the 64-input slabs outnumber an XCD's resident
// blocks): 16384 -> 8192 nodes, B = 4096: 0.294 -> 0.278 -> 0.253 ms; B = 8192: 0.675 -> 0.568 -> 0.578 (0.513 in chunks
// of rows, dwn_row_chunks); B = 16384: 1.357 -> 1.195 -> 1.15 (1.046); 32768 -> 16384, B = 4096: 0.736 -> 0.594 -> 0.593
// (0.589); 24576 -> 12288: 0.416.  Inputs read once or
// twice lose by it (24576 -> 8192: 0.340 -> 0.363 ms; 49152 -> 8192: 0.471 -> 0.531) and keep the in-order gather, and
// so do layers with less than 2 MB of rows per tile (8192 -> 4096: 0.143 -> 0.148 ms at B = 4096, 0.259 -> 0.269 at
// 8192; 10000 -> 5000, B = 8192: 0.338 -> 0.387) and batches of fewer than 32 tiles (B = 2048, 32 tiles: 0.161 -> 0.153 ->
// 0.144 ms; B = 1024: no difference).
#define DWN_PACE_GBS 5000.0  // base pace: the bytes of a tile step at this rate
// Inputs read six times (equal widths at k = 6) take it with the packed rows and sixteen inputs per wavefront once the
// 64-input slabs outnumber an XCD's resident blocks: 12288 -> 12288 at B = 4096 0.433 -> 0.352 ms, 16384 -> 16384 0.640 ->
// 0.591; at 8192 -> 8192 the in-order gather stays ahead (0.253 against 0.268 ms).
// Returns the fan-in it applies to (3 or 6), 0 = the in-order gather.
static inline int dwn_walk_rows(int BT, int I, int N, int k, int O, int gx_tiled) {
    if (O != 1 || gx_tiled) return 0;
    if ((long long)N * 320 < (2LL << 20) || BT < 32) return 0;
    if ((long long)N * k == 3LL * I) return 3;
    if ((long long)N * k == 6LL * I && I > 64 * DWN_RESIDENT) return 6;
    return 0;
}
static int dwn_backward_fast(const void *saved, const int32_t *inv_ptr, const int32_t *inv_pos, const float *luts,
                             const float *gy, int gy_tiled, float alpha, float beta, const float *scale, float *gx,
                             int gx_tiled, float *gluts, void *ws, int B, int I, int N, int k, int O, hipStream_t s,
                             const DwnGroupHead *head = nullptr, const float *alpha_n = nullptr,
                             const float *beta_n = nullptr, const DwnFusedPrev *prev = nullptr,
                             const DwnRowChunk *rc = nullptr) {
    const long long NO = (long long)N * O;
    const int L = 1 << k;
    const uint8_t *addrT = (const uint8_t *)saved;
    float *D = (float *)ws;
    float *gyT = (float *)((char *)ws + dwn_table_bytes(N, k, O));
    const int BT = dwn_bt(B), BP = BT * 64;
    float *partial = (float *)((char *)ws + dwn_table_bytes(N, k, O) + dwn_gyT_bytes(B, N, O));
    int col_tiles, chunks, tpc;
    if (!rc && gx && gluts && !prev && !head && !gy_tiled && !gx_tiled) {
        const int n = dwn_row_chunks(BT, I, N, k, O);
        if (n > 1) {  // in chunks of rows, each through this function again
            int total = 0, sets = 0;
            for (int c = 0; c < n; ++c) {
                dwn_hist_grid(NO, dwn_row_chunk_tiles(BT, n, c), col_tiles, chunks, tpc);
                total += chunks;
            }
            for (int c = 0; c < n; ++c) {
                const int t0 = dwn_row_chunk_begin(BT, n, c), tiles = dwn_row_chunk_tiles(BT, n, c);
                const int rows = std::min(B - t0 * 64, tiles * 64);
                const DwnRowChunk r = {partial, sets, c == n - 1 ? total : 0, c == 0};
                const int rcode = dwn_backward_fast(addrT + (size_t)t0 * N * 64, inv_ptr, inv_pos, luts, gy + (size_t)t0 * 64 * NO, 0,
                                                    alpha, beta, scale, gx + (size_t)t0 * 64 * I, 0, gluts, ws, rows, I, N, k, O, s,
                                                    nullptr, alpha_n, beta_n, nullptr, &r);
                if (rcode) return rcode;
                dwn_hist_grid(NO, tiles, col_tiles, chunks, tpc);
                sets += chunks;
            }
            return DL_OK;
        }
    }
    if (rc) partial = rc->partial_base + (size_t)rc->set_offset * NO * L;
    dwn_hist_grid(NO, BT, col_tiles, chunks, tpc);
    const bool sform = !scale && beta >= -0.5f && beta <= 0.5f;
    // The coefficient tables of the gather depend on the tables only, so their blocks ride in the histogram's launch
    // (extra rows of its grid, dispatched last: they fill the tail in which the histogram blocks drain); the
    // fixed-order sum of the histogram partials rides in the gather's launch the same way.
    // the walking gather of a layer too wide for one XCD's resident blocks packs two D-form rows into a register; for
    // |beta| <= 1/2 its table then holds the differences of the S form (the bits the other gathers compute from it)
    const int walk_rows = gx ? dwn_walk_rows(BT, I, N, k, O, gx_tiled) : 0;
    const bool walk_pack = walk_rows == 6 || (walk_rows == 3 && dl_ceil_div(I, 4 * DWN_WI) > DWN_RESIDENT);
    const bool gather = gx || prev;  // (prev without gx: the input gradient is summed for the bins in front, not stored)
    const int fused_wi = prev && (gx_tiled || !gx) && O == 1 && sform ? dwn_fused_wi(I, N, k) : 0;
    const bool fused_pack = fused_wi && dwn_fused_pack(I, N, k);
    DwnTables tb = {gather && (!rc || rc->first) ? luts : nullptr, D, scale, alpha_n, beta_n, alpha, beta, (int)NO, k, O,
                    sform ? (walk_pack || fused_pack ? 2 : 1) : 0};
    const dim3 hgrid(col_tiles, chunks + dl_ceil_div(dwn_table_blocks(tb), col_tiles));
    if (!gluts) {
        // the table gradient of this layer is already there (the gather of the layer behind filled its bins): only the
        // coefficient tables remain to be built.  gy is tile-major in that case.
        if (dwn_table_blocks(tb)) DL_TIMED("dwn_build_tables", s, (dwn_build_tables<<<dwn_table_blocks(tb), 256, 0, s>>>(tb)));
    } else if (head)
        DL_TIMED("dwn_bwd_hist_groups", s, (dwn_bwd_hist_tiled<true><<<hgrid, 256, 0, s>>>(
                                               gy, addrT, gluts, (int)NO, O, L, BT, tpc, partial, chunks, tb, gather ? gyT : nullptr, B,
                                               head->groups, head->gsize, head->inv_tau)));
    else if (gy_tiled)
        DL_TIMED("dwn_bwd_hist_tiled", s,
                 (dwn_bwd_hist_tiled<false><<<hgrid, 256, 0, s>>>(gy, addrT, gluts, (int)NO, O, L, BT, tpc, partial, chunks, tb)));
    else if (gather)
        DL_TIMED("dwn_bwd_transpose_hist", s, (dwn_bwd_transpose_hist<true><<<hgrid, 256, 0, s>>>(
                                                  gy, addrT, gyT, gluts, B, (int)NO, O, L, BP, BT, tpc, partial, scale, chunks, tb)));
    else
        DL_TIMED("dwn_bwd_transpose_hist", s, (dwn_bwd_transpose_hist<false><<<hgrid, 256, 0, s>>>(
                                                  gy, addrT, gyT, gluts, B, (int)NO, O, L, BP, BT, tpc, partial, scale, chunks, tb)));
    // (the row-major histogram's scale is applied in the sum; the tile-major ones scale afterwards)
    DwnReduce red = {gluts && chunks > 1 ? partial : nullptr, gluts, NO * L, chunks, (head || gy_tiled) ? nullptr : scale, L, O};
    if (rc) {  // a chunk of rows: the last one adds the sets of all chunks
        red.partial = rc->total_sets ? rc->partial_base : nullptr;
        red.chunks = rc->total_sets;
    }
    if (!gather && dwn_reduce_blocks(red))
        DL_TIMED("dwn_reduce_partials", s, (dwn_reduce_partials<<<dwn_reduce_blocks(red), 256, 0, s>>>(red)));
    if (fused_wi) {
        // the gather that also fills the bins of the layer in front
        const float *src = gy_tiled ? gy : gyT;
        const DwnFusedSplit f = dwn_fused_split(BT, I, prev->k, 4 * (fused_pack ? DWN_WI : fused_wi));
        const int fan = (long long)N * k % I == 0 ? (int)((long long)N * k / I) : 0;  // every input read `fan` times?
        const int gather_blocks = DL_XCDS * f.part * f.groups, grid = gather_blocks + dwn_reduce_blocks(red), Lp = 1 << prev->k;
#define DWN_GXH(K_, WI_, FAN_)                                                                                                \
    DL_TIMED("dwn_bwd_gx_hist", s, (dwn_bwd_gx_walk<K_, WI_, FAN_><<<grid, 256, 0, s>>>(src, addrT, D, inv_ptr, inv_pos, gx, prev->addrT, \
                                                                                  prev->partial, I, N, BT, f.slabs, f.split, f.part, f.tpb, Lp, gather_blocks, red)))
#define DWN_GXH_K(K_)                                                \
    if (fused_pack)                                                  \
        DL_TIMED("dwn_bwd_gx_hist", s, (dwn_bwd_gx_walk<K_, DWN_WI, 6, true, false, true, true><<<grid, 256, 0, s>>>(src, addrT, D, inv_ptr, inv_pos, gx, prev->addrT, \
                                                                                  prev->partial, I, N, BT, f.slabs, f.split, f.part, f.tpb, Lp, gather_blocks, red))); \
    else if (fused_wi != DWN_WI && fan == 6) DWN_GXH(K_, DWN_WI_SMALL, 6); \
    else if (fused_wi != DWN_WI && fan == 12) DWN_GXH(K_, DWN_WI_SMALL, 12); \
    else if (fused_wi != DWN_WI) DWN_GXH(K_, DWN_WI_SMALL, 0);       \
    else if (fan == 1) DWN_GXH(K_, DWN_WI, 1);                       \
    else if (fan == 2) DWN_GXH(K_, DWN_WI, 2);                       \
    else if (fan == 3) DWN_GXH(K_, DWN_WI, 3);                       \
    else DWN_GXH(K_, DWN_WI, 0)
        switch (k) {
            case 1: DWN_GXH_K(1); break;
            case 2: DWN_GXH_K(2); break;
            case 3: DWN_GXH_K(3); break;
            case 4: DWN_GXH_K(4); break;
            case 5: DWN_GXH_K(5); break;
            default: DWN_GXH_K(6); break;
        }
#undef DWN_GXH_K
#undef DWN_GXH
        const DwnReduce pred = {prev->partial, prev->gluts, (long long)I * Lp, f.sets, nullptr, Lp, 1};
        DL_TIMED("dwn_reduce_partials", s, (dwn_reduce_partials<<<dwn_reduce_blocks(pred), 256, 0, s>>>(pred)));
    } else if (walk_rows) {
        // row-major input gradient of a big layer whose inputs are all read three times: the walking gather, paced
        const float *src = gy_tiled ? gy : gyT;
        const int slabs = dl_ceil_div(I, 4 * (walk_pack && walk_rows == 3 ? 2 * DWN_WI : DWN_WI));
        int split = 1;
        while (split < DL_XCDS && dl_ceil_div(slabs, split) > DWN_RESIDENT) split *= 2;
        const int part = dl_ceil_div(slabs, split), ncls = DL_XCDS / split, tiles_cls = dl_ceil_div(BT, ncls);
        int groups = DWN_RESIDENT / part;
        if (groups > tiles_cls / 8) groups = tiles_cls / 8;  // at least eight tiles per block
        if (groups < 1) groups = 1;
        const int tpb = dl_ceil_div(tiles_cls, groups);
        groups = dl_ceil_div(tiles_cls, tpb);
        const int gb = DL_XCDS * part * groups;
        // base pace: the bytes one tile step moves (every XCD reads the rows of `groups` tiles and writes its slabs'
        // share of them) at DWN_PACE_GBS, in ticks of 10 ns; the device-side scale moves it from there
        const double step_bytes = (double)DL_XCDS * groups * ((double)N * 320 + (double)I / split * 256);
        const int pace = (int)(step_bytes / (DWN_PACE_GBS * 1e9) * 1e8);
        // the band of late tile starts the steering aims for: where the rows the gather reads (the gradient the histogram
        // has just written, the saved addresses) still sit in the 256 MB Infinity Cache, falling behind costs little and
        // the best pace has 15-24 % late starts; beyond that size the step time has an edge (B = 8192 at the headline's
        // widths: 0.579 ms at 3200 GB/s with no late starts, 0.590 at 3400 with 0.2 %, 0.614 at 3600 with 63 %) and the
        // pace stays just on its slow side
        const bool cached = (double)N * BT * 64 * 5 <= DWN_PACE_CACHE_MB * 1e6;
        const int band = cached ? (DWN_PACE_LATE_LO << 8) | (DWN_PACE_LATE_HI << 16) : (DWN_PACE_EDGE_LO << 8) | (DWN_PACE_EDGE_HI << 16);
        const int slot = band + (int)(((unsigned)I * 2654435761u ^ (unsigned)N * 40503u ^ (unsigned)BT * 97u ^ (unsigned)k ^ (sform ? 0u : 7u)) % DWN_PACE_SLOTS);
#define DWN_WALK_F(K_, DF_)                                                                                      \
    DL_TIMED("dwn_bwd_gx", s,                                                                                    \
             (dwn_bwd_gx_walk<K_, DWN_WI, 3, false, true, DF_><<<gb + dwn_reduce_blocks(red), 256, 0, s>>>(      \
                 src, addrT, D, inv_ptr, inv_pos, gx, nullptr, nullptr, I, N, BT, slabs, split, part, tpb, 0, gb, red, B, pace, slot)))
#define DWN_WALK(K_)                                                                                             \
    if (walk_rows == 6)                                                                                          \
        DL_TIMED("dwn_bwd_gx", s,                                                                                \
                 (dwn_bwd_gx_walk<K_, DWN_WI, 6, false, true, true, true><<<gb + dwn_reduce_blocks(red), 256, 0, s>>>( \
                     src, addrT, D, inv_ptr, inv_pos, gx, nullptr, nullptr, I, N, BT, slabs, split, part, tpb, 0, gb, red, B, pace, slot))); \
    else if (walk_pack)                                                                                          \
        DL_TIMED("dwn_bwd_gx", s,                                                                                \
                 (dwn_bwd_gx_walk<K_, 2 * DWN_WI, 3, false, true, true, true><<<gb + dwn_reduce_blocks(red), 256, 0, s>>>( \
                     src, addrT, D, inv_ptr, inv_pos, gx, nullptr, nullptr, I, N, BT, slabs, split, part, tpb, 0, gb, red, B, pace, slot))); \
    else if (sform) DWN_WALK_F(K_, false);                                                                       \
    else DWN_WALK_F(K_, true)
        switch (k) {
            case 1: DWN_WALK(1); break;
            case 2: DWN_WALK(2); break;
            case 3: DWN_WALK(3); break;
            case 4: DWN_WALK(4); break;
            case 5: DWN_WALK(5); break;
            default: DWN_WALK(6); break;
        }
#undef DWN_WALK
#undef DWN_WALK_F
    } else if (gx) {
        const float *src = gy_tiled ? gy : gyT;
        switch (k) {
            case 1: dwn_launch_gx<1>(src, addrT, D, inv_ptr, inv_pos, gx, B, I, N, O, sform, gx_tiled, red, s); break;
            case 2: dwn_launch_gx<2>(src, addrT, D, inv_ptr, inv_pos, gx, B, I, N, O, sform, gx_tiled, red, s); break;
            case 3: dwn_launch_gx<3>(src, addrT, D, inv_ptr, inv_pos, gx, B, I, N, O, sform, gx_tiled, red, s); break;
            case 4: dwn_launch_gx<4>(src, addrT, D, inv_ptr, inv_pos, gx, B, I, N, O, sform, gx_tiled, red, s); break;
            case 5: dwn_launch_gx<5>(src, addrT, D, inv_ptr, inv_pos, gx, B, I, N, O, sform, gx_tiled, red, s); break;
            default: dwn_launch_gx<6>(src, addrT, D, inv_ptr, inv_pos, gx, B, I, N, O, sform, gx_tiled, red, s); break;
        }
    }
    if (scale && (gy_tiled || head))  // the row-major histogram applies the scale when it flushes
        DL_TIMED("dwn_scale_tables", s,
                 (dwn_scale_tables<<<dl_ceil_div(NO * L, 256), 256, 0, s>>>(gluts, scale, NO * L, L, O)));
    return dl_launch_status();
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
    if (!dwn_fast(N, k, O)) {
        if (!x) return DL_ERR_NULL;
        return dwn_generic_backward(x, idx32, inv_ptr, inv_pos, luts, gy, alpha, beta, nullptr, gx, gluts, B, I, N, k, O, s,
                                    nullptr, nullptr, fabsf(beta), ws, ws_bytes);
    }
    if (!saved || !ws) return DL_ERR_NULL;
    if (ws_bytes < dl_dwn_bwd_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    return dwn_backward_fast(saved, inv_ptr, inv_pos, luts, gy, 0, alpha, beta, nullptr, gx, 0, gluts, ws, B, I, N, k, O, s);
}

// The same backward with every node's own alpha and beta (device arrays [N]); beta_abs_max = max |beta_n| decides
// which form of the coefficient table is safe for all nodes.
extern "C" int dl_dwn_layer_bwd_nodes(const float *x, const void *saved, const int32_t *idx32, const int32_t *inv_ptr,
                                      const int32_t *inv_pos, const float *luts, const float *gy, const float *alpha_n,
                                      const float *beta_n, float beta_abs_max, float *gx, float *gluts, void *ws,
                                      size_t ws_bytes, int B, int I, int N, int k, int O, void *stream) {
    if (!idx32 || !luts || !gy || !gluts || !alpha_n || !beta_n) return DL_ERR_NULL;
    if (gx && (!inv_ptr || !inv_pos)) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (!dwn_fast(N, k, O)) {
        if (!x) return DL_ERR_NULL;
        return dwn_generic_backward(x, idx32, inv_ptr, inv_pos, luts, gy, 0.0f, 0.0f, nullptr, gx, gluts, B, I, N, k, O, s,
                                    alpha_n, beta_n, beta_abs_max, ws, ws_bytes);
    }
    if (!saved || !ws) return DL_ERR_NULL;
    if (ws_bytes < dl_dwn_bwd_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    // beta handed to the form choice only: |beta| <= 1/2 for every node -> the shared 64-entry form
    return dwn_backward_fast(saved, inv_ptr, inv_pos, luts, gy, 0, 0.0f, beta_abs_max, nullptr, gx, 0, gluts, ws, B, I, N, k,
                             O, s, nullptr, alpha_n, beta_n);
}

extern "C" int dl_dwn_stable_layer_bwd(const float *x, const void *saved, const int32_t *idx32, const int32_t *inv_ptr,
                                       const int32_t *inv_pos, const float *luts, const float *gy,
                                       const float *gradient_scale, float *gx, float *gluts, void *ws, size_t ws_bytes,
                                       int B, int I, int N, int k, int O, void *stream) {
    if (!idx32 || !luts || !gy || !gluts || !gradient_scale) return DL_ERR_NULL;
    if (gx && (!inv_ptr || !inv_pos)) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (!dwn_fast(N, k, O)) {
        if (!x) return DL_ERR_NULL;
        return dwn_generic_backward(x, idx32, inv_ptr, inv_pos, luts, gy, 0.0f, 0.0f, gradient_scale, gx, gluts, B, I, N, k,
                                    O, s);
    }
    if (!saved || !ws) return DL_ERR_NULL;
    if (ws_bytes < dl_dwn_bwd_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    return dwn_backward_fast(saved, inv_ptr, inv_pos, luts, gy, 0, 0.0f, 0.0f, gradient_scale, gx, 0, gluts, ws, B, I, N, k,
                             O, s);
}

extern "C" int dl_table_sigmoid_fwd(const float *raw, float *luts, long long count, void *stream) {
    if (!raw || !luts) return DL_ERR_NULL;
    if (count <= 0 || count > 0x7fffffffLL * 256) return DL_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    DL_TIMED("dwn_table_sigmoid", s, (dwn_table_sigmoid<<<dl_ceil_div(count, 256), 256, 0, s>>>(raw, luts, count)));
    return dl_launch_status();
}

extern "C" int dl_table_sigmoid_bwd(const float *gluts, const float *luts, float *graw, long long count, void *stream) {
    if (!gluts || !luts || !graw) return DL_ERR_NULL;
    if (count <= 0 || count > 0x7fffffffLL * 256) return DL_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    DL_TIMED("dwn_table_sigmoid_bwd", s,
             (dwn_table_sigmoid_bwd<<<dl_ceil_div(count, 256), 256, 0, s>>>(gluts, luts, graw, count)));
    return dl_launch_status();
}

// ---------------------------------------------------------------------------------
// Bit-sliced inference for a layer between two bit-plane tensors.  Lanes are NODES here: a lane keeps its column's
// truth table as 2^k bits (table entry >= 0.5), fetches the k plane words of its inputs for a batch tile (64 rows in
// one 64-bit word each) and evaluates the table on all 64 rows at once as a multiplexer tree of bitwise operations:
// level j halves the table with the word of input j,  v[i] = v[2i] ^ ((v[2i] ^ v[2i+1]) & x_j).  About 6 vector
// instructions per (node, tile) instead of 13 vector + 26 scalar in the lookup kernel, and the result of a lane is
// already the plane word of its column.  A block takes 256 columns and walks `tiles_per_block` tiles with the same
// indices and tables in registers.
// SAVE: the training forward of a chained hidden layer - the same planes out, plus the address of every
// (node, row) for the backward ([tile][node][64] bytes): the k plane words are turned into 16 words of four
// address bytes each (a nibble of rows times 0x204081 puts its four bits at the bottom of four bytes).
template <int K, bool SAVE = false>
__global__ __launch_bounds__(256) void dwn_eval_bitsliced(const u64 *__restrict__ planes, const int *__restrict__ idx32,
                                                           const float *__restrict__ luts, u64 *__restrict__ planes_out,
                                                           int B, int I, int N, int O, int BT, int tiles_per_block,
                                                           uint8_t *__restrict__ addrT = nullptr) {
    constexpr int L = 1 << K;
    typedef unsigned u4v __attribute__((ext_vector_type(4)));
    __shared__ u4v stage[SAVE ? 4 : 1][SAVE ? 64 * 5 : 1];  // per wavefront: 64 nodes x 64 address bytes, rows padded to 80
    const int NO = N * O;
    const int lane = threadIdx.x & 63;
    const int wave = dl_uniform(threadIdx.x >> 6);
    const int wc0 = (blockIdx.x * 4 + wave) * 64;  // my wavefront's first column
    if (wc0 >= NO) return;
    const int c = min(wc0 + lane, NO - 1);
    // truth tables of the wavefront's 64 columns: row u of the tables is read with lane = entry and voted on
    unsigned t_lo = 0u, t_hi = 0u;
    {
        float tv[64];  // all 64 rows asked for at once: one trip to memory, not one per handful of rows
#pragma unroll
        for (int u = 0; u < 64; ++u) tv[u] = lane < L ? luts[(size_t)min(wc0 + u, NO - 1) * L + lane] : 0.0f;
#pragma unroll
        for (int u = 0; u < 64; ++u) {
            const u64 bits = __ballot(tv[u] >= 0.5f);
            if (lane == u) { t_lo = (unsigned)bits; t_hi = (unsigned)(bits >> 32); }
        }
    }
    int off[K];  // word offsets of my inputs inside a tile's planes
#pragma unroll
    for (int j = 0; j < K; ++j) off[j] = idx32[(size_t)(c / O) * K + j];
    const int t_begin = blockIdx.y * tiles_per_block;
    const int t_end = min(BT, t_begin + tiles_per_block);
    u64 w[K], wn[K];
    auto fetch = [&](int t, u64 (&dst)[K]) {
#pragma unroll
        for (int j = 0; j < K; ++j) dst[j] = planes[(size_t)t * I + off[j]];
    };
    if (t_begin < t_end) fetch(t_begin, w);
    for (int t = t_begin; t < t_end; ++t) {
        if (t + 1 < t_end) fetch(t + 1, wn);
        unsigned vlo[L / 2 > 0 ? L / 2 : 1], vhi[L / 2 > 0 ? L / 2 : 1];
        const unsigned x0lo = (unsigned)w[0], x0hi = (unsigned)(w[0] >> 32);
#pragma unroll
        for (int i = 0; i < L / 2; ++i) {  // level of input 0: the leaves are table bits, spread to 0 / ~0
            const unsigned src0 = (2 * i < 32) ? t_lo : t_hi, src1 = (2 * i + 1 < 32) ? t_lo : t_hi;
            const unsigned m0 = (unsigned)__builtin_amdgcn_sbfe((int)src0, (2 * i) & 31, 1);
            const unsigned m1 = (unsigned)__builtin_amdgcn_sbfe((int)src1, (2 * i + 1) & 31, 1);
            const unsigned d = m0 ^ m1;
            vlo[i] = m0 ^ (d & x0lo);
            vhi[i] = m0 ^ (d & x0hi);
        }
#pragma unroll
        for (int j = 1; j < K; ++j) {
            const unsigned xlo = (unsigned)w[j], xhi = (unsigned)(w[j] >> 32);
#pragma unroll
            for (int i = 0; i < (L >> (j + 1)); ++i) {
                vlo[i] = vlo[2 * i] ^ ((vlo[2 * i] ^ vlo[2 * i + 1]) & xlo);
                vhi[i] = vhi[2 * i] ^ ((vhi[2 * i] ^ vhi[2 * i + 1]) & xhi);
            }
        }
        const int rows = min(64, B - t * 64);  // rows past B stay 0, like the planes packed from x
        const u64 valid = rows == 64 ? ~0ull : ((1ull << rows) - 1ull);
        if (wc0 + lane < NO) planes_out[(size_t)t * NO + wc0 + lane] = (((u64)vhi[0] << 32) | vlo[0]) & valid;
        if (SAVE && wc0 + lane < NO && c % O == 0) {
            u4v *dst = reinterpret_cast<u4v *>(addrT + ((size_t)t * N + c / O) * 64);
            // word q = the address bytes of rows 4q .. 4q + 3.  Bit j of those four bytes: nibble q of plane j times
            // 0x204081 has the nibble's bit r at bit 8r (no two partial products meet, so nothing carries), times 2^j
            // puts it at bit j of byte r.  The nibbles are taken as bytes of two masked copies of the plane word (even
            // and odd nibbles); from j = 3 on the copies carry the nibble at bits 3..6 and the constant 2^(j-3), which
            // keeps both factors inside 24 bits.
            unsigned word[16];
#pragma unroll
            for (int q = 0; q < 16; ++q) word[q] = 0u;
#pragma unroll
            for (int j = 0; j < K; ++j) {
                constexpr unsigned SPREAD = 0x204081u;
                const int sh = j >= 3 ? 3 : 0;
                const unsigned factor = SPREAD << (j - sh), keep = 0x01010101u << j, nibbles = 0x0F0F0F0Fu << sh;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const unsigned half = h ? (unsigned)(w[j] >> 32) : (unsigned)w[j];
                    const unsigned even = (half << sh) & nibbles, odd = ((half >> 4) << sh) & nibbles;
#pragma unroll
                    for (int q = 0; q < 8; ++q) {
                        const unsigned nib = (((q & 1) ? odd : even) >> (8 * (q >> 1))) & 0xFFu;
                        word[h * 8 + q] |= __umul24(nib, factor) & keep;
                    }
                }
            }
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const u4v v = {word[4 * q4], word[4 * q4 + 1], word[4 * q4 + 2], word[4 * q4 + 3]};
                if (O == 1)
                    stage[wave][lane * 5 + q4] = v;
                else
                    dst[q4] = v;
            }
        }
        if (SAVE && O == 1) {
            // one output per node: the wavefront's 64 nodes own 4 KB in a row.  Through the LDS, so that every store
            // instruction writes 1 KB of whole lines instead of a quarter of 64 lines.
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int node = q4 * 16 + (lane >> 2);
                const u4v v = stage[wave][node * 5 + (lane & 3)];
                if (wc0 + node < NO)
                    *reinterpret_cast<u4v *>(addrT + ((size_t)t * N + wc0) * 64 + (size_t)q4 * 1024 + lane * 16) = v;
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
#pragma unroll
        for (int j = 0; j < K; ++j) w[j] = wn[j];
    }
}

template <int K>
static void dwn_launch_eval_bitsliced(const u64 *planes, const int *idx32, const float *luts, u64 *planes_out, int B, int I,
                                      int N, int O, hipStream_t s, uint8_t *addrT = nullptr) {
    const int BT = dwn_bt(B);
    const int col_blocks = dl_ceil_div((long long)N * O, 256);
    // about 1024 blocks, one resident round: each repays its tables over more tiles (2048: 45 us per launch of the deep
    // stack's training forward, 1024: 41, 4096: 53)
    int chunks = col_blocks >= 1024 ? 1 : 1024 / col_blocks;
    if (chunks > BT) chunks = BT;
    const int tpb = dl_ceil_div(BT, chunks);
    if (addrT)
        DL_TIMED("dwn_fwd_bitsliced", s, (dwn_eval_bitsliced<K, true><<<dim3(col_blocks, dl_ceil_div(BT, tpb)), 256, 0, s>>>(
                                             planes, idx32, luts, planes_out, B, I, N, O, BT, tpb, addrT)));
    else
        DL_TIMED("dwn_eval_bitsliced", s, (dwn_eval_bitsliced<K><<<dim3(col_blocks, dl_ceil_div(BT, tpb)), 256, 0, s>>>(
                                              planes, idx32, luts, planes_out, B, I, N, O, BT, tpb)));
}

// ---------------------------------------------------------------------------------
// Chained layers: activations between two DWN layers never take their [B, N] fp32 form.
extern "C" size_t dl_dwn_planes_bytes(int B, int C) { return (B > 0 && C > 0) ? dwn_planes_bytes(B, C) : 256; }
extern "C" size_t dl_dwn_tiled_bytes(int B, int C) {
    return (B > 0 && C > 0) ? dl_align256((size_t)dwn_bt(B) * C * 64 * sizeof(float)) : 256;
}

extern "C" int dl_dwn_pack_planes(const float *x, void *planes, int B, int I, void *stream) {
    if (!x || !planes) return DL_ERR_NULL;
    if (B <= 0 || I <= 0) return DL_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    const int BT = dwn_bt(B);
    if (I % 4 == 0 && ((uintptr_t)x & 15) == 0)
        DL_TIMED("dwn_pack_planes", s, (dwn_pack_planes<4><<<dim3(dl_ceil_div(I, 1024), dwn_pack_grid_y(BT)), 256, 0, s>>>(x, (u64 *)planes, B, I)));
    else
        DL_TIMED("dwn_pack_planes", s, (dwn_pack_planes<1><<<dim3(dl_ceil_div(I, 256), dwn_pack_grid_y(BT)), 256, 0, s>>>(x, (u64 *)planes, B, I)));
    return dl_launch_status();
}

extern "C" int dl_dwn_layer_fwd_planes(const void *planes_in, const int32_t *idx32, const float *luts, float *y,
                                       void *planes_out, void *saved, int B, int I, int N, int k, int O, void *stream) {
    if (!planes_in || !idx32 || !luts || !saved || (!y && !planes_out)) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    if (!dwn_fast(N, k, O)) return DL_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    const u64 *planes = (const u64 *)planes_in;
    uint8_t *addrT = (uint8_t *)saved;
    u64 *po = (u64 *)planes_out;
    if (!y) {  // a hidden layer of a chain: only planes and saved addresses leave it - the bit-sliced form
        switch (k) {
            case 1: dwn_launch_eval_bitsliced<1>(planes, idx32, luts, po, B, I, N, O, s, addrT); break;
            case 2: dwn_launch_eval_bitsliced<2>(planes, idx32, luts, po, B, I, N, O, s, addrT); break;
            case 3: dwn_launch_eval_bitsliced<3>(planes, idx32, luts, po, B, I, N, O, s, addrT); break;
            case 4: dwn_launch_eval_bitsliced<4>(planes, idx32, luts, po, B, I, N, O, s, addrT); break;
            case 5: dwn_launch_eval_bitsliced<5>(planes, idx32, luts, po, B, I, N, O, s, addrT); break;
            default: dwn_launch_eval_bitsliced<6>(planes, idx32, luts, po, B, I, N, O, s, addrT); break;
        }
        return dl_launch_status();
    }
    switch (k) {
        case 1: dwn_launch_lookup<1>(planes, idx32, luts, y, addrT, po, B, I, N, O, s); break;
        case 2: dwn_launch_lookup<2>(planes, idx32, luts, y, addrT, po, B, I, N, O, s); break;
        case 3: dwn_launch_lookup<3>(planes, idx32, luts, y, addrT, po, B, I, N, O, s); break;
        case 4: dwn_launch_lookup<4>(planes, idx32, luts, y, addrT, po, B, I, N, O, s); break;
        case 5: dwn_launch_lookup<5>(planes, idx32, luts, y, addrT, po, B, I, N, O, s); break;
        default: dwn_launch_lookup<6>(planes, idx32, luts, y, addrT, po, B, I, N, O, s); break;
    }
    return dl_launch_status();
}

// ---- GroupSum head on the last layer of a chain
// logits[b][g] = inv_tau * (sum of the per-tile partial sums of group g, tiles in ascending order)
__global__ __launch_bounds__(256) void dwn_group_finish(const float *__restrict__ partial, float *__restrict__ logits, int B,
                                                         int BP, int F, int groups, int gsize, int slots, float inv_tau) {
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    if (e >= (long long)B * groups) return;
    const int g = (int)(e / B), b = (int)(e % B);
    const int c_lo = g * gsize, c_hi = min(F, c_lo + gsize);
    float sum = 0.0f;
    if (c_lo < c_hi)
        for (int ct = c_lo / DWN_TC; ct <= (c_hi - 1) / DWN_TC; ++ct)
            sum += partial[((size_t)ct * slots + (g - (ct * DWN_TC) / gsize)) * BP + b];
    logits[(size_t)b * groups + g] = sum * inv_tau;
}
// groups the columns of one tile can touch, and the size of a group (features padded up to groups * gsize)
static inline int dwn_group_size(int F, int groups) { return (F + groups - 1) / groups; }
static inline int dwn_group_slots(int gsize) { return (DWN_TC - 1) / gsize + 2; }

extern "C" size_t dl_dwn_groups_workspace_bytes(int B, int N, int O, int groups) {
    if (B <= 0 || N <= 0 || O <= 0 || groups <= 0) return 256;
    const long long F = (long long)N * O;
    const int slots = dwn_group_slots(dwn_group_size((int)F, groups));
    return dl_align256((size_t)dl_ceil_div(F, DWN_TC) * slots * dwn_bt(B) * 64 * sizeof(float));
}

extern "C" int dl_dwn_layer_fwd_planes_groups(const void *planes_in, const int32_t *idx32, const float *luts, float *logits,
                                              void *saved, void *ws, size_t ws_bytes, int B, int I, int N, int k, int O,
                                              int groups, float tau, void *stream) {
    if (!planes_in || !idx32 || !luts || !logits || !saved || !ws) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    if (groups <= 0 || !(tau > 0.0f)) return DL_ERR_SHAPE;
    if (!dwn_fast(N, k, O)) return DL_ERR_UNSUPPORTED;
    const int F = N * O, gsize = dwn_group_size(F, groups), slots = dwn_group_slots(gsize);
    if (slots > DWN_GS_SLOTS) return DL_ERR_UNSUPPORTED;  // groups narrower than half a column tile
    if (ws_bytes < dl_dwn_groups_workspace_bytes(B, N, O, groups)) return DL_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    const u64 *planes = (const u64 *)planes_in;
    uint8_t *addrT = (uint8_t *)saved;
    float *partial = (float *)ws;
    switch (k) {
        case 1: dwn_launch_lookup<1>(planes, idx32, luts, partial, addrT, nullptr, B, I, N, O, s, gsize, slots); break;
        case 2: dwn_launch_lookup<2>(planes, idx32, luts, partial, addrT, nullptr, B, I, N, O, s, gsize, slots); break;
        case 3: dwn_launch_lookup<3>(planes, idx32, luts, partial, addrT, nullptr, B, I, N, O, s, gsize, slots); break;
        case 4: dwn_launch_lookup<4>(planes, idx32, luts, partial, addrT, nullptr, B, I, N, O, s, gsize, slots); break;
        case 5: dwn_launch_lookup<5>(planes, idx32, luts, partial, addrT, nullptr, B, I, N, O, s, gsize, slots); break;
        default: dwn_launch_lookup<6>(planes, idx32, luts, partial, addrT, nullptr, B, I, N, O, s, gsize, slots); break;
    }
    DL_TIMED("dwn_group_finish", s,
             (dwn_group_finish<<<dl_ceil_div((long long)B * groups, 256), 256, 0, s>>>(partial, logits, B, dwn_bt(B) * 64, F,
                                                                                     groups, gsize, slots, 1.0f / tau)));
    return dl_launch_status();
}

// ---- inference on binary activations
extern "C" int dl_dwn_layer_eval_planes(const void *planes_in, const int32_t *idx32, const float *luts, float *y,
                                        void *planes_out, int B, int I, int N, int k, int O, void *stream) {
    if (!planes_in || !idx32 || !luts || (!y && !planes_out)) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    if (!dwn_fast(N, k, O)) return DL_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    const u64 *planes = (const u64 *)planes_in;
    u64 *po = (u64 *)planes_out;
    if (!y) {  // a hidden layer of an inference chain: planes in, planes out
        switch (k) {
            case 1: dwn_launch_eval_bitsliced<1>(planes, idx32, luts, po, B, I, N, O, s); break;
            case 2: dwn_launch_eval_bitsliced<2>(planes, idx32, luts, po, B, I, N, O, s); break;
            case 3: dwn_launch_eval_bitsliced<3>(planes, idx32, luts, po, B, I, N, O, s); break;
            case 4: dwn_launch_eval_bitsliced<4>(planes, idx32, luts, po, B, I, N, O, s); break;
            case 5: dwn_launch_eval_bitsliced<5>(planes, idx32, luts, po, B, I, N, O, s); break;
            default: dwn_launch_eval_bitsliced<6>(planes, idx32, luts, po, B, I, N, O, s); break;
        }
        return dl_launch_status();
    }
    uint8_t *none = (uint8_t *)const_cast<float *>(luts);  // descriptor base of the unused address stores
    switch (k) {
        case 1: dwn_launch_lookup<1>(planes, idx32, luts, y, none, po, B, I, N, O, s, 0, 0, true); break;
        case 2: dwn_launch_lookup<2>(planes, idx32, luts, y, none, po, B, I, N, O, s, 0, 0, true); break;
        case 3: dwn_launch_lookup<3>(planes, idx32, luts, y, none, po, B, I, N, O, s, 0, 0, true); break;
        case 4: dwn_launch_lookup<4>(planes, idx32, luts, y, none, po, B, I, N, O, s, 0, 0, true); break;
        case 5: dwn_launch_lookup<5>(planes, idx32, luts, y, none, po, B, I, N, O, s, 0, 0, true); break;
        default: dwn_launch_lookup<6>(planes, idx32, luts, y, none, po, B, I, N, O, s, 0, 0, true); break;
    }
    return dl_launch_status();
}

// Eval forward of one layer on [B, I] fp32 input, exact for any values: the input is packed into bit-planes while
// being checked; if every value is 0 or 1 the bit-plane kernel answers, otherwise the generic one does (both are
// launched, one of them returns at once - no host synchronisation).
extern "C" size_t dl_dwn_eval_workspace_bytes(int B, int I, int N, int k, int O) {
    return dwn_fast(N, k, O) && B > 0 && I > 0 ? dwn_planes_bytes(B, I) + 256 : 256;
}
extern "C" int dl_dwn_layer_eval_ws(const float *x, const int32_t *idx32, const float *luts, float *y, void *ws,
                                    size_t ws_bytes, int B, int I, int N, int k, int O, void *stream) {
    if (!x || !idx32 || !luts || !y) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (!dwn_fast(N, k, O)) return dwn_generic_eval(x, idx32, luts, y, B, I, N, k, O, nullptr, s);
    if (!ws) return DL_ERR_NULL;
    if (ws_bytes < dl_dwn_eval_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    u64 *planes = (u64 *)ws;
    int *flag = (int *)((char *)ws + dwn_planes_bytes(B, I));
    const int BT = dwn_bt(B);
    dwn_set_flag<<<1, 64, 0, s>>>(flag, 1);
    if (I % 4 == 0 && ((uintptr_t)x & 15) == 0)
        DL_TIMED("dwn_pack_planes", s,
                 (dwn_pack_planes<4, true><<<dim3(dl_ceil_div(I, 1024), dwn_pack_grid_y(BT)), 256, 0, s>>>(x, planes, B, I, flag)));
    else
        DL_TIMED("dwn_pack_planes", s,
                 (dwn_pack_planes<1, true><<<dim3(dl_ceil_div(I, 256), dwn_pack_grid_y(BT)), 256, 0, s>>>(x, planes, B, I, flag)));
    uint8_t *none = (uint8_t *)const_cast<float *>(luts);
    switch (k) {
        case 1: dwn_launch_lookup<1>(planes, idx32, luts, y, none, nullptr, B, I, N, O, s, 0, 0, true, flag); break;
        case 2: dwn_launch_lookup<2>(planes, idx32, luts, y, none, nullptr, B, I, N, O, s, 0, 0, true, flag); break;
        case 3: dwn_launch_lookup<3>(planes, idx32, luts, y, none, nullptr, B, I, N, O, s, 0, 0, true, flag); break;
        case 4: dwn_launch_lookup<4>(planes, idx32, luts, y, none, nullptr, B, I, N, O, s, 0, 0, true, flag); break;
        case 5: dwn_launch_lookup<5>(planes, idx32, luts, y, none, nullptr, B, I, N, O, s, 0, 0, true, flag); break;
        default: dwn_launch_lookup<6>(planes, idx32, luts, y, none, nullptr, B, I, N, O, s, 0, 0, true, flag); break;
    }
    return dwn_generic_eval(x, idx32, luts, y, B, I, N, k, O, flag, s);
}

extern "C" int dl_dwn_layer_eval_planes_groups(const void *planes_in, const int32_t *idx32, const float *luts,
                                               float *logits, void *ws, size_t ws_bytes, int B, int I, int N, int k, int O,
                                               int groups, float tau, void *stream) {
    if (!planes_in || !idx32 || !luts || !logits || !ws) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    if (groups <= 0 || !(tau > 0.0f)) return DL_ERR_SHAPE;
    if (!dwn_fast(N, k, O)) return DL_ERR_UNSUPPORTED;
    const int F = N * O, gsize = dwn_group_size(F, groups), slots = dwn_group_slots(gsize);
    if (slots > DWN_GS_SLOTS) return DL_ERR_UNSUPPORTED;
    if (ws_bytes < dl_dwn_groups_workspace_bytes(B, N, O, groups)) return DL_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    const u64 *planes = (const u64 *)planes_in;
    float *partial = (float *)ws;
    uint8_t *none = (uint8_t *)const_cast<float *>(luts);
    switch (k) {
        case 1: dwn_launch_lookup<1>(planes, idx32, luts, partial, none, nullptr, B, I, N, O, s, gsize, slots, true); break;
        case 2: dwn_launch_lookup<2>(planes, idx32, luts, partial, none, nullptr, B, I, N, O, s, gsize, slots, true); break;
        case 3: dwn_launch_lookup<3>(planes, idx32, luts, partial, none, nullptr, B, I, N, O, s, gsize, slots, true); break;
        case 4: dwn_launch_lookup<4>(planes, idx32, luts, partial, none, nullptr, B, I, N, O, s, gsize, slots, true); break;
        case 5: dwn_launch_lookup<5>(planes, idx32, luts, partial, none, nullptr, B, I, N, O, s, gsize, slots, true); break;
        default: dwn_launch_lookup<6>(planes, idx32, luts, partial, none, nullptr, B, I, N, O, s, gsize, slots, true); break;
    }
    DL_TIMED("dwn_group_finish", s,
             (dwn_group_finish<<<dl_ceil_div((long long)B * groups, 256), 256, 0, s>>>(partial, logits, B, dwn_bt(B) * 64, F,
                                                                                     groups, gsize, slots, 1.0f / tau)));
    return dl_launch_status();
}

extern "C" int dl_dwn_layer_bwd_groups(const void *saved, const int32_t *inv_ptr, const int32_t *inv_pos, const float *luts,
                                       const float *glogits, int groups, float tau, float alpha, float beta, float *gx,
                                       int gx_tiled, float *gluts, void *ws, size_t ws_bytes, int B, int I, int N, int k,
                                       int O, void *stream) {
    if (!saved || !luts || !glogits || !gluts || !ws) return DL_ERR_NULL;
    if (gx && (!inv_ptr || !inv_pos)) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    if (groups <= 0 || !(tau > 0.0f)) return DL_ERR_SHAPE;
    if (!dwn_fast(N, k, O)) return DL_ERR_UNSUPPORTED;
    if (ws_bytes < dl_dwn_bwd_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    const DwnGroupHead head = {groups, dwn_group_size(N * O, groups), 1.0f / tau};
    return dwn_backward_fast(saved, inv_ptr, inv_pos, luts, glogits, 0, alpha, beta, nullptr, gx, gx_tiled, gluts, ws, B, I, N,
                             k, O, (hipStream_t)stream, &head);
}

extern "C" int dl_dwn_layer_bwd_tiled(const void *saved, const int32_t *inv_ptr, const int32_t *inv_pos,
                                      const float *luts, const float *gy, int gy_tiled, float alpha, float beta,
                                      float *gx, int gx_tiled, float *gluts, void *ws, size_t ws_bytes, int B, int I, int N,
                                      int k, int O, void *stream) {
    if (!saved || !luts || !gy || !gluts || !ws) return DL_ERR_NULL;
    if (gx && (!inv_ptr || !inv_pos)) return DL_ERR_NULL;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    if (!dwn_fast(N, k, O)) return DL_ERR_UNSUPPORTED;
    if (ws_bytes < dl_dwn_bwd_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    return dwn_backward_fast(saved, inv_ptr, inv_pos, luts, gy, gy_tiled, alpha, beta, nullptr, gx, gx_tiled, gluts, ws, B, I, N, k, O,
                             (hipStream_t)stream);
}

// The chained backward with every node's own alpha and beta (device arrays [N]); beta_abs_max = max |beta_n| decides
// which form of the coefficient table is safe for all nodes.  gy_form: 0 = gy row-major [B, N*O], 1 = tile-major
// [B/64][N*O][64], 2 = the [B, groups] gradient of a GroupSum head's logits (groups, tau as in dl_dwn_layer_bwd_groups).
extern "C" int dl_dwn_layer_bwd_chain_nodes(const void *saved, const int32_t *inv_ptr, const int32_t *inv_pos,
                                            const float *luts, const float *gy, int gy_form, int groups, float tau,
                                            const float *alpha_n, const float *beta_n, float beta_abs_max, float *gx,
                                            int gx_tiled, float *gluts, void *ws, size_t ws_bytes, int B, int I, int N,
                                            int k, int O, void *stream) {
    if (!saved || !luts || !gy || !gluts || !ws || !alpha_n || !beta_n) return DL_ERR_NULL;
    if (gx && (!inv_ptr || !inv_pos)) return DL_ERR_NULL;
    if (gy_form < 0 || gy_form > 2) return DL_ERR_SHAPE;
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    if (gy_form == 2 && (groups <= 0 || !(tau > 0.0f))) return DL_ERR_SHAPE;
    if (!dwn_fast(N, k, O)) return DL_ERR_UNSUPPORTED;
    if (ws_bytes < dl_dwn_bwd_workspace_bytes(B, I, N, k, O)) return DL_ERR_WORKSPACE;
    const DwnGroupHead head = {groups, gy_form == 2 ? dwn_group_size(N * O, groups) : 1, gy_form == 2 ? 1.0f / tau : 1.0f};
    return dwn_backward_fast(saved, inv_ptr, inv_pos, luts, gy, gy_form == 1, 0.0f, beta_abs_max, nullptr, gx, gx_tiled, gluts,
                             ws, B, I, N, k, O, (hipStream_t)stream, gy_form == 2 ? &head : nullptr, alpha_n, beta_n);
}

// ---- chained backward with the histogram of the layer in front folded into the gather
// 1 when dl_dwn_layer_bwd_chain_fused can fill the table gradient of the layer in front (k_prev inputs per node, one
// output per node) from this layer's tile-major input gradient: k <= 6 on both sides, one output per node, the compact
// coefficient table (every |beta| <= 1/2), CSR lists short enough for the multi-input gather.
extern "C" int dl_dwn_chain_fusable(int B, int I, int N, int k, int O, int k_prev, float beta_abs_max) {
    if (dwn_check(B, I, N, k, O) || !dwn_fast(N, k, O) || O != 1) return 0;
    if (k_prev <= 0 || k_prev > DL_MAX_FAST_K || !dwn_fast(I, k_prev, 1)) return 0;
    if (!(beta_abs_max <= 0.5f)) return 0;
    return dwn_fused_wi(I, N, k) != 0;
}
extern "C" size_t dl_dwn_bwd_fused_workspace_bytes(int B, int I, int N, int k, int O, int k_prev) {
    if (!dwn_fast(N, k, O) || k_prev <= 0 || k_prev > DL_MAX_FAST_K) return 256;
    return dl_dwn_bwd_workspace_bytes(B, I, N, k, O) + dwn_fused_partial_bytes(B, I, N, k, k_prev);
}
// dl_dwn_layer_bwd_chain_nodes with two options.  gluts == NULL: this layer's table gradient has already been computed
// (by the call for the layer behind it); gy must then be tile-major (gy_form 1).  prev_saved != NULL: the layer in front
// (I nodes of k_prev inputs, one output each; prev_saved = what its forward saved) gets its table gradient prev_gluts
// [I, 2^k_prev] from this call; requires gx tile-major and dl_dwn_chain_fusable(...) == 1.
extern "C" int dl_dwn_layer_bwd_chain_fused(const void *saved, const int32_t *inv_ptr, const int32_t *inv_pos,
                                            const float *luts, const float *gy, int gy_form, int groups, float tau,
                                            const float *alpha_n, const float *beta_n, float beta_abs_max, float *gx,
                                            int gx_tiled, float *gluts, const void *prev_saved, int k_prev,
                                            float *prev_gluts, void *ws, size_t ws_bytes, int B, int I, int N, int k, int O,
                                            void *stream) {
    if (!saved || !luts || !gy || !ws || !alpha_n || !beta_n) return DL_ERR_NULL;
    if ((gx || prev_saved) && (!inv_ptr || !inv_pos)) return DL_ERR_NULL;
    if (gy_form < 0 || gy_form > 2) return DL_ERR_SHAPE;
    if (!gluts && gy_form != 1) return DL_ERR_SHAPE;
    if (!gluts && !gx && !prev_saved) return DL_ERR_NULL;  // nothing to do
    int rc = dwn_check(B, I, N, k, O);
    if (rc) return rc;
    if (gy_form == 2 && (groups <= 0 || !(tau > 0.0f))) return DL_ERR_SHAPE;
    if (!dwn_fast(N, k, O)) return DL_ERR_UNSUPPORTED;
    DwnFusedPrev prev = {nullptr, nullptr, 0, nullptr};
    size_t need = dl_dwn_bwd_workspace_bytes(B, I, N, k, O);
    if (prev_saved) {
        if (!prev_gluts || (gx && !gx_tiled)) return DL_ERR_NULL;  // gx == NULL: only the bins of the layer in front
        if ((uintptr_t)prev_saved & 15) return DL_ERR_UNSUPPORTED;  // its addresses are read sixteen at a time
        if (!dl_dwn_chain_fusable(B, I, N, k, O, k_prev, beta_abs_max)) return DL_ERR_UNSUPPORTED;
        prev = DwnFusedPrev{(const uint8_t *)prev_saved, prev_gluts, k_prev, (float *)((char *)ws + need)};
        need = dl_dwn_bwd_fused_workspace_bytes(B, I, N, k, O, k_prev);
    }
    if (ws_bytes < need) return DL_ERR_WORKSPACE;
    const DwnGroupHead head = {groups, gy_form == 2 ? dwn_group_size(N * O, groups) : 1, gy_form == 2 ? 1.0f / tau : 1.0f};
    return dwn_backward_fast(saved, inv_ptr, inv_pos, luts, gy, gy_form == 1, 0.0f, beta_abs_max, nullptr, gx, gx_tiled, gluts,
                             ws, B, I, N, k, O, (hipStream_t)stream, gy_form == 2 ? &head : nullptr, alpha_n, beta_n,
                             prev_saved ? &prev : nullptr);
}
