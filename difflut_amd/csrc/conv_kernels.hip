// Patch extraction of the convolutional LUT layer and its adjoint.
//   rows    r = (image b, output position oy, ox), row-major: r = (b * OH + oy) * OW + ox
//   columns c = (channel ch, dy, dx):                          c = (ch * KH + dy) * KW + dx
//   patches[r][c] = x[b, ch, oy*SH + dy - PH, ox*SW + dx - PW], 0 outside the image
// Neighbouring rows are neighbouring output positions, so with lane = row the loads of one column
// are (stride SW) contiguous in x and a 64-row tile of a column is 256 contiguous bytes tile-major.
#include "dl_common.h"

struct ConvGeom {
    int B, C, H, W, KH, KW, SH, SW, PH, PW, OH, OW;
};

#define CONV_MAX_COLS 4096  // columns whose offsets fit the per-block table

// per-column offset inside an image (ch*H*W + dy*W + dx) and (dy, dx) packed, built once per block
__device__ __forceinline__ void conv_fill_columns(const ConvGeom &g, int cols, int *off, int *dydx) {
    for (int c = threadIdx.x; c < cols; c += blockDim.x) {
        const int dx = c % g.KW, dy = (c / g.KW) % g.KH, ch = c / (g.KW * g.KH);
        off[c] = (ch * g.H + dy) * g.W + dx;
        dydx[c] = (dy << 16) | dx;
    }
}

// grid = ceil(rows / 64) blocks of 256 threads; block t writes rows 64 t .. 64 t + 63 (all columns), coalesced.
// flip (nullable, [rows][cols] bytes): bit-flip augmentation of the patch matrix, v -> v + (1 - 2 v) where set
// (base_layer.py:149-264 applied to the patches, convolutional.py:205-207).
__global__ __launch_bounds__(256) void conv_unfold_rows(const float *__restrict__ x, float *__restrict__ patches, ConvGeom g,
                                                         long long rows, int cols, const uint8_t *__restrict__ flip) {
    __shared__ int off[CONV_MAX_COLS], dydx[CONV_MAX_COLS];
    __shared__ long long base[64];
    __shared__ int y0s[64], x0s[64];
    conv_fill_columns(g, cols, off, dydx);
    if (threadIdx.x < 64) {
        const long long r = (long long)blockIdx.x * 64 + threadIdx.x;
        const long long rr = r < rows ? r : rows - 1;
        const int ox = (int)(rr % g.OW), oy = (int)((rr / g.OW) % g.OH);
        const long long b = rr / ((long long)g.OW * g.OH);
        const int y0 = oy * g.SH - g.PH, x0 = ox * g.SW - g.PW;
        y0s[threadIdx.x] = y0;
        x0s[threadIdx.x] = x0;
        base[threadIdx.x] = (b * g.C * g.H + y0) * (long long)g.W + x0;
    }
    __syncthreads();
    const long long r0 = (long long)blockIdx.x * 64;
    const int live = (int)min((long long)64, rows - r0);
    float *out = patches + r0 * cols;
    for (int e = threadIdx.x; e < live * cols; e += 256) {
        const int r = e / cols, c = e - r * cols;
        const int y = y0s[r] + (dydx[c] >> 16), xx = x0s[r] + (dydx[c] & 0xffff);
        const bool in = y >= 0 && y < g.H && xx >= 0 && xx < g.W;
        float v = in ? x[base[r] + off[c]] : 0.0f;
        if (flip && flip[r0 * cols + e]) v = v + (1.0f - 2.0f * v);
        out[e] = v;
    }
}

// The same patches as the bit-planes a DWN layer reads: word (t, c) holds in bit r (patches[64 t + r][c] >= 0.5).
// grid = ceil(rows / 64) blocks of 256 threads; lane = row, the four wavefronts share the columns.
__global__ __launch_bounds__(256) void conv_unfold_planes(const float *__restrict__ x, unsigned long long *__restrict__ planes,
                                                           ConvGeom g, long long rows, int cols,
                                                           const uint8_t *__restrict__ flip) {
    __shared__ int off[CONV_MAX_COLS], dydx[CONV_MAX_COLS];
    conv_fill_columns(g, cols, off, dydx);
    __syncthreads();
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const long long r = (long long)blockIdx.x * 64 + lane;
    const bool live = r < rows;
    const long long rr = live ? r : rows - 1;
    const int ox = (int)(rr % g.OW), oy = (int)((rr / g.OW) % g.OH);
    const long long b = rr / ((long long)g.OW * g.OH);
    const int y0 = oy * g.SH - g.PH, x0 = ox * g.SW - g.PW;
    const float *img = x + (b * g.C * g.H + y0) * (long long)g.W + x0;
    unsigned long long *out = planes + (size_t)blockIdx.x * cols;
    const int per = (cols + 3) / 4;
    const int c0 = w * per, c1 = min(cols, c0 + per);
    for (int cb = c0; cb < c1; cb += 64) {  // a lane keeps word cb + lane; 64 consecutive words leave together
        unsigned long long mine = 0;
        const int cnt = min(64, c1 - cb);
        for (int q = 0; q < cnt; ++q) {
            const int c = cb + q;
            const int y = y0 + (dydx[c] >> 16), xx = x0 + (dydx[c] & 0xffff);
            const bool in = live && y >= 0 && y < g.H && xx >= 0 && xx < g.W;
            float v = in ? img[off[c]] : 0.0f;
            if (flip && live && flip[r * cols + c]) v = v + (1.0f - 2.0f * v);  // the value the reference thresholds
            const unsigned long long mask = __ballot(live && v >= 0.5f);
            if (q == lane) mine = mask;
        }
        if (lane < cnt) out[cb + lane] = mine;
    }
}

// Adjoint: gx[b,ch,y,xx] = sum over (dy,dx) of gpatches[(b,oy,ox)][(ch,dy,dx)] with oy*SH + dy - PH = y,
// ox*SW + dx - PW = xx.  One thread per pixel, terms added in (dy, dx) order.  gpatches row-major
// [rows][cols] or (tiled) tile-major [rows/64][cols][64].
__global__ __launch_bounds__(256) void conv_fold(const float *__restrict__ gp, float *__restrict__ gx, ConvGeom g, int cols,
                                                  int tiled) {
    const long long total = (long long)g.B * g.C * g.H * g.W;
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    const int xx = (int)(e % g.W), y = (int)((e / g.W) % g.H);
    const int ch = (int)((e / ((long long)g.W * g.H)) % g.C);
    const long long b = e / ((long long)g.W * g.H * g.C);
    float acc = 0.0f;
    for (int dy = 0; dy < g.KH; ++dy) {
        const int ny = y + g.PH - dy;
        if (ny < 0 || ny % g.SH) continue;
        const int oy = ny / g.SH;
        if (oy >= g.OH) continue;
        for (int dx = 0; dx < g.KW; ++dx) {
            const int nx = xx + g.PW - dx;
            if (nx < 0 || nx % g.SW) continue;
            const int ox = nx / g.SW;
            if (ox >= g.OW) continue;
            const long long r = (b * g.OH + oy) * g.OW + ox;
            const int c = (ch * g.KH + dy) * g.KW + dx;
            acc += tiled ? gp[((r >> 6) * cols + c) * 64 + (r & 63)] : gp[r * cols + c];
        }
    }
    gx[e] = acc;
}

static int conv_geom(ConvGeom &g, int B, int C, int H, int W, int KH, int KW, int SH, int SW, int PH, int PW) {
    if (B <= 0 || C <= 0 || H <= 0 || W <= 0 || KH <= 0 || KW <= 0 || SH <= 0 || SW <= 0 || PH < 0 || PW < 0)
        return DL_ERR_SHAPE;
    if (H + 2 * PH < KH || W + 2 * PW < KW) return DL_ERR_SHAPE;
    if (KH > 0xffff || KW > 0xffff || (long long)C * KH * KW > CONV_MAX_COLS) return DL_ERR_UNSUPPORTED;
    if ((long long)C * H * W > 0x7fffffffLL) return DL_ERR_UNSUPPORTED;
    g = {B, C, H, W, KH, KW, SH, SW, PH, PW, (H + 2 * PH - KH) / SH + 1, (W + 2 * PW - KW) / SW + 1};
    if ((long long)B * g.OH * g.OW > 0x7fffffffLL * 64) return DL_ERR_UNSUPPORTED;
    return DL_OK;
}

extern "C" long long dl_unfold_rows(int B, int H, int W, int KH, int KW, int SH, int SW, int PH, int PW) {
    ConvGeom g;
    if (conv_geom(g, B, 1, H, W, KH, KW, SH, SW, PH, PW)) return 0;
    return (long long)B * g.OH * g.OW;
}

extern "C" int dl_unfold_flip(const float *x, const uint8_t *flip, float *patches, void *planes, int B, int C, int H, int W,
                              int KH, int KW, int SH, int SW, int PH, int PW, void *stream);
extern "C" int dl_unfold(const float *x, float *patches, void *planes, int B, int C, int H, int W, int KH, int KW, int SH,
                         int SW, int PH, int PW, void *stream) {
    return dl_unfold_flip(x, nullptr, patches, planes, B, C, H, W, KH, KW, SH, SW, PH, PW, stream);
}

extern "C" int dl_unfold_flip(const float *x, const uint8_t *flip, float *patches, void *planes, int B, int C, int H, int W,
                              int KH, int KW, int SH, int SW, int PH, int PW, void *stream) {
    if (!x || (!patches && !planes)) return DL_ERR_NULL;
    ConvGeom g;
    int rc = conv_geom(g, B, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    const long long rows = (long long)B * g.OH * g.OW;
    const int cols = C * KH * KW, grid = dl_ceil_div(rows, 64);
    if (patches) DL_TIMED("conv_unfold_rows", s, (conv_unfold_rows<<<grid, 256, 0, s>>>(x, patches, g, rows, cols, flip)));
    if (planes)
        DL_TIMED("conv_unfold_planes", s,
                 (conv_unfold_planes<<<grid, 256, 0, s>>>(x, (unsigned long long *)planes, g, rows, cols, flip)));
    return dl_launch_status();
}

extern "C" int dl_fold(const float *gpatches, int tiled, float *gx, int B, int C, int H, int W, int KH, int KW, int SH,
                       int SW, int PH, int PW, void *stream) {
    if (!gpatches || !gx) return DL_ERR_NULL;
    ConvGeom g;
    int rc = conv_geom(g, B, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    const long long total = (long long)B * C * H * W;
    DL_TIMED("conv_fold", s, (conv_fold<<<dl_ceil_div(total, 256), 256, 0, s>>>(gpatches, gx, g, C * KH * KW, tiled)));
    return dl_launch_status();
}
