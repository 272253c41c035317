// Launchers of the generic (any k) DWN kernels, defined in dwn_generic.hip.
// scale == null: EFD weights alpha * beta^h; otherwise scale[n] / (h + 1), which also multiplies the table gradient.
// alpha_n / beta_n (nullable, device [N]): every node's own alpha and beta instead of the scalars.
#pragma once
#include <hip/hip_runtime.h>

int dwn_generic_forward(const float *x, const int *idx32, const float *luts, float *y, int B, int I, int N, int k, int O,
                        hipStream_t s);
int dwn_generic_backward(const float *x, const int *idx32, const int *inv_ptr, const int *inv_pos, const float *luts,
                         const float *gy, float alpha, float beta, const float *scale, float *gx, float *gluts, int B, int I,
                         int N, int k, int O, hipStream_t s, const float *alpha_n = nullptr, const float *beta_n = nullptr,
                         float beta_abs_max = 1.0f, void *ws = nullptr, size_t ws_bytes = 0);
// bytes of workspace with which the EFD backward (|beta| <= 1/2) takes its input gradient from smoothed tables
size_t dwn_generic_smooth_bytes(int N, int k, int O);
// Eval forward for any input values; returns at once when *skip_if_set (device, nullable) is non-zero.
int dwn_generic_eval(const float *x, const int *idx32, const float *luts, float *y, int B, int I, int N, int k, int O,
                     const int *skip_if_set, hipStream_t s);
