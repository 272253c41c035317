/* difflut_hip.h - C ABI of the MI355X (gfx950) DiffLUT hot path.
 *
 * One shared library, libdifflut_hip.so, built from difflut_amd/csrc/ by hipcc.
 * Plain pointers and sizes only; every pointer is DEVICE memory unless it says
 * host.  `stream` is a hipStream_t passed as void*.  Nothing here allocates or
 * frees device memory and nothing synchronises the device (except
 * dl_profile_read, which waits for the kernels it reports on): outputs and
 * workspaces come from the caller, kernels are enqueued on `stream`.
 * The library itself holds two things in device memory, per GPU, for the life of the process: the scratch of
 * dl_dwn_layer_fwd_static (DL_DWN_STATIC_SCRATCH_BYTES) and 34 KB of pacing state of the input-gradient kernel
 * for big layers (how fast its blocks step through the batch, adjusted from launch to launch; it changes
 * durations only, never a result).
 *
 * Return value of every int function: 0 = ok, negative = argument error
 * (DL_ERR_*), positive = a hipError_t from a launch.  dl_error_string() turns
 * either into text.
 *
 * Each entry point names the reference interface it replaces (paths relative
 * to the aplesner/difflut checkout).
 *
 * Shapes: B batch rows, I layer inputs, N nodes, k inputs per node, L = 2^k
 * table entries, O outputs per node, M = N*k selections of a learnable layer.
 * All float tensors are fp32, row-major, contiguous.  Workspaces, `saved` buffers, bit-planes and tile-major
 * tensors must be 16-byte aligned (what hipMalloc and torch's allocator return is enough); fp32 tensors
 * take vectorised paths when they are 16-byte aligned and their row length is a multiple of 4.
 *
 * Size limits (DL_ERR_UNSUPPORTED beyond them, checked on the host before anything is launched):
 * k <= DL_MAX_K; N * O * 2^k < 2^31 table entries per layer; I <= 2^28 for the k <= 6 DWN kernels;
 * B <= 4 000 000 rows for the probabilistic entry points and dl_thermometer_planes (their batch tiles are a
 * grid dimension); C * KH * KW <= 4096 patch columns for dl_unfold / dl_fold.  The DWN layers take
 * B <= 2^31 - 65 rows as long as their 1-D grids fit 31 bits: ceil(N*O/128) * T and ceil(I/4) * T + N*O*2^k/1024
 * blocks, T = ceil(B/64) rounded up to a multiple of 8.  The gathers and the bit-plane packing take any B that fits an int.
 */
#ifndef DIFFLUT_HIP_H
#define DIFFLUT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DL_OK 0
#define DL_ERR_NULL (-1)        /* a required pointer is null */
#define DL_ERR_SHAPE (-2)       /* a size is <= 0 or inconsistent */
#define DL_ERR_UNSUPPORTED (-3) /* k, O or an option outside what the kernels cover */
#define DL_ERR_WORKSPACE (-4)   /* workspace smaller than the matching *_workspace_bytes() */
#define DL_ERR_INDEX (-5)       /* an index table entry is outside [0, I) (host-checked entry points only) */
#define DL_ERR_SCRATCH (-6)     /* dl_dwn_layer_fwd_static: the call needs more than DL_DWN_STATIC_SCRATCH_BYTES */

#define DL_MAX_FAST_K 6  /* tables of up to 64 entries sit one-per-lane in a wavefront */
#define DL_MAX_K 16      /* generic kernels */

int dl_version(void);
const char *dl_error_string(int code);

/* ------------------------------------------------------------------------
 * RandomLayer mapping gather.
 * Replaces mapping_cuda.forward / .backward
 *   (difflut/layers/cuda/mapping_cuda.cpp:25-74, mapping_cuda_kernel.cu:30-56,136-162),
 * called from RandomLayer.get_mapping (difflut/layers/random_layer.py:258-304).
 * idx is [N,k]; idx_bits says whether it holds int16 (16) or int32 (32) entries,
 * the two dtypes the reference registers (random_layer.py:214).
 * ------------------------------------------------------------------------ */
/* m[b,n,j] = x[b, idx[n,j]]          x [B,I] -> m [B,N,k] */
int dl_gather_fwd(const float *x, const void *idx, int idx_bits, float *m,
                  int B, int I, int N, int k, void *stream);
/* gx[b,i] = sum_{(n,j): idx[n,j]=i} gm[b,n,j]; gx [B,I] is overwritten.
 * inv_ptr [I+1] / inv_pos [N*k] is the inverse of idx in CSR form (inv_pos holds
 * flat positions n*k+j, ascending inside each input): the sum is a gather in a
 * fixed order, so results are run-to-run identical (the reference uses atomics). */
int dl_gather_bwd(const float *gm, const int32_t *inv_ptr, const int32_t *inv_pos, float *gx,
                  int B, int I, int N, int k, void *stream);

/* ------------------------------------------------------------------------
 * RandomLayer + DWN nodes, whole layer in one call.
 * Replaces the per-node loop of RandomLayer.forward (random_layer.py:306-340)
 * over efd_cuda.forward/.backward (difflut/nodes/cuda/efd_cuda.cpp:22-45,
 * efd_cuda_kernel.cu:12-43,79-189) and the layer-wide efd_fused_cuda.forward/
 * .backward (efd_fused_cuda.cpp:19-34, efd_fused_cuda_kernel.cu:11-197).
 *   idx32 [N,k] int32 (the registered int16/int32 table widened once by the host)
 *   luts  [N,O,L]     (the N node tables [O,L] of dwn_node.py:423 stacked)
 *   y     [B,N*O]
 * Training forward: addr = sum_j [x[b,idx[n,j]] >= 0.5] << j;  y[b,n,d] = luts[n,d,addr].
 * `saved` (dl_dwn_saved_bytes) receives what the backward needs instead of x:
 * for k <= DL_MAX_FAST_K the address of every (node, row), node-major.
 * `ws` (dl_dwn_fwd_workspace_bytes) is scratch that may be reused after the call.
 * ------------------------------------------------------------------------ */
size_t dl_dwn_saved_bytes(int B, int I, int N, int k, int O);
size_t dl_dwn_fwd_workspace_bytes(int B, int I, int N, int k, int O);
size_t dl_dwn_bwd_workspace_bytes(int B, int I, int N, int k, int O);
int dl_dwn_layer_fwd(const float *x, const int32_t *idx32, const float *luts, float *y,
                     void *saved, void *ws, size_t ws_bytes,
                     int B, int I, int N, int k, int O, void *stream);
/* dl_dwn_layer_fwd for callers that cannot allocate device memory at all - code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc - and so cannot bring a workspace either.  It has no
 * counterpart in the reference.  Same arguments minus `ws`, same kernels, same results: the bit-planes that
 * dl_dwn_layer_fwd puts into `ws` go to a device array owned by the library instead
 * (DL_DWN_STATIC_SCRATCH_BYTES on every GPU the library runs on, held until the process ends).  The call
 * allocates and frees nothing.  Limit: ceil(B/64) * I * 8 <= DL_DWN_STATIC_SCRATCH_BYTES when
 * k <= DL_MAX_FAST_K (e.g. B = 4096 with I = 16384), otherwise DL_ERR_SCRATCH; larger k uses no scratch.
 * All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams, two threads)
 * race on it and must be serialised by the caller.  Nothing in it has to survive between calls.
 * The first call on each device also looks up the device address of the array (hipGetSymbolAddress, which may
 * load the code object): make that call before any stream capture begins; every later call on the device only
 * enqueues kernels and can be captured. */
#define DL_DWN_STATIC_SCRATCH_BYTES (8u << 20)
int dl_dwn_layer_fwd_static(const float *x, const int32_t *idx32, const float *luts, float *y,
                            void *saved, int B, int I, int N, int k, int O, void *stream);
/* Extended-finite-difference backward (dwn_node.py:167-229):
 *   gx[b,i]     = sum_{(n,j): idx=i} alpha * sum_d gy[b,n,d] *
 *                 sum_kappa s(kappa_j) luts[n,d,kappa] beta^popc((addr ^ kappa) & ~(1<<j))
 *   gluts[n,d,e] = sum_b [addr(b,n) = e] gy[b,n,d]
 * gx may be null (input does not need a gradient); gx and gluts are overwritten.
 * x is only read when k > DL_MAX_FAST_K (then `saved` is unused) and may be null otherwise.  For k > DL_MAX_FAST_K the
 * workspace is optional (ws may be null): with dl_dwn_bwd_workspace_bytes of it, |beta| <= 1/2 and k <= 12 the input
 * gradient is taken from tables smoothed once per call (two loads per row and connection); without, from the 2^k-term
 * sum of the formula per row and connection.  The table gradient of that path is summed with atomics. */
int dl_dwn_layer_bwd(const float *x, const void *saved, const int32_t *idx32,
                     const int32_t *inv_ptr, const int32_t *inv_pos,
                     const float *luts, const float *gy, float alpha, float beta,
                     float *gx, float *gluts, void *ws, size_t ws_bytes,
                     int B, int I, int N, int k, int O, void *stream);
/* dl_dwn_layer_bwd with every node's own alpha and beta: the reference keeps them as per-node buffers and reads
 * each node's pair in its forward (dwn_node.py:417-418, 450), so a state dict may carry different values per node.
 * alpha_n, beta_n: device arrays [N]; beta_abs_max = max_n |beta_n[n]| (host value). */
int dl_dwn_layer_bwd_nodes(const float *x, const void *saved, const int32_t *idx32,
                           const int32_t *inv_ptr, const int32_t *inv_pos,
                           const float *luts, const float *gy, const float *alpha_n, const float *beta_n,
                           float beta_abs_max, float *gx, float *gluts, void *ws, size_t ws_bytes,
                           int B, int I, int N, int k, int O, void *stream);
/* Chained DWN layers.  No counterpart in the reference, which materialises the [B, N] fp32
 * activations between layers (random_layer.py:306-340 per layer): a following DWN layer only
 * thresholds them, so layer l can hand layer l+1 its output as bit-planes
 * ([ceil(B/64)][C] uint64, bit r of word (t, c) = (value[64t+r][c] >= 0.5)), and layer l+1 can hand
 * back its input gradient tile-major ([ceil(B/64)][C][64] fp32), which is the form the backward
 * of layer l reads.  k <= DL_MAX_FAST_K only (DL_ERR_UNSUPPORTED otherwise).
 *   dl_dwn_pack_planes      : x [B,I] fp32 -> planes
 *   dl_dwn_layer_fwd_planes : planes_in -> y [B,N*O] (nullable) and/or planes_out (nullable); saved as above
 *   dl_dwn_layer_bwd_tiled  : gy row-major [B,N*O] or (gy_tiled) tile-major; gx (nullable) row-major
 *                             [B,I] or (gx_tiled) tile-major; workspace dl_dwn_bwd_workspace_bytes */
size_t dl_dwn_planes_bytes(int B, int C);
size_t dl_dwn_tiled_bytes(int B, int C);
int dl_dwn_pack_planes(const float *x, void *planes, int B, int I, void *stream);
int dl_dwn_layer_fwd_planes(const void *planes_in, const int32_t *idx32, const float *luts, float *y,
                            void *planes_out, void *saved, int B, int I, int N, int k, int O, void *stream);
int dl_dwn_layer_bwd_tiled(const void *saved, const int32_t *inv_ptr, const int32_t *inv_pos,
                           const float *luts, const float *gy, int gy_tiled, float alpha, float beta,
                           float *gx, int gx_tiled, float *gluts, void *ws, size_t ws_bytes,
                           int B, int I, int N, int k, int O, void *stream);
/* GroupSum head on the last layer of a chain (utils/modules.py:116-163 after random_layer.py:306-340).
 * No counterpart in the reference, which writes the layer's [B, N*O] output, sums it per group and in
 * the backward expands the [B, groups] gradient to [B, N*O] again.  Here the last layer hands out
 *   logits[b][g] = (sum of its columns g*gs .. (g+1)*gs - 1) / tau,  gs = ceil(N*O / groups)
 * (columns past N*O count as 0, as the zero-padding of GroupSum does) and its backward takes the
 * gradient of the logits: column c gets glogits[b][c / gs] / tau.  Groups must be at least 64 columns
 * wide (DL_ERR_UNSUPPORTED otherwise), k <= DL_MAX_FAST_K.  Sums run in a fixed order (reproducible).
 *   workspace of the forward: dl_dwn_groups_workspace_bytes; of the backward: dl_dwn_bwd_workspace_bytes */
size_t dl_dwn_groups_workspace_bytes(int B, int N, int O, int groups);
int dl_dwn_layer_fwd_planes_groups(const void *planes_in, const int32_t *idx32, const float *luts, float *logits,
                                   void *saved, void *ws, size_t ws_bytes, int B, int I, int N, int k, int O,
                                   int groups, float tau, void *stream);
int dl_dwn_layer_bwd_groups(const void *saved, const int32_t *inv_ptr, const int32_t *inv_pos, const float *luts,
                            const float *glogits, int groups, float tau, float alpha, float beta,
                            float *gx, int gx_tiled, float *gluts, void *ws, size_t ws_bytes,
                            int B, int I, int N, int k, int O, void *stream);
/* The chained backward with every node's own alpha and beta (device arrays [N]; the reference reads each node's
 * buffers, difflut/nodes/dwn_node.py:417-418,450).  beta_abs_max = max |beta_n| (a host value) selects the form of
 * the coefficient table.  gy_form: 0 = gy row-major [B, N*O], 1 = tile-major [B/64][N*O][64], 2 = the [B, groups]
 * gradient of a GroupSum head's logits (groups, tau as in dl_dwn_layer_bwd_groups; ignored otherwise). */
int dl_dwn_layer_bwd_chain_nodes(const void *saved, const int32_t *inv_ptr, const int32_t *inv_pos, const float *luts,
                                 const float *gy, int gy_form, int groups, float tau, const float *alpha_n,
                                 const float *beta_n, float beta_abs_max, float *gx, int gx_tiled, float *gluts,
                                 void *ws, size_t ws_bytes, int B, int I, int N, int k, int O, void *stream);
/* dl_dwn_layer_bwd_chain_nodes that can also produce the table gradient of the layer IN FRONT.  In a chain this layer's
 * input gradient is that layer's output gradient (random_layer.py:306-340 run layer by layer), so the gather adds every
 * batch tile it has just summed into that layer's bins, and that layer's own pass over its [B, N] output gradient is
 * left out.  No counterpart in the reference, which runs each node's backward on its own (efd_cuda_kernel.cu:195-331).
 *   prev_saved (nullable, 16-byte aligned): what the forward of the layer in front saved (I nodes of k_prev inputs, ONE
 *     output each);
 *     prev_gluts [I, 2^k_prev] then receives its table gradient.  Needs gx tile-major (gx_tiled = 1) and
 *     dl_dwn_chain_fusable(...) == 1 (k, k_prev <= DL_MAX_FAST_K, O == 1, beta_abs_max <= 1/2, N k < 32 I);
 *     workspace dl_dwn_bwd_fused_workspace_bytes.  Bins are summed per block and then in block order: reproducible,
 *     but a different order of additions than dl_dwn_layer_bwd_tiled's for the same table.
 *   gluts (nullable): NULL when this layer's own table gradient has already been produced by the call for the layer
 *     behind it; gy must then be tile-major (gy_form 1) and gx or prev_saved non-NULL.
 *   gx (nullable with prev_saved): NULL when nobody reads this layer's input gradient after the bins of the layer in
 *     front are filled (that layer is the first of the chain and its input needs no gradient): the sums are then made
 *     for the bins only and not stored (B x I x 4 bytes less to write). */
int dl_dwn_chain_fusable(int B, int I, int N, int k, int O, int k_prev, float beta_abs_max);
size_t dl_dwn_bwd_fused_workspace_bytes(int B, int I, int N, int k, int O, int k_prev);
int dl_dwn_layer_bwd_chain_fused(const void *saved, const int32_t *inv_ptr, const int32_t *inv_pos, const float *luts,
                                 const float *gy, int gy_form, int groups, float tau, const float *alpha_n,
                                 const float *beta_n, float beta_abs_max, float *gx, int gx_tiled, float *gluts,
                                 const void *prev_saved, int k_prev, float *prev_gluts, void *ws, size_t ws_bytes,
                                 int B, int I, int N, int k, int O, void *stream);
/* The eval forward below with a workspace (dl_dwn_eval_workspace_bytes): the same result for any input, and
 * the bit-plane kernels' speed when every input value is exactly 0 or 1 (checked on the device while packing;
 * no host synchronisation - both kernels are launched and one returns at once). */
size_t dl_dwn_eval_workspace_bytes(int B, int I, int N, int k, int O);
int dl_dwn_layer_eval_ws(const float *x, const int32_t *idx32, const float *luts, float *y, void *ws,
                         size_t ws_bytes, int B, int I, int N, int k, int O, void *stream);
/* Inference on binary activations (DWNNode.forward_eval, dwn_node.py:457-483, for inputs that are exactly
 * 0 or 1 - what a thermometer encoder or a preceding layer's eval output delivers; there its address
 * floor(sum_j x_j 2^j) equals the thresholded one).  planes_in as dl_dwn_pack_planes /
 * dl_thermometer_planes / a preceding call write them; y (nullable) = (table entry >= 0.5) as 0/1 fp32
 * [B, N*O]; planes_out (nullable) = the same bits as planes for the next layer.  The *_groups form
 * returns GroupSum of that output instead (utils/modules.py:116-163; workspace
 * dl_dwn_groups_workspace_bytes, groups >= 64 columns wide).  No counterpart in the reference, which
 * runs its layers on [B, N] fp32 tensors in eval mode too.  k <= DL_MAX_FAST_K. */
int dl_dwn_layer_eval_planes(const void *planes_in, const int32_t *idx32, const float *luts, float *y,
                             void *planes_out, int B, int I, int N, int k, int O, void *stream);
int dl_dwn_layer_eval_planes_groups(const void *planes_in, const int32_t *idx32, const float *luts, float *logits,
                                    void *ws, size_t ws_bytes, int B, int I, int N, int k, int O,
                                    int groups, float tau, void *stream);
/* Eval forward (DWNNode.forward_eval, dwn_node.py:457-483): addr = floor(sum_j x_j 2^j)
 * with no thresholding of x (clamped to the table), y = (luts[n,d,addr] >= 0.5) as 0/1. */
int dl_dwn_layer_eval(const float *x, const int32_t *idx32, const float *luts, float *y,
                      int B, int I, int N, int k, int O, void *stream);

/* ------------------------------------------------------------------------
 * RandomLayer + gradient-stabilised DWN nodes (node type "dwn_stable").
 * Replaces the node loop over dwn_stable_cuda.forward/.backward
 * (difflut/nodes/cuda/dwn_stable_cuda_kernel.cu:13-74, 84-242) and
 * GradientStabilizedFunctionCPU (difflut/nodes/dwn_stable_node.py:113-206).
 * The training forward is the DWN lookup on luts = sigmoid(raw_luts): dl_table_sigmoid_fwd, then
 * dl_dwn_layer_fwd.  The backward is the EFD sum with the weight 1/(h+1) in place of
 * alpha*beta^h, h = popc((addr ^ kappa) & ~(1<<j)), times the node's gradient scale:
 *   gx[b,i]      = sum_{(n,j): idx=i} scale[n] * sum_d gy[b,n,d] *
 *                  sum_kappa s(kappa_j) luts[n,d,kappa] / (h + 1)
 *   gluts[n,d,e] = scale[n] * sum_b [addr(b,n) = e] gy[b,n,d]
 * gradient_scale [N] is a DEVICE array (the nodes' `gradient_scale` parameters stacked), so no
 * value has to be read back by the host.  saved / ws / x as for dl_dwn_layer_bwd.
 * dl_table_sigmoid_bwd is the adjoint of the table sigmoid: graw = gluts * luts * (1 - luts)
 * (what autograd applies for `_get_luts`, dwn_stable_node.py:289-295, hybrid_node.py:309-315).
 * ------------------------------------------------------------------------ */
int dl_table_sigmoid_fwd(const float *raw, float *luts, long long count, void *stream);
int dl_table_sigmoid_bwd(const float *gluts, const float *luts, float *graw, long long count, void *stream);
int dl_dwn_stable_layer_bwd(const float *x, const void *saved, const int32_t *idx32,
                            const int32_t *inv_ptr, const int32_t *inv_pos,
                            const float *luts, const float *gy, const float *gradient_scale,
                            float *gx, float *gluts, void *ws, size_t ws_bytes,
                            int B, int I, int N, int k, int O, void *stream);

/* ------------------------------------------------------------------------
 * RandomLayer + hybrid nodes (node type "hybrid"): thresholded lookup forward (dl_table_sigmoid_fwd,
 * then dl_dwn_layer_fwd), probabilistic backward.  Replaces the node loop over
 * hybrid_cuda.forward/.backward (difflut/nodes/cuda/hybrid_cuda_kernel.cu:7-126, 129-243) and
 * HybridFunctionCPU (difflut/nodes/hybrid_node.py:105-204):
 *   p[b,n,a]     = prod_j (x_j a_j + (1 - x_j)(1 - a_j)),  x_j = x[b, idx[n,j]] as given
 *   gluts[n,d,a] = sum_b p[b,n,a] gy[b,n,d]
 *   gx[b,i]      = sum_{(n,j): idx=i} sum_d gy[b,n,d] sum_a luts[n,d,a] p[b,n,a]
 *                  (a_j - x_j) / (x_j (1 - x_j) + 1e-8)
 * computed as dy/dx_j of the multilinear interpolation times q/(q + 1e-8), q = x_j (1 - x_j):
 * the same value, and like the reference exactly 0 where x_j is 0 or 1.
 * luts [N,O,L]; gx [B,I] (nullable) and gluts [N,O,L] are overwritten.
 * ------------------------------------------------------------------------ */
size_t dl_hybrid_bwd_workspace_bytes(int B, int I, int N, int k, int O);
int dl_hybrid_layer_bwd(const float *x, const int32_t *idx32,
                        const int32_t *inv_ptr, const int32_t *inv_pos,
                        const float *luts, const float *gy, float *gx, float *gluts,
                        void *ws, size_t ws_bytes,
                        int B, int I, int N, int k, int O, void *stream);

/* ------------------------------------------------------------------------
 * RandomLayer + Probabilistic nodes, whole layer in one call.
 * Replaces the node loop over probabilistic_cuda.forward/.backward
 * (difflut/nodes/cuda/probabilistic_cuda.cpp:22-49, probabilistic_cuda_kernel.cu:7-307)
 * and the CPU branch of ProbabilisticNode.forward_train (probabilistic_node.py:284-300).
 *   raw_w [N,L,O] (the node parameters raw_weights [L,O] stacked), temperature T:
 *   y[b,n,d] = sum_a sigmoid(raw_w[n,a,d] / max(T,1e-6)) * prod_j (x_j a_j + (1-x_j)(1-a_j)),
 *   x_j = x[b, idx[n,j]] used as given (no clamping: inputs are probabilities).
 * Backward is the exact derivative of that expression (what autograd gives the
 * reference's CPU path): gx [B,I] (nullable), graw [N,L,O]; both overwritten.
 * Both directions re-tile their [batch, feature] operands (lanes = batch rows inside
 * the kernels).
 * ------------------------------------------------------------------------ */
size_t dl_prob_saved_bytes(int B, int I, int N, int k, int O);
size_t dl_prob_bwd_workspace_bytes(int B, int I, int N, int k, int O);
/* `saved` (dl_prob_saved_bytes) receives the sigmoid table and the re-tiled input. */
int dl_prob_layer_fwd(const float *x, const int32_t *idx32, const float *raw_w, float temperature,
                      float *y, void *saved, size_t saved_bytes,
                      int B, int I, int N, int k, int O, void *stream);
/* `saved` may be null: then both are rebuilt from x, raw_w and temperature. */
int dl_prob_layer_bwd(const float *x, const void *saved, const int32_t *idx32,
                      const int32_t *inv_ptr, const int32_t *inv_pos,
                      const float *raw_w, float temperature, const float *gy,
                      float *gx, float *graw, void *ws, size_t ws_bytes,
                      int B, int I, int N, int k, int O, void *stream);
/* The same forward and backward with every node's own temperature (device array [N]; the reference reads each
 * node's `temperature` buffer, difflut/nodes/probabilistic_node.py:277-282, 224-239). */
int dl_prob_layer_fwd_nodes(const float *x, const int32_t *idx32, const float *raw_w, const float *temperature_n,
                            float *y, void *saved, size_t saved_bytes, int B, int I, int N, int k, int O, void *stream);
int dl_prob_layer_bwd_nodes(const float *x, const void *saved, const int32_t *idx32, const int32_t *inv_ptr,
                            const int32_t *inv_pos, const float *raw_w, const float *temperature_n, const float *gy,
                            float *gx, float *graw, void *ws, size_t ws_bytes, int B, int I, int N, int k, int O,
                            void *stream);
/* Eval forward (probabilistic_node.py:302-328): y = (sigmoid(raw_w[n,addr,d]/T) >= 0.5). */
int dl_prob_layer_eval(const float *x, const int32_t *idx32, const float *raw_w, float temperature,
                       float *y, int B, int I, int N, int k, int O, void *stream);
/* The same with a workspace (dl_prob_eval_workspace_bytes): the binarised sigmoid tables are looked up through
 * the DWN eval path, i.e. through bit-planes when every input value is exactly 0 or 1 (decided on the device,
 * same result for any input). */
size_t dl_prob_eval_workspace_bytes(int B, int I, int N, int k, int O);
int dl_prob_layer_eval_ws(const float *x, const int32_t *idx32, const float *raw_w, float temperature, float *y,
                          void *ws, size_t ws_bytes, int B, int I, int N, int k, int O, void *stream);
int dl_prob_layer_eval_ws_nodes(const float *x, const int32_t *idx32, const float *raw_w, const float *temperature_n,
                                float *y, void *ws, size_t ws_bytes, int B, int I, int N, int k, int O, void *stream);

/* ------------------------------------------------------------------------
 * LearnableLayer soft connectivity (training) and hard selection (eval).
 * Replaces F.softmax(W / tau, -1) followed by torch.matmul(x, S.t()) and its
 * autograd (difflut/layers/learnable_layer.py:254-255), the forward-only
 * learnable_mapping_cuda.soft_forward (learnable_mapping_cuda_kernel.cu:99-223),
 * and learnable_mapping_cuda.forward/.backward for argmax selection
 * (learnable_mapping_cuda_kernel.cu:22-81,236-257; learnable_layer.py:216-236).
 *   x [B,I], W [M,I], m [B,M];   S = softmax(W / tau) along I, never materialised.
 * precision: 0 = fp32 operands on the fp32 matrix cores (reference numerics),
 *            1 = bf16 operands, fp32 accumulation (tolerance documented with the tests).
 * stats (dl_soft_map_saved_bytes bytes) is written by the forward and read by the backward.
 *   gx = gm * S,   gW = S * (G - r) / tau with G = gm^T x and r[o] = sum_b gm[b,o] m[b,o].
 * ------------------------------------------------------------------------ */
/* size of `stats`: what the forward keeps for the backward (row maximum and 1/sum; with
 * precision 1 also the bf16 softmax numerators, M*I*2 bytes) */
size_t dl_soft_map_saved_bytes(int B, int I, int M, int precision);
/* scratch of either direction (one size for both): the backward's r [M] and partial gx products and,
 * with precision 1, the bf16 copies of x and gm.  The forward only needs it with precision 1. */
size_t dl_soft_map_workspace_bytes(int B, int I, int M, int precision);
int dl_soft_map_fwd(const float *x, const float *W, float tau, float *m, float *stats,
                    void *ws, size_t ws_bytes, int B, int I, int M, int precision, void *stream);
int dl_soft_map_bwd(const float *x, const float *W, float tau, const float *m, const float *stats,
                    const float *gm, float *gx, float *gW, void *ws, size_t ws_bytes,
                    int B, int I, int M, int precision, void *stream);
/* sel[o] = argmax_i W[o,i] (lowest index on ties), int32 [M]. */
int dl_row_argmax(const float *W, int32_t *sel, int M, int I, void *stream);
/* m[b,o] = x[b, sel[o]] */
int dl_hard_select_fwd(const float *x, const int32_t *sel, float *m, int B, int I, int M, void *stream);
/* gx[b,i] = sum_{o: sel[o]=i} gm[b,o]; CSR inverse of sel as for dl_gather_bwd (k = 1). */
int dl_hard_select_bwd(const float *gm, const int32_t *inv_ptr, const int32_t *inv_pos, float *gx,
                       int B, int I, int M, void *stream);

/* ------------------------------------------------------------------------
 * Either side of the layers in the training configurations.
 * Thermometer encode (difflut/encoder/thermometer.py:89-116):
 *   bits[b, f*nbits + j] = (x[b,f] > thr[f,j]) as 0/1, x [B,F], thr [F,nbits].
 * GroupSum (difflut/utils/modules.py:116-163): features zero-padded to a multiple of
 *   groups, y[b,g] = sum of group g / tau; backward gx[b,f] = gy[b, f / group_size] / tau.
 * ------------------------------------------------------------------------ */
int dl_thermometer_encode(const float *x, const float *thr, float *bits, int B, int F, int nbits,
                          void *stream);
/* The same comparison written as the bit-planes a chained DWN layer reads (dl_dwn_layer_fwd_planes,
 * width F*nbits): no counterpart in the reference, which materialises the [B, F*nbits] fp32 tensor
 * (thermometer.py:108-116) for the first layer to threshold again.  planes: dl_dwn_planes_bytes(B, F*nbits). */
int dl_thermometer_planes(const float *x, const float *thr, void *planes, int B, int F, int nbits,
                          void *stream);
int dl_group_sum_fwd(const float *x, float *y, int B, int F, int groups, float tau, void *stream);
/* Cross-entropy with mean reduction on the [B, C] logits that GroupSum returns (the loss of the training
 * configurations; torch.nn.CrossEntropyLoss in the reference's examples and tests, e.g.
 * tests/test_layers/test_convolutional_learning.py): *loss = mean_b(logsumexp(logits[b]) - logits[b][labels[b]]),
 * glogits = d loss / d logits = (softmax - onehot) / B, both from one pass over the logits; the B row losses
 * are added in a fixed order.  labels are int64 class indices; rows whose label is outside [0, C) add nothing.
 * Workspace: dl_cross_entropy_workspace_bytes(B). */
size_t dl_cross_entropy_workspace_bytes(int B);
int dl_cross_entropy(const float *logits, const long long *labels, float *loss, float *glogits, void *ws,
                     size_t ws_bytes, int B, int C, void *stream);
int dl_group_sum_bwd(const float *gy, float *gx, int B, int F, int groups, float tau, void *stream);

/* ------------------------------------------------------------------------
 * Adam update of parameter banks (the [N, O, 2^k] tensors the layers keep their nodes' tables in): the arithmetic
 * of torch.optim.Adam without amsgrad - what the reference's training scripts apply to the per-node parameters
 * (experiments and examples construct torch.optim.Adam(model.parameters(), lr=...)) - for `count` tensors in one
 * launch.  params / grads / exp_avg / exp_avg_sq and numel are HOST arrays of `count` device pointers / element
 * counts; `step` is the 1-based step number (bias corrections 1 - beta^step are computed on the host in double).
 * In place: params, exp_avg, exp_avg_sq. */
/* Gradient stabilisation of a layer's output gradient (LUTLayerMixin._apply_gradient_stabilization,
 * difflut/layers/base_layer.py:266-339): out = (g - mean) * sqrt(target_std / (mean((g - mean)^2) + eps)) over the
 * whole [rows, cols] tensor (per_row = 0, "layerwise") or per row (per_row = 1, "batchwise"); the mean is subtracted
 * only when subtract_mean is set.  Sums in double, fixed order.  out may equal g only for per_row = 1.  The layerwise
 * form needs dl_grad_stabilize_workspace_bytes(rows, cols, 0) bytes. */
size_t dl_grad_stabilize_workspace_bytes(long long rows, long long cols, int per_row);
int dl_grad_stabilize(const float *g, float *out, long long rows, long long cols, int per_row, float target_std,
                      int subtract_mean, float eps, void *ws, size_t ws_bytes, void *stream);
#define DL_ADAM_MAX_TENSORS 8 /* tensors per launch; more are taken in several launches */
int dl_adam_step(void *const *params, const void *const *grads, void *const *exp_avg, void *const *exp_avg_sq,
                 const long long *numel, int count, float lr, float beta1, float beta2, float eps, float weight_decay,
                 int step, int maximize, void *stream);

/* ------------------------------------------------------------------------
 * Convolutional LUT layer: patch extraction and its adjoint.
 * Replaces nn.Unfold + transpose + contiguous + view in ConvolutionalLayer.forward
 * (difflut/layers/convolutional.py:199-205) and what autograd does for them in the backward.
 *   x [B,C,H,W];  rows r = (b, oy, ox) row-major, OH = (H + 2 PH - KH) / SH + 1 (OW alike);
 *   columns c = (ch, dy, dx) row-major;  patches[r][c] = x[b, ch, oy SH + dy - PH, ox SW + dx - PW], 0 outside.
 * dl_unfold writes `patches` [rows, C KH KW] fp32 (nullable) and/or `planes` (nullable): the same matrix
 * as the bit-planes of (value >= 0.5) that dl_dwn_layer_fwd_planes reads (dl_dwn_planes_bytes(rows, C KH KW));
 * the bit-plane form has no counterpart in the reference.  dl_fold sums a gradient of the patch matrix,
 * row-major or (tiled) tile-major [rows/64][C KH KW][64] as dl_dwn_layer_bwd_tiled writes it, back into
 * gx [B,C,H,W] (overwritten; fixed summation order).  C KH KW <= 4096.  dl_unfold_rows returns B OH OW (0 if
 * the geometry is invalid).
 * ------------------------------------------------------------------------ */
long long dl_unfold_rows(int B, int H, int W, int KH, int KW, int SH, int SW, int PH, int PW);
int dl_unfold(const float *x, float *patches, void *planes, int B, int C, int H, int W,
              int KH, int KW, int SH, int SW, int PH, int PW, void *stream);
int dl_fold(const float *gpatches, int tiled, float *gx, int B, int C, int H, int W,
            int KH, int KW, int SH, int SW, int PH, int PW, void *stream);
/* dl_unfold with the layer's bit-flip augmentation applied to the patch matrix on the way
 * (LUTLayerMixin._apply_bit_flip, difflut/layers/base_layer.py:149-264, called on the patches at
 * convolutional.py:205-207): flip [rows, C KH KW] bytes (nullable), non-zero = that entry becomes v + (1 - 2 v)
 * before it is written or thresholded.  The flip is noise, not a function of x: dl_fold is its backward too. */
int dl_unfold_flip(const float *x, const uint8_t *flip, float *patches, void *planes, int B, int C, int H, int W,
                   int KH, int KW, int SH, int SW, int PH, int PW, void *stream);

/* ------------------------------------------------------------------------
 * Per-kernel timing.  No counterpart in the reference (it has no tracing at all).
 * After dl_profile_enable(1) every kernel launched by the entry points above is
 * bracketed by HIP events on its stream (at most 64 kernels between two reads).
 * dl_profile_read waits for those events, writes the elapsed milliseconds in
 * launch order to ms[], the kernel names separated by ';' to names (host
 * buffers), returns the number of entries and starts a new recording.
 * ------------------------------------------------------------------------ */
int dl_profile_enable(int on);
int dl_profile_read(char *names, size_t names_bytes, float *ms, int max_entries);

#ifdef __cplusplus
}
#endif
#endif /* DIFFLUT_HIP_H */
