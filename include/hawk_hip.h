/*
 * libhawk_hip: C ABI of the MI355X (gfx950) kernels for Hawk's RG-LRU hot path.
 *
 * Plain pointers and sizes only.  Every pointer named "device" must be device memory of
 * the GPU that is current when the call is made.  All calls are asynchronous on `stream`
 * (a hipStream_t passed as void*; NULL is the default stream) unless stated otherwise,
 * never synchronise the device, never allocate or free memory, and may be called from any
 * host thread.  The only host-side state is bookkeeping that no caller can observe: a bit per
 * device recording that a kernel's dynamic-LDS limit has been raised there, and the device
 * address of the fixed scratch array of hawk_rglru_scan_fwd_static.  Every function returns a hawk_status; nothing
 * throws or aborts.
 *
 * Tensors are dense row-major: activations [B,T,D] (strides T*D, D, 1), Lambda [D] fp32,
 * conv weight [W,D] fp32, conv bias [D] fp32, conv state [B,W-1,D], recurrent state [B,D].
 * `dtype` is the element type of the activation tensors of that call.
 *
 * Citations name the interface of the upstream tree (fattorib/hawk-pytorch, paths under
 * hawk/) that each entry point replaces.
 */
#ifndef HAWK_HIP_H_
#define HAWK_HIP_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum hawk_status {
    HAWK_OK = 0,
    HAWK_ERR_NULL_POINTER = 1,  /* a required pointer is NULL */
    HAWK_ERR_BAD_SHAPE = 2,     /* a size is < 1, too large (D and row strides above 2^24 elements,
                                   more than 2^31 - 1 tiles), or breaks a stated divisibility rule */
    HAWK_ERR_BAD_DTYPE = 3,     /* dtype is not a hawk_dtype this entry point supports */
    HAWK_ERR_WORKSPACE = 4,     /* workspace missing or smaller than the size query says */
    HAWK_ERR_LAUNCH = 5,        /* the HIP runtime refused a launch or copy */
    HAWK_ERR_ALIGNMENT = 6,     /* a tensor pointer is not aligned to its element size */
    HAWK_ERR_SCRATCH_LIMIT = 7  /* the problem needs more carry words than the library's fixed
                                   scratch array holds (hawk_rglru_scan_fwd_static only) */
} hawk_status;

typedef enum hawk_dtype {
    HAWK_DTYPE_BF16 = 0, /* bf16 storage, fp32 arithmetic and state */
    HAWK_DTYPE_F32 = 1
} hawk_dtype;

/* Library version (major*10000 + minor*100 + patch) and a static message per status. */
int hawk_version(void);
const char* hawk_status_string(int status);

/* *id <- the identifier of the graph capture `stream` is recording into, or 0 when it is not
 * capturing (hipStreamGetCaptureInfo).  A host that hands launches a workspace can key one
 * buffer per (stream, capture) with it: launches recorded on one stream replay in order, so they
 * can share what eager launches on one stream share.  No upstream counterpart. */
int hawk_stream_capture_id(void* stream, unsigned long long* id);

/* ---------------------------------------------------------------------------------------
 * Scan workspace.  The scan passes carries between tiles through a caller-owned device
 * buffer.  Query its size for a problem shape, allocate it, zero it ONCE with
 * hawk_scan_workspace_init (stream-ordered), then pass it to any number of later scan
 * calls of that or any smaller shape.  Calls that share a workspace must be ordered on
 * one stream; concurrent streams need a workspace each.
 * Upstream allocates nothing comparable: its kernels walk T serially
 * (hawk/scan_fused.py:83, :199).
 * ------------------------------------------------------------------------------------- */
size_t hawk_scan_workspace_bytes(int B, int T, int D, int dtype);
int hawk_scan_workspace_init(void* workspace_device, size_t workspace_bytes, void* stream);
/* Synchronises `stream` and reports in *flag whether any scan on this workspace gave up
 * waiting for a carry (0 = all carries arrived).  A non-zero flag means results of that
 * launch are invalid and the workspace must be re-initialised.  workspace_device == NULL
 * asks about the current device's fixed scratch array (hawk_rglru_scan_fwd_static), which the
 * caller cannot re-initialise: reading a raised flag there lowers it again (a one-word fill
 * kernel on `stream`), so one lost carry is reported once. */
int hawk_scan_workspace_status(const void* workspace_device, void* stream, int* flag);

/* ---------------------------------------------------------------------------------------
 * RG-LRU scan forward.
 *   r = sigmoid(a_rg_lru), i = sigmoid(x_rg_lru), alpha = exp(-8 r softplus(Lambda)),
 *   h_t = alpha_t h_{t-1} + sqrt(1 - alpha_t^2) (i_t x_t),  h_{-1} = 0.
 * Replaces sequential_scan_forward / sequential_scan_fwd_kernel
 * (hawk/scan_fused.py:319-360, :34-109).  Lambda stays fp32 for both dtypes.  Any D >= 1
 * is accepted (upstream requires D % 64 == 0); even D takes the two-channels-per-lane
 * path.  The workspace may be NULL when T fits one tile.
 * Every scan entry point is reproducible: its outputs are a function of the inputs and of
 * (B, T, D, dtypes) alone, never of timing, so two launches on the same data agree bit for
 * bit.  The same sequence inside another batch size may differ in the last bit of fp32
 * intermediate sums (launches with few independent chains group their carries in wider
 * windows).
 * ------------------------------------------------------------------------------------- */
int hawk_rglru_scan_fwd(const void* x, const void* x_rg_lru, const void* a_rg_lru,
                        const float* a_param, void* h, int B, int T, int D, int dtype,
                        void* workspace_device, size_t workspace_bytes, void* stream);

/* hawk_rglru_scan_fwd for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops, harnesses that forbid allocation).  It has no counterpart
 * upstream.  Same kernels, same arguments and same results bit for bit, but the carry words
 * live in an array of HAWK_STATIC_SCRATCH_BYTES that is part of the library's device code:
 * every GPU the library is used on holds one such array from the first call there until the
 * process ends.  The call allocates and frees nothing.
 *   limit   hawk_rglru_scan_fwd_static_bytes(B, T, D, dtype), the bytes of the array a shape
 *           uses, must not exceed HAWK_STATIC_SCRATCH_BYTES: at most
 *           ceil(T / 128) * B * D * 24 + 1024 bytes, and 0 when T <= 128; beyond it the call
 *           returns HAWK_ERR_SCRATCH_LIMIT and launches nothing.  B=8, T=4096, D=2560 needs
 *           15.0 MiB.
 *   sharing every call on a GPU uses that GPU's one array, so calls must not overlap there:
 *           order them on one stream (or with events).  Two overlapping calls race.
 *   set-up  the first call on a device looks up the array's device address (the device must
 *           be current, as for every call).  Nothing is ever cleared: the array starts as
 *           zeros, a launch leaves its ticket counter at zero, and carry words are tagged with
 *           their launch's epoch, so the call records nothing but its kernel into a graph. */
#define HAWK_STATIC_SCRATCH_BYTES (16u << 20)
size_t hawk_rglru_scan_fwd_static_bytes(int B, int T, int D, int dtype);
int hawk_rglru_scan_fwd_static(const void* x, const void* x_rg_lru, const void* a_rg_lru,
                               const float* a_param, void* h, int B, int T, int D, int dtype,
                               void* stream);

/* RG-LRU scan backward (reverse time).  Inputs are the forward's inputs, the saved h and
 * the upstream gradient; outputs are dx, dx_rg_lru, da_rg_lru in `dtype` and
 * da_param [D] fp32, already reduced over batch and time.
 * Replaces sequential_scan_backward / sequential_scan_bwd_kernel and the trailing
 * .sum(dim=0) (hawk/scan_fused.py:363-424, :112-317).  T = 1 is handled (the upstream
 * kernel needs T >= 2).  The workspace is always required. */
int hawk_rglru_scan_bwd(const void* x, const void* x_rg_lru, const void* a_rg_lru,
                        const float* a_param, const void* h_saved, const void* grad_out,
                        void* dx, void* dx_rg_lru, void* da_rg_lru, float* da_param, int B,
                        int T, int D, int dtype, void* workspace_device,
                        size_t workspace_bytes, void* stream);

/* Mixed-precision variants of the two scan entry points: x, x_rg_lru, a_rg_lru (and, in
 * the backward, their three gradients) have in_dtype; h (and, in the backward, h_saved and
 * grad_out) have out_dtype / state_dtype.  Supported pairs: (bf16, bf16), (f32, f32) and
 * (f32, bf16).  The last one is what the model produces under autocast (fp32 conv output
 * and gate logits, bf16 h): upstream first casts all inputs to bf16 with three extra
 * kernels (custom_fwd(cast_inputs=bfloat16), hawk/scan_fused.py:428) and autograd casts the
 * three gradients back to fp32 with three more; here the rounding happens in registers.
 * The plain entry points above are these with both dtypes equal. */
int hawk_rglru_scan_fwd_mixed(const void* x, const void* x_rg_lru, const void* a_rg_lru,
                              const float* a_param, void* h, int B, int T, int D, int in_dtype,
                              int out_dtype, void* workspace_device, size_t workspace_bytes,
                              void* stream);
int hawk_rglru_scan_bwd_mixed(const void* x, const void* x_rg_lru, const void* a_rg_lru,
                              const float* a_param, const void* h_saved, const void* grad_out,
                              void* dx, void* dx_rg_lru, void* da_rg_lru, float* da_param,
                              int B, int T, int D, int in_dtype, int state_dtype,
                              void* workspace_device, size_t workspace_bytes, void* stream);

/* Scan fused with the step that follows it in a Hawk block, out = gelu(y) * h with the
 * exact (erf) GELU (Hawk.epilogue before its projection, hawk/hawk.py:134-135, applied to
 * the scan's result at hawk/hawk.py:186).  Dtypes as in the mixed variants; y, out, h_last
 * and dy have the out / state dtype.
 *   y        [B,T,D] gate input; rows are ldy >= D elements apart and batches T rows apart,
 *            so the second half of the fused projection of hawk/hawk.py:164-166 can be
 *            passed in place (ldy = 2 D).  y and dy need only be aligned to their element
 *            size; 4-byte alignment and even row strides let bf16 move as pairs.
 *   h        [B,T,D] dense, or NULL when the state sequence is not needed (no backward)
 *   out      [B,T,D] dense
 *   h_last   [B,D] or NULL: h at t = T-1, what RNNCache.update_cache keeps (hawk.py:190)
 * Forward: reads 4 tensors, writes 1 or 2, where the unfused sequence reads 5 and writes 2. */
int hawk_rglru_scan_gated_fwd(const void* x, const void* x_rg_lru, const void* a_rg_lru,
                              const float* a_param, const void* y, long long ldy, void* h,
                              void* out, void* h_last, int B, int T, int D, int in_dtype,
                              int out_dtype, void* workspace_device, size_t workspace_bytes,
                              void* stream);

/* Backward of the above.  grad_out is the gradient of `out`; dy [B,T,D] (rows lddy >= D
 * elements apart) receives grad_out * h * gelu'(y); the other outputs are as in
 * hawk_rglru_scan_bwd.  Replaces the autograd of gelu and of the product together with
 * sequential_scan_backward (hawk/scan_fused.py:363-424): reads 6 tensors and writes 4
 * where the unfused sequence reads 8 and writes 5. */
int hawk_rglru_scan_gated_bwd(const void* x, const void* x_rg_lru, const void* a_rg_lru,
                              const float* a_param, const void* y, long long ldy,
                              const void* h_saved, const void* grad_out, void* dx,
                              void* dx_rg_lru, void* da_rg_lru, void* dy, long long lddy,
                              float* da_param, int B, int T, int D, int in_dtype,
                              int state_dtype, void* workspace_device, size_t workspace_bytes,
                              void* stream);

/* ---------------------------------------------------------------------------------------
 * Temporal causal depthwise conv1d.
 *   y[b,t,c] = bias[c] + sum_{s<W} w[W-1-s,c] x[b,t-s,c]
 * Rows before t = 0 are zero, or are taken from `state` [B,W-1,D] (oldest row first,
 * dtype of x) when it is not NULL.  Replaces Conv1D.forward (hawk/external.py:49-98).
 * x and y may have different dtypes (upstream returns fp32 for bf16 x by promotion).
 * 1 <= W <= 8.
 * ------------------------------------------------------------------------------------- */
int hawk_conv1d_fwd(const void* x, const float* w, const float* bias, const void* state,
                    void* y, int B, int T, int D, int W, int x_dtype, int y_dtype,
                    void* stream);

/* The same with rows of x and y further apart than D elements (x_row_stride, y_row_stride >= D,
 * in elements; batch rows lie T rows apart): the x half of the block's [B,T,2D] input
 * projection (hawk/hawk.py:163-164, a chunk of one tensor) is read in place instead of
 * being copied out first.  `state` stays dense.  Same upstream lines as hawk_conv1d_fwd. */
int hawk_conv1d_fwd_strided(const void* x, long long x_row_stride, const float* w, const float* bias,
                            const void* state, void* y, long long y_row_stride, int B, int T, int D,
                            int W, int x_dtype, int y_dtype, void* stream);

/* Size of the scratch buffer hawk_conv1d_bwd needs for its dw/db partial sums. */
size_t hawk_conv1d_bwd_workspace_bytes(int B, int T, int D, int W);

/* Conv1d backward with zero history: dx (x_dtype), dw [W,D] fp32, db [D] fp32.
 * Upstream has no hand-written backward; this is the adjoint autograd builds from
 * hawk/external.py:78-93.  grad_y has dtype gy_dtype. */
int hawk_conv1d_bwd(const void* grad_y, const void* x, const float* w, void* dx, float* dw,
                    float* db, int B, int T, int D, int W, int x_dtype, int gy_dtype,
                    void* workspace_device, size_t workspace_bytes, void* stream);

/* The same with rows of x and dx further apart than D elements: x is read from, and dx written
 * into, the x half of a [B,T,2D] tensor in place (the gradient of the input projection's
 * output is then one tensor that this call and hawk_rglru_scan_gated_bwd fill side by side,
 * where autograd would concatenate two).  grad_y is dense. */
int hawk_conv1d_bwd_strided(const void* grad_y, const void* x, long long x_row_stride, const float* w,
                            void* dx, long long dx_row_stride, float* dw, float* db, int B, int T, int D,
                            int W, int x_dtype, int gy_dtype, void* workspace_device,
                            size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------
 * Decode steps (one new token per batch row).
 * ------------------------------------------------------------------------------------- */

/* conv_state [B,W-1,D] is consumed and updated in place (rolled up one row, x_new written
 * last); y [B,D] is the conv output for the new token.  Replaces the
 * concat / RNNCache.update_conv_cache / Conv1D / last-row slice sequence
 * (hawk/hawk.py:169-179, hawk/cache.py:37-43).  state, x_new share `dtype`; y has y_dtype. */
int hawk_conv1d_step(void* conv_state, const void* x_new, const float* w, const float* bias,
                     void* y, int B, int D, int W, int dtype, int y_dtype, void* stream);

/* h = alpha * recc_state + sqrt(1-alpha^2) (i x); recc_state [B,D] (state_dtype) is read,
 * then overwritten with h; h_out [B,D] (`dtype`) also receives h.  Replaces
 * Hawk.inference_prologue + step + RNNCache.update_cache (hawk/hawk.py:137-151, :196-198,
 * hawk/cache.py:29-35).  x, x_rg_lru, a_rg_lru are [B,D] of `dtype`. */
int hawk_rglru_step(const void* x, const void* x_rg_lru, const void* a_rg_lru,
                    const float* a_param, void* recc_state, void* h_out, int B, int D,
                    int dtype, int state_dtype, void* stream);

/* The same step with the work around it folded in (one launch instead of five):
 *   bias_i, bias_a  [D] fp32 or NULL: added to x_rg_lru / a_rg_lru first, so the two
 *                   block-diagonal projections (hawk/external.py:224-233, called at
 *                   hawk/hawk.py:181-182) can leave their bias out
 *   y, out          out [B,D] <- gelu(y) * h, the gate of Hawk.epilogue (hawk/hawk.py:134-135);
 *                   y is [B,D] with rows ldy >= D elements apart (the gate half of the
 *                   input projection, passed in place), aligned to its element size
 *   h_out           may be NULL here (the state itself lands in recc_state) */
int hawk_rglru_step_gated(const void* x, const void* x_rg_lru, const void* a_rg_lru,
                          const float* bias_i, const float* bias_a, const float* a_param,
                          const void* y, long long ldy, void* recc_state, void* h_out, void* out,
                          int B, int D, int dtype, int state_dtype, void* stream);

/* ---------------------------------------------------------------------------------------
 * Block-diagonal gate projections (matrix cores, bf16 operands, fp32 accumulation).
 * ------------------------------------------------------------------------------------- */

/* 1 if the (D, num_blocks) pair is served: D divisible by num_blocks and a block width of
 * 32, 64, 128 or 256.  Other shapes stay with the caller's library GEMM. */
int hawk_gate_proj_supported(int D, int num_blocks);

/* 1 if hawk_decode_core_step serves the shape: a (D, num_blocks) pair the gate projections
 * serve and a conv window of 1 <= W <= 8 rows. */
int hawk_decode_core_supported(int D, int num_blocks, int W);

/* One decode step of a layer's whole recurrent core, one launch instead of
 * hawk_conv1d_step + hawk_gate_proj_fwd + hawk_rglru_step_gated (upstream: the window concat,
 * RNNCache.update_conv_cache, Conv1D, the two BlockDiagonalLinear calls evaluated twice,
 * Hawk.inference_prologue, the step, RNNCache.update_cache and Hawk.epilogue's gate:
 * hawk/hawk.py:134-151, :169-182, :196-198, hawk/cache.py:29-43):
 *   conv_state [B, W-1, D]  rolled up one row in place, x_new written last
 *   x_new      [B, D], rows ldx >= D elements apart, ldx a multiple of 8 (the x half of the
 *              input projection, passed in place); 16-byte aligned
 *   conv_w [W, D], conv_b [D] fp32; w_i, w_a [num_blocks, bw, bw] of w_dtype (16-byte
 *              aligned); b_i, b_a [D] fp32 or NULL; a_param [D] fp32
 *   y          [B, D], rows ldy >= D elements apart (the gate half of the input projection)
 *   recc_state [B, D] of state_dtype: read, then overwritten with the new state h
 *   out        [B, D] <- gelu(y) * h
 * conv_state, x_new, y and out are bf16 (`dtype` must be HAWK_DTYPE_BF16).  The conv output
 * and the two logits are rounded to bf16 where the three separate calls round them, so both
 * routes give the same result.  y, recc_state and out are accessed 16 bytes at a time when
 * they are 16-byte aligned (32 for an fp32 recc_state) and ldy is a multiple of 8. */
int hawk_decode_core_step(void* conv_state, const void* x_new, long long ldx, const float* conv_w,
                          const float* conv_b, const void* w_i, const float* b_i, const void* w_a,
                          const float* b_a, const float* a_param, const void* y, long long ldy,
                          void* recc_state, void* out, int B, int D, int num_blocks, int W,
                          int dtype, int w_dtype, int state_dtype, void* stream);

/* The same step with a workspace: hawk_decode_core_workspace_bytes(B, D, num_blocks) bytes of
 * device memory (4-byte aligned) that hold zeros before the first call (hipMemsetAsync, or
 * hawk_scan_workspace_init) and are left holding zeros by every call, so one buffer serves all
 * layers and steps issued in order on one stream; concurrent streams need one each.  With it the
 * output columns of a block are produced by up to four workgroups instead of one (a block's
 * 2 x bw x bw weights then pass through four L1 caches, not one, and a batch of 256 rows with
 * 10 blocks occupies 320 workgroups instead of 80); the workgroup that is last to have read a
 * conv window rolls it.  Results are bit-identical to hawk_decode_core_step.  A NULL workspace
 * makes the call hawk_decode_core_step.  Same upstream lines as above. */
size_t hawk_decode_core_workspace_bytes(int B, int D, int num_blocks);
int hawk_decode_core_step_ws(void* conv_state, const void* x_new, long long ldx, const float* conv_w,
                             const float* conv_b, const void* w_i, const float* b_i, const void* w_a,
                             const float* b_a, const float* a_param, const void* y, long long ldy,
                             void* recc_state, void* out, int B, int D, int num_blocks, int W,
                             int dtype, int w_dtype, int state_dtype, void* workspace_device,
                             size_t workspace_bytes, void* stream);

/* Both gate logits of M = B*T tokens in one pass over x:
 *   x_rg_lru[m, h*bw+j] = b_i[h*bw+j] + sum_i x[m, h*bw+i] w_i[h, i, j]     (same for a_rg_lru)
 * Replaces the two BlockDiagonalLinear calls of hawk/hawk.py:181-182 (einsum + bias,
 * hawk/external.py:224-233).  x [M,D] has x_dtype; w_i, w_a [num_blocks, bw, bw] have
 * w_dtype; b_i, b_a [D] are fp32 or NULL; the outputs [M,D] have out_dtype.  x and the
 * weights are rounded to bf16 in registers (what bf16 autocast does to this einsum); the
 * sums and the bias add are fp32.  x, the weights and the outputs must be 16-byte aligned
 * (HAWK_ERR_ALIGNMENT otherwise).  Row counts up to 512 (decode) run a variant that is cut
 * by output columns instead of rows; results are the same sums in the same order. */
int hawk_gate_proj_fwd(const void* x, const void* w_i, const float* b_i, const void* w_a,
                       const float* b_a, void* x_rg_lru, void* a_rg_lru, int M, int D,
                       int num_blocks, int x_dtype, int w_dtype, int out_dtype, void* stream);

/* The temporal conv and both gate projections of its output in one pass over the conv's input:
 *   u[b, t, c]  = conv_b[c] + sum_k conv_w[k, c] x[b, t - (3 - k), c]   (rows before t = 0 are zero)
 *   x_rg_lru, a_rg_lru = hawk_gate_proj_fwd(u)
 * Replaces Conv1D.forward followed by the two BlockDiagonalLinear calls (hawk/hawk.py:172-182,
 * hawk/external.py:49-95, :224-233) for a sequence without conv history: the same arithmetic in
 * the same order as hawk_conv1d_fwd (bf16 output) followed by hawk_gate_proj_fwd, bit for bit,
 * without reading u back.  x [B,T,D] bf16, rows x_row_stride >= D elements apart (a multiple
 * of 8: the x half of the block's input projection is read in place); u, x_rg_lru, a_rg_lru
 * [B,T,D] bf16, dense; conv_w [4,D], conv_b [D] fp32; gate weights and biases as in
 * hawk_gate_proj_fwd.  temporal_width must be 4 and T >= 32 (HAWK_ERR_BAD_SHAPE otherwise; use
 * the two separate calls then). */
int hawk_conv_gate_proj_fwd(const void* x, long long x_row_stride, const float* conv_w,
                            const float* conv_b, const void* w_i, const float* b_i, const void* w_a,
                            const float* b_a, void* u, void* x_rg_lru, void* a_rg_lru, int B, int T,
                            int D, int num_blocks, int temporal_width, int w_dtype, void* stream);

/* Gradient of the two projections with respect to x, in one pass over both logit gradients:
 *   dx[m, h*bw+i] = sum_j d_x_rg_lru[m, h*bw+j] w_i[h, i, j] + sum_j d_a_rg_lru[m, h*bw+j] w_a[h, i, j]
 *                   (+ addend[m, h*bw+i])
 * (what autograd derives from the einsum of hawk/external.py:230, twice, plus the add of
 * the two results).  addend [M,D] (dx_dtype) may be NULL; it is the gradient x receives from
 * its other consumer, the scan (hawk/hawk.py:186), whose accumulation autograd would
 * otherwise do in a separate pass; it may alias dx.  Gradients have g_dtype, weights
 * w_dtype, dx has dx_dtype; operands are rounded to bf16 in registers, sums are fp32. */
int hawk_gate_proj_bwd_input(const void* d_x_rg_lru, const void* d_a_rg_lru, const void* w_i,
                             const void* w_a, const void* addend, void* dx, int M, int D,
                             int num_blocks, int g_dtype, int w_dtype, int dx_dtype, void* stream);

/* Gradients of the weights and biases of the two projections:
 *   dw_g[h, i, j] = sum_m x[m, h*bw+i] d_g[m, h*bw+j],   db_g[c] = sum_m d_g[m, c]
 * (autograd of hawk/external.py:230 with respect to w and b).  dw_i, dw_a
 * [num_blocks, bw, bw] and db_i, db_a [D] (may be NULL) are fp32 and are overwritten.  The
 * row range is split over workgroups; their partial sums live in the caller's workspace
 * (size from the query) and are added in a fixed order, so results are reproducible. */
size_t hawk_gate_proj_bwd_weights_workspace_bytes(int M, int D, int num_blocks);
int hawk_gate_proj_bwd_weights(const void* x, const void* d_x_rg_lru, const void* d_a_rg_lru,
                               float* dw_i, float* db_i, float* dw_a, float* db_a, int M, int D,
                               int num_blocks, int x_dtype, int g_dtype, void* workspace_device,
                               size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------
 * The recurrent core of a block as one call per direction.
 * Hawk.forward between the input projection and the output projection (hawk/hawk.py:169-198:
 * Conv1D, the two BlockDiagonalLinear gates, rnn_scan / the fused scan, gelu(y) * h) on the
 * projection's output xy [B,T,2D] bf16 in place (x half, then y half; rows xy_row_stride >= 2D
 * elements apart, a multiple of 8; D a multiple of 8).  The kernels and the results are those of
 * hawk_conv_gate_proj_fwd + hawk_rglru_scan_gated_fwd and of hawk_rglru_scan_gated_bwd +
 * hawk_gate_proj_bwd_input (onto the scan's dx, in place) + hawk_conv1d_bwd_strided +
 * hawk_gate_proj_bwd_weights, bit for bit; what the single calls cannot do is share their small
 * launches: here fp32 gate weights are rounded to bf16 by one launch for both gates, and the three
 * closing reductions of the backward run as one launch.
 * ------------------------------------------------------------------------------------- */

/* fp32 -> bf16 (round to nearest even) of both gates' weights [num_blocks, bw, bw] in one launch;
 * bw a multiple of 4.  What `w.to(torch.bfloat16)` gives, twice. */
int hawk_gate_weights_to_bf16(const float* w_i, const float* w_a, void* w_i_bf16, void* w_a_bf16,
                              int num_blocks, int block_width, void* stream);

/* Forward.  Gate weights have w_dtype; when they are fp32 and w_bf16 is not NULL, they are first
 * rounded into w_bf16 ([2][num_blocks][bw][bw] bf16: w_i, then w_a), which the kernels then read
 * and which hawk_block_core_bwd can be handed as its weights (w_dtype bf16).  u, x_rg_lru,
 * a_rg_lru, out [B,T,D] bf16 dense; h [B,T,D] bf16 and h_last [B,D] bf16 may be NULL (h is what
 * the backward needs).  temporal_width must be 4 and T >= 32 (HAWK_ERR_BAD_SHAPE otherwise: use
 * the single calls).  scan_workspace as for hawk_rglru_scan_fwd. */
int hawk_block_core_fwd(const void* xy, long long xy_row_stride, const float* conv_w,
                        const float* conv_b, const void* w_i, const float* b_i, const void* w_a,
                        const float* b_a, int w_dtype, void* w_bf16, const float* a_param, void* u,
                        void* x_rg_lru, void* a_rg_lru, void* h, void* out, void* h_last, int B, int T,
                        int D, int num_blocks, int temporal_width, void* scan_workspace,
                        size_t scan_workspace_bytes, void* stream);

/* Backward.  grad_out [B,T,D] bf16 dense; d_xy [B,T,2D] bf16 (rows d_xy_row_stride elements
 * apart) receives both halves; du, d_x_rg_lru, d_a_rg_lru [B,T,D] bf16 are the caller's scratch
 * for the gradients in between (du ends as the gradient of the conv output).  d_conv_w
 * [temporal_width, D], d_conv_b [D], dw_i, dw_a [num_blocks, bw, bw], db_i, db_a [D] (may be
 * NULL), da_param [D]: fp32, overwritten.  The three workspaces are those of the single calls
 * (hawk_scan_workspace_bytes, hawk_gate_proj_bwd_weights_workspace_bytes,
 * hawk_conv1d_bwd_workspace_bytes). */
int hawk_block_core_bwd(const void* xy, long long xy_row_stride, const void* u, const void* x_rg_lru,
                        const void* a_rg_lru, const void* h_saved, const float* conv_w,
                        const void* w_i, const void* w_a, int w_dtype, const float* a_param,
                        const void* grad_out, void* d_xy, long long d_xy_row_stride, void* du,
                        void* d_x_rg_lru, void* d_a_rg_lru, float* d_conv_w, float* d_conv_b,
                        float* dw_i, float* db_i, float* dw_a, float* db_a, float* da_param, int B, int T,
                        int D, int num_blocks, int temporal_width, void* scan_workspace,
                        size_t scan_workspace_bytes, void* gate_workspace,
                        size_t gate_workspace_bytes, void* conv_workspace,
                        size_t conv_workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------
 * A measurement aid with no counterpart in the reference: copy kernels that move n_reads
 * tensors in and n_writes tensors out (`bytes` each, 16-byte aligned, all distinct) with the scan
 * kernels' memory instructions and no arithmetic to speak of, so that a benchmark can state on its
 * own tensors what the part delivers for a mix of reads and writes.  shape 0: flat, a workgroup
 * takes 16 KiB of every tensor (bytes a multiple of 16384).  shape S >= 1: the scan's workgroup
 * shape, eight waves stacked in time on 16 rows x 256 bytes each, over [rows, row_pitch_bytes]
 * tensors (row_pitch_bytes a multiple of 256, rows a multiple of 128 * S), with the tiles taken in
 * the order a scan launch over sequences of S row groups (128 * S rows) takes them: position along
 * the sequence slowest, then sequence, then column tile; S = 1 is plain memory order, S = T / 128
 * the order of a [B, T, D] scan.  Every 32-bit word of output i receives the sum of the inputs'
 * words at its place plus i.  Supported mixes (reads + writes): 1+1, 1+2, 1+3, 2+1, 3+1, 5+3;
 * HAWK_ERR_BAD_SHAPE otherwise.
 * ------------------------------------------------------------------------------------- */
int hawk_stream_probe(const void* const* reads, int n_reads, void* const* writes, int n_writes,
                      size_t bytes, size_t row_pitch_bytes, int shape, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* HAWK_HIP_H_ */
