/*
 * m2dscan -- C ABI of the MI355X (gfx950) wavefront 2-D selective scan.
 *
 * A torch-free HIP shared library (libm2dscan.so) exports exactly these symbols.  They
 * are what a binding for the reference's native module would call in place of its two
 * pybind entry points
 *     wf_fwd(hs, x, deltaT, deltaL, BT, BL, AT, AL)                     wf_cuda_bind.cpp:24-33
 *     wf_bwd(hs, x, deltaT, deltaL, AT, AL, grad_output, dDAT, dDAL, omega)   wf_cuda_bind.cpp:35-46
 * together with the tensor algebra the reference performs around them in Python
 * (output projection wavefront_cuda.py:156, its backward :176-178, parameter gradients
 * :97-139, d_x assembly :193-194): one fused forward producing y and one fused backward
 * producing the nine gradients, neither of which materialises the (B,H,W,E,N) state.
 *
 * Conventions
 *   - All tensor arguments are DEVICE pointers to contiguous, channel-last arrays in
 *     the reference's layout:  x, deltaT, deltaL, y, dy, dx, d_deltaT, d_deltaL : (B,H,W,E)
 *                              BT, BL, C, d_BT, d_BL, d_C : (B,H,W,N)
 *                              AT, AL, d_AT, d_AL : (E,N)        D, d_D : (E)
 *     every one of them in the element type named by m2d_desc.dtype (the reference
 *     requires one common dtype too, wf_cuda.cu:182).  State and accumulation are fp32.
 *   - The caller owns every buffer, including workspace and checkpoints; the library
 *     allocates nothing and keeps no mutable global state, so calls are re-entrant.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  Calls only
 *     enqueue work; they do not synchronise.
 *   - Every function returns an m2d_status; nothing is launched unless it is M2D_OK.
 */
#ifndef M2DSCAN_H
#define M2DSCAN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum m2d_status {
  M2D_OK = 0,
  M2D_ERR_NULL_POINTER = 1,   /* a required pointer argument is NULL */
  M2D_ERR_BAD_SHAPE = 2,      /* a dimension is < 1, or H < 2 or W < 2 (reference: wavefront_cuda.py:323-324) */
  M2D_ERR_UNSUPPORTED = 3,    /* dtype / N outside what the kernels are built for, or one image too large
                                 for 32-bit offsets (H*W >= 2^24 cells or H*W*E >= 2^30 elements) */
  M2D_ERR_WORKSPACE = 4,      /* workspace or checkpoint buffer smaller than required */
  M2D_ERR_MISALIGNED = 5,     /* a tensor pointer is not 16-byte aligned / workspace not 256-byte aligned */
  M2D_ERR_HIP = 6,            /* a HIP runtime call or kernel launch failed */
  M2D_ERR_TOO_LARGE = 7       /* m2d_scan_fwd_noalloc: the problem needs more scratch than the library's static buffer */
} m2d_status;

typedef enum m2d_dtype {
  M2D_F32 = 0,                /* fp32 in, fp32 out */
  M2D_BF16 = 1                /* bf16 in, bf16 out, fp32 state and accumulation */
} m2d_dtype;

/* Problem descriptor.  N must be 16 in this build (the reference's d_state default,
 * models/mamba2d.py:23).  flags: bit 0 = M2D_FLAG_FLIP, scan from the bottom-right
 * corner (equivalent to torch.flip(x,(1,2)) of every spatial tensor before and of the
 * outputs after, models/mamba2d.py:163-173); the other flags are described below. */
typedef struct m2d_desc {
  int32_t B, H, W, E, N;
  int32_t dtype;              /* m2d_dtype */
  int32_t flags;
  int32_t ckpt_interval;      /* steps between the state snapshots that m2d_scan_fwd keeps for m2d_scan_bwd:
                                 0 (the library chooses), 2, 4, 8 or 16.
                                 2: two snapshots per block of 4 steps; the backward then recomputes one step in two
                                    and computes every gate once (its kernel is bound by instruction issue, not by
                                    memory: it trades bytes for instructions).  Only where every image (or stack of
                                    small images) is swept as one stream with all 16 states of a channel in one lane;
                                    the other schedules (few large images) keep 4, also when 2 is asked for.
                                 4: one snapshot per block; the backward recomputes the block.
                                 8, 16: a half / a quarter of the snapshots of 4; the backward replays the forward
                                    over the blocks in between (4 or 12 steps of every 8 or 16) before it sweeps them.
                                 0 picks 2 where it exists, else 4.  The forward and the backward of one problem
                                 must use the same value.  Ignored by the m2d_proj_* entry points. */
} m2d_desc;

#define M2D_FLAG_FLIP 1
/* m2d_proj_fwd / m2d_proj_bwd only: round weights and biases to desc->dtype before use, which is
 * what the reference's cast of its weights to x.dtype does (wavefront_cuda.py:327-332).  Without
 * the flag bf16 activations still meet bf16-rounded weight matrices (not biases) wherever the
 * products run on the matrix cores (channel counts that are a multiple of 8). */
#define M2D_FLAG_ROUND_WEIGHTS 2
/* m2d_scan_fwd / m2d_scan_bwd only: AT, AL and D are the parameters as the reference's module holds
 * them, fp32: AT and AL point to A_log (E,N) with A = -exp(A_log) (models/mamba2d.py:95-101,
 * wavefront_cuda.py:72-73), D to (E); the library rounds A and D to desc->dtype as the reference's
 * casts do (wavefront_cuda.py:90-91, 332).  d_AT, d_AL, d_D are then fp32 gradients with respect to
 * A_log and D. */
#define M2D_FLAG_RAW_PARAMS 4
/* B_T, B_L and C travel from m2d_proj_fwd to m2d_scan_fwd / m2d_scan_bwd in the form the scan
 * kernels read, saving the scan its repacking pass: with this flag m2d_proj_fwd writes, to its BT
 * argument, one fp32 record of 48 values per position (B,H,W,48) -- the values rounded to
 * desc->dtype, in the library's own order -- and leaves BL and C alone (they may be NULL); the
 * scan calls read those records through their BT argument and ignore BL and C.  The records are
 * only meaningful to this library. */
#define M2D_FLAG_PACKED_BC 8
/* The gradients of the two step sizes travel from m2d_scan_bwd to m2d_proj_bwd as gradients with
 * respect to what the softplus was applied to (wavefront_cuda.py:85-86): with this flag m2d_scan_bwd
 * writes d_delta * (1 - exp(-delta)) to d_deltaT and d_deltaL, and m2d_proj_bwd takes its d_deltaT and
 * d_deltaL arguments as such and does not read deltaT and deltaL (they may be NULL).  This saves
 * m2d_proj_bwd reading the two step-size tensors and a pass of its own intermediate through memory. */
#define M2D_FLAG_DPRE 16
/* Scheduling hints for m2d_scan_fwd / m2d_scan_bwd (results agree to rounding either way; sizes
 * queried and calls made for one problem must carry the same hints).  The library normally decides by
 * itself: with few images it spreads the 16 states of a channel over the lanes of a wave (a wave per
 * channel instead of per 4 channels), which shortens a sweep when the device is far from full.
 * M2D_FLAG_SPLIT_STATES asks for that layout wherever it exists, M2D_FLAG_WHOLE_STATES forbids it. */
#define M2D_FLAG_SPLIT_STATES 32
#define M2D_FLAG_WHOLE_STATES 64
/* Test aid for the linked sweep (grids of many bands and few images, whose bands run on workgroups of their own
 * inside one launch and wait for each other's boundary rows; see m2d_scan_link_error).  With this flag the
 * workgroups of one band (forward: the second; backward: the last but one) wait for a neighbour that never
 * reports, and every wait of the launch gives up after a few polls instead of about a million: the launch runs
 * the path of a wait that gives up, and still ends normally.  What that path does: the workgroup sets the error
 * word, tells its dependants not to wait, and overwrites its band's rows of y (forward) or of dx, d_deltaT,
 * d_deltaL and its channels' shares of d_AT, d_AL, d_D (backward) with NaN, as does every band that depended
 * on it; so a linked sweep that failed shows in the caller's tensors.  Ignored by other schedules. */
#define M2D_FLAG_TEST_DEAD_LINK 128

/* The sums over channels d_BT, d_BL, d_C travel from m2d_scan_bwd to m2d_proj_bwd_parts unfinished.  The scan's
 * backward kernel adds them up over the channels of a workgroup and normally a small second kernel adds the
 * workgroups of an image and rounds; where the only reader is the projections' backward, that reader can do the
 * last step while it loads them.  With this flag m2d_scan_bwd writes, to its d_BT argument, the fp32 records
 * [parts][B*H*W][d_C | d_BT | d_BL][16] with parts = m2d_scan_sum_parts(desc) (the caller sizes the buffer with
 * it), and leaves d_BL and d_C alone (they may be NULL).  The records are only meaningful to this library. */
#define M2D_FLAG_SUM_PARTS 256

/* bf16 tensors keep their state snapshots rounded to bf16 (the reference keeps every state of its hidden-state tensor
 * in the tensors' type); with this flag m2d_scan_fwd keeps them in fp32 and m2d_scan_bwd reads them so: twice the
 * checkpoint bytes of an interval of 4 steps, which the flag implies (ckpt_interval 0 or 4; others are refused), and
 * the whole-state kernels in workgroups of 4 sweeping waves, which is slower wherever another plan would have been
 * chosen.  Both passes of a problem must agree on it.  No effect on fp32 tensors. */
#define M2D_FLAG_FP32_SNAPSHOTS 512

#define M2D_PASS_FWD 0
#define M2D_PASS_BWD 1

/* Library version (major*10000 + minor*100 + patch). */
int m2d_version(void);

/* Human-readable text for a status code (static storage). */
const char* m2d_status_str(int status);

/* Validates a descriptor without touching the GPU. */
int m2d_desc_check(const m2d_desc* desc);

/* Bytes of scratch the forward (M2D_PASS_FWD) or backward (M2D_PASS_BWD) pass needs.
 * `have_ckpt` != 0 means the caller passes a checkpoint buffer to that pass (forward:
 * to be filled; backward: filled by the forward), which reduces the scratch.
 * Returns 0 for an invalid descriptor. */
size_t m2d_scan_workspace_bytes(const m2d_desc* desc, int pass, int have_ckpt);

/* Bytes of the checkpoint buffer (anti-diagonal state snapshots every desc->ckpt_interval steps
 * plus band-boundary rows; linear in H*W, at 4 steps about 1/4 of the reference's hs tensor, at 2 steps 1/2:
 * the snapshots have the width of the tensors' type, fp32 or bf16, as every state of hs has in the
 * reference, wf_cuda.cu:5,59-67). */
size_t m2d_scan_ckpt_bytes(const m2d_desc* desc);

/* Fused forward:  y = sum_n h*C + x*D  with h from the recurrence of wf_cuda.cu:40-69.
 * Replaces wf_fwd (wf_cuda_bind.cpp:24) + wavefront_cuda.py:152-156.
 * ckpt may be NULL (inference); if given it is filled for a later m2d_scan_bwd. */
int m2d_scan_fwd(const m2d_desc* desc,
                 const void* x, const void* deltaT, const void* deltaL,
                 const void* AT, const void* AL,
                 const void* BT, const void* BL, const void* C, const void* D,
                 void* y,
                 void* ckpt, size_t ckpt_bytes,
                 void* workspace, size_t workspace_bytes,
                 void* stream);

/* Debugging aid for grids of many bands and few images, whose bands run on workgroups of their own
 * inside one launch and wait for each other's boundary rows (a bounded wait: a workgroup that has
 * polled about two million times -- seconds of wall time, which only another tenant of the device
 * holding the compute units can cause -- gives up, so that the launch always ends; the results are then
 * invalid, and the workgroup and every band after it overwrite their rows of the outputs with NaN).
 * Synchronises `stream` and reads, from the workspace of the last m2d_scan_fwd or
 * m2d_scan_bwd call of this descriptor on it, whether any workgroup gave up: *gave_up = 0 or 1 (always
 * 0 for problems that do not run that way).  No counterpart in the reference (its diagonals are
 * ordered by kernel launches, wf_cuda.cu:203,259). */
int m2d_scan_link_error(const m2d_desc* desc, const void* workspace, void* stream, int* gave_up);

/* What the library will do with a problem: one line of text per pass (M2D_PASS_FWD / M2D_PASS_BWD), e.g.
 * "m2d_bwd_split_kernel: linked sweep, 19 bands, 152 workgroups of 8 waves, 8 channels each, 4 states per lane".
 * Writes at most `cap` bytes including the terminating 0; host only, touches no device.  Returns M2D_OK or the
 * status m2d_desc_check gives.  No counterpart in the reference (which has one schedule). */
int m2d_scan_plan(const m2d_desc* desc, int pass, char* text, size_t cap);

/* m2d_scan_fwd without a checkpoint buffer and without a workspace argument, for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * it).  It has no counterpart in the reference, whose Python side allocates every buffer with
 * torch.empty.  The scratch that m2d_scan_fwd takes as `workspace` lives in a static device array
 * of M2D_NOALLOC_SCRATCH_BYTES inside the library (each GPU the library runs on holds one copy until
 * the process ends); the call allocates and frees nothing.  A problem whose
 * m2d_scan_workspace_bytes(desc, M2D_PASS_FWD, 0) exceeds that size is rejected with
 * M2D_ERR_TOO_LARGE before anything is launched (this check comes first: a call with NULL tensors on
 * a problem that is too large reports M2D_ERR_TOO_LARGE).  All calls on one GPU share the array: two calls
 * that overlap on one GPU (different streams or threads) race; calls on one stream are ordered.  Besides
 * boundary rows, the array holds the progress counts of a linked sweep: an overlapping call that clears
 * them in mid-flight can make the other launch's waits give up (its rows of y then say NaN, see
 * m2d_scan_link_error). */
#define M2D_NOALLOC_SCRATCH_BYTES (32u << 20)
int m2d_scan_fwd_noalloc(const m2d_desc* desc,
                         const void* x, const void* deltaT, const void* deltaL,
                         const void* AT, const void* AL,
                         const void* BT, const void* BL, const void* C, const void* D,
                         void* y,
                         void* stream);

/* Fused backward: the nine gradients of the forward above for upstream gradient dy.
 * Replaces wavefront_cuda.py:169-196 (state recompute, wf_bwd of wf_cuda_bind.cpp:35,
 * fused_backward_math, output-projection backward).  ckpt may be NULL, in which case
 * the checkpoints are rebuilt inside the call (one extra forward sweep).  A ckpt buffer
 * belongs to the inputs and the descriptor of the forward that filled it: besides the state
 * snapshots it holds what that forward derived from AT, AL and D, which this call reuses.
 * d_AT, d_AL, d_D are written (not accumulated). */
int m2d_scan_bwd(const m2d_desc* desc,
                 const void* x, const void* deltaT, const void* deltaL,
                 const void* AT, const void* AL,
                 const void* BT, const void* BL, const void* C, const void* D,
                 const void* dy,
                 const void* ckpt, size_t ckpt_bytes,
                 void* dx, void* d_deltaT, void* d_deltaL,
                 void* d_AT, void* d_AL,
                 void* d_BT, void* d_BL, void* d_C, void* d_D,
                 void* workspace, size_t workspace_bytes,
                 void* stream);

/* ---- Projections either side of the scan -------------------------------------------------
 * The reference computes the scan's parameters from x with stock operators (proj_params,
 * models/kernels/wavefront_cuda.py:63-95) and differentiates them with autograd
 * (wavefront_cuda.py:262-296).  The two calls below do the same work in hand-written kernels.
 * desc->H and desc->W only enter through the number of positions P = B*H*W; of the flags
 * M2D_FLAG_ROUND_WEIGHTS, M2D_FLAG_PACKED_BC (forward) and M2D_FLAG_DPRE (backward) are read.  Activations have the element type of desc->dtype; weights,
 * biases and their gradients are fp32.  dt_rank <= 32, E <= 4096.
 *
 *   x_proj_w  (2*dt_rank + 3*N, E)     dt_proj{T,L}_w (E, dt_rank)     dt_proj{T,L}_b (E)
 *   lowrank   (B,H,W, 2*dt_rank)       the inputs of the two dt projections, T then L
 */
size_t m2d_proj_workspace_bytes(const m2d_desc* desc, int dt_rank, int pass);

/* lowrank | BT | BL | C = split(x @ x_proj_w^T);  delta{T,L} = softplus(lowrank{T,L} @ dt_proj{T,L}_w^T + b)
 * (wavefront_cuda.py:75-86).  All six outputs are written. */
int m2d_proj_fwd(const m2d_desc* desc, int dt_rank,
                 const void* x,
                 const float* x_proj_w, const float* dt_projT_w, const float* dt_projT_b,
                 const float* dt_projL_w, const float* dt_projL_b,
                 void* lowrank, void* deltaT, void* deltaL, void* BT, void* BL, void* C,
                 void* workspace, size_t workspace_bytes,
                 void* stream);

/* Backward of m2d_proj_fwd for the gradients d_deltaT ... d_C that m2d_scan_bwd produced.
 * dx is read and written: on entry the scan's own gradient for x, on return that plus the
 * gradient through the projections (wavefront_cuda.py:303-311).  The five weight gradients are
 * written (not accumulated). */
int m2d_proj_bwd(const m2d_desc* desc, int dt_rank,
                 const void* x, const void* lowrank, const void* deltaT, const void* deltaL,
                 const float* x_proj_w, const float* dt_projT_w, const float* dt_projL_w,
                 const void* d_deltaT, const void* d_deltaL,
                 const void* d_BT, const void* d_BL, const void* d_C,
                 void* dx,
                 float* d_x_proj_w, float* d_dt_projT_w, float* d_dt_projT_b,
                 float* d_dt_projL_w, float* d_dt_projL_b,
                 void* workspace, size_t workspace_bytes,
                 void* stream);

/* Number of per-workgroup partial sums that m2d_scan_bwd leaves with M2D_FLAG_SUM_PARTS for this descriptor
 * (0 for an invalid one); host only. */
int m2d_scan_sum_parts(const m2d_desc* desc);

/* m2d_proj_bwd for gradients d_BT, d_BL, d_C that arrive as the partial sums of M2D_FLAG_SUM_PARTS: d_BT points to
 * sum_parts records as described there, which are added up in their order as they are loaded and rounded to
 * desc->dtype; d_BL and d_C are ignored.  sum_parts = 0 is m2d_proj_bwd.  Only where the products run on the matrix
 * cores (bf16, E a multiple of 8); otherwise M2D_ERR_UNSUPPORTED. */
int m2d_proj_bwd_parts(const m2d_desc* desc, int dt_rank, int sum_parts,
                       const void* x, const void* lowrank, const void* deltaT, const void* deltaL,
                       const float* x_proj_w, const float* dt_projT_w, const float* dt_projL_w,
                       const void* d_deltaT, const void* d_deltaL,
                       const void* d_BT, const void* d_BL, const void* d_C,
                       void* dx,
                       float* d_x_proj_w, float* d_dt_projT_w, float* d_dt_projT_b,
                       float* d_dt_projL_w, float* d_dt_projL_b,
                       void* workspace, size_t workspace_bytes,
                       void* stream);

/* ---- Two operators of the residual block around the scan (inference forward) -------------------
 * The reference's blocks normalise channel-last activations with nn.LayerNorm over 64 to 512
 * channels (models/mamba2d.py:57,220,248,363; models/utils.py:13,232-233) and run a depthwise 3x3
 * convolution in the local path (models/utils.py:101-114).  Both are bandwidth-bound; these kernels
 * read the input once and write the output once.  dtype is the element type of x and y, weight_dtype
 * that of the weights (m2d_dtype each); arithmetic is fp32.  Every array must be 16-byte aligned.
 *
 * y[r,:] = (x[r,:] - mean) / sqrt(var + eps) * weight + bias over the C values of each of `rows` rows
 * (biased variance, as nn.LayerNorm).  C must be a multiple of 8 (bf16) / 4 (fp32), at most 4096 / 2048. */
int m2d_layernorm_fwd(int64_t rows, int C, int dtype, int weight_dtype,
                      const void* x, const void* weight, const void* bias, float eps, void* y, void* stream);

/* y = depthwise 3x3 cross-correlation of x (B,H,W,C), stride 1, zero padding 1, no bias; weight is the
 * (C,1,3,3) tensor of nn.Conv2d(C, C, 3, padding=1, groups=C).  C must be a multiple of 8 (bf16) / 4 (fp32). */
int m2d_dwconv3x3_fwd(int B, int H, int W, int C, int dtype, int weight_dtype,
                      const void* x, const void* weight, void* y, void* stream);

/* y = scale * relu(x)^2 + bias over n elements with one scale and one bias (StarReLU, models/utils.py:26-44).
 * n must be a multiple of 8 (bf16) / 4 (fp32). */
int m2d_starrelu_fwd(int64_t n, int dtype, int weight_dtype, const void* x, const void* scale, const void* bias,
                     void* y, void* stream);

/* y[r,c] = x[r,c] * scale[c] + residual[r,c] (+ residual2[r,c]): the residual update of a block with its
 * learned per-channel scale (models/mamba2d.py:258-259, models/utils.py:46-55).  residual2 may be NULL; it
 * takes the second term of a token mixer whose answer is a sum (scan path + local path,
 * models/mamba2d.py:176), which then is never written out on its own.  y may be x or a residual. */
int m2d_scale_residual_fwd(int64_t rows, int C, int dtype, int weight_dtype, const void* x, const void* scale,
                           const void* residual, const void* residual2, void* y, void* stream);

/* The residual update with the LayerNorm that follows it (models/mamba2d.py:258-259: the first update feeds
 * norm2 of the same block, the second norm1 of the next block or the LayerNorm that ends the stage):
 * x_out = x * scale[c] + residual (+ residual2, may be NULL), y = LayerNorm(x_out) over C with weight, bias, eps,
 * where the norm sees x_out as stored (rounded to the element type).  Same limits as m2d_layernorm_fwd;
 * x_out may be x or a residual. */
int m2d_scale_residual_layernorm_fwd(int64_t rows, int C, int dtype, int weight_dtype, const void* x, const void* scale,
                                     const void* residual, const void* residual2, const void* weight, const void* bias,
                                     float eps, void* x_out, void* y, void* stream);

/* Rotary embedding and per-head LayerNorm of q and k in the attention stages (models/utils.py:253-301):
 * qkv is the output of the qkv projection, (B, L, 3, heads, head_dim); cos and sin are (L, head_dim) tables
 * of qkv's element type in which the two features of a pair (2i, 2i+1) hold the same angle (cos 1, sin 0 on
 * features that do not rotate); rotated[2i] = x[2i] cos - x[2i+1] sin, rotated[2i+1] = x[2i+1] cos + x[2i] sin.
 * q and k receive LayerNorm(rotated) with their own weights, laid out (B, heads, L, head_dim), or, with
 * token_major != 0, (B, L, heads, head_dim): the layout of the projection itself, which an attention
 * kernel that takes strides reads as it is and answers in, so that its output needs no transposing copy.
 * head_dim must be 8, 16, ... 256 (bf16) / 4, 8, ... 128 (fp32), a power of two. */
int m2d_rope_qknorm_fwd(int B, int L, int heads, int head_dim, int dtype, int weight_dtype,
                        const void* qkv, const void* cos, const void* sin,
                        const void* q_weight, const void* q_bias, const void* k_weight, const void* k_bias,
                        float eps, int token_major, void* q, void* k, void* stream);

/* The whole attention of a rotary stage (models/utils.py:253-316) for heads of 32 features and up to 256
 * tokens, bf16: out[b, l, head, :] = softmax_l'(scale * q[l] . k[l']) v[l'] with q and k rotated and
 * LayerNormed per head as m2d_rope_qknorm_fwd does, v taken as it is; qkv is (B, L, 3, heads, 32), cos and sin
 * are (L, 32) bf16, out is (B, L, heads, 32), the input of the output projection.  Scores, softmax and the
 * sums are fp32; the probabilities enter the second product rounded to bf16.
 * head_dim other than 32 or L > 256: M2D_ERR_UNSUPPORTED. */
int m2d_rope_attention_fwd(int B, int L, int heads, int head_dim, int weight_dtype,
                           const void* qkv, const void* cos, const void* sin,
                           const void* q_weight, const void* q_bias, const void* k_weight, const void* k_bias,
                           float eps, float scale, void* out, void* stream);

/* y = post(pre(x) weight^T + bias) for the narrow linear layers of a block on bf16 activations: in_proj and
 * out_proj of the token mixer (models/mamba2d.py:166-176), the pointwise convolutions of the local path
 * (models/utils.py:87-118) and the MLP (models/utils.py:58-81), together with the activation the block
 * applies before or after the layer.  x (P,K) and y (P,N) are bf16; weight (N,K), bias (N, may be NULL) and
 * the activation parameters have weight_dtype.  pre_act / post_act: 0 nothing, 1 GELU (exact form),
 * 2 StarReLU with the one-element scale and bias given (device pointers, ignored otherwise).
 * K must be a multiple of 32 up to 512 and N a multiple of 16 (the weight matrix is held in LDS as bf16,
 * in slices of 64 or more outputs per workgroup); M2D_ERR_UNSUPPORTED otherwise. */
#define M2D_ACT_NONE 0
#define M2D_ACT_GELU 1
#define M2D_ACT_STARRELU 2
int m2d_linear_fwd(int64_t P, int K, int N, int weight_dtype, const void* x, const void* weight, const void* bias,
                   int pre_act, const void* pre_scale, const void* pre_bias,
                   int post_act, const void* post_scale, const void* post_bias, void* y, void* stream);

/* m2d_linear_fwd with a LayerNorm over the K inputs in front of the layer (ln_weight, ln_bias: (K), weight_dtype):
 * y = post(LayerNorm(x) weight^T + bias), for a norm whose only reader is the layer (local_norm before pwconv1,
 * models/mamba2d.py:57,161; norm2 before fc1, :248).  The normalised rows are rounded to bf16 as a LayerNorm
 * kernel would store them, and never written.  K up to 128; otherwise as m2d_linear_fwd. */
int m2d_layernorm_linear_fwd(int64_t P, int K, int N, int weight_dtype, const void* x,
                             const void* ln_weight, const void* ln_bias, float eps,
                             const void* weight, const void* bias,
                             int post_act, const void* post_scale, const void* post_bias, void* y, void* stream);

/* y = fc2(GELU(fc1 x)) of the MLP (models/utils.py:58-81) where both weight matrices fit LDS together:
 * C = 32 or 64 channels and hidden = 4 C.  x and y are (P, C) bf16; w1 (hidden, C), b1 (hidden), w2 (C, hidden),
 * b2 (C) have weight_dtype; b1 and b2 may be NULL.  The hidden activations stay in registers; they enter the
 * second product rounded to bf16, as the stock path stores them.  With ln_weight and ln_bias (C each, weight_dtype;
 * both or neither) the rows of x pass through LayerNorm(eps) first (norm2 of the block, models/mamba2d.py:248),
 * rounded to bf16 as a LayerNorm kernel would store them.  Other sizes: M2D_ERR_UNSUPPORTED. */
int m2d_mlp_fwd(int64_t P, int C, int hidden, int weight_dtype, const void* x,
                const void* ln_weight, const void* ln_bias, float eps,
                const void* w1, const void* b1, const void* w2, const void* b2, void* y, void* stream);

/* Measurement aid; no counterpart in the reference.  While enabled, every m2d_scan_fwd /
 * m2d_scan_bwd call records a pair of HIP events on its stream around the main scan kernel of
 * the pass (not around the small set-up and reduction kernels).  m2d_profile_last_ms waits for
 * the most recent such pair and returns the elapsed milliseconds.  The events are process-wide:
 * enable it only from a single-threaded benchmark. */
int m2d_profile_enable(int on);
int m2d_profile_last_ms(int pass, float* ms);

/* ---- The reference's native entry points at their own boundary -----------------------------------
 * wf_fwd and wf_bwd as the reference's extension exports them (wf_cuda_bind.cpp:24-46), for callers of its
 * custom operators mamba2d::wf_fwd / mamba2d::wf_bwd (wavefront_cuda.py:25-57): they materialise the state
 * tensor hs (B,H,W,E,N), which the fused calls above never do, take any number of states N and the three
 * element types the reference dispatches (wf_cuda.cu:182,240), and are not on the fast path.  dtype names the one
 * element type of every tensor: M2D_F32, M2D_BF16 (fp32 arithmetic, every stored value rounded once) or M2D_F64.
 *
 * m2d_wf_fwd fills hs with the recurrence of wf_cuda.cu:40-69.
 * m2d_wf_bwd is wf_cuda.cu:108-160: grad_output (B,H,W,E,N) holds dL/dhs on entry and dBX on return, dDAT and
 * dDAL (B,H,W,E,N) are written, omega (2,B,H,E,N) is scratch; x is not read (as in the reference).
 * All pointers are device pointers to contiguous arrays; one launch per call, nothing is allocated. */
#define M2D_F64 2
int m2d_wf_fwd(int B, int H, int W, int E, int N, int dtype, void* hs, const void* x, const void* deltaT,
               const void* deltaL, const void* BT, const void* BL, const void* AT, const void* AL, void* stream);
int m2d_wf_bwd(int B, int H, int W, int E, int N, int dtype, const void* hs, const void* x, const void* deltaT,
               const void* deltaL, const void* AT, const void* AL, void* grad_output, void* dDAT, void* dDAL,
               void* omega, void* stream);

/* Measurement aid; no counterpart in the reference.  What the vector ALUs of the current device issue per
 * second, measured by a small kernel that fills the device with `waves_per_simd` waves per SIMD (1 to 8; the scan
 * kernels run 2), each lane running 65536 operations of one kind on registers:
 *   M2D_RATE_FMA, M2D_RATE_EXP                      v_fma_f32 / v_exp_f32, 16 independent chains per lane
 *   M2D_RATE_FMA_DEPENDENT, M2D_RATE_EXP_DEPENDENT  one chain per lane: every operation waits for the one before
 *   M2D_RATE_SCAN_FWD_UNIT                          the forward scan's arithmetic per (cell, channel, state): two gate
 *                                                   exponents with their multiply-adds, five multiply-adds
 * *per_second receives lane-operations per second over the whole device (units per second for the last kind).
 * `scratch` is a device buffer of at least 1 KiB x compute units x waves_per_simd that the kernel writes its
 * (meaningless) results to.  The call times six launches with a pair of events and synchronises on them. */
#define M2D_RATE_FMA 0
#define M2D_RATE_FMA_DEPENDENT 1
#define M2D_RATE_EXP 2
#define M2D_RATE_EXP_DEPENDENT 3
#define M2D_RATE_SCAN_FWD_UNIT 4
int m2d_valu_rate_probe(int kind, int waves_per_simd, void* scratch, size_t scratch_bytes, void* stream, double* per_second);

#ifdef __cplusplus
}
#endif
#endif /* M2DSCAN_H */
