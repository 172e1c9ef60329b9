/*
 * xlstm_amd — C ABI of the MI355X (gfx950) sLSTM forward / decode engine.
 *
 * Plain C: raw device pointers, sizes, enums and an opaque stream handle.  No
 * C++ or torch types cross this boundary.  The caller owns every buffer
 * (inputs, outputs and the workspace); the library allocates nothing and
 * never synchronises the device.  Every entry point returns 0 on success or a
 * negative XS_ERR_* code; xs_last_error() gives the text for the calling thread.
 *
 * What each entry point replaces in the reference (NX-AI/xlstm, paths relative
 * to its root) is cited at its declaration.
 */
#ifndef XLSTM_AMD_H
#define XLSTM_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XS_ABI_VERSION 16

/* element types */
enum { XS_F32 = 0, XS_BF16 = 1 };

/* error codes */
enum {
  XS_OK = 0,
  XS_ERR_NULL = -1,        /* a required pointer is NULL */
  XS_ERR_SHAPE = -2,       /* a dimension is out of range or inconsistent */
  XS_ERR_DTYPE = -3,       /* unsupported dtype combination */
  XS_ERR_ALIGN = -4,       /* pointer or stride not aligned as documented */
  XS_ERR_UNSUPPORTED = -5, /* shape is valid but not covered by a kernel */
  XS_ERR_WORKSPACE = -6,   /* workspace missing or too small */
  XS_ERR_LAUNCH = -7,      /* the HIP runtime refused the launch */
  XS_ERR_DEVICE = -8       /* device does not fit the grid (co-residency) */
};

/*
 * Arguments of one cell call.  All pointers are DEVICE pointers.
 *
 *   wx     [B, T, 4, NH, dh]  gate pre-activations (gate order i,f,z,o), element
 *                             type wx_dtype.  The innermost 4*NH*dh elements are
 *                             contiguous; rows/steps are addressed through
 *                             wx_stride_b / wx_stride_t (in ELEMENTS), so the
 *                             [B,S,4H] tensor the layer produces is read in place
 *                             (the reference permutes and copies it first:
 *                             xlstm/blocks/slstm/cell.py:327-352, :768-774).
 *   r      [NH, 4*dh, dh]     recurrent matrix, r[h][g*dh + a][d] multiplies input
 *                             unit d of head h into gate g of output unit a —
 *                             the K-contiguous layout of the reference's vanilla
 *                             backend (cell.py:601-617).  r_dtype is XS_F32 or
 *                             XS_BF16; with wx_dtype == XS_F32 it must be XS_F32.
 *   bias   [NH, 4, dh]        float32 (cell.py:253-257, external view).
 *   s0     [4, B, NH*dh]      float32 initial y,c,n,m or NULL for zeros (cell.py:441-469).
 *   reset  [B, T] uint8       or NULL.  Non-zero at (b,t) => y,c,n,m of row b are
 *                             zeroed before step t (start of a packed document).
 *                             Row stride reset_stride_b in bytes.  Not in the
 *                             reference (only the unused `lengths`, cell.py:496).
 *   h_out  [T, B, NH*dh]      hidden state after every step, element type
 *                             wx_dtype, contiguous (the reference's
 *                             all_states[0][1:], cell.py:502).
 *   s_out  [4, B, NH*dh]      float32 state after the last step (cell.py:471-476).
 *                             Must not overlap s0 (other compute units still read it).
 *   workspace                 at least xs_slstm_workspace_bytes() bytes, 256-byte
 *                             aligned.  Holds the status block (below), one
 *                             placement word per workgroup and the exchange
 *                             ring through which the compute units of a head
 *                             pass h_t to each other (a few MiB).  Two calls
 *                             that may overlap in time need different workspaces;
 *                             two sequence calls that overlap on one GPU also
 *                             compete for its compute units (each needs all of
 *                             its workgroups running at once), so one of them
 *                             waits, within spin_limit, until the other is done.
 *   stream                    hipStream_t (NULL = the null stream).
 *   spin_limit                bound on every wait between compute units (a step: between
 *                             the waves of a workgroup), in poll iterations; 0 selects
 *                             the default.  When a wait runs out the kernel records it
 *                             in the status block and finishes without waiting any further.
 *   h_prev [B, NH*dh]         optional, xs_slstm_step with bf16 wx only (ignored
 *                             otherwise): the y plane of s0 rounded to bf16, i.e.
 *                             the h_out of the previous step.  The kernel rounds
 *                             y to bf16 anyway before it multiplies by r; given
 *                             this copy it reads half the bytes and the result is
 *                             bit for bit the same.  The caller vouches for the
 *                             copy: it is not compared with s0.  Not in the
 *                             reference.
 *   coef_out                  optional, xs_slstm_forward only: a training forward.  The
 *                             nine float32 coefficients per step and element that
 *                             xs_slstm_backward_prepare would otherwise recompute, in the
 *                             order xs_slstm_backward reads them with split == 2:
 *                             [T][ceil(B/4)][NH][dh/64][4 rows][9][64 units]
 *                             (T * ceil(B/4)*4 * 9 * H floats).  Takes the place of the
 *                             state history and gate cache that the reference's forward
 *                             keeps for its backward (slstm.cc:79-108).  Only where the
 *                             call runs in row tiles of 4 rows of one kernel: bf16 wx, head
 *                             dim 128 or 256, a batch whose row tiles of 4 rows fit the
 *                             device; otherwise XS_ERR_UNSUPPORTED before anything is
 *                             launched (call again without it and use
 *                             xs_slstm_backward_prepare).  h_out and s_out are bit for bit
 *                             those of a call without it.
 *   r_tiled                   optional, xs_slstm_step only: r in the element type of wx as
 *                             xs_slstm_tile_r_for_steps lays it out, made once per change
 *                             of the parameters.  With it a step at a head dim beyond 256
 *                             (bf16; with h_prev) or 128 (f32), a multiple of 64, runs a
 *                             kernel whose operands are brought to LDS by waves of their
 *                             own (13 -> 8 us a step at 4 heads of 512); the result is bit
 *                             for bit the same.  Ignored elsewhere.  Not in the reference.
 */
typedef struct xs_slstm_args {
  int32_t B, T, NH, dh;
  int32_t wx_dtype, r_dtype;
  const void *wx;
  int64_t wx_stride_b, wx_stride_t;
  const void *r;
  const float *bias;
  const float *s0;
  const uint8_t *reset;
  int64_t reset_stride_b;
  void *h_out;
  float *s_out;
  void *workspace;
  size_t workspace_bytes;
  void *stream;
  int64_t spin_limit;
  const void *h_prev;
  float *coef_out;
  const void *r_tiled;
} xs_slstm_args;

/* Status block at the start of the workspace, written by the kernels. */
typedef struct xs_slstm_status {
  uint32_t aborted;     /* 1 if a bounded wait ran out: the results are invalid, and every workgroup that finished after
                           the give-up has overwritten its part of h_out and s_out with NaN (a step: the workgroup
                           whose waves gave up on each other writes NaN for its tile) */
  uint32_t abort_wg;    /* workgroup that gave up first */
  uint32_t abort_step;  /* timestep it was waiting for */
  uint32_t max_spins;   /* largest number of poll iterations any wait needed */
  uint32_t xcd_mixed;   /* number of head groups whose workgroups ran on more than one XCD */
  uint32_t launches;    /* kernel launches the call was split into */
  uint32_t step_kernel; /* 1 if the call ran the single-token step kernel (xs_slstm_step, or xs_slstm_forward with T == 1) */
  uint32_t rows_per_workgroup; /* sequence kernels: batch rows a workgroup handles (4, 8, 16, 32 = two row tiles, 64 = four
                                  row tiles: the kernel with MFMA waves and gating waves), of the last launch; 0 after a step */
  uint32_t pipelined_step; /* 1 if the step ran the pipelined step kernel (bf16, head dim 256, whole tiles, a state, no mask,
                              h_prev given), 0 if the tile kernel; 0 after a sequence call */
  uint32_t reserved[7];
} xs_slstm_status;

/* Library / ABI identification.  Replaces nothing (the reference keys its JIT
 * modules by config, cell.py:509-534). */
int xs_abi_version(void);

/* Text of the last error on the calling thread ("" if none). */
const char *xs_last_error(void);

/* Bytes of workspace a call with these dimensions needs. */
size_t xs_slstm_workspace_bytes(int32_t B, int32_t T, int32_t NH, int32_t dh);

/*
 * Sequence forward: T steps in ONE persistent launch (per batch chunk).
 * Replaces sLSTMFunc.forward -> ForwardPass::Run, i.e. the per-timestep
 * cuBLAS GEMM + pointwise kernel loop
 * (xlstm/blocks/slstm/src/cuda/slstm.cc:53-135,
 *  xlstm/blocks/slstm/src/cuda/slstm_forward.cu:217-267) and the vanilla loop
 * (xlstm/blocks/slstm/src/vanilla/__init__.py:17-74).
 * A call with T == 1 whose recurrent matrix is in the dtype of wx is what the
 * reference's layer makes for every decoded token (xlstm/blocks/slstm/layer.py:113-115);
 * it runs the step kernel of xs_slstm_step (same bits, status.step_kernel = 1).
 */
int xs_slstm_forward(const xs_slstm_args *args);

/*
 * xs_slstm_forward for callers that cannot allocate device memory or pass a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments and results as xs_slstm_forward, except that args->workspace and args->workspace_bytes are
 * ignored: the status block, the placement words and the exchange ring live in an array of
 * XS_STATIC_SCRATCH_BYTES that is part of the library's device image (each GPU the library runs on holds it
 * until the process ends).  It calls no allocator, host or device.  4 MiB + 64 KiB hold every bfloat16 call on a
 * device of 256 compute units; a call whose launches need more (float32 with four row tiles per workgroup on all
 * compute units, e.g. B >= 128 at NH 4 x dh 512: 8 MiB) returns XS_ERR_WORKSPACE before anything is launched.  All calls on one GPU share its array: calls that overlap in
 * time on one GPU race (give each stream its own workspace through xs_slstm_forward instead); what must start
 * clean is cleared by fill kernels at the start of every call.  The status block is not reachable by the caller.
 */
#define XS_STATIC_SCRATCH_BYTES ((4u << 20) + (64u << 10))
int xs_slstm_forward_static(const xs_slstm_args *args);

/*
 * Single-token decode step (T must be 1): state in, state out, no waits
 * between compute units; bit-identical to the same step inside a sequence
 * call.  The recurrent matrix must be in the dtype of wx (keep a bf16 copy
 * for bf16 decoding instead of converting it every token).  Replaces the
 * T == 1 use of the same reference entry (xlstm/blocks/slstm/layer.py:113-115
 * calls the cell's forward with S = 1).
 */
int xs_slstm_step(const xs_slstm_args *args);

/*
 * xs_slstm_tile_r_for_steps   r ([NH, 4*dh, dh] in dtype, the forward's layout; dh a multiple of 64) into the slabs that
 *   xs_slstm_step reads it in when xs_slstm_args::r_tiled is given: [NH][unit/32][k/KS][gate][unit%32][k%KS] with KS
 *   = 128 bytes of K (NH*4*dh*dh elements).  No counterpart in the reference, whose step GEMM reads R as it lies
 *   (slstm_forward.cu:176-182).
 */
int xs_slstm_tile_r_for_steps(const void *r, void *r_tiled, int32_t NH, int32_t dh, int32_t dtype, void *stream);

/*
 * The operations around the cell inside an sLSTM layer (bf16 only; the layer keeps its
 * PyTorch path for everything else).  They enqueue one kernel each and allocate nothing.
 *
 * xs_causal_conv_silu: out[b,t,c] = silu(bias[c] + sum_j weight[c,j] * x[b, t-(K-1)+j, c]),
 * the causal depthwise convolution of xlstm/components/conv.py:113-127 followed by the
 * activation of xlstm/blocks/slstm/layer.py:136-137.  Inputs before t = 0 are read from
 * conv_state (the K-1 tokens before this call, conv.py:118-122) or are zero.  With a reset
 * mask (not in the reference) a tap that would reach before the start of the token's document
 * reads zero.
 */
typedef struct xs_conv_args {
  int32_t B, T, D, K;        /* K taps, 2..4; D a multiple of 8 */
  int32_t dtype;             /* XS_BF16 */
  const void *x;             /* [B,T,D], strides in elements, innermost contiguous */
  int64_t x_stride_b, x_stride_t;
  const void *conv_state;    /* [B,K-1,D] or NULL; tokens contiguous, rows conv_state_stride_b apart */
  int64_t conv_state_stride_b; /* in elements; 0 = (K-1)*D */
  const void *weight;        /* [D,K] (nn.Conv1d's [D,1,K]) */
  const void *bias;          /* [D] or NULL */
  const uint8_t *reset;      /* [B,T] or NULL, row stride reset_stride_b bytes */
  int64_t reset_stride_b;
  void *out;                 /* [B,T,D] contiguous */
  void *stream;
  void *ring_out;            /* NULL, or with T == 1 a [B,K,D] contiguous buffer that receives the K-1 inputs
                                before x followed by x: the state of the next step (conv.py:142-149) */
} xs_conv_args;

int xs_causal_conv_silu(const xs_conv_args *args);

/*
 * xs_headwise_gates: the four block-diagonal gate projections and their concatenation,
 *   out[m, g*H + h*dh + o] = sum_d A_g[m, h*dh + d] * w[g][h, o, d],   H = NH*dh,
 * with A_g = x_conv for the slots g = i, f and x for g = z, o
 * (xlstm/blocks/slstm/layer.py:144-153: four LinearHeadwiseExpand modules,
 * xlstm/components/linear_headwise.py:75-82, then torch.cat).  `out` is the cell's wx.
 * w[] is in SLOT order i, f, z, o; the reference wires its module named fgate to the i slot
 * and igate to the f slot (layer.py:144-149).
 */
typedef struct xs_gates_args {
  int32_t M, NH, dh;         /* M = B*T tokens; dh a multiple of 64 */
  int32_t dtype;             /* XS_BF16 */
  const void *x;             /* [M, H], row stride in elements */
  int64_t x_stride_row;
  const void *x_conv;        /* [M, H] */
  int64_t x_conv_stride_row;
  const void *w[4];          /* each [NH, dh, dh] contiguous */
  void *out;                 /* [M, 4*H] */
  int64_t out_stride_row;
  void *stream;
} xs_gates_args;

int xs_headwise_gates(const xs_gates_args *args);

/*
 * xs_headwise_group_norm: the per-head group norm behind the cell,
 *   out[b,t,h,:] = (x[b,t,h,:] - mean) / sqrt(var + eps) * (1 + weight[h,:])
 * with mean and (biased) variance over the dh units of head h of one token
 * (MultiHeadLayerNorm.forward, xlstm/components/ln.py:51-68, with the residual weight of
 * ln.py:29-33, as called by xlstm/blocks/slstm/layer.py:159).  x is addressed by strides so that
 * the cell's [T,B,H] output is read where it lies; out is token-major, the layer's output layout.
 */
typedef struct xs_norm_args {
  int32_t B, T, NH, dh;      /* dh a multiple of 4, at most 1024 */
  int32_t dtype;             /* XS_BF16 */
  float eps;
  const void *x;             /* element (b,t,h,d) at b*x_stride_b + t*x_stride_t + h*x_stride_h + d */
  int64_t x_stride_b, x_stride_t, x_stride_h;
  const void *weight;        /* [NH*dh] or NULL (scale 1) */
  void *out;                 /* [B,T,NH*dh] contiguous */
  void *stream;
} xs_norm_args;

int xs_headwise_group_norm(const xs_norm_args *args);

/*
 * Backward pass of the cell (training), by the rule of the reference's native kernel: the stabiliser m is a
 * constant of the differentiation (xlstm/blocks/slstm/src/cuda/slstm_pointwise.cu:118-196).  Two calls replace the
 * reference's per-timestep launches (slstm_backward.cu:291-319) and the state history and gate cache its forward
 * writes for them (slstm.cc:79-108); the forward entry points above store nothing for training.
 *
 * xs_slstm_backward_prepare  walks forward in time over raw = wx + R.y_{t-1} + bias, recomputing R.y_{t-1} from the
 *   outputs h_out of the forward call (y_{-1} the y plane of s0; zero where reset[b,t] is set) and r, and writes nine
 *   float32 coefficients per step and element into coef [T,B,9,H] (with split != 0: T * ceil(B/16)*16 * 9 * H floats,
 *   in the order the split kernel reads them).
 * xs_slstm_backward          one launch for all T steps, reverse in time: d_wx [B,T,4,NH,dh] (float32, or bf16 with d_wx_dtype; the gradient
 *   with respect to the raw gates: the gradient of wx, and with the outputs what the gradients of R and the bias are
 *   sums of, slstm_backward.cu:381-386, 52-108) and d_s0 [4,B,H] (the m part is zero).
 *
 * dtype is the type of wx, d_h and r_t (XS_F32 or XS_BF16).  r_t is R transposed - element (input unit d, gate
 * unit k = g*dh + a) of head h is the reference's external view recurrent_kernel[h][d][g][a] (cell.py:234-242) -
 * tiled as MFMA operands: [NH][d/16][k/KC][(k%KC)/EPC][d%16][k%EPC] with EPC = 16 bytes of elements (8 bf16, 4 f32)
 * and KC = 4*EPC, so that what the 64 lanes of a wave load for one k-step is 1 KiB in a row.  Head dims: 64, 128, 256
 * (512 with bf16 and split; up to 1024 with bf16 and 512 with f32 with split == 3, one launch per step).
 * The caller owns every buffer; both calls only enqueue kernels on `stream`.
 */
typedef struct xs_slstm_bwd_args {
  int32_t B, T, NH, dh;
  int32_t dtype;
  const void *wx;            /* [B,T,4,NH,dh], strides in elements, innermost 4*H contiguous (prepare) */
  int64_t wx_stride_b, wx_stride_t;
  const float *ry;           /* unused (an earlier version took R.y_{t-1} of all steps here); pass NULL */
  const float *bias;         /* [NH,4,dh] (prepare) */
  const float *s0;           /* [4,B,H] or NULL (prepare) */
  const uint8_t *reset;      /* [B,T] or NULL, row stride reset_stride_b bytes (both) */
  int64_t reset_stride_b;
  float *coef;               /* [T,B,9,H] ([T,ceil(B/16)*16,9,H] with split, [T,ceil(B/4)*4,9,H] with split == 2, [T,ceil(B/64)*64,9,H] with split == 3): written by prepare, read by backward */
  const void *d_h;           /* [T,B,H]: gradient with respect to h_out (backward) */
  const float *d_s_final;    /* [4,B,H] or NULL: gradient with respect to the final state; y, c, n are used (backward) */
  const void *r_t;           /* (backward) */
  void *d_wx;                /* [B,T,4,NH,dh] float32 (or bf16: d_wx_dtype below), strides in elements (backward, params) */
  int64_t d_wx_stride_b, d_wx_stride_t;
  float *d_s0;               /* [4,B,H] (backward) */
  void *stream;
  /* backward, optional: a head spread over dh/64 compute units (head dims 64, 128, 256; 512 in bf16).  With split != 0,
   * r_t holds R transposed with K ordered k = 256*(a/64) + 64*g + a%64 (a the hidden unit, g the gate), tiled as MFMA
   * operands per owner of the output columns and per wave: [NH][dh/64][8][K/8/KC][4][KC/EPC][16][EPC], EPC the elements
   * of 16 bytes and KC = 4*EPC; exchange is a 16-byte aligned buffer of 4 * NH * ceil(B/16) * 16 * 4*dh elements of
   * dtype and counters 1 + 2 * NH * ceil(B/16) 32-bit words; the library initialises both in front of the kernel, and the
   * FIRST word is nonzero after the call when a bounded wait between the compute units of a head ran out, or when the
   * workgroups of a head did not run on one XCD as the exchange assumes (d_s0 is NaN then).
   * split == 2 (XS_BF16, head dims 64, 128, 256): row tiles of 4 rows instead of 16, four times the workgroups, a
   * shorter step; for batches whose NH * ceil(B/4) * dh/64 workgroups fit the device.  Then K is ordered k = 4*a + g,
   * r_t is tiled the same way, coef is [T][ceil(B/4)][NH][dh/64][4 rows][9][64 units], exchange has
   * 4 * NH * ceil(B/4) * 4 * 4*dh elements and counters 1 + 2 * NH * ceil(B/4) words.
   * The call is refused (XS_ERR_DEVICE) when its workgroups do not all fit the device at once.
   * split == 3 (both calls; head dims 512 to 1024 with XS_BF16, 256 to 512 with XS_F32, in steps of 64:
   * up to what the forward entry points cover): ONE LAUNCH PER STEP instead of one per call, the reference's own
   * decomposition (slstm_backward.cu:291-319), for head dims whose slice of R no compute unit can keep in registers.
   * prepare launches, once per four steps, a kernel that multiplies the outputs of the steps before (h_out) by r in one
   * pass over r and runs the forward's update step by step, the backward call T + 1 times a kernel that multiplies the gate deltas of the step behind by R
   * transposed and forms the step's gradient.  Then coef has T * ceil(B/64)*64 * 9 * H floats, in the order the walk's
   * waves write and the reverse pass's read them; r_t is R transposed (element (d, k = g*dh + a))
   * in slabs of 256 bytes of K per tile of 32 input units, [NH][d/32][k/KS][d%32][k%KS] with KS = 128 (bf16) or 64
   * (f32), so that what a workgroup stages per slab is 8 KiB in a row; counters is not used, nothing waits and nothing
   * can give up; and exchange is a 16-byte aligned buffer of at least
   * max(16*B*H + 4*NH*dh*dh*sizeof(dtype), 8*ceil(B/64)*64*H*sizeof(dtype)) bytes: the walk's state and its copy of r
   * (prepare), the gate deltas from launch to launch (backward). */
  int32_t split;
  void *exchange;
  uint32_t *counters;
  int64_t spin_limit;        /* bound of the waits between the compute units of a head, in looks; 0 = default; negative:
                                every such wait gives up at its first look (forces the error path from the host: the
                                kernel still runs to its end, counters[0] is set and d_s0 is NaN) */
  /* backward, the two options of the reference's native backward pass (cell.py:84-87):
   * recurrent_cut != 0       no gradient passes from a step to the y it started from: the product with R transposed is
   *                          left out (sLSTMFunc.backward_cut, slstm.cc:223-304, slstm_backward_cut.cu:265-312); c and n
   *                          still pass theirs on, and d_s0's y plane is zero.
   * recurrent_clipval > 0    the gradient that reaches y_t from step t+1 is clipped to +-recurrent_clipval before d_h is
   *                          added (slstm_pointwise.cu:136-143); the y plane of d_s_final counts as coming from outside
   *                          (the reference receives it through the same argument as d_h) and is not clipped.
   *                          0, negative or not finite: no clipping. */
  int32_t recurrent_cut;
  float recurrent_clipval;
  /* the forward call's outputs and recurrent matrix, and the gradients of the parameters */
  const void *h_out;         /* [T,B,H] in dtype: what the forward call returned (prepare, params) */
  const void *r;             /* [NH,4*dh,dh] in dtype, the forward's layout (prepare) */
  float *d_r;                /* [NH,4*dh,dh] float32: gradient of r in that layout (params) */
  float *d_bias;             /* [NH,4,dh] float32 (params) */
  /* the type of d_wx: XS_F32 (0, the default), or XS_BF16 with dtype == XS_BF16 - the gate deltas are then written
   * rounded to bf16, as the reference returns dx in the type of its kernels (slstm.cc:137-221), the reverse kernel
   * writes and xs_slstm_backward_params reads half the bytes, and a caller whose input is bf16 needs no conversion
   * (d_wx must then be 16-byte aligned and its strides multiples of 8 elements) */
  int32_t d_wx_dtype;
} xs_slstm_bwd_args;

int xs_slstm_backward_prepare(const xs_slstm_bwd_args *args);
int xs_slstm_backward(const xs_slstm_bwd_args *args);

/*
 * xs_slstm_backward_params   the gradients of the recurrent matrix and the bias from the gate deltas that
 *   xs_slstm_backward left in d_wx and the forward's outputs: d_r[h][g*dh+a][d] = sum over rows and steps of
 *   d_wx[b,t,g,h,a] * y_{t-1}[b,h,d] (y_{-1} the y plane of s0; zero where reset[b,t] is set), d_bias[h][g][a] = sum of
 *   d_wx[b,t,g,h,a].  Replaces the strided-batched GEMM and the bias aggregation behind the reference's time loop
 *   (slstm_backward.cu:381-386, 52-108).  Uses B, T, NH, dh (a multiple of 64), dtype, d_wx and its strides, h_out, s0,
 *   reset, d_r, d_bias, stream.  With bf16 the deltas are rounded to bf16 for the product (float32 sums), as the
 *   reference's gate cache is.  The sums over slices of B*T are added with float atomics: their last bits depend on
 *   the order the compute units finish in.
 */
int xs_slstm_backward_params(const xs_slstm_bwd_args *args);

/*
 * xs_slstm_backward_tile_r   brings the recurrent matrix into the operand order of the reverse kernel that `split`
 *   names: reads r ([NH,4*dh,dh] in dtype, the forward's layout) and writes r_t (NH*4*dh*dh elements of dtype) as
 *   described at xs_slstm_bwd_args above, so that a caller need not know the tilings.  The reference hands its GEMM R
 *   as it lies and a transpose flag (slstm_backward.cu:308-319); here the kernels keep R transposed in registers or read
 *   it slab by slab, in an order of their own.  Uses NH, dh, dtype, split, r, r_t, stream.  Call it once per change of
 *   the parameters, in front of xs_slstm_backward.
 */
int xs_slstm_backward_tile_r(const xs_slstm_bwd_args *args);

/*
 * Measurement (no counterpart in the reference): one stage of the dependency chain of a timestep of the sequence
 * kernel, run alone for `steps` iterations in which every iteration needs the result of the one before, with the
 * product kernel's instructions, layouts and exchange protocol.  The caller times the call (events on `stream`) at two
 * step counts and divides the difference; the sum of the three stages is the serial bound of a step.
 *   XS_STAGE_EXCHANGE     `members` compute units (8, 16, 32 or 64; one XCD, or with two_xcds != 0 half each on XCDs 0
 *                         and 4 with device-scope stores) publish a 16 x 16 bf16 tile each and poll the group's tile of
 *                         `rows` batch rows until it is complete.  Workspace: 256 + 8 * members * 512 bytes; word 0 is
 *                         nonzero afterwards if a wait ran out (other work held compute units), word 1 the longest wait.
 *                         With rows <= 4 inside one XCD: the layout of the kernel for such tiles, every wave polls the
 *                         whole tile.
 *   XS_STAGE_CONTRACTION  one workgroup: a wave's 8 MFMAs over K = 256 in four chains, their fold, the three row shifts
 *                         that bring a unit's four gates together.
 *   XS_STAGE_GATING       one workgroup: the exponential gating of one element per lane, y rounded to bf16.
 *   XS_STAGE_LAUNCH       `steps` launches of an empty kernel, back to back: the floor of a dependent launch.
 *   XS_STAGE_CHAIN        the three stages as ONE loop in the order of the kernel for tiles of 4 rows (barrier, pause,
 *                         poll, MFMAs, fold, row shifts, gating, publication) on head groups of 16 compute units placed as the product places
 *                         them, as many as the device holds, tiles of `rows` batch rows; constant W.x, no mask, no output
 *                         tensor, none of the product kernel's other waves: what a step costs when only the chain is
 *                         left.  Workspace: 256 + (compute units / 16) * 8 * 16 * 512 bytes; words 0 and 1 as above.
 */
enum { XS_STAGE_EXCHANGE = 0, XS_STAGE_CONTRACTION = 1, XS_STAGE_GATING = 2, XS_STAGE_LAUNCH = 3, XS_STAGE_CHAIN = 4 };
typedef struct xs_measure_args {
  int32_t stage, members, two_xcds, rows, steps;
  void *workspace;
  size_t workspace_bytes;
  void *stream;
} xs_measure_args;

int xs_measure_stage(const xs_measure_args *args);

#ifdef __cplusplus
}
#endif
#endif /* XLSTM_AMD_H */
