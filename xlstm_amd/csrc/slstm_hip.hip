// sLSTM forward / decode engine for MI355X (gfx950, CDNA4): kernels + C ABI.
//
// One persistent launch runs all T timesteps.  A head's recurrent matrix R
// [dh x 4dh] is split by OUTPUT UNIT over G = ceil(dh/16) workgroups ("head
// group"); each workgroup keeps its 64 columns of R (4 gates x 16 units) in
// VGPRs for the whole sequence, computes R.h with MFMA (K split over the 4
// waves, partial sums reduced through LDS), and runs the exponential-gating
// pointwise update with c, n, m in fp32 registers.  The only thing exchanged
// per step is h_t: every workgroup stores its 16 units of h_t into a ring of
// 8 step slots in the workspace (laid out [row tile][member][16 rows][16 units],
// so that polls and stores move whole cache lines) and the other members of the
// group poll those very words until none of them carries the "not written yet"
// pattern the ring was pre-filled with.  One memory round trip per step, no
// flags, no atomics-with-return, no grid barrier.  A decode step (T = 1) is a
// different kernel: a tiled GEMM + gating with no waits between workgroups.
//
// Equations follow xlstm/blocks/slstm/src/vanilla/slstm.py:19-37 with the
// per-element n == 0 rule of xlstm/blocks/slstm/src/cuda/slstm_pointwise.cu:79.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "xlstm_amd.h"

#include "slstm_device_common.h"
#include "slstm_seq_kernel.h"
#include "slstm_seq_roles_kernel.h"
#include "slstm_step_kernel.h"
#include "slstm_step_pipe_kernel.h"
#include "slstm_layer_kernels.h"
#include "slstm_backward_kernels.h"
#include "slstm_backward_quad_kernel.h"
#include "slstm_backward_step_kernel.h"
#include "slstm_step_feed_kernel.h"
#include "slstm_backward_params_kernel.h"
#include "slstm_serial_bound.h"

// ---------------------------------------------------------------------------
// Scratch of the entry point that allocates nothing (xs_slstm_forward_static): status block, placement words and
// exchange ring in an array that every GPU the library runs on holds until the process ends.  In host code the
// array's name is only a stand-in: the device address comes from hipGetSymbolAddress, once per device.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[XS_STATIC_SCRATCH_BYTES];

namespace {

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

constexpr size_t kStatusBytes = 256;
constexpr int kMaxWg = 4096;
constexpr size_t kHeaderBytes = kStatusBytes + (size_t)kMaxWg * 4;  // status block + placement words (multiple of 256)

// upper bound on the elements of the exchange ring [8 slots][head groups][G][rows][16]:
// the head groups of one launch never cover more than B rounded up to 64 rows per head
inline size_t xbuf_elems(int B, int NH, int dh) {
  // (with row tiles of 4 or 8 rows a block still spans 16 rows, hence the factor 4)
  return (size_t)8 * NH * ((dh + 15) / 16) * ((size_t)(B + 63) / 64 * 64) * 16 * 4;
}

typedef void (*SeqKernel)(SeqParams);

template <bool BF16, int NCH, bool FULL>
SeqKernel pick_mt(int MT, bool burst) {
  switch (MT) {
    case 1: return (burst && NCH <= 4) ? slstm_seq_kernel<BF16, NCH, 1, FULL, NCH <= 4> : slstm_seq_kernel<BF16, NCH, 1, FULL, false>;
    case 2: return slstm_seq_kernel<BF16, NCH, 2, FULL, NCH <= 4>;
    default: return nullptr;
  }
}

template <bool BF16, bool FULL>
SeqKernel pick_roles_kernel(int nch) {
  switch (nch) {
    case 1: return slstm_seq_roles_kernel<BF16, 1, FULL>;
    case 2: return slstm_seq_roles_kernel<BF16, 2, FULL>;
    case 4: return slstm_seq_roles_kernel<BF16, 4, FULL>;
    case 8: return slstm_seq_roles_kernel<BF16, 8, FULL>;
    default: return nullptr;
  }
}

template <bool BF16, bool FULL>
SeqKernel pick_kernel(int nch, int MT, bool burst) {
  switch (nch) {
    case 1: return pick_mt<BF16, 1, FULL>(MT, burst);
    case 2: return pick_mt<BF16, 2, FULL>(MT, burst);
    case 4: return pick_mt<BF16, 4, FULL>(MT, burst);
    case 8: return pick_mt<BF16, 8, FULL>(MT, burst);
    default: return nullptr;
  }
}

int validate(const xs_slstm_args *a, bool step, bool own_scratch = false) {
  if (!a) return fail(XS_ERR_NULL, "args is NULL");
  if (a->B < 0 || a->T < 0 || a->NH <= 0 || a->dh <= 0) return fail(XS_ERR_SHAPE, "bad dims B=%d T=%d NH=%d dh=%d", a->B, a->T, a->NH, a->dh);
  if (step && a->T != 1) return fail(XS_ERR_SHAPE, "xs_slstm_step needs T == 1, got %d", a->T);
  if (step && a->r_dtype != a->wx_dtype) return fail(XS_ERR_DTYPE, "xs_slstm_step needs the recurrent matrix in the dtype of wx");
  if (a->wx_dtype != XS_F32 && a->wx_dtype != XS_BF16) return fail(XS_ERR_DTYPE, "wx_dtype %d not supported", a->wx_dtype);
  if (a->r_dtype != XS_F32 && a->r_dtype != XS_BF16) return fail(XS_ERR_DTYPE, "r_dtype %d not supported", a->r_dtype);
  if (a->wx_dtype == XS_F32 && a->r_dtype != XS_F32) return fail(XS_ERR_DTYPE, "float32 wx needs a float32 recurrent matrix");
  if (!a->r || !a->bias || !a->s_out) return fail(XS_ERR_NULL, "r, bias and s_out are required");
  if (a->s0) {  // other workgroups still read s0 while the first ones write s_out
    const uintptr_t lo0 = (uintptr_t)a->s0, lo1 = (uintptr_t)a->s_out;
    const uintptr_t bytes = (uintptr_t)16 * (uintptr_t)a->B * (uintptr_t)a->NH * (uintptr_t)a->dh;
    if (lo0 < lo1 + bytes && lo1 < lo0 + bytes && bytes) return fail(XS_ERR_SHAPE, "s_out must not overlap s0");
  }
  if (a->B > 0 && a->T > 0 && (!a->wx || !a->h_out)) return fail(XS_ERR_NULL, "wx and h_out are required");
  if (a->dh % 8 != 0) return fail(XS_ERR_UNSUPPORTED, "head dim %d is not a multiple of 8", a->dh);
  const long long H = (long long)a->NH * a->dh;
  if (a->B > 0 && a->T > 0) {
    if (a->wx_stride_t < 4 * H || (a->B > 1 && a->wx_stride_b < 4 * H))
      return fail(XS_ERR_SHAPE, "wx strides (%lld, %lld) overlap the innermost 4*H = %lld elements", (long long)a->wx_stride_b, (long long)a->wx_stride_t, 4 * H);
    if (a->reset && a->reset_stride_b < a->T) return fail(XS_ERR_SHAPE, "reset row stride %lld < T", (long long)a->reset_stride_b);
  }
  const uintptr_t al = 16;
  const long long esz = a->wx_dtype == XS_BF16 ? 2 : 4;
  if (a->B > 0 && a->T > 0 &&
      (((uintptr_t)a->wx % al) || ((a->wx_stride_b * esz) % 16) || ((a->wx_stride_t * esz) % 16)))
    return fail(XS_ERR_ALIGN, "wx and its row/step strides must be 16-byte aligned");
  if (((uintptr_t)a->r % al) || ((uintptr_t)a->h_out % al) || ((uintptr_t)a->s0 % al) || ((uintptr_t)a->s_out % al) ||
      ((uintptr_t)a->h_prev % al))
    return fail(XS_ERR_ALIGN, "r, h_out, s0, s_out and h_prev must be 16-byte aligned");
  if (a->h_prev && !a->s0) return fail(XS_ERR_NULL, "h_prev is a copy of the y plane of s0: s0 is required with it");
  if (!own_scratch) {  // (the entry point with a scratch array of its own checks what the launches really need)
    if (!a->workspace || a->workspace_bytes < xs_slstm_workspace_bytes(a->B, a->T, a->NH, a->dh))
      return fail(XS_ERR_WORKSPACE, "workspace missing or smaller than xs_slstm_workspace_bytes()");
    if ((uintptr_t)a->workspace % 256) return fail(XS_ERR_ALIGN, "workspace must be 256-byte aligned");
  }
  return XS_OK;
}

// compute units of the current device (an attribute query: no device synchronisation, cheap per call)
int device_cus() {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
    return -1;
  return cus;
}

// Raises a kernel's dynamic-LDS limit once per (kernel, device); the attribute call is not free and
// a decode loop would otherwise pay it every token.
int ensure_dynamic_lds(const void *kernel, size_t bytes) {
  struct Done { const void *kernel; int device; size_t bytes; };
  static std::mutex mu;
  static Done done[256];  // (a fixed table: nothing on the launch path allocates, host memory included)
  static int ndone = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(XS_ERR_DEVICE, "cannot query the current device");
  std::lock_guard<std::mutex> lock(mu);
  for (int i = 0; i < ndone; ++i)
    if (done[i].kernel == kernel && done[i].device == dev && done[i].bytes >= bytes) return XS_OK;
  const hipError_t ea = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (ea != hipSuccess) return fail(XS_ERR_LAUNCH, "cannot reserve %zu bytes of LDS: %s", bytes, hipGetErrorString(ea));
  if (ndone < 256) done[ndone++] = Done{kernel, dev, bytes};  // (a full table only means the attribute is set again next time)
  return XS_OK;
}

int run_step(const xs_slstm_args *a) {
  hipStream_t stream = (hipStream_t)a->stream;
  const int B = a->B, NH = a->NH, dh = a->dh;
  const bool bf16 = a->wx_dtype == XS_BF16;
  if (B == 0) return XS_OK;
  const int epc = bf16 ? 8 : 4;
  int nch = 1;
  while (nch * 16 * epc < dh) nch *= 2;  // the sequence kernel's K quarters are nch slabs wide
  if (nch > 8) return fail(XS_ERR_UNSUPPORTED, "head dim %d too large for %s operands (max %d)", dh, bf16 ? "bf16" : "fp32", 8 * 16 * epc);
  if ((long long)B * 4 * NH * dh * (bf16 ? 2 : 4) < 32) return fail(XS_ERR_SHAPE, "wx too small");
  StepParams p;
  p.wx = a->wx; p.wx_sb = a->wx_stride_b;
  p.r = a->r; p.r_bf16 = a->r_dtype == XS_BF16;
  p.bias = a->bias; p.s0 = a->s0;
  p.reset = a->reset; p.reset_sb = a->reset_stride_b;
  p.h_out = a->h_out; p.s_out = a->s_out;
  p.status = (xs_slstm_status *)a->workspace;
  p.B = B; p.NH = NH; p.dh = dh;
  p.n_unit_tiles = (dh + 31) / 32;
  p.n_row_tiles = (B + 63) / 64;
  p.spin_limit = a->spin_limit > 0 ? (a->spin_limit < (1ll << 30) ? (int)a->spin_limit : (1 << 30)) : (1 << 22);
  const long long nwg = (long long)NH * p.n_unit_tiles * p.n_row_tiles;
  if (nwg > 0x7FFFFFFF) return fail(XS_ERR_UNSUPPORTED, "too many tiles for one step launch");
  const dim3 grid((unsigned)nwg);
  int nch_log2 = 0;
  while ((1 << nch_log2) < nch) ++nch_log2;
  // steady-state decode: whole tiles, a state, no mask -> the variant without clamping
  const bool full = a->s0 && !a->reset && B % 64 == 0 && dh % 32 == 0 && dh == nch * 16 * epc;
  // slab width in MFMA k-steps: the whole K range when it fits LDS (dh <= 256 bf16 / 128 fp32)
  const int slabch = nch == 1 ? 4 : (nch == 2 ? 8 : 2);
  const int nbuf = slabch >= 4 ? 1 : 2;
  // one slab: eight waves in two roles (operands + MFMA / pointwise operands + gating), the sums of one row tile cross in 16 KiB of LDS
  const bool split = slabch >= 4;
  const size_t lds = (size_t)nbuf * (64 + 128) * (slabch * 64 + 16) + (split ? 4 * 256 * 16 : 0);
  typedef void (*StepKernel)(StepParams, int);
  StepKernel kern;
  const bool hint = full && bf16 && a->h_prev != nullptr;  // operand already in bf16 (h_out of the previous step)
  p.h_prev = hint ? a->h_prev : nullptr;
  // the steady state of bf16 decoding with the previous h at hand, head dim 256: the pipelined kernel (row tiles move
  // through fetch, MFMA, gating and store one behind the other); its buffer offsets are 31-bit
  if (hint && dh == 256 && 63ll * a->wx_stride_b * 2 + 4ll * NH * dh * 2 < (1ll << 31) && 4ll * B * NH * dh * 4 < (1ll << 31)) {
    const size_t plds = (size_t)2 * 64 * 256 + 3 * 64 * 128 + 4 * 64 * 64 + 2 * 128 * 256 + 64;  // h, c/n/m, W.x, R (later the sums), counters
    void (*pk)(StepParams) = slstm_step_pipe_kernel<8>;
    const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(pk), plds);
    if (rc != XS_OK) return rc;
    hipLaunchKernelGGL(pk, grid, dim3(kStepPipeThreads), plds, stream, p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "step kernel launch failed: %s", hipGetErrorString(e));
    return XS_OK;
  }
  // R prepared in slabs (xs_slstm_tile_r_for_steps) and the recurrent operand in the type of the operands: the kernel
  // whose feeder waves bring the slabs to LDS, for the head dims whose K range is walked in slabs
  if (a->r_tiled && slabch == 2 && dh % 64 == 0 && (!bf16 || a->h_prev || !a->s0) && (long long)B * NH * dh * (bf16 ? 2 : 4) < (1ll << 31)) {
    StepFeedParams q;
    q.B = B; q.NH = NH; q.dh = dh; q.nch = nch;
    q.wx = a->wx; q.wx_sb = a->wx_stride_b;
    q.r_tiled = a->r_tiled;
    q.h_prev = a->s0 ? (bf16 ? a->h_prev : (const void *)a->s0) : nullptr;
    q.bias = a->bias; q.s0 = a->s0; q.reset = a->reset; q.reset_sb = a->reset_stride_b;
    q.h_out = a->h_out; q.s_out = a->s_out; q.status = (xs_slstm_status *)a->workspace;
    if (((uintptr_t)a->r_tiled % 16) || ((uintptr_t)q.h_prev % 16)) return fail(XS_ERR_ALIGN, "r_tiled and h_prev must be 16-byte aligned");
    void (*fk)(StepFeedParams) = bf16 ? slstm_step_feed_kernel<true> : slstm_step_feed_kernel<false>;
    const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(fk), (size_t)step_feed_lds_bytes());
    if (rc != XS_OK) return rc;
    const long long fwg = (long long)NH * (dh / 32) * ((B + 63) / 64);
    hipLaunchKernelGGL(fk, dim3((unsigned)fwg), dim3(512), step_feed_lds_bytes(), stream, q);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "step kernel launch failed: %s", hipGetErrorString(e));
    return XS_OK;
  }
#define XS_PICK(BF, SC, SP) (full ? slstm_step_tile_kernel<BF, SC, true, false, SP> : slstm_step_tile_kernel<BF, SC, false, false, SP>)
#define XS_PICK_HINT(SC, SP) (hint ? slstm_step_tile_kernel<true, SC, true, true, SP> : XS_PICK(true, SC, SP))
  if (bf16) kern = slabch == 4 ? XS_PICK_HINT(4, true) : (slabch == 8 ? XS_PICK_HINT(8, true) : XS_PICK_HINT(2, false));
  else kern = slabch == 4 ? XS_PICK(false, 4, true) : (slabch == 8 ? XS_PICK(false, 8, true) : XS_PICK(false, 2, false));
#undef XS_PICK_HINT
#undef XS_PICK
  if (lds > 64 * 1024) {  // the single-slab variant at dh = 256 needs 99 KiB of the 160 KiB of LDS
    const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), lds);
    if (rc != XS_OK) return rc;
  }
  hipLaunchKernelGGL(kern, grid, dim3(split ? 512 : 256), lds, stream, p, nch_log2);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "step kernel launch failed: %s", hipGetErrorString(e));
  return XS_OK;
}

// need != nullptr: launch nothing, only report the bytes of workspace the launches of this call touch
int run_forward(const xs_slstm_args *a, size_t *need = nullptr) {
  hipStream_t stream = (hipStream_t)a->stream;
  const int B = a->B, T = a->T, NH = a->NH, dh = a->dh;
  const long long H = (long long)NH * dh;
  const bool bf16 = a->wx_dtype == XS_BF16;
  const bool dry = need != nullptr;
  if (dry) *need = kHeaderBytes;

  // status block + per-workgroup placement words start clean
  if (!dry)
    hipLaunchKernelGGL(fill_u32_kernel, dim3(4), dim3(256), 0, stream, (uint32_t *)a->workspace,
                       (kStatusBytes + (size_t)kMaxWg * 4) / 4, 0u);
  if (B == 0) return XS_OK;
  if (T == 0) {
    if (dry) return XS_OK;
    const size_t n = (size_t)4 * B * H;
    hipLaunchKernelGGL(copy_state_kernel, dim3(256), dim3(256), 0, stream, a->s0, a->s_out, n);
    return hipGetLastError() == hipSuccess ? XS_OK : fail(XS_ERR_LAUNCH, "state copy launch failed");
  }

  // kernel shape
  const int epc = bf16 ? 8 : 4;
  int nch = 1;
  while (nch * 16 * epc < dh) nch *= 2;  // four waves cover nch * 16 * epc input units
  if (nch > 8) return fail(XS_ERR_UNSUPPORTED, "head dim %d too large for %s operands (max %d)", dh, bf16 ? "bf16" : "fp32", 8 * 16 * epc);
  const int G = (dh + 15) / 16;
  const int cus = device_cus();
  if (cus <= 0) return fail(XS_ERR_DEVICE, "cannot query the device");
  if (G > cus) return fail(XS_ERR_UNSUPPORTED, "ceil(dh/16) = %d workgroups of one head exceed the %d compute units; they must all be resident", G, cus);

  // Every workgroup of a head group waits for the others, so all groups of a launch must be resident at once, and
  // the placement deals groups out per XCD: a group of up to 32 workgroups sits on ONE XCD, a larger even one on
  // an XCD pair, anything else is spread over the device.  What a launch may hold is therefore counted per XCD
  // (one workgroup per compute unit), not per device: with 24 workgroups per group an XCD of 32 compute units
  // holds one group, not 32 * 8 / 24 of the device's.
  const int cus_per_xcd = cus / 8 > 0 ? cus / 8 : 1;
  int capacity;  // head groups per launch
  if (G <= 32) capacity = 8 * (cus_per_xcd / G);
  else if (G <= 64 && G % 2 == 0) capacity = 4 * ((2 * cus_per_xcd) / G);
  else capacity = cus / G;
  if (capacity < 1) return fail(XS_ERR_DEVICE, "a head group of %d workgroups does not fit the %d compute units of this device's XCDs", G, cus);
  // Heads are independent (block-diagonal R): when the groups of all heads do not fit at once, the heads go in
  // several launches, as many per launch as fit.
  const int heads_per_launch = NH < capacity ? NH : capacity;
  int launch_no = 0;
  for (int head0 = 0; head0 < NH; head0 += heads_per_launch) {
  const int NHL = head0 + heads_per_launch <= NH ? heads_per_launch : NH - head0;

  // batch tiling: the fewest rows per workgroup such that all groups of one launch are co-resident
  const int tiles = (B + 15) / 16;
  const int max_groups_per_head = capacity / NHL;  // >= 1
  int MT = 1;
  while (MT < 4 && (tiles + MT - 1) / MT > max_groups_per_head) MT *= 2;
  {
    // The gating waves of the kernel of four row tiles address W.x, the mask and h_out as a scalar base plus a 32-bit
    // offset per lane inside four rows / one row tile.  Where four rows span more than that (sequences of a gigabyte
    // per row), the batch goes through the kernel of two row tiles in more launches instead.
    const long long esz = bf16 ? 2 : 4;
    const bool offsets_fit = 4ll * a->wx_stride_b * esz + 4ll * NH * dh * esz < 0xFFFFFF00ll &&
                             (!a->reset || 4ll * a->reset_stride_b < 0xFFFFFF00ll) && 16ll * NH * dh * esz < (1ll << 31);
    if (MT == 4 && !offsets_fit) MT = 2;
  }
  int rows_per_wg = 16 * MT;
  if (MT == 1) {  // spare compute units: smaller row tiles, smaller exchanges
    for (int r = 4; r < 16; r *= 2)
      if ((B + r - 1) / r <= max_groups_per_head) { rows_per_wg = r; break; }
  }
  const int rows_per_launch = rows_per_wg * max_groups_per_head;

  for (int b0 = 0; b0 < B; b0 += rows_per_launch) {
    const int bend = b0 + rows_per_launch < B ? b0 + rows_per_launch : B;
    // the variant without per-chunk masks: no K tail and, with several row tiles, no missing rows in this launch
    const bool full = dh == nch * 16 * epc && (MT == 1 || (bend - b0) % rows_per_wg == 0);
    // the feeder fetches W.x in bursts where the prefetch waves cannot cover it: row tiles of 8 rows or more
    const bool burst = rows_per_wg >= 8;
    // four row tiles per workgroup: the kernel with MFMA waves and gating waves; one or two: the kernel in which
    // every compute wave does both
    const bool roles = MT == 4;
    SeqKernel kern;
    if (roles)
      kern = bf16 ? (full ? pick_roles_kernel<true, true>(nch) : pick_roles_kernel<true, false>(nch))
                  : (full ? pick_roles_kernel<false, true>(nch) : pick_roles_kernel<false, false>(nch));
    else
      kern = bf16 ? (full ? pick_kernel<true, true>(nch, MT, burst) : pick_kernel<true, false>(nch, MT, burst))
                  : (full ? pick_kernel<false, true>(nch, MT, burst) : pick_kernel<false, false>(nch, MT, burst));
    // row tiles of at most 4 rows, bf16, whole K ranges up to 512: the compute waves split the columns by unit, not K
    const bool quad = bf16 && MT == 1 && rows_per_wg == 4 && full && nch <= 4 && G <= 32;
    if (quad) {
      kern = nch == 1 ? slstm_seq_kernel<true, 1, 1, true, false, false, true>
                      : (nch == 2 ? slstm_seq_kernel<true, 2, 1, true, false, false, true> : slstm_seq_kernel<true, 4, 1, true, false, false, true>);
    }
    if (a->coef_out) {  // a training forward: the same kernel, leaving the backward pass its coefficients
      if (!quad || (dh != 128 && dh != 256) || rows_per_launch < B)
        return fail(XS_ERR_UNSUPPORTED, "coef_out: the call does not run in row tiles of 4 rows of one kernel (bf16, head dim 128 or 256, "
                                        "ceil(B/4) * NH * dh/16 workgroups on the device at once)");
      if (((uintptr_t)a->coef_out % 4)) return fail(XS_ERR_ALIGN, "coef_out must be 4-byte aligned");
      kern = nch == 1 ? slstm_seq_kernel<true, 1, 1, true, false, false, true, true> : slstm_seq_kernel<true, 2, 1, true, false, false, true, true>;
    }
#ifdef XS_SMALL_BATCH_FMA
    // the measured alternative for small batches (see the kernel): only in a library built for that measurement
    if (MT == 1 && rows_per_wg == 4 && nch <= 2 && full) {
      if (bf16) kern = nch == 1 ? slstm_seq_kernel<true, 1, 1, true, false, true> : slstm_seq_kernel<true, 2, 1, true, false, true>;
      else kern = nch == 1 ? slstm_seq_kernel<false, 1, 1, true, false, true> : slstm_seq_kernel<false, 2, 1, true, false, true>;
    }
#endif
    if (!kern) return fail(XS_ERR_UNSUPPORTED, "no kernel for nch=%d MT=%d", nch, MT);
    const int NBT = (bend - b0 + rows_per_wg - 1) / rows_per_wg;
    const int ngroups = NHL * NBT;
    if (dry) {
      const size_t ring = (size_t)kRing * ngroups * G * 16 * MT * 16 * (bf16 ? 2 : 4);
      if (kHeaderBytes + ring > *need) *need = kHeaderBytes + ring;
      continue;
    }
    if (launch_no++ > 0)  // the placement words of the previous launch must not pass for this one's
      hipLaunchKernelGGL(fill_u32_kernel, dim3(4), dim3(256), 0, stream,
                         (uint32_t *)((char *)a->workspace + kStatusBytes), (size_t)kMaxWg, 0u);
    // grid shapes of the three placements the kernel knows: one XCD per group, two XCDs per group, spread
    const int grid = G <= 32 ? 8 * G * ((ngroups + 7) / 8)
                             : ((G <= 64 && G % 2 == 0) ? 8 * (G / 2) * ((ngroups + 3) / 4) : ngroups * G);
    if (grid > kMaxWg) return fail(XS_ERR_UNSUPPORTED, "grid %d too large", grid);
    {  // every word of the exchange ring starts as "not written yet"
      const size_t words = ((size_t)kRing * ngroups * G * 16 * MT * 16 * (bf16 ? 2 : 4) + 3) / 4;
      const int blocks = (int)((words + 256 * 4 - 1) / (256 * 4));
      hipLaunchKernelGGL(fill_u32_kernel, dim3(blocks < 1 ? 1 : (blocks > 1024 ? 1024 : blocks)), dim3(256), 0, stream,
                         (uint32_t *)((char *)a->workspace + kHeaderBytes), words, kSentinel32);
    }
    SeqParams p;
    p.wx = a->wx; p.wx_sb = a->wx_stride_b; p.wx_st = a->wx_stride_t;
    p.r = a->r; p.r_bf16 = a->r_dtype == XS_BF16;
    p.bias = a->bias; p.s0 = a->s0;
    p.reset = a->reset; p.reset_sb = a->reset_stride_b;
    p.h_out = a->h_out; p.s_out = a->s_out;
    p.status = (xs_slstm_status *)a->workspace;
    p.wg_xcc = (uint32_t *)((char *)a->workspace + kStatusBytes);
    p.xbuf = (char *)a->workspace + kHeaderBytes;
    p.B = B; p.T = T; p.NH = NH; p.dh = dh;
    p.b0 = b0; p.bend = bend; p.G = G; p.NBT = NBT; p.rows_per_wg = rows_per_wg;
    p.head0 = head0; p.NHL = NHL;
    p.spin_limit = a->spin_limit;
    p.coef_out = a->coef_out;
    // a prefetch wave issues 2 (bf16) or 4 (fp32) scalar loads per batch row of a tile; 8 per wave and iteration
    // and 16 in all are what the scalar cache sustains, a tile that needs more goes without (prefetch waves that
    // fall behind hold up the barriers: measured 2x slower)
    {
      const int rows_in_tile = rows_per_wg < 16 ? rows_per_wg : 16;
      const int want = (rows_in_tile * (bf16 ? 2 : 4) + 7) / 8;
      p.prefetch = want <= max_prefetch_waves(nch) ? want : 0;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(roles ? kRolesThreads : kThreads + 64 * p.prefetch), 0, stream, p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "sequence kernel launch failed: %s", hipGetErrorString(e));
  }
  }  // heads of one launch
  return XS_OK;
}

// the type of d_wx that a backward call asks for
int d_wx_type(const xs_slstm_bwd_args *a, int *is_bf16) {
  *is_bf16 = 0;
  if (a->d_wx_dtype == XS_F32) return XS_OK;
  if (a->d_wx_dtype != XS_BF16 || a->dtype != XS_BF16) return fail(XS_ERR_DTYPE, "d_wx_dtype must be XS_F32, or XS_BF16 with dtype XS_BF16");
  if (a->d_wx && (((uintptr_t)a->d_wx % 16) || (a->d_wx_stride_b % 8) || (a->d_wx_stride_t % 8)))
    return fail(XS_ERR_ALIGN, "d_wx in bf16 must be 16-byte aligned and its strides multiples of 8 elements");
  *is_bf16 = 1;
  return XS_OK;
}

// ---- backward pass with one launch per step (split == 3): slstm_fwd_walk_kernel and slstm_bwd_step_kernel.  Both keep
// what a launch hands to the next in the caller's `exchange` buffer: the forward walk (a launch per kFwdWalkSteps
// steps) a state [4,B,H] float32 (its y plane holds the y of the initial state in the type of the operands) and R in
// the walk's slabs; the reverse pass two
// sets of gate deltas in the type of the operands, in tiles of 64 rows.
int run_backward_stepwise(const xs_slstm_bwd_args *a, bool prepare) {
  const bool bf16 = a->dtype == XS_BF16;
  const int esz = bf16 ? 2 : 4;
  const int B = a->B, T = a->T, NH = a->NH, dh = a->dh;
  const long long H = (long long)NH * dh, BH = (long long)B * H;
  hipStream_t stream = (hipStream_t)a->stream;
  int dwx_bf16 = 0;
  {
    const int rc = d_wx_type(a, &dwx_bf16);
    if (rc != XS_OK) return rc;
  }
  if (!a->exchange) return fail(XS_ERR_NULL, "exchange is required with one launch per step");
  if (((uintptr_t)a->exchange % 16) || ((uintptr_t)a->coef % 16)) return fail(XS_ERR_ALIGN, "exchange and coef must be 16-byte aligned");
  const long long nwg = (long long)NH * (dh / 32) * ((B + 63) / 64);
  if (nwg > 0x7FFFFFFF) return fail(XS_ERR_UNSUPPORTED, "too many tiles for one step launch");
  if (prepare) {
    if (!a->wx || !a->r || !a->bias || !a->h_out) return fail(XS_ERR_NULL, "wx, r, bias and h_out are required");
    if (a->wx_stride_t < 4 * H || (B > 1 && a->wx_stride_b < 4 * H)) return fail(XS_ERR_SHAPE, "wx strides overlap the innermost 4*H elements");
    if (((uintptr_t)a->wx % 16) || ((a->wx_stride_b * esz) % 16) || ((a->wx_stride_t * esz) % 16))
      return fail(XS_ERR_ALIGN, "wx and its row/step strides must be 16-byte aligned");
    if (((uintptr_t)a->r % 16) || ((uintptr_t)a->s0 % 16) || ((uintptr_t)a->bias % 16) || ((uintptr_t)a->h_out % 16))
      return fail(XS_ERR_ALIGN, "r, s0, bias and h_out must be 16-byte aligned");
    if (BH * esz >= (1ll << 31)) return fail(XS_ERR_UNSUPPORTED, "a step's outputs of 2 GiB or more");
    char *const ws = (char *)a->exchange;
    float *const state = (float *)ws;              // [4,B,H]; the y plane: the y of the initial state in the type of the operands
    char *const r_tiled = ws + 16 * BH;
    void (*init)(const void *, void *, const float *, void *, int, int, int) = bf16 ? slstm_fwd_walk_init_kernel<true> : slstm_fwd_walk_init_kernel<false>;
    hipLaunchKernelGGL(init, dim3(1024), dim3(256), 0, stream, a->r, (void *)r_tiled, a->s0, (void *)state, B, NH, dh);
    FwdWalkParams p;
    p.B = B; p.T = T; p.NH = NH; p.dh = dh;
    p.wx = a->wx; p.wx_sb = a->wx_stride_b; p.wx_st = a->wx_stride_t;
    p.r_tiled = r_tiled; p.bias = a->bias; p.state = state;
    p.h_out = a->h_out; p.h_init = a->s0 ? (const void *)state : nullptr;
    p.reset = a->reset; p.reset_sb = a->reset_stride_b; p.coef = a->coef;
    void (*kern)(FwdWalkParams) = bf16 ? slstm_fwd_walk_kernel<true> : slstm_fwd_walk_kernel<false>;
    {
      const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), (size_t)fwd_walk_lds_bytes());
      if (rc != XS_OK) return rc;
    }
    for (int t = 0; t < T; t += kFwdWalkSteps) {  // (a launch covers kFwdWalkSteps steps: one pass over R for all of them)
      p.t = t;
      p.nsteps = T - t < kFwdWalkSteps ? T - t : kFwdWalkSteps;
      p.state_in = t == 0 ? a->s0 : state;
      hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(kBwdStepThreads), fwd_walk_lds_bytes(), stream, p);
    }
  } else {
    if (!a->d_h || !a->r_t || !a->d_wx || !a->d_s0) return fail(XS_ERR_NULL, "d_h, r_t, d_wx and d_s0 are required");
    if (((uintptr_t)a->r_t % 16) || ((uintptr_t)a->d_h % 16) || ((uintptr_t)a->d_s0 % 16) || ((uintptr_t)a->d_s_final % 16))
      return fail(XS_ERR_ALIGN, "r_t, d_h, d_s0 and d_s_final must be 16-byte aligned");
    if (((uintptr_t)a->d_wx % 16) || (a->d_wx_stride_b % 4) || (a->d_wx_stride_t % 4))
      return fail(XS_ERR_ALIGN, "d_wx and its row/step strides must be 16-byte aligned");
    if (a->d_wx_stride_t < 4 * H || (B > 1 && a->d_wx_stride_b < 4 * H)) return fail(XS_ERR_SHAPE, "d_wx strides overlap the innermost 4*H elements");
    BwdStepParams q;
    q.B = B; q.T = T; q.NH = NH; q.dh = dh;
    q.coef = a->coef; q.d_h = a->d_h; q.d_s_final = a->d_s_final; q.r_t = a->r_t;
    q.reset = a->reset; q.reset_sb = a->reset_stride_b;
    q.d_wx = (float *)a->d_wx; q.d_wx_sb = a->d_wx_stride_b; q.d_wx_st = a->d_wx_stride_t; q.d_wx_bf16 = dwx_bf16; q.d_s0 = a->d_s0;
    q.cut = a->recurrent_cut != 0;
    q.clip = (a->recurrent_clipval > 0.0f && a->recurrent_clipval < __builtin_inff()) ? a->recurrent_clipval : 0.0f;
    char *const deltas[2] = {(char *)a->exchange, (char *)a->exchange + 4ll * ((B + 63) / 64 * 64) * H * esz};  // (tiles of 64 rows)
    void (*kern)(BwdStepParams) = bf16 ? slstm_bwd_step_kernel<true> : slstm_bwd_step_kernel<false>;
    {
      const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), (size_t)bwd_step_lds_bytes());
      if (rc != XS_OK) return rc;
    }
    for (int t = T - 1; t >= -1; --t) {
      q.t = t; q.first = t == T - 1;
      q.delta_out = deltas[(t + 1) & 1];
      q.delta_in = deltas[t & 1];  // (what the launch of step t + 1 wrote)
      hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(kBwdStepThreads), bwd_step_lds_bytes(), stream, q);
    }
  }
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "backward step kernel launch failed: %s", hipGetErrorString(e));
  return XS_OK;
}

// ---- backward pass: the forward walk that leaves the coefficients, and the reverse-time kernel
int run_backward(const xs_slstm_bwd_args *a, bool prepare) {
  if (!a) return fail(XS_ERR_NULL, "args is NULL");
  if (a->B < 0 || a->T < 0 || a->NH <= 0 || a->dh <= 0) return fail(XS_ERR_SHAPE, "bad dims B=%d T=%d NH=%d dh=%d", a->B, a->T, a->NH, a->dh);
  if (a->dtype != XS_F32 && a->dtype != XS_BF16) return fail(XS_ERR_DTYPE, "dtype must be XS_F32 or XS_BF16");
  if (a->split == 3) {
    // one launch per step: the head dims the forward covers beyond those of the persistent kernels, and those next below
    const int lo = a->dtype == XS_BF16 ? 512 : 256;
    if (a->dh % 64 != 0 || a->dh < lo || a->dh > 2 * lo)
      return fail(XS_ERR_UNSUPPORTED, "backward pass with one launch per step: head dim %d not supported (%d to %d in steps of 64)", a->dh, lo, 2 * lo);
  } else if (a->dh != 64 && a->dh != 128 && a->dh != 256 && !(a->dh == 512 && a->dtype == XS_BF16 && (prepare || a->split)))
    return fail(XS_ERR_UNSUPPORTED, "backward pass: head dim %d not supported (64, 128, 256; 512 in bf16 over several compute units; "
                "up to 1024 in bf16 and 512 in float32 with one launch per step, split = 3)", a->dh);
  if (a->B == 0 || a->T == 0) return XS_OK;
  const bool bf16 = a->dtype == XS_BF16;
  const long long H = (long long)a->NH * a->dh;
  int dwx_bf16 = 0;
  if (!prepare) {
    const int rc = d_wx_type(a, &dwx_bf16);
    if (rc != XS_OK) return rc;
  }
  if (!a->coef) return fail(XS_ERR_NULL, "coef is required");
  if (a->reset && a->reset_stride_b < a->T) return fail(XS_ERR_SHAPE, "reset row stride %lld < T", (long long)a->reset_stride_b);
  hipStream_t stream = (hipStream_t)a->stream;
  if (a->split == 3) return run_backward_stepwise(a, prepare);
  if (prepare) {
    if (!a->wx || !a->r || !a->h_out || !a->bias) return fail(XS_ERR_NULL, "wx, r, h_out and bias are required");
    if (a->wx_stride_t < 4 * H || (a->B > 1 && a->wx_stride_b < 4 * H)) return fail(XS_ERR_SHAPE, "wx strides overlap the innermost 4*H elements");
    {  // (W.x and the outputs go straight into LDS in pieces of 16 bytes, R is read in such pieces)
      const long long esz = bf16 ? 2 : 4;
      if (((uintptr_t)a->wx % 16) || ((a->wx_stride_b * esz) % 16) || ((a->wx_stride_t * esz) % 16))
        return fail(XS_ERR_ALIGN, "wx and its row/step strides must be 16-byte aligned");
      if (((uintptr_t)a->r % 16) || ((uintptr_t)a->h_out % 16) || ((uintptr_t)a->s0 % 16) || ((uintptr_t)a->coef % 16))
        return fail(XS_ERR_ALIGN, "r, h_out, s0 and coef must be 16-byte aligned");
    }
    BwdPrepParams p;
    p.B = a->B; p.T = a->T; p.NH = a->NH; p.dh = a->dh;
    p.wx = a->wx; p.wx_sb = a->wx_stride_b; p.wx_st = a->wx_stride_t;
    p.r = a->r; p.h_out = a->h_out; p.bias = a->bias; p.s0 = a->s0; p.reset = a->reset; p.reset_sb = a->reset_stride_b; p.coef = a->coef;
    p.tiled = a->split == 2 ? 4 : (a->split ? 16 : 0);
    // (batch row, head) pairs dealt out over the XCDs, the dh / 64 slices of a pair on one of them
    const long long blocks = ((long long)a->B * a->NH + 7) / 8 * 8 * (a->dh / 64);
    if (blocks > 0x7FFFFFFF) return fail(XS_ERR_UNSUPPORTED, "too many elements for one launch");
    void (*kp)(BwdPrepParams) = nullptr;
    switch (a->dh) {
      case 64: kp = bf16 ? slstm_bwd_prepare_kernel<true, 64> : slstm_bwd_prepare_kernel<false, 64>; break;
      case 128: kp = bf16 ? slstm_bwd_prepare_kernel<true, 128> : slstm_bwd_prepare_kernel<false, 128>; break;
      case 256: kp = bf16 ? slstm_bwd_prepare_kernel<true, 256> : slstm_bwd_prepare_kernel<false, 256>; break;
      default: kp = slstm_bwd_prepare_kernel<true, 512>; break;  // (512 with bf16: checked above)
    }
    const int plds = bwd_prepare_lds_bytes(bf16, a->dh);
    const int rc = ensure_dynamic_lds((const void *)kp, (size_t)plds);
    if (rc != XS_OK) return rc;
    hipLaunchKernelGGL(kp, dim3((unsigned)blocks), dim3(kPrepThreads), plds, stream, p);
  } else {
    if (!a->d_h || !a->r_t || !a->d_wx || !a->d_s0) return fail(XS_ERR_NULL, "d_h, r_t, d_wx and d_s0 are required");
    if (((uintptr_t)a->r_t % 16)) return fail(XS_ERR_ALIGN, "r_t must be 16-byte aligned");
    // (d_h and the coefficients are fetched in pieces of 16 bytes, d_wx is written in pairs of floats)
    if (((uintptr_t)a->d_h % 16) || ((uintptr_t)a->coef % 16)) return fail(XS_ERR_ALIGN, "d_h and coef must be 16-byte aligned");
    if (((uintptr_t)a->d_wx % 8) || (a->d_wx_stride_b % 2) || (a->d_wx_stride_t % 2))
      return fail(XS_ERR_ALIGN, "d_wx must be 8-byte aligned and its strides even");
    if (a->d_wx_stride_t < 4 * H || (a->B > 1 && a->d_wx_stride_b < 4 * H)) return fail(XS_ERR_SHAPE, "d_wx strides overlap the innermost 4*H elements");
    // (0, negative, NaN or infinite: no clipping)
    const float clip = (a->recurrent_clipval > 0.0f && a->recurrent_clipval < __builtin_inff()) ? a->recurrent_clipval : 0.0f;
    if (a->split == 2) {
      // row tiles of 4 rows (bf16, head dims up to 256): four times the workgroups of the 16-row kernel, a shorter step
      if (!bf16 || (a->dh != 64 && a->dh != 128 && a->dh != 256))
        return fail(XS_ERR_UNSUPPORTED, "backward pass with row tiles of 4 rows: bf16 and head dim 64, 128 or 256 (got %d)", a->dh);
      if (!a->exchange || !a->counters) return fail(XS_ERR_NULL, "exchange and counters are required with split");
      if (((uintptr_t)a->exchange % 16)) return fail(XS_ERR_ALIGN, "exchange must be 16-byte aligned");
      if (a->reset && 3 * a->reset_stride_b + a->T >= 0x7FFFFF00ll) return fail(XS_ERR_UNSUPPORTED, "reset rows too far apart for row tiles of 4 rows");
      if (3 * H * 2 + 1024 >= 0x7FFFFF00ll) return fail(XS_ERR_UNSUPPORTED, "rows too long for row tiles of 4 rows");
      const int S = a->dh / 64;
      const long long ngroups = (long long)a->NH * ((a->B + 3) / 4);
      const long long grid = (ngroups + 7) / 8 * 8 * S;
      if (grid > device_cus()) return fail(XS_ERR_DEVICE, "%lld workgroups of the backward pass with row tiles of 4 rows do not fit %d compute units at once", grid, device_cus());
      BwdSplitParams q;
      q.B = a->B; q.T = a->T; q.NH = a->NH; q.dh = a->dh;
      q.coef = a->coef; q.d_h = a->d_h; q.d_s_final = a->d_s_final; q.r_ts = a->r_t;
      q.reset = a->reset; q.reset_sb = a->reset_stride_b;
      q.d_wx = (float *)a->d_wx; q.d_wx_sb = a->d_wx_stride_b; q.d_wx_st = a->d_wx_stride_t; q.d_s0 = a->d_s0;
      q.xch = a->exchange; q.abort_word = a->counters; q.progress = a->counters + 1; q.placement = a->counters + 1 + ngroups;
      q.main_locals = (int)(grid / 8);
      // prefetching workgroups per XCD: one per 40 KB that the XCD's groups read per step (a compute unit draws some
      // 65 GB/s from memory, a step takes about a microsecond), as far as there are compute units left
      int prefetchers = 0;
      {
        const long long groups_per_xcd = (ngroups + 7) / 8;
        const long long step_bytes = groups_per_xcd * S * (kBwdQuadCoefBytes + 4 * 64 * 2);
        long long want = (step_bytes + 39999) / 40000;
        const long long room = (device_cus() - grid) / 8;
        if (want > room) want = room;
        if (want > 8) want = 8;
        prefetchers = (int)(want < 0 ? 0 : want);
      }
      q.spin_limit = a->spin_limit != 0 ? a->spin_limit : kDefaultSpinLimit;
      q.cut = a->recurrent_cut != 0; q.clip = clip;
      const long long n16 = (long long)kBwdRing * ngroups * 4 * 4 * a->dh * 2 / 16;
      hipLaunchKernelGGL(slstm_bwd_arm_kernel, dim3((unsigned)((n16 + 255) / 256 < 1024 ? (n16 + 255) / 256 : 1024)), dim3(256), 0, stream,
                         (uint4 *)a->exchange, n16, a->counters, (int)(1 + 2 * ngroups));
      void (*kq)(BwdSplitParams) = a->dh == 64 ? slstm_bwd_quad_kernel<1> : (a->dh == 128 ? slstm_bwd_quad_kernel<2> : slstm_bwd_quad_kernel<4>);
      if (dwx_bf16) kq = a->dh == 64 ? slstm_bwd_quad_kernel<1, true> : (a->dh == 128 ? slstm_bwd_quad_kernel<2, true> : slstm_bwd_quad_kernel<4, true>);
      const int lds = bwd_quad_lds_bytes();
      {
        const int rc = ensure_dynamic_lds((const void *)kq, (size_t)lds);
        if (rc != XS_OK) return rc;
      }
      hipLaunchKernelGGL(kq, dim3((unsigned)(grid + 8 * prefetchers)), dim3(kBwdQuadThreads), lds, stream, q);
      const hipError_t es = hipGetLastError();
      if (es != hipSuccess) return fail(XS_ERR_LAUNCH, "backward kernel launch failed: %s", hipGetErrorString(es));
      return XS_OK;
    }
    if (a->split) {
      if (a->dh != 64 && a->dh != 128 && a->dh != 256 && !(a->dh == 512 && bf16))
        return fail(XS_ERR_UNSUPPORTED, "backward pass over several compute units per head: head dim %d not supported", a->dh);
      if (!a->exchange || !a->counters) return fail(XS_ERR_NULL, "exchange and counters are required with split");
      const int S = a->dh / 64;
      const long long ngroups = (long long)a->NH * ((a->B + 15) / 16);
      const long long grid = (ngroups + 7) / 8 * 8 * S;
      if (grid > device_cus()) return fail(XS_ERR_DEVICE, "%lld workgroups of the split backward pass do not fit %d compute units at once", grid, device_cus());
      BwdSplitParams q;
      q.B = a->B; q.T = a->T; q.NH = a->NH; q.dh = a->dh;
      q.coef = a->coef; q.d_h = a->d_h; q.d_s_final = a->d_s_final; q.r_ts = a->r_t;
      q.reset = a->reset; q.reset_sb = a->reset_stride_b;
      q.d_wx = (float *)a->d_wx; q.d_wx_sb = a->d_wx_stride_b; q.d_wx_st = a->d_wx_stride_t; q.d_s0 = a->d_s0;
      if (((uintptr_t)a->exchange % 16)) return fail(XS_ERR_ALIGN, "exchange must be 16-byte aligned");
      q.xch = a->exchange; q.abort_word = a->counters; q.progress = a->counters + 1; q.placement = a->counters + 1 + ngroups;
      q.main_locals = (int)(grid / 8);
      // prefetching workgroups per XCD, as for the row tiles of 4 rows below: one per 40 KB that the XCD's groups read
      // per step, as far as there are compute units left
      int prefetchers = 0;
      {
        const long long groups_per_xcd = (ngroups + 7) / 8;
        const long long step_bytes = groups_per_xcd * S * (kBwdCoefBytes + 16 * 64 * (bf16 ? 2 : 4));
        long long want = (step_bytes + 39999) / 40000;
        const long long room = (device_cus() - grid) / 8;
        if (want > room) want = room;
        if (want > 8) want = 8;
        prefetchers = (int)(want < 0 ? 0 : want);
      }
      q.spin_limit = a->spin_limit != 0 ? a->spin_limit : kDefaultSpinLimit;  // (negative: every wait gives up at once)
      q.cut = a->recurrent_cut != 0; q.clip = clip;
      const long long n16 = (long long)kBwdRing * ngroups * 16 * 4 * a->dh * (bf16 ? 2 : 4) / 16;
      hipLaunchKernelGGL(slstm_bwd_arm_kernel, dim3((unsigned)((n16 + 255) / 256 < 1024 ? (n16 + 255) / 256 : 1024)), dim3(256), 0, stream,
                         (uint4 *)a->exchange, n16, a->counters, (int)(1 + 2 * ngroups));
      void (*ks)(BwdSplitParams) = nullptr;
      bool feed = true;  // (feeder waves where the registers allow twelve waves)
      if (a->dh == 64) ks = bf16 ? slstm_bwd_split_kernel<true, 1, true> : slstm_bwd_split_kernel<false, 1, true>;
      else if (a->dh == 128) ks = bf16 ? slstm_bwd_split_kernel<true, 2, true> : slstm_bwd_split_kernel<false, 2, true>;
      else if (a->dh == 256 && bf16) ks = slstm_bwd_split_kernel<true, 4, true>;
      else if (a->dh == 256) { ks = slstm_bwd_split_kernel<false, 4, false>; feed = false; }
      else { ks = slstm_bwd_split_kernel<true, 8, false>; feed = false; }
      if (dwx_bf16) {
        if (a->dh == 64) ks = slstm_bwd_split_kernel<true, 1, true, true>;
        else if (a->dh == 128) ks = slstm_bwd_split_kernel<true, 2, true, true>;
        else if (a->dh == 256) ks = slstm_bwd_split_kernel<true, 4, true, true>;
        else ks = slstm_bwd_split_kernel<true, 8, false, true>;
      }
      const int lds = bwd_split_lds_bytes(feed, bf16);
      {
        const int rc = ensure_dynamic_lds((const void *)ks, (size_t)lds);
        if (rc != XS_OK) return rc;
      }
      hipLaunchKernelGGL(ks, dim3((unsigned)(grid + 8 * prefetchers)), dim3(feed ? 768 : 512), lds, stream, q);
      const hipError_t es = hipGetLastError();
      if (es != hipSuccess) return fail(XS_ERR_LAUNCH, "backward kernel launch failed: %s", hipGetErrorString(es));
      return XS_OK;
    }
    BwdParams p;
    p.B = a->B; p.T = a->T; p.NH = a->NH; p.dh = a->dh;
    p.coef = a->coef; p.d_h = a->d_h; p.d_s_final = a->d_s_final; p.r_t = a->r_t;
    p.reset = a->reset; p.reset_sb = a->reset_stride_b;
    p.d_wx = (float *)a->d_wx; p.d_wx_sb = a->d_wx_stride_b; p.d_wx_st = a->d_wx_stride_t; p.d_wx_bf16 = dwx_bf16; p.d_s0 = a->d_s0;
    p.cut = a->recurrent_cut != 0; p.clip = clip;
    void (*kern)(BwdParams) = nullptr;
    int waves = 0;
#ifndef XS_BWD_NB256
#define XS_BWD_NB256 2
#endif
    if (a->dh == 64) { kern = bf16 ? slstm_bwd_kernel<true, 1, 4> : slstm_bwd_kernel<false, 1, 4>; waves = 4; }
    else if (a->dh == 128) { kern = bf16 ? slstm_bwd_kernel<true, 1, 8> : slstm_bwd_kernel<false, 1, 8>; waves = 8; }
    else { kern = bf16 ? slstm_bwd_kernel<true, XS_BWD_NB256, 16 / XS_BWD_NB256> : slstm_bwd_kernel<false, XS_BWD_NB256, 16 / XS_BWD_NB256>; waves = 16 / XS_BWD_NB256; }
    const int esz = bf16 ? 2 : 4;
    const size_t lds = (size_t)16 * (4 * a->dh + 16 / esz) * esz;  // the delta tile
    if (lds > 64 * 1024) {
      const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), lds);
      if (rc != XS_OK) return rc;
    }
    const long long blocks = (long long)a->NH * ((a->B + 15) / 16);
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(waves * 64), lds, stream, p);
  }
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "backward kernel launch failed: %s", hipGetErrorString(e));
  return XS_OK;
}

// ---- backward pass: R in the operand order of the reverse kernels (xs_slstm_bwd_args::r_t), one thread per element of
// the result: its place says which (gate unit k = g dh + a, input unit d) it holds, and R[h][k][d] is read from the
// forward's layout.  mode = xs_slstm_bwd_args::split.
template <typename T>
__global__ __launch_bounds__(256) void slstm_bwd_tile_r_kernel(const T *r, T *r_t, int NH, int dh, int mode, int epc) {
  const long long per_head = 4ll * dh * dh, n = (long long)NH * per_head;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long o = (long long)blockIdx.x * blockDim.x + threadIdx.x; o < n; o += stride) {
    const int h = (int)(o / per_head);
    long long v = o - (long long)h * per_head;
    int k, d;
    if (mode == 0) {         // [d / 16][k / KC][(k % KC) / EPC][d % 16][k % EPC], KC = 4 EPC
      const int e = (int)(v % epc); v /= epc;
      const int r16 = (int)(v & 15); v >>= 4;
      const int c = (int)(v & 3); v >>= 2;
      const int nkc = 4 * dh / (4 * epc);
      const int kc = (int)(v % nkc); v /= nkc;
      k = (kc * 4 + c) * epc + e;
      d = (int)v * 16 + r16;
    } else if (mode == 3) {  // [d / 32][k / KS][d % 32][k % KS], KS = 32 EPC / 2 (256 bytes)
      const int ks = 16 * epc;
      const int e = (int)(v % ks); v /= ks;
      const int r32 = (int)(v & 31); v >>= 5;
      const int nsl = 4 * dh / ks;
      const int sl = (int)(v % nsl); v /= nsl;
      k = sl * ks + e;
      d = (int)v * 32 + r32;
    } else {                 // [dh / 64][8 waves][k-steps of a wave][4 column blocks][4][16 columns][EPC], K reordered
      const int ksteps = 4 * dh / 8 / (4 * epc);
      const int e = (int)(v % epc); v /= epc;
      const int r16 = (int)(v & 15); v >>= 4;
      const int c = (int)(v & 3); v >>= 2;
      const int cb = (int)(v & 3); v >>= 2;
      const int kst = (int)(v % ksteps); v /= ksteps;
      const int w = (int)(v & 7); v >>= 3;
      const int kk = ((w * ksteps + kst) * 4 + c) * epc + e;  // the kernel's K index
      d = ((int)v * 4 + cb) * 16 + r16;
      if (mode == 1) k = ((kk & 255) >> 6) * dh + (kk >> 8) * 64 + (kk & 63);  // kk = 256 (a / 64) + 64 g + a % 64
      else k = (kk & 3) * dh + (kk >> 2);                                     // kk = 4 a + g
    }
    r_t[o] = r[((long long)h * 4 * dh + k) * dh + d];
  }
}

int run_backward_tile_r(const xs_slstm_bwd_args *a) {
  if (!a) return fail(XS_ERR_NULL, "args is NULL");
  if (a->NH <= 0 || a->dh <= 0) return fail(XS_ERR_SHAPE, "bad dims NH=%d dh=%d", a->NH, a->dh);
  if (a->dtype != XS_F32 && a->dtype != XS_BF16) return fail(XS_ERR_DTYPE, "dtype must be XS_F32 or XS_BF16");
  if (a->split < 0 || a->split > 3) return fail(XS_ERR_UNSUPPORTED, "split = %d", a->split);
  if (!a->r || !a->r_t) return fail(XS_ERR_NULL, "r and r_t are required");
  const bool bf16 = a->dtype == XS_BF16;
  const int epc = bf16 ? 8 : 4;
  if (a->split == 2 && !bf16) return fail(XS_ERR_UNSUPPORTED, "row tiles of 4 rows go with XS_BF16");
  if (a->dh % 64 != 0) return fail(XS_ERR_UNSUPPORTED, "head dim %d is not one of the backward kernels'", a->dh);
  hipStream_t stream = (hipStream_t)a->stream;
  const long long n = 4ll * a->NH * a->dh * a->dh;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  if (bf16) hipLaunchKernelGGL(slstm_bwd_tile_r_kernel<uint16_t>, dim3(blocks), dim3(256), 0, stream, (const uint16_t *)a->r, (uint16_t *)a->r_t, a->NH, a->dh, a->split, epc);
  else hipLaunchKernelGGL(slstm_bwd_tile_r_kernel<uint32_t>, dim3(blocks), dim3(256), 0, stream, (const uint32_t *)a->r, (uint32_t *)a->r_t, a->NH, a->dh, a->split, epc);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "tiling kernel launch failed: %s", hipGetErrorString(e));
  return XS_OK;
}

// ---- backward pass: the gradients of R and the bias from the gate deltas and the forward's outputs
int run_backward_params(const xs_slstm_bwd_args *a) {
  if (!a) return fail(XS_ERR_NULL, "args is NULL");
  if (a->B < 0 || a->T < 0 || a->NH <= 0 || a->dh <= 0) return fail(XS_ERR_SHAPE, "bad dims B=%d T=%d NH=%d dh=%d", a->B, a->T, a->NH, a->dh);
  if (a->dtype != XS_F32 && a->dtype != XS_BF16) return fail(XS_ERR_DTYPE, "dtype must be XS_F32 or XS_BF16");
  if (a->dh % 64 != 0) return fail(XS_ERR_UNSUPPORTED, "backward pass: head dim %d is not a multiple of 64", a->dh);
  if (!a->d_r || !a->d_bias) return fail(XS_ERR_NULL, "d_r and d_bias are required");
  const bool bf16 = a->dtype == XS_BF16;
  const long long H = (long long)a->NH * a->dh;
  int dwx_bf16 = 0;
  {
    const int rc = d_wx_type(a, &dwx_bf16);
    if (rc != XS_OK) return rc;
  }
  hipStream_t stream = (hipStream_t)a->stream;
  const size_t nr = (size_t)a->NH * 4 * a->dh * a->dh, nb = (size_t)4 * H;
  if (((uintptr_t)a->d_r % 4) || ((uintptr_t)a->d_bias % 4)) return fail(XS_ERR_ALIGN, "d_r and d_bias must be 4-byte aligned");
  const bool empty = a->B == 0 || a->T == 0;
  if (!empty) {
    if (!a->d_wx || !a->h_out) return fail(XS_ERR_NULL, "d_wx and h_out are required");
    if (a->d_wx_stride_t < 4 * H || (a->B > 1 && a->d_wx_stride_b < 4 * H)) return fail(XS_ERR_SHAPE, "d_wx strides overlap the innermost 4*H elements");
    if (((uintptr_t)a->d_wx % 16) || (a->d_wx_stride_b % 4) || (a->d_wx_stride_t % 4))
      return fail(XS_ERR_ALIGN, "d_wx and its row/step strides must be 16-byte aligned");
    if (((uintptr_t)a->h_out % 16) || ((uintptr_t)a->s0 % 16)) return fail(XS_ERR_ALIGN, "h_out and s0 must be 16-byte aligned");
    if (a->reset && a->reset_stride_b < a->T) return fail(XS_ERR_SHAPE, "reset row stride %lld < T", (long long)a->reset_stride_b);
    // (a chunk of 32 steps is read through one buffer descriptor: its offsets are 31-bit)
    if (32ll * a->d_wx_stride_t * (dwx_bf16 ? 2 : 4) >= (1ll << 31) || 32ll * a->B * H * (bf16 ? 2 : 4) >= (1ll << 31))
      return fail(XS_ERR_UNSUPPORTED, "32 steps of d_wx or of the outputs span 2 GiB or more: run the batch in slices of rows");
  }
  // (the slices of K are added into the results: they start at zero)
  hipLaunchKernelGGL(fill_u32_kernel, dim3(256), dim3(256), 0, stream, (uint32_t *)a->d_r, nr, 0u);
  hipLaunchKernelGGL(fill_u32_kernel, dim3(4), dim3(256), 0, stream, (uint32_t *)a->d_bias, nb, 0u);
  if (!empty) {
    BwdParamParams p;
    p.B = a->B; p.T = a->T; p.NH = a->NH; p.dh = a->dh;
    p.d_wx = (const float *)a->d_wx; p.d_wx_sb = a->d_wx_stride_b; p.d_wx_st = a->d_wx_stride_t; p.d_wx_bf16 = dwx_bf16;
    p.h_out = a->h_out; p.s0 = a->s0; p.reset = a->reset; p.reset_sb = a->reset_stride_b;
    p.d_r = a->d_r; p.d_bias = a->d_bias;
    p.tchunks = (a->T + kParamKC - 1) / kParamKC;
    const int nt = a->dh % 256 == 0 ? 256 : (a->dh % 128 == 0 ? 128 : 64);
    const int tiles = (4 * a->dh / kParamMT) * (a->dh / nt);
    const long long nchunks = (long long)a->B * p.tchunks;
    // slices of K: enough workgroups for two per compute unit, no slice shorter than four chunks
    const int cus = device_cus() > 0 ? device_cus() : 256;
    long long ks = (2ll * cus + (long long)a->NH * tiles - 1) / ((long long)a->NH * tiles);  // (4 or 8 per compute unit: 10 to 30 % slower)
    // (head, slice) groups are dealt out over the XCDs, group i on XCD i % 8: a multiple of 8 of them keeps every XCD
    // busy (4 heads of 1024 are 512 tiles and one slice each by the rule above: four XCDs idle, twice the time)
    while ((a->NH * ks) % 8 != 0 && a->NH * ks < 64) ++ks;
    if (ks > nchunks / 4) ks = nchunks / 4;
    if (ks < 1) ks = 1;
    p.ksplit = (int)ks;
    const long long groups = (long long)a->NH * ks;
    const long long grid = (groups + 7) / 8 * 8 * tiles;
    if (grid > 0x7FFFFFFF) return fail(XS_ERR_UNSUPPORTED, "too many tiles for one launch");
    void (*kern)(BwdParamParams);
    if (bf16) kern = nt == 256 ? slstm_bwd_param_kernel<true, 256> : (nt == 128 ? slstm_bwd_param_kernel<true, 128> : slstm_bwd_param_kernel<true, 64>);
    else kern = nt == 256 ? slstm_bwd_param_kernel<false, 256> : (nt == 128 ? slstm_bwd_param_kernel<false, 128> : slstm_bwd_param_kernel<false, 64>);
    const size_t lds = (size_t)bwd_param_lds_bytes(bf16, nt);
    if (lds > 64 * 1024) {
      const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), lds);
      if (rc != XS_OK) return rc;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), lds, stream, p);
  }
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "parameter gradient kernel launch failed: %s", hipGetErrorString(e));
  return XS_OK;
}

int run_conv(const xs_conv_args *a) {
  if (!a) return fail(XS_ERR_NULL, "args is NULL");
  if (a->B < 0 || a->T < 0 || a->D <= 0) return fail(XS_ERR_SHAPE, "bad dims B=%d T=%d D=%d", a->B, a->T, a->D);
  if (a->dtype != XS_BF16) return fail(XS_ERR_DTYPE, "xs_causal_conv_silu computes on bf16 tensors only");
  if (a->K < 2 || a->K > 4) return fail(XS_ERR_UNSUPPORTED, "convolution of %d taps not supported (2..4)", a->K);
  if (a->D % 8 != 0) return fail(XS_ERR_UNSUPPORTED, "D = %d is not a multiple of 8", a->D);
  if (a->ring_out && (a->T != 1 || a->reset)) return fail(XS_ERR_SHAPE, "ring_out goes with a single unmasked token (T == 1, no reset mask)");
  if (a->B == 0 || a->T == 0) return XS_OK;
  if (!a->x || !a->weight || !a->out) return fail(XS_ERR_NULL, "x, weight and out are required");
  if ((uintptr_t)a->ring_out % 16) return fail(XS_ERR_ALIGN, "ring_out must be 16-byte aligned");
  if (a->ring_out && a->conv_state) {  // other threads still read the old ring while the first ones write the new one
    const uintptr_t lo0 = (uintptr_t)a->conv_state, lo1 = (uintptr_t)a->ring_out;
    const uintptr_t sb = (uintptr_t)(a->conv_state_stride_b ? a->conv_state_stride_b : (long long)(a->K - 1) * a->D) * 2;
    const uintptr_t n0 = sb * (uintptr_t)(a->B - 1) + (uintptr_t)(a->K - 1) * a->D * 2, n1 = (uintptr_t)a->B * a->K * a->D * 2;
    if (lo0 < lo1 + n1 && lo1 < lo0 + n0) return fail(XS_ERR_SHAPE, "ring_out must not overlap conv_state");
  }
  if (a->x_stride_t < a->D || (a->B > 1 && a->x_stride_b < a->D)) return fail(XS_ERR_SHAPE, "x strides overlap the innermost D elements");
  if (a->reset && a->reset_stride_b < a->T) return fail(XS_ERR_SHAPE, "reset row stride %lld < T", (long long)a->reset_stride_b);
  if (a->conv_state && a->conv_state_stride_b && (a->conv_state_stride_b < (long long)(a->K - 1) * a->D || a->conv_state_stride_b % 8))
    return fail(XS_ERR_SHAPE, "conv_state row stride %lld too small or not 16-byte aligned", (long long)a->conv_state_stride_b);
  if (((uintptr_t)a->x % 16) || ((a->x_stride_b * 2) % 16) || ((a->x_stride_t * 2) % 16) || ((uintptr_t)a->conv_state % 16) ||
      ((uintptr_t)a->weight % 16) || ((uintptr_t)a->bias % 16) || ((uintptr_t)a->out % 16))
    return fail(XS_ERR_ALIGN, "x and its strides, conv_state, weight, bias and out must be 16-byte aligned");
  const long long threads = (long long)a->B * a->T * (a->D / 8);
  const long long blocks = ((threads + 255) / 256 + 7) / 8 * 8;  // a multiple of 8: the kernel deals them out by XCD
  if (blocks > 0x7FFFFFFF) return fail(XS_ERR_UNSUPPORTED, "too many tokens for one launch");
  ConvParams p;
  p.x = (const uint16_t *)a->x; p.x_sb = a->x_stride_b; p.x_st = a->x_stride_t;
  p.state = (const uint16_t *)a->conv_state;
  p.state_sb = a->conv_state_stride_b ? a->conv_state_stride_b : (long long)(a->K - 1) * a->D;
  p.w = (const uint16_t *)a->weight; p.bias = (const uint16_t *)a->bias;
  p.reset = a->reset; p.reset_sb = a->reset_stride_b;
  p.out = (uint16_t *)a->out;
  p.ring_out = (uint16_t *)a->ring_out;
  p.B = a->B; p.T = a->T; p.D = a->D;
  hipStream_t stream = (hipStream_t)a->stream;
  void (*kern)(ConvParams) = a->K == 2 ? causal_conv_silu_kernel<2> : (a->K == 3 ? causal_conv_silu_kernel<3> : causal_conv_silu_kernel<4>);
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), 0, stream, p);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "convolution kernel launch failed: %s", hipGetErrorString(e));
  return XS_OK;
}

int run_gates(const xs_gates_args *a) {
  if (!a) return fail(XS_ERR_NULL, "args is NULL");
  if (a->M < 0 || a->NH <= 0 || a->dh <= 0) return fail(XS_ERR_SHAPE, "bad dims M=%d NH=%d dh=%d", a->M, a->NH, a->dh);
  if (a->dtype != XS_BF16) return fail(XS_ERR_DTYPE, "xs_headwise_gates computes on bf16 tensors only");
  if (a->dh % 64 != 0) return fail(XS_ERR_UNSUPPORTED, "head dim %d is not a multiple of 64", a->dh);
  if (a->M == 0) return XS_OK;
  const long long H = (long long)a->NH * a->dh;
  if (!a->x || !a->x_conv || !a->out || !a->w[0] || !a->w[1] || !a->w[2] || !a->w[3])
    return fail(XS_ERR_NULL, "x, x_conv, the four weights and out are required");
  if (a->x_stride_row < H || a->x_conv_stride_row < H || a->out_stride_row < 4 * H)
    return fail(XS_ERR_SHAPE, "a row stride is smaller than the row");
  if (((uintptr_t)a->x % 16) || ((uintptr_t)a->x_conv % 16) || ((uintptr_t)a->out % 16) || ((a->x_stride_row * 2) % 16) ||
      ((a->x_conv_stride_row * 2) % 16) || ((a->out_stride_row * 2) % 16) || ((uintptr_t)a->w[0] % 16) ||
      ((uintptr_t)a->w[1] % 16) || ((uintptr_t)a->w[2] % 16) || ((uintptr_t)a->w[3] % 16))
    return fail(XS_ERR_ALIGN, "x, x_conv, out, their row strides and the weights must be 16-byte aligned");
  GatesParams p;
  p.x = (const uint16_t *)a->x; p.xc = (const uint16_t *)a->x_conv;
  p.x_sr = a->x_stride_row; p.xc_sr = a->x_conv_stride_row;
  for (int g = 0; g < 4; ++g) p.w[g] = (const uint16_t *)a->w[g];
  p.out = (uint16_t *)a->out; p.out_sr = a->out_stride_row;
  p.M = a->M; p.NH = a->NH; p.dh = a->dh;
  hipStream_t stream = (hipStream_t)a->stream;
  if (a->dh == 128 || a->dh == 256) {
    // weights resident in registers, workgroups walk over token tiles
    const int cus = device_cus();
    if (cus <= 0) return fail(XS_ERR_DEVICE, "cannot query the device");
    const int combos = 2 * a->NH;  // (head, operand)
    const int bm = a->dh == 256 ? 64 : 32;  // tokens per tile: threads / 8
    p.m_tiles = (a->M + bm - 1) / bm;
    p.n_tiles = combos;
    int parts = cus / combos;
    if (parts < 1) parts = 1;
    if (parts > p.m_tiles) parts = p.m_tiles;
    if ((long long)((a->M + 63) / 64) * combos < cus) {
      // too few token tiles to fill the device that way (a decode step): split the units instead
      p.m_tiles = (a->M + 63) / 64;
      p.n_tiles = 4 * a->NH * (a->dh / 64);
      const size_t lds = (size_t)128 * (a->dh * 2 + 16);
      void (*kern)(GatesParams) = a->dh == 256 ? headwise_gates_slab_kernel<4> : headwise_gates_slab_kernel<2>;
      if (lds > 64 * 1024) {
        const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), lds);
        if (rc != XS_OK) return rc;
      }
      hipLaunchKernelGGL(kern, dim3((unsigned)(p.m_tiles * p.n_tiles)), dim3(256), lds, stream, p);
    } else if (a->dh == 256)
      hipLaunchKernelGGL(headwise_gates_resident_kernel<4>, dim3((unsigned)(combos * parts)), dim3(512), 0, stream, p, combos, parts);
    else
      hipLaunchKernelGGL(headwise_gates_resident_kernel<2>, dim3((unsigned)(combos * parts)), dim3(256), 0, stream, p, combos, parts);
  } else {
    // tile: 128 tokens when there are enough of them to fill the compute units, 128 units when dh allows
    const int bn = a->dh % 128 == 0 ? 128 : 64;
    const int bm = a->M >= 4096 ? 128 : 64;
    p.m_tiles = (a->M + bm - 1) / bm;
    p.n_tiles = 4 * a->NH * (a->dh / bn);
    const long long grid = (long long)8 * ((p.m_tiles + 7) / 8) * p.n_tiles;
    if (grid > 0x7FFFFFFF) return fail(XS_ERR_UNSUPPORTED, "too many tiles for one launch");
    void (*kern)(GatesParams) = bm == 128 ? (bn == 128 ? headwise_gates_kernel<128, 128> : headwise_gates_kernel<128, 64>)
                                          : (bn == 128 ? headwise_gates_kernel<64, 128> : headwise_gates_kernel<64, 64>);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), 0, stream, p);
  }
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "gate projection kernel launch failed: %s", hipGetErrorString(e));
  return XS_OK;
}

int run_group_norm(const xs_norm_args *a) {
  if (!a) return fail(XS_ERR_NULL, "args is NULL");
  if (a->B < 0 || a->T < 0 || a->NH <= 0 || a->dh <= 0) return fail(XS_ERR_SHAPE, "bad dims B=%d T=%d NH=%d dh=%d", a->B, a->T, a->NH, a->dh);
  if (a->dtype != XS_BF16) return fail(XS_ERR_DTYPE, "xs_headwise_group_norm computes on bf16 tensors only");
  if (a->dh % 4 != 0 || a->dh > 1024) return fail(XS_ERR_UNSUPPORTED, "head dim %d is not a multiple of 4 up to 1024", a->dh);
  if (a->B == 0 || a->T == 0) return XS_OK;
  if (!a->x || !a->out) return fail(XS_ERR_NULL, "x and out are required");
  if (((uintptr_t)a->x % 8) || ((uintptr_t)a->out % 8) || ((uintptr_t)a->weight % 8) || (a->x_stride_b % 4) || (a->x_stride_t % 4) || (a->x_stride_h % 4))
    return fail(XS_ERR_ALIGN, "x, weight, out and the strides of x must be 8-byte aligned");
  const long long groups = (long long)a->B * a->T * a->NH;
  const long long blocks = (groups + 3) / 4;
  if (blocks > 0x7FFFFFFF) return fail(XS_ERR_UNSUPPORTED, "too many tokens for one launch");
  NormParams p;
  p.x = (const uint16_t *)a->x; p.x_sb = a->x_stride_b; p.x_st = a->x_stride_t; p.x_sh = a->x_stride_h;
  p.weight = (const uint16_t *)a->weight; p.out = (uint16_t *)a->out; p.eps = a->eps;
  p.B = a->B; p.T = a->T; p.NH = a->NH; p.dh = a->dh;
  const int pieces = (a->dh + 255) / 256;
  void (*kern)(NormParams) = pieces == 1 ? headwise_group_norm_kernel<1> : (pieces == 2 ? headwise_group_norm_kernel<2> : headwise_group_norm_kernel<4>);
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)a->stream, p);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "group norm kernel launch failed: %s", hipGetErrorString(e));
  return XS_OK;
}

// ---- measurement: one stage of the dependency chain of a timestep, alone (slstm_serial_bound.h)
int run_stage(const xs_measure_args *a) {
  if (!a) return fail(XS_ERR_NULL, "args is NULL");
  if (a->steps <= 0) return fail(XS_ERR_SHAPE, "steps must be positive");
  hipStream_t stream = (hipStream_t)a->stream;
  StageParams p{};
  p.steps = a->steps;
  p.words = nullptr;
  if (a->stage == XS_STAGE_LAUNCH) {
    for (int i = 0; i < a->steps; ++i) hipLaunchKernelGGL(stage_empty_kernel, dim3(1), dim3(64), 0, stream);
  } else {
    if (!a->workspace || ((uintptr_t)a->workspace % 256)) return fail(XS_ERR_WORKSPACE, "a 256-byte aligned workspace is required");
    p.words = (unsigned int *)a->workspace;
    if (a->stage == XS_STAGE_EXCHANGE) {
      const int G = a->members;
      if (G != 8 && G != 16 && G != 32 && G != 64) return fail(XS_ERR_SHAPE, "members must be 8, 16, 32 or 64");
      if (a->rows < 1 || a->rows > 16) return fail(XS_ERR_SHAPE, "rows must be 1..16");
      const int cus = device_cus();
      const int per_xcd = a->two_xcds ? G / 2 : G;
      if (cus <= 0 || per_xcd > cus / 8) return fail(XS_ERR_DEVICE, "%d workgroups do not fit one XCD of this device at once", per_xcd);
      const size_t ring = (size_t)kRing * G * 512;
      if (a->workspace_bytes < 256 + ring) return fail(XS_ERR_WORKSPACE, "the exchange stage needs %zu bytes of workspace", 256 + ring);
      p.members = G; p.two_xcds = a->two_xcds ? 1 : 0; p.rows = a->rows;
      p.ring = (char *)a->workspace + 256;
      p.spin_limit = kDefaultSpinLimit;
      hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, stream, (uint32_t *)a->workspace, (size_t)64, 0u);
      hipLaunchKernelGGL(fill_u32_kernel, dim3(64), dim3(256), 0, stream, (uint32_t *)p.ring, ring / 4, kSentinel32);
      void (*k)(StageParams) = G == 8 ? stage_exchange_kernel<1> : (G == 16 ? stage_exchange_kernel<2> : (G == 32 ? stage_exchange_kernel<4> : stage_exchange_kernel<8>));
      // tiles of at most 4 rows inside one XCD: the layout and the polls of the kernel for such tiles
      if (a->rows <= 4 && !a->two_xcds && G <= 32)
        k = G == 8 ? stage_exchange_quad_kernel<4> : (G == 16 ? stage_exchange_quad_kernel<8> : stage_exchange_quad_kernel<16>);
      hipLaunchKernelGGL(k, dim3(8 * per_xcd), dim3(256), 0, stream, p);
    } else if (a->stage == XS_STAGE_CHAIN) {
      const int G = 16;  // (head dim 256)
      const int cus = device_cus();
      const int per_xcd = cus > 0 ? (cus / 8) / G : 0;  // head groups per XCD, as many as fit: the product's launch at config 2
      if (per_xcd < 1) return fail(XS_ERR_DEVICE, "a head group of %d workgroups does not fit one XCD of this device", G);
      if (a->rows < 1 || a->rows > 16) return fail(XS_ERR_SHAPE, "rows must be 1..16");
      const size_t ring = (size_t)8 * per_xcd * kRing * G * 512;
      if (a->workspace_bytes < 256 + ring) return fail(XS_ERR_WORKSPACE, "the chain stage needs %zu bytes of workspace", 256 + ring);
      p.members = G; p.two_xcds = 0; p.rows = a->rows;
      p.ring = (char *)a->workspace + 256;
      p.spin_limit = kDefaultSpinLimit;
      hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, stream, (uint32_t *)a->workspace, (size_t)64, 0u);
      hipLaunchKernelGGL(fill_u32_kernel, dim3(64), dim3(256), 0, stream, (uint32_t *)p.ring, ring / 4, kSentinel32);
      hipLaunchKernelGGL(stage_chain_kernel, dim3(8 * per_xcd * G), dim3(256), 0, stream, p);
    } else if (a->stage == XS_STAGE_CONTRACTION) {
      if (a->workspace_bytes < 256) return fail(XS_ERR_WORKSPACE, "256 bytes of workspace are required");
      hipLaunchKernelGGL(stage_contraction_kernel<2>, dim3(1), dim3(256), 0, stream, p);
    } else if (a->stage == XS_STAGE_GATING) {
      if (a->workspace_bytes < 256) return fail(XS_ERR_WORKSPACE, "256 bytes of workspace are required");
      hipLaunchKernelGGL(stage_gating_kernel, dim3(1), dim3(256), 0, stream, p);
    } else {
      return fail(XS_ERR_SHAPE, "unknown stage %d", a->stage);
    }
  }
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "measurement kernel launch failed: %s", hipGetErrorString(e));
  return XS_OK;
}

// host side of the static scratch array: its device address, per device
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void *g_scratch_ptr[kMaxDevices] = {};

int static_scratch(void **out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(XS_ERR_DEVICE, "cannot query the current device");
  if (dev < 0 || dev >= kMaxDevices) return fail(XS_ERR_DEVICE, "device %d beyond the %d this entry point keeps scratch for", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));  // this device's copy of the array
    if (e != hipSuccess || !ptr) return fail(XS_ERR_DEVICE, "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return XS_OK;
}

}  // namespace

extern "C" {

int xs_abi_version(void) { return XS_ABI_VERSION; }

const char *xs_last_error(void) { return g_err; }

size_t xs_slstm_workspace_bytes(int32_t B, int32_t T, int32_t NH, int32_t dh) {
  if (B < 0 || T < 0 || NH <= 0 || dh <= 0) return 0;
  return kHeaderBytes + xbuf_elems(B, NH, dh) * 4;
}

int xs_slstm_forward(const xs_slstm_args *args) {
  g_err[0] = 0;
  const int rc = validate(args, false);
  if (rc != XS_OK) return rc;
  if (args->coef_out) {  // a training forward: is this one of the calls that can leave the coefficients? (launches nothing)
    if (args->T < 1 || args->B < 1) return fail(XS_ERR_UNSUPPORTED, "coef_out: nothing to do for an empty call");
    size_t need = 0;
    const int rd = run_forward(args, &need);
    if (rd != XS_OK) return rd;
    return run_forward(args);  // (also for one token: the step kernels keep no gate values)
  }
  // one token: the tiled step kernel (no waits between compute units, bit-identical to the sequence kernel)
  if (args->T == 1 && args->B > 0 && args->r_dtype == args->wx_dtype) return run_step(args);
  return run_forward(args);
}

int xs_slstm_forward_static(const xs_slstm_args *args) {
  g_err[0] = 0;
  int rc = validate(args, false, true);
  if (rc != XS_OK) return rc;
  if (args->coef_out) return fail(XS_ERR_UNSUPPORTED, "coef_out goes with xs_slstm_forward");
  xs_slstm_args a = *args;
  rc = static_scratch(&a.workspace);
  if (rc != XS_OK) return rc;
  a.workspace_bytes = XS_STATIC_SCRATCH_BYTES;
  if (a.T == 1 && a.B > 0 && a.r_dtype == a.wx_dtype) return run_step(&a);  // (touches the status block only)
  size_t need = 0;
  rc = run_forward(&a, &need);  // what the launches of this call would touch; launches nothing
  if (rc != XS_OK) return rc;
  if (need > (size_t)XS_STATIC_SCRATCH_BYTES)
    return fail(XS_ERR_WORKSPACE, "this call needs %zu bytes of scratch, the static array holds %zu: use xs_slstm_forward with a workspace",
                need, (size_t)XS_STATIC_SCRATCH_BYTES);
  return run_forward(&a);
}

int xs_slstm_step(const xs_slstm_args *args) {
  g_err[0] = 0;
  const int rc = validate(args, true);
  if (rc != XS_OK) return rc;
  if (args->coef_out) return fail(XS_ERR_UNSUPPORTED, "coef_out goes with xs_slstm_forward");
  return run_step(args);
}

int xs_slstm_backward_prepare(const xs_slstm_bwd_args *args) {
  g_err[0] = 0;
  return run_backward(args, true);
}

int xs_slstm_backward(const xs_slstm_bwd_args *args) {
  g_err[0] = 0;
  return run_backward(args, false);
}

int xs_measure_stage(const xs_measure_args *args) {
  g_err[0] = 0;
  return run_stage(args);
}

int xs_slstm_backward_params(const xs_slstm_bwd_args *args) {
  g_err[0] = 0;
  return run_backward_params(args);
}

int xs_slstm_tile_r_for_steps(const void *r, void *r_tiled, int32_t NH, int32_t dh, int32_t dtype, void *stream) {
  g_err[0] = 0;
  if (!r || !r_tiled) return fail(XS_ERR_NULL, "r and r_tiled are required");
  if (NH <= 0 || dh <= 0 || dh % 64 != 0) return fail(XS_ERR_SHAPE, "bad dims NH=%d dh=%d (a multiple of 64)", NH, dh);
  if (dtype != XS_F32 && dtype != XS_BF16) return fail(XS_ERR_DTYPE, "dtype must be XS_F32 or XS_BF16");
  if (((uintptr_t)r % 16) || ((uintptr_t)r_tiled % 16)) return fail(XS_ERR_ALIGN, "r and r_tiled must be 16-byte aligned");
  void (*init)(const void *, void *, const float *, void *, int, int, int) = dtype == XS_BF16 ? slstm_fwd_walk_init_kernel<true> : slstm_fwd_walk_init_kernel<false>;
  hipLaunchKernelGGL(init, dim3(1024), dim3(256), 0, (hipStream_t)stream, r, r_tiled, (const float *)nullptr, (void *)nullptr, 0, NH, dh);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "tiling kernel launch failed: %s", hipGetErrorString(e));
  return XS_OK;
}

int xs_slstm_backward_tile_r(const xs_slstm_bwd_args *args) {
  g_err[0] = 0;
  return run_backward_tile_r(args);
}

int xs_causal_conv_silu(const xs_conv_args *args) {
  g_err[0] = 0;
  return run_conv(args);
}

int xs_headwise_gates(const xs_gates_args *args) {
  g_err[0] = 0;
  return run_gates(args);
}

int xs_headwise_group_norm(const xs_norm_args *args) {
  g_err[0] = 0;
  return run_group_norm(args);
}

}  // extern "C"
