// sLSTM forward / decode engine for MI355X (gfx950, CDNA4): kernels + C ABI.
//
// One persistent launch runs all T timesteps.  A head's recurrent matrix R
// [dh x 4dh] is split by OUTPUT UNIT over G = ceil(dh/16) workgroups ("head
// group"); each workgroup keeps its 64 columns of R (4 gates x 16 units) in
// VGPRs for the whole sequence, computes R.h with MFMA (K split over the 4
// waves, partial sums reduced through LDS), and runs the exponential-gating
// pointwise update with c, n, m in fp32 registers.  The only thing exchanged
// per step is h_t: every workgroup stores its 16 units of h_t straight into
// the output tensor h_out[t] and the other members of the group poll those
// very words until none of them carries the "not written yet" pattern the
// buffer was pre-filled with.  One memory round trip per step, no flags, no
// atomics-with-return, no grid barrier.
//
// Equations follow xlstm/blocks/slstm/src/vanilla/slstm.py:19-37 with the
// per-element n == 0 rule of xlstm/blocks/slstm/src/cuda/slstm_pointwise.cu:79.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "xlstm_amd.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kThreads = 256;           // 4 waves
constexpr int kTileStride = 20;         // floats between unit columns of a partial tile in LDS
constexpr int kTileFloats = 16 * kTileStride;
constexpr uint32_t kSentinel32 = 0xFFFFFFFFu;  // fp32 "not written yet"
constexpr uint32_t kSentinel16 = 0xFFFFu;      // bf16 "not written yet"
constexpr long long kDefaultSpinLimit = 1ll << 22;

struct SeqParams {
  const void *wx;
  long long wx_sb, wx_st;
  const void *r;
  int r_bf16;
  const float *bias;
  const float *s0;
  const unsigned char *reset;
  long long reset_sb;
  void *h_out;
  float *s_out;
  xs_slstm_status *status;
  uint32_t *wg_xcc;
  int B, T, NH, dh;
  int b0, bend;  // batch rows [b0, bend) handled by this launch
  int G;         // workgroups per head group
  int NBT;       // batch tiles (independent groups) per head
  int rows_per_wg;
  long long spin_limit;
};

__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __uint_as_float(b << 16); }

// round-to-nearest-even; NaN becomes the canonical quiet NaN so that the
// "not written yet" pattern 0xFFFF can never be produced by a real value
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0u;
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return float_to_bf16_bits(lo) | (float_to_bf16_bits(hi) << 16);
}

__device__ __forceinline__ bool chunk_has_sentinel_bf16(const uint4 &v) {
  auto bad = [](uint32_t w) { return ((w & 0xFFFFu) == kSentinel16) || ((w >> 16) == kSentinel16); };
  return bad(v.x) || bad(v.y) || bad(v.z) || bad(v.w);
}
__device__ __forceinline__ bool chunk_has_sentinel_f32(const uint4 &v) {
  return v.x == kSentinel32 || v.y == kSentinel32 || v.z == kSentinel32 || v.w == kSentinel32;
}

// 16-byte load that is served beyond this compute unit's vector L1
__device__ __forceinline__ uint4 load16_agent(const void *p) {
  const unsigned long long *q = reinterpret_cast<const unsigned long long *>(p);
  unsigned long long lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  unsigned long long hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  uint4 v;
  v.x = (uint32_t)lo; v.y = (uint32_t)(lo >> 32); v.z = (uint32_t)hi; v.w = (uint32_t)(hi >> 32);
  return v;
}

__device__ __forceinline__ float logsigmoid_f(float x) {
  // min(x,0) - log1p(exp(-|x|))
  return fminf(x, 0.0f) - log1pf(expf(-fabsf(x)));
}
__device__ __forceinline__ float sigmoid_f(float x) {
  if (x >= 0.0f) return 1.0f / (1.0f + expf(-x));
  float e = expf(x);
  return e / (1.0f + e);
}

struct CellState { float y, c, n, m; };

// One exponential-gating update (vanilla/slstm.py:19-37; per-element n == 0 rule).
__device__ __forceinline__ void slstm_pointwise(float iraw, float fraw, float zraw, float oraw, CellState &s) {
  const float lfm = s.m + logsigmoid_f(fraw);
  const float mnew = (s.n == 0.0f) ? iraw : fmaxf(iraw, lfm);
  const float og = sigmoid_f(oraw);
  const float ig = fminf(expf(iraw - mnew), 1.0f);
  const float fg = fminf(expf(lfm - mnew), 1.0f);
  const float cnew = fg * s.c + ig * tanhf(zraw);
  const float nnew = fg * s.n + ig;
  s.y = og * cnew / nnew;
  s.c = cnew; s.n = nnew; s.m = mnew;
}

// ---------------------------------------------------------------------------
// fill kernels (plain vector stores; also used instead of memset so that a
// caller may capture the call in a graph)
// ---------------------------------------------------------------------------
__global__ void fill_u32_kernel(uint32_t *p, size_t n, uint32_t v) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = v;
}

__global__ void copy_state_kernel(const float *s0, float *s_out, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) s_out[i] = s0 ? s0[i] : 0.0f;
}

// ---------------------------------------------------------------------------
// persistent sequence kernel
//   BF16: wx / h_out / MFMA operands are bf16 (fp32 accumulate, fp32 c,n,m);
//         otherwise everything is fp32 (v_mfma_f32_16x16x4_f32).
//   NCH : 16-byte chunks of h each lane holds per batch row; one wave covers
//         NCH*32 (bf16) or NCH*16 (fp32) input units, the four waves 4x that.
//   MT  : 16-row batch tiles handled one after the other by a workgroup.
// ---------------------------------------------------------------------------
template <bool BF16, int NCH, int MT>
__global__ __launch_bounds__(kThreads) void slstm_seq_kernel(SeqParams p) {
  constexpr int EPC = BF16 ? 8 : 4;      // elements per 16-byte chunk
  constexpr int KW = NCH * 4 * EPC;      // input units per wave

  __shared__ float part[2][4][4][kTileFloats];  // [buffer][wave][gate][unit*stride + row]

  // ---- role of this workgroup (XCD-aware: workgroup i is dispatched to XCD i % 8,
  //      a head group takes consecutive slots of ONE XCD so its exchange stays in one L2)
  const int wg = blockIdx.x;
  const int ngroups = p.NH * p.NBT;
  int gi, member;  // head group index, position inside the group
  if (p.G <= 32) {
    const int xcd = wg & 7;
    const int local = wg >> 3;
    const int slot = local / p.G;
    member = local - slot * p.G;
    gi = slot * 8 + xcd;
  } else {  // a group larger than one XCD is spread over all of them
    gi = wg / p.G;
    member = wg - gi * p.G;
  }
  if (threadIdx.x == 0 && p.wg_xcc) {
    // XCC_ID hardware register (id 20), bits [3:0]
    p.wg_xcc[wg] = (gi < ngroups ? 0x100u : 0u) | (uint32_t)(gi << 16) |
                   (__builtin_amdgcn_s_getreg(20 | (3 << 11)) & 0xFu);
  }
  if (gi >= ngroups) return;
  const int head = gi / p.NBT;
  const int bt = gi - head * p.NBT;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int q = lane >> 4;     // lane group: which 16-byte chunk of a 4-chunk K slab
  const int r16 = lane & 15;   // MFMA row (A) / column (B, C)

  const int dh = p.dh;
  const int H = p.NH * dh;
  const int a0 = member * 16;
  const int rowbase = p.b0 + bt * p.rows_per_wg;
  const long long BH = (long long)p.B * H;

  // ---- R slice -> registers (once).  B operand: column n = unit a0 + r16 of gate g,
  //      K chunk c of this wave/lane group.
  uint4 rreg[4][NCH];
  {
    const int a = a0 + r16;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int k0 = wave * KW + c * 4 * EPC + q * EPC;
        uint4 v = make_uint4(0, 0, 0, 0);
        if (a < dh && k0 < dh) {
          const long long off = ((long long)head * 4 * dh + (long long)g * dh + a) * dh + k0;
          if (BF16) {
            if (p.r_bf16) {
              v = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.r) + off);
            } else {
              const float4 lo = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(p.r) + off);
              const float4 hi = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(p.r) + off + 4);
              v.x = pack_bf16x2(lo.x, lo.y); v.y = pack_bf16x2(lo.z, lo.w);
              v.z = pack_bf16x2(hi.x, hi.y); v.w = pack_bf16x2(hi.z, hi.w);
            }
          } else {
            v = *reinterpret_cast<const uint4 *>(reinterpret_cast<const float *>(p.r) + off);
          }
        }
        rreg[g][c] = v;
      }
    }
  }

  // ---- pointwise role: one (batch row, unit) element per thread and batch tile
  const int pb = tid & 15;
  const int pa = tid >> 4;
  const int ua = a0 + pa;
  const bool unit_ok = ua < dh;
  const int col = head * dh + ua;  // column in [.., H]
  float bias_g[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) bias_g[g] = unit_ok ? p.bias[((long long)head * 4 + g) * dh + ua] : 0.0f;

  CellState st[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int brow = rowbase + mt * 16 + pb;
    st[mt] = CellState{0.0f, 0.0f, 0.0f, 0.0f};
    if (p.s0 && unit_ok && brow < p.bend) {
      const long long o = (long long)brow * H + col;
      st[mt].y = p.s0[o]; st[mt].c = p.s0[BH + o]; st[mt].n = p.s0[2 * BH + o]; st[mt].m = p.s0[3 * BH + o];
    }
  }

  const long long spin_limit = p.spin_limit > 0 ? p.spin_limit : kDefaultSpinLimit;
  bool aborted = false;
  uint32_t max_spins = 0;
  int it = 0;  // (t, mt) iteration counter, selects the LDS buffer

  for (int t = 0; t < p.T; ++t) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt, ++it) {
      // ---- 1. A operand: h_{t-1} of batch row (rowbase + mt*16 + r16), this wave's K slab
      const int arow = rowbase + mt * 16 + r16;
      uint4 areg[NCH];
      bool need[NCH];
      const bool row_ok = arow < p.bend;
      // a row that starts a document contributes R.0 = 0 exactly
      const bool row_reset = row_ok && p.reset && p.reset[(long long)arow * p.reset_sb + t] != 0;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int k0 = wave * KW + c * 4 * EPC + q * EPC;
        areg[c] = make_uint4(0, 0, 0, 0);
        need[c] = row_ok && !row_reset && k0 < dh;
      }
      if (t == 0) {
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
          const int k0 = wave * KW + c * 4 * EPC + q * EPC;
          if (need[c] && p.s0) {
            const float *src = p.s0 + (long long)arow * H + head * dh + k0;
            if (BF16) {
              const float4 lo = *reinterpret_cast<const float4 *>(src);
              const float4 hi = *reinterpret_cast<const float4 *>(src + 4);
              areg[c].x = pack_bf16x2(lo.x, lo.y); areg[c].y = pack_bf16x2(lo.z, lo.w);
              areg[c].z = pack_bf16x2(hi.x, hi.y); areg[c].w = pack_bf16x2(hi.z, hi.w);
            } else {
              areg[c] = *reinterpret_cast<const uint4 *>(src);
            }
          }
        }
      } else {
        const char *hprev = reinterpret_cast<const char *>(p.h_out) +
                            ((long long)(t - 1) * BH + (long long)arow * H + head * dh) * (BF16 ? 2 : 4);
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
          const int k0 = wave * KW + c * 4 * EPC + q * EPC;
          if (need[c]) areg[c] = load16_agent(hprev + (long long)k0 * (BF16 ? 2 : 4));
        }
        if (!aborted) {
          uint32_t spins = 0;
          for (;;) {
            bool any_bad = false;
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
              if (need[c]) {
                const bool bad = BF16 ? chunk_has_sentinel_bf16(areg[c]) : chunk_has_sentinel_f32(areg[c]);
                if (bad) {
                  any_bad = true;
                  const int k0 = wave * KW + c * 4 * EPC + q * EPC;
                  areg[c] = load16_agent(hprev + (long long)k0 * (BF16 ? 2 : 4));
                }
              }
            }
            if (!any_bad) break;
            ++spins;
            if ((spins & 1023u) == 0u &&
                __hip_atomic_load(&p.status->aborted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) {
              aborted = true;
              break;
            }
            if ((long long)spins >= spin_limit) {
              aborted = true;
              if (atomicExch(&p.status->aborted, 1u) == 0u) {
                p.status->abort_wg = (uint32_t)wg;
                p.status->abort_step = (uint32_t)t;
              }
              break;
            }
          }
          max_spins = spins > max_spins ? spins : max_spins;
        }
      }

      // ---- 2. partial R.h over this wave's K slab, all four gates
      f32x4 acc[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) acc[g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        if (BF16) {
          const bf16x8 av = __builtin_bit_cast(bf16x8, areg[c]);
#pragma unroll
          for (int g = 0; g < 4; ++g)
            acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, __builtin_bit_cast(bf16x8, rreg[g][c]), acc[g], 0, 0, 0);
        } else {
          const uint32_t aw[4] = {areg[c].x, areg[c].y, areg[c].z, areg[c].w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              const uint32_t bw[4] = {rreg[g][c].x, rreg[g][c].y, rreg[g][c].z, rreg[g][c].w};
              acc[g] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(aw[e]), __uint_as_float(bw[e]), acc[g], 0, 0, 0);
            }
          }
        }
      }

      // ---- 3. partial tiles -> LDS.  C layout: lane holds unit column r16, batch rows 4q..4q+3
      const int buf = it & 1;
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<f32x4 *>(&part[buf][wave][g][r16 * kTileStride + 4 * q]) = acc[g];
      __syncthreads();

      // ---- 4. reduce over waves + exponential gating for element (row pb, unit pa)
      const int brow = rowbase + mt * 16 + pb;
      const bool elem_ok = unit_ok && brow < p.bend;
      float raw[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        // fixed summation order: wave 0 + wave 1 + wave 2 + wave 3
        float ry = part[buf][0][g][pa * kTileStride + pb];
        ry += part[buf][1][g][pa * kTileStride + pb];
        ry += part[buf][2][g][pa * kTileStride + pb];
        ry += part[buf][3][g][pa * kTileStride + pb];
        float wxv = 0.0f;
        if (elem_ok) {
          const long long o = (long long)brow * p.wx_sb + (long long)t * p.wx_st + (long long)g * H + col;
          wxv = BF16 ? bf16_bits_to_float(reinterpret_cast<const uint16_t *>(p.wx)[o])
                     : reinterpret_cast<const float *>(p.wx)[o];
        }
        raw[g] = (wxv + ry) + bias_g[g];
      }
      if (elem_ok) {
        if (p.reset && p.reset[(long long)brow * p.reset_sb + t] != 0) st[mt] = CellState{0.0f, 0.0f, 0.0f, 0.0f};
        slstm_pointwise(raw[0], raw[1], raw[2], raw[3], st[mt]);
        // ---- 5. publish h_t (this IS the output tensor; peers poll these words)
        const long long o = (long long)t * BH + (long long)brow * H + col;
        if (BF16) {
          __hip_atomic_store(reinterpret_cast<uint16_t *>(p.h_out) + o, (uint16_t)float_to_bf16_bits(st[mt].y),
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
          float y = st[mt].y;
          if (y != y) y = __uint_as_float(0x7FC00000u);
          __hip_atomic_store(reinterpret_cast<float *>(p.h_out) + o, y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
  }

  // ---- final state
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int brow = rowbase + mt * 16 + pb;
    if (unit_ok && brow < p.bend) {
      const long long o = (long long)brow * H + col;
      p.s_out[o] = st[mt].y; p.s_out[BH + o] = st[mt].c; p.s_out[2 * BH + o] = st[mt].n; p.s_out[3 * BH + o] = st[mt].m;
    }
  }
  if (lane == 0 && max_spins) atomicMax(&p.status->max_spins, max_spins);
}

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

typedef void (*SeqKernel)(SeqParams);

template <bool BF16, int NCH>
SeqKernel pick_mt(int MT) {
  switch (MT) {
    case 1: return slstm_seq_kernel<BF16, NCH, 1>;
    case 2: return slstm_seq_kernel<BF16, NCH, 2>;
    case 4: return slstm_seq_kernel<BF16, NCH, 4>;
    default: return nullptr;
  }
}

template <bool BF16>
SeqKernel pick_kernel(int nch, int MT) {
  switch (nch) {
    case 1: return pick_mt<BF16, 1>(MT);
    case 2: return pick_mt<BF16, 2>(MT);
    case 4: return pick_mt<BF16, 4>(MT);
    case 8: return pick_mt<BF16, 8>(MT);
    default: return nullptr;
  }
}

int validate(const xs_slstm_args *a, bool step) {
  if (!a) return fail(XS_ERR_NULL, "args is NULL");
  if (a->B < 0 || a->T < 0 || a->NH <= 0 || a->dh <= 0) return fail(XS_ERR_SHAPE, "bad dims B=%d T=%d NH=%d dh=%d", a->B, a->T, a->NH, a->dh);
  if (step && a->T != 1) return fail(XS_ERR_SHAPE, "xs_slstm_step needs T == 1, got %d", a->T);
  if (a->wx_dtype != XS_F32 && a->wx_dtype != XS_BF16) return fail(XS_ERR_DTYPE, "wx_dtype %d not supported", a->wx_dtype);
  if (a->r_dtype != XS_F32 && a->r_dtype != XS_BF16) return fail(XS_ERR_DTYPE, "r_dtype %d not supported", a->r_dtype);
  if (a->wx_dtype == XS_F32 && a->r_dtype != XS_F32) return fail(XS_ERR_DTYPE, "float32 wx needs a float32 recurrent matrix");
  if (!a->r || !a->bias || !a->s_out) return fail(XS_ERR_NULL, "r, bias and s_out are required");
  if (a->B > 0 && a->T > 0 && (!a->wx || !a->h_out)) return fail(XS_ERR_NULL, "wx and h_out are required");
  const int epc = a->wx_dtype == XS_BF16 ? 8 : 4;
  if (a->dh % 8 != 0) return fail(XS_ERR_UNSUPPORTED, "head dim %d is not a multiple of 8", a->dh);
  const long long H = (long long)a->NH * a->dh;
  if (a->B > 0 && a->T > 0) {
    if (a->wx_stride_t < 4 * H || (a->B > 1 && a->wx_stride_b < 4 * H))
      return fail(XS_ERR_SHAPE, "wx strides (%lld, %lld) overlap the innermost 4*H = %lld elements", (long long)a->wx_stride_b, (long long)a->wx_stride_t, 4 * H);
    if (a->reset && a->reset_stride_b < a->T) return fail(XS_ERR_SHAPE, "reset row stride %lld < T", (long long)a->reset_stride_b);
  }
  const uintptr_t al = 16;
  if (((uintptr_t)a->r % al) || ((uintptr_t)a->h_out % al) || ((uintptr_t)a->s0 % al) || ((uintptr_t)a->s_out % al))
    return fail(XS_ERR_ALIGN, "r, h_out, s0 and s_out must be 16-byte aligned");
  if (!a->workspace || a->workspace_bytes < xs_slstm_workspace_bytes(a->B, a->T, a->NH, a->dh))
    return fail(XS_ERR_WORKSPACE, "workspace missing or smaller than xs_slstm_workspace_bytes()");
  if ((uintptr_t)a->workspace % 256) return fail(XS_ERR_ALIGN, "workspace must be 256-byte aligned");
  (void)epc;
  return XS_OK;
}

int device_cus() {
  static int cus = -1;
  if (cus < 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return -1;
    cus = prop.multiProcessorCount;
  }
  return cus;
}

int run_forward(const xs_slstm_args *a) {
  hipStream_t stream = (hipStream_t)a->stream;
  const int B = a->B, T = a->T, NH = a->NH, dh = a->dh;
  const long long H = (long long)NH * dh;
  const bool bf16 = a->wx_dtype == XS_BF16;

  // status block + per-workgroup placement words start clean
  hipLaunchKernelGGL(fill_u32_kernel, dim3(4), dim3(256), 0, stream, (uint32_t *)a->workspace,
                     (kStatusBytes + (size_t)kMaxWg * 4) / 4, 0u);
  if (B == 0) return XS_OK;
  if (T == 0) {
    const size_t n = (size_t)4 * B * H;
    if (a->s0 != a->s_out)
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
  if ((long long)NH * G > cus) return fail(XS_ERR_UNSUPPORTED, "NH * ceil(dh/16) = %lld workgroups exceed the %d compute units; they must all be resident", (long long)NH * G, cus);

  // batch tiling: the fewest rows per workgroup such that all groups of one launch are co-resident
  const int tiles = (B + 15) / 16;
  const int max_groups_per_head = cus / (NH * G);  // >= 1
  int MT = 1;
  while (MT < 4 && (tiles + MT - 1) / MT > max_groups_per_head) MT *= 2;
  const int rows_per_wg = 16 * MT;
  const int rows_per_launch = rows_per_wg * max_groups_per_head;

  SeqKernel kern = bf16 ? pick_kernel<true>(nch, MT) : pick_kernel<false>(nch, MT);
  if (!kern) return fail(XS_ERR_UNSUPPORTED, "no kernel for nch=%d MT=%d", nch, MT);

  // pre-fill h_out with the "not written yet" pattern
  {
    const size_t words = ((size_t)T * B * H * (bf16 ? 2 : 4) + 3) / 4;
    const int blocks = (int)((words + 256 * 8 - 1) / (256 * 8));
    hipLaunchKernelGGL(fill_u32_kernel, dim3(blocks < 1 ? 1 : (blocks > 2048 ? 2048 : blocks)), dim3(256), 0, stream,
                       (uint32_t *)a->h_out, words, kSentinel32);
  }

  uint32_t launches = 0;
  for (int b0 = 0; b0 < B; b0 += rows_per_launch) {
    const int bend = b0 + rows_per_launch < B ? b0 + rows_per_launch : B;
    const int NBT = (bend - b0 + rows_per_wg - 1) / rows_per_wg;
    const int ngroups = NH * NBT;
    const int grid = G <= 32 ? 8 * G * ((ngroups + 7) / 8) : ngroups * G;
    if (grid > kMaxWg) return fail(XS_ERR_UNSUPPORTED, "grid %d too large", grid);
    SeqParams p;
    p.wx = a->wx; p.wx_sb = a->wx_stride_b; p.wx_st = a->wx_stride_t;
    p.r = a->r; p.r_bf16 = a->r_dtype == XS_BF16;
    p.bias = a->bias; p.s0 = a->s0;
    p.reset = a->reset; p.reset_sb = a->reset_stride_b;
    p.h_out = a->h_out; p.s_out = a->s_out;
    p.status = (xs_slstm_status *)a->workspace;
    p.wg_xcc = (uint32_t *)((char *)a->workspace + kStatusBytes);
    p.B = B; p.T = T; p.NH = NH; p.dh = dh;
    p.b0 = b0; p.bend = bend; p.G = G; p.NBT = NBT; p.rows_per_wg = rows_per_wg;
    p.spin_limit = a->spin_limit;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), 0, stream, p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "sequence kernel launch failed: %s", hipGetErrorString(e));
    ++launches;
  }
  (void)launches;
  return XS_OK;
}

}  // namespace

extern "C" {

int xs_abi_version(void) { return XS_ABI_VERSION; }

const char *xs_last_error(void) { return g_err; }

size_t xs_slstm_workspace_bytes(int32_t, int32_t, int32_t, int32_t) { return kStatusBytes + (size_t)kMaxWg * 4; }

int xs_slstm_forward(const xs_slstm_args *args) {
  g_err[0] = 0;
  const int rc = validate(args, false);
  if (rc != XS_OK) return rc;
  return run_forward(args);
}

int xs_slstm_step(const xs_slstm_args *args) {
  g_err[0] = 0;
  const int rc = validate(args, true);
  if (rc != XS_OK) return rc;
  return run_forward(args);
}

}  // extern "C"
