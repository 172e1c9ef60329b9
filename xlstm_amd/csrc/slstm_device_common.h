// Device helpers shared by the sequence kernel and the decode step kernel: vector types, bf16
// conversion, the "not written yet" tests of the exchange ring, the exponential-gating update
// and the fill kernels.  Included by slstm_hip.hip only (one translation unit).
#pragma once

namespace {


typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kThreads = 384;           // 4 compute waves + feeder wave + drainer wave (+ up to 2 prefetch waves)
constexpr int kMaxPrefetchWaves = 2;
constexpr int kTileStride = 20;         // floats between unit columns of a partial tile in LDS
constexpr int kTileFloats = 16 * kTileStride;
constexpr uint32_t kSentinel32 = 0xFFFFFFFFu;  // fp32 "not written yet"
constexpr uint32_t kSentinel16 = 0xFFFFu;      // bf16 "not written yet"
constexpr long long kDefaultSpinLimit = 1ll << 22;
// what the outputs of a call hold after one of its bounded waits ran out (a quiet NaN; as bf16 it is 0x7FC0)
constexpr float kPoison = __builtin_bit_cast(float, 0x7FC00000u);

__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __uint_as_float(b << 16); }

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// two floats -> two bf16, round-to-nearest-even, one v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
}

// one float -> bf16 for the exchange ring.  A NaN whose payload would round to the
// "not written yet" pattern 0xFFFF becomes the canonical quiet NaN, so that pattern can
// never be produced by a value.
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
  const uint32_t b = pack_bf16x2(f, 0.0f) & 0xFFFFu;
  return b == 0xFFFFu ? 0x7FC0u : b;
}

// "Not written yet" tests without branches (they sit on the critical path between the arrival of
// h and the MFMAs).  A mark is the element-wise unsigned maximum of words: the pattern is all
// ones, so an element of the maximum equals the pattern iff one of the inputs did.
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
template <bool BF16>
__device__ __forceinline__ uint32_t mark_join(uint32_t a, uint32_t b) {
  if (BF16)  // v_pk_max_u16
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2_t, a), __builtin_bit_cast(u16x2_t, b)));
  return a > b ? a : b;
}
template <bool BF16>
__device__ __forceinline__ uint32_t chunk_mark(const uint4 &v) {
  return mark_join<BF16>(mark_join<BF16>(v.x, v.y), mark_join<BF16>(v.z, v.w));
}
template <bool BF16>
__device__ __forceinline__ bool mark_has_sentinel(uint32_t m) {
  if (BF16) return (int)((m & 0xFFFFu) == kSentinel16) | (int)(m >= 0xFFFF0000u);
  return m == kSentinel32;
}
__device__ __forceinline__ bool chunk_has_sentinel_bf16(const uint4 &v) { return mark_has_sentinel<true>(chunk_mark<true>(v)); }
__device__ __forceinline__ bool chunk_has_sentinel_f32(const uint4 &v) { return mark_has_sentinel<false>(chunk_mark<false>(v)); }

struct CellState { float y, c, n, m; };

// One exponential-gating update (vanilla/slstm.py:19-37; per-element n == 0 rule), the same code in
// both kernels and both precisions.  exp, log and the reciprocals are the hardware's (v_exp_f32,
// v_log_f32, v_rcp_f32; about 1 ulp each): against the float64 oracle this is as close as the libm
// routines were (h within 5e-7, state within 5e-6 over 2048 steps; the float32 recurrence itself
// sets that floor) at less than half the instructions, and gating is on the critical path of a step.
__device__ __forceinline__ void slstm_pointwise(float iraw, float fraw, float zraw, float oraw, CellState &s) {
  // m + logsigmoid(f).  The argument of the logarithm lies in (1, 2], so the bare v_log_f32 (a base-2 logarithm)
  // serves: __logf would wrap it in a dozen instructions of range handling, all on the critical path of a step.
  const float lfm = s.m + (fminf(fraw, 0.0f) - 0.69314718055994531f * __builtin_amdgcn_logf(1.0f + __expf(-fabsf(fraw))));
  const float mnew = (s.n == 0.0f) ? iraw : fmaxf(iraw, lfm);
  const float og = __builtin_amdgcn_rcpf(1.0f + __expf(-oraw));                      // sigmoid(o)
  const float ig = fminf(__expf(iraw - mnew), 1.0f);
  const float fg = fminf(__expf(lfm - mnew), 1.0f);
  const float tz = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __expf(2.0f * zraw));  // tanh(z)
  const float cnew = fg * s.c + ig * tz;
  const float nnew = fg * s.n + ig;
  s.y = og * cnew * __builtin_amdgcn_rcpf(nnew);
  s.c = cnew; s.n = nnew; s.m = mnew;
}

// The same update with the gate values kept (a training forward leaves the backward pass its coefficients): the same
// expressions in the same order, so the state and y have the bits of slstm_pointwise.
struct GateValues { float og, ig, fg, tz, rn; };
__device__ __forceinline__ void slstm_pointwise_keep(float iraw, float fraw, float zraw, float oraw, CellState &s, GateValues &k) {
  const float lfm = s.m + (fminf(fraw, 0.0f) - 0.69314718055994531f * __builtin_amdgcn_logf(1.0f + __expf(-fabsf(fraw))));
  const float mnew = (s.n == 0.0f) ? iraw : fmaxf(iraw, lfm);
  k.og = __builtin_amdgcn_rcpf(1.0f + __expf(-oraw));
  k.ig = fminf(__expf(iraw - mnew), 1.0f);
  k.fg = fminf(__expf(lfm - mnew), 1.0f);
  k.tz = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __expf(2.0f * zraw));
  const float cnew = k.fg * s.c + k.ig * k.tz;
  const float nnew = k.fg * s.n + k.ig;
  k.rn = __builtin_amdgcn_rcpf(nnew);
  s.y = k.og * cnew * k.rn;
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

}  // namespace
