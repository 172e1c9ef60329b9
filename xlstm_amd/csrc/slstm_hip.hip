// sLSTM forward / decode engine for MI355X (gfx950, CDNA4): kernels + C ABI.
//
// One persistent launch runs all T timesteps.  A head's recurrent matrix R
// [dh x 4dh] is split by OUTPUT UNIT over G = ceil(dh/16) workgroups ("head
// group"); each workgroup keeps its 64 columns of R (4 gates x 16 units) in
// VGPRs for the whole sequence, computes R.h with MFMA (K split over the 4
// waves, partial sums reduced through LDS), and runs the exponential-gating
// pointwise update with c, n, m in fp32 registers.  The only thing exchanged
// per step is h_t: every workgroup stores its 16 units of h_t into a compact
// exchange buffer (one 512-byte / 1-KiB block per workgroup and step, so that
// polls and stores move whole cache lines spread over all L2 channels) and
// the other members of the group poll those very words until none of them
// carries the "not written yet" pattern the buffer was pre-filled with.  One
// memory round trip per step, no flags, no atomics-with-return, no grid barrier.
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
#include <vector>

#include "xlstm_amd.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kThreads = 384;           // 4 compute waves + feeder wave + drainer wave
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
  void *xbuf;    // exchange ring [head group][kRing][row tile][member][16 rows][16 units], pre-filled with the "not written yet" pattern
  int B, T, NH, dh;
  int b0, bend;  // batch rows [b0, bend) handled by this launch
  int G;         // workgroups per head group
  int NBT;       // batch tiles (independent groups) per head
  int rows_per_wg;
  long long spin_limit;
};

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
  const float lfm = s.m + (fminf(fraw, 0.0f) - __logf(1.0f + __expf(-fabsf(fraw))));  // m + logsigmoid(f)
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
//
// Six waves per workgroup, one barrier per (step, tile) iteration shared by all:
//   waves 0-3  compute: poll h_{t-1}, MFMA, reduce through LDS, gating, publish h_t.
//              Their vector-memory queue only ever holds L2-resident traffic (the
//              exchange ring), because vector memory completes in order within a wave
//              and anything slower would sit in front of the latency-critical polls.
//   wave 4     feeder: streams W.x and the reset flags of FUTURE iterations from HBM
//              into an LDS ring (kLookahead iterations in flight).
//   wave 5     drainer: writes h of PAST iterations from an LDS staging ring to the
//              output tensor in HBM.
//
// Exchange ring: kRing slots, slot t % kRing holds h_t as [row tile][member][16 rows][16 units].
// A word is either data or the "not written yet" pattern.  A workgroup re-arms its own
// words of slot (t-2) % kRing after its poll of step t has completed: by then every peer
// has published h_{t-1}, hence has finished reading h_{t-2}.  The re-arm is acknowledged
// before the workgroup's poll of step t+1 completes, i.e. before it publishes h_{t+1};
// a peer polling slot (t-2) % kRing for h_{t-2+kRing} has seen that publication, so it
// can only ever read the pattern or the new data there, never the stale h_{t-2}.
// ---------------------------------------------------------------------------
constexpr int kLookahead = 4;  // iterations of W.x the feeder keeps in flight
constexpr int kRing = 8;       // slots of the exchange ring
constexpr int kPollStagger = 6;  // s_sleep units (64 cycles) between the two polls of a step (measured best of 2 .. 16)

__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint32_t uniform(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

// 16 bytes per lane from a buffer straight into LDS (no registers): lane i's bytes land at
// lds_addr + 16 * i.  Issued as inline assembly on purpose: the compiler then knows nothing of
// these loads, and the waits for them are written by hand with exact counts (s_waitcnt vmcnt).
// rsrc and lds_addr must be wave-uniform values (see uniform()).
__device__ __forceinline__ void lds_direct_load_b128(u32x4_t rsrc, uint32_t lds_addr, int voffset, int soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen sc1 lds"
               :: "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset) : "memory", "m0");
}

template <bool BF16, int NCH, int MT>
__global__ __launch_bounds__(kThreads) void slstm_seq_kernel(SeqParams p) {
  constexpr int EPC = BF16 ? 8 : 4;      // elements per 16-byte chunk
  constexpr int KW = NCH * 4 * EPC;      // input units per wave
  constexpr int ESZ = BF16 ? 2 : 4;
  constexpr int WCH = 16 / EPC;          // 16-byte chunks holding the 16 units of one (row, gate)
  constexpr int ROWS = 16 * MT;          // batch rows of a workgroup
  // With four row tiles a tile is polled by the peers three iterations after it was computed, so
  // it can leave through the drainer wave (two iterations late) and the compute waves issue no
  // stores at all: their waits for poll data then never include a store acknowledgement (loads
  // and stores share one counter and complete out of order with each other).
  constexpr bool kDrainerPublishes = MT >= 4;
  // ... and the polls of a tile are then issued TWO iterations ahead, straight into LDS (dynamic
  // shared memory, [2][compute wave][NCH][lane] 16-byte pieces), because the load latency of a
  // freshly published tile (about 3000 to 5000 cycles) is longer than one iteration.
  constexpr bool kDeepPrefetch = kDrainerPublishes;
  extern __shared__ __attribute__((aligned(16))) unsigned char seq_dyn_lds[];

  __shared__ float part[2][4][4][kTileFloats];  // [buffer][wave][gate][unit*stride + row]
  __shared__ float wxs[2][4][kTileFloats];      // [slot][gate][row*stride + unit]   W.x of one iteration
  __shared__ float hst[4][256];                 // [slot][row*16 + unit]             h on its way to HBM
  __shared__ uint32_t rfl[4][16];               // [slot][row]                       reset flags
  __shared__ uint32_t cross_s;
  __shared__ uint32_t pubflag[4];               // [compute wave] iterations whose h is staged in hst

  // ---- role of this workgroup (XCD-aware: workgroup i is dispatched to XCD i % 8,
  //      a head group takes consecutive slots of ONE XCD so its exchange stays in one L2)
  const int wg = blockIdx.x;
  const int ngroups = p.NH * p.NBT;
  int gi, member;  // head group index, position inside the group
  const bool one_xcd_layout = p.G <= 32;
  if (one_xcd_layout) {
    const int xcd = wg & 7;
    const int local = wg >> 3;
    const int slot = local / p.G;
    member = local - slot * p.G;
    gi = slot * 8 + xcd;
  } else if (p.G <= 64 && (p.G & 1) == 0) {
    // two XCDs per group (workgroup i runs on XCD i % 8): members 0 .. G/2-1 on the even XCD of a
    // pair, the rest on the odd one, so that half of a member's polls stay inside its own L2
    const int xcd = wg & 7;
    const int local = wg >> 3;
    const int half = p.G >> 1;
    const int slot = local / half;
    member = (xcd & 1) * half + (local - slot * half);
    gi = slot * 4 + (xcd >> 1);
  } else {  // larger groups are spread over all XCDs
    gi = wg / p.G;
    member = wg - gi * p.G;
  }
  if (gi >= ngroups) return;
  const int head = gi / p.NBT;
  const int bt = gi - head * p.NBT;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const long long spin_limit = p.spin_limit > 0 ? p.spin_limit : kDefaultSpinLimit;

  // ---- placement handshake: do all members of this head group share one XCD (one L2)?
  //      If so h is published with plain stores (they land in that L2); otherwise with
  //      device-scope stores that are written through to memory.
  if (tid == 0) {
    const uint32_t my_xcc = __builtin_amdgcn_s_getreg(20 | (3 << 11)) & 0xFu;  // XCC_ID, bits [3:0]
    __hip_atomic_store(&p.wg_xcc[wg], 0x80000000u | ((uint32_t)gi << 8) | my_xcc, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    uint32_t cross = one_xcd_layout ? 0u : 1u;
    if (one_xcd_layout) {
      const int xcd = wg & 7;
      const int slot = (wg >> 3) / p.G;
      for (int j = 0; j < p.G; ++j) {
        const int peer = ((slot * p.G + j) << 3) | xcd;
        uint32_t w = 0;
        long long spins = 0;
        while (((w = __hip_atomic_load(&p.wg_xcc[peer], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) & 0x80000000u) == 0u) {
          if (++spins >= spin_limit) {  // a peer never started: the grid is not co-resident
            if (atomicExch(&p.status->aborted, 1u) == 0u) {
              p.status->abort_wg = (uint32_t)wg;
              p.status->abort_step = 0xFFFFFFFFu;
            }
            cross = 1u;
            break;
          }
        }
        if ((w & 0xFu) != my_xcc) cross = 1u;
      }
      if (cross) atomicAdd(&p.status->xcd_mixed, 1u);
    }
    cross_s = cross;
  }
  if (tid < 4) pubflag[tid] = 0u;

  const int dh = p.dh;
  const int H = p.NH * dh;
  const int a0 = member * 16;
  const int rowbase = p.b0 + bt * p.rows_per_wg;
  // rows [rowbase, rend) belong to this workgroup; with few rows per head the batch is cut into
  // tiles of fewer than 16 rows so that more compute units share the work and every exchange is smaller
  const int rend = (rowbase + p.rows_per_wg < p.bend) ? rowbase + p.rows_per_wg : p.bend;
  const long long BH = (long long)p.B * H;
  const int NIT = p.T * MT;
  const int NITpad = (NIT + kLookahead - 1) / kLookahead * kLookahead;  // barriers every wave executes

  // =========================================================================
  // wave 4: feeder.  Every iteration issues exactly WCH + 1 loads (addresses of
  // rows / chunks / steps that do not exist are clamped to ones that do and the
  // result is zeroed), so that the outstanding-load count at each use is exact.
  // =========================================================================
  if (wave == 4) {
    const int fb = lane & 15;  // batch row inside the tile
    const int fg = lane >> 4;  // gate
    uint4 ring[kLookahead][WCH];
    uint32_t fring[kLookahead];
    const char *wxb = reinterpret_cast<const char *>(p.wx);
    const unsigned char *flagb = p.reset ? p.reset : reinterpret_cast<const unsigned char *>(p.wx);
    const long long flag_sb = p.reset ? p.reset_sb : 0;
    const uint32_t flag_on = p.reset ? 0xFFu : 0u;

    auto issue = [&](int it, uint4 (&dst)[WCH], uint32_t &flag) {
      const int itc = it < NIT ? it : NIT - 1;
      const int t = itc / MT;
      const int mt = itc - t * MT;
      const int brow = rowbase + mt * 16 + fb;
      const int browc = brow < rend ? brow : rend - 1;
      const long long e0 = (long long)browc * p.wx_sb + (long long)t * p.wx_st + (long long)fg * H + head * dh + a0;
#pragma unroll
      for (int c = 0; c < WCH; ++c) {
        const int cc = (a0 + c * EPC < dh) ? c : 0;
        dst[c] = *reinterpret_cast<const uint4 *>(wxb + (e0 + cc * EPC) * ESZ);
      }
      flag = flagb[(long long)browc * flag_sb + (p.reset ? t : 0)];
    };
    auto put = [&](int it, const uint4 (&src)[WCH], uint32_t flag_next, int it_next) {
      const int t = it / MT;
      const int mt = it - t * MT;
      const bool row_ok = rowbase + mt * 16 + fb < rend;
      float *dst = &wxs[it & 1][fg][fb * kTileStride];
#pragma unroll
      for (int c = 0; c < WCH; ++c) {
        uint4 v = src[c];
        if (!row_ok || a0 + c * EPC >= dh) v = make_uint4(0, 0, 0, 0);
        if (BF16) {
          f32x4 lo, hi;
          lo[0] = bf16_bits_to_float(v.x & 0xFFFFu); lo[1] = bf16_bits_to_float(v.x >> 16);
          lo[2] = bf16_bits_to_float(v.y & 0xFFFFu); lo[3] = bf16_bits_to_float(v.y >> 16);
          hi[0] = bf16_bits_to_float(v.z & 0xFFFFu); hi[1] = bf16_bits_to_float(v.z >> 16);
          hi[2] = bf16_bits_to_float(v.w & 0xFFFFu); hi[3] = bf16_bits_to_float(v.w >> 16);
          *reinterpret_cast<f32x4 *>(dst + c * 8) = lo;
          *reinterpret_cast<f32x4 *>(dst + c * 8 + 4) = hi;
        } else {
          *reinterpret_cast<uint4 *>(dst + c * 4) = v;
        }
      }
      // reset flag of the NEXT iteration (needed before that iteration's MFMA)
      const int tn = it_next / MT;
      const int mtn = it_next - tn * MT;
      const bool rown_ok = it_next < NIT && rowbase + mtn * 16 + fb < rend;
      if (fg == 0) rfl[it_next & 3][fb] = rown_ok ? (flag_next & flag_on) : 0u;
    };

#pragma unroll
    for (int u = 0; u < kLookahead; ++u) issue(u, ring[u], fring[u]);
    if (fg == 0) rfl[0][fb] = (rowbase + fb < rend) ? (fring[0] & flag_on) : 0u;
    lds_barrier();  // prologue barrier
#ifdef XS_PROFILE
    long long fprof[3] = {0, 0, 0};
    long long ft = clock64();
#define XS_FTICK(i) do { const long long now_ = clock64(); fprof[i] += now_ - ft; ft = now_; } while (0)
#else
#define XS_FTICK(i) do { } while (0)
#endif
    for (int it0 = 0; it0 < NITpad; it0 += kLookahead) {
#pragma unroll
      for (int u = 0; u < kLookahead; ++u) {
        const int it = it0 + u;
        put(it, ring[u], fring[(u + 1) % kLookahead], it + 1);
        XS_FTICK(0);
        issue(it + kLookahead, ring[u], fring[u]);
        XS_FTICK(1);
        lds_barrier();  // barrier #it
        XS_FTICK(2);
      }
    }
    lds_barrier();  // final barrier
#ifdef XS_PROFILE
    if (lane == 0 && member == 0 && gi == 0) {
      long long *dst = reinterpret_cast<long long *>(p.wg_xcc + 4096 - 128) + 4 * 8;
      for (int i = 0; i < 3; ++i) dst[i] = fprof[i];
    }
#endif
    return;
  }

  // =========================================================================
  // wave 5: drainer.  h of iteration it is staged in LDS by the compute waves
  // between barriers #it and #it+1; it is written to HBM two iterations later.
  // =========================================================================
  if (wave == 5) {
    const int drow = lane >> 2;   // batch row inside the tile
    const int dq = lane & 3;      // which 4 of the 16 units
    bool dcross = false;
    auto drain = [&](int it, bool publish) {
      const int t = it / MT;
      const int mt = it - t * MT;
      const int brow = rowbase + mt * 16 + drow;
      const f32x4 v = *reinterpret_cast<const f32x4 *>(&hst[it & 3][drow * 16 + dq * 4]);
      if (kDrainerPublishes && publish) {
        // h_t of this tile goes to the exchange ring from here, and the words of h_{t-2} are re-armed,
        // so the compute waves wait on nothing but their polls.  Every lane stores: words outside
        // the batch or the head belong to this member's block and are never polled.
        constexpr int TB = 16 * 16 * ESZ;  // one member's tile; a ring slot is [row tile][member][16 rows][16 units]
        const int xsl = p.G * MT * TB;
        char *const blk = reinterpret_cast<char *>(p.xbuf) + (long long)gi * kRing * xsl + ((long long)mt * p.G + member) * TB +
                          (drow * 16 + dq * 4) * ESZ;
        unsigned long long *cur = reinterpret_cast<unsigned long long *>(blk + (t % kRing) * xsl);
        unsigned long long *old = reinterpret_cast<unsigned long long *>(blk + ((t + kRing - 2) % kRing) * xsl);
        unsigned long long w0, w1 = 0;
        if (BF16) {
          w0 = (unsigned long long)(float_to_bf16_bits(v[0]) | (float_to_bf16_bits(v[1]) << 16)) |
               ((unsigned long long)(float_to_bf16_bits(v[2]) | (float_to_bf16_bits(v[3]) << 16)) << 32);
        } else {
          w0 = (unsigned long long)__float_as_uint(v[0]) | ((unsigned long long)__float_as_uint(v[1]) << 32);
          w1 = (unsigned long long)__float_as_uint(v[2]) | ((unsigned long long)__float_as_uint(v[3]) << 32);
        }
        if (dcross) {
          __hip_atomic_store(cur, w0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (!BF16) __hip_atomic_store(cur + 1, w1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(old, ~0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (!BF16) __hip_atomic_store(old + 1, ~0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
          cur[0] = w0;
          if (!BF16) cur[1] = w1;
          old[0] = ~0ull;
          if (!BF16) old[1] = ~0ull;
        }
      }
      if (brow < rend && a0 + dq * 4 < dh) {
        const long long o = (long long)t * BH + (long long)brow * H + head * dh + a0 + dq * 4;
        if (BF16) {
          uint2 w;
          w.x = float_to_bf16_bits(v[0]) | (float_to_bf16_bits(v[1]) << 16);
          w.y = float_to_bf16_bits(v[2]) | (float_to_bf16_bits(v[3]) << 16);
          *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(p.h_out) + o) = w;
        } else {
          *reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(p.h_out) + o) = v;
        }
      }
    };
    lds_barrier();  // prologue barrier
    dcross = cross_s != 0u;
#ifdef XS_PROFILE
    long long dprof[2] = {0, 0};
    long long dt = clock64();
#endif
    if (kDrainerPublishes) {
      // iteration j leaves as soon as the four compute waves have staged it (they raise their
      // counters after the LDS write): the peers fetch a tile two iterations before they use it
      bool gave_up = false;
      for (int j = 0; j < NITpad; ++j) {
        lds_barrier();  // barrier #j
#ifdef XS_PROFILE
        { const long long now_ = clock64(); dprof[1] += now_ - dt; dt = now_; }
#endif
        if (j < NIT) {
          long long spins = 0;
          while (!gave_up) {
            const uint32_t want = (uint32_t)j + 1u;
            const uint32_t f0 = __hip_atomic_load(&pubflag[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            const uint32_t f1 = __hip_atomic_load(&pubflag[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            const uint32_t f2 = __hip_atomic_load(&pubflag[2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            const uint32_t f3 = __hip_atomic_load(&pubflag[3], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (f0 >= want && f1 >= want && f2 >= want && f3 >= want) break;
            __builtin_amdgcn_s_sleep(1);
            if (++spins >= spin_limit) {  // cannot happen while the compute waves run; never wait forever
              gave_up = true;
              if (lane == 0 && atomicExch(&p.status->aborted, 1u) == 0u) {
                p.status->abort_wg = (uint32_t)wg;
                p.status->abort_step = (uint32_t)(j / MT);
              }
            }
          }
          drain(j, true);
        }
#ifdef XS_PROFILE
        { const long long now_ = clock64(); dprof[0] += now_ - dt; dt = now_; }
#endif
      }
      lds_barrier();  // final barrier
    } else {
    for (int j = 0; j < NITpad; ++j) {
      if (j >= 2 && j - 2 < NIT) drain(j - 2, true);
#ifdef XS_PROFILE
      { const long long now_ = clock64(); dprof[0] += now_ - dt; dt = now_; }
#endif
      lds_barrier();  // barrier #j
#ifdef XS_PROFILE
      { const long long now_ = clock64(); dprof[1] += now_ - dt; dt = now_; }
#endif
    }
    lds_barrier();  // final barrier
    for (int it = (NITpad >= 2 ? NITpad - 2 : 0); it < NIT; ++it) drain(it, false);
    }
#ifdef XS_PROFILE
    if (lane == 0 && member == 0 && gi == 0) {
      long long *dst = reinterpret_cast<long long *>(p.wg_xcc + 4096 - 128) + 5 * 8;
      for (int i = 0; i < 2; ++i) dst[i] = dprof[i];
    }
#endif
    return;
  }

  // =========================================================================
  // waves 0-3: compute
  // =========================================================================
  __builtin_amdgcn_s_setprio(3);
  const int q = lane >> 4;     // lane group: which 16-byte chunk of a 4-chunk K slab
  const int r16 = lane & 15;   // MFMA row (A) / column (B, C)

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
  const int pa = tid & 15;  // unit inside the workgroup's 16
  const int pb = tid >> 4;  // batch row inside the tile
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
    if (p.s0 && unit_ok && brow < rend) {
      const long long o = (long long)brow * H + col;
      st[mt].y = p.s0[o]; st[mt].c = p.s0[BH + o]; st[mt].n = p.s0[2 * BH + o]; st[mt].m = p.s0[3 * BH + o];
    }
  }

  bool aborted = false;
  uint32_t max_spins = 0;
  int it = 0;  // (t, mt) iteration counter, selects the LDS buffers
#ifdef XS_PROFILE
  long long prof[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#define XS_TICK(i) do { const long long now_ = clock64(); prof[i] += now_ - tick_; tick_ = now_; } while (0)
  long long tick_ = clock64();
#else
#define XS_TICK(i) do { } while (0)
#endif

  lds_barrier();  // prologue barrier: reset flags of iteration 0 and the placement verdict are in LDS
  const bool cross = cross_s != 0u;

  // exchange ring layout [head group][slot][member][ROWS][16 units]: what a group publishes in
  // one step is contiguous (512 B per member for bf16, one tile), which spreads a step's polls
  // over all L2 channels (measured: lines 256 B .. 2 KiB apart are served 1.5x faster than
  // lines 4 KiB or more apart)
  constexpr int XBLOCK = ROWS * 16 * ESZ;            // bytes one member publishes per step
  constexpr int XTILE = 16 * 16 * ESZ;               // ... per row tile
  const int xslot = p.G * XBLOCK;                    // bytes one group publishes per step
  // a slot is laid out [row tile][member][16 rows][16 units]: what the group publishes for one row
  // tile is contiguous, so the polls of an iteration spread over all L2 channels
  char *const xbase = reinterpret_cast<char *>(p.xbuf) + (long long)gi * kRing * xslot;

  // With several row tiles per workgroup (MT > 1) the polls of the NEXT (t, mt) iteration are
  // issued right after the MFMAs of the current one have consumed the operand registers: the
  // peers published that tile MT - 1 iterations ago, so the data is there and the exchange
  // latency hides behind barrier, gating and publish.  The completion check, the re-arm and
  // their order are unchanged.  (With MT == 1 the tile is published only at the end of the
  // peers' current iteration, so there is nothing to fetch early.)
  uint4 areg[NCH];
  bool prefetched = false;
  // poll address of chunk c of row tile mt = per-lane part (one register) + a compile-time constant:
  // unit k of row r of row tile mt lives at [mt][member k/16][r][k%16]
  const int xlane = ((wave * KW + q * EPC) >> 4) * XTILE + (r16 * 16 + ((q * EPC) & 15)) * ESZ;
  const int xtile_stride = p.G * XTILE;
  auto xconst = [&](int c, int mt_) { return ((c * 4 * EPC) >> 4) * XTILE + mt_ * xtile_stride; };
  auto dma_slot = [&](int itx, int c) { return seq_dyn_lds + ((((itx & 1) * 4 + wave) * NCH + c) << 10); };
  for (int t = 0; t < p.T; ++t) {
    // all 16-byte polls of this step go through one buffer descriptor based at slot (t-1)
    // (the descriptor ends with the slot: a chunk past the last member reads zeros)
    const __amdgpu_buffer_rsrc_t hrs = __builtin_amdgcn_make_buffer_rsrc(
        xbase + ((t + kRing - 1) % kRing) * xslot, 0, xslot, 0x00020000);
    char *const hcur = xbase + (t % kRing) * xslot;
    char *const hold = xbase + ((t + kRing - 2) % kRing) * xslot;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt, ++it) {
      // ---- 1. A operand: h_{t-1} of batch row (rowbase + mt*16 + r16), this wave's K slab
      XS_TICK(5);
      const int arow = rowbase + mt * 16 + r16;
      bool need[NCH];
      const bool row_ok = arow < rend;
      const bool row_reset = rfl[it & 3][r16] != 0u;  // a row that starts a document contributes R.0 = 0 exactly
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int k0 = wave * KW + c * 4 * EPC + q * EPC;
        if (!(MT > 1 && prefetched)) areg[c] = make_uint4(0, 0, 0, 0);
        need[c] = row_ok && k0 < dh;
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
        if (kDeepPrefetch) {
          // this tile was requested two iterations ago; the only younger requests are the NCH of the next tile
#ifdef XS_PROFILE
          const long long w0_ = clock64();
#endif
          if (it + 1 < NIT) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NCH) : "memory");
          else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#ifdef XS_PROFILE
          prof[7] += clock64() - w0_;
#endif
#pragma unroll
          for (int c = 0; c < NCH; ++c) areg[c] = *reinterpret_cast<const uint4 *>(dma_slot(it, c) + lane * 16);
        } else if (MT == 1) {
          // Two polls in flight, about half a round trip apart (kPollStagger), re-issued alternately:
          // a poll returns every ~300 cycles instead of every ~600, which halves both the wait for h
          // and the skew between the four waves at the barrier.  Lanes whose batch row does not exist
          // ask for an offset past the descriptor's end: zeros, no memory traffic, so the doubled poll
          // rate stays far below what a compute unit can pull from the L2.  The decisions are
          // wave-uniform (ballot) so that the waits keep exact counts.
          const int xl = row_ok ? xlane : 0x7FFFFF00;
          uint4 breg[NCH];
#pragma unroll
          for (int c = 0; c < NCH; ++c)
            areg[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(hrs, xl, xconst(c, mt), 16));
          __builtin_amdgcn_s_sleep(kPollStagger);
#pragma unroll
          for (int c = 0; c < NCH; ++c)
            breg[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(hrs, xl, xconst(c, mt), 16));
          if (!aborted) {
            uint32_t spins = 0;
            for (;;) {
              uint32_t ma = 0u;
#pragma unroll
              for (int c = 0; c < NCH; ++c) ma = mark_join<BF16>(ma, need[c] ? chunk_mark<BF16>(areg[c]) : 0u);
              if (__builtin_amdgcn_ballot_w64(mark_has_sentinel<BF16>(ma)) == 0ull) break;
#pragma unroll
              for (int c = 0; c < NCH; ++c)
                areg[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(hrs, xl, xconst(c, mt), 16));
              uint32_t mb = 0u;
#pragma unroll
              for (int c = 0; c < NCH; ++c) mb = mark_join<BF16>(mb, need[c] ? chunk_mark<BF16>(breg[c]) : 0u);
              if (__builtin_amdgcn_ballot_w64(mark_has_sentinel<BF16>(mb)) == 0ull) {
#pragma unroll
                for (int c = 0; c < NCH; ++c) areg[c] = breg[c];
                break;
              }
#pragma unroll
              for (int c = 0; c < NCH; ++c)
                breg[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(hrs, xl, xconst(c, mt), 16));
              spins += 2;
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
#ifdef XS_PROFILE
            prof[6] += spins;
#endif
          }
        } else {
          // every lane loads every chunk (no divergent branches on the way to the MFMAs); what is
          // not needed is left out of the test below and zeroed afterwards
          if (!(MT > 1 && prefetched)) {
#pragma unroll
            for (int c = 0; c < NCH; ++c)
              areg[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(hrs, xlane, xconst(c, mt), 16));
          }
        }
        // (tiles fetched ahead through LDS are checked once outside the loop: inside it the wave
        // waits for ALL of its outstanding loads, the next tile's requests included)
        // first look at everything at once: one mark over all chunks this lane needs
        uint32_t mark = 0u;
#pragma unroll
        for (int c = 0; c < NCH; ++c) mark = mark_join<BF16>(mark, need[c] ? chunk_mark<BF16>(areg[c]) : 0u);
        if (!aborted && mark_has_sentinel<BF16>(mark)) {
          uint32_t spins = 0;
          for (;;) {
            bool any_bad = false;
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
              if (need[c]) {
                const bool bad = BF16 ? chunk_has_sentinel_bf16(areg[c]) : chunk_has_sentinel_f32(areg[c]);
                if (bad) {
                  any_bad = true;
                  areg[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(hrs, xlane, xconst(c, mt), 16));
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
#ifdef XS_PROFILE
          prof[6] += spins;
#endif
        }
      }
      // (a whole wave rarely has anything to clear: one uniform branch instead of 4 selects per chunk)
      bool clear_any = row_reset;
#pragma unroll
      for (int c = 0; c < NCH; ++c) clear_any |= !need[c];
      if (__builtin_amdgcn_ballot_w64(clear_any) != 0ull) {
#pragma unroll
        for (int c = 0; c < NCH; ++c)
          if (row_reset || !need[c]) areg[c] = make_uint4(0, 0, 0, 0);
      }

      // ---- 2. partial R.h over this wave's K slab, all four gates
      XS_TICK(0);
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

      if (kDeepPrefetch) {
        // request the tile of iteration it + 2 (its LDS slot is the one just read); step 0 takes its
        // operand from s0.  A chunk past the last member reads zeros (the descriptor ends with the slot).
        const int nmt = (mt + 2) % MT;
        const int nt = t + (mt + 2 >= MT ? 1 : 0);
        if (nt >= 1 && nt < p.T) {
          const unsigned long long sb = reinterpret_cast<unsigned long long>(xbase + ((nt + kRing - 1) % kRing) * xslot);
          const u32x4_t rs = {uniform((uint32_t)sb), uniform((uint32_t)(sb >> 32) & 0xFFFFu), uniform((uint32_t)xslot), 0x00020000u};
          const uint32_t lds0 = uniform((uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)dma_slot(it, 0)));
#pragma unroll
          for (int c = 0; c < NCH; ++c) lds_direct_load_b128(rs, lds0 + (c << 10), xlane, xconst(c, nmt));
        }
      } else if (MT > 1) {
        // early polls of the next iteration's tile (see above); step 0 takes its operand from s0
        const int nmt = (mt + 1) % MT;
        const int nt = t + (mt + 1 == MT ? 1 : 0);
        prefetched = nt >= 1 && nt < p.T;
        if (prefetched) {
          // unconditional loads (a select on the loaded value would make the wave wait for it right
          // here); the descriptor ends with the slot, so a chunk past the last member reads zeros,
          // and chunks that are not needed are zeroed when consumed
          const __amdgpu_buffer_rsrc_t hrn = __builtin_amdgcn_make_buffer_rsrc(
              xbase + ((nt + kRing - 1) % kRing) * xslot, 0, xslot, 0x00020000);
#pragma unroll
          for (int c = 0; c < NCH; ++c)
            areg[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(hrn, xlane, xconst(c, nmt), 16));
        }
      }

      // ---- 3. partial tiles -> LDS.  C layout: lane holds unit column r16, batch rows 4q..4q+3
      const int buf = it & 1;
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<f32x4 *>(&part[buf][wave][g][r16 * kTileStride + 4 * q]) = acc[g];
      XS_TICK(1);
      lds_barrier();  // barrier #it
      XS_TICK(2);

      // ---- 4. reduce over waves + exponential gating for element (row pb, unit pa)
      float raw[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        // fixed summation order: wave 0 + wave 1 + wave 2 + wave 3
        float ry = part[buf][0][g][pa * kTileStride + pb];
        ry += part[buf][1][g][pa * kTileStride + pb];
        ry += part[buf][2][g][pa * kTileStride + pb];
        ry += part[buf][3][g][pa * kTileStride + pb];
        raw[g] = (wxs[buf][g][pb * kTileStride + pa] + ry) + bias_g[g];
      }
      if (rfl[it & 3][pb] != 0u) st[mt] = CellState{0.0f, 0.0f, 0.0f, 0.0f};
      slstm_pointwise(raw[0], raw[1], raw[2], raw[3], st[mt]);
#ifdef XS_PROFILE
      asm volatile("" :: "v"(st[mt].y));
#endif
      XS_TICK(3);
      // ---- 5. publish h_t to the peers, re-arm the words of h_{t-2}, stage h_t for the drainer
      float y = st[mt].y;
      if (!BF16 && y != y) y = __uint_as_float(0x7FC00000u);  // keep the "not written yet" NaN pattern unique
      // (With four row tiles the drainer wave publishes: see there.)  Every lane stores, every
      // iteration: lanes outside the batch or the head write words of their own block that nobody
      // polls, and the re-arm of steps 0 and 1 hits slots that still hold the pattern.
      if (!kDrainerPublishes) {
        const long long xo = ((long long)mt * p.G + member) * (XTILE / ESZ) + pb * 16 + pa;
        if (BF16) {
          const uint16_t v = (uint16_t)float_to_bf16_bits(y);
          uint16_t *dst = reinterpret_cast<uint16_t *>(hcur) + xo;
          uint16_t *old = reinterpret_cast<uint16_t *>(hold) + xo;
          if (cross) {
            __hip_atomic_store(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(old, (uint16_t)kSentinel16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          } else {
            *dst = v;
            *old = (uint16_t)kSentinel16;
          }
        } else {
          float *dst = reinterpret_cast<float *>(hcur) + xo;
          float *old = reinterpret_cast<float *>(hold) + xo;
          if (cross) {
            __hip_atomic_store(dst, y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(old, __uint_as_float(kSentinel32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          } else {
            *dst = y;
            *old = __uint_as_float(kSentinel32);
          }
        }
      }
      hst[it & 3][tid] = y;
      if (kDrainerPublishes && lane == 0)
        __hip_atomic_store(&pubflag[wave], (uint32_t)it + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      XS_TICK(4);
    }
  }
  for (int j = NIT; j < NITpad; ++j) lds_barrier();  // padding iterations of the feeder
  lds_barrier();                                     // final barrier
#ifdef XS_PROFILE
  if (lane == 0 && member == 0 && gi == 0) {
    long long *dst = reinterpret_cast<long long *>(p.wg_xcc + 4096 - 128) + wave * 8;
    for (int i = 0; i < 8; ++i) dst[i] = prof[i];
  }
#endif

  // ---- final state
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int brow = rowbase + mt * 16 + pb;
    if (unit_ok && brow < rend) {
      const long long o = (long long)brow * H + col;
      p.s_out[o] = st[mt].y; p.s_out[BH + o] = st[mt].c; p.s_out[2 * BH + o] = st[mt].n; p.s_out[3 * BH + o] = st[mt].m;
    }
  }
  if (lane == 0 && max_spins) atomicMax(&p.status->max_spins, max_spins);
}

// ---------------------------------------------------------------------------
// decode step kernel, LDS-staged: a workgroup owns 64 batch rows x 32 units x 4 gates.
// K is walked in slabs of SLABCH MFMA k-steps (WIDE: 64 bf16 / 32 fp32 input units, so that
// every global load instruction moves whole 128-byte lines); each slab of h (converted to the
// operand type) and of R goes to LDS, double-buffered, one barrier per slab, and the global
// loads of up to kStepRing slabs are in flight at once (all of them at dh = 256).  The product
// is formed transposed (units on the MFMA M axis), so a lane ends with 4 consecutive units of
// one batch row and the state, W.x and h move as 16-byte / 8-byte accesses that are issued
// before the K loop and consumed after it.  The slabs are accumulated in the sequence kernel's
// four K quarters and the quarters are added in its order, so step-by-step decoding
// reproduces a sequence call bit for bit.
// ---------------------------------------------------------------------------
struct StepParams {
  const void *wx;
  long long wx_sb;
  const void *r;
  int r_bf16;
  const float *bias;
  const float *s0;
  const unsigned char *reset;
  long long reset_sb;
  void *h_out;
  float *s_out;
  xs_slstm_status *status;
  int B, NH, dh;
  int n_unit_tiles, n_row_tiles;
};

// Workgroup i runs on XCD i % 8.  The workgroups of one head share its h rows and its R, so they
// are placed on as few XCDs as possible (one when there are 8 or more heads): every operand is
// then fetched from HBM once and re-read from ONE L2 instead of being fetched by all eight.
__device__ __forceinline__ void step_tile_of(const StepParams &p, int i, int &head, int &ut, int &rt) {
  const int tiles = p.n_unit_tiles * p.n_row_tiles;
  int tile;
  if (p.NH % 8 == 0) {
    const int hpx = p.NH / 8;  // heads per XCD
    const int m = i >> 3;
    head = (i & 7) * hpx + m % hpx;
    tile = m / hpx;
  } else if (8 % p.NH == 0 && tiles % (8 / p.NH) == 0) {
    const int xph = 8 / p.NH;  // XCDs per head
    head = (i & 7) % p.NH;
    tile = (i >> 3) * xph + (i & 7) / p.NH;
  } else {
    head = i / tiles;
    tile = i - head * tiles;
  }
  ut = tile % p.n_unit_tiles;
  rt = tile / p.n_unit_tiles;
}

// FULL: the tile lies entirely inside the problem (64 rows, 32 units, every K slab), there is an
// initial state and no reset mask - the decode steady state.  All clamping and masking is then
// compiled out, which matters: the kernel is bound by the number of instructions a wave issues.
// SLABCH = MFMA k-steps per slab.  With 4 (dh <= 128) or 8 (dh <= 256, bf16) the whole K range
// is ONE slab: everything is staged once, one barrier, and the registers that carried the
// loads are free again before the MFMA loop (which then batches its LDS reads).
template <bool BF16, int SLABCH, bool FULL>
__global__ __launch_bounds__(256) void slstm_step_tile_kernel(StepParams p, int nch_log2) {
  constexpr int EPC = BF16 ? 8 : 4;
  constexpr int CHK = 4 * EPC;                // input units per MFMA k-step ("chunk")
  constexpr int SLABK = SLABCH * CHK;         // input units per slab
  constexpr int kStepRing = SLABCH >= 4 ? 1 : 4;  // slabs whose loads are in flight
  constexpr int NBUF = SLABCH >= 4 ? 1 : 2;       // LDS buffers
  constexpr int RS = SLABCH * 64 + 16;        // bytes per LDS row: data + pad (conflict-free 16-byte reads)
  constexpr int HITEMS = (SLABK * 4 / 16) / 4;  // 16-byte pieces of fp32 h each thread stages per slab
  constexpr int RITEMS = SLABCH * 2;            // 16-byte pieces of R each thread stages per slab
  constexpr int ESZ = BF16 ? 2 : 4;
  extern __shared__ __attribute__((aligned(16))) unsigned char step_lds[];
  unsigned char(*hbuf)[64 * RS] = reinterpret_cast<unsigned char(*)[64 * RS]>(step_lds);
  unsigned char(*rbuf)[128 * RS] = reinterpret_cast<unsigned char(*)[128 * RS]>(step_lds + NBUF * 64 * RS);

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int q = lane >> 4;
  const int r16 = lane & 15;
  int head, unit_tile, row_tile;
  step_tile_of(p, blockIdx.x, head, unit_tile, row_tile);
  const int a0 = unit_tile * 32;
  const int rowbase = row_tile * 64;
  const int dh = p.dh;
  const int H = p.NH * dh;
  const long long BH = (long long)p.B * H;
  const int nch = 1 << nch_log2;              // chunks per K quarter (as in the sequence kernel)
  const int nslab = (4 * nch) / SLABCH;

  if (blockIdx.x == 0 && tid < 16)
    reinterpret_cast<uint32_t *>(p.status)[tid] = 0u;  // a step never waits, so it never aborts

  const bool has_s0 = FULL || p.s0 != nullptr;
  const bool has_reset = !FULL && p.reset != nullptr;
  const float *s0p = has_s0 ? p.s0 : reinterpret_cast<const float *>(p.wx);                  // stand-ins are only read
  const unsigned char *rsp = has_reset ? p.reset : reinterpret_cast<const unsigned char *>(p.wx);  // in their first 32 bytes

  // ---- staging roles: consecutive lanes take consecutive 16-byte pieces of a row / column.
  // A single slab is staged in NSPLIT phases (K halves): a thread's first HITEMS / NSPLIT items
  // lie in the first half of K, so the MFMA loop can start on it while the second half lands.
  constexpr int HPIECES = SLABK * 4 / 16;     // 16-byte pieces of fp32 h per row and slab
  constexpr int RPIECES = SLABCH * 4;         // 16-byte pieces of R per column and slab
  constexpr int NSPLIT = SLABCH >= 4 ? 2 : 1;
  constexpr int HPP = HPIECES / NSPLIT, HIP = HITEMS / NSPLIT;  // pieces per row, items per thread: per phase
  constexpr int RPP = RPIECES / NSPLIT, RIP = RITEMS / NSPLIT;
  auto hrow_of = [&](int j) { return (tid + 256 * (j % HIP)) / HPP; };
  auto hpiece_of = [&](int j) { return (j / HIP) * HPP + (tid + 256 * (j % HIP)) % HPP; };
  auto rcol_of = [&](int j) { return (tid + 256 * (j % RIP)) / RPP; };
  auto rpiece_of = [&](int j) { return (j / RIP) * RPP + (tid + 256 * (j % RIP)) % RPP; };
  const float *hsrc[HITEMS];
  bool hzero[HITEMS];
#pragma unroll
  for (int j = 0; j < HITEMS; ++j) {
    const int brow = rowbase + hrow_of(j);
    if (FULL) {
      hzero[j] = false;
      hsrc[j] = s0p + (long long)brow * H + head * dh + hpiece_of(j) * 4;
    } else {
      const int browc = brow < p.B ? brow : p.B - 1;
      const uint32_t flag = rsp[has_reset ? (long long)browc * p.reset_sb : 0];
      hzero[j] = !(brow < p.B) || !has_s0 || (has_reset && flag != 0u);
      hsrc[j] = s0p + (has_s0 ? (long long)browc * H + head * dh : 0);
    }
  }
  const char *rsrc[RITEMS];
  bool rok[RITEMS];
#pragma unroll
  for (int j = 0; j < RITEMS; ++j) {
    const int colx = rcol_of(j);                  // column of the workgroup's 128: gate colx/32, unit colx%32
    const int a = a0 + (colx & 31);
    rok[j] = FULL || a < dh;
    rsrc[j] = reinterpret_cast<const char *>(p.r) +
              ((long long)head * 4 * dh + (long long)(colx >> 5) * dh + (rok[j] ? a : 0)) * dh * ESZ +
              (FULL ? rpiece_of(j) * 16 : 0);
  }
  uint4 hring[kStepRing][HITEMS], rring[kStepRing][RITEMS];
  auto load_slab = [&](int sidx, uint4 (&hst)[HITEMS], uint4 (&rst)[RITEMS]) {
    const int kbase = sidx * SLABK;
#pragma unroll
    for (int ph = 0; ph < NSPLIT; ++ph) {
#pragma unroll
      for (int j = ph * HIP; j < (ph + 1) * HIP; ++j) {
        if (FULL) {
          hst[j] = *reinterpret_cast<const uint4 *>(hsrc[j] + kbase);
        } else {
          const int k = kbase + hpiece_of(j) * 4;
          hst[j] = *reinterpret_cast<const uint4 *>(hsrc[j] + ((has_s0 && k < dh) ? k : 0));
        }
      }
#pragma unroll
      for (int j = ph * RIP; j < (ph + 1) * RIP; ++j) {
        if (FULL) {
          rst[j] = *reinterpret_cast<const uint4 *>(rsrc[j] + kbase * ESZ);
        } else {
          const int k = kbase + rpiece_of(j) * EPC;
          rst[j] = *reinterpret_cast<const uint4 *>(rsrc[j] + (long long)(k < dh ? k : 0) * ESZ);
        }
      }
    }
  };
  // phase < 0: the whole slab; otherwise the items of that K phase only
  auto store_slab = [&](int sidx, int buf, const uint4 (&hst)[HITEMS], const uint4 (&rst)[RITEMS], int phase) {
    const int kbase = sidx * SLABK;
#pragma unroll
    for (int j = 0; j < HITEMS; ++j) {
      if (phase >= 0 && j / HIP != phase) continue;
      const int piece = hpiece_of(j);
      uint4 v = hst[j];
      if (!FULL && (hzero[j] || kbase + piece * 4 >= dh)) v = make_uint4(0, 0, 0, 0);
      unsigned char *dst = &hbuf[buf][hrow_of(j) * RS];
      if (BF16) {
        uint2 w;
        w.x = pack_bf16x2(__uint_as_float(v.x), __uint_as_float(v.y));
        w.y = pack_bf16x2(__uint_as_float(v.z), __uint_as_float(v.w));
        *reinterpret_cast<uint2 *>(dst + piece * 8) = w;
      } else {
        *reinterpret_cast<uint4 *>(dst + piece * 16) = v;
      }
    }
#pragma unroll
    for (int j = 0; j < RITEMS; ++j) {
      if (phase >= 0 && j / RIP != phase) continue;
      const int piece = rpiece_of(j);
      uint4 w = rst[j];
      if (!FULL && (!rok[j] || kbase + piece * EPC >= dh)) w = make_uint4(0, 0, 0, 0);
      *reinterpret_cast<uint4 *>(&rbuf[buf][rcol_of(j) * RS + piece * 16]) = w;
    }
  };

#ifdef XS_PROFILE
  long long pstamp[6];
  pstamp[0] = clock64();
  const long long pwall0 = wall_clock64();
#endif
#pragma unroll
  for (int u = 0; u < kStepRing; ++u)
    if (u < nslab) load_slab(u, hring[u], rring[u]);

  // ---- wave tiling 2 x 2: wave (wr, wu) owns rows 32*wr .. +31 (two MFMA row tiles, index ut below)
  // and units 16*wu .. +15 of all four gates, so a k-step reads 2 h and 4 R fragments from LDS for
  // its 8 MFMAs.  Pointwise operands of this lane: batch rows rowbase + 32*wr + 16*ut + r16,
  // units a0 + 16*wu + 4q .. +3.
  const int wr = wave >> 1, wu = wave & 1;
  const int ua = a0 + wu * 16 + 4 * q;
  const int uac = (FULL || ua < dh) ? ua : 0;
  const long long col = (long long)head * dh + uac;
  uint2 wxb[2][4];
  float4 wxf[2][4], bias4[4], c4[2], n4[2], m4[2];
  uint32_t pflag[2];
#pragma unroll
  for (int g = 0; g < 4; ++g)
    bias4[g] = *reinterpret_cast<const float4 *>(p.bias + ((long long)head * 4 + g) * dh + uac);
#pragma unroll
  for (int ut = 0; ut < 2; ++ut) {
    const int brow = rowbase + 32 * wr + 16 * ut + r16;
    const int browc = (FULL || brow < p.B) ? brow : p.B - 1;
    pflag[ut] = FULL ? 0u : rsp[has_reset ? (long long)browc * p.reset_sb : 0];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const long long o = (long long)browc * p.wx_sb + (long long)g * H + col;
      if (BF16) wxb[ut][g] = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(p.wx) + o);
      else wxf[ut][g] = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(p.wx) + o);
    }
    const long long so = (long long)browc * H + col;
    c4[ut] = *reinterpret_cast<const float4 *>(s0p + (has_s0 ? BH + so : 0));
    n4[ut] = *reinterpret_cast<const float4 *>(s0p + (has_s0 ? 2 * BH + so : 0));
    m4[ut] = *reinterpret_cast<const float4 *>(s0p + (has_s0 ? 3 * BH + so : 0));
  }

  // ---- K loop
  f32x4 acc[2][4], tot[2][4];
#pragma unroll
  for (int ut = 0; ut < 2; ++ut)
#pragma unroll
    for (int g = 0; g < 4; ++g) { acc[ut][g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f}; tot[ut][g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f}; }

#ifdef XS_PROFILE
  pstamp[1] = clock64();
#endif
  store_slab(0, 0, hring[0], rring[0], SLABCH >= 4 ? 0 : -1);
  __syncthreads();
#ifdef XS_PROFILE
  pstamp[2] = clock64();
#endif
  if (SLABCH >= 4) {
    // single slab: the number of chunks per K quarter is the compile-time constant SLABCH / 4 ->
    // straight-line MFMA code; the second K half goes to LDS after the MFMAs of the first
    constexpr int NQ = SLABCH / 4;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      if (w == 2) {
        store_slab(0, 0, hring[0], rring[0], 1);
        __syncthreads();
      }
#pragma unroll
      for (int cq = 0; cq < (NQ > 0 ? NQ : 1); ++cq) {
        const int ch = w * NQ + cq;
        uint4 hv[2], rv[4];
#pragma unroll
        for (int ut = 0; ut < 2; ++ut)
          hv[ut] = *reinterpret_cast<const uint4 *>(&hbuf[0][(32 * wr + 16 * ut + r16) * RS + ch * 64 + q * 16]);
#pragma unroll
        for (int g = 0; g < 4; ++g)
          rv[g] = *reinterpret_cast<const uint4 *>(&rbuf[0][(g * 32 + wu * 16 + r16) * RS + ch * 64 + q * 16]);
#pragma unroll
        for (int ut = 0; ut < 2; ++ut)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            if (BF16) {
              acc[ut][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, rv[g]), __builtin_bit_cast(bf16x8, hv[ut]), acc[ut][g], 0, 0, 0);
            } else {
              const uint32_t rw[4] = {rv[g].x, rv[g].y, rv[g].z, rv[g].w};
              const uint32_t hw[4] = {hv[ut].x, hv[ut].y, hv[ut].z, hv[ut].w};
#pragma unroll
              for (int e = 0; e < 4; ++e)
                acc[ut][g] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(rw[e]), __uint_as_float(hw[e]), acc[ut][g], 0, 0, 0);
            }
          }
      }
#pragma unroll
      for (int ut = 0; ut < 2; ++ut)
#pragma unroll
        for (int g = 0; g < 4; ++g) {  // fold the quarter into the running sum (quarter 0 first)
          tot[ut][g] = (w == 0) ? acc[ut][g] : tot[ut][g] + acc[ut][g];
          acc[ut][g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
  } else {
  for (int s0i = 0; s0i < nslab; s0i += kStepRing) {
#pragma unroll
    for (int u = 0; u < kStepRing; ++u) {
      const int sidx = s0i + u;
      if (sidx < nslab) {
        const int buf = sidx & (NBUF - 1);
#pragma unroll
        for (int ch = 0; ch < SLABCH; ++ch) {
          uint4 hv[2], rv[4];
#pragma unroll
          for (int ut = 0; ut < 2; ++ut)
            hv[ut] = *reinterpret_cast<const uint4 *>(&hbuf[buf][(32 * wr + 16 * ut + r16) * RS + ch * 64 + q * 16]);
#pragma unroll
          for (int g = 0; g < 4; ++g)
            rv[g] = *reinterpret_cast<const uint4 *>(&rbuf[buf][(g * 32 + wu * 16 + r16) * RS + ch * 64 + q * 16]);
#pragma unroll
          for (int ut = 0; ut < 2; ++ut)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              if (BF16) {
                acc[ut][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, rv[g]), __builtin_bit_cast(bf16x8, hv[ut]), acc[ut][g], 0, 0, 0);
              } else {
                const uint32_t rw[4] = {rv[g].x, rv[g].y, rv[g].z, rv[g].w};
                const uint32_t hw[4] = {hv[ut].x, hv[ut].y, hv[ut].z, hv[ut].w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  acc[ut][g] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(rw[e]), __uint_as_float(hw[e]), acc[ut][g], 0, 0, 0);
              }
            }
          const int chunks_done = sidx * SLABCH + ch + 1;
          if ((chunks_done & (nch - 1)) == 0) {  // end of a K quarter: fold it into the running sum (quarter 0 first)
#pragma unroll
            for (int ut = 0; ut < 2; ++ut)
#pragma unroll
              for (int g = 0; g < 4; ++g) {
                tot[ut][g] = (chunks_done == nch) ? acc[ut][g] : tot[ut][g] + acc[ut][g];
                acc[ut][g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
              }
          }
        }
        // slab sidx went to LDS one iteration ago: its ring entry takes the loads of slab sidx + kStepRing
        if (sidx + kStepRing < nslab) load_slab(sidx + kStepRing, hring[u], rring[u]);
        if (sidx + 1 < nslab) {
          const int un = (u + 1) % kStepRing;
          store_slab(sidx + 1, (sidx + 1) & (NBUF - 1), hring[un], rring[un], -1);  // the other buffer was last read before the previous barrier
          __syncthreads();
        }
      }
    }
  }

  }
#ifdef XS_PROFILE
  asm volatile("" :: "v"(tot[0][0][0]), "v"(tot[1][3][3]));
  pstamp[3] = clock64();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  pstamp[4] = clock64();
#endif
  // ---- gating
#pragma unroll
  for (int ut = 0; ut < 2; ++ut) {
    const int brow = rowbase + 32 * wr + 16 * ut + r16;
    const bool reset_row = !FULL && (!has_s0 || (has_reset && pflag[ut] != 0u));
    const float cin[4] = {c4[ut].x, c4[ut].y, c4[ut].z, c4[ut].w};
    const float nin[4] = {n4[ut].x, n4[ut].y, n4[ut].z, n4[ut].w};
    const float min_[4] = {m4[ut].x, m4[ut].y, m4[ut].z, m4[ut].w};
    float yv[4], cv[4], nv[4], mv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float raw[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float wxv;
        if (BF16) {
          const uint32_t wd = i < 2 ? wxb[ut][g].x : wxb[ut][g].y;
          wxv = bf16_bits_to_float((i & 1) ? (wd >> 16) : (wd & 0xFFFFu));
        } else {
          const float wf[4] = {wxf[ut][g].x, wxf[ut][g].y, wxf[ut][g].z, wxf[ut][g].w};
          wxv = wf[i];
        }
        const float bf[4] = {bias4[g].x, bias4[g].y, bias4[g].z, bias4[g].w};
        raw[g] = (wxv + tot[ut][g][i]) + bf[i];
      }
      CellState st{0.0f, reset_row ? 0.0f : cin[i], reset_row ? 0.0f : nin[i], reset_row ? 0.0f : min_[i]};
      slstm_pointwise(raw[0], raw[1], raw[2], raw[3], st);
      yv[i] = st.y; cv[i] = st.c; nv[i] = st.n; mv[i] = st.m;
    }
    if (FULL || (brow < p.B && ua < dh)) {
      const long long o = (long long)brow * H + head * dh + ua;
      // streaming stores: the lines leave the L2 while the kernel still runs instead of being
      // written back when it ends (measured: 0.65 us per step at B = 256, D = 2048)
      __builtin_nontemporal_store(f32x4{yv[0], yv[1], yv[2], yv[3]}, reinterpret_cast<f32x4 *>(p.s_out + o));
      __builtin_nontemporal_store(f32x4{cv[0], cv[1], cv[2], cv[3]}, reinterpret_cast<f32x4 *>(p.s_out + BH + o));
      __builtin_nontemporal_store(f32x4{nv[0], nv[1], nv[2], nv[3]}, reinterpret_cast<f32x4 *>(p.s_out + 2 * BH + o));
      __builtin_nontemporal_store(f32x4{mv[0], mv[1], mv[2], mv[3]}, reinterpret_cast<f32x4 *>(p.s_out + 3 * BH + o));
      if (BF16) {
        uint2 hw;
        hw.x = float_to_bf16_bits(yv[0]) | (float_to_bf16_bits(yv[1]) << 16);
        hw.y = float_to_bf16_bits(yv[2]) | (float_to_bf16_bits(yv[3]) << 16);
        // (h stays an ordinary store: as a streaming store its 8-byte pieces cost 0.8 us per step)
        *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(p.h_out) + o) = hw;
      } else {
        *reinterpret_cast<float4 *>(reinterpret_cast<float *>(p.h_out) + o) = make_float4(yv[0], yv[1], yv[2], yv[3]);
      }
    }
  }
#ifdef XS_PROFILE
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (tid == 0 && blockIdx.x == 9) {
    pstamp[5] = clock64();
    long long *dst = reinterpret_cast<long long *>(reinterpret_cast<char *>(p.status) + 64);
    for (int i = 0; i < 6; ++i) dst[i] = pstamp[i] - pstamp[0];
  }
  if (tid == 0) {
    long long *wt = reinterpret_cast<long long *>(reinterpret_cast<char *>(p.status) + 256);
    wt[2 * blockIdx.x] = pwall0;
    wt[2 * blockIdx.x + 1] = wall_clock64();
  }
#endif
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
constexpr size_t kHeaderBytes = kStatusBytes + (size_t)kMaxWg * 4;  // status block + placement words (multiple of 256)

// upper bound on the elements of the exchange ring [8 slots][head groups][G][rows][16]:
// the head groups of one launch never cover more than B rounded up to 64 rows per head
inline size_t xbuf_elems(int B, int NH, int dh) {
  // (with row tiles of 4 or 8 rows a block still spans 16 rows, hence the factor 4)
  return (size_t)8 * NH * ((dh + 15) / 16) * ((size_t)(B + 63) / 64 * 64) * 16 * 4;
}

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
  if (step && a->r_dtype != a->wx_dtype) return fail(XS_ERR_DTYPE, "xs_slstm_step needs the recurrent matrix in the dtype of wx");
  if (a->wx_dtype != XS_F32 && a->wx_dtype != XS_BF16) return fail(XS_ERR_DTYPE, "wx_dtype %d not supported", a->wx_dtype);
  if (a->r_dtype != XS_F32 && a->r_dtype != XS_BF16) return fail(XS_ERR_DTYPE, "r_dtype %d not supported", a->r_dtype);
  if (a->wx_dtype == XS_F32 && a->r_dtype != XS_F32) return fail(XS_ERR_DTYPE, "float32 wx needs a float32 recurrent matrix");
  if (!a->r || !a->bias || !a->s_out) return fail(XS_ERR_NULL, "r, bias and s_out are required");
  if (a->s0 && a->s0 == a->s_out) return fail(XS_ERR_SHAPE, "s_out must not alias s0");
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
  const long long esz = a->wx_dtype == XS_BF16 ? 2 : 4;
  if (a->B > 0 && a->T > 0 &&
      (((uintptr_t)a->wx % al) || ((a->wx_stride_b * esz) % 16) || ((a->wx_stride_t * esz) % 16)))
    return fail(XS_ERR_ALIGN, "wx and its row/step strides must be 16-byte aligned");
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

// Raises a kernel's dynamic-LDS limit once per (kernel, device); the attribute call is not free and
// a decode loop would otherwise pay it every token.
int ensure_dynamic_lds(const void *kernel, size_t bytes) {
  struct Done { const void *kernel; int device; size_t bytes; };
  static std::mutex mu;
  static std::vector<Done> done;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(XS_ERR_DEVICE, "cannot query the current device");
  std::lock_guard<std::mutex> lock(mu);
  for (const Done &d : done)
    if (d.kernel == kernel && d.device == dev && d.bytes >= bytes) return XS_OK;
  const hipError_t ea = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (ea != hipSuccess) return fail(XS_ERR_LAUNCH, "cannot reserve %zu bytes of LDS: %s", bytes, hipGetErrorString(ea));
  done.push_back(Done{kernel, dev, bytes});
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
  const size_t lds = (size_t)nbuf * (64 + 128) * (slabch * 64 + 16);
  typedef void (*StepKernel)(StepParams, int);
  StepKernel kern;
#define XS_PICK(BF, SC) (full ? slstm_step_tile_kernel<BF, SC, true> : slstm_step_tile_kernel<BF, SC, false>)
  if (bf16) kern = slabch == 4 ? XS_PICK(true, 4) : (slabch == 8 ? XS_PICK(true, 8) : XS_PICK(true, 2));
  else kern = slabch == 4 ? XS_PICK(false, 4) : (slabch == 8 ? XS_PICK(false, 8) : XS_PICK(false, 2));
#undef XS_PICK
  if (lds > 64 * 1024) {  // the single-slab variant at dh = 256 needs 99 KiB of the 160 KiB of LDS
    const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), lds);
    if (rc != XS_OK) return rc;
  }
  hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, p, nch_log2);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(XS_ERR_LAUNCH, "step kernel launch failed: %s", hipGetErrorString(e));
  return XS_OK;
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
  int rows_per_wg = 16 * MT;
  if (MT == 1) {  // spare compute units: smaller row tiles, smaller exchanges
    for (int r = 4; r < 16; r *= 2)
      if ((B + r - 1) / r <= max_groups_per_head) { rows_per_wg = r; break; }
  }
  const int rows_per_launch = rows_per_wg * max_groups_per_head;

  SeqKernel kern = bf16 ? pick_kernel<true>(nch, MT) : pick_kernel<false>(nch, MT);
  if (!kern) return fail(XS_ERR_UNSUPPORTED, "no kernel for nch=%d MT=%d", nch, MT);

  uint32_t launches = 0;
  for (int b0 = 0; b0 < B; b0 += rows_per_launch) {
    const int bend = b0 + rows_per_launch < B ? b0 + rows_per_launch : B;
    const int NBT = (bend - b0 + rows_per_wg - 1) / rows_per_wg;
    const int ngroups = NH * NBT;
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
    p.spin_limit = a->spin_limit;
    // with four row tiles the polled tiles are staged in dynamic LDS: [2][4 waves][nch] KiB
    const size_t dyn_lds = MT >= 4 ? (size_t)nch * 8192 : 0;
    if (dyn_lds) {
      const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), dyn_lds);
      if (rc != XS_OK) return rc;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), dyn_lds, stream, p);
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

size_t xs_slstm_workspace_bytes(int32_t B, int32_t T, int32_t NH, int32_t dh) {
  if (B < 0 || T < 0 || NH <= 0 || dh <= 0) return 0;
  return kHeaderBytes + xbuf_elems(B, NH, dh) * 4;
}

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
  return run_step(args);
}

}  // extern "C"
