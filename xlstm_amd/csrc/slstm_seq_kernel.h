// The persistent sequence kernel: all T timesteps of a call in one launch.
// Included by slstm_hip.hip only (one translation unit), after slstm_device_common.h.
#pragma once

namespace {

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
  int head0;     // first head of this launch (more heads than fit the device at once go in several launches)
  int NHL;       // heads of this launch
  int rows_per_wg;
  long long spin_limit;
  int prefetch;  // number of prefetch waves launched behind the six others (0 .. kMaxPrefetchWaves)
  float *coef_out;  // COEF variant: the backward pass's nine coefficients per step and element,
                    // [T][ceil(B/4)][NH][dh/64][4 rows][9][64 units] (what slstm_bwd_quad_kernel reads); else unused
};

// ---------------------------------------------------------------------------
// persistent sequence kernel
//   BF16: wx / h_out / MFMA operands are bf16 (fp32 accumulate, fp32 c,n,m);
//         otherwise everything is fp32 (v_mfma_f32_16x16x4_f32).
//   NCH : 16-byte chunks of h each lane holds per batch row; one wave covers
//         NCH*32 (bf16) or NCH*16 (fp32) input units, the four waves 4x that.
//   MT  : 16-row batch tiles handled one after the other by a workgroup.
//
// Six to eight waves per workgroup, one barrier per (step, tile) iteration shared by all:
//   waves 0-3  compute: poll h_{t-1}, MFMA, reduce through LDS, gating, publish h_t.
//              Their vector-memory queue only ever holds L2-resident traffic (the
//              exchange ring), because vector memory completes in order within a wave
//              and anything slower would sit in front of the latency-critical polls.
//   wave 4     feeder: streams W.x and the reset flags of FUTURE iterations from HBM
//              into an LDS ring (four iterations in flight; with two row tiles, bursts of eight).
//   wave 5     drainer: writes h of PAST iterations from an LDS staging ring to the
//              output tensor in HBM.
//   waves 6..  prefetchers (0 to 2 of them, chosen by the host): they touch the W.x lines of the step
//              kPrefetchAhead ahead with SCALAR loads.  A compute unit returns vector-memory data in order across
//              its waves, so every feeder load that misses to HBM delays the polls issued behind it (measured: an
//              L2 hit takes 200 cycles alone and 600 with another wave's misses in flight, unchanged at 210 when
//              those misses go through the scalar cache).  With the lines already in the L2 the feeder's loads
//              are short.  A scalar miss brings 64 bytes and a wave keeps about 15 of them in flight, so a
//              prefetch wave is given at most 8 loads per iteration, and the scalar cache serves about 16 per
//              iteration in all (measured: two waves of 8 gain 18 %, four waves of 8 lose a factor of 2 because
//              they hold up the barriers), so tiles of 16 rows go without.
//
// Exchange ring: kRing slots, slot t % kRing holds h_t as [row tile][member][16 rows][16 units].
// A word is either data or the "not written yet" pattern.  A workgroup re-arms its own
// words of slot (t-2) % kRing after its poll of step t has completed: by then every peer
// has published h_{t-1}, hence has finished reading h_{t-2}.  The re-arm is acknowledged
// before the workgroup's poll of step t+1 completes, i.e. before it publishes h_{t+1};
// a peer polling slot (t-2) % kRing for h_{t-2+kRing} has seen that publication, so it
// can only ever read the pattern or the new data there, never the stale h_{t-2}.
// ---------------------------------------------------------------------------
constexpr int kRing = 8;       // slots of the exchange ring
// Measurement builds (-DXS_PROFILE): the waves of workgroup 0 leave their per-phase cycle sums in the last 128 of the
// 4096 placement words of the workspace header, 8 counters of 8 bytes per wave slot.
constexpr int kStampWord = 4096 - 128;
// prefetch waves a kernel may be launched with (8 waves per workgroup = two per SIMD = 256 VGPRs each, which the
// largest variants need)
constexpr int max_prefetch_waves(int nch) { return nch >= 8 ? 1 : kMaxPrefetchWaves; }
constexpr int kPrefetchAhead = 8;  // steps between the scalar-cache touch of a W.x line and the step that uses it (4: 17 % slower; 12, 16: the same)

__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint32_t uniform(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

// ---- role of a workgroup (XCD-aware: workgroup i is dispatched to XCD i % 8; a head group takes consecutive slots of
//      ONE XCD so its exchange stays in one L2): head group index and position inside the group
__device__ __forceinline__ void seq_place(const SeqParams &p, int wg, int &gi, int &member) {
  if (p.G <= 32) {
    const int xcd = wg & 7;
    const int local = wg >> 3;
    const int slot = local / p.G;
    member = local - slot * p.G;
    gi = slot * 8 + xcd;
  } else if (p.G <= 64 && (p.G & 1) == 0) {
    // two XCDs per group (workgroup i runs on XCD i % 8): XCDs j and j + 4, members 0 .. G/2-1 on the first, the rest
    // on the second, so that half of a member's polls stay inside its own L2.  (Measured at head dim 1024, batch 64,
    // three runs each: 13.5 ms with the pairs (j, j + 4), 13.7 with (j, j + 1), 13.8 with (j, j + 2).)
    const int xcd = wg & 7;
    const int local = wg >> 3;
    const int half = p.G >> 1;
    const int slot = local / half;
    member = (xcd >> 2) * half + (local - slot * half);
    gi = slot * 4 + (xcd & 3);
  } else {  // larger groups are spread over all XCDs
    gi = wg / p.G;
    member = wg - gi * p.G;
  }
}

// ---- placement handshake (one thread of the workgroup): do all members of this head group share one XCD (one L2)?
//      If so h is published with plain stores (they land in that L2); otherwise with device-scope stores that are
//      written through to memory.  Returns 1 for "more than one XCD".
__device__ __forceinline__ uint32_t seq_handshake(const SeqParams &p, int wg, int gi, long long spin_limit) {
  const bool one_xcd_layout = p.G <= 32;
  if (wg == 0) {
    atomicAdd(&p.status->launches, 1u);  // a long batch is run as several launches of row chunks
    p.status->rows_per_workgroup = (uint32_t)p.rows_per_wg;
  }
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
  return cross;
}

// FULL: the head dim fills the K range of the four waves exactly (dh == 16 * NCH * elements per chunk) and, with
// more than one row tile, every batch row of every tile exists.  The per-chunk "is this chunk needed" masks of
// the arrival test are then compiled out (with one row tile, lanes of rows that do not exist read zeros from
// past the end of the buffer descriptor, which never look like the "not written yet" pattern).  That matters:
// the compute waves are bound by the number of instructions between the arrival of h and the MFMAs.
// BURST: the feeder fetches W.x in bursts of several iterations (see there); the host asks for it with two row
// tiles and with one row tile of 8 or 16 rows, for head dims up to 512 (bf16).
// FMAC: the contraction of a row tile of at most 4 rows with FMA instructions and a reduction across the wave instead
// of MFMA (the alternative for small batches; measured, slower at every batch size, so the host never picks it
// unless the library is built with XS_SMALL_BATCH_FMA for that measurement).  Each lane multiplies its 8 (bf16) or
// 4 (fp32) inputs of every real row - fetched from the lane that holds them - into its own column's weights, and
// the four lane groups' partial sums over K are added with two cross-lane steps.  The sums are formed in a different
// order than the MFMA forms them, so the bits differ from the MFMA path (and from the decode kernel).
// QUAD: row tiles of at most 4 rows (bf16, FULL, one row tile): the four compute waves split the workgroup's 64
// columns by UNIT instead of splitting K, see "waves 0-3, QUAD" below.
// COEF (with QUAD): a training forward: the compute waves also leave the nine coefficients per step and element that the
// backward pass would otherwise recompute in a forward walk of its own (slstm_bwd_prepare_kernel), see "COEF" below.
template <bool BF16, int NCH, int MT, bool FULL, bool BURST, bool FMAC = false, bool QUAD = false, bool COEF = false>
__global__ __launch_bounds__(kThreads + 64 * max_prefetch_waves(NCH)) void slstm_seq_kernel(SeqParams p) {
  static_assert(!COEF || QUAD, "coefficients for the backward pass come from the unit-split compute waves only");
  static_assert(!FMAC || MT == 1, "the FMA contraction is for one row tile of at most 4 rows");
  static_assert(!QUAD || (BF16 && MT == 1 && FULL && !BURST && !FMAC), "the unit-split compute waves exist for bf16, one full row tile");
  constexpr int EPC = BF16 ? 8 : 4;      // elements per 16-byte chunk
  constexpr int KW = NCH * 4 * EPC;      // input units per wave
  constexpr int ESZ = BF16 ? 2 : 4;
  constexpr int WCH = 16 / EPC;          // 16-byte chunks holding the 16 units of one (row, gate)
  constexpr int ROWS = 16 * MT;          // batch rows of a workgroup
  static_assert(MT == 1 || MT == 2, "workgroups of four row tiles run slstm_seq_roles_kernel");

  __shared__ float part[2][4][4][kTileFloats];  // [buffer][wave][gate][unit*stride + row]
  __shared__ float wxs[2][4][kTileFloats];      // [slot][gate][row*stride + unit]   W.x of one iteration
  __shared__ float hst[4][256];                 // [slot][row*16 + unit]             h on its way to HBM
  __shared__ float cst[COEF ? 4 : 1][COEF ? 9 * 64 : 1];  // [slot][coefficient][row*16 + unit]  (COEF) on their way to HBM
  __shared__ uint32_t rfl[4][16];               // [slot][row]                       reset flags
  __shared__ uint32_t cross_s;

  // ---- role of this workgroup
  const int wg = blockIdx.x;
  const int ngroups = p.NHL * p.NBT;
  int gi, member;  // head group index, position inside the group
  seq_place(p, wg, gi, member);
  if (gi >= ngroups) return;
  const int head = p.head0 + gi / p.NBT;
  const int bt = gi % p.NBT;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const long long spin_limit = p.spin_limit > 0 ? p.spin_limit : kDefaultSpinLimit;

  if (tid == 0) cross_s = seq_handshake(p, wg, gi, spin_limit);

  const int dh = p.dh;
  const int H = p.NH * dh;
  const int a0 = member * 16;
  const int rowbase = p.b0 + bt * p.rows_per_wg;
  // rows [rowbase, rend) belong to this workgroup; with few rows per head the batch is cut into
  // tiles of fewer than 16 rows so that more compute units share the work and every exchange is smaller
  const int rend = (rowbase + p.rows_per_wg < p.bend) ? rowbase + p.rows_per_wg : p.bend;
  const long long BH = (long long)p.B * H;
  const int NIT = p.T * MT;
  // How far ahead the feeder fetches W.x.  A compute unit returns vector-memory data in order across its waves, so
  // while feeder loads that miss to HBM are in flight the polls of the compute waves wait behind them.
  //   plain   a load per iteration, four iterations ahead (with row tiles of 4 rows the prefetch waves keep those
  //           loads from missing);
  //   BURST   bursts of kBurst iterations, one burst ahead (a ring of two bursts in registers): the polls then wait
  //           behind W.x during one memory latency per burst instead of all the time.
  // Measured with bursts: two row tiles, B 128 x dh 256 2.46 -> 2.11 us per step, B 64 x 8 heads x dh 256 2.64 -> 2.25,
  // B 64 x dh 512 2.68 -> 2.42; one row tile of 16 rows (B 64 x dh 256) 1.31 -> 1.20, of 8 rows (B 32, on top of the
  // prefetch waves) 1.03 -> 0.96.  Not with row tiles of 4 rows, where the prefetch waves cover every line (config 2:
  // 6 % slower), not with four row tiles (those iterations are bound by their arithmetic, the time per step is the
  // same with W.x in the Infinity Cache; 12 % slower), not with a 1024-wide head (9 % slower).  At which iteration
  // of a burst the next one is requested makes no difference (0, 1, 4 tried).
  constexpr bool kBursts = BURST;
  constexpr int kBurst = kBursts ? (BF16 ? 8 : 4) : 1;
  constexpr int kFeedRing = kBursts ? 2 * kBurst : 4;
  const int NITpad = (NIT + kFeedRing - 1) / kFeedRing * kFeedRing;  // barriers every wave executes

  // =========================================================================
  // wave 4: feeder.  Every iteration issues exactly WCH + 1 loads (addresses of
  // rows / chunks / steps that do not exist are clamped to ones that do and the
  // result is zeroed), so that the outstanding-load count at each use is exact.
  // =========================================================================
  if (wave == 4) {
    const int fb = lane & 15;  // batch row inside the tile
    const int fg = lane >> 4;  // gate
    uint4 ring[kFeedRing][WCH];
    uint32_t fring[kFeedRing];
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
    for (int u = 0; u < (kBursts ? kBurst : kFeedRing); ++u) issue(u, ring[u], fring[u]);
    if (fg == 0) rfl[0][fb] = (rowbase + fb < rend) ? (fring[0] & flag_on) : 0u;
    lds_barrier();  // prologue barrier
#ifdef XS_PROFILE
    long long fprof[3] = {0, 0, 0};
    long long ft = clock64();
#define XS_FTICK(i) do { const long long now_ = clock64(); fprof[i] += now_ - ft; ft = now_; } while (0)
#else
#define XS_FTICK(i) do { } while (0)
#endif
    for (int it0 = 0; it0 < NITpad; it0 += kFeedRing) {
#pragma unroll
      for (int u = 0; u < kFeedRing; ++u) {
        const int it = it0 + u;
        if constexpr (kBursts) {
          if (u % kBurst == 0) {  // the burst behind the one that starts now; its registers held the burst before
#pragma unroll
            for (int v = 0; v < kBurst; ++v) {
              const int slot = (u + kBurst + v) % kFeedRing;
              issue(it + kBurst + v, ring[slot], fring[slot]);
            }
          }
          XS_FTICK(1);
          put(it, ring[u], fring[(u + 1) % kFeedRing], it + 1);
          XS_FTICK(0);
        } else {
          put(it, ring[u], fring[(u + 1) % kFeedRing], it + 1);
          XS_FTICK(0);
          issue(it + kFeedRing, ring[u], fring[u]);
          XS_FTICK(1);
        }
        lds_barrier();  // barrier #it
        XS_FTICK(2);
      }
    }
    lds_barrier();  // final barrier
#ifdef XS_PROFILE
    if (lane == 0 && member == 0 && gi == 0) {
      long long *dst = reinterpret_cast<long long *>(p.wg_xcc + kStampWord) + 4 * 8;
      for (int i = 0; i < 3; ++i) dst[i] = fprof[i];
    }
#endif
    return;
  }

  // =========================================================================
  // wave 5: drainer.  h of iteration it is staged in LDS by the compute waves
  // between barriers #it and #it+1; it is written to HBM two iterations later
  // =========================================================================
  if (wave == 5) {
    const int drow = lane >> 2;   // batch row inside the tile
    const int dq = lane & 3;      // which 4 of the 16 units
    auto drain = [&](int it, bool poison = false) {
      const int t = it / MT;
      const int mt = it - t * MT;
      const int brow = rowbase + mt * 16 + drow;
      f32x4 v = *reinterpret_cast<const f32x4 *>(&hst[it & 3][drow * 16 + dq * 4]);
      if (poison) v = f32x4{kPoison, kPoison, kPoison, kPoison};
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
    // COEF: the coefficients of step t are staged one iteration later than its h (in the shadow of the next step's
    // poll), between barriers #t+1 and #t+2, and leave three iterations behind: 4 rows x 9 coefficients x 16 units into
    // the piece of the (row tile, head, slice of 64 units) that the backward's reverse kernel reads per step
    float *coef_dst = nullptr;
    long long coef_step = 0;
    if constexpr (COEF) {
      const int ntiles = (p.B + 3) >> 2, S = dh >> 6;
      coef_step = (long long)ntiles * p.NH * S * (4 * 9 * 64);
      coef_dst = p.coef_out + ((((long long)(rowbase >> 2)) * p.NH + head) * S + (a0 >> 6)) * (4 * 9 * 64)
                 + (lane >> 4) * (9 * 64) + (a0 & 63) + (lane & 15);
    }
    auto drain_coef = [&](int t) {
      if constexpr (COEF) {
        float *dst = coef_dst + t * coef_step;
#pragma unroll
        for (int j = 0; j < 9; ++j) dst[j * 64] = cst[t & 3][j * 64 + lane];
      }
    };
    lds_barrier();  // prologue barrier
#ifdef XS_PROFILE
    long long dprof[2] = {0, 0};
    long long dt = clock64();
#endif
    for (int j = 0; j < NITpad; ++j) {
      if (j >= 2 && j - 2 < NIT) drain(j - 2);
      if (COEF && j >= 3 && j - 3 < NIT) drain_coef(j - 3);
#ifdef XS_PROFILE
      { const long long now_ = clock64(); dprof[0] += now_ - dt; dt = now_; }
#endif
      lds_barrier();  // barrier #j
#ifdef XS_PROFILE
      { const long long now_ = clock64(); dprof[1] += now_ - dt; dt = now_; }
#endif
    }
    lds_barrier();  // final barrier
    for (int it = (NITpad >= 2 ? NITpad - 2 : 0); it < NIT; ++it) drain(it);
    if (COEF)
      for (int it = (NITpad >= 3 ? NITpad - 3 : 0); it < NIT; ++it) drain_coef(it);
    // A bounded wait ran out somewhere: whatever this workgroup computed from then on is built on operands that
    // never arrived.  A caller that does not read the status block must not mistake it for a result, so the
    // workgroup's part of h_out becomes NaN (the compute waves do the same to s_out).  Any workgroup that consumed
    // such operands did so after the flag was raised, and looks at the flag here, later still.
    if (__hip_atomic_load(&p.status->aborted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)
      for (int it = 0; it < NIT; ++it) drain(it, true);
#ifdef XS_PROFILE
    if (lane == 0 && member == 0 && gi == 0) {
      long long *dst = reinterpret_cast<long long *>(p.wg_xcc + kStampWord) + 5 * 8;
      for (int i = 0; i < 2; ++i) dst[i] = dprof[i];
    }
#endif
    return;
  }

  // =========================================================================
  // waves 6 and up: prefetchers.  They take part in every barrier (plain s_barrier: they have no LDS traffic of
  // their own and must not wait for their loads there) and issue nothing but scalar loads whose results are never
  // read: they all land in one scalar register that stays reserved for the whole loop.  Wave 6 + k takes the
  // batch rows k, k + n, ... of a tile.
  // =========================================================================
  if (wave >= 6) {
    const int pfi = (int)uniform((uint32_t)wave) - 6, npf = p.prefetch;  // (uniform: the loops below run on the scalar unit)
    constexpr int LM = 128 / (16 * ESZ);  // members whose 16 units share one 128-byte line of W.x: 4 (bf16) / 2 (fp32)
    const long long row_bytes = 4ll * H * ESZ;
    const long long cluster = ((long long)head * dh + (member / LM) * LM * 16) * ESZ;  // first byte of the shared line in a gate's block
    const char *const wxb = reinterpret_cast<const char *>(p.wx);
    uint32_t sink = 0;
    __builtin_amdgcn_s_barrier();  // prologue barrier
    for (int itp = 0; itp < NITpad; ++itp) {
      const int itn = itp + kPrefetchAhead * MT;  // the iteration whose lines are touched now
      const int tp = itn / MT;
      const int row0 = rowbase + (itn - tp * MT) * 16;
      const int nrows = rend - row0 < 16 ? rend - row0 : 16;
      if (tp < p.T) {
        for (int r = pfi; r < nrows; r += npf) {
          const long long rowoff = ((long long)(row0 + r) * p.wx_sb + (long long)tp * p.wx_st) * ESZ;
          for (int g = member % LM; g < 4; g += LM) {  // the members that share a line split the gates between them
#pragma unroll
            for (int half = 0; half < 2; ++half) {  // (a miss of the scalar cache brings 64 bytes into the L2, not the line)
              long long o = (long long)g * H * ESZ + cluster + half * 64;
              o = o < row_bytes - 4 ? o : row_bytes - 4;  // (a line of the last head may reach past the row)
              const unsigned long long a = reinterpret_cast<unsigned long long>(wxb + rowoff + o);
              const unsigned long long au = (unsigned long long)uniform((uint32_t)a) | ((unsigned long long)uniform((uint32_t)(a >> 32)) << 32);
              asm volatile("s_load_dword %0, %1, 0x0" : "+s"(sink) : "s"(au));
            }
          }
        }
      }
      __builtin_amdgcn_s_barrier();  // barrier #itp
    }
    __builtin_amdgcn_s_barrier();  // final barrier
    asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(sink));
    return;
  }

  // =========================================================================
  // waves 0-3, QUAD: row tiles of at most 4 rows.  With K split over the four waves (below), a step's chain runs
  // through LDS: partial tiles out, a barrier, sixteen partial values back in and added up, and only one of the four
  // waves gates real rows.  Here wave w owns units 4 w .. 4 w + 3 of the workgroup's 16 with all four gates (16
  // columns) and the WHOLE of K: it polls the whole h tile of the group (4 rows x dh, 16 bytes per lane from the 16
  // lanes whose MFMA row is a real one), multiplies, and gates its own 16 elements; nothing crosses between the waves.
  // The batch rows sit at MFMA rows 0, 4, 8, 12, so the sum of (row b, column n) arrives in lane group b, lane n, and
  // the four gates of a unit meet in the unit's lane through three row shifts (no LDS).  K is accumulated in the same
  // four quarters and folded in the same order as everywhere else: the same bits.  The barrier of the step (the
  // feeder's W.x, the drainer's h) is passed in front of the poll.  The exchange ring is [slot][member][4 rows]
  // [16 units]: the group's h of a step is 8 dh bytes in a row.
  // =========================================================================
  if constexpr (QUAD) {
    __builtin_amdgcn_s_setprio(3);
    constexpr int NK = 4 * NCH;                // MFMA k-steps over the head dim (dh = 32 NK)
    const int q = lane >> 4, r16 = lane & 15;
    uint4 rreg[NK];
    {
      const int a = a0 + 4 * wave + (r16 & 3);
      const long long rowoff = ((long long)head * 4 * dh + (long long)(r16 >> 2) * dh + a) * dh;
#pragma unroll
      for (int ks = 0; ks < NK; ++ks) {
        const long long off = rowoff + ks * 32 + q * 8;
        if (p.r_bf16) {
          rreg[ks] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.r) + off);
        } else {
          const float4 lo = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(p.r) + off);
          const float4 hi = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(p.r) + off + 4);
          rreg[ks] = uint4{pack_bf16x2(lo.x, lo.y), pack_bf16x2(lo.z, lo.w), pack_bf16x2(hi.x, hi.y), pack_bf16x2(hi.z, hi.w)};
        }
      }
    }
    // gating role: lane group = batch row of the tile, lanes 0-3 of the group = the wave's four units
    const int gb = q, gu = 4 * wave + (r16 & 3);
    const bool gate_lane = r16 < 4;
    const int ua = a0 + gu, col = head * dh + ua;
    const int brow = rowbase + gb;
    float bias_g[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) bias_g[g] = p.bias[((long long)head * 4 + g) * dh + ua];
    CellState st{0.0f, 0.0f, 0.0f, 0.0f};
    if (p.s0 && brow < rend) {
      const long long o = (long long)brow * H + col;
      st.y = p.s0[o]; st.c = p.s0[BH + o]; st.n = p.s0[2 * BH + o]; st.m = p.s0[3 * BH + o];
    }
    bool aborted = false;
    uint32_t max_spins = 0;
    // COEF: what the coefficients of the step before are made of, kept until the next step's poll is out
    GateValues kept{0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    float kept_y = 0.0f, kept_c = 0.0f, kept_n = 0.0f, kept_f = 0.0f;
    auto stage_coefficients = [&](int t) {  // the nine coefficients of step t (see slstm_bwd_prepare_kernel) -> LDS
      if constexpr (COEF) {
        const float omf = __builtin_amdgcn_rcpf(1.0f + __expf(kept_f));  // 1 - sigmoid(f)
        if (gate_lane) {
          float *dst = &cst[t & 3][gb * 16 + gu];
          dst[0 * 64] = kept.og * kept.rn;
          dst[1 * 64] = kept_y * kept.rn;
          dst[2 * 64] = kept.ig * kept.tz;
          dst[3 * 64] = kept.ig;
          dst[4 * 64] = kept.fg * omf * kept_c;
          dst[5 * 64] = kept.fg * omf * kept_n;
          dst[6 * 64] = kept.ig * (1.0f - kept.tz * kept.tz);
          dst[7 * 64] = (1.0f - kept.og) * kept_y;
          dst[8 * 64] = kept.fg;
        }
      }
    };
#ifdef XS_PROFILE
    long long qprof[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    long long qtick = clock64();
#define XS_QTICK(i) do { const long long now_ = clock64(); qprof[i] += now_ - qtick; qtick = now_; } while (0)
#else
#define XS_QTICK(i) do { } while (0)
#endif
    lds_barrier();  // prologue barrier
    const bool cross = cross_s != 0u;
    constexpr int QTILE = 4 * 16 * 2;          // bytes a member publishes per step
    const int xslot = p.G * QTILE;
    char *const xbase = reinterpret_cast<char *>(p.xbuf) + (long long)gi * kRing * xslot;
    // operand: MFMA row r16 is batch row r16 / 4 when r16 % 4 == 0, nothing otherwise; k-step ks, lane group q: units
    // 32 ks + 8 q .. + 7 = member 2 ks + q / 2, its units 8 (q % 2) .. + 7
    const int arow = rowbase + (r16 >> 2);
    const bool a_lane = (r16 & 3) == 0 && arow < rend;
    const int xl = a_lane ? (q >> 1) * QTILE + (r16 >> 2) * 32 + (q & 1) * 16 : 0x7FFFFF00;
    const long long xo = (long long)member * (QTILE / 2) + gb * 16 + gu;
#ifndef XS_QUAD_PAD
#define XS_QUAD_PAD 4
#endif
    asm volatile(".p2align 5\n\t.rept %0\n\ts_nop 0\n\t.endr" :: "n"(XS_QUAD_PAD));
    for (int t = 0; t < p.T; ++t) {
      const __amdgpu_buffer_rsrc_t hrs = __builtin_amdgcn_make_buffer_rsrc(xbase + ((t + kRing - 1) % kRing) * xslot, 0, xslot, 0x00020000);
      uint16_t *const hcur = reinterpret_cast<uint16_t *>(xbase + (t % kRing) * xslot);
      uint16_t *const hold = reinterpret_cast<uint16_t *>(xbase + ((t + kRing - 2) % kRing) * xslot);
      uint4 areg[NK];
      // The step's barrier and what the gating needs from LDS come FIRST, then one s_sleep, then the poll: whatever
      // stands between the poll's return and the MFMAs is on the chain.  Measured at B 16 x T 2048 x 4 heads of 256 (ms
      // per call): barrier and LDS reads under the poll 1.81, in front of it 1.63, with the s_sleep 1.52 (two of
      // them 1.53 - 1.57, four 1.66).  What the s_sleep gives is not the delay - the same cycles spent in s_nop cost
      // instead (32 cycles 1.61, 64 1.69, 128 1.91), and it does as well behind the poll's issue or in front of the
      // barrier (1.52 - 1.53) - but the issue slots: a wave asleep leaves its SIMD to the feeder, drainer and prefetch
      // waves, which these waves' raised priority otherwise keeps waiting (no s_sleep but priority 0 from the barrier
      // to the poll: 1.53).  Then the loop's start moved over the eight phases of a 32-byte line of code:
      // 1.517 .. 1.573, the best one taken.  (K split over the waves, below: 1.70.)
      const int buf = t & 1;
      float wxv[4];
      XS_QTICK(5);
      lds_barrier();  // barrier #t: W.x of this step is in LDS, the h of two steps ago has been drained
      XS_QTICK(2);
#pragma unroll
      for (int g = 0; g < 4; ++g) wxv[g] = wxs[buf][g][gb * kTileStride + gu];
      const bool row_reset = rfl[t & 3][r16 >> 2] != 0u;   // (the operand's row: it contributes R.0 = 0 exactly)
      const bool gate_reset = rfl[t & 3][gb] != 0u;
#ifndef XS_QUAD_SLEEP
#define XS_QUAD_SLEEP 1
#endif
      if (XS_QUAD_SLEEP > 0) __builtin_amdgcn_s_sleep(XS_QUAD_SLEEP);
      asm volatile("");  // (the compiler keeps what stands in front of this statement in front of the poll)
#ifdef XS_PROFILE
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#endif
      XS_QTICK(1);
      if (t > 0) {
#pragma unroll
        for (int ks = 0; ks < NK; ++ks)
          areg[ks] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(hrs, xl, ks * 2 * QTILE, 16));
        stage_coefficients(t - 1);  // (COEF; while the poll is on its way)
      } else {
#pragma unroll
        for (int ks = 0; ks < NK; ++ks) {
          areg[ks] = make_uint4(0, 0, 0, 0);
          if (a_lane && p.s0) {
            const float *src = p.s0 + (long long)arow * H + head * dh + ks * 32 + q * 8;
            const float4 lo = *reinterpret_cast<const float4 *>(src);
            const float4 hi = *reinterpret_cast<const float4 *>(src + 4);
            areg[ks] = uint4{pack_bf16x2(lo.x, lo.y), pack_bf16x2(lo.z, lo.w), pack_bf16x2(hi.x, hi.y), pack_bf16x2(hi.z, hi.w)};
          }
        }
      }
      if (t > 0 && !aborted) {
        uint32_t spins = 0;
        for (;;) {
          uint32_t ma = 0u;
#pragma unroll
          for (int ks = 0; ks < NK; ++ks) ma = mark_join<true>(ma, chunk_mark<true>(areg[ks]));
          if (__builtin_amdgcn_ballot_w64(mark_has_sentinel<true>(ma)) == 0ull) break;
#pragma unroll
          for (int ks = 0; ks < NK; ++ks)
            areg[ks] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(hrs, xl, ks * 2 * QTILE, 16));
          spins += 1;
          if ((spins & 1023u) == 0u && __hip_atomic_load(&p.status->aborted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) {
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
        qprof[6] += spins;
#endif
      }
      XS_QTICK(0);
      if (__builtin_amdgcn_ballot_w64(row_reset) != 0ull) {
#pragma unroll
        for (int ks = 0; ks < NK; ++ks)
          if (row_reset) areg[ks] = make_uint4(0, 0, 0, 0);
      }
      // the four quarters of K, each its own chain from zero, folded in the order of the other kernels' waves
      f32x4 acc[4];
#pragma unroll
      for (int w4 = 0; w4 < 4; ++w4) acc[w4] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int c = 0; c < NCH; ++c)
#pragma unroll
        for (int w4 = 0; w4 < 4; ++w4)
          acc[w4] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, areg[w4 * NCH + c]),
                                                            __builtin_bit_cast(bf16x8, rreg[w4 * NCH + c]), acc[w4], 0, 0, 0);
      float mine = acc[0][0];
      mine += acc[1][0];
      mine += acc[2][0];
      mine += acc[3][0];
      // lane (row, gate g, unit u) -> the unit's lane (row, 0, u): lanes 4, 8, 12 further on in the row of 16
      const int mi = __float_as_int(mine);
      const float ry1 = __int_as_float(__builtin_amdgcn_update_dpp(0, mi, 0x104, 0xF, 0xF, true));  // row_shl:4
      const float ry2 = __int_as_float(__builtin_amdgcn_update_dpp(0, mi, 0x108, 0xF, 0xF, true));  // row_shl:8
      const float ry3 = __int_as_float(__builtin_amdgcn_update_dpp(0, mi, 0x10C, 0xF, 0xF, true));  // row_shl:12
      const float raw0 = (wxv[0] + mine) + bias_g[0], raw1 = (wxv[1] + ry1) + bias_g[1];
      const float raw2 = (wxv[2] + ry2) + bias_g[2], raw3 = (wxv[3] + ry3) + bias_g[3];
#ifdef XS_PROFILE
      asm volatile("" :: "v"(raw0), "v"(raw1), "v"(raw2), "v"(raw3));
#endif
      XS_QTICK(7);
      if (gate_reset) st = CellState{0.0f, 0.0f, 0.0f, 0.0f};
      if constexpr (COEF) {
        kept_c = st.c; kept_n = st.n; kept_f = raw1;
        slstm_pointwise_keep(raw0, raw1, raw2, raw3, st, kept);
        kept_y = st.y;
      } else {
        slstm_pointwise(raw0, raw1, raw2, raw3, st);
      }
      const float y = st.y;
#ifdef XS_PROFILE
      asm volatile("" :: "v"(y));
#endif
      XS_QTICK(3);
      if (gate_lane) {
        const uint16_t v = (uint16_t)float_to_bf16_bits(y);
        if (cross) {
          __hip_atomic_store(hcur + xo, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(hold + xo, (uint16_t)kSentinel16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
          hcur[xo] = v;
          hold[xo] = (uint16_t)kSentinel16;
        }
        hst[t & 3][gb * 16 + gu] = y;
      }
#pragma unroll
      for (int ks = 0; ks < NK; ++ks)  // (the operand registers stay reserved to the end of the iteration)
        asm volatile("" :: "v"(areg[ks].x), "v"(areg[ks].y), "v"(areg[ks].z), "v"(areg[ks].w));
      XS_QTICK(4);
    }
    if (COEF && p.T > 0) stage_coefficients(p.T - 1);
    for (int j = NIT; j < NITpad; ++j) lds_barrier();  // padding iterations of the feeder
    lds_barrier();                                     // final barrier
#ifdef XS_PROFILE
    // slots: 0 poll (issue to complete operand), 1 LDS reads + s_sleep, 2 barrier, 3 gating, 4 publication + staging,
    // 5 loop top, 6 polls repeated, 7 MFMAs + fold + row shifts
    if (lane == 0 && member == 0 && gi == 0) {
      long long *dst = reinterpret_cast<long long *>(p.wg_xcc + kStampWord) + wave * 8;
      for (int i = 0; i < 8; ++i) dst[i] = qprof[i];
    }
#endif
    const bool poisoned = __hip_atomic_load(&p.status->aborted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
    if (gate_lane && brow < rend) {
      const long long o = (long long)brow * H + col;
      if (poisoned) st = CellState{kPoison, kPoison, kPoison, kPoison};
      p.s_out[o] = st.y; p.s_out[BH + o] = st.c; p.s_out[2 * BH + o] = st.n; p.s_out[3 * BH + o] = st.m;
    }
    if (lane == 0 && max_spins) atomicMax(&p.status->max_spins, max_spins);
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

  // exchange ring layout [head group][slot][row tile][member][16 rows][16 units]: what a group
  // publishes for one row tile is contiguous (512 B per member for bf16), which spreads the polls
  // of an iteration over all L2 channels (measured: lines 256 B .. 2 KiB apart are served 1.5x
  // faster than lines 4 KiB or more apart)
  constexpr int XBLOCK = ROWS * 16 * ESZ;            // bytes one member publishes per step
  constexpr int XTILE = 16 * 16 * ESZ;               // ... per row tile
  const int xslot = p.G * XBLOCK;                    // bytes one group publishes per step
  char *const xbase = reinterpret_cast<char *>(p.xbuf) + (long long)gi * kRing * xslot;

  // How h_{t-1} is fetched depends on the number of row tiles per workgroup:
  //   MT == 1  nothing can be fetched early (the peers publish the tile at the end of their current
  //            iteration): two staggered polls in flight, see below;
  //   MT == 2  the polls of the NEXT (t, mt) iteration are issued right after the MFMAs of the
  //            current one have consumed the operand registers (the peers published that tile one
  //            iteration ago);
  // The completion test, the re-arm and their order are the same in both.
  uint4 areg[NCH];
  bool prefetched = false;
  // poll address of chunk c of row tile mt = per-lane part (one register) + a compile-time constant:
  // unit k of row r of row tile mt lives at [mt][member k/16][r][k%16]
  const int xlane = ((wave * KW + q * EPC) >> 4) * XTILE + (r16 * 16 + ((q * EPC) & 15)) * ESZ;
  const int xtile_stride = p.G * XTILE;
  auto xconst = [&](int c, int mt_) { return ((c * 4 * EPC) >> 4) * XTILE + mt_ * xtile_stride; };
  // Where the time loop of the compute waves starts relative to a 32-byte boundary of the code moves the time per step
  // by 3 % (config 2, all eight phases measured twice: 1.690 / 1.707 / 1.717 / 1.718 / 1.720 / 1.738 / 1.751 / 1.752 ms,
  // the same 32 bytes further on): the instruction fetch of a wave that comes out of a poll or a barrier.  Without the
  // alignment the phase is whatever the code in front of the loop leaves (one more store there cost 1 %); with it the
  // phase is chosen, per variant where one has been measured.
#ifndef XS_LOOP_PAD
#define XS_LOOP_PAD ((BF16 && NCH == 2 && MT == 1 && FULL && !BURST && !FMAC) ? 3 : 0)
#endif
  asm volatile(".p2align 5\n\t.rept %0\n\ts_nop 0\n\t.endr" :: "n"(XS_LOOP_PAD));
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
      uint32_t needmask[NCH];
      const bool row_ok = (FULL && MT > 1) ? true : arow < rend;
      // a row that starts a document contributes R.0 = 0 exactly.  (Fetching this flag behind the poll's issue, so that
      // the poll goes out an LDS round trip earlier, measured 2.5 % SLOWER: an earlier poll more often comes back
      // incomplete, and the next one is a full round trip away.)
      const bool row_reset = rfl[it & 3][r16] != 0u;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int k0 = wave * KW + c * 4 * EPC + q * EPC;
        if (!(MT > 1 && prefetched)) areg[c] = make_uint4(0, 0, 0, 0);
        need[c] = FULL ? true : (row_ok && k0 < dh);
        needmask[c] = need[c] ? 0xFFFFFFFFu : 0u;  // (masks, not selects: the tests below stay straight-line code)
      }
      // ---- 2. (defined here, used below) partial R.h over this wave's K slab, all four gates, from the operand
      //      registers given; rows that start a document and chunks that are not needed count as zeros
      f32x4 acc[4];
      auto multiply = [&](uint4 (&op)[NCH]) {
        // (a whole wave rarely has anything to clear: one uniform branch instead of 4 selects per chunk)
        bool clear_any = row_reset;
#pragma unroll
        for (int c = 0; c < NCH; ++c) clear_any |= !need[c];
        if (__builtin_amdgcn_ballot_w64(clear_any) != 0ull) {
#pragma unroll
          for (int c = 0; c < NCH; ++c)
            if (row_reset || !need[c]) op[c] = make_uint4(0, 0, 0, 0);
        }
        XS_TICK(0);
#pragma unroll
        for (int g = 0; g < 4; ++g) acc[g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        if constexpr (FMAC) {
          float sum[4][4];  // [gate][row]: this lane's column, this lane group's slice of K
#pragma unroll
          for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int r = 0; r < 4; ++r) sum[g][r] = 0.0f;
#pragma unroll
          for (int c = 0; c < NCH; ++c) {
            float w[4][EPC];  // the weights of this lane's column
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              const uint32_t rw[4] = {rreg[g][c].x, rreg[g][c].y, rreg[g][c].z, rreg[g][c].w};
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                if (BF16) { w[g][2 * e] = bf16_bits_to_float(rw[e] & 0xFFFFu); w[g][2 * e + 1] = __uint_as_float(rw[e] & 0xFFFF0000u); }
                else w[g][e] = __uint_as_float(rw[e]);
              }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              if (r >= rend - rowbase) break;  // (wave-uniform: only the rows that exist cost anything)
              // the inputs of row r for this lane group's slice of K sit in lane 16 q + r
              const uint32_t hw[4] = {(uint32_t)__shfl((int)op[c].x, (lane & 48) + r), (uint32_t)__shfl((int)op[c].y, (lane & 48) + r),
                                      (uint32_t)__shfl((int)op[c].z, (lane & 48) + r), (uint32_t)__shfl((int)op[c].w, (lane & 48) + r)};
              float hx[EPC];
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                if (BF16) { hx[2 * e] = bf16_bits_to_float(hw[e] & 0xFFFFu); hx[2 * e + 1] = __uint_as_float(hw[e] & 0xFFFF0000u); }
                else hx[e] = __uint_as_float(hw[e]);
              }
#pragma unroll
              for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int e = 0; e < EPC; ++e) sum[g][r] = fmaf(hx[e], w[g][e], sum[g][r]);
            }
          }
          // add the four lane groups' slices; the result tile keeps the MFMA's layout (rows 4q .. 4q+3 of column r16)
#pragma unroll
          for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              float v = sum[g][r];
              v += __shfl_xor(v, 16);
              v += __shfl_xor(v, 32);
              acc[g][r] = q == 0 ? v : 0.0f;
            }
          return;
        }
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
          if (BF16) {
            const bf16x8 av = __builtin_bit_cast(bf16x8, op[c]);
#pragma unroll
            for (int g = 0; g < 4; ++g)
              acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, __builtin_bit_cast(bf16x8, rreg[g][c]), acc[g], 0, 0, 0);
          } else {
            const uint32_t aw[4] = {op[c].x, op[c].y, op[c].z, op[c].w};
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
      };
      bool multiplied = false;
      if (t == 0) {
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
          const int k0 = wave * KW + c * 4 * EPC + q * EPC;
          if ((FULL ? row_ok : need[c]) && p.s0) {
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
        if (MT == 1) {
          multiply(areg);
          multiplied = true;
        }
      } else {
        if (MT == 1) {
          // ONE poll in flight, re-issued when it comes back incomplete.  With W.x out of the way of the polls
          // (prefetch waves) a poll takes 200 to 300 cycles and finds everything in place in 92 % of the steps:
          // the peers' h is in the L2 before this wave's own loop has come round.  A second poll half a round
          // trip behind the first, which paid while polls took 600 cycles, then only costs: the compiler
          // parks a wait for it behind the first MFMA (10 % of a step at config 2, and the time per step jumped
          // by +-15 % with the distance between the two and with unrelated changes to the code).  A pause in front of
          // the poll does not pay either (64 cycles: the same; 128: 2 % slower; 192: 6 % slower).
          // Lanes whose batch row does not exist ask for an offset past the descriptor's end: zeros, no memory
          // traffic.  The decision is wave-uniform (ballot) and the MFMAs are issued right where the set is
          // found complete.
          const int xl = row_ok ? xlane : 0x7FFFFF00;
#pragma unroll
          for (int c = 0; c < NCH; ++c)
            areg[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(hrs, xl, xconst(c, mt), 16));
          uint32_t spins = 0;
          if (!aborted) {
            for (;;) {
              uint32_t ma = 0u;
#pragma unroll
              for (int c = 0; c < NCH; ++c) ma = mark_join<BF16>(ma, chunk_mark<BF16>(areg[c]) & needmask[c]);
              if (__builtin_amdgcn_ballot_w64(mark_has_sentinel<BF16>(ma)) == 0ull) {
                multiply(areg);
                multiplied = true;
                break;
              }
#pragma unroll
              for (int c = 0; c < NCH; ++c)
                areg[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(hrs, xl, xconst(c, mt), 16));
              spins += 1;
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
        // first look at everything at once: one mark over all chunks this lane needs
        uint32_t mark = 0u;
        if (MT != 1) {  // (with one row tile the loop above has seen a complete set, or given up)
#pragma unroll
          for (int c = 0; c < NCH; ++c) mark = mark_join<BF16>(mark, chunk_mark<BF16>(areg[c]) & needmask[c]);
        }
        if (MT != 1 && !aborted && mark_has_sentinel<BF16>(mark)) {
          uint32_t spins = 0;
          // The loop ENDS with the test of what it loaded.  The compiler lays a loop with lane-dependent exits out
          // so that the wave leaves it at the bottom; with the reloads at the bottom it took the operand registers
          // for possibly still being loaded behind the loop and put a wait for ALL outstanding loads (the next
          // tile's requests included) in front of the MFMAs.  The two ways out on a failure leave before a reload.
          bool bad[NCH];
          bool any_bad;
          auto test_chunks = [&]() {
            any_bad = false;
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
              bad[c] = need[c] && (BF16 ? chunk_has_sentinel_bf16(areg[c]) : chunk_has_sentinel_f32(areg[c]));
              any_bad |= bad[c];
            }
          };
          test_chunks();
          while (any_bad) {
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
#pragma unroll
            for (int c = 0; c < NCH; ++c)
              if (bad[c])
                areg[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(hrs, xlane, xconst(c, mt), 16));
            test_chunks();
          }
          max_spins = spins > max_spins ? spins : max_spins;
#ifdef XS_PROFILE
          prof[6] += spins;
#endif
        }
      }
      if (MT == 1) {
        // (every path above has multiplied, except a wait that ran out: nothing may refer to the poll registers
        // behind the loop, or the compiler keeps copies of them alive across it and waits for the poll in flight)
        if (!multiplied) {
#pragma unroll
          for (int g = 0; g < 4; ++g) acc[g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
      } else if (!multiplied) {
        multiply(areg);
      }

      if (MT > 1) {
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
      // Every lane stores, every iteration: lanes outside the batch or the head write words of their own
      // block that nobody polls, and the re-arm of steps 0 and 1 hits slots that still hold the pattern.
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
      hst[it & 3][tid] = y;
      if (MT == 1) {
        // (the operand registers stay reserved to the end of the iteration: measured as fast or faster)
#pragma unroll
        for (int c = 0; c < NCH; ++c)
          asm volatile("" :: "v"(areg[c].x), "v"(areg[c].y), "v"(areg[c].z), "v"(areg[c].w));
      }
      XS_TICK(4);
    }
  }
  for (int j = NIT; j < NITpad; ++j) lds_barrier();  // padding iterations of the feeder
  lds_barrier();                                     // final barrier
#ifdef XS_PROFILE
  if (lane == 0 && member == 0 && gi == 0) {
    long long *dst = reinterpret_cast<long long *>(p.wg_xcc + kStampWord) + wave * 8;
    for (int i = 0; i < 8; ++i) dst[i] = prof[i];
  }
#endif

  // ---- final state (NaN when a bounded wait ran out anywhere in the call: see the drainer)
  const bool poisoned = __hip_atomic_load(&p.status->aborted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int brow = rowbase + mt * 16 + pb;
    if (unit_ok && brow < rend) {
      const long long o = (long long)brow * H + col;
      if (poisoned) st[mt] = CellState{kPoison, kPoison, kPoison, kPoison};
      p.s_out[o] = st[mt].y; p.s_out[BH + o] = st[mt].c; p.s_out[2 * BH + o] = st[mt].n; p.s_out[3 * BH + o] = st[mt].m;
    }
  }
  if (lane == 0 && max_spins) atomicMax(&p.status->max_spins, max_spins);
}

}  // namespace
