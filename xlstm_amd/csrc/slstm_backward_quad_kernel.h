// The reverse pass of the sLSTM backward for row tiles of 4 batch rows (bf16, head dims 64, 128, 256).  Included by
// slstm_hip.hip only (one translation unit), after slstm_backward_kernels.h, whose parameter block, exchange ring
// protocol, arm kernel and prefetching workgroups it shares.
//
// slstm_bwd_split_kernel walks 16 rows per workgroup: two elements per thread in the gradient of a step, 32 KiB of gate
// deltas per workgroup and poll round, partial tiles of 16 rows through LDS, two barriers.  A batch of few rows (16 at
// four heads, say) then keeps 16 compute units busy and the step is as long as its longest wave.  Here a workgroup
// owns 4 rows x 64 units: one element per thread in four of its eight compute waves, 8 KiB of deltas per group and
// round of which a wave polls 1 KiB, partial tiles of 4 rows, ONE barrier per step, four times the workgroups.  What
// stays: a head over S = dh / 64 workgroups by output unit, a wave holding its eighth of K of the slice of R transposed in
// registers for the whole call, deltas polled straight into MFMA operand registers, words that are data or the all-ones
// pattern, the publisher re-arming its words of two steps ago, bounded waits.
//
// K is ordered (unit of the head, gate): the four deltas of an element are 8 bytes in a row and a thread publishes them
// with one store; a group's slot is [4 rows][K] bf16, a wave's store 512 bytes in a row.  Wave w multiplies k-steps
// 4w ... 4w + 3 (at head dim 256), i.e. the deltas of units 32w ... 32w + 31 of the head: it polls ONE publisher's
// half.  The four batch rows sit at MFMA rows 0, 4, 8, 12 (the rows between are zero), so the sum of (row b, column n)
// arrives in lane group b, lane n, first element.
#pragma once

namespace {

constexpr int kBwdQuadCoefBytes = 4 * 9 * 64 * 4;  // a step's coefficients of a workgroup: 4 rows, 9 of them, 64 units
// a slot of the feeder waves: the coefficients, d_h (4 rows of 128 bytes in a landing zone of 1 KiB), the reset flags of the
// 4 rows as words (in a landing zone of 256 bytes)
constexpr int kBwdQuadSlot = kBwdQuadCoefBytes + 1024 + 256;
constexpr int kBwdQuadSlots = 8;
constexpr int kBwdQuadFeeders = 4;                 // feeder waves: wave 8 + f brings the inputs of the steps n = f (mod 4)
constexpr int kBwdQuadDepth = 6;                   // steps the feeder waves request ahead
static_assert(kBwdQuadDepth >= 3 && kBwdQuadDepth <= kBwdQuadSlots && kBwdQuadDepth <= kBwdQuadFeeders + 2, "feeder depth");
constexpr int kBwdQuadThreads = (8 + kBwdQuadFeeders) * 64;
constexpr int kBwdQuadPart = 4 * kBwdPartStride;   // floats of a wave's partial tile
constexpr int bwd_quad_lds_bytes() { return 2 * 8 * kBwdQuadPart * 4 + kBwdQuadSlots * kBwdQuadSlot; }

// s_sleep units (64 cycles each) in front of a wave's first look at the step's deltas: of the waves that do not form the
// step's gradient (they leave the barrier with nothing else to do, a quarter of a step before anything is published),
// and of the waves that have just published.  Reverse kernel at B 16, T 2048, 4 heads of 256, ms: (0, 0) 2.43, (4, 0)
// 2.42, (6, 2) 2.31, (8, 2) 2.20, (8, 4) 2.17, (10, 0) 2.24, (12, 2) 2.20, (16, 4) 2.33; at half the batch (one group per
// XCD) 2.13, 2.21, 2.09, 2.02, 2.09, 2.04, 2.10, 2.32.  A look that comes back incomplete costs its whole round trip, and
// so does every cycle slept past the arrival.
constexpr int kBwdQuadSleepIdle = 8, kBwdQuadSleepPublished = 2;

template <int S, bool DWX16 = false>  // S workgroups per group, dh = 64 S; DWX16: d_wx takes the gate deltas rounded to bf16
__global__ __launch_bounds__(kBwdQuadThreads) void slstm_bwd_quad_kernel(BwdSplitParams p) {
  constexpr int UW = 64;
  constexpr int dh = S * UW;
  constexpr int K = 4 * dh;
  constexpr int KSTEPS = K / 8 / 32;          // MFMA k-steps of a wave: its eighth of K
  constexpr int SLOT = 4 * K * 2;             // bytes of a group's slot
  constexpr int PART = kBwdQuadPart;
  extern __shared__ __attribute__((aligned(16))) float part[];  // [2][8 waves][4 rows][kBwdPartStride], then the feeder's slots
  const int H = p.NH * dh;
  const long long BH = (long long)p.B * H;
  const int ntiles = (p.B + 3) >> 2;
  const int ngroups = p.NH * ntiles;
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
#ifdef XS_PROFILE
  const long long wg_start = wall_clock64();
#endif
  if (local >= p.main_locals) {
    bwd_tile_prefetch<true, S, 4, kBwdQuadDepth>(p, xcd, local - p.main_locals, (int)(gridDim.x >> 3) - p.main_locals);
    return;
  }
  const int group = (local / S) * 8 + xcd, s = local % S;
  if (group >= ngroups) return;
  const int head = group % p.NH;
  const int row0 = (group / p.NH) * 4;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, q = lane >> 4, r16 = lane & 15;
  char *const feed = reinterpret_cast<char *>(part + 2 * 8 * PART);
  bwd_note_placement(p, group);
  // look_step[w]: 1 + the step of the call whose first look compute wave w has issued (for the feeder waves, see there)
  __shared__ volatile int look_step[8];
  if (tid < 8) look_step[tid] = 0;
  const int rows_there = p.B - row0 < 4 ? p.B - row0 : 4;
  if (wave >= 8) {
    // ---- the feeder waves: the inputs of step n into slot n % 8, kBwdQuadDepth steps ahead, with loads that write LDS
    //      directly (no registers; their waits are written by hand)
    const uint32_t feed_lds = (uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)feed);
    const long long coef_piece0 = (((long long)(row0 >> 2) * p.NH + head) * S + s) * kBwdQuadCoefBytes;  // + t * coef_step
    const long long coef_step = (long long)ntiles * p.NH * S * kBwdQuadCoefBytes;
    const uint32_t dh_records = (uint32_t)(((long long)(rows_there - 1) * H + 64) * 2);
    const int dh_voff = (lane >> 3) * H * 2 + (lane & 7) * 16;  // (rows 4 to 7 lie past the records: zeros into the landing zone)
    const unsigned long long fb = reinterpret_cast<unsigned long long>(p.reset ? p.reset + (long long)row0 * p.reset_sb : reinterpret_cast<const uint8_t *>(p.coef));
    const uint32_t flag_records = p.reset ? (uint32_t)((long long)(rows_there - 1) * p.reset_sb + p.T) : 0u;  // (no mask: every flag reads zero)
    const u32x4_t frs = {uniform((uint32_t)fb), uniform((uint32_t)(fb >> 32) & 0xFFFFu), uniform(flag_records), 0x00020000u};
    const uint32_t flag_lane = lane < rows_there ? (uint32_t)(lane * p.reset_sb) : 0x7FFFFF00u;
    auto request = [&](int n) {
      const int t = p.T - 1 - n;
      const unsigned long long cb = reinterpret_cast<unsigned long long>(p.coef) + (unsigned long long)(coef_piece0 + t * coef_step);
      const u32x4_t crs = {uniform((uint32_t)cb), uniform((uint32_t)(cb >> 32) & 0xFFFFu), (uint32_t)kBwdQuadCoefBytes, 0x00020000u};
      const uint32_t slot = feed_lds + (n & (kBwdQuadSlots - 1)) * kBwdQuadSlot;
#pragma unroll
      for (int k = 0; k < 9; ++k) bwd_fetch_to_lds_b128(crs, uniform(slot + k * 1024), (uint32_t)(k * 1024 + lane * 16));
      const unsigned long long db = reinterpret_cast<unsigned long long>(p.d_h) + (unsigned long long)((((long long)t * p.B + row0) * H + (long long)head * dh + s * UW) * 2);
      const u32x4_t drs = {uniform((uint32_t)db), uniform((uint32_t)(db >> 32) & 0xFFFFu), dh_records, 0x00020000u};
      bwd_fetch_to_lds_b128(drs, uniform(slot + kBwdQuadCoefBytes), (uint32_t)dh_voff);
      bwd_fetch_to_lds_u8(frs, uniform(slot + kBwdQuadCoefBytes + 1024), lane < rows_there ? flag_lane + (uint32_t)t : 0x7FFFFF00u);
    };
    // Feeder wave f owns the steps n = f (mod kBwdQuadFeeders): it asks for step n's inputs behind barrier A(n - depth)
    // and waits for them - for everything it has in flight - in front of barrier A(n - 2), behind which the compute
    // waves read them; its next request goes out behind that barrier at the earliest (depth <= feeders + 2), so it never
    // has two requests in flight and no wait needs a count.  (One wave with several requests in flight and counted
    // waits, `s_waitcnt vmcnt(33)` for "all but the last three requests", waited a request's whole latency every step:
    // the wait counter of a wave has 6 bits, and these loads seem to weigh more than one each.)
    const int f = wave - 8;
#ifdef XS_PROFILE
    long long fprof[6] = {0, 0, 0, 0, 0, 0}, ftick = clock64();
#endif
    for (int n = f; n < kBwdQuadDepth && n < p.T; n += kBwdQuadFeeders) request(n);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (among them the inputs of steps 0 and 1)
    __syncthreads();           // P: the compute waves read the inputs of steps 0 and 1 behind it
    for (int m = 0; m < p.T; ++m) {
      // in front of barrier A(m) the inputs of step m + 2 are in place: the compute waves read them behind it
      if ((m + 2) % kBwdQuadFeeders == f) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#ifdef XS_PROFILE
      fprof[4] += clock64() - ftick;  // (the wait, if it was this wave's turn)
#endif
      __syncthreads();  // A(m)
#ifdef XS_PROFILE
      fprof[5] += clock64() - ftick;  // (the step)
      ftick = clock64();
#endif
      const int n = m + kBwdQuadDepth;  // (into the slot of step n - 8, read in front of A(n - 9))
      if (n % kBwdQuadFeeders == f && n < p.T) {
        // The request goes out behind the compute waves' looks at the next step's deltas: a compute unit returns its
        // loads in the order they were issued, and these take longer than a look.  (A bounded wait: nobody depends on it.)
        if (p.cut == 0 && m + 1 < p.T) {
          for (int spin = 0; spin < 512; ++spin) {
            const int seen = lane < 8 ? look_step[lane] : 0x7FFFFFFF;
            if (__builtin_amdgcn_ballot_w64(seen < m + 2) == 0ull) break;
            __builtin_amdgcn_s_sleep(1);
          }
        }
#ifdef XS_PROFILE
        fprof[2] += clock64() - ftick;  // (the compute waves' looks are out)
        if ((m & 63) >= 32 && (m & 63) < 36) {  // (measurement: how long a request takes; sampled, every wait below is in the way)
          const long long f0 = clock64();
          request(n);
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          fprof[0] += clock64() - f0; fprof[1] += 1;
        } else
#endif
        request(n);
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#ifdef XS_PROFILE
    __syncthreads();  // (the compute waves have cleared the m plane of d_s0)
    if (group == 0 && s == 0 && lane == 0 && f == 0 && (long long)p.B * H >= 64) {
      long long *out = reinterpret_cast<long long *>(p.d_s0 + 3ll * p.B * H) + 24;
      for (int i = 0; i < 6; ++i) out[i] = fprof[i];
    }
#endif
    return;
  }
  // ---- this wave's share of the workgroup's slice of R transposed -> registers, once
  uint4 bq[KSTEPS][4];
  {
    const char *base = reinterpret_cast<const char *>(p.r_ts) + ((((long long)(head * S + s) * 8 + wave) * KSTEPS * 4 * 64) << 4);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) bq[ks][cb] = *reinterpret_cast<const uint4 *>(base + (((ks * 4 + cb) * 64 + lane) << 4));
  }
  // ---- the thread's element (waves 0 to 3): row `wave` of the tile, unit s 64 + lane of the head
  const bool grad_wave = wave < 4;
  const int prow = wave & 3, pu = lane;
  const int row = row0 + prow;
  const bool there = grad_wave && row < p.B;
  const long long ecol = (long long)head * dh + s * UW + pu;
  float dy = 0.0f, dc = 0.0f, dn = 0.0f;
  if (there && p.d_s_final) {
    const long long o = (long long)row * H + ecol;
    dy = p.d_s_final[o]; dc = p.d_s_final[BH + o]; dn = p.d_s_final[2 * BH + o];
  }
  const int pub_off = prow * (K * 2) + (s * UW + pu) * 8;
  const int wave_u = (int)uniform((uint32_t)wave);
  // + k-step * 64; the lanes between the real rows ask past the end of the slot and get zeros without a request to the L2
  // (with copies of the real rows there a look moved four times the bytes through the compute unit's one return path)
  const int poll_off = (r16 & 3) == 0 ? (r16 >> 2) * (K * 2) + q * 16 : 0x7FFFFF00;
  char *const ring = reinterpret_cast<char *>(p.xch) + (long long)group * SLOT;
  const long long ring_stride = (long long)ngroups * SLOT;
  const bool cut = p.cut != 0;
  float c9[9], dht = 0.0f;
  bool restart = false;
  auto read_inputs = [&](int n) {  // the inputs of step n of the call, from the feeder's slot
    const char *slot = feed + (n & (kBwdQuadSlots - 1)) * kBwdQuadSlot;
    const float *src = reinterpret_cast<const float *>(slot) + prow * (9 * 64) + pu;
#pragma unroll
    for (int j = 0; j < 9; ++j) c9[j] = src[j * 64];
    dht = __uint_as_float((uint32_t)*reinterpret_cast<const uint16_t *>(slot + kBwdQuadCoefBytes + prow * 128 + pu * 2) << 16);
    restart = *reinterpret_cast<const uint32_t *>(slot + kBwdQuadCoefBytes + 1024 + prow * 4) != 0u;
  };
  bool gave_up = false, zero_dy = false;
#ifdef XS_PROFILE
  // measurement build: when a wave passes fixed points of the loop, in cycles since it left the step's barrier, summed
  // over the steps; waves 0 (forms the gradient, polls its own workgroup), 4 and 6 (poll only; 6 polls another workgroup)
  // of the first workgroup leave theirs in the m plane of d_s0
  long long bprof[8] = {0, 0, 0, 0, 0, 0, 0, 0}, btick = clock64(), blook = 0;
#define XS_BTICK(i) do { const long long now_ = clock64(); bprof[i] += now_ - btick; if ((i) == 5) btick = now_; } while (0)
#else
#define XS_BTICK(i) do { } while (0)
#endif
  auto add_up = [&](int n) {  // what reaches y of the thread's element from step n of the call: the eight partial results, in the order of the waves
    const float *tiles = part + (n & 1) * 8 * PART + prow * kBwdPartStride + pu;
    float sum = 0.0f;
#pragma unroll
    for (int w = 0; w < 8; ++w) sum += tiles[w * PART];
    return sum;
  };
  __syncthreads();  // P
  if (grad_wave) read_inputs(0);
  // (where the loop starts relative to a 32-byte boundary of the code is left to the compiler: no phase measured better)
  for (int n = 0; n < p.T; ++n) {
    const int t = p.T - 1 - n;
    if (grad_wave) {
      if (n > 0) dy = (cut || zero_dy) ? 0.0f : add_up(n - 1);
#ifdef XS_PROFILE
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#endif
      XS_BTICK(0);
      // ---- the gradient of the step for the thread's element
      float delta[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if (there) {
        const float dyt = dht + bwd_recurrent_dy(dy, p.clip, n == 0);
        const float dct = dc + dyt * c9[0];
        const float dnt = dn - dyt * c9[1];
        delta[0] = c9[2] * dct + c9[3] * dnt;
        delta[1] = c9[4] * dct + c9[5] * dnt;
        delta[2] = c9[6] * dct;
        delta[3] = c9[7] * dyt;
        dc = restart ? 0.0f : c9[8] * dct;  // (a row that starts a document at t took nothing from the step before)
        dn = restart ? 0.0f : c9[8] * dnt;
      }
      zero_dy = restart;
      if (!cut) {
        // ---- publish (rows outside the batch: zeros), re-arm the words of two steps ago
        // (the pattern stays unique: a half of all ones, which only a NaN can give, becomes 0xFFFE, a NaN as well)
        const u16x2_t lo = __builtin_elementwise_min(__builtin_bit_cast(u16x2_t, pack_bf16x2(delta[0], delta[1])), u16x2_t{0xFFFE, 0xFFFE});
        const u16x2_t hi = __builtin_elementwise_min(__builtin_bit_cast(u16x2_t, pack_bf16x2(delta[2], delta[3])), u16x2_t{0xFFFE, 0xFFFE});
        // (plain stores: as stores of device scope, which the forward's kernels use, they measured 0.1 to 0.5 ms slower here)
        *reinterpret_cast<uint2 *>(ring + (n % kBwdRing) * ring_stride + pub_off) = uint2{__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi)};
        *reinterpret_cast<uint2 *>(ring + ((n + kBwdRing - 2) % kBwdRing) * ring_stride + pub_off) = uint2{0xFFFFFFFFu, 0xFFFFFFFFu};
      }
      XS_BTICK(1);
      // ---- while the deltas are on their way: d_wx, the progress word, the next step's inputs
      //      (with the first look issued in front of these instead of behind them, and a longer sleep in front of it, the
      //      kernel took 2.33 ms at config 2 instead of 2.20: the look then waits for the stores behind it as well)
      if (s == 0 && tid == 0) p.progress[group] = (unsigned int)n;
      if (there) {
        const long long wo = (long long)row * p.d_wx_sb + (long long)t * p.d_wx_st + ecol;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          if constexpr (DWX16) reinterpret_cast<uint16_t *>(p.d_wx)[wo + (long long)g * H] = (uint16_t)(pack_bf16x2(delta[g], 0.0f) & 0xFFFFu);
          else p.d_wx[wo + (long long)g * H] = delta[g];
        }
      }
      if (n + 1 < p.T) read_inputs(n + 1);
      if (!cut && S > 1) __builtin_amdgcn_s_sleep(kBwdQuadSleepPublished);
    } else {
      if (!cut) __builtin_amdgcn_s_sleep(kBwdQuadSleepIdle);
    }
    XS_BTICK(2);
    if (!cut) {
      // ---- delta [4 rows x K/8] . R^T [K/8 x 64] from the A operand registers `a`: the wave's partial result, to LDS.
      //      Two sets of tiles, used in turn: a wave writes the tiles of step n + 2 only after a peer has published step
      //      n + 2, for which that peer needed all of this workgroup's deltas of step n + 1, which were computed from the
      //      sums of step n.
      auto multiply = [&](const u32x4_t (&a)[KSTEPS]) {
        XS_BTICK(3);
        f32x4 acc[4];
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) acc[cb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
          for (int cb = 0; cb < 4; ++cb)
            acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[ks]), __builtin_bit_cast(bf16x8, bq[ks][cb]), acc[cb], 0, 0, 0);
        float *const tiles = part + (n & 1) * 8 * PART + wave * PART + q * kBwdPartStride + r16;
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) tiles[cb * 16] = acc[cb][0];
      };
      // (a negative spin limit is the host's way to make every wait run out at its first look: the error path, forced)
      auto complete = [&](const u32x4_t (&a)[KSTEPS]) {
        uint32_t mark = 0u;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) mark = mark_join<true>(mark, chunk_mark<true>(__builtin_bit_cast(uint4, a[ks])));
        return (__builtin_amdgcn_ballot_w64(mark_has_sentinel<true>(mark)) == 0ull && p.spin_limit >= 0) || gave_up;
      };
      long long spins = 0;
      auto another_round = [&]() {  // false: the wait has run out (or somebody else's has)
#ifdef XS_PROFILE
        bprof[6] += 1;
#endif
        if (++spins > p.spin_limit || ((spins & 255) == 0 && __hip_atomic_load(p.abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
          __hip_atomic_store(p.abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          gave_up = true;
        }
      };
      // ---- the deltas of the wave's eighth of K: polled straight into the A operand registers
      // (two looks in flight half a round trip apart, so that an incomplete one is followed sooner: 0.15 to 0.4 ms slower,
      // as was every variant that asks more often)
      {
        u32x4_t areg[KSTEPS];
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(ring + (n % kBwdRing) * ring_stride, 0, SLOT, 0x00020000);
        constexpr int kPastL1 = 16;  // (the load's scope bits: served by the L2)
        if (lane == 0) look_step[wave] = n + 1;
        for (;;) {
#ifdef XS_PROFILE
          blook = clock64() - btick;
#endif
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks)
            areg[ks] = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rs, poll_off, (wave_u * KSTEPS + ks) * 64, kPastL1));
          if (complete(areg)) break;
          another_round();
        }
#ifdef XS_PROFILE
        bprof[7] += blook;
#endif
        multiply(areg);
      }
    }
    XS_BTICK(4);
    __syncthreads();  // A(n)
    XS_BTICK(5);
  }
  // ---- gradient w.r.t. the initial state (the stabiliser's part is zero by the rule; NaN all over when a wait ran out)
  const bool mixed = S > 1 && !cut && bwd_placement_mixed(p, group);
  if (grad_wave) {
    dy = (cut || zero_dy) ? 0.0f : add_up(p.T - 1);
    if (there) {
      const bool poisoned = mixed || __hip_atomic_load(p.abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
      const long long o = (long long)row * H + ecol;
      p.d_s0[o] = poisoned ? kPoison : dy;
      p.d_s0[BH + o] = poisoned ? kPoison : dc;
      p.d_s0[2 * BH + o] = poisoned ? kPoison : dn;
      p.d_s0[3 * BH + o] = 0.0f;
    }
  }
#ifdef XS_PROFILE
  __syncthreads();
  if (tid == 0 && s == 0) p.progress[group] = 0x40000000u + (unsigned int)(wall_clock64() - wg_start);  // (how long the group took, in 10 ns)
  if (group == 0 && s == 0 && lane == 0 && (wave == 0 || wave == 4 || wave == 6) && BH >= 64) {
    long long *out = reinterpret_cast<long long *>(p.d_s0 + 3 * BH) + (wave == 0 ? 0 : (wave == 4 ? 8 : 16));
    for (int i = 0; i < 8; ++i) out[i] = bprof[i];
  }
#endif
}

}  // namespace
