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
// half.  The four batch rows sit at MFMA rows 0, 4, 8, 12 and the rows between hold copies (a row of the product depends
// on the same row of the operand only), so the sum of (row b, column n) arrives in lane group b, lane n, first element.
#pragma once

namespace {

constexpr int kBwdQuadLoads = 11;                  // loads of one request of the feeder wave
constexpr int kBwdQuadCoefBytes = 4 * 9 * 64 * 4;  // a step's coefficients of a workgroup: 4 rows, 9 of them, 64 units
// a slot of the feeder wave: the coefficients, d_h (4 rows of 128 bytes in a landing zone of 1 KiB), the reset flags of the
// 4 rows as words (in a landing zone of 256 bytes)
constexpr int kBwdQuadSlot = kBwdQuadCoefBytes + 1024 + 256;
constexpr int kBwdQuadSlots = 4;
constexpr int kBwdQuadPart = 4 * kBwdPartStride;   // floats of a wave's partial tile
constexpr int bwd_quad_lds_bytes() { return 2 * 8 * kBwdQuadPart * 4 + kBwdQuadSlots * kBwdQuadSlot; }

#ifndef XS_BQ_SLEEP_IDLE
#define XS_BQ_SLEEP_IDLE 4   // s_sleep units (64 cycles each) of the waves that do not form the step's gradient, in front of their poll
#endif
#ifndef XS_BQ_SLEEP_PUB
#define XS_BQ_SLEEP_PUB 2    // ... of the waves that have just published, in front of theirs
#endif

template <int S>  // S workgroups per group, dh = 64 S
__global__ __launch_bounds__(576) void slstm_bwd_quad_kernel(BwdSplitParams p) {
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
  if (local >= p.main_locals) {
    bwd_prefetch<true, 4>(p, xcd);
    return;
  }
  const int group = (local / S) * 8 + xcd, s = local % S;
  if (group >= ngroups) return;
  const int head = group % p.NH;
  const int row0 = (group / p.NH) * 4;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, q = lane >> 4, r16 = lane & 15;
  char *const feed = reinterpret_cast<char *>(part + 2 * 8 * PART);
  const int rows_there = p.B - row0 < 4 ? p.B - row0 : 4;
  if (wave == 8) {
    // ---- the feeder wave: the inputs of step n into slot n % 4, four steps ahead, with loads that write LDS directly.
    //      Every wait is counted by hand: a request is kBwdQuadLoads loads, and loads return in the order they were issued.
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
      const uint32_t slot = feed_lds + (n & 3) * kBwdQuadSlot;
#pragma unroll
      for (int k = 0; k < 9; ++k) bwd_fetch_to_lds_b128(crs, uniform(slot + k * 1024), (uint32_t)(k * 1024 + lane * 16));
      const unsigned long long db = reinterpret_cast<unsigned long long>(p.d_h) + (unsigned long long)((((long long)t * p.B + row0) * H + (long long)head * dh + s * UW) * 2);
      const u32x4_t drs = {uniform((uint32_t)db), uniform((uint32_t)(db >> 32) & 0xFFFFu), dh_records, 0x00020000u};
      bwd_fetch_to_lds_b128(drs, uniform(slot + kBwdQuadCoefBytes), (uint32_t)dh_voff);
      bwd_fetch_to_lds_u8(frs, uniform(slot + kBwdQuadCoefBytes + 1024), lane < rows_there ? flag_lane + (uint32_t)t : 0x7FFFFF00u);
    };
    // `behind` requests may still be in flight
    auto wait_all_but = [&](int behind) {
      if (behind >= 2) asm volatile("s_waitcnt vmcnt(22)" ::: "memory");
      else if (behind == 1) asm volatile("s_waitcnt vmcnt(11)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };
    static_assert(kBwdQuadLoads == 11, "the waits above count 11 loads per request");
    int issued = 0;  // requests 0 ... issued - 1 are out
    for (; issued < 4 && issued < p.T; ++issued) request(issued);
    wait_all_but(issued - 2);  // (requests 0 and 1 have landed)
    __syncthreads();           // P: the compute waves read the inputs of steps 0 and 1 behind it
    for (int m = 0; m < p.T; ++m) {
      // in front of barrier A(m) the inputs of step m + 2 are in place: the compute waves read them behind it
      wait_all_but(issued - (m + 3));
      __syncthreads();  // A(m)
      if (issued < p.T) { request(issued); ++issued; }  // (= m + 4, into the slot of step m, read in front of A(m - 1))
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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
  const int poll_off = (r16 >> 2) * (K * 2) + q * 16;  // + k-step * 64; (lanes between the real rows ask for the real row's bytes)
  char *const ring = reinterpret_cast<char *>(p.xch) + (long long)group * SLOT;
  const long long ring_stride = (long long)ngroups * SLOT;
  const bool cut = p.cut != 0;
  float c9[9], dht = 0.0f;
  bool restart = false;
  auto read_inputs = [&](int n) {  // the inputs of step n of the call, from the feeder's slot
    const char *slot = feed + (n & 3) * kBwdQuadSlot;
    const float *src = reinterpret_cast<const float *>(slot) + prow * (9 * 64) + pu;
#pragma unroll
    for (int j = 0; j < 9; ++j) c9[j] = src[j * 64];
    dht = __uint_as_float((uint32_t)*reinterpret_cast<const uint16_t *>(slot + kBwdQuadCoefBytes + prow * 128 + pu * 2) << 16);
    restart = *reinterpret_cast<const uint32_t *>(slot + kBwdQuadCoefBytes + 1024 + prow * 4) != 0u;
  };
  bool gave_up = false, zero_dy = false;
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
        *reinterpret_cast<uint2 *>(ring + (n % kBwdRing) * ring_stride + pub_off) = uint2{__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi)};
        *reinterpret_cast<uint2 *>(ring + ((n + kBwdRing - 2) % kBwdRing) * ring_stride + pub_off) = uint2{0xFFFFFFFFu, 0xFFFFFFFFu};
      }
      // ---- while the deltas are on their way: d_wx, the progress word, the next step's inputs
      if (s == 0 && tid == 0) p.progress[group] = (unsigned int)n;
      if (there) {
        float *dw = p.d_wx + (long long)row * p.d_wx_sb + (long long)t * p.d_wx_st + ecol;
#pragma unroll
        for (int g = 0; g < 4; ++g) dw[(long long)g * H] = delta[g];
      }
      if (n + 1 < p.T) read_inputs(n + 1);
      if (!cut && S > 1) __builtin_amdgcn_s_sleep(XS_BQ_SLEEP_PUB);
    } else {
      if (!cut) __builtin_amdgcn_s_sleep(XS_BQ_SLEEP_IDLE);
    }
    if (!cut) {
      // ---- the deltas of the wave's eighth of K: polled straight into the A operand registers
      uint4 areg[KSTEPS];
      {
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(ring + (n % kBwdRing) * ring_stride, 0, SLOT, 0x00020000);
        constexpr int kPastL1 = 16;  // (the load's scope bits: served by the L2)
        long long spins = 0;
        for (;;) {
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks)
            areg[ks] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rs, poll_off, (wave_u * KSTEPS + ks) * 64, kPastL1));
          uint32_t mark = 0u;
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks) mark = mark_join<true>(mark, chunk_mark<true>(areg[ks]));
          // (a negative spin limit is the host's way to make every wait run out at its first look: the error path, forced)
          if ((__builtin_amdgcn_ballot_w64(mark_has_sentinel<true>(mark)) == 0ull && p.spin_limit >= 0) || gave_up) break;
          if (++spins > p.spin_limit || ((spins & 255) == 0 && __hip_atomic_load(p.abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
            __hip_atomic_store(p.abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            gave_up = true;
            break;
          }
        }
      }
      // ---- delta [4 rows x K/8] . R^T [K/8 x 64]: the wave's partial result, to LDS.  Two sets of tiles, used in turn: a
      //      wave writes the tiles of step n + 2 only after a peer has published step n + 2, for which that peer needed
      //      all of this workgroup's deltas of step n + 1, which were computed from the sums of step n.
      f32x4 acc[4];
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) acc[cb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
          acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, areg[ks]), __builtin_bit_cast(bf16x8, bq[ks][cb]), acc[cb], 0, 0, 0);
      float *const tiles = part + (n & 1) * 8 * PART + wave * PART + q * kBwdPartStride + r16;
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) tiles[cb * 16] = acc[cb][0];
    }
    __syncthreads();  // A(n)
  }
  // ---- gradient w.r.t. the initial state (the stabiliser's part is zero by the rule; NaN all over when a wait ran out)
  if (grad_wave) {
    dy = (cut || zero_dy) ? 0.0f : add_up(p.T - 1);
    if (there) {
      const bool poisoned = __hip_atomic_load(p.abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
      const long long o = (long long)row * H + ecol;
      p.d_s0[o] = poisoned ? kPoison : dy;
      p.d_s0[BH + o] = poisoned ? kPoison : dc;
      p.d_s0[2 * BH + o] = poisoned ? kPoison : dn;
      p.d_s0[3 * BH + o] = 0.0f;
    }
  }
}

}  // namespace
