// Measurement kernels: the stages of the dependency chain of one timestep of the sequence kernel, each run alone as a
// loop in which every iteration needs the result of the one before.  Included by slstm_hip.hip only.
//
// A timestep of slstm_seq_kernel is a chain: the peers' h arrives -> MFMAs over this workgroup's 64 columns -> the
// gates of a unit brought together -> exponential gating -> h published -> it arrives at the peers.  stage_chain_kernel
// runs that chain, as the kernel for row tiles of 4 rows makes it, with the same instructions, layouts and protocol
// and nothing else: what a step of this structure costs when only the chain is left, the serial bound that bench.py
// reports next to the measured time per step.  The other kernels run its stages alone (each its own loop: their sum is
// more than the chain) and the exchange in the layouts of the other sequence kernels.
#pragma once

namespace {

struct StageParams {
  int members;          // exchange: workgroups that exchange (one per compute unit)
  int two_xcds;         // exchange: members on XCDs 0 and 4 (half each), device-scope stores
  int rows;             // exchange: batch rows of the tile that exist (the others are never fetched)
  int steps;
  char *ring;           // exchange: [kRing slots][members][16 rows][16 units] bf16, all ones at the start
  unsigned int *words;  // [0] abort flag (zero at the start), [1] spins of the longest wait, [8...] results nobody reads
  long long spin_limit;
};

// ---- (1) the exchange: every workgroup publishes 16 rows x 16 units of bf16 (512 bytes, one 2-byte store per thread,
//      as the product kernel does), re-arms its words of two steps ago, and its four waves poll their quarter of the
//      group's row tile (NCH chunks of 16 bytes per lane) until no word carries the "not written yet" pattern.  What
//      a workgroup publishes next is computed from what it polled.
template <int NCH>
__global__ __launch_bounds__(256) void stage_exchange_kernel(StageParams p) {
  const int wg = blockIdx.x, xcd = wg & 7, local = wg >> 3;
  int member;
  if (p.two_xcds) {
    if (xcd != 0 && xcd != 4) return;
    member = (xcd >> 2) * (p.members >> 1) + local;
    if (local >= (p.members >> 1)) return;
  } else {
    if (xcd != 0 || local >= p.members) return;
    member = local;
  }
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, q = lane >> 4, r16 = lane & 15;
  constexpr int KW = NCH * 32;                       // input units per wave
  constexpr int XTILE = 16 * 16 * 2;                 // bytes a member publishes per step
  const int xslot = p.members * XTILE;
  const int pb = tid >> 4, pa = tid & 15;
  const int xlane = r16 < p.rows ? ((wave * KW + q * 8) >> 4) * XTILE + (r16 * 16 + ((q * 8) & 15)) * 2 : 0x7FFFFF00;
  uint32_t carry = (uint32_t)tid;
  uint32_t max_spins = 0;
  bool dead = false;
  for (int t = 0; t < p.steps; ++t) {
    char *const cur = p.ring + (t % kRing) * xslot;
    char *const old = p.ring + ((t + kRing - 2) % kRing) * xslot;
    const uint16_t v = (uint16_t)(carry & 0x7FFFu);
    uint16_t *dst = reinterpret_cast<uint16_t *>(cur) + member * (XTILE / 2) + pb * 16 + pa;
    uint16_t *rearm = reinterpret_cast<uint16_t *>(old) + member * (XTILE / 2) + pb * 16 + pa;
    if (p.two_xcds) {
      __hip_atomic_store(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(rearm, (uint16_t)kSentinel16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      *dst = v;
      *rearm = (uint16_t)kSentinel16;
    }
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(cur, 0, xslot, 0x00020000);
    uint4 areg[NCH];
    uint32_t spins = 0;
    for (;;) {
#pragma unroll
      for (int c = 0; c < NCH; ++c)
        areg[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rs, xlane, ((c * 32) >> 4) * XTILE, 16));
      uint32_t ma = 0u;
#pragma unroll
      for (int c = 0; c < NCH; ++c) ma = mark_join<true>(ma, chunk_mark<true>(areg[c]));
      if (__builtin_amdgcn_ballot_w64(mark_has_sentinel<true>(ma)) == 0ull || dead) break;
      if (++spins >= (uint32_t)p.spin_limit ||
          ((spins & 1023u) == 0u && __hip_atomic_load(p.words, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
        __hip_atomic_store(p.words, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        dead = true;
        break;
      }
    }
    max_spins = spins > max_spins ? spins : max_spins;
#pragma unroll
    for (int c = 0; c < NCH; ++c) carry += areg[c].x ^ areg[c].w;
    carry = (uint32_t)__shfl((int)carry, (lane + 1) & 63);  // (every thread's next word depends on a polled one)
    // The workgroup's one barrier per step, as in the product kernel, and part of the protocol: a wave polls a quarter
    // of the members only, and may re-arm its words of two steps ago only when ALL members have published the step
    // before, which it knows once its three sister waves have seen their quarters.
    __syncthreads();
  }
  if (lane == 0 && max_spins) atomicMax(p.words + 1, max_spins);
  if (member == 0 && tid == 0) p.words[8] = carry;
}

// ---- (1b) the exchange as the kernel for row tiles of 4 rows makes it: [slot][member][4 rows][16 units], EVERY wave
//      polls the group's whole tile (NK chunks of 16 bytes from the 16 lanes whose MFMA row is a real one) and publishes
//      its own 16 values; the step's barrier and a pause of 64 cycles in front of the poll
template <int NK>
__global__ __launch_bounds__(256) void stage_exchange_quad_kernel(StageParams p) {
  const int wg = blockIdx.x, xcd = wg & 7, member = wg >> 3;
  if (xcd != 0 || member >= p.members) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, q = lane >> 4, r16 = lane & 15;
  constexpr int QTILE = 4 * 16 * 2;
  const int xslot = p.members * QTILE;
  const bool a_lane = (r16 & 3) == 0 && (r16 >> 2) < p.rows;
  const int xl = a_lane ? (q >> 1) * QTILE + (r16 >> 2) * 32 + (q & 1) * 16 : 0x7FFFFF00;
  const long long xo = (long long)member * (QTILE / 2) + q * 16 + 4 * wave + (r16 & 3);
  uint32_t carry = (uint32_t)tid, max_spins = 0;
  bool dead = false;
  for (int t = 0; t < p.steps; ++t) {
    uint16_t *const cur = reinterpret_cast<uint16_t *>(p.ring + (t % kRing) * xslot);
    uint16_t *const old = reinterpret_cast<uint16_t *>(p.ring + ((t + kRing - 2) % kRing) * xslot);
    if (r16 < 4) {
      cur[xo] = (uint16_t)(carry & 0x7FFFu);
      old[xo] = (uint16_t)kSentinel16;
    }
    __syncthreads();
    __builtin_amdgcn_s_sleep(1);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char *>(cur), 0, xslot, 0x00020000);
    uint4 areg[NK];
    uint32_t spins = 0;
    for (;;) {
#pragma unroll
      for (int ks = 0; ks < NK; ++ks)
        areg[ks] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rs, xl, ks * 2 * QTILE, 16));
      uint32_t ma = 0u;
#pragma unroll
      for (int ks = 0; ks < NK; ++ks) ma = mark_join<true>(ma, chunk_mark<true>(areg[ks]));
      if (__builtin_amdgcn_ballot_w64(mark_has_sentinel<true>(ma)) == 0ull || dead) break;
      if (++spins >= (uint32_t)p.spin_limit ||
          ((spins & 1023u) == 0u && __hip_atomic_load(p.words, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
        __hip_atomic_store(p.words, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        dead = true;
        break;
      }
    }
    max_spins = spins > max_spins ? spins : max_spins;
    // (every lane's next word depends on a polled one: lanes 0-3 of a row of 16 publish, lanes 0, 4, 8, 12 poll)
    uint32_t mix = areg[0].x;
#pragma unroll
    for (int ks = 1; ks < NK; ++ks) mix ^= areg[ks].x;
    carry += mix + (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mix, 0x104, 0xF, 0xF, true);
  }
  if (lane == 0 && max_spins) atomicMax(p.words + 1, max_spins);
  if (member == 0 && tid == 0) p.words[8] = carry;
}

// ---- (2) the contraction of a step as that kernel makes it: a wave's NK MFMAs over the whole of K in four chains, the
//      fold of the four quarters, the three row shifts that bring a unit's gates together (no LDS, no barrier)
template <int NCH>
__global__ __launch_bounds__(256) void stage_contraction_kernel(StageParams p) {
  constexpr int NK = 4 * NCH;
  const int tid = threadIdx.x;
  uint4 rreg[NK];
#pragma unroll
  for (int ks = 0; ks < NK; ++ks) rreg[ks] = make_uint4(0x3C003C00u + tid, 0x3C013C01u, 0x3C023C02u + ks, 0x3C033C03u);
  float feed = 0.25f;
  for (int t = 0; t < p.steps; ++t) {
    uint4 areg[NK];
    const uint32_t w = pack_bf16x2(feed, feed);
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) areg[ks] = make_uint4(w, w + ks, w, w);
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
    const int mi = __float_as_int(mine);
    const float r1 = __int_as_float(__builtin_amdgcn_update_dpp(0, mi, 0x104, 0xF, 0xF, true));
    const float r2 = __int_as_float(__builtin_amdgcn_update_dpp(0, mi, 0x108, 0xF, 0xF, true));
    const float r3 = __int_as_float(__builtin_amdgcn_update_dpp(0, mi, 0x10C, 0xF, 0xF, true));
    feed = ((mine + r1) + (r2 + r3)) * 1e-6f + 0.25f;
  }
  if (tid == 0) reinterpret_cast<float *>(p.words)[9] = feed;
}

// ---- (3) the gating of one element per lane (one wave per SIMD, as in the product kernel), the four raw gate values
//      of a step formed from the y of the step before, y rounded to bf16 as it is published
__global__ __launch_bounds__(256) void stage_gating_kernel(StageParams p) {
  const int tid = threadIdx.x;
  CellState st{0.0f, 0.0f, 0.0f, 0.0f};
  const float k0 = 0.5f + 0.001f * tid, k1 = 3.0f + 0.002f * tid, k2 = -0.7f, k3 = 0.3f;
  for (int t = 0; t < p.steps; ++t) {
    const float y = bf16_bits_to_float(float_to_bf16_bits(st.y));
    slstm_pointwise(k0 + y, k1 - y, k2 + 2.0f * y, k3 + y, st);
  }
  if (tid == 0) reinterpret_cast<float *>(p.words)[10] = st.y + st.c;
}

// ---- the whole chain in one loop, in the product kernel's order (the kernel for row tiles of 4 rows): barrier, pause,
//      poll of the whole tile, MFMAs, fold, row shifts, gating, publication; constant W.x and bias, no reset flags, no
//      output tensor, no feeder, drainer or prefetch waves.  Head groups of 16 members placed as the product places
//      them (consecutive slots of one XCD).
__global__ __launch_bounds__(256) void stage_chain_kernel(StageParams p) {
  constexpr int NCH = 2, NK = 4 * NCH, QTILE = 4 * 16 * 2;
  const int wg = blockIdx.x, xcd = wg & 7, local = wg >> 3;
  const int slot = local / p.members, member = local - slot * p.members;
  const int group = slot * 8 + xcd;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, q = lane >> 4, r16 = lane & 15;
  const int xslot = p.members * QTILE;
  char *const xbase = p.ring + (long long)group * kRing * xslot;
  const bool a_lane = (r16 & 3) == 0 && (r16 >> 2) < p.rows;
  const int xl = a_lane ? (q >> 1) * QTILE + (r16 >> 2) * 32 + (q & 1) * 16 : 0x7FFFFF00;
  const long long xo = (long long)member * (QTILE / 2) + q * 16 + 4 * wave + (r16 & 3);
  uint4 rreg[NK];
#pragma unroll
  for (int ks = 0; ks < NK; ++ks) {
    const uint32_t w = pack_bf16x2(0.001f * (float)((r16 >> 2) + 1), -0.0007f * (float)(ks + 1 + (lane & 3)));
    rreg[ks] = make_uint4(w, w, w, w);
  }
  const float wx_g[4] = {0.5f + 0.01f * (r16 & 3), 3.0f + 0.02f * q, -0.7f, 0.3f};
  CellState st{0.0f, 0.0f, 0.0f, 0.0f};
  uint32_t max_spins = 0;
  bool dead = false;
  // (the loop's start relative to a 32-byte line of code, chosen like the product kernel's: the best of the eight,
  // 0.64 us per step; the others 0.67 (three of them) and 0.78 (four))
#ifndef XS_CHAIN_PAD
#define XS_CHAIN_PAD 4
#endif
  asm volatile(".p2align 5\n\t.rept %0\n\ts_nop 0\n\t.endr" :: "n"(XS_CHAIN_PAD));
  for (int t = 0; t < p.steps; ++t) {
    uint16_t *const cur = reinterpret_cast<uint16_t *>(xbase + (t % kRing) * xslot);
    uint16_t *const old = reinterpret_cast<uint16_t *>(xbase + ((t + kRing - 2) % kRing) * xslot);
    lds_barrier();
    __builtin_amdgcn_s_sleep(1);
    uint4 areg[NK];
    if (t == 0) {
#pragma unroll
      for (int ks = 0; ks < NK; ++ks) areg[ks] = make_uint4(0, 0, 0, 0);
    } else {
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(xbase + ((t + kRing - 1) % kRing) * xslot, 0, xslot, 0x00020000);
      uint32_t spins = 0;
      for (;;) {
#pragma unroll
        for (int ks = 0; ks < NK; ++ks)
          areg[ks] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rs, xl, ks * 2 * QTILE, 16));
        uint32_t ma = 0u;
#pragma unroll
        for (int ks = 0; ks < NK; ++ks) ma = mark_join<true>(ma, chunk_mark<true>(areg[ks]));
        if (__builtin_amdgcn_ballot_w64(mark_has_sentinel<true>(ma)) == 0ull || dead) break;
        if (++spins >= (uint32_t)p.spin_limit ||
            ((spins & 1023u) == 0u && __hip_atomic_load(p.words, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
          __hip_atomic_store(p.words, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          dead = true;
          break;
        }
      }
      max_spins = spins > max_spins ? spins : max_spins;
    }
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
    const int mi = __float_as_int(mine);
    const float ry1 = __int_as_float(__builtin_amdgcn_update_dpp(0, mi, 0x104, 0xF, 0xF, true));
    const float ry2 = __int_as_float(__builtin_amdgcn_update_dpp(0, mi, 0x108, 0xF, 0xF, true));
    const float ry3 = __int_as_float(__builtin_amdgcn_update_dpp(0, mi, 0x10C, 0xF, 0xF, true));
    slstm_pointwise(wx_g[0] + mine, wx_g[1] + ry1, wx_g[2] + ry2, wx_g[3] + ry3, st);
    if (r16 < 4) {
      cur[xo] = (uint16_t)float_to_bf16_bits(st.y);
      old[xo] = (uint16_t)kSentinel16;
    }
  }
  if (lane == 0 && max_spins) atomicMax(p.words + 1, max_spins);
  if (wg == 0 && tid == 0) reinterpret_cast<float *>(p.words)[11] = st.y;
}

__global__ void stage_empty_kernel() {}

}  // namespace
