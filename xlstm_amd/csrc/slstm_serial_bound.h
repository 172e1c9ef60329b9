// Measurement kernels: the stages of the dependency chain of one timestep of the sequence kernel, each run alone as a
// loop in which every iteration needs the result of the one before.  Included by slstm_hip.hip only.
//
// A timestep of slstm_seq_kernel (one row tile per workgroup) is a chain: the peers' h arrives -> MFMAs over this
// workgroup's 64 columns -> partial sums through LDS, one barrier -> exponential gating -> h published -> it arrives at
// the peers.  The three kernels below run (1) publish -> arrive among G compute units, (2) MFMAs + the reduction
// through LDS, (3) the gating, with the same instructions, layouts and protocol as the product kernel and nothing
// else.  The sum of their times per iteration is what a step of this structure costs when nothing but the chain is
// left: the serial bound that bench.py reports next to the measured time per step.
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

// ---- (2) the contraction of a step in one workgroup: every wave 4 gates x NCH MFMAs on its quarter of K, partial
//      tiles to LDS, the barrier, and the sums of an element (16 partial values and the step's W.x) out of LDS
template <int NCH>
__global__ __launch_bounds__(256) void stage_contraction_kernel(StageParams p) {
  __shared__ float part[2][4][4][kTileFloats];
  __shared__ float wxs[4][kTileFloats];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, q = lane >> 4, r16 = lane & 15;
  const int pa = tid & 15, pb = tid >> 4;
  uint4 rreg[4][NCH];
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int c = 0; c < NCH; ++c) rreg[g][c] = make_uint4(0x3C003C00u + tid, 0x3C013C01u, 0x3C023C02u + g, 0x3C033C03u + c);
  for (int i = tid; i < 4 * kTileFloats; i += 256) (&wxs[0][0])[i] = 0.001f * i;
  __syncthreads();
  float feed = 0.25f;
  for (int t = 0; t < p.steps; ++t) {
    uint4 areg[NCH];
    const uint32_t w = pack_bf16x2(feed, feed);
#pragma unroll
    for (int c = 0; c < NCH; ++c) areg[c] = make_uint4(w, w + c, w, w);
    f32x4 acc[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) acc[g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const bf16x8 av = __builtin_bit_cast(bf16x8, areg[c]);
#pragma unroll
      for (int g = 0; g < 4; ++g)
        acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, __builtin_bit_cast(bf16x8, rreg[g][c]), acc[g], 0, 0, 0);
    }
    const int buf = t & 1;
#pragma unroll
    for (int g = 0; g < 4; ++g) *reinterpret_cast<f32x4 *>(&part[buf][wave][g][r16 * kTileStride + 4 * q]) = acc[g];
    lds_barrier();
    float raw = 0.0f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float ry = part[buf][0][g][pa * kTileStride + pb];
      ry += part[buf][1][g][pa * kTileStride + pb];
      ry += part[buf][2][g][pa * kTileStride + pb];
      ry += part[buf][3][g][pa * kTileStride + pb];
      raw += wxs[g][pb * kTileStride + pa] + ry;
    }
    feed = raw * 1e-6f + 0.25f;
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

// ---- the whole chain in one loop: poll -> MFMAs -> partial sums through LDS, barrier -> sums -> gating -> publish,
//      in the product kernel's order, with constant W.x and bias, no reset flags, no output tensor, no feeder, drainer
//      or prefetch waves.  Head groups of 16 members placed as the product places them (consecutive slots of one XCD).
__global__ __launch_bounds__(256) void stage_chain_kernel(StageParams p) {
  constexpr int NCH = 2, KW = NCH * 32, XTILE = 16 * 16 * 2;
  __shared__ float part[2][4][4][kTileFloats];
  const int wg = blockIdx.x, xcd = wg & 7, local = wg >> 3;
  const int slot = local / p.members, member = local - slot * p.members;
  const int group = slot * 8 + xcd;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, q = lane >> 4, r16 = lane & 15;
  const int pa = tid & 15, pb = tid >> 4;
  const int xslot = p.members * XTILE;
  char *const xbase = p.ring + (long long)group * kRing * xslot;
  const int xlane = r16 < p.rows ? ((wave * KW + q * 8) >> 4) * XTILE + (r16 * 16 + ((q * 8) & 15)) * 2 : 0x7FFFFF00;
  uint4 rreg[4][NCH];
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const uint32_t w = pack_bf16x2(0.001f * (float)(g + 1), -0.0007f * (float)(c + 1 + (lane & 3)));
      rreg[g][c] = make_uint4(w, w, w, w);
    }
  const float wx_g[4] = {0.5f + 0.01f * pa, 3.0f + 0.02f * pb, -0.7f, 0.3f};
  CellState st{0.0f, 0.0f, 0.0f, 0.0f};
  uint32_t max_spins = 0;
  bool dead = false;
  for (int t = 0; t < p.steps; ++t) {
    char *const cur = xbase + (t % kRing) * xslot;
    char *const old = xbase + ((t + kRing - 2) % kRing) * xslot;
    f32x4 acc[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) acc[g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    if (t > 0) {
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(xbase + ((t + kRing - 1) % kRing) * xslot, 0, xslot, 0x00020000);
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
      for (int c = 0; c < NCH; ++c) {
        const bf16x8 av = __builtin_bit_cast(bf16x8, areg[c]);
#pragma unroll
        for (int g = 0; g < 4; ++g)
          acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, __builtin_bit_cast(bf16x8, rreg[g][c]), acc[g], 0, 0, 0);
      }
    }
    const int buf = t & 1;
#pragma unroll
    for (int g = 0; g < 4; ++g) *reinterpret_cast<f32x4 *>(&part[buf][wave][g][r16 * kTileStride + 4 * q]) = acc[g];
    lds_barrier();
    float raw[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float ry = part[buf][0][g][pa * kTileStride + pb];
      ry += part[buf][1][g][pa * kTileStride + pb];
      ry += part[buf][2][g][pa * kTileStride + pb];
      ry += part[buf][3][g][pa * kTileStride + pb];
      raw[g] = wx_g[g] + ry;
    }
    slstm_pointwise(raw[0], raw[1], raw[2], raw[3], st);
    const uint16_t v = (uint16_t)float_to_bf16_bits(st.y);
    reinterpret_cast<uint16_t *>(cur)[member * (XTILE / 2) + pb * 16 + pa] = v;
    reinterpret_cast<uint16_t *>(old)[member * (XTILE / 2) + pb * 16 + pa] = (uint16_t)kSentinel16;
  }
  if (lane == 0 && max_spins) atomicMax(p.words + 1, max_spins);
  if (wg == 0 && tid == 0) reinterpret_cast<float *>(p.words)[11] = st.y;
}

__global__ void stage_empty_kernel() {}

}  // namespace
