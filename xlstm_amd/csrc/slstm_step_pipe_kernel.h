// The pipelined decode step kernel: the steady state of bf16 decoding (whole tiles, a carried state, no mask, the
// previous h available in bf16, head dim 256).  Included by slstm_hip.hip only, after slstm_step_kernel.h.
#pragma once

namespace {

// A decode step is bound by HBM (the state is read and written once), and inside a compute unit by four different
// things: how many requests the unit keeps in flight while the operands arrive, LDS reads during the MFMAs, VALU
// issue during the gating, the write path at the end.  The tile kernel (slstm_step_tile_kernel) runs them one after
// the other for the whole 64 x 32 tile, and because all workgroups do so in step, the memory system sees all
// reads, then all writes.  Here the tile is cut into four ROW TILES of 16 rows that move through the stages one
// behind the other: the gating of the first row tiles runs while the operands of the last still arrive, and their
// stores leave while the last are gated.  Measured at B 256 x D 2048 (8 heads): 6.3 us per step against 7.5.
//
// Everything the workgroup reads goes STRAIGHT INTO LDS (buffer_load ... lds, whole lines, hand-issued and
// hand-counted).  Twelve waves:
//
//   waves 0-3   MFMA waves, wave g = gate g, raised priority.  They request h of all four row tiles (the MFMA
//               operand, bf16), then R; both come from the L2.  They issue no stores, so their one wait is exact.
//               Each keeps its 32 columns of R (2 unit tiles x K) in registers, read once from LDS (fetched as MFMA
//               fragments straight from memory a load touches 16 half lines and the fetch took twice as long).  Per
//               row tile: 16 MFMAs while the h fragments of the next row tile are read, sums to LDS (into the part
//               of the R area that the wave itself has emptied).
//   waves 4-11  gating waves, two per SIMD: wave 4 + v + 4 j gates the row tiles j and j + 2, rows 4 v .. 4 v + 3.
//               At once they request the old c, n, m and W.x of their two row tiles, the earlier one first: these
//               come from memory or the Infinity Cache, 2 to 3 thousand cycles away, and a compute unit keeps only
//               some 32 KiB of requests in flight, so they have to be the first in the queue.  Then, per row tile:
//               2 elements per lane (two neighbouring units of one row), all operands from LDS, results to global
//               memory.  One gating wave per SIMD leaves it idle 40 % of the time (a chain of dependent
//               transcendentals and LDS round trips: 1250 cycles per row tile for 750 cycles of issue).
//
// The stages are chained by counters in LDS, not by workgroup barriers: a wave that has seen its own share land adds
// one to h_landed (MFMA waves) or s_landed[r] (the four gating waves of row tile r) and goes on when all four have;
// an MFMA wave whose sums of row tile r are in LDS adds one to summed[r], which the gating waves of r wait for.
// K is accumulated in the sequence kernel's four quarters and the quarters are added in its order: the same bits
// as every other path.
//
// What the order of the requests is worth (same kernel otherwise, us per step): everything requested by the MFMA
// waves, row tile by row tile, R as MFMA fragments 8.0; R through LDS 7.4; the far-away operands requested first
// and by the gating waves 7.0; two gating waves per SIMD 6.6; h before R, a gating group waiting only for its own
// row tiles, the next row tile's h fragments read under the MFMAs 6.3.  Pauses in front of either role's requests
// (256 to 4096 cycles) only cost.
template <int N>
__device__ __forceinline__ void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }

// Bounded like every other wait of the engine (the other waves of the workgroup always get there); false when the
// bound ran out.  The caller then marks the workgroup as given up, and what it stores is NaN.
__device__ __forceinline__ bool wait_lds_counter(uint32_t *counter, uint32_t want, int spin_limit) {
  for (int spins = 0; spins < spin_limit; ++spins) {
    if (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= want) return true;
    __builtin_amdgcn_s_sleep(1);
  }
  return __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= want;
}

constexpr int kStepPipeThreads = 768;  // 4 MFMA waves + 8 gating waves

template <int NK>  // MFMA k-steps over the head dim: dh = 32 * NK
__global__ __launch_bounds__(kStepPipeThreads) void slstm_step_pipe_kernel(StepParams p) {
  static_assert(NK == 8, "head dim 256 (with 128 the sums of a gate do not fit the R columns of that gate)");
  constexpr int DH = 32 * NK;
  constexpr int NQ = NK / 4;            // k-steps per K quarter, as in the sequence kernel
  constexpr int NHB = DH / 128;         // 256-byte column blocks of an h row
  constexpr int SROW = 36;              // floats per row of a sum tile (32 units + pad: conflict-free 16-byte writes)
  constexpr int kHalfR = 128 * 256;     // bytes of one K half of the R slab
  // loads per row tile: h 4 per column block (2 per MFMA wave); c / n / m 2 each + W.x 1 per gate = 10 (3 / 3 / 2 / 2 per gating wave)
  constexpr int LH = 4 * NHB / 4;
  constexpr int LS = 10;

  extern __shared__ __attribute__((aligned(16))) unsigned char step_lds[];
  unsigned char *const hbuf = step_lds;                               // [NHB][64 rows][256 B], pieces swizzled
  unsigned char *const cnm = hbuf + NHB * 64 * 256;                   // [3][64 rows][128 B]
  unsigned char *const wxl = cnm + 3 * 64 * 128;                      // [4 gates][64 rows][64 B]
  unsigned char *const rbuf = wxl + 4 * 64 * 64;                      // [2 K halves][128 columns][256 B], pieces swizzled
  uint32_t *const counters = reinterpret_cast<uint32_t *>(rbuf + 2 * kHalfR);  // h_landed, -, -, -, summed[4], s_landed[4], gave_up
  // sums of (row tile rt, gate g), [16 rows][SROW] floats: inside the 8 KiB of K half rt / 2 that held gate g's columns
  auto sums_of = [&](int rt, int g) { return reinterpret_cast<float *>(rbuf + (rt >> 1) * kHalfR + g * 8192 + (rt & 1) * (16 * SROW * 4)); };

  const int wave = (int)uniform((uint32_t)(threadIdx.x >> 6));
  const int lane = threadIdx.x & 63;
  int head, unit_tile, row_tile;
  step_tile_of(p, blockIdx.x, head, unit_tile, row_tile);
  const int a0 = unit_tile * 32;
  const int rowbase = row_tile * 64;
  const int H = p.NH * DH;
  const long long BH = (long long)p.B * H;

  // the status block: one launch, the step kernel, the pipelined one.  (Device-scope stores, like the stores of a
  // workgroup that gives up: both reach the same place in the same order they were made.  Workgroup 0 is the first
  // to be dispatched, and nobody gives up before its operands are a memory round trip overdue.)
  if (blockIdx.x == 0 && threadIdx.x < 16)
    __hip_atomic_store(reinterpret_cast<uint32_t *>(p.status) + threadIdx.x,
                       (threadIdx.x == 5 || threadIdx.x == 6 || threadIdx.x == 8) ? 1u : 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (threadIdx.x < 13) counters[threadIdx.x] = 0u;
  lds_barrier();  // the only workgroup barrier: the counters start at zero
  // a wait inside the workgroup ran out: the workgroup's outputs become NaN and the status block says so
  auto give_up = [&]() {
    if (lane == 0) {
      __hip_atomic_store(&counters[12], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      __hip_atomic_store(&p.status->abort_wg, (uint32_t)blockIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&p.status->aborted, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  };

  // ---- the old c, n, m and W.x (what is furthest away): a gating wave requests its share of the two row tiles its
  //      group gates, the earlier row tile first (10 loads per row tile, 3 + 2 or 2 + 3 per wave)
  auto issue_state_and_wx = [&]() {
    const int gv = (wave - 4) & 3, gj = (wave - 4) >> 2;
    // one descriptor for the state planes and one for W.x, both based at this workgroup's first row and unit (the host
    // checks that the offsets fit 31 bits); everything that changes from load to load is in the lane's offset
    const unsigned long long sb = reinterpret_cast<unsigned long long>(p.s0) + ((unsigned long long)rowbase * H + (unsigned long long)head * DH + a0) * 4;
    const unsigned long long xb = reinterpret_cast<unsigned long long>(p.wx) + ((unsigned long long)rowbase * p.wx_sb + (unsigned long long)head * DH + a0) * 2;
    const u32x4_t srs = {uniform((uint32_t)sb), uniform((uint32_t)(sb >> 32) & 0xFFFFu), uniform((uint32_t)(3 * BH * 4 + 64ll * H * 4)), 0x00020000u};
    const u32x4_t xrs = {uniform((uint32_t)xb), uniform((uint32_t)(xb >> 32) & 0xFFFFu), uniform((uint32_t)(63 * p.wx_sb * 2 + 3ll * H * 2 + 64)), 0x00020000u};
    const uint32_t cl = (uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)cnm);
    const uint32_t xl = (uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)wxl);
    const int svoff = (lane >> 3) * H * 4 + (lane & 7) * 16;               // c, n, m: 8 rows x 128 bytes per load
    const int xvoff = (int)((lane >> 2) * p.wx_sb * 2) + (lane & 3) * 16;  // W.x: 16 rows x 64 bytes of one gate per load
#pragma unroll
    for (int rti = 0; rti < 2; ++rti) {
      const int rt = gj + 2 * rti;
#pragma unroll
      for (int i = 0; i < LS; ++i) {
        if (((i + 2 * rti) & 3) != gv) continue;  // (wave-uniform)
        if (i < 6) {
          const int plane = i >> 1, r0 = 16 * rt + 8 * (i & 1);
          lds_direct_fetch_b128(srs, uniform(cl + plane * (64 * 128) + r0 * 128), svoff + (int)((plane + 1) * BH * 4) + r0 * H * 4);
        } else {
          const int g = i - 6;
          lds_direct_fetch_b128(xrs, uniform(xl + (g * 64 + 16 * rt) * 64), xvoff + (int)(16 * rt * p.wx_sb * 2) + g * H * 2);
        }
      }
    }
  };
#ifdef XS_PROFILE
  const long long pt0 = clock64();
  long long *const pdst = reinterpret_cast<long long *>(reinterpret_cast<char *>(p.status) + 256);
#define XS_PSTAMP(slot) do { if (blockIdx.x == 9 && lane == 0) pdst[slot] = clock64() - pt0; } while (0)
#else
#define XS_PSTAMP(slot) do { } while (0)
#endif
  if (wave < 4) {
    // =====================================================================
    // MFMA waves
    // =====================================================================
    const int q = lane >> 4, r16 = lane & 15;
    // (the gating waves' requests go first: what they ask for is the furthest away)
    {
      const unsigned long long hb = reinterpret_cast<unsigned long long>(p.h_prev), rb = reinterpret_cast<unsigned long long>(p.r);
      const u32x4_t hrs = {uniform((uint32_t)hb), uniform((uint32_t)(hb >> 32) & 0xFFFFu), uniform((uint32_t)(BH * 2)), 0x00020000u};
      const u32x4_t rrs = {uniform((uint32_t)rb), uniform((uint32_t)(rb >> 32) & 0xFFFFu), uniform((uint32_t)((long long)H * 4 * DH * 2)), 0x00020000u};
      const uint32_t hl = (uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)hbuf);
      const uint32_t rl = (uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)rbuf);
      const int sub = lane >> 4, pos = lane & 15;  // a load covers 4 rows / columns of 256 bytes: row sub of them, position pos
      // h first (all four row tiles: 8 loads), then R: the MFMAs of a row tile then never wait for its h, which returned
      // late when requested behind R (requests return in order, and the gating waves' far-away ones are among them).
      // h: rows 4 wave .. + 3 of every row tile, one column block per load; piece (pos ^ (row & 7)) goes to position pos
#pragma unroll
      for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int blk = 0; blk < NHB; ++blk) {
          const int row = 16 * rt + 4 * wave + sub;
          const int voff = (int)(((long long)(rowbase + row) * H + head * DH) * 2) + (blk * 16 + (pos ^ (row & 7))) * 16;
          lds_direct_fetch_b128(hrs, uniform(hl + blk * (64 * 256) + (16 * rt + 4 * wave) * 256), voff);
        }
      // R of this workgroup's 128 columns, one K half of 4 columns per load, 16 loads per wave: its own gate's 32 columns
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const int colx = 4 * (wave * 8 + k) + sub;  // column of the workgroup's 128: gate colx / 32 (= wave), unit colx % 32
          const int voff = (int)(((long long)head * 4 * DH + (long long)(colx >> 5) * DH + a0 + (colx & 31)) * DH * 2) + (half * 16 + (pos ^ (colx & 7))) * 16;
          lds_direct_fetch_b128(rrs, uniform(rl + half * kHalfR + (wave * 8 + k) * 1024), voff);
        }
    }
    if (wave == 0) XS_PSTAMP(0);
    // byte offset inside a 256-byte row of this lane's piece of k-step c of a column block: position (4c + q) ^ (row & 7)
    const int swz[4] = {((0 + q) ^ (r16 & 7)) << 4, ((4 + q) ^ (r16 & 7)) << 4, ((8 + q) ^ (r16 & 7)) << 4, ((12 + q) ^ (r16 & 7)) << 4};
    // ---- everything this wave asked for (R comes last); each wave fetched its own gate's columns of R, so its own wait
    //      suffices for those.  A operand: unit a0 + 16 ut + r16 of gate `wave`, k-step ch, this lane group's 8 inputs.
    wait_vmcnt<0>();
    if (lane == 0) __hip_atomic_fetch_add(&counters[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    uint4 rf[2][NK];
#pragma unroll
    for (int ut = 0; ut < 2; ++ut)
#pragma unroll
      for (int ch = 0; ch < NK; ++ch)
        rf[ut][ch] = *reinterpret_cast<const uint4 *>(rbuf + (ch >> 2) * kHalfR + (wave * 32 + ut * 16 + r16) * 256 + swz[ch & 3]);
    if (wave == 0) XS_PSTAMP(1);
    if (!wait_lds_counter(&counters[0], 4u, p.spin_limit)) give_up();  // h of all row tiles, from all four MFMA waves
    asm volatile("" ::: "memory");
    // B operand: h of row 16 rt + r16, k-step ch.  The fragments of the next row tile are read while the MFMAs of this
    // one run (everything has landed: nothing else stands between the row tiles but the LDS round trip).
    auto h_frag = [&](int rt, int ch) {
      return *reinterpret_cast<const uint4 *>(hbuf + (ch >> 2) * (64 * 256) + (16 * rt + r16) * 256 + swz[ch & 3]);
    };
    uint4 hv[NK], hn[NK];
#pragma unroll
    for (int ch = 0; ch < NK; ++ch) hv[ch] = h_frag(0, ch);
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
      if (wave == 0) XS_PSTAMP(2 + 3 * rt);
      if (rt < 3) {
#pragma unroll
        for (int ch = 0; ch < NK; ++ch) hn[ch] = h_frag(rt + 1, ch);
      }
      f32x4 tot[2], acc[2];
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        acc[0] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        acc[1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int cq = 0; cq < NQ; ++cq) {
          const int ch = w * NQ + cq;
#pragma unroll
          for (int ut = 0; ut < 2; ++ut)
            acc[ut] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, rf[ut][ch]), __builtin_bit_cast(bf16x8, hv[ch]), acc[ut], 0, 0, 0);
        }
#pragma unroll
        for (int ut = 0; ut < 2; ++ut) tot[ut] = (w == 0) ? acc[ut] : tot[ut] + acc[ut];  // quarter 0 first
      }
#pragma unroll
      for (int ch = 0; ch < NK; ++ch) hv[ch] = hn[ch];
      // sums of gate `wave`: lane holds units 16 ut + 4 q .. + 3 of row r16
#pragma unroll
      for (int ut = 0; ut < 2; ++ut)
        *reinterpret_cast<f32x4 *>(sums_of(rt, wave) + r16 * SROW + 16 * ut + 4 * q) = tot[ut];
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      if (lane == 0) __hip_atomic_fetch_add(&counters[4 + rt], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      if (wave == 0) XS_PSTAMP(3 + 3 * rt);
    }
    return;
  }

  // =======================================================================
  // gating waves: wave 4 + v + 4 j gates the row tiles j and j + 2; lane l -> row 4 v + l / 16 of the row tile, units
  // 2 (l % 16) and + 1.  Two gating waves per SIMD: one wave's chain of dependent transcendentals and its LDS round
  // trips leave the SIMD idle about 40 % of the time (one row tile took 1250 cycles for 750 cycles of issue).
  // =======================================================================
  const int v = (wave - 4) & 3;
  const int rt0 = (wave - 4) >> 2;
  const int prow = 4 * v + (lane >> 4);
  const int pair = lane & 15;
  const int ua = a0 + 2 * pair;
  typedef float f32x2v __attribute__((ext_vector_type(2)));
  f32x2v bias2[4];
  {
    // the bias first (hand-issued as well: a load the compiler knew of would make it wait for everything behind it)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float *src = p.bias + ((long long)head * 4 + g) * DH + ua;
      asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(bias2[g]) : "v"(src) : "memory");
    }
  }
  issue_state_and_wx();
  if (wave == 4) XS_PSTAMP(15);
#pragma unroll
  for (int rti = 0; rti < 2; ++rti) {
    const int rt = rt0 + 2 * rti;
    const int row = 16 * rt + prow;  // row of the workgroup's 64
    if (rti == 0) {
      // this wave's share of the row tile's old state and W.x: only its 2 or 3 requests for the second row tile are
      // younger (no stores yet: the count is exact)
      if (v < 2) wait_vmcnt<2>(); else wait_vmcnt<3>();
      asm volatile("" : "+v"(bias2[0]), "+v"(bias2[1]), "+v"(bias2[2]), "+v"(bias2[3]) :: "memory");  // (the bias landed before them)
      if (lane == 0) __hip_atomic_fetch_add(&counters[8 + rt], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      if (wave == 4) XS_PSTAMP(16);
    }
    if (!wait_lds_counter(&counters[8 + rt], 4u, p.spin_limit) || !wait_lds_counter(&counters[4 + rt], 4u, p.spin_limit)) give_up();
    asm volatile("" ::: "memory");
    if (wave == 4 || wave == 8) XS_PSTAMP(17 + 2 * rt);
    float2 s2[4];
    uint32_t wx2[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      s2[g] = *reinterpret_cast<const float2 *>(sums_of(rt, g) + prow * SROW + 2 * pair);
      wx2[g] = *reinterpret_cast<const uint32_t *>(wxl + (g * 64 + row) * 64 + pair * 4);
    }
    const float2 c2 = *reinterpret_cast<const float2 *>(cnm + (0 * 64 + row) * 128 + pair * 8);
    const float2 n2 = *reinterpret_cast<const float2 *>(cnm + (1 * 64 + row) * 128 + pair * 8);
    const float2 m2 = *reinterpret_cast<const float2 *>(cnm + (2 * 64 + row) * 128 + pair * 8);
    // (an MFMA wave that gave up said so before it reported its sums; this wave's own give_up is in LDS order before this read)
    const bool poisoned = __hip_atomic_load(&counters[12], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != 0u;
    float yv[2], cv[2], nv[2], mv[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      float raw[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const float wxv = bf16_bits_to_float(i ? (wx2[g] >> 16) : (wx2[g] & 0xFFFFu));
        raw[g] = (wxv + (i ? s2[g].y : s2[g].x)) + bias2[g][i];
      }
      CellState st{0.0f, i ? c2.y : c2.x, i ? n2.y : n2.x, i ? m2.y : m2.x};
      slstm_pointwise(raw[0], raw[1], raw[2], raw[3], st);
      yv[i] = poisoned ? kPoison : st.y; cv[i] = poisoned ? kPoison : st.c;
      nv[i] = poisoned ? kPoison : st.n; mv[i] = poisoned ? kPoison : st.m;
    }
    if (rti == 0) {
      // The second row tile's share, before this row tile's stores go out: loads and stores share the counter and a
      // wait behind the stores would also wait for their acknowledgement (400 cycles, measured).
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(yv[0]), "+v"(yv[1]) :: "memory");
      if (lane == 0) __hip_atomic_fetch_add(&counters[8 + rt + 2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    const long long o = (long long)(rowbase + row) * H + head * DH + ua;
    // streaming stores: 16 lanes write one whole 128-byte line of each state plane
    __builtin_nontemporal_store(f32x2v{yv[0], yv[1]}, reinterpret_cast<f32x2v *>(p.s_out + o));
    __builtin_nontemporal_store(f32x2v{cv[0], cv[1]}, reinterpret_cast<f32x2v *>(p.s_out + BH + o));
    __builtin_nontemporal_store(f32x2v{nv[0], nv[1]}, reinterpret_cast<f32x2v *>(p.s_out + 2 * BH + o));
    __builtin_nontemporal_store(f32x2v{mv[0], mv[1]}, reinterpret_cast<f32x2v *>(p.s_out + 3 * BH + o));
    *reinterpret_cast<uint32_t *>(reinterpret_cast<uint16_t *>(p.h_out) + o) = float_to_bf16_bits(yv[0]) | (float_to_bf16_bits(yv[1]) << 16);
  }
#ifdef XS_PROFILE
  if (wave == 8) XS_PSTAMP(24);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (wave == 8) XS_PSTAMP(25);
#endif
}

}  // namespace
