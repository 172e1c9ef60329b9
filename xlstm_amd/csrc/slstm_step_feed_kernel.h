// The decode step (T = 1) for the head dims whose K range does not fit LDS in one piece (beyond 256 in bf16, 128 in
// float32), with R prepared once: included by slstm_hip.hip only, behind slstm_backward_step_kernel.h, whose forward
// walk it shares its build with.
//
// slstm_step_tile_kernel walks K in slabs whose loads sit in registers of the waves that multiply; the compiler places
// the waits of such a loop so that a slab costs a whole memory latency (13 us a step at 4 heads of 512, 20 at 1024,
// whatever the batch).  Here four feeder waves bring the slabs straight into a ring of LDS slots, slabs ahead of the
// four waves that multiply, with hand-counted waits and one barrier per slab.  That wants R slab by slab in memory
// (xs_slstm_tile_r_for_steps: [NH][unit / 32][k / KS][gate][unit % 32][k % KS], KS = 128 bytes of K) and the
// recurrent operand in the type of the operands: the bf16 copy of the state's y that the previous step left
// (xs_slstm_args::h_prev), the state's y plane itself in float32.  A workgroup owns 64 batch rows x 32 units x 4 gates;
// the slabs are accumulated in the sequence kernel's four K quarters and the quarters are added in its order, so a step
// reproduces a sequence call bit for bit, as slstm_step_tile_kernel does.
#pragma once

namespace {

struct StepFeedParams {
  int B, NH, dh;
  int nch;                   // MFMA k-steps per K quarter (as in the sequence kernel)
  const void *wx;            // [B, 4, NH, dh], row stride wx_sb elements
  long long wx_sb;
  const void *r_tiled;
  const void *h_prev;        // [B,H] in the type of the operands, or null: zeros (no initial state)
  const float *bias;         // [NH,4,dh]
  const float *s0;           // [4,B,H] or null
  const uint8_t *reset;      // [B] (row stride reset_sb) or null
  long long reset_sb;
  void *h_out;               // [B,H] in the type of the operands
  float *s_out;              // [4,B,H]
  xs_slstm_status *status;
};

constexpr int kStepFeedSlots = 6;
constexpr int kStepFeedSlot = (128 + 64) * 128;  // bytes of a slab in LDS: R of 4 gates x 32 units, the operand rows of 64 batch rows
constexpr int step_feed_lds_bytes() { return kStepFeedSlots * kStepFeedSlot; }

template <bool BF16>
__global__ __launch_bounds__(512) void slstm_step_feed_kernel(StepFeedParams p) {
  constexpr int ESZ = BF16 ? 2 : 4;
  constexpr int D = kStepFeedSlots;
  extern __shared__ __attribute__((aligned(1024))) unsigned char sfeed_lds[];
  const int dh = p.dh, NH = p.NH;
  const int H = NH * dh;
  const long long BH = (long long)p.B * H;
  const int n_ut = dh >> 5, n_rt = (p.B + 63) >> 6;
  int head, tile;  // (workgroup i runs on XCD i % 8: the tiles of a head on as few XCDs as possible, as step_tile_of does)
  {
    const int i = blockIdx.x, tiles = n_ut * n_rt;
    if (NH % 8 == 0) {
      const int hpx = NH / 8, m = i >> 3;
      head = (i & 7) * hpx + m % hpx;
      tile = m / hpx;
    } else if (8 % NH == 0 && tiles % (8 / NH) == 0) {
      head = (i & 7) % NH;
      tile = (i >> 3) * (8 / NH) + (i & 7) / NH;
    } else {
      head = i / tiles;
      tile = i - head * tiles;
    }
  }
  const int a0 = (tile % n_ut) * 32, rowbase = (tile / n_ut) * 64;
  const int tid = threadIdx.x, lane = tid & 63, q = lane >> 4, r16 = lane & 15;
  const int wave = (int)uniform((uint32_t)(tid >> 6));
  const int nslab = dh * ESZ >> 7;
  const uint32_t lds0 = (uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)sfeed_lds);
  if (blockIdx.x == 0 && tid < 16)
    reinterpret_cast<uint32_t *>(p.status)[tid] = (tid == 5 || tid == 6) ? 1u : 0u;  // a step never waits, so it never aborts; one launch; step_kernel = 1

  if (wave >= 4) {
    // ---- feeder wave f: per slab 4 of the 16 KiB of R and 2 of the 8 KiB of operand rows (16 batch rows), 1 KiB (8
    //      rows of 128 bytes) per load, straight into LDS, piece g of row r (16 bytes) at position g ^ (r & 7) of the
    //      row.  Rows past the batch, rows that start a document and a step without a state ask out of range: zeros.
    const int f = wave - 4, sub = lane >> 3, pos = lane & 7;
    const unsigned long long hb = reinterpret_cast<unsigned long long>(p.h_prev ? p.h_prev : p.r_tiled);
    const unsigned long long rb = reinterpret_cast<unsigned long long>(p.r_tiled) + ((long long)head * n_ut + (a0 >> 5)) * nslab * (128 * 128);
    const u32x4_t hrs = {uniform((uint32_t)hb), uniform((uint32_t)(hb >> 32) & 0xFFFFu), (uint32_t)(BH * ESZ), 0x00020000u};
    const u32x4_t rrs = {uniform((uint32_t)rb), uniform((uint32_t)(rb >> 32) & 0xFFFFu), (uint32_t)(nslab * (128 * 128)), 0x00020000u};
    uint32_t hvo[2], rvo[4];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int row = 8 * (2 * f + k) + sub, brow = rowbase + row;
      bool zero = brow >= p.B || !p.h_prev;
      if (!zero && p.reset) zero = p.reset[(long long)brow * p.reset_sb] != 0;
      hvo[k] = zero ? 0x80000000u : (uint32_t)(((long long)brow * H + head * dh) * ESZ + ((pos ^ (row & 7)) << 4));
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int row = 8 * (4 * f + k) + sub;  // gate row / 32, unit row % 32 of the tile
      rvo[k] = (uint32_t)(row * 128 + ((pos ^ (row & 7)) << 4));
    }
    auto request = [&](int s) {
      const int sc = s < nslab ? s : nslab - 1;
      const uint32_t slot = lds0 + (uint32_t)(s % D) * kStepFeedSlot;
#pragma unroll
      for (int k = 0; k < 4; ++k)
        bwd_fetch_to_lds_b128(rrs, uniform(slot + (4 * f + k) * 1024), rvo[k] + (uint32_t)sc * (128 * 128));
#pragma unroll
      for (int k = 0; k < 2; ++k)
        bwd_fetch_to_lds_b128(hrs, uniform(slot + 128 * 128 + (2 * f + k) * 1024), hvo[k] + (uint32_t)sc * 128u);
    };
    for (int s = 0; s < D - 1; ++s) request(s);
    for (int s = 0; s < nslab; ++s) {
      asm volatile("s_waitcnt vmcnt(%0)" :: "n"(6 * (D - 2)) : "memory");  // (slab s has landed)
      lds_barrier();
      request(s + D - 1);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (nothing may land in LDS that another workgroup has been given)
    return;
  }
  const int wr = wave >> 1, wu = wave & 1;

  // ---- pointwise operands of this lane's elements (rows rowbase + 32 wr + 16 ut + r16, units a0 + 16 wu + 4 q .. + 3),
  //      asked for in front of the K loop
  const int ua = a0 + 16 * wu + 4 * q;
  const bool has_s0 = p.s0 != nullptr;
  f32x4 bias4[4], wx4[2][4], c4[2], n4[2], m4[2];
  bool there[2], restart[2];
  long long eo[2];
#pragma unroll
  for (int g = 0; g < 4; ++g) bias4[g] = *reinterpret_cast<const f32x4 *>(p.bias + ((long long)head * 4 + g) * dh + ua);
#pragma unroll
  for (int ut = 0; ut < 2; ++ut) {
    const int row = rowbase + 32 * wr + 16 * ut + r16;
    there[ut] = row < p.B;
    const int rowc = there[ut] ? row : p.B - 1;
    eo[ut] = (long long)rowc * H + head * dh + ua;
    restart[ut] = !has_s0 || (p.reset && p.reset[(long long)rowc * p.reset_sb] != 0);
    const f32x4 zero = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    c4[ut] = has_s0 ? __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p.s0 + BH + eo[ut])) : zero;
    n4[ut] = has_s0 ? __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p.s0 + 2 * BH + eo[ut])) : zero;
    m4[ut] = has_s0 ? __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p.s0 + 3 * BH + eo[ut])) : zero;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const long long o = (long long)rowc * p.wx_sb + (long long)g * H + head * dh + ua;
      if (BF16) {
        const uint2 w = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(p.wx) + o);
        wx4[ut][g] = f32x4{bf16_bits_to_float(w.x & 0xFFFFu), bf16_bits_to_float(w.x >> 16), bf16_bits_to_float(w.y & 0xFFFFu), bf16_bits_to_float(w.y >> 16)};
      } else {
        wx4[ut][g] = *reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(p.wx) + o);
      }
    }
  }

  // ---- R [4 x 32 units x K] . h [64 rows x K], transposed: acc[ut][g][i] = gate g of unit ua + i, row 32 wr + 16 ut + r16;
  //      a K quarter of the sequence kernel is nch k-steps = nch / 2 slabs
  f32x4 acc[2][4], tot[2][4];
#pragma unroll
  for (int ut = 0; ut < 2; ++ut)
#pragma unroll
    for (int g = 0; g < 4; ++g) { acc[ut][g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f}; tot[ut][g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f}; }
  {
    const int swz[2] = {((0 + q) ^ (r16 & 7)) << 4, ((4 + q) ^ (r16 & 7)) << 4};
    const int rrow = (16 * wu + r16) * 128;                 // (gate g: 32 rows further each)
    const int hrow = 128 * 128 + (32 * wr + r16) * 128;     // (row tile ut: 16 rows further)
    const int qslabs = p.nch >> 1;
    for (int s = 0; s < nslab; ++s) {
      lds_barrier();
      const unsigned char *slot = sfeed_lds + (s % D) * kStepFeedSlot;
#pragma unroll
      for (int ch = 0; ch < 2; ++ch) {
        uint4 rv[4], hv[2];
#pragma unroll
        for (int g = 0; g < 4; ++g) rv[g] = *reinterpret_cast<const uint4 *>(slot + rrow + g * (32 * 128) + swz[ch]);
#pragma unroll
        for (int ut = 0; ut < 2; ++ut) hv[ut] = *reinterpret_cast<const uint4 *>(slot + hrow + 16 * ut * 128 + swz[ch]);
#pragma unroll
        for (int ut = 0; ut < 2; ++ut)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            if (BF16) {
              acc[ut][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, rv[g]), __builtin_bit_cast(bf16x8, hv[ut]), acc[ut][g], 0, 0, 0);
            } else {
              const uint32_t rw[4] = {rv[g].x, rv[g].y, rv[g].z, rv[g].w}, hw[4] = {hv[ut].x, hv[ut].y, hv[ut].z, hv[ut].w};
#pragma unroll
              for (int e = 0; e < 4; ++e)
                acc[ut][g] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(rw[e]), __uint_as_float(hw[e]), acc[ut][g], 0, 0, 0);
            }
          }
      }
      if ((s + 1) % qslabs == 0) {  // end of a K quarter: fold it into the running sum (quarter 0 first)
        const bool first = s + 1 == qslabs;
#pragma unroll
        for (int ut = 0; ut < 2; ++ut)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            tot[ut][g] = first ? acc[ut][g] : tot[ut][g] + acc[ut][g];
            acc[ut][g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
          }
      }
    }
    if (nslab % qslabs != 0) {  // (a last quarter that the head dim ends inside)
#pragma unroll
      for (int ut = 0; ut < 2; ++ut)
#pragma unroll
        for (int g = 0; g < 4; ++g) tot[ut][g] = nslab < qslabs ? acc[ut][g] : tot[ut][g] + acc[ut][g];
    }
  }

  // ---- gating and stores (the expressions of slstm_step_tile_kernel)
#pragma unroll
  for (int ut = 0; ut < 2; ++ut) {
    f32x4 yv, cv, nv, mv;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float raw[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) raw[g] = (wx4[ut][g][i] + tot[ut][g][i]) + bias4[g][i];
      CellState st{0.0f, restart[ut] ? 0.0f : c4[ut][i], restart[ut] ? 0.0f : n4[ut][i], restart[ut] ? 0.0f : m4[ut][i]};
      slstm_pointwise(raw[0], raw[1], raw[2], raw[3], st);
      yv[i] = st.y; cv[i] = st.c; nv[i] = st.n; mv[i] = st.m;
    }
    if (!there[ut]) continue;
    const long long o = eo[ut];
    __builtin_nontemporal_store(yv, reinterpret_cast<f32x4 *>(p.s_out + o));
    __builtin_nontemporal_store(cv, reinterpret_cast<f32x4 *>(p.s_out + BH + o));
    __builtin_nontemporal_store(nv, reinterpret_cast<f32x4 *>(p.s_out + 2 * BH + o));
    __builtin_nontemporal_store(mv, reinterpret_cast<f32x4 *>(p.s_out + 3 * BH + o));
    if (BF16) {
      uint2 hw;
      hw.x = float_to_bf16_bits(yv[0]) | (float_to_bf16_bits(yv[1]) << 16);
      hw.y = float_to_bf16_bits(yv[2]) | (float_to_bf16_bits(yv[3]) << 16);
      *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(p.h_out) + o) = hw;
    } else {
      *reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(p.h_out) + o) = yv;
    }
  }
}

}  // namespace
