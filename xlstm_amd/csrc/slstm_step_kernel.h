// The decode step kernel (T = 1).  Included by slstm_hip.hip only (one translation unit),
// after slstm_device_common.h.
#pragma once

namespace {

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
// 16 bytes per lane from a buffer straight into LDS, lane i's bytes at lds_addr + 16 * i (see lds_direct_load_b128;
// this one leaves the cache policy alone: operands, not polls)
__device__ __forceinline__ void lds_direct_fetch_b128(u32x4_t rsrc, uint32_t lds_addr, int voffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :: "s"(lds_addr), "v"(voffset), "s"(rsrc) : "memory", "m0");
}

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
  const void *h_prev;  // optional bf16 copy of the y plane of s0 (see the HB variant)
  int spin_limit;      // bound of the waits between the waves of a workgroup (the pipelined kernel)
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
// HB (only with BF16 and FULL): the recurrent operand comes from StepParams::h_prev, a bf16 copy of
// the y plane of s0 (the h_out of the previous step), instead of being converted from float32:
// half the bytes of the most re-read operand (every unit tile of a row tile reads all of it).
// SPLIT (single-slab variants only): eight waves in two roles.  Waves 0-3 fetch and stage the operands, run the
// MFMAs and gate MFMA row tile 1: they ask for its W.x right behind the operands (W.x comes from HBM unless the
// previous kernel has just written it) and for its old state (which the previous step left in the Infinity Cache)
// once every operand has landed.  Waves 4-7 fetch the pointwise operands of row tile 0, take its sums from the
// MFMA waves through LDS and gate it.  With one role a wave that issues loads faster than the memory system
// takes them stalls in the issue, so the MFMAs could not start before the last pointwise operand had been
// REQUESTED (5.9k of a step's 13k cycles at B = 256, D = 2048) although their own operands had long arrived; and
// the gating (bound by instruction issue and its waits) ran on one wave per SIMD.  What is not needed first must
// also be ASKED FOR later, because everything in flight shares the memory system's queues: with all pointwise
// operands requested up front by the gating waves the first K half is staged at 4.4-4.6k cycles instead of 2.9k.
// Measured slower or equal: the gating waves fetching and staging the second K half (it then arrives later and
// the MFMA waves wait for it), the gating waves fetching row tile 1's operands late and handing them over
// through LDS, streaming loads for the once-read operands.
template <bool BF16, int SLABCH, bool FULL, bool HB = false, bool SPLIT = false>
__global__ __launch_bounds__(SPLIT ? 512 : 256) void slstm_step_tile_kernel(StepParams p, int nch_log2) {
  static_assert(!HB || (BF16 && FULL), "the bf16 operand hint is a steady-state bf16 path");
  static_assert(!SPLIT || SLABCH >= 4, "two roles only with the whole K range in one slab");
  constexpr int HBYTES = HB ? 2 : 4;          // bytes per element of the recurrent operand as it is read
  constexpr int EPC = BF16 ? 8 : 4;
  constexpr int CHK = 4 * EPC;                // input units per MFMA k-step ("chunk")
  constexpr int SLABK = SLABCH * CHK;         // input units per slab
  constexpr int kStepRing = SLABCH >= 4 ? 1 : 4;  // slabs whose loads are in flight
  constexpr int NBUF = SLABCH >= 4 ? 1 : 2;       // LDS buffers
  constexpr int RS = SLABCH * 64 + 16;        // bytes per LDS row: data + pad (conflict-free 16-byte reads)
  constexpr int HITEMS = (SLABK * HBYTES / 16) / 4;  // 16-byte pieces of h each thread stages per slab
  constexpr int RITEMS = SLABCH * 2;            // 16-byte pieces of R each thread stages per slab
  constexpr int ESZ = BF16 ? 2 : 4;
  extern __shared__ __attribute__((aligned(16))) unsigned char step_lds[];
  unsigned char(*hbuf)[64 * RS] = reinterpret_cast<unsigned char(*)[64 * RS]>(step_lds);
  unsigned char(*rbuf)[128 * RS] = reinterpret_cast<unsigned char(*)[128 * RS]>(step_lds + NBUF * 64 * RS);
  // SPLIT: the sums of MFMA row tile 0, [wave][gate][lane] x 16 bytes, behind the operand buffers
  // DIRECT (the steady-state bf16 decode variant): the operands go from memory straight into LDS, no registers and
  // no LDS writes in between.  Such a load fills 1 KiB of consecutive LDS, so the rows cannot be padded: each K
  // half is an array of 256-byte rows (16 pieces of 16 bytes), and piece p of row r sits at position p ^ (r & 7),
  // which keeps the MFMA loop's 16-byte reads (8 consecutive rows, one piece) free of bank conflicts.
  constexpr bool DIRECT = SPLIT && HB && SLABCH == 8;
  constexpr int kHalfH = 64 * 256, kHalfR = 128 * 256;  // bytes of one K half of h / of R
  unsigned char *const hdir = step_lds;
  unsigned char *const rdir = step_lds + 2 * kHalfH;
  f32x4 *const totbuf = reinterpret_cast<f32x4 *>(step_lds + (DIRECT ? 2 * (kHalfH + kHalfR) : NBUF * (64 + 128) * RS));

  const int tid = threadIdx.x & 255;
  const bool gating_role = SPLIT && uniform((uint32_t)(threadIdx.x >> 8)) != 0u;  // scalar: the roles meet at barriers
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

  if (blockIdx.x == 0 && threadIdx.x < 16)
    reinterpret_cast<uint32_t *>(p.status)[tid] = (tid == 5 || tid == 6) ? 1u : 0u;  // a step never waits, so it never aborts; one launch; step_kernel = 1

  const bool has_s0 = FULL || p.s0 != nullptr;
  const bool has_reset = !FULL && p.reset != nullptr;
  const float *s0p = has_s0 ? p.s0 : reinterpret_cast<const float *>(p.wx);                  // stand-ins are only read
  const unsigned char *rsp = has_reset ? p.reset : reinterpret_cast<const unsigned char *>(p.wx);  // in their first 32 bytes

  // ---- staging roles: consecutive lanes take consecutive 16-byte pieces of a row / column.
  // A single slab is staged in NSPLIT phases (K halves): a thread's first HITEMS / NSPLIT items
  // lie in the first half of K, so the MFMA loop can start on it while the second half lands.
  constexpr int HPIECES = SLABK * HBYTES / 16;  // 16-byte pieces of h per row and slab
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
    if (HB) {  // hsrc counts in float units below: a bf16 row is half as long, a 16-byte piece is 4 floats wide
      hzero[j] = false;
      hsrc[j] = reinterpret_cast<const float *>(reinterpret_cast<const uint16_t *>(p.h_prev) + (long long)brow * H + head * dh) +
                hpiece_of(j) * 4;
    } else if (FULL) {
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
  // phase < 0: the whole slab; otherwise the items of that K phase only (as in store_slab)
  auto load_slab = [&](int sidx, uint4 (&hst)[HITEMS], uint4 (&rst)[RITEMS], int phase) {
    const int kbase = sidx * SLABK;
#pragma unroll
    for (int ph = 0; ph < NSPLIT; ++ph) {
      if (phase >= 0 && ph != phase) continue;
#pragma unroll
      for (int j = ph * HIP; j < (ph + 1) * HIP; ++j) {
        if (HB) {
          hst[j] = *reinterpret_cast<const uint4 *>(hsrc[j] + kbase / 2);
        } else if (FULL) {
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
      if (HB) {
        *reinterpret_cast<uint4 *>(dst + piece * 16) = v;  // already in the operand type
      } else if (BF16) {
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
  long long pstamp[10];
  for (int i = 0; i < 10; ++i) pstamp[i] = 0;
  pstamp[0] = clock64();
  const long long pwall0 = wall_clock64();
#endif
  // ---- wave tiling 2 x 2: wave (wr, wu) owns rows 32*wr .. +31 (two MFMA row tiles, index ut below)
  // and units 16*wu .. +15 of all four gates, so a k-step reads 2 h and 4 R fragments from LDS for
  // its 8 MFMAs.  Pointwise operands of this lane: batch rows rowbase + 32*wr + 16*ut + r16,
  // units a0 + 16*wu + 4q .. +3.
  const int wr = wave >> 1, wu = wave & 1;
  // DIRECT: byte offset inside a 256-byte row of this lane's piece of k-step c of a K half: position (4c + q) ^ (row & 7),
  // and the rows this lane reads (of h and of R) all have row & 7 == r16 & 7
  const int swz[4] = {((0 + q) ^ (r16 & 7)) << 4, ((4 + q) ^ (r16 & 7)) << 4, ((8 + q) ^ (r16 & 7)) << 4, ((12 + q) ^ (r16 & 7)) << 4};
  const int ua = a0 + wu * 16 + 4 * q;
  const int uac = (FULL || ua < dh) ? ua : 0;
  const long long col = (long long)head * dh + uac;
  uint2 wxb[2][4];
  float4 wxf[2][4], bias4[4], c4[2], n4[2], m4[2];
  uint32_t pflag[2];
  auto load_bias_and_flags = [&]() {
#pragma unroll
    for (int g = 0; g < 4; ++g)
      bias4[g] = *reinterpret_cast<const float4 *>(p.bias + ((long long)head * 4 + g) * dh + uac);
#pragma unroll
    for (int ut = 0; ut < 2; ++ut) {
      const int brow = rowbase + 32 * wr + 16 * ut + r16;
      const int browc = (FULL || brow < p.B) ? brow : p.B - 1;
      pflag[ut] = FULL ? 0u : rsp[has_reset ? (long long)browc * p.reset_sb : 0];
    }
  };
  auto load_wx = [&](int ut_lo, int ut_hi) {  // W.x of MFMA row tiles [ut_lo, ut_hi)
#pragma unroll
    for (int ut = 0; ut < 2; ++ut) {
      if (ut < ut_lo || ut >= ut_hi) continue;
      const int brow = rowbase + 32 * wr + 16 * ut + r16;
      const int browc = (FULL || brow < p.B) ? brow : p.B - 1;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const long long o = (long long)browc * p.wx_sb + (long long)g * H + col;
        if (BF16) wxb[ut][g] = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(p.wx) + o);
        else wxf[ut][g] = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(p.wx) + o);
      }
    }
  };
  auto load_state = [&](int ut_lo, int ut_hi) {  // the old c, n, m of MFMA row tiles [ut_lo, ut_hi)
#pragma unroll
    for (int ut = 0; ut < 2; ++ut) {
      if (ut < ut_lo || ut >= ut_hi) continue;
      const int brow = rowbase + 32 * wr + 16 * ut + r16;
      const int browc = (FULL || brow < p.B) ? brow : p.B - 1;
      const long long so = (long long)browc * H + col;
      c4[ut] = *reinterpret_cast<const float4 *>(s0p + (has_s0 ? BH + so : 0));
      n4[ut] = *reinterpret_cast<const float4 *>(s0p + (has_s0 ? 2 * BH + so : 0));
      m4[ut] = *reinterpret_cast<const float4 *>(s0p + (has_s0 ? 3 * BH + so : 0));
    }
  };
  f32x4 acc[2][4], tot[2][4];
  // ---- gating of MFMA row tile ut, and its stores
  auto gate_and_store = [&](int ut) {
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
  };
#ifdef XS_PROFILE
  auto profile_end = [&]() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (tid == 0 && blockIdx.x == 9) {
      pstamp[5] = clock64();
      long long *dst = reinterpret_cast<long long *>(reinterpret_cast<char *>(p.status) + 64);
      for (int i = SPLIT ? 4 : 0; i < 6; ++i) dst[i] = pstamp[i] - pstamp[0];
    }
    if (tid == 0) {
      long long *wt = reinterpret_cast<long long *>(reinterpret_cast<char *>(p.status) + 256);
      wt[2 * blockIdx.x] = pwall0;
      wt[2 * blockIdx.x + 1] = wall_clock64();
    }
  };
#endif

  if (SPLIT && gating_role) {
    // The compute unit returns vector-memory data in the order of the requests, across waves: a short pause lets
    // the MFMA waves ask for their operands first (8 and 20 units of 64 cycles measured alike, 0 is 3 % slower).
    __builtin_amdgcn_s_sleep(8);
    load_bias_and_flags();
    load_wx(0, 1);
    load_state(0, 1);
    lds_barrier();  // first K half staged
    lds_barrier();  // second K half staged
    lds_barrier();  // sums of row tile 0 in LDS
#pragma unroll
    for (int g = 0; g < 4; ++g) tot[0][g] = totbuf[(wave * 4 + g) * 64 + lane];
#ifdef XS_PROFILE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    pstamp[4] = clock64();
#endif
    gate_and_store(0);
#ifdef XS_PROFILE
    profile_end();
#endif
    return;  // (no path from here into the code below: the compiler's load bookkeeping of the two roles stays apart)
  }
  // ---- operands, K loop (SPLIT: the MFMA waves).  No load is issued before the roles part: where the two paths
  // touch in the compiler's control-flow graph it waits for every load the other path might have in flight.
  if (DIRECT) {
    // Every load between the first hand-issued operand request and the hand-written wait for the first K half is
    // hand-issued too, so that wait's count is a constant of this file, not of what the compiler emits: the
    // compiler's own loads of this role (the bias) go out BEFORE the requests (the assembly statements clobber
    // memory, so the compiler moves no load across them), W.x goes out behind them as assembly.
    load_bias_and_flags();
    {
      const unsigned long long hb = reinterpret_cast<unsigned long long>(p.h_prev), rb = reinterpret_cast<unsigned long long>(p.r);
      const u32x4_t hrs = {uniform((uint32_t)hb), uniform((uint32_t)(hb >> 32) & 0xFFFFu), uniform((uint32_t)(BH * 2)), 0x00020000u};
      const u32x4_t rrs = {uniform((uint32_t)rb), uniform((uint32_t)(rb >> 32) & 0xFFFFu), uniform((uint32_t)((long long)H * 4 * dh * 2)), 0x00020000u};
      const uint32_t hl = (uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)hdir);
      const uint32_t rl = (uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)rdir);
      const int wv = (int)uniform((uint32_t)wave);
      const int sub = lane >> 4, pos = lane & 15;  // a load covers 4 rows: row sub of them, position pos
#pragma unroll
      for (int half = 0; half < 2; ++half) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {  // h: 16 loads per half and workgroup
          const int row = 4 * (wv * 4 + k) + sub;
          const int voff = (int)(((long long)(rowbase + row) * H + head * dh) * 2) + (half * 16 + (pos ^ (row & 7))) * 16;
          lds_direct_fetch_b128(hrs, uniform(hl + half * kHalfH + (wv * 4 + k) * 1024), voff);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {  // R: 32 loads per half and workgroup
          const int colx = 4 * (wv * 8 + k) + sub;  // column of the workgroup's 128: gate colx / 32, unit colx % 32
          const int voff = (int)(((long long)head * 4 * dh + (long long)(colx >> 5) * dh + a0 + (colx & 31)) * dh * 2) +
                           (half * 16 + (pos ^ (colx & 7))) * 16;
          lds_direct_fetch_b128(rrs, uniform(rl + half * kHalfR + (wv * 8 + k) * 1024), voff);
        }
      }
    }
  } else {
#pragma unroll
    for (int u = 0; u < kStepRing; ++u)
      if (u < nslab) load_slab(u, hring[u], rring[u], -1);
  }

  if (!SPLIT) { load_bias_and_flags(); load_wx(0, 2); load_state(0, 2); }
#pragma unroll
  for (int ut = 0; ut < 2; ++ut)
#pragma unroll
    for (int g = 0; g < 4; ++g) { acc[ut][g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f}; tot[ut][g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f}; }

  // W.x comes from HBM when the previous kernel did not just write it, the old state from the Infinity Cache: the
  // requests for this role's W.x go out early, those for its state once every operand has landed
  if (DIRECT) {
    // W.x of this role's row tile (4 gates x 4 units of one row per lane): hand-issued, see above.  The compiler takes
    // the registers for written when the statement has been issued; they are read behind the wait for all loads in
    // front of the second K half, which names them as operands so that nothing that reads them moves above it.
    const int brow = rowbase + 32 * wr + 16 + r16;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const uint16_t *src = reinterpret_cast<const uint16_t *>(p.wx) + ((long long)brow * p.wx_sb + (long long)g * H + col);
      asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(wxb[1][g]) : "v"(src) : "memory");
    }
  } else if (SPLIT) {
    load_bias_and_flags();
    load_wx(1, 2);
  }
#ifdef XS_PROFILE
  pstamp[1] = clock64();
#endif
  if (DIRECT) {
    // In flight behind the first K half's 12 requests, all hand-issued: 12 requests of the second half and 4 of W.x.
    // At most 16 left = the first K half is in LDS.
    asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  } else {
    store_slab(0, 0, hring[0], rring[0], SLABCH >= 4 ? 0 : -1);
  }
  if (SPLIT) lds_barrier(); else __syncthreads();
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
#ifdef XS_PROFILE
        asm volatile("" :: "v"(tot[0][0][0]), "v"(tot[1][3][3]));
        pstamp[6] = clock64();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        pstamp[7] = clock64();
#endif
        if (DIRECT)  // the second K half and the hand-issued W.x
          asm volatile("s_waitcnt vmcnt(0)" : "+v"(wxb[1][0]), "+v"(wxb[1][1]), "+v"(wxb[1][2]), "+v"(wxb[1][3]) :: "memory");
        else store_slab(0, 0, hring[0], rring[0], 1);
        if (SPLIT) lds_barrier(); else __syncthreads();
        // every operand has landed: the requests for the state this role gates go out now and arrive behind the
        // MFMAs of the second half
        if (SPLIT) load_state(1, 2);
#ifdef XS_PROFILE
        pstamp[8] = clock64();
#endif
      }
#pragma unroll
      for (int cq = 0; cq < (NQ > 0 ? NQ : 1); ++cq) {
        const int ch = w * NQ + cq;
        uint4 hv[2], rv[4];
#pragma unroll
        for (int ut = 0; ut < 2; ++ut)
          hv[ut] = DIRECT ? *reinterpret_cast<const uint4 *>(hdir + (ch >> 2) * kHalfH + (32 * wr + 16 * ut + r16) * 256 + swz[ch & 3])
                          : *reinterpret_cast<const uint4 *>(&hbuf[0][(32 * wr + 16 * ut + r16) * RS + ch * 64 + q * 16]);
#pragma unroll
        for (int g = 0; g < 4; ++g)
          rv[g] = DIRECT ? *reinterpret_cast<const uint4 *>(rdir + (ch >> 2) * kHalfR + (g * 32 + wu * 16 + r16) * 256 + swz[ch & 3])
                         : *reinterpret_cast<const uint4 *>(&rbuf[0][(g * 32 + wu * 16 + r16) * RS + ch * 64 + q * 16]);
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
        if (sidx + kStepRing < nslab) load_slab(sidx + kStepRing, hring[u], rring[u], -1);
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
#endif
  if (SPLIT) {
#pragma unroll
    for (int g = 0; g < 4; ++g) totbuf[(wave * 4 + g) * 64 + lane] = tot[0][g];
    lds_barrier();  // sums of row tile 0 in LDS
#ifdef XS_PROFILE
    if (tid == 0 && blockIdx.x == 9) {
      long long *dst = reinterpret_cast<long long *>(reinterpret_cast<char *>(p.status) + 64);
      for (int i = 0; i < 4; ++i) dst[i] = pstamp[i] - pstamp[0];
      for (int i = 6; i < 10; ++i) dst[i] = pstamp[i] - pstamp[0];
    }
#endif
    gate_and_store(1);
    return;
  }
#ifdef XS_PROFILE
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  pstamp[4] = clock64();
#endif
  gate_and_store(0);
  gate_and_store(1);
#ifdef XS_PROFILE
  profile_end();
#endif
}

}  // namespace
