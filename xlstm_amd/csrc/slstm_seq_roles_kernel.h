// The persistent sequence kernel for workgroups of FOUR row tiles (64 batch rows), with the work split by role.
// Included by slstm_hip.hip only, after slstm_seq_kernel.h (same parameters, same exchange ring, same bits).
#pragma once

namespace {

// With four row tiles per workgroup a tile is needed by the peers again only four iterations after it was computed, so
// nothing in an iteration waits for another compute unit: an iteration is throughput, not latency.  The kernel with
// the common roles (slstm_seq_kernel, MT = 4) still runs it as ONE chain per SIMD - operand tile out of LDS, 32
// MFMAs, partial sums through LDS, barrier, gating with 9 transcendentals, staging - and the MFMA pipe idles 80 % of
// the time.  Here the chain is cut in two and the halves of consecutive iterations run side by side, two waves per
// SIMD:
//
//   waves 0-3  MFMA waves (K quarter = wave; their 64 columns of R in registers).  A wave fetches its piece of the next
//              operand tile one iteration ahead straight into a second set of registers: ordinary loads that the
//              compiler tracks, issued right behind the wait for the current tile, so that this wait (the only one
//              in these waves, which issue no stores) never covers them.  Per iteration: arrival test, 32 MFMAs,
//              partial sums to LDS, barrier.  No W.x, no gating, no LDS round trip for the operands.
//   waves 4-7  gating waves (rows 4 (wave - 4) .. + 3 of every tile, one element per lane).  Per iteration: barrier,
//              partial sums out of LDS, exponential gating, h to the exchange ring and to the output tensor.  They
//              fetch their own W.x and reset flags straight from memory into a ring of registers, eight iterations
//              ahead, with hand-issued loads and hand-counted waits (loads and stores share one counter, and a wait
//              the compiler places would be a wait for everything).  There is no feeder and no drainer wave.
//
// Barrier #it means "the partial sums of iteration it are in LDS"; the gating waves reach it when they are done with
// iteration it - 1.  The sums are formed in the same order as everywhere else: the same bits.
constexpr int kRolesThreads = 512;

template <bool BF16, int NCH, bool FULL>
__global__ __launch_bounds__(kRolesThreads) void slstm_seq_roles_kernel(SeqParams p) {
  constexpr int MT = 4;
  constexpr int NMW = 4;                 // MFMA waves
  constexpr int CPW = NCH;               // 16-byte chunks of an operand row per lane and MFMA wave
  constexpr int EPC = BF16 ? 8 : 4;      // elements per 16-byte chunk
  constexpr int KW = CPW * 4 * EPC;      // input units per MFMA wave
  constexpr int ESZ = BF16 ? 2 : 4;
  constexpr int D = 8;                   // iterations the gating waves fetch W.x ahead (a ring of registers)
  __shared__ float part[2][NMW][4][kTileFloats];  // [buffer][wave][gate][unit*stride + row]

  __shared__ uint32_t rfl[4][16];               // [slot][row] reset flags, written two iterations ahead by the gating waves
  __shared__ uint32_t cross_s;

  const int wg = blockIdx.x;
  const int ngroups = p.NHL * p.NBT;
  int gi, member;
  seq_place(p, wg, gi, member);
  if (gi >= ngroups) return;
  const int head = p.head0 + gi / p.NBT;
  const int bt = gi % p.NBT;
  const int tid = threadIdx.x;
  const int wave = (int)uniform((uint32_t)(tid >> 6));
  const int lane = tid & 63;
  const long long spin_limit = p.spin_limit > 0 ? p.spin_limit : kDefaultSpinLimit;
  if (tid == 0) cross_s = seq_handshake(p, wg, gi, spin_limit);

  const int dh = p.dh;
  const int H = p.NH * dh;
  const int a0 = member * 16;
  const int rowbase = p.b0 + bt * p.rows_per_wg;
  const int rend = (rowbase + p.rows_per_wg < p.bend) ? rowbase + p.rows_per_wg : p.bend;
  const long long BH = (long long)p.B * H;
  const int NIT = p.T * MT;
  constexpr int XTILE = 16 * 16 * ESZ;               // bytes one member publishes per row tile
  const int xslot = p.G * MT * XTILE;                // bytes one group publishes per step
  char *const xbase = reinterpret_cast<char *>(p.xbuf) + (long long)gi * kRing * xslot;
  if (wave < NMW) __builtin_amdgcn_s_setprio(3);

  if (wave >= NMW) {
    // =====================================================================
    // gating waves
    // =====================================================================
    const int pel = (wave - NMW) * 64 + lane;  // element inside a tile: row * 16 + unit
    const int pa = pel & 15, pb = pel >> 4;
    const int ua = a0 + pa;
    const bool unit_ok = ua < dh;
    const int col = head * dh + (unit_ok ? ua : a0);  // (a unit that does not exist reads a neighbour's words and counts as zero)
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
    // (everything the compiler knows of has landed before the first hand-issued load goes out)
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(bias_g[0]), "+v"(bias_g[1]), "+v"(bias_g[2]), "+v"(bias_g[3]) :: "memory");
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      asm volatile("" : "+v"(st[mt].y), "+v"(st[mt].c), "+v"(st[mt].n), "+v"(st[mt].m));

    // ---- W.x and the reset flag of iteration it -> ring slot it % D.  Exactly 5 loads per iteration (rows, units and
    //      iterations that do not exist are clamped to ones that do and the result is zeroed), so the count at each use is exact.
    uint32_t wxr[D][4], flr[D];
    const char *const wxb = reinterpret_cast<const char *>(p.wx);
    const unsigned char *const flagb = p.reset ? p.reset : reinterpret_cast<const unsigned char *>(p.wx);
    const long long flag_sb = p.reset ? p.reset_sb : 0;
    const uint32_t flag_on = p.reset ? 0xFFu : 0u;
    auto issue = [&](int it, uint32_t (&dst)[4], uint32_t &flag) {
      const int itc = it < NIT ? it : NIT - 1;
      const int t = itc / MT, mt = itc - t * MT;
      const int brow = rowbase + mt * 16 + pb;
      const int browc = brow < rend ? brow : rend - 1;
      const char *src = wxb + ((long long)browc * p.wx_sb + (long long)t * p.wx_st + col) * ESZ;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const char *sg = src + (long long)g * H * ESZ;
        if (BF16) asm volatile("global_load_ushort %0, %1, off" : "=v"(dst[g]) : "v"(sg) : "memory");
        else asm volatile("global_load_dword %0, %1, off" : "=v"(dst[g]) : "v"(sg) : "memory");
      }
      const unsigned char *sf = flagb + (long long)browc * flag_sb + (p.reset ? t : 0);
      asm volatile("global_load_ubyte %0, %1, off" : "=v"(flag) : "v"(sf) : "memory");
    };
#pragma unroll
    for (int u = 0; u < D; ++u) issue(u, wxr[u], flr[u]);
    // the flags of iterations 0 and 1 go to LDS before the first barrier (the MFMA waves clear the operand rows of
    // documents that start); from then on the flag of iteration it + 2 is written during iteration it
    asm volatile("s_waitcnt vmcnt(%[cnt])" : "+v"(flr[0]), "+v"(flr[1]) : [cnt] "n"(5 * (D - 2)) : "memory");
    if (pa == 0) {
      rfl[0][pb] = (rowbase + pb < rend) ? (flr[0] & flag_on) : 0u;
      rfl[1][pb] = (NIT > 1 && rowbase + 16 + pb < rend) ? (flr[1] & flag_on) : 0u;
    }
    lds_barrier();  // prologue barrier
    const bool cross = cross_s != 0u;

    auto gate_tile = [&](int it, int mt, const uint32_t (&wxv)[4], uint32_t flag, uint32_t flag_ahead) {
      const int t = it / MT;
      const int buf = it & 1;
      const int brow = rowbase + mt * 16 + pb;
      const bool row_ok = brow < rend;
      float raw[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        // fixed summation order: wave 0 + wave 1 + wave 2 + wave 3
        float ry = part[buf][0][g][pa * kTileStride + pb];
        ry += part[buf][1][g][pa * kTileStride + pb];
        ry += part[buf][2][g][pa * kTileStride + pb];
        ry += part[buf][3][g][pa * kTileStride + pb];
        float wx = BF16 ? bf16_bits_to_float(wxv[g]) : __uint_as_float(wxv[g]);
        if (!row_ok || !unit_ok) wx = 0.0f;
        raw[g] = (wx + ry) + bias_g[g];
      }
      if (row_ok && (flag & flag_on) != 0u) st[mt] = CellState{0.0f, 0.0f, 0.0f, 0.0f};
      slstm_pointwise(raw[0], raw[1], raw[2], raw[3], st[mt]);
      // ---- publish h_t to the peers, re-arm the words of h_{t-2}, write h_t to the output tensor.  Every lane stores to
      //      the ring (lanes outside the batch or the head write words of their own block that nobody polls).
      float y = st[mt].y;
      if (!BF16 && y != y) y = __uint_as_float(0x7FC00000u);  // keep the "not written yet" NaN pattern unique
      char *const blk = xbase + ((long long)mt * p.G + member) * XTILE + (pb * 16 + pa) * ESZ;
      char *const cur = blk + (t % kRing) * xslot;
      char *const old = blk + ((t + kRing - 2) % kRing) * xslot;
      if (BF16) {
        const uint16_t v = (uint16_t)float_to_bf16_bits(y);
        if (cross) {
          __hip_atomic_store(reinterpret_cast<uint16_t *>(cur), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(reinterpret_cast<uint16_t *>(old), (uint16_t)kSentinel16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
          *reinterpret_cast<uint16_t *>(cur) = v;
          *reinterpret_cast<uint16_t *>(old) = (uint16_t)kSentinel16;
        }
        if (row_ok && unit_ok)
          reinterpret_cast<uint16_t *>(p.h_out)[(long long)t * BH + (long long)brow * H + col] = v;
      } else {
        if (cross) {
          __hip_atomic_store(reinterpret_cast<float *>(cur), y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(reinterpret_cast<float *>(old), __uint_as_float(kSentinel32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
          *reinterpret_cast<float *>(cur) = y;
          *reinterpret_cast<float *>(old) = __uint_as_float(kSentinel32);
        }
        if (row_ok && unit_ok)
          reinterpret_cast<float *>(p.h_out)[(long long)t * BH + (long long)brow * H + col] = y;
      }
      // the reset flags of iteration it + 2 for the MFMA waves
      const int it2 = it + 2, t2 = it2 / MT, mt2 = it2 - t2 * MT;
      if (pa == 0) rfl[it2 & 3][pb] = (it2 < NIT && rowbase + mt2 * 16 + pb < rend) ? (flag_ahead & flag_on) : 0u;
    };

#ifdef XS_PROFILE
    long long gprof[4] = {0, 0, 0, 0};
    long long gt_ = clock64();
#define XS_GTICK(i) do { const long long now_ = clock64(); gprof[i] += now_ - gt_; gt_ = now_; } while (0)
#else
#define XS_GTICK(i) do { } while (0)
#endif
    for (int it0 = 0; it0 < NIT; it0 += D) {
#pragma unroll
      for (int u = 0; u < D; ++u) {
        const int it = it0 + u;
        if (it >= NIT) break;  // (uniform)
        XS_GTICK(3);
        lds_barrier();  // barrier #it: the partial sums of iteration it are in LDS
        XS_GTICK(0);
        // The loads of the iterations up to it + 2 have landed when at most those of the 5 iterations behind are
        // outstanding (stores of the last iteration may be waited for as well; they are a whole iteration old).
        const int u2 = (u + 2) % D;
        asm volatile("s_waitcnt vmcnt(%[cnt])"
                     : "+v"(wxr[u][0]), "+v"(wxr[u][1]), "+v"(wxr[u][2]), "+v"(wxr[u][3]), "+v"(flr[u]), "+v"(flr[u2])
                     : [cnt] "n"(5 * (D - 3)) : "memory");
        XS_GTICK(1);
        gate_tile(it, u % MT, wxr[u], flr[u], flr[u2]);
        XS_GTICK(2);
        issue(it + D, wxr[u], flr[u]);
      }
    }
#ifdef XS_PROFILE
    if (lane == 0 && member == 0 && gi == 0 && wave == NMW) {
      long long *dst = reinterpret_cast<long long *>(p.wg_xcc + 4096 - 128) + 5 * 8;
      for (int i = 0; i < 4; ++i) dst[i] = gprof[i];
    }
#endif
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // ---- final state; NaN all over this workgroup's outputs when a bounded wait ran out anywhere in the call
    const bool poisoned = __hip_atomic_load(&p.status->aborted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int brow = rowbase + mt * 16 + pb;
      if (unit_ok && brow < rend) {
        const long long o = (long long)brow * H + col;
        if (poisoned) st[mt] = CellState{kPoison, kPoison, kPoison, kPoison};
        p.s_out[o] = st[mt].y; p.s_out[BH + o] = st[mt].c; p.s_out[2 * BH + o] = st[mt].n; p.s_out[3 * BH + o] = st[mt].m;
        if (poisoned) {
          for (int t = 0; t < p.T; ++t) {
            const long long ho = (long long)t * BH + o;
            if (BF16) reinterpret_cast<uint16_t *>(p.h_out)[ho] = (uint16_t)0x7FC0u;
            else reinterpret_cast<float *>(p.h_out)[ho] = kPoison;
          }
        }
      }
    }
    return;
  }

  // =======================================================================
  // MFMA waves
  // =======================================================================
  const int q = lane >> 4;     // lane group: which 16-byte chunk of a 4-chunk K slab
  const int r16 = lane & 15;   // MFMA row (A) / column (B, C)
  // ---- R slice -> registers (once).  B operand: column n = unit a0 + r16 of gate g, K chunk c of this wave / lane group.
  uint4 rreg[4][CPW];
  {
    const int a = a0 + r16;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
#pragma unroll
      for (int c = 0; c < CPW; ++c) {
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
  // (R has landed before the first hand-issued request goes out: the counts below are of hand-issued loads only)
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int c = 0; c < CPW; ++c)
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(rreg[g][c].x), "+v"(rreg[g][c].y), "+v"(rreg[g][c].z), "+v"(rreg[g][c].w) :: "memory");
  bool aborted = false;
  uint32_t max_spins = 0;
  lds_barrier();  // prologue barrier: the reset flags of iterations 0 and 1 and the placement verdict are in LDS

  // poll address of chunk c of row tile mt = per-lane part + a compile-time constant: unit k of row r of row tile mt
  // lives at [mt][member k/16][r][k%16].  Lanes whose batch row does not exist ask for an offset past the descriptor's
  // end: zeros, no memory traffic.
  const int xlane_ok = ((wave * KW + q * EPC) >> 4) * XTILE + (r16 * 16 + ((q * EPC) & 15)) * ESZ;
  const int xtile_stride = p.G * XTILE;
  auto xconst = [&](int c, int mt_) { return ((c * 4 * EPC) >> 4) * XTILE + mt_ * xtile_stride; };
  uint4 aset[2][CPW];  // the operand tile being consumed and the one on its way
#pragma unroll
  for (int s_ = 0; s_ < 2; ++s_)
#pragma unroll
    for (int c = 0; c < CPW; ++c) aset[s_][c] = make_uint4(0, 0, 0, 0);
  // requests the piece of iteration itr's tile this wave multiplies; step 0 takes its operand from s0.
  // A chunk past the last member reads zeros (the descriptor ends with the slot).
  auto ring_rsrc = [&](int t_) {
    return __builtin_amdgcn_make_buffer_rsrc(xbase + ((t_ + kRing - 1) % kRing) * xslot, 0, xslot, 0x00020000);
  };
  auto request = [&](int itr, uint4 (&dst)[CPW]) -> bool {
    const int nt = itr / MT, nmt = itr - nt * MT;
    if (!(itr < NIT && nt >= 1)) return false;
    const __amdgpu_buffer_rsrc_t rs = ring_rsrc(nt);
    const int xl = (FULL || rowbase + nmt * 16 + r16 < rend) ? xlane_ok : 0x7FFFFF00;
#pragma unroll
    for (int c = 0; c < CPW; ++c) dst[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rs, xl, xconst(c, nmt), 16));
    return true;
  };
#ifdef XS_PROFILE
  long long mprof[6] = {0, 0, 0, 0, 0, 0};
  long long mt_ = clock64();
#define XS_MTICK(i) do { const long long now_ = clock64(); mprof[i] += now_ - mt_; mt_ = now_; } while (0)
#else
#define XS_MTICK(i) do { } while (0)
#endif
  bool next_requested = false;
  int it = 0;
  for (int t = 0; t < p.T; ++t) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt, ++it) {
      uint4 (&cur)[CPW] = aset[mt & 1];   // (it & 1 == mt & 1)
      uint4 (&nxt)[CPW] = aset[(mt + 1) & 1];
      // ---- 1. A operand: h_{t-1} of batch row (rowbase + mt*16 + r16), this wave's K slab
      const int arow = rowbase + mt * 16 + r16;
      const bool row_ok = FULL ? true : arow < rend;
      const bool row_reset = rfl[it & 3][r16] != 0u;
      bool need[CPW];
#pragma unroll
      for (int c = 0; c < CPW; ++c) need[c] = FULL ? true : (row_ok && wave * KW + c * 4 * EPC + q * EPC < dh);
      XS_MTICK(0);
      const bool this_requested = next_requested;
      if (!this_requested) {  // step 0: the operand comes from the initial state (or is zero)
#pragma unroll
        for (int c = 0; c < CPW; ++c) {
          const int k0 = wave * KW + c * 4 * EPC + q * EPC;
          uint4 v = make_uint4(0, 0, 0, 0);
          if (need[c] && p.s0) {
            const float *src = p.s0 + (long long)arow * H + head * dh + k0;
            if (BF16) {
              const float4 lo = *reinterpret_cast<const float4 *>(src);
              const float4 hi = *reinterpret_cast<const float4 *>(src + 4);
              v.x = pack_bf16x2(lo.x, lo.y); v.y = pack_bf16x2(lo.z, lo.w);
              v.z = pack_bf16x2(hi.x, hi.y); v.w = pack_bf16x2(hi.z, hi.w);
            } else {
              v = *reinterpret_cast<const uint4 *>(src);
            }
          }
          cur[c] = v;
        }
      }
      // this tile's piece, requested one iteration ago, has to be here now (the compiler's wait: nothing younger is in flight) ...
#pragma unroll
      for (int c = 0; c < CPW; ++c) asm volatile("" : "+v"(cur[c].x), "+v"(cur[c].y), "+v"(cur[c].z), "+v"(cur[c].w));
      XS_MTICK(2);
      // ... and the next tile's goes out
      next_requested = request(it + 1, nxt);
      XS_MTICK(1);
      if (this_requested) {
        // one look at everything at once: one mark over all chunks this lane needs
        auto any_missing = [&]() {
          uint32_t mark = 0u;
#pragma unroll
          for (int c = 0; c < CPW; ++c)
            mark = mark_join<BF16>(mark, chunk_mark<BF16>(cur[c]) & (need[c] ? 0xFFFFFFFFu : 0u));
          return __builtin_amdgcn_ballot_w64(mark_has_sentinel<BF16>(mark)) != 0ull;
        };
        if (!aborted && any_missing()) {
          // the tile had not been published completely when it was requested: poll it again, bounded (behind the next
          // tile's requests, which are waited for with it)
          uint32_t spins = 0;
          const __amdgpu_buffer_rsrc_t rs = ring_rsrc(t);
          const int xl = row_ok ? xlane_ok : 0x7FFFFF00;
          for (;;) {
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
            for (int c = 0; c < CPW; ++c) cur[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rs, xl, xconst(c, mt), 16));
            if (!any_missing()) break;
          }
          max_spins = spins > max_spins ? spins : max_spins;
        }
      }
      // ---- 2. partial R.h over this wave's K slab; rows that start a document and chunks that are not needed count as zeros
      uint4 areg[CPW];
#pragma unroll
      for (int c = 0; c < CPW; ++c) areg[c] = (row_reset || !need[c]) ? make_uint4(0, 0, 0, 0) : cur[c];
      XS_MTICK(3);
      f32x4 acc[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) acc[g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int c = 0; c < CPW; ++c) {
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
      // ---- 3. partial tiles -> LDS.  C layout: lane holds unit column r16, batch rows 4q..4q+3
      const int buf = it & 1;
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<f32x4 *>(&part[buf][wave][g][r16 * kTileStride + 4 * q]) = acc[g];
      XS_MTICK(4);
      lds_barrier();  // barrier #it
      XS_MTICK(5);
    }
  }
#ifdef XS_PROFILE
  if (lane == 0 && member == 0 && gi == 0 && wave < 4) {
    long long *dst = reinterpret_cast<long long *>(p.wg_xcc + 4096 - 128) + wave * 8;
    for (int i = 0; i < 6; ++i) dst[i] = mprof[i];
  }
#endif
  if (lane == 0 && max_spins) atomicMax(&p.status->max_spins, max_spins);
}

}  // namespace
