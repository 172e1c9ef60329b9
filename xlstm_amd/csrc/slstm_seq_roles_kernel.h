// The persistent sequence kernel for workgroups of FOUR row tiles (64 batch rows), with the work split by role.
// Included by slstm_hip.hip only, after slstm_seq_kernel.h (same parameters, same exchange ring, same bits).
#pragma once

#include <type_traits>

namespace {

// With four row tiles per workgroup a tile is needed by the peers again only four iterations after it was computed, so
// an iteration does not wait for another compute unit as long as a tile's h gets round in less than four iterations
// (across two XCDs it just does; see the measurements at the end of this comment).  The kernel with
// the common roles (slstm_seq_kernel, MT = 4) still runs it as ONE chain per SIMD - operand tile out of LDS, 32
// MFMAs, partial sums through LDS, barrier, gating with 9 transcendentals, staging - and the MFMA pipe idles 80 % of
// the time.  Here the chain is cut in two and the halves of consecutive iterations run side by side, two waves per
// SIMD:
//
//   waves 0-3  MFMA waves (K quarter = wave; their 64 columns of R in registers).  A wave fetches its piece of the next
//              operand tile one iteration ahead straight into a second set of registers: ordinary loads that the
//              compiler tracks, issued right behind the wait for the current tile, so that this wait (the only one
//              in these waves, which issue no stores) never covers them.  Per iteration: arrival test, 32 MFMAs,
//              partial sums to LDS, barrier.  No W.x, no gating, no reset flags (a row that starts a document has
//              its sums discarded by the gating waves: the same +0 as a zero operand row gives).
//   waves 4-7  gating waves (rows 4 (wave - 4) .. + 3 of every tile, one element per lane).  Per iteration: barrier,
//              partial sums out of LDS, exponential gating, h to the exchange ring and to the output tensor.  They
//              fetch their own W.x and reset flags eight iterations ahead, from memory straight into rings in LDS
//              (no registers in flight), with hand-issued loads and hand-counted waits (loads and stores share one
//              counter, and a wait the compiler places would be a wait for everything).  There is no feeder and no
//              drainer wave.
//
// Measured and dropped (all bit-identical; us per step at head dim 1024 / 512 / 256 against 3.5 / 2.5 / 4.4 as it is):
//  - the MFMA loop written by hand with exact waits, the loads of the tile TWO iterations on between the MFMA groups of
//    the current one: 5.4 / 2.8 / 5.0 (a tile is asked for before all peers have published it, and every miss costs
//    a full round trip);
//  - the same with the loads of the NEXT tile in two halves, four at the top and four between the first MFMA groups
//    (head dim 1024 only): 3.7.  The MFMA waves get shorter, the gating waves longer by as much: their memory
//    instructions then always find the compute unit's one texture path busy;
//  - the gating waves' stores and fetch moved up behind the barrier, under the latency of the partial sums: 5.5 / 3.0 /
//    5.1, for the same reason (that is when the MFMA waves issue their requests);
//  - a ring of 16 slots instead of 8 (twice as long for the stores to complete before a wait counts them): no change;
//  - the MFMA waves asking for the next tile at different times (wave w behind the first w/4 of its MFMAs, so that the
//    requests of one wave leave while the other three multiply): 3.45 against 3.38; in two groups: 3.50.  The late waves
//    then wait for the arrival instead (a request takes 1,200 cycles and more to come back from the other XCD);
//  - no barrier in the loop (counters in LDS hand the sums over and the buffers back, one buffer per row tile) and the
//    gating by ONE wave per row tile, four elements per lane (the sums are then 16-byte reads and W.x needs no
//    staging), or by TWO waves per row tile, two elements per lane: the same bits, the gating waves busy a fifth of the
//    time - and 5.0 to 5.3 us per step.  Timestamps of one workgroup and per-workgroup sums of all 256 showed why: h of
//    a tile is stored 1,400 to 2,000 cycles behind the sums instead of 1,000 (one wave gates two or four elements),
//    which is too late for the request that the MFMA waves issue one iteration ahead; every request then finds
//    unwritten words and is repeated, a repeat costs a round trip inside the wave that should multiply, and all
//    workgroups alike wait 1,900 cycles per iteration for their operand.  The step is a loop - MFMAs, sums through LDS,
//    gating, store, the way to the other XCD, request, arrival test - that a tile's h goes round once, about 7,000 cycles,
//    and four tiles are in flight: the roles as they are finish just early enough for the requests to be valid;
//  - the arrival test left to the hardware (the MFMAs run on what arrived; an unwritten word is a NaN and makes the sums of
//    its batch row NaNs; the words are looked at only then): the same bits, 400 cycles less in the MFMA waves - and 4.03
//    against 3.33 (2.69 against 2.47 at head dim 512).  Waves that come round sooner ask sooner, find the tile
//    unwritten more often, and then multiply twice: the pace of the loop is the peers' h, not the waves' work.  With
//    the request moved behind a quarter, half, three quarters, all of the MFMAs: 4.05, 3.92, 3.80, 3.57;
//  - (the two XCDs of a head group are (i, i + 4): 3.30 against 3.34 with (i, i + 1) and 3.37 with (i, i + 2).)
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
  constexpr int D = 8;                   // iterations the gating waves fetch W.x ahead (slots of their rings in LDS)
  __shared__ float part[2][NMW][4][kTileFloats];  // [buffer][wave][gate][unit*stride + row]

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

    const int gw = wave - NMW;
    const bool has_mask = p.reset != nullptr;
    const long long flag_sb = has_mask ? p.reset_sb : 0;
    bool lane_ok[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) lane_ok[mt] = FULL ? true : (unit_ok && rowbase + mt * 16 + pb < rend);
#ifdef XS_PROFILE
    long long gprof[6] = {0, 0, 0, 0, 0, 0};
    long long gt_ = clock64();
#define XS_GTICK(i) do { const long long now_ = clock64(); gprof[i] += now_ - gt_; gt_ = now_; } while (0)
#else
#define XS_GTICK(i) do { } while (0)
#endif
    const int lane_ring = member * XTILE + (pb * 16 + pa) * ESZ;
    const uint32_t lane_h = (uint32_t)((pb * H + pa) * ESZ);
    char *const h_member = reinterpret_cast<char *>(p.h_out) + (long long)(head * dh + a0) * ESZ;
    const __amdgpu_buffer_rsrc_t ring = __builtin_amdgcn_make_buffer_rsrc(xbase, 0, kRing * xslot, 0x00020000);
    bool cross_xcd = false;  // (known behind the prologue barrier)
    // ---- h of a tile: to the peers (and the words of h_{t-2} re-armed), and to the output tensor.  Every lane stores to
    //      the ring (lanes outside the batch or the head write words of their own block that nobody polls).
    auto store_tile = [&](int t, int mt, uint32_t hbits) {
      const int tile_off = mt * p.G * XTILE;
      const int off_cur = (t % kRing) * xslot + tile_off;
      const int off_old = ((t + kRing - 2) % kRing) * xslot + tile_off;
      char *const hdst = h_member + ((long long)t * BH + (long long)(rowbase + mt * 16) * H) * ESZ;
      if (BF16) {
        if (cross_xcd) {  // (groups that span two L2s publish past them)
          __builtin_amdgcn_raw_buffer_store_b16((uint16_t)hbits, ring, lane_ring, off_cur, 16);
          __builtin_amdgcn_raw_buffer_store_b16((uint16_t)kSentinel16, ring, lane_ring, off_old, 16);
        } else {
          __builtin_amdgcn_raw_buffer_store_b16((uint16_t)hbits, ring, lane_ring, off_cur, 0);
          __builtin_amdgcn_raw_buffer_store_b16((uint16_t)kSentinel16, ring, lane_ring, off_old, 0);
        }
        if (lane_ok[mt]) *reinterpret_cast<uint16_t *>(hdst + lane_h) = (uint16_t)hbits;
      } else {
        if (cross_xcd) {
          __builtin_amdgcn_raw_buffer_store_b32(hbits, ring, lane_ring, off_cur, 16);
          __builtin_amdgcn_raw_buffer_store_b32(kSentinel32, ring, lane_ring, off_old, 16);
        } else {
          __builtin_amdgcn_raw_buffer_store_b32(hbits, ring, lane_ring, off_cur, 0);
          __builtin_amdgcn_raw_buffer_store_b32(kSentinel32, ring, lane_ring, off_old, 0);
        }
        if (lane_ok[mt]) *reinterpret_cast<uint32_t *>(hdst + lane_h) = hbits;
      }
    };
    if constexpr (FULL) {
      // ---- Every row and unit exists (the common case, and the fast one).  W.x of an iteration takes ONE load per wave,
      //      D iterations ahead, into a ring of registers: lane l fetches units 4 (l & 3) .. + 3 of gate (l >> 2) & 3 for
      //      row l >> 4 of the wave's four rows, as a 32-bit offset on top of a base that the scalar unit steps.  When
      //      they are needed the pieces go through a private corner of LDS to the lanes that gate them (same wave: no
      //      barrier, LDS keeps a wave's order).  The loads are hand-issued and the waits hand-counted (two loads per
      //      iteration; loads and stores share one counter, and a wait the compiler places would be a wait for
      //      everything).  The compiler does not know that a ring register is in flight between the load and the wait:
      //      it must not copy or reuse one in between, and xlstm_amd/isa_check.py checks the compiled code for exactly
      //      that.  (The rings in LDS of the loop for ragged tiles below have no such condition; here they cost 15 %
      //      at config 5's full length, 16.4 against 13.9 ms, and nothing at half of it.)
      constexpr int WB = 4 * ESZ;                 // bytes a lane fetches
      typedef uint32_t wxq_t __attribute__((ext_vector_type(WB / 4)));
      typedef typename std::conditional<BF16, uint16_t, uint32_t>::type wxe_t;
      __shared__ __attribute__((aligned(16))) wxe_t wxt[4][16][16];  // [gating wave][row * 4 + gate][unit]
      const uint32_t lane_wxq =
          (uint32_t)(((long long)(lane >> 4) * p.wx_sb + (long long)((lane >> 2) & 3) * H + 4 * (lane & 3)) * ESZ);
      const uint32_t lane_flagq = (uint32_t)((long long)(lane >> 4) * flag_sb);
      const char *const wx_wave = reinterpret_cast<const char *>(p.wx) + (long long)(head * dh + a0) * ESZ;
      const unsigned char *const flagb = has_mask ? p.reset : reinterpret_cast<const unsigned char *>(p.wx);
      wxq_t wxq[D];
      uint32_t flq[D];
      // the offsets of the D / MT steps a round of D iterations fetches for (clamped to the last step: what the rounds
      // past the end fetch is never looked at), kept as offsets that the scalar unit adds per iteration
      long long pf_wx[D / MT], pf_flag[D / MT];
      auto set_prefetch_steps = [&](int tfirst) {
#pragma unroll
        for (int d = 0; d < D / MT; ++d) {
          const int tp = tfirst + d < p.T ? tfirst + d : p.T - 1;
          pf_wx[d] = (long long)tp * p.wx_st * ESZ;
          pf_flag[d] = has_mask ? tp : 0;
        }
      };
      auto fetch = [&](int u, wxq_t &dst, uint32_t &flag) {  // iteration (round, u): step u / MT of the round, row tile u % MT
        const int mt = u % MT;
        const char *src = wx_wave + (long long)(rowbase + mt * 16 + 4 * gw) * p.wx_sb * ESZ + pf_wx[u / MT];
        const unsigned char *sf = flagb + (long long)(rowbase + mt * 16 + 4 * gw) * flag_sb + pf_flag[u / MT];
        // One statement: the bases are in scalar registers before it starts, and the wait states in front keep a base
        // that the compiler has just moved there with a vector instruction (a reload of a spilled scalar) from being
        // read too early; the compiler does not look for that inside a statement like this.
        if (BF16)
          asm volatile("s_nop 4\n\tglobal_load_dwordx2 %0, %2, %3\n\tglobal_load_ubyte %1, %4, %5"
                       : "=&v"(dst), "=&v"(flag) : "v"(lane_wxq), "s"(src), "v"(lane_flagq), "s"(sf) : "memory");
        else
          asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %2, %3\n\tglobal_load_ubyte %1, %4, %5"
                       : "=&v"(dst), "=&v"(flag) : "v"(lane_wxq), "s"(src), "v"(lane_flagq), "s"(sf) : "memory");
      };
      set_prefetch_steps(0);
#pragma unroll
      for (int u = 0; u < D; ++u) fetch(u, wxq[u], flq[u]);
      lds_barrier();  // prologue barrier
      cross_xcd = cross_s != 0u;
      // (everything fetched so far has landed before the loop is entered: whatever the compiler does to the ring
      // registers at the loop's entry, it does to landed data)
#pragma unroll
      for (int u = 0; u < D; ++u) asm volatile("s_waitcnt vmcnt(0)" : "+v"(wxq[u]), "+v"(flq[u]) :: "memory");
      // (two copies of the loop: calls without a mask run the one without the selects)
      auto gating_loop = [&](auto mask_c) {
        constexpr bool MASK = decltype(mask_c)::value;
        for (int it0 = 0; it0 < NIT; it0 += D) {
          const int t0 = it0 / MT;
          set_prefetch_steps(t0 + D / MT);
#pragma unroll
          for (int u = 0; u < D; ++u) {
            if (it0 + u >= NIT) break;  // (uniform)
            const int mt = u % MT;
            const int buf = u & 1;  // (D is even: the parity of the iteration)
            // Before the barrier, while the MFMA waves still work on this iteration: W.x through the LDS corner.
            // The loads of this iteration have landed when no more than the loads of the D - 1 iterations behind it are
            // outstanding (the stores in between count as well, so this waits for a little more: operations that are
            // several iterations old).
            asm volatile("s_waitcnt vmcnt(%[cnt])" : "+v"(wxq[u]), "+v"(flq[u]) : [cnt] "n"(2 * (D - 1)) : "memory");
            XS_GTICK(1);
            *reinterpret_cast<wxq_t *>(&wxt[gw][lane >> 2][4 * (lane & 3)]) = wxq[u];
            float wxf[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              const uint32_t wxbits = wxt[gw][(lane >> 4) * 4 + g][pa];
              wxf[g] = BF16 ? bf16_bits_to_float(wxbits) : __uint_as_float(wxbits);
            }
            // a row that starts a document: zero state, and R.h counts as the +0 a zero operand row gives
            const bool restart = MASK && (flq[u] & 0xFFu) != 0u;
            asm volatile("" : "+v"(wxf[0]), "+v"(wxf[1]), "+v"(wxf[2]), "+v"(wxf[3]));  // (here, not behind the barrier)
            XS_GTICK(3);
            lds_barrier();  // barrier #it: the partial sums of iteration it are in LDS
            XS_GTICK(0);
            float raw[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              // fixed summation order: wave 0 + wave 1 + wave 2 + wave 3
              float ry = part[buf][0][g][pa * kTileStride + pb];
              ry += part[buf][1][g][pa * kTileStride + pb];
              ry += part[buf][2][g][pa * kTileStride + pb];
              ry += part[buf][3][g][pa * kTileStride + pb];
              if (MASK && restart) ry = 0.0f;
              raw[g] = (wxf[g] + ry) + bias_g[g];
            }
            if (MASK && restart) st[mt] = CellState{0.0f, 0.0f, 0.0f, 0.0f};
#ifdef XS_PROFILE
            asm volatile("" : "+v"(raw[0]), "+v"(raw[1]), "+v"(raw[2]), "+v"(raw[3]));
            XS_GTICK(4);
#endif
            slstm_pointwise(raw[0], raw[1], raw[2], raw[3], st[mt]);
            float y = st[mt].y;
            uint32_t hbits;
            if (BF16) {
              hbits = float_to_bf16_bits(y);
            } else {
              if (y != y) y = __uint_as_float(0x7FC00000u);  // keep the "not written yet" NaN pattern unique
              hbits = __float_as_uint(y);
            }
#ifdef XS_PROFILE
            asm volatile("" : "+v"(hbits));
            XS_GTICK(5);
#endif
            store_tile(t0 + u / MT, mt, hbits);
            XS_GTICK(2);
            fetch(u, wxq[u], flq[u]);  // iteration it + D, into the slot of this one
          }
        }
      };
      if (has_mask) gating_loop(std::integral_constant<bool, true>{});
      else gating_loop(std::integral_constant<bool, false>{});
    } else {
      // ---- W.x and the reset flags travel from memory STRAIGHT INTO LDS (no registers), D - 1 iterations ahead, into a
      //      ring of D slots per gating wave.  Nothing of a load in flight is visible to the compiler, so it cannot move or
      //      copy a destination that has not landed, and the waits are counted by hand: exactly one load (two with a mask)
      //      per iteration, loads and stores share one counter, and a wait the compiler places would be a wait for
      //      everything.  A 16-byte load per lane: the wave's 16 (row, gate) pieces of 16 units land as
      //      [row * 4 + gate][unit], which is how the lanes that gate them read them back.  Rows and units that do not
      //      exist ask for an offset past the end of the buffer descriptor: zeros, no memory access.
      constexpr int UPL = 16 / ESZ;                 // units a lane fetches (8 bf16 / 4 fp32)
      constexpr int LPP = 16 / UPL;                 // lanes per piece
      typedef typename std::conditional<BF16, uint16_t, uint32_t>::type wxe_t;
      __shared__ __attribute__((aligned(16))) wxe_t wxring[4][D][16][16];  // [gating wave][slot][row * 4 + gate][unit]
      __shared__ uint32_t flring[4][D][64];                                  // [gating wave][slot][lane]: the row's flag byte
      constexpr uint32_t kPastEnd = 0xFFFFFF00u;    // (= the descriptors' size)
      const int dl_piece = lane / LPP, dl_part = lane % LPP;
      const bool dl_active = lane < 16 * LPP;       // (bf16: the lower half of the wave fetches)
      uint32_t voff_wx[MT], voff_flag[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int row0 = rowbase + mt * 16 + 4 * gw;  // first row of this wave in the tile
        const bool piece_ok = row0 + (dl_piece >> 2) < rend && a0 + dl_part * UPL < dh;
        voff_wx[mt] = piece_ok ? (uint32_t)(((long long)(dl_piece >> 2) * p.wx_sb + (long long)(dl_piece & 3) * H + dl_part * UPL) * ESZ)
                               : kPastEnd;
        voff_flag[mt] = row0 + (lane >> 4) < rend ? (uint32_t)((long long)(lane >> 4) * flag_sb) : kPastEnd;
      }
      const char *const wx_wave = reinterpret_cast<const char *>(p.wx) + (long long)(head * dh + a0) * ESZ;
      // The offsets of the D / MT steps a round of D iterations fetches for (clamped to the last step: what the rounds
      // past the end fetch is never looked at), kept as offsets that the scalar unit adds per iteration.
      constexpr int NPF = D / MT;
      long long pf_wx[NPF], pf_flag[NPF];
      auto set_prefetch_steps = [&](int tfirst) {
#pragma unroll
        for (int d = 0; d < NPF; ++d) {
          const int tp = tfirst + d < p.T ? tfirst + d : p.T - 1;
          pf_wx[d] = (long long)tp * p.wx_st * ESZ;
          pf_flag[d] = tp;
        }
      };
      auto descriptor = [&](const void *base) {  // raw bytes from base, kPastEnd of them
        const unsigned long long a = reinterpret_cast<unsigned long long>(base);
        return u32x4_t{uniform((uint32_t)a), uniform((uint32_t)(a >> 32) & 0xFFFFu), kPastEnd, 0x00020000u};
      };
      // (The wait states in front: the descriptor may sit in scalar registers that the compiler has just written with a
      // vector instruction, e.g. the reload of a spilled scalar, and it does not look for that hazard inside a statement
      // like this.  M0 = the LDS address of lane 0's bytes.)
      auto fetch = [&](auto mask_c, int mt, int d, int slot) {  // row tile mt of step pf[d] -> ring slot
        const uint32_t vw = voff_wx[mt], vf = voff_flag[mt];
        const long long step_flag = pf_flag[d];
        const char *src = wx_wave + (long long)(rowbase + mt * 16 + 4 * gw) * p.wx_sb * ESZ + pf_wx[d];
        const u32x4_t rs = descriptor(src);
        const uint32_t lds = uniform((uint32_t)(unsigned long long)((__attribute__((address_space(3))) wxe_t *)&wxring[gw][slot][0][0]));
        if (dl_active)
          asm volatile("s_nop 4\n\ts_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                       :: "s"(lds), "v"(vw), "s"(rs) : "memory", "m0");
        if (decltype(mask_c)::value) {
          const unsigned char *sf = p.reset + (long long)(rowbase + mt * 16 + 4 * gw) * flag_sb + step_flag;
          const u32x4_t fs = descriptor(sf);
          const uint32_t fl = uniform((uint32_t)(unsigned long long)((__attribute__((address_space(3))) uint32_t *)&flring[gw][slot][0]));
          asm volatile("s_nop 4\n\ts_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_ubyte %1, %2, 0 offen lds"
                       :: "s"(fl), "v"(vf), "s"(fs) : "memory", "m0");
        }
      };
      // W.x of the iteration in a ring slot -> the lanes that gate it.  Its loads have landed when no more than the loads
      // of the D - 1 iterations fetched behind it are outstanding (the stores in between count as well, so this waits for
      // a little more: operations that are several iterations old).
      auto stage = [&](auto mask_c, int slot, float (&wxf)[4], uint32_t &flag) {
        constexpr bool MASK = decltype(mask_c)::value;
        asm volatile("s_waitcnt vmcnt(%[cnt])" :: [cnt] "n"((MASK ? 2 : 1) * (D - 1)) : "memory");
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const uint32_t wxbits = wxring[gw][slot][(lane >> 4) * 4 + g][pa];
          wxf[g] = BF16 ? bf16_bits_to_float(wxbits) : __uint_as_float(wxbits);
        }
        flag = MASK ? (flring[gw][slot][lane] & 0xFFu) : 0u;
        asm volatile("" : "+v"(wxf[0]), "+v"(wxf[1]), "+v"(wxf[2]), "+v"(wxf[3]), "+v"(flag));  // (here, not where they are used)
      };
      // Per iteration: barrier #it, the partial sums out of LDS, the gating, the tile's three stores, the fetch for
      // iteration it + D into the ring slot just freed, and W.x of iteration it + 1 out of the ring, so that nothing of it
      // is left to do behind the next barrier.  The memory instructions come late in the iteration on purpose: right behind
      // the barrier the MFMA waves issue their requests for the next operand tile, and memory instructions of both kinds
      // queue in the one texture path of the compute unit (measured: with the stores and the fetch of the previous tile
      // moved up behind the barrier, 2.4 -> 3.0 us per step at head dim 512 and 3.5 -> 5.5 at 1024).
      // (Two copies of the loop: calls without a mask run the one without the flag loads and the selects.)
      auto gating_loop = [&](auto mask_c) {
        constexpr bool MASK = decltype(mask_c)::value;
        set_prefetch_steps(0);
#pragma unroll
        for (int j = 0; j < D; ++j) fetch(mask_c, j % MT, j / MT, j);
        float wxf[4];
        uint32_t flag_now;
        stage(mask_c, 0, wxf, flag_now);
        lds_barrier();  // prologue barrier
        cross_xcd = cross_s != 0u;
        for (int it0 = 0; it0 < NIT; it0 += D) {
          const int t0 = it0 / MT;
          set_prefetch_steps(t0 + D / MT);
#pragma unroll
          for (int u = 0; u < D; ++u) {
            if (it0 + u >= NIT) break;  // (uniform)
            const int mt = u % MT;
            const int buf = u & 1;  // (D is even: the parity of the iteration)
            XS_GTICK(3);
            lds_barrier();  // barrier #it: the partial sums of iteration it are in LDS
            XS_GTICK(0);
            // a row that starts a document: zero state, and R.h counts as the +0 a zero operand row gives
            const bool restart = MASK && flag_now != 0u;
            float raw[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              // fixed summation order: wave 0 + wave 1 + wave 2 + wave 3
              float ry = part[buf][0][g][pa * kTileStride + pb];
              ry += part[buf][1][g][pa * kTileStride + pb];
              ry += part[buf][2][g][pa * kTileStride + pb];
              ry += part[buf][3][g][pa * kTileStride + pb];
              if (MASK && restart) ry = 0.0f;
              raw[g] = (wxf[g] + ry) + bias_g[g];
            }
            if (MASK && restart) st[mt] = CellState{0.0f, 0.0f, 0.0f, 0.0f};
#ifdef XS_PROFILE
            asm volatile("" : "+v"(raw[0]), "+v"(raw[1]), "+v"(raw[2]), "+v"(raw[3]));
            XS_GTICK(4);
#endif
            slstm_pointwise(raw[0], raw[1], raw[2], raw[3], st[mt]);
            float y = st[mt].y;
            uint32_t hbits;
            if (BF16) {
              hbits = float_to_bf16_bits(y);
            } else {
              if (y != y) y = __uint_as_float(0x7FC00000u);  // keep the "not written yet" NaN pattern unique
              hbits = __float_as_uint(y);
            }
#ifdef XS_PROFILE
            asm volatile("" : "+v"(hbits));
            XS_GTICK(5);
#endif
            store_tile(t0 + u / MT, mt, hbits);
            fetch(mask_c, mt, u / MT, u);  // iteration it + D, into the slot of this one
            XS_GTICK(2);
            stage(mask_c, (u + 1) % D, wxf, flag_now);
            XS_GTICK(1);
          }
        }
      };
      if (has_mask) gating_loop(std::integral_constant<bool, true>{});
      else gating_loop(std::integral_constant<bool, false>{});
    }
#ifdef XS_PROFILE
    if (lane == 0 && member == 0 && gi == 0 && wave == NMW) {
      long long *dst = reinterpret_cast<long long *>(p.wg_xcc + kStampWord) + 5 * 8;
      for (int i = 0; i < 6; ++i) dst[i] = gprof[i];
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
  lds_barrier();  // prologue barrier: the placement verdict is in LDS

  // poll address of chunk c of row tile mt = per-lane part + a constant: unit k of row r of row tile mt lives at
  // [mt][member k/16][r][k%16] of a ring slot
  const int xlane_ok = ((wave * KW + q * EPC) >> 4) * XTILE + (r16 * 16 + ((q * EPC) & 15)) * ESZ;
  const int xtile_stride = p.G * XTILE;
  auto xconst = [&](int c, int mt_) { return ((c * 4 * EPC) >> 4) * XTILE + mt_ * xtile_stride; };
#ifdef XS_PROFILE
  long long mprof[6] = {0, 0, 0, 0, 0, 0};
  long long mt_ = clock64();
#define XS_MTICK(i) do { const long long now_ = clock64(); mprof[i] += now_ - mt_; mt_ = now_; } while (0)
#else
#define XS_MTICK(i) do { } while (0)
#endif

  // ---- partial R.h over this wave's K slab -> LDS (C layout: lane holds unit column r16, batch rows 4q..4q+3), barrier #it
  auto multiply_and_hand_over = [&](int it, const uint4 (&areg)[CPW]) {
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
    XS_MTICK(3);
    const int buf = it & 1;
#pragma unroll
    for (int g = 0; g < 4; ++g)
      *reinterpret_cast<f32x4 *>(&part[buf][wave][g][r16 * kTileStride + 4 * q]) = acc[g];
    XS_MTICK(4);
    lds_barrier();  // barrier #it
    XS_MTICK(5);
  };
  auto row_exists = [&](int mt) { return FULL ? true : rowbase + mt * 16 + r16 < rend; };
  auto chunk_needed = [&](int mt, int c) { return FULL ? true : (row_exists(mt) && wave * KW + c * 4 * EPC + q * EPC < dh); };

  // ---- step 0: the operand comes from the initial state (or is zero)
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    uint4 areg[CPW];
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      const int k0 = wave * KW + c * 4 * EPC + q * EPC;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (chunk_needed(mt, c) && p.s0) {
        const float *src = p.s0 + (long long)(rowbase + mt * 16 + r16) * H + head * dh + k0;
        if (BF16) {
          const float4 lo = *reinterpret_cast<const float4 *>(src);
          const float4 hi = *reinterpret_cast<const float4 *>(src + 4);
          v.x = pack_bf16x2(lo.x, lo.y); v.y = pack_bf16x2(lo.z, lo.w);
          v.z = pack_bf16x2(hi.x, hi.y); v.w = pack_bf16x2(hi.z, hi.w);
        } else {
          v = *reinterpret_cast<const uint4 *>(src);
        }
      }
      areg[c] = v;
    }
    multiply_and_hand_over(mt, areg);
  }

  if (p.T > 1) {
    // ---- steps 1 .. T-1: a wave fetches its piece of the next tile one iteration ahead into a
    //      second set of registers, right behind the wait for the current tile, so that this wait (the only one in these
    //      waves, which issue no stores) never covers the new loads.
    //      Lanes whose batch row does not exist ask for an offset past the descriptor's end: zeros, no memory traffic;
    //      a chunk past the last member reads zeros as well (the descriptor ends with the slot).
    auto ring_rsrc = [&](int t_) {  // the slot that holds h_{t_ - 1}
      return __builtin_amdgcn_make_buffer_rsrc(xbase + ((t_ + kRing - 1) % kRing) * xslot, 0, xslot, 0x00020000);
    };
    uint4 aset[2][CPW];
    auto request = [&](int itr, uint4 (&dst)[CPW]) {
      if (itr >= NIT) return;
      const int nt = itr / MT, nmt = itr - nt * MT;
      const __amdgpu_buffer_rsrc_t rs = ring_rsrc(nt);
      const int xl = row_exists(nmt) ? xlane_ok : 0x7FFFFF00;
#pragma unroll
      for (int c = 0; c < CPW; ++c) dst[c] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rs, xl, xconst(c, nmt), 16));
    };
#pragma unroll
    for (int c = 0; c < CPW; ++c) aset[1][c] = make_uint4(0, 0, 0, 0);
    request(MT, aset[0]);
    int it = MT;
    for (int t = 1; t < p.T; ++t) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt, ++it) {
        uint4 (&cur)[CPW] = aset[mt & 1];   // (it & 1 == mt & 1)
        uint4 (&nxt)[CPW] = aset[(mt + 1) & 1];
        bool need[CPW];
#pragma unroll
        for (int c = 0; c < CPW; ++c) need[c] = chunk_needed(mt, c);
        XS_MTICK(0);
        // this tile's piece, requested one iteration ago, has to be here now (the compiler's wait: nothing younger is in flight) ...
#pragma unroll
        for (int c = 0; c < CPW; ++c) asm volatile("" : "+v"(cur[c].x), "+v"(cur[c].y), "+v"(cur[c].z), "+v"(cur[c].w));
        XS_MTICK(1);
        // ... and the next tile's goes out
        request(it + 1, nxt);
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
          const int xl = row_exists(mt) ? xlane_ok : 0x7FFFFF00;
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
        uint4 areg[CPW];
#pragma unroll
        for (int c = 0; c < CPW; ++c) areg[c] = need[c] ? cur[c] : make_uint4(0, 0, 0, 0);
        XS_MTICK(2);
        multiply_and_hand_over(it, areg);
      }
    }
  }
#ifdef XS_PROFILE
  if (lane == 0 && member == 0 && gi == 0 && wave < 4) {
    long long *dst = reinterpret_cast<long long *>(p.wg_xcc + kStampWord) + wave * 8;
    for (int i = 0; i < 6; ++i) dst[i] = mprof[i];
  }
#endif
  if (lane == 0 && max_spins) atomicMax(&p.status->max_spins, max_spins);
}

}  // namespace
