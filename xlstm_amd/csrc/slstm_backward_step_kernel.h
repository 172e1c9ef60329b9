// The backward pass with ONE LAUNCH PER STEP, for the head dims whose slice of R no compute unit can keep in its
// registers (1024 in bf16, 512 in float32: 4 dh x 64 operands are 512 KiB, the whole register file), where the
// persistent kernels of slstm_backward_kernels.h do not reach.  Included by slstm_hip.hip only.
//
// It is the reference's own decomposition (slstm_backward.cu:291-319: per timestep one pointwise launch and one
// strided-batched GEMM with R transposed; the forward that fills its caches likewise, slstm_forward.cu:176-182), each
// step fused into one kernel:
//
//   slstm_fwd_walk_kernel   the forward walk (what slstm_bwd_prepare_kernel does for the smaller head dims): the launch
//                           of step t multiplies the outputs of step t - 1, which the forward call stored, by R, adds
//                           W.x and the bias, runs the forward's update on the state that the walk keeps in memory, and
//                           leaves the step's nine coefficients.
//   slstm_bwd_step_kernel   the reverse pass: the launch of step t first forms what reaches y_t through the recurrence -
//                           the gate deltas of step t + 1 (left in memory by the launch before, in the type of the
//                           operands) times R transposed - and then the gradient of step t from it, its nine
//                           coefficients and d_h, element by element.  What the steps hand on besides the deltas - the
//                           gradients of c and n - lives in planes 1 and 2 of d_s0 between the launches; a last launch
//                           (t = -1) forms what reaches the y of the initial state.
//
// Both: a workgroup owns 64 batch rows x 32 hidden units (the walk: x 4 gates).  K is walked in slabs of 256 bytes per
// row that four feeder waves bring straight into a ring of LDS slots, slabs ahead of the four waves that multiply, one
// barrier per slab; R lies in memory slab by slab, so a slab of a tile is one piece.  (With the loads in registers of
// the multiplying waves, whose waits the compiler places, a slab took a whole memory latency: 73 us per step of the
// reverse pass at 4 heads of 1024 instead of 19, 29 us per step of the walk.)  The product is formed transposed (units
// on the MFMA M axis), so a lane ends with 4 consecutive units of one batch row and everything pointwise moves as
// 16-byte accesses, asked for in front of the K loop.  Each element of what the launches hand to each other is read
// and written by the same lane of the same workgroup of every launch.  No launch waits for another workgroup: nothing
// here can give up.
#pragma once

namespace {

struct BwdStepParams {
  int B, T, NH, dh;
  int t;                     // the step of this launch; -1: only the gradient of the initial state's y
  int first;                 // the call's last step (its first launch): what reaches y comes from d_s_final
  const float *coef;         // [T][ceil(B/64)][NH][dh/32][2 row tiles of a wave][4 waves][9][64 lanes][4]: as the walk's waves wrote them
  const void *d_h;           // [T,B,H] in the type of the operands
  const float *d_s_final;    // [4,B,H] or null
  const void *r_t;           // R transposed, element (input unit d, gate unit k = g dh + a) of head h, in slabs of 256 bytes of K:
                             // [NH][d / 32][k / KS][d % 32][k % KS], KS = 128 (bf16) or 64 (float32) - what a workgroup
                             // stages per slab is 8 KiB in a row (rows of K, 8 or 16 KiB apart, all fall on one memory channel)
  const void *delta_in;      // the gate deltas of step t + 1 in the type of the operands, tiled the same way:
                             // [ceil(B / 64)][NH][k / KS][b % 64][k % KS]
  void *delta_out;           // ... of step t
  const uint8_t *reset;      // [B,T] or null
  long long reset_sb;
  float *d_wx;               // [B,T,4,NH,dh] float32 (bf16 with d_wx_bf16), strides in elements
  long long d_wx_sb, d_wx_st;
  int d_wx_bf16;
  float *d_s0;               // [4,B,H]
  int cut;
  float clip;
};

constexpr int kBwdStepThreads = 512;    // waves 0-3: MFMAs and the gradient; waves 4-7: bring the operands to LDS
// (Two rings instead - 3 slots for the deltas, which come from the L2, 12 for R transposed, which comes from memory
// every step, with feeder waves of their own - measured 20.4 instead of 19.3 us per step at B 64 x 4 heads of 1024:
// the loop is not waiting for R transposed alone; the kernel moves 60 MB per launch at 3 to 4 TB/s throughout.)
constexpr int kBwdStepSlots = 6;        // slabs in LDS: one being multiplied, the others landing
constexpr int kBwdStepSlot = (64 + 32) * 256;  // bytes of a slab in LDS: the deltas of 64 rows, R transposed of 32 units
constexpr int bwd_step_lds_bytes() { return kBwdStepSlots * kBwdStepSlot; }

template <bool BF16>
__global__ __launch_bounds__(kBwdStepThreads) void slstm_bwd_step_kernel(BwdStepParams p) {
  constexpr int ESZ = BF16 ? 2 : 4;
  constexpr int D = kBwdStepSlots;
  extern __shared__ __attribute__((aligned(1024))) unsigned char bstep_lds[];
  const int dh = p.dh, NH = p.NH;
  const int H = NH * dh;
  const long long BH = (long long)p.B * H;
  const long long KB = (long long)4 * dh * ESZ;  // bytes of a row of K
  const int n_ut = dh >> 5, n_rt = (p.B + 63) >> 6;
  // Workgroup i runs on XCD i % 8: the tiles of a head go to as few XCDs as possible, so that the head's deltas and
  // its rows of R transposed are fetched into few L2s (as the decode step kernel places its tiles).
  int head, tile;
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
  const int t = p.t;
  const bool last_launch = t < 0;
  const bool multiply = !p.first && !p.cut;
  const int nslab = (int)(KB >> 8);
  const long long dtile = ((long long)(rowbase >> 6) * NH + head) * nslab * (64 * 256);  // this row tile's deltas of the head
  const uint32_t lds0 = (uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)bstep_lds);

  if (wave >= 4) {
    // ---- a feeder wave: per slab 4 of the 16 KiB of deltas and 2 of the 8 KiB of R transposed, 1 KiB (4 rows of 256
    //      bytes) per load, straight into LDS.  Such a load fills consecutive LDS, so the rows cannot be padded: piece
    //      g of row r (16 bytes) sits at position g ^ (r & 7) of the row, which keeps the 16-byte reads of the MFMA
    //      waves (8 consecutive rows, one piece) free of bank conflicts.  Slab s is asked for D - 1 slabs ahead, into
    //      the slot that the MFMA waves left before the barrier just passed; the waits are for a constant count
    //      (slabs past the end are asked for like the others - the last slab again, into a slot that nobody reads).
    if (!multiply) return;
    const int f = wave - 4, sub = lane >> 4, pos = lane & 15;
    const bool live = rowbase + 16 * f < p.B;  // (this wave's 16 rows of deltas: not fetched when the batch ends in front of them)
    const unsigned long long db = reinterpret_cast<unsigned long long>(p.delta_in) + dtile;
    const unsigned long long rb = reinterpret_cast<unsigned long long>(p.r_t) + ((long long)head * (dh >> 5) + (a0 >> 5)) * nslab * (32 * 256);
    const u32x4_t drs = {uniform((uint32_t)db), uniform((uint32_t)(db >> 32) & 0xFFFFu), (uint32_t)(nslab * (64 * 256)), 0x00020000u};
    const u32x4_t rrs = {uniform((uint32_t)rb), uniform((uint32_t)(rb >> 32) & 0xFFFFu), (uint32_t)(nslab * (32 * 256)), 0x00020000u};
    uint32_t dvo[4], rvo[2];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int row = 4 * (4 * f + k) + sub;
      dvo[k] = (uint32_t)(row * 256 + ((pos ^ (row & 7)) << 4));
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int row = 4 * (2 * f + k) + sub;
      rvo[k] = (uint32_t)(row * 256 + ((pos ^ (row & 7)) << 4));
    }
    auto request = [&](int s) {
      const int sc = s < nslab ? s : nslab - 1;
      const uint32_t slot = lds0 + (uint32_t)(s % D) * kBwdStepSlot;
      if (live) {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          bwd_fetch_to_lds_b128(drs, uniform(slot + (4 * f + k) * 1024), dvo[k] + (uint32_t)sc * (64 * 256));
      }
#pragma unroll
      for (int k = 0; k < 2; ++k)
        bwd_fetch_to_lds_b128(rrs, uniform(slot + 64 * 256 + (2 * f + k) * 1024), rvo[k] + (uint32_t)sc * (32 * 256));
    };
    for (int s = 0; s < D - 1; ++s) request(s);
    for (int s = 0; s < nslab; ++s) {
      if (live) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(6 * (D - 2)) : "memory");  // (slab s has landed)
      else asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * (D - 2)) : "memory");
      lds_barrier();
      request(s + D - 1);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (nothing may land in LDS that another workgroup has been given)
    return;
  }
  const int wr = wave >> 1, wu = wave & 1;

  // ---- what the gradient of the step needs of this lane's elements: batch rows rowbase + 32 wr + 16 ut + r16,
  //      units a0 + 16 wu + 4 q .. + 3; asked for in front of the K loop
  const int ua = a0 + 16 * wu + 4 * q;
  f32x4 cf[2][9], dhv[2], dcv[2], dnv[2], dyv[2];
  bool there[2], restart[2], cut_off[2];
  long long eo[2];
#pragma unroll
  for (int ut = 0; ut < 2; ++ut) {
    const int row = rowbase + 32 * wr + 16 * ut + r16;
    there[ut] = row < p.B;
    const int rowc = there[ut] ? row : p.B - 1;
    eo[ut] = (long long)rowc * H + head * dh + ua;
    const unsigned char *flags = p.reset ? p.reset + (long long)rowc * p.reset_sb : nullptr;
    restart[ut] = flags && !last_launch && flags[t] != 0;
    // (a row that starts a document at step t + 1 took nothing from y_t)
    cut_off[ut] = flags && !p.first && flags[t + 1] != 0;
    const f32x4 zero = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    dyv[ut] = (p.first && p.d_s_final) ? *reinterpret_cast<const f32x4 *>(p.d_s_final + eo[ut]) : zero;
    if (last_launch) continue;
    const float *carry = p.first ? p.d_s_final : p.d_s0;
    dcv[ut] = carry ? *reinterpret_cast<const f32x4 *>(carry + BH + eo[ut]) : zero;
    dnv[ut] = carry ? *reinterpret_cast<const f32x4 *>(carry + 2 * BH + eo[ut]) : zero;
    // (the coefficients lie as the walk's waves wrote them: per tile, row tile of the wave, wave and coefficient the 64
    // lanes' 16 bytes in a row - a load is 1 KiB in one piece; the lanes of rows past the batch ask for nothing)
    const float *cs = p.coef + ((((long long)t * n_rt * NH * n_ut + ((long long)(rowbase >> 6) * NH + head) * n_ut + (a0 >> 5)) * 2 + ut) * 4 + wave) * (9 * 256) + lane * 4;
#pragma unroll
    for (int j = 0; j < 9; ++j) cf[ut][j] = there[ut] ? *reinterpret_cast<const f32x4 *>(cs + j * 256) : zero;
    const long long ho = (long long)t * BH + eo[ut];
    if (BF16) {
      const uint2 w = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(p.d_h) + ho);
      dhv[ut] = f32x4{bf16_bits_to_float(w.x & 0xFFFFu), bf16_bits_to_float(w.x >> 16), bf16_bits_to_float(w.y & 0xFFFFu), bf16_bits_to_float(w.y >> 16)};
    } else {
      dhv[ut] = *reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(p.d_h) + ho);
    }
  }

  // ---- delta_{t+1} [64 rows x K] . R^T [K x 32 units], transposed: acc[ut][i] = unit ua + i, row 32 wr + 16 ut + r16
  f32x4 acc[2] = {f32x4{0.0f, 0.0f, 0.0f, 0.0f}, f32x4{0.0f, 0.0f, 0.0f, 0.0f}};
  if (multiply) {
    // this lane's pieces of a slab: k-step ch, lane group q -> piece 4 ch + q of the row, at position piece ^ (row & 7)
    // (all rows this lane reads have row & 7 == r16 & 7)
    int swz[4];
#pragma unroll
    for (int ch = 0; ch < 4; ++ch) swz[ch] = ((4 * ch + q) ^ (r16 & 7)) << 4;
    const int drow[2] = {(32 * wr + r16) * 256, (32 * wr + 16 + r16) * 256};
    const int rrow = 64 * 256 + (16 * wu + r16) * 256;
    for (int s = 0; s < nslab; ++s) {
      lds_barrier();  // (slab s is in LDS; the feeder waves may overwrite the slot of slab s - 1)
      const unsigned char *slot = bstep_lds + (s % D) * kBwdStepSlot;
      uint4 rv[4], dv[2][4];
#pragma unroll
      for (int ch = 0; ch < 4; ++ch) {
        rv[ch] = *reinterpret_cast<const uint4 *>(slot + rrow + swz[ch]);
#pragma unroll
        for (int ut = 0; ut < 2; ++ut) dv[ut][ch] = *reinterpret_cast<const uint4 *>(slot + drow[ut] + swz[ch]);
      }
#pragma unroll
      for (int ch = 0; ch < 4; ++ch)
#pragma unroll
        for (int ut = 0; ut < 2; ++ut) {
          if (BF16) {
            acc[ut] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, rv[ch]), __builtin_bit_cast(bf16x8, dv[ut][ch]), acc[ut], 0, 0, 0);
          } else {
            const uint32_t rw[4] = {rv[ch].x, rv[ch].y, rv[ch].z, rv[ch].w}, dw[4] = {dv[ut][ch].x, dv[ut][ch].y, dv[ut][ch].z, dv[ut][ch].w};
#pragma unroll
            for (int e = 0; e < 4; ++e)
              acc[ut] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(rw[e]), __uint_as_float(dw[e]), acc[ut], 0, 0, 0);
          }
        }
    }
  }

  // ---- the gradient of the step (the rule of slstm_bwd_kernel), 4 units of one row at a time
#pragma unroll
  for (int ut = 0; ut < 2; ++ut) {
    if (!there[ut]) continue;
    f32x4 dy;
#pragma unroll
    for (int i = 0; i < 4; ++i) dy[i] = p.first ? dyv[ut][i] : (cut_off[ut] ? 0.0f : acc[ut][i]);
    if (last_launch) {
      *reinterpret_cast<f32x4 *>(p.d_s0 + eo[ut]) = dy;
      *reinterpret_cast<f32x4 *>(p.d_s0 + 3 * BH + eo[ut]) = f32x4{0.0f, 0.0f, 0.0f, 0.0f};  // (the stabiliser's part is zero by the rule)
      continue;
    }
    f32x4 delta[4], dc_prev, dn_prev;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float dyt = dhv[ut][i] + bwd_recurrent_dy(dy[i], p.clip, p.first != 0);
      const float dct = dcv[ut][i] + dyt * cf[ut][0][i];
      const float dnt = dnv[ut][i] - dyt * cf[ut][1][i];
      delta[0][i] = cf[ut][2][i] * dct + cf[ut][3][i] * dnt;
      delta[1][i] = cf[ut][4][i] * dct + cf[ut][5][i] * dnt;
      delta[2][i] = cf[ut][6][i] * dct;
      delta[3][i] = cf[ut][7][i] * dyt;
      // (a row that starts a document at t took nothing from the step before)
      dc_prev[i] = restart[ut] ? 0.0f : cf[ut][8][i] * dct;
      dn_prev[i] = restart[ut] ? 0.0f : cf[ut][8][i] * dnt;
    }
    const int row = rowbase + 32 * wr + 16 * ut + r16;
    const long long wo = (long long)row * p.d_wx_sb + (long long)t * p.d_wx_st + head * dh + ua;
    unsigned char *dout = reinterpret_cast<unsigned char *>(p.delta_out) + dtile + (row & 63) * 256;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int kb = (g * dh + ua) * ESZ;  // byte of the row of K: slab kb / 256, inside it kb % 256
      unsigned char *dst = dout + (long long)(kb >> 8) * (64 * 256) + (kb & 255);
      if (!BF16 || !p.d_wx_bf16) __builtin_nontemporal_store(delta[g], reinterpret_cast<f32x4 *>(p.d_wx + wo + (long long)g * H));  // (as plain stores: 19.9 instead of 19.4 us per step)
      if (BF16) {
        uint2 w;
        w.x = pack_bf16x2(delta[g][0], delta[g][1]);
        w.y = pack_bf16x2(delta[g][2], delta[g][3]);
        if (p.d_wx_bf16) *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(p.d_wx) + wo + (long long)g * H) = w;
        *reinterpret_cast<uint2 *>(dst) = w;
      } else {
        *reinterpret_cast<f32x4 *>(dst) = delta[g];
      }
    }
    *reinterpret_cast<f32x4 *>(p.d_s0 + BH + eo[ut]) = dc_prev;
    *reinterpret_cast<f32x4 *>(p.d_s0 + 2 * BH + eo[ut]) = dn_prev;
  }
}

// ---------------------------------------------------------------------------------------------------------------
// The forward walk.  What a step multiplies by R is known in advance - the outputs that the forward call stored - so
// only the pointwise part of the walk is a chain in time: a launch covers kFwdWalkSteps steps, multiplies their
// operand rows (64 batch rows x the steps) by R in ONE pass over R, keeps the sums of all its steps in registers and
// then walks through the steps.  R is read from memory once per kFwdWalkSteps steps instead of once per step (14.2 us
// a step at B 64 x 4 heads of 1024 with one step per launch).
struct FwdWalkParams {
  int B, T, NH, dh;
  int t;                     // the first step of this launch
  int nsteps;                // its steps: kFwdWalkSteps, fewer at the end of the sequence
  const void *wx;            // [B,T,4,NH,dh], strides in elements
  long long wx_sb, wx_st;
  const void *r_tiled;       // R in the type of the operands, in slabs of 128 bytes of K per tile of 32 units:
                             // [NH][a / 32][k / KS][gate][a % 32][k % KS], KS = 64 (bf16) or 32 (float32)
  const void *h_out;         // [T,B,H] in the type of the operands: the forward's outputs
  const void *h_init;        // [B,H] in that type: the y of the initial state, or null: zeros
  const float *bias;         // [NH,4,dh]
  const float *state_in;     // [4,B,H]: planes 1-3 are c, n, m in front of step t (step 0: the initial state), or null: zeros
  float *state;              // [4,B,H]: planes 1-3 take c, n, m behind the launch's last step
  const uint8_t *reset;      // [B,T] or null
  long long reset_sb;
  float *coef;               // [T][ceil(B/64)][NH][dh/32][2 row tiles of a wave][4 waves][9][64 lanes][4] (the lanes' 4 units)
};

constexpr int kFwdWalkSteps = 4;
constexpr int kFwdWalkSlots = 3;
constexpr int kFwdWalkSlot = (128 + kFwdWalkSteps * 64) * 128;  // bytes of a slab in LDS: R of 4 gates x 32 units, the outputs of 64 rows x the steps
constexpr int fwd_walk_lds_bytes() { return kFwdWalkSlots * kFwdWalkSlot; }

// R [NH][4 dh][dh] into the walk's slabs, and the y plane of the initial state into the type of the operands
template <bool BF16>
__global__ __launch_bounds__(256) void slstm_fwd_walk_init_kernel(const void *r, void *r_tiled, const float *s0, void *h_init, int B, int NH, int dh) {
  constexpr int ESZ = BF16 ? 2 : 4;
  const int nslab = dh * ESZ >> 7;
  const long long pieces = (long long)NH * 4 * dh * nslab * 8;  // 16-byte pieces of R
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < pieces; i += stride) {
    const int piece = (int)(i & 7);
    long long v = i >> 3;
    const int j = (int)(v & 31); v >>= 5;
    const int g = (int)(v & 3); v >>= 2;
    const int slab = (int)(v % nslab); v /= nslab;
    const int ut = (int)(v % (dh >> 5));
    const int head = (int)(v / (dh >> 5));
    const char *src = reinterpret_cast<const char *>(r) + (((long long)head * 4 + g) * dh + ut * 32 + j) * dh * ESZ + slab * 128 + piece * 16;
    reinterpret_cast<uint4 *>(r_tiled)[i] = *reinterpret_cast<const uint4 *>(src);
  }
  const long long BH = (long long)B * NH * dh;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < BH; i += stride) {
    const float y = s0 ? s0[i] : 0.0f;
    if (BF16) reinterpret_cast<uint16_t *>(h_init)[i] = (uint16_t)(pack_bf16x2(y, 0.0f) & 0xFFFFu);
    else reinterpret_cast<float *>(h_init)[i] = y;
  }
}

template <bool BF16>
__global__ __launch_bounds__(kBwdStepThreads) void slstm_fwd_walk_kernel(FwdWalkParams p) {
  constexpr int ESZ = BF16 ? 2 : 4;
  constexpr int D = kFwdWalkSlots, TB = kFwdWalkSteps;
  extern __shared__ __attribute__((aligned(1024))) unsigned char fwalk_lds[];
  const int dh = p.dh, NH = p.NH;
  const int H = NH * dh;
  const long long BH = (long long)p.B * H;
  const int n_ut = dh >> 5, n_rt = (p.B + 63) >> 6;
  int head, tile;  // (placed as in slstm_bwd_step_kernel)
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
  const int t0 = p.t;
  const int nslab = dh * ESZ >> 7;
  const uint32_t lds0 = (uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)fwalk_lds);

  if (wave >= 4) {
    // ---- feeder wave f: per slab the 8 KiB of operand rows of step t0 + f (64 rows x 128 bytes) and 4 of the 16 KiB
    //      of R, 1 KiB (8 rows of 128 bytes) per load, straight into LDS, piece g of row r (16 bytes) at position
    //      g ^ (r & 7) of the row.  Rows past the batch, rows that start a document at that step, a step past the
    //      end and a walk without an initial state ask out of range: the loads return zeros.
    const int f = wave - 4, sub = lane >> 3, pos = lane & 7;
    const int tt = t0 + f;  // this wave's step
    const void *hsrc = tt == 0 ? p.h_init : reinterpret_cast<const void *>(reinterpret_cast<const char *>(p.h_out) + (long long)(tt - 1) * BH * ESZ);
    const bool step_there = f < p.nsteps && hsrc != nullptr;
    const unsigned long long hb = reinterpret_cast<unsigned long long>(step_there ? hsrc : p.r_tiled);
    const unsigned long long rb = reinterpret_cast<unsigned long long>(p.r_tiled) + ((long long)head * n_ut + (a0 >> 5)) * nslab * (128 * 128);
    const u32x4_t hrs = {uniform((uint32_t)hb), uniform((uint32_t)(hb >> 32) & 0xFFFFu), (uint32_t)(BH * ESZ), 0x00020000u};
    const u32x4_t rrs = {uniform((uint32_t)rb), uniform((uint32_t)(rb >> 32) & 0xFFFFu), (uint32_t)(nslab * (128 * 128)), 0x00020000u};
    uint32_t hvo[8], rvo[4];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int row = 8 * k + sub, brow = rowbase + row;
      bool zero = brow >= p.B || !step_there;
      if (!zero && p.reset) zero = p.reset[(long long)brow * p.reset_sb + tt] != 0;
      hvo[k] = zero ? 0x80000000u : (uint32_t)(((long long)brow * H + head * dh) * ESZ + ((pos ^ (row & 7)) << 4));
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int row = 8 * (4 * f + k) + sub;  // gate row / 32, unit row % 32 of the tile
      rvo[k] = (uint32_t)(row * 128 + ((pos ^ (row & 7)) << 4));
    }
    auto request = [&](int s) {
      const int sc = s < nslab ? s : nslab - 1;
      const uint32_t slot = lds0 + (uint32_t)(s % D) * kFwdWalkSlot;
#pragma unroll
      for (int k = 0; k < 4; ++k)
        bwd_fetch_to_lds_b128(rrs, uniform(slot + (4 * f + k) * 1024), rvo[k] + (uint32_t)sc * (128 * 128));
#pragma unroll
      for (int k = 0; k < 8; ++k)
        bwd_fetch_to_lds_b128(hrs, uniform(slot + 128 * 128 + (8 * f + k) * 1024), hvo[k] + (uint32_t)sc * 128u);
    };
    for (int s = 0; s < D - 1; ++s) request(s);
    for (int s = 0; s < nslab; ++s) {
      asm volatile("s_waitcnt vmcnt(%0)" :: "n"(12 * (D - 2)) : "memory");  // (slab s has landed)
      lds_barrier();
      request(s + D - 1);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    return;
  }
  const int wr = wave >> 1, wu = wave & 1;

  // ---- pointwise operands of this lane's elements (rows rowbase + 32 wr + 16 ut + r16, units a0 + 16 wu + 4 q .. + 3)
  const int ua = a0 + 16 * wu + 4 * q;
  f32x4 cv[2], nv[2], mv[2];
  bool there[2];
  uint32_t restart_bits = 0u;  // bit 2 j + ut: the row starts from nothing at step t0 + j
  long long eo[2], wo[2];
  typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
  struct StepWx { typename std::conditional<BF16, u32x2_t, f32x4>::type g[2][4]; };
  auto load_wx = [&](int j, StepWx &w) {
#pragma unroll
    for (int ut = 0; ut < 2; ++ut)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const long long o = wo[ut] + (long long)(t0 + j) * p.wx_st + (long long)g * H;
        if constexpr (BF16) w.g[ut][g] = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t *>(reinterpret_cast<const uint16_t *>(p.wx) + o));
        else w.g[ut][g] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(p.wx) + o));
      }
  };
#pragma unroll
  for (int ut = 0; ut < 2; ++ut) {
    const int row = rowbase + 32 * wr + 16 * ut + r16;
    there[ut] = row < p.B;
    const int rowc = there[ut] ? row : p.B - 1;
    eo[ut] = (long long)rowc * H + head * dh + ua;
    wo[ut] = (long long)rowc * p.wx_sb + head * dh + ua;
#pragma unroll
    for (int j = 0; j < TB; ++j) {
      const bool rs = (j == 0 && !p.state_in) || (p.reset && j < p.nsteps && p.reset[(long long)rowc * p.reset_sb + t0 + j] != 0);
      restart_bits |= rs ? (1u << (2 * j + ut)) : 0u;
    }
    const f32x4 zero = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    cv[ut] = p.state_in ? *reinterpret_cast<const f32x4 *>(p.state_in + BH + eo[ut]) : zero;
    nv[ut] = p.state_in ? *reinterpret_cast<const f32x4 *>(p.state_in + 2 * BH + eo[ut]) : zero;
    mv[ut] = p.state_in ? *reinterpret_cast<const f32x4 *>(p.state_in + 3 * BH + eo[ut]) : zero;
  }
  // (float32: one set of W.x registers, asked for per step - two sets did not fit beside the sums of four steps)
  StepWx wxa, wxb;
  if constexpr (BF16) load_wx(0, wxa);

  // ---- R [4 x 32 units x K] . y_{t-1} [64 rows x K] for every step of the launch, transposed:
  //      acc[j][ut][g][i] = gate g of unit ua + i, row 32 wr + 16 ut + r16, step t0 + j
  f32x4 acc[TB][2][4];
#pragma unroll
  for (int j = 0; j < TB; ++j)
#pragma unroll
    for (int ut = 0; ut < 2; ++ut)
#pragma unroll
      for (int g = 0; g < 4; ++g) acc[j][ut][g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  {
    // this lane's pieces of a slab: k-step ch, lane group q -> piece 4 ch + q of the row, at position piece ^ (row & 7)
    // (all rows this lane reads have row & 7 == r16 & 7)
    const int swz[2] = {((0 + q) ^ (r16 & 7)) << 4, ((4 + q) ^ (r16 & 7)) << 4};
    const int rrow = (16 * wu + r16) * 128;                 // (gate g: 32 rows further each)
    const int hrow = 128 * 128 + (32 * wr + r16) * 128;     // (row tile ut: 16 rows further, step j: 64 rows further)
    for (int s = 0; s < nslab; ++s) {
      lds_barrier();
      const unsigned char *slot = fwalk_lds + (s % D) * kFwdWalkSlot;
#pragma unroll
      for (int ch = 0; ch < 2; ++ch) {
        uint4 rv[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) rv[g] = *reinterpret_cast<const uint4 *>(slot + rrow + g * (32 * 128) + swz[ch]);
#pragma unroll
        for (int j = 0; j < TB; ++j) {
          uint4 hv[2];
#pragma unroll
          for (int ut = 0; ut < 2; ++ut) hv[ut] = *reinterpret_cast<const uint4 *>(slot + hrow + (j * 64 + 16 * ut) * 128 + swz[ch]);
#pragma unroll
          for (int ut = 0; ut < 2; ++ut)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              if (BF16) {
                acc[j][ut][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, rv[g]), __builtin_bit_cast(bf16x8, hv[ut]), acc[j][ut][g], 0, 0, 0);
              } else {
                const uint32_t rw[4] = {rv[g].x, rv[g].y, rv[g].z, rv[g].w}, hw[4] = {hv[ut].x, hv[ut].y, hv[ut].z, hv[ut].w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  acc[j][ut][g] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(rw[e]), __uint_as_float(hw[e]), acc[j][ut][g], 0, 0, 0);
              }
            }
        }
      }
    }
  }

  // ---- the walk through the launch's steps: the forward's update with the gate values kept, and the nine
  //      coefficients of each step's gradient (W.x of the next step is asked for while this one is worked)
  f32x4 bias4[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) bias4[g] = *reinterpret_cast<const f32x4 *>(p.bias + ((long long)head * 4 + g) * dh + ua);
  auto one_step = [&](int j, const StepWx &w) {
#pragma unroll
    for (int ut = 0; ut < 2; ++ut) {
      const bool restart = (restart_bits >> (2 * j + ut)) & 1u;
      f32x4 cf[9];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float raw[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          float wv;
          if constexpr (BF16) {
            const uint32_t wd = i < 2 ? w.g[ut][g][0] : w.g[ut][g][1];
            wv = bf16_bits_to_float((i & 1) ? (wd >> 16) : (wd & 0xFFFFu));
          } else {
            wv = w.g[ut][g][i];
          }
          raw[g] = (wv + acc[j][ut][g][i]) + bias4[g][i];
        }
        CellState st{0.0f, restart ? 0.0f : cv[ut][i], restart ? 0.0f : nv[ut][i], restart ? 0.0f : mv[ut][i]};
        const float c_old = st.c, n_old = st.n;
        GateValues k;
        slstm_pointwise_keep(raw[0], raw[1], raw[2], raw[3], st, k);
        const float omf = __builtin_amdgcn_rcpf(1.0f + __expf(raw[1]));  // 1 - sigmoid(f)
        cf[0][i] = k.og * k.rn;
        cf[1][i] = st.y * k.rn;
        cf[2][i] = k.ig * k.tz;
        cf[3][i] = k.ig;
        cf[4][i] = k.fg * omf * c_old;
        cf[5][i] = k.fg * omf * n_old;
        cf[6][i] = k.ig * (1.0f - k.tz * k.tz);
        cf[7][i] = (1.0f - k.og) * st.y;
        cf[8][i] = k.fg;
        cv[ut][i] = st.c; nv[ut][i] = st.n; mv[ut][i] = st.m;
      }
      if (there[ut]) {
        float *cd = p.coef + ((((long long)(t0 + j) * n_rt * NH * n_ut + ((long long)(rowbase >> 6) * NH + head) * n_ut + (a0 >> 5)) * 2 + ut) * 4 + wave) * (9 * 256) + lane * 4;
#pragma unroll
        // (a store is 1 KiB in one piece: with the coefficients in planes of H floats per batch row two waves shared each
        // 128-byte line of a plane)
        for (int jj = 0; jj < 9; ++jj) *reinterpret_cast<f32x4 *>(cd + jj * 256) = cf[jj];
      }
    }
  };
#pragma unroll
  for (int j = 0; j < TB; ++j) {
    if (j < p.nsteps) {
      if constexpr (BF16) {
        StepWx &cur = (j & 1) ? wxb : wxa;
        StepWx &nxt = (j & 1) ? wxa : wxb;
        if (j + 1 < p.nsteps) load_wx(j + 1, nxt);
        one_step(j, cur);
      } else {
        load_wx(j, wxa);
        one_step(j, wxa);
      }
    }
  }
#pragma unroll
  for (int ut = 0; ut < 2; ++ut) {
    if (!there[ut]) continue;
    *reinterpret_cast<f32x4 *>(p.state + BH + eo[ut]) = cv[ut];
    *reinterpret_cast<f32x4 *>(p.state + 2 * BH + eo[ut]) = nv[ut];
    *reinterpret_cast<f32x4 *>(p.state + 3 * BH + eo[ut]) = mv[ut];
  }
}

}  // namespace
