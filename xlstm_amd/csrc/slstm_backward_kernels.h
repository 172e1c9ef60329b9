// Backward pass of the sLSTM cell: two kernels.  Included by slstm_hip.hip only.
//
// What they replace in the reference: SLSTMPointwiseBackward (xlstm/blocks/slstm/src/cuda/slstm_pointwise.cu:118-196) and
// the per-timestep launches around it (slstm_backward.cu:291-319: one pointwise launch and one strided-batched GEMM with
// R transposed per step), plus the state history [4,T+1,B,H] and the gate cache [T,B,4H] that the reference's forward
// writes for them (slstm.cc:79-108).  The rule is the native kernel's: the stabiliser m is a constant of the
// differentiation (its gradient is written as zero, slstm_pointwise.cu:187-190).
//
//   slstm_bwd_prepare_kernel   one thread per (batch row, hidden unit) walks FORWARD through time over
//                              raw = W.x + R.h_{t-1} + bias (R.h_{t-1} for all steps at once is one batched GEMM over the
//                              stored outputs, done by the caller) and leaves, per step and element, the nine
//                              coefficients that make the gradient of a step a handful of multiply-adds:
//                                dc' = dc + dy a0          dn' = dn - dy a1
//                                d_i = a2 dc' + a3 dn'     d_f = a4 dc' + a5 dn'     d_z = a6 dc'     d_o = a7 dy
//                                dc_prev = a8 dc'          dn_prev = a8 dn'
//                              (a0 = o/n', a1 = y'/n', a2 = i' tanh z, a3 = i', a4 = f'(1 - sig f) c, a5 = f'(1 - sig f) n,
//                              a6 = i'(1 - tanh^2 z), a7 = (1 - o) y', a8 = f').  No transcendental is left for the
//                              reverse pass, and the forward kernels stay as they are: an inference call stores nothing.
//   slstm_bwd_kernel           one persistent launch for all T steps, reverse in time.  A workgroup owns one head and 16
//                              batch rows: per step the gate deltas of its rows (16 x 4 dh) go through LDS as the A
//                              operand of MFMAs against R transposed (K = 4 dh gate units, N = dh input units), whose
//                              result - the gradient that reaches y_{t-1} through the recurrence - stays in the
//                              registers of the lanes that need it for the next step (the accumulator layout is the
//                              layout of the pointwise part).  R transposed is read from the L2 every step.
//
// This is a first version: a head is not spread over compute units (no exchange between workgroups), so a step is bound
// by one compute unit's path to the L2 (4 dh x dh operands per step), and head dims are 64, 128 or 256.
#pragma once

namespace {

struct BwdPrepParams {
  int B, T, NH, dh;
  const void *wx;            // [B,T,4,NH,dh], strides in elements
  long long wx_sb, wx_st;
  const float *ry;           // [T,B,NH,4,dh] float32: R.h_{t-1}
  const float *bias;         // [NH,4,dh]
  const float *s0;           // [4,B,H] or null
  const uint8_t *reset;      // [B,T] or null
  long long reset_sb;
  float *coef;               // [T,B,9,H]
};

template <bool BF16>
__global__ __launch_bounds__(256) void slstm_bwd_prepare_kernel(BwdPrepParams p) {
  const int H = p.NH * p.dh;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)p.B * H) return;
  const int b = (int)(idx / H), col = (int)(idx - (long long)b * H);
  const int head = col / p.dh, a = col - head * p.dh;
  const long long BH = (long long)p.B * H;
  float bias_g[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) bias_g[g] = p.bias[((long long)head * 4 + g) * p.dh + a];
  float c = 0.0f, n = 0.0f, m = 0.0f;
  if (p.s0) { c = p.s0[BH + idx]; n = p.s0[2 * BH + idx]; m = p.s0[3 * BH + idx]; }
  auto load_raw = [&](int t, float (&raw)[4]) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const long long wo = (long long)b * p.wx_sb + (long long)t * p.wx_st + (long long)g * H + col;
      const float w = BF16 ? bf16_bits_to_float(reinterpret_cast<const uint16_t *>(p.wx)[wo]) : reinterpret_cast<const float *>(p.wx)[wo];
      raw[g] = (w + p.ry[((((long long)t * p.B + b) * p.NH + head) * 4 + g) * p.dh + a]) + bias_g[g];
    }
  };
  float nxt[4];
  load_raw(0, nxt);
  for (int t = 0; t < p.T; ++t) {
    float raw[4] = {nxt[0], nxt[1], nxt[2], nxt[3]};
    if (t + 1 < p.T) load_raw(t + 1, nxt);  // (one step ahead: the loads of a thread's next step do not depend on this one)
    if (p.reset && p.reset[(long long)b * p.reset_sb + t]) { c = 0.0f; n = 0.0f; m = 0.0f; }
    // the forward's update (slstm_pointwise), with the gate values kept
    const float sigf_neg = __expf(-fabsf(raw[1]));
    const float lfm = m + (fminf(raw[1], 0.0f) - 0.69314718055994531f * __builtin_amdgcn_logf(1.0f + sigf_neg));
    const float mnew = (n == 0.0f) ? raw[0] : fmaxf(raw[0], lfm);
    const float og = __builtin_amdgcn_rcpf(1.0f + __expf(-raw[3]));
    const float ig = fminf(__expf(raw[0] - mnew), 1.0f);
    const float fg = fminf(__expf(lfm - mnew), 1.0f);
    const float tz = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __expf(2.0f * raw[2]));
    const float one_minus_fsig = __builtin_amdgcn_rcpf(1.0f + __expf(raw[1]));  // 1 - sigmoid(f) = sigmoid(-f)
    const float cnew = fg * c + ig * tz;
    const float nnew = fg * n + ig;
    const float rn = __builtin_amdgcn_rcpf(nnew);
    const float ynew = og * cnew * rn;
    float *dst = p.coef + ((long long)t * p.B + b) * 9 * H + col;
    dst[0] = og * rn;
    dst[(long long)H] = ynew * rn;
    dst[2ll * H] = ig * tz;
    dst[3ll * H] = ig;
    dst[4ll * H] = fg * one_minus_fsig * c;
    dst[5ll * H] = fg * one_minus_fsig * n;
    dst[6ll * H] = ig * (1.0f - tz * tz);
    dst[7ll * H] = (1.0f - og) * ynew;
    dst[8ll * H] = fg;
    c = cnew; n = nnew; m = mnew;
  }
}

struct BwdParams {
  int B, T, NH, dh;
  const float *coef;         // [T,B,9,H]
  const void *d_h;           // [T,B,H] in the type of the operands (bf16 or float32): gradient w.r.t. h_out
  const float *d_s_final;    // [4,B,H] or null: gradient w.r.t. the final state (y, c, n are used)
  const void *r_t;           // R transposed, element (input unit d, gate unit k = g dh + a) of head h, in the type of the operands,
                             // tiled as MFMA fragments: [NH][d / 16][k / KC][(k % KC) / EPC][d % 16][k % EPC], EPC = elements
                             // of 16 bytes, KC = 4 EPC (the 64 lanes' operands of one MFMA k-step are 1 KiB in a row)
  const uint8_t *reset;      // [B,T] or null
  long long reset_sb;
  float *d_wx;               // [B,T,4,NH,dh] float32, strides in elements
  long long d_wx_sb, d_wx_st;
  float *d_s0;               // [4,B,H]
};

// NW waves, each with NB 16-column blocks of the result (dh = 16 NB NW: wave w owns input units 16 NB w .. + 16 NB - 1).
// More waves with fewer blocks each keep more loads in flight: a step is made of memory latency.
template <bool BF16, int NB, int NW>
__global__ __launch_bounds__(NW * 64) void slstm_bwd_kernel(BwdParams p) {
  constexpr int ESZ = BF16 ? 2 : 4;
  constexpr int EPC = 16 / ESZ;              // elements of a 16-byte chunk
  constexpr int dh = NB * NW * 16;
  constexpr int K = 4 * dh;
  constexpr int LDK = K + EPC;               // row stride of the delta tile in LDS (16 bytes of padding: rows start in different banks)
  extern __shared__ __attribute__((aligned(16))) char bwd_lds[];
  const int H = p.NH * dh;
  const long long BH = (long long)p.B * H;
  const int head = blockIdx.x % p.NH;
  const int row0 = (blockIdx.x / p.NH) * 16;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, q = lane >> 4, r16 = lane & 15;
  // the lane's elements (i, nb): batch row row0 + 4 q + i, unit (wave NB + nb) 16 + r16 of the head: where the MFMA leaves
  // the result for that row and unit
  float dy[NB][4], dc[NB][4], dn[NB][4];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = row0 + 4 * q + i;
      const long long o = (long long)row * H + head * dh + (wave * NB + nb) * 16 + r16;
      const bool there = row < p.B && p.d_s_final;
      dy[nb][i] = there ? p.d_s_final[o] : 0.0f;
      dc[nb][i] = there ? p.d_s_final[BH + o] : 0.0f;
      dn[nb][i] = there ? p.d_s_final[2 * BH + o] : 0.0f;
    }
  const char *const rt_head = reinterpret_cast<const char *>(p.r_t) + (long long)head * dh * K * ESZ;
  // R transposed does not depend on the step: its fragments are fetched in groups of GK k-steps into two sets of
  // registers, the next group (at the end of a step: the first group of the next step) while the MFMAs of this one run
  constexpr int KSTEPS = K / (4 * EPC);      // 16-byte chunks of a row per lane group
  constexpr int GK = 4;
  constexpr int NG = KSTEPS / GK;            // (even)
  uint4 bq[2][GK][NB];
  auto fetch_group = [&](int j, uint4 (&dst)[GK][NB]) {
#pragma unroll
    for (int g = 0; g < GK; ++g)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        // (tiled: the 64 lanes' chunks of one (column block, k-step) are 1 KiB in a row)
        dst[g][nb] = *reinterpret_cast<const uint4 *>(rt_head + ((((long long)(wave * NB + nb) * KSTEPS + (j * GK + g)) * 64 + lane) << 4));
      }
  };
  fetch_group(0, bq[0]);
  for (int t = p.T - 1; t >= 0; --t) {
    // ---- the gradient of the step, element by element (two rows of the lane at a time, their loads first); the gate
    //      deltas go to LDS (the A operand) and to d_wx
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      float cf[2][NB][9], dh_in[2][NB];
      bool there[2], restart[2];
#pragma unroll
      for (int ii = 0; ii < 2; ++ii) {
        const int row = row0 + 4 * q + 2 * half + ii;
        there[ii] = row < p.B;
        restart[ii] = there[ii] && p.reset && p.reset[(long long)row * p.reset_sb + t];
        const long long e = (long long)t * p.B + (there[ii] ? row : row0);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const int unit = (wave * NB + nb) * 16 + r16;
          const float *src = p.coef + e * 9 * H + head * dh + unit;
#pragma unroll
          for (int j = 0; j < 9; ++j) cf[ii][nb][j] = src[(long long)j * H];
          const long long ho = e * H + head * dh + unit;
          dh_in[ii][nb] = BF16 ? bf16_bits_to_float(reinterpret_cast<const uint16_t *>(p.d_h)[ho]) : reinterpret_cast<const float *>(p.d_h)[ho];
        }
      }
#pragma unroll
      for (int ii = 0; ii < 2; ++ii) {
        const int i = 2 * half + ii;
        const int row = row0 + 4 * q + i;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const int unit = (wave * NB + nb) * 16 + r16;
          float delta[4] = {0.0f, 0.0f, 0.0f, 0.0f};
          if (there[ii]) {
            const float dyt = dh_in[ii][nb] + dy[nb][i];
            const float dct = dc[nb][i] + dyt * cf[ii][nb][0];
            const float dnt = dn[nb][i] - dyt * cf[ii][nb][1];
            delta[0] = cf[ii][nb][2] * dct + cf[ii][nb][3] * dnt;
            delta[1] = cf[ii][nb][4] * dct + cf[ii][nb][5] * dnt;
            delta[2] = cf[ii][nb][6] * dct;
            delta[3] = cf[ii][nb][7] * dyt;
            // (a row that starts a document at t took nothing from the step before)
            dc[nb][i] = restart[ii] ? 0.0f : cf[ii][nb][8] * dct;
            dn[nb][i] = restart[ii] ? 0.0f : cf[ii][nb][8] * dnt;
            float *dw = p.d_wx + (long long)row * p.d_wx_sb + (long long)t * p.d_wx_st + head * dh + unit;
#pragma unroll
            for (int g = 0; g < 4; ++g) dw[(long long)g * H] = delta[g];
          }
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int k = g * dh + unit;
            if (BF16) reinterpret_cast<uint16_t *>(bwd_lds)[(4 * q + i) * LDK + k] = (uint16_t)(pack_bf16x2(delta[g], 0.0f) & 0xFFFFu);
            else reinterpret_cast<float *>(bwd_lds)[(4 * q + i) * LDK + k] = delta[g];
          }
        }
      }
    }
    __syncthreads();
    // ---- what reaches y_{t-1} through the recurrence: delta [16 rows x K] . R^T [K x dh], this wave's dh / 4 columns
    f32x4 acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < NG; ++j) {
      fetch_group(j + 1 < NG ? j + 1 : 0, bq[(j + 1) & 1]);
#pragma unroll
      for (int g = 0; g < GK; ++g) {
        const int k0 = (j * GK + g) * 4 * EPC + q * EPC;
        const uint4 av = *reinterpret_cast<const uint4 *>(bwd_lds + ((long long)r16 * LDK + k0) * ESZ);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const uint4 bv = bq[j & 1][g][nb];
          if (BF16) {
            acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av), __builtin_bit_cast(bf16x8, bv), acc[nb], 0, 0, 0);
          } else {
            const uint32_t aw[4] = {av.x, av.y, av.z, av.w}, bw[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
            for (int e = 0; e < 4; ++e)
              acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(aw[e]), __uint_as_float(bw[e]), acc[nb], 0, 0, 0);
          }
        }
      }
    }
    __syncthreads();  // (the tile is written again in the next step)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = row0 + 4 * q + i;
      const bool restart_row = row < p.B && p.reset && p.reset[(long long)row * p.reset_sb + t];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) dy[nb][i] = restart_row ? 0.0f : acc[nb][i];
    }
  }
  // ---- gradient w.r.t. the initial state (the stabiliser's part is zero by the rule)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = row0 + 4 * q + i;
    if (row >= p.B) continue;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      const long long o = (long long)row * H + head * dh + (wave * NB + nb) * 16 + r16;
      p.d_s0[o] = dy[nb][i]; p.d_s0[BH + o] = dc[nb][i]; p.d_s0[2 * BH + o] = dn[nb][i]; p.d_s0[3 * BH + o] = 0.0f;
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// The reverse pass with a head SPREAD OVER S = dh / 64 workgroups (compute units), the forward's idea turned round:
// workgroup s of a (head, 16-row tile) group owns 64 hidden units.  Its slice of R transposed - the 256 gate units of
// its own 64 units by all dh input units, 128 KiB in bf16 at head dim 256 - stays in the registers of its eight waves
// for the whole call, its MFMAs need only the gate deltas of its OWN units, and what travels per step is a
// reduce-scatter of partial sums: every workgroup writes its 16 x dh partial result, waits for the S - 1 others of its
// group (one arrival counter per step parity, two buffers: a workgroup that is a step ahead writes the other one), and
// adds up, in the order of the workgroups, the S partial sums of its own 64 columns.  Nothing is read from memory per
// step but the coefficients of the workgroup's own 16 x 64 elements.
//
// All workgroups of a group run on one XCD (workgroup i is dispatched to XCD i % 8) and must be resident at once; the
// host launches at most as many as there are compute units.  Waits are bounded: when one runs out the call's abort
// word is set, every workgroup stops waiting, and the gradient of the initial state is overwritten with NaN.
struct BwdSplitParams {
  int B, T, NH, dh;
  const float *coef;
  const void *d_h;
  const float *d_s_final;
  const void *r_ts;          // R transposed per workgroup slice, tiled as MFMA fragments:
                             // [NH][S][dh / 16][KSTEPS][64 lanes][16 bytes], k = g 64 + (unit % 64) inside a slice
  const uint8_t *reset;
  long long reset_sb;
  float *d_wx;
  long long d_wx_sb, d_wx_st;
  float *d_s0;
  float *xch;                // [2][groups][S][16][dh] partial sums
  unsigned int *cnt;         // [groups][2] arrival counters, then one abort word; zero at the start of a call
  long long spin_limit;
};

template <bool BF16, int NB>  // eight waves, NB 16-column blocks each: dh = 128 NB, S = 2 NB workgroups per group
__global__ __launch_bounds__(512) void slstm_bwd_split_kernel(BwdSplitParams p) {
  constexpr int ESZ = BF16 ? 2 : 4;
  constexpr int EPC = 16 / ESZ;
  constexpr int dh = NB * 128;
  constexpr int UW = 64;                      // hidden units of a workgroup
  constexpr int S = dh / UW;
  constexpr int KS = 4 * UW;                  // gate units of a workgroup: its share of K
  constexpr int KSTEPS = KS / (4 * EPC);
  constexpr int LDK = KS + EPC;
  __shared__ __attribute__((aligned(16))) char tile[16 * LDK * ESZ];
  __shared__ int gave_up;
  const int H = p.NH * dh;
  const long long BH = (long long)p.B * H;
  const int ngroups = p.NH * ((p.B + 15) / 16);
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  const int group = (local / S) * 8 + xcd, s = local % S;
  if (group >= ngroups) return;
  const int head = group % p.NH;
  const int row0 = (group / p.NH) * 16;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, q = lane >> 4, r16 = lane & 15;
  unsigned int *const abort_word = p.cnt + 2 * ngroups;
  if (tid == 0) gave_up = 0;
  // ---- this workgroup's slice of R transposed -> registers, once
  uint4 bq[KSTEPS][NB];
  {
    const char *base = reinterpret_cast<const char *>(p.r_ts) + ((long long)(head * S + s) * (dh / 16) * KSTEPS * 64 << 4);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        bq[ks][nb] = *reinterpret_cast<const uint4 *>(base + ((((long long)(wave * NB + nb) * KSTEPS + ks) * 64 + lane) << 4));
  }
  // ---- the thread's two elements: row prow, units s 64 + 2 pu, + 1 of the head
  const int prow = tid >> 5, pu = (tid & 31) * 2;
  const int row = row0 + prow;
  const bool there = row < p.B;
  const long long ecol = (long long)head * dh + s * UW + pu;
  float dy[2] = {0.0f, 0.0f}, dc[2] = {0.0f, 0.0f}, dn[2] = {0.0f, 0.0f};
  if (there && p.d_s_final) {
    const long long o = (long long)row * H + ecol;
#pragma unroll
    for (int e = 0; e < 2; ++e) { dy[e] = p.d_s_final[o + e]; dc[e] = p.d_s_final[BH + o + e]; dn[e] = p.d_s_final[2 * BH + o + e]; }
  }
  __syncthreads();
  // the step's inputs of the thread's elements, fetched one step ahead (while the workgroup waits for its peers)
  f32x2 c9[9], dh2;
  bool restart = false;
  auto fetch_step = [&](int t) {
    if (!there) return;
    restart = p.reset && p.reset[(long long)row * p.reset_sb + t];
    const long long e = (long long)t * p.B + row;
    const float *cf = p.coef + e * 9 * H + ecol;
#pragma unroll
    for (int j = 0; j < 9; ++j) c9[j] = *reinterpret_cast<const f32x2 *>(cf + (long long)j * H);
    if (BF16) {
      const uint32_t w = *reinterpret_cast<const uint32_t *>(reinterpret_cast<const uint16_t *>(p.d_h) + e * H + ecol);
      dh2 = f32x2{__uint_as_float(w << 16), __uint_as_float(w & 0xFFFF0000u)};
    } else {
      dh2 = *reinterpret_cast<const f32x2 *>(reinterpret_cast<const float *>(p.d_h) + e * H + ecol);
    }
  };
  fetch_step(p.T - 1);
  for (int t = p.T - 1; t >= 0; --t) {
    const int n = p.T - 1 - t, par = n & 1;
    // ---- the gradient of the step for the thread's elements; gate deltas to d_wx and, as the A operand, to LDS
    float delta[4][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}, {0.0f, 0.0f}, {0.0f, 0.0f}};
    const bool restart_now = restart;
    if (there) {
      const float dh_in[2] = {dh2[0], dh2[1]};
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const float dyt = dh_in[k] + dy[k];
        const float dct = dc[k] + dyt * c9[0][k];
        const float dnt = dn[k] - dyt * c9[1][k];
        delta[0][k] = c9[2][k] * dct + c9[3][k] * dnt;
        delta[1][k] = c9[4][k] * dct + c9[5][k] * dnt;
        delta[2][k] = c9[6][k] * dct;
        delta[3][k] = c9[7][k] * dyt;
        dc[k] = restart_now ? 0.0f : c9[8][k] * dct;  // (a row that starts a document at t took nothing from the step before)
        dn[k] = restart_now ? 0.0f : c9[8][k] * dnt;
      }
      float *dw = p.d_wx + (long long)row * p.d_wx_sb + (long long)t * p.d_wx_st + ecol;
#pragma unroll
      for (int g = 0; g < 4; ++g) *reinterpret_cast<f32x2 *>(dw + (long long)g * H) = f32x2{delta[g][0], delta[g][1]};
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int k = g * UW + pu;
      if (BF16) *reinterpret_cast<uint32_t *>(tile + ((long long)prow * LDK + k) * 2) = pack_bf16x2(delta[g][0], delta[g][1]);
      else *reinterpret_cast<f32x2 *>(tile + ((long long)prow * LDK + k) * 4) = f32x2{delta[g][0], delta[g][1]};
    }
    __syncthreads();
    // ---- this workgroup's share of what reaches y_{t-1}: delta [16 x KS] . R^T slice [KS x dh], 16 NB columns per wave
    f32x4 acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const uint4 av = *reinterpret_cast<const uint4 *>(tile + ((long long)r16 * LDK + ks * 4 * EPC + q * EPC) * ESZ);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        const uint4 bv = bq[ks][nb];
        if (BF16) {
          acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av), __builtin_bit_cast(bf16x8, bv), acc[nb], 0, 0, 0);
        } else {
          const uint32_t aw[4] = {av.x, av.y, av.z, av.w}, bw[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
          for (int e = 0; e < 4; ++e)
            acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(aw[e]), __uint_as_float(bw[e]), acc[nb], 0, 0, 0);
        }
      }
    }
    // ---- partial sums out (past the first-level cache: the peers read them), then the group's arrival counter
    float *const mine = p.xch + ((((long long)par * ngroups + group) * S + s) * 16) * dh;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        __hip_atomic_store(mine + (long long)(4 * q + i) * dh + (wave * NB + nb) * 16 + r16, acc[nb][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // The stores above are device-scope stores: acknowledged means visible to every compute unit.  Waiting for the
    // acknowledgements and then for the workgroup's other waves orders them in front of the counter without a fence
    // (a device-scope fence writes back and invalidates caches: two of them cost more than the rest of the step).
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (t > 0) fetch_step(t - 1);  // (behind the wait for the acknowledgements, which would be a wait for these loads too)
    __syncthreads();  // (every wave's partial sums are out; the tile may be written again)
    if (tid == 0) {
      unsigned int *const counter = p.cnt + 2 * group + par;
      __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const unsigned int want = (unsigned int)S * (unsigned int)((n >> 1) + 1);
      if (!gave_up) {
        long long spins = 0;
        while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want) {
          if (++spins > p.spin_limit || ((spins & 255) == 0 && __hip_atomic_load(abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
            __hip_atomic_store(abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            gave_up = 1;
            break;
          }
          __builtin_amdgcn_s_sleep(1);
        }
      }
    }
    __syncthreads();
    // ---- the S partial sums of the thread's two columns, in the order of the workgroups (device-scope loads: not from
    //      the first-level cache, which may still hold what the buffer held two steps ago)
    {
      const float *src = p.xch + ((((long long)par * ngroups + group) * S) * 16 + prow) * dh + s * UW + pu;
      float sum0 = 0.0f, sum1 = 0.0f;
#pragma unroll
      for (int peer = 0; peer < S; ++peer) {
        sum0 += __hip_atomic_load(src + (long long)peer * 16 * dh, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        sum1 += __hip_atomic_load(src + (long long)peer * 16 * dh + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      dy[0] = restart_now ? 0.0f : sum0;
      dy[1] = restart_now ? 0.0f : sum1;
    }
  }
  // ---- gradient w.r.t. the initial state (the stabiliser's part is zero by the rule; NaN all over when a wait ran out)
  if (there) {
    const bool poisoned = gave_up || __hip_atomic_load(abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const long long o = (long long)row * H + ecol;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      p.d_s0[o + e] = poisoned ? kPoison : dy[e];
      p.d_s0[BH + o + e] = poisoned ? kPoison : dc[e];
      p.d_s0[2 * BH + o + e] = poisoned ? kPoison : dn[e];
      p.d_s0[3 * BH + o + e] = 0.0f;
    }
  }
}

}  // namespace
