// The reverse pass with ONE LAUNCH PER STEP, for the head dims whose slice of R transposed no compute unit can keep in
// its registers (1024 in bf16, 512 in float32: 4 dh x 64 operands are 512 KiB, the whole register file), where the
// persistent kernels of slstm_backward_kernels.h do not reach.  Included by slstm_hip.hip only.
//
// It is the reference's own decomposition (slstm_backward.cu:291-319: per timestep one pointwise launch and one
// strided-batched GEMM with R transposed), fused into one kernel per step and turned round: the launch of step t first
// forms what reaches y_t through the recurrence - the gate deltas of step t + 1 (left in memory by the launch before,
// in the type of the operands) times R transposed - and then the gradient of step t from it, its nine coefficients
// and d_h, element by element.  A workgroup owns 64 batch rows x 32 hidden units: K = 4 dh gate units are walked in
// slabs of 256 bytes per row that go through LDS (two buffers, one barrier per slab, the loads of four slabs in flight
// in registers); the product is formed transposed (units on the MFMA M axis), so a lane ends with 4 consecutive units
// of one batch row and everything pointwise moves as 16-byte accesses, asked for in front of the K loop.  What the
// steps hand on besides the deltas - the gradients of c and n - lives in planes 1 and 2 of d_s0 between the launches
// (each element is read and written by the same lane of the same workgroup of every launch); a last launch (t = -1)
// forms what reaches the y of the initial state.  No launch waits for another workgroup: nothing here can give up.
#pragma once

namespace {

struct BwdStepParams {
  int B, T, NH, dh;
  int t;                     // the step of this launch; -1: only the gradient of the initial state's y
  int first;                 // the call's last step (its first launch): what reaches y comes from d_s_final
  const float *coef;         // [T,B,9,H]
  const void *d_h;           // [T,B,H] in the type of the operands
  const float *d_s_final;    // [4,B,H] or null
  const void *r_t;           // [NH][dh][4 dh]: R transposed, element (input unit d, gate unit k = g dh + a), K contiguous
  const void *delta_in;      // [B][NH][4 dh] in the type of the operands: the gate deltas of step t + 1
  void *delta_out;           // ... of step t
  const uint8_t *reset;      // [B,T] or null
  long long reset_sb;
  float *d_wx;               // [B,T,4,NH,dh] float32, strides in elements
  long long d_wx_sb, d_wx_st;
  float *d_s0;               // [4,B,H]
  int cut;
  float clip;
};

constexpr int kBwdStepThreads = 256;
constexpr int kBwdStepRow = 256 + 16;   // bytes of an LDS row: a slab's 256 bytes and padding (conflict-free 16-byte reads)
constexpr int kBwdStepRing = 4;         // slabs whose loads are in flight
constexpr int bwd_step_lds_bytes() { return 2 * (64 + 32) * kBwdStepRow; }

template <bool BF16>
__global__ __launch_bounds__(kBwdStepThreads) void slstm_bwd_step_kernel(BwdStepParams p) {
  constexpr int ESZ = BF16 ? 2 : 4;
  constexpr int RS = kBwdStepRow;
  extern __shared__ __attribute__((aligned(16))) unsigned char bstep_lds[];
  unsigned char(*dbuf)[64 * RS] = reinterpret_cast<unsigned char(*)[64 * RS]>(bstep_lds);
  unsigned char(*rbuf)[32 * RS] = reinterpret_cast<unsigned char(*)[32 * RS]>(bstep_lds + 2 * 64 * RS);
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
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, q = lane >> 4, r16 = lane & 15;
  const int wr = wave >> 1, wu = wave & 1;
  const int t = p.t;
  const bool last_launch = t < 0;
  const bool multiply = !p.first && !p.cut;

  // ---- staging roles: consecutive lanes take consecutive 16-byte pieces of a row (16 pieces a slab)
  const unsigned char *dsrc[4], *rsrc[2];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int idx = tid + 256 * j, row = rowbase + (idx >> 4);
    const int rowc = row < p.B ? row : p.B - 1;  // (rows past the batch read a row that is there; their results are dropped)
    dsrc[j] = reinterpret_cast<const unsigned char *>(p.delta_in) + ((long long)rowc * NH + head) * KB + (idx & 15) * 16;
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int idx = tid + 256 * j;
    rsrc[j] = reinterpret_cast<const unsigned char *>(p.r_t) + ((long long)head * dh + a0 + (idx >> 4)) * KB + (idx & 15) * 16;
  }
  uint4 dring[kBwdStepRing][4], rring[kBwdStepRing][2];
  auto load_slab = [&](int s, uint4 (&d)[4], uint4 (&r)[2]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) d[j] = *reinterpret_cast<const uint4 *>(dsrc[j] + (long long)s * 256);
#pragma unroll
    for (int j = 0; j < 2; ++j) r[j] = *reinterpret_cast<const uint4 *>(rsrc[j] + (long long)s * 256);
  };
  auto store_slab = [&](int buf, const uint4 (&d)[4], const uint4 (&r)[2]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int idx = tid + 256 * j;
      *reinterpret_cast<uint4 *>(&dbuf[buf][(idx >> 4) * RS + (idx & 15) * 16]) = d[j];
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int idx = tid + 256 * j;
      *reinterpret_cast<uint4 *>(&rbuf[buf][(idx >> 4) * RS + (idx & 15) * 16]) = r[j];
    }
  };
  const int nslab = (int)(KB >> 8);
  if (multiply) {
#pragma unroll
    for (int u = 0; u < kBwdStepRing; ++u)
      if (u < nslab) load_slab(u, dring[u], rring[u]);
  }

  // ---- what the gradient of the step needs of this lane's elements: batch rows rowbase + 32 wr + 16 ut + r16,
  //      units a0 + 16 wu + 4 q .. + 3; asked for behind the first operands
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
    const float *cs = p.coef + ((long long)t * p.B + rowc) * 9 * H + head * dh + ua;
#pragma unroll
    for (int j = 0; j < 9; ++j) cf[ut][j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(cs + (long long)j * H));
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
    store_slab(0, dring[0], rring[0]);
    __syncthreads();
    for (int s0i = 0; s0i < nslab; s0i += kBwdStepRing) {
#pragma unroll
      for (int u = 0; u < kBwdStepRing; ++u) {
        const int sidx = s0i + u;
        if (sidx < nslab) {
          const int buf = sidx & 1;
#pragma unroll
          for (int ch = 0; ch < 4; ++ch) {
            const uint4 rv = *reinterpret_cast<const uint4 *>(&rbuf[buf][(16 * wu + r16) * RS + ch * 64 + q * 16]);
#pragma unroll
            for (int ut = 0; ut < 2; ++ut) {
              const uint4 dv = *reinterpret_cast<const uint4 *>(&dbuf[buf][(32 * wr + 16 * ut + r16) * RS + ch * 64 + q * 16]);
              if (BF16) {
                acc[ut] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, rv), __builtin_bit_cast(bf16x8, dv), acc[ut], 0, 0, 0);
              } else {
                const uint32_t rw[4] = {rv.x, rv.y, rv.z, rv.w}, dw[4] = {dv.x, dv.y, dv.z, dv.w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  acc[ut] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(rw[e]), __uint_as_float(dw[e]), acc[ut], 0, 0, 0);
              }
            }
          }
          // slab sidx went to LDS one iteration ago: its ring entry takes the loads of slab sidx + kBwdStepRing
          if (sidx + kBwdStepRing < nslab) load_slab(sidx + kBwdStepRing, dring[u], rring[u]);
          if (sidx + 1 < nslab) {
            const int un = (u + 1) % kBwdStepRing;
            store_slab((sidx + 1) & 1, dring[un], rring[un]);  // (the other buffer was last read before the previous barrier)
            __syncthreads();
          }
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
    float *dw = p.d_wx + (long long)row * p.d_wx_sb + (long long)t * p.d_wx_st + head * dh + ua;
    unsigned char *dout = reinterpret_cast<unsigned char *>(p.delta_out) + ((long long)row * NH + head) * KB;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      __builtin_nontemporal_store(delta[g], reinterpret_cast<f32x4 *>(dw + (long long)g * H));
      if (BF16) {
        uint2 w;
        w.x = pack_bf16x2(delta[g][0], delta[g][1]);
        w.y = pack_bf16x2(delta[g][2], delta[g][3]);
        *reinterpret_cast<uint2 *>(dout + ((long long)g * dh + ua) * 2) = w;
      } else {
        *reinterpret_cast<f32x4 *>(dout + ((long long)g * dh + ua) * 4) = delta[g];
      }
    }
    *reinterpret_cast<f32x4 *>(p.d_s0 + BH + eo[ut]) = dc_prev;
    *reinterpret_cast<f32x4 *>(p.d_s0 + 2 * BH + eo[ut]) = dn_prev;
  }
}

}  // namespace
