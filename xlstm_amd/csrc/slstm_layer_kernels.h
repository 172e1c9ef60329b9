// The kernels around the cell inside an sLSTM layer: causal depthwise convolution + SiLU, the four
// block-diagonal gate projections that produce the cell's input W.x, and the per-head group norm behind it.  bf16 operands,
// float32 arithmetic.  Included by slstm_hip.hip only (one translation unit), after
// slstm_device_common.h.
#pragma once

#include <type_traits>

namespace {

// ---------------------------------------------------------------------------
// causal depthwise convolution over time + SiLU (xlstm/components/conv.py:113-127 followed by
// the activation of xlstm/blocks/slstm/layer.py:136-137).  One thread: 8 channels of one token.
// Tap j of a kernel of KS taps multiplies the input KS-1-j tokens back; inputs before t = 0 come
// from `state` (the KS-1 tokens before this call) or are zero; with a reset mask a tap that
// would reach before the start of the token's document reads zero.  A decode step (T = 1) can also
// write the ring of the next step: the inputs of its taps, oldest first.
// ---------------------------------------------------------------------------
struct ConvParams {
  const uint16_t *x;
  long long x_sb, x_st;
  const uint16_t *state;  // [B, KS-1, D] or null; rows state_sb elements apart
  long long state_sb;
  const uint16_t *w;      // [D, KS]
  const uint16_t *bias;   // [D] or null
  const unsigned char *reset;
  long long reset_sb;
  uint16_t *out;          // [B, T, D]
  uint16_t *ring_out;     // [B, KS, D] or null (T == 1): the inputs of the taps, oldest first
  int B, T, D;
};

template <int KS>
__global__ __launch_bounds__(256) void causal_conv_silu_kernel(ConvParams p) {
  const int pieces = p.D >> 3;
  // workgroup i runs on XCD i % 8: give every XCD one contiguous range of tokens (the grid is a multiple of 8),
  // so that neighbouring tokens, which share all but one of their taps, find them in the same L2
  const long long wg = (long long)(blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const long long idx = wg * 256 + threadIdx.x;
  if (idx >= (long long)p.B * p.T * pieces) return;
  const int piece = (int)(idx % pieces);
  const long long bt = idx / pieces;
  const int t = (int)(bt % p.T);
  const int b = (int)(bt / p.T);
  const int c0 = piece * 8;

  // weights of the 8 channels: 8 * KS consecutive bf16
  uint16_t wv[8 * KS];
  {
    const uint4 *wp = reinterpret_cast<const uint4 *>(p.w + (long long)c0 * KS);
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      const uint4 v = wp[j];
      const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        wv[8 * j + 2 * e] = (uint16_t)(d[e] & 0xFFFFu);
        wv[8 * j + 2 * e + 1] = (uint16_t)(d[e] >> 16);
      }
    }
  }
  float acc[8];
  if (p.bias) {
    const uint4 v = *reinterpret_cast<const uint4 *>(p.bias + c0);
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc[2 * e] = bf16_bits_to_float(d[e] & 0xFFFFu);
      acc[2 * e + 1] = bf16_bits_to_float(d[e] >> 16);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
  }
  bool alive = true;  // no document start between the tap and the token so far
#pragma unroll
  for (int back = 0; back < KS; ++back) {
    const int j = KS - 1 - back;
    const int ts = t - back;
    if (back > 0 && p.reset) {  // the tap at `back` is dropped if a document starts in (t - back, t]
      const int tm = t - back + 1;
      if (tm >= 0 && p.reset[(long long)b * p.reset_sb + tm] != 0) alive = false;
    }
    const uint16_t *src = nullptr;
    if (alive) {
      if (ts >= 0) src = p.x + (long long)b * p.x_sb + (long long)ts * p.x_st + c0;
      else if (p.state) src = p.state + (long long)b * p.state_sb + (long long)(KS - 1 + ts) * p.D + c0;
    }
    if (p.ring_out) {  // (T == 1, no mask: `alive` holds; a missing state reads as zeros)
      const uint4 v = src ? *reinterpret_cast<const uint4 *>(src) : make_uint4(0, 0, 0, 0);
      *reinterpret_cast<uint4 *>(p.ring_out + ((long long)b * KS + j) * p.D + c0) = v;
    }
    if (src) {
      const uint4 v = *reinterpret_cast<const uint4 *>(src);
      const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[2 * e] += bf16_bits_to_float(wv[(2 * e) * KS + j]) * bf16_bits_to_float(d[e] & 0xFFFFu);
        acc[2 * e + 1] += bf16_bits_to_float(wv[(2 * e + 1) * KS + j]) * bf16_bits_to_float(d[e] >> 16);
      }
    }
  }
  uint32_t o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float a = acc[2 * e], c = acc[2 * e + 1];
    o[e] = pack_bf16x2(a * __builtin_amdgcn_rcpf(1.0f + __expf(-a)), c * __builtin_amdgcn_rcpf(1.0f + __expf(-c)));
  }
  *reinterpret_cast<uint4 *>(p.out + ((long long)b * p.T + t) * p.D + c0) = make_uint4(o[0], o[1], o[2], o[3]);
}

// ---------------------------------------------------------------------------
// the four headwise gate projections and their concatenation
// (xlstm/blocks/slstm/layer.py:144-153, xlstm/components/linear_headwise.py:75-82):
//   out[m, g*H + h*dh + o] = sum_d A_g[m, h*dh + d] * W_g[h, o, d]
// with A_g = x_conv for the slots i and f, x for z and o.  A workgroup computes BM tokens x BN output
// units of one (slot, head); K = dh is walked in stages of 64 inputs (128-byte rows), each staged
// through LDS once; the loads of the next stage are in flight during the MFMAs of the current one.
// Four waves as 2 x 2.  The product is formed transposed (units on the MFMA M axis), so a lane ends
// with 4 consecutive units of one token.  Workgroup i runs on XCD i % 8: the tiles of one block of
// tokens are given to ONE XCD, so that x and x_conv are fetched from HBM once.
// ---------------------------------------------------------------------------
struct GatesParams {
  const uint16_t *x, *xc;
  long long x_sr, xc_sr;
  const uint16_t *w[4];
  uint16_t *out;
  long long out_sr;
  int M, NH, dh;
  int m_tiles, n_tiles;
};

constexpr int kGateRowBytes = 144;  // 128 bytes of data + 16 of padding: conflict-free 16-byte reads

template <int BM, int BN>
__global__ __launch_bounds__(256) void headwise_gates_kernel(GatesParams p) {
  constexpr int AI = BM * 8 / 256;  // 16-byte pieces of the token tile a thread stages per K stage
  constexpr int WI = BN * 8 / 256;  // ... of the weight tile
  constexpr int TM = BM / 32, TN = BN / 32;  // MFMA tiles of a wave: TM token tiles x TN unit tiles
  __shared__ __attribute__((aligned(16))) unsigned char abuf[BM * kGateRowBytes];
  __shared__ __attribute__((aligned(16))) unsigned char wbuf[BN * kGateRowBytes];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int q = lane >> 4, r16 = lane & 15;
  const int wm = wave >> 1, wn = wave & 1;

  const int xcd = blockIdx.x & 7;
  const int jj = blockIdx.x >> 3;
  const int mtile = (jj / p.n_tiles) * 8 + xcd;
  if (mtile >= p.m_tiles) return;  // the whole workgroup leaves before any barrier
  int nt = jj % p.n_tiles;
  const int npu = p.dh / BN;  // unit tiles per (slot, head)
  const int ut = nt % npu; nt /= npu;
  const int slot_in_pair = nt & 1; nt >>= 1;
  const int pair = nt & 1;
  const int head = nt >> 1;
  const int slot = pair * 2 + slot_in_pair;
  const int m0 = mtile * BM;
  const int n0 = ut * BN;
  const int dh = p.dh;

  const uint16_t *abase = pair ? p.x : p.xc;
  const long long asr = pair ? p.x_sr : p.xc_sr;
  const uint16_t *wbase = p.w[slot] + ((long long)head * dh + n0) * dh;

  const uint16_t *asrc[AI];
  int adst[AI];
#pragma unroll
  for (int j = 0; j < AI; ++j) {
    const int e = tid + 256 * j;
    const int row = e >> 3, pc = e & 7;
    const int m = m0 + row < p.M ? m0 + row : p.M - 1;
    asrc[j] = abase + (long long)m * asr + (long long)head * dh + pc * 8;
    adst[j] = row * kGateRowBytes + pc * 16;
  }
  const uint16_t *wsrc[WI];
  int wdst[WI];
#pragma unroll
  for (int j = 0; j < WI; ++j) {
    const int e = tid + 256 * j;
    const int row = e >> 3, pc = e & 7;
    wsrc[j] = wbase + (long long)row * dh + pc * 8;
    wdst[j] = row * kGateRowBytes + pc * 16;
  }

  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  uint4 areg[AI], wreg[WI];
#pragma unroll
  for (int j = 0; j < AI; ++j) areg[j] = *reinterpret_cast<const uint4 *>(asrc[j]);
#pragma unroll
  for (int j = 0; j < WI; ++j) wreg[j] = *reinterpret_cast<const uint4 *>(wsrc[j]);

  const int nstage = dh >> 6;
  for (int s = 0; s < nstage; ++s) {
    if (s) __syncthreads();  // every wave is done reading the previous stage
#pragma unroll
    for (int j = 0; j < AI; ++j) *reinterpret_cast<uint4 *>(&abuf[adst[j]]) = areg[j];
#pragma unroll
    for (int j = 0; j < WI; ++j) *reinterpret_cast<uint4 *>(&wbuf[wdst[j]]) = wreg[j];
    __syncthreads();
    if (s + 1 < nstage) {
#pragma unroll
      for (int j = 0; j < AI; ++j) areg[j] = *reinterpret_cast<const uint4 *>(asrc[j] + (s + 1) * 64);
#pragma unroll
      for (int j = 0; j < WI; ++j) wreg[j] = *reinterpret_cast<const uint4 *>(wsrc[j] + (s + 1) * 64);
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      uint4 av[TM], wv[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        av[i] = *reinterpret_cast<const uint4 *>(&abuf[(wm * (BM / 2) + 16 * i + r16) * kGateRowBytes + ks * 64 + q * 16]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        wv[j] = *reinterpret_cast<const uint4 *>(&wbuf[(wn * (BN / 2) + 16 * j + r16) * kGateRowBytes + ks * 64 + q * 16]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wv[j]), __builtin_bit_cast(bf16x8, av[i]), acc[i][j], 0, 0, 0);
    }
  }

  // lane (r16, q) holds token m0 + wm*BM/2 + 16 i + r16, units n0 + wn*BN/2 + 16 j + 4 q .. +3
  const long long colbase = (long long)slot * p.NH * dh + (long long)head * dh + n0 + wn * (BN / 2) + 4 * q;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + wm * (BM / 2) + 16 * i + r16;
    if (m < p.M) {
      uint16_t *orow = p.out + (long long)m * p.out_sr + colbase;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        uint2 v;
        v.x = pack_bf16x2(acc[i][j][0], acc[i][j][1]);
        v.y = pack_bf16x2(acc[i][j][2], acc[i][j][3]);
        *reinterpret_cast<uint2 *>(orow + 16 * j) = v;
      }
    }
  }
}

// The same projections for head dims 128 and 256 with the weights RESIDENT in registers.  A workgroup
// owns one (head, operand) pair - all units of the slots i and f (operand x_conv) or z and o (operand x)
// of one head - and walks over tiles of 64 tokens (32 at dh = 128).  Each of its 2 * dh / 64 waves keeps the MFMA
// fragments of 64 units of one slot for the whole K range in VGPRs (128 at dh = 256), so the weights are
// read once per workgroup, every token tile is read from memory exactly once in the whole launch, and LDS
// carries the token fragments only: global -> registers -> LDS, two buffers, one barrier per K stage of
// 64 inputs, the loads of stage k + 2 issued before the MFMAs of stage k.  (The kernel above reads a
// token tile once per 128 output units - eight times at dh = 256 - and is bound by the fill rate of
// the L1, the workgroups that share a tile asking the same L2 channel at the same time.)
template <int I, typename T>
__device__ __forceinline__ T &pick_set(T &a, T &b) {
  if constexpr (I != 0) return b;
  else return a;
}

template <int NST>
__global__ __launch_bounds__(128 * NST) void headwise_gates_resident_kernel(GatesParams p, int combos, int parts) {
  constexpr int NW = 2 * NST;        // waves
  constexpr int NT = 64 * NW;        // threads
  constexpr int BM = NT / 8;         // tokens per tile: a thread stages ONE 16-byte piece per K stage
  constexpr int TM = BM / 16;
  constexpr int dh = NST * 64;
  __shared__ __attribute__((aligned(16))) unsigned char abuf[2][BM * kGateRowBytes];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int q = lane >> 4, r16 = lane & 15;
  const int combo = blockIdx.x % combos, part = blockIdx.x / combos;
  const int pair = combo & 1, head = combo >> 1;
  const int slot = pair * 2 + wave / NST;
  const int u0 = (wave % NST) * 64;  // this wave's units of the slot

  const int my_tiles = part < p.m_tiles ? (p.m_tiles - part + parts - 1) / parts : 0;
  if (my_tiles == 0) return;  // the whole workgroup leaves before any barrier

  // resident weight fragments: units u0 + 16 j + r16, inputs 64 s + 32 ks + 8 q .. +7
  uint4 wfrag[NST][2][4];
  {
    const uint16_t *wbase = p.w[slot] + ((long long)head * dh + u0 + r16) * dh + 8 * q;
#pragma unroll
    for (int s = 0; s < NST; ++s)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          wfrag[s][ks][j] = *reinterpret_cast<const uint4 *>(wbase + (long long)(16 * j) * dh + s * 64 + ks * 32);
  }

  const uint16_t *abase = (pair ? p.x : p.xc) + (long long)head * dh;
  const long long asr = pair ? p.x_sr : p.xc_sr;
  const int arow = tid >> 3;
  const int adst = arow * kGateRowBytes + (tid & 7) * 16;
  const int apc = (tid & 7) * 8;
  // stage k of this workgroup: token tile part + parts * (k / NST), inputs 64 * (k % NST) .. +63
  const int nstages = my_tiles * NST;
  // (no branches around the loads and LDS writes of the pipeline: past the last stage they repeat it, so the
  // compiler can count outstanding loads exactly instead of waiting for all of them at every join)
  auto load_stage = [&](int k) -> uint4 {
    k = k < nstages ? k : nstages - 1;
    const int m0 = (part + parts * (k / NST)) * BM;
    const int m = m0 + arow < p.M ? m0 + arow : p.M - 1;
    return *reinterpret_cast<const uint4 *>(abase + (long long)m * asr + (k % NST) * 64 + apc);
  };

  f32x4 acc[TM][4];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  uint4 areg0 = load_stage(0), areg1 = load_stage(1);  // two named registers, not an array (it would be placed in LDS)
  *reinterpret_cast<uint4 *>(&abuf[0][adst]) = areg0;
  __syncthreads();

  const long long colbase = (long long)slot * p.NH * dh + (long long)head * dh + u0 + 4 * q;
  // NST is even, so stage k lives in LDS buffer k & 1 = s & 1 and in register set k & 1 alike
  auto stage = [&](int k, auto sc) {
    constexpr int s = decltype(sc)::value;
    uint4 &mine = pick_set<s & 1>(areg0, areg1);         // held stage k, in LDS since the previous stage
    uint4 &other = pick_set<(s + 1) & 1>(areg0, areg1);  // holds stage k + 1, loaded one stage ago
    mine = load_stage(k + 2);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      uint4 av[TM];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        av[i] = *reinterpret_cast<const uint4 *>(&abuf[s & 1][(16 * i + r16) * kGateRowBytes + ks * 64 + q * 16]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wfrag[s][ks][j]), __builtin_bit_cast(bf16x8, av[i]), acc[i][j], 0, 0, 0);
    }
    *reinterpret_cast<uint4 *>(&abuf[(s + 1) & 1][adst]) = other;  // stage k + 1 goes to the other buffer, last read at stage k - 1
    __syncthreads();
  };
  for (int k0 = 0; k0 < nstages; k0 += NST) {
    stage(k0, std::integral_constant<int, 0>{});
    stage(k0 + 1, std::integral_constant<int, 1>{});
    if constexpr (NST > 2) {
      stage(k0 + 2, std::integral_constant<int, 2>{});
      stage(k0 + 3, std::integral_constant<int, 3>{});
    }
    // the token tile is complete: lane (r16, q) holds token m0 + 16 i + r16, units u0 + 16 j + 4 q .. +3
    const int m0 = (part + parts * (k0 / NST)) * BM;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = m0 + 16 * i + r16;
      if (m < p.M) {
        uint16_t *orow = p.out + (long long)m * p.out_sr + colbase;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint2 v;
          v.x = pack_bf16x2(acc[i][j][0], acc[i][j][1]);
          v.y = pack_bf16x2(acc[i][j][2], acc[i][j][3]);
          *reinterpret_cast<uint2 *>(orow + 16 * j) = v;
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
  }
}

// The same projections for FEW tokens (a decode step: M = batch size), head dims 128 and 256.  There the
// weights are the traffic (4 * H * dh elements against M * H of x) and every compute unit should fetch its
// share of them once: a workgroup computes 64 tokens x 64 units of one (slot, head) with the WHOLE K range
// staged through LDS in one go - all global loads of the two operand tiles are in flight together, one
// barrier, then 4 * NST MFMA k-steps per wave (four waves as 2 x 2, 32 x 32 outputs each).
template <int NST>
__global__ __launch_bounds__(256) void headwise_gates_slab_kernel(GatesParams p) {
  constexpr int dh = NST * 64;
  constexpr int RB = dh * 2 + 16;           // bytes per LDS row: data + pad (conflict-free 16-byte reads)
  constexpr int PPR = dh / 8;               // 16-byte pieces per row
  constexpr int ITEMS = 64 * PPR / 256;     // pieces of each operand tile a thread stages
  extern __shared__ __attribute__((aligned(16))) unsigned char slab_lds[];
  unsigned char *abuf = slab_lds, *wbuf = slab_lds + 64 * RB;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int q = lane >> 4, r16 = lane & 15;
  const int wm = wave >> 1, wn = wave & 1;
  // blockIdx -> (token tile, slot, head, unit tile); unit tiles fastest so that neighbours share x rows in one L2
  constexpr int npu = dh / 64;
  int nt = blockIdx.x % p.n_tiles;
  const int mtile = blockIdx.x / p.n_tiles;
  const int ut = nt % npu; nt /= npu;
  const int slot = nt & 3;
  const int head = nt >> 2;
  const int m0 = mtile * 64, n0 = ut * 64;

  const uint16_t *abase = (slot >= 2 ? p.x : p.xc) + (long long)head * dh;
  const long long asr = slot >= 2 ? p.x_sr : p.xc_sr;
  const uint16_t *wbase = p.w[slot] + ((long long)head * dh + n0) * dh;
  uint4 areg[ITEMS], wreg[ITEMS];
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const int e = tid + 256 * j;
    const int row = e / PPR, pc = e % PPR;
    const int m = m0 + row < p.M ? m0 + row : p.M - 1;
    areg[j] = *reinterpret_cast<const uint4 *>(abase + (long long)m * asr + pc * 8);
    wreg[j] = *reinterpret_cast<const uint4 *>(wbase + (long long)row * dh + pc * 8);
  }
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const int e = tid + 256 * j;
    const int row = e / PPR, pc = e % PPR;
    *reinterpret_cast<uint4 *>(&abuf[row * RB + pc * 16]) = areg[j];
    *reinterpret_cast<uint4 *>(&wbuf[row * RB + pc * 16]) = wreg[j];
  }
  __syncthreads();

  f32x4 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int ks = 0; ks < 2 * NST; ++ks) {
    uint4 av[2], wv[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) av[i] = *reinterpret_cast<const uint4 *>(&abuf[(wm * 32 + 16 * i + r16) * RB + ks * 64 + q * 16]);
#pragma unroll
    for (int j = 0; j < 2; ++j) wv[j] = *reinterpret_cast<const uint4 *>(&wbuf[(wn * 32 + 16 * j + r16) * RB + ks * 64 + q * 16]);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wv[j]), __builtin_bit_cast(bf16x8, av[i]), acc[i][j], 0, 0, 0);
  }
  // lane (r16, q) holds token m0 + 32 wm + 16 i + r16, units n0 + 32 wn + 16 j + 4 q .. +3
  const long long colbase = (long long)slot * p.NH * dh + (long long)head * dh + n0 + wn * 32 + 4 * q;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = m0 + wm * 32 + 16 * i + r16;
    if (m < p.M) {
      uint16_t *orow = p.out + (long long)m * p.out_sr + colbase;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        uint2 v;
        v.x = pack_bf16x2(acc[i][j][0], acc[i][j][1]);
        v.y = pack_bf16x2(acc[i][j][2], acc[i][j][3]);
        *reinterpret_cast<uint2 *>(orow + 16 * j) = v;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// per-head group norm behind the cell (xlstm/components/ln.py:51-68 as called by
// xlstm/blocks/slstm/layer.py:159): for every token and head, (x - mean) / sqrt(var + eps) * (1 + weight)
// over the dh units of the head, biased variance, float32 arithmetic.  One wave per (token, head); a lane
// holds 4 consecutive units per 256 units of head dim.  The input is addressed by strides, so the cell's
// [S,B,H] output is read as it lies in memory and the result is written token-major [B,S,H].
// ---------------------------------------------------------------------------
struct NormParams {
  const uint16_t *x;
  long long x_sb, x_st, x_sh;
  const uint16_t *weight;  // [NH*dh] or null
  uint16_t *out;           // [B, T, NH*dh]
  float eps;
  int B, T, NH, dh;
};

template <int PIECES>  // 8-byte pieces per lane: ceil(dh / 256)
__global__ __launch_bounds__(256) void headwise_group_norm_kernel(NormParams p) {
  const int lane = threadIdx.x & 63;
  const long long g = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);  // (b, t, head)
  if (g >= (long long)p.B * p.T * p.NH) return;
  const int head = (int)(g % p.NH);
  const long long bt = g / p.NH;
  const int t = (int)(bt % p.T);
  const int b = (int)(bt / p.T);
  const uint16_t *src = p.x + (long long)b * p.x_sb + (long long)t * p.x_st + (long long)head * p.x_sh;
  float v[PIECES][4];
  float sum = 0.0f;
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int u = (lane + 64 * j) * 4;
    if (u < p.dh) {
      const uint2 w = *reinterpret_cast<const uint2 *>(src + u);
      v[j][0] = bf16_bits_to_float(w.x & 0xFFFFu); v[j][1] = bf16_bits_to_float(w.x >> 16);
      v[j][2] = bf16_bits_to_float(w.y & 0xFFFFu); v[j][3] = bf16_bits_to_float(w.y >> 16);
    } else {
      v[j][0] = v[j][1] = v[j][2] = v[j][3] = 0.0f;
    }
    sum += (v[j][0] + v[j][1]) + (v[j][2] + v[j][3]);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
  const float mean = sum / (float)p.dh;
  float sq = 0.0f;
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int u = (lane + 64 * j) * 4;
    if (u < p.dh) {
#pragma unroll
      for (int e = 0; e < 4; ++e) { const float d = v[j][e] - mean; sq += d * d; }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o, 64);
  const float rstd = rsqrtf(sq / (float)p.dh + p.eps);
  uint16_t *dst = p.out + ((long long)b * p.T + t) * p.NH * p.dh + (long long)head * p.dh;
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int u = (lane + 64 * j) * 4;
    if (u < p.dh) {
      float sc[4] = {1.0f, 1.0f, 1.0f, 1.0f};
      if (p.weight) {
        const uint2 w = *reinterpret_cast<const uint2 *>(p.weight + (long long)head * p.dh + u);
        sc[0] += bf16_bits_to_float(w.x & 0xFFFFu); sc[1] += bf16_bits_to_float(w.x >> 16);
        sc[2] += bf16_bits_to_float(w.y & 0xFFFFu); sc[3] += bf16_bits_to_float(w.y >> 16);
      }
      uint2 o2;
      o2.x = pack_bf16x2((v[j][0] - mean) * rstd * sc[0], (v[j][1] - mean) * rstd * sc[1]);
      o2.y = pack_bf16x2((v[j][2] - mean) * rstd * sc[2], (v[j][3] - mean) * rstd * sc[3]);
      *reinterpret_cast<uint2 *>(dst + u) = o2;
    }
  }
}

}  // namespace
