// Backward pass of the sLSTM cell: two kernels.  Included by slstm_hip.hip only.
//
// What they replace in the reference: SLSTMPointwiseBackward (xlstm/blocks/slstm/src/cuda/slstm_pointwise.cu:118-196) and
// the per-timestep launches around it (slstm_backward.cu:291-319: one pointwise launch and one strided-batched GEMM with
// R transposed per step), plus the state history [4,T+1,B,H] and the gate cache [T,B,4H] that the reference's forward
// writes for them (slstm.cc:79-108).  The rule is the native kernel's: the stabiliser m is a constant of the
// differentiation (its gradient is written as zero, slstm_pointwise.cu:187-190).
//
//   slstm_bwd_prepare_kernel   one thread per (batch row, hidden unit) walks FORWARD through time over
//                              raw = W.x + R.h_{t-1} + bias (R.h_{t-1} from the stored outputs, by MFMA waves of the same
//                              workgroup a block of steps ahead) and leaves, per step and element, the nine
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
//                              layout of the pointwise part).  R transposed is read from the L2 every step: a step is
//                              bound by one compute unit's path to the L2 (4 dh x dh operands per step).  Head dims 64,
//                              128, 256; used for launches that the split kernel cannot hold.
//   slstm_bwd_split_kernel     the same pass with a head spread over dh / 64 compute units that exchange their gate
//                              deltas every step (head dims 64 - one unit, the same step - 128, 256, 512 in bf16); described in front of it.
#pragma once

namespace {

struct BwdPrepParams {
  int B, T, NH, dh;
  const void *wx;            // [B,T,4,NH,dh], strides in elements
  long long wx_sb, wx_st;
  const void *r;             // [NH, 4 dh, dh] in the type of the operands: R as the forward takes it (K contiguous)
  const void *h_out;         // [T,B,H] in the type of the operands: the forward's outputs
  const float *bias;         // [NH,4,dh]
  const float *s0;           // [4,B,H] or null
  const uint8_t *reset;      // [B,T] or null
  long long reset_sb;
  float *coef;               // [T,B,9,H], or with tiled = R (16 or 4) [T][ceil(B/R)][NH][dh/64][R rows][9][64 units]: what a
                             // workgroup of the split kernels reads per step is one piece of 36 (9) KiB (planes 4 KiB apart,
                             // as in the plain layout, all fall on the same memory channel)
  int tiled;
};

// 16 bytes (or one byte) per lane from a buffer straight into LDS, lane i's bytes at lds_addr + 16 i (+ 4 i).  The wait
// states in front: the descriptor may sit in scalar registers that a vector instruction has just written, and the
// compiler does not look for that hazard inside a statement like this.
__device__ __forceinline__ void bwd_fetch_to_lds_b128(u32x4_t rsrc, uint32_t lds_addr, uint32_t voffset) {
  asm volatile("s_nop 4\n\ts_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :: "s"(lds_addr), "v"(voffset), "s"(rsrc) : "memory", "m0");
}
__device__ __forceinline__ void bwd_fetch_to_lds_u8(u32x4_t rsrc, uint32_t lds_addr, uint32_t voffset) {
  asm volatile("s_nop 4\n\ts_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_ubyte %1, %2, 0 offen lds"
               :: "s"(lds_addr), "v"(voffset), "s"(rsrc) : "memory", "m0");
}

// One workgroup per (batch row, 64 hidden units), twelve waves:
//   wave 0        walks through time: lane = unit, the forward's own update with the gate values kept, nine
//                 coefficients per step into LDS.
//   wave 1        brings the steps' inputs to an LDS ring - W.x of the slice, the row's output of the step before (the
//                 operand of R), the reset flag: three loads a step - in blocks of kPrepBlock steps, up to three blocks
//                 ahead, with loads that write LDS directly and waits written by hand.  (With the inputs fetched by the
//                 walking wave itself, into registers six steps ahead, the kernel took 0.95 ms at config 2 and 0.36 ms
//                 without its loads: a wave has at most 63 memory operations in flight, the nine stores of a step among
//                 them, against a way to HBM and back of several microseconds.)
//   waves 2, 3    store what the walking wave leaves in LDS (five and four coefficients each), a block behind it: with
//                 its own nine stores a step in its 63 operations in flight, the acknowledgements of those stores set
//                 the walking wave's pace.
//   waves 4 - 11  R.y_{t-1} of the slice's 64 units x 4 gates for the steps of the NEXT block: MFMAs over the outputs in
//                 the ring (rows that start a document zero; in front of step 0 the y of the initial state) against
//                 their 32 columns of R, which stay in registers for the whole call; results into the ring, where the
//                 walking wave finds them next to W.x.  The reference caches the gate values of the forward instead
//                 (slstm.cc:79-108); an earlier version of this kernel read R.h from a tensor that a library GEMM over
//                 all steps had written (1 KiB per step and workgroup more to fetch, 0.5 GB at config 2).
constexpr int kPrepBlock = 8;
constexpr int kPrepRing = 4;  // blocks in the ring
constexpr int kPrepThreads = 768;
constexpr int bwd_prepare_slot_bytes(bool bf16, int dh) { return 4 * 64 * (bf16 ? 2 : 4) + 64 * 16 + 16 + dh * (bf16 ? 2 : 4); }
constexpr int bwd_prepare_lds_bytes(bool bf16, int dh) {  // the ring of inputs and two blocks of results
  return kPrepRing * kPrepBlock * bwd_prepare_slot_bytes(bf16, dh) + 2 * kPrepBlock * 9 * 64 * 4;
}
template <bool BF16, int DH>
__global__ __launch_bounds__(kPrepThreads) void slstm_bwd_prepare_kernel(BwdPrepParams p) {
  constexpr int ESZ = BF16 ? 2 : 4;
  constexpr int EPC = 16 / ESZ;               // elements of a 16-byte chunk
  constexpr int WXB = 4 * 64 * ESZ;           // W.x of a step: [4 gates][64 units]
  constexpr int RYB = 64 * 16;                // R.y of a step: [64 units][4 gates] float32
  constexpr int HOFF = WXB + RYB + 16;        // ... the row's reset flag, then the operand row: y_{t-1} of the head, DH elements
  constexpr int SLOT = bwd_prepare_slot_bytes(BF16, DH);
  constexpr int NR = kPrepRing;
  constexpr int KSTEPS = DH / (4 * EPC);      // 16-byte chunks of an operand row per lane group
  extern __shared__ __attribute__((aligned(16))) char prep_lds[];
  char *const ring = prep_lds;                                                    // [NR][kPrepBlock] slots of inputs
  float *const outs = reinterpret_cast<float *>(prep_lds + NR * kPrepBlock * SLOT);  // [2][kPrepBlock][9][64]: results
  const int H = p.NH * DH;
  // The DH / 64 workgroups of a (batch row, head) read the same operand rows (the head's outputs): they take
  // consecutive slots of ONE XCD (workgroup i runs on XCD i % 8), so those rows come from HBM into one L2 once.
  // (Dealt out in launch order they sat on different XCDs and each fetched its own copy: 539 MB read at
  // B 16 x T 2048 x 4 heads of 256 for 340 of W.x, outputs and R.)
  constexpr int SPH = DH >> 6;                       // slices per head
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int pair = (slot / SPH) * 8 + xcd;           // (batch row, head) pair
  if (pair >= p.B * p.NH) return;
  const int b = pair / p.NH, head = pair - b * p.NH, a0 = (slot % SPH) << 6;
  const int col0 = head * DH + a0;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = (int)uniform((uint32_t)(tid >> 6));
  const int nblocks = (p.T + kPrepBlock - 1) / kPrepBlock;
  const uint32_t ring_lds = (uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)ring);
  const long long BH = (long long)p.B * H;
  // Barriers, the same for every wave: P (block 0's inputs have landed), then barrier k in front of the walking wave's
  // block k (the MFMA waves have left R.y of block k in the ring, the inputs of block k + 1 have landed), then one
  // behind the last block.
  if (wave >= 4) {
    // ---- an MFMA wave: columns 32 mw .. + 31 of the slice's 256, column c = 4 * unit + gate (the order the walking
    //      wave reads them in)
    const int mw = wave - 4, q = lane >> 4, r16 = lane & 15;
    uint4 rreg[KSTEPS][2];
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
      const int c = 32 * mw + 16 * cb + r16;
      const long long row = (long long)head * 4 * DH + (long long)(c & 3) * DH + a0 + (c >> 2);
      const char *src = reinterpret_cast<const char *>(p.r) + row * DH * ESZ;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) rreg[ks][cb] = *reinterpret_cast<const uint4 *>(src + (ks * 4 + q) * 16);
    }
    auto block_product = [&](int k) {  // R.y of the steps of block k: rows 0 .. 7 of the MFMA tile, the rest is padding
      const int t = k * kPrepBlock + (r16 & 7);
      const char *slot = ring + ((k % NR) * kPrepBlock + (r16 & 7)) * SLOT;
      bool zero = r16 >= kPrepBlock || t >= p.T;
      if (p.reset && !zero) zero = (*reinterpret_cast<const uint32_t *>(slot + WXB + RYB) & 0xFFu) != 0u;
      f32x4 acc[2] = {f32x4{0.0f, 0.0f, 0.0f, 0.0f}, f32x4{0.0f, 0.0f, 0.0f, 0.0f}};
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        uint4 av = *reinterpret_cast<const uint4 *>(slot + HOFF + (ks * 4 + q) * 16);
        if (t == 0) {  // in front of the first step: the y of the initial state, rounded as the forward rounds it
          av = uint4{0u, 0u, 0u, 0u};
          if (p.s0) {
            const float *src = p.s0 + (long long)b * H + (long long)head * DH + (ks * 4 + q) * EPC;
            const float4 lo = *reinterpret_cast<const float4 *>(src);
            if (BF16) {
              const float4 hi = *reinterpret_cast<const float4 *>(src + 4);
              av = uint4{pack_bf16x2(lo.x, lo.y), pack_bf16x2(lo.z, lo.w), pack_bf16x2(hi.x, hi.y), pack_bf16x2(hi.z, hi.w)};
            } else {
              av = __builtin_bit_cast(uint4, lo);
            }
          }
        }
        if (zero) av = uint4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) {
          if (BF16) {
            acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av), __builtin_bit_cast(bf16x8, rreg[ks][cb]), acc[cb], 0, 0, 0);
          } else {
            const uint32_t aw[4] = {av.x, av.y, av.z, av.w}, bw[4] = {rreg[ks][cb].x, rreg[ks][cb].y, rreg[ks][cb].z, rreg[ks][cb].w};
#pragma unroll
            for (int e = 0; e < 4; ++e)
              acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(aw[e]), __uint_as_float(bw[e]), acc[cb], 0, 0, 0);
          }
        }
      }
      if (q < 2) {  // lane (q, r16) holds steps 4 q .. 4 q + 3 of column r16 of each block of 16 columns
#pragma unroll
        for (int cb = 0; cb < 2; ++cb)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            *reinterpret_cast<float *>(ring + ((k % NR) * kPrepBlock + 4 * q + e) * SLOT + WXB + (32 * mw + 16 * cb + r16) * 4) = acc[cb][e];
      }
    };
    __syncthreads();  // P
    block_product(0);
    for (int k = 0; k < nblocks; ++k) {
      __syncthreads();  // barrier k
      if (k + 1 < nblocks) block_product(k + 1);
    }
    __syncthreads();    // (behind the last block)
    return;
  }
  if (wave >= 2) {
    // ---- a storer wave: five (wave 2) or four (wave 3) of the nine coefficients of every step, a block behind the
    //      walking wave
    const int col = col0 + lane, a = a0 + lane, j0 = wave == 2 ? 0 : 5, nj = wave == 2 ? 5 : 4;
    auto store_block = [&](int k) {
#pragma unroll
      for (int i = 0; i < kPrepBlock; ++i) {
        const int t = k * kPrepBlock + i;
        if (t >= p.T) break;
        float *dst = p.coef + ((long long)t * p.B + b) * 9 * H + col;
        long long js = H;
        if (p.tiled) {
          const int tr = p.tiled;
          const long long piece = (((long long)t * ((p.B + tr - 1) / tr) + b / tr) * p.NH + head) * (DH >> 6) + (a >> 6);
          dst = p.coef + (piece * tr + b % tr) * (9 * 64) + (a & 63);
          js = 64;
        }
        const float *src = outs + (((k & 1) * kPrepBlock + i) * 9 + j0) * 64 + lane;
#pragma unroll
        for (int j = 0; j < 5; ++j)
          if (j < nj) dst[(j0 + j) * js] = src[j * 64];
      }
    };
    __syncthreads();  // P
    for (int k = 0; k < nblocks; ++k) {
      __syncthreads();  // barrier k
      if (k > 0) store_block(k - 1);
    }
    __syncthreads();    // the last block's results are in LDS
    store_block(nblocks - 1);
    return;
  }
  if (wave == 1) {
    // ---- the loader wave.  Block k sits in ring part k % NR; it is asked for behind barrier k - NR + 1 (when the
    //      walking wave is through with block k - NR, which sat there) and has landed in front of barrier k - 1, when
    //      the MFMA waves take its operand rows.
    auto descriptor = [&](const void *base, uint32_t bytes) {
      const unsigned long long a = reinterpret_cast<unsigned long long>(base);
      return u32x4_t{uniform((uint32_t)a), uniform((uint32_t)(a >> 32) & 0xFFFFu), bytes, 0x00020000u};
    };
    constexpr int LPG = 64 * ESZ / 16;        // lanes that cover a gate's 64 units of W.x
    constexpr int HL = DH * ESZ / 16;         // lanes that cover an operand row (16 .. 64)
    auto request_block = [&](int k) {  // 3 x 8 loads, whatever T is (steps past the end ask for the last step again)
#pragma unroll
      for (int i = 0; i < kPrepBlock; ++i) {
        int t = k * kPrepBlock + i;
        t = t < p.T ? t : p.T - 1;
        const uint32_t slot = ring_lds + ((k % NR) * kPrepBlock + i) * SLOT;
        {  // W.x: a gate's 64 units are 128 bytes (bf16: 8 lanes) or 256 (float32: 16 lanes)
          const char *base = reinterpret_cast<const char *>(p.wx) + ((long long)b * p.wx_sb + (long long)t * p.wx_st + col0) * ESZ;
          const uint32_t voff = (uint32_t)(((long long)(lane / LPG) * H) * ESZ + (lane % LPG) * 16);
          const u32x4_t rs = descriptor(base, (uint32_t)((3ll * H + 64) * ESZ));
          const uint32_t dst = uniform(slot);
          if (lane < 4 * LPG) bwd_fetch_to_lds_b128(rs, dst, voff);  // (only these lanes write LDS)
        }
        {  // the operand row: the head's outputs of step t - 1 (step 0: any row, the MFMA waves take the initial state)
          const int tp = t > 0 ? t - 1 : 0;
          const char *base = reinterpret_cast<const char *>(p.h_out) + ((long long)tp * BH + (long long)b * H + (long long)head * DH) * ESZ;
          const u32x4_t rs = descriptor(base, (uint32_t)(DH * ESZ));
          const uint32_t dst = uniform(slot + HOFF);
          if (lane < HL) bwd_fetch_to_lds_b128(rs, dst, (uint32_t)lane * 16u);
        }
        {  // the row's reset flag (lane 0; without a mask: nothing is read, the word is not used)
          const unsigned char *base = p.reset ? p.reset + (long long)b * p.reset_sb + t : reinterpret_cast<const unsigned char *>(p.wx);
          const u32x4_t rs = descriptor(base, 1u);
          const uint32_t dst = uniform(slot + WXB + RYB);
          if (lane == 0) bwd_fetch_to_lds_u8(rs, dst, 0u);
        }
      }
    };
    // (blocks past the end are asked for like the others - their steps are the last step again, their ring part is
    // free - so that every wait below is for the same count)
    request_block(0);
    request_block(1);
    request_block(2);
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(3 * kPrepBlock * 2) : "memory");  // (block 0 has landed)
    __syncthreads();  // P
    for (int k = 0; k < nblocks; ++k) {
      asm volatile("s_waitcnt vmcnt(%0)" :: "n"(3 * kPrepBlock) : "memory");    // (block k + 1 has landed)
      __syncthreads();  // barrier k: the walking wave is through with block k - 1
      request_block(k + NR - 1);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();    // (behind the last block)
    return;
  }
  // ---- the walking wave: lane = unit of the slice
  const int a = a0 + lane;
  const long long idx = (long long)b * H + col0 + lane;
  float bias_g[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) bias_g[g] = p.bias[((long long)head * 4 + g) * DH + a];
  float c = 0.0f, n = 0.0f, m = 0.0f;
  if (p.s0) { c = p.s0[BH + idx]; n = p.s0[2 * BH + idx]; m = p.s0[3 * BH + idx]; }
  const bool has_mask = p.reset != nullptr;
  // (a block's inputs are read from LDS in one go, in front of its eight steps: read per step, each read would be
  // waited for with nothing else to do, and the compiler does not move them up past the writes of the results)
  struct StepInputs { f32x4 ry; typename std::conditional<BF16, uint16_t, float>::type wx[4]; uint32_t flag; };
  auto read_inputs = [&](const char *slot, StepInputs &in) {
    in.ry = *reinterpret_cast<const f32x4 *>(slot + WXB + lane * 16);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if constexpr (BF16) in.wx[g] = *reinterpret_cast<const uint16_t *>(slot + (g * 64 + lane) * 2);
      else in.wx[g] = *reinterpret_cast<const float *>(slot + (g * 64 + lane) * 4);
    }
    in.flag = has_mask ? *reinterpret_cast<const uint32_t *>(slot + WXB + RYB) : 0u;
  };
  auto one_step = [&](const StepInputs &in, float *out) {
    float raw[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float w;
      if constexpr (BF16) w = bf16_bits_to_float(in.wx[g]);
      else w = in.wx[g];
      raw[g] = (w + in.ry[g]) + bias_g[g];
    }
    const bool restart = (in.flag & 0xFFu) != 0u;
    if (restart) { c = 0.0f; n = 0.0f; m = 0.0f; }
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
    out[0 * 64] = og * rn;
    out[1 * 64] = ynew * rn;
    out[2 * 64] = ig * tz;
    out[3 * 64] = ig;
    out[4 * 64] = fg * one_minus_fsig * c;
    out[5 * 64] = fg * one_minus_fsig * n;
    out[6 * 64] = ig * (1.0f - tz * tz);
    out[7 * 64] = (1.0f - og) * ynew;
    out[8 * 64] = fg;
    c = cnew; n = nnew; m = mnew;
  };
  __syncthreads();  // P
  for (int k = 0; k < nblocks; ++k) {
    __syncthreads();  // barrier k
    StepInputs in[kPrepBlock];
#pragma unroll
    for (int i = 0; i < kPrepBlock; ++i) read_inputs(ring + ((k % NR) * kPrepBlock + i) * SLOT, in[i]);
#pragma unroll
    for (int i = 0; i < kPrepBlock; ++i) {
      const int t = k * kPrepBlock + i;
      if (t < p.T) one_step(in[i], outs + ((k & 1) * kPrepBlock + i) * 9 * 64 + lane);
    }
  }
  __syncthreads();  // (behind the last block)
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
  float *d_wx;               // [B,T,4,NH,dh] float32 (bf16 with d_wx_bf16), strides in elements
  long long d_wx_sb, d_wx_st;
  int d_wx_bf16;
  float *d_s0;               // [4,B,H]
  int cut;                   // no gradient from a step to the y it started from (slstm_backward_cut.cu:265-312)
  float clip;                // > 0: that gradient is clipped to +-clip before d_h is added (slstm_pointwise.cu:136-143); 0: not
};

// The gradient that reached y_t through the recurrence, as the step's gradient takes it in: clipped when the call asks
// for it, except at the last step, where it is the y part of d_s_final and comes from outside.
__device__ __forceinline__ float bwd_recurrent_dy(float dy, float clip, bool last_step) {
  return (clip > 0.0f && !last_step) ? __builtin_amdgcn_fmed3f(dy, -clip, clip) : dy;
}

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
            const float dyt = dh_in[ii][nb] + bwd_recurrent_dy(dy[nb][i], p.clip, t == p.T - 1);
            const float dct = dc[nb][i] + dyt * cf[ii][nb][0];
            const float dnt = dn[nb][i] - dyt * cf[ii][nb][1];
            delta[0] = cf[ii][nb][2] * dct + cf[ii][nb][3] * dnt;
            delta[1] = cf[ii][nb][4] * dct + cf[ii][nb][5] * dnt;
            delta[2] = cf[ii][nb][6] * dct;
            delta[3] = cf[ii][nb][7] * dyt;
            // (a row that starts a document at t took nothing from the step before)
            dc[nb][i] = restart[ii] ? 0.0f : cf[ii][nb][8] * dct;
            dn[nb][i] = restart[ii] ? 0.0f : cf[ii][nb][8] * dnt;
            const long long wo = (long long)row * p.d_wx_sb + (long long)t * p.d_wx_st + head * dh + unit;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              if (p.d_wx_bf16) reinterpret_cast<uint16_t *>(p.d_wx)[wo + (long long)g * H] = (uint16_t)(pack_bf16x2(delta[g], 0.0f) & 0xFFFFu);
              else p.d_wx[wo + (long long)g * H] = delta[g];
            }
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
    //      (nothing when the call cuts that path)
    f32x4 acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    if (!p.cut) {
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
// The reverse pass with a head SPREAD OVER S = dh / 64 workgroups (compute units), built like the forward's sequence
// kernel: workgroup s of a (head, 16-row tile) group owns 64 hidden units.  It computes the step's gate deltas of its
// own 16 x 64 elements, publishes them to its peers, and computes what reaches ITS 64 units of y_{t-1}:
// delta [16 x 4 dh] . R^T [4 dh x 64].  That slice of R transposed (128 KiB in bf16 at head dim 256) stays in the
// registers of the eight waves for the whole call, each wave holding one eighth of K for all 64 columns; the eight
// partial results are added up through LDS.  Per step a workgroup writes its 16 x 256 deltas (8 KiB in bf16) and reads
// the group's 16 x 4 dh, straight into MFMA operand registers; nothing else is read from memory per step but the
// coefficients and d_h of its own elements (by feeder waves, or two steps ahead: see FEED below).
//
// The exchange is a ring of kBwdRing slots per group, slot n % kBwdRing for the n-th step of the call, laid out as
// MFMA A operands: [K / KC][16 rows][4][16 bytes] with KC = 32 (bf16) or 16 (float32) and K index
// k = 256 s + 64 gate + unit % 64.  A word is data or the "not written yet" pattern (all ones, which no value takes:
// a NaN that would is changed into another NaN).  A reader polls its 16-byte chunks until none holds the pattern.  A workgroup that
// publishes step n also re-arms its words of step n - 2: it has read all deltas of step n - 1, which every peer
// computed from a complete set of step n - 2.  The re-arm is acknowledged before the workgroup's poll of step n
// returns (accesses of a wave complete in order), so before it publishes step n + 1; a peer that polls the slot again
// for step n - 2 + kBwdRing has seen that publication and finds the pattern or the new data, never the old.  The
// library fills the ring with the pattern in front of the kernel.
//
// All workgroups of a group run on one XCD (workgroup i is dispatched to XCD i % 8): plain stores reach the XCD's L2,
// and the polls read past the first-level cache.  All workgroups must be resident at once; the host launches at most
// as many as there are compute units.  Waits are bounded: when one runs out the call's abort word is set, every wave
// stops waiting, and the gradient of the initial state is overwritten with NaN.
constexpr int kBwdRing = 4;

struct BwdSplitParams {
  int B, T, NH, dh;
  const float *coef;         // [T][ceil(B/16)][NH][S][16 rows][9][64 units]
  const void *d_h;
  const float *d_s_final;
  const void *r_ts;          // R transposed per workgroup and wave, tiled as MFMA B operands:
                             // [NH][S][8 waves][KSTEPS][4 column blocks][64 lanes][16 bytes]
  const uint8_t *reset;
  long long reset_sb;
  float *d_wx;               // (bf16 in the DWX16 variants of the kernels)
  long long d_wx_sb, d_wx_st;
  float *d_s0;
  void *xch;                 // [kBwdRing][groups][K / KC][16][4][16 bytes], all ones at the start
  unsigned int *abort_word;  // zero at the start of a call
  unsigned int *progress;    // [groups]: the step of the call that the group has reached (for the prefetching workgroups)
  unsigned int *placement;   // [groups], zero at the start: the XCDs that the group's workgroups found themselves on, one bit each
  int main_locals;           // workgroups per XCD that compute; those behind them (one per XCD, if any) prefetch
  long long spin_limit;
  int cut;                   // as in BwdParams
  float clip;
};

// fills the exchange ring with the "not written yet" pattern and clears the abort word in front of the split kernel
// (a kernel, not a memset: a caller may capture the call in a graph)
__global__ __launch_bounds__(256) void slstm_bwd_arm_kernel(uint4 *xch, long long n16, unsigned int *words, int nwords) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
    xch[i] = uint4{0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu};
  if (blockIdx.x == 0)
    for (int i = threadIdx.x; i < nwords; i += blockDim.x) words[i] = 0u;
}

// Prefetching workgroups: they bring what an XCD's groups will read from memory - coefficients and d_h - into the XCD's
// L2, a few steps ahead of them.  A compute unit returns its loads in the order they were issued, whichever wave issued
// them: a miss that goes to HBM holds up every poll of the exchange ring behind it, and a step took 2.7 us at config 2
// with the inputs fetched by the workgroup itself (by its polling waves or by others, one step ahead or two) against
// 2.0 us with inputs that were already in the L2.  So other compute units take the misses.  Nothing depends on these
// workgroups: they follow the groups' progress words at a distance, and stop when those stop.
//
// `which` of the `of` prefetching workgroups of this XCD (a compute unit draws some 65 GB/s from memory: the host
// launches as many as the XCD's groups need); they share a step's lines by position.  The groups' progress words are
// read by the lanes of one wave side by side, the lines of a step - the coefficients and d_h of all groups of the XCD -
// are dealt out over the threads as one flat range, and a workgroup that has fallen behind what the feeder waves have
// already asked for skips ahead.  (An earlier version, one workgroup per XCD with a call per group and tensor and the
// progress words read one after the other, took longer than the compute units take for the step once an XCD held more
// than two or three groups; the feeder waves then missed to HBM, every poll of their compute unit came back behind those
// misses, and at the end the prefetch kept the kernel alive for as long again: 5 us per step at B 64 x 4 heads of 256
// instead of 2, 16 at B 192.)
constexpr int kBwdAhead = 12;  // steps the prefetch may run ahead at most (1.2 MiB of a 4 MiB L2 at config 2)
// ROWS: batch rows of a row tile; DEPTH: steps the feeder waves ask ahead
template <bool BF16, int S, int ROWS, int DEPTH>
__device__ __forceinline__ void bwd_tile_prefetch(const BwdSplitParams &p, int xcd, int which, int of) {
  constexpr int ESZ = BF16 ? 2 : 4;
  constexpr int dh = 64 * S;
  constexpr int PIECE = ROWS * 9 * 64 * 4;          // bytes of a workgroup's coefficients of one step
  constexpr int CL = S * PIECE / 128;               // lines of a group's coefficients of one step (its S workgroups' pieces lie in a row)
  constexpr int PER_ROW = dh * ESZ / 128;           // lines of a row of d_h
  constexpr int DL = ROWS * PER_ROW;
  const int H = p.NH * dh, ntiles = (p.B + ROWS - 1) / ROWS, ngroups = p.NH * ntiles;
  const int tid = threadIdx.x, nthreads = blockDim.x, lane = tid & 63;
  if (xcd >= ngroups || of < 1) return;
  const int G = (ngroups - xcd + 7) >> 3;           // groups of this XCD: xcd, xcd + 8, ...
  // steps the prefetch may run ahead of the groups' progress: about 2 MiB of the XCD's 4 MiB L2, and more than the
  // feeder waves run ahead
  int ahead = (2 << 20) / (G * (CL + DL) * 128);
  ahead = ahead > kBwdAhead ? kBwdAhead : (ahead < DEPTH + 2 ? DEPTH + 2 : ahead);
  // A touch is a load that writes LDS, not a register: nothing waits for these loads before the end, and a register
  // that a load in flight is going to write would be handed out again by the compiler in the meantime.  Every touch of
  // every wave lands in the same kilobyte, which nobody reads.
  __shared__ uint4 dump[64];
  const uint32_t dump_lds = (uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)dump);
  __shared__ int slowest;      // the least progress among the XCD's groups; -1: stop
  const long long coef_step = (long long)ngroups * S * PIECE;  // bytes of one step's coefficients, all groups
  const long long dh_step = (long long)p.B * H * ESZ;
  for (int m = 0; m < p.T; ++m) {
    if (m >= ahead && (m & 1) == 0) {  // (every other step: the groups' progress is read through the L2)
      if (tid == 0) slowest = 0x7FFFFFFF;
      __syncthreads();
      if (tid < 64) {
        int spins = 0;
        for (;;) {
          int least = 0x7FFFFFFF;
          for (int j = lane; j < G; j += 64) {
            const int at = (int)__hip_atomic_load(p.progress + xcd + 8 * j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            least = at < least ? at : least;
          }
          if (__builtin_amdgcn_ballot_w64(least < m - ahead) == 0ull) {  // (lanes without a group: the largest int)
            if (lane < G) atomicMin(&slowest, least);
            break;
          }
          if (++spins > (1 << 16) || __hip_atomic_load(p.abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
            if (lane == 0) slowest = -1;
            break;
          }
          __builtin_amdgcn_s_sleep(8);
        }
      }
      __syncthreads();
      const int at = slowest;
      if (at < 0) break;
      // (fallen behind what the feeder waves have already asked for: skip to where a touch can still come first)
      if (m < at + DEPTH + 1) m = (at + DEPTH + 1) & ~1;
      if (m >= p.T) break;
    }
    const int t = p.T - 1 - m;
    const unsigned long long cb = reinterpret_cast<unsigned long long>(p.coef) + (unsigned long long)(t * coef_step);
    const unsigned long long db = reinterpret_cast<unsigned long long>(p.d_h) + (unsigned long long)(t * dh_step);
    const u32x4_t crs = {uniform((uint32_t)cb), uniform((uint32_t)(cb >> 32) & 0xFFFFu), uniform((uint32_t)coef_step), 0x00020000u};
    const u32x4_t drs = {uniform((uint32_t)db), uniform((uint32_t)(db >> 32) & 0xFFFFu), uniform((uint32_t)dh_step), 0x00020000u};
    // (uniform trip counts: lanes past the end ask past the buffer's end)
    for (int i0 = which * nthreads; i0 < G * CL; i0 += of * nthreads) {
      const int i = i0 + tid;
      const int j = i / CL, l = i - j * CL;
      const int g = xcd + 8 * j, head = g % p.NH, tile = g / p.NH;
      const uint32_t coff = i < G * CL ? (uint32_t)(((tile * p.NH + head) * S) * PIECE + l * 128) : 0xFFFFFF00u;
      bwd_fetch_to_lds_b128(crs, uniform(dump_lds), coff);
    }
    for (int i0 = which * nthreads; i0 < G * DL; i0 += of * nthreads) {
      const int i = i0 + tid;
      const int j = i / DL, l = i - j * DL;
      const int g = xcd + 8 * j, head = g % p.NH, tile = g / p.NH;
      const int row = tile * ROWS + l / PER_ROW;
      const uint32_t doff = (i < G * DL && row < p.B) ? (uint32_t)(((long long)row * H + head * dh) * ESZ + (l % PER_ROW) * 128) : 0xFFFFFF00u;
      bwd_fetch_to_lds_b128(drs, uniform(dump_lds), doff);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// The workgroups of a group exchange their deltas with plain stores through the L2 of the XCD that they are launched
// on by position (workgroup i on XCD i mod 8).  Each leaves the XCD it really runs on in the group's placement word, and
// at the end of the call looks at what the others left: with more than one XCD among them the exchange may have read
// words that were never written back (or a slot's previous content), so the call is flagged like one whose waits ran out.
__device__ __forceinline__ void bwd_note_placement(const BwdSplitParams &p, int group) {
  if (threadIdx.x == 0) atomicOr(p.placement + group, 1u << (__builtin_amdgcn_s_getreg(20 | (3 << 11)) & 0xFu));  // XCC_ID, bits [3:0]
}
__device__ __forceinline__ bool bwd_placement_mixed(const BwdSplitParams &p, int group) {
  const unsigned int seen = __hip_atomic_load(p.placement + group, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const bool mixed = (seen & (seen - 1u)) != 0u;
  if (mixed && threadIdx.x == 0) __hip_atomic_store(p.abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return mixed;
}

constexpr int kBwdPartStride = 68;  // floats between the rows of a wave's partial tile in LDS (no bank conflicts)
constexpr int kBwdCoefBytes = 16 * 9 * 64 * 4;  // a step's coefficients of a workgroup: 16 rows, 9 of them, 64 units
constexpr int bwd_feed_slot_bytes(bool bf16) { return kBwdCoefBytes + 16 * 64 * (bf16 ? 2 : 4); }  // ... and its d_h
constexpr int bwd_split_lds_bytes(bool feed, bool bf16) {
  return feed ? 8 * 16 * kBwdPartStride * 4 + 2 * bwd_feed_slot_bytes(bf16) : 2 * 8 * 16 * kBwdPartStride * 4;
}

// FEED: four more waves that do nothing but bring the steps' inputs from memory to LDS, two steps ahead, with loads
// that write LDS directly (no registers, and every wait of these waves is written by hand: a wave's loads return in
// the order they were issued, and the compiler waits for all of them wherever it waits for one).  The same order is
// why the polling waves must not fetch the inputs themselves: a poll issued behind a step's 40 KiB of coefficients
// comes back no sooner than they do, from HBM, and the step took 2.9 us at config 2 that way instead of 1.5 us
// without the fetch.  Twelve waves leave 168 registers a lane, which the variants with 128 registers of R transposed
// (float32 at head dim 256, bf16 at 512) do not fit: they run without feeders.
//
// With feeders a step has two barriers: B', behind which the slot that the step's inputs were read from is free for
// the inputs of the step after the next, and A, in front of which the wave's partial tile is written and the next
// step's inputs have landed.  (Without: one barrier, two sets of partial tiles.)
// DWX16: d_wx takes the gate deltas rounded to bf16.  (A template flag, not a branch on a kernel argument: with the
// branch in the step the compiler kept the exchange ring's descriptor in vector registers and wrapped every poll in a
// loop over the lanes' values.)
template <bool BF16, int S, bool FEED, bool DWX16 = false>  // eight compute waves; S workgroups per group, dh = 64 S (S = 1: one workgroup
                                        // per head and row tile, the same step with nobody else to wait for)
__global__ __launch_bounds__(FEED ? 768 : 512) void slstm_bwd_split_kernel(BwdSplitParams p) {
  static_assert(!DWX16 || BF16, "gate deltas in bf16 go with bf16 operands");
  constexpr int ESZ = BF16 ? 2 : 4;
  constexpr int EPC = 16 / ESZ;               // elements of a 16-byte chunk
  constexpr int KC = 4 * EPC;                 // K of one chunk row: what one MFMA (bf16) or four (float32) take
  constexpr int UW = 64;                      // hidden units of a workgroup
  constexpr int dh = S * UW;
  constexpr int K = 4 * dh;
  constexpr int KSTEPS = K / 8 / KC;          // chunks of a wave: its eighth of K
  constexpr int SLOT = 16 * K * ESZ;          // bytes of a group's slot
  constexpr int PART = 16 * kBwdPartStride;   // floats of a wave's partial tile
  extern __shared__ __attribute__((aligned(16))) float part[];  // [2][8 waves][16 rows][kBwdPartStride]
  const int H = p.NH * dh;
  const long long BH = (long long)p.B * H;
  const int ngroups = p.NH * ((p.B + 15) / 16);
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  if (local >= p.main_locals) {
    bwd_tile_prefetch<BF16, S, 16, 2>(p, xcd, local - p.main_locals, (int)(gridDim.x >> 3) - p.main_locals);
    return;
  }
  const int group = (local / S) * 8 + xcd, s = local % S;
  if (group >= ngroups) return;
  const int head = group % p.NH;
  const int row0 = (group / p.NH) * 16;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, q = lane >> 4, r16 = lane & 15;
  bwd_note_placement(p, group);
  constexpr int FSLOT = bwd_feed_slot_bytes(BF16);
  char *const feed = reinterpret_cast<char *>(part + 8 * PART);  // [2 slots][16 rows][9][64 units] float32, then d_h [16][64]
  const long long coef_piece0 = ((((long long)(row0 >> 4)) * p.NH + head) * S + s) * kBwdCoefBytes;  // + t * coef_step
  const long long coef_step = (long long)((p.B + 15) >> 4) * p.NH * S * kBwdCoefBytes;
  if (FEED && wave >= 8) {
    const int f = (int)uniform((uint32_t)wave) - 8;
    const uint32_t feed_lds = (uint32_t)(unsigned long long)((__attribute__((address_space(3))) unsigned char *)feed);
    const int rows_there = p.B - row0 < 16 ? p.B - row0 : 16;
    const uint32_t dh_records = uniform((uint32_t)(((long long)(rows_there - 1) * H + 64) * ESZ));
    // d_h: a load covers 8 rows of 128 bytes (bf16; the waves' two halves twice over) or 4 rows of 256 bytes
    const int dh_part = BF16 ? (f & 1) : f;
    const int dh_voff = BF16 ? ((dh_part * 8 + (lane >> 3)) * H * 2 + (lane & 7) * 16) : ((dh_part * 4 + (lane >> 4)) * H * 4 + (lane & 15) * 16);
    auto request = [&](int n) {  // the inputs of step n of the call -> slot n % 2: ten loads a wave
      const int t = p.T - 1 - n;
      const unsigned long long cb = reinterpret_cast<unsigned long long>(p.coef) + (unsigned long long)(coef_piece0 + t * coef_step);
      const u32x4_t crs = {uniform((uint32_t)cb), uniform((uint32_t)(cb >> 32) & 0xFFFFu), (uint32_t)kBwdCoefBytes, 0x00020000u};
      const uint32_t slot = feed_lds + (n & 1) * FSLOT;
#pragma unroll
      for (int k = 0; k < 9; ++k) bwd_fetch_to_lds_b128(crs, uniform(slot + (f * 9 + k) * 1024), (uint32_t)((f * 9 + k) * 1024 + lane * 16));
      const unsigned long long db = reinterpret_cast<unsigned long long>(p.d_h) + (unsigned long long)((((long long)t * p.B + row0) * H + (long long)head * dh + s * UW) * ESZ);
      const u32x4_t drs = {uniform((uint32_t)db), uniform((uint32_t)(db >> 32) & 0xFFFFu), dh_records, 0x00020000u};
      bwd_fetch_to_lds_b128(drs, uniform(slot + kBwdCoefBytes + dh_part * 1024), (uint32_t)dh_voff);  // (with the wait states behind the descriptor's scalar writes)
    };
    // Slot n % 2 is free behind barrier B'(n), but the inputs of step n + 2 are asked for only behind barrier A(n),
    // when the compute waves add up, read LDS and do arithmetic: right behind B' they publish and poll, and 38 KiB
    // of requests in front of those in the compute unit's queue cost the group a poll round (4.6 -> 4.2 ms at
    // config 2).
    request(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (p.T > 1) request(1);
    __syncthreads();  // (slot 0 is in place)
    for (int n = 0; n < p.T; ++n) {
      __syncthreads();  // B'(n): slot n % 2 has been read
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (the inputs of step n + 1, requested a step ago, have landed)
      __syncthreads();  // A(n)
      if (n + 2 < p.T) request(n + 2);
    }
    return;
  }
  // ---- this wave's share of the workgroup's slice of R transposed -> registers, once
  uint4 bq[KSTEPS][4];
  {
    const char *base = reinterpret_cast<const char *>(p.r_ts) + ((((long long)(head * S + s) * 8 + wave) * KSTEPS * 4 * 64) << 4);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) bq[ks][cb] = *reinterpret_cast<const uint4 *>(base + (((ks * 4 + cb) * 64 + lane) << 4));
  }
  // ---- the thread's two elements: row prow, units s 64 + pu, + 1 of the head
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
  // where the thread's deltas of gate g go in a slot, and where the wave's chunks come from
  int pub_off[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int k = s * 4 * UW + g * UW + pu;
    pub_off[g] = (((k / KC) * 16 + prow) * 4 + (k % KC) / EPC) * 16 + (k % EPC) * ESZ;
  }
  const int poll_off = (r16 * 4 + q) * 16;
  const int wave_u = (int)uniform((uint32_t)wave);  // (on the scalar unit: the polls' slot offsets are scalar operands)
  char *const ring = reinterpret_cast<char *>(p.xch) + (long long)group * SLOT;
  const long long ring_stride = (long long)ngroups * SLOT;
  // the step's inputs of the thread's elements, two sets used in turn: each is requested two steps ahead, right after
  // a poll has come back, so that the next poll (loads return in order) does not queue up behind it
  struct StepIn { f32x2 c9[9], dh2; bool restart; };
  StepIn in0, in1;
  auto fetch_step = [&](StepIn &in, int t) {
    in.restart = false;
    if (!there || t < 0) return;
    in.restart = p.reset && p.reset[(long long)row * p.reset_sb + t];
    const long long e = (long long)t * p.B + row;
    const float *cf = p.coef + ((((long long)t * ((p.B + 15) >> 4) + (row0 >> 4)) * p.NH + head) * S + s) * (16 * 9 * 64) + prow * (9 * 64) + pu;
#pragma unroll
    for (int j = 0; j < 9; ++j) in.c9[j] = *reinterpret_cast<const f32x2 *>(cf + j * 64);
    if (BF16) {
      const uint32_t w = *reinterpret_cast<const uint32_t *>(reinterpret_cast<const uint16_t *>(p.d_h) + e * H + ecol);
      in.dh2 = f32x2{__uint_as_float(w << 16), __uint_as_float(w & 0xFFFF0000u)};
    } else {
      in.dh2 = *reinterpret_cast<const f32x2 *>(reinterpret_cast<const float *>(p.d_h) + e * H + ecol);
    }
  };
  bool gave_up = false;
  uint32_t restart_raw = 0u;  // (FEED) the reset flag of the thread's row at the next step, as loaded
  auto step = [&](StepIn &in, int t) {
    const int n = p.T - 1 - t;
    if (FEED) {
      const char *slot = feed + (n & 1) * FSLOT;
      const float *src = reinterpret_cast<const float *>(slot) + prow * (9 * 64) + pu;
#pragma unroll
      for (int j = 0; j < 9; ++j) in.c9[j] = *reinterpret_cast<const f32x2 *>(src + j * 64);
      if (BF16) {
        const uint32_t w = *reinterpret_cast<const uint32_t *>(slot + kBwdCoefBytes + prow * 128 + pu * 2);
        in.dh2 = f32x2{__uint_as_float(w << 16), __uint_as_float(w & 0xFFFF0000u)};
      } else {
        in.dh2 = *reinterpret_cast<const f32x2 *>(slot + kBwdCoefBytes + prow * 256 + pu * 4);
      }
      in.restart = restart_raw != 0u;
      __syncthreads();  // B'(n)
    }
    // ---- the gradient of the step for the thread's elements
    float delta[4][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}, {0.0f, 0.0f}, {0.0f, 0.0f}};
    const bool restart_now = in.restart;
    if (there) {
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const float dyt = in.dh2[k] + bwd_recurrent_dy(dy[k], p.clip, n == 0);
        const float dct = dc[k] + dyt * in.c9[0][k];
        const float dnt = dn[k] - dyt * in.c9[1][k];
        delta[0][k] = in.c9[2][k] * dct + in.c9[3][k] * dnt;
        delta[1][k] = in.c9[4][k] * dct + in.c9[5][k] * dnt;
        delta[2][k] = in.c9[6][k] * dct;
        delta[3][k] = in.c9[7][k] * dyt;
        dc[k] = restart_now ? 0.0f : in.c9[8][k] * dct;  // (a row that starts a document at t took nothing from the step before)
        dn[k] = restart_now ? 0.0f : in.c9[8][k] * dnt;
      }
    }
    // ---- publish the deltas (rows outside the batch: zeros), re-arm the words of two steps ago.  A call that cuts
    //      the gradient through y needs none of the exchange: every workgroup is on its own.
    const bool cut = p.cut != 0;
    if (!cut) {
      char *const cur = ring + (n % kBwdRing) * ring_stride;
      char *const old = ring + ((n + kBwdRing - 2) % kBwdRing) * ring_stride;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        if (BF16) {
          // (the pattern stays unique: a half of all ones, which only a NaN can give, becomes 0xFFFE, a NaN as well)
          const u16x2_t w = __builtin_elementwise_min(__builtin_bit_cast(u16x2_t, pack_bf16x2(delta[g][0], delta[g][1])), u16x2_t{0xFFFE, 0xFFFE});
          *reinterpret_cast<uint32_t *>(cur + pub_off[g]) = __builtin_bit_cast(uint32_t, w);
        } else {
          float d0 = delta[g][0], d1 = delta[g][1];
          if (d0 != d0) d0 = kPoison;
          if (d1 != d1) d1 = kPoison;
          *reinterpret_cast<f32x2 *>(cur + pub_off[g]) = f32x2{d0, d1};
        }
      }
#pragma unroll
      for (int g = 0; g < 4; ++g) {  // (behind all of the step's deltas: those are waited for)
        if (BF16) *reinterpret_cast<uint32_t *>(old + pub_off[g]) = 0xFFFFFFFFu;
        else *reinterpret_cast<f32x2 *>(old + pub_off[g]) = f32x2{__uint_as_float(kSentinel32), __uint_as_float(kSentinel32)};
      }
    }
    // ---- between the publication and the first look at the peers' deltas, which need a while to land: the step's
    //      gate deltas to d_wx and a short sleep (reverse kernel at config 2: 4.25 ms with these stores behind the poll,
    //      4.14 with them here, 4.11 / 4.06 with 256 / 512 cycles of sleep on top, 4.16 / 4.50 with 1024 / 1536)
    //      (other shapes, us per step without / with the 512 cycles: bf16 at head dim 128 1.32 / 1.37, at 512 3.07 / 3.17,
    //      float32 at 128 3.99 / 3.36)
    if (s == 0 && tid == 0) p.progress[group] = (unsigned int)n;
    if (FEED && there && p.reset && t > 0) restart_raw = p.reset[(long long)row * p.reset_sb + t - 1];  // (used by the next step)
    if (there) {
      const long long wo = (long long)row * p.d_wx_sb + (long long)t * p.d_wx_st + ecol;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        if constexpr (DWX16) *reinterpret_cast<uint32_t *>(reinterpret_cast<uint16_t *>(p.d_wx) + wo + (long long)g * H) = pack_bf16x2(delta[g][0], delta[g][1]);
        else *reinterpret_cast<f32x2 *>(p.d_wx + wo + (long long)g * H) = f32x2{delta[g][0], delta[g][1]};
      }
    }
    if (cut) {
      if (!FEED) fetch_step(in, t - 2);
      __syncthreads();  // (the step's one barrier behind the publication: the feeders count on it)
      dy[0] = 0.0f;
      dy[1] = 0.0f;
      return;
    }
    if (S > 1) __builtin_amdgcn_s_sleep(8);  // (a workgroup that is its own group has its deltas in the L2 by the time it asks)
    // ---- the group's deltas of the wave's eighth of K: polled straight into the A operand registers
    uint4 areg[KSTEPS];
    {
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(ring + (n % kBwdRing) * ring_stride, 0, SLOT, 0x00020000);
      constexpr int kPastL1 = 16;  // (the load's scope bits: served by the L2)
      long long spins = 0;
      for (;;) {
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks)
          areg[ks] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rs, poll_off, (wave_u * KSTEPS + ks) * 1024, kPastL1));
        uint32_t mark = 0u;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) mark = mark_join<BF16>(mark, chunk_mark<BF16>(areg[ks]));
        // (a negative spin limit is the host's way to make every wait run out at its first look: the error path, forced)
        if ((__builtin_amdgcn_ballot_w64(mark_has_sentinel<BF16>(mark)) == 0ull && p.spin_limit >= 0) || gave_up) break;
        if (++spins > p.spin_limit || ((spins & 255) == 0 && __hip_atomic_load(p.abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
          __hip_atomic_store(p.abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          gave_up = true;
          break;
        }
      }
    }
    // ---- behind the poll: the inputs of the step after the next
    if (!FEED) fetch_step(in, t - 2);
    // ---- delta [16 x K/8] . R^T [K/8 x 64]: the wave's partial result, to LDS
    f32x4 acc[4];
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) acc[cb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const uint4 av = areg[ks];
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) {
        const uint4 bv = bq[ks][cb];
        if (BF16) {
          acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av), __builtin_bit_cast(bf16x8, bv), acc[cb], 0, 0, 0);
        } else {
          const uint32_t aw[4] = {av.x, av.y, av.z, av.w}, bw[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
          for (int e = 0; e < 4; ++e)
            acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(aw[e]), __uint_as_float(bw[e]), acc[cb], 0, 0, 0);
        }
      }
    }
    // (two sets of tiles, used in turn: a wave writes the tiles of step n + 2 only after every peer has published
    // step n + 2, for which it needed all of this workgroup's deltas of step n + 1, computed from the sums below)
    float *const tiles = part + (FEED ? 0 : (n & 1) * 8 * PART);
#pragma unroll
    for (int cb = 0; cb < 4; ++cb)
#pragma unroll
      for (int i = 0; i < 4; ++i) tiles[wave * PART + (4 * q + i) * kBwdPartStride + cb * 16 + r16] = acc[cb][i];
    __syncthreads();
    // ---- the eight partial results of the thread's two columns, in the order of the waves
    float sum0 = 0.0f, sum1 = 0.0f;
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      const f32x2 v = *reinterpret_cast<const f32x2 *>(tiles + w * PART + prow * kBwdPartStride + pu);
      sum0 += v[0];
      sum1 += v[1];
    }
    dy[0] = restart_now ? 0.0f : sum0;
    dy[1] = restart_now ? 0.0f : sum1;
  };
  if (!FEED) {
    fetch_step(in0, p.T - 1);
    fetch_step(in1, p.T - 2);
  } else {
    if (there && p.reset) restart_raw = p.reset[(long long)row * p.reset_sb + p.T - 1];
    __syncthreads();  // (the feeders' first slot is in place)
  }
  // (where this loop starts relative to a 32-byte boundary of the code, which moves the forward's sequence kernel by
  // 3 %, makes no difference here: all eight phases within 0.5 %)
  for (int t = p.T - 1; t >= 0; t -= 2) {
    step(in0, t);
    if (t > 0) step(in1, t - 1);
  }
  // ---- gradient w.r.t. the initial state (the stabiliser's part is zero by the rule; NaN all over when a wait ran out)
  const bool mixed = S > 1 && p.cut == 0 && bwd_placement_mixed(p, group);
  if (there) {
    const bool poisoned = gave_up || mixed || __hip_atomic_load(p.abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
