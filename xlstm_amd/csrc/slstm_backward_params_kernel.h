// Gradients of the recurrent matrix and the bias: the third kernel of the backward pass.  Included by slstm_hip.hip only.
//
//   d R[h][g dh + a][d] = sum over rows b and steps t of  delta[b,t,g,h,a] * y_{t-1}[b,h,d]
//   d bias[h][g][a]     = sum over rows b and steps t of  delta[b,t,g,h,a]
//
// delta is what the reverse kernel left in d_wx, y_{t-1} the operand the forward step t multiplied by R: the output of
// step t - 1 (the y of the initial state in front of step 0), zero for a row that starts a document at t.  In the
// reference this is one strided-batched GEMM over the gate cache and the state history behind the time loop and a
// reduction kernel for the bias (xlstm/blocks/slstm/src/cuda/slstm_backward.cu:381-386, 52-108).
//
// Per head a product [4 dh x K] . [K x dh] with K = B T in the millions of flops per output element and both operands
// stored K-major: delta[k][m] and y[k][n] have their m, n contiguous in memory, the MFMA wants 8 consecutive k per
// lane.  A workgroup (eight waves) owns 128 rows m x NT columns n of one head's result for one slice of K.  It brings
// chunks of 32 k to LDS as they lie in memory (delta rounded to the operand type on the way, one barrier per chunk, the
// loads of the next two chunks in flight under the MFMAs) and every lane gathers its 8 k of an operand fragment with eight 16-bit
// LDS reads that fill the halves of four registers (rows of 132 / NT + 4 elements: the four lane groups of a read hit
// different banks).  float32 operands take the 16x16x4 MFMA, whose fragments are single values: no gathering.  The
// slices of K are added into d_r with float atomics (the entry point clears it first); the bias sums fall out of the
// delta values as they pass through the threads that stage them.
//
// Bound: delta is read once (16 bytes per step and element in float32: 537 MB at B 16 x T 2048 x D 1024), y_{t-1} once
// per 128 rows of the result from the L2; 68.7 GFLOP there, 27 us of bf16 MFMA.
#pragma once

namespace {

struct BwdParamParams {
  int B, T, NH, dh;
  const float *d_wx;         // [B,T,4,NH,dh] float32 (bf16 with d_wx_bf16), strides in elements: the gate deltas
  long long d_wx_sb, d_wx_st;
  int d_wx_bf16;
  const void *h_out;         // [T,B,H] in the operand type: the forward's outputs
  const float *s0;           // [4,B,H] or null
  const uint8_t *reset;      // [B,T] or null
  long long reset_sb;
  float *d_r;                // [NH, 4 dh, dh] float32, zero at the start
  float *d_bias;             // [NH, 4, dh] float32, zero at the start
  int ksplit;                // slices of K
  int tchunks;               // chunks of 32 steps per batch row: ceil(T / 32)
};

constexpr int kParamKC = 32;     // k per chunk
constexpr int kParamMT = 128;    // rows of the result per workgroup
constexpr int kParamPad = 4;     // elements of padding per LDS row
constexpr int bwd_param_lds_bytes(bool bf16, int nt) {
  return 2 * kParamKC * ((kParamMT + kParamPad) + (nt + kParamPad)) * (bf16 ? 2 : 4);
}

template <bool BF16, int NT>  // NT: columns of the result per workgroup (64, 128 or 256; dh is a multiple of it)
__global__ __launch_bounds__(512) void slstm_bwd_param_kernel(BwdParamParams p) {
  typedef typename std::conditional<BF16, uint16_t, float>::type elem_t;
  constexpr int ESZ = BF16 ? 2 : 4;
  constexpr int WN = NT / 64;              // waves along n
  constexpr int WM = 8 / WN;               // waves along m
  constexpr int MTILES = kParamMT / WM / 16;  // 16-row tiles of a wave: 1, 2 or 4
  constexpr int LDA = kParamMT + kParamPad, LDB = NT + kParamPad;
  constexpr int NROWTHREADS = NT / 8;      // threads that stage one row of y (8 elements each)
  constexpr int YPASS = kParamKC * NROWTHREADS / 512;  // passes over the y chunk: 1/2 (NT 64: half the threads idle), 1, 2
  extern __shared__ __attribute__((aligned(16))) unsigned char param_lds[];
  elem_t *const As = reinterpret_cast<elem_t *>(param_lds);                        // [2][32 k][LDA]
  elem_t *const Bs = reinterpret_cast<elem_t *>(param_lds) + 2 * kParamKC * LDA;   // [2][32 k][LDB]

  const int dh = p.dh, H = p.NH * dh;
  const int tiles_m = 4 * dh / kParamMT, tiles_n = dh / NT, tiles = tiles_m * tiles_n;
  // placement: the workgroups of one (head, K slice) share its stream of y chunks; they take consecutive slots of ONE
  // XCD (workgroup i runs on XCD i % 8), so that stream is fetched into one L2 once
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int group = (slot / tiles) * 8 + xcd, tile = slot % tiles;
  if (group >= p.NH * p.ksplit) return;
  const int head = group / p.ksplit, ks = group % p.ksplit;
  const int m0 = (tile / tiles_n) * kParamMT, n0 = (tile % tiles_n) * NT;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, q = lane >> 4, r16 = lane & 15;
  const int wm = wave / WN, wn = wave % WN;
  const long long BH = (long long)p.B * H;

  // this workgroup's chunks: a contiguous range of the B * tchunks chunks (chunk = 32 steps of one batch row)
  const long long nchunks = (long long)p.B * p.tchunks;
  const long long c_lo = nchunks * ks / p.ksplit, c_hi = nchunks * (ks + 1) / p.ksplit;

  // ---- staging roles.  delta: thread -> step tid / 16 of the chunk, 8 consecutive m from 8 (tid % 16); y: thread ->
  //      step (tid / NROWTHREADS) (+ 512 / NROWTHREADS per pass), 8 consecutive n
  const int dk = tid >> 4, dm = (tid & 15) * 8;
  const int dcol = m0 + dm;                       // row of the head's result = gate * dh + unit
  const long long d_off = (long long)(dcol / dh) * H + (long long)head * dh + dcol % dh;
  const int yk = tid / NROWTHREADS, yn = (tid % NROWTHREADS) * 8;
  const bool y_thread = tid < kParamKC * NROWTHREADS;  // (NT 64: 256 threads cover the chunk)
  float bsum[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
  const bool dbf16 = BF16 && p.d_wx_bf16 != 0;  // the deltas lie in bf16 (only with bf16 operands)

  struct Staged { float4 d[2]; uint4 y[YPASS < 1 ? 1 : YPASS][BF16 ? 1 : 2]; uint32_t flag[YPASS < 1 ? 1 : YPASS]; };
  // The loads of a chunk have no branch around them: they go through buffer descriptors that end where the chunk's
  // valid rows end, so a step past the end of the sequence, the step in front of step 0 and a call without a mask
  // read zeros (with `if (t < T)` and the like around the loads: 0.28 instead of 0.23 ms at B 16 x T 2048 x D 1024).
  // What the initial state contributes - y in front of step 0 - is added by the first slice of K in a short loop of its
  // own behind the main one.
  auto fetch = [&](long long c, Staged &s) {
    const int b = (int)(c / p.tchunks), t0 = (int)(c % p.tchunks) * kParamKC;
    const int nrows = p.T - t0 < kParamKC ? p.T - t0 : kParamKC;  // (>= 1)
    {  // delta: rows t0 .. of the batch row, this thread's 8 m of row dk
      const int dsz = dbf16 ? 2 : 4;
      const char *base = reinterpret_cast<const char *>(p.d_wx) + ((long long)b * p.d_wx_sb + (long long)t0 * p.d_wx_st) * dsz;
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<char *>(base), 0, (int)(((long long)(nrows - 1) * p.d_wx_st + 4ll * H) * dsz), 0x00020000);
      const int vo = (int)(((long long)dk * p.d_wx_st + d_off) * dsz);
      s.d[0] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rs, vo, 0, 0));
      // (deltas in bf16: the thread's 8 values are the first 16 bytes; the second load asks past the end and reads zeros)
      s.d[1] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rs, dbf16 ? (int)0x80000000 : vo + 16, 0, 0));
    }
    // y_{t-1}: the outputs of steps t0 - 1 .. (row -1, in front of step 0, lies in front of the descriptor: zeros)
    const int tb = t0 > 0 ? t0 - 1 : 0;  // the step the descriptor starts at
    const long long col = (long long)head * dh + n0;
    const char *ybase = reinterpret_cast<const char *>(p.h_out) + ((long long)tb * BH + (long long)b * H + col) * ESZ;
    const int yrows = t0 + nrows - 1 - tb;  // rows of h_out behind ybase that the chunk's steps use (0: only step 0)
    const __amdgpu_buffer_rsrc_t yrs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char *>(ybase), 0, yrows > 0 ? (int)(((long long)(yrows - 1) * BH + NT) * ESZ) : 0, 0x00020000);
    const __amdgpu_buffer_rsrc_t frs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(p.reset ? p.reset + (long long)b * p.reset_sb + t0 : reinterpret_cast<const uint8_t *>(p.d_wx)), 0,
        p.reset ? nrows : 0, 0x00020000);
#pragma unroll
    for (int ps = 0; ps < (YPASS < 1 ? 1 : YPASS); ++ps) {
      const int k = yk + ps * (512 / NROWTHREADS);          // the chunk's step t0 + k
      const int row = t0 + k - 1 - tb;                      // its operand's row behind ybase; -1 in front of step 0
      // (threads beyond the chunk - NT 64: the upper half of the workgroup - ask out of range too)
      const int vo = (y_thread && row >= 0) ? (int)(((long long)row * BH + yn) * ESZ) : (int)0x80000000;
      s.y[ps][0] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(yrs, vo, 0, 0));
      if (!BF16) s.y[ps][BF16 ? 0 : 1] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(yrs, vo, 16, 0));
      s.flag[ps] = __builtin_amdgcn_raw_buffer_load_b8(frs, y_thread ? k : (int)0x80000000, 0, 0);
    }
  };
  // the chunk of the initial state: k = 32 batch rows from b0, delta of step 0 against the y of s0 (rows that start a
  // document at step 0 and rows past the batch: zeros)
  auto fetch_initial = [&](int b0, Staged &s) {
    {
      const int b = b0 + dk;
      s.d[0] = s.d[1] = float4{0.0f, 0.0f, 0.0f, 0.0f};
      if (b < p.B) {
        const char *src = reinterpret_cast<const char *>(p.d_wx) + ((long long)b * p.d_wx_sb + d_off) * (dbf16 ? 2 : 4);
        s.d[0] = *reinterpret_cast<const float4 *>(src);
        if (!dbf16) s.d[1] = *reinterpret_cast<const float4 *>(src + 16);
      }
    }
#pragma unroll
    for (int ps = 0; ps < (YPASS < 1 ? 1 : YPASS); ++ps) {
      const int b = b0 + yk + ps * (512 / NROWTHREADS);
#pragma unroll
      for (int e = 0; e < (BF16 ? 1 : 2); ++e) s.y[ps][e] = uint4{0u, 0u, 0u, 0u};
      s.flag[ps] = 0u;
      if (!y_thread || b >= p.B) continue;
      if (p.reset) s.flag[ps] = p.reset[(long long)b * p.reset_sb];
      const long long col = (long long)head * dh + n0 + yn;
      const float4 lo = *reinterpret_cast<const float4 *>(p.s0 + (long long)b * H + col);
      const float4 hi = *reinterpret_cast<const float4 *>(p.s0 + (long long)b * H + col + 4);
      if (BF16) {
        s.y[ps][0] = uint4{pack_bf16x2(lo.x, lo.y), pack_bf16x2(lo.z, lo.w), pack_bf16x2(hi.x, hi.y), pack_bf16x2(hi.z, hi.w)};
      } else {
        s.y[ps][0] = __builtin_bit_cast(uint4, lo);
        s.y[ps][BF16 ? 0 : 1] = __builtin_bit_cast(uint4, hi);
      }
    }
  };
  auto stage = [&](const Staged &s, int buf, bool count_bias = true) {
    float dv[8] = {s.d[0].x, s.d[0].y, s.d[0].z, s.d[0].w, s.d[1].x, s.d[1].y, s.d[1].z, s.d[1].w};
    if (dbf16) {  // (8 bf16 in the first 16 bytes)
      const uint32_t w[4] = {__float_as_uint(s.d[0].x), __float_as_uint(s.d[0].y), __float_as_uint(s.d[0].z), __float_as_uint(s.d[0].w)};
#pragma unroll
      for (int j = 0; j < 4; ++j) { dv[2 * j] = bf16_bits_to_float(w[j] & 0xFFFFu); dv[2 * j + 1] = bf16_bits_to_float(w[j] >> 16); }
    }
    if (n0 == 0 && count_bias) {
#pragma unroll
      for (int j = 0; j < 8; ++j) bsum[j] += dv[j];
    }
    elem_t *a = As + ((long long)buf * kParamKC + dk) * LDA + dm;
    if (BF16) {
      *reinterpret_cast<uint2 *>(a) = uint2{pack_bf16x2(dv[0], dv[1]), pack_bf16x2(dv[2], dv[3])};
      *reinterpret_cast<uint2 *>(a + 4) = uint2{pack_bf16x2(dv[4], dv[5]), pack_bf16x2(dv[6], dv[7])};
    } else {
      *reinterpret_cast<float4 *>(a) = s.d[0];
      *reinterpret_cast<float4 *>(a + 4) = s.d[1];
    }
    if (y_thread) {
#pragma unroll
      for (int ps = 0; ps < (YPASS < 1 ? 1 : YPASS); ++ps) {
        elem_t *bdst = Bs + ((long long)buf * kParamKC + yk + ps * (512 / NROWTHREADS)) * LDB + yn;
        const bool keep = (s.flag[ps] & 0xFFu) == 0u;  // (a row that starts a document at this step: the forward's operand was zero)
        const uint4 y0 = keep ? s.y[ps][0] : uint4{0u, 0u, 0u, 0u};
        if (BF16) {
          *reinterpret_cast<uint2 *>(bdst) = uint2{y0.x, y0.y};
          *reinterpret_cast<uint2 *>(bdst + 4) = uint2{y0.z, y0.w};
        } else {
          *reinterpret_cast<uint4 *>(bdst) = y0;
          *reinterpret_cast<uint4 *>(bdst + 4) = keep ? s.y[ps][BF16 ? 0 : 1] : uint4{0u, 0u, 0u, 0u};
        }
      }
    }
  };

  f32x4 acc[MTILES][4];
#pragma unroll
  for (int i = 0; i < MTILES; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  const int am = wm * (MTILES * 16) + r16;   // this lane's row of an A fragment inside the workgroup's 128 (+ 16 per tile)
  const int bn = wn * 64 + r16;              // ... column of a B fragment (+ 16 per tile)

  // Two chunks are in flight beyond the one in LDS (two sets of staging registers, used in turn): with one, every
  // chunk cost a whole memory latency (0.36 ms at B 16 x T 2048 x D 1024; 64 KiB a compute unit in flight are what
  // keeps the memory system busy)
  auto compute = [&](int buf) {
    const elem_t *A = As + (long long)buf * kParamKC * LDA, *Bm = Bs + (long long)buf * kParamKC * LDB;
    if constexpr (BF16) {
      // one MFMA k-step = the whole chunk: lane group q takes k = 8 q .. 8 q + 7
      uint4 af[MTILES], bf[4];
      auto gather = [&](const uint16_t *base, int ld, int col) {  // 8 k of one column: halves of four registers
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
          w[e] = (uint32_t)base[(8 * q + 2 * e) * ld + col] | ((uint32_t)base[(8 * q + 2 * e + 1) * ld + col] << 16);
        return uint4{w[0], w[1], w[2], w[3]};
      };
#pragma unroll
      for (int i = 0; i < MTILES; ++i) af[i] = gather(A, LDA, am + 16 * i);
#pragma unroll
      for (int j = 0; j < 4; ++j) bf[j] = gather(Bm, LDB, bn + 16 * j);
#pragma unroll
      for (int i = 0; i < MTILES; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[i]), __builtin_bit_cast(bf16x8, bf[j]), acc[i][j], 0, 0, 0);
    } else {
#pragma unroll
      for (int k4 = 0; k4 < kParamKC / 4; ++k4) {  // lane group q takes k = 4 k4 + q
        float af[MTILES], bf[4];
#pragma unroll
        for (int i = 0; i < MTILES; ++i) af[i] = A[(4 * k4 + q) * LDA + am + 16 * i];
#pragma unroll
        for (int j = 0; j < 4; ++j) bf[j] = Bm[(4 * k4 + q) * LDB + bn + 16 * j];
#pragma unroll
        for (int i = 0; i < MTILES; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[i], bf[j], acc[i][j], 0, 0, 0);
      }
    }
  };
  Staged sa, sb;
  if (c_lo < c_hi) {
    fetch(c_lo, sa);
    if (c_lo + 1 < c_hi) fetch(c_lo + 1, sb);
    stage(sa, 0);
    if (c_lo + 2 < c_hi) fetch(c_lo + 2, sa);
  }
  __syncthreads();
  // (With every fetch issued whatever the chunk number, so that the compiler counts exactly two chunks in flight at
  // each stage - its waits then read vmcnt(11) and (7) instead of (5) and (4) - the kernel is not faster, 0.244
  // against 0.229 ms at B 16 x T 2048 x D 1024.  Nor is the gathering from LDS what bounds it: with one 16-byte read
  // per fragment in place of the eight 16-bit reads (wrong values, a timing probe) it takes 0.209 ms.  It moves its
  // 604 MB at 2.6 TB/s, in pieces of 512 bytes per step and row.)
  auto iteration = [&](long long c, Staged &next, int buf) {  // `next` holds chunk c + 1 and is refilled with chunk c + 3
    compute(buf);
    if (c + 1 < c_hi) stage(next, buf ^ 1);  // (the other buffer: everybody left it before the barrier that opened this chunk)
    if (c + 3 < c_hi) fetch(c + 3, next);
    __syncthreads();
  };
  for (long long c = c_lo; c < c_hi; c += 2) {
    iteration(c, sb, 0);
    if (c + 1 < c_hi) iteration(c + 1, sa, 1);
  }
  if (ks == 0 && p.s0) {  // what the initial state contributes (the deltas of step 0 are in the bias sums already)
    for (int b0 = 0; b0 < p.B; b0 += kParamKC) {
      fetch_initial(b0, sa);
      stage(sa, 0, false);
      __syncthreads();
      compute(0);
      __syncthreads();
    }
  }

  // ---- the slice's share of d_r: lane (q, r16) holds rows 4 q .. 4 q + 3, column r16 of every 16 x 16 tile
#pragma unroll
  for (int i = 0; i < MTILES; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int row = m0 + wm * (MTILES * 16) + 16 * i + 4 * q + e, col = n0 + wn * 64 + 16 * j + r16;
        atomicAdd(p.d_r + ((long long)head * 4 * dh + row) * dh + col, acc[i][j][e]);
      }
  // ---- ... and of the bias (the workgroups of the first column tile): the 32 threads that staged a group of 8 m add
  //      up through LDS (the staging buffers are free behind the last barrier)
  if (n0 == 0) {
    float *red = reinterpret_cast<float *>(param_lds);  // [32 steps][128 m]
#pragma unroll
    for (int j = 0; j < 8; ++j) red[dk * kParamMT + dm + j] = bsum[j];
    __syncthreads();
    if (tid < kParamMT) {
      float sum = 0.0f;
#pragma unroll 8
      for (int k = 0; k < kParamKC; ++k) sum += red[k * kParamMT + tid];
      const int row = m0 + tid;  // = gate * dh + unit
      atomicAdd(p.d_bias + (long long)head * 4 * dh + row, sum);
    }
  }
}

}  // namespace
