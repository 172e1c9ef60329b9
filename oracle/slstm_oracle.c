/*
 * TEST INFRASTRUCTURE ONLY — CPU restatement of the sLSTM cell forward pass.
 *
 * This file is the parity oracle for the HIP engine.  Nothing shipped in the
 * product path may link, import or call it; only tests, the smoke check and
 * the benchmark's CPU-baseline leg do.
 *
 * What it restates (reference NX-AI/xlstm, paths relative to its root):
 *   - time loop and recurrent contraction:
 *       xlstm/blocks/slstm/src/vanilla/__init__.py:17-74   (slstm_forward)
 *   - exponential-gating pointwise update:
 *       xlstm/blocks/slstm/src/vanilla/slstm.py:8-37       (slstm_forward_pointwise)
 *   - per-element "n == 0" stabiliser rule of the native kernel:
 *       xlstm/blocks/slstm/src/cuda/slstm_pointwise.cu:79-83
 *   - parameter / input layouts (external views):
 *       xlstm/blocks/slstm/cell.py:234-257 (R_ext[NH,dh_in,4,dh_out], b_ext[NH,4,dh])
 *       xlstm/blocks/slstm/cell.py:339-342 (input [B,S,4,NH,dh], gate order i,f,z,o)
 *       xlstm/blocks/slstm/cell.py:496-506 (output y[1:], final state [4,B,H] = y,c,n,m)
 *
 * Pinning status of each function:
 *   slstm_oracle_forward_{f64,f32}: pinned by (a) golden vectors written from
 *     the reference's vanilla cell (tests/golden/), (b) closed forms from a
 *     zero state, (c) an R == 0 elementwise scan evaluated independently,
 *     (d) a brute-force triple loop for the contraction, (e) stabiliser
 *     invariance, (f) chunked == whole and step-by-step == sequence.
 *   reset mask: not present in the reference (the only hook is the unused
 *     `lengths` argument, cell.py:496).  Defined here as "zero y,c,n,m of the
 *     row before the step"; pinned by "packed run == every document run alone
 *     from a zero state".
 *
 * Layouts (all row-major, contiguous):
 *   wx    [B, T, 4, NH, dh]   gate pre-activations W x (gate order i,f,z,o)
 *   r_ext [NH, dh, 4, dh]     r_ext[h][d][g][a]: input unit d -> gate g, output unit a
 *   b_ext [NH, 4, dh]
 *   s0    [4, B, NH*dh]       initial y, c, n, m (may be NULL = zeros)
 *   reset [B, T] uint8        may be NULL; non-zero => row state is zeroed before step t
 *   h_out [T, B, NH*dh]       y after each step
 *   s_out [4, B, NH*dh]       y, c, n, m after the last step
 *
 * n0_rule: 0 = per element (native-kernel rule), 1 = whole tensor
 *          (`torch.all(n == 0)`, vanilla/slstm.py:25).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define DEFINE_ORACLE(NAME, REAL, EXP, LOG1P, TANH, FABS)                              \
  static REAL NAME##_logsigmoid(REAL x) {                                              \
    /* min(x,0) - log1p(exp(-|x|)) : the numerically stable log-sigmoid */             \
    REAL mn = x < (REAL)0 ? x : (REAL)0;                                               \
    return mn - LOG1P(EXP(-FABS(x)));                                                  \
  }                                                                                    \
  static REAL NAME##_sigmoid(REAL x) {                                                 \
    if (x >= (REAL)0) {                                                                \
      return (REAL)1 / ((REAL)1 + EXP(-x));                                            \
    } else {                                                                           \
      REAL e = EXP(x);                                                                 \
      return e / ((REAL)1 + e);                                                        \
    }                                                                                  \
  }                                                                                    \
  int NAME(const REAL *wx, const REAL *r_ext, const REAL *b_ext, const REAL *s0,       \
           const uint8_t *reset, REAL *h_out, REAL *s_out, int B, int T, int NH,       \
           int dh, int n0_rule) {                                                      \
    const size_t H = (size_t)NH * dh;                                                  \
    const size_t BH = (size_t)B * H;                                                   \
    REAL *st = (REAL *)calloc(4 * BH, sizeof(REAL));                                   \
    REAL *ry_all = (REAL *)malloc((size_t)B * 4 * H * sizeof(REAL));                   \
    REAL *ynew = (REAL *)malloc(BH * sizeof(REAL));                                    \
    if (!st || !ry_all || !ynew) {                                                         \
      free(st); free(ry_all); free(ynew);                                                  \
      return -1;                                                                       \
    }                                                                                  \
    if (s0) memcpy(st, s0, 4 * BH * sizeof(REAL));                                     \
    REAL *y = st, *c = st + BH, *n = st + 2 * BH, *m = st + 3 * BH;                    \
    for (int t = 0; t < T; ++t) {                                                      \
      if (reset) {                                                                     \
        for (int b = 0; b < B; ++b) {                                                  \
          if (reset[(size_t)b * T + t]) {                                              \
            for (size_t k = 0; k < H; ++k) {                                           \
              y[b * H + k] = 0; c[b * H + k] = 0; n[b * H + k] = 0; m[b * H + k] = 0;  \
            }                                                                          \
          }                                                                            \
        }                                                                              \
      }                                                                                \
      int all_n_zero = 1;                                                              \
      if (n0_rule == 1) {                                                              \
        for (size_t k = 0; k < BH; ++k) {                                              \
          if (n[k] != (REAL)0) { all_n_zero = 0; break; }                              \
        }                                                                              \
      }                                                                                \
      _Pragma("omp parallel for schedule(static)")                                     \
      for (int b = 0; b < B; ++b) {                                                    \
        /* Ry[g][h][a] = sum_d y[b][h][d] * r_ext[h][d][g][a], d ascending */          \
        REAL *ry = ry_all + (size_t)b * 4 * H;                                         \
        for (size_t k = 0; k < 4 * H; ++k) ry[k] = 0;                                  \
        for (int h = 0; h < NH; ++h) {                                                 \
          for (int d = 0; d < dh; ++d) {                                               \
            const REAL yv = y[b * H + (size_t)h * dh + d];                             \
            for (int g = 0; g < 4; ++g) {                                              \
              const REAL *rrow = r_ext + (((size_t)h * dh + d) * 4 + g) * dh;          \
              REAL *dst = ry + ((size_t)g * NH + h) * dh;                              \
              for (int a = 0; a < dh; ++a) dst[a] += yv * rrow[a];                     \
            }                                                                          \
          }                                                                            \
        }                                                                              \
        const REAL *wxt = wx + ((size_t)b * T + t) * 4 * H;                            \
        for (int h = 0; h < NH; ++h) {                                                 \
          for (int a = 0; a < dh; ++a) {                                               \
            const size_t k = (size_t)h * dh + a;                                       \
            const size_t idx = b * H + k;                                              \
            REAL raw[4];                                                               \
            for (int g = 0; g < 4; ++g) {                                              \
              raw[g] = wxt[g * H + k] + ry[g * H + k] +                                \
                       b_ext[((size_t)h * 4 + g) * dh + a];                            \
            }                                                                          \
            const REAL lfm = m[idx] + NAME##_logsigmoid(raw[1]);                       \
            REAL mnew;                                                                 \
            int nz = (n0_rule == 1) ? all_n_zero : (n[idx] == (REAL)0);                \
            if (nz) mnew = raw[0];                                                     \
            else mnew = raw[0] > lfm ? raw[0] : lfm;                                   \
            const REAL og = NAME##_sigmoid(raw[3]);                                    \
            REAL ig = EXP(raw[0] - mnew);                                              \
            if (ig > (REAL)1) ig = 1;                                                  \
            REAL fg = EXP(lfm - mnew);                                                 \
            if (fg > (REAL)1) fg = 1;                                                  \
            const REAL cnew = fg * c[idx] + ig * TANH(raw[2]);                         \
            const REAL nnew = fg * n[idx] + ig;                                        \
            ynew[idx] = og * cnew / nnew;                                              \
            c[idx] = cnew; n[idx] = nnew; m[idx] = mnew;                               \
          }                                                                            \
        }                                                                              \
      }                                                                                \
      memcpy(y, ynew, BH * sizeof(REAL));                                              \
      if (h_out) memcpy(h_out + (size_t)t * BH, y, BH * sizeof(REAL));                 \
    }                                                                                  \
    if (s_out) memcpy(s_out, st, 4 * BH * sizeof(REAL));                               \
    free(st); free(ry_all); free(ynew);                                                    \
    return 0;                                                                          \
  }

DEFINE_ORACLE(slstm_oracle_forward_f64, double, exp, log1p, tanh, fabs)
DEFINE_ORACLE(slstm_oracle_forward_f32, float, expf, log1pf, tanhf, fabsf)
