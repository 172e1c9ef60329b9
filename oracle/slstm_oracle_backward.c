/*
 * TEST INFRASTRUCTURE ONLY — CPU restatement (float64) of the sLSTM cell's backward pass.
 *
 * Nothing shipped in the product path may link, import or call it.  It exists so that a backward pass of the engine
 * has an oracle before it has a kernel.
 *
 * What it restates (reference NX-AI/xlstm, paths relative to its root):
 *   - the pointwise gradient:      xlstm/blocks/slstm/src/cuda/slstm_pointwise.cu:118-196 (SLSTMPointwiseBackward)
 *   - the recurrent contraction with R transposed, the gradient of R and of the bias over time:
 *                                  xlstm/blocks/slstm/src/cuda/slstm_backward.cu:291-303, 314-319, 381-386, 52-108
 *   - the forward it differentiates: xlstm/blocks/slstm/src/vanilla/__init__.py:17-74, vanilla/slstm.py:8-37
 *
 * The rule of the native kernel: the stabiliser m is a constant of the differentiation (its gradient is written as
 * zero, slstm_pointwise.cu:187-190).  For every loss that depends on the outputs y only this IS the gradient: y does
 * not depend on the choice of m (c and n scale alike), so the paths through m cancel.  For a loss on the final c, n
 * or m it is not the derivative of the forward as written; the vanilla path's autograd differs there, and so does
 * this restatement (tests/golden/bwd_state_loss.npz documents the difference).
 *
 * Two options of the reference's native backward are restated as well:
 *   recurrent_cut      no gradient passes from a step to the y it started from: the contraction with R transposed is
 *                      left out (xlstm/blocks/slstm/src/cuda/slstm_backward_cut.cu:265-312 against
 *                      slstm_backward.cu:314-319; chosen by cell.py:580-583).  c and n still pass their gradients on.
 *   recurrent_clipval  the gradient that reaches y_t through the recurrence is clipped to +-clipval before the
 *                      gradient from outside is added (slstm_pointwise.cu:136-143).  What comes from outside (d_h, and
 *                      at the last step the y part of d_s_final, which the reference receives through the same
 *                      argument, slstm_backward.cu:367-370; ds starts as zeros, slstm.cc:178-179) is not clipped.  <= 0 or not finite: no clipping.
 *
 * Pinning status:
 *   slstm_oracle_backward_f64: pinned by (a) central finite differences of slstm_oracle_forward_f64 for losses that
 *     are linear forms of the outputs, in every input (W.x, R, bias, initial y/c/n), (b) the gradients that the
 *     reference's vanilla cell returns through autograd for such losses (tests/golden/bwd_*.npz), (c) rows that a
 *     reset mask cuts: the gradient of a packed row equals the gradients of its documents run alone, (d) the
 *     d_s_final argument (y, c, n) by the chain rule: the gradients of a sequence equal those of its two halves when
 *     the second half's d_s0 is the first half's d_s_final, (e) recurrent_cut by the gradient of the same outputs
 *     computed with R = 0 from inputs that already contain R y_{t-1} (the pinned path), (f) recurrent_clipval by a
 *     step-by-step restatement in numpy around one-step calls (tests/test_oracle_backward.py).
 *
 * Layouts as in slstm_oracle.c; d_h [T, B, NH*dh] is the gradient of the loss with respect to h_out, d_s_final
 * [4, B, NH*dh] (may be NULL) with respect to the final state; outputs d_wx [B, T, 4, NH, dh], d_r_ext [NH, dh, 4, dh],
 * d_b_ext [NH, 4, dh], d_s0 [4, B, NH*dh] (the m part is zero).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static double bw_logsigmoid(double x) { return (x < 0 ? x : 0) - log1p(exp(-fabs(x))); }
static double bw_sigmoid(double x) {
  if (x >= 0) return 1.0 / (1.0 + exp(-x));
  const double e = exp(x);
  return e / (1.0 + e);
}

int slstm_oracle_backward_f64(const double *wx, const double *r_ext, const double *b_ext, const double *s0,
                              const uint8_t *reset, const double *d_h, const double *d_s_final, double *d_wx,
                              double *d_r_ext, double *d_b_ext, double *d_s0, int B, int T, int NH, int dh, int n0_rule,
                              int recurrent_cut, double recurrent_clipval) {
  const size_t H = (size_t)NH * dh, BH = (size_t)B * H;
  /* ---- forward, keeping what the backward needs: the state BEFORE every step (after the reset) and after it, and
   *      the gate values the native kernel caches (exp(i - m'), raw f, tanh z, sigmoid o) */
  double *sb = (double *)calloc((size_t)T * 4 * BH + 1, sizeof(double)); /* [T][4][B][H] state before step t */
  double *sa = (double *)calloc((size_t)T * 4 * BH + 1, sizeof(double)); /* [T][4][B][H] state after step t */
  double *gc = (double *)calloc((size_t)T * 4 * BH + 1, sizeof(double)); /* [T][4][B][H] cached gate values */
  double *cur = (double *)calloc(4 * BH, sizeof(double));
  double *dcur = (double *)calloc(4 * BH, sizeof(double)); /* gradient w.r.t. the state after step t (y, c, n, m) */
  double *delta = (double *)calloc(4 * BH, sizeof(double)); /* [4][B][H] gradient w.r.t. the raw gates of a step */
  if (!sb || !sa || !gc || !cur || !dcur || !delta) return -1;
  if (s0) memcpy(cur, s0, 4 * BH * sizeof(double));
  for (int t = 0; t < T; ++t) {
    if (reset)
      for (int b = 0; b < B; ++b)
        if (reset[(size_t)b * T + t])
          for (int s = 0; s < 4; ++s) memset(cur + s * BH + (size_t)b * H, 0, H * sizeof(double));
    double *y = cur, *c = cur + BH, *n = cur + 2 * BH, *m = cur + 3 * BH;
    memcpy(sb + (size_t)t * 4 * BH, cur, 4 * BH * sizeof(double));
    int all_n_zero = 1;
    if (n0_rule == 1)
      for (size_t k = 0; k < BH; ++k)
        if (n[k] != 0) { all_n_zero = 0; break; }
    double *after = sa + (size_t)t * 4 * BH, *g = gc + (size_t)t * 4 * BH;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b)
      for (int h = 0; h < NH; ++h)
        for (int a = 0; a < dh; ++a) {
          const size_t k = (size_t)h * dh + a, idx = (size_t)b * H + k;
          double raw[4];
          for (int q = 0; q < 4; ++q) {
            double ry = 0;
            for (int d = 0; d < dh; ++d)
              ry += y[(size_t)b * H + (size_t)h * dh + d] * r_ext[(((size_t)h * dh + d) * 4 + q) * dh + a];
            raw[q] = wx[((size_t)b * T + t) * 4 * H + q * H + k] + ry + b_ext[((size_t)h * 4 + q) * dh + a];
          }
          const double lfm = m[idx] + bw_logsigmoid(raw[1]);
          const int nz = (n0_rule == 1) ? all_n_zero : (n[idx] == 0);
          const double mnew = nz ? raw[0] : (raw[0] > lfm ? raw[0] : lfm);
          const double og = bw_sigmoid(raw[3]);
          double ig = exp(raw[0] - mnew), fg = exp(lfm - mnew);
          if (ig > 1) ig = 1;
          if (fg > 1) fg = 1;
          const double zv = tanh(raw[2]);
          const double cnew = fg * c[idx] + ig * zv, nnew = fg * n[idx] + ig;
          after[idx] = og * cnew / nnew; after[BH + idx] = cnew; after[2 * BH + idx] = nnew; after[3 * BH + idx] = mnew;
          g[idx] = ig; g[BH + idx] = raw[1]; g[2 * BH + idx] = zv; g[3 * BH + idx] = og;
        }
    memcpy(cur, after, 4 * BH * sizeof(double));
  }
  /* ---- backward in time */
  memset(d_r_ext, 0, (size_t)NH * dh * 4 * dh * sizeof(double));
  memset(d_b_ext, 0, (size_t)NH * 4 * dh * sizeof(double));
  if (d_s_final) memcpy(dcur, d_s_final, 4 * BH * sizeof(double));
  const int clip = isfinite(recurrent_clipval) && recurrent_clipval > 0;
  for (int t = T - 1; t >= 0; --t) {
    const double *before = sb + (size_t)t * 4 * BH, *after = sa + (size_t)t * 4 * BH, *g = gc + (size_t)t * 4 * BH;
    for (size_t idx = 0; idx < BH; ++idx) {
      /* slstm_pointwise.cu:139-190 */
      double dy_recurrent = dcur[idx];
      if (clip && t < T - 1) { /* (at the last step dcur holds what came from outside: the y part of d_s_final) */
        if (dy_recurrent > recurrent_clipval) dy_recurrent = recurrent_clipval;
        if (dy_recurrent < -recurrent_clipval) dy_recurrent = -recurrent_clipval;
      }
      const double dy_total = d_h[(size_t)t * BH + idx] + dy_recurrent;
      double dc_total = dcur[BH + idx], dn_total = dcur[2 * BH + idx];
      const double ig = g[idx], fraw = g[BH + idx], zv = g[2 * BH + idx], og = g[3 * BH + idx];
      const double c_old = before[BH + idx], n_old = before[2 * BH + idx], m_old = before[3 * BH + idx];
      const double y_new = after[idx], n_new = after[2 * BH + idx], m_new = after[3 * BH + idx];
      double fg = exp(bw_logsigmoid(fraw) + m_old - m_new);
      if (fg > 1) fg = 1;
      const double fsig = bw_sigmoid(fraw);
      const double dy_inter = dy_total / n_new;
      dc_total += dy_inter * og;
      dn_total -= dy_inter * y_new;
      delta[idx] = ig * (zv * dc_total + dn_total);
      delta[BH + idx] = fg * (dc_total * c_old + dn_total * n_old) * (1 - fsig);
      delta[2 * BH + idx] = dc_total * ig * (1 - zv * zv);
      delta[3 * BH + idx] = (1 - og) * y_new * dy_total;
      dcur[idx] = 0; dcur[BH + idx] = fg * dc_total; dcur[2 * BH + idx] = fg * dn_total; dcur[3 * BH + idx] = 0;
    }
    /* gradient of W.x and the bias; of R and of the y the step started from (slstm_backward.cu:314-319, 381-386) */
    /* (heads do not meet: one thread per head keeps every sum in the order of the plain loops) */
#pragma omp parallel for schedule(static)
    for (int h = 0; h < NH; ++h)
      for (int b = 0; b < B; ++b)
        for (int q = 0; q < 4; ++q)
          for (int a = 0; a < dh; ++a) {
            const size_t k = (size_t)h * dh + a;
            const double dv = delta[q * BH + (size_t)b * H + k];
            d_wx[((size_t)b * T + t) * 4 * H + q * H + k] = dv;
            d_b_ext[((size_t)h * 4 + q) * dh + a] += dv;
            for (int d = 0; d < dh; ++d) {
              const size_t yi = (size_t)b * H + (size_t)h * dh + d;
              d_r_ext[(((size_t)h * dh + d) * 4 + q) * dh + a] += before[yi] * dv;
              if (!recurrent_cut) dcur[yi] += dv * r_ext[(((size_t)h * dh + d) * 4 + q) * dh + a];
            }
          }
    /* a row that starts a document at t took nothing from the step before */
    if (reset)
      for (int b = 0; b < B; ++b)
        if (reset[(size_t)b * T + t])
          for (int s = 0; s < 4; ++s) memset(dcur + s * BH + (size_t)b * H, 0, H * sizeof(double));
  }
  memcpy(d_s0, dcur, 4 * BH * sizeof(double));
  free(sb); free(sa); free(gc); free(cur); free(dcur); free(delta);
  return 0;
}
