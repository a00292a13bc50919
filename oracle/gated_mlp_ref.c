/*
 * Plain-C restatement of the gated-MLP hot path (TEST INFRASTRUCTURE: a checker for tests/,
 * smoke() and the cpu_baseline leg of bench.py; never linked into the product library).
 *
 * Follows the reference's eager definition and closed-form backward
 *   EagerGatedMLP.forward   src/triton_gated_mlp/gated_mlp.py:92-98
 *   eager_fwd / eager_bwd   src/triton_gated_mlp/gated_mlp.py:105-156
 *   silu' = s(1 + x(1-s))   src/triton_gated_mlp/gated_mlp.py:40-43, ops/act.py:42-45
 *   hidden_act table        src/triton_gated_mlp/gated_mlp.py:17-37 (torch defaults: erf GELU,
 *                           LeakyReLU slope 0.01); act codes 0..6 = silu, gelu, relu, leaky_relu,
 *                           sigmoid, tanh, identity; derivatives at kinks as torch.autograd
 * with scalar loops in double precision, independent of torch and NumPy, so that the torch oracle
 * (oracle/eager.py) and the NumPy Philox (oracle/philox.py) each have a second implementation to
 * be checked against.  Layouts: row-major; W_gate, W_up [N,K]; W_down [K,N]; keep [M,N] uint8 or
 * NULL; biases may be NULL.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

static double sigmoid(double v) { return 1.0 / (1.0 + exp(-v)); }

static double act_fwd(int act, double v) {
  switch (act) {
    case 0: return v * sigmoid(v);
    case 1: return 0.5 * v * (1.0 + erf(v / sqrt(2.0)));
    case 2: return v > 0.0 ? v : 0.0;
    case 3: return v > 0.0 ? v : 0.01 * v;
    case 4: return sigmoid(v);
    case 5: return tanh(v);
    default: return v;
  }
}

static double act_grad(int act, double v) {
  switch (act) {
    case 0: { double s = sigmoid(v); return s * (1.0 + v * (1.0 - s)); }
    case 1: return 0.5 * (1.0 + erf(v / sqrt(2.0))) + v * exp(-0.5 * v * v) / sqrt(2.0 * M_PI);
    case 2: return v > 0.0 ? 1.0 : 0.0;
    case 3: return v > 0.0 ? 1.0 : 0.01;
    case 4: { double s = sigmoid(v); return s * (1.0 - s); }
    case 5: { double t = tanh(v); return 1.0 - t * t; }
    default: return 1.0;
  }
}

/* G, U, H: [M,N] outputs; Y: [M,K] output. */
void gmlp_ref_forward(const double* x, const double* wg, const double* bg, const double* wu,
                      const double* bu, const double* wd, const double* bd, const uint8_t* keep,
                      double p, int act, int64_t M, int64_t K, int64_t N, double* G, double* U,
                      double* H, double* Y) {
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      double g = bg ? bg[n] : 0.0, u = bu ? bu[n] : 0.0;
      for (int64_t k = 0; k < K; ++k) {
        g += x[m * K + k] * wg[n * K + k];
        u += x[m * K + k] * wu[n * K + k];
      }
      double h = act_fwd(act, g) * u;
      if (keep && p > 0.0) h = keep[m * N + n] ? h / (1.0 - p) : 0.0;
      G[m * N + n] = g;
      U[m * N + n] = u;
      H[m * N + n] = h;
    }
  for (int64_t m = 0; m < M; ++m)
    for (int64_t k = 0; k < K; ++k) {
      double y = bd ? bd[k] : 0.0;
      for (int64_t n = 0; n < N; ++n) y += H[m * N + n] * wd[k * N + n];
      Y[m * K + k] = y;
    }
}

/* Gradients for upstream dY [M,K].  G, U, H as produced by gmlp_ref_forward.
 * Outputs: dX [M,K], dWg [N,K], dWu [N,K], dWd [K,N], dbg [N], dbu [N], dbd [K] (bias outputs
 * may be NULL). */
void gmlp_ref_backward(const double* x, const double* wg, const double* wu, const double* wd,
                       const uint8_t* keep, double p, int act, const double* G, const double* U,
                       const double* H, const double* dY, int64_t M, int64_t K, int64_t N,
                       double* dX, double* dWg, double* dWu, double* dWd, double* dbg, double* dbu,
                       double* dbd) {
  double* dG = (double*)malloc(sizeof(double) * (size_t)(M * N));
  double* dU = (double*)malloc(sizeof(double) * (size_t)(M * N));
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      double dh = 0.0;
      for (int64_t k = 0; k < K; ++k) dh += dY[m * K + k] * wd[k * N + n];
      if (keep && p > 0.0) dh = keep[m * N + n] ? dh / (1.0 - p) : 0.0;
      double g = G[m * N + n];
      dU[m * N + n] = dh * act_fwd(act, g);
      dG[m * N + n] = dh * U[m * N + n] * act_grad(act, g);
    }
  for (int64_t m = 0; m < M; ++m)
    for (int64_t k = 0; k < K; ++k) {
      double a = 0.0;
      for (int64_t n = 0; n < N; ++n) a += dU[m * N + n] * wu[n * K + k] + dG[m * N + n] * wg[n * K + k];
      dX[m * K + k] = a;
    }
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t k = 0; k < K; ++k) {
      double a = 0.0, b = 0.0;
      for (int64_t m = 0; m < M; ++m) {
        a += dG[m * N + n] * x[m * K + k];
        b += dU[m * N + n] * x[m * K + k];
      }
      dWg[n * K + k] = a;
      dWu[n * K + k] = b;
    }
    double sg = 0.0, su = 0.0;
    for (int64_t m = 0; m < M; ++m) { sg += dG[m * N + n]; su += dU[m * N + n]; }
    if (dbg) dbg[n] = sg;
    if (dbu) dbu[n] = su;
  }
  for (int64_t k = 0; k < K; ++k) {
    for (int64_t n = 0; n < N; ++n) {
      double a = 0.0;
      for (int64_t m = 0; m < M; ++m) a += dY[m * K + k] * H[m * N + n];
      dWd[k * N + n] = a;
    }
    double s = 0.0;
    for (int64_t m = 0; m < M; ++m) s += dY[m * K + k];
    if (dbd) dbd[k] = s;
  }
  free(dG);
  free(dU);
}

/* Philox4x32-10 (Salmon et al., SC'11), scalar. */
void gmlp_ref_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; ++r) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* keep[e] = word(e) >= threshold; e = m*N + n; see oracle/philox.py for the definition. */
void gmlp_ref_keep_mask(uint8_t* keep, int64_t M, int64_t N, uint32_t threshold, uint64_t seed,
                        uint64_t offset) {
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  for (int64_t e = 0; e < M * N; ++e) {
    uint64_t e4 = (uint64_t)e >> 2;
    uint32_t ctr[4] = {(uint32_t)e4, (uint32_t)(e4 >> 32), (uint32_t)offset, (uint32_t)(offset >> 32)};
    uint32_t w[4];
    gmlp_ref_philox4x32_10(ctr, key, w);
    keep[e] = w[e & 3] >= threshold;
  }
}
