// bnn_oracle.cpp -- TEST INFRASTRUCTURE ONLY (see bnn_oracle.h).
//
// Plain host C++ restatement of the reference's HMC math.  Build with -ffp-contract=off so that
// every fused multiply-add below is an explicit fmaf()/fma() call and nothing else is fused.
#include "bnn_oracle.h"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>
#include <limits>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

// ---------------------------------------------------------------------------------------------
// parameter layout, ffma.h:35-44: W1[k*D1 + c] | b1[c] | w2[c] | b2
// ---------------------------------------------------------------------------------------------
struct Layout {
  int d0, d1, oW1, ob1, ow2, ob2, P;
  Layout(int d0_, int d1_) : d0(d0_), d1(d1_) {
    oW1 = 0;
    ob1 = d0 * d1;
    ow2 = ob1 + d1;
    ob2 = ow2 + d1;
    P = ob2 + 1;
  }
};

// float constants derived the way the reference derives them from its double constexprs
// (ffma.h:289-300, 113-118: lit<T>(double expression))
struct Consts {
  float scale_recp, df, df_recp, loss_norm, l_scale, g_scale;  // Student-t
  float sig_recp, gauss_norm;                                  // Gaussian
  float prior_recp, prior_norm, prior_neg_recp2;
  explicit Consts(const orc_model& m) {
    const double pi = 3.14159265358979323846;
    scale_recp = (float)(1.0 / m.lik_scale);
    df = (float)m.lik_df;
    df_recp = (float)(1.0 / m.lik_df);
    // global_params.h:41-45
    double norm = std::log(std::fabs(m.lik_scale)) + 0.5 * std::log(m.lik_df) + 0.5 * std::log(pi) +
                  std::lgamma(0.5 * m.lik_df) - std::lgamma(0.5 * (m.lik_df + 1.0));
    loss_norm = (float)norm;
    l_scale = -0.5f * (df + 1.0f);      // ffma.h:297
    g_scale = (df + 1.0f) * scale_recp; // ffma.h:300
    sig_recp = (float)(1.0 / m.lik_scale);
    gauss_norm = (float)(std::log(std::fabs(m.lik_scale)) + 0.5 * std::log(2.0 * pi));
    prior_recp = (float)(1.0 / m.prior_scale);
    prior_norm = (float)(0.5 * std::log(2.0 * pi) + std::log(m.prior_scale));  // global_params.h:51-52
    prior_neg_recp2 = (float)(-1.0 / (m.prior_scale * m.prior_scale));         // global_params.h:49-50
  }
};

// kernel_helpers.h:34-42
inline float tanh_fwd(float x) {
  float e = exp2f(x * -2.88539008177792681472f);
  float denom = 1.0f + e;
  float sigm = 1.0f / denom;
  return std::fabs(x) < 0.0048176045529544353485f ? x : fmaf(sigm, 2.0f, -1.0f);
}
// kernel_helpers.h:43
inline float tanh_bwd(float out, float dgrad) { return fmaf(-out, out, 1.0f) * dgrad; }

inline void row_loglik(const orc_model& m, const Consts& c, float y, float yhat, float b2,
                       float* ell, float* g) {
  if (m.lik_kind == ORC_LIK_STUDENT_T) {
    // ffma.h:293-301
    float diff = (y - yhat - b2) * c.scale_recp;
    float diff2 = diff * diff;
    *ell = c.l_scale * log1pf(diff2 * c.df_recp) - c.loss_norm;
    *g = diff * c.g_scale / (diff2 + c.df);
  } else {
    float diff = (y - yhat - b2) * c.sig_recp;
    *ell = -0.5f * (diff * diff) - c.gauss_norm;
    *g = diff * c.sig_recp;
  }
}

// ffma.h:113-118
inline void prior_terms(const Consts& c, float w, float* logp, float* grad) {
  float lp = w * c.prior_recp;
  *logp = -(lp * lp) * 0.5f - c.prior_norm;
  *grad = w * c.prior_neg_recp2;
}

// ---------------------------------------------------------------------------------------------
// Philox4x32-10 (Salmon, Moraes, Dror, Shaw, SC'11).  Published algorithm, restated.
// ---------------------------------------------------------------------------------------------
inline void philox(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
  uint32_t k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; ++r) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// natural log from +,-,*,/ only (the classic argument reduction x = 2^k (1+f), s = f/(2+f),
// degree-14 odd series in s) so that host and device agree bit for bit.  x must be a positive
// normal double.
inline double det_log(double x) {
  const double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10,
               Lg1 = 6.666666666666735130e-01, Lg2 = 3.999999999940941908e-01,
               Lg3 = 2.857142874366239149e-01, Lg4 = 2.222219843214978396e-01,
               Lg5 = 1.818357216161805012e-01, Lg6 = 1.531383769920937332e-01,
               Lg7 = 1.479819860511658591e-01;
  uint64_t bits;
  std::memcpy(&bits, &x, 8);
  uint32_t hx = (uint32_t)(bits >> 32);
  uint32_t lx = (uint32_t)bits;
  int k = (int)(hx >> 20) - 1023;
  hx &= 0x000fffffu;
  uint32_t i = (hx + 0x95f64u) & 0x100000u;
  hx |= (i ^ 0x3ff00000u);
  k += (int)(i >> 20);
  bits = ((uint64_t)hx << 32) | lx;
  double m;
  std::memcpy(&m, &bits, 8);
  double f = m - 1.0;
  double hfsq = 0.5 * f * f;
  double s = f / (2.0 + f);
  double z = s * s;
  double w = z * z;
  double t1 = w * (Lg2 + w * (Lg4 + w * Lg6));
  double t2 = z * (Lg1 + w * (Lg3 + w * (Lg5 + w * Lg7)));
  double R = t2 + t1;
  double dk = (double)k;
  return s * (hfsq + R) + dk * ln2_lo - hfsq + f + dk * ln2_hi;
}

// square root from a bit-level seed and Newton steps on 1/sqrt(x) (mul/add/fma only) so that host
// and device agree bit for bit; accurate to about one ulp.  x must be a positive normal double.
inline double det_sqrt(double x) {
  uint64_t bits;
  std::memcpy(&bits, &x, 8);
  bits = 0x5fe6eb50c7b537a9ull - (bits >> 1);
  double r;
  std::memcpy(&r, &bits, 8);
  for (int it = 0; it < 5; ++it) r = r * (1.5 - 0.5 * x * r * r);
  double s = x * r;
  return s + 0.5 * r * std::fma(-s, s, x);
}

// Wichura, Algorithm AS 241 (Appl. Statist. 37, 1988), routine PPND16: the normal quantile.
inline double ppnd16(double p) {
  const double a0 = 3.3871328727963666080e0, a1 = 1.3314166789178437745e+2,
               a2 = 1.9715909503065514427e+3, a3 = 1.3731693765509461125e+4,
               a4 = 4.5921953931549871457e+4, a5 = 6.7265770927008700853e+4,
               a6 = 3.3430575583588128105e+4, a7 = 2.5090809287301226727e+3,
               b1 = 4.2313330701600911252e+1, b2 = 6.8718700749205790830e+2,
               b3 = 5.3941960214247511077e+3, b4 = 2.1213794301586595867e+4,
               b5 = 3.9307895800092710610e+4, b6 = 2.8729085735721942674e+4,
               b7 = 5.2264952788528545610e+3;
  const double c0 = 1.42343711074968357734e0, c1 = 4.63033784615654529590e0,
               c2 = 5.76949722146069140550e0, c3 = 3.64784832476320460504e0,
               c4 = 1.27045825245236838258e0, c5 = 2.41780725177450611770e-1,
               c6 = 2.27238449892691845833e-2, c7 = 7.74545014278341407640e-4,
               d1 = 2.05319162663775882187e0, d2 = 1.67638483018380384940e0,
               d3 = 6.89767334985100004550e-1, d4 = 1.48103976427480074590e-1,
               d5 = 1.51986665636164571966e-2, d6 = 5.47593808499534494600e-4,
               d7 = 1.05075007164441684324e-9;
  const double e0 = 6.65790464350110377720e0, e1 = 5.46378491116411436990e0,
               e2 = 1.78482653991729133580e0, e3 = 2.96560571828504891230e-1,
               e4 = 2.65321895265761230930e-2, e5 = 1.24266094738807843860e-3,
               e6 = 2.71155556874348757815e-5, e7 = 2.01033439929228813265e-7,
               f1 = 5.99832206555887937690e-1, f2 = 1.36929880922735805310e-1,
               f3 = 1.48753612908506148525e-2, f4 = 7.86869131145613259100e-4,
               f5 = 1.84631831751005468180e-5, f6 = 1.42151175831644588870e-7,
               f7 = 2.04426310338993978564e-15;
  double q = p - 0.5;
  if (std::fabs(q) <= 0.425) {
    double r = 0.180625 - q * q;
    double num = (((((((a7 * r + a6) * r + a5) * r + a4) * r + a3) * r + a2) * r + a1) * r + a0);
    double den = (((((((b7 * r + b6) * r + b5) * r + b4) * r + b3) * r + b2) * r + b1) * r + 1.0);
    return q * num / den;
  }
  double r = q < 0.0 ? p : 1.0 - p;
  r = det_sqrt(-det_log(r));
  double val;
  if (r <= 5.0) {
    r -= 1.6;
    double num = (((((((c7 * r + c6) * r + c5) * r + c4) * r + c3) * r + c2) * r + c1) * r + c0);
    double den = (((((((d7 * r + d6) * r + d5) * r + d4) * r + d3) * r + d2) * r + d1) * r + 1.0);
    val = num / den;
  } else {
    r -= 5.0;
    double num = (((((((e7 * r + e6) * r + e5) * r + e4) * r + e3) * r + e2) * r + e1) * r + e0);
    double den = (((((((f7 * r + f6) * r + f5) * r + f4) * r + f3) * r + f2) * r + f1) * r + 1.0);
    val = num / den;
  }
  return q < 0.0 ? -val : val;
}

inline uint32_t rng_word(uint32_t seed, uint32_t id, uint32_t stream, uint32_t t, uint64_t index) {
  uint64_t blk = index >> 2;
  uint32_t ctr[4] = {(uint32_t)blk, t, stream, (uint32_t)(blk >> 32)};
  uint32_t key[2] = {seed, id};
  uint32_t out[4];
  philox(ctr, key, out);
  return out[index & 3];
}

inline double u01(uint32_t k) { return ((double)k + 0.5) * (1.0 / 4294967296.0); }

inline float normal(uint32_t seed, uint32_t id, uint32_t stream, uint32_t t, uint64_t index) {
  return (float)ppnd16(u01(rng_word(seed, id, stream, t, index)));
}

// ---------------------------------------------------------------------------------------------
// log-posterior and gradient, FP32 per-row arithmetic (ffma.h:225-360)
// ---------------------------------------------------------------------------------------------
constexpr int ROW_BLOCK = 16;  // rows whose terms are summed in FP32 before going to double
                               // (the reference sums 17 or 24 rows per warp in registers)

void eval_f32_range(const orc_model& m, const Consts& c, const Layout& L, const float* X,
                    const float* y, const float* w, int row_begin, int row_end, float* ell,
                    double* gacc /* P, likelihood part only, accumulated */, float* yhat_out) {
  const int d0 = L.d0, d1 = L.d1;
  const float* W1 = w + L.oW1;
  const float* b1 = w + L.ob1;
  const float* w2 = w + L.ow2;
  const float b2 = w[L.ob2];
  std::vector<float> h(d1), delta(d1), gblk(L.P);
  for (int r0 = row_begin; r0 < row_end; r0 += ROW_BLOCK) {
    int r1 = std::min(r0 + ROW_BLOCK, row_end);
    std::fill(gblk.begin(), gblk.end(), 0.0f);
    for (int i = r0; i < r1; ++i) {
      const float* x = X + (size_t)i * d0;
      // layer 1: FMA chain over k ascending starting from the bias (ffma.h:225-255)
      for (int cc = 0; cc < d1; ++cc) h[cc] = b1[cc];
      for (int k = 0; k < d0; ++k) {
        const float xk = x[k];
        const float* wr = W1 + (size_t)k * d1;
        for (int cc = 0; cc < d1; ++cc) h[cc] = fmaf(wr[cc], xk, h[cc]);
      }
      for (int cc = 0; cc < d1; ++cc) h[cc] = tanh_fwd(h[cc]);  // ffma.h:256-263
      // layer 2 dot (ffma.h:265-281); b2 enters through the residual (ffma.h:293)
      float yh = 0.0f;
      for (int cc = 0; cc < d1; ++cc) yh = fmaf(w2[cc], h[cc], yh);
      float li, gi;
      row_loglik(m, c, y[i], yh, b2, &li, &gi);
      if (ell) ell[i] = li;
      if (yhat_out) yhat_out[i] = yh;
      // backward (ffma.h:306-360)
      gblk[L.ob2] += gi;
      for (int cc = 0; cc < d1; ++cc) {
        gblk[L.ow2 + cc] = fmaf(gi, h[cc], gblk[L.ow2 + cc]);
        float dl = tanh_bwd(h[cc], w2[cc] * gi);
        delta[cc] = dl;
        gblk[L.ob1 + cc] += dl;
      }
      for (int k = 0; k < d0; ++k) {
        const float xk = x[k];
        float* gr = gblk.data() + (size_t)k * d1;
        for (int cc = 0; cc < d1; ++cc) gr[cc] = fmaf(xk, delta[cc], gr[cc]);
      }
    }
    for (int p = 0; p < L.P; ++p) gacc[p] += (double)gblk[p];
  }
}

// Rows are cut into fixed chunks of ROW_CHUNK rows (whatever the number of threads); each chunk is
// summed on its own in block order and the chunk sums are added in chunk order, so the result does
// not depend on how many threads ran.
constexpr int ROW_CHUNK = 64 * ROW_BLOCK;

void eval_f32(const orc_model& m, const float* X, const float* y, const float* w, float* ell,
              float* prior, float* grad, float* yhat) {
  Consts c(m);
  Layout L(m.d0, m.d1);
  const int n_chunks = (m.n + ROW_CHUNK - 1) / ROW_CHUNK;
  std::vector<double> gacc((size_t)std::max(n_chunks, 1) * L.P, 0.0);
#ifdef _OPENMP
#pragma omp parallel for schedule(static) if (n_chunks > 1)
#endif
  for (int ch = 0; ch < n_chunks; ++ch)
    eval_f32_range(m, c, L, X, y, w, ch * ROW_CHUNK, std::min(m.n, (ch + 1) * ROW_CHUNK), ell,
                   gacc.data() + (size_t)ch * L.P, yhat);
  for (int ch = 1; ch < n_chunks; ++ch)
    for (int p = 0; p < L.P; ++p) gacc[p] += gacc[(size_t)ch * L.P + p];
  for (int p = 0; p < L.P; ++p) {
    float lp, gp;
    prior_terms(c, w[p], &lp, &gp);
    if (prior) prior[p] = lp;
    if (grad) grad[p] = (float)((double)gp + gacc[p]);  // block 0 seeds with the prior gradient
  }
}

void eval_f64(const orc_model& m, const float* X, const float* y, const double* w, double* ell,
              double* prior, double* grad) {
  const double pi = 3.14159265358979323846;
  Layout L(m.d0, m.d1);
  const int d0 = L.d0, d1 = L.d1;
  const double* W1 = w + L.oW1;
  const double* b1 = w + L.ob1;
  const double* w2 = w + L.ow2;
  const double b2 = w[L.ob2];
  std::vector<double> h(d1), g(L.P, 0.0);
  double lik_norm, prior_norm = 0.5 * std::log(2.0 * pi) + std::log(m.prior_scale);
  if (m.lik_kind == ORC_LIK_STUDENT_T)
    lik_norm = std::log(std::fabs(m.lik_scale)) + 0.5 * std::log(m.lik_df) + 0.5 * std::log(pi) +
               std::lgamma(0.5 * m.lik_df) - std::lgamma(0.5 * (m.lik_df + 1.0));
  else
    lik_norm = std::log(std::fabs(m.lik_scale)) + 0.5 * std::log(2.0 * pi);
  for (int i = 0; i < m.n; ++i) {
    const float* x = X + (size_t)i * d0;
    double yh = 0.0;
    for (int cc = 0; cc < d1; ++cc) {
      double a = b1[cc];
      for (int k = 0; k < d0; ++k) a += W1[(size_t)k * d1 + cc] * (double)x[k];
      h[cc] = std::tanh(a);
      yh += w2[cc] * h[cc];
    }
    double d = ((double)y[i] - yh - b2) / m.lik_scale, li, gi;
    if (m.lik_kind == ORC_LIK_STUDENT_T) {
      li = -0.5 * (m.lik_df + 1.0) * std::log1p(d * d / m.lik_df) - lik_norm;
      gi = d * (m.lik_df + 1.0) / m.lik_scale / (d * d + m.lik_df);
    } else {
      li = -0.5 * d * d - lik_norm;
      gi = d / m.lik_scale;
    }
    if (ell) ell[i] = li;
    g[L.ob2] += gi;
    for (int cc = 0; cc < d1; ++cc) {
      g[L.ow2 + cc] += gi * h[cc];
      double dl = (1.0 - h[cc] * h[cc]) * w2[cc] * gi;
      g[L.ob1 + cc] += dl;
      for (int k = 0; k < d0; ++k) g[(size_t)k * d1 + cc] += (double)x[k] * dl;
    }
  }
  for (int p = 0; p < L.P; ++p) {
    double s = w[p] / m.prior_scale;
    if (prior) prior[p] = -0.5 * s * s - prior_norm;
    if (grad) grad[p] = g[p] - w[p] / (m.prior_scale * m.prior_scale);
  }
}

// one leapfrog position/momentum update, ffma.h:106-112.  mom_correction is 2 for the first step
// of a trajectory (half kick) and 1 afterwards.  Written as two explicit FMAs.
inline void leapfrog_update(float& w, float& mom, float g_prev, float eps, int mom_correction) {
  float e = mom_correction == 2 ? eps * 0.5f : eps;
  mom = fmaf(e, g_prev, mom);
  w = fmaf(eps, mom, w);
}

bool g_cut_short = true;  // see orc_set_cut_short

}  // namespace

extern "C" {

void orc_set_threads(int threads) {
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#else
  (void)threads;
#endif
}
void orc_set_cut_short(int on) { g_cut_short = on != 0; }

int orc_num_params(int d0, int d1) { return Layout(d0, d1).P; }

void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  philox(ctr, key, out);
}
double orc_det_log(double x) { return det_log(x); }
double orc_det_sqrt(double x) { return det_sqrt(x); }
double orc_ppnd16(double p) { return ppnd16(p); }
uint32_t orc_rng_word(uint32_t seed, uint32_t id, uint32_t stream, uint32_t t, uint64_t index) {
  return rng_word(seed, id, stream, t, index);
}
float orc_normal(uint32_t seed, uint32_t id, uint32_t stream, uint32_t t, uint64_t index) {
  return normal(seed, id, stream, t, index);
}
void orc_momentum(uint32_t seed, uint32_t chain_id, uint32_t t, int P, float* out) {
  for (int p = 0; p < P; ++p) out[p] = normal(seed, chain_id, ORC_STREAM_MOMENTUM, t, (uint64_t)p);
}
float orc_log_uniform(uint32_t seed, uint32_t chain_id, uint32_t t) {
  return (float)det_log(u01(rng_word(seed, chain_id, ORC_STREAM_ACCEPT, t, 0)));
}

void orc_gen_window(uint32_t seed, uint32_t window, int n, int d0, int d1, float teacher_scale,
                    float noise_sigma, float* X, float* y, float* teacher) {
  Layout L(d0, d1);
  std::vector<float> th(L.P);
  for (int p = 0; p < L.P; ++p)
    th[p] = teacher_scale * normal(seed, window, ORC_STREAM_TEACHER, 0, (uint64_t)p);
  if (teacher) std::memcpy(teacher, th.data(), sizeof(float) * L.P);
  std::vector<float> h(d1);
  for (int i = 0; i < n; ++i) {
    float* x = X + (size_t)i * d0;
    for (int k = 0; k < d0; ++k)
      x[k] = normal(seed, window, ORC_STREAM_X, 0, (uint64_t)i * d0 + k);
    for (int cc = 0; cc < d1; ++cc) h[cc] = th[L.ob1 + cc];
    for (int k = 0; k < d0; ++k)
      for (int cc = 0; cc < d1; ++cc) h[cc] = fmaf(th[(size_t)k * d1 + cc], x[k], h[cc]);
    float yh = th[L.ob2];
    for (int cc = 0; cc < d1; ++cc) yh = fmaf(th[L.ow2 + cc], tanh_fwd(h[cc]), yh);
    y[i] = fmaf(noise_sigma, normal(seed, window, ORC_STREAM_NOISE, 0, (uint64_t)i), yh);
  }
}

float orc_tanh_fwd(float x) { return tanh_fwd(x); }
float orc_tanh_bwd(float out, float dgrad) { return tanh_bwd(out, dgrad); }
void orc_row_loglik(const orc_model* m, float y, float yhat, float b2, float* ell, float* g) {
  Consts c(*m);
  row_loglik(*m, c, y, yhat, b2, ell, g);
}
void orc_prior_terms(const orc_model* m, float w, float* logp, float* grad) {
  Consts c(*m);
  prior_terms(c, w, logp, grad);
}

void orc_eval_f32(const orc_model* m, const float* X, const float* y, const float* w, float* ell,
                  float* prior, float* grad, float* yhat) {
  eval_f32(*m, X, y, w, ell, prior, grad, yhat);
}
void orc_eval_f64(const orc_model* m, const float* X, const float* y, const double* w, double* ell,
                  double* prior, double* grad) {
  eval_f64(*m, X, y, w, ell, prior, grad);
}

void orc_mcmc_step(const orc_model* m, const float* X, const float* y, const float* w_prev,
                   const float* mom_prev, const float* grad_prev, float eps, int L, float* w_next,
                   float* mom_next, float* grad_cur, float* loss_values) {
  const int P = orc_num_params(m->d0, m->d1);
  std::vector<float> w(w_prev, w_prev + P), mom(mom_prev, mom_prev + P), g(grad_prev, grad_prev + P);
  std::vector<float> gn(P);
  for (int s = 0; s < L; ++s) {
    // ffma.h:408 (first launch: MOM_CORRECTION 2), 414-419 (middle), 420-426 (last: OUTPUT_LOSS)
    for (int p = 0; p < P; ++p) leapfrog_update(w[p], mom[p], g[p], eps, s == 0 ? 2 : 1);
    // A position that has left the finite numbers never comes back (inf + x is inf or NaN), its
    // log-prior is -inf or NaN, so the log accept ratio of this trajectory is -inf or NaN whatever
    // the remaining steps do: the transition rejects and counts as -inf for the adaptation.  The
    // remaining steps are skipped and every output is NaN.
    bool finite = true;
    for (int p = 0; p < P; ++p) finite = finite && std::isfinite(w[p]);
    if (!finite && g_cut_short) {
      const float nan = std::numeric_limits<float>::quiet_NaN();
      std::fill(w.begin(), w.end(), nan);
      std::fill(mom.begin(), mom.end(), nan);
      std::fill(g.begin(), g.end(), nan);
      std::fill(loss_values, loss_values + m->n + P, nan);
      break;
    }
    bool last = (s == L - 1);
    eval_f32(*m, X, y, w.data(), last ? loss_values : nullptr,
             last ? loss_values + m->n : nullptr, gn.data(), nullptr);
    g.swap(gn);
  }
  std::memcpy(w_next, w.data(), sizeof(float) * P);
  std::memcpy(mom_next, mom.data(), sizeof(float) * P);
  std::memcpy(grad_cur, g.data(), sizeof(float) * P);
}

float orc_log_acpt(int n_loss, int P, const float* prev_loss, const float* new_loss,
                   const float* prev_mom, const float* new_mom, const float* grad_cur, float eps) {
  // kernel_helpers.h:163-175: per-element FP32 terms; the sum itself is taken in double
  double acc = 0.0;
  for (int i = 0; i < n_loss; ++i) acc += (double)(new_loss[i] - prev_loss[i]);
  for (int i = 0; i < P; ++i) {
    float nm = fmaf(eps * 0.5f, grad_cur[i], new_mom[i]);  // final half kick
    float t = prev_mom[i] * prev_mom[i];
    t = fmaf(-nm, nm, t);
    acc += (double)(0.5f * t);
  }
  return (float)acc;
}

int orc_accept(float log_u, float log_acpt) { return log_u < log_acpt ? 1 : 0; }

float orc_adapt_eps(const orc_hmc* h, float eps, float log_acpt) {
  // main.h:267-276
  float la = (log_acpt == log_acpt) ? log_acpt : -std::numeric_limits<float>::infinity();
  float log_mean_acpt_r = la < 0.0f ? la : 0.0f;
  float dec_adj = -h->decrement / (1.0f + h->decrement);
  float inc_adj = h->increment;
  float adj = log_mean_acpt_r < (float)std::log((double)h->target_rate) ? dec_adj : inc_adj;
  return eps + eps * adj;
}

// main.h:117-293 from a given state: position w0 (NULL = zeros, main.h:166-183), step size eps0 and
// the index t0 of the first transition (which selects the RNG counters and the sample slots).
static int run_chain_impl(const orc_model* m, const orc_hmc* h, const float* X, const float* y,
                          const float* w0, float eps0, int t0, int n_trans, float* samples,
                          float* log_acpt_trace, int* accept_trace, float* eps_trace, float* final_w,
                          float* final_eps) {
  const int P = orc_num_params(m->d0, m->d1);
  const int n = m->n;
  std::vector<float> w(P, 0.0f), mom(P, 0.0f), g(P, 0.0f);
  std::vector<float> w_next(P), mom_next(P), g_cur(P), loss(n + P), prev_loss(n + P), prev_g(P),
      prev_w(P, 0.0f), mom0(P);
  if (w0) {
    std::copy(w0, w0 + P, w.begin());
    std::copy(w0, w0 + P, prev_w.begin());
  }
  float eps = eps0;
  // bootstrap main.h:191-202: with zero momentum and zero gradient the update is a no-op, so one
  // step evaluates the log-posterior rows and the gradient at the start
  orc_mcmc_step(m, X, y, w.data(), mom.data(), g.data(), eps, 1, w_next.data(), mom_next.data(),
                g_cur.data(), loss.data());
  prev_g = g_cur;
  prev_loss = loss;
  int n_acc = 0;
  for (int i = 0; i < n_trans; ++i) {
    const int step = t0 + i;
    orc_momentum(h->seed, h->chain_id, (uint32_t)step, P, mom0.data());  // main.h:207-216
    // main.h:218-223: trajectory from (prev_w, mom0, prev_g)
    orc_mcmc_step(m, X, y, prev_w.data(), mom0.data(), prev_g.data(), eps, h->leapfrog_steps,
                  w_next.data(), mom_next.data(), g_cur.data(), loss.data());
    float la = orc_log_acpt(n + P, P, prev_loss.data(), loss.data(), mom0.data(), mom_next.data(),
                            g_cur.data(), eps);  // main.h:228-232
    float lu = orc_log_uniform(h->seed, h->chain_id, (uint32_t)step);  // main.h:235-239
    int acc = orc_accept(lu, la);
    if (acc) {  // main.h:242-253
      prev_w = w_next;
      prev_g = g_cur;
      prev_loss = loss;
      ++n_acc;
    }  // else main.h:254-265: the saved state stays
    if (log_acpt_trace) log_acpt_trace[i] = la;
    if (accept_trace) accept_trace[i] = acc;
    if (step < h->adapt_steps) eps = orc_adapt_eps(h, eps, la);  // main.h:267-276
    if (eps_trace) eps_trace[i] = eps;
    if (step >= h->burn_in && step - h->burn_in < h->n_samples && samples)  // main.h:277-283
      std::memcpy(samples + (size_t)(step - h->burn_in) * P, prev_w.data(), sizeof(float) * P);
  }
  if (final_w) std::memcpy(final_w, prev_w.data(), sizeof(float) * P);
  if (final_eps) *final_eps = eps;
  return n_acc;
}

int orc_run_chain(const orc_model* m, const orc_hmc* h, const float* X, const float* y,
                  float* samples, float* log_acpt_trace, int* accept_trace, float* eps_trace,
                  float* final_w, float* final_eps) {
  return run_chain_impl(m, h, X, y, nullptr, h->eps0, 0, h->burn_in + h->n_samples, samples,
                        log_acpt_trace, accept_trace, eps_trace, final_w, final_eps);
}

int orc_run_chain_from(const orc_model* m, const orc_hmc* h, const float* X, const float* y,
                       const float* w0, float eps0, int t0, int n_trans, float* samples,
                       float* log_acpt_trace, int* accept_trace, float* eps_trace, float* final_w,
                       float* final_eps) {
  return run_chain_impl(m, h, X, y, w0, eps0, t0, n_trans, samples, log_acpt_trace, accept_trace,
                        eps_trace, final_w, final_eps);
}

void orc_final_loss(const orc_model* m, const float* X, const float* y, const float* samples,
                    int n_samples, double* loss1, double* loss2, double* full) {
  // main.h:85-112: running means of the data log-lik, the log-prior and their sum
  const int P = orc_num_params(m->d0, m->d1);
  std::vector<float> ell(m->n), prior(P);
  double l1 = 0, l2 = 0, fl = 0;
  for (int s = 0; s < n_samples; ++s) {
    eval_f32(*m, X, y, samples + (size_t)s * P, ell.data(), prior.data(), nullptr, nullptr);
    double s1 = 0, s2 = 0;
    for (int i = 0; i < m->n; ++i) s1 += (double)ell[i];
    for (int p = 0; p < P; ++p) s2 += (double)prior[p];
    // get_loss_values returns FP32 sums (kernel_helpers.h:205-214)
    double f1 = (double)(float)s1, f2 = (double)(float)s2, ds = (double)s;
    l1 = (l1 * ds + f1) / (ds + 1);
    l2 = (l2 * ds + f2) / (ds + 1);
    fl = (fl * ds + (f1 + f2)) / (ds + 1);
  }
  *loss1 = l1;
  *loss2 = l2;
  *full = fl;
}

double orc_bench_grad_evals(const orc_model* m, const float* X, const float* y, int threads,
                            double seconds, int* threads_used, long* evals_done) {
  const int P = orc_num_params(m->d0, m->d1);
  Consts c(*m);
  Layout L(m->d0, m->d1);
#ifdef _OPENMP
  if (threads <= 0) threads = omp_get_max_threads();
#else
  threads = 1;
#endif
  long total = 0;
  double elapsed = 0.0;
  // every thread integrates its own chain on the shared window: leapfrog update + gradient, which is
  // what one launch of the reference's step kernel does
#ifdef _OPENMP
#pragma omp parallel num_threads(threads) reduction(+ : total) reduction(max : elapsed)
#endif
  {
    int tid = 0;
#ifdef _OPENMP
    tid = omp_get_thread_num();
#endif
    std::vector<float> w(P), mom(P), g(P, 0.0f);
    std::vector<double> gacc(P);
    for (int p = 0; p < P; ++p) {
      w[p] = 0.1f * normal(12345u, (uint32_t)tid, ORC_STREAM_TEACHER, 0, (uint64_t)p);
      mom[p] = normal(12345u, (uint32_t)tid, ORC_STREAM_MOMENTUM, 0, (uint64_t)p);
    }
    const float eps = 1e-6f;
    auto t0 = std::chrono::steady_clock::now();
    long done = 0;
    double el = 0.0;
    do {
      for (int p = 0; p < P; ++p) leapfrog_update(w[p], mom[p], g[p], eps, 1);
      std::fill(gacc.begin(), gacc.end(), 0.0);
      eval_f32_range(*m, c, L, X, y, w.data(), 0, m->n, nullptr, gacc.data(), nullptr);
      for (int p = 0; p < P; ++p) {
        float lp, gp;
        prior_terms(c, w[p], &lp, &gp);
        g[p] = (float)((double)gp + gacc[p]);
      }
      ++done;
      el = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    } while (el < seconds);
    total += done;
    elapsed = el;
  }
  if (threads_used) *threads_used = threads;
  if (evals_done) *evals_done = total;
  return (double)total / elapsed;
}

}  // extern "C"
