// Counter-based RNG shared by host and device code of the library.
//
// Replaces the reference's per-transition thrust::minstd_rand + discard momentum sampler
// (include/mcmc/main.h:207-216) and its host std::default_random_engine accept draw
// (include/mcmc/main.h:235-239) with one generator that is a pure function of
// (seed, chain, stream, transition, index): Philox4x32-10 -> 32-bit word -> u = (k + 0.5) / 2^32 ->
// normal quantile (Wichura AS 241, PPND16) or log u.  log and sqrt are built from + - * / and fma
// only, with contraction disabled, so host and device produce identical bits.
#pragma once

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define BNN_HD __host__ __device__ inline
#else
#define BNN_HD inline
#endif

namespace bnn {

enum Stream : uint32_t {
  STREAM_X = 0,         // synthetic features
  STREAM_TEACHER = 1,   // synthetic teacher weights
  STREAM_NOISE = 2,     // synthetic target noise
  STREAM_MOMENTUM = 3,  // HMC momentum resampling
  STREAM_ACCEPT = 4     // Metropolis uniform
};

struct u32x4 {
  uint32_t v[4];
};

BNN_HD u32x4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                           uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  u32x4 o;
  o.v[0] = c0;
  o.v[1] = c1;
  o.v[2] = c2;
  o.v[3] = c3;
  return o;
}

BNN_HD double bits_to_double(uint64_t b) {
  double d;
  memcpy(&d, &b, 8);
  return d;
}
BNN_HD uint64_t double_to_bits(double d) {
  uint64_t b;
  memcpy(&b, &d, 8);
  return b;
}

// The three functions below must round identically on host and device: no contraction.
#if defined(__clang__)
#pragma clang fp contract(off)
#endif

// natural log of a positive normal double: x = 2^k (1 + f), s = f / (2 + f), odd series in s
BNN_HD double det_log(double x) {
#if defined(__clang__)
#pragma clang fp contract(off)
#endif
  const double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10,
               Lg1 = 6.666666666666735130e-01, Lg2 = 3.999999999940941908e-01,
               Lg3 = 2.857142874366239149e-01, Lg4 = 2.222219843214978396e-01,
               Lg5 = 1.818357216161805012e-01, Lg6 = 1.531383769920937332e-01,
               Lg7 = 1.479819860511658591e-01;
  uint64_t bits = double_to_bits(x);
  uint32_t hx = (uint32_t)(bits >> 32);
  const uint32_t lx = (uint32_t)bits;
  int k = (int)(hx >> 20) - 1023;
  hx &= 0x000fffffu;
  const uint32_t i = (hx + 0x95f64u) & 0x100000u;
  hx |= (i ^ 0x3ff00000u);
  k += (int)(i >> 20);
  const double m = bits_to_double(((uint64_t)hx << 32) | lx);
  const double f = m - 1.0;
  const double hfsq = 0.5 * f * f;
  const double s = f / (2.0 + f);
  const double z = s * s;
  const double w = z * z;
  const double t1 = w * (Lg2 + w * (Lg4 + w * Lg6));
  const double t2 = z * (Lg1 + w * (Lg3 + w * (Lg5 + w * Lg7)));
  const double R = t2 + t1;
  const double dk = (double)k;
  return s * (hfsq + R) + dk * ln2_lo - hfsq + f + dk * ln2_hi;
}

// square root of a positive normal double: bit-level seed, Newton steps on 1/sqrt(x), one
// fma-corrected step on sqrt(x); about one ulp
BNN_HD double det_sqrt(double x) {
#if defined(__clang__)
#pragma clang fp contract(off)
#endif
  double r = bits_to_double(0x5fe6eb50c7b537a9ull - (double_to_bits(x) >> 1));
  for (int it = 0; it < 5; ++it) r = r * (1.5 - 0.5 * x * r * r);
  const double s = x * r;
  return s + 0.5 * r * __builtin_fma(-s, s, x);
}

// normal quantile, Wichura's algorithm AS 241 (PPND16)
BNN_HD double ppnd16(double p) {
#if defined(__clang__)
#pragma clang fp contract(off)
#endif
  const double q = p - 0.5;
  if (__builtin_fabs(q) <= 0.425) {
    const double r = 0.180625 - q * q;
    const double num =
        (((((((2.5090809287301226727e+3 * r + 3.3430575583588128105e+4) * r +
              6.7265770927008700853e+4) * r + 4.5921953931549871457e+4) * r +
            1.3731693765509461125e+4) * r + 1.9715909503065514427e+3) * r +
          1.3314166789178437745e+2) * r + 3.3871328727963666080e0);
    const double den =
        (((((((5.2264952788528545610e+3 * r + 2.8729085735721942674e+4) * r +
              3.9307895800092710610e+4) * r + 2.1213794301586595867e+4) * r +
            5.3941960214247511077e+3) * r + 6.8718700749205790830e+2) * r +
          4.2313330701600911252e+1) * r + 1.0);
    return q * num / den;
  }
  double r = q < 0.0 ? p : 1.0 - p;
  r = det_sqrt(-det_log(r));
  double val;
  if (r <= 5.0) {
    r -= 1.6;
    const double num =
        (((((((7.74545014278341407640e-4 * r + 2.27238449892691845833e-2) * r +
              2.41780725177450611770e-1) * r + 1.27045825245236838258e0) * r +
            3.64784832476320460504e0) * r + 5.76949722146069140550e0) * r +
          4.63033784615654529590e0) * r + 1.42343711074968357734e0);
    const double den =
        (((((((1.05075007164441684324e-9 * r + 5.47593808499534494600e-4) * r +
              1.51986665636164571966e-2) * r + 1.48103976427480074590e-1) * r +
            6.89767334985100004550e-1) * r + 1.67638483018380384940e0) * r +
          2.05319162663775882187e0) * r + 1.0);
    val = num / den;
  } else {
    r -= 5.0;
    const double num =
        (((((((2.01033439929228813265e-7 * r + 2.71155556874348757815e-5) * r +
              1.24266094738807843860e-3) * r + 2.65321895265761230930e-2) * r +
            2.96560571828504891230e-1) * r + 1.78482653991729133580e0) * r +
          5.46378491116411436990e0) * r + 6.65790464350110377720e0);
    const double den =
        (((((((2.04426310338993978564e-15 * r + 1.42151175831644588870e-7) * r +
              1.84631831751005468180e-5) * r + 7.86869131145613259100e-4) * r +
            1.48753612908506148525e-2) * r + 1.36929880922735805310e-1) * r +
          5.99832206555887937690e-1) * r + 1.0);
    val = num / den;
  }
  return q < 0.0 ? -val : val;
}

BNN_HD double u01(uint32_t k) {
#if defined(__clang__)
#pragma clang fp contract(off)
#endif
  return ((double)k + 0.5) * (1.0 / 4294967296.0);
}

// word `index` of stream (stream, t) under key (seed, id): word index % 4 of the Philox block with
// counter (index / 4, t, stream, index >> 34)
BNN_HD uint32_t rng_word(uint32_t seed, uint32_t id, uint32_t stream, uint32_t t, uint64_t index) {
  const uint64_t blk = index >> 2;
  const u32x4 o = philox4x32_10((uint32_t)blk, t, stream, (uint32_t)(blk >> 32), seed, id);
  const uint32_t sel = (uint32_t)index & 3u;
  return sel == 0 ? o.v[0] : (sel == 1 ? o.v[1] : (sel == 2 ? o.v[2] : o.v[3]));
}

BNN_HD float word_to_normal(uint32_t k) { return (float)ppnd16(u01(k)); }

BNN_HD float rng_normal(uint32_t seed, uint32_t id, uint32_t stream, uint32_t t, uint64_t index) {
  return word_to_normal(rng_word(seed, id, stream, t, index));
}

BNN_HD float rng_log_uniform(uint32_t seed, uint32_t id, uint32_t t) {
  return (float)det_log(u01(rng_word(seed, id, STREAM_ACCEPT, t, 0)));
}

}  // namespace bnn
