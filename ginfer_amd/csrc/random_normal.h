// A counter-based generator of normal numbers, written once for the host and for the device: element i of a tensor
// with a 64-bit key is a pure function of (key, i), and that function uses only operations that round the same
// way everywhere (32-bit add, multiply, divide and square root, each rounded once; integer and bit operations), in
// one fixed order, with no contraction into fused multiply-adds.  So a model whose weights are drawn on the GPU holds
// bit for bit the numbers of the model folder that the host writes for the same seed.  The reference has no
// random-weights mode (it loads checkpoints only, ginfer/model/qwen2.cc:28-49).
//
// normal = sqrt(-2 ln u1) * cos(2 pi u2), u1 in (0, 1] and u2 in [0, 1) from 24 bits each of one 64-bit hash;
// the logarithm and the cosine are short polynomials of our own (the libraries' differ between host and device in the
// last bit): ln through (m - 1) / (m + 1) of the mantissa, the cosine by quadrant from 2 bits of u2 and a Taylor
// polynomial over [0, pi / 2).  Both are exact to a few units of the last place, far below what a weight's
// distribution can show.
//
// Every source that includes this file is compiled with -ffp-contract=off.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define GA_HOST_DEVICE __host__ __device__
#else
#define GA_HOST_DEVICE
#endif

GA_HOST_DEVICE inline uint64_t ga_mix64(uint64_t z) {          // the finaliser of splitmix64
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

GA_HOST_DEVICE inline float ga_bits_to_float(uint32_t b) {
  float f;
  __builtin_memcpy(&f, &b, 4);
  return f;
}

GA_HOST_DEVICE inline uint32_t ga_float_to_bits(float f) {
  uint32_t b;
  __builtin_memcpy(&b, &f, 4);
  return b;
}

// A standard normal number for element i of the tensor with this key.
GA_HOST_DEVICE inline float ga_normal_from_counter(uint64_t key, uint64_t i) {
  const uint64_t h = ga_mix64(ga_mix64(key) ^ (i * 0xD1342543DE82EF95ull));
  // u1 = n1 / 2^24 with n1 in [1, 2^24]; ln u1 = (exponent of n1 - 24) ln 2 + ln(mantissa in [1, 2))
  const uint32_t n1 = (uint32_t)(h >> 40) + 1u;
  const uint32_t bits = ga_float_to_bits((float)n1);             // exact: n1 has at most 25 bits, and 2^24 is a power of two
  const float e = (float)((int)(bits >> 23) - 127 - 24);
  const float m = ga_bits_to_float((bits & 0x007FFFFFu) | 0x3F800000u);
  const float s = (m - 1.0f) / (m + 1.0f);                       // in [0, 1/3]
  const float s2 = s * s;
  float p = 1.0f / 13.0f;
  p = p * s2 + 1.0f / 11.0f;
  p = p * s2 + 1.0f / 9.0f;
  p = p * s2 + 1.0f / 7.0f;
  p = p * s2 + 1.0f / 5.0f;
  p = p * s2 + 1.0f / 3.0f;
  p = p * s2 + 1.0f;
  const float ln_u1 = e * 0.693147180559945f + 2.0f * s * p;      // <= 0
  const float r = __builtin_sqrtf(-2.0f * ln_u1);
  // u2 = n2 / 2^24: its first 2 bits name the quadrant, the other 22 the angle in it
  const uint32_t n2 = (uint32_t)(h >> 8) & 0x00FFFFFFu;
  const uint32_t quadrant = n2 >> 22;
  const float t = (float)(n2 & 0x003FFFFFu) * (1.5707963267948966f / 4194304.0f);    // in [0, pi / 2)
  const float t2 = t * t;
  float c = 1.0f / 479001600.0f;
  c = c * t2 - 1.0f / 3628800.0f;
  c = c * t2 + 1.0f / 40320.0f;
  c = c * t2 - 1.0f / 720.0f;
  c = c * t2 + 1.0f / 24.0f;
  c = c * t2 - 0.5f;
  c = c * t2 + 1.0f;
  float sn = 1.0f / 6227020800.0f;
  sn = sn * t2 - 1.0f / 39916800.0f;
  sn = sn * t2 + 1.0f / 362880.0f;
  sn = sn * t2 - 1.0f / 5040.0f;
  sn = sn * t2 + 1.0f / 120.0f;
  sn = sn * t2 - 1.0f / 6.0f;
  sn = sn * t2 + 1.0f;
  sn = sn * t;
  const float cosine = quadrant == 0 ? c : quadrant == 1 ? -sn : quadrant == 2 ? -c : sn;
  return r * cosine;
}

// mean + std * normal, rounded once to 32-bit
GA_HOST_DEVICE inline float ga_weight_from_counter(uint64_t key, uint64_t i, float mean, float std) {
  const float z = ga_normal_from_counter(key, i) * std;
  return z + mean;
}
