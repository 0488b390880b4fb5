// Reproducible synthetic data for benchmarks and parity runs (host side).
//
// Counter-based: element i of (seed, stream) is a pure function of
// (seed, stream, i), so buffers can be generated in parallel, in pieces, and
// identically on any machine.  The reference harness fills buffers with
// closed-form patterns (test/perf/host_api/test_allreduce.cpp:20-32); seeded
// random data has no counterpart there.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>

#include "flagcx_amd/fx_synth.h"

namespace {

inline uint64_t mix64(uint64_t z) {  // SplitMix64 output function
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

inline uint64_t streamKey(uint64_t seed, uint64_t stream) {
  return mix64(mix64(seed + 0x9E3779B97F4A7C15ull) ^ (stream * 0xD1B54A32D192ED03ull + 0x8CB92BA72F3D8DD7ull));
}

inline uint64_t draw(uint64_t key, uint64_t j) { return mix64(key + (j + 1) * 0x9E3779B97F4A7C15ull); }

inline uint16_t toBf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// fp32 -> binary16 by scaling into the target grid and rounding with the
// FPU's own round-to-nearest-even.
inline uint16_t toF16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  float a = std::fabs(f);
  if (std::isnan(f)) return (uint16_t)(sign | 0x7e00u);
  if (a >= 65520.0f) return (uint16_t)(sign | 0x7c00u);
  if (a < 6.103515625e-05f) {  // subnormal half: units of 2^-24
    float q = std::nearbyintf(a * 16777216.0f);
    return (uint16_t)(sign | (uint16_t)q);
  }
  int e;
  float m = std::frexp(a, &e);                      // a = m * 2^e, m in [0.5, 1)
  float q = std::nearbyintf(m * 2048.0f);           // 11 significant bits
  if (q == 2048.0f) {
    q = 1024.0f;
    e++;
  }
  uint32_t bits = ((uint32_t)(e + 14) << 10) + ((uint32_t)q - 1024u);
  return (uint16_t)(sign | bits);
}

struct Job {
  void *dst;
  size_t n;
  int dtype, dist;
  double a, b;
  uint64_t key;
};

inline void store(const Job &jb, size_t i, double v) {
  switch (jb.dtype) {
    case flagcxFloat32: ((float *)jb.dst)[i] = (float)v; break;
    case flagcxFloat64: ((double *)jb.dst)[i] = v; break;
    case flagcxBfloat16: ((uint16_t *)jb.dst)[i] = toBf16((float)v); break;
    case flagcxFloat16: ((uint16_t *)jb.dst)[i] = toF16((float)v); break;
    case flagcxInt32: ((int32_t *)jb.dst)[i] = (int32_t)(int64_t)v; break;
    default: break;
  }
}

// Pairs [p0, p1): pair p yields elements 2p and 2p+1 from one 64-bit draw.
void fillPairs(const Job &jb, size_t p0, size_t p1) {
  const double kTwoPi = 6.283185307179586476925286766559;
  for (size_t p = p0; p < p1; p++) {
    const uint64_t r = draw(jb.key, p);
    const uint32_t hi = (uint32_t)(r >> 32), lo = (uint32_t)r;
    double v0, v1;
    if (jb.dist == FX_SYNTH_NORMAL) {
      const double u1 = ((double)hi + 0.5) * (1.0 / 4294967296.0);
      const double u2 = ((double)lo + 0.5) * (1.0 / 4294967296.0);
      const double rad = std::sqrt(-2.0 * std::log(u1));
      v0 = jb.a + jb.b * rad * std::cos(kTwoPi * u2);
      v1 = jb.a + jb.b * rad * std::sin(kTwoPi * u2);
    } else if (jb.dist == FX_SYNTH_UNIFORM_INT) {
      const uint64_t range = (uint64_t)((int64_t)jb.b - (int64_t)jb.a) + 1ull;
      v0 = (double)((int64_t)jb.a + (int64_t)(((uint64_t)hi * range) >> 32));
      v1 = (double)((int64_t)jb.a + (int64_t)(((uint64_t)lo * range) >> 32));
    } else {
      v0 = jb.a + (jb.b - jb.a) * ((double)hi * (1.0 / 4294967296.0));
      v1 = jb.a + (jb.b - jb.a) * ((double)lo * (1.0 / 4294967296.0));
    }
    store(jb, 2 * p, v0);
    if (2 * p + 1 < jb.n) store(jb, 2 * p + 1, v1);
  }
}

}  // namespace

extern "C" {
#pragma GCC visibility push(default)

int fx_synth_fill(void *dst, size_t n, int dtype, int dist, double a, double b, uint64_t seed, uint64_t stream,
                  int nthreads) {
  if (n == 0) return flagcxSuccess;
  if (!dst) return flagcxInvalidArgument;
  if (dtype != flagcxFloat32 && dtype != flagcxFloat64 && dtype != flagcxBfloat16 && dtype != flagcxFloat16 &&
      dtype != flagcxInt32)
    return flagcxNotSupported;
  if (dist < FX_SYNTH_UNIFORM || dist > FX_SYNTH_UNIFORM_INT) return flagcxInvalidArgument;
  if (dist == FX_SYNTH_UNIFORM_INT && b < a) return flagcxInvalidArgument;
  Job jb{dst, n, dtype, dist, a, b, streamKey(seed, stream)};
  const size_t pairs = (n + 1) / 2;
  int nt = nthreads < 1 ? 1 : nthreads;
  if ((size_t)nt > pairs / 4096 + 1) nt = (int)(pairs / 4096 + 1);
  if (nt == 1) {
    fillPairs(jb, 0, pairs);
    return flagcxSuccess;
  }
  std::vector<std::thread> th;
  for (int t = 0; t < nt; t++) {
    size_t p0 = pairs * (size_t)t / nt, p1 = pairs * (size_t)(t + 1) / nt;
    th.emplace_back(fillPairs, std::cref(jb), p0, p1);
  }
  for (auto &t : th) t.join();
  return flagcxSuccess;
}

#pragma GCC visibility pop
}
