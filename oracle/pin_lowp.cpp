// TEST INFRASTRUCTURE — exhaustive pinning of lowp.hpp.
//   part 1 (needs oracle/_ref): kRefHost narrowing of ALL 2^32 f32 bit patterns and widening of
//           all narrow codes, compared bit-for-bit with the compiled reference classes.
//   part 2 (always): kIeee f8E4M3FN narrowing of all 2^32 patterns compared with a nearest-value
//           search over the table of the 253 finite f8 values (ties to even code), an algorithm
//           that shares nothing with narrow_f32; kIeee f16 against the x86 F16C instruction.
// Prints one summary line per check; exit status 0 only if every count is 0.
#include "lowp.hpp"
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <immintrin.h>
#include <vector>

#ifdef WITH_REF
extern "C" {
uint8_t ref_f32_to_f8e4m3fn(float);
float ref_f8e4m3fn_to_f32(uint8_t);
uint16_t ref_f32_to_f16(float);
float ref_f16_to_f32(uint16_t);
uint16_t ref_f32_to_bf16(float);
float ref_bf16_to_f32(uint16_t);
}
#endif

using namespace orc;

static uint8_t f8_nearest_search(float x, const std::vector<double> &vals) {
  // vals[c] = value of positive code c (0..0x7E), strictly increasing.
  const uint32_t u = f32_bits(x);
  const uint8_t sign = uint8_t((u >> 31) << 7);
  if (std::isnan(x))
    return 0x7F;
  const double a = std::fabs(double(x));
  if (a >= vals[0x7E])
    return sign | 0x7E;
  int lo = 0, hi = 0x7E; // vals[lo] <= a < vals[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) / 2;
    if (vals[mid] <= a)
      lo = mid;
    else
      hi = mid;
  }
  const double dl = a - vals[lo], dh = vals[hi] - a;
  int code = dl < dh ? lo : (dh < dl ? hi : ((lo & 1) ? hi : lo));
  return sign | uint8_t(code);
}

int main() {
  long long bad_total = 0;
#ifdef WITH_REF
  {
    long long bad8 = 0, bad16 = 0, badbf = 0;
#pragma omp parallel for schedule(static) reduction(+ : bad8, bad16, badbf)
    for (long long i = 0; i < (1LL << 32); ++i) {
      const float x = bits_f32(uint32_t(i));
      bad8 += f32_to_f8e4m3fn(x, kRefHost) != ref_f32_to_f8e4m3fn(x);
      bad16 += f32_to_f16(x, kRefHost) != ref_f32_to_f16(x);
      badbf += f32_to_bf16(x, kRefHost) != ref_f32_to_bf16(x);
    }
    std::printf("refhost narrow vs reference, all 2^32 f32: f8 mismatches=%lld f16=%lld bf16=%lld\n",
                bad8, bad16, badbf);
    long long badw = 0;
    for (int c = 0; c < 256; ++c)
      badw += f32_bits(f8e4m3fn_to_f32(uint8_t(c))) != f32_bits(ref_f8e4m3fn_to_f32(uint8_t(c)));
    for (int c = 0; c < 65536; ++c) {
      badw += f32_bits(f16_to_f32(uint16_t(c))) != f32_bits(ref_f16_to_f32(uint16_t(c)));
      badw += f32_bits(bf16_to_f32(uint16_t(c))) != f32_bits(ref_bf16_to_f32(uint16_t(c)));
    }
    std::printf("widen vs reference, all codes: mismatches=%lld\n", badw);
    bad_total += bad8 + bad16 + badbf + badw;
  }
#endif
  {
    std::vector<double> vals(0x7F);
    for (int c = 0; c < 0x7F; ++c) {
      const int e = c >> 3, m = c & 7;
      vals[c] = e == 0 ? std::ldexp(double(m), -9) : std::ldexp(1.0 + m / 8.0, e - 7);
    }
    long long bad8 = 0, bad16 = 0, diff_modes = 0;
#pragma omp parallel for schedule(static) reduction(+ : bad8, bad16, diff_modes)
    for (long long i = 0; i < (1LL << 32); ++i) {
      const float x = bits_f32(uint32_t(i));
      const uint8_t got = f32_to_f8e4m3fn(x, kIeee);
      bad8 += got != f8_nearest_search(x, vals);
      diff_modes += got != f32_to_f8e4m3fn(x, kRefHost);
      if (!std::isnan(x)) {
        const uint16_t hw = uint16_t(_cvtss_sh(x, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
        bad16 += f32_to_f16(x, kIeee) != hw;
      }
    }
    std::printf("ieee narrow, all 2^32 f32: f8 vs nearest-search mismatches=%lld, f16 vs F16C=%lld "
                "(f8 ieee!=refhost on %lld patterns)\n",
                bad8, bad16, diff_modes);
    bad_total += bad8 + bad16;
  }
  return bad_total == 0 ? 0 : 1;
}
