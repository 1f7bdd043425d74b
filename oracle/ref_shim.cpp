// TEST INFRASTRUCTURE — C entry points over the REFERENCE's own number classes.
// Compiled only where /root/reference is mounted, together with the reference's
// DataTypes.cpp taken from where it lies (see Makefile target `_ref`); the output
// goes to oracle/_ref/ and is never committed.  Used to validate lowp.hpp and to
// mint the golden tables under tests/golden/.
#include "mlir-executor/Runtime/Backend/Common/DataTypes.h"
#include <cmath>
#include <cstdint>

extern "C" {
uint8_t ref_f32_to_f8e4m3fn(float x) { return uint8_t(mtrt::F8E4M3FN(x).getRawBits()); }
float ref_f8e4m3fn_to_f32(uint8_t b) { return float(mtrt::F8E4M3FN::fromRawBits(int8_t(b))); }
uint16_t ref_f32_to_f16(float x) { return uint16_t(mtrt::Float16(x).getRawBits()); }
float ref_f16_to_f32(uint16_t b) { return float(mtrt::Float16::fromRawBits(int16_t(b))); }
uint16_t ref_f32_to_bf16(float x) { return uint16_t(mtrt::BFloat16(x).getRawBits()); }
float ref_bf16_to_f32(uint16_t b) { return float(mtrt::BFloat16::fromRawBits(int16_t(b))); }
int8_t ref_int4_from_int(int32_t v) { return int8_t(int(mtrt::Int4(int(v)))); }
uint8_t ref_int4_raw_from_int(int32_t v) { return uint8_t(mtrt::Int4(int(v)).getRawBits()); }
int8_t ref_int4_from_raw(uint8_t nibble) { return int8_t(int(mtrt::Int4::fromRawBits(int8_t(nibble)))); }
// _fptosi_f32_i4 (CoreModule.cpp:72-98): Int4(std::trunc(x))
int8_t ref_fptosi_f32_i4(float x) { return int8_t(int(mtrt::Int4(int(std::trunc(x))))); }

void ref_f32_to_f8e4m3fn_bulk(const float *x, uint8_t *o, int64_t n) {
  for (int64_t i = 0; i < n; ++i) o[i] = ref_f32_to_f8e4m3fn(x[i]);
}
void ref_f32_to_f16_bulk(const float *x, uint16_t *o, int64_t n) {
  for (int64_t i = 0; i < n; ++i) o[i] = ref_f32_to_f16(x[i]);
}
void ref_f32_to_bf16_bulk(const float *x, uint16_t *o, int64_t n) {
  for (int64_t i = 0; i < n; ++i) o[i] = ref_f32_to_bf16(x[i]);
}
}
