// host_math.cpp -- g++ build of the kernels' scalar arithmetic (arcq_math.h) so that CPU tests
// can sweep it exhaustively.  Not part of the shipped GPU path; exports array wrappers only.
#include <stdint.h>

#include "arcq_math.h"

extern "C" {

void arcq_host_ue4m3(const float *t, int n, float *val, uint8_t *byte) {
  for (int i = 0; i < n; ++i) byte[i] = (uint8_t)arcq::ue4m3_scale(t[i], &val[i]);
}

void arcq_host_ue8m0(const float *t, int n, float *val, uint8_t *byte) {
  for (int i = 0; i < n; ++i) byte[i] = (uint8_t)arcq::ue8m0_scale(t[i], &val[i]);
}

void arcq_host_e2m1(const float *x, int n, float *val, uint8_t *code) {
  for (int i = 0; i < n; ++i) {
    code[i] = (uint8_t)arcq::e2m1_code(x[i]);
    val[i] = arcq::e2m1_value(code[i]);
  }
}

void arcq_host_scale_values(const uint8_t *b, int n, int fmt, float *val) {
  for (int i = 0; i < n; ++i) val[i] = fmt == 0 ? arcq::nvfp4_scale_value(b[i]) : arcq::mxfp4_scale_value(b[i]);
}

}  // extern "C"
