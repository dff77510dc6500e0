// Thin C-ABI shim around the reference's own, dependency-free MX element math.
// It holds no algorithm of its own: the header is compiled from where it lies
// in the reference tree (include path given by the Makefile) and its functions
// are exported so that the oracle restatement can be checked against them and
// golden vectors can be written.  Output goes to oracle/_ref/ only.
#include "mxfp_quant.h"

extern "C" {

// MxFP4Quant(float max) constructor path (src/csrc/qtypes.cpp:69-77):
// returns the float scale produced by mx_get_shared_scale for a block maximum.
float ref_mx_shared_scale(float amax) {
  int shared_exp = (int)get_biased_exponent(amax);
  return mx_get_shared_scale(shared_exp, 8, 6.0f);
}

int ref_biased_exponent(float v) {
  return get_biased_exponent(v);
}

// quantize_elemwise as MxFP4Quant::quantize calls it (qtypes.cpp:91-98).
float ref_e2m1_round(float scaled_in) {
  return quantize_elemwise(scaled_in, 3, 2, 6.0f, rd_even, true, true);
}

void ref_e2m1_round_n(const float* in, float* out, long n) {
  for (long i = 0; i < n; i++)
    out[i] = quantize_elemwise(in[i], 3, 2, 6.0f, rd_even, true, true);
}

void ref_mx_shared_scale_n(const float* amax, float* out, long n) {
  for (long i = 0; i < n; i++)
    out[i] = ref_mx_shared_scale(amax[i]);
}
}
