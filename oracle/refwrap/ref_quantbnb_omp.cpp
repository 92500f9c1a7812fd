// Test infrastructure: exposes the reference host quantiser of
// src/quantBnB-omp/main.cpp (HeCBench tree) as a C entry point.  The reference
// source is compiled where it lies; nothing of it is copied here.
#define main hecbench_quantbnb_omp_main
#include "main.cpp"
#undef main

extern "C" __attribute__((visibility("default"))) uint8_t ref_dquantize(float x) { return dQuantize<0>(code, 0.f, x); }
extern "C" __attribute__((visibility("default"))) void ref_dquantize_n(const float* A, uint8_t* out, long n) {
  for (long i = 0; i < n; ++i) out[i] = dQuantize<0>(code, 0.f, A[i]);
}
extern "C" __attribute__((visibility("default"))) const float* ref_code_table(void) { return code; }
// The reference program itself (argv: <number of elements> <repeat>), host-only.
extern "C" __attribute__((visibility("default"))) int ref_quantbnb_omp_main(int argc, char** argv) { return hecbench_quantbnb_omp_main(argc, argv); }
