// Test infrastructure: the reference AQLM kernel and launcher
// (src/quantAQLM-hip/main.cu, HeCBench tree) behind C entry points.
#define main hecbench_quantaqlm_main
#include "main.cu"
#undef main

// The reference launcher: synchronises, times itself and prints one line.
extern "C" __attribute__((visibility("default"))) void ref_code1x16_matvec(const void* A, const void* B, void* C, const void* codebook,
                                    int prob_m, int prob_k, const int sizes[4], int codebook_stride) {
  code1x16_matvec(A, B, C, codebook, prob_m, prob_k, make_int4(sizes[0], sizes[1], sizes[2], sizes[3]),
                  codebook_stride);
}

// The reference kernel with the reference launch shape, without the host-side
// synchronisation and printing (for event timing).
extern "C" __attribute__((visibility("default"))) void ref_code1x16_launch(const void* A, const void* B, void* C, const void* codebook,
                                    int prob_m, int prob_k, const int sizes[4], int codebook_stride,
                                    void* stream) {
  int sms;
  hipDeviceGetAttribute(&sms, hipDeviceAttributeMultiprocessorCount, 0);
  int waves = 0, thread_m;
  do {
    waves++;
    thread_m = ceildiv(prob_m, waves * sms);
  } while (thread_m > THREAD_M);
  int blocks = ceildiv(prob_m, thread_m);
  int threads = 64 * thread_m;
  Code1x16MatVec<64><<<blocks, threads, sizeof(int4) * 64 * F, (hipStream_t)stream>>>(
      (const int4*)A, (const int4*)B, (int4*)C, (const int4*)codebook, prob_m, prob_k,
      make_int4(sizes[0], sizes[1], sizes[2], sizes[3]), codebook_stride);
}
