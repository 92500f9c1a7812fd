// Test infrastructure: the reference LUT-GEMM kernels (src/lut-gemm-hip,
// HeCBench tree) and the host-side fixture loops of its main.cu behind C entry
// points.  The BLAS check of the reference (tests.h) is never instantiated.
#define main hecbench_lutgemm_main
#include "main.cu"
#undef main
#include "kernels.cu"
#include "nQWeight_fp16.cu"

// matmul() of the reference on caller-owned device buffers.
extern "C" __attribute__((visibility("default"))) void ref_lut_matmul(void* out_f16, void* in_f16, unsigned* bW, void* alpha_f16,
                               void* qbias_f16, int K, int N, int nb, int num_groups) {
  nQWeight_fp16* w = new nQWeight_fp16();  // deliberately leaked: its destructor frees the buffers
  w->bWeight = bW;
  w->alpha = alpha_f16;
  w->q_bias = qbias_f16;
  w->num_groups = num_groups;
  w->group_size = K / num_groups;
  w->mSize = N;
  w->kSize = K;
  w->nb = nb;
  w->is_row_wise_quantize = false;
  matmul(out_f16, in_f16, *w, 1);
}

// Host fixture of the reference at a small fixed shape: random bit planes,
// alphas, biases (srand(123) streams of tests.h) and the dense weights its own
// host loop dequantizeFrom_qW() derives from them.
template <int N, int K, int NB>
static void fixture(float* qW, unsigned* bW, float* alpha, float* q_bias, float* weight, float* input) {
  typedef int3_col_wise_matmul_fp16<1, N, K, NB, 128> Fx;
  Fx* f = (Fx*)calloc(1, sizeof(Fx));
  f->qW = qW; f->bW = bW; f->alpha = alpha; f->q_bias = q_bias; f->weight = weight; f->input = input;
  f->makeRandomInput();
  f->makeRandomWeight();
  f->makeRandomAlpha();
  f->dequantizeFrom_qW();
  free(f);
}
extern "C" __attribute__((visibility("default"))) void ref_lut_fixture_256x256x3(float* qW, unsigned* bW, float* alpha, float* q_bias,
                                          float* weight, float* input) {
  fixture<256, 256, 3>(qW, bW, alpha, q_bias, weight, input);
}
extern "C" __attribute__((visibility("default"))) void ref_lut_fixture_128x384x4(float* qW, unsigned* bW, float* alpha, float* q_bias,
                                          float* weight, float* input) {
  fixture<128, 384, 4>(qW, bW, alpha, q_bias, weight, input);
}
