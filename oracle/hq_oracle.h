/*
 * hq_oracle.h — CPU restatement of the HeCBench weight-only quantized-inference
 * kernels (quant3MatMul, lut-gemm, quantAQLM, quantBnB) plus the NF4/FP4
 * blockwise dequant.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the
 * smoke check and the benchmark's cpu_baseline leg may call it, and only as the
 * checker / reported baseline.  The shipped library (libhq.so) never links or
 * calls anything declared here.
 *
 * Every function cites the reference lines (relative to the HeCBench tree) whose
 * arithmetic it restates.  Functions marked PARITY UNPINNED have no counterpart
 * or no check in the reference; they are pinned only by closed forms and brute
 * force in tests/.
 *
 *   q3 unpack / fp32 matvec : pinned by the reference known answer -49152.f
 *                             (src/quant3MatMul-hip/main.cu:36-53,84-105)
 *   q3 fp16 ("faster")      : pinned by the same known answer
 *   q3 batched GEMM         : PARITY UNPINNED (no batched kernel in the reference)
 *   NF4 / FP4 dequant       : PARITY UNPINNED (no NF4/FP4 code in the reference)
 *   dynamic 8-bit quantize  : pinned by the reference host function compiled
 *                             into oracle/_ref (src/quantBnB-omp/main.cpp)
 *   LUT-GEMM                : bit packing + dequant formula pinned by the
 *                             reference host loops compiled into oracle/_ref
 *                             (src/lut-gemm-hip/main.cu:118-146)
 *   AQLM                    : the reference checks nothing; pinned by a golden output of the
 *                             reference kernel itself (tests/golden/aqlm_reference_kernel.npz,
 *                             bit-identical in mode 1) and by closed forms
 *   int8 activation quant   : pinned by the reference host loops compiled into
 *                             oracle/_ref (src/quantVLLM-cuda/reference.h)
 *   4-bit blockwise quantize: PARITY UNPINNED (no counterpart in the reference)
 *   gemv fp16 / int8 / int4 : the reference's own statement of the result is its device-side
 *                             checker (src/gemv-hip/gemv.cu:134-190); pinned by closed forms and,
 *                             on a GPU, by the reference kernels compiled into oracle/_ref
 *   mxfp4 quantise-dequantise: pinned by the reference's verification table
 *                             (src/mxfp4-cuda/verify.h) and, on a GPU, by the reference kernel
 *                             compiled into oracle/_ref
 */
#ifndef HQ_ORACLE_H
#define HQ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- IEEE binary16 helpers (round-to-nearest-even, subnormals kept) ---- */
uint16_t hqo_f32_to_f16(float f);
float    hqo_f16_to_f32(uint16_t h);
uint16_t hqo_f64_to_f16(double d);
/* fp16 fused multiply-add a*b+c with a single rounding (device __hfma). */
uint16_t hqo_hfma(uint16_t a, uint16_t b, uint16_t c);
uint16_t hqo_hadd(uint16_t a, uint16_t b);
uint16_t hqo_hmul(uint16_t a, uint16_t b);

/* ---- GPTQ 3-bit (quant3MatMul) ---------------------------------------- */
/* codes[k*N+n] in 0..7  <->  mat[(3*(k/32)+j)*N + n], j=0..2.
 * Layout derived from src/quant3MatMul-hip/kernels.h:42-86. */
void hqo_q3_pack(const uint8_t* codes, int K, int N, int32_t* mat);
void hqo_q3_unpack(const int32_t* mat, int K, int N, uint8_t* codes);

/* Threads for the loops over independent outputs of hqo_dequant_4bit, hqo_lut_gemv_f64,
 * hqo_aqlm_matvec and hqo_q3_gemm (1 = serial, the default; results do not depend on it): the
 * benchmark times the restatements serially and again over the host cores. */
void hqo_set_threads(int n);
int hqo_max_threads(void);

/* fp32 kernel, src/quant3MatMul-hip/kernels.h:12-90: per 256-row block
 * res += (scale*float(q) - zero) * x  sequentially in fp32 (no FMA
 * contraction), block partials added to mul[] in block order.  mul is
 * accumulated into (the reference caller zeroes it, main.cu:80). */
void hqo_q3_matvec_f32(const float* x, const int32_t* mat, float* mul,
                       const float* scales, const float* zeros, int K, int N);

/* The same kernel with the columns spread over OpenMP threads (identical results: each
 * column keeps its arithmetic order).  Returns the number of threads used. */
int hqo_q3_matvec_f32_omp(const float* x, const int32_t* mat, float* mul,
                          const float* scales, const float* zeros, int K, int N);

/* Same sum in double precision, written to y (overwrites). */
void hqo_q3_matvec_f64(const double* x, const int32_t* mat, double* y,
                       const float* scales, const float* zeros, int K, int N);

/* "faster" kernel, src/quant3MatMul-hip/kernels.h:93-169: scale/zero rounded
 * to fp16, per 32-value group a fresh half2 accumulator collects 16
 * hfma2(hfma2(q, scale, -zero), x, acc) terms, widened and added in fp32. */
void hqo_q3_matvec_f16(const uint16_t* x_f16, const int32_t* mat, float* mul,
                       const float* scales, const float* zeros, int K, int N);

/* Batched GEMM, PARITY UNPINNED: out[m][n] = sum_k A[m][k]*(s[n]*q[k][n]-z[n]).
 * mode 0: exact in double; mode 1: weight rounded once to fp16
 * (w16 = fp16_rn(s*q - z) in fp32), products accumulated in double. */
void hqo_q3_gemm(const uint16_t* A_f16, const int32_t* mat, double* out,
                 const float* scales, const float* zeros, int M, int K, int N,
                 int mode);

/* ---- NF4 / FP4 blockwise dequant (PARITY UNPINNED) --------------------- */
extern const float hqo_nf4_table[16];
extern const float hqo_fp4_table[16];
/* out[2i] = f16(table[byte>>4]*absmax[2i/bs]); out[2i+1] = f16(table[byte&15]*...) */
void hqo_dequant_4bit(const uint8_t* packed, const float* absmax,
                      uint16_t* out_f16, int64_t n_elems, int blocksize,
                      int table /*0=NF4, 1=FP4*/);

/* Inverse of hqo_dequant_4bit (PARITY UNPINNED): blockwise absmax, nearest table code. */
void hqo_quantize_4bit(const void* x, int x_is_f16, uint8_t* packed, float* absmax, int64_t n,
                       int blocksize, int table);

/* ---- bitsandbytes dynamic 8-bit quantize (quantBnB) -------------------- */
/* src/quantBnB-hip/main.cu:13-66 with STOCHASTIC=0. */
uint8_t hqo_dquantize(const float* code256, float x);
void    hqo_quantize_dynamic8(const float* code256, const float* A, uint8_t* out,
                              int64_t n);
/* The signed dynamic map bitsandbytes builds (256 sorted fp32 values). */
void    hqo_dynamic_map(float* code256);

/* ---- per-token int8 activation quantisation (quantVLLM) ------------------ */
/* src/quantVLLM-cuda/reference.h:1-93; dtype 0 = fp32, 1 = fp16 bits, 2 = bf16 bits.
 * Pinned by the reference host loops compiled into oracle/_ref. */
void hqo_int8_quant_static(const void* x, int dtype, int8_t* out, int64_t tokens, int hidden,
                           float scale, int has_azp, int32_t azp);
void hqo_int8_quant_dynamic(const void* x, int dtype, int8_t* out, float* scales,
                            int32_t* azp /*nullable*/, int64_t tokens, int hidden);

/* ---- LUT-GEMM (BCQ) ----------------------------------------------------- */
/* bit packing of src/lut-gemm-hip/main.cu:118-134:
 * signs[(k*nb + b)*N + n] in {-1,+1} -> bW[((k/32)*nb + b)*N + n] bit (k%32). */
void hqo_bcq_pack(const int8_t* signs, int K, int N, int nb, uint32_t* bW);
/* dense weights, src/lut-gemm-hip/main.cu:136-146 (W[k*N+n], double). */
void hqo_bcq_dequant(const uint32_t* bW, const uint16_t* alpha_f16,
                     const uint16_t* qbias_f16 /*nullable*/, int K, int N, int nb,
                     int group, double* W);
/* y[n] = sum_k x[k]*W[k][n] in double (x, alpha, bias are fp16 inputs). */
void hqo_lut_gemv_f64(const uint32_t* bW, const uint16_t* alpha_f16,
                      const uint16_t* qbias_f16, const uint16_t* x_f16, double* y,
                      int K, int N, int nb, int group);
/* Reference evaluation order, src/lut-gemm-hip/mv_fp16.h:133-227: fp16 LUT
 * built by the doubling chain, fp16 partial sums, fp16 alpha multiply, and the
 * per-K-tile fp16 results added to the output in tile order (the GPU's atomic
 * order is arbitrary; tile order is one admissible outcome). */
void hqo_lut_gemv_f16(const uint32_t* bW, const uint16_t* alpha_f16,
                      const uint16_t* qbias_f16, const uint16_t* x_f16,
                      uint16_t* y_f16, int K, int N, int nb, int group);

/* ---- AQLM 1x16 ------------------------------------------------------------ */
/* src/quantAQLM-hip/main.cu:29-101.  mode 0: double accumulation;
 * mode 1: the reference's arithmetic (4 chained hfma2 per code, halves widened
 * and summed in fp32 in lane order, fp32 shuffle-down tree over 64 lanes).
 * scales_f16 NULL => no scale (reference behaviour); else y = f16(scale*acc). */
void hqo_aqlm_matvec(const int16_t* codes, const uint16_t* codebooks_f16,
                     const uint16_t* scales_f16, const uint16_t* x_f16,
                     uint16_t* y_f16, double* y_f64 /*nullable*/, int M, int K,
                     const int cb_a_sizes[4], int cb_stride_int4, int mode);

/* ---- gemv (src/gemv-hip) --------------------------------------------------- */
/* mode 0: mat fp16 [rows][n]; 1: int8 [rows][n]; 2: 4-bit codes, uint8 [rows][n/2], column j in the
 * low nibble of byte j/2 for even j.  res = scale * sum_j (q - zero_point) * vec[j] in double with
 * scale/zero_point rounded to fp16 first (ignored for mode 0); res_f16 / res_f64 may be NULL. */
void hqo_gemv(const void* mat, int mode, const uint16_t* vec_f16, uint16_t* res_f16, double* res_f64,
              int rows, int n, float scale, float zero_point);

/* ---- mxfp4 quantise-dequantise (src/mxfp4-hip/main.cu:19-142) ---------------- */
/* in/out: fp16 or bf16 bit patterns, n a multiple of 32 (groups of 32 share a power-of-two scale). */
void hqo_mxfp4_qdq(const uint16_t* in, uint16_t* out, int64_t n, int is_bf16);

#ifdef __cplusplus
}
#endif
#endif
