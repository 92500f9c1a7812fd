/*
 * hq.h — C ABI of libhq: weight-only quantized-inference kernels for AMD
 * Instinct MI355X (gfx950 / CDNA4).
 *
 * The entry points replace the host launch wrappers of the HeCBench benchmarks
 * quant3MatMul, lut-gemm, quantAQLM and quantBnB (citations are relative to the
 * HeCBench tree).  Conventions shared by every entry point:
 *
 *   - all data pointers are DEVICE pointers owned by the caller;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     calls are asynchronous on that stream and never synchronise;
 *   - outputs are OVERWRITTEN unless HQ_FLAG_ACCUMULATE is given, so no
 *     pre-zeroing memset is needed (the reference wrappers accumulate with
 *     atomics and make the caller memset first);
 *   - return value: 0 on success, a negative HQ_ERR_* code for a rejected
 *     argument (nothing is launched), or a positive hipError_t value;
 *   - nothing is printed; hq_strerror() turns a code into text;
 *   - a NaN or an infinity among the activations makes the affected outputs non-finite (the
 *     fixed-point matrix-core paths give NaN where the reference arithmetic would give +-Inf);
 *   - the library keeps one small workspace per (device, stream) pair (split-K
 *     partial sums, arrival counters, re-ordered GEMM activations), allocated by
 *     hq_init() / hq_reserve_workspace() or by the first call that needs more than
 *     is there (that call then runs hipMalloc, which fails under stream capture:
 *     reserve first).  A workspace grows geometrically, lives until hq_shutdown()
 *     and is used by every call on its stream: calls on different streams may
 *     overlap, two host threads must not issue calls on the SAME stream at the
 *     same time (the calls of one stream share the workspace in stream order).
 */
#ifndef HQ_H
#define HQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HQ_OK 0
#define HQ_ERR_NULL_POINTER (-1)
#define HQ_ERR_BAD_SHAPE (-2)
#define HQ_ERR_BAD_ENUM (-3)
#define HQ_ERR_MISALIGNED (-4)
#define HQ_ERR_UNSUPPORTED_DEVICE (-5)
#define HQ_ERR_TOO_LARGE (-6)

/* element types of the activation vector / matrix */
#define HQ_DTYPE_F32 0
#define HQ_DTYPE_F16 1
#define HQ_DTYPE_BF16 2 /* accepted by the activation quantisers and hq_mxfp4_qdq only */

/* flags */
#define HQ_FLAG_ACCUMULATE 1u /* y += result (reference wrapper semantics) */

/* 4-bit code books of hq_dequant_nf4 / hq_quantize_4bit.
 * NF4: the QLoRA normal-float table (checked against its quantile construction).
 * FP4: bit 3 sign, low bits {0, 1/192, 2/3, 1, 1/3, 1/2, 1/6, 1/4} -- parity unpinned: the HeCBench
 * tree holds no FP4 source, so the table is this library's statement of the bitsandbytes one. */
#define HQ_TABLE_NF4 0
#define HQ_TABLE_FP4 1

/* Version of this ABI (bumped on incompatible change). */
int hq_abi_version(void);

/* Text for a return code of this library (HQ_ERR_* or a hipError_t value). */
const char* hq_strerror(int code);

/* Prepare the current HIP device: checks that it is a gfx950 part, allocates
 * the per-device workspace.  Optional (the first compute call does the same),
 * but calling it keeps the allocation out of the first timed call.
 * Mirrors the device query of the AQLM launcher, src/quantAQLM-hip/main.cu:108-121. */
int hq_init(void);

/* Sizes the workspace of (current device, stream) for split-K matvecs up to max_N columns and
 * batched GEMMs up to max_K input features, so that later calls on that stream never allocate
 * (needed before stream capture).  No counterpart in the reference. */
int hq_reserve_workspace(void* stream, int max_K, int max_N);

/* Host-only size queries behind hq_reserve_workspace (plain arithmetic: no device is touched, so they also
 * answer for a device that is not present).  hq_q3_workspace_need: floats and arrival counters one
 * hq_q3_matvec(K, N, batch_M) call takes from its stream's workspace on a device of compute_units compute
 * units, computed by the very plan functions of the launch.  hq_reserve_need: what
 * hq_reserve_workspace(stream, max_K, max_N) makes sure of - at least the need of every call with K <= max_K
 * and N <= max_N, whatever the batch.  Counterpart of the compute-unit query that sizes the launch in
 * src/quantAQLM-hip/main.cu:108-121. */
int hq_q3_workspace_need(int compute_units, int K, int N, int batch_M, int64_t* floats, int64_t* counters);
int hq_reserve_need(int compute_units, int max_K, int max_N, int64_t* floats, int64_t* counters);

/* Waits for the current device, then frees every workspace the library holds on any device.
 * Optional; the library can be used again afterwards (workspaces are re-created on demand). */
int hq_shutdown(void);

/* Launch-shape override for tests and sweeps, not part of the stable interface: name is one of
 * HQ_Q3_WAVES, HQ_Q3_STEPS, HQ_Q3_KSPLIT, HQ_Q3_TILE, HQ_Q3_SMALL_BATCH, HQ_Q3_ROW_BLOCKS, HQ_LUT_PATH, HQ_LUT_KSPLIT, HQ_NF4_PIPE,
 * HQ_AQLM_ROWS, HQ_Q8_WGS, HQ_Q8_FAST, HQ_GEMV_LDS, HQ_GEMV_SPLIT, HQ_SPLITK_FENCES (an environment variable of the same name seeds
 * the knob once per process); clear != 0 returns the knob to the library's own choice.  Results
 * never depend on a knob beyond the documented tolerances. */
int hq_set_tunable(const char* name, int value, int clear);

/* Device facts the benchmark drivers print next to the roofline numbers.
 * Any pointer may be NULL. */
int hq_device_info(int* compute_units, int* wavefront_size, int* lds_bytes_per_cu,
                   int* memory_clock_khz, int* memory_bus_bits, char* name, int name_len);

/*
 * Blockwise 4-bit dequantisation to fp16 (NF4 or FP4 code book).
 *   out[2i]   = fp16_rn(table[packed[i] >> 4]  * absmax[(2i)   / blocksize])
 *   out[2i+1] = fp16_rn(table[packed[i] & 15]  * absmax[(2i+1) / blocksize])
 * fp32 multiply, one round-to-nearest-even to fp16 (bit-exact contract).
 * n_elems >= 0; blocksize > 0 and even.  Stands in the place of the quantBnB
 * benchmark's kernel launch, src/quantBnB-hip/main.cu:176 (the reference
 * benchmark itself holds the 8-bit quantiser, see hq_quantize_dynamic8).
 */
int hq_dequant_nf4(const uint8_t* packed, const float* absmax, void* out_fp16,
                   int64_t n_elems, int blocksize, int table, void* stream);

/*
 * bitsandbytes dynamic-map 8-bit quantisation: out[i] = index of the entry of
 * the sorted 256-entry table `code` nearest to A[i], with the reference's
 * search and tie rules.  Replaces kQuantize<256,256><<<...>>>(code, A, out, n),
 * src/quantBnB-hip/main.cu:90-130,176.  Bit-exact contract.
 */
int hq_quantize_dynamic8(const float* code, const float* A, uint8_t* out, int64_t n,
                         void* stream);

/*
 * GPTQ 3-bit matvec / batched GEMM:
 *   y[m][n] = sum_k x[m][k] * (scales[n] * q[k][n] - zeros[n]),  m < batch_M
 * qweight is int32[3*K/32][N] row-major: the 32 codes of k-group g of column n
 * form a 96-bit little-endian string in words qweight[(3g+j)*N + n], j=0..2,
 * code i at bits 3i..3i+2 (src/quant3MatMul-hip/kernels.h:42-86).  zeros holds
 * the pre-multiplied scale*zero_point.
 *   x        : [batch_M][K] row-major, fp32 (HQ_DTYPE_F32) or fp16 (HQ_DTYPE_F16)
 *   y        : fp32 [batch_M][N]
 *   K % 32 == 0, N % 4 == 0, batch_M >= 1; qweight and x 16-byte aligned; for batch_M > 1 scales, zeros
 *   and y 16-byte aligned as well (whichever kernel the plan picks, so that a pointer that works at one
 *   batch size or on one device works at every other), for batch_M == 1 4-byte aligned.
 * Products are accumulated in fp32 for both dtypes (the reference's fp16
 * variant accumulates 16 terms in fp16).
 * batch_M == 1 replaces vecquant3matmul / vecquant3matmul_faster
 * (src/quant3MatMul-hip/kernels.h:171-217) — pass HQ_FLAG_ACCUMULATE for their
 * "mul +=" behaviour.  batch_M > 1 requires HQ_DTYPE_F16 and has no counterpart in
 * the reference; which kernel serves it (hq_q3_matvec_plan tells):
 *   - the matvec's kernel, four rows side by side: batches 2 ... 4 (at 0.1 ... 0.6 us more than
 *     batch 1); batches up to 64 as row blocks of four, one workgroup per column tile, 4096
 *     elements of K and row block, where that makes at most four workgroups per compute unit
 *     (5 and 6 rows: at most one) and K <= 32768; otherwise 5 ... 8 rows as two passes of one
 *     workgroup unless N / 128 is at least 7/8 of the compute units or K is longer than that;
 *     every activation enters with an error of at most 2^-19 of the largest magnitude
 *     among its 32 neighbours (exactly, if within 2^8 of it);
 *   - everything else: the MFMA GEMM path, which pre-scales every activation row by a
 *     power of two, so accuracy does not depend on the magnitude of the activations:
 *     entries within 2^21 of their row's largest magnitude enter the matrix cores
 *     exactly, smaller ones lose low bits (those 2^32 below it vanish).
 */
int hq_q3_matvec(const void* x, int x_dtype, const int32_t* qweight, const float* scales,
                 const float* zeros, float* y, int K, int N, int batch_M, unsigned flags,
                 void* stream);

/*
 * Which kernel hq_q3_matvec runs for this shape on the current device with the current
 * tunables (for tests and tuning; negative = error code).
 */
#define HQ_Q3_PLAN_MATVEC 0 /* batch_M == 1 */
#define HQ_Q3_PLAN_GEMM 2   /* batched MFMA GEMM */
#define HQ_Q3_PLAN_BLOCK 3  /* batch_M 2 ... 64: the matvec's kernel, four rows per pass or workgroup */
int hq_q3_matvec_plan(int K, int N, int batch_M);

/*
 * hq_q3_matvec for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): same arguments, same kernels and bit-identical results, but the
 * scratch the kernels need (split-K partial sums and arrival counters of batches 1 and 2, the batched
 * path's re-ordered activations, row sums, row scales and K-split sums) is a fixed 10 MiB + 64 KiB array in device
 * memory that each GPU holds from library load to process end, instead of the stream's workspace.
 * The call runs no hipMalloc, hipFree or allocating library routine.  Limits: a batch that the MFMA
 * GEMM serves (hq_q3_matvec_plan) needs K <= 16384; a split-K matvec needs tiles * splits * batch_M <= 8192 (the one-per-round split falls
 * back to one workgroup per compute unit where it would not fit) and N <= 1032192; beyond them
 * HQ_ERR_TOO_LARGE.  All calls on one GPU
 * share that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race;
 * issue them on one stream or order them with events.  Call hq_init() once per device beforehand,
 * outside any capture (it resolves the array's address).  No counterpart in the reference.
 */
int hq_q3_matvec_noalloc(const void* x, int x_dtype, const int32_t* qweight, const float* scales,
                         const float* zeros, float* y, int K, int N, int batch_M, unsigned flags,
                         void* stream);

/*
 * LUT-GEMM binary-coded-quantisation matvec (fp16 in, fp16 out):
 *   y[n] = sum_k x[k] * ( q_bias[k/G][n] + sum_b alpha[k/G][b][n] * s(k,b,n) ),
 *   s = +1 if bit (k%32) of bW[k/32][b][n] is set, else -1
 * Layouts (src/lut-gemm-hip/nQWeight_fp16.h:24-26): bW uint32[K/32][nbits][N],
 * alpha fp16[K/G][nbits][N], q_bias fp16[K/G][N] or NULL, x fp16[K], y fp16[N].
 * K % 32 == 0, G % 32 == 0, K % G == 0, 1 <= nbits <= 8; any N.  x 16-byte aligned, bW 4-byte,
 * alpha, q_bias and y 2-byte (16-byte aligned operands and N % 64 == 0 take the aligned loads).
 * Sums are kept in fp32 and rounded to fp16 once.  Replaces
 * matmul(output, input, nqW, m), src/lut-gemm-hip/kernels.cu:27-31.
 */
int hq_lut_gemv(const uint32_t* bW, const void* alpha_fp16, const void* q_bias_fp16,
                const void* x_fp16, void* y_fp16, int K, int N, int nbits, int group_size,
                void* stream);

/* Which kernel hq_lut_gemv takes for a problem (pointers matter through their alignment only; nothing is
 * launched): HQ_LUT_PLAN_TABLE, or a matrix-core plan, with HQ_LUT_PLAN_RAGGED or-ed in when N is not a
 * multiple of 64 or an operand is not 16-byte aligned.  Negative: the HQ_ERR_* code hq_lut_gemv would return
 * for the shape.  The reference kernel takes any N (src/lut-gemm-hip/mv_fp16.h:229-236); so do the
 * matrix-core plans for N >= 64 and K % 128 == 0. */
#define HQ_LUT_PLAN_TABLE 0        /* 256-entry tables per 8-element sub-vector in LDS */
#define HQ_LUT_PLAN_MFMA 1         /* group size a multiple of 128 */
#define HQ_LUT_PLAN_MFMA_GROUPED 2 /* group size 64 or 32 */
#define HQ_LUT_PLAN_RAGGED 16
int hq_lut_gemv_plan(const uint32_t* bW, const void* alpha_fp16, const void* q_bias_fp16, int K, int N,
                     int nbits, int group_size);

/*
 * AQLM 1x16 code-book matvec (fp16 in, fp16 out):
 *   y[m] = fp16_rn( scale[m] * sum_g dot8(codebook[cb(m)][u16(codes[m][g])], x[8g..8g+7]) )
 * codes int16[M][K/8] (read as unsigned), codebooks fp16[..][65536][8] with
 * consecutive code books codebook_stride_int4*16 bytes apart, cb(m) = first j
 * with m < codebook_a_sizes[j].  scales_fp16 may be NULL (the reference kernel
 * applies no scale).  K % 64 == 0 (as in the reference).  fp32 accumulation, one rounding.  Replaces
 * code1x16_matvec, src/quantAQLM-hip/main.cu:103-139 (without its internal
 * synchronisation, timing and printing).
 */
int hq_aqlm_matvec(const int16_t* codes, const void* codebooks_fp16, const void* scales_fp16,
                   const void* x_fp16, void* y_fp16, int M, int K,
                   const int codebook_a_sizes[4], int codebook_stride_int4, void* stream);

/*
 * Device-side packers and the 4-bit blockwise quantiser (inverses of the unpack /
 * dequantise steps above, so the family round-trips on the GPU).
 *
 * hq_q3_pack: codes uint8[K][N] (values 0..7) -> qweight int32[3K/32][N] in the layout of
 *   hq_q3_matvec; the host loop it replaces is the weight initialisation of
 *   src/quant3MatMul-hip/main.cu:35-43 (generalised from the all-ones pattern).
 * hq_bcq_pack: signs int8[K][nbits][N] (> 0 means +1) -> bW uint32[K/32][nbits][N];
 *   replaces the packing loop of makeRandomWeight, src/lut-gemm-hip/main.cu:118-134.
 * hq_quantize_4bit: x fp32/fp16 [n] -> packed nibbles (high nibble first) and one fp32
 *   absmax per block; code = nearest table entry of x/absmax (NF4: a value exactly on the
 *   midpoint of two entries takes the lower code).  No counterpart in the HeCBench tree.
 */
int hq_q3_pack(const uint8_t* codes, int32_t* qweight, int K, int N, void* stream);
int hq_bcq_pack(const int8_t* signs, uint32_t* bW, int K, int N, int nbits, void* stream);
int hq_quantize_4bit(const void* x, int x_dtype, uint8_t* packed, float* absmax, int64_t n_elems,
                     int blocksize, int table, void* stream);

/*
 * Per-token int8 activation quantisation, the step in front of a W8A8 matmul.
 * x is [num_tokens][hidden_size] row-major in fp32, fp16 or bf16; out int8 of the same shape.
 *   static : out = sat8(rne(x / scale))                       (has_azp == 0)
 *            out = sat8(sat32(rne(x / scale)) + azp)          (has_azp != 0)
 *   dynamic: azp == NULL: scales[t] = max|x_t| / 127, out = sat8(rne(x * (127 / max|x_t|)))
 *            azp != NULL: scales[t] = (max_t - min_t) / 255, azp[t] = rne(-128 - min_t / scales[t]),
 *                         out = sat8(sat32(rne(x / scales[t])) + azp[t])
 * Results are those of fp32 IEEE arithmetic (true division, round to nearest even): bit-exact with
 * the reference host loops (src/quantVLLM-cuda/reference.h:1-93) wherever those are defined (a NaN
 * quotient, or a quotient plus zero point beyond int32, is undefined there).  Any element alignment
 * is accepted; x 16-byte and out 8-byte aligned take the vector path at every hidden size.  Replaces
 * static_scaled_int8_quant / dynamic_scaled_int8_quant, src/quantVLLM-hip/main.cu:133-168.
 */
int hq_int8_quant_static(const void* x, int x_dtype, int8_t* out, int64_t num_tokens, int hidden_size,
                         float scale, int has_azp, int32_t azp, void* stream);
int hq_int8_quant_dynamic(const void* x, int x_dtype, int8_t* out, float* scales, int32_t* azp,
                          int64_t num_tokens, int hidden_size, void* stream);

/*
 * Dense / weight-quantised matrix-vector products with an fp16 vector and fp16 result
 * (mat is [rows][n] row-major, sums in fp32, one rounding to fp16):
 *   hq_gemv_fp16: res[r] = sum_j mat[r][j] * vec[j]                     mat fp16;  n % 8 == 0
 *   hq_gemv_int8: res[r] = scale * sum_j (mat[r][j] - zero_point) * vec[j]   mat int8;  n % 16 == 0
 *   hq_gemv_int4: the same with 4-bit unsigned codes, two per byte: column j is the low nibble
 *                 of byte j/2 for even j, the high nibble for odd j;  n % 32 == 0
 * scale and zero_point are rounded to fp16 first, as the reference launchers do.  mat and vec
 * 16-byte aligned.  Replace solve_gemv_with_params / solve_gemv_int8_quantized_with_params /
 * solve_gemv_int4_quantized_with_params, src/gemv-hip/gemv.cu:10-133 (kernels
 * src/gemv-hip/kernels.h:66-311); the reference's block_dim_x/block_dim_y tuning arguments have no
 * counterpart (the launch shape is chosen from the CU count).
 */
int hq_gemv_fp16(const void* mat_fp16, const void* vec_fp16, void* res_fp16, int rows, int n, void* stream);
int hq_gemv_int8(const int8_t* mat, const void* vec_fp16, void* res_fp16, int rows, int n, float scale,
                 float zero_point, void* stream);
int hq_gemv_int4(const uint8_t* mat_packed, const void* vec_fp16, void* res_fp16, int rows, int n, float scale,
                 float zero_point, void* stream);

/*
 * Microscaling fp4 quantise-dequantise: groups of 32 consecutive elements share the scale
 * 2^(e-2), 2^e being the group's largest magnitude rounded to a power of two (carry at a
 * mantissa of 0.75); out = scale * e2m1(in / scale) with round-to-nearest-even onto
 * {0, .5, 1, 1.5, 2, 3, 4, 6} and saturation.  dtype HQ_DTYPE_F16 or HQ_DTYPE_BF16; n_elems a
 * multiple of 32; 16-byte aligned pointers; in and out must not overlap.  Bit-exact with the reference
 * kernel for finite data, except where its arithmetic breaks down: a group maximum that rounds to zero
 * (the reference divides by zero; here signed zeros) and a finite group maximum whose power-of-two
 * rounding leaves the format (fp16 >= 61440, bf16 >= 0x7f60: the reference writes NaN for the group;
 * here the scale is 2^14 / 2^126 and the results are finite or infinite).  Replaces mxfp4<T>(y, a, numel, niters), src/mxfp4-hip/main.cu:144-171
 * (kernel main.cu:109-142), without its timing loop and printing.
 */
int hq_mxfp4_qdq(const void* in, void* out, int64_t n_elems, int dtype, void* stream);

/*
 * Memory-system probes for the benchmark report (no counterpart in the reference): the rate this device
 * delivers to the simplest kernels, measured next to the library kernels instead of quoted from a data sheet.
 *   hq_probe_stream(mode, src, dst, bytes, stream): mode 0 reads `bytes` bytes of src and writes nothing
 *     (dst must still be a valid 16-byte buffer), mode 1 copies them to dst.  bytes a multiple of 16.
 *   hq_probe_gather16(table, table_bytes, gathers, sink16, stream): at least `gathers` independent 16-byte
 *     reads at pseudo-random entries of a table of table_bytes bytes (a power of two) - the access pattern
 *     of a code-book lookup, bounded by cache requests per second; sink16 is a 16-byte buffer that is
 *     never written in practice.  hq_probe_gather16_count(gathers) returns the exact number of reads that
 *     call performs on the current device (the request rounded up to whole trips of every lane).
 *   hq_probe_lds(offsets64, width_bits, write, repeats, sink16, stream): one workgroup of four waves per compute
 *     unit; lane l of every wave repeats one LDS access of width_bits (32, 64 or 128) bits, a read or (write != 0)
 *     a write, at byte offset offsets64[l] (device array of 64 offsets below 8192 - 16, multiples of the access size)
 *     inside its wave's own LDS region - the lane pattern of any kernel's LDS operand can be put under a
 *     profiler's bank-conflict counter next to patterns whose conflicts are known.
 */
int hq_probe_stream(int mode, const void* src, void* dst, int64_t bytes, void* stream);
int hq_probe_gather16(const void* table, int64_t table_bytes, int64_t gathers, void* sink16, void* stream);
int64_t hq_probe_gather16_count(int64_t gathers);
int hq_probe_lds(const uint32_t* offsets64, int width_bits, int write, int repeats, void* sink16, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HQ_H */
