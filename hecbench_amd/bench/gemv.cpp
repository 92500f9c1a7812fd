// gemv: the command line, inputs, printed lines and acceptance band of the HeCBench benchmark
// (src/gemv-hip/main.cu, gemv.cu, simple_tensor.h) on top of libhq.
//
//   gemv [-s <size>] [-i <iter>] [-x <block_x>] [-y <block_y>] [-u <scale>] [-v <zero_point>]
//
// block_x / block_y are accepted and echoed as the reference does, but the library picks its
// own launch shape.  Extra lines give GB/s of algorithmic bytes and a PASS / FAIL verdict of
// the reference's check (|result - exact| <= 0.125 * size / 512, widened by the fp16 rounding of
// the result) evaluated on the host.
#include <getopt.h>

#include "bench_common.h"

namespace {

// The reference fills every tensor from a fresh std::mt19937(19937) (simple_tensor.h:76-99).
std::vector<uint16_t> random_half(size_t n) {
  std::vector<uint16_t> v(n);
  std::mt19937 gen(19937);
  std::uniform_real_distribution<float> dis(0.0, 1.0);
  for (auto& x : v) x = f32_to_f16_bits(dis(gen));
  return v;
}
std::vector<int8_t> random_int8(size_t n) {
  std::vector<int8_t> v(n);
  std::mt19937 gen(19937);
  std::uniform_int_distribution<int> dis(-128, 127);
  for (auto& x : v) x = (int8_t)dis(gen);
  return v;
}
std::vector<uint8_t> random_int4_pairs(size_t nbytes) {
  std::vector<uint8_t> v(nbytes);
  std::mt19937 gen(19937);
  std::uniform_int_distribution<int> dis(0, 15);
  for (auto& b : v) {
    const int x = dis(gen), y = dis(gen);  // X = low nibble, Y = high nibble
    b = (uint8_t)((x & 15) | ((y & 15) << 4));
  }
  return v;
}

template <typename Weight>  // Weight(row, col) -> dequantised weight as double
int check(const std::vector<uint16_t>& res, const std::vector<uint16_t>& vec, unsigned size, Weight w) {
  const double delta = 0.125 * size / 512;  // gemv.cu:143
  int bad = 0;
  std::vector<double> x(size);
  for (unsigned j = 0; j < size; ++j) x[j] = f16_bits_to_f32(vec[j]);
#pragma omp parallel for reduction(+ : bad)
  for (int i = 0; i < (int)size; ++i) {
    double s = 0;
    for (unsigned j = 0; j < size; ++j) s += w((unsigned)i, j) * x[j];
    const double got = f16_bits_to_f32(res[i]);
    // the band of the reference plus the rounding of the fp16 result itself (half an ulp), which the
    // reference's band does not leave room for once |result| exceeds 256
    if (std::fabs(s - got) > delta + std::fabs(s) * (1.0 / 2048)) {
      if (bad < 10) std::printf("!!![idx=%d] %f != %f, diff=%f\n", i, got, s, s - got);
      ++bad;
    }
  }
  return bad;
}

template <typename Call>
void run(const char* title, unsigned iter, double bytes, Call call) {
  std::printf("%s\n", title);
  call();  // warm-up, as the first timed call would otherwise include the module load
  HIP_OK(hipDeviceSynchronize());
  auto start = std::chrono::steady_clock::now();
  for (unsigned i = 0; i < iter; ++i) call();
  HIP_OK(hipDeviceSynchronize());
  auto end = std::chrono::steady_clock::now();
  const double ns = std::chrono::duration<double, std::nano>(end - start).count();
  std::printf("Average kernel execution time: %f (us)\n", (ns * 1e-3) / iter);
  std::printf("  (%.1f GB/s of algorithmic bytes, %.1f%% of 8000 GB/s)\n", bytes / (ns / iter),
              100.0 * bytes / (ns / iter) / 8000.0);
  std::printf("Check correctness on the device\n");
}

}  // namespace

int main(int argc, char** argv) {
  static struct option long_options[] = {{"size", required_argument, 0, 's'},   {"iter", required_argument, 0, 'i'},
                                         {"block_x", required_argument, 0, 'x'}, {"block_y", required_argument, 0, 'y'},
                                         {"scale", required_argument, 0, 'u'},  {"zero_point", required_argument, 0, 'v'},
                                         {0, 0, 0, 0}};
  unsigned size = 512, iter = 1, block_dim_x = 32, block_dim_y = 4;
  float scale = 0.0625f, zero_point = 0.01f;
  int opt;
  while ((opt = getopt_long(argc, argv, "s:i:k:x:y:g:u:v:", long_options, NULL)) != -1) {
    switch (opt) {
      case 's': size = (unsigned)std::atoi(optarg); break;
      case 'i': iter = (unsigned)std::atoi(optarg); break;
      case 'x': block_dim_x = (unsigned)std::atoi(optarg); break;
      case 'y': block_dim_y = (unsigned)std::atoi(optarg); break;
      case 'u': scale = (float)std::atof(optarg); break;
      case 'v': zero_point = (float)std::atof(optarg); break;
      default:
        std::printf("Invalid option. Usage: %s [-s <size> -i <iter> -x <block_x> -y <block_y> -u <scale> -v "
                    "<zero_point>]\n", argv[0]);
        return -1;
    }
  }
  if (size == 0 || size % 32 || iter == 0) {
    std::printf("size must be a positive multiple of 32 and iter positive\n");
    return -1;
  }
  const unsigned grid_dim_x = 1;
  std::printf("size=%u, iter=%u\n", size, iter);
  std::printf("GPU block_dim\t(%d, %d)\n", block_dim_x, block_dim_y);
  std::printf("GPU grid_dim\t(%d, %d)\n", grid_dim_x, size / block_dim_y);
  std::printf("num_per_thread=%d\n", size / (block_dim_x * grid_dim_x));
  HQ_OK_OR_DIE(hq_init());

  const size_t nn = (size_t)size * size;
  const std::vector<uint16_t> vec = random_half(size);
  DevBuf<uint16_t> d_vec(size), d_res(size);
  d_vec.upload(vec);
  int bad = 0;
  const float sc = f16_bits_to_f32(f32_to_f16_bits(scale)), zp = f16_bits_to_f32(f32_to_f16_bits(zero_point));
  {
    const std::vector<uint16_t> mat = random_half(nn);
    DevBuf<uint16_t> d_mat(nn);
    d_mat.upload(mat);
    run("GEMV FP16 ..", iter, 2.0 * nn + 4.0 * size,
        [&] { HQ_OK_OR_DIE(hq_gemv_fp16(d_mat.p, d_vec.p, d_res.p, (int)size, (int)size, nullptr)); });
    bad += check(d_res.download(), vec, size, [&](unsigned i, unsigned j) { return (double)f16_bits_to_f32(mat[(size_t)i * size + j]); });
  }
  std::printf("int8/int4: scale=%f, zero_point=%f\n", scale, zero_point);
  {
    const std::vector<int8_t> mat = random_int8(nn);
    DevBuf<int8_t> d_mat(nn);
    d_mat.upload(mat);
    run("GEMV int8 quantized...", iter, 1.0 * nn + 4.0 * size,
        [&] { HQ_OK_OR_DIE(hq_gemv_int8(d_mat.p, d_vec.p, d_res.p, (int)size, (int)size, scale, zero_point, nullptr)); });
    bad += check(d_res.download(), vec, size, [&](unsigned i, unsigned j) { return ((double)mat[(size_t)i * size + j] - zp) * sc; });
  }
  {
    const std::vector<uint8_t> mat = random_int4_pairs(nn / 2);
    DevBuf<uint8_t> d_mat(nn / 2);
    d_mat.upload(mat);
    run("GEMV int4 quantized...", iter, 0.5 * nn + 4.0 * size,
        [&] { HQ_OK_OR_DIE(hq_gemv_int4(d_mat.p, d_vec.p, d_res.p, (int)size, (int)size, scale, zero_point, nullptr)); });
    bad += check(d_res.download(), vec, size, [&](unsigned i, unsigned j) {
      const uint8_t b = mat[((size_t)i * size + j) / 2];
      return ((double)((j & 1) ? (b >> 4) : (b & 15)) - zp) * sc;
    });
  }
  std::printf("%s\n", bad ? "FAIL" : "PASS");
  return bad ? 1 : 0;
}
