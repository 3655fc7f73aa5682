// cp4_bench_mem tensor_file [results_file] [device]
// The reference's BenchBothMem driver (Cuda_kernels/bench/BenchBothMem.cu):
// algorithmic KiB moved per shape and rank, same CSV layout as the timing
// driver.  The dense column is the dense filter's footprint
// 4*(N*T*H*W + N*C*H*W + T*C*Y*X) bytes.
#include <cstdlib>
#include <iomanip>

#include "bench_common.h"
#include "cp4/capi.h"
#include "cp4/cp4conv2d.h"

int main(int argc, char** argv) {
  std::ofstream of;
  std::streambuf* buf = std::cout.rdbuf();
  int device = 0;
  switch (argc) {
    case 4: device = std::atoi(argv[3]);  // fallthrough
    case 3: of.open(argv[2]); buf = of.rdbuf();  // fallthrough
    case 2: break;
    default:
      std::cerr << "USAGE: cp4_bench_mem  Tensor_file  [Results_file]  [device_number]\n";
      return 1;
  }
  std::ostream results(buf);
  results << std::showpoint << std::setw(5);
  // the reference's header, column names included (BenchBothTime.cu:49, BenchBothMem.cu:49):
  // scripts keyed on it read both files; the "cuDNN" column is the vendor library's dense
  // convolution, MIOpen here
  results << "N C H W pad T Y X, cuDNN, Rank 1, Rank 2, Rank 4, Rank 8, Rank 16" << std::endl;
  std::vector<tensor_shape> shapes;
  if (!read_shapes(argv[1], &shapes)) return 1;
  if (cp4_set_device(device) != CP4_OK) {
    std::cerr << cp4_last_error_message() << "\n";
    return 1;
  }
  for (auto& p : shapes) {
    results << p.N << " " << p.C << " " << p.H << " " << p.W << " " << p.pad << " " << p.T << " "
            << p.Y << " " << p.X;
    const size_t dense = sizeof(float) * ((size_t)p.N * p.T * p.H * p.W +
                                          (size_t)p.N * p.C * p.H * p.W +
                                          (size_t)p.T * p.C * p.Y * p.X);
    results << ", " << dense / 1024;
    for (unsigned r = 1; r <= 16; r *= 2) {
      p.Rank = r;
      results << ", " << CP::run_convolution(p, 47).second / 1024;
    }
    results << std::endl;
  }
  return 0;
}
