// cp4_bench_time tensor_file [results_file] [device]
// The reference's BenchBothTime driver (Cuda_kernels/bench/BenchBothTime.cu):
// for every unique shape of the list, mean microseconds over 47 forward
// launches for ranks 1, 2, 4, 8, 16, as CSV.  The first data column is the
// vendor library's dense convolution (cuDNN in the reference,
// BenchBothTime.cu:90; MIOpen here through namespace NV); shapes it cannot
// take (2*pad != Y-1) print "nan".
#include <cstdlib>
#include <iomanip>

#include "bench_common.h"
#include "cp4/capi.h"
#include "cp4/cp4conv2d.h"
#include "cp4/nvconv2d.h"

int main(int argc, char** argv) {
  std::ofstream of;
  std::streambuf* buf = std::cout.rdbuf();
  int device = 0;
  switch (argc) {
    case 4: device = std::atoi(argv[3]);  // fallthrough
    case 3: of.open(argv[2]); buf = of.rdbuf();  // fallthrough
    case 2: break;
    default:
      std::cerr << "USAGE: cp4_bench_time  Tensor_file  [Results_file]  [device_number]\n";
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
            << p.Y << " " << p.X << ", ";
    if (2 * p.pad + 1 == p.Y && p.Y == p.X)
      results << NV::run_convolution(p, 47).first;
    else
      results << "nan";
    for (unsigned r = 1; r <= 16; r *= 2) {
      p.Rank = r;
      results << ", " << CP::run_convolution(p, 47).first;
    }
    results << std::endl;
  }
  return 0;
}
