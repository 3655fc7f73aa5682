// cp4_conv2d_forward N C H W pad T Y X Rank device
// The reference's standalone executable (Cuda_kernels/cp4Conv2d.cu:196-236):
// one forward launch of the given shape, meant to be run under a profiler.
// Unlike the reference it prints the time and bytes it measured.
#include <cstdlib>
#include <iostream>

#include "cp4/capi.h"
#include "cp4/cp4conv2d.h"

int main(int argc, char** argv) {
  tensor_shape p;
  p.N = 5; p.C = 32; p.H = 1024; p.W = 1024; p.pad = 1; p.T = 32; p.Y = 3; p.X = 3; p.Rank = 8;
  int device = 0;
  if (argc != 11) {
    std::cerr << "Using Default shape" << std::endl;
  } else {
    p.N = std::atoi(argv[1]); p.C = std::atoi(argv[2]); p.H = std::atoi(argv[3]);
    p.W = std::atoi(argv[4]); p.pad = std::atoi(argv[5]); p.T = std::atoi(argv[6]);
    p.Y = std::atoi(argv[7]); p.X = std::atoi(argv[8]); p.Rank = std::atoi(argv[9]);
    device = std::atoi(argv[10]);
  }
  if (cp4_set_device(device) != CP4_OK) {
    std::cerr << cp4_last_error_message() << "\n";
    return 1;
  }
  const auto r = CP::run_convolution(p, 1);
  std::cout << r.first << " us, " << r.second << " bytes" << std::endl;
  return 0;
}
