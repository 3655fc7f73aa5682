// Shape-list reader shared by the two bench drivers: whitespace rows
// "N C H W pad T Y X", '#' comments and blank lines skipped, duplicates
// dropped keeping first-seen order (Cuda_kernels/bench/BenchBothTime.cu:14-25,
// 59-82; file format as in Cuda_kernels/bench/tensors_alexnet.txt).
#ifndef CP4_BENCH_COMMON_H
#define CP4_BENCH_COMMON_H

#include <fstream>
#include <iostream>
#include <set>
#include <sstream>
#include <string>
#include <vector>

#include "cp4/tensor.h"

inline std::vector<tensor_shape> get_unique_ordered_shapes(const std::vector<tensor_shape>& in) {
  std::vector<tensor_shape> out;
  std::set<tensor_shape> seen;
  for (const auto& s : in)
    if (seen.insert(s).second) out.push_back(s);
  return out;
}

inline bool read_shapes(const char* path, std::vector<tensor_shape>* shapes) {
  std::ifstream f(path);
  if (!f.is_open()) {
    std::cerr << "Couldn't open tensors file.\n";
    return false;
  }
  std::string line;
  while (std::getline(f, line)) {
    if (line.empty() || line[0] == '#') continue;
    std::stringstream ss(line);
    tensor_shape p;
    if (!(ss >> p.N >> p.C >> p.H >> p.W >> p.pad >> p.T >> p.Y >> p.X)) continue;
    shapes->push_back(p);
  }
  *shapes = get_unique_ordered_shapes(*shapes);
  return true;
}

#endif
