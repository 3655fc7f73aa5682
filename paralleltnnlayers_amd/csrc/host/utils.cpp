// random_fill, cp4recom, AllClose (Cuda_kernels/Utils.cu) on the C ABI.
#include "cp4/utils.h"

#include <cstdio>
#include <cstdlib>

#include "cp4/capi.h"

namespace {
void check(cp4_status st, const char* where) {
  if (st == CP4_OK) return;
  std::fprintf(stderr, "cp4 assert: %s (%s) in %s\n", cp4_status_string(st),
               cp4_last_error_message(), where);
  std::exit((int)st);
}
}  // namespace

Tensor random_fill(std::initializer_list<unsigned> lst) {
  Tensor A(lst);
  // fixed seed, as curandSetPseudoRandomGeneratorSeed(gen, 1234ULL) in Utils.cu:27
  check(cp4_random_uniform(A.device(), A.size(), 1234ULL, nullptr), "random_fill");
  A.download();
  return A;
}

Tensor cp4recom(Tensor const& FT, Tensor const& FC, Tensor const& FY, Tensor const& FX) {
  cp4_shape s{};
  s.Rank = FT.shape[1];
  s.T = FT.shape[0];
  s.C = FC.shape[0];
  s.Y = FY.shape[0];
  s.X = FX.shape[0];
  Tensor Out{s.T, s.C, s.Y, s.X};
  for (const Tensor* t : {&FT, &FC, &FY, &FX}) t->upload();
  check(cp4_recompose(&s, FT.device(), FC.device(), FY.device(), FX.device(), Out.device(),
                      nullptr),
        "cp4recom");
  Out.download();
  return Out;
}

bool AllClose(Tensor const& A, Tensor const& B, float tolerance) {
  if (A.size() != B.size()) return false;
  A.upload();
  B.upload();
  long long bad = 0;
  check(cp4_count_exceeding(A.device(), B.device(), A.size(), tolerance, &bad, nullptr),
        "AllClose");
  return bad == 0;
}
