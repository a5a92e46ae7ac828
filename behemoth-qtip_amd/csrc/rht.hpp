// Launch wrappers of rht.hip, bound to one device + stream.
#pragma once
#include <cmath>
#include <memory>
#include <utility>
#include <vector>

#include "qtip_internal.hpp"

namespace qtipmi {

class Rht {
 public:
  void init(int device, hipStream_t stream);
  // x <- (hadK^(T) (x) H_{n/K}) (x * rs[row] * cs[col]) / sqrt(n) on `rows` rows of length n, stride ld; rs / cs may be null
  void hadamard_rows(float* X, long rows, int n, long ld, bool transpose, const float* rs = nullptr,
                     const float* cs = nullptr);
  void transpose(const float* in, long rows, long cols, long ld_in, float* out, long ld_out);
  void scale(float* X, long rows, long cols, long ld, float a);
  void add_diag(float* H, long n, float a);
  // fixed-order fp64 reductions; mode 0: sum A^2, 1: sum A*B, 2: sum (A-B)^2, 3: trace of the rows x rows matrix A
  double reduce(const float* A, long lda, const float* B, long ldb, long rows, long cols, int mode);

 private:
  const uint32_t* device_had(int K, bool transpose);
  int dev_ = 0;
  int cus_ = 1;  // compute units of the device: resident workgroups of the row kernel that walks rows
  hipStream_t s_ = nullptr;
  DBuf<double> partial_;
  std::vector<std::pair<int, std::unique_ptr<DBuf<uint32_t>>>> had_;
};

}  // namespace qtipmi
