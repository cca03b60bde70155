// Tables of the base-2 exponential and logarithm that float64 kernels carry with them (straight-line and interpreter):
// 64 values 2^(j/64); 256 pairs (R[j], G[j]) = (1/(1+j/256) rounded, -log2 of that rounded value); the polynomial
// coefficients c5..c1 of 2^r - 1 and l7..l1 of log2(1+u). 64 + 512 + 12 doubles.
#pragma once
#include <cmath>
#include <vector>

namespace spnc_hip {

constexpr unsigned DOUBLE_MATH_TABLE_VALUES = 64 + 512 + 12;

inline std::vector<double> doubleMathTables() {
  std::vector<double> t;
  for (int j = 0; j < 64; ++j) t.push_back(double(exp2l((long double)j / 64.0L)));
  for (int j = 0; j < 256; ++j) {
    const double recip = double(1.0L / (1.0L + (long double)j / 256.0L));
    t.push_back(recip);
    t.push_back(j == 0 ? 0.0 : double(-log2l((long double)recip)));
  }
  static const double poly[12] = {0x1.5d87fe78a6731p-10, 0x1.3b2ab6fba4e77p-7, 0x1.c6b08d704a0cp-5, 0x1.ebfbdff82c58fp-3, 0x1.62e42fefa39efp-1,
                                  0x1.a61762a7aded9p-3, -0x1.ec709dc3a03fdp-3, 0x1.2776c50ef9bfep-2, -0x1.71547652b82fep-2,
                                  0x1.ec709dc3a03fdp-2, -0x1.71547652b82fep-1, 0x1.71547652b82fep+0};
  t.insert(t.end(), poly, poly + 12);
  return t;
}

}  // namespace spnc_hip
