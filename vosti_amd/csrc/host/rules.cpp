#include "rules.h"

#include <algorithm>
#include <cmath>

namespace vosti {

void rotary_inverse_frequencies(double theta, int rotary_dim, float* out) {
  const float theta32 = (float)theta;
  for (int j = 0; 2 * j < rotary_dim; ++j) {
    const float exponent = (float)(2 * j) / (float)rotary_dim;
    const float power = (float)std::pow((double)theta32, (double)exponent);
    out[j] = 1.0f / power;
  }
}

float rotary_stretched_frequencies(double theta, int rotary_dim, double factor, double original, double fast, double slow, float* out) {
  const double pi = 3.14159265358979323846;
  const int half = rotary_dim / 2;
  auto turn = [&](double t) { return rotary_dim * std::log(original / (2.0 * pi * t)) / (2.0 * std::log(theta)); };
  const bool stretch = factor > 0.0;
  const double lo = stretch ? std::max(std::floor(turn(fast)), 0.0) : 0.0;
  const double hi = stretch ? std::min(std::ceil(turn(slow)), (double)(rotary_dim - 1)) : 0.0;
  for (int j = 0; j < half; ++j) {
    const double f = std::pow(theta, -2.0 * j / rotary_dim);
    if (!stretch) {
      out[j] = (float)f;
      continue;
    }
    const double ramp = std::min(std::max((j - lo) / std::max(hi - lo, 0.001), 0.0), 1.0);
    out[j] = (float)(f / factor * ramp + f * (1.0 - ramp));
  }
  return stretch ? (float)(0.1 * std::log(factor) + 1.0) : 1.0f;
}

void rotary_linear_frequencies(double theta, int rotary_dim, double factor, float* out) {
  for (int j = 0; j < rotary_dim / 2; ++j) out[j] = (float)(std::pow(theta, -2.0 * j / rotary_dim) / factor);
}

static int bucket(int n) {      // the smallest of 1, 2, 3, 4, 6, 8, 12, 16, ... that is at least n
  for (int b = 1;; b *= 2) {
    if (b >= n) return b;
    if (b >= 2 && b + b / 2 >= n) return b + b / 2;
  }
}

int graph_row_bucket(int rows) { return rows > 512 ? rows : bucket(std::max(rows, 1)); }
int graph_width_bucket(int pages) { return 8 * bucket((std::max(pages, 1) + 7) / 8); }

}  // namespace vosti
