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

static int bucket(int n) {      // the smallest of 1, 2, 3, 4, 6, 8, 12, 16, ... that is at least n
  for (int b = 1;; b *= 2) {
    if (b >= n) return b;
    if (b >= 2 && b + b / 2 >= n) return b + b / 2;
  }
}

int graph_row_bucket(int rows) { return rows > 512 ? rows : bucket(std::max(rows, 1)); }
int graph_width_bucket(int pages) { return 8 * bucket((std::max(pages, 1) + 7) / 8); }

}  // namespace vosti
