// Rules that every host of the kernels follows, written once: the native engine calls them directly, the
// Python package through the host library's C interface.  Two hosts that each computed them their own way
// could differ in a last bit (of a rotation frequency) or in a bucket's border, and with them the logits or
// the recorded graphs.
#pragma once

namespace vosti {

// inv_freq[j] = 1 / theta^(2j / rotary_dim), j < rotary_dim / 2, as 32-bit values
// (python/vosti_kernels/rotary.py:80-90 writes 1.0 / (theta ** (arange(0, D, 2).float() / D)) in 32-bit).  The
// exponent is the 32-bit quotient; the power is the 32-bit number nearest to the exact power of the 32-bit
// theta and exponent (computed in 64-bit, then rounded once), so that it does not depend on whose powf runs;
// the reciprocal is a 32-bit division.
void rotary_inverse_frequencies(double theta, int rotary_dim, float* out);

// Recorded decode steps have one of 1, 2, 3, 4, 6, 8, 12, 16, 24, ... rows (a step with fewer is filled up with
// rows that read one key and store nothing; the reference pads its graphs likewise,
// python/vosti_kernels/graph_overlay.py:177-389), and block tables one of these numbers times eight pages, so
// that a long generation walks through few recordings.  More than 512 rows are recorded as they are.
int graph_row_bucket(int rows);
int graph_width_bucket(int pages);

// Recorded graphs kept; the least recently replayed one goes first.
constexpr int kMaxGraphs = 24;

}  // namespace vosti
