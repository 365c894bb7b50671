// Entropy (KL-divergence) calibration: _contrib_calibrate_entropy of the reference
// (src/operator/quantization/calibrate.cc:33-186), called by the histogram collector
// (python/mxnet/contrib/quantization.py:262-285).  All arithmetic is binary32 in the
// reference's order of operations, so the chosen threshold is the same number.
#include <cmath>
#include <limits>
#include <numeric>
#include <vector>

#include "mxq_graph_pass.h"
#include "mxq_shim.h"

namespace mxq_graph {

namespace {

// Replaces zeros by eps and takes the same mass off the non-zero entries
// (calibrate.cc:33-64).  Empty result: the distribution is all zero, or has so many
// zeros that the correction would reach 1.
std::vector<float> Smooth(const std::vector<float>& p, const float eps = 0.0001f) {
  size_t zeros = 0;
  for (const float v : p) zeros += (v == 0.f);
  const size_t nonzeros = p.size() - zeros;
  if (nonzeros == 0) return {};
  const float eps1 = eps * static_cast<float>(zeros) / static_cast<float>(nonzeros);
  if (eps1 >= 1.0) return {};
  std::vector<float> out(p);
  for (size_t i = 0; i < p.size(); ++i) {
    // eps * is_zero - eps1 * is_nonzero with 0/1 flags, then one addition
    const float is_zero = p[i] == 0.f ? 1.f : 0.f, is_nonzero = p[i] != 0.f ? 1.f : 0.f;
    out[i] += eps * is_zero - eps1 * is_nonzero;
  }
  return out;
}

// KL(p || q) of the two histograms after normalising each (calibrate.cc:66-87).
float Divergence(std::vector<float> p, std::vector<float> q) {
  CHECK_EQ(p.size(), q.size());
  const float p_sum = std::accumulate(p.begin(), p.end(), 0.f);
  const float q_sum = std::accumulate(q.begin(), q.end(), 0.f);
  for (float& v : p) v = v / p_sum;
  for (float& v : q) v = v / q_sum;
  float kl = 0;
  for (size_t i = 0; i < p.size(); ++i) {
    CHECK(p[i] > 0 && q[i] > 0);
    kl += p[i] * std::log(p[i] / q[i]);
  }
  return kl;
}

}  // namespace

void CalibrateEntropy(const float* hist, const float* hist_edges, size_t num_bins,
                      int num_quantized_bins, float* threshold, float* divergence) {
  CHECK(num_bins % 2 == 1) << "the histogram needs an odd number of bins";
  CHECK(num_quantized_bins >= 1 && static_cast<size_t>(num_quantized_bins) <= num_bins)
      << "num_quantized_bins out of range";
  const long zero_bin = static_cast<long>(num_bins / 2);
  const long half_quantized = num_quantized_bins / 2;
  const size_t candidates = static_cast<size_t>(zero_bin + 1 - half_quantized);
  std::vector<float> thresholds(candidates, 0.f), divergences(candidates, 0.f);
  // candidate i keeps bins [zero_bin - i, zero_bin + i]; everything outside is folded
  // into the two edge bins of the reference distribution p
  for (long i = half_quantized; i <= zero_bin; ++i) {
    const size_t start = static_cast<size_t>(zero_bin - i), stop = static_cast<size_t>(zero_bin + i + 1);
    const size_t width = stop - start;
    thresholds[i - half_quantized] = hist_edges[stop];
    std::vector<size_t> sliced(width, 0);
    std::vector<float> p(width, 0.f);
    for (size_t j = 0; j < num_bins; ++j) {
      if (j <= start) {
        p[0] += hist[j];
      } else if (j >= stop) {
        p.back() += hist[j];
      } else {
        sliced[j - start] = static_cast<size_t>(hist[j]);
        p[j - start] = hist[j];
      }
    }
    // q: the kept bins merged into num_quantized_bins levels (the last level takes the
    // remainder), then spread back evenly over the non-empty bins of each level
    const size_t merged = width / static_cast<size_t>(num_quantized_bins);
    std::vector<float> level(num_quantized_bins, 0.f);
    for (int j = 0; j < num_quantized_bins; ++j) {
      long long s = 0;
      for (size_t k = j * merged; k < (j + 1) * merged; ++k) s += static_cast<long long>(sliced[k]);
      level[j] = static_cast<float>(static_cast<int>(s));
    }
    {
      long long s = 0;
      for (size_t k = num_quantized_bins * merged; k < width; ++k) s += static_cast<long long>(sliced[k]);
      level.back() += static_cast<float>(static_cast<int>(s));
    }
    std::vector<float> q(width, 0.f);
    for (int j = 0; j < num_quantized_bins; ++j) {
      const size_t lo = j * merged;
      const size_t hi = (j == num_quantized_bins - 1) ? width : (j + 1) * merged;
      int nonempty = 0;
      for (size_t k = lo; k < hi; ++k) nonempty += sliced[k] != 0;
      if (nonempty == 0) continue;
      for (size_t k = lo; k < hi; ++k)
        if (p[k]) q[k] = level[j] / nonempty;
    }
    const std::vector<float> ps = Smooth(p), qs = Smooth(q);
    divergences[i - half_quantized] =
        qs.empty() ? std::numeric_limits<float>::infinity() : Divergence(ps, qs);
  }
  size_t best = 0;
  float best_divergence = std::numeric_limits<float>::max();
  for (size_t i = 0; i < divergences.size(); ++i) {
    if (divergences[i] < best_divergence) {
      best_divergence = divergences[i];
      best = i;
    }
  }
  *divergence = best_divergence;
  *threshold = thresholds[best];
}

}  // namespace mxq_graph
