// Entry points of the quantization graph passes and of entropy calibration.
#ifndef MXQ_GRAPH_PASS_H_
#define MXQ_GRAPH_PASS_H_

#include <map>
#include <set>
#include <string>
#include <utility>
#include <vector>

#include "mxq_graph.h"

namespace mxq_graph {

// The graph attributes MXQuantizeSymbol attaches before running the pass
// (src/c_api/c_api_symbolic.cc:936-957).
struct QuantizeOptions {
  std::set<std::string> excluded_nodes;  // node names
  std::set<std::string> excluded_ops;    // float operator names
  std::set<std::string> offline_params;  // variables quantized ahead of time
  std::string quantized_dtype = "int8";  // out_type of the inserted quantize / requantize
  std::string quantize_mode = "smart";   // "full" or "smart"
  std::string quantize_granularity = "tensor-wise";
  int dev_type = 2;                      // Context::DeviceType: 1 cpu, 2 gpu
};

struct QuantizeResult {
  Graph graph;
  std::vector<std::string> calib_nodes;
};

QuantizeResult QuantizeGraph(const Graph& src, const QuantizeOptions& opt);
Graph SetCalibTable(const Graph& g, const std::map<std::string, std::pair<float, float>>& table);

// _contrib_calibrate_entropy (src/operator/quantization/calibrate.cc:89-186): the
// threshold whose clipped and re-quantized histogram is closest (KL divergence) to the
// observed one.  hist has an odd number of bins, hist_edges one more entry.
void CalibrateEntropy(const float* hist, const float* hist_edges, size_t num_bins,
                      int num_quantized_bins, float* threshold, float* divergence);

}  // namespace mxq_graph

#endif  // MXQ_GRAPH_PASS_H_
