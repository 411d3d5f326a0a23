#include "graph.h"

namespace wkf {

TensorData Resolver::run_matmul(const NodeP&) { throw Error(WKF_ERR_UNSUPPORTED, "mat_mul: not built yet"); }

}  // namespace wkf
