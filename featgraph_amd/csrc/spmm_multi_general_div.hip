// The several-rows-per-wave SpMM kernel as the generalised operator with the message FG_MSG_DIV (three reducers, tiles
// of 16, 32 and 64 floats).
#include "spmm_multi_kernel.hpp"

namespace fg {

int spmm_multi_general_div(const SpmmArgs &a, int64_t blocks, hipStream_t stream) {
  return launch_multi_general<FG_MSG_DIV>(a, blocks, stream);
}

}  // namespace fg
