// The several-workgroups-per-row kernels for one element type: launches in which some row has a top-k.
#include "ets_split_launch.h"

namespace ets_host {

ets_status launch_split_topk_bf16(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream) {
  return launch_split<ets::kDtypeBFloat16, true>(s, p, rows, stream);
}

}  // namespace ets_host
