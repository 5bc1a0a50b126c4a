// The several-workgroups-per-row kernels for one element type: launches without top-k rows, and
// the multinomial rows' five launches.
#include "ets_split_launch.h"

namespace ets_host {

ets_status launch_split_bf16(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream, bool topk_rows) {
  return topk_rows ? launch_split_topk_bf16(s, p, rows, stream) : launch_split<ets::kDtypeBFloat16, false>(s, p, rows, stream);
}

ets_status launch_split_walk_bf16(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream) {
  return launch_split_walk<ets::kDtypeBFloat16>(s, p, rows, stream);
}

}  // namespace ets_host
