// The several-workgroups-per-row kernels for one element type: launches without top-k rows, and
// the multinomial rows' five launches.
#include "ets_split_launch.h"

namespace ets_host {

ets_status launch_split_f32(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream, bool topk_rows) {
  return topk_rows ? launch_split_topk_f32(s, p, rows, stream) : launch_split<ets::kDtypeFloat, false>(s, p, rows, stream);
}

ets_status launch_split_walk_f32(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream) {
  return launch_split_walk<ets::kDtypeFloat>(s, p, rows, stream);
}

}  // namespace ets_host
