// sample_rows_kernel for one element type (a translation unit per type: they compile side by side).
#include "ets_rows_launch.h"

namespace ets_host {

ets_status launch_rows_f32(ets_sampler* s, const ets::RowParams& p, int32_t batch, hipStream_t stream, int draw) {
  return launch_rows<ets::kDtypeFloat>(s, p, batch, stream, draw);
}

}  // namespace ets_host
