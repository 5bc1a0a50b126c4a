// Launch of sample_rows_kernel (one workgroup per row) for one element type; included by the
// translation unit of that type.
#pragma once

#include "ets_host.h"

namespace ets_host {

template <int DT, bool ALIGNED, int DRAW, bool LOOP>
ets_status launch_rows_looped(ets_sampler* s, const ets::RowParams& p, int grid, hipStream_t stream) {
  static std::atomic<size_t> set_bytes[kMaxDevices];
  const size_t lds = s->lds_bytes;
  ets_status st = allow_dynamic_lds(s, reinterpret_cast<const void*>(&ets::sample_rows_kernel<DT, ALIGNED, DRAW, LOOP>), lds, set_bytes);
  if (st != ETS_OK) return st;
  hipLaunchKernelGGL((ets::sample_rows_kernel<DT, ALIGNED, DRAW, LOOP>), dim3(grid), dim3(ets::kBlock), lds, stream, p);
  ETS_HIP(s, hipGetLastError());
  return ETS_OK;
}

template <int DT, bool ALIGNED, int DRAW>
ets_status launch_rows_impl(ets_sampler* s, const ets::RowParams& p_in, int32_t batch, hipStream_t stream) {
  ets::RowParams p = p_in;
  p.rows = batch;
  p.ticket = (s->wb ? s->wb->tickets : s->d_tickets) + DRAW;
  // a workgroup per row while the scratch rows last; beyond that the rows are handed out by ticket
  return batch > p.grid_cap ? launch_rows_looped<DT, ALIGNED, DRAW, true>(s, p, p.grid_cap, stream)
                            : launch_rows_looped<DT, ALIGNED, DRAW, false>(s, p, batch, stream);
}

template <int DT>
ets_status launch_rows(ets_sampler* s, const ets::RowParams& p, int32_t batch, hipStream_t stream, int draw) {
  // 128-bit loads need a 16-byte aligned base and row pitch
  const size_t esz = ets::ElemSize<DT>::value;
  const bool aligned = (reinterpret_cast<uintptr_t>(p.logits) % 16 == 0) && ((static_cast<size_t>(p.row_stride) * esz) % 16 == 0);
  // one kernel instantiation per draw
  const bool use_topk = draw == ets::kDrawTopK;
  const bool use_mult = draw == ets::kDrawMultinomial;
  if (draw == ets::kDrawAny) {
    // rows of different draws in one launch (the looping instantiation serves every batch size)
    ets::RowParams q = p;
    q.rows = batch;
    q.ticket = (s->wb ? s->wb->tickets : s->d_tickets) + 4;  // (0 .. 2: the launches of one draw, 3: the finish kernel)
    const int grid = batch < q.grid_cap ? batch : q.grid_cap;
    return aligned ? launch_rows_looped<DT, true, ets::kDrawAny, true>(s, q, grid, stream)
                   : launch_rows_looped<DT, false, ets::kDrawAny, true>(s, q, grid, stream);
  }
  if (use_topk) {
    return aligned ? launch_rows_impl<DT, true, ets::kDrawTopK>(s, p, batch, stream)
                   : launch_rows_impl<DT, false, ets::kDrawTopK>(s, p, batch, stream);
  }
  if (use_mult) {
    return aligned ? launch_rows_impl<DT, true, ets::kDrawMultinomial>(s, p, batch, stream)
                   : launch_rows_impl<DT, false, ets::kDrawMultinomial>(s, p, batch, stream);
  }
  return aligned ? launch_rows_impl<DT, true, ets::kDrawTopP>(s, p, batch, stream)
                 : launch_rows_impl<DT, false, ets::kDrawTopP>(s, p, batch, stream);
}

}  // namespace ets_host
