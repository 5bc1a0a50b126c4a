// Launches of the several-workgroups-per-row kernels (ets_split.h) for one element type; included
// by the translation units of that type.
#pragma once

#include <cstdlib>

#include "ets_host.h"

namespace ets_host {

// Top-k launches are compiled in translation units of their own.
ets_status launch_split_topk_f32(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream);
ets_status launch_split_topk_f16(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream);
ets_status launch_split_topk_bf16(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream);

template <int DT>
void launch_split_pass1(const ets::SplitParams& sp, int32_t rows, hipStream_t stream) {
  if (rows <= 256) {
    const int per_block = (ets::kPass1Block / 64) * 2;
    hipLaunchKernelGGL((ets::split_pass1_kernel<DT, 2>), dim3((sp.ns + per_block - 1) / per_block, rows), dim3(ets::kPass1Block),
                       0, stream, sp);
  } else {
    const int per_block = (ets::kPass1Block / 64) * 4;
    hipLaunchKernelGGL((ets::split_pass1_kernel<DT, 4>), dim3((sp.ns + per_block - 1) / per_block, rows), dim3(ets::kPass1Block),
                       0, stream, sp);
  }
}

// A call that brings its own work buffers laid them out for at most max_row_wgs workgroups per row.
inline ets_status check_row_wgs(ets_sampler* s, int row_wgs) {
  if (s->wb && row_wgs > s->wb->max_row_wgs)
    return fail(s, ETS_INTERNAL, "more workgroups per row than the call's work buffers were laid out for");
  return ETS_OK;
}

// Whether a launch of `rows` rows may run pass 1 inside pass 2 (every workgroup resident at once, a wave's
// slots in its registers, finite temperatures, nothing beside it on another stream, room for the records
// that the workgroups hand to each other); `spin_limit`: how often a workgroup reads the others' records
// before it works their slots out itself.  ETS_FUSE=0 switches it off, ETS_FUSE_SPIN_LIMIT sets the limit
// (read at every launch, so that a test can switch between them inside one process).
inline bool fused_launch_fits(const ets_sampler* s, const ets::SplitParams& sp, const ets::RowParams& p, int32_t rows, int32_t* spin_limit) {
  const char* const fuse_text = std::getenv("ETS_FUSE");
  const int fuse_env = fuse_text ? std::atoi(fuse_text) : 1;
  const char* const spin_text = std::getenv("ETS_FUSE_SPIN_LIMIT");
  // (256 reads are about 0.4 ms: the usual wait is a read or two, and a launch whose workgroups cannot all be
  // resident -- another launch of the same kind on another stream holds the compute units -- should not stall
  // for long before its workgroups help themselves, which costs them some twenty microseconds)
  const int spin_env = spin_text ? std::atoi(spin_text) : 256;
  *spin_limit = spin_env < 0 ? 0 : spin_env;
  const int per_wg_slots = ((sp.ns + sp.row_wgs - 1) / sp.row_wgs + ets::kWaves - 1) / ets::kWaves * ets::kWaves;
  const float abs_inv = p.inv_temperature < 0.0f ? -p.inv_temperature : p.inv_temperature;
  // (rows with parameters of their own: the caller has looked at their temperatures)
  const bool inv_ordinary = p.row_cfg ? s->cfg_inv_ordinary : abs_inv < 3.0e38f;
  return fuse_env != 0 && inv_ordinary && s->beside_rows == 0 && sp.arrive != nullptr &&
         static_cast<int64_t>(rows) * sp.row_wgs <= (s->num_cus > 0 ? s->num_cus : 0) && per_wg_slots <= ets::kFusedSlots * ets::kWaves &&
         (!s->wb || static_cast<size_t>(rows) * sp.ns_stride * sizeof(float4) <= s->wb->pack_bytes);
}

// The three launches for top-p (and, with TOPK, top-k) rows.
// TOPK: some row may be a top-k row (the kernels of a launch without one leave that case out).
template <int DT, bool TOPK>
ets_status launch_split(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream) {
  ets_status st = ETS_OK;
  constexpr bool k16 = DT == ets::kDtypeBFloat16 || DT == ets::kDtypeHalf;
  if (!s->wb) {
    st = ensure_split(s);
    if (st != ETS_OK) return st;
    if (k16) {
      st = ensure_phist(s);
      if (st != ETS_OK) return st;
    }
  }
  ets::SplitParams sp = s->wb ? s->wb->split : s->split;
  sp.row = p;
  sp.row.rows = rows;
  sp.row.ticket = (s->wb ? s->wb->tickets : s->d_tickets) + 3;  // (0 .. 2 are the one-workgroup-per-row kernel's, by draw)
  sp.phist_words = DT == ets::kDtypeBFloat16 ? kPhistWordsBFloat16 : (DT == ets::kDtypeHalf ? kPhistWordsHalf : 0);
  sp.row_wgs = pass2_workgroups(s, rows, sp.ns, s->beside_rows);
  st = check_row_wgs(s, sp.row_wgs);
  if (st != ETS_OK) return st;
  sp.list_region = list_region(sp.ns, sp.row_wgs);
  static const int short_lists = [] {
    const char* e = std::getenv("ETS_SHORT_LISTS");  // 0: pass 2 lists every possible candidate, always
    return e ? std::atoi(e) : 1;
  }();
  sp.short_lists = short_lists;
  const size_t lut_bytes = (DT == ets::kDtypeBFloat16 ? sizeof(float) * ets::kLutCountWords : 0) + sizeof(uint32_t) * sp.phist_words;
  // (a launch that neither writes the probabilities nor fills the phase clocks runs kernels without those branches)
  const bool extras = sp.timers != nullptr || p.probs != nullptr;
  // Pass 1 inside pass 2 (one read of the logits, one launch fewer): plain top-p launches that fit
  // (fused_launch_fits) and ask for neither probabilities nor debug records.
  int32_t spin_limit = 0;
  const bool fused = (!extras || (ETS_PHASE_CLOCKS && p.probs == nullptr)) && fused_launch_fits(s, sp, p, rows, &spin_limit);
  bool* dirty = arrive_dirty_flag(s);
  if (fused) {
    {
      if (*dirty) {
        hipLaunchKernelGGL(ets::split_launch_number_kernel<DT>, dim3(1), dim3(64), 0, stream, sp.arrive);
        ETS_HIP(s, hipGetLastError());
      }
      *dirty = true;  // (until this call's finish kernel, which numbers the next launch, has been launched)
      sp.spin_limit = spin_limit;
      static std::atomic<size_t> set_bytes_f[kMaxDevices];
      constexpr bool kClocks = ETS_PHASE_CLOCKS != 0;  // (a profiling build: the fused kernel with its phase clocks)
      st = allow_dynamic_lds(s, reinterpret_cast<const void*>(&ets::split_pass2_kernel<DT, true, false, TOPK, kClocks, true>), lut_bytes, set_bytes_f);
      if (st != ETS_OK) return st;
      hipLaunchKernelGGL((ets::split_pass2_kernel<DT, true, false, TOPK, kClocks, true>), dim3(sp.row_wgs * rows), dim3(ets::kBlock), lut_bytes,
                         stream, sp);
    }
  } else {
    launch_split_pass1<DT>(sp, rows, stream);
    ETS_HIP(s, hipGetLastError());
  }
  if (fused) {
  } else if (extras) {
    static std::atomic<size_t> set_bytes2[kMaxDevices];
    st = allow_dynamic_lds(s, reinterpret_cast<const void*>(&ets::split_pass2_kernel<DT, true, false, TOPK, true>), lut_bytes, set_bytes2);
    if (st != ETS_OK) return st;
    hipLaunchKernelGGL((ets::split_pass2_kernel<DT, true, false, TOPK, true>), dim3(sp.row_wgs, rows), dim3(ets::kBlock), lut_bytes,
                       stream, sp);
  } else {
    static std::atomic<size_t> set_bytes2[kMaxDevices];
    st = allow_dynamic_lds(s, reinterpret_cast<const void*>(&ets::split_pass2_kernel<DT, true, false, TOPK, false>), lut_bytes, set_bytes2);
    if (st != ETS_OK) return st;
    hipLaunchKernelGGL((ets::split_pass2_kernel<DT, true, false, TOPK, false>), dim3(sp.row_wgs, rows), dim3(ets::kBlock), lut_bytes,
                       stream, sp);
  }
  ETS_HIP(s, hipGetLastError());
  if (rows > p.grid_cap) {
    // more rows than workgroups: a workgroup takes up to kChainRows rows at a time
    static const int chain_rows_max = [] {
      const char* e = std::getenv("ETS_CHAIN_ROWS");
      const int v = e ? std::atoi(e) : ets::kChainRows;
      return v < 1 ? 1 : (v > ets::kChainRows ? ets::kChainRows : v);
    }();
    const int per_wg = (rows + p.grid_cap - 1) / p.grid_cap;
    sp.chain_rows = per_wg < chain_rows_max ? per_wg : chain_rows_max;
    // every row of a unit needs room for its records and at least one prepared slot in its share of the key buffer
    const int by_lds = static_cast<int>(s->lds_bytes / (ets::chain_rec_bytes(sp.ns) + sizeof(ets::PrepSlot)));
    if (sp.chain_rows > by_lds) sp.chain_rows = by_lds < 1 ? 1 : by_lds;
    const int units = (rows + sp.chain_rows - 1) / sp.chain_rows;
    const dim3 grid(units < p.grid_cap ? units : p.grid_cap);
    if (extras) {
      static std::atomic<size_t> set_bytes[kMaxDevices];
      st = allow_dynamic_lds(s, reinterpret_cast<const void*>(&ets::split_finish_kernel<DT, true, TOPK, true>), s->lds_bytes, set_bytes);
      if (st != ETS_OK) return st;
      hipLaunchKernelGGL((ets::split_finish_kernel<DT, true, TOPK, true>), grid, dim3(ets::kBlock), s->lds_bytes, stream, sp);
    } else {
      static std::atomic<size_t> set_bytes[kMaxDevices];
      st = allow_dynamic_lds(s, reinterpret_cast<const void*>(&ets::split_finish_kernel<DT, true, TOPK, false>), s->lds_bytes, set_bytes);
      if (st != ETS_OK) return st;
      hipLaunchKernelGGL((ets::split_finish_kernel<DT, true, TOPK, false>), grid, dim3(ets::kBlock), s->lds_bytes, stream, sp);
    }
  } else {
    if (extras) {
      static std::atomic<size_t> set_bytes[kMaxDevices];
      st = allow_dynamic_lds(s, reinterpret_cast<const void*>(&ets::split_finish_kernel<DT, false, TOPK, true>), s->lds_bytes, set_bytes);
      if (st != ETS_OK) return st;
      hipLaunchKernelGGL((ets::split_finish_kernel<DT, false, TOPK, true>), dim3(rows), dim3(ets::kBlock), s->lds_bytes, stream, sp);
    } else {
      static std::atomic<size_t> set_bytes[kMaxDevices];
      st = allow_dynamic_lds(s, reinterpret_cast<const void*>(&ets::split_finish_kernel<DT, false, TOPK, false>), s->lds_bytes, set_bytes);
      if (st != ETS_OK) return st;
      hipLaunchKernelGGL((ets::split_finish_kernel<DT, false, TOPK, false>), dim3(rows), dim3(ets::kBlock), s->lds_bytes, stream, sp);
    }
  }
  ETS_HIP(s, hipGetLastError());
  if (fused) *dirty = false;
  return ETS_OK;
}

// Multinomial rows: five launches (ets_split.h, split_walk_kernel); four when pass 1 runs inside the first pass 2.
template <int DT>
ets_status launch_split_walk(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream) {
  ets_status st = ETS_OK;
  if (!s->wb) {
    st = ensure_split(s);
    if (st != ETS_OK) return st;
  }
  ets::SplitParams sp = s->wb ? s->wb->split : s->split;
  sp.row = p;
  sp.row.rows = rows;
  sp.phist_words = 0;
  sp.short_lists = 0;
  sp.row_wgs = pass2_workgroups(s, rows, sp.ns, s->beside_rows);
  st = check_row_wgs(s, sp.row_wgs);
  if (st != ETS_OK) return st;
  sp.list_region = 0;
  // (pass 1 inside the first pass 2 when the launch fits: four launches instead of five)
  int32_t spin_limit = 0;
  const bool fused = fused_launch_fits(s, sp, p, rows, &spin_limit);
  bool* dirty = arrive_dirty_flag(s);
  if (!fused) {
    launch_split_pass1<DT>(sp, rows, stream);
    ETS_HIP(s, hipGetLastError());
  }
  const size_t lut_bytes = DT == ets::kDtypeBFloat16 ? sizeof(float) * ets::kLutCountWords : 0;
  // the walk kernel's LDS: the row's records and as many prepared slots as fit beside them
  const uint32_t walk_lds = static_cast<uint32_t>(ets::chain_rec_bytes(sp.ns) + 16 * sizeof(ets::PrepSlot));
  static std::atomic<size_t> set_sum[kMaxDevices], set_walk[kMaxDevices], set_k0[kMaxDevices], set_k1[kMaxDevices];
  st = allow_dynamic_lds(s, reinterpret_cast<const void*>(&ets::split_pass2_kernel<DT, false, false>), lut_bytes, set_sum);
  if (st != ETS_OK) return st;
  st = allow_dynamic_lds(s, reinterpret_cast<const void*>(&ets::split_pass2_kernel<DT, false, true>), lut_bytes, set_walk);
  if (st != ETS_OK) return st;
  st = allow_dynamic_lds(s, reinterpret_cast<const void*>(&ets::split_walk_kernel<DT, 0>), walk_lds, set_k0);
  if (st != ETS_OK) return st;
  st = allow_dynamic_lds(s, reinterpret_cast<const void*>(&ets::split_walk_kernel<DT, 1>), walk_lds, set_k1);
  if (st != ETS_OK) return st;
  if (fused) {
    if (*dirty) {
      hipLaunchKernelGGL(ets::split_launch_number_kernel<DT>, dim3(1), dim3(64), 0, stream, sp.arrive);
      ETS_HIP(s, hipGetLastError());
    }
    *dirty = true;  // (until the first walk kernel, which numbers the next launch, has been launched)
    sp.spin_limit = spin_limit;
    static std::atomic<size_t> set_fused[kMaxDevices];
    st = allow_dynamic_lds(s, reinterpret_cast<const void*>(&ets::split_pass2_kernel<DT, false, false, false, true, true>), lut_bytes, set_fused);
    if (st != ETS_OK) return st;
    hipLaunchKernelGGL((ets::split_pass2_kernel<DT, false, false, false, true, true>), dim3(sp.row_wgs * rows), dim3(ets::kBlock), lut_bytes,
                       stream, sp);
  } else {
    hipLaunchKernelGGL((ets::split_pass2_kernel<DT, false, false>), dim3(sp.row_wgs, rows), dim3(ets::kBlock), lut_bytes, stream, sp);
  }
  ETS_HIP(s, hipGetLastError());
  hipLaunchKernelGGL((ets::split_walk_kernel<DT, 0>), dim3(rows), dim3(ets::kWalkBlock), walk_lds, stream, sp, walk_lds);
  ETS_HIP(s, hipGetLastError());
  if (fused) *dirty = false;
  hipLaunchKernelGGL((ets::split_pass2_kernel<DT, false, true>), dim3(sp.row_wgs, rows), dim3(ets::kBlock), lut_bytes, stream, sp);
  ETS_HIP(s, hipGetLastError());
  hipLaunchKernelGGL((ets::split_walk_kernel<DT, 1>), dim3(rows), dim3(ets::kWalkBlock), walk_lds, stream, sp, walk_lds);
  ETS_HIP(s, hipGetLastError());
  return ETS_OK;
}

}  // namespace ets_host
