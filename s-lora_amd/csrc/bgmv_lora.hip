// Decode shrink and expand of the same projections in one launch (see the comment in front
// of LoraArgs).  A file of its own so that it compiles next to bgmv_decode.hip, whose device
// code it shares through bgmv_device.hpp.
//
// Replaces the back-to-back dispatch_bgmv pairs of
// slora/models/peft/lora_unordered_batch_infer.py:267-273, 287-293, 307-313, 438-444.

#include "bgmv_device.hpp"

namespace slora {
namespace {

// ---------------------------------------------------------------------------
// shrink and expand of the same projections in ONE launch
// ---------------------------------------------------------------------------
// The reference issues shrink and expand of a projection back to back
// (slora/models/peft/lora_unordered_batch_infer.py:267-273): two launches, the second of
// which cannot start before the first has drained.  Here one workgroup per item does both
// halves of its item: the shrink of its 8 rows (shrink_body, unchanged), then the 8 pages of
// B^T with the same page ids (expand_body, unchanged: wavefront w takes pages w and w + 4).
// An expand page needs the whole delta row of its run, i.e. the rows of ALL items of the run
// (rank / 8 workgroups): the hand-over between them is one counter per (run, projection)
// behind the plan.  A workgroup stores its rows with device-scope stores, waits for them,
// counts itself in and polls until the run's `need` workgroups of this launch have done so;
// then it reads the rows with device-scope loads.  The counter is never reset: it grows by
// `need` per launch, launches on one plan do not overlap, so the value a workgroup's own
// increment returns tells which launch this is ((old / need + 1) * need is the count to wait
// for).  Producers and consumers are the same workgroups, and the items of a run are
// neighbours in their XCD's queue: workgroups are handed out in index order, so whoever a
// workgroup waits for is resident or about to be as soon as anything finishes.  The wait is
// bounded all the same (spin_limit polls, then a sticky flag in the counters' header and the
// workgroup goes on) so that no wavefront can wait for ever.
struct LoraArgs {
  ShrinkArgs s;
  ExpandArgs e;
  int* sync;       // the plan's counters
  int rank_cap;    // of the plan: a run has ceil(min(rank, rank_cap) / 8) items
  int spin_limit;  // polls after which a waiting workgroup gives up
};

// First half of the hand-over, called by all threads of the workgroup after its shrink rows
// are stored: waits for the stores, meets, counts the workgroup in.  Returns (in wavefront 0)
// the count to wait for; 0 if the run has no other workgroup.
__device__ __forceinline__ int lora_arrive(const LoraArgs& p, const Item& it, int proj_abs) {
  const int listed = it.r < p.rank_cap ? it.r : p.rank_cap;
  const int need = (listed + kRB - 1) / kRB;
  // wait until the stores of this wavefront are acknowledged (vmcnt(0); a workgroup-scope fence
  // alone need not wait for global stores), i.e. have reached the level the other workgroups read from
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  int target = 0;
  if (need > 1 && threadIdx.x == 0) {
    int* cnt = p.sync + kSyncHeader + ((int64_t)it.tok[0] * 4 + proj_abs);
    const int old = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    target = (old / need + 1) * need;
  }
  return target;
}

// Second half: wavefront 0 polls until the run's workgroups of this launch have all counted
// in (bounded), then the workgroup meets again.
__device__ __forceinline__ void lora_wait(const LoraArgs& p, const Item& it, int proj_abs, int target) {
  if (threadIdx.x < kWave) {
    target = __builtin_amdgcn_readfirstlane(target);
    if (target != 0) {
      const int* cnt = p.sync + kSyncHeader + ((int64_t)it.tok[0] * 4 + proj_abs);
      int spins = 0;
      while (__hip_atomic_load(cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - target < 0) {
        if (++spins > p.spin_limit) {  // never expected; leaves a mark instead of waiting for ever
          if (threadIdx.x == 0) {
            p.sync[SY_TIMEOUT] = 1;
            __hip_atomic_fetch_or(const_cast<int*>(p.s.plan) + PH_STATUS, kPlanStatusTimeout, __ATOMIC_RELAXED,
                                  __HIP_MEMORY_SCOPE_AGENT);
          }
          break;
        }
        __builtin_amdgcn_s_sleep(4);
      }
    }
  }
  __syncthreads();
  // the rows are read with device-scope loads; keep them behind the wait
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

template <typename T, int NV>
__device__ __forceinline__ int lora_body(const LoraArgs& p, int unit, int proj, u32x4* s_x, uint16_t* s_strip) {
  Item it;
  const int n_items = shrink_body<T, true, NV, true>(p.s, unit, proj, s_x, it);
  if (it.n_tok <= 0) return n_items;  // no such item (uniform over the workgroup)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int proj_abs = p.s.qkvo0 + proj;
  const int r = it.r;
  const ExpandArgs& e = p.e;
  // The usual case in straight-line code: both pages of this wavefront (w and w + 4 of the item's
  // block) are whole one-pass pages inside the output, on the vector path.  Their loads and the y
  // values go out between the two halves of the hand-over, so they are in flight while it completes.
  const bool fast = (r & (r - 1)) == 0 && r >= 8 && r <= 128 && r <= e.x_cols && it.more == 0 && (e.x_cols & 7) == 0 &&
                    e.page_elems == ExpandPass<NV>::kElems && e.pages_shift[proj] == -1 && (e.h_out[proj] & 7) == 0 &&
                    e.y_aligned != 0;
  const int target = lora_arrive(p, it, proj_abs);
  if (!fast) {
    lora_wait(p, it, proj_abs, target);
    expand_body<T, 1, true, NV, true>(e, unit, proj * 2, s_strip);
    expand_body<T, 1, true, NV, true>(e, unit, proj * 2 + 1, s_strip);
    return n_items;
  }
  const int lg_r = __builtin_ctz((unsigned)r);
  const int h_stride = e.h_out[proj];
  const uint16_t* y = reinterpret_cast<const uint16_t*>(e.y[proj]);
  typedef const int __attribute__((address_space(4))) * ConstWords;
  ConstWords rec = (ConstWords)p.s.plan + kPlanHeaderWords + (int64_t)unit * kItemWords;
  int pg[2];
  u32x4 wv[2][NV], yv[2][kTT];
  int n_page0[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    pg[i] = rec[IT_PAGES + proj_abs * kRB + wave + 4 * i];
    const uint16_t* wpage = reinterpret_cast<const uint16_t*>(e.w) + (int64_t)(pg[i] >= 0 ? pg[i] : 0) * e.page_elems;
#pragma unroll
    for (int c = 0; c < NV; ++c) wv[i][c] = ldg16_stream(wpage + (c * kWave + lane) * 8);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int k = it.j0 + wave + 4 * i;
    n_page0[i] = (int)(((int64_t)k * e.page_elems) >> lg_r);
    const bool y_ok = lane * 8 < (ExpandPass<NV>::kElems >> lg_r);
#pragma unroll
    for (int t = 0; t < kTT; ++t)  // lanes with no outputs re-read the page's first ones; the values are not used
      yv[i][t] = ldg16_stream(y + (int64_t)(t < it.n_tok ? it.tok[t] : it.tok[0]) * h_stride +
                              (y_ok ? n_page0[i] + lane * 8 : n_page0[i]));
  }
  const float scale = load_scale(e.scales, e.scales_dtype, it.a);
  lora_wait(p, it, proj_abs, target);
  const int d0 = (lane & ((r >> 3) - 1)) * 8;
  const uint16_t* x = reinterpret_cast<const uint16_t*>(e.x[proj]);
  u32x4 xv[kTT];
#pragma unroll
  for (int t = 0; t < kTT; ++t)
    xv[t] = ldg16_coherent(x + (int64_t)(t < it.n_tok ? it.tok[t] : it.tok[0]) * e.x_cols + d0);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    if (pg[i] >= 0)
      expand_update<T, NV>(e, proj, it, lg_r, wv[i], xv, yv[i], n_page0[i], h_stride, scale, s_strip);
  }
  return n_items;
}

// Grid: x = item, y = projection of the launch.  LDS: the shrink's staging area (dynamic) and a
// strip per wavefront for the expand.
template <typename T, int NV>
__global__ __launch_bounds__(256, NV > 8 ? 3 : 4) void bgmv_lora_kernel(const LoraArgs p) {
  extern __shared__ u32x4 s_x[];  // [lds_tt][h_in / 8]
  __shared__ __align__(16) uint16_t s_out[4][ExpandPass<NV>::kStrip];
  int unit = (int)blockIdx.x;
  const int n_items = lora_body<T, NV>(p, unit, (int)blockIdx.y, s_x, s_out[threadIdx.x >> 6]);
  if (p.s.strided) {  // the items beyond the grid, if the batch has that many
    for (unit += (int)gridDim.x; unit < n_items; unit += (int)gridDim.x) {
      __syncthreads();  // the staging area of the item before is free
      lora_body<T, NV>(p, unit, (int)blockIdx.y, s_x, s_out[threadIdx.x >> 6]);
    }
  }
}

template <typename T, int NV>
int launch_lora_nv(const LoraArgs& p, int64_t grid, int nproj, size_t lds, hipStream_t stream) {
  auto kernel = bgmv_lora_kernel<T, NV>;
  static PerDeviceOnce once;
  if (lds > 48 * 1024 && !raise_dynamic_lds(reinterpret_cast<const void*>(kernel), 128 * 1024, once))
    return SLORA_ERR_LAUNCH;
  hipLaunchKernelGGL(kernel, dim3((uint32_t)grid, (uint32_t)nproj), dim3(256), lds, stream, p);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

template <typename T>
int launch_lora(LoraArgs p, int64_t grid, int nproj, hipStream_t stream) {
  if (grid <= 0) return SLORA_OK;
  if (grid > 0x7fffffffLL / 8) return SLORA_ERR_UNSUPPORTED;
  const size_t row_bytes = (size_t)p.s.h_in * 2;
  int tt = kTT;
  while (tt > 1 && tt * row_bytes > 64 * 1024) --tt;
  const size_t lds = tt * row_bytes;
  if (lds > 128 * 1024 - 8 * 1024) return SLORA_ERR_UNSUPPORTED;
  p.s.lds_tt = tt;
  p.e.n_units = (int)grid;
  p.e.interleave = 0;
  // Only the 4096-element pass is instantiated: wider pages take the same kernel's general paths
  // (several passes per page), correct and slower.
  return launch_lora_nv<T, 8>(p, grid, nproj, lds, stream);
}

int lora_common(const void* plan, int64_t n_items, int64_t rank_cap, void* const y[3], void* const delta[3],
                const int64_t h_out[3], int nproj, int qkvo0, const void* x, const void* wa, const void* wb,
                const slora_tables* tables, const int64_t* bins, const void* scales, int scales_dtype, int64_t batch,
                int64_t h_in, int64_t delta_cols, int64_t page_elems, int64_t n_pages, int dtype, void* stream) {
  LoraArgs p{};
  int64_t grid_s = 0, grid_e = 0;
  int rc = shrink_prepare(plan, n_items, rank_cap, delta, nproj, qkvo0, x, wa, tables, bins, batch, h_in, delta_cols,
                          page_elems, n_pages, dtype, p.s, grid_s);
  if (rc != SLORA_OK) return rc == kNothingToDo ? SLORA_OK : rc;
  const void* xs[3] = {delta[0], delta[1], delta[2]};
  rc = expand_prepare(plan, n_items, rank_cap, y, xs, h_out, nproj, qkvo0, wb, tables, bins, scales, scales_dtype,
                      batch, delta_cols, page_elems, n_pages, dtype, p.e, grid_e);
  if (rc == kNothingToDo)  // no output to update: the shrink half alone
    return slora_bgmv_shrink_planned(plan, rank_cap, n_items, nproj, delta[0], delta[1], delta[2], x, wa, tables, bins,
                                     batch, h_in, delta_cols, page_elems, n_pages, qkvo0, dtype, stream);
  if (rc != SLORA_OK) return rc;
  if (grid_s != grid_e) return SLORA_ERR_BAD_SHAPE;
  // the delta rows are read 8 bytes at a time by device-scope loads
  if ((delta_cols & 7) != 0) return SLORA_ERR_UNSUPPORTED;
  p.sync = const_cast<int*>(static_cast<const int*>(plan)) + plan_sync_offset(batch, rank_cap);
  p.rank_cap = (int)rank_cap;
  p.spin_limit = 1 << 16;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  return dtype == SLORA_DTYPE_F16 ? launch_lora<F16>(p, grid_s, nproj, s) : launch_lora<BF16>(p, grid_s, nproj, s);
}

}  // namespace
}  // namespace slora

extern "C" {

int slora_bgmv_lora_planned(void* plan, int64_t rank_cap, int64_t n_items, int nproj, void* y0, void* y1, void* y2,
                            void* delta0, void* delta1, void* delta2, const void* x, const void* w_a, const void* w_b,
                            const slora_tables* tables, const int64_t* bins, const void* scales, int scales_dtype,
                            int64_t batch, int64_t h_in, int64_t delta_cols, int64_t h_out0, int64_t h_out1,
                            int64_t h_out2, int64_t page_elems, int64_t n_pages, int qkvo, int dtype, void* stream) {
  if (plan == nullptr) return SLORA_ERR_NULL_POINTER;
  if (rank_cap <= 0 || rank_cap > SLORA_MAX_RANK) return SLORA_ERR_BAD_SHAPE;
  if (nproj != 1 && nproj != 3) return SLORA_ERR_BAD_SHAPE;
  if (nproj == 3 && qkvo != 0) return SLORA_ERR_BAD_SHAPE;
  if (nproj == 1 && (qkvo < 0 || qkvo > 3)) return SLORA_ERR_BAD_SHAPE;
  void* ys[3] = {y0, y1, y2};
  void* ds[3] = {delta0, delta1, delta2};
  const int64_t hs[3] = {h_out0, h_out1, h_out2};
  return slora::lora_common(plan, n_items, rank_cap, ys, ds, hs, nproj, qkvo, x, w_a, w_b, tables, bins, scales,
                            scales_dtype, batch, h_in, delta_cols, page_elems, n_pages, dtype, stream);
}

}  // extern "C"
