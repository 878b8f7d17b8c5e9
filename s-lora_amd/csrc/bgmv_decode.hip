// Decode-time batched gather matrix-vector products over the paged adapter
// pool: shrink (x[H] -> delta[r]) and expand (delta[r] -> y[H_out] +=).
//
// Both kernels are bandwidth kernels and, at decode sizes, latency kernels: a
// call moves a few tens of MB, so what counts is how many DEPENDENT memory
// round trips separate kernel start from the weight loads, and how many bytes
// are in flight at once.  The unit of work is one pool page per wavefront task
// (an A row for shrink, one page of the flattened B^T for expand): a wavefront
// issues all 16-byte loads of its pages before it waits for any.  A workgroup
// covers one "item": 8 consecutive rows/pages of the projection blocks of one
// "run" (up to kTT tokens that share an adapter, so the pages are fetched once
// for all of them); the run's activations are staged once in LDS.
//   single projection: 4 wavefronts x 2 pages;   q/k/v fused: 8 wavefronts x 3 pages.
//
// Two ways to find the items:
//  * stateless (dispatch_bgmv as the reference calls it): a workgroup per
//    (token, 8-row block); every wavefront scans the per-token adapter ids
//    itself (ballots, no barrier), then walks bins -> a_len/a_start -> a_loc ->
//    page: four dependent round trips, and blocks beyond the adapter's rank or
//    of tokens that do not lead a run exit;
//  * planned: slora_bgmv_plan_build() writes the item list (tokens and page
//    ids) once per batch; every later call launches exactly one workgroup per
//    item, reads the item in one round trip and goes straight to the weights.
//
// Replaces slora/csrc/bgmv/bgmv_impl.cuh:14-241 of the reference.

#include "bgmv_device.hpp"

namespace slora {
namespace {

// NV: the straight-line path of this instantiation holds pages of up to 512 * NV elements
// (8: hidden <= 4096; larger ones cost registers, so the host picks the smallest that fits)
template <typename T, bool PLANNED, int NV>
__global__ __launch_bounds__(256, NV == 8 ? 4 : 1) void bgmv_shrink_kernel(const ShrinkArgs p) {
  extern __shared__ u32x4 s_x[];  // [lds_tt][h_in / 8]
  int unit = (int)blockIdx.x;
  Item it;
  const int n_items = shrink_body<T, PLANNED, NV>(p, unit, (int)blockIdx.y, s_x, it);
  if (PLANNED && p.strided) {
    // a launch sized for a fraction of the plan's capacity: the items beyond the grid, if the
    // batch has that many, are walked here (uniform over the workgroup)
    for (unit += (int)gridDim.x; unit < n_items; unit += (int)gridDim.x) {
      __syncthreads();  // the staging area of the item before is free
      shrink_body<T, PLANNED, NV>(p, unit, (int)blockIdx.y, s_x, it);
    }
  }
}

// ---------------------------------------------------------------------------
// plan build: one workgroup
// ---------------------------------------------------------------------------
constexpr int kPlanThreads = 1024;
constexpr int kPlanWaves = kPlanThreads / kWave;

// exclusive prefix sum of `v` over the workgroup; *total receives the sum
__device__ __forceinline__ int block_exclusive_scan(int v, int* s_wave, int* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int inc = v;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const int up = __shfl_up(inc, o, kWave);
    if (lane >= o) inc += up;
  }
  if (lane == kWave - 1) s_wave[wave] = inc;
  __syncthreads();
  int before = 0, tot = 0;
  for (int wv = 0; wv < kPlanWaves; ++wv) {
    const int c = s_wave[wv];
    if (wv < wave) before += c;
    tot += c;
  }
  __syncthreads();
  *total = tot;
  return before + inc - v;
}

constexpr int kMaxLdsBins = 8192;  // adapter ids kept in LDS (larger batches read the rest from memory)
constexpr int kMaxLdsRuns = 2048;  // run descriptors kept in LDS

// Builds the item list.  Runs are sorted by adapter, then cut into 8 queues of
// equal work, one per XCD: consecutive workgroup ids go to the XCDs in turn, so
// queue q's k-th item is stored at index k*8 + q.  All items of a run, and all
// runs of an adapter (up to a cut), then execute on one XCD: the run's
// activations and an adapter's pages shared by several runs are fetched by a
// single L2.  Queues are padded to the longest with empty items.
__global__ __launch_bounds__(kPlanThreads) void bgmv_plan_kernel(int* __restrict__ plan, Tables t, int batch,
                                                                 int rank_cap, int max_items,
                                                                 int* __restrict__ scratch, int* __restrict__ sync,
                                                                 int sync_words) {
  __shared__ int s_bins[kMaxLdsBins];
  __shared__ int s_ra[kMaxLdsRuns], s_rb[kMaxLdsRuns], s_rn[kMaxLdsRuns];
  __shared__ int s_wave[kPlanWaves];
  __shared__ int s_max_rank, s_total;
  __shared__ int s_qstart[kXcds], s_qlen[kXcds];
  const int tid = threadIdx.x;
  for (int i = tid; i < sync_words; i += kPlanThreads) sync[i] = 0;
  if (tid == 0) {
    s_max_rank = 0;
    s_total = 0;
  }
  if (tid < kXcds) {
    s_qstart[tid] = 0x7fffffff;
    s_qlen[tid] = 0;
  }
  auto adapter_of = [&](int q) -> int {
    const int64_t a = t.bins[q];
    return ((uint64_t)a < (uint64_t)t.n_adapters && a <= 0x7fffffffLL) ? (int)a : -1;
  };
  for (int i = tid; i < batch && i < kMaxLdsBins; i += kPlanThreads) s_bins[i] = adapter_of(i);
  __syncthreads();
  auto bin_at = [&](int q) -> int { return q < kMaxLdsBins ? s_bins[q] : adapter_of(q); };

  // ---- runs, in token order ----
  int n_runs = 0;
  for (int b0 = 0; b0 < batch; b0 += kPlanThreads) {
    const int b = b0 + tid;
    bool leader = false;
    int a = -1, r = 0;
    if (b < batch) {
      a = bin_at(b);
      if (a >= 0) {
        int pos = 0;
        for (int q = 0; q < b; ++q) pos += (bin_at(q) == a) ? 1 : 0;
        const int64_t len = t.a_len[a];
        r = len > 0 ? (int)(len >> 2) : 0;
        leader = (pos % kTT) == 0 && r > 0;
      }
    }
    int tot = 0;
    const int idx = n_runs + block_exclusive_scan(leader ? 1 : 0, s_wave, &tot);
    if (leader) {
      const int r_listed = r < rank_cap ? r : rank_cap;
      const int n_it = (r_listed + kRB - 1) / kRB;
      int* sc = scratch + (int64_t)idx * SC_WORDS;
      sc[SC_ADAPTER] = a;
      sc[SC_TOKEN] = b;
      sc[SC_RANK] = r;
      sc[SC_ITEMS] = n_it;
      if (idx < kMaxLdsRuns) {
        s_ra[idx] = a;
        s_rb[idx] = b;
        s_rn[idx] = n_it;
      }
      atomicMax(&s_max_rank, r);
      atomicAdd(&s_total, n_it);
    }
    n_runs += tot;
  }
  __syncthreads();
  const int total = s_total;

  // ---- order by (adapter, token): work in front of every run, then its queue ----
  for (int rho = tid; rho < n_runs; rho += kPlanThreads) {
    int* sc = scratch + (int64_t)rho * SC_WORDS;
    const int a = sc[SC_ADAPTER], b = sc[SC_TOKEN], n = sc[SC_ITEMS];
    int before = 0;
    for (int o = 0; o < n_runs; ++o) {
      int oa, ob, on;
      if (o < kMaxLdsRuns) {
        oa = s_ra[o];
        ob = s_rb[o];
        on = s_rn[o];
      } else {
        const int* so = scratch + (int64_t)o * SC_WORDS;
        oa = so[SC_ADAPTER];
        ob = so[SC_TOKEN];
        on = so[SC_ITEMS];
      }
      if (oa < a || (oa == a && ob < b)) before += on;
    }
    int q = (int)(((int64_t)before * kXcds) / (total > 0 ? total : 1));
    if (q > kXcds - 1) q = kXcds - 1;
    sc[SC_WORK] = before;
    sc[SC_QUEUE] = q;
    atomicMin(&s_qstart[q], before);
    atomicAdd(&s_qlen[q], n);
  }
  __syncthreads();
  int max_len = 0;
  for (int q = 0; q < kXcds; ++q) max_len = s_qlen[q] > max_len ? s_qlen[q] : max_len;
  int n_items = kXcds * max_len;
  const bool overflow = n_items > max_items;  // cannot happen with the capacity slora_bgmv_plan_bytes() reserves
  if (overflow) n_items = 0;

  // ---- records: padding first, then every run's items ----
  for (int pos = tid; pos < n_items; pos += kPlanThreads) {
    if (pos / kXcds >= s_qlen[pos % kXcds]) {
      int* rec = plan + kPlanHeaderWords + (int64_t)pos * kItemWords;
      for (int q = 0; q < kItemWords; ++q) rec[q] = q >= IT_PAGES && q < IT_BASE ? -1 : 0;
    }
  }
  for (int rho = tid; rho < n_runs && !overflow; rho += kPlanThreads) {
    const int* sc = scratch + (int64_t)rho * SC_WORDS;
    const int a = sc[SC_ADAPTER], b = sc[SC_TOKEN], r = sc[SC_RANK], n_it = sc[SC_ITEMS];
    const int q = sc[SC_QUEUE];
    const int k0 = sc[SC_WORK] - s_qstart[q];
    const int64_t base = t.a_start[a];
    int toks[kTT];
    int n = 0;
    for (int c = b; c < batch && n < kTT; ++c)
      if (bin_at(c) == a) toks[n++] = c;
    for (int c = n; c < kTT; ++c) toks[c] = 0;
    for (int i = 0; i < n_it; ++i) {
      int* rec = plan + kPlanHeaderWords + ((int64_t)(k0 + i) * kXcds + q) * kItemWords;
      rec[IT_ADAPTER] = a;
      rec[IT_RANK] = r;
      rec[IT_NTOK] = n;
      rec[IT_J0] = i * kRB;
      for (int c = 0; c < kTT; ++c) rec[IT_TOK + c] = toks[c];
      rec[IT_BASE] = (int)(uint32_t)(uint64_t)base;
      rec[IT_BASE + 1] = (int)(uint32_t)((uint64_t)base >> 32);
      rec[IT_MORE] = (i == n_it - 1 && r > rank_cap) ? 1 : 0;
      for (int c = IT_MORE + 1; c < kItemWords; ++c) rec[c] = 0;
    }
  }
  __syncthreads();
  // ---- page ids: one thread per (item, projection), its 8 lookups in flight together ----
  for (int task = tid; task < n_items * 4; task += kPlanThreads) {
    const int item = task >> 2, proj = task & 3;
    int* rec = plan + kPlanHeaderWords + (int64_t)item * kItemWords;
    const int r = rec[IT_RANK], j0 = rec[IT_J0], n_tok = rec[IT_NTOK];
    const int64_t base = (int64_t)(((uint64_t)(uint32_t)rec[IT_BASE + 1] << 32) | (uint32_t)rec[IT_BASE]);
    int64_t pg[kRB];
#pragma unroll
    for (int jr = 0; jr < kRB; ++jr)
      pg[jr] = (n_tok > 0 && j0 + jr < r) ? lookup_page(t, base + (int64_t)proj * r + j0 + jr) : (int64_t)-1;
#pragma unroll
    for (int jr = 0; jr < kRB; ++jr)
      rec[IT_PAGES + proj * kRB + jr] = (pg[jr] >= 0 && pg[jr] <= 0x7fffffffLL) ? (int)pg[jr] : -1;
  }
  if (tid == 0) {
    plan[PH_MAGIC] = kPlanMagic;
    plan[PH_NITEMS] = n_items;
    plan[PH_MAXRANK] = s_max_rank;
    plan[PH_BATCH] = batch;
    plan[PH_TT] = kTT;
    plan[PH_RANKCAP] = rank_cap;
    plan[PH_NRUNS] = n_runs;
    plan[PH_STATUS] = 0;
  }
}

// The same plan for batches of up to kFastPlanBatch tokens, built by several
// workgroups.  Every workgroup derives the runs, their order and the queues by
// itself, entirely in LDS (the work is small and identical everywhere, so no
// exchange between workgroups is needed); the item records, which are most of the
// bytes and carry the page lookups, are then shared out: 16 lanes write one record
// as twelve 16-byte stores, eight of them holding four page ids each whose lookups
// are in flight together.
constexpr int kFastPlanBatch = 1024;

__global__ __launch_bounds__(kPlanThreads) void bgmv_plan_fast_kernel(int* __restrict__ plan, Tables t, int batch,
                                                                      int rank_cap, int max_items,
                                                                      int* __restrict__ sync, int sync_words) {
  __shared__ int s_bins[kFastPlanBatch];    // adapter of a token, -1: none
  __shared__ int s_run[kFastPlanBatch];     // token -> run, valid at a run's first token
  __shared__ int s_ra[kFastPlanBatch], s_rr[kFastPlanBatch], s_rn[kFastPlanBatch];  // run: adapter, rank, items
  __shared__ int s_blo[kFastPlanBatch], s_bhi[kFastPlanBatch];                      // run: a_start of its adapter
  __shared__ int s_ntok[kFastPlanBatch];
  __shared__ int s_toks[kFastPlanBatch * kTT];
  __shared__ int s_before[kFastPlanBatch + 1];  // sorted position -> items in front of the run there
  __shared__ int s_order[kFastPlanBatch];       // sorted position -> run
  __shared__ int s_wave[kPlanWaves];
  __shared__ int s_max_rank, s_total;
  __shared__ int s_qstart[kXcds], s_qlen[kXcds];
  const int tid = threadIdx.x;
  for (int i = (int)blockIdx.x * kPlanThreads + tid; i < sync_words; i += (int)gridDim.x * kPlanThreads) sync[i] = 0;
  if (tid == 0) {
    s_max_rank = 0;
    s_total = 0;
  }
  if (tid < kXcds) {
    s_qstart[tid] = 0x7fffffff;
    s_qlen[tid] = 0;
  }
  // one token per thread (batch <= kPlanThreads == kFastPlanBatch)
  int a = -1;
  if (tid < batch) {
    const int64_t a64 = t.bins[tid];
    a = ((uint64_t)a64 < (uint64_t)t.n_adapters && a64 <= 0x7fffffffLL) ? (int)a64 : -1;
  }
  int64_t len = 0, base = 0;
  if (a >= 0) {
    len = t.a_len[a];
    base = t.a_start[a];
  }
  s_bins[tid] = a;
  s_ntok[tid] = 0;
  __syncthreads();
  // my number among the tokens of my adapter, and the first token of my group of kTT
  int pos = 0, first = tid;
  const int q_end = tid < batch ? tid : 0;
  for (int q = 0; q < q_end; ++q) {
    if (s_bins[q] == a) {
      if (pos % kTT == 0) first = q;
      ++pos;
    }
  }
  if (pos % kTT == 0) first = tid;
  const int r = (a >= 0 && len > 0) ? (int)(len >> 2) : 0;
  const bool member = r > 0;
  const bool leader = member && first == tid;
  int n_runs = 0;
  const int idx = block_exclusive_scan(leader ? 1 : 0, s_wave, &n_runs);
  int n_it = 0;
  if (leader) {
    const int r_listed = r < rank_cap ? r : rank_cap;
    n_it = (r_listed + kRB - 1) / kRB;
    s_run[tid] = idx;
    s_ra[idx] = a;
    s_rr[idx] = r;
    s_rn[idx] = n_it;
    s_blo[idx] = (int)(uint32_t)(uint64_t)base;
    s_bhi[idx] = (int)(uint32_t)((uint64_t)base >> 32);
    atomicMax(&s_max_rank, r);
    atomicAdd(&s_total, n_it);
  }
  __syncthreads();
  if (member) {
    const int run = s_run[first];
    s_toks[run * kTT + pos % kTT] = tid;
    atomicAdd(&s_ntok[run], 1);
  }
  const int total = s_total;
  // order by (adapter, first token): items in front of my run, and runs in front of it
  if (leader) {
    int before = 0, rank_pos = 0;
    for (int o = 0; o < n_runs; ++o) {
      const int oa = s_ra[o];
      if (oa < a || (oa == a && o < idx)) {  // runs are numbered in token order
        before += s_rn[o];
        ++rank_pos;
      }
    }
    int q = (int)(((int64_t)before * kXcds) / (total > 0 ? total : 1));
    if (q > kXcds - 1) q = kXcds - 1;
    s_before[rank_pos] = before;
    s_order[rank_pos] = idx;
    atomicMin(&s_qstart[q], before);
    atomicAdd(&s_qlen[q], n_it);
  }
  __syncthreads();
  int max_len = 0;
  for (int q = 0; q < kXcds; ++q) max_len = s_qlen[q] > max_len ? s_qlen[q] : max_len;
  int n_items = kXcds * max_len;
  if (n_items > max_items) n_items = 0;  // cannot happen with the capacity slora_bgmv_plan_bytes() reserves

  // ---- records ----
  const int sub = tid & 15;
  const int n_groups = (int)gridDim.x * (kPlanThreads / 16);
  for (int rec_i = (int)blockIdx.x * (kPlanThreads / 16) + (tid >> 4); rec_i < n_items; rec_i += n_groups) {
    const int q = rec_i % kXcds, k = rec_i / kXcds;
    const bool real = k < s_qlen[q];
    int run = 0, i = 0;
    if (real) {
      const int srt = s_qstart[q] + k;  // index of the item in sorted order
      int lo = 0, hi = n_runs;          // last sorted position whose `before` is <= srt
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (s_before[mid] <= srt) lo = mid; else hi = mid;
      }
      run = s_order[lo];
      i = srt - s_before[lo];
    }
    const int ra = s_ra[run], rr = s_rr[run], rn = s_rn[run], n_tok = s_ntok[run];
    const int64_t rbase = (int64_t)(((uint64_t)(uint32_t)s_bhi[run] << 32) | (uint32_t)s_blo[run]);
    const int j0 = i * kRB;
    int w0 = 0, w1 = 0, w2 = 0, w3 = 0;
    if (sub >= 2 && sub < 10) {
      const int proj = (sub - 2) >> 1, jr0 = ((sub - 2) & 1) * 4;
      int64_t pg[4];
#pragma unroll
      for (int c = 0; c < 4; ++c)
        pg[c] = lookup_page_nobranch(t, rbase + (int64_t)proj * rr + j0 + jr0 + c,
                                     real && n_tok > 0 && j0 + jr0 + c < rr && t.n_loc > 0);
      w0 = (pg[0] >= 0 && pg[0] <= 0x7fffffffLL) ? (int)pg[0] : -1;
      w1 = (pg[1] >= 0 && pg[1] <= 0x7fffffffLL) ? (int)pg[1] : -1;
      w2 = (pg[2] >= 0 && pg[2] <= 0x7fffffffLL) ? (int)pg[2] : -1;
      w3 = (pg[3] >= 0 && pg[3] <= 0x7fffffffLL) ? (int)pg[3] : -1;
    } else if (real) {
      if (sub == 0) {
        w0 = ra, w1 = rr, w2 = n_tok < kTT ? n_tok : kTT, w3 = j0;
      } else if (sub == 1) {
        w0 = n_tok > 0 ? s_toks[run * kTT + 0] : 0;
        w1 = n_tok > 1 ? s_toks[run * kTT + 1] : 0;
        w2 = n_tok > 2 ? s_toks[run * kTT + 2] : 0;
        w3 = n_tok > 3 ? s_toks[run * kTT + 3] : 0;
      } else if (sub == 10) {
        w0 = s_blo[run], w1 = s_bhi[run];
        w2 = (i == rn - 1 && rr > rank_cap) ? 1 : 0;
      }
    }
    if (sub < 12) {
      int4 v = make_int4(w0, w1, w2, w3);
      *reinterpret_cast<int4*>(plan + kPlanHeaderWords + (int64_t)rec_i * kItemWords + sub * 4) = v;
    }
  }
  if (blockIdx.x == 0 && tid == 0) {
    plan[PH_MAGIC] = kPlanMagic;
    plan[PH_NITEMS] = n_items;
    plan[PH_MAXRANK] = s_max_rank;
    plan[PH_BATCH] = batch;
    plan[PH_TT] = kTT;
    plan[PH_RANKCAP] = rank_cap;
    plan[PH_NRUNS] = n_runs;
    plan[PH_STATUS] = 0;
  }
}

// The same plan for batches of up to kSortPlanBatch tokens: instead of counting, for every token,
// the tokens of its adapter in front of it (quadratic in the batch), the tokens are sorted by
// (adapter, token) in LDS -- a bitonic network over 32-bit keys adapter << 13 | token -- after which
// a run is four neighbours, the order of the runs is the order of the keys, and everything else is
// prefix sums.  As in bgmv_plan_fast_kernel every workgroup derives the order by itself and the
// records are shared out.  LDS (dynamic): keys[n], before[n + 1], spos[n] (16 bit) with n the batch
// rounded up to a power of two.  Needs n_adapters < 2^19.
constexpr int kSortPlanBatch = 8192;
constexpr int kCountPlanBatch = 64;  // up to here bgmv_plan_fast_kernel is the quicker one
constexpr int kSortTokBits = 13;
constexpr int kSortMaxAdapters = 1 << (32 - kSortTokBits);

// exclusive running maximum of `v` over the workgroup (-1 in front of the first thread)
__device__ __forceinline__ int block_exclusive_max(int v, int* s_wave) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int inc = v;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const int up = __shfl_up(inc, o, kWave);
    if (lane >= o) inc = up > inc ? up : inc;
  }
  if (lane == kWave - 1) s_wave[wave] = inc;
  __syncthreads();
  int before = -1;
  for (int wv = 0; wv < kPlanWaves; ++wv)
    if (wv < wave) before = s_wave[wv] > before ? s_wave[wv] : before;
  __syncthreads();
  const int prev = __shfl_up(inc, 1, kWave);
  const int mine = lane == 0 ? -1 : prev;
  return mine > before ? mine : before;
}

__global__ __launch_bounds__(kPlanThreads) void bgmv_plan_sort_kernel(int* __restrict__ plan, Tables t, int batch,
                                                                      int rank_cap, int max_items, int n,
                                                                      int* __restrict__ sync, int sync_words) {
  extern __shared__ __align__(16) unsigned char s_dyn[];
  uint32_t* s_key = reinterpret_cast<uint32_t*>(s_dyn);                // sorted: adapter << 13 | token, ~0: no member
  int* s_before = reinterpret_cast<int*>(s_key + n);                   // run -> items in front of it
  uint16_t* s_spos = reinterpret_cast<uint16_t*>(s_before + (n + 1));  // run -> sorted position of its first token
  __shared__ int s_wave[kPlanWaves];
  __shared__ int s_max_rank;
  __shared__ int s_qstart[kXcds], s_qlen[kXcds];
  constexpr uint32_t kNone = 0xffffffffu;
  const int tid = threadIdx.x;
  for (int i = (int)blockIdx.x * kPlanThreads + tid; i < sync_words; i += (int)gridDim.x * kPlanThreads) sync[i] = 0;
  if (tid == 0) s_max_rank = 0;
  if (tid < kXcds) {
    s_qstart[tid] = 0x7fffffff;
    s_qlen[tid] = 0;
  }
  // keys: tokens of an adapter that exists and has a rank
  for (int i = tid; i < n; i += kPlanThreads) {
    uint32_t key = kNone;
    if (i < batch) {
      const int64_t a64 = t.bins[i];
      if ((uint64_t)a64 < (uint64_t)t.n_adapters && t.a_len[a64] >= 4) key = ((uint32_t)a64 << kSortTokBits) | (uint32_t)i;
    }
    s_key[i] = key;
  }
  __syncthreads();
  // bitonic network, ascending
  for (int k = 2; k <= n; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      const int lj = __builtin_ctz((unsigned)j);
      for (int pr = tid; pr < (n >> 1); pr += kPlanThreads) {
        const int i = ((pr >> lj) << (lj + 1)) | (pr & (j - 1)), o = i + j;
        const uint32_t x = s_key[i], y = s_key[o];
        const bool up = (i & k) == 0;
        if ((x > y) == up) {
          s_key[i] = y;
          s_key[o] = x;
        }
      }
      __syncthreads();
    }
  }
  // E consecutive sorted positions per thread
  constexpr int kMaxE = kSortPlanBatch / kPlanThreads;
  const int E = n >= kPlanThreads ? n / kPlanThreads : 1;
  const int s0 = tid * E;
  const bool active = s0 < n;
  uint32_t key[kMaxE];
  int rank[kMaxE];
  bool head[kMaxE];
#pragma unroll
  for (int e = 0; e < kMaxE; ++e) {
    key[e] = (active && e < E) ? s_key[s0 + e] : kNone;
    rank[e] = 0;
    if (key[e] != kNone) rank[e] = (int)(t.a_len[key[e] >> kSortTokBits] >> 2);
  }
  int last_head = -1;
#pragma unroll
  for (int e = 0; e < kMaxE; ++e) {
    const int sp = s0 + e;
    const uint32_t prev = e > 0 ? key[e - 1] : ((active && sp > 0) ? s_key[sp - 1] : kNone);
    head[e] = key[e] != kNone && (sp == 0 || (prev >> kSortTokBits) != (key[e] >> kSortTokBits));
    if (head[e]) last_head = sp;
  }
  int hp = block_exclusive_max(last_head, s_wave);  // where the adapter of my first position starts
  int n_lead = 0, n_it_sum = 0;
  bool leader[kMaxE];
  int n_it[kMaxE];
#pragma unroll
  for (int e = 0; e < kMaxE; ++e) {
    const int sp = s0 + e;
    if (head[e]) hp = sp;
    leader[e] = key[e] != kNone && ((sp - hp) % kTT) == 0;
    const int r_listed = rank[e] < rank_cap ? rank[e] : rank_cap;
    n_it[e] = leader[e] ? (r_listed + kRB - 1) / kRB : 0;
    n_lead += leader[e] ? 1 : 0;
    n_it_sum += n_it[e];
  }
  int n_runs = 0, total = 0;
  int run = block_exclusive_scan(n_lead, s_wave, &n_runs);
  int before = block_exclusive_scan(n_it_sum, s_wave, &total);
#pragma unroll
  for (int e = 0; e < kMaxE; ++e) {
    if (leader[e]) {
      int q = (int)(((int64_t)before * kXcds) / (total > 0 ? total : 1));
      if (q > kXcds - 1) q = kXcds - 1;
      s_before[run] = before;
      s_spos[run] = (uint16_t)(s0 + e);
      atomicMin(&s_qstart[q], before);
      atomicAdd(&s_qlen[q], n_it[e]);
      atomicMax(&s_max_rank, rank[e]);
      ++run;
      before += n_it[e];
    }
  }
  __syncthreads();
  int max_len = 0;
  for (int q = 0; q < kXcds; ++q) max_len = s_qlen[q] > max_len ? s_qlen[q] : max_len;
  int n_items = kXcds * max_len;
  if (n_items > max_items) n_items = 0;  // cannot happen with the capacity slora_bgmv_plan_bytes() reserves

  // ---- records: 16 lanes each, as in bgmv_plan_fast_kernel ----
  const int sub = tid & 15;
  const int n_groups = (int)gridDim.x * (kPlanThreads / 16);
  for (int rec_i = (int)blockIdx.x * (kPlanThreads / 16) + (tid >> 4); rec_i < n_items; rec_i += n_groups) {
    const int q = rec_i % kXcds, k = rec_i / kXcds;
    const bool real = k < s_qlen[q];
    int ra = 0, rr = 0, rn = 0, n_tok = 0, i = 0;
    int toks[kTT] = {0, 0, 0, 0};
    int64_t rbase = 0;
    if (real) {
      const int srt = s_qstart[q] + k;  // index of the item in sorted order
      int lo = 0, hi = n_runs;          // last run whose `before` is <= srt
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (s_before[mid] <= srt) lo = mid; else hi = mid;
      }
      i = srt - s_before[lo];
      const int sp = s_spos[lo];
      const uint32_t k0 = s_key[sp];
      ra = (int)(k0 >> kSortTokBits);
#pragma unroll
      for (int c = 0; c < kTT; ++c) {
        const uint32_t kc = sp + c < n ? s_key[sp + c] : kNone;
        if (kc != kNone && (kc >> kSortTokBits) == (k0 >> kSortTokBits)) {
          toks[c] = (int)(kc & ((1u << kSortTokBits) - 1u));
          n_tok = c + 1;
        }
      }
      rr = (int)(t.a_len[ra] >> 2);
      rbase = t.a_start[ra];
      const int r_listed = rr < rank_cap ? rr : rank_cap;
      rn = (r_listed + kRB - 1) / kRB;
    }
    const int j0 = i * kRB;
    int w0 = 0, w1 = 0, w2 = 0, w3 = 0;
    if (sub >= 2 && sub < 10) {
      const int proj = (sub - 2) >> 1, jr0 = ((sub - 2) & 1) * 4;
      int64_t pg[4];
#pragma unroll
      for (int c = 0; c < 4; ++c)
        pg[c] = lookup_page_nobranch(t, rbase + (int64_t)proj * rr + j0 + jr0 + c,
                                     real && n_tok > 0 && j0 + jr0 + c < rr && t.n_loc > 0);
      w0 = (pg[0] >= 0 && pg[0] <= 0x7fffffffLL) ? (int)pg[0] : -1;
      w1 = (pg[1] >= 0 && pg[1] <= 0x7fffffffLL) ? (int)pg[1] : -1;
      w2 = (pg[2] >= 0 && pg[2] <= 0x7fffffffLL) ? (int)pg[2] : -1;
      w3 = (pg[3] >= 0 && pg[3] <= 0x7fffffffLL) ? (int)pg[3] : -1;
    } else if (real) {
      if (sub == 0) {
        w0 = ra, w1 = rr, w2 = n_tok, w3 = j0;
      } else if (sub == 1) {
        w0 = toks[0], w1 = toks[1], w2 = toks[2], w3 = toks[3];
      } else if (sub == 10) {
        w0 = (int)(uint32_t)(uint64_t)rbase, w1 = (int)(uint32_t)((uint64_t)rbase >> 32);
        w2 = (i == rn - 1 && rr > rank_cap) ? 1 : 0;
      }
    }
    if (sub < 12) {
      int4 v = make_int4(w0, w1, w2, w3);
      *reinterpret_cast<int4*>(plan + kPlanHeaderWords + (int64_t)rec_i * kItemWords + sub * 4) = v;
    }
  }
  if (blockIdx.x == 0 && tid == 0) {
    plan[PH_MAGIC] = kPlanMagic;
    plan[PH_NITEMS] = n_items;
    plan[PH_MAXRANK] = s_max_rank;
    plan[PH_BATCH] = batch;
    plan[PH_TT] = kTT;
    plan[PH_RANKCAP] = rank_cap;
    plan[PH_NRUNS] = n_runs;
    plan[PH_STATUS] = 0;
  }
}

template <typename T, bool PLANNED, int NV>
int launch_shrink_nv(ShrinkArgs p, int nproj, int64_t units, size_t lds, hipStream_t stream) {
  auto kernel = bgmv_shrink_kernel<T, PLANNED, NV>;
  const int64_t grid = units;
  if (lds > kLdsSoftLimit) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess) {
      (void)hipGetLastError();
      return SLORA_ERR_LAUNCH;
    }
  }
  if (grid <= 0) return SLORA_OK;
  if (grid > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kernel, dim3((uint32_t)grid, (uint32_t)nproj), dim3(256), lds, stream, p);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

template <typename T, bool PLANNED>
int launch_shrink(ShrinkArgs p, int nproj, int64_t units, hipStream_t stream) {
  // as many tokens staged at once as fit the LDS budget: a full run of kTT tokens up to
  // hidden 8192 (four workgroups per compute unit at 5120, two at 8192), fewer beyond
  const size_t row_bytes = (size_t)p.h_in * 2;
  int tt = kTT;
  while (tt > 1 && tt * row_bytes > 64 * 1024) --tt;
  const size_t lds = tt * row_bytes;
  if (lds > kLdsHardLimit) return SLORA_ERR_UNSUPPORTED;
  p.lds_tt = tt;
  const int nvec = p.h_in >> 3;
  if (nvec <= 8 * kWave) return launch_shrink_nv<T, PLANNED, 8>(p, nproj, units, lds, stream);
  if (nvec <= 10 * kWave) return launch_shrink_nv<T, PLANNED, 10>(p, nproj, units, lds, stream);
  if (nvec <= 12 * kWave) return launch_shrink_nv<T, PLANNED, 12>(p, nproj, units, lds, stream);
  if (nvec <= 16 * kWave) return launch_shrink_nv<T, PLANNED, 16>(p, nproj, units, lds, stream);
  return launch_shrink_nv<T, PLANNED, 8>(p, nproj, units, lds, stream);  // general path only
}

// Five workgroups per compute unit for the q/k/v launch (its 3000 workgroups come in rounds,
// more of them resident hide more of each other's waits), four for a single projection (all of
// its workgroups are resident at once, and four leave 128 registers: nothing spills).
// Grid, two forms.  Two-dimensional (x = unit, y = projection * 2 + half): all workgroups of
// one projection half run before those of the next.  One-dimensional (p.interleave): id L
// -> unit 8 * (L / (8 * S)) + L % 8, sub (L / 8) % S with S = 2 * NPROJ, so a unit still sits
// on XCD unit % 8 and its S workgroups follow each other.  The second form is for outputs
// narrower than a page (grouped-query k and v): most of their workgroups find no page and
// exit, and spread between the others they cost nothing, while in phases of their own they
// are all a phase consists of.
// NV: see expand_page.  The wider instantiations hold more of a page in registers and get one
// workgroup per compute unit fewer.
template <typename T, int NPROJ, bool PLANNED, int NV>
__global__ __launch_bounds__(256, NV > 8 ? (NV > 12 ? 3 : 4) : (NPROJ == 3 ? 5 : 4)) void bgmv_expand_kernel(
    const ExpandArgs p) {
  __shared__ __align__(16) uint16_t s_out[4][ExpandPass<NV>::kStrip];
  int unit = (int)blockIdx.x, sub = (int)blockIdx.y;
  if (p.interleave) {
    constexpr int S = 2 * NPROJ;
    const int g = unit >> 3;
    unit = (g / S) * 8 + (unit & 7);
    sub = g % S;
    if (unit >= p.n_units) return;
  }
  const int n_items = expand_body<T, NPROJ, PLANNED, NV>(p, unit, sub, s_out[threadIdx.x >> 6]);
  if (PLANNED && p.strided) {  // the items beyond the grid, if the batch has that many
    const int stride = p.interleave ? (int)gridDim.x / (2 * NPROJ) : (int)gridDim.x;  // units of the grid
    for (unit += stride; unit < n_items; unit += stride)
      expand_body<T, NPROJ, PLANNED, NV>(p, unit, sub, s_out[threadIdx.x >> 6]);
  }
}

template <typename T, int NPROJ, bool PLANNED, int NV>
int launch_expand_nv(ExpandArgs p, int64_t items, hipStream_t stream) {
  dim3 grid((uint32_t)items, 2 * NPROJ);
  if (p.interleave) grid = dim3((uint32_t)((items + 7) / 8 * 8 * 2 * NPROJ), 1);
  hipLaunchKernelGGL((bgmv_expand_kernel<T, NPROJ, PLANNED, NV>), grid, dim3(256), 0, stream, p);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

template <typename T, int NPROJ, bool PLANNED>
int launch_expand(ExpandArgs p, int64_t items, hipStream_t stream) {
  if (items <= 0) return SLORA_OK;
  if (items > 0x7fffffffLL / (2 * NPROJ + 1)) return SLORA_ERR_UNSUPPORTED;
  p.n_units = (int)items;
  p.interleave = 0;
  for (int i = 0; i < NPROJ; ++i)
    if (p.pages_shift[i] > 0) p.interleave = 1;  // an output narrower than a page
  // planned launches: the instantiation whose pass holds the whole page (the stateless kernels keep
  // the 4096-element pass)
  if (PLANNED) {
    const int64_t pv = p.page_elems >> 3;
    if (pv > 8 * kWave && pv <= 10 * kWave) return launch_expand_nv<T, NPROJ, PLANNED, PLANNED ? 10 : 8>(p, items, stream);
    if (pv > 10 * kWave && pv <= 12 * kWave) return launch_expand_nv<T, NPROJ, PLANNED, PLANNED ? 12 : 8>(p, items, stream);
    if (pv > 12 * kWave && pv <= 16 * kWave) return launch_expand_nv<T, NPROJ, PLANNED, PLANNED ? 16 : 8>(p, items, stream);
  }
  return launch_expand_nv<T, NPROJ, PLANNED, 8>(p, items, stream);
}

template <typename T>
int dispatch_shrink(const ShrinkArgs& p, int nproj, bool planned, int64_t units, hipStream_t s) {
  return planned ? launch_shrink<T, true>(p, nproj, units, s) : launch_shrink<T, false>(p, nproj, units, s);
}

template <typename T>
int dispatch_expand(const ExpandArgs& p, int nproj, bool planned, int64_t grid, hipStream_t s) {
  if (nproj == 3)
    return planned ? launch_expand<T, 3, true>(p, grid, s) : launch_expand<T, 3, false>(p, grid, s);
  return planned ? launch_expand<T, 1, true>(p, grid, s) : launch_expand<T, 1, false>(p, grid, s);
}

int shrink_common(const void* plan, int64_t n_items, int64_t rank_cap, void* const y[3], int nproj, int qkvo0,
                  const void* x, const void* w, const slora_tables* tables, const int64_t* bins, int64_t batch,
                  int64_t h_in, int64_t y_cols, int64_t page_elems, int64_t n_pages, int dtype, void* stream) {
  ShrinkArgs p{};
  int64_t grid = 0;
  const int rc = shrink_prepare(plan, n_items, rank_cap, y, nproj, qkvo0, x, w, tables, bins, batch, h_in, y_cols,
                                page_elems, n_pages, dtype, p, grid);
  if (rc != SLORA_OK) return rc == kNothingToDo ? SLORA_OK : rc;
  const bool planned = plan != nullptr;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  return dtype == SLORA_DTYPE_F16 ? dispatch_shrink<F16>(p, nproj, planned, grid, s)
                                  : dispatch_shrink<BF16>(p, nproj, planned, grid, s);
}

int expand_common(const void* plan, int64_t n_items, int64_t rank_cap, void* const y[3], const void* const x[3],
                  const int64_t h_out[3], int nproj, int qkvo0, const void* w, const slora_tables* tables,
                  const int64_t* bins, const void* scales, int scales_dtype, int64_t batch, int64_t x_cols,
                  int64_t page_elems, int64_t n_pages, int dtype, void* stream) {
  ExpandArgs p{};
  int64_t grid = 0;
  const int rc = expand_prepare(plan, n_items, rank_cap, y, x, h_out, nproj, qkvo0, w, tables, bins, scales,
                                scales_dtype, batch, x_cols, page_elems, n_pages, dtype, p, grid);
  if (rc != SLORA_OK) return rc == kNothingToDo ? SLORA_OK : rc;
  const bool planned = plan != nullptr;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  return dtype == SLORA_DTYPE_F16 ? dispatch_expand<F16>(p, nproj, planned, grid, s)
                                  : dispatch_expand<BF16>(p, nproj, planned, grid, s);
}

}  // namespace
}  // namespace slora

extern "C" {

int slora_bgmv_shrink(void* y, const void* x, const void* w, const slora_tables* tables, const int64_t* bins,
                      int64_t batch, int64_t h_in, int64_t y_cols, int64_t page_elems, int64_t n_pages, int qkvo,
                      int dtype, void* stream) {
  void* ys[3] = {y, nullptr, nullptr};
  if (qkvo < 0 || qkvo > 3) return SLORA_ERR_BAD_SHAPE;
  return slora::shrink_common(nullptr, 0, 0, ys, 1, qkvo, x, w, tables, bins, batch, h_in, y_cols, page_elems,
                              n_pages, dtype, stream);
}

int slora_bgmv_shrink_qkv(void* y_q, void* y_k, void* y_v, const void* x, const void* w,
                          const slora_tables* tables, const int64_t* bins, int64_t batch, int64_t h_in,
                          int64_t y_cols, int64_t page_elems, int64_t n_pages, int dtype, void* stream) {
  void* ys[3] = {y_q, y_k, y_v};
  return slora::shrink_common(nullptr, 0, 0, ys, 3, 0, x, w, tables, bins, batch, h_in, y_cols, page_elems, n_pages,
                              dtype, stream);
}

int slora_bgmv_expand(void* y, const void* x, const void* w, const slora_tables* tables, const int64_t* bins,
                      const void* scales, int scales_dtype, int64_t batch, int64_t x_cols, int64_t h_out,
                      int64_t page_elems, int64_t n_pages, int qkvo, int dtype, void* stream) {
  void* ys[3] = {y, nullptr, nullptr};
  const void* xs[3] = {x, nullptr, nullptr};
  const int64_t hs[3] = {h_out, 0, 0};
  if (qkvo < 0 || qkvo > 3) return SLORA_ERR_BAD_SHAPE;
  return slora::expand_common(nullptr, 0, 0, ys, xs, hs, 1, qkvo, w, tables, bins, scales, scales_dtype, batch,
                              x_cols, page_elems, n_pages, dtype, stream);
}

int slora_bgmv_expand_qkv(void* y_q, void* y_k, void* y_v, const void* x_q, const void* x_k, const void* x_v,
                          const void* w, const slora_tables* tables, const int64_t* bins, const void* scales,
                          int scales_dtype, int64_t batch, int64_t x_cols, int64_t h_out_q, int64_t h_out_k,
                          int64_t h_out_v, int64_t page_elems, int64_t n_pages, int dtype, void* stream) {
  void* ys[3] = {y_q, y_k, y_v};
  const void* xs[3] = {x_q, x_k, x_v};
  const int64_t hs[3] = {h_out_q, h_out_k, h_out_v};
  return slora::expand_common(nullptr, 0, 0, ys, xs, hs, 3, 0, w, tables, bins, scales, scales_dtype, batch, x_cols,
                              page_elems, n_pages, dtype, stream);
}

int64_t slora_bgmv_plan_bytes(int64_t batch, int64_t rank_cap) {
  if (batch < 0 || rank_cap <= 0 || rank_cap > SLORA_MAX_RANK || batch > (1 << 24)) return SLORA_ERR_BAD_SHAPE;
  return 4 * slora::plan_words(batch, rank_cap);
}

int slora_bgmv_plan_build(void* plan, int64_t plan_bytes, const slora_tables* tables, const int64_t* bins,
                          int64_t batch, int64_t rank_cap, int64_t n_pages, void* stream) {
  using namespace slora;
  if (plan == nullptr) return SLORA_ERR_NULL_POINTER;
  const int64_t need = slora_bgmv_plan_bytes(batch, rank_cap);
  if (need < 0) return (int)need;
  if (plan_bytes < need) return SLORA_ERR_BAD_SHAPE;
  if (!aligned16(plan)) return SLORA_ERR_ALIGNMENT;
  Tables t{};
  int rc = fill_tables(t, tables, bins, n_pages);
  if (rc != SLORA_OK) return rc;
  const int64_t max_items = plan_max_items(batch, rank_cap);
  if (max_items > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
  int* sync = static_cast<int*>(plan) + plan_sync_offset(batch, rank_cap);
  const int sync_words = (int)plan_sync_words(batch);
  // Three builders, one plan (word for word): counting in LDS with a token per thread is the quickest
  // up to a few dozen tokens (4 us for one token, 10 us for 32), sorting from there on (15 us for 256
  // tokens, 23 us for 1024, 90 us for 8192: the counting builder takes 27 and 86 us for the first
  // two), and one workgroup with scratch memory serves what the sorted keys cannot hold.
  const bool sortable = batch <= kSortPlanBatch && t.n_adapters < kSortMaxAdapters;
  if (batch <= (sortable ? kCountPlanBatch : kFastPlanBatch)) {
    int64_t grid = (max_items + kPlanThreads / 16 - 1) / (kPlanThreads / 16);
    grid = grid < 1 ? 1 : (grid > 16 ? 16 : grid);
    hipLaunchKernelGGL(bgmv_plan_fast_kernel, dim3((uint32_t)grid), dim3(kPlanThreads), 0,
                       reinterpret_cast<hipStream_t>(stream), static_cast<int*>(plan), t, (int)batch, (int)rank_cap,
                       (int)max_items, sync, sync_words);
    return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
  }
  if (sortable) {
    int n = 64;
    while (n < batch) n <<= 1;
    const size_t lds = (size_t)n * 4 + (size_t)(n + 1) * 4 + (size_t)n * 2 + 16;
    static PerDeviceOnce once;
    if (!raise_dynamic_lds(reinterpret_cast<const void*>(bgmv_plan_sort_kernel), kSortPlanBatch * 10 + 32, once))
      return SLORA_ERR_LAUNCH;
    int64_t grid = (max_items + kPlanThreads / 16 - 1) / (kPlanThreads / 16);
    grid = grid < 1 ? 1 : (grid > 16 ? 16 : grid);
    hipLaunchKernelGGL(bgmv_plan_sort_kernel, dim3((uint32_t)grid), dim3(kPlanThreads), lds,
                       reinterpret_cast<hipStream_t>(stream), static_cast<int*>(plan), t, (int)batch, (int)rank_cap,
                       (int)max_items, n, sync, sync_words);
    return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
  }
  int* scratch = static_cast<int*>(plan) + kPlanHeaderWords + max_items * kItemWords;
  hipLaunchKernelGGL(bgmv_plan_kernel, dim3(1), dim3(kPlanThreads), 0, reinterpret_cast<hipStream_t>(stream),
                     static_cast<int*>(plan), t, (int)batch, (int)rank_cap, (int)max_items, scratch, sync, sync_words);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

int slora_bgmv_shrink_planned(const void* plan, int64_t rank_cap, int64_t n_items, int nproj, void* y0, void* y1,
                              void* y2, const void* x, const void* w, const slora_tables* tables,
                              const int64_t* bins, int64_t batch, int64_t h_in, int64_t y_cols, int64_t page_elems,
                              int64_t n_pages, int qkvo, int dtype, void* stream) {
  if (plan == nullptr) return SLORA_ERR_NULL_POINTER;
  if (rank_cap <= 0 || rank_cap > SLORA_MAX_RANK) return SLORA_ERR_BAD_SHAPE;
  if (nproj != 1 && nproj != 3) return SLORA_ERR_BAD_SHAPE;
  if (nproj == 3 && qkvo != 0) return SLORA_ERR_BAD_SHAPE;
  void* ys[3] = {y0, y1, y2};
  return slora::shrink_common(plan, n_items, rank_cap, ys, nproj, qkvo, x, w, tables, bins, batch, h_in, y_cols,
                              page_elems, n_pages, dtype, stream);
}

int slora_bgmv_expand_planned(const void* plan, int64_t rank_cap, int64_t n_items, int nproj, void* y0, void* y1,
                              void* y2, const void* x0, const void* x1, const void* x2, const void* w,
                              const slora_tables* tables, const int64_t* bins, const void* scales, int scales_dtype,
                              int64_t batch, int64_t x_cols, int64_t h_out0, int64_t h_out1, int64_t h_out2,
                              int64_t page_elems, int64_t n_pages, int qkvo, int dtype, void* stream) {
  if (plan == nullptr) return SLORA_ERR_NULL_POINTER;
  if (rank_cap <= 0 || rank_cap > SLORA_MAX_RANK) return SLORA_ERR_BAD_SHAPE;
  if (nproj != 1 && nproj != 3) return SLORA_ERR_BAD_SHAPE;
  if (nproj == 3 && qkvo != 0) return SLORA_ERR_BAD_SHAPE;
  void* ys[3] = {y0, y1, y2};
  const void* xs[3] = {x0, x1, x2};
  const int64_t hs[3] = {h_out0, h_out1, h_out2};
  return slora::expand_common(plan, n_items, rank_cap, ys, xs, hs, nproj, qkvo, w, tables, bins, scales,
                              scales_dtype, batch, x_cols, page_elems, n_pages, dtype, stream);
}

}  // extern "C"
