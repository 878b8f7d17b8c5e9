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

#include "common.hpp"
#include "cabi_util.hpp"

namespace slora {
namespace {

constexpr int kTT = 4;                    // most tokens merged into one run
constexpr int kRB = 8;                    // rows / pages per item
constexpr int kVecPerPass = 8;            // 16-byte vectors a lane holds per 4096-element pass over a page

struct Tables {
  const int64_t* a_start;
  const int64_t* a_len;
  const int64_t* a_loc;
  const int64_t* bins;
  int64_t n_adapters, n_loc, n_pages;
};

// page id for entry `li` of a_loc, or -1 if anything is out of range
__device__ __forceinline__ int64_t lookup_page(const Tables& t, int64_t li) {
  if ((uint64_t)li >= (uint64_t)t.n_loc) return -1;
  const int64_t page = t.a_loc[li];
  return (uint64_t)page < (uint64_t)t.n_pages ? page : -1;
}

// ---------------------------------------------------------------------------
// plan: the items of a batch
// ---------------------------------------------------------------------------
// int32 words: a 16-word header, then one 48-word (192-byte) record per item:
//   [0] adapter  [1] rank  [2] n_tok  [3] j0 = first row of the item
//   [4..8)   token indices
//   [8..40)  page id of a_loc entry p*rank + j0 + i at [8 + p*8 + i]  (p = q,k,v,o; -1 = none)
//   [40..42) a_start[adapter] (int64)
//   [42]     1 if this is the run's last stored item and rank > rank_cap (rows the plan does not list)
constexpr int kPlanMagic = 0x534c5032;  // "SLP2"
constexpr int kPlanHeaderWords = 16;
constexpr int kItemWords = 48;
enum { PH_MAGIC = 0, PH_NITEMS = 1, PH_MAXRANK = 2, PH_BATCH = 3, PH_TT = 4, PH_RANKCAP = 5, PH_NRUNS = 6 };
enum { IT_ADAPTER = 0, IT_RANK = 1, IT_NTOK = 2, IT_J0 = 3, IT_TOK = 4, IT_PAGES = 8, IT_BASE = 40, IT_MORE = 42 };

struct Item {
  int64_t a;     // adapter
  int64_t base;  // a_start[a]
  int r;         // rank
  int n_tok;     // tokens in the run (0: nothing to do)
  int j0;        // first row / page of the item inside each projection block
  int more;      // rows beyond the listed ones exist (rank > rank_cap)
  int tok[kTT];  // token indices
  int plan_items;  // items of the plan the record was read from (0: no plan, or not a plan)
};

__device__ __forceinline__ int item_token(const Item& it, int t) {
  int tk = 0;
#pragma unroll
  for (int k = 0; k < kTT; ++k)
    if (k == t) tk = it.tok[k];
  return tk;
}

// Stateless discovery by ONE wavefront: which tokens share token b's adapter,
// is b the first of a run of kTT, and who are the others.  No LDS, no barrier;
// every wavefront of the workgroup computes the same answer.  The adapter ids
// are loaded 512 at a time so the loads of a group overlap.
__device__ __forceinline__ void discover_run(const Tables& t, int batch, int b, Item& it) {
  const int lane = threadIdx.x & 63;
  it.n_tok = 0;
  it.r = 0;
  it.more = 0;
  it.plan_items = 0;
  constexpr int kGroup = 8;  // chunks of 64 ids loaded together
  const int64_t a = t.bins[b];
  int64_t v[kGroup];
#pragma unroll
  for (int c = 0; c < kGroup; ++c) {
    const int tkn = c * kWave + lane;
    v[c] = tkn < batch ? t.bins[tkn] : (int64_t)-1;
  }
  if ((uint64_t)a >= (uint64_t)t.n_adapters) return;
  // in flight while the ids are compared
  const int64_t len = t.a_len[a];
  const int64_t base_a = t.a_start[a];
  int pos_b = 0, n_tok = 0;
  bool started = false;
  for (int g0 = 0; g0 < batch; g0 += kGroup * kWave) {
    if (g0 != 0) {
#pragma unroll
      for (int c = 0; c < kGroup; ++c) {
        const int tkn = g0 + c * kWave + lane;
        v[c] = tkn < batch ? t.bins[tkn] : (int64_t)-1;
      }
    }
#pragma unroll
    for (int c = 0; c < kGroup; ++c) {
      const int base = g0 + c * kWave;
      if (base < batch && n_tok < kTT) {
        const int tkn = base + lane;
        uint64_t mask = __ballot(tkn < batch && v[c] == a);
        bool collect = started;
        if (!started) {
          if (base + kWave <= b) {
            pos_b += __popcll(mask);
          } else {
            const int l_b = b - base;
            pos_b += __popcll(mask & ((1ull << l_b) - 1ull));
            if (pos_b % kTT != 0) return;  // b is not the first token of a run
            mask &= ~((1ull << l_b) - 1ull);
            started = true;
            collect = true;
          }
        }
        if (collect) {
          while (mask != 0 && n_tok < kTT) {
            const int i = __builtin_ctzll(mask);
            mask &= mask - 1;
#pragma unroll
            for (int k = 0; k < kTT; ++k)
              if (k == n_tok) it.tok[k] = base + i;
            ++n_tok;
          }
        }
      }
    }
    if (n_tok == kTT) break;
  }
  it.n_tok = n_tok;
  it.a = a;
  it.base = base_a;
  it.r = len > 0 ? (int)(len >> 2) : 0;
}

// Item record of a plan.  The record's address comes from the workgroup id
// only.  Every field (and the page ids of rows jr0 and jr1 of projection pp) is
// read up front and pinned in scalar registers before the first branch, so the
// compiler cannot sink the loads below the early exits: header check, record
// and page ids are ONE round trip of independent scalar loads.
__device__ __forceinline__ void load_item(const int* __restrict__ plan, int idx, int pp, int jr0, int jr1, Item& it,
                                          int& page0, int& page1) {
  // The header and the records do not change while a kernel that reads them runs
  // (the counters behind them do, through another pointer): reading them through
  // the constant address space keeps these loads scalar whatever else the kernel
  // stores.
  typedef const int __attribute__((address_space(4))) * ConstWords;
  ConstWords head = (ConstWords)plan;
  ConstWords rec = head + kPlanHeaderWords + (int64_t)idx * kItemWords;
  int magic = head[PH_MAGIC], n_items = head[PH_NITEMS];
  int a = rec[IT_ADAPTER], r = rec[IT_RANK], n_tok = rec[IT_NTOK], j0 = rec[IT_J0];
  int t0 = rec[IT_TOK + 0], t1 = rec[IT_TOK + 1], t2 = rec[IT_TOK + 2], t3 = rec[IT_TOK + 3];
  int more = rec[IT_MORE];
  int base_lo = rec[IT_BASE], base_hi = rec[IT_BASE + 1];
  int pg0 = rec[IT_PAGES + pp * kRB + jr0], pg1 = rec[IT_PAGES + pp * kRB + jr1];
  asm volatile(""
               : "+s"(magic), "+s"(n_items), "+s"(a), "+s"(r), "+s"(n_tok), "+s"(j0), "+s"(t0), "+s"(t1), "+s"(t2),
                 "+s"(t3), "+s"(more), "+s"(base_lo), "+s"(base_hi), "+s"(pg0), "+s"(pg1));
  static_assert(kTT == 4, "the record holds four token ids");
  it.tok[0] = t0;
  it.tok[1] = t1;
  it.tok[2] = t2;
  it.tok[3] = t3;
  const bool ok = (magic == kPlanMagic) & (idx < n_items);
  it.plan_items = magic == kPlanMagic ? n_items : 0;
  it.a = a;
  it.r = r;
  it.n_tok = ok ? n_tok : 0;
  it.j0 = j0;
  it.more = more;
  it.base = (int64_t)(((uint64_t)(uint32_t)base_hi << 32) | (uint32_t)base_lo);
  page0 = pg0;
  page1 = pg1;
}

// a_loc entry `li` -> page id without a branch around the load: an unwanted or
// out-of-range index reads a_start[0] instead (the table has at least one adapter
// whenever a kernel is launched) and is rejected afterwards
__device__ __forceinline__ int64_t lookup_page_nobranch(const Tables& t, int64_t li, bool want) {
  const bool in = want & ((uint64_t)li < (uint64_t)t.n_loc);
  const int64_t page = *(in ? t.a_loc + li : t.a_start);
  return (in & ((uint64_t)page < (uint64_t)t.n_pages)) ? page : (int64_t)-1;
}

// ---------------------------------------------------------------------------
// shrink
// ---------------------------------------------------------------------------
struct ShrinkArgs {
  void* y[3];
  const void* x;
  const void* w;
  const int* plan;  // nullptr: stateless
  Tables t;
  int64_t page_elems;
  int batch, h_in, y_cols, qkvo0, blocks, lds_tt;
  int strided;  // planned launch with fewer workgroups than the plan may have items (see planned_grid)
};

// The common case in straight-line code: the whole page in one pass (hidden <= 512 * NV
// elements), all tokens of the run fit the LDS staging area, no rows beyond the item.
// Every global load is unconditional (absent tokens / rows read a valid dummy address
// and are discarded) so that no branch separates the loads: first the activations, then
// both weight pages; the LDS stores wait for the activations only.
// NV: 16-byte vectors a lane holds of a page (8 = hidden up to 4096).
template <typename T, int NV>
__device__ __forceinline__ void shrink_fast(const ShrinkArgs& p, const Item& it, int proj, int r_eff,
                                            const int64_t (&page)[2], u32x4* s_x) {
  constexpr int XS = (NV + 3) / 4;  // activation vectors a thread stages per token
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nvec = p.h_in >> 3;
  const u32x4* xg = reinterpret_cast<const u32x4*>(p.x);
  const uint16_t* wbase = reinterpret_cast<const uint16_t*>(p.w);

  u32x4 xr[kTT][XS];
#pragma unroll
  for (int t = 0; t < kTT; ++t) {
    const int tk = t < it.n_tok ? it.tok[t] : it.tok[0];
    const u32x4* xrow = xg + (int64_t)tk * nvec;
#pragma unroll
    for (int i = 0; i < XS; ++i) {
      const int v = i * 256 + tid;
      xr[t][i] = xrow[v < nvec ? v : 0];
    }
  }
  __builtin_amdgcn_sched_barrier(0);  // keep the activation loads in front: the LDS stores wait for them only
  u32x4 wv[2][NV];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const u32x4* src = reinterpret_cast<const u32x4*>(wbase + (page[i] >= 0 ? page[i] : 0) * p.page_elems);
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      const int v = c * kWave + lane;
      wv[i][c] = ldg16_stream(src + (v < nvec ? v : 0));
    }
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int t = 0; t < kTT; ++t)
#pragma unroll
    for (int i = 0; i < XS; ++i) {
      const int v = i * 256 + tid;
      if (t < it.n_tok && v < nvec) s_x[t * nvec + v] = xr[t][i];
    }
  __syncthreads();

  float acc[2][kTT];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int t = 0; t < kTT; ++t) acc[i][t] = 0.f;
#pragma unroll
  for (int t = 0; t < kTT; ++t) {
    if (t < it.n_tok) {
#pragma unroll
      for (int c = 0; c < NV; ++c) {
        const int v = c * kWave + lane;
        if (v < nvec) {
          const u32x4 xv = s_x[t * nvec + v];
#pragma unroll
          for (int i = 0; i < 2; ++i) acc[i][t] = dot8<T>(wv[i][c], xv, acc[i][t]);
        }
      }
    }
  }
  uint16_t* y = reinterpret_cast<uint16_t*>(p.y[proj]);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = it.j0 + wave + 4 * i;
#pragma unroll
    for (int t = 0; t < kTT; ++t) {
      if (t < it.n_tok) {
        const float sum = wave_sum(acc[i][t]);
        if (lane == 0 && page[i] >= 0 && row < r_eff) {
          y[(int64_t)it.tok[t] * p.y_cols + row] = T::from_float(sum);
        }
      }
    }
  }
}

// 4 wavefronts; wavefront w takes rows j0+w and j0+w+4 of one projection.  A
// q/k/v call launches three workgroups per item (grid y = projection: workgroup ids
// run item-fastest, so with a multiple of 8 items all three land on the item's XCD
// and share its activations in that L2).
// Grid: x = item (planned) or token * blocks + block (stateless), y = projection of the
// launch.  s_x: [lds_tt][h_in / 8] LDS words.
template <typename T, bool PLANNED, int NV>
__device__ __forceinline__ int shrink_body(const ShrinkArgs& p, int unit, int proj, u32x4* s_x) {
  constexpr int NW = 4;
  constexpr int NTASK = 2;
  constexpr int NT = NW * kWave;
  constexpr int kSlab = 512 / NT;  // 16-byte vectors per thread, token and 4096-element slab
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  Item it;
  const int* rec = PLANNED ? p.plan + kPlanHeaderWords + (int64_t)unit * kItemWords : nullptr;
  int plan_pg0 = -1, plan_pg1 = -1;
  if (PLANNED) {
    load_item(p.plan, unit, p.qkvo0 + proj, wave, wave + 4, it, plan_pg0, plan_pg1);
  } else {
    const int b = unit / p.blocks;
    discover_run(p.t, p.batch, b, it);
    it.j0 = (unit - b * p.blocks) * kRB;
  }
  // page ids of this wavefront's two rows, read before any branch
  int64_t page2[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int jr = wave + 4 * i;
    if (PLANNED)
      page2[i] = i == 0 ? plan_pg0 : plan_pg1;
    else
      page2[i] = lookup_page_nobranch(p.t, it.base + (int64_t)it.r * (p.qkvo0 + proj) + it.j0 + jr,
                                      it.n_tok > 0 && p.t.n_loc > 0);
  }
  if (it.n_tok <= 0) return it.plan_items;
  const int r_eff = it.r < p.y_cols ? it.r : p.y_cols;
  if (it.j0 >= r_eff) return it.plan_items;  // uniform over the workgroup

  const int nvec = p.h_in >> 3;
  if (nvec <= NV * kWave && it.n_tok <= p.lds_tt && !(PLANNED && it.more)) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
      if (it.j0 + wave + 4 * i >= r_eff) page2[i] = -1;
    shrink_fast<T, NV>(p, it, proj, r_eff, page2, s_x);
    return it.plan_items;
  }
  const uint16_t* wbase = reinterpret_cast<const uint16_t*>(p.w);
  int row[NTASK];
  const u32x4* wrow[NTASK];
  u32x4 wv[NTASK][kVecPerPass];

  // rows jb .. jb+7 of the run: page pointers, and the first pass of this
  // wavefront's pages goes in flight before anything waits
  auto open_block = [&](int jb, bool from_plan) {
#pragma unroll
    for (int i = 0; i < NTASK; ++i) {
      const int jr = wave + 4 * i;  // row inside the block
      row[i] = jb + jr;
      wrow[i] = nullptr;
      if (row[i] < r_eff) {
        int64_t page;
        if (PLANNED && from_plan)
          page = rec[IT_PAGES + (p.qkvo0 + proj) * kRB + jr];
        else
          page = lookup_page(p.t, it.base + (int64_t)it.r * (p.qkvo0 + proj) + row[i]);
        if (page >= 0) wrow[i] = reinterpret_cast<const u32x4*>(wbase + page * p.page_elems);
      }
    }
#pragma unroll
    for (int i = 0; i < NTASK; ++i)
#pragma unroll
      for (int c = 0; c < kVecPerPass; ++c) {
        const int v = c * kWave + lane;
        wv[i][c] = (wrow[i] != nullptr && v < nvec) ? wrow[i][v] : zero16();
      }
  };
  open_block(it.j0, true);
  // a plan lists rows up to rank_cap; the run's last listed block also takes the rows beyond
  const int j_end = (PLANNED && it.more) ? r_eff : it.j0 + kRB;

  const u32x4* xg = reinterpret_cast<const u32x4*>(p.x);
  const int vec_per_pass = kVecPerPass * kWave;

  for (int t0 = 0; t0 < it.n_tok; t0 += p.lds_tt) {
    const int nt = it.n_tok - t0 < p.lds_tt ? it.n_tok - t0 : p.lds_tt;
    if (t0 != 0) __syncthreads();
    // stage the activations of these tokens: every row is read once per
    // workgroup; all loads of a slab are issued before the first LDS store
    for (int v0 = 0; v0 < nvec; v0 += kSlab * NT) {
      u32x4 xr[kTT][kSlab];
#pragma unroll
      for (int t = 0; t < kTT; ++t) {
        const u32x4* xrow = xg + (int64_t)item_token(it, t0 + t) * nvec;
#pragma unroll
        for (int i = 0; i < kSlab; ++i) {
          const int v = v0 + i * NT + tid;
          xr[t][i] = (t < nt && v < nvec) ? xrow[v] : zero16();
        }
      }
#pragma unroll
      for (int t = 0; t < kTT; ++t)
#pragma unroll
        for (int i = 0; i < kSlab; ++i) {
          const int v = v0 + i * NT + tid;
          if (t < nt && v < nvec) s_x[t * nvec + v] = xr[t][i];
        }
    }
    __syncthreads();

    for (int jb = it.j0; jb < j_end; jb += kRB) {
      if (jb != it.j0 || t0 != 0) open_block(jb, jb == it.j0);
      float acc[NTASK][kTT];
#pragma unroll
      for (int i = 0; i < NTASK; ++i)
#pragma unroll
        for (int t = 0; t < kTT; ++t) acc[i][t] = 0.f;
      for (int v0 = 0; v0 < nvec; v0 += vec_per_pass) {
        if (v0 != 0) {
#pragma unroll
          for (int i = 0; i < NTASK; ++i)
#pragma unroll
            for (int c = 0; c < kVecPerPass; ++c) {
              const int v = v0 + c * kWave + lane;
              wv[i][c] = (wrow[i] != nullptr && v < nvec) ? wrow[i][v] : zero16();
            }
        }
#pragma unroll
        for (int t = 0; t < kTT; ++t) {
          if (t < nt) {
#pragma unroll
            for (int c = 0; c < kVecPerPass; ++c) {
              const int v = v0 + c * kWave + lane;
              if (v < nvec) {
                const u32x4 xv = s_x[t * nvec + v];
#pragma unroll
                for (int i = 0; i < NTASK; ++i) acc[i][t] = dot8<T>(wv[i][c], xv, acc[i][t]);
              }
            }
          }
        }
      }
      uint16_t* y = reinterpret_cast<uint16_t*>(p.y[proj]);
#pragma unroll
      for (int i = 0; i < NTASK; ++i) {
#pragma unroll
        for (int t = 0; t < kTT; ++t) {
          if (t < nt) {
            const float s = wave_sum(acc[i][t]);
            if (lane == 0 && wrow[i] != nullptr) {
              y[(int64_t)item_token(it, t0 + t) * p.y_cols + row[i]] = T::from_float(s);
            }
          }
        }
      }
    }
  }
  return it.plan_items;
}

// NV: the straight-line path of this instantiation holds pages of up to 512 * NV elements
// (8: hidden <= 4096; larger ones cost registers, so the host picks the smallest that fits)
template <typename T, bool PLANNED, int NV>
__global__ __launch_bounds__(256) void bgmv_shrink_kernel(const ShrinkArgs p) {
  extern __shared__ u32x4 s_x[];  // [lds_tt][h_in / 8]
  int unit = (int)blockIdx.x;
  const int n_items = shrink_body<T, PLANNED, NV>(p, unit, (int)blockIdx.y, s_x);
  if (PLANNED && p.strided) {
    // a launch sized for a fraction of the plan's capacity: the items beyond the grid, if the
    // batch has that many, are walked here (uniform over the workgroup)
    for (unit += (int)gridDim.x; unit < n_items; unit += (int)gridDim.x) {
      __syncthreads();  // the staging area of the item before is free
      shrink_body<T, PLANNED, NV>(p, unit, (int)blockIdx.y, s_x);
    }
  }
}

// ---------------------------------------------------------------------------
// expand
// ---------------------------------------------------------------------------
struct ExpandArgs {
  void* y[3];
  const void* x[3];
  const void* w;
  const void* scales;
  const int* plan;
  Tables t;
  int64_t page_elems;
  int scales_dtype;
  int batch, x_cols, qkvo0, blocks, y_aligned;
  int interleave;  // one-dimensional grid: the workgroups of an item follow each other (see bgmv_expand_kernel)
  int strided;     // planned launch with fewer workgroups than the plan may have items (see planned_grid)
  int n_units;     // items (planned) or token blocks (stateless) of the launch
  int h_out[3];
  // pages per rank row of each projection: a rank-r adapter's B^T fills ceil(r * h_out /
  // page_elems) pages.  pages_shift >= 0: page_elems = h_out << pages_shift (the count is a
  // shift); -1: h_out >= page_elems (all r pages); -2: neither (a division on the device).
  int pages_shift[3];
};

// One exchange of a reduce-scatter over the lanes that share an output: a lane holds N
// partial sums (one per load of the pass); the lane with `up` keeps the upper N/2 and
// hands the lower N/2 to its partner, the other lane the reverse, and each adds what it
// receives to what it keeps.  CTRL is the DPP pattern that names the partner.
template <int CTRL, int N>
__device__ __forceinline__ void rs_stage(float (&v)[kVecPerPass], bool up) {
#pragma unroll
  for (int i = 0; i < N / 2; ++i) {
    const float keep = up ? v[i + N / 2] : v[i];
    const float send = up ? v[i] : v[i + N / 2];
    const int got = __builtin_amdgcn_update_dpp(0, __float_as_int(send), CTRL, 0xf, 0xf, false);
    v[i] = keep + __int_as_float(got);
  }
}

// Sum the 8 partial sums of a pass (one per load) over the LPO lanes that share an
// output and file them, scaled and rounded to the storage type, in the wavefront's LDS
// strip at [c * OPW + g] (load c, lane group g): the strip then holds the pass's outputs
// in order.  The sums are reduce-scattered: every exchange halves what a lane holds, so
// that the LPO lanes of a group end up with 8 / LPO different loads each (lane li of the
// group with loads li * 8 / LPO + i) and every lane writes only sums nobody else has.
// The first exchanges use the mirror patterns (their partners differ in all lower lane
// bits, which is fine while every lane still holds every load), the last ones xor 2 and
// xor 1, which keep the upper bits that by then decide what a lane holds.
template <typename T, int LPO>
__device__ __forceinline__ void file_sums(float (&v)[kVecPerPass], float scale, int lane, uint16_t* s_strip) {
  static_assert(LPO == 1 || LPO == 2 || LPO == 4 || LPO == 8 || LPO == 16, "lanes per output");
  constexpr int OPW = kWave / LPO;
  constexpr int kRowMirror = 0x140, kHalfMirror = 0x141, kXor2 = 0x4E, kXor1 = 0xB1;
  if (LPO == 16) {
    rs_stage<kRowMirror, 8>(v, (lane & 8) != 0);
    rs_stage<kHalfMirror, 4>(v, (lane & 4) != 0);
    rs_stage<kXor2, 2>(v, (lane & 2) != 0);
    v[0] = dpp_add<kXor1>(v[0]);  // both lanes of the last pair hold the sum; either may write it
  } else if (LPO == 8) {
    rs_stage<kHalfMirror, 8>(v, (lane & 4) != 0);
    rs_stage<kXor2, 4>(v, (lane & 2) != 0);
    rs_stage<kXor1, 2>(v, (lane & 1) != 0);
  } else if (LPO == 4) {
    rs_stage<kXor2, 8>(v, (lane & 2) != 0);
    rs_stage<kXor1, 4>(v, (lane & 1) != 0);
  } else if (LPO == 2) {
    rs_stage<kXor1, 8>(v, (lane & 1) != 0);
  }
  constexpr int NV = LPO >= 8 ? 1 : kVecPerPass / LPO;  // sums this lane holds now
  const int li = lane % LPO, g = lane / LPO;
  const int c0 = LPO == 16 ? li >> 1 : li * NV;
#pragma unroll
  for (int i = 0; i < NV; ++i) s_strip[(c0 + i) * OPW + g] = T::from_float(v[i] * scale);
}

// One page of the flattened (h_out, r) matrix B^T for one run, rank r a power
// of two (8..128) that divides the page: r/8 lanes share an output, so a
// wavefront-wide 16-byte load covers 512/r consecutive outputs.  The reduced,
// scaled sums of a pass are transposed through an LDS strip of the wavefront
// so that the read-modify-write of y is one 16-byte load and one 16-byte store
// per lane and token.
// NV: 16-byte vectors a lane holds per pass, i.e. a pass covers 512 * NV elements; the host
// picks the smallest NV whose pass holds the whole page (8, 10, 12, 16: pages of up to 4096,
// 5120, 6144, 8192 elements), so that every load of the page is issued before the first wait.
// Wider pages take several passes.
// FULL: every element of the page belongs to an output inside h_out and every rank
// column is used (the caller checks: whole passes, page inside the output, delta as wide
// as the rank) -- then no load needs its result masked.
template <int NV>
struct ExpandPass {
  static constexpr int kElems = NV * kWave * 8;            // elements per pass
  static constexpr int kGroups = (NV + kVecPerPass - 1) / kVecPerPass;  // groups of 8 loads whose sums are filed together
  static constexpr int kStrip = kGroups * kVecPerPass * kWave;          // 16-bit entries of a wavefront's LDS strip
};

template <typename T, bool FULL, int NV>
__device__ __forceinline__ void expand_page(const ExpandArgs& p, int proj, const Item& it, int r_eff,
                                            const uint16_t* wpage, int64_t flat0, float scale, uint16_t* s_strip) {
  constexpr int kPass = ExpandPass<NV>::kElems;
  const int lane = threadIdx.x & 63;
  const int r = it.r;
  const int lg_r = __builtin_ctz((unsigned)r);
  const int lpo = r >> 3;
  const int d0 = (lane & (lpo - 1)) * 8;
  const bool d_ok = FULL || d0 < r_eff;
  const int page_elems = (int)p.page_elems;
  const int out_per_pass = kPass >> lg_r;
  const int opw = kWave >> (lg_r - 3);  // outputs a wavefront-wide load covers
  const int n_page0 = (int)(flat0 >> lg_r);  // first output of this page
  // outputs of this page: [n_page0, n_end); later pages own what lies beyond
  const int n_page_end = n_page0 + (page_elems >> lg_r);
  const int h_stride = p.h_out[proj];
  const int n_end = h_stride < n_page_end ? h_stride : n_page_end;
  uint16_t* y = reinterpret_cast<uint16_t*>(p.y[proj]);
  const uint16_t* x = reinterpret_cast<const uint16_t*>(p.x[proj]);

  // first pass of the page and the run's delta fragments go in flight together
  u32x4 wv[NV];
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int e = (c * kWave + lane) * 8;
    if (FULL) {
      wv[c] = ldg16_stream(wpage + e);
    } else {
      const bool w_ok = d_ok && e < page_elems && n_page0 + (e >> lg_r) < n_end;
      wv[c] = w_ok ? ldg16_stream(wpage + e) : zero16();
    }
  }
  u32x4 xv[kTT];
#pragma unroll
  for (int t = 0; t < kTT; ++t) {
    if (FULL)  // a token the run does not have re-reads the first one's row; its sums are never used
      xv[t] = ldg16(x + (int64_t)(t < it.n_tok ? it.tok[t] : it.tok[0]) * p.x_cols + d0);
    else
      xv[t] = (t < it.n_tok && d_ok) ? ldg16(x + (int64_t)it.tok[t] * p.x_cols + d0) : zero16();
  }

  for (int e0 = 0; e0 < page_elems; e0 += kPass) {
    if (e0 != 0) {
#pragma unroll
      for (int c = 0; c < NV; ++c) {
        const int e = e0 + (c * kWave + lane) * 8;
        if (FULL) {
          wv[c] = ldg16_stream(wpage + e);
        } else {
          const bool w_ok = d_ok && e < page_elems && n_page0 + (e >> lg_r) < n_end;
          wv[c] = w_ok ? ldg16_stream(wpage + e) : zero16();
        }
      }
    }
    // this lane's 8 consecutive outputs of the pass (of its first 512 outputs: a pass has more
    // only for rank 8 and NV > 8, and those follow in further steps)
    const int n_pass0 = n_page0 + (e0 >> lg_r);
    const int n_mine = n_pass0 + lane * 8;
    const bool y_ok = lane * 8 < out_per_pass && n_mine < n_end;
    u32x4 yv[kTT];
#pragma unroll
    for (int t = 0; t < kTT; ++t) {
      if (FULL) {  // lanes with no outputs re-read the page's first ones; the values are not used
        yv[t] = ldg16_stream(y + (int64_t)(t < it.n_tok ? it.tok[t] : it.tok[0]) * h_stride +
                             (y_ok ? n_mine : n_page0));
      } else {
        const uint16_t* yp = y + (int64_t)it.tok[t] * h_stride + n_mine;
        yv[t] = (t < it.n_tok && y_ok) ? ldg16_stream(yp) : zero16();
      }
    }
#pragma unroll
    for (int t = 0; t < kTT; ++t) {
      if (t < it.n_tok) {
        // partial sums of the pass, eight loads at a time (a last group of fewer loads is
        // padded with zeros, which add nothing)
#pragma unroll
        for (int g8 = 0; g8 < ExpandPass<NV>::kGroups; ++g8) {
          float part[kVecPerPass];
#pragma unroll
          for (int c = 0; c < kVecPerPass; ++c)
            part[c] = g8 * kVecPerPass + c < NV ? dot8<T>(wv[g8 * kVecPerPass + c], xv[t], 0.f) : 0.f;
          uint16_t* strip = s_strip + g8 * kVecPerPass * opw;
          switch (lpo) {
            case 1: file_sums<T, 1>(part, scale, lane, strip); break;
            case 2: file_sums<T, 2>(part, scale, lane, strip); break;
            case 4: file_sums<T, 4>(part, scale, lane, strip); break;
            case 8: file_sums<T, 8>(part, scale, lane, strip); break;
            default: file_sums<T, 16>(part, scale, lane, strip); break;
          }
        }
        // the same wavefront wrote the strip: its LDS operations complete in order
        const u32x4 dv = *reinterpret_cast<const u32x4*>(s_strip + (y_ok ? lane * 8 : 0));
        if (y_ok) {
          u32x4 out;
#pragma unroll
          for (int q = 0; q < 4; ++q) out[q] = T::add2(yv[t][q], dv[q]);
          stg16_stream(y + (int64_t)it.tok[t] * h_stride + n_mine, out);
        }
        if (NV > kVecPerPass) {
          // outputs 512.. of the pass (rank 8 only): y is loaded here, behind the sums
          for (int s0 = 8 * kWave; s0 < out_per_pass; s0 += 8 * kWave) {
            const int n2 = n_pass0 + s0 + lane * 8;
            if (s0 + lane * 8 < out_per_pass && n2 < n_end) {
              uint16_t* yp = y + (int64_t)it.tok[t] * h_stride + n2;
              const u32x4 y2 = ldg16_stream(yp);
              const u32x4 d2 = *reinterpret_cast<const u32x4*>(s_strip + s0 + lane * 8);
              u32x4 out;
#pragma unroll
              for (int q = 0; q < 4; ++q) out[q] = T::add2(y2[q], d2[q]);
              stg16_stream(yp, out);
            }
          }
        }
      }
    }
  }
}

// Any rank, any alignment: one lane per output whose first element lies in this
// page, element-wise loads through a_loc (an output's r elements may continue
// on the next page).
template <typename T>
__device__ __forceinline__ void expand_scalar(const ExpandArgs& p, int proj, const Item& it, int r_eff, int k,
                                              int64_t base_li, float scale) {
  const int h_out = p.h_out[proj];
  const int r = it.r;
  const int64_t pe = p.page_elems;
  int64_t n_lo = (k * pe + r - 1) / r, n_hi = ((k + 1) * pe + r - 1) / r;
  if (n_hi > h_out) n_hi = h_out;
  const uint16_t* wbase = reinterpret_cast<const uint16_t*>(p.w);
  uint16_t* y = reinterpret_cast<uint16_t*>(p.y[proj]);
  const uint16_t* x = reinterpret_cast<const uint16_t*>(p.x[proj]);
  const int lane = threadIdx.x & 63;
  for (int64_t n = n_lo + lane; n < n_hi; n += kWave) {
    for (int t = 0; t < it.n_tok; ++t) {
      const int bt = item_token(it, t);
      float acc = 0.f;
      for (int d = 0; d < r_eff; ++d) {
        const int64_t flat = n * r + d;
        const int64_t pg = flat / pe, off = flat - pg * pe;
        const int64_t page = lookup_page(p.t, base_li + pg);
        if (page < 0) continue;
        const float wf = T::to_float(wbase[page * pe + off]);
        acc = __builtin_fmaf(wf, T::to_float(x[(int64_t)bt * p.x_cols + d]), acc);
      }
      uint16_t* yp = y + (int64_t)bt * h_out + n;
      *yp = T::add(*yp, T::from_float(acc * scale));
    }
  }
}

// Page kk of projection `proj` for the item's run; `page` is its pool page id
// or -2 to look it up in a_loc.
template <typename T, int NV>
__device__ __forceinline__ void expand_one(const ExpandArgs& p, int proj, const Item& it, int r_eff, int kk,
                                           int64_t page, bool vec_ok, uint16_t* s_strip) {
  const int64_t base_li = it.base + (int64_t)it.r * (p.qkvo0 + proj);
  if (!vec_ok) {
    expand_scalar<T>(p, proj, it, r_eff, kk, base_li, load_scale(p.scales, p.scales_dtype, it.a));
    return;
  }
  if (page == -2) page = lookup_page(p.t, base_li + kk);
  if (page < 0) return;
  const uint16_t* wpage = reinterpret_cast<const uint16_t*>(p.w) + page * p.page_elems;
  const int64_t flat0 = (int64_t)kk * p.page_elems;
  const float scale = load_scale(p.scales, p.scales_dtype, it.a);
  // the whole page lies inside the output, in whole passes, and delta is as wide as the rank
  const bool full = r_eff == it.r && p.page_elems % ExpandPass<NV>::kElems == 0 &&
                    flat0 + p.page_elems <= (int64_t)p.h_out[proj] * it.r;
  if (full)
    expand_page<T, true, NV>(p, proj, it, r_eff, wpage, flat0, scale, s_strip);
  else
    expand_page<T, false, NV>(p, proj, it, r_eff, wpage, flat0, scale, s_strip);
}

// Expand has nothing to share between wavefronts (the delta row is 16 bytes per
// lane), so every wavefront takes exactly one page: a workgroup is 4 wavefronts
// = half of one projection's 8-page block of an item, and an item gets
// 2 * NPROJ workgroups.
// Grid: x = item (planned) or token * blocks + block (stateless), y = projection * 2 +
// half: workgroup ids run item-fastest, so with a multiple of 8 items every workgroup of
// an item lands on XCD item % 8.
template <typename T, int NPROJ, bool PLANNED, int NV>
__device__ __forceinline__ int expand_body(const ExpandArgs& p, int unit, int sub, uint16_t* s_strip) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int proj = sub >> 1;
  const int jr = (sub & 1) * 4 + wave;  // page inside the item's block

  Item it;
  int plan_pg = -1, plan_pg_unused = -1;
  if (PLANNED) {
    load_item(p.plan, unit, p.qkvo0 + proj, jr, jr, it, plan_pg, plan_pg_unused);
  } else {
    const int b = unit / p.blocks;
    discover_run(p.t, p.batch, b, it);
    it.j0 = (unit - b * p.blocks) * kRB;
  }
  if (it.n_tok <= 0) return it.plan_items;
  const int r = it.r;
  const int r_eff = r < p.x_cols ? r : p.x_cols;
  if (r_eff <= 0) return it.plan_items;
  const int k = it.j0 + jr;
  // pages that hold this projection's h_out * r elements
  const int sh = p.pages_shift[proj];
  int n_pg = r;
  if (sh >= 0)
    n_pg = (r + (1 << sh) - 1) >> sh;
  else if (sh == -2)
    n_pg = r > 512 ? (int)(((int64_t)p.h_out[proj] * r + p.page_elems - 1) / p.page_elems)
                   : (int)(((uint32_t)p.h_out[proj] * (uint32_t)r + (uint32_t)p.page_elems - 1u) /
                           (uint32_t)p.page_elems);
  if (n_pg > r) n_pg = r;
  // Pages the launch does not enumerate: the stateless grid stops at the delta
  // width and a plan at rank_cap; an adapter of larger rank has more, which
  // the wavefronts of the last enumerated block take in further rounds.
  bool extra = false;
  if (PLANNED)
    extra = it.more != 0;
  else
    extra = it.j0 + kRB >= p.blocks * kRB;
  const bool has_work = k < n_pg || extra;
  if (!has_work) return it.plan_items;
  const bool pow2 = (r & (r - 1)) == 0;
  // the vector path reads and writes y 16 bytes at a time: rows and page boundaries must fall on multiples of 8 outputs
  const bool vec_ok = pow2 && r >= 8 && r <= 128 && (r_eff & 7) == 0 && (p.x_cols & 7) == 0 &&
                      (p.page_elems & (8 * r - 1)) == 0 && (p.h_out[proj] & 7) == 0 && p.y_aligned != 0;
  if (k < n_pg) {
    const int64_t page = PLANNED ? (int64_t)plan_pg : (int64_t)-2;
    expand_one<T, NV>(p, proj, it, r_eff, k, page, vec_ok, s_strip);
  }
  if (extra) {
#pragma unroll 1
    for (int kk = k + kRB; kk < n_pg; kk += kRB) expand_one<T, NV>(p, proj, it, r_eff, kk, -2, vec_ok, s_strip);
  }
  return it.plan_items;
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
constexpr int kXcds = 8;
enum { SC_ADAPTER = 0, SC_TOKEN = 1, SC_RANK = 2, SC_ITEMS = 3, SC_WORK = 4, SC_QUEUE = 5, SC_WORDS = 6 };

// Builds the item list.  Runs are sorted by adapter, then cut into 8 queues of
// equal work, one per XCD: consecutive workgroup ids go to the XCDs in turn, so
// queue q's k-th item is stored at index k*8 + q.  All items of a run, and all
// runs of an adapter (up to a cut), then execute on one XCD: the run's
// activations and an adapter's pages shared by several runs are fetched by a
// single L2.  Queues are padded to the longest with empty items.
__global__ __launch_bounds__(kPlanThreads) void bgmv_plan_kernel(int* __restrict__ plan, Tables t, int batch,
                                                                 int rank_cap, int max_items,
                                                                 int* __restrict__ scratch) {
  __shared__ int s_bins[kMaxLdsBins];
  __shared__ int s_ra[kMaxLdsRuns], s_rb[kMaxLdsRuns], s_rn[kMaxLdsRuns];
  __shared__ int s_wave[kPlanWaves];
  __shared__ int s_max_rank, s_total;
  __shared__ int s_qstart[kXcds], s_qlen[kXcds];
  const int tid = threadIdx.x;
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
                                                                      int rank_cap, int max_items) {
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
                                                                      int rank_cap, int max_items, int n) {
  extern __shared__ __align__(16) unsigned char s_dyn[];
  uint32_t* s_key = reinterpret_cast<uint32_t*>(s_dyn);                // sorted: adapter << 13 | token, ~0: no member
  int* s_before = reinterpret_cast<int*>(s_key + n);                   // run -> items in front of it
  uint16_t* s_spos = reinterpret_cast<uint16_t*>(s_before + (n + 1));  // run -> sorted position of its first token
  __shared__ int s_wave[kPlanWaves];
  __shared__ int s_max_rank;
  __shared__ int s_qstart[kXcds], s_qlen[kXcds];
  constexpr uint32_t kNone = 0xffffffffu;
  const int tid = threadIdx.x;
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
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
int fill_tables(Tables& t, const slora_tables* in, const int64_t* bins, int64_t n_pages) {
  if (in == nullptr || in->a_start == nullptr || in->a_len == nullptr || in->a_loc == nullptr || bins == nullptr)
    return SLORA_ERR_NULL_POINTER;
  if (in->n_adapters < 0 || in->n_loc < 0 || n_pages < 0) return SLORA_ERR_BAD_SHAPE;
  if (n_pages == 0 && in->n_loc > 0) return SLORA_ERR_BAD_SHAPE;  // page ids, but no pool they could name
  t.a_start = in->a_start;
  t.a_len = in->a_len;
  t.a_loc = in->a_loc;
  t.bins = bins;
  t.n_adapters = in->n_adapters;
  t.n_loc = in->n_loc;
  t.n_pages = n_pages;
  return SLORA_OK;
}

constexpr size_t kLdsSoftLimit = 64 * 1024;
constexpr size_t kLdsHardLimit = 160 * 1024 - 256;

// item capacity of a plan: every run's items plus the padding that evens out the 8 queues
// (a whole number of groups of 8, so that a launch sized for the capacity keeps item i on XCD i % 8)
int64_t plan_max_items(int64_t batch, int64_t rank_cap) {
  const int64_t per_run = (rank_cap + kRB - 1) / kRB;
  return (batch * per_run + kXcds - 1) / kXcds * kXcds + kXcds * (per_run + 1);
}
// int32 words of the builder's scratch area behind the items
int64_t plan_scratch_words(int64_t batch) { return batch * SC_WORDS; }
int64_t plan_words(int64_t batch, int64_t rank_cap) {
  return kPlanHeaderWords + plan_max_items(batch, rank_cap) * kItemWords + plan_scratch_words(batch);
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

// Grid of a planned launch: the items the caller read back.  Without that count (a plan rebuilt
// in place, or built inside a graph capture) the plan's capacity is the only bound the host
// has, several times what a batch usually needs, and every workgroup of an item that does not
// exist still costs its hand-out and one round trip.  Such launches get a quarter of the
// capacity (a multiple of 8, so that item i stays on XCD i % 8) and their workgroups walk the
// items in strides of the grid: a usual batch fits the grid, a batch of many short runs makes
// a workgroup do up to four items one after the other.
int64_t planned_grid(int64_t n_items, int64_t batch, int64_t rank_cap, int& strided) {
  const int64_t cap = plan_max_items(batch, rank_cap);
  strided = 0;
  if (n_items > 0 && n_items < cap) return n_items;
  if (cap <= 64 * kXcds) return cap;
  strided = 1;
  return (cap / 4 + kXcds - 1) / kXcds * kXcds;
}

constexpr int kNothingToDo = 1;  // a valid call with no work; callers turn it into SLORA_OK

// Checks the arguments of a shrink call and fills the kernel arguments and grid.
int shrink_prepare(const void* plan, int64_t n_items, int64_t rank_cap, void* const y[3], int nproj, int qkvo0,
                   const void* x, const void* w, const slora_tables* tables, const int64_t* bins, int64_t batch,
                   int64_t h_in, int64_t y_cols, int64_t page_elems, int64_t n_pages, int dtype, ShrinkArgs& p,
                   int64_t& grid) {
  if (dtype != SLORA_DTYPE_F16 && dtype != SLORA_DTYPE_BF16) return SLORA_ERR_BAD_DTYPE;
  if (batch < 0 || h_in < 0 || y_cols < 0 || page_elems < 0 || n_items < 0) return SLORA_ERR_BAD_SHAPE;
  if (qkvo0 < 0 || qkvo0 + nproj > 4) return SLORA_ERR_BAD_SHAPE;
  if (batch == 0 || y_cols == 0) return kNothingToDo;
  int rc = fill_tables(p.t, tables, bins, n_pages);
  if (rc != SLORA_OK) return rc;
  // no adapter or no adapter page: every lookup would be rejected
  if (p.t.n_adapters == 0 || p.t.n_loc == 0) return kNothingToDo;
  if (x == nullptr || w == nullptr) return SLORA_ERR_NULL_POINTER;
  for (int i = 0; i < nproj; ++i)
    if (y[i] == nullptr) return SLORA_ERR_NULL_POINTER;
  if (h_in == 0 || (h_in & 7) != 0 || (page_elems & 7) != 0 || h_in > page_elems) return SLORA_ERR_UNSUPPORTED;
  if (y_cols > SLORA_MAX_RANK || batch > (1 << 24) || h_in > (1 << 21) || page_elems > (1LL << 30))
    return SLORA_ERR_UNSUPPORTED;
  if (!aligned16(x) || !aligned16(w)) return SLORA_ERR_ALIGNMENT;
  for (int i = 0; i < 3; ++i) p.y[i] = i < nproj ? y[i] : nullptr;
  p.x = x;
  p.w = w;
  p.plan = static_cast<const int*>(plan);
  p.page_elems = page_elems;
  p.batch = (int)batch;
  p.h_in = (int)h_in;
  p.y_cols = (int)y_cols;
  p.qkvo0 = qkvo0;
  p.blocks = (int)((y_cols + kRB - 1) / kRB);
  p.strided = 0;
  grid = plan != nullptr ? planned_grid(n_items, batch, rank_cap, p.strided) : batch * p.blocks;
  return SLORA_OK;
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

int expand_prepare(const void* plan, int64_t n_items, int64_t rank_cap, void* const y[3], const void* const x[3],
                   const int64_t h_out[3], int nproj, int qkvo0, const void* w, const slora_tables* tables,
                   const int64_t* bins, const void* scales, int scales_dtype, int64_t batch, int64_t x_cols,
                   int64_t page_elems, int64_t n_pages, int dtype, ExpandArgs& p, int64_t& grid) {
  if (dtype != SLORA_DTYPE_F16 && dtype != SLORA_DTYPE_BF16) return SLORA_ERR_BAD_DTYPE;
  if (scales_dtype != SLORA_DTYPE_F16 && scales_dtype != SLORA_DTYPE_BF16 && scales_dtype != SLORA_DTYPE_F32)
    return SLORA_ERR_BAD_DTYPE;
  if (batch < 0 || x_cols < 0 || page_elems < 0 || n_items < 0) return SLORA_ERR_BAD_SHAPE;
  for (int i = 0; i < nproj; ++i)
    if (h_out[i] < 0) return SLORA_ERR_BAD_SHAPE;
  if (qkvo0 < 0 || qkvo0 + nproj > 4) return SLORA_ERR_BAD_SHAPE;
  if (batch == 0 || x_cols == 0) return kNothingToDo;
  int rc = fill_tables(p.t, tables, bins, n_pages);
  if (rc != SLORA_OK) return rc;
  if (p.t.n_adapters == 0 || p.t.n_loc == 0) return kNothingToDo;
  if (w == nullptr || scales == nullptr) return SLORA_ERR_NULL_POINTER;
  for (int i = 0; i < nproj; ++i)
    if (y[i] == nullptr || x[i] == nullptr) return SLORA_ERR_NULL_POINTER;
  if (page_elems == 0 || (page_elems & 7) != 0) return SLORA_ERR_UNSUPPORTED;
  if (x_cols > SLORA_MAX_RANK || batch > (1 << 24) || page_elems > (1LL << 30)) return SLORA_ERR_UNSUPPORTED;
  for (int i = 0; i < nproj; ++i)
    if (h_out[i] > (1 << 21)) return SLORA_ERR_UNSUPPORTED;
  if (!aligned16(w)) return SLORA_ERR_ALIGNMENT;
  if ((x_cols & 7) == 0)
    for (int i = 0; i < nproj; ++i)
      if (!aligned16(x[i])) return SLORA_ERR_ALIGNMENT;
  int64_t h_max = 0;
  for (int i = 0; i < 3; ++i) {
    p.y[i] = i < nproj ? y[i] : nullptr;
    p.x[i] = i < nproj ? x[i] : nullptr;
    p.h_out[i] = i < nproj ? (int)h_out[i] : 0;
    p.pages_shift[i] = -2;
    if (i < nproj && h_out[i] > 0) {
      if (h_out[i] >= page_elems) {
        p.pages_shift[i] = -1;
      } else if (page_elems % h_out[i] == 0) {
        const int64_t q = page_elems / h_out[i];
        if ((q & (q - 1)) == 0) p.pages_shift[i] = __builtin_ctzll((unsigned long long)q);
      }
    }
    if (i < nproj && h_out[i] > h_max) h_max = h_out[i];
  }
  if (h_max == 0) return kNothingToDo;
  p.y_aligned = 1;
  for (int i = 0; i < nproj; ++i)
    if (!aligned16(y[i])) p.y_aligned = 0;
  p.w = w;
  p.scales = scales;
  p.scales_dtype = scales_dtype;
  p.plan = static_cast<const int*>(plan);
  p.page_elems = page_elems;
  p.batch = (int)batch;
  p.x_cols = (int)x_cols;
  p.qkvo0 = qkvo0;
  // stateless: the rank is only known on the device; the grid covers the pages of a rank
  // up to the delta width (an adapter uses min(rank, ceil(h_out*rank/page_elems)) pages)
  p.blocks = (int)((x_cols + kRB - 1) / kRB);
  p.strided = 0;
  grid = plan != nullptr ? planned_grid(n_items, batch, rank_cap, p.strided) : batch * p.blocks;
  return SLORA_OK;
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
                       (int)max_items);
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
                       (int)max_items, n);
    return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
  }
  int* scratch = static_cast<int*>(plan) + kPlanHeaderWords + max_items * kItemWords;
  hipLaunchKernelGGL(bgmv_plan_kernel, dim3(1), dim3(kPlanThreads), 0, reinterpret_cast<hipStream_t>(stream),
                     static_cast<int*>(plan), t, (int)batch, (int)rank_cap, (int)max_items, scratch);
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
