// Device code and host-side argument checks shared by the decode kernels (bgmv_decode.hip:
// shrink, expand, plan builders) and the one-launch shrink + expand kernel (bgmv_lora.hip).
// Everything here is a template or lives in an unnamed namespace, so each of the two files
// gets its own copy and they compile in parallel.
#pragma once

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
// Behind the records: the one-workgroup builder's scratch (6 words per token), then the
// hand-over counters of the one-launch LoRA (kSyncHeader words, then 4 per token: entry
// [first token of a run][projection], see lora_handover), zeroed by every build.
constexpr int kPlanMagic = 0x534c5033;  // "SLP3"
constexpr int kSyncHeader = 4;          // [0]: set when a hand-over gave up waiting (never expected)
enum { SY_TIMEOUT = 0 };
constexpr int kPlanHeaderWords = 16;
constexpr int kItemWords = 48;
enum { PH_MAGIC = 0, PH_NITEMS = 1, PH_MAXRANK = 2, PH_BATCH = 3, PH_TT = 4, PH_RANKCAP = 5, PH_NRUNS = 6, PH_STATUS = 7 };
// PH_STATUS (0 after a build; read back with slora_plan_status): bit 0 = a launch named another batch size
// or rank cap than the plan was built for and did nothing; bit 1 = a hand-over of the one-launch LoRA gave up
enum { kPlanStatusMismatch = 1, kPlanStatusTimeout = 2 };
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
__device__ __forceinline__ void load_item(const int* __restrict__ plan, int idx, int pp, int jr0, int jr1, int batch,
                                          int rank_cap, Item& it, int& page0, int& page1) {
  // The header and the records do not change while a kernel that reads them runs
  // (the counters behind them do, through another pointer): reading them through
  // the constant address space keeps these loads scalar whatever else the kernel
  // stores.
  typedef const int __attribute__((address_space(4))) * ConstWords;
  ConstWords head = (ConstWords)plan;
  ConstWords rec = head + kPlanHeaderWords + (int64_t)idx * kItemWords;
  int magic = head[PH_MAGIC], n_items = head[PH_NITEMS], plan_batch = head[PH_BATCH], plan_cap = head[PH_RANKCAP];
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
  // a plan of another batch or rank cap lists other tokens and rows: nothing is done, and the plan says so
  const bool mine = (magic == kPlanMagic) & (plan_batch == batch) & (plan_cap == rank_cap);
  if ((magic == kPlanMagic) & !mine & (idx == 0) & (threadIdx.x == 0)) const_cast<int*>(plan)[PH_STATUS] = kPlanStatusMismatch;
  const bool ok = mine & (idx < n_items);
  it.plan_items = mine ? n_items : 0;
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
  int rank_cap;  // of the plan the caller names (planned launches)
  int strided;  // planned launch with fewer workgroups than the plan may have items (see planned_grid)
};

// The common case in straight-line code: the whole page in one pass (hidden <= 512 * NV
// elements), all tokens of the run fit the LDS staging area, no rows beyond the item.
// Every global load is unconditional (absent tokens / rows read a valid dummy address
// and are discarded) so that no branch separates the loads: first the activations, then
// both weight pages; the LDS stores wait for the activations only.
// NV: 16-byte vectors a lane holds of a page (8 = hidden up to 4096).
// COH: the results are read by other workgroups of the same launch (st16_coherent).
template <typename T, int NV, bool COH>
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
          uint16_t* dst = y + (int64_t)it.tok[t] * p.y_cols + row;
          if (COH) st16_coherent(dst, T::from_float(sum)); else *dst = T::from_float(sum);
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
// `it` receives the item (n_tok = 0: nothing was done).
template <typename T, bool PLANNED, int NV, bool COH = false>
__device__ __forceinline__ int shrink_body(const ShrinkArgs& p, int unit, int proj, u32x4* s_x, Item& it) {
  constexpr int NW = 4;
  constexpr int NTASK = 2;
  constexpr int NT = NW * kWave;
  constexpr int kSlab = 512 / NT;  // 16-byte vectors per thread, token and 4096-element slab
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const int* rec = PLANNED ? p.plan + kPlanHeaderWords + (int64_t)unit * kItemWords : nullptr;
  int plan_pg0 = -1, plan_pg1 = -1;
  if (PLANNED) {
    load_item(p.plan, unit, p.qkvo0 + proj, wave, wave + 4, p.batch, p.rank_cap, it, plan_pg0, plan_pg1);
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
    shrink_fast<T, NV, COH>(p, it, proj, r_eff, page2, s_x);
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
              uint16_t* dst = y + (int64_t)item_token(it, t0 + t) * p.y_cols + row[i];
              if (COH) st16_coherent(dst, T::from_float(s)); else *dst = T::from_float(s);
            }
          }
        }
      }
    }
  }
  return it.plan_items;
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
  int rank_cap;  // of the plan the caller names (planned launches)
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

// Sizes of a pass of NV 16-byte vectors per lane (see expand_page).
template <int NV>
struct ExpandPass {
  static constexpr int kElems = NV * kWave * 8;            // elements per pass
  static constexpr int kGroups = (NV + kVecPerPass - 1) / kVecPerPass;  // groups of 8 loads whose sums are filed together
  static constexpr int kStrip = kGroups * kVecPerPass * kWave;          // 16-bit entries of a wavefront's LDS strip
};

// The arithmetic of one pass: for every token of the run, the pass's NV loads times the
// token's delta fragment, reduced over the lanes that share an output, filed in the
// wavefront's LDS strip in output order, added to y (yv: the lane's 8 outputs of the first
// 512 of the pass, already loaded) and stored.  n_pass0: first output of the pass.
template <typename T, int NV>
__device__ __forceinline__ void expand_update(const ExpandArgs& p, int proj, const Item& it, int lg_r,
                                              const u32x4 (&wv)[NV], const u32x4 (&xv)[kTT], const u32x4 (&yv)[kTT],
                                              int n_pass0, int n_end, float scale, uint16_t* s_strip) {
  const int lane = threadIdx.x & 63;
  const int lpo = 1 << (lg_r - 3);
  const int opw = kWave >> (lg_r - 3);  // outputs a wavefront-wide load covers
  const int out_per_pass = ExpandPass<NV>::kElems >> lg_r;
  const int h_stride = p.h_out[proj];
  uint16_t* y = reinterpret_cast<uint16_t*>(p.y[proj]);
  const int n_mine = n_pass0 + lane * 8;
  const bool y_ok = lane * 8 < out_per_pass && n_mine < n_end;
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
// COH: the delta rows were written by other workgroups of the same launch (ldg16_coherent).
template <typename T, bool FULL, int NV, bool COH>
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
    const uint16_t* xp = x + (int64_t)(t < it.n_tok ? it.tok[t] : it.tok[0]) * p.x_cols + (d_ok ? d0 : 0);
    // (FULL: a token the run does not have re-reads the first one's row; its sums are never used)
    if (FULL)
      xv[t] = COH ? ldg16_coherent(xp) : ldg16(xp);
    else
      xv[t] = (t < it.n_tok && d_ok) ? (COH ? ldg16_coherent(xp) : ldg16(xp)) : zero16();
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
    expand_update<T, NV>(p, proj, it, lg_r, wv, xv, yv, n_pass0, n_end, scale, s_strip);
  }
}

// Any rank, any alignment: one lane per output whose first element lies in this
// page, element-wise loads through a_loc (an output's r elements may continue
// on the next page).
template <typename T, bool COH>
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
        const uint16_t* xp = x + (int64_t)bt * p.x_cols + d;
        acc = __builtin_fmaf(wf, T::to_float(COH ? ld16_coherent(xp) : *xp), acc);
      }
      uint16_t* yp = y + (int64_t)bt * h_out + n;
      *yp = T::add(*yp, T::from_float(acc * scale));
    }
  }
}

// Page kk of projection `proj` for the item's run; `page` is its pool page id
// or -2 to look it up in a_loc.
template <typename T, int NV, bool COH>
__device__ __forceinline__ void expand_one(const ExpandArgs& p, int proj, const Item& it, int r_eff, int kk,
                                           int64_t page, bool vec_ok, uint16_t* s_strip) {
  const int64_t base_li = it.base + (int64_t)it.r * (p.qkvo0 + proj);
  if (!vec_ok) {
    expand_scalar<T, COH>(p, proj, it, r_eff, kk, base_li, load_scale(p.scales, p.scales_dtype, it.a));
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
    expand_page<T, true, NV, COH>(p, proj, it, r_eff, wpage, flat0, scale, s_strip);
  else
    expand_page<T, false, NV, COH>(p, proj, it, r_eff, wpage, flat0, scale, s_strip);
}

// Expand has nothing to share between wavefronts (the delta row is 16 bytes per
// lane), so every wavefront takes exactly one page: a workgroup is 4 wavefronts
// = half of one projection's 8-page block of an item, and an item gets
// 2 * NPROJ workgroups.
// Grid: x = item (planned) or token * blocks + block (stateless), y = projection * 2 +
// half: workgroup ids run item-fastest, so with a multiple of 8 items every workgroup of
// an item lands on XCD item % 8.
template <typename T, int NPROJ, bool PLANNED, int NV, bool COH = false>
__device__ __forceinline__ int expand_body(const ExpandArgs& p, int unit, int sub, uint16_t* s_strip) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int proj = sub >> 1;
  const int jr = (sub & 1) * 4 + wave;  // page inside the item's block

  Item it;
  int plan_pg = -1, plan_pg_unused = -1;
  if (PLANNED) {
    load_item(p.plan, unit, p.qkvo0 + proj, jr, jr, p.batch, p.rank_cap, it, plan_pg, plan_pg_unused);
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
    expand_one<T, NV, COH>(p, proj, it, r_eff, k, page, vec_ok, s_strip);
  }
  if (extra) {
#pragma unroll 1
    for (int kk = k + kRB; kk < n_pg; kk += kRB)
      expand_one<T, NV, COH>(p, proj, it, r_eff, kk, -2, vec_ok, s_strip);
  }
  return it.plan_items;
}

// ---------------------------------------------------------------------------
// plan sizes and argument checks (host)
// ---------------------------------------------------------------------------
constexpr int kXcds = 8;
enum { SC_ADAPTER = 0, SC_TOKEN = 1, SC_RANK = 2, SC_ITEMS = 3, SC_WORK = 4, SC_QUEUE = 5, SC_WORDS = 6 };
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
// int32 words of the hand-over counters behind the scratch area, and where they start
int64_t plan_sync_words(int64_t batch) { return kSyncHeader + 4 * batch; }
int64_t plan_sync_offset(int64_t batch, int64_t rank_cap) {
  return kPlanHeaderWords + plan_max_items(batch, rank_cap) * kItemWords + plan_scratch_words(batch);
}
int64_t plan_words(int64_t batch, int64_t rank_cap) {
  return plan_sync_offset(batch, rank_cap) + plan_sync_words(batch);
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
  p.rank_cap = (int)rank_cap;
  p.strided = 0;
  grid = plan != nullptr ? planned_grid(n_items, batch, rank_cap, p.strided) : batch * p.blocks;
  return SLORA_OK;
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
  p.rank_cap = (int)rank_cap;
  p.strided = 0;
  grid = plan != nullptr ? planned_grid(n_items, batch, rank_cap, p.strided) : batch * p.blocks;
  return SLORA_OK;
}

}  // namespace
}  // namespace slora
