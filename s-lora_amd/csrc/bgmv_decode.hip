// Decode-time batched gather matrix-vector products over the paged adapter
// pool: shrink (x[H] -> delta[r]) and expand (delta[r] -> y[H_out] +=).
//
// Both kernels are bandwidth kernels.  One workgroup of 8 wavefronts is
// launched per (token, 64 KiB slice of the token's adapter weights); tokens of
// the same adapter are merged into runs so a slice is fetched once per run.
// Every wavefront owns 8 KiB of weights (one A row / 8 contiguous 1 KiB pieces
// of B^T) and issues all of its 16-byte loads before it waits for any.
//
// Replaces slora/csrc/bgmv/bgmv_impl.cuh:14-241 of the reference.

#include "common.hpp"
#include "cabi_util.hpp"

namespace slora {
namespace {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / kWave;  // 8
constexpr int kTT = 4;                    // most tokens merged into one run
constexpr int kVecPerPass = 8;            // 16-byte vectors a lane holds per pass over a row

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
// shrink
// ---------------------------------------------------------------------------
struct ShrinkArgs {
  void* y[3];
  const void* x;
  const void* w;
  Tables t;
  int64_t page_elems;
  int batch, h_in, y_cols, nproj, qkvo0, rb_per_proj, tt;
};

template <typename T, int TT>
__global__ __launch_bounds__(kThreads) void bgmv_shrink_kernel(const ShrinkArgs p) {
  extern __shared__ u32x4 s_x[];  // [run tokens][h_in / 8]
  __shared__ uint64_t s_masks[kWaves];
  __shared__ int s_members[TT];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  int b, rb;
  map_block(blockIdx.x, (uint32_t)(p.rb_per_proj * p.nproj), b, rb);
  if (b >= p.batch) return;
  const int proj = rb / p.rb_per_proj;
  const int j0 = (rb - proj * p.rb_per_proj) * kWaves;
  const int64_t a = p.t.bins[b];
  if ((uint64_t)a >= (uint64_t)p.t.n_adapters) return;
  const int64_t len = p.t.a_len[a];
  const int r = (int)(len >> 2);
  const int r_eff = r < p.y_cols ? r : p.y_cols;
  if (j0 >= r_eff) return;
  const int n_tok = find_run<kThreads>(p.t.bins, p.batch, b, a, p.tt, s_masks, s_members);
  if (n_tok == 0) return;

  const int nvec = p.h_in >> 3;
  const int j = j0 + wave;
  const u32x4* wrow = nullptr;
  if (j < r_eff) {
    const int64_t page = lookup_page(p.t, p.t.a_start[a] + (int64_t)r * (p.qkvo0 + proj) + j);
    if (page >= 0) wrow = reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.w) + page * p.page_elems);
  }

  // first pass of this wave's row goes in flight before anything waits
  u32x4 wv[kVecPerPass];
#pragma unroll
  for (int i = 0; i < kVecPerPass; ++i) {
    const int v = i * kWave + lane;
    wv[i] = (wrow != nullptr && v < nvec) ? wrow[v] : zero16();
  }

  __syncthreads();  // s_members
  int members[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) members[t] = t < n_tok ? s_members[t] : 0;

  // stage the run's activations: every row is read once per workgroup
  const u32x4* xg = reinterpret_cast<const u32x4*>(p.x);
  for (int t = 0; t < n_tok; ++t) {
    const u32x4* xrow = xg + (int64_t)members[t] * nvec;
    for (int v = tid; v < nvec; v += kThreads) s_x[t * nvec + v] = xrow[v];
  }
  __syncthreads();

  float acc[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) acc[t] = 0.f;

  const int vec_per_pass = kVecPerPass * kWave;
  for (int v0 = 0; v0 < nvec; v0 += vec_per_pass) {
    // next pass in flight while this one is consumed
    u32x4 wn[kVecPerPass];
    const int v1 = v0 + vec_per_pass;
    if (v1 < nvec) {
#pragma unroll
      for (int i = 0; i < kVecPerPass; ++i) {
        const int v = v1 + i * kWave + lane;
        wn[i] = (wrow != nullptr && v < nvec) ? wrow[v] : zero16();
      }
    }
    if (wrow != nullptr) {
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        if (t < n_tok) {
#pragma unroll
          for (int i = 0; i < kVecPerPass; ++i) {
            const int v = v0 + i * kWave + lane;
            if (v < nvec) acc[t] = dot8<T>(wv[i], s_x[t * nvec + v], acc[t]);
          }
        }
      }
    }
    if (v1 < nvec) {
#pragma unroll
      for (int i = 0; i < kVecPerPass; ++i) wv[i] = wn[i];
    }
  }

  uint16_t* y = reinterpret_cast<uint16_t*>(p.y[proj]);
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    if (t < n_tok) {
      const float s = wave_sum(acc[t]);
      if (lane == 0 && wrow != nullptr) y[(int64_t)members[t] * p.y_cols + j] = T::from_float(s);
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
  Tables t;
  const void* scales;
  int64_t page_elems;
  int scales_dtype;
  int batch, x_cols, nproj, qkvo0, tt;
  int h_out[3];
  int blocks[3];  // workgroups per token for each projection
  int blocks_total;
};

constexpr int kChunks = 8;  // 1 KiB pieces of B^T per wavefront

// One run of tokens, adapter rank a multiple of 8.  LPO lanes share one output
// (each holds 8 consecutive rank entries), so a wavefront-wide 16-byte load
// covers OPW = 64 / LPO consecutive outputs = one contiguous piece of B^T.
template <typename T, int TT, int LPO>
__device__ __forceinline__ void expand_body(const ExpandArgs& p, int proj, int n_wg0, int r, int r_eff,
                                            int64_t base_li, float scale, int n_tok, const int* s_members) {
  constexpr int OPW = kWave / LPO;
  constexpr int ROUNDS = (kChunks / LPO) > 0 ? (kChunks / LPO) : 1;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane % LPO, g = lane / LPO;
  const int d0 = li * 8;
  const bool d_ok = d0 < r_eff;
  const int h_out = p.h_out[proj];
  const int n_wave0 = n_wg0 + wave * kChunks * OPW;
  const uint16_t* wbase = reinterpret_cast<const uint16_t*>(p.w);
  const uint32_t page_elems = (uint32_t)p.page_elems;

  u32x4 wv[kChunks];
#pragma unroll
  for (int c = 0; c < kChunks; ++c) {
    const int n = n_wave0 + c * OPW + g;
    wv[c] = zero16();
    if (d_ok && n < h_out) {
      const uint32_t flat = (uint32_t)n * (uint32_t)r + (uint32_t)d0;
      const uint32_t pg = flat / page_elems;
      const uint32_t off = flat - pg * page_elems;
      const int64_t page = lookup_page(p.t, base_li + pg);
      if (page >= 0) wv[c] = ldg16(wbase + page * p.page_elems + off);
    }
  }

  uint16_t* y = reinterpret_cast<uint16_t*>(p.y[proj]);
  const uint16_t* x = reinterpret_cast<const uint16_t*>(p.x[proj]);
  for (int t = 0; t < n_tok; ++t) {
    const int bt = s_members[t];
    float xs[8];
    {
      u32x4 xv = zero16();
      if (d_ok) xv = ldg16(x + (int64_t)bt * p.x_cols + d0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // entries at or beyond r_eff do not take part (lanes are whole vectors
        // because r_eff is a multiple of 8 on this path)
        xs[2 * i] = T::lo(xv[i]) * scale;
        xs[2 * i + 1] = T::hi(xv[i]) * scale;
      }
    }
    float res[ROUNDS];
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) res[rd] = 0.f;
#pragma unroll
    for (int c = 0; c < kChunks; ++c) {
      float s = dot8f<T>(wv[c], xs, 0.f);
      s = group_sum<LPO>(s);
      // after LPO chunks every lane of the wavefront holds exactly one output
      if (li == (c % LPO)) res[c / LPO < ROUNDS ? c / LPO : 0] = s;
    }
    uint16_t* yrow = y + (int64_t)bt * h_out;
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int c = rd * LPO + li;
      const int n = n_wave0 + c * OPW + g;
      if (c < kChunks && n < h_out) yrow[n] = T::add(yrow[n], T::from_float(res[rd]));
    }
  }
}

// Any rank, any alignment: one lane per output, element-wise loads.
template <typename T>
__device__ __forceinline__ void expand_scalar(const ExpandArgs& p, int proj, int n_wg0, int span, int r,
                                              int r_eff, int64_t base_li, float scale, int n_tok,
                                              const int* s_members) {
  const int h_out = p.h_out[proj];
  const int n_end = n_wg0 + span < h_out ? n_wg0 + span : h_out;
  const uint16_t* wbase = reinterpret_cast<const uint16_t*>(p.w);
  uint16_t* y = reinterpret_cast<uint16_t*>(p.y[proj]);
  const uint16_t* x = reinterpret_cast<const uint16_t*>(p.x[proj]);
  const uint32_t page_elems = (uint32_t)p.page_elems;
  for (int n = n_wg0 + (int)threadIdx.x; n < n_end; n += kThreads) {
    for (int t = 0; t < n_tok; ++t) {
      const int bt = s_members[t];
      float acc = 0.f;
      for (int d = 0; d < r_eff; ++d) {
        const uint32_t flat = (uint32_t)n * (uint32_t)r + (uint32_t)d;
        const uint32_t pg = flat / page_elems;
        const uint32_t off = flat - pg * page_elems;
        const int64_t page = lookup_page(p.t, base_li + pg);
        if (page < 0) continue;
        const float wf = T::to_float(wbase[page * p.page_elems + off]);
        acc = __builtin_fmaf(wf, T::to_float(x[(int64_t)bt * p.x_cols + d]) * scale, acc);
      }
      uint16_t* yp = y + (int64_t)bt * h_out + n;
      *yp = T::add(*yp, T::from_float(acc));
    }
  }
}

template <typename T, int TT>
__global__ __launch_bounds__(kThreads) void bgmv_expand_kernel(const ExpandArgs p) {
  __shared__ uint64_t s_masks[kWaves];
  __shared__ int s_members[TT];

  int b, blk;
  map_block(blockIdx.x, (uint32_t)p.blocks_total, b, blk);
  if (b >= p.batch) return;
  int proj = 0;
  if (blk >= p.blocks[0]) {
    blk -= p.blocks[0];
    proj = 1;
    if (blk >= p.blocks[1]) {
      blk -= p.blocks[1];
      proj = 2;
    }
  }
  const int64_t a = p.t.bins[b];
  if ((uint64_t)a >= (uint64_t)p.t.n_adapters) return;
  const int r = (int)(p.t.a_len[a] >> 2);
  const int r_eff = r < p.x_cols ? r : p.x_cols;
  if (r_eff <= 0) return;
  const int nv = (r_eff + 7) >> 3;
  int lpo = 1;
  while (lpo < nv) lpo <<= 1;
  const int span = kWaves * kChunks * (kWave / lpo);  // outputs per workgroup at this rank
  const int n_wg0 = blk * span;
  if (n_wg0 >= p.h_out[proj]) return;
  const int n_tok = find_run<kThreads>(p.t.bins, p.batch, b, a, p.tt, s_masks, s_members);
  if (n_tok == 0) return;
  __syncthreads();

  const int64_t base_li = p.t.a_start[a] + (int64_t)r * (p.qkvo0 + proj);
  const float scale = load_scale(p.scales, p.scales_dtype, a);
  const bool vec_ok = (r & 7) == 0 && (r_eff & 7) == 0 && (p.x_cols & 7) == 0;
  if (!vec_ok) {
    expand_scalar<T>(p, proj, n_wg0, span, r, r_eff, base_li, scale, n_tok, s_members);
    return;
  }
  switch (lpo) {
    case 1: expand_body<T, TT, 1>(p, proj, n_wg0, r, r_eff, base_li, scale, n_tok, s_members); break;
    case 2: expand_body<T, TT, 2>(p, proj, n_wg0, r, r_eff, base_li, scale, n_tok, s_members); break;
    case 4: expand_body<T, TT, 4>(p, proj, n_wg0, r, r_eff, base_li, scale, n_tok, s_members); break;
    case 8: expand_body<T, TT, 8>(p, proj, n_wg0, r, r_eff, base_li, scale, n_tok, s_members); break;
    case 16: expand_body<T, TT, 16>(p, proj, n_wg0, r, r_eff, base_li, scale, n_tok, s_members); break;
    case 32: expand_body<T, TT, 32>(p, proj, n_wg0, r, r_eff, base_li, scale, n_tok, s_members); break;
    default: expand_body<T, TT, 64>(p, proj, n_wg0, r, r_eff, base_li, scale, n_tok, s_members); break;
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
int fill_tables(Tables& t, const slora_tables* in, const int64_t* bins, int64_t n_pages) {
  if (in == nullptr || in->a_start == nullptr || in->a_len == nullptr || in->a_loc == nullptr || bins == nullptr)
    return SLORA_ERR_NULL_POINTER;
  if (in->n_adapters < 0 || in->n_loc < 0 || n_pages < 0) return SLORA_ERR_BAD_SHAPE;
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

template <typename T>
int launch_shrink(const ShrinkArgs& a, hipStream_t stream) {
  ShrinkArgs p = a;
  // as many tokens per run as fit the LDS budget
  const size_t row_bytes = (size_t)p.h_in * 2;
  int tt = kTT;
  while (tt > 1 && tt * row_bytes > kLdsSoftLimit) --tt;
  const size_t lds = tt * row_bytes;
  if (lds > kLdsHardLimit) return SLORA_ERR_UNSUPPORTED;
  p.tt = tt;
  auto kernel = bgmv_shrink_kernel<T, kTT>;
  if (lds > kLdsSoftLimit) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess) {
      (void)hipGetLastError();
      return SLORA_ERR_LAUNCH;
    }
  }
  const int64_t groups = (p.batch + 7) / 8;
  const int64_t grid = groups * 8 * p.rb_per_proj * p.nproj;
  if (grid <= 0) return SLORA_OK;
  if (grid > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kernel, dim3((uint32_t)grid), dim3(kThreads), lds, stream, p);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

template <typename T>
int launch_expand(const ExpandArgs& a, hipStream_t stream) {
  ExpandArgs p = a;
  p.tt = kTT;
  const int nv_max = (p.x_cols + 7) / 8;
  int lpo_max = 1;
  while (lpo_max < nv_max) lpo_max <<= 1;
  const int span_min = kWaves * kChunks * (kWave / lpo_max);
  p.blocks_total = 0;
  for (int i = 0; i < 3; ++i) {
    p.blocks[i] = i < p.nproj ? (p.h_out[i] + span_min - 1) / span_min : 0;
    p.blocks_total += p.blocks[i];
  }
  const int64_t groups = (p.batch + 7) / 8;
  const int64_t grid = groups * 8 * p.blocks_total;
  if (grid <= 0) return SLORA_OK;
  if (grid > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
  hipLaunchKernelGGL((bgmv_expand_kernel<T, kTT>), dim3((uint32_t)grid), dim3(kThreads), 0, stream, p);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

int shrink_common(void* const y[3], int nproj, int qkvo0, const void* x, const void* w, const slora_tables* tables,
                  const int64_t* bins, int64_t batch, int64_t h_in, int64_t y_cols, int64_t page_elems,
                  int64_t n_pages, int dtype, void* stream) {
  if (dtype != SLORA_DTYPE_F16 && dtype != SLORA_DTYPE_BF16) return SLORA_ERR_BAD_DTYPE;
  if (batch < 0 || h_in < 0 || y_cols < 0 || page_elems < 0) return SLORA_ERR_BAD_SHAPE;
  if (qkvo0 < 0 || qkvo0 + nproj > 4) return SLORA_ERR_BAD_SHAPE;
  if (batch == 0 || y_cols == 0) return SLORA_OK;
  ShrinkArgs p{};
  int rc = fill_tables(p.t, tables, bins, n_pages);
  if (rc != SLORA_OK) return rc;
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
  p.page_elems = page_elems;
  p.batch = (int)batch;
  p.h_in = (int)h_in;
  p.y_cols = (int)y_cols;
  p.nproj = nproj;
  p.qkvo0 = qkvo0;
  p.rb_per_proj = (int)((y_cols + kWaves - 1) / kWaves);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  return dtype == SLORA_DTYPE_F16 ? launch_shrink<F16>(p, s) : launch_shrink<BF16>(p, s);
}

int expand_common(void* const y[3], const void* const x[3], const int64_t h_out[3], int nproj, int qkvo0,
                  const void* w, const slora_tables* tables, const int64_t* bins, const void* scales,
                  int scales_dtype, int64_t batch, int64_t x_cols, int64_t page_elems, int64_t n_pages, int dtype,
                  void* stream) {
  if (dtype != SLORA_DTYPE_F16 && dtype != SLORA_DTYPE_BF16) return SLORA_ERR_BAD_DTYPE;
  if (scales_dtype != SLORA_DTYPE_F16 && scales_dtype != SLORA_DTYPE_BF16 && scales_dtype != SLORA_DTYPE_F32)
    return SLORA_ERR_BAD_DTYPE;
  if (batch < 0 || x_cols < 0 || page_elems < 0) return SLORA_ERR_BAD_SHAPE;
  for (int i = 0; i < nproj; ++i)
    if (h_out[i] < 0) return SLORA_ERR_BAD_SHAPE;
  if (qkvo0 < 0 || qkvo0 + nproj > 4) return SLORA_ERR_BAD_SHAPE;
  if (batch == 0 || x_cols == 0) return SLORA_OK;
  ExpandArgs p{};
  int rc = fill_tables(p.t, tables, bins, n_pages);
  if (rc != SLORA_OK) return rc;
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
  for (int i = 0; i < 3; ++i) {
    p.y[i] = i < nproj ? y[i] : nullptr;
    p.x[i] = i < nproj ? x[i] : nullptr;
    p.h_out[i] = i < nproj ? (int)h_out[i] : 0;
  }
  p.w = w;
  p.scales = scales;
  p.scales_dtype = scales_dtype;
  p.page_elems = page_elems;
  p.batch = (int)batch;
  p.x_cols = (int)x_cols;
  p.nproj = nproj;
  p.qkvo0 = qkvo0;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  return dtype == SLORA_DTYPE_F16 ? launch_expand<F16>(p, s) : launch_expand<BF16>(p, s);
}

}  // namespace
}  // namespace slora

extern "C" {

int slora_bgmv_shrink(void* y, const void* x, const void* w, const slora_tables* tables, const int64_t* bins,
                      int64_t batch, int64_t h_in, int64_t y_cols, int64_t page_elems, int64_t n_pages, int qkvo,
                      int dtype, void* stream) {
  void* ys[3] = {y, nullptr, nullptr};
  if (qkvo < 0 || qkvo > 3) return SLORA_ERR_BAD_SHAPE;
  return slora::shrink_common(ys, 1, qkvo, x, w, tables, bins, batch, h_in, y_cols, page_elems, n_pages, dtype,
                              stream);
}

int slora_bgmv_shrink_qkv(void* y_q, void* y_k, void* y_v, const void* x, const void* w,
                          const slora_tables* tables, const int64_t* bins, int64_t batch, int64_t h_in,
                          int64_t y_cols, int64_t page_elems, int64_t n_pages, int dtype, void* stream) {
  void* ys[3] = {y_q, y_k, y_v};
  return slora::shrink_common(ys, 3, 0, x, w, tables, bins, batch, h_in, y_cols, page_elems, n_pages, dtype, stream);
}

int slora_bgmv_expand(void* y, const void* x, const void* w, const slora_tables* tables, const int64_t* bins,
                      const void* scales, int scales_dtype, int64_t batch, int64_t x_cols, int64_t h_out,
                      int64_t page_elems, int64_t n_pages, int qkvo, int dtype, void* stream) {
  void* ys[3] = {y, nullptr, nullptr};
  const void* xs[3] = {x, nullptr, nullptr};
  const int64_t hs[3] = {h_out, 0, 0};
  if (qkvo < 0 || qkvo > 3) return SLORA_ERR_BAD_SHAPE;
  return slora::expand_common(ys, xs, hs, 1, qkvo, w, tables, bins, scales, scales_dtype, batch, x_cols, page_elems,
                              n_pages, dtype, stream);
}

int slora_bgmv_expand_qkv(void* y_q, void* y_k, void* y_v, const void* x_q, const void* x_k, const void* x_v,
                          const void* w, const slora_tables* tables, const int64_t* bins, const void* scales,
                          int scales_dtype, int64_t batch, int64_t x_cols, int64_t h_out_q, int64_t h_out_k,
                          int64_t h_out_v, int64_t page_elems, int64_t n_pages, int dtype, void* stream) {
  void* ys[3] = {y_q, y_k, y_v};
  const void* xs[3] = {x_q, x_k, x_v};
  const int64_t hs[3] = {h_out_q, h_out_k, h_out_v};
  return slora::expand_common(ys, xs, hs, 3, 0, w, tables, bins, scales, scales_dtype, batch, x_cols, page_elems,
                              n_pages, dtype, stream);
}

}  // extern "C"
