// Prefill-time segmented gather-GEMM over the paged adapter pool.
//
// A request owns a run of consecutive token rows and one adapter.  Shrink is
// [tokens x H] . [H x r] with the r weight rows gathered page by page; expand
// is [tokens x r] . [r x H_out] accumulated into the output, with B^T laid end
// to end over the adapter's pages.  Both contractions run on the matrix cores
// (v_mfma_f32_16x16x32 f16/bf16, float accumulate); both operands are
// K-contiguous in memory, so MFMA fragments are plain 16-byte global loads.
//
// Replaces slora/models/peft/triton_kernel/lora/lora_prefill.py:10-164 of the
// reference.

#include <type_traits>

#include "common.hpp"
#include "cabi_util.hpp"

namespace slora {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

template <typename T>
__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c);
template <>
__device__ __forceinline__ f32x4 mfma16<F16>(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4 mfma16<BF16>(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0,
                                                 0);
}

struct SegTables {
  const int64_t* a_start;
  const int64_t* a_len;
  const int64_t* a_loc;
  const int32_t* b_start_loc;
  const int32_t* b_seq_len;
  const int64_t* b_indicies;
  int64_t n_adapters, n_loc, n_pages;
  int n_requests, n_tokens;
};

__device__ __forceinline__ int64_t seg_page(const SegTables& t, int64_t li) {
  if ((uint64_t)li >= (uint64_t)t.n_loc) return -1;
  const int64_t page = t.a_loc[li];
  return (uint64_t)page < (uint64_t)t.n_pages ? page : -1;
}

__device__ __forceinline__ bool aligned16_dev(const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; }

// a_loc entry `li` -> page id with the load outside any branch: an unwanted or
// out-of-range index reads a_start[0] instead (there is at least one adapter
// whenever a request reaches this point) and is rejected afterwards.  Callers
// issue several of these back to back so the loads overlap.
__device__ __forceinline__ int64_t seg_page_nobranch(const SegTables& t, int64_t li, bool want) {
  const bool in = want & ((uint64_t)li < (uint64_t)t.n_loc);
  const int64_t page = *(in ? t.a_loc + li : t.a_start);
  return (in & ((uint64_t)page < (uint64_t)t.n_pages)) ? page : (int64_t)-1;
}

// Request `req`: its adapter, rank, first row and row count clipped to the
// buffers.  False if the request has nothing to do.
__device__ __forceinline__ bool seg_lookup(const SegTables& t, int req, int64_t& a, int& r, int& row0, int& rows) {
  a = t.b_indicies[req];
  if ((uint64_t)a >= (uint64_t)t.n_adapters) return false;
  r = (int)(t.a_len[a] >> 2);
  row0 = t.b_start_loc[req];
  rows = t.b_seq_len[req];
  if (row0 < 0 || rows <= 0) return false;
  if (row0 >= t.n_tokens) return false;
  if (rows > t.n_tokens - row0) rows = t.n_tokens - row0;
  return true;
}

// ---------------------------------------------------------------------------
// shrink
// ---------------------------------------------------------------------------
struct SegShrinkArgs {
  void* o[3];  // one output per projection of the launch (q, k, v when nproj = 3)
  const void* x;
  const void* w;
  SegTables t;
  int64_t x_stride, w_stride, o_stride;  // elements per row
  int h_in, max_rank, qkvo, m_tiles;
  int nproj;  // 1: projection qkvo; 3: q, k and v in one pass over x (qkvo = 0)
  int col_split;  // 1, 2 or 4 workgroups share a tile's rank columns (16-column tiles t with t % col_split == group)
  int vec_ok;  // every row start is 16-byte aligned and h_in % 8 == 0
};

constexpr int kShrThreads = 256;
constexpr int kShrWaves = kShrThreads / kWave;  // K is split over the 4 wavefronts (one per SIMD: 512 registers each)
constexpr int kShrMF = 4;                       // 16-row A fragments per tile
constexpr int kShrTM = 16 * kShrMF;             // token rows per tile
constexpr int kShrNB = 64;                      // rank columns per pass
constexpr int kShrLd = kShrNB + 4;              // LDS row pitch (floats) -> conflict-free C-tile stores

// Element-wise fallback for layouts the vector path cannot read.
template <typename T>
__device__ void shrink_generic(const SegShrinkArgs& p, int pj, int r_eff, int64_t base_li, int row0, int m0, int m_cnt) {
  const uint16_t* x = reinterpret_cast<const uint16_t*>(p.x);
  const uint16_t* w = reinterpret_cast<const uint16_t*>(p.w);
  uint16_t* o = reinterpret_cast<uint16_t*>(p.o[pj]);
  for (int idx = threadIdx.x; idx < m_cnt * p.max_rank; idx += kShrThreads) {
    const int m = idx / p.max_rank, j = idx - m * p.max_rank;
    const int64_t row = row0 + m0 + m;
    float acc = 0.f;
    if (j < r_eff) {
      const int64_t page = seg_page(p.t, base_li + j);
      if (page >= 0) {
        const uint16_t* wr = w + page * p.w_stride;
        const uint16_t* xr = x + row * p.x_stride;
        for (int k = 0; k < p.h_in; ++k) acc = __builtin_fmaf(T::to_float(xr[k]), T::to_float(wr[k]), acc);
      }
    }
    o[row * p.o_stride + j] = T::from_float(acc);
  }
}

// Two lane orders of a 16-row x 64-k block (two MFMA K steps, one 128-byte line per row).
// MFMA order: register s (K step s) of lane (lr, lg) holds row lr, 16-byte piece 4*s + lg.
// Line order: register g holds row 8*g + lr%8, piece lg + 4*(lr/8) -- one load instruction
// covers 8 whole lines instead of 16 half lines, which the vector cache serves about 1.4x
// faster.  Both orders keep a value inside its 16-lane row, at most 8 lanes away: one DPP
// move per register converts between them, and the conversion is its own inverse.
__device__ __forceinline__ void swap_halves(u32x4& a, u32x4& b) {
  constexpr int kRowRor8 = 0x128;  // rotate by 8 inside each row of 16 lanes
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int va = (int)a[q], vb = (int)b[q];
    // a keeps its lanes 0..7 of every 16 and takes b's lanes 0..7 into 8..15;
    // b takes a's lanes 8..15 into 0..7 and keeps its lanes 8..15
    a[q] = (uint32_t)__builtin_amdgcn_update_dpp(va, vb, kRowRor8, 0xF, 0xC, false);
    b[q] = (uint32_t)__builtin_amdgcn_update_dpp(vb, va, kRowRor8, 0xF, 0x3, false);
  }
}

// One wavefront's share of the K loop of a (16 * MF)-token x (16 * NT)-rank tile: the
// 64-k blocks wave, wave + kShrWaves, ...  A block's fragments are loaded in line order
// (xline / wline: the rows of the lane's two loads per fragment) and converted when
// they are multiplied; the loads of one block are in flight while the previous one
// is multiplied.  No load sits inside a branch (the wait counters then stay
// exact): the main loop only runs where all of its blocks exist, and the tail
// re-reads the last block where one does not.
template <typename T, int NT, int MF>
__device__ __forceinline__ void shrink_k_loop(const uint16_t* const (&xline)[kShrMF][2],
                                              const uint16_t* const (&wline)[4][2], int wave, int piece, int h_in,
                                              f32x4 (&acc)[kShrMF][4]) {
  const int blocks = (h_in + 63) >> 6;
  const int n = (blocks - wave + kShrWaves - 1) / kShrWaves;  // blocks of this wavefront
  if (n <= 0) return;
  const bool ragged_k = (h_in & 63) != 0;
  struct Block {
    u32x4 a[MF][2], b[NT][2];
  };
  auto load_block = [&](int i, Block& blk) {
    if (i >= n) i = n - 1;
    int k = (i * kShrWaves + wave) * 64 + piece * 8;
    const bool k_in = k < h_in;
    if (!k_in) k = 0;
#pragma unroll
    for (int f = 0; f < MF; ++f)
#pragma unroll
      for (int g = 0; g < 2; ++g) blk.a[f][g] = ldg16_stream(xline[f][g] + k);
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int g = 0; g < 2; ++g) blk.b[t][g] = ldg16(wline[t][g] + k);
    if (ragged_k && !k_in) {
#pragma unroll
      for (int f = 0; f < MF; ++f) blk.a[f][0] = blk.a[f][1] = zero16();
#pragma unroll
      for (int t = 0; t < NT; ++t) blk.b[t][0] = blk.b[t][1] = zero16();
    }
  };
  auto mul_block = [&](Block& blk) {
#pragma unroll
    for (int f = 0; f < MF; ++f) swap_halves(blk.a[f][0], blk.a[f][1]);
#pragma unroll
    for (int t = 0; t < NT; ++t) swap_halves(blk.b[t][0], blk.b[t][1]);
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int f = 0; f < MF; ++f) acc[f][t] = mfma16<T>(blk.a[f][s], blk.b[t][s], acc[f][t]);
  };
  Block c0, c1;
  load_block(0, c0);
  int i = 0;
  for (; i + 2 < n; i += 2) {
    load_block(i + 1, c1);
    mul_block(c0);
    load_block(i + 2, c0);
    mul_block(c1);
  }
  // one or two blocks are left; block i is loaded
  load_block(i + 1, c1);
  mul_block(c0);
  if (i + 1 < n) mul_block(c1);
}

// The same loop with a ring of D blocks, D - 1 of them in flight while one is multiplied
// (same blocks in the same order: identical sums).  For launches with few workgroups, where
// a wavefront waits for its own loads and nobody else's fill the compute unit: 1024 tokens
// of rank 64 take 16 -> 14.5 us, 4096 tokens 25 -> 23.5 us with D = 4.  With every compute
// unit streaming (C3) the deeper ring is slower (37 -> 44 us): a wavefront's loads return in
// order, so the weight rows (cache hits) queue behind the activations of the blocks ahead.
// A load past the last block re-reads it; only multiplications are skipped.
template <typename T, int NT, int MF, int D>
__device__ __forceinline__ void shrink_k_loop_ring(const uint16_t* const (&xline)[kShrMF][2],
                                                   const uint16_t* const (&wline)[4][2], int wave, int piece,
                                                   int h_in, f32x4 (&acc)[kShrMF][4]) {
  const int blocks = (h_in + 63) >> 6;
  const int n = (blocks - wave + kShrWaves - 1) / kShrWaves;  // blocks of this wavefront
  if (n <= 0) return;
  const bool ragged_k = (h_in & 63) != 0;
  struct Block {
    u32x4 a[MF][2], b[NT][2];
  };
  auto load_block = [&](int i, Block& blk) {
    if (i >= n) i = n - 1;
    int k = (i * kShrWaves + wave) * 64 + piece * 8;
    const bool k_in = k < h_in;
    if (!k_in) k = 0;
#pragma unroll
    for (int f = 0; f < MF; ++f)
#pragma unroll
      for (int g = 0; g < 2; ++g) blk.a[f][g] = ldg16_stream(xline[f][g] + k);
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int g = 0; g < 2; ++g) blk.b[t][g] = ldg16(wline[t][g] + k);
    if (ragged_k && !k_in) {
#pragma unroll
      for (int f = 0; f < MF; ++f) blk.a[f][0] = blk.a[f][1] = zero16();
#pragma unroll
      for (int t = 0; t < NT; ++t) blk.b[t][0] = blk.b[t][1] = zero16();
    }
  };
  auto mul_block = [&](Block& blk) {
#pragma unroll
    for (int f = 0; f < MF; ++f) swap_halves(blk.a[f][0], blk.a[f][1]);
#pragma unroll
    for (int t = 0; t < NT; ++t) swap_halves(blk.b[t][0], blk.b[t][1]);
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int f = 0; f < MF; ++f) acc[f][t] = mfma16<T>(blk.a[f][s], blk.b[t][s], acc[f][t]);
  };
  Block ring[D];
#pragma unroll
  for (int d = 0; d < D - 1; ++d) load_block(d, ring[d]);
  for (int i = 0; i < n; i += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      load_block(i + d + D - 1, ring[(d + D - 1) % D]);
      if (i + d < n) mul_block(ring[d]);
    }
  }
}

// The same share of the K loop for q, k and v at once: a 64-k block of the activations is
// loaded once and multiplied with the block of each projection's weight rows in turn.  Two
// activation blocks and two weight blocks are held; while one product runs, the weight block
// it does not use is refilled with what is needed two products later (q, k, v of block i,
// then q, k, v of block i + 1, ...), so every load has one product's time to arrive.  As in
// shrink_k_loop no load sits inside a branch; loads past the last block re-read it.
template <typename T, int NT, int MF>
__device__ __forceinline__ void shrink_k_loop_qkv(const uint16_t* const (&xline)[kShrMF][2],
                                                  const uint16_t* const (&wline)[3][4][2], int wave, int piece,
                                                  int h_in, f32x4 (&acc)[3][kShrMF][4]) {
  const int blocks = (h_in + 63) >> 6;
  const int n = (blocks - wave + kShrWaves - 1) / kShrWaves;  // blocks of this wavefront
  if (n <= 0) return;
  const bool ragged_k = (h_in & 63) != 0;
  struct ABlock {
    u32x4 a[MF][2];
  };
  struct BBlock {
    u32x4 b[NT][2];
  };
  auto k_of = [&](int i, bool& k_in) {
    if (i >= n) i = n - 1;
    int k = (i * kShrWaves + wave) * 64 + piece * 8;
    k_in = k < h_in;
    return k_in ? k : 0;
  };
  auto load_a = [&](int i, ABlock& blk) {
    bool k_in;
    const int k = k_of(i, k_in);
#pragma unroll
    for (int f = 0; f < MF; ++f)
#pragma unroll
      for (int g = 0; g < 2; ++g) blk.a[f][g] = ldg16_stream(xline[f][g] + k);
    if (ragged_k && !k_in) {
#pragma unroll
      for (int f = 0; f < MF; ++f) blk.a[f][0] = blk.a[f][1] = zero16();
    }
  };
  auto load_b = [&](int i, int pj, BBlock& blk) {
    bool k_in;
    const int k = k_of(i, k_in);
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int g = 0; g < 2; ++g) blk.b[t][g] = ldg16(wline[pj][t][g] + k);
    if (ragged_k && !k_in) {
#pragma unroll
      for (int t = 0; t < NT; ++t) blk.b[t][0] = blk.b[t][1] = zero16();
    }
  };
  auto to_mfma_order = [&](ABlock& blk) {
#pragma unroll
    for (int f = 0; f < MF; ++f) swap_halves(blk.a[f][0], blk.a[f][1]);
  };
  auto mul = [&](const ABlock& a, BBlock& b, f32x4 (&c)[kShrMF][4]) {
#pragma unroll
    for (int t = 0; t < NT; ++t) swap_halves(b.b[t][0], b.b[t][1]);
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int f = 0; f < MF; ++f) c[f][t] = mfma16<T>(a.a[f][s], b.b[t][s], c[f][t]);
  };
  ABlock a0, a1;
  BBlock bx, by;
  load_a(0, a0);
  load_b(0, 0, bx);
  load_b(0, 1, by);
  int i = 0;
  // block i: activations in a0, q in bx, k in by
  for (; i + 2 < n; i += 2) {
    load_a(i + 1, a1);
    to_mfma_order(a0);
    mul(a0, bx, acc[0]);
    load_b(i, 2, bx);
    mul(a0, by, acc[1]);
    load_b(i + 1, 0, by);
    mul(a0, bx, acc[2]);
    load_b(i + 1, 1, bx);
    // block i + 1: activations in a1, q in by, k in bx
    load_a(i + 2, a0);
    to_mfma_order(a1);
    mul(a1, by, acc[0]);
    load_b(i + 1, 2, by);
    mul(a1, bx, acc[1]);
    load_b(i + 2, 0, bx);
    mul(a1, by, acc[2]);
    load_b(i + 2, 1, by);
  }
  // one or two blocks are left; block i is loaded as at the top of the loop
  load_a(i + 1, a1);
  to_mfma_order(a0);
  mul(a0, bx, acc[0]);
  load_b(i, 2, bx);
  mul(a0, by, acc[1]);
  load_b(i + 1, 0, by);
  mul(a0, bx, acc[2]);
  load_b(i + 1, 1, bx);
  const bool second = i + 1 < n;
  if (second) {
    to_mfma_order(a1);
    mul(a1, by, acc[0]);
  }
  load_b(i + 1, 2, by);
  if (second) {
    mul(a1, bx, acc[1]);
    mul(a1, by, acc[2]);
  }
}

// ---------------------------------------------------------------------------
// K loop fed through LDS (large batches)
// ---------------------------------------------------------------------------
// With every compute unit streaming, what a register-fed loop can keep in flight (64 KB per
// compute unit at 324 registers per lane) is what bounds it.  Here the 64-k blocks of a tile --
// 64 token rows of x and the 16-row units of weight rows of every projection -- travel from
// memory straight into a ring of LDS stages (global_load_lds_dwordx4: no registers held while a
// load is in flight), up to 128 KB per compute unit, and the MFMA fragments are read from
// there.  The four wavefronts split the tile's OUTPUT (two row fragments x half of the units
// each) instead of K, so every output is one chain of products over all of K and nothing is
// summed across wavefronts.
//
// A wave-wide load fills one 1 KiB chunk of a stage: 8 rows x 128 bytes, lane i at slot i.
// Which 16-byte piece of its row a lane fetches is its slot's column xor the row (within the
// chunk), so that the later fragment reads -- 16 rows at one piece index -- fall on 8 different
// 16-byte columns: no bank conflicts on either side (SQ_LDS_BANK_CONFLICT reads 0).
constexpr int kShrRingBytes = 128 * 1024;

template <int U>  // 16-row units of weight rows per block: projections x 16-column tiles of the rank
struct ShrRing {
  static constexpr int kLoads = 8 + 2 * U;        // chunks per stage: 8 of x, 2 per unit
  static constexpr int kLpw = (kLoads + 3) / 4;   // loads a wavefront issues per stage
  static constexpr int kStage = kLoads * 1024;    // bytes
  static constexpr int kStages = kShrRingBytes / kStage < 8 ? kShrRingBytes / kStage : 8;
  static constexpr int kUpw = (U + 1) / 2;        // units per wavefront column
};

// s_waitcnt for "at most n vector memory operations of this wavefront outstanding" (gfx9 encoding)
template <int N>
__device__ __forceinline__ void wait_vm() {
  static_assert(N >= 0 && N < 64, "vmcnt is six bits");
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x0F70);
}

// The compiler may not move LDS accesses across these: the barrier builtin alone says nothing
// about memory, and __syncthreads() would wait for every outstanding load (the ring's included).
__device__ __forceinline__ void ring_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
// LDS writes of this wavefront done (lgkmcnt(0), nothing else), then the barrier
__device__ __forceinline__ void lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

constexpr int kShrOutPitch = kShrNB + 8;  // 16-bit entries per row of the output staging tile (rows stay 16-byte aligned)
constexpr int kShrOutBytes = kShrTM * kShrOutPitch * 2;

// One pass (64 rank columns from nb0) over ALL tiles of a part -- rows row_first .. + m_rows of one
// request -- as one stream of 64-k blocks: the loads run kStages - 1 blocks ahead of the products
// across tile boundaries, so the ring never drains between the tiles of a part.  A tile's sums go
// through a staging tile in LDS (s_out, behind the ring) and leave as whole 16-byte pieces, the
// columns behind the adapter's rank (up to max_rank) as zeros.
template <typename T, int NPROJ, int NT>
__device__ __forceinline__ void shrink_part_lds_pass(const SegShrinkArgs& p, unsigned char* ring, uint16_t* s_out,
                                                     int64_t row_first, int m_rows, int r_eff, int64_t base_li,
                                                     int rank, int nb0, int nb_cnt) {
  constexpr int U = NPROJ * NT;
  using R = ShrRing<U>;
  constexpr int NU = R::kUpw;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;
  const uint16_t* xg = reinterpret_cast<const uint16_t*>(p.x);
  const uint16_t* wg = reinterpret_cast<const uint16_t*>(p.w);

  // ---- what this lane fetches: the chunks wave, wave + 4, ... of every stage (a chunk past the
  // last one repeats it: same data to the same place).  Chunks 0..7 are x (loads q = 0, 1 of every
  // wavefront), the others weight rows, whose addresses do not change over the part.
  const int crow = lane >> 3, piece = (lane & 7) ^ crow;
  const uint16_t* src_w[R::kLpw];  // entries 0, 1 unused
  int chunk[R::kLpw];
  {
    int64_t pg[R::kLpw];
#pragma unroll
    for (int q = 0; q < R::kLpw; ++q) {
      int l = wave + 4 * q;
      if (l >= R::kLoads) l = R::kLoads - 1;
      chunk[q] = l;
      const int a = l - 8, u = a >> 1, pj = u / NT, t = u - pj * NT;
      const int j = nb0 + t * 16 + (a & 1) * 8 + crow;  // rank row (weight chunks)
      pg[q] = seg_page_nobranch(p.t, base_li + (int64_t)pj * rank + j, q >= 2 && j < r_eff && p.t.n_loc > 0);
    }
#pragma unroll
    for (int q = 0; q < R::kLpw; ++q)  // a row that does not exist reads pool page 0: its products only reach columns that are zeroed
      src_w[q] = wg + (pg[q] >= 0 ? pg[q] : 0) * p.w_stride + piece * 8;
  }
  typedef __attribute__((address_space(3))) unsigned char* LdsBytes;
  typedef const __attribute__((address_space(1))) void* GlobalPtr;
  LdsBytes lds = (LdsBytes)ring;
  const int nblk = p.h_in >> 6;
  const int n_mt = (m_rows + kShrTM - 1) / kShrTM;

  // the block the next load fetches: (i_tile, i_blk); its x rows (rows past the end of the part
  // repeat the last one: their results are not stored)
  int i_tile = 0, i_blk = 0;
  const uint16_t* src_x[2];
  auto x_rows_of = [&](int tile) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      int m = tile * kShrTM + chunk[q] * 8 + crow;
      if (m >= m_rows) m = m_rows - 1;
      src_x[q] = xg + (row_first + m) * p.x_stride + piece * 8;
    }
  };
  x_rows_of(0);
  auto issue = [&](int stage) {
#pragma unroll
    for (int q = 0; q < R::kLpw; ++q) {
      // the LDS address of a chunk is the same in every lane (it travels in M0)
      const int off = __builtin_amdgcn_readfirstlane(stage * R::kStage + chunk[q] * 1024);
      const uint16_t* src = (q < 2 ? src_x[q] : src_w[q]) + (int64_t)i_blk * 64;
      if (q < 2)  // x is read once: nontemporal, so that it does not push the weight rows out of L2
        __builtin_amdgcn_global_load_lds((GlobalPtr)src, (__attribute__((address_space(3))) void*)(lds + off), 16, 0, 2);
      else
        __builtin_amdgcn_global_load_lds((GlobalPtr)src, (__attribute__((address_space(3))) void*)(lds + off), 16, 0, 0);
    }
    // advance; past the last block of the part the last block is fetched again, into a stage nobody reads
    if (i_blk + 1 < nblk) {
      ++i_blk;
    } else if (i_tile + 1 < n_mt) {
      ++i_tile;
      i_blk = 0;
      x_rows_of(i_tile);
    }
  };

  // ---- fragment reads: lane (lr, lg) of K step s wants row lr, piece 4 s + lg of a 16-row unit
  const int lr = lane & 15, lg = lane >> 4;
  int frag_off[2];
#pragma unroll
  for (int sk = 0; sk < 2; ++sk) frag_off[sk] = (((lr >> 3) * 64) + (lr & 7) * 8 + ((4 * sk + lg) ^ (lr & 7))) * 16;
  const int u0 = wn * NU;

#pragma unroll
  for (int b = 0; b < R::kStages - 1; ++b) issue(b);
  int stage = 0, refill = R::kStages - 1;
  for (int tile = 0; tile < n_mt; ++tile) {
    f32x4 acc[2][NU];
#pragma unroll
    for (int fi = 0; fi < 2; ++fi)
#pragma unroll
      for (int ui = 0; ui < NU; ++ui) acc[fi][ui] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int b = 0; b < nblk; ++b) {
      // this wavefront's share of the block has landed; meet: everybody's has, and everybody is
      // done with the block before, whose stage is refilled next
      wait_vm<(R::kStages - 2) * R::kLpw>();
      ring_barrier();
      issue(refill);
      LdsBytes base = lds + stage * R::kStage;
#pragma unroll
      for (int sk = 0; sk < 2; ++sk) {
        u32x4 a[2];
#pragma unroll
        for (int fi = 0; fi < 2; ++fi)
          a[fi] = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(base + (2 * (2 * wm + fi)) * 1024 +
                                                                                    frag_off[sk]);
#pragma unroll
        for (int ui = 0; ui < NU; ++ui) {
          int u = u0 + ui;
          if (u >= U) u = U - 1;  // a unit past the last one is multiplied again and not stored
          const u32x4 bfr = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(base + (8 + 2 * u) * 1024 +
                                                                                               frag_off[sk]);
#pragma unroll
          for (int fi = 0; fi < 2; ++fi) acc[fi][ui] = mfma16<T>(a[fi], bfr, acc[fi][ui]);
        }
      }
      stage = stage + 1 == R::kStages ? 0 : stage + 1;
      refill = refill + 1 == R::kStages ? 0 : refill + 1;
    }
    // ---- the tile's sums: lane holds column lr, rows 4 lg + i of fragment (2 wm + fi), unit u0 + ui.
    // (s_out is free: whoever read it for the tile before has passed this tile's barriers since)
    const int m_cnt = m_rows - tile * kShrTM < kShrTM ? m_rows - tile * kShrTM : kShrTM;
#pragma unroll
    for (int pj = 0; pj < NPROJ; ++pj) {
#pragma unroll
      for (int ui = 0; ui < NU; ++ui) {
        const int u = u0 + ui;
        if (u < U && u / NT == pj) {
          const int c = (u - pj * NT) * 16 + lr;
#pragma unroll
          for (int fi = 0; fi < 2; ++fi)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              s_out[((2 * wm + fi) * 16 + 4 * lg + i) * kShrOutPitch + c] =
                  T::from_float(nb0 + c < r_eff ? acc[fi][ui][i] : 0.f);
        }
      }
      lds_barrier();
      // rows of 8 columns (16 bytes) each; columns behind the adapter's tiles are zeros
      uint16_t* og = reinterpret_cast<uint16_t*>(p.o[pj]);
      const int64_t orow0 = row_first + (int64_t)tile * kShrTM;
      if ((nb_cnt & 7) == 0 && (p.o_stride & 7) == 0 && (nb0 & 7) == 0 && aligned16_dev(og)) {
        const int pieces = nb_cnt >> 3;
        for (int idx = tid; idx < m_cnt * pieces; idx += kShrThreads) {
          const int m = idx / pieces, c8 = (idx - m * pieces) * 8;
          u32x4 v = zero16();
          if (c8 < NT * 16) v = *reinterpret_cast<const u32x4*>(s_out + m * kShrOutPitch + c8);
          *reinterpret_cast<u32x4*>(og + (orow0 + m) * p.o_stride + nb0 + c8) = v;
        }
      } else {
        for (int idx = tid; idx < m_cnt * nb_cnt; idx += kShrThreads) {
          const int m = idx / nb_cnt, c = idx - m * nb_cnt;
          og[(orow0 + m) * p.o_stride + nb0 + c] = c < NT * 16 ? s_out[m * kShrOutPitch + c] : (uint16_t)0;
        }
      }
      if (NPROJ > 1) lds_barrier();  // the staging tile is rewritten for the next projection
    }
  }
  wait_vm<0>();  // the loads past the end
  ring_barrier();  // the ring and the staging tile are free again
}

// A part through the LDS ring: per pass of 64 rank columns the 16-column tiles that hold columns
// of the adapter are multiplied; a pass behind the adapter's rank only writes zeros.
template <typename T, int NPROJ>
__device__ __forceinline__ void shrink_part_lds(const SegShrinkArgs& p, unsigned char* ring, int64_t row_first,
                                                int m_rows, int r_eff, int64_t base_li, int rank) {
  uint16_t* s_out = reinterpret_cast<uint16_t*>(ring + kShrRingBytes);
  for (int nb0 = 0; nb0 < p.max_rank; nb0 += kShrNB) {
    const int nb_cnt = p.max_rank - nb0 < kShrNB ? p.max_rank - nb0 : kShrNB;
    const int n_tiles = (r_eff - nb0 + 15) >> 4 < 4 ? (r_eff - nb0 + 15) >> 4 : 4;
    switch (n_tiles > 0 ? n_tiles : 0) {
      case 1: shrink_part_lds_pass<T, NPROJ, 1>(p, ring, s_out, row_first, m_rows, r_eff, base_li, rank, nb0, nb_cnt); break;
      case 2: shrink_part_lds_pass<T, NPROJ, 2>(p, ring, s_out, row_first, m_rows, r_eff, base_li, rank, nb0, nb_cnt); break;
      case 3: shrink_part_lds_pass<T, NPROJ, 3>(p, ring, s_out, row_first, m_rows, r_eff, base_li, rank, nb0, nb_cnt); break;
      case 4: shrink_part_lds_pass<T, NPROJ, 4>(p, ring, s_out, row_first, m_rows, r_eff, base_li, rank, nb0, nb_cnt); break;
      default: {
        // no column of the adapter in this pass: zeros
#pragma unroll
        for (int pj = 0; pj < NPROJ; ++pj) {
          uint16_t* og = reinterpret_cast<uint16_t*>(p.o[pj]);
          for (int idx = threadIdx.x; idx < m_rows * nb_cnt; idx += kShrThreads) {
            const int m = idx / nb_cnt, c = idx - m * nb_cnt;
            og[(row_first + m) * p.o_stride + nb0 + c] = 0;
          }
        }
        break;
      }
    }
  }
}

// One tile: token rows row_first .. row_first + m_cnt (m_cnt <= kShrTM) of a request
// whose weight rows start at a_loc[base_li]; of every 64 rank columns the 16-column
// tiles t with t % p.col_split == cg.  All threads of the workgroup call it together;
// it ends with a barrier.
template <typename T, int NPROJ, bool DEEP>
__device__ __forceinline__ void shrink_tile(const SegShrinkArgs& p, float* s_part, int64_t row_first, int m_cnt,
                                            int r_eff, int64_t base_li, int rank, int cg) {
  const int cs = p.col_split;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint16_t* xg = reinterpret_cast<const uint16_t*>(p.x);
  const uint16_t* wg = reinterpret_cast<const uint16_t*>(p.w);
  const int lr = lane & 15, lg = lane >> 4;  // MFMA order: fragment row / k-group of this lane
  const int lrow = lr & 7, piece = lg + 4 * (lr >> 3);  // line order: row inside a half fragment, 16-byte piece

  // token rows of the lane's two loads per A fragment (clamped; rows past the end
  // contribute nothing because their results are never stored)
  const uint16_t* xline[kShrMF][2];
#pragma unroll
  for (int f = 0; f < kShrMF; ++f)
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      int m = f * 16 + 8 * g + lrow;
      if (m >= m_cnt) m = m_cnt - 1;
      xline[f][g] = xg + (row_first + m) * p.x_stride;
    }

  for (int nb0 = 0; nb0 < p.max_rank; nb0 += kShrNB) {
    const int nb_cnt = p.max_rank - nb0 < kShrNB ? p.max_rank - nb0 : kShrNB;
    // this workgroup's tiles of the pass: cg, cg + cs, ...; n_own of them hold columns of the adapter
    const int n_tiles = (r_eff - nb0 + 15) >> 4 < 4 ? (r_eff - nb0 + 15) >> 4 : 4;
    const int n_own = n_tiles > cg ? (n_tiles - cg + cs - 1) / cs : 0;
    f32x4 acc[NPROJ][kShrMF][4];
    if (n_own > 0) {
      // weight rows of the lane's two loads per B fragment, for every projection of the
      // launch (projection pj's rows start rank entries of a_loc behind the one before):
      // the page lookups go out together; a row that does not exist (j >= r_eff, bad page
      // id) reads pool page 0 -- its products only reach output columns that are zeroed below
      const uint16_t* wline[NPROJ][4][2];
      {
        int64_t pg[NPROJ][4][2];
#pragma unroll
        for (int pj = 0; pj < NPROJ; ++pj)
#pragma unroll
          for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int g = 0; g < 2; ++g) {
              const int j = nb0 + (cg + cs * t) * 16 + 8 * g + lrow;
              pg[pj][t][g] = seg_page_nobranch(p.t, base_li + (int64_t)pj * rank + j,
                                               t < n_own && j < r_eff && p.t.n_loc > 0);
            }
#pragma unroll
        for (int pj = 0; pj < NPROJ; ++pj)
#pragma unroll
          for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int g = 0; g < 2; ++g) wline[pj][t][g] = wg + (pg[pj][t][g] >= 0 ? pg[pj][t][g] : 0) * p.w_stride;
      }
#pragma unroll
      for (int pj = 0; pj < NPROJ; ++pj)
#pragma unroll
        for (int f = 0; f < kShrMF; ++f)
#pragma unroll
          for (int t = 0; t < 4; ++t) acc[pj][f][t] = f32x4{0.f, 0.f, 0.f, 0.f};

      // fragments that hold no row or no rank column are neither loaded nor multiplied
      auto k_loop = [&](auto mf) {
        constexpr int MF = decltype(mf)::value;
        if constexpr (NPROJ == 1) {
          if (DEEP) {
            switch (n_own) {
              case 1: shrink_k_loop_ring<T, 1, MF, 4>(xline, wline[0], wave, piece, p.h_in, acc[0]); break;
              case 2: shrink_k_loop_ring<T, 2, MF, 4>(xline, wline[0], wave, piece, p.h_in, acc[0]); break;
              case 3: shrink_k_loop_ring<T, 3, MF, 4>(xline, wline[0], wave, piece, p.h_in, acc[0]); break;
              default: shrink_k_loop_ring<T, 4, MF, 4>(xline, wline[0], wave, piece, p.h_in, acc[0]); break;
            }
          } else {
            switch (n_own) {
              case 1: shrink_k_loop<T, 1, MF>(xline, wline[0], wave, piece, p.h_in, acc[0]); break;
              case 2: shrink_k_loop<T, 2, MF>(xline, wline[0], wave, piece, p.h_in, acc[0]); break;
              case 3: shrink_k_loop<T, 3, MF>(xline, wline[0], wave, piece, p.h_in, acc[0]); break;
              default: shrink_k_loop<T, 4, MF>(xline, wline[0], wave, piece, p.h_in, acc[0]); break;
            }
          }
        } else {
          switch (n_own) {
            case 1: shrink_k_loop_qkv<T, 1, MF>(xline, wline, wave, piece, p.h_in, acc); break;
            case 2: shrink_k_loop_qkv<T, 2, MF>(xline, wline, wave, piece, p.h_in, acc); break;
            case 3: shrink_k_loop_qkv<T, 3, MF>(xline, wline, wave, piece, p.h_in, acc); break;
            default: shrink_k_loop_qkv<T, 4, MF>(xline, wline, wave, piece, p.h_in, acc); break;
          }
        }
      };
      switch ((m_cnt + 15) >> 4) {
        case 1: k_loop(std::integral_constant<int, 1>{}); break;
        case 2: k_loop(std::integral_constant<int, 2>{}); break;
        case 3: k_loop(std::integral_constant<int, 3>{}); break;
        default: k_loop(std::integral_constant<int, 4>{}); break;
      }
    }
    // the partial tiles of the four wavefronts are summed through LDS, one projection at a time
#pragma unroll
    for (int pj = 0; pj < NPROJ; ++pj) {
      if (n_own > 0) {
        // C tile: lane holds column lr, rows 4*lg + i; fragment t is column tile cg + cs * t
        float* mine = s_part + wave * (kShrTM * kShrLd);
#pragma unroll
        for (int f = 0; f < kShrMF; ++f)
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (t < n_own) {
#pragma unroll
              for (int i = 0; i < 4; ++i)
                mine[(f * 16 + lg * 4 + i) * kShrLd + (cg + cs * t) * 16 + lr] = acc[pj][f][t][i];
            }
      }
      __syncthreads();
      uint16_t* og = reinterpret_cast<uint16_t*>(p.o[pj]);
      for (int idx = tid; idx < kShrTM * kShrNB; idx += kShrThreads) {
        const int m = idx / kShrNB, c = idx - m * kShrNB;
        if (m < m_cnt && c < nb_cnt && ((c >> 4) & (cs - 1)) == cg) {
          float v = 0.f;
          if (nb0 + c < r_eff) {
#pragma unroll
            for (int wv = 0; wv < kShrWaves; ++wv) v += s_part[wv * (kShrTM * kShrLd) + m * kShrLd + c];
          }
          og[(row_first + m) * p.o_stride + nb0 + c] = T::from_float(v);
        }
      }
      __syncthreads();
    }
  }
}

// 16 token rows: the unit work is shared out in
constexpr int kShrUnit = 16;
constexpr int kShrMaxGrid = 256;  // one workgroup per compute unit
constexpr int kShrDeepTokens = 4096;  // batches up to this size use the deeper K loop (see shrink_k_loop_ring)
constexpr int kShrChunk = 256;    // requests described at a time (one per thread)

// inclusive prefix sum of `v` over the workgroup; *total receives the sum
__device__ __forceinline__ int64_t shrink_block_scan(int64_t v, int64_t* s_wave, int64_t* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int64_t inc = v;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const int64_t up = __shfl_up(inc, o, kWave);
    if (lane >= o) inc += up;
  }
  if (lane == kWave - 1) s_wave[wave] = inc;
  __syncthreads();
  int64_t before = 0, tot = 0;
#pragma unroll
  for (int wv = 0; wv < kShrWaves; ++wv) {
    const int64_t c = s_wave[wv];
    if (wv < wave) before += c;
    tot += c;
  }
  __syncthreads();
  *total = tot;
  return before + inc;
}

// Cost of walking `units` 16-row units of a rank-r request as tiles of up to kShrMF units, in
// eighths of what a weight row costs: measured per tile 6.7 us + 0.2 us per weight row, plus
// 0.177 us per activation row (hidden 4096; all three scale alike with the hidden size).
// 32-bit: callers keep a request to 4096 units, so that 256 requests still sum below 2^32.
constexpr uint32_t kShrCostUnit = 7 * kShrUnit;
__device__ __forceinline__ uint32_t shrink_tile_cost(int r_own) { return 268u + 8u * (uint32_t)r_own; }
__device__ __forceinline__ uint32_t shrink_chunk_cost(int units, int r_eff) {
  const uint32_t tiles = ((uint32_t)units + kShrMF - 1) / kShrMF;
  return tiles * shrink_tile_cost(r_eff) + (uint32_t)units * kShrCostUnit;
}

// About the fewest even chunks of a request of `units` units such that none costs more than
// t.  Float arithmetic (a chain of exact integer divisions costs microseconds on a lone
// wavefront): the count only steers the balance, and every wavefront computes the same one.
__device__ __forceinline__ int shrink_chunks_needed(int units, int r_eff, uint32_t t) {
  // largest chunk: m whole tiles, then e more units of one more tile
  const float a = (float)shrink_tile_cost(r_eff), full = a + (float)(kShrMF * kShrCostUnit);
  const float m = __builtin_floorf((float)t * __builtin_amdgcn_rcpf(full));
  const float rem = (float)t - m * full;
  float e = __builtin_floorf((rem - a) * (1.0f / (float)kShrCostUnit));
  e = e < 0.f ? 0.f : (e > (float)(kShrMF - 1) ? (float)(kShrMF - 1) : e);
  float size = m * (float)kShrMF + e;
  if (!(size >= 1.f)) return units;
  if (size > (float)units) size = (float)units;
  int n = (int)__builtin_ceilf((float)units * __builtin_amdgcn_rcpf(size));
  return n < 1 ? 1 : (n > units ? units : n);
}

// The requests are cut into units of 16 token rows, a unit of a rank-r request
// costing kShrTM + r: its share of the bytes a full tile moves -- 16 activation
// rows and a quarter of the r weight rows (a weight row measures as costly as an
// activation row).  Laid end to end in request order, the units' cost line is
// cut into gridDim.x equal parts, XCD-major: consecutive workgroup ids go to the
// 8 XCDs in turn, so workgroup id -> part (id % 8) * (gridDim.x / 8) + id / 8
// gives every XCD one contiguous eighth (neighbouring tiles of a request, which
// read the same weight rows, share an L2) and every workgroup the same cost,
// whatever the mix of request lengths and ranks.  A workgroup owns the units
// whose start falls into its part and walks them as tiles of up to kShrMF units.
// RING: the K loop fed through LDS (shrink_part_lds; launches whose every workgroup has whole tiles
// and whole 64-k blocks), otherwise from registers (shrink_tile), DEEP with three blocks in flight
// per wavefront.  The ring kernels need half the register file at most, and with no more than 256
// registers a wavefront the matrix instructions accumulate in ordinary registers instead of being
// copied in and out of the accumulation registers around every block.
template <typename T, int NPROJ, bool DEEP, bool RING>
__global__ __launch_bounds__(kShrThreads, RING ? 2 : 1) void sgmm_shrink_kernel(const SegShrinkArgs p) {
  extern __shared__ float s_part[];  // [kShrWaves][kShrTM][kShrLd]
  __shared__ int64_t s_wave[kShrWaves];
  __shared__ int s_row0[kShrChunk], s_rows[kShrChunk], s_ub[kShrChunk], s_ue[kShrChunk], s_rank[kShrChunk];
  __shared__ int64_t s_base[kShrChunk];
  __shared__ int s_first, s_last;
  const int tid = threadIdx.x;
  // XCD-major position of the workgroup; col_split neighbours share the rows of a part
  const int slot = (int)(blockIdx.x & 7) * ((int)gridDim.x >> 3) + (int)(blockIdx.x >> 3);
  const int parts = (int)gridDim.x / p.col_split;
  const int part = slot / p.col_split, cg = slot - part * p.col_split;
  const int row_cap = p.m_tiles * kShrTM;  // rows of a request past max_input_len are not touched

  // request -> cost of one of its units (0: nothing to do).  The loads sit outside
  // every branch, in two dependent groups: (adapter id, first row, row count), then
  // that adapter's (length, start) -- an invalid request re-reads entry 0.
  auto describe = [&](int req, int64_t& base_li, int& r, int& row0, int& rows, int& units) -> int64_t {
    const bool mine = tid < kShrChunk && req < p.t.n_requests;
    const int rq = mine ? req : 0;
    const int64_t a = p.t.b_indicies[rq];
    row0 = p.t.b_start_loc[rq];
    rows = p.t.b_seq_len[rq];
    const bool a_ok = (uint64_t)a < (uint64_t)p.t.n_adapters;
    const int64_t len = p.t.a_len[a_ok ? a : 0];
    const int64_t start = p.t.a_start[a_ok ? a : 0];
    r = (int)(len >> 2);
    units = 0;
    if (!mine || !a_ok || row0 < 0 || rows <= 0 || row0 >= p.t.n_tokens) return 0;
    if (rows > p.t.n_tokens - row0) rows = p.t.n_tokens - row0;
    if (rows > row_cap) rows = row_cap;
    base_li = start + (int64_t)r * p.qkvo;
    units = (rows + kShrUnit - 1) / kShrUnit;
    return kShrTM + (r < p.max_rank ? r : p.max_rank);
  };

  // total cost (one pass when the requests fit one thread each)
  int64_t total = 0;
  if (p.t.n_requests > kShrChunk) {
    for (int c0 = 0; c0 < p.t.n_requests; c0 += kShrChunk) {
      int64_t base_li = 0;
      int r = 0, row0 = 0, rows = 0, units = 0;
      const int64_t cu = describe(c0 + tid, base_li, r, row0, rows, units);
      int64_t tot = 0;
      shrink_block_scan(cu * units, s_wave, &tot);
      total += tot;
    }
  }
  // Few requests: no workgroup is given rows of two requests (each would cost it a tile's
  // fixed share); request j is cut into n_j even chunks, one workgroup each.
  const bool aligned = p.t.n_requests <= kShrChunk && p.t.n_requests <= parts && p.m_tiles <= 1024;
  int64_t carry = 0;  // cost in front of the current chunk of requests
  for (int c0 = 0; c0 < p.t.n_requests; c0 += kShrChunk) {
    int64_t base_li = 0;
    int r = 0, row0 = 0, rows = 0, units = 0;
    const int64_t cu = describe(c0 + tid, base_li, r, row0, rows, units);
    int64_t tot = 0;
    int ub = 0, ue = 0;
    if (!aligned) {
      const int64_t cp = carry + shrink_block_scan(cu * units, s_wave, &tot) - cu * units;  // cost in front of me
      if (p.t.n_requests <= kShrChunk) total = tot;
      if (total <= 0) return;
      if (units > 0) {
        // units of my request whose start cost cp + u * cu lies in [lo, hi)
        const int64_t lo = total * part / parts, hi = total * (part + 1) / parts;
        const int64_t b = lo > cp ? (lo - cp + cu - 1) / cu : 0;
        const int64_t e = hi > cp ? (hi - cp + cu - 1) / cu : 0;
        ub = b < units ? (int)b : units;
        ue = e < units ? (int)e : units;
      }
    }
    if (tid == 0) {
      s_first = kShrChunk;
      s_last = -1;
    }
    __syncthreads();
    if (tid < kShrChunk) {
      s_ub[tid] = ub;
      s_ue[tid] = ue;
      s_row0[tid] = row0;
      s_rows[tid] = units > 0 ? rows : 0;
      s_rank[tid] = r;
      s_base[tid] = base_li;
      if (ue > ub) {
        atomicMin(&s_first, tid);
        atomicMax(&s_last, tid);
      }
    }
    __syncthreads();
    if (aligned) {
      // Every wavefront repeats the search on its own (shuffles only, no barrier): lane
      // l looks after requests l, l + 64, ...  T, the cost of the dearest chunk, is
      // bisected down to the least value whose n_j still sum to at most the grid
      // (8 rounds: 1/256 of the range).
      constexpr int kPerLane = kShrChunk / kWave;
      const int lane = tid & 63;
      int un[kPerLane], re[kPerLane];
      uint32_t t_hi = 0;  // one chunk per request always fits: n_requests <= parts
      uint32_t t_sum = 0;
#pragma unroll
      for (int q = 0; q < kPerLane; ++q) {
        const int idx = lane + q * kWave;
        un[q] = (s_rows[idx] + kShrUnit - 1) / kShrUnit;
        re[q] = s_rank[idx] < p.max_rank ? s_rank[idx] : p.max_rank;
        re[q] = (re[q] + p.col_split - 1) / p.col_split;  // weight rows one workgroup of the split reads
        if (idx >= p.t.n_requests) un[q] = 0;
        const uint32_t c = un[q] > 0 ? shrink_chunk_cost(un[q], re[q]) : 0u;
        t_hi = c > t_hi ? c : t_hi;
        t_sum += c;
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const uint32_t other = (uint32_t)__shfl_xor((int)t_hi, o, kWave);
        t_hi = other > t_hi ? other : t_hi;
        t_sum += (uint32_t)__shfl_xor((int)t_sum, o, kWave);
      }
      uint32_t t_lo = 0;  // infeasible (or untested) bound
      auto fits = [&](uint32_t t) {
        int sum = 0;
#pragma unroll
        for (int q = 0; q < kPerLane; ++q)
          if (q * kWave < p.t.n_requests) sum += un[q] > 0 ? shrink_chunks_needed(un[q], re[q], t) : 0;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, kWave);
        return sum <= parts;
      };
      // The even share is a lower bound (cutting only adds cost).  Guesses a quarter above
      // it, a quarter above that, ... until one fits; then three rounds of bisection
      // between the last two: T ends within a few percent of the least feasible one.
      {
        uint32_t guess = t_sum / (uint32_t)parts;
        t_lo = guess;
        for (int k = 0; k < 12; ++k) {
          guess += (guess >> 2) + 1u;
          if (guess >= t_hi) break;
          if (fits(guess)) {
            t_hi = guess;
            break;
          }
          t_lo = guess;
        }
      }
      for (int round = 0; round < 3 && t_hi - t_lo > 1; ++round) {
        const uint32_t t_mid = t_lo + (t_hi - t_lo) / 2;
        if (fits(t_mid)) t_hi = t_mid; else t_lo = t_mid;
      }
      // chunks in request order; the request that owns chunk `part` gets its units
      int before = 0;
#pragma unroll
      for (int q = 0; q < kPerLane; ++q) {
        if (q * kWave >= p.t.n_requests) break;
        const int n_mine = un[q] > 0 ? shrink_chunks_needed(un[q], re[q], t_hi) : 0;
        int inc = n_mine;
#pragma unroll
        for (int o = 1; o < kWave; o <<= 1) {
          const int up = __shfl_up(inc, o, kWave);
          if (lane >= o) inc += up;
        }
        const int mine_before = before + inc - n_mine;
        if (tid < kWave && n_mine > 0 && part >= mine_before && part < mine_before + n_mine) {
          const int64_t i = part - mine_before;
          const int idx = lane + q * kWave;
          s_ub[idx] = (int)((int64_t)un[q] * i / n_mine);
          s_ue[idx] = (int)((int64_t)un[q] * (i + 1) / n_mine);
          s_first = idx;
          s_last = idx;
        }
        before += __shfl(inc, kWave - 1, kWave);
      }
      __syncthreads();
    }
    // everything read back from LDS is the same in every lane: say so, so that the
    // tile code keeps it in scalar registers and branches on it uniformly
    auto uni = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
    const int first = uni(s_first), last = uni(s_last);
    for (int j = first; j <= last; ++j) {
      const int u0 = uni(s_ub[j]), u1 = uni(s_ue[j]);
      const int rj = uni(s_rank[j]);
      const int r_eff = rj < p.max_rank ? rj : p.max_rank;
      const int rw0 = uni(s_row0[j]), rows = uni(s_rows[j]);
      const int64_t bl = s_base[j];
      const int64_t base_li =
          (int64_t)(((uint64_t)(uint32_t)uni((int)((uint64_t)bl >> 32)) << 32) | (uint32_t)uni((int)(uint32_t)bl));
      if constexpr (RING) {
        // all tiles of the request's share as one stream of blocks (the launcher picks this
        // instantiation only for layouts the vector path reads)
        const int m0 = u0 * kShrUnit, m_end = u1 * kShrUnit < rows ? u1 * kShrUnit : rows;
        if (m_end > m0)
          shrink_part_lds<T, NPROJ>(p, reinterpret_cast<unsigned char*>(s_part), (int64_t)rw0 + m0, m_end - m0, r_eff,
                                    base_li, rj);
      }
      for (int u = u0; !RING && u < u1; u += kShrMF) {
        const int m0 = u * kShrUnit;
        int m_end = (u + kShrMF < u1 ? u + kShrMF : u1) * kShrUnit;
        if (m_end > rows) m_end = rows;
        if (m_end <= m0) continue;
        if (!p.vec_ok) {
          if (cg == 0)
            for (int pj = 0; pj < NPROJ; ++pj)
              shrink_generic<T>(p, pj, r_eff, base_li + (int64_t)pj * rj, rw0, m0, m_end - m0);
          __syncthreads();
        } else {
          shrink_tile<T, NPROJ, DEEP>(p, s_part, (int64_t)rw0 + m0, m_end - m0, r_eff, base_li, rj, cg);
        }
      }
    }
    carry += tot;
    __syncthreads();  // the tables are rewritten by the next chunk
  }
}

// ---------------------------------------------------------------------------
// shrink with a plan: the split of the requests over the workgroups depends only on
// the batch (request lengths, adapters' ranks), not on the layer or projection, so it
// can be computed once per prefill step and read back by the 4 x n_layers shrink
// calls of that step with one scalar load per workgroup.
// ---------------------------------------------------------------------------
constexpr int kSegPlanMagic = 0x53475031;
constexpr int kSegPlanHeaderWords = 16;
constexpr int kSegPartWords = 8;
enum SegPlanHeader { SP_MAGIC = 0, SP_PARTS, SP_SPLIT, SP_NREQ, SP_NTOKENS, SP_MAXRANK, SP_ROWCAP, SP_STATUS };  // SP_STATUS: as PH_STATUS of the decode plan (word 7)
enum SegPart { PT_ROW = 0, PT_ROWS, PT_RANK, PT_START_LO, PT_START_HI };

// One workgroup.  Same scheme as the few-requests case of sgmm_shrink_kernel (request j
// in n_j even chunks, T bisected), with more rounds; record `part` = chunk `part` in
// request order, empty records behind the last chunk.
__global__ __launch_bounds__(kShrThreads) void sgmm_plan_kernel(int* plan, SegTables t, int parts, int col_split,
                                                                int max_rank, int row_cap) {
  __shared__ int64_t s_wave[kShrWaves];
  const int tid = threadIdx.x;
  for (int i = tid; i < parts * kSegPartWords; i += kShrThreads) plan[kSegPlanHeaderWords + i] = 0;
  const bool mine = tid < t.n_requests;
  const int rq = mine ? tid : 0;
  const int64_t a = t.b_indicies[rq];
  const int row0 = t.b_start_loc[rq];
  int rows = t.b_seq_len[rq];
  const bool a_ok = (uint64_t)a < (uint64_t)t.n_adapters;
  const int64_t len = t.a_len[a_ok ? a : 0];
  const int64_t start = t.a_start[a_ok ? a : 0];
  const int r = (int)(len >> 2);
  int units = 0;
  if (mine && a_ok && row0 >= 0 && rows > 0 && row0 < t.n_tokens) {
    if (rows > t.n_tokens - row0) rows = t.n_tokens - row0;
    if (rows > row_cap) rows = row_cap;
    units = (rows + kShrUnit - 1) / kShrUnit;
  }
  int r_own = r < max_rank ? r : max_rank;
  r_own = (r_own + col_split - 1) / col_split;
  const uint32_t cost = units > 0 ? shrink_chunk_cost(units, r_own) : 0u;
  int64_t t_sum = 0;
  shrink_block_scan((int64_t)cost, s_wave, &t_sum);
  // the dearest single request bounds T from above (one chunk per request always fits)
  uint32_t t_hi = cost;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const uint32_t other = (uint32_t)__shfl_xor((int)t_hi, o, kWave);
    t_hi = other > t_hi ? other : t_hi;
  }
  if ((tid & 63) == 0) s_wave[tid >> 6] = t_hi;
  __syncthreads();
#pragma unroll
  for (int wv = 0; wv < kShrWaves; ++wv) t_hi = (uint32_t)s_wave[wv] > t_hi ? (uint32_t)s_wave[wv] : t_hi;
  __syncthreads();
  uint32_t t_lo = (uint32_t)(t_sum / parts);  // the even share: a lower bound
  if (t_lo > t_hi) t_lo = t_hi;
  for (int round = 0; round < 20 && t_hi - t_lo > 1; ++round) {
    const uint32_t t_mid = t_lo + (t_hi - t_lo) / 2;
    int64_t sum = 0;
    shrink_block_scan(units > 0 ? shrink_chunks_needed(units, r_own, t_mid) : 0, s_wave, &sum);
    if (sum <= parts) t_hi = t_mid; else t_lo = t_mid;
  }
  const int n_mine = units > 0 ? shrink_chunks_needed(units, r_own, t_hi) : 0;
  int64_t n_all = 0;
  const int64_t before = shrink_block_scan(n_mine, s_wave, &n_all) - n_mine;
  for (int i = 0; i < n_mine && before + i < parts; ++i) {
    const int ub = (int)((int64_t)units * i / n_mine), ue = (int)((int64_t)units * (i + 1) / n_mine);
    const int m0 = ub * kShrUnit;
    const int m_end = ue * kShrUnit < rows ? ue * kShrUnit : rows;
    int* rec = plan + kSegPlanHeaderWords + (before + i) * kSegPartWords;
    rec[PT_ROW] = row0 + m0;
    rec[PT_ROWS] = m_end - m0;
    rec[PT_RANK] = r;
    rec[PT_START_LO] = (int)(uint32_t)start;
    rec[PT_START_HI] = (int)((uint64_t)start >> 32);
  }
  if (tid == 0) {
    plan[SP_MAGIC] = kSegPlanMagic;
    plan[SP_PARTS] = parts;
    plan[SP_SPLIT] = col_split;
    plan[SP_NREQ] = t.n_requests;
    plan[SP_NTOKENS] = t.n_tokens;
    plan[SP_MAXRANK] = max_rank;
    plan[SP_ROWCAP] = row_cap;
    plan[SP_STATUS] = 0;
  }
}

template <typename T, int NPROJ, bool DEEP, bool RING>
__global__ __launch_bounds__(kShrThreads, RING ? 2 : 1) void sgmm_shrink_planned_kernel(const SegShrinkArgs p,
                                                                                        const int* plan) {
  extern __shared__ float s_part[];  // [kShrWaves][kShrTM][kShrLd], or the ring and its staging tile
  const int slot = (int)(blockIdx.x & 7) * ((int)gridDim.x >> 3) + (int)(blockIdx.x >> 3);
  const int parts = (int)gridDim.x / p.col_split;
  // (an integer division runs on the vector unit: say that its result is the same in every lane)
  const int part = __builtin_amdgcn_readfirstlane(slot / p.col_split), cg = slot - part * p.col_split;
  // header and record of this part in one group of scalar loads (the plan does not change while
  // this kernel runs: reading it through the constant address space keeps the loads scalar
  // whatever else the kernel writes)
  typedef const int __attribute__((address_space(4))) * ConstWords;
  ConstWords head = (ConstWords)plan;
  ConstWords rec = head + kSegPlanHeaderWords + part * kSegPartWords;
  int magic = head[SP_MAGIC], n_parts = head[SP_PARTS], split = head[SP_SPLIT];
  int row_first = rec[PT_ROW], m_rows = rec[PT_ROWS], r = rec[PT_RANK], lo = rec[PT_START_LO], hi = rec[PT_START_HI];
  asm volatile("" : "+s"(magic), "+s"(n_parts), "+s"(split), "+s"(row_first), "+s"(m_rows), "+s"(r), "+s"(lo), "+s"(hi));
  if (magic != kSegPlanMagic || n_parts != parts || split != p.col_split) {  // not a plan of this launch shape: nothing is done
    if (magic == kSegPlanMagic && blockIdx.x == 0 && threadIdx.x == 0) const_cast<int*>(plan)[SP_STATUS] = 1;
    return;
  }
  if (m_rows <= 0 || row_first < 0 || m_rows > p.t.n_tokens - row_first) return;
  const int r_eff = r < p.max_rank ? r : p.max_rank;
  const int64_t base_li = (int64_t)(((uint64_t)(uint32_t)hi << 32) | (uint32_t)lo) + (int64_t)r * p.qkvo;
  if constexpr (RING) {  // all tiles of the part as one stream of blocks
    shrink_part_lds<T, NPROJ>(p, reinterpret_cast<unsigned char*>(s_part), row_first, m_rows, r_eff, base_li, r);
    return;
  }
  for (int m0 = 0; !RING && m0 < m_rows; m0 += kShrTM) {
    const int m_cnt = m_rows - m0 < kShrTM ? m_rows - m0 : kShrTM;
    if (!p.vec_ok) {
      if (cg == 0)
        for (int pj = 0; pj < NPROJ; ++pj)
          shrink_generic<T>(p, pj, r_eff, base_li + (int64_t)pj * r, row_first, m0, m_cnt);
      __syncthreads();
    } else {
      shrink_tile<T, NPROJ, DEEP>(p, s_part, (int64_t)row_first + m0, m_cnt, r_eff, base_li, r, cg);
    }
  }
}

// ---------------------------------------------------------------------------
// expand
// ---------------------------------------------------------------------------
struct SegExpandArgs {
  void* o;
  const void* x;
  const void* w;
  const void* scales;
  SegTables t;
  int64_t x_stride, w_stride, o_stride;
  int64_t page_elems;
  int scales_dtype;
  int feat_out, max_rank, qkvo, m_tiles, m_span, n_chunks;
  int vec_ok;
  int row_cap;  // rows of a request at or past this are not touched (max_input_len, rounded up to a row tile)
  // q, k and v in one launch (nproj == 3): n_chunks counts the output groups of all three, projection
  // pj owning groups chunk_end[pj - 1] .. chunk_end[pj]; o, x, feat_out, o_stride and qkvo above are then
  // taken from these by the workgroup (expand_select)
  int nproj;
  int chunk_end[3];
  void* o3[3];
  const void* x3[3];
  int feat3[3];
  int64_t o_stride3[3];
};

// The arguments as one projection's workgroup sees them, and its output group inside that projection.
template <int NPROJ>
__device__ __forceinline__ SegExpandArgs expand_select(const SegExpandArgs& in, int& group) {
  SegExpandArgs p = in;
  if (NPROJ == 3) {
    const int pj = group >= in.chunk_end[1] ? 2 : (group >= in.chunk_end[0] ? 1 : 0);
    group -= pj == 0 ? 0 : in.chunk_end[pj - 1];
    p.o = pj == 2 ? in.o3[2] : (pj == 1 ? in.o3[1] : in.o3[0]);
    p.x = pj == 2 ? in.x3[2] : (pj == 1 ? in.x3[1] : in.x3[0]);
    p.feat_out = pj == 2 ? in.feat3[2] : (pj == 1 ? in.feat3[1] : in.feat3[0]);
    p.o_stride = pj == 2 ? in.o_stride3[2] : (pj == 1 ? in.o_stride3[1] : in.o_stride3[0]);
    p.qkvo = pj;
  }
  return p;
}

constexpr int kExpThreads = 256;
constexpr int kExpWaves = kExpThreads / kWave;  // 4 wavefronts, one 64-output block each
constexpr int kExpMF = 2;                       // 16-row MFMA fragments per row tile
constexpr int kExpTMW = 16 * kExpMF;            // token rows per row tile
constexpr int kExpOB = 64;                      // outputs per wavefront
constexpr int kExpGroup = kExpOB * kExpWaves;   // outputs per workgroup: 512 contiguous bytes of every row
constexpr int kExpSpanTiles = 16;                    // most row tiles a workgroup of the per-request kernel walks
// workgroups of the walking kernel: as many per compute unit as its registers allow (156; 224 for ranks above 64)
template <int KS>
constexpr int kExpWalkGrid = KS <= 2 ? 768 : 512;
constexpr int kExpMinGrid = 512;                     // shorter spans rather than fewer workgroups than this

template <typename T>
__device__ void expand_generic(const SegExpandArgs& p, int r, int r_eff, int64_t base_li, float scale, int row0,
                               int m0, int m_cnt, int n0, int n_cnt) {
  const uint16_t* x = reinterpret_cast<const uint16_t*>(p.x);
  const uint16_t* w = reinterpret_cast<const uint16_t*>(p.w);
  uint16_t* o = reinterpret_cast<uint16_t*>(p.o);
  const uint32_t page_elems = (uint32_t)p.page_elems;
  for (int idx = threadIdx.x; idx < m_cnt * n_cnt; idx += kExpThreads) {
    const int m = idx / n_cnt, n = n0 + (idx - m * n_cnt);
    const int64_t row = row0 + m0 + m;
    float acc = 0.f;
    for (int d = 0; d < r_eff; ++d) {
      const uint32_t flat = (uint32_t)n * (uint32_t)r + (uint32_t)d;
      const uint32_t pg = flat / page_elems, off = flat - pg * page_elems;
      const int64_t page = seg_page(p.t, base_li + pg);
      if (page < 0) continue;
      acc = __builtin_fmaf(T::to_float(x[row * p.x_stride + d]), T::to_float(w[page * p.w_stride + off]), acc);
    }
    uint16_t* op = o + row * p.o_stride + n;
    *op = T::from_float(T::to_float(*op) + acc * scale);
  }
}

// One wavefront = one 64-output block x a walk over token-row tiles of kExpTMW rows.
// KS = number of 32-wide K steps that cover the rank (1, 2 or 4).  The B^T
// fragments of the block are loaded once and stay in registers; every row tile
// then loads its delta fragments and y values together, multiplies and stores,
// with the next tile's loads already in flight.
//
// MFMA orientation: rows = outputs, columns = tokens, so a lane's C values are
// consecutive outputs of ONE token row.  The row -> output map
//   tile t, row m  <->  output  32*(t/2) + 8*(m/4) + 4*(t%2) + (m%4)   (inside a block)
// gives lane group g = m/4 the outputs 8g..8g+7 (tiles 0,1) and 32+8g..32+8g+7
// (tiles 2,3): each 16-byte access of the four lane groups of a token is one
// contiguous 64-byte run.
//
// y itself is read and written in another lane order.  In the MFMA order the four
// lanes of a token cover 64 bytes per instruction, so an instruction touches 16
// half cache lines; the vector cache handles 8 whole lines per instruction about
// 1.4x faster.  In the "line order" instruction g covers tokens 8g .. 8g+7 of a
// fragment, lane (lr, lg) holding 16-byte piece lg + 4*(lr/8) of token 8g + lr%8.
// Both orders keep a value in the same 16-lane row, at most 8 lanes away, so one
// DPP move per register converts between them (swap_halves, its own inverse).
struct ExpandStage {
  u32x4 y[kExpMF][2];  // y values in line order
};

// The workgroup's delta rows go through LDS (every wavefront multiplies the same
// rows): row stride KS*64 + 16 bytes, the pad spreading the 16 rows of an MFMA-order
// read over all banks.
template <int KS>
constexpr int kExpLdsRow = KS * 64 + 16;
constexpr int kExpChunkRows = 4 * kExpTMW;  // rows staged at a time

// B^T fragments of outputs nb .. nb + 63 (MFMA A operand)
template <typename T, int KS>
__device__ __forceinline__ void expand_load_weights(const SegExpandArgs& p, int r, int r_eff, int64_t base_li, int nb,
                                                    u32x4 (&a)[4][KS]) {
  const int lane = threadIdx.x & 63;
  const int lr = lane & 15, lg = lane >> 4;
  const uint16_t* wg = reinterpret_cast<const uint16_t*>(p.w);
  const uint32_t page_elems = (uint32_t)p.page_elems;
  // phase 1: every page id (loads back to back, no branch in between)
  int64_t page[4][KS];
  uint32_t off[4][KS];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int n = nb + 32 * (t >> 1) + 8 * (lr >> 2) + 4 * (t & 1) + (lr & 3);
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int d = s * 32 + lg * 8;
      const bool want = n < p.feat_out && d < r_eff && p.t.n_loc > 0;
      const uint32_t flat = (uint32_t)n * (uint32_t)r + (uint32_t)d;
      const uint32_t pg = flat / page_elems;
      off[t][s] = flat - pg * page_elems;
      page[t][s] = seg_page_nobranch(p.t, base_li + pg, want);
    }
  }
  // phase 2: every fragment, from a valid dummy address where there is none
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const bool ok = page[t][s] >= 0;
      a[t][s] = ldg16(wg + (ok ? page[t][s] * p.w_stride + off[t][s] : 0));
    }
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int s = 0; s < KS; ++s)
      if (page[t][s] < 0) a[t][s] = zero16();
}

// y values of rows m0w .. m0w + kExpTMW - 1 of the request, outputs nb .. nb + 63, in line
// order; rows at or past m_end read row m_safe instead and are never stored.
__device__ __forceinline__ void expand_load_rows(const SegExpandArgs& p, int row0, int m0w, int m_end, int m_safe,
                                                 int nb, ExpandStage& st) {
  const int lane = threadIdx.x & 63;
  const int lr = lane & 15, lg = lane >> 4;
  const uint16_t* og = reinterpret_cast<const uint16_t*>(p.o);
  const int n_line = nb + 8 * (lg + 4 * (lr >> 3));
#pragma unroll
  for (int f = 0; f < kExpMF; ++f)
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      const int m = m0w + f * 16 + 8 * g + (lr & 7);
      const int64_t row = row0 + (m < m_end ? m : m_safe);
      st.y[f][g] = ldg16_stream(og + row * p.o_stride + (n_line < p.feat_out ? n_line : 0));
    }
}

// Delta rows of one chunk (kExpChunkRows rows from m_chunk; rows at or past m_end repeat
// row m_safe) as the whole workgroup loads them: an instruction covers whole 128-byte
// lines, lane t of the workgroup takes pieces t, t + 256, ...
template <int KS>
struct ExpandChunk {
  u32x4 v[KS * 2];  // kExpChunkRows * KS * 4 pieces / kExpThreads
};

template <int KS>
__device__ __forceinline__ void expand_chunk_load(const SegExpandArgs& p, int row0, int m_chunk, int m_end, int m_safe,
                                                  ExpandChunk<KS>& c) {
  constexpr int kPieces = KS * 4;  // 16-byte pieces of a row
  const uint16_t* xg = reinterpret_cast<const uint16_t*>(p.x);
#pragma unroll
  for (int u = 0; u < KS * 2; ++u) {
    const int idx = (int)threadIdx.x + u * kExpThreads;
    const int row = idx / kPieces, d = (idx - row * kPieces) * 8;
    const int m = m_chunk + row;
    // columns at or past max_rank may not exist in the row; the fragments zero them anyway
    c.v[u] = ldg16(xg + (int64_t)(row0 + (m < m_end ? m : m_safe)) * p.x_stride + (d < p.max_rank ? d : 0));
  }
}

template <int KS>
__device__ __forceinline__ void expand_chunk_store(const ExpandChunk<KS>& c, char* s_chunk) {
  constexpr int kPieces = KS * 4;
#pragma unroll
  for (int u = 0; u < KS * 2; ++u) {
    const int idx = (int)threadIdx.x + u * kExpThreads;
    const int row = idx / kPieces, piece = idx - row * kPieces;
    *reinterpret_cast<u32x4*>(s_chunk + row * kExpLdsRow<KS> + piece * 16) = c.v[u];
  }
}

// One row tile: multiply the staged delta rows m_rel .. m_rel + 31 of the span by the
// block's B^T fragments, add to y and store.
template <typename T, int KS>
__device__ __forceinline__ void expand_finish(const SegExpandArgs& p, float scale, int r_eff, int row0, int m0w,
                                              int m_end, int nb, const u32x4 (&a)[4][KS], const char* s_tile,
                                              const ExpandStage& st) {
  const int lane = threadIdx.x & 63;
  const int lr = lane & 15, lg = lane >> 4;
  uint16_t* og = reinterpret_cast<uint16_t*>(p.o);
  // delta fragments (MFMA B operand) in MFMA order, zero past the adapter's rank
  u32x4 b[kExpMF][KS];
#pragma unroll
  for (int f = 0; f < kExpMF; ++f)
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      b[f][s] = *reinterpret_cast<const u32x4*>(s_tile + (f * 16 + lr) * kExpLdsRow<KS> + s * 64 + lg * 16);
      if (s * 32 + lg * 8 >= r_eff) b[f][s] = zero16();
    }
  f32x4 acc[kExpMF][4];
#pragma unroll
  for (int f = 0; f < kExpMF; ++f)
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      acc[f][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KS; ++s) acc[f][t] = mfma16<T>(a[t][s], b[f][s], acc[f][t]);
    }
  // C tile t: lane holds token column lr, rows 4*lg + i  ->  output 32*(t/2) + 8*lg + 4*(t%2) + i
  const int n_line = nb + 8 * (lg + 4 * (lr >> 3));
#pragma unroll
  for (int f = 0; f < kExpMF; ++f) {
    u32x4 y0 = st.y[f][0], y1 = st.y[f][1];
    swap_halves(y0, y1);  // line order -> MFMA order: y0 = outputs nb + 8*lg .., y1 = outputs nb + 32 + 8*lg ..
    u32x4 out[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const u32x4& yv = h == 0 ? y0 : y1;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        // outputs n + 2q, n + 2q + 1  <-  tile 2h + (2q)/4, element (2q)%4 and the next
        const int e0 = 2 * q;
        const float d0 = acc[f][2 * h + (e0 >> 2)][e0 & 3] * scale;
        const float d1 = acc[f][2 * h + ((e0 + 1) >> 2)][(e0 + 1) & 3] * scale;
        const uint16_t lo = T::from_float(T::lo(yv[q]) + d0);
        const uint16_t hi = T::from_float(T::hi(yv[q]) + d1);
        out[h][q] = (uint32_t)lo | ((uint32_t)hi << 16);
      }
    }
    swap_halves(out[0], out[1]);  // back to line order
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      const int m = m0w + f * 16 + 8 * g + (lr & 7);
      if (m < m_end && n_line < p.feat_out)
        stg16_stream(og + (int64_t)(row0 + m) * p.o_stride + n_line, out[g]);
    }
  }
}

// The whole workgroup enters and stays to the end: the delta rows go through LDS in
// chunks of kExpChunkRows rows, two buffers, one barrier per chunk.  Between barriers
// the wavefront walks the chunk's row tiles for its own outputs nb .. nb + 63, the
// next tile's y values and the next chunk's delta rows always in flight.
template <typename T, int KS>
__device__ __forceinline__ void expand_mfma(const SegExpandArgs& p, int r, int r_eff, int64_t base_li, float scale,
                                            int row0, int m0, int m_end, int nb, char* s_x) {
  constexpr int kChunkBytes = kExpChunkRows * kExpLdsRow<KS>;
  const bool live = nb < p.feat_out;  // a wavefront past the last output only helps with the staging
  u32x4 a[4][KS];
  ExpandStage cur;
  ExpandChunk<KS> chunk;
  // in program order: the first y values and delta rows (they need nothing but the
  // row), then the B^T fragments behind their page ids
  expand_load_rows(p, row0, m0, m_end, m0, nb, cur);
  expand_chunk_load<KS>(p, row0, m0, m_end, m0, chunk);
  expand_load_weights<T, KS>(p, r, r_eff, base_li, live ? nb : 0, a);
  expand_chunk_store<KS>(chunk, s_x);
  __syncthreads();
  int buf = 0;
#pragma unroll 1
  for (int mc = m0; mc < m_end; mc += kExpChunkRows) {
    expand_chunk_load<KS>(p, row0, mc + kExpChunkRows, m_end, m0, chunk);
    if (live) {
#pragma unroll 1
      for (int m0w = mc; m0w < mc + kExpChunkRows && m0w < m_end; m0w += kExpTMW) {
        ExpandStage nxt;  // past the end every lane re-reads row m0; nothing of it is stored
        expand_load_rows(p, row0, m0w + kExpTMW, m_end, m0, nb, nxt);
        expand_finish<T, KS>(p, scale, r_eff, row0, m0w, m_end, nb, a,
                             s_x + buf * kChunkBytes + (m0w - mc) * kExpLdsRow<KS>, cur);
        cur = nxt;
      }
    }
    buf ^= 1;
    expand_chunk_store<KS>(chunk, s_x + buf * kChunkBytes);  // last read two barriers ago
    __syncthreads();
  }
}

// Workgroup = (request, span of p.m_span token rows, group of 256 outputs): wavefront
// w takes the group's w-th block of 64 outputs, keeps that block's B^T fragments
// and walks the span's row tiles, so the four wavefronts together read and write
// 512 contiguous bytes of every row.
template <typename T, int KS, int NPROJ>
__global__ __launch_bounds__(kExpThreads) void sgmm_expand_kernel(const SegExpandArgs p_all) {
  const int wave = threadIdx.x >> 6;
  // the output group is the fastest index: consecutive workgroup ids go to
  // the 8 XCDs in turn, so every XCD owns 1/8 of the output columns of ALL
  // requests -- disjoint pieces of B^T per L2 and an even share of the y traffic
  int blk = blockIdx.x;
  int group = blk % p_all.n_chunks;
  blk /= p_all.n_chunks;
  const SegExpandArgs p = expand_select<NPROJ>(p_all, group);
  const int req = blk / p.m_tiles;
  const int m0 = (blk - req * p.m_tiles) * p.m_span;
  // The request's three entries are independent loads: all go out before the first
  // test, so a workgroup beyond the request's length leaves after one round trip;
  // the adapter's entries (length, start, scale) are the second round trip.
  int64_t a = p.t.b_indicies[req];
  int row0 = p.t.b_start_loc[req];
  int rows = p.t.b_seq_len[req];
  asm volatile("" : "+s"(a), "+s"(row0), "+s"(rows));
  if (row0 < 0 || rows <= 0 || row0 >= p.t.n_tokens) return;
  if (rows > p.t.n_tokens - row0) rows = p.t.n_tokens - row0;
  if (m0 >= rows) return;
  if ((uint64_t)a >= (uint64_t)p.t.n_adapters) return;
  const int r = (int)(p.t.a_len[a] >> 2);
  const int r_eff = r < p.max_rank ? r : p.max_rank;
  if (r_eff <= 0) return;
  const int m_end = rows - m0 < p.m_span ? rows : m0 + p.m_span;
  const int64_t base_li = p.t.a_start[a] + (int64_t)r * p.qkvo;
  const float scale = load_scale(p.scales, p.scales_dtype, a);
  if (!p.vec_ok || (r & 7) != 0 || (r_eff & 7) != 0 || r_eff > 128) {
    const int n0 = group * kExpGroup;
    const int n_end = n0 + kExpGroup < p.feat_out ? n0 + kExpGroup : p.feat_out;
    expand_generic<T>(p, r, r_eff, base_li, scale, row0, m0, m_end - m0, n0, n_end - n0);
    return;
  }
  const int nb = group * kExpGroup + wave * kExpOB;
  // KS 32-wide steps cover max_rank (chosen on the host); a smaller adapter
  // rank leaves the upper fragments zero
  extern __shared__ __align__(16) char s_delta[];
  expand_mfma<T, KS>(p, r, r_eff, base_li, scale, row0, m0, m_end, nb, s_delta);
}

// The same work for batches of up to kExpReqs requests, shared out evenly: every
// workgroup of an output group gets the same number of row tiles, whatever the
// requests' lengths, and pays the lookups of a request (adapter, start, scale) once,
// from LDS.  Thread j describes request j (two dependent groups of loads, outside
// every branch); a prefix sum over the requests' tile counts lays them end to end;
// workgroup (group, slice) walks tiles [total * slice / slices, total * (slice + 1) / slices)
// of that line, request by request.
constexpr int kExpReqs = 256;

template <typename T, int KS, int NPROJ>
__global__ __launch_bounds__(kExpThreads) void sgmm_expand_walk_kernel(const SegExpandArgs p_all) {
  extern __shared__ __align__(16) char s_delta[];
  __shared__ int s_row0[kExpReqs], s_rows[kExpReqs], s_rank[kExpReqs], s_tile0[kExpReqs];
  __shared__ int64_t s_base[kExpReqs];
  __shared__ float s_scale[kExpReqs];
  __shared__ int s_wsum[kExpWaves];
  __shared__ int s_first;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int group = (int)blockIdx.x % p_all.n_chunks;
  const int slice = (int)blockIdx.x / p_all.n_chunks, slices = (int)gridDim.x / p_all.n_chunks;
  const SegExpandArgs p = expand_select<NPROJ>(p_all, group);

  // request tid: an invalid one re-reads entry 0 and gets no tiles
  const bool mine = tid < p.t.n_requests;
  const int rq = mine ? tid : 0;
  const int64_t a = p.t.b_indicies[rq];
  int row0 = p.t.b_start_loc[rq];
  int rows = p.t.b_seq_len[rq];
  const bool a_ok = (uint64_t)a < (uint64_t)p.t.n_adapters;
  const int64_t a_safe = a_ok ? a : 0;
  const int64_t len = p.t.a_len[a_safe];
  const int64_t start = p.t.a_start[a_safe];
  const float scale = load_scale(p.scales, p.scales_dtype, a_safe);
  const int r = (int)(len >> 2);
  const bool valid = mine && a_ok && row0 >= 0 && rows > 0 && row0 < p.t.n_tokens && r > 0 && p.max_rank > 0;
  if (valid) {
    if (rows > p.t.n_tokens - row0) rows = p.t.n_tokens - row0;
    if (rows > p.row_cap) rows = p.row_cap;
  } else {
    rows = 0;
  }
  const int tiles = (rows + kExpTMW - 1) / kExpTMW;
  int inc = tiles;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const int up = __shfl_up(inc, o, kWave);
    if (lane >= o) inc += up;
  }
  if (lane == kWave - 1) s_wsum[wave] = inc;
  if (tid == 0) s_first = 0;
  __syncthreads();
  int before = 0, total = 0;
#pragma unroll
  for (int wv = 0; wv < kExpWaves; ++wv) {
    const int c = s_wsum[wv];
    if (wv < wave) before += c;
    total += c;
  }
  const int tile0 = before + inc - tiles;  // tiles in front of my request
  const int t_begin = (int)((int64_t)total * slice / slices), t_end = (int)((int64_t)total * (slice + 1) / slices);
  s_row0[tid] = row0;
  s_rows[tid] = rows;
  s_rank[tid] = r;
  s_tile0[tid] = tile0;
  s_base[tid] = start + (int64_t)r * p.qkvo;
  s_scale[tid] = scale;
  if (tiles > 0 && t_begin >= tile0 && t_begin < tile0 + tiles) s_first = tid;
  __syncthreads();
  if (t_begin >= t_end) return;

  auto uni = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
  const int nb = group * kExpGroup + wave * kExpOB;
  int t = t_begin;
  for (int j = uni(s_first); t < t_end && j < p.t.n_requests; ++j) {
    const int rows_j = uni(s_rows[j]);
    const int tiles_j = (rows_j + kExpTMW - 1) / kExpTMW;
    const int tile0_j = uni(s_tile0[j]);
    if (tiles_j == 0 || t >= tile0_j + tiles_j) continue;
    const int last = t_end - tile0_j < tiles_j ? t_end - tile0_j : tiles_j;  // my tiles of request j: [t - tile0_j, last)
    const int m0 = (t - tile0_j) * kExpTMW;
    const int m_end = last * kExpTMW < rows_j ? last * kExpTMW : rows_j;
    t = tile0_j + last;
    const int rj = uni(s_rank[j]);
    const int r_eff = rj < p.max_rank ? rj : p.max_rank;
    const int rw0 = uni(s_row0[j]);
    const int64_t bl = s_base[j];
    const int64_t base_li =
        (int64_t)(((uint64_t)(uint32_t)uni((int)((uint64_t)bl >> 32)) << 32) | (uint32_t)uni((int)(uint32_t)bl));
    const float scale_j = __builtin_bit_cast(float, uni(__builtin_bit_cast(int, s_scale[j])));
    if (!p.vec_ok || (rj & 7) != 0 || (r_eff & 7) != 0 || r_eff > 128) {
      const int n0 = group * kExpGroup;
      const int n_end = n0 + kExpGroup < p.feat_out ? n0 + kExpGroup : p.feat_out;
      expand_generic<T>(p, rj, r_eff, base_li, scale_j, rw0, m0, m_end - m0, n0, n_end - n0);
    } else {
      expand_mfma<T, KS>(p, rj, r_eff, base_li, scale_j, rw0, m0, m_end, nb, s_delta);
    }
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
int fill_seg_tables(SegTables& t, const slora_tables* in, const int32_t* b_start_loc, const int32_t* b_seq_len,
                    const int64_t* b_indicies, int64_t n_requests, int64_t n_tokens, int64_t n_pages) {
  if (in == nullptr || in->a_start == nullptr || in->a_len == nullptr || in->a_loc == nullptr ||
      b_start_loc == nullptr || b_seq_len == nullptr || b_indicies == nullptr)
    return SLORA_ERR_NULL_POINTER;
  if (in->n_adapters < 0 || in->n_loc < 0 || n_pages < 0) return SLORA_ERR_BAD_SHAPE;
  if (n_pages == 0 && in->n_loc > 0) return SLORA_ERR_BAD_SHAPE;  // page ids, but no pool they could name
  if (n_requests > (1 << 24) || n_tokens > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
  t.a_start = in->a_start;
  t.a_len = in->a_len;
  t.a_loc = in->a_loc;
  t.b_start_loc = b_start_loc;
  t.b_seq_len = b_seq_len;
  t.b_indicies = b_indicies;
  t.n_adapters = in->n_adapters;
  t.n_loc = in->n_loc;
  t.n_pages = n_pages;
  t.n_requests = (int)n_requests;
  t.n_tokens = (int)n_tokens;
  return SLORA_OK;
}

// Workgroups of a shrink launch and how many of them share a tile's rank columns: at most
// one workgroup per 16-row unit and kShrMaxGrid.  A small batch leaves most of them without
// rows while each of the others streams all weight rows of its tile, so the rank columns of
// a tile are then shared by 2 or 4 workgroups: the split with the least estimated time of
// the slowest workgroup (14.2 us + per tile 0.2 us per weight row it reads + 0.177 us per
// row; further tiles 6.7 us each).  Batches beyond kShrDeepTokens are not split (they take the
// kernels that stream whole tiles through LDS).  grid = 0: nothing to do.
void shrink_geometry(int64_t n_tokens, int64_t n_requests, int64_t m_tiles, int64_t max_rank, int64_t& grid, int& cs) {
  grid = 0;
  cs = 1;
  int64_t units = (n_tokens + kShrUnit - 1) / kShrUnit + n_requests;
  const int64_t by_len = n_requests * m_tiles * kShrMF;
  if (by_len < units) units = by_len;
  if (units <= 0) return;
  float best = 0.f;
  for (int c = 1; c <= 4; c *= 2) {
    if (c > 1 && max_rank < 16 * c) break;  // fewer 16-column tiles than workgroups to share them
    if (c > 1 && n_tokens > kShrDeepTokens) break;  // such batches stream through the LDS ring, whole tiles per workgroup
    const int64_t row_parts = kShrMaxGrid / c;
    int64_t rows = (n_tokens + row_parts - 1) / row_parts;
    rows = (rows + kShrUnit - 1) / kShrUnit * kShrUnit;
    const float tiles = (float)((rows + kShrTM - 1) / kShrTM);
    const float t = 14.2f + tiles * (0.2f * (float)max_rank / (float)c) + (tiles - 1.f) * 6.7f + 0.177f * (float)rows;
    if (c == 1 || t < best) {
      best = t;
      cs = c;
    }
  }
  grid = (units * cs + 8 * cs - 1) / (8 * cs) * (8 * cs);
  if (grid > kShrMaxGrid) grid = kShrMaxGrid;
}

// a plan holds one record per row part: usable where no part spans two requests
bool shrink_plan_usable(int64_t n_requests, int64_t m_tiles, int64_t grid, int cs) {
  return grid > 0 && n_requests <= kShrChunk && n_requests <= grid / cs && m_tiles <= 1024;
}

// DEEP: the instantiation whose single-projection K loop keeps three blocks in flight (for
// launches with few workgroups, see shrink_k_loop_ring)
template <typename T, int NPROJ, bool DEEP, bool RING>
int launch_seg_shrink_kernel(const SegShrinkArgs& q, const int* plan, int64_t grid, size_t lds, hipStream_t stream) {
  const void* kernel = plan != nullptr ? reinterpret_cast<const void*>(sgmm_shrink_planned_kernel<T, NPROJ, DEEP, RING>)
                                       : reinterpret_cast<const void*>(sgmm_shrink_kernel<T, NPROJ, DEEP, RING>);
  static PerDeviceOnce once[2];
  if (!raise_dynamic_lds(kernel, (int)lds, once[plan != nullptr])) return SLORA_ERR_LAUNCH;
  if (plan != nullptr)
    hipLaunchKernelGGL((sgmm_shrink_planned_kernel<T, NPROJ, DEEP, RING>), dim3((uint32_t)grid), dim3(kShrThreads), lds,
                       stream, q, plan);
  else
    hipLaunchKernelGGL((sgmm_shrink_kernel<T, NPROJ, DEEP, RING>), dim3((uint32_t)grid), dim3(kShrThreads), lds, stream,
                       q);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

template <typename T, int NPROJ, bool DEEP>
int launch_seg_shrink(const SegShrinkArgs& p, const int* plan, hipStream_t stream) {
  int64_t grid = 0;
  SegShrinkArgs q = p;
  shrink_geometry(p.t.n_tokens, p.t.n_requests, p.m_tiles, p.max_rank, grid, q.col_split);
  if (grid <= 0) return SLORA_OK;
  if (plan != nullptr && !shrink_plan_usable(p.t.n_requests, p.m_tiles, grid, q.col_split)) return SLORA_ERR_BAD_SHAPE;
  // Large batches (every compute unit has a tile of its own) with whole 64-k blocks: the K loop through
  // the LDS ring.  Beyond kShrDeepTokens for q/k/v too, so that the fused launch stays bit for bit the
  // three calls.
  if constexpr (!DEEP) {
    const bool ring = p.t.n_tokens > kShrDeepTokens && q.col_split == 1 && p.vec_ok && (p.h_in & 63) == 0 && p.h_in >= 64;
    if (ring)
      return launch_seg_shrink_kernel<T, NPROJ, false, true>(q, plan, grid, kShrRingBytes + kShrOutBytes, stream);
  }
  return launch_seg_shrink_kernel<T, NPROJ, DEEP, false>(q, plan, grid, sizeof(float) * kShrWaves * kShrTM * kShrLd, stream);
}

template <typename T, int KS, int NPROJ>
int launch_seg_expand_ks(const SegExpandArgs& p, int64_t grid, hipStream_t stream) {
  const bool walk = p.t.n_requests <= kExpReqs && p.t.n_tokens <= (1 << 22);  // tile counts stay far inside 32 bits
  auto kernel = walk ? sgmm_expand_walk_kernel<T, KS, NPROJ> : sgmm_expand_kernel<T, KS, NPROJ>;
  constexpr int lds = 2 * kExpChunkRows * kExpLdsRow<KS>;  // 68 KiB for ranks up to 128
  static PerDeviceOnce once[2];
  if (lds > 64 * 1024 && !raise_dynamic_lds(reinterpret_cast<const void*>(kernel), lds, once[walk]))
    return SLORA_ERR_LAUNCH;
  if (walk) {
    // as many slices per output group as fill the chip, at most one per row tile
    const int64_t tiles = ((int64_t)p.t.n_tokens + kExpTMW - 1) / kExpTMW + p.t.n_requests;
    int64_t slices = (kExpWalkGrid<KS> + p.n_chunks - 1) / p.n_chunks;
    if (slices > tiles) slices = tiles;
    grid = slices * p.n_chunks;
  }
  hipLaunchKernelGGL(kernel, dim3((uint32_t)grid), dim3(kExpThreads), lds, stream, p);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

template <typename T>
int launch_seg_expand(const SegExpandArgs& p, hipStream_t stream) {
  const int64_t grid = (int64_t)p.t.n_requests * p.m_tiles * p.n_chunks;
  if (grid <= 0) return SLORA_OK;
  if (grid > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
  if (p.nproj == 3) {
    if (p.max_rank <= 32) return launch_seg_expand_ks<T, 1, 3>(p, grid, stream);
    if (p.max_rank <= 64) return launch_seg_expand_ks<T, 2, 3>(p, grid, stream);
    return launch_seg_expand_ks<T, 4, 3>(p, grid, stream);
  }
  if (p.max_rank <= 32) return launch_seg_expand_ks<T, 1, 1>(p, grid, stream);
  if (p.max_rank <= 64) return launch_seg_expand_ks<T, 2, 1>(p, grid, stream);
  return launch_seg_expand_ks<T, 4, 1>(p, grid, stream);
}

int seg_shrink_common(const int* plan, bool planned, void* const o[3], int nproj, const void* x, const void* w,
                      const slora_tables* tables,
                      const int32_t* b_start_loc, const int32_t* b_seq_len, const int64_t* b_indicies,
                      int64_t n_requests, int64_t max_input_len, int64_t n_tokens, int64_t h_in, int64_t max_rank,
                      int64_t x_row_stride, int64_t w_row_stride, int64_t o_row_stride, int64_t n_pages, int qkvo,
                      int dtype, void* stream) {
  if (dtype != SLORA_DTYPE_F16 && dtype != SLORA_DTYPE_BF16) return SLORA_ERR_BAD_DTYPE;
  if (n_requests < 0 || max_input_len < 0 || n_tokens < 0 || h_in < 0 || max_rank < 0) return SLORA_ERR_BAD_SHAPE;
  if (qkvo < 0 || qkvo + nproj > 4) return SLORA_ERR_BAD_SHAPE;
  if (x_row_stride < h_in || w_row_stride < h_in || o_row_stride < max_rank) return SLORA_ERR_BAD_SHAPE;
  if (n_requests == 0 || max_input_len == 0 || n_tokens == 0 || max_rank == 0) return SLORA_OK;
  SegShrinkArgs p{};
  int rc = fill_seg_tables(p.t, tables, b_start_loc, b_seq_len, b_indicies, n_requests, n_tokens, n_pages);
  if (rc != SLORA_OK) return rc;
  if (p.t.n_adapters == 0) return SLORA_OK;  // no request can name an adapter
  if (x == nullptr || w == nullptr) return SLORA_ERR_NULL_POINTER;
  for (int i = 0; i < nproj; ++i)
    if (o[i] == nullptr) return SLORA_ERR_NULL_POINTER;
  if (h_in == 0 || h_in > (1 << 21) || max_rank > SLORA_MAX_RANK) return SLORA_ERR_UNSUPPORTED;
  if (planned && (reinterpret_cast<uintptr_t>(plan) & 15) != 0) return SLORA_ERR_ALIGNMENT;
  if (max_input_len > n_tokens) max_input_len = n_tokens;  // no request is longer than the batch
  for (int i = 0; i < 3; ++i) p.o[i] = i < nproj ? o[i] : nullptr;
  p.nproj = nproj;
  p.x = x;
  p.w = w;
  p.x_stride = x_row_stride;
  p.w_stride = w_row_stride;
  p.o_stride = o_row_stride;
  p.h_in = (int)h_in;
  p.max_rank = (int)max_rank;
  p.qkvo = qkvo;
  p.m_tiles = (int)((max_input_len + kShrTM - 1) / kShrTM);
  p.col_split = 1;
  p.vec_ok = (h_in % 8 == 0) && (x_row_stride % 8 == 0) && (w_row_stride % 8 == 0) && aligned16(x) && aligned16(w);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (nproj == 3)
    return dtype == SLORA_DTYPE_F16 ? launch_seg_shrink<F16, 3, false>(p, plan, s)
                                    : launch_seg_shrink<BF16, 3, false>(p, plan, s);
  if (n_tokens <= kShrDeepTokens)
    return dtype == SLORA_DTYPE_F16 ? launch_seg_shrink<F16, 1, true>(p, plan, s)
                                    : launch_seg_shrink<BF16, 1, true>(p, plan, s);
  return dtype == SLORA_DTYPE_F16 ? launch_seg_shrink<F16, 1, false>(p, plan, s)
                                  : launch_seg_shrink<BF16, 1, false>(p, plan, s);
}

// One projection (nproj 1: o[0], x[0], feat_out[0], o_row_stride[0], any qkvo) or q, k and v in one
// launch (nproj 3, qkvo 0): the output groups of the three projections side by side in one grid.
int seg_expand_common(void* const o[3], const void* const x[3], int nproj, const void* w, const slora_tables* tables,
                      const void* scales, int scales_dtype, const int32_t* b_start_loc, const int32_t* b_seq_len,
                      const int64_t* b_indicies, int64_t n_requests, int64_t max_input_len, int64_t n_tokens,
                      const int64_t feat_out[3], int64_t page_elems, int64_t max_rank, int64_t x_row_stride,
                      int64_t w_row_stride, const int64_t o_row_stride[3], int64_t n_pages, int qkvo, int dtype,
                      void* stream) {
  if (dtype != SLORA_DTYPE_F16 && dtype != SLORA_DTYPE_BF16) return SLORA_ERR_BAD_DTYPE;
  if (scales_dtype != SLORA_DTYPE_F16 && scales_dtype != SLORA_DTYPE_BF16 && scales_dtype != SLORA_DTYPE_F32)
    return SLORA_ERR_BAD_DTYPE;
  if (n_requests < 0 || max_input_len < 0 || n_tokens < 0 || max_rank < 0 || page_elems < 0) return SLORA_ERR_BAD_SHAPE;
  for (int i = 0; i < nproj; ++i)
    if (feat_out[i] < 0) return SLORA_ERR_BAD_SHAPE;
  if (qkvo < 0 || qkvo + nproj > 4) return SLORA_ERR_BAD_SHAPE;
  if (page_elems == 0) page_elems = feat_out[0];  // the reference's convention: page width == output width
  if (x_row_stride < max_rank || w_row_stride < page_elems) return SLORA_ERR_BAD_SHAPE;
  int64_t feat_max = 0;
  for (int i = 0; i < nproj; ++i) {
    if (o_row_stride[i] < feat_out[i]) return SLORA_ERR_BAD_SHAPE;
    if (feat_out[i] > feat_max) feat_max = feat_out[i];
  }
  if (n_requests == 0 || max_input_len == 0 || n_tokens == 0 || max_rank == 0 || feat_max == 0) return SLORA_OK;
  if (max_input_len > n_tokens) max_input_len = n_tokens;  // no request is longer than the batch
  SegExpandArgs p{};
  int rc = fill_seg_tables(p.t, tables, b_start_loc, b_seq_len, b_indicies, n_requests, n_tokens, n_pages);
  if (rc != SLORA_OK) return rc;
  if (p.t.n_adapters == 0) return SLORA_OK;  // no request can name an adapter
  if (w == nullptr || scales == nullptr) return SLORA_ERR_NULL_POINTER;
  for (int i = 0; i < nproj; ++i)
    if (feat_out[i] > 0 && (o[i] == nullptr || x[i] == nullptr)) return SLORA_ERR_NULL_POINTER;
  if (feat_max > (1 << 21) || max_rank > SLORA_MAX_RANK || page_elems > (1LL << 30)) return SLORA_ERR_UNSUPPORTED;
  p.o = o[0];
  p.x = x[0];
  p.w = w;
  p.scales = scales;
  p.scales_dtype = scales_dtype;
  p.x_stride = x_row_stride;
  p.w_stride = w_row_stride;
  p.o_stride = o_row_stride[0];
  p.page_elems = page_elems;
  p.feat_out = (int)feat_out[0];
  p.max_rank = (int)max_rank;
  p.qkvo = qkvo;
  p.nproj = nproj;
  p.vec_ok = (page_elems % 8 == 0) && (x_row_stride % 8 == 0) && (w_row_stride % 8 == 0) && aligned16(w);
  int64_t chunks = 0;
  for (int i = 0; i < 3; ++i) {
    if (i < nproj) {
      chunks += (feat_out[i] + kExpGroup - 1) / kExpGroup;
      p.o3[i] = o[i];
      p.x3[i] = x[i];
      p.feat3[i] = (int)feat_out[i];
      p.o_stride3[i] = o_row_stride[i];
      if (feat_out[i] > 0)
        p.vec_ok = p.vec_ok && (feat_out[i] % 8 == 0) && (o_row_stride[i] % 8 == 0) && aligned16(o[i]) && aligned16(x[i]);
    }
    p.chunk_end[i] = (int)chunks;
  }
  p.n_chunks = (int)chunks;
  // rows a workgroup walks: up to kExpSpanTiles tiles, fewer while that leaves the chip short of workgroups
  int64_t tiles = kExpSpanTiles;
  while (tiles > 1 &&
         n_requests * ((max_input_len + kExpTMW * tiles - 1) / (kExpTMW * tiles)) * p.n_chunks < kExpMinGrid)
    tiles >>= 1;
  p.m_span = (int)(kExpTMW * tiles);
  p.row_cap = max_input_len > (1 << 30) ? (1 << 30) : (int)((max_input_len + kExpTMW - 1) / kExpTMW * kExpTMW);
  p.m_tiles = (int)((max_input_len + p.m_span - 1) / p.m_span);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  return dtype == SLORA_DTYPE_F16 ? launch_seg_expand<F16>(p, s) : launch_seg_expand<BF16>(p, s);
}

}  // namespace
}  // namespace slora

extern "C" {

int slora_sgmm_shrink(void* o, const void* x, const void* w, const slora_tables* tables, const int32_t* b_start_loc,
                      const int32_t* b_seq_len, const int64_t* b_indicies, int64_t n_requests, int64_t max_input_len,
                      int64_t n_tokens, int64_t h_in, int64_t max_rank, int64_t x_row_stride, int64_t w_row_stride,
                      int64_t o_row_stride, int64_t n_pages, int qkvo, int dtype, void* stream) {
  void* const os[3] = {o, nullptr, nullptr};
  return slora::seg_shrink_common(nullptr, false, os, 1, x, w, tables, b_start_loc, b_seq_len, b_indicies, n_requests,
                                  max_input_len, n_tokens, h_in, max_rank, x_row_stride, w_row_stride, o_row_stride,
                                  n_pages, qkvo, dtype, stream);
}

int64_t slora_sgmm_plan_bytes(void) {
  return (int64_t)sizeof(int) * (slora::kSegPlanHeaderWords + slora::kShrMaxGrid * slora::kSegPartWords);
}

int slora_sgmm_plan_build(void* plan, int64_t plan_bytes, const slora_tables* tables, const int32_t* b_start_loc,
                          const int32_t* b_seq_len, const int64_t* b_indicies, int64_t n_requests,
                          int64_t max_input_len, int64_t n_tokens, int64_t max_rank, int* usable, void* stream) {
  using namespace slora;
  if (usable == nullptr) return SLORA_ERR_NULL_POINTER;
  *usable = 0;
  if (n_requests < 0 || max_input_len < 0 || n_tokens < 0 || max_rank < 0) return SLORA_ERR_BAD_SHAPE;
  if (plan == nullptr) return SLORA_ERR_NULL_POINTER;
  if (plan_bytes < slora_sgmm_plan_bytes()) return SLORA_ERR_BAD_SHAPE;
  if ((reinterpret_cast<uintptr_t>(plan) & 15) != 0) return SLORA_ERR_ALIGNMENT;
  if (max_rank > SLORA_MAX_RANK) return SLORA_ERR_UNSUPPORTED;
  if (n_requests == 0 || max_input_len == 0 || n_tokens == 0 || max_rank == 0) return SLORA_OK;
  SegTables t{};
  int rc = fill_seg_tables(t, tables, b_start_loc, b_seq_len, b_indicies, n_requests, n_tokens, 1);
  if (rc != SLORA_OK) return rc;
  if (t.n_adapters == 0) return SLORA_OK;
  if (max_input_len > n_tokens) max_input_len = n_tokens;
  const int64_t m_tiles = (max_input_len + kShrTM - 1) / kShrTM;
  int64_t grid = 0;
  int cs = 1;
  shrink_geometry(n_tokens, n_requests, m_tiles, max_rank, grid, cs);
  if (!shrink_plan_usable(n_requests, m_tiles, grid, cs)) return SLORA_OK;
  hipLaunchKernelGGL(sgmm_plan_kernel, dim3(1), dim3(kShrThreads), 0, reinterpret_cast<hipStream_t>(stream),
                     static_cast<int*>(plan), t, (int)(grid / cs), cs, (int)max_rank, (int)(m_tiles * kShrTM));
  if (hipGetLastError() != hipSuccess) return SLORA_ERR_LAUNCH;
  *usable = 1;
  return SLORA_OK;
}

int slora_sgmm_shrink_planned(const void* plan, void* o, const void* x, const void* w, const slora_tables* tables,
                              const int32_t* b_start_loc, const int32_t* b_seq_len, const int64_t* b_indicies,
                              int64_t n_requests, int64_t max_input_len, int64_t n_tokens, int64_t h_in,
                              int64_t max_rank, int64_t x_row_stride, int64_t w_row_stride, int64_t o_row_stride,
                              int64_t n_pages, int qkvo, int dtype, void* stream) {
  if (plan == nullptr) return SLORA_ERR_NULL_POINTER;
  void* const os[3] = {o, nullptr, nullptr};
  return slora::seg_shrink_common(static_cast<const int*>(plan), true, os, 1, x, w, tables, b_start_loc, b_seq_len,
                                  b_indicies, n_requests, max_input_len, n_tokens, h_in, max_rank, x_row_stride,
                                  w_row_stride, o_row_stride, n_pages, qkvo, dtype, stream);
}

int slora_sgmm_shrink_qkv(const void* plan, void* o_q, void* o_k, void* o_v, const void* x, const void* w,
                          const slora_tables* tables, const int32_t* b_start_loc, const int32_t* b_seq_len,
                          const int64_t* b_indicies, int64_t n_requests, int64_t max_input_len, int64_t n_tokens,
                          int64_t h_in, int64_t max_rank, int64_t x_row_stride, int64_t w_row_stride,
                          int64_t o_row_stride, int64_t n_pages, int dtype, void* stream) {
  void* const os[3] = {o_q, o_k, o_v};
  return slora::seg_shrink_common(static_cast<const int*>(plan), plan != nullptr, os, 3, x, w, tables, b_start_loc,
                                  b_seq_len, b_indicies, n_requests, max_input_len, n_tokens, h_in, max_rank,
                                  x_row_stride, w_row_stride, o_row_stride, n_pages, 0, dtype, stream);
}

int slora_sgmm_expand(void* o, const void* x, const void* w, const slora_tables* tables, const void* scales,
                      int scales_dtype, const int32_t* b_start_loc, const int32_t* b_seq_len,
                      const int64_t* b_indicies, int64_t n_requests, int64_t max_input_len, int64_t n_tokens,
                      int64_t feat_out, int64_t page_elems, int64_t max_rank, int64_t x_row_stride,
                      int64_t w_row_stride, int64_t o_row_stride, int64_t n_pages, int qkvo, int dtype,
                      void* stream) {
  void* const os[3] = {o, nullptr, nullptr};
  const void* const xs[3] = {x, nullptr, nullptr};
  const int64_t feats[3] = {feat_out, 0, 0}, o_strides[3] = {o_row_stride, 0, 0};
  return slora::seg_expand_common(os, xs, 1, w, tables, scales, scales_dtype, b_start_loc, b_seq_len, b_indicies,
                                  n_requests, max_input_len, n_tokens, feats, page_elems, max_rank, x_row_stride,
                                  w_row_stride, o_strides, n_pages, qkvo, dtype, stream);
}

int slora_sgmm_expand_qkv(void* o_q, void* o_k, void* o_v, const void* x_q, const void* x_k, const void* x_v,
                          const void* w, const slora_tables* tables, const void* scales, int scales_dtype,
                          const int32_t* b_start_loc, const int32_t* b_seq_len, const int64_t* b_indicies,
                          int64_t n_requests, int64_t max_input_len, int64_t n_tokens, int64_t feat_out_q,
                          int64_t feat_out_kv, int64_t page_elems, int64_t max_rank, int64_t x_row_stride,
                          int64_t w_row_stride, int64_t o_row_stride_q, int64_t o_row_stride_kv, int64_t n_pages,
                          int dtype, void* stream) {
  void* const os[3] = {o_q, o_k, o_v};
  const void* const xs[3] = {x_q, x_k, x_v};
  const int64_t feats[3] = {feat_out_q, feat_out_kv, feat_out_kv};
  const int64_t o_strides[3] = {o_row_stride_q, o_row_stride_kv, o_row_stride_kv};
  return slora::seg_expand_common(os, xs, 3, w, tables, scales, scales_dtype, b_start_loc, b_seq_len, b_indicies,
                                  n_requests, max_input_len, n_tokens, feats, page_elems, max_rank, x_row_stride,
                                  w_row_stride, o_strides, n_pages, 0, dtype, stream);
}

}  // extern "C"
