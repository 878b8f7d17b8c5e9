// Moving adapters in and out of the unified paged pool: the producers of every
// byte the LoRA kernels read.
//
//   slora_pool_scatter_rows   pool[loc[i]] = rows[i] for several pool buffers at once
//                             (slora/server/router/model_infer/infer_adapter.py:56-57,
//                             81-82: `key_buffer[l][loc] = w_combined[0]`, one
//                             index_put per layer and side in the reference)
//   slora_var_len_copy        new_loc[new_start[i] + k] = old_loc[old_start[i] + k]
//                             (infer_adapter.py:261-280, launch_var_len_copy_triton)
//   slora_tables_compact      the index tables after some adapters are dropped, and the
//                             page ids they give back (infer_adapter.py:186-258)
//
//   slora_pool_gather_a       A_p as a dense (hidden, rank) matrix out of its r pool pages
//                             (slora/models/peft/lora_single_batch_infer.py:38-46), the
//                             left operand of merging an adapter into the base weights
//   slora_pool_alloc / slora_pool_alloc_contiguous / slora_pool_free
//                             the page allocator over the pool's free map
//                             (slora/common/mem_allocator.py:30-59, 185-199)
//
// All of it is plain byte/integer movement, bound by HBM bandwidth (the first) or
// by a handful of dependent round trips (the rest).

#include <mutex>

#include "common.hpp"
#include "cabi_util.hpp"

namespace slora {
namespace {

// ---------------------------------------------------------------------------
// workspace of slora_pool_alloc_contiguous_static
// ---------------------------------------------------------------------------
// The allocator's workspace (best start, per-workgroup free counts and last used
// pages) for maps of up to kStaticMapPages pages, held by every GPU the library
// runs on until the process ends.  In host code the array's name is only a
// handle: the address the kernels get comes from hipGetSymbolAddress, once per
// device, with that device current (every GPU has its own copy at its own
// address).
constexpr int64_t kStaticMapPages = int64_t(1) << 24;  // 16 Mi pages: 128 GiB of 8 KiB pages
constexpr int64_t kStaticMapBlocks = kStaticMapPages / (256 * 16);
constexpr int64_t kStaticScratchBytes = 16 + kStaticMapBlocks * 4 + 8 + kStaticMapBlocks * 8;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices];  // per device: the address of `scratch` there, nullptr = not asked yet

// the current device's copy of `scratch`, or nullptr if the runtime cannot name it
void* static_scratch() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

// ---------------------------------------------------------------------------
// scatter rows into pool pages
// ---------------------------------------------------------------------------
constexpr int kScatterBufs = 64;  // pool buffers served by one launch (pointers travel as kernel arguments)

struct ScatterArgs {
  void* dst[kScatterBufs];
  const void* src[kScatterBufs];
  const int64_t* loc;
  int64_t n_rows, n_pages;
  int64_t row_bytes, dst_stride, src_stride;  // bytes
  int n_bufs;
  int vec_ok;  // rows, strides and bases are multiples of 16 bytes
};

// One workgroup per (row, buffer): buffer-fastest, so the few workgroups that
// read the same loc entry run together.  A row of 8 KiB is two 16-byte loads and
// stores per lane, all loads issued before the stores.
__global__ __launch_bounds__(256) void pool_scatter_kernel(const ScatterArgs p) {
  const int64_t row = blockIdx.x / p.n_bufs;
  const int buf = (int)(blockIdx.x - row * p.n_bufs);
  const int64_t page = p.loc[row];
  if ((uint64_t)page >= (uint64_t)p.n_pages) return;  // a page id outside the pool is skipped, not written
  const char* s = static_cast<const char*>(p.src[buf]) + row * p.src_stride;
  char* d = static_cast<char*>(p.dst[buf]) + page * p.dst_stride;
  if (p.vec_ok) {
    const int64_t nvec = p.row_bytes >> 4;
    for (int64_t v0 = 0; v0 < nvec; v0 += 4 * 256) {
      u32x4 t[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t v = v0 + u * 256 + threadIdx.x;
        t[u] = ldg16_stream(s + ((v < nvec ? v : 0) << 4));
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t v = v0 + u * 256 + threadIdx.x;
        if (v < nvec) stg16_stream(d + (v << 4), t[u]);
      }
    }
  } else {
    for (int64_t b = threadIdx.x; b < p.row_bytes; b += 256) d[b] = s[b];
  }
}

// ---------------------------------------------------------------------------
// pack one adapter's matrices straight into its pool pages
// ---------------------------------------------------------------------------
// The adapter loader of the reference first builds w_combined on the host
// (slora/models/peft/layer_weights/lora_layer_weight.py:84-93: A_p^T as r rows of hidden
// elements, and the (h_out, r) row-major B_p^T cut into r rows) and then index_puts its rows
// into the pool (infer_adapter.py:56-57, 81-82).  Both halves are the same operation: a
// (rows x cols) row-major source matrix -- A_p is (hidden x r), B_p is (r x h_out) -- is
// written transposed, as the (cols x rows) matrix whose rows are dst_pitch elements apart,
// end to end over the pool pages loc[first .. first + n_slot): element (c, k) goes to flat
// position c * dst_pitch + k, page flat / page_elems, offset flat % page_elems.  A_p uses
// dst_pitch = page_elems (every column of A_p gets a page of its own), B_p uses dst_pitch =
// rows (= r: dense).  Positions of the slot that no source element reaches are zeroed, as
// index_put of the zero-padded w_combined would leave them.
constexpr int kPackMats = 64;  // matrices per launch (their descriptions travel as kernel arguments)

struct PackEntry {
  void* dst;        // pool buffer
  const void* src;  // (rows x cols) row-major, 16-bit elements
  int64_t first;    // index of the slot's first page id in loc
  int rows, cols, dst_pitch, n_slot;
};
struct PackArgs {
  PackEntry m[kPackMats];
  const int64_t* loc;
  int64_t n_loc, n_pages, page_elems;
  int n_mats, tiles_k;  // tiles_k: 64-wide tiles along k the grid provides per 64 columns
};

// 64 x 64 tiles through LDS: the source is read along its rows (cols contiguous), the
// pages are written along k (contiguous).
__global__ __launch_bounds__(256) void pool_pack_kernel(const PackArgs p) {
  __shared__ uint16_t s_t[64][66];
  const PackEntry e = p.m[blockIdx.y];
  const int tile_c = (int)blockIdx.x / p.tiles_k, tile_k = (int)blockIdx.x - tile_c * p.tiles_k;
  const int c0 = tile_c * 64, k0 = tile_k * 64;
  const int64_t slot_elems = (int64_t)e.n_slot * p.page_elems;
  if (k0 >= e.dst_pitch || (int64_t)c0 * e.dst_pitch >= slot_elems) return;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
  const uint16_t* src = static_cast<const uint16_t*>(e.src);
  for (int kk = ty; kk < 64; kk += 4) {
    const int k = k0 + kk, c = c0 + tx;
    s_t[kk][tx] = (k < e.rows && c < e.cols) ? src[(int64_t)k * e.cols + c] : (uint16_t)0;
  }
  __syncthreads();
  uint16_t* dst = static_cast<uint16_t*>(e.dst);
  for (int cc = ty; cc < 64; cc += 4) {
    const int c = c0 + cc, k = k0 + tx;
    if (k >= e.dst_pitch) continue;
    const int64_t flat = (int64_t)c * e.dst_pitch + k;
    if (flat >= slot_elems) continue;
    const int64_t pg = flat / p.page_elems, off = flat - pg * p.page_elems;
    const int64_t li = e.first + pg;
    if ((uint64_t)li >= (uint64_t)p.n_loc) continue;
    const int64_t page = p.loc[li];
    if ((uint64_t)page >= (uint64_t)p.n_pages) continue;  // a page id outside the pool is skipped
    dst[page * p.page_elems + off] = s_t[tx][cc];
  }
}

// ---------------------------------------------------------------------------
// variable-length copy of page-id lists
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void var_len_copy_kernel(const int64_t* __restrict__ old_start,
                                                           const int64_t* __restrict__ len,
                                                           const int64_t* __restrict__ old_loc,
                                                           const int64_t* __restrict__ new_start,
                                                           int64_t* __restrict__ new_loc, int64_t n_old_loc,
                                                           int64_t n_new_loc) {
  const int64_t i = blockIdx.x;
  const int64_t n = len[i], os = old_start[i], ns = new_start[i];
  if (n <= 0 || os < 0 || ns < 0 || os > n_old_loc - n || ns > n_new_loc - n) return;  // a list outside its table is skipped
  for (int64_t k = threadIdx.x; k < n; k += 256) new_loc[ns + k] = old_loc[os + k];
}

// ---------------------------------------------------------------------------
// table compaction
// ---------------------------------------------------------------------------
constexpr int kCompactThreads = 1024;
constexpr int kCompactWaves = kCompactThreads / kWave;

// inclusive prefix sums of two values over the workgroup, totals returned through tot_*
__device__ __forceinline__ void compact_scan2(int64_t& a, int64_t& b, int64_t* s_a, int64_t* s_b, int64_t& tot_a,
                                              int64_t& tot_b) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const int64_t ua = __shfl_up(a, o, kWave), ub = __shfl_up(b, o, kWave);
    if (lane >= o) {
      a += ua;
      b += ub;
    }
  }
  if (lane == kWave - 1) {
    s_a[wave] = a;
    s_b[wave] = b;
  }
  __syncthreads();
  int64_t ba = 0, bb = 0;
  tot_a = 0;
  tot_b = 0;
  for (int wv = 0; wv < kCompactWaves; ++wv) {
    if (wv < wave) {
      ba += s_a[wv];
      bb += s_b[wv];
    }
    tot_a += s_a[wv];
    tot_b += s_b[wv];
  }
  __syncthreads();
  a += ba;
  b += bb;
}

struct CompactArgs {
  const int64_t* a_start;
  const int64_t* a_len;
  const int64_t* a_loc;
  const void* a_scaling;
  const uint8_t* keep;
  int64_t* new_start;
  int64_t* new_len;
  int64_t* new_loc;
  void* new_scaling;
  int64_t* removed;
  int64_t* counts;  // [4]: kept adapters, kept page ids, dropped adapters, dropped page ids
  int64_t* work;    // [n_adapters] destination offset of every adapter's list
  int64_t n_adapters, n_loc;
  int scale_bytes;
};

// One workgroup.  Pass 1 (a thread per adapter, 1024 at a time with running
// totals): kept adapters are numbered in order and get the running sum of kept
// lengths as their new start; dropped adapters get their offset in the list of
// returned page ids.  Pass 2 (a wavefront per adapter): the lists are copied,
// lanes over consecutive entries.
__global__ __launch_bounds__(kCompactThreads) void tables_compact_kernel(const CompactArgs p) {
  __shared__ int64_t s_a[kCompactWaves], s_b[kCompactWaves];
  const int tid = threadIdx.x;
  int64_t kept = 0, kept_loc = 0, dropped = 0, dropped_loc = 0;
  for (int64_t i0 = 0; i0 < p.n_adapters; i0 += kCompactThreads) {
    const int64_t i = i0 + tid;
    const bool in = i < p.n_adapters;
    int64_t len = in ? p.a_len[i] : 0;
    const int64_t start = in ? p.a_start[i] : 0;
    const bool k = in && p.keep[i] != 0;
    if (len < 0 || start < 0 || start > p.n_loc - len) len = 0;  // a list outside a_loc counts as empty
    // kept: (count, length) ; dropped: (count, length) -- two scans
    int64_t kc = k ? 1 : 0, kl = k ? len : 0, tkc, tkl;
    compact_scan2(kc, kl, s_a, s_b, tkc, tkl);
    int64_t dc = (in && !k) ? 1 : 0, dl = (in && !k) ? len : 0, tdc, tdl;
    compact_scan2(dc, dl, s_a, s_b, tdc, tdl);
    if (in) {
      if (k) {
        const int64_t idx = kept + kc - 1, off = kept_loc + kl - len;
        p.new_start[idx] = off;
        p.new_len[idx] = len;
        if (p.scale_bytes == 2)
          static_cast<uint16_t*>(p.new_scaling)[idx] = static_cast<const uint16_t*>(p.a_scaling)[i];
        else
          static_cast<uint32_t*>(p.new_scaling)[idx] = static_cast<const uint32_t*>(p.a_scaling)[i];
        p.work[i] = off;
      } else {
        p.work[i] = dropped_loc + dl - len;
      }
    }
    kept += tkc;
    kept_loc += tkl;
    dropped += tdc;
    dropped_loc += tdl;
  }
  if (tid == 0) {
    p.counts[0] = kept;
    p.counts[1] = kept_loc;
    p.counts[2] = dropped;
    p.counts[3] = dropped_loc;
  }
  __threadfence_block();
  __syncthreads();  // work[] written above is read by other wavefronts below
  const int lane = tid & 63, wave = tid >> 6;
  for (int64_t i = wave; i < p.n_adapters; i += kCompactWaves) {
    int64_t len = p.a_len[i];
    const int64_t start = p.a_start[i];
    if (len < 0 || start < 0 || start > p.n_loc - len) len = 0;
    int64_t* dst = (p.keep[i] != 0 ? p.new_loc : p.removed) + p.work[i];
    for (int64_t e = lane; e < len; e += kWave) dst[e] = p.a_loc[start + e];
  }
}


// ---------------------------------------------------------------------------
// A_p out of the pool: out[k, d] = pool[loc[first + d]][k]
// ---------------------------------------------------------------------------
// 64 x 64 tiles through LDS: pages are read along k (contiguous), the dense
// matrix is written along d (contiguous).  Columns r .. out_cols are zero.
__global__ __launch_bounds__(256) void gather_a_kernel(const uint16_t* __restrict__ pool, int64_t page_elems,
                                                       int64_t n_pages, const int64_t* __restrict__ loc,
                                                       int64_t n_loc, int64_t first, int r, int h,
                                                       uint16_t* __restrict__ out, int out_cols) {
  __shared__ uint16_t s_t[64][66];
  const int k0 = blockIdx.x * 64, d0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
  for (int dd = ty; dd < 64; dd += 4) {
    const int d = d0 + dd, k = k0 + tx;
    uint16_t v = 0;
    if (d < r && k < h && (uint64_t)(first + d) < (uint64_t)n_loc) {
      const int64_t page = loc[first + d];
      if ((uint64_t)page < (uint64_t)n_pages) v = pool[page * page_elems + k];
    }
    s_t[dd][tx] = v;
  }
  __syncthreads();
  for (int kk = ty; kk < 64; kk += 4) {
    const int k = k0 + kk, d = d0 + tx;
    if (k < h && d < out_cols) out[(int64_t)k * out_cols + d] = s_t[tx][kk];
  }
}

// ---------------------------------------------------------------------------
// checksum of pool pages: out[i] = xor of the 32-bit words of page loc[i].  One wavefront
// per page, 16-byte loads, nothing else: the plainest read of scattered pages there is,
// which makes its duration the streaming ceiling the LoRA kernels are measured against.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void page_xor_kernel(const u32x4* __restrict__ pool, int64_t page_vecs,
                                                       int64_t n_pages, const int64_t* __restrict__ loc, int64_t n,
                                                       uint32_t* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (i >= n) return;
  const int64_t page = loc[i];
  u32x4 acc = zero16();
  if ((uint64_t)page < (uint64_t)n_pages) {
    const u32x4* src = pool + page * page_vecs;
    for (int64_t v0 = 0; v0 < page_vecs; v0 += 8 * kWave) {
      u32x4 v[8];
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const int64_t k = v0 + c * kWave + lane;
        v[c] = k < page_vecs ? ldg16_stream(src + k) : zero16();
      }
#pragma unroll
      for (int c = 0; c < 8; ++c) acc ^= v[c];
    }
  }
  uint32_t r = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) r ^= (uint32_t)__shfl_xor((int)r, o, kWave);
  if (lane == 0) out[i] = r;
}

// The same walk with a write: every 32-bit word of page loc[i] is xor-ed with `key` in place
// (key 0 leaves the data as it is and still reads and writes every byte).  One wavefront per
// page, all loads of a pass issued before the first store: the plainest read-modify-write of
// scattered rows, timed by the benchmark as the floor of the kernels that update an output in
// place (the expand kernels' y).
__global__ __launch_bounds__(256) void page_rmw_kernel(u32x4* __restrict__ pool, int64_t page_vecs, int64_t n_pages,
                                                       const int64_t* __restrict__ loc, int64_t n, uint32_t key) {
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (i >= n) return;
  const int64_t page = loc[i];
  if ((uint64_t)page >= (uint64_t)n_pages) return;
  u32x4* row = pool + page * page_vecs;
  for (int64_t v0 = 0; v0 < page_vecs; v0 += 8 * kWave) {
    u32x4 v[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int64_t k = v0 + c * kWave + lane;
      v[c] = k < page_vecs ? ldg16_stream(row + k) : zero16();
    }
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int64_t k = v0 + c * kWave + lane;
      if (k < page_vecs) stg16_stream(row + k, v[c] ^ u32x4{key, key, key, key});
    }
  }
}

// ---------------------------------------------------------------------------
// page allocator over the free map (1 byte per page, 1 = free)
// ---------------------------------------------------------------------------
constexpr int kMapThreads = 256;
constexpr int kMapPerThread = 16;                            // one 16-byte load of the map per thread
constexpr int kMapBlock = kMapThreads * kMapPerThread;       // pages per workgroup
constexpr int kMapWaves = kMapThreads / kWave;

// the 16 map bytes of this thread (0 beyond the end), as 0/1 flags
__device__ __forceinline__ void map_load16(const uint8_t* __restrict__ map, int64_t tot, int64_t base, int (&f)[16],
                                           bool vec) {
  if (vec && base + 16 <= tot) {
    const u32x4 v = ldg16(map + base);
#pragma unroll
    for (int i = 0; i < 16; ++i) f[i] = ((v[i >> 2] >> ((i & 3) * 8)) & 0xffu) != 0 ? 1 : 0;
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) f[i] = (base + i < tot && map[base + i] != 0) ? 1 : 0;
  }
}

// workgroup b: number of free pages, and (for the contiguous search) the index of its
// last used page (-1: none), into block_free[b] / block_last_used[b]
__global__ __launch_bounds__(kMapThreads) void map_block_stats_kernel(const uint8_t* __restrict__ map, int64_t tot,
                                                                      int* __restrict__ block_free,
                                                                      int64_t* __restrict__ block_last_used, int vec) {
  __shared__ int s_cnt[kMapWaves];
  __shared__ long long s_last[kMapWaves];
  const int64_t base = (int64_t)blockIdx.x * kMapBlock + (int64_t)threadIdx.x * kMapPerThread;
  int f[16];
  map_load16(map, tot, base, f, vec != 0);
  int cnt = 0;
  long long last = -1;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    cnt += f[i];
    if (!f[i] && base + i < tot) last = base + i;
  }
  for (int o = 32; o > 0; o >>= 1) {
    cnt += __shfl_xor(cnt, o, kWave);
    const long long ol = __shfl_xor(last, o, kWave);
    last = ol > last ? ol : last;
  }
  if ((threadIdx.x & 63) == 0) {
    s_cnt[threadIdx.x >> 6] = cnt;
    s_last[threadIdx.x >> 6] = last;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int c = 0;
    long long l = -1;
    for (int w = 0; w < kMapWaves; ++w) {
      c += s_cnt[w];
      l = s_last[w] > l ? s_last[w] : l;
    }
    block_free[blockIdx.x] = c;
    if (block_last_used != nullptr) block_last_used[blockIdx.x] = l;
  }
}

// `mem_cum_sum <= need_size and mem_state == 1` (mem_allocator.py:34-38): the free
// pages whose rank among the free pages is <= need, in index order, are written to
// out[rank - 1] and marked used.  result[0] = pages handed out.
__global__ __launch_bounds__(kMapThreads) void map_alloc_kernel(uint8_t* __restrict__ map, int64_t tot, int64_t need,
                                                                const int* __restrict__ block_free, int n_blocks,
                                                                int64_t* __restrict__ out, int64_t* __restrict__ result,
                                                                int vec) {
  __shared__ long long s_part[kMapWaves];
  __shared__ int s_scan[kMapWaves];
  // free pages in front of this workgroup, and in total
  long long before = 0, total = 0;
  for (int b = threadIdx.x; b < n_blocks; b += kMapThreads) {
    const int c = block_free[b];
    if (b < (int)blockIdx.x) before += c;
    total += c;
  }
  for (int o = 32; o > 0; o >>= 1) {
    before += __shfl_xor(before, o, kWave);
    total += __shfl_xor(total, o, kWave);
  }
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = before;
  __syncthreads();
  before = 0;
  for (int w = 0; w < kMapWaves; ++w) before += s_part[w];
  __syncthreads();
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = total;
  __syncthreads();
  total = 0;
  for (int w = 0; w < kMapWaves; ++w) total += s_part[w];
  if (blockIdx.x == 0 && threadIdx.x == 0) result[0] = total < need ? total : need;
  if (before >= need) return;  // uniform

  const int64_t base = (int64_t)blockIdx.x * kMapBlock + (int64_t)threadIdx.x * kMapPerThread;
  int f[16];
  map_load16(map, tot, base, f, vec != 0);
  int mine = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) mine += f[i];
  // exclusive scan of `mine` over the workgroup
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int inc = mine;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const int up = __shfl_up(inc, o, kWave);
    if (lane >= o) inc += up;
  }
  if (lane == kWave - 1) s_scan[wave] = inc;
  __syncthreads();
  long long rank = before + inc - mine;  // free pages in front of this thread's first page
  for (int w = 0; w < wave; ++w) rank += s_scan[w];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    if (f[i]) {
      ++rank;
      if (rank <= need) {
        out[rank - 1] = base + i;
        map[base + i] = 0;
      }
    }
  }
}

// First start s with pages [s, s + need) all free (mem_allocator.py:45-52).  A page i
// ends such a window iff the nearest used page at or before i lies before i - need + 1.
// Every workgroup takes the last used page in front of it from block_last_used, scans
// its own pages and proposes the smallest start it sees with a 64-bit atomic min.
__global__ __launch_bounds__(kMapThreads) void map_find_run_kernel(const uint8_t* __restrict__ map, int64_t tot,
                                                                   int64_t need,
                                                                   const int64_t* __restrict__ block_last_used,
                                                                   unsigned long long* __restrict__ best, int vec) {
  __shared__ long long s_last[kMapWaves];
  long long prev = -1;  // last used page in front of this workgroup
  for (int b = threadIdx.x; b < (int)blockIdx.x; b += kMapThreads) {
    const long long l = block_last_used[b];
    prev = l > prev ? l : prev;
  }
  for (int o = 32; o > 0; o >>= 1) {
    const long long ol = __shfl_xor(prev, o, kWave);
    prev = ol > prev ? ol : prev;
  }
  if ((threadIdx.x & 63) == 0) s_last[threadIdx.x >> 6] = prev;
  __syncthreads();
  prev = -1;
  for (int w = 0; w < kMapWaves; ++w) prev = s_last[w] > prev ? s_last[w] : prev;
  __syncthreads();

  const int64_t base = (int64_t)blockIdx.x * kMapBlock + (int64_t)threadIdx.x * kMapPerThread;
  int f[16];
  map_load16(map, tot, base, f, vec != 0);
  long long mine = -1;  // last used page among this thread's pages
#pragma unroll
  for (int i = 0; i < 16; ++i)
    if (!f[i] && base + i < tot) mine = base + i;
  // inclusive max-scan over the workgroup, then shifted to "in front of this thread"
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  long long run = mine;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const long long up = __shfl_up(run, o, kWave);
    if (lane >= o) run = up > run ? up : run;
  }
  if (lane == kWave - 1) s_last[wave] = run;
  __syncthreads();
  long long front = __shfl_up(run, 1, kWave);
  if (lane == 0) front = -1;
  front = front > prev ? front : prev;
  for (int w = 0; w < wave; ++w) front = s_last[w] > front ? s_last[w] : front;
  long long last_used = front;
  unsigned long long cand = ~0ull;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const long long idx = base + i;
    if (idx < tot) {
      if (!f[i]) last_used = idx;
      const long long start = idx - need + 1;
      if (f[i] && start >= 0 && last_used < start && (unsigned long long)start < cand) cand = (unsigned long long)start;
    }
  }
  for (int o = 32; o > 0; o >>= 1) {
    const unsigned long long oc = __shfl_xor(cand, o, kWave);
    cand = oc < cand ? oc : cand;
  }
  if (lane == 0 && cand != ~0ull) atomicMin(best, cand);
}

// pages [*best, *best + need) are marked used and listed; result = {start or -1, pages}
__global__ __launch_bounds__(kMapThreads) void map_take_run_kernel(uint8_t* __restrict__ map, int64_t tot, int64_t need,
                                                                   const unsigned long long* __restrict__ best,
                                                                   int64_t* __restrict__ out,
                                                                   int64_t* __restrict__ result) {
  const unsigned long long b = *best;
  const bool found = b != ~0ull && (long long)b + need <= tot;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    result[0] = found ? (int64_t)b : -1;
    result[1] = found ? need : 0;
  }
  if (!found) return;
  for (int64_t k = (int64_t)blockIdx.x * kMapThreads + threadIdx.x; k < need; k += (int64_t)gridDim.x * kMapThreads) {
    out[k] = (int64_t)b + k;
    map[(int64_t)b + k] = 0;
  }
}

__global__ __launch_bounds__(256) void map_init_best_kernel(unsigned long long* best) { *best = ~0ull; }

// mem_state[free_index] = 1 (mem_allocator.py:185-199); ids outside the map are skipped
__global__ __launch_bounds__(256) void map_free_kernel(uint8_t* __restrict__ map, int64_t tot,
                                                       const int64_t* __restrict__ idx, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) {
    const int64_t pg = idx[i];
    if ((uint64_t)pg < (uint64_t)tot) map[pg] = 1;
  }
}

}  // namespace
}  // namespace slora

extern "C" {

int slora_pool_scatter_rows(void* const* dst_bufs, const void* const* src_bufs, int n_bufs, const int64_t* loc,
                            int64_t n_rows, int64_t row_bytes, int64_t dst_row_stride_bytes,
                            int64_t src_row_stride_bytes, int64_t n_pages, void* stream) {
  using namespace slora;
  if (n_bufs < 0 || n_rows < 0 || row_bytes < 0 || n_pages < 0) return SLORA_ERR_BAD_SHAPE;
  if (dst_row_stride_bytes < row_bytes || src_row_stride_bytes < row_bytes) return SLORA_ERR_BAD_SHAPE;
  if (n_bufs == 0 || n_rows == 0 || row_bytes == 0) return SLORA_OK;
  if (dst_bufs == nullptr || src_bufs == nullptr || loc == nullptr) return SLORA_ERR_NULL_POINTER;
  for (int i = 0; i < n_bufs; ++i)
    if (dst_bufs[i] == nullptr || src_bufs[i] == nullptr) return SLORA_ERR_NULL_POINTER;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  for (int b0 = 0; b0 < n_bufs; b0 += kScatterBufs) {
    ScatterArgs p{};
    p.n_bufs = n_bufs - b0 < kScatterBufs ? n_bufs - b0 : kScatterBufs;
    bool vec = (row_bytes % 16 == 0) && (dst_row_stride_bytes % 16 == 0) && (src_row_stride_bytes % 16 == 0);
    for (int i = 0; i < p.n_bufs; ++i) {
      p.dst[i] = dst_bufs[b0 + i];
      p.src[i] = src_bufs[b0 + i];
      vec = vec && aligned16(p.dst[i]) && aligned16(p.src[i]);
    }
    p.loc = loc;
    p.n_rows = n_rows;
    p.n_pages = n_pages;
    p.row_bytes = row_bytes;
    p.dst_stride = dst_row_stride_bytes;
    p.src_stride = src_row_stride_bytes;
    p.vec_ok = vec ? 1 : 0;
    const int64_t grid = n_rows * p.n_bufs;
    if (grid > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(pool_scatter_kernel, dim3((uint32_t)grid), dim3(256), 0, s, p);
    if (hipGetLastError() != hipSuccess) return SLORA_ERR_LAUNCH;
  }
  return SLORA_OK;
}

int slora_pool_pack_transposed(void* const* dst_bufs, const void* const* src_mats, const int64_t* first,
                               const int64_t* rows, const int64_t* cols, const int64_t* dst_pitch,
                               const int64_t* n_slot, int n_mats, const int64_t* loc, int64_t n_loc,
                               int64_t page_elems, int64_t n_pages, void* stream) {
  using namespace slora;
  if (n_mats < 0 || n_loc < 0 || page_elems < 0 || n_pages < 0) return SLORA_ERR_BAD_SHAPE;
  if (n_mats == 0) return SLORA_OK;
  if (dst_bufs == nullptr || src_mats == nullptr || first == nullptr || rows == nullptr || cols == nullptr ||
      dst_pitch == nullptr || n_slot == nullptr || loc == nullptr)
    return SLORA_ERR_NULL_POINTER;
  if (page_elems == 0) return SLORA_ERR_BAD_SHAPE;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  for (int m0 = 0; m0 < n_mats; m0 += kPackMats) {
    PackArgs p{};
    p.n_mats = n_mats - m0 < kPackMats ? n_mats - m0 : kPackMats;
    int64_t max_tiles = 0;
    int tiles_k = 1;
    for (int i = 0; i < p.n_mats; ++i) {
      const int j = m0 + i;
      if (rows[j] < 0 || cols[j] < 0 || dst_pitch[j] < rows[j] || n_slot[j] < 0 || first[j] < 0)
        return SLORA_ERR_BAD_SHAPE;
      if (rows[j] > (1 << 24) || cols[j] > (1 << 24) || dst_pitch[j] > (1 << 30) || n_slot[j] > (1 << 20))
        return SLORA_ERR_UNSUPPORTED;
      // the transposed matrix must fit its slot
      if (cols[j] > 0 && (cols[j] - 1) * dst_pitch[j] + rows[j] > n_slot[j] * page_elems) return SLORA_ERR_BAD_SHAPE;
      if (dst_bufs[j] == nullptr || (src_mats[j] == nullptr && rows[j] * cols[j] > 0)) return SLORA_ERR_NULL_POINTER;
      const int tk = (int)((dst_pitch[j] + 63) / 64);
      if (tk > tiles_k) tiles_k = tk;
    }
    p.tiles_k = tiles_k;
    for (int i = 0; i < p.n_mats; ++i) {
      const int j = m0 + i;
      p.m[i].dst = dst_bufs[j];
      p.m[i].src = src_mats[j];
      p.m[i].first = first[j];
      p.m[i].rows = (int)rows[j];
      p.m[i].cols = (int)cols[j];
      p.m[i].dst_pitch = (int)dst_pitch[j];
      p.m[i].n_slot = (int)n_slot[j];
      // columns the slot has room for (source columns, then zero fill)
      const int64_t c_cover = dst_pitch[j] > 0 ? (n_slot[j] * page_elems + dst_pitch[j] - 1) / dst_pitch[j] : 0;
      const int64_t tiles = (c_cover + 63) / 64 * tiles_k;
      if (tiles > max_tiles) max_tiles = tiles;
    }
    p.loc = loc;
    p.n_loc = n_loc;
    p.n_pages = n_pages;
    p.page_elems = page_elems;
    if (max_tiles == 0) continue;
    if (max_tiles > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(pool_pack_kernel, dim3((uint32_t)max_tiles, (uint32_t)p.n_mats), dim3(256), 0, s, p);
    if (hipGetLastError() != hipSuccess) return SLORA_ERR_LAUNCH;
  }
  return SLORA_OK;
}

int slora_var_len_copy(const int64_t* old_a_start, const int64_t* old_a_len, const int64_t* old_a_loc,
                       const int64_t* new_a_start, int64_t* new_a_loc, int64_t n_adapters, int64_t n_old_loc,
                       int64_t n_new_loc, void* stream) {
  using namespace slora;
  if (n_adapters < 0 || n_old_loc < 0 || n_new_loc < 0) return SLORA_ERR_BAD_SHAPE;
  if (n_adapters == 0) return SLORA_OK;
  if (old_a_start == nullptr || old_a_len == nullptr || old_a_loc == nullptr || new_a_start == nullptr ||
      new_a_loc == nullptr)
    return SLORA_ERR_NULL_POINTER;
  if (n_adapters > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(var_len_copy_kernel, dim3((uint32_t)n_adapters), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), old_a_start, old_a_len, old_a_loc, new_a_start, new_a_loc,
                     n_old_loc, n_new_loc);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

int slora_tables_compact(const slora_tables* tables, const void* a_scaling, int scales_dtype, const uint8_t* keep,
                         int64_t* new_a_start, int64_t* new_a_len, int64_t* new_a_loc, void* new_a_scaling,
                         int64_t* removed_pages, int64_t* counts, int64_t* work, void* stream) {
  using namespace slora;
  if (tables == nullptr || counts == nullptr) return SLORA_ERR_NULL_POINTER;
  if (tables->n_adapters < 0 || tables->n_loc < 0) return SLORA_ERR_BAD_SHAPE;
  if (scales_dtype != SLORA_DTYPE_F16 && scales_dtype != SLORA_DTYPE_BF16 && scales_dtype != SLORA_DTYPE_F32)
    return SLORA_ERR_BAD_DTYPE;
  if (tables->n_adapters > 0 &&
      (tables->a_start == nullptr || tables->a_len == nullptr || a_scaling == nullptr || keep == nullptr ||
       new_a_start == nullptr || new_a_len == nullptr || new_a_scaling == nullptr || work == nullptr))
    return SLORA_ERR_NULL_POINTER;
  if (tables->n_loc > 0 && (tables->a_loc == nullptr || new_a_loc == nullptr || removed_pages == nullptr))
    return SLORA_ERR_NULL_POINTER;
  CompactArgs p{};
  p.a_start = tables->a_start;
  p.a_len = tables->a_len;
  p.a_loc = tables->a_loc;
  p.a_scaling = a_scaling;
  p.keep = keep;
  p.new_start = new_a_start;
  p.new_len = new_a_len;
  p.new_loc = new_a_loc;
  p.new_scaling = new_a_scaling;
  p.removed = removed_pages;
  p.counts = counts;
  p.work = work;
  p.n_adapters = tables->n_adapters;
  p.n_loc = tables->n_loc;
  p.scale_bytes = scales_dtype == SLORA_DTYPE_F32 ? 4 : 2;
  hipLaunchKernelGGL(tables_compact_kernel, dim3(1), dim3(kCompactThreads), 0, reinterpret_cast<hipStream_t>(stream),
                     p);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

int slora_pool_gather_a(void* out, int64_t out_cols, const void* pool, const int64_t* a_loc, int64_t n_loc,
                        int64_t first, int64_t rank, int64_t h, int64_t page_elems, int64_t n_pages, void* stream) {
  using namespace slora;
  if (out == nullptr || pool == nullptr || a_loc == nullptr) return SLORA_ERR_NULL_POINTER;
  if (h < 0 || rank < 0 || out_cols < rank || page_elems < h || n_pages < 0 || first < 0 || n_loc < 0)
    return SLORA_ERR_BAD_SHAPE;
  if (h == 0 || out_cols == 0) return SLORA_OK;
  if (h > (1 << 21) || out_cols > SLORA_MAX_RANK) return SLORA_ERR_UNSUPPORTED;
  const dim3 grid((uint32_t)((h + 63) / 64), (uint32_t)((out_cols + 63) / 64));
  hipLaunchKernelGGL(gather_a_kernel, grid, dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     static_cast<const uint16_t*>(pool), page_elems, n_pages, a_loc, n_loc, first, (int)rank, (int)h,
                     static_cast<uint16_t*>(out), (int)out_cols);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

int slora_pool_page_checksums(uint32_t* out, const void* pool, const int64_t* loc, int64_t n, int64_t page_bytes,
                              int64_t n_pages, void* stream) {
  using namespace slora;
  if (n < 0 || page_bytes < 0 || n_pages < 0) return SLORA_ERR_BAD_SHAPE;
  if (n == 0) return SLORA_OK;
  if (out == nullptr || pool == nullptr || loc == nullptr) return SLORA_ERR_NULL_POINTER;
  if (page_bytes % 16 != 0) return SLORA_ERR_UNSUPPORTED;
  if (!aligned16(pool)) return SLORA_ERR_ALIGNMENT;
  const int64_t grid = (n + 3) / 4;
  if (grid > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(page_xor_kernel, dim3((uint32_t)grid), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     static_cast<const u32x4*>(pool), page_bytes / 16, n_pages, loc, n, out);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

int slora_pool_page_xor(void* pool, const int64_t* loc, int64_t n, int64_t page_bytes, int64_t n_pages, uint32_t key,
                        void* stream) {
  using namespace slora;
  if (n < 0 || page_bytes < 0 || n_pages < 0) return SLORA_ERR_BAD_SHAPE;
  if (n == 0) return SLORA_OK;
  if (pool == nullptr || loc == nullptr) return SLORA_ERR_NULL_POINTER;
  if (page_bytes % 16 != 0) return SLORA_ERR_UNSUPPORTED;
  if (!aligned16(pool)) return SLORA_ERR_ALIGNMENT;
  const int64_t grid = (n + 3) / 4;
  if (grid > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(page_rmw_kernel, dim3((uint32_t)grid), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     static_cast<u32x4*>(pool), page_bytes / 16, n_pages, loc, n, key);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

int64_t slora_pool_alloc_workspace_bytes(int64_t tot_size) {
  if (tot_size < 0) return SLORA_ERR_BAD_SHAPE;
  const int64_t nb = (tot_size + slora::kMapBlock - 1) / slora::kMapBlock;
  return 16 + nb * 4 + 8 + nb * 8;  // best start, free counts, (alignment), last used pages
}

int slora_pool_alloc(uint8_t* mem_state, int64_t tot_size, int64_t need, int64_t* out_index, int64_t* result,
                     void* workspace, void* stream) {
  using namespace slora;
  if (tot_size < 0 || need < 0) return SLORA_ERR_BAD_SHAPE;
  if (result == nullptr || workspace == nullptr) return SLORA_ERR_NULL_POINTER;
  if (tot_size > 0 && mem_state == nullptr) return SLORA_ERR_NULL_POINTER;
  if (need > 0 && out_index == nullptr) return SLORA_ERR_NULL_POINTER;
  const int64_t nb = (tot_size + kMapBlock - 1) / kMapBlock;
  if (nb > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  int* block_free = reinterpret_cast<int*>(static_cast<char*>(workspace) + 16);
  const int vec = aligned16(mem_state) ? 1 : 0;
  if (nb == 0) {
    hipLaunchKernelGGL(map_alloc_kernel, dim3(1), dim3(kMapThreads), 0, s, mem_state, tot_size, need, block_free, 0,
                       out_index, result, vec);
    return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
  }
  hipLaunchKernelGGL(map_block_stats_kernel, dim3((uint32_t)nb), dim3(kMapThreads), 0, s, mem_state, tot_size,
                     block_free, static_cast<int64_t*>(nullptr), vec);
  hipLaunchKernelGGL(map_alloc_kernel, dim3((uint32_t)nb), dim3(kMapThreads), 0, s, mem_state, tot_size, need,
                     block_free, (int)nb, out_index, result, vec);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

int slora_pool_alloc_contiguous(uint8_t* mem_state, int64_t tot_size, int64_t need, int64_t* out_index,
                                int64_t* result, void* workspace, void* stream) {
  using namespace slora;
  if (tot_size < 0 || need <= 0) return SLORA_ERR_BAD_SHAPE;
  if (result == nullptr || workspace == nullptr || out_index == nullptr) return SLORA_ERR_NULL_POINTER;
  if (tot_size > 0 && mem_state == nullptr) return SLORA_ERR_NULL_POINTER;
  const int64_t nb = (tot_size + kMapBlock - 1) / kMapBlock;
  if (nb > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  unsigned long long* best = static_cast<unsigned long long*>(workspace);
  int* block_free = reinterpret_cast<int*>(static_cast<char*>(workspace) + 16);
  int64_t* block_last = reinterpret_cast<int64_t*>(static_cast<char*>(workspace) + 16 + ((nb * 4 + 7) / 8) * 8);
  const int vec = aligned16(mem_state) ? 1 : 0;
  hipLaunchKernelGGL(map_init_best_kernel, dim3(1), dim3(1), 0, s, best);
  if (nb > 0) {
    hipLaunchKernelGGL(map_block_stats_kernel, dim3((uint32_t)nb), dim3(kMapThreads), 0, s, mem_state, tot_size,
                       block_free, block_last, vec);
    hipLaunchKernelGGL(map_find_run_kernel, dim3((uint32_t)nb), dim3(kMapThreads), 0, s, mem_state, tot_size, need,
                       block_last, best, vec);
  }
  int64_t grid = (need + kMapThreads - 1) / kMapThreads;
  if (grid > 1024) grid = 1024;
  hipLaunchKernelGGL(map_take_run_kernel, dim3((uint32_t)grid), dim3(kMapThreads), 0, s, mem_state, tot_size, need,
                     best, out_index, result);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

int slora_pool_alloc_contiguous_static(uint8_t* mem_state, int64_t tot_size, int64_t need, int64_t* out_index,
                                       int64_t* result, void* stream) {
  using namespace slora;
  if (tot_size > kStaticMapPages) return SLORA_ERR_TOO_LARGE;
  static_assert(kStaticMapBlocks * kMapBlock == kStaticMapPages, "the static workspace is sized in whole map blocks");
  static_assert(kStaticMapPages == SLORA_POOL_STATIC_MAX_PAGES, "the header states the capacity");
  if (tot_size >= 0 && slora_pool_alloc_workspace_bytes(tot_size) > kStaticScratchBytes) return SLORA_ERR_TOO_LARGE;
  void* ws = static_scratch();
  if (ws == nullptr) return SLORA_ERR_LAUNCH;
  // same kernels as slora_pool_alloc_contiguous; its first launch resets the best start, and the
  // per-workgroup entries it reads are all rewritten by the launch in front of the reader
  return slora_pool_alloc_contiguous(mem_state, tot_size, need, out_index, result, ws, stream);
}

int slora_pool_free(uint8_t* mem_state, int64_t tot_size, const int64_t* free_index, int64_t n, void* stream) {
  using namespace slora;
  if (tot_size < 0 || n < 0) return SLORA_ERR_BAD_SHAPE;
  if (n == 0) return SLORA_OK;
  if (mem_state == nullptr || free_index == nullptr) return SLORA_ERR_NULL_POINTER;
  const int64_t grid = (n + 255) / 256;
  if (grid > 0x7fffffffLL) return SLORA_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(map_free_kernel, dim3((uint32_t)grid), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     mem_state, tot_size, free_index, n);
  return hipGetLastError() == hipSuccess ? SLORA_OK : SLORA_ERR_LAUNCH;
}

}  // extern "C"
