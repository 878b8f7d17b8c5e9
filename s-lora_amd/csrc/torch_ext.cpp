// slora_hip._kernels -- the thin PyTorch-ROCm extension in front of libslora_hip.so.
//
// Exports the operator surface the reference's LoRA engine imports:
//   dispatch_bgmv                       (slora/csrc/lora_ops.cc:76-78, 135)
//   lora_get_qkvo_fwd_shrink / _expand  (slora/models/peft/triton_kernel/lora/lora_prefill.py:139, 105)
// with the same positional arguments, in-place semantics and RuntimeErrors, plus the
// calls this library adds (q/k/v in one launch, per-batch plans, pool helpers).  Every
// function checks its tensors, takes the current HIP stream of the tensors' device and
// calls the C ABI of include/slora_hip.h; nothing is computed here and nothing
// synchronises.  The only state is the two plan caches below, each behind a mutex.
#include <torch/extension.h>

#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <cstdlib>
#include <mutex>
#include <string>
#include <vector>

#include "slora_hip.h"

namespace {

using at::Tensor;

// ---------------------------------------------------------------------------
// checks (messages follow lora_ops.cc:13-42)
// ---------------------------------------------------------------------------
#define SL_CHECK_INPUT(t)                                          \
  do {                                                             \
    TORCH_CHECK((t).is_cuda(), #t " must be a CUDA tensor");       \
    TORCH_CHECK((t).is_contiguous(), #t " must be contiguous");    \
  } while (0)
#define SL_CHECK_DIM(d, t) TORCH_CHECK((t).dim() == (d), #t " must be a " #d "D tensor")
#define SL_CHECK_INDEX(t) \
  TORCH_CHECK((t).scalar_type() == at::kLong, #t " must be an int64 tensor, got ", (t).scalar_type())
#define SL_CHECK_EQ(a, b) TORCH_CHECK((a) == (b), "CHECK_EQ(" #a ", " #b ") failed. ", (a), " vs ", (b))

int dtype_code(const Tensor& t, const char* what) {
  switch (t.scalar_type()) {
    case at::kHalf: return SLORA_DTYPE_F16;
    case at::kBFloat16: return SLORA_DTYPE_BF16;
    case at::kFloat: return SLORA_DTYPE_F32;
    default: TORCH_CHECK(false, what, " must be float16, bfloat16 or float32, got ", t.scalar_type());
  }
  return -1;
}

void* stream_of(const Tensor& t) { return c10::hip::getCurrentHIPStream(t.get_device()).stream(); }

// 0 when the stream is not being captured into a graph, else the id of the capture (never 0)
uint64_t capture_id_of(void* stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  unsigned long long id = 0;
  if (hipStreamGetCaptureInfo(static_cast<hipStream_t>(stream), &st, &id) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  if (st == hipStreamCaptureStatusNone) return 0;
  return id != 0 ? (uint64_t)id : ~(uint64_t)0;
}

// non-zero return code of the C ABI -> the RuntimeError a TORCH_CHECK of the reference would raise
void check_rc(int rc, const char* what, const std::string& detail = std::string()) {
  TORCH_CHECK(rc == SLORA_OK, what, ": ", slora_strerror(rc), detail.empty() ? "" : " ", detail);
}

// A tensor this library writes through a raw pointer counts as modified in place, so
// that anything keyed on tensor versions (the plan caches here, autograd's checks) sees it.
void mark_written(const Tensor& t) {
  if (t.defined() && !t.is_inference()) t.unsafeGetTensorImpl()->bump_version();
}

slora_tables tables_of(const Tensor& a_start, const Tensor& a_len, const Tensor& a_loc) {
  slora_tables t;
  t.a_start = a_start.data_ptr<int64_t>();
  t.a_len = a_len.data_ptr<int64_t>();
  t.a_loc = a_loc.data_ptr<int64_t>();
  t.n_adapters = a_start.numel();
  t.n_loc = a_loc.numel();
  return t;
}

// ---------------------------------------------------------------------------
// identity of the index tensors a cached plan was built from
// ---------------------------------------------------------------------------
// The very same tensor object (a weak reference keeps its TensorImpl's address from
// being handed to another tensor) at the same version: every in-place torch operation
// and every writer of this library raises the version.  Inference tensors carry no
// version and are never cached.
struct TensorId {
  typedef c10::intrusive_ptr<c10::TensorImpl, c10::UndefinedTensorImpl> ImplPtr;
  c10::weak_intrusive_ptr<c10::TensorImpl, c10::UndefinedTensorImpl> weak;
  const c10::TensorImpl* impl = nullptr;
  const void* data = nullptr;
  int64_t numel = 0;
  uint32_t version = 0;

  TensorId() : weak(ImplPtr()) {}
  explicit TensorId(const Tensor& t)
      : weak(t.getIntrusivePtr()),
        impl(t.unsafeGetTensorImpl()),
        data(t.data_ptr()),
        numel(t.numel()),
        version(t._version()) {}
  bool matches(const Tensor& t) const {
    return impl == t.unsafeGetTensorImpl() && !weak.expired() && data == t.data_ptr() && numel == t.numel() &&
           version == (uint32_t)t._version();
  }
};

bool cacheable(std::initializer_list<const Tensor*> ts) {
  for (const Tensor* t : ts)
    if (t->is_inference()) return false;
  return true;
}

bool env_cache_default() {
  const char* v = std::getenv("SLORA_PLAN_CACHE");  // read once, at import
  return !(v != nullptr && v[0] == '0' && v[1] == '\0');
}
bool g_cache_enabled = env_cache_default();

// status word of a plan buffer, read back on the buffer's current stream
int64_t plan_status_of(const Tensor& buf) {
  int status = 0;
  check_rc(slora_plan_status(buf.data_ptr(), &status, stream_of(buf)), "plan status");
  return status;
}

// ---------------------------------------------------------------------------
// decode plans
// ---------------------------------------------------------------------------
struct BgmvPlan {
  Tensor buf;  // int32 device buffer of slora_bgmv_plan_bytes() bytes
  int64_t rank_cap = 0, batch = 0;
  int64_t n_items = 0;  // 0 = not read back: launches are sized for the plan's capacity
  int64_t max_rank = 0, n_runs = 0;
};

void check_tables(const Tensor& start_indicies, const Tensor& lora_ranks, const Tensor& loc_indicies,
                  const Tensor& indicies) {
  SL_CHECK_INPUT(start_indicies);
  SL_CHECK_INPUT(lora_ranks);
  SL_CHECK_INPUT(loc_indicies);
  SL_CHECK_INPUT(indicies);
  SL_CHECK_DIM(1, indicies);
  SL_CHECK_INDEX(start_indicies);
  SL_CHECK_INDEX(lora_ranks);
  SL_CHECK_INDEX(loc_indicies);
  SL_CHECK_INDEX(indicies);
  SL_CHECK_EQ(start_indicies.numel(), lora_ranks.numel());
}

void check_scales(const Tensor& lora_scales, const Tensor& start_indicies) {
  SL_CHECK_INPUT(lora_scales);
  (void)dtype_code(lora_scales, "lora_scales");
  TORCH_CHECK(lora_scales.numel() >= start_indicies.numel(), "CHECK_EQ(lora_scales.size(0), start_indicies.size(0)) failed. ",
              lora_scales.numel(), " vs ", start_indicies.numel());
}

void build_plan_into(const Tensor& buf, const Tensor& start_indicies, const Tensor& lora_ranks,
                     const Tensor& loc_indicies, const Tensor& indicies, int64_t rank_cap, int64_t n_pages,
                     void* stream, const char* what) {
  const slora_tables t = tables_of(start_indicies, lora_ranks, loc_indicies);
  const int rc = slora_bgmv_plan_build(buf.data_ptr(), buf.numel() * 4, &t, indicies.data_ptr<int64_t>(),
                                       indicies.numel(), rank_cap, n_pages, stream);
  check_rc(rc, what);
}

Tensor alloc_plan_buffer(int64_t batch, int64_t rank_cap, const Tensor& like, const char* what) {
  const int64_t nbytes = slora_bgmv_plan_bytes(batch, rank_cap);
  if (nbytes < 0) check_rc((int)nbytes, what, "(batch=" + std::to_string(batch) + " rank_cap=" + std::to_string(rank_cap) + ")");
  return at::empty({(std::max<int64_t>(nbytes, 64) + 3) / 4}, like.options().dtype(at::kInt));
}

std::shared_ptr<BgmvPlan> make_plan(const Tensor& start_indicies, const Tensor& lora_ranks, const Tensor& loc_indicies,
                                    const Tensor& indicies, int64_t rank_cap, int64_t n_pages, bool readback) {
  check_tables(start_indicies, lora_ranks, loc_indicies, indicies);
  auto plan = std::make_shared<BgmvPlan>();
  plan->rank_cap = rank_cap;
  plan->batch = indicies.numel();
  plan->buf = alloc_plan_buffer(plan->batch, rank_cap, indicies, "make_plan");
  build_plan_into(plan->buf, start_indicies, lora_ranks, loc_indicies, indicies, rank_cap, n_pages, stream_of(indicies),
                  "make_plan");
  if (readback && plan->batch > 0) {
    const Tensor head = plan->buf.slice(0, 0, 8).cpu();  // one synchronisation
    const int32_t* h = head.data_ptr<int32_t>();
    plan->n_items = h[1];
    plan->max_rank = h[2];
    plan->n_runs = h[6];
  }
  return plan;
}

void rebuild_plan(const std::shared_ptr<BgmvPlan>& plan, const Tensor& start_indicies, const Tensor& lora_ranks,
                  const Tensor& loc_indicies, const Tensor& indicies, int64_t n_pages) {
  check_tables(start_indicies, lora_ranks, loc_indicies, indicies);
  TORCH_CHECK(indicies.numel() == plan->batch, "plan was built for ", plan->batch, " tokens, this batch has ",
              indicies.numel());
  build_plan_into(plan->buf, start_indicies, lora_ranks, loc_indicies, indicies, plan->rank_cap, n_pages,
                  stream_of(indicies), "rebuild_plan");
  // the new batch's item count is not known on the host (nothing is read back, so that the call can be
  // recorded into a graph): launches with this plan are sized for its capacity from now on
  plan->n_items = 0;
  plan->max_rank = 0;
  plan->n_runs = 0;
}

// Plans built on behalf of callers that pass none.  The reference's engine issues all
// 8 x n_layers dispatch_bgmv calls of a decode step with the same four index tensors
// (slora/models/peft/lora_unordered_batch_infer.py:254-318, 428-448): the first call of a
// step builds the plan, the others reuse it.  A build does not wait for the device: the
// item count travels to a pinned host word behind an event, launches use the plan's
// capacity until it has arrived and the exact count afterwards.  Callers that pass new
// tensor objects every call (slices) never hit; after kMissStreak builds in a row that
// nobody reused the cache pauses for kCoolDown calls.
class PlanCache {
 public:
  static constexpr int kCapacity = 4, kMissStreak = 8, kCoolDown = 256;

  struct Entry {
    TensorId ids[4];
    int64_t rank_cap = 0, n_pages = 0;
    void* stream = nullptr;
    int device = -1;
    std::shared_ptr<BgmvPlan> plan;
    int32_t* host_head = nullptr;  // pinned, 8 words: the plan's header once `landed` has fired
    hipEvent_t landed = nullptr;
    bool pending = false;
    uint64_t used = 0;
    uint64_t capture = 0;  // the graph capture the plan was built in (its build is a node of that graph), 0: none
  };

  ~PlanCache() {
    // process teardown: the runtime may be gone already; pinned words and events are left to it
  }

  void clear() {
    std::lock_guard<std::mutex> lock(mu_);
    for (Entry& e : entries_) e.plan.reset();
    streak_ = paused_ = 0;
  }

  // nullptr: no plan for this call (cache off, inference tensors, cooling down).
  // While the stream is being captured into a graph a plan is built and reused as well, within
  // that capture only: its build kernel becomes a node of the graph, so every replay rebuilds
  // the plan from what the index tensors hold then, and the buffer comes from the graph's own
  // memory pool.  Such a plan's item count is never read back (no host copy may be captured
  // usefully): its launches are sized for the plan's capacity.
  std::shared_ptr<BgmvPlan> get(const Tensor& start_indicies, const Tensor& lora_ranks, const Tensor& loc_indicies,
                                const Tensor& indicies, int64_t rank_cap, int64_t n_pages, void* stream) {
    if (!g_cache_enabled || indicies.numel() == 0 || rank_cap <= 0 || rank_cap > SLORA_MAX_RANK) return nullptr;
    if (!cacheable({&start_indicies, &lora_ranks, &loc_indicies, &indicies})) return nullptr;
    const uint64_t capture = capture_id_of(stream);
    std::lock_guard<std::mutex> lock(mu_);
    if (paused_ > 0) {
      --paused_;
      return nullptr;
    }
    const Tensor* ts[4] = {&start_indicies, &lora_ranks, &loc_indicies, &indicies};
    const int device = indicies.get_device();
    ++clock_;
    for (Entry& e : entries_) {
      if (!e.plan || e.rank_cap != rank_cap || e.n_pages != n_pages || e.stream != stream || e.device != device ||
          e.capture != capture)
        continue;
      bool same = true;
      for (int i = 0; i < 4 && same; ++i) same = e.ids[i].matches(*ts[i]);
      if (!same) continue;
      if (e.pending && capture == 0 && hipEventQuery(e.landed) == hipSuccess) {
        e.pending = false;
        e.plan->n_items = e.host_head[1];
        e.plan->max_rank = e.host_head[2];
        e.plan->n_runs = e.host_head[6];
      }
      e.used = clock_;
      ++hits_;
      streak_ = 0;
      return e.plan;
    }
    if (++streak_ > kMissStreak) {
      streak_ = 0;
      paused_ = kCoolDown;
      return nullptr;
    }
    // build into the least recently used slot
    if ((int)entries_.size() < kCapacity) entries_.emplace_back();
    Entry* slot = nullptr;
    for (Entry& e : entries_) {
      if (capture != 0 && e.pending) continue;  // no waiting for a copy while a graph is being captured
      if (!e.plan) { slot = &e; break; }
      if (slot == nullptr || e.used < slot->used) slot = &e;
    }
    if (slot == nullptr) return nullptr;
    if (slot->pending) {  // its copy may still be in flight: wait for it before the words are reused
      (void)hipEventSynchronize(slot->landed);
      slot->pending = false;
    }
    auto plan = std::make_shared<BgmvPlan>();
    plan->rank_cap = rank_cap;
    plan->batch = indicies.numel();
    plan->buf = alloc_plan_buffer(plan->batch, rank_cap, indicies, "dispatch_bgmv (plan)");
    build_plan_into(plan->buf, start_indicies, lora_ranks, loc_indicies, indicies, rank_cap, n_pages, stream,
                    "dispatch_bgmv (plan)");
    if (capture == 0 && slot->host_head == nullptr) {
      void* p = nullptr;
      if (hipHostMalloc(&p, 8 * sizeof(int32_t), hipHostMallocDefault) == hipSuccess) slot->host_head = static_cast<int32_t*>(p);
      else (void)hipGetLastError();
    }
    if (capture == 0 && slot->landed == nullptr &&
        hipEventCreateWithFlags(&slot->landed, hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      slot->landed = nullptr;
    }
    if (capture == 0 && slot->host_head != nullptr && slot->landed != nullptr &&
        hipMemcpyAsync(slot->host_head, plan->buf.data_ptr(), 8 * sizeof(int32_t), hipMemcpyDeviceToHost,
                       static_cast<hipStream_t>(stream)) == hipSuccess &&
        hipEventRecord(slot->landed, static_cast<hipStream_t>(stream)) == hipSuccess) {
      slot->pending = true;
    } else {
      (void)hipGetLastError();
    }
    for (int i = 0; i < 4; ++i) slot->ids[i] = TensorId(*ts[i]);
    slot->rank_cap = rank_cap;
    slot->n_pages = n_pages;
    slot->stream = stream;
    slot->device = device;
    slot->capture = capture;
    slot->plan = plan;
    slot->used = clock_;
    ++builds_;
    return plan;
  }

  int64_t hits() const { return hits_; }
  int64_t builds() const { return builds_; }
  void reset_stats() { hits_ = builds_ = 0; }

 private:
  std::mutex mu_;
  std::vector<Entry> entries_;
  uint64_t clock_ = 0;
  int64_t hits_ = 0, builds_ = 0;
  int streak_ = 0, paused_ = 0;
};

PlanCache& plan_cache() {
  static PlanCache* c = new PlanCache();  // never destroyed: no HIP calls at exit
  return *c;
}

// `plan` argument of the Python calls: None = automatic, False = none, else a BgmvPlan
std::shared_ptr<BgmvPlan> resolve_plan(const py::object& plan, const Tensor& start_indicies, const Tensor& lora_ranks,
                                       const Tensor& loc_indicies, const Tensor& indicies, int64_t rank_cap,
                                       int64_t n_pages, void* stream, int64_t batch) {
  std::shared_ptr<BgmvPlan> p;
  if (plan.is_none()) {
    p = plan_cache().get(start_indicies, lora_ranks, loc_indicies, indicies, rank_cap, n_pages, stream);
  } else if (py::isinstance<py::bool_>(plan)) {
    TORCH_CHECK(!plan.cast<bool>(), "plan must be a BgmvPlan, None or False");
  } else {
    p = plan.cast<std::shared_ptr<BgmvPlan>>();
  }
  if (p) TORCH_CHECK(p->batch == batch, "plan was built for ", p->batch, " tokens, this call has ", batch);
  return p;
}

void dispatch_bgmv(const Tensor& y, const Tensor& x, const Tensor& w, const Tensor& start_indicies,
                   const Tensor& lora_ranks, const Tensor& loc_indicies, const Tensor& indicies, int64_t qkvo,
                   const Tensor& lora_scales, const py::object& plan) {
  SL_CHECK_INPUT(y);
  SL_CHECK_INPUT(x);
  SL_CHECK_INPUT(w);
  check_tables(start_indicies, lora_ranks, loc_indicies, indicies);
  check_scales(lora_scales, start_indicies);
  SL_CHECK_DIM(2, y);
  SL_CHECK_DIM(2, x);
  SL_CHECK_DIM(3, w);
  SL_CHECK_EQ(indicies.size(0), x.size(0));
  SL_CHECK_EQ(y.size(0), x.size(0));
  const int64_t batch = x.size(0), h_in = x.size(1), h_out = y.size(1);
  const bool dt_ok = (x.scalar_type() == at::kHalf || x.scalar_type() == at::kBFloat16) &&
                     y.scalar_type() == x.scalar_type() && w.scalar_type() == x.scalar_type();
  TORCH_CHECK(dt_ok && h_in < 65536 && h_out < 65536, "No suitable kernel. h_in=", h_in, " h_out=", h_out,
              " dtype=", x.scalar_type());
  const int64_t page_elems = w.size(1) * w.size(2), n_pages = w.size(0);
  const slora_tables t = tables_of(start_indicies, lora_ranks, loc_indicies);
  const int code = dtype_code(x, "x");
  void* stream = stream_of(x);
  const std::shared_ptr<BgmvPlan> p = resolve_plan(plan, start_indicies, lora_ranks, loc_indicies, indicies,
                                                   std::min(h_in, h_out), n_pages, stream, batch);
  const int64_t* bins = indicies.data_ptr<int64_t>();
  int rc;
  if (h_in < h_out) {  // direction rule of slora/csrc/bgmv/bgmv_impl.cuh:221
    const int sc = dtype_code(lora_scales, "lora_scales");
    if (p)
      rc = slora_bgmv_expand_planned(p->buf.data_ptr(), p->rank_cap, p->n_items, 1, y.data_ptr(), nullptr, nullptr,
                                     x.data_ptr(), nullptr, nullptr, w.data_ptr(), &t, bins, lora_scales.data_ptr(), sc,
                                     batch, h_in, h_out, 0, 0, page_elems, n_pages, (int)qkvo, code, stream);
    else
      rc = slora_bgmv_expand(y.data_ptr(), x.data_ptr(), w.data_ptr(), &t, bins, lora_scales.data_ptr(), sc, batch, h_in,
                             h_out, page_elems, n_pages, (int)qkvo, code, stream);
  } else {
    if (p)
      rc = slora_bgmv_shrink_planned(p->buf.data_ptr(), p->rank_cap, p->n_items, 1, y.data_ptr(), nullptr, nullptr,
                                     x.data_ptr(), w.data_ptr(), &t, bins, batch, h_in, h_out, page_elems, n_pages,
                                     (int)qkvo, code, stream);
    else
      rc = slora_bgmv_shrink(y.data_ptr(), x.data_ptr(), w.data_ptr(), &t, bins, batch, h_in, h_out, page_elems, n_pages,
                             (int)qkvo, code, stream);
  }
  TORCH_CHECK(rc != SLORA_ERR_UNSUPPORTED, "No suitable kernel. h_in=", h_in, " h_out=", h_out, " dtype=", x.scalar_type());
  if (rc != SLORA_OK)
    check_rc(rc, "dispatch_bgmv",
             "(h_in=" + std::to_string(h_in) + " h_out=" + std::to_string(h_out) + " qkvo=" + std::to_string(qkvo) + ")");
}

void check_rows_2d(const Tensor& t, const char* name, int64_t rows, int64_t cols, at::ScalarType dt) {
  TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
  TORCH_CHECK(t.dim() == 2, name, " must be a 2D tensor");
  TORCH_CHECK(t.size(0) == rows && (cols < 0 || t.size(1) == cols) && t.scalar_type() == dt, name, " must be [", rows,
              ", ", cols < 0 ? t.size(1) : cols, "] ", dt);
}

void dispatch_bgmv_qkv_shrink(const Tensor& y_q, const Tensor& y_k, const Tensor& y_v, const Tensor& x, const Tensor& w,
                              const Tensor& start_indicies, const Tensor& lora_ranks, const Tensor& loc_indicies,
                              const Tensor& indicies, const py::object& plan) {
  SL_CHECK_INPUT(x);
  SL_CHECK_DIM(2, x);
  SL_CHECK_INPUT(w);
  SL_CHECK_DIM(3, w);
  check_tables(start_indicies, lora_ranks, loc_indicies, indicies);
  const int64_t batch = x.size(0), h_in = x.size(1);
  SL_CHECK_INPUT(y_q);
  SL_CHECK_DIM(2, y_q);
  const int64_t y_cols = y_q.size(1);
  check_rows_2d(y_q, "y_q", batch, y_cols, x.scalar_type());
  check_rows_2d(y_k, "y_k", batch, y_cols, x.scalar_type());
  check_rows_2d(y_v, "y_v", batch, y_cols, x.scalar_type());
  SL_CHECK_EQ(indicies.size(0), x.size(0));
  const bool dt_ok = (x.scalar_type() == at::kHalf || x.scalar_type() == at::kBFloat16) && w.scalar_type() == x.scalar_type();
  TORCH_CHECK(dt_ok, "No suitable kernel. h_in=", h_in, " h_out=", y_cols, " dtype=", x.scalar_type());
  const slora_tables t = tables_of(start_indicies, lora_ranks, loc_indicies);
  void* stream = stream_of(x);
  const int64_t page_elems = w.size(1) * w.size(2), n_pages = w.size(0);
  const std::shared_ptr<BgmvPlan> p =
      resolve_plan(plan, start_indicies, lora_ranks, loc_indicies, indicies, y_cols, n_pages, stream, batch);
  const int code = dtype_code(x, "x");
  int rc;
  if (p)
    rc = slora_bgmv_shrink_planned(p->buf.data_ptr(), p->rank_cap, p->n_items, 3, y_q.data_ptr(), y_k.data_ptr(),
                                   y_v.data_ptr(), x.data_ptr(), w.data_ptr(), &t, indicies.data_ptr<int64_t>(), batch,
                                   h_in, y_cols, page_elems, n_pages, 0, code, stream);
  else
    rc = slora_bgmv_shrink_qkv(y_q.data_ptr(), y_k.data_ptr(), y_v.data_ptr(), x.data_ptr(), w.data_ptr(), &t,
                               indicies.data_ptr<int64_t>(), batch, h_in, y_cols, page_elems, n_pages, code, stream);
  TORCH_CHECK(rc != SLORA_ERR_UNSUPPORTED, "No suitable kernel. h_in=", h_in, " h_out=", y_cols, " dtype=", x.scalar_type());
  check_rc(rc, "dispatch_bgmv_qkv_shrink");
}

void dispatch_bgmv_qkv_expand(const Tensor& y_q, const Tensor& y_k, const Tensor& y_v, const Tensor& x_q,
                              const Tensor& x_k, const Tensor& x_v, const Tensor& w, const Tensor& start_indicies,
                              const Tensor& lora_ranks, const Tensor& loc_indicies, const Tensor& indicies,
                              const Tensor& lora_scales, const py::object& plan) {
  SL_CHECK_INPUT(x_q);
  SL_CHECK_DIM(2, x_q);
  SL_CHECK_INPUT(w);
  SL_CHECK_DIM(3, w);
  check_tables(start_indicies, lora_ranks, loc_indicies, indicies);
  check_scales(lora_scales, start_indicies);
  const int64_t batch = x_q.size(0), x_cols = x_q.size(1);
  const at::ScalarType dt = x_q.scalar_type();
  check_rows_2d(x_k, "x_k", batch, x_cols, dt);
  check_rows_2d(x_v, "x_v", batch, x_cols, dt);
  check_rows_2d(y_q, "y_q", batch, -1, dt);
  check_rows_2d(y_k, "y_k", batch, -1, dt);
  check_rows_2d(y_v, "y_v", batch, -1, dt);
  SL_CHECK_EQ(indicies.size(0), x_q.size(0));
  const bool dt_ok = (dt == at::kHalf || dt == at::kBFloat16) && w.scalar_type() == dt;
  TORCH_CHECK(dt_ok, "No suitable kernel. h_in=", x_cols, " h_out=", y_q.size(1), " dtype=", dt);
  const slora_tables t = tables_of(start_indicies, lora_ranks, loc_indicies);
  void* stream = stream_of(x_q);
  const int64_t page_elems = w.size(1) * w.size(2), n_pages = w.size(0);
  const std::shared_ptr<BgmvPlan> p =
      resolve_plan(plan, start_indicies, lora_ranks, loc_indicies, indicies, x_cols, n_pages, stream, batch);
  const int code = dtype_code(x_q, "x_q"), sc = dtype_code(lora_scales, "lora_scales");
  int rc;
  if (p)
    rc = slora_bgmv_expand_planned(p->buf.data_ptr(), p->rank_cap, p->n_items, 3, y_q.data_ptr(), y_k.data_ptr(),
                                   y_v.data_ptr(), x_q.data_ptr(), x_k.data_ptr(), x_v.data_ptr(), w.data_ptr(), &t,
                                   indicies.data_ptr<int64_t>(), lora_scales.data_ptr(), sc, batch, x_cols, y_q.size(1),
                                   y_k.size(1), y_v.size(1), page_elems, n_pages, 0, code, stream);
  else
    rc = slora_bgmv_expand_qkv(y_q.data_ptr(), y_k.data_ptr(), y_v.data_ptr(), x_q.data_ptr(), x_k.data_ptr(),
                               x_v.data_ptr(), w.data_ptr(), &t, indicies.data_ptr<int64_t>(), lora_scales.data_ptr(), sc,
                               batch, x_cols, y_q.size(1), y_k.size(1), y_v.size(1), page_elems, n_pages, code, stream);
  TORCH_CHECK(rc != SLORA_ERR_UNSUPPORTED, "No suitable kernel. h_in=", x_cols, " h_out=", y_q.size(1), " dtype=", dt);
  check_rc(rc, "dispatch_bgmv_qkv_expand");
}

// Shrink and expand of one projection in one launch: delta = x A (left in `delta`), y += scale * delta B.
// With plan=False (or no plan for the batch) the two stateless launches are issued instead.
void dispatch_bgmv_lora(const Tensor& y, const Tensor& delta, const Tensor& x, const Tensor& w_a, const Tensor& w_b,
                        const Tensor& start_indicies, const Tensor& lora_ranks, const Tensor& loc_indicies,
                        const Tensor& indicies, int64_t qkvo, const Tensor& lora_scales, const py::object& plan) {
  SL_CHECK_INPUT(x);
  SL_CHECK_DIM(2, x);
  SL_CHECK_INPUT(w_a);
  SL_CHECK_DIM(3, w_a);
  SL_CHECK_INPUT(w_b);
  SL_CHECK_DIM(3, w_b);
  check_tables(start_indicies, lora_ranks, loc_indicies, indicies);
  check_scales(lora_scales, start_indicies);
  const int64_t batch = x.size(0), h_in = x.size(1);
  const at::ScalarType dt = x.scalar_type();
  check_rows_2d(delta, "delta", batch, -1, dt);
  check_rows_2d(y, "y", batch, -1, dt);
  SL_CHECK_EQ(indicies.size(0), x.size(0));
  const int64_t d_cols = delta.size(1), h_out = y.size(1);
  const bool dt_ok = (dt == at::kHalf || dt == at::kBFloat16) && w_a.scalar_type() == dt && w_b.scalar_type() == dt;
  TORCH_CHECK(dt_ok && h_in < 65536 && h_out < 65536, "No suitable kernel. h_in=", h_in, " h_out=", h_out, " dtype=", dt);
  TORCH_CHECK(w_a.sizes() == w_b.sizes(), "w_a and w_b must be pools of one shape (they share page ids)");
  const int64_t page_elems = w_a.size(1) * w_a.size(2), n_pages = w_a.size(0);
  const slora_tables t = tables_of(start_indicies, lora_ranks, loc_indicies);
  const int code = dtype_code(x, "x"), sc = dtype_code(lora_scales, "lora_scales");
  void* stream = stream_of(x);
  const std::shared_ptr<BgmvPlan> p =
      resolve_plan(plan, start_indicies, lora_ranks, loc_indicies, indicies, d_cols, n_pages, stream, batch);
  const int64_t* bins = indicies.data_ptr<int64_t>();
  int rc;
  if (p && d_cols % 8 == 0) {
    rc = slora_bgmv_lora_planned(p->buf.data_ptr(), p->rank_cap, p->n_items, 1, y.data_ptr(), nullptr, nullptr,
                                 delta.data_ptr(), nullptr, nullptr, x.data_ptr(), w_a.data_ptr(), w_b.data_ptr(), &t, bins,
                                 lora_scales.data_ptr(), sc, batch, h_in, d_cols, h_out, 0, 0, page_elems, n_pages,
                                 (int)qkvo, code, stream);
  } else {
    rc = slora_bgmv_shrink(delta.data_ptr(), x.data_ptr(), w_a.data_ptr(), &t, bins, batch, h_in, d_cols, page_elems,
                           n_pages, (int)qkvo, code, stream);
    if (rc == SLORA_OK)
      rc = slora_bgmv_expand(y.data_ptr(), delta.data_ptr(), w_b.data_ptr(), &t, bins, lora_scales.data_ptr(), sc, batch,
                             d_cols, h_out, page_elems, n_pages, (int)qkvo, code, stream);
  }
  TORCH_CHECK(rc != SLORA_ERR_UNSUPPORTED, "No suitable kernel. h_in=", h_in, " h_out=", h_out, " dtype=", dt);
  check_rc(rc, "dispatch_bgmv_lora");
}

// The same for q, k and v in one launch (they share x).
void dispatch_bgmv_qkv_lora(const Tensor& y_q, const Tensor& y_k, const Tensor& y_v, const Tensor& d_q, const Tensor& d_k,
                            const Tensor& d_v, const Tensor& x, const Tensor& w_a, const Tensor& w_b,
                            const Tensor& start_indicies, const Tensor& lora_ranks, const Tensor& loc_indicies,
                            const Tensor& indicies, const Tensor& lora_scales, const py::object& plan) {
  SL_CHECK_INPUT(x);
  SL_CHECK_DIM(2, x);
  SL_CHECK_INPUT(w_a);
  SL_CHECK_DIM(3, w_a);
  SL_CHECK_INPUT(w_b);
  SL_CHECK_DIM(3, w_b);
  check_tables(start_indicies, lora_ranks, loc_indicies, indicies);
  check_scales(lora_scales, start_indicies);
  const int64_t batch = x.size(0), h_in = x.size(1);
  const at::ScalarType dt = x.scalar_type();
  check_rows_2d(d_q, "d_q", batch, -1, dt);
  const int64_t d_cols = d_q.size(1);
  check_rows_2d(d_k, "d_k", batch, d_cols, dt);
  check_rows_2d(d_v, "d_v", batch, d_cols, dt);
  check_rows_2d(y_q, "y_q", batch, -1, dt);
  check_rows_2d(y_k, "y_k", batch, -1, dt);
  check_rows_2d(y_v, "y_v", batch, -1, dt);
  SL_CHECK_EQ(indicies.size(0), x.size(0));
  const bool dt_ok = (dt == at::kHalf || dt == at::kBFloat16) && w_a.scalar_type() == dt && w_b.scalar_type() == dt;
  TORCH_CHECK(dt_ok, "No suitable kernel. h_in=", h_in, " h_out=", y_q.size(1), " dtype=", dt);
  TORCH_CHECK(w_a.sizes() == w_b.sizes(), "w_a and w_b must be pools of one shape (they share page ids)");
  const int64_t page_elems = w_a.size(1) * w_a.size(2), n_pages = w_a.size(0);
  const slora_tables t = tables_of(start_indicies, lora_ranks, loc_indicies);
  const int code = dtype_code(x, "x"), sc = dtype_code(lora_scales, "lora_scales");
  void* stream = stream_of(x);
  const std::shared_ptr<BgmvPlan> p =
      resolve_plan(plan, start_indicies, lora_ranks, loc_indicies, indicies, d_cols, n_pages, stream, batch);
  const int64_t* bins = indicies.data_ptr<int64_t>();
  int rc;
  if (p && d_cols % 8 == 0) {
    rc = slora_bgmv_lora_planned(p->buf.data_ptr(), p->rank_cap, p->n_items, 3, y_q.data_ptr(), y_k.data_ptr(),
                                 y_v.data_ptr(), d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), x.data_ptr(),
                                 w_a.data_ptr(), w_b.data_ptr(), &t, bins, lora_scales.data_ptr(), sc, batch, h_in, d_cols,
                                 y_q.size(1), y_k.size(1), y_v.size(1), page_elems, n_pages, 0, code, stream);
  } else {
    rc = slora_bgmv_shrink_qkv(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), x.data_ptr(), w_a.data_ptr(), &t, bins,
                               batch, h_in, d_cols, page_elems, n_pages, code, stream);
    if (rc == SLORA_OK)
      rc = slora_bgmv_expand_qkv(y_q.data_ptr(), y_k.data_ptr(), y_v.data_ptr(), d_q.data_ptr(), d_k.data_ptr(),
                                 d_v.data_ptr(), w_b.data_ptr(), &t, bins, lora_scales.data_ptr(), sc, batch, d_cols,
                                 y_q.size(1), y_k.size(1), y_v.size(1), page_elems, n_pages, code, stream);
  }
  TORCH_CHECK(rc != SLORA_ERR_UNSUPPORTED, "No suitable kernel. h_in=", h_in, " h_out=", y_q.size(1), " dtype=", dt);
  check_rc(rc, "dispatch_bgmv_qkv_lora");
}

// ---------------------------------------------------------------------------
// prefill
// ---------------------------------------------------------------------------
void check_2d_strided(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor");
  TORCH_CHECK(t.dim() == 2, name, " must be a 2D tensor");
  TORCH_CHECK(t.size(1) <= 1 || t.stride(1) == 1, name, " must have unit column stride, got ", t.stride(1));
}
void check_1d(const Tensor& t, const char* name, at::ScalarType dt) {
  TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor");
  TORCH_CHECK(t.dim() == 1 && t.is_contiguous(), name, " must be a contiguous 1D tensor");
  TORCH_CHECK(t.scalar_type() == dt, name, " must be ", dt, ", got ", t.scalar_type());
}

void check_segments(const Tensor& b_lora_start, const Tensor& b_lora_ranks, const Tensor& b_start_loc,
                    const Tensor& b_seq_len, const Tensor& b_indicies) {
  check_1d(b_lora_start, "b_lora_start", at::kLong);
  check_1d(b_lora_ranks, "b_lora_ranks", at::kLong);
  check_1d(b_indicies, "b_indicies", at::kLong);
  check_1d(b_start_loc, "b_start_loc", at::kInt);
  check_1d(b_seq_len, "b_seq_len", at::kInt);
  TORCH_CHECK(b_start_loc.numel() == b_seq_len.numel() && b_seq_len.numel() == b_indicies.numel(),
              "b_start_loc, b_seq_len and b_indicies must have one entry per request");
  TORCH_CHECK(b_lora_start.numel() == b_lora_ranks.numel(), "b_lora_start and b_lora_ranks must have one entry per adapter");
}

slora_tables prefill_common(const Tensor& x, const Tensor& w, const Tensor& o, const Tensor& b_loc,
                            const Tensor& b_lora_start, const Tensor& b_lora_ranks, const Tensor& b_start_loc,
                            const Tensor& b_seq_len, const Tensor& b_indicies) {
  check_2d_strided(x, "x");
  check_2d_strided(w, "w");
  check_2d_strided(o, "o");
  check_1d(b_loc, "b_loc", at::kLong);
  check_segments(b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies);
  const at::ScalarType dt = x.scalar_type();
  TORCH_CHECK((dt == at::kHalf || dt == at::kBFloat16) && w.scalar_type() == dt && o.scalar_type() == dt,
              "x, w and o must share a dtype of float16 or bfloat16, got ", dt, ", ", w.scalar_type(), ", ", o.scalar_type());
  TORCH_CHECK(x.size(0) == o.size(0), "x and o must have the same number of rows, got ", x.size(0), " and ", o.size(0));
  return tables_of(b_lora_start, b_lora_ranks, b_loc);
}

struct SgmmPlan {
  Tensor buf;
  bool usable = false;
  int64_t n_requests = 0, n_tokens = 0, max_rank = 0, max_input_len = 0;
};

std::shared_ptr<SgmmPlan> make_prefill_plan(const Tensor& b_lora_start, const Tensor& b_lora_ranks,
                                            const Tensor& b_start_loc, const Tensor& b_seq_len, const Tensor& b_indicies,
                                            int64_t n_tokens, int64_t max_rank, int64_t max_input_len) {
  check_segments(b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies);
  auto plan = std::make_shared<SgmmPlan>();
  const int64_t nbytes = slora_sgmm_plan_bytes();
  plan->buf = at::empty({nbytes / 4}, b_seq_len.options().dtype(at::kInt));
  // the plan reads no page ids: the loc table only has to be non-null
  slora_tables t = tables_of(b_lora_start, b_lora_ranks, b_lora_start);
  t.n_loc = 0;
  int usable = 0;
  const int rc = slora_sgmm_plan_build(plan->buf.data_ptr(), nbytes, &t, b_start_loc.data_ptr<int32_t>(),
                                       b_seq_len.data_ptr<int32_t>(), b_indicies.data_ptr<int64_t>(), b_seq_len.numel(),
                                       max_input_len, n_tokens, max_rank, &usable, stream_of(b_seq_len));
  check_rc(rc, "make_prefill_plan", "(n_tokens=" + std::to_string(n_tokens) + " max_rank=" + std::to_string(max_rank) + ")");
  plan->usable = usable != 0;
  plan->n_requests = b_seq_len.numel();
  plan->n_tokens = n_tokens;
  plan->max_rank = max_rank;
  plan->max_input_len = max_input_len;
  return plan;
}

// Same rules as PlanCache, for the shrink calls of a prefill step (they all pass the same
// five index tensors, lora_unordered_batch_infer.py:334-410).
class PrefillPlanCache {
 public:
  static constexpr int kCapacity = 2, kMissStreak = 8, kCoolDown = 256;
  struct Entry {
    TensorId ids[5];
    int64_t n_tokens = 0, max_rank = 0, max_input_len = 0;
    void* stream = nullptr;
    int device = -1;
    std::shared_ptr<SgmmPlan> plan;
    uint64_t used = 0;
    uint64_t capture = 0;  // as in PlanCache::Entry
  };
  void clear() {
    std::lock_guard<std::mutex> lock(mu_);
    entries_.clear();
    streak_ = paused_ = 0;
  }
  std::shared_ptr<SgmmPlan> get(const Tensor& b_lora_start, const Tensor& b_lora_ranks, const Tensor& b_start_loc,
                                const Tensor& b_seq_len, const Tensor& b_indicies, int64_t n_tokens, int64_t max_rank,
                                int64_t max_input_len, void* stream) {
    if (!g_cache_enabled || b_seq_len.numel() == 0 || n_tokens <= 0 || max_rank <= 0 || max_rank > SLORA_MAX_RANK ||
        max_input_len <= 0)
      return nullptr;
    if (!cacheable({&b_lora_start, &b_lora_ranks, &b_start_loc, &b_seq_len, &b_indicies})) return nullptr;
    const uint64_t capture = capture_id_of(stream);  // a plan built inside a capture serves that capture only
    std::lock_guard<std::mutex> lock(mu_);
    if (paused_ > 0) {
      --paused_;
      return nullptr;
    }
    const Tensor* ts[5] = {&b_lora_start, &b_lora_ranks, &b_start_loc, &b_seq_len, &b_indicies};
    const int device = b_seq_len.get_device();
    ++clock_;
    for (Entry& e : entries_) {
      if (e.n_tokens != n_tokens || e.max_rank != max_rank || e.max_input_len != max_input_len || e.stream != stream ||
          e.device != device || e.capture != capture)
        continue;
      bool same = true;
      for (int i = 0; i < 5 && same; ++i) same = e.ids[i].matches(*ts[i]);
      if (!same) continue;
      e.used = clock_;
      ++hits_;
      streak_ = 0;
      return e.plan;
    }
    if (++streak_ > kMissStreak) {
      streak_ = 0;
      paused_ = kCoolDown;
      return nullptr;
    }
    if ((int)entries_.size() < kCapacity) entries_.emplace_back();
    Entry* slot = &entries_[0];
    for (Entry& e : entries_)
      if (!e.plan) { slot = &e; break; } else if (e.used < slot->used) slot = &e;
    slot->plan = make_prefill_plan(b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies, n_tokens, max_rank,
                                   max_input_len);
    for (int i = 0; i < 5; ++i) slot->ids[i] = TensorId(*ts[i]);
    slot->n_tokens = n_tokens;
    slot->max_rank = max_rank;
    slot->max_input_len = max_input_len;
    slot->stream = stream;
    slot->device = device;
    slot->capture = capture;
    slot->used = clock_;
    ++builds_;
    return slot->plan;
  }
  int64_t hits() const { return hits_; }
  int64_t builds() const { return builds_; }
  void reset_stats() { hits_ = builds_ = 0; }

 private:
  std::mutex mu_;
  std::vector<Entry> entries_;
  uint64_t clock_ = 0;
  int64_t hits_ = 0, builds_ = 0;
  int streak_ = 0, paused_ = 0;
};

PrefillPlanCache& prefill_plan_cache() {
  static PrefillPlanCache* c = new PrefillPlanCache();
  return *c;
}

std::shared_ptr<SgmmPlan> resolve_prefill_plan(const py::object& plan, const Tensor& b_lora_start,
                                               const Tensor& b_lora_ranks, const Tensor& b_start_loc,
                                               const Tensor& b_seq_len, const Tensor& b_indicies, int64_t n_tokens,
                                               int64_t max_rank, int64_t max_input_len, void* stream, const char* what) {
  std::shared_ptr<SgmmPlan> p;
  if (plan.is_none()) {
    p = prefill_plan_cache().get(b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies, n_tokens, max_rank,
                                 max_input_len, stream);
  } else if (py::isinstance<py::bool_>(plan)) {
    TORCH_CHECK(!plan.cast<bool>(), "plan must be an SgmmPlan, None or False");
  } else {
    p = plan.cast<std::shared_ptr<SgmmPlan>>();
    TORCH_CHECK(p->n_requests == b_seq_len.numel() && p->n_tokens == n_tokens && p->max_rank == max_rank &&
                    p->max_input_len == max_input_len,
                what, ": the plan was built for another batch (", p->n_requests, " requests, ", p->n_tokens,
                " tokens, max_rank ", p->max_rank, ", max_input_len ", p->max_input_len, ")");
  }
  return (p && p->usable) ? p : nullptr;
}

void lora_get_qkvo_fwd_shrink(const Tensor& x, const Tensor& w, const Tensor& o, const Tensor& b_loc,
                              const Tensor& b_lora_start, const Tensor& b_lora_ranks, const Tensor& b_start_loc,
                              const Tensor& b_seq_len, const Tensor& b_indicies, int64_t hidden_size, int64_t qkvo,
                              int64_t max_rank, int64_t max_input_len, const py::object& plan) {
  const slora_tables t = prefill_common(x, w, o, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies);
  TORCH_CHECK(x.size(1) >= hidden_size && w.size(1) >= hidden_size && o.size(1) >= max_rank,
              "x/w narrower than hidden_size or o narrower than max_rank");
  void* stream = stream_of(x);
  const std::shared_ptr<SgmmPlan> p =
      resolve_prefill_plan(plan, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies, x.size(0), max_rank,
                           max_input_len, stream, "lora_get_qkvo_fwd_shrink");
  const int code = dtype_code(x, "x");
  int rc;
  if (p)
    rc = slora_sgmm_shrink_planned(p->buf.data_ptr(), o.data_ptr(), x.data_ptr(), w.data_ptr(), &t,
                                   b_start_loc.data_ptr<int32_t>(), b_seq_len.data_ptr<int32_t>(),
                                   b_indicies.data_ptr<int64_t>(), b_seq_len.numel(), max_input_len, x.size(0), hidden_size,
                                   max_rank, x.stride(0), w.stride(0), o.stride(0), w.size(0), (int)qkvo, code, stream);
  else
    rc = slora_sgmm_shrink(o.data_ptr(), x.data_ptr(), w.data_ptr(), &t, b_start_loc.data_ptr<int32_t>(),
                           b_seq_len.data_ptr<int32_t>(), b_indicies.data_ptr<int64_t>(), b_seq_len.numel(), max_input_len,
                           x.size(0), hidden_size, max_rank, x.stride(0), w.stride(0), o.stride(0), w.size(0), (int)qkvo,
                           code, stream);
  if (rc != SLORA_OK)
    check_rc(rc, "lora_get_qkvo_fwd_shrink",
             "(hidden_size=" + std::to_string(hidden_size) + " max_rank=" + std::to_string(max_rank) +
                 " qkvo=" + std::to_string(qkvo) + ")");
}

// q, k and v shrink of one layer in one pass over x (no counterpart in the reference, which
// issues the three calls of lora_unordered_batch_infer.py:334-347, 374-381, 400-407)
void lora_get_qkvo_fwd_shrink_qkv(const Tensor& x, const Tensor& w, const Tensor& o_q, const Tensor& o_k,
                                  const Tensor& o_v, const Tensor& b_loc, const Tensor& b_lora_start,
                                  const Tensor& b_lora_ranks, const Tensor& b_start_loc, const Tensor& b_seq_len,
                                  const Tensor& b_indicies, int64_t hidden_size, int64_t max_rank,
                                  int64_t max_input_len, const py::object& plan) {
  const slora_tables t = prefill_common(x, w, o_q, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies);
  check_2d_strided(o_k, "o_k");
  check_2d_strided(o_v, "o_v");
  TORCH_CHECK(o_k.scalar_type() == o_q.scalar_type() && o_v.scalar_type() == o_q.scalar_type() &&
                  o_k.sizes() == o_q.sizes() && o_v.sizes() == o_q.sizes() && o_k.stride(0) == o_q.stride(0) &&
                  o_v.stride(0) == o_q.stride(0),
              "o_q, o_k and o_v must share dtype, shape and row stride");
  TORCH_CHECK(x.size(1) >= hidden_size && w.size(1) >= hidden_size && o_q.size(1) >= max_rank,
              "x/w narrower than hidden_size or o narrower than max_rank");
  void* stream = stream_of(x);
  const std::shared_ptr<SgmmPlan> p =
      resolve_prefill_plan(plan, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies, x.size(0), max_rank,
                           max_input_len, stream, "lora_get_qkvo_fwd_shrink_qkv");
  const int rc = slora_sgmm_shrink_qkv(p ? p->buf.data_ptr() : nullptr, o_q.data_ptr(), o_k.data_ptr(), o_v.data_ptr(),
                                       x.data_ptr(), w.data_ptr(), &t, b_start_loc.data_ptr<int32_t>(),
                                       b_seq_len.data_ptr<int32_t>(), b_indicies.data_ptr<int64_t>(), b_seq_len.numel(),
                                       max_input_len, x.size(0), hidden_size, max_rank, x.stride(0), w.stride(0),
                                       o_q.stride(0), w.size(0), dtype_code(x, "x"), stream);
  if (rc != SLORA_OK)
    check_rc(rc, "lora_get_qkvo_fwd_shrink_qkv",
             "(hidden_size=" + std::to_string(hidden_size) + " max_rank=" + std::to_string(max_rank) + ")");
}

void lora_get_qkvo_fwd_expand(const Tensor& x, const Tensor& w, const Tensor& o, const Tensor& scale, const Tensor& b_loc,
                              const Tensor& b_lora_start, const Tensor& b_lora_ranks, const Tensor& b_start_loc,
                              const Tensor& b_seq_len, const Tensor& b_indicies, int64_t feat_out, int64_t qkvo,
                              int64_t max_rank, int64_t max_input_len) {
  const slora_tables t = prefill_common(x, w, o, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies);
  TORCH_CHECK(scale.is_cuda() && scale.is_contiguous(), "scale must be a contiguous CUDA tensor");
  const int sc = dtype_code(scale, "scale");
  TORCH_CHECK(scale.numel() >= b_lora_start.numel(), "scale must have one entry per adapter");
  TORCH_CHECK(o.size(1) >= feat_out && x.size(1) >= max_rank, "o narrower than feat_out or x narrower than max_rank");
  const int rc = slora_sgmm_expand(o.data_ptr(), x.data_ptr(), w.data_ptr(), &t, scale.data_ptr(), sc,
                                   b_start_loc.data_ptr<int32_t>(), b_seq_len.data_ptr<int32_t>(),
                                   b_indicies.data_ptr<int64_t>(), b_seq_len.numel(), max_input_len, x.size(0), feat_out,
                                   w.size(1), max_rank, x.stride(0), w.stride(0), o.stride(0), w.size(0), (int)qkvo,
                                   dtype_code(x, "x"), stream_of(x));
  if (rc != SLORA_OK)
    check_rc(rc, "lora_get_qkvo_fwd_expand",
             "(feat_out=" + std::to_string(feat_out) + " max_rank=" + std::to_string(max_rank) +
                 " qkvo=" + std::to_string(qkvo) + ")");
}

// q, k and v expand of one layer in one launch (no counterpart in the reference, which issues the
// three calls of lora_unordered_batch_infer.py:349-372, 383-398, 409-424): the results are those of the
// three calls bit for bit.  o_k and o_v share width and row stride (grouped-query models: narrower
// than o_q); x_q, x_k and x_v share shape and row stride.
void lora_get_qkvo_fwd_expand_qkv(const Tensor& x_q, const Tensor& x_k, const Tensor& x_v, const Tensor& w,
                                  const Tensor& o_q, const Tensor& o_k, const Tensor& o_v, const Tensor& scale,
                                  const Tensor& b_loc, const Tensor& b_lora_start, const Tensor& b_lora_ranks,
                                  const Tensor& b_start_loc, const Tensor& b_seq_len, const Tensor& b_indicies,
                                  int64_t feat_out_q, int64_t feat_out_kv, int64_t max_rank, int64_t max_input_len) {
  const slora_tables t = prefill_common(x_q, w, o_q, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies);
  for (const Tensor* a : {&x_k, &x_v, &o_k, &o_v}) check_2d_strided(*a, "x_k / x_v / o_k / o_v");
  TORCH_CHECK(x_k.scalar_type() == x_q.scalar_type() && x_v.scalar_type() == x_q.scalar_type() &&
                  o_k.scalar_type() == x_q.scalar_type() && o_v.scalar_type() == x_q.scalar_type(),
              "x_q, x_k, x_v, o_q, o_k and o_v must share their dtype");
  TORCH_CHECK(x_k.sizes() == x_q.sizes() && x_v.sizes() == x_q.sizes() && x_k.stride(0) == x_q.stride(0) &&
                  x_v.stride(0) == x_q.stride(0),
              "x_q, x_k and x_v must share shape and row stride");
  TORCH_CHECK(o_k.sizes() == o_v.sizes() && o_k.stride(0) == o_v.stride(0) && o_k.size(0) == o_q.size(0),
              "o_k and o_v must share shape and row stride, and have as many rows as o_q");
  TORCH_CHECK(scale.is_cuda() && scale.is_contiguous(), "scale must be a contiguous CUDA tensor");
  const int sc = dtype_code(scale, "scale");
  TORCH_CHECK(scale.numel() >= b_lora_start.numel(), "scale must have one entry per adapter");
  TORCH_CHECK(o_q.size(1) >= feat_out_q && o_k.size(1) >= feat_out_kv && x_q.size(1) >= max_rank,
              "o narrower than feat_out or x narrower than max_rank");
  const int rc = slora_sgmm_expand_qkv(o_q.data_ptr(), o_k.data_ptr(), o_v.data_ptr(), x_q.data_ptr(), x_k.data_ptr(),
                                       x_v.data_ptr(), w.data_ptr(), &t, scale.data_ptr(), sc,
                                       b_start_loc.data_ptr<int32_t>(), b_seq_len.data_ptr<int32_t>(),
                                       b_indicies.data_ptr<int64_t>(), b_seq_len.numel(), max_input_len, x_q.size(0),
                                       feat_out_q, feat_out_kv, w.size(1), max_rank, x_q.stride(0), w.stride(0),
                                       o_q.stride(0), o_k.stride(0), w.size(0), dtype_code(x_q, "x"), stream_of(x_q));
  if (rc != SLORA_OK)
    check_rc(rc, "lora_get_qkvo_fwd_expand_qkv",
             "(feat_out_q=" + std::to_string(feat_out_q) + " feat_out_kv=" + std::to_string(feat_out_kv) +
                 " max_rank=" + std::to_string(max_rank) + ")");
}

// ---------------------------------------------------------------------------
// pool helpers (slora/server/router/model_infer/infer_adapter.py, slora/common/mem_allocator.py)
// ---------------------------------------------------------------------------
void load_rows_into_pool(const std::vector<Tensor>& buffers, const std::vector<Tensor>& rows, const Tensor& loc) {
  TORCH_CHECK(buffers.size() == rows.size(), buffers.size(), " pool buffers but ", rows.size(), " row blocks");
  if (buffers.empty()) return;
  SL_CHECK_INPUT(loc);
  SL_CHECK_INDEX(loc);
  const int64_t n_rows = loc.numel();
  const Tensor& b0 = buffers[0];
  const int64_t row_elems = b0.size(0) > 0 ? b0.numel() / b0.size(0) : 0;
  std::vector<void*> dst(buffers.size());
  std::vector<const void*> src(buffers.size());
  for (size_t i = 0; i < buffers.size(); ++i) {
    const Tensor &b = buffers[i], &r = rows[i];
    TORCH_CHECK(b.is_cuda() && b.is_contiguous(), "buffers[", i, "] must be a contiguous CUDA tensor");
    TORCH_CHECK(r.is_cuda() && r.is_contiguous(), "rows[", i, "] must be a contiguous CUDA tensor");
    TORCH_CHECK(b.scalar_type() == b0.scalar_type() && r.scalar_type() == b0.scalar_type(),
                "pool buffers and rows must share one dtype");
    TORCH_CHECK(b.sizes() == b0.sizes(), "pool buffers must share one shape");
    TORCH_CHECK(r.dim() >= 1 && r.size(0) == n_rows && r.numel() == n_rows * row_elems, "rows[", i, "] must be [", n_rows,
                ", ...] with the pool's row shape, got ", r.sizes());
    dst[i] = b.data_ptr();
    src[i] = r.data_ptr();
  }
  const int64_t row_bytes = row_elems * b0.element_size();
  const int rc = slora_pool_scatter_rows(dst.data(), src.data(), (int)buffers.size(), loc.data_ptr<int64_t>(), n_rows,
                                         row_bytes, row_bytes, row_bytes, b0.size(0), stream_of(loc));
  check_rc(rc, "load_rows_into_pool");
  for (const Tensor& b : buffers) mark_written(b);
}

// (rows x cols) matrices written transposed into the pool pages loc[first .. first + n_slot)
void pack_transposed_into_pool(const std::vector<Tensor>& buffers, const std::vector<Tensor>& mats,
                               const std::vector<int64_t>& first, const std::vector<int64_t>& dst_pitch,
                               const std::vector<int64_t>& n_slot, const Tensor& loc) {
  const size_t n = buffers.size();
  TORCH_CHECK(mats.size() == n && first.size() == n && dst_pitch.size() == n && n_slot.size() == n,
              "buffers, mats, first, dst_pitch and n_slot must have one entry per matrix");
  if (n == 0) return;
  SL_CHECK_INPUT(loc);
  SL_CHECK_INDEX(loc);
  const Tensor& b0 = buffers[0];
  const int64_t page_elems = b0.size(0) > 0 ? b0.numel() / b0.size(0) : 0;
  std::vector<void*> dst(n);
  std::vector<const void*> src(n);
  std::vector<int64_t> rows(n), cols(n);
  for (size_t i = 0; i < n; ++i) {
    const Tensor &b = buffers[i], &m = mats[i];
    TORCH_CHECK(b.is_cuda() && b.is_contiguous(), "buffers[", i, "] must be a contiguous CUDA tensor");
    TORCH_CHECK(m.is_cuda() && m.is_contiguous() && m.dim() == 2, "mats[", i, "] must be a contiguous 2D CUDA tensor");
    TORCH_CHECK(b.element_size() == 2 && m.scalar_type() == b.scalar_type(),
                "pool buffers and matrices must share one 16-bit dtype");
    TORCH_CHECK(b.sizes() == b0.sizes(), "pool buffers must share one shape");
    dst[i] = b.data_ptr();
    src[i] = m.data_ptr();
    rows[i] = m.size(0);
    cols[i] = m.size(1);
  }
  const int rc = slora_pool_pack_transposed(dst.data(), src.data(), first.data(), rows.data(), cols.data(),
                                            dst_pitch.data(), n_slot.data(), (int)n, loc.data_ptr<int64_t>(), loc.numel(),
                                            page_elems, b0.size(0), stream_of(loc));
  check_rc(rc, "pack_transposed_into_pool");
  for (const Tensor& b : buffers) mark_written(b);
}

void launch_var_len_copy(const Tensor& old_a_start, const Tensor& old_a_len, const Tensor& old_location,
                         const Tensor& new_a_start, const Tensor& new_a_location) {
  for (const Tensor* t : {&old_a_start, &old_a_len, &old_location, &new_a_start, &new_a_location}) {
    TORCH_CHECK(t->is_cuda() && t->is_contiguous(), "index tables must be contiguous CUDA tensors");
    TORCH_CHECK(t->scalar_type() == at::kLong, "index tables must be int64 tensors, got ", t->scalar_type());
  }
  const int64_t n = old_a_start.numel();
  TORCH_CHECK(old_a_len.numel() == n && new_a_start.numel() == n,
              "old_a_start, old_a_len and new_a_start must have one entry per adapter");
  const int rc = slora_var_len_copy(old_a_start.data_ptr<int64_t>(), old_a_len.data_ptr<int64_t>(),
                                    old_location.data_ptr<int64_t>(), new_a_start.data_ptr<int64_t>(),
                                    new_a_location.data_ptr<int64_t>(), n, old_location.numel(), new_a_location.numel(),
                                    stream_of(old_location));
  check_rc(rc, "launch_var_len_copy");
  mark_written(new_a_location);
}

// outputs sized for the worst case; counts = {kept adapters, kept page ids, dropped adapters, dropped page ids}
std::vector<Tensor> compact_adapter_tables_raw(const Tensor& a_start, const Tensor& a_len, const Tensor& a_loc,
                                               const Tensor& a_scaling, const Tensor& keep) {
  SL_CHECK_INPUT(a_start);
  SL_CHECK_INPUT(a_len);
  SL_CHECK_INPUT(a_loc);
  SL_CHECK_INDEX(a_start);
  SL_CHECK_INDEX(a_len);
  SL_CHECK_INDEX(a_loc);
  SL_CHECK_INPUT(a_scaling);
  SL_CHECK_INPUT(keep);
  const int64_t n = a_start.numel(), n_loc = a_loc.numel();
  TORCH_CHECK(a_len.numel() == n && a_scaling.numel() == n && keep.numel() == n,
              "a_start, a_len, a_scaling and keep must have one entry per adapter");
  const int sc = dtype_code(a_scaling, "a_scaling");
  TORCH_CHECK(keep.scalar_type() == at::kBool || keep.scalar_type() == at::kByte, "keep must be a bool or uint8 tensor, got ",
              keep.scalar_type());
  const auto i64 = a_start.options();
  Tensor new_start = at::empty({n}, i64), new_len = at::empty({n}, i64), new_loc = at::empty({n_loc}, i64);
  Tensor new_scaling = at::empty({n}, a_scaling.options()), removed = at::empty({n_loc}, i64);
  Tensor counts = at::zeros({4}, i64), work = at::empty({std::max<int64_t>(n, 1)}, i64);
  const slora_tables t = tables_of(a_start, a_len, a_loc);
  const int rc = slora_tables_compact(&t, a_scaling.data_ptr(), sc, static_cast<const uint8_t*>(keep.data_ptr()),
                                      new_start.data_ptr<int64_t>(), new_len.data_ptr<int64_t>(),
                                      new_loc.data_ptr<int64_t>(), new_scaling.data_ptr(), removed.data_ptr<int64_t>(),
                                      counts.data_ptr<int64_t>(), work.data_ptr<int64_t>(), stream_of(a_start));
  check_rc(rc, "compact_adapter_tables");
  return {new_start, new_len, new_loc, new_scaling, removed, counts};
}

int64_t pool_alloc_workspace_bytes(int64_t tot_size) { return slora_pool_alloc_workspace_bytes(tot_size); }

void check_map(const Tensor& mem_state) {
  TORCH_CHECK(mem_state.is_cuda() && mem_state.is_contiguous() && mem_state.dim() == 1, "mem_state must be a contiguous 1D CUDA tensor");
  TORCH_CHECK(mem_state.scalar_type() == at::kBool || mem_state.scalar_type() == at::kByte, "mem_state must be bool or uint8");
}

void pool_alloc(const Tensor& mem_state, int64_t need, const Tensor& out_index, const Tensor& result, const Tensor& work) {
  check_map(mem_state);
  TORCH_CHECK(out_index.is_cuda() && out_index.scalar_type() == at::kLong && out_index.numel() >= need, "out_index must hold `need` int64");
  TORCH_CHECK(result.is_cuda() && result.scalar_type() == at::kLong && result.numel() >= 2, "result must hold two int64");
  TORCH_CHECK(work.is_cuda() && work.nbytes() >= (size_t)slora_pool_alloc_workspace_bytes(mem_state.numel()), "workspace too small");
  const int rc = slora_pool_alloc(static_cast<uint8_t*>(mem_state.data_ptr()), mem_state.numel(), need,
                                  out_index.data_ptr<int64_t>(), result.data_ptr<int64_t>(), work.data_ptr(),
                                  stream_of(mem_state));
  check_rc(rc, "PageAllocator.alloc");
  mark_written(mem_state);
  mark_written(out_index);
}

void pool_alloc_contiguous(const Tensor& mem_state, int64_t need, const Tensor& out_index, const Tensor& result,
                           const c10::optional<Tensor>& work) {
  check_map(mem_state);
  TORCH_CHECK(out_index.is_cuda() && out_index.scalar_type() == at::kLong && out_index.numel() >= need, "out_index must hold `need` int64");
  TORCH_CHECK(result.is_cuda() && result.scalar_type() == at::kLong && result.numel() >= 2, "result must hold two int64");
  int rc;
  if (work.has_value()) {
    TORCH_CHECK(work->is_cuda() && work->nbytes() >= (size_t)slora_pool_alloc_workspace_bytes(mem_state.numel()), "workspace too small");
    rc = slora_pool_alloc_contiguous(static_cast<uint8_t*>(mem_state.data_ptr()), mem_state.numel(), need,
                                     out_index.data_ptr<int64_t>(), result.data_ptr<int64_t>(), work->data_ptr(),
                                     stream_of(mem_state));
  } else {  // the library's own static workspace: nothing allocated
    rc = slora_pool_alloc_contiguous_static(static_cast<uint8_t*>(mem_state.data_ptr()), mem_state.numel(), need,
                                            out_index.data_ptr<int64_t>(), result.data_ptr<int64_t>(), stream_of(mem_state));
  }
  check_rc(rc, "PageAllocator.alloc_contiguous");
  mark_written(mem_state);
  mark_written(out_index);
}

void pool_free(const Tensor& mem_state, const Tensor& free_index) {
  check_map(mem_state);
  SL_CHECK_INPUT(free_index);
  SL_CHECK_INDEX(free_index);
  const int rc = slora_pool_free(static_cast<uint8_t*>(mem_state.data_ptr()), mem_state.numel(),
                                 free_index.data_ptr<int64_t>(), free_index.numel(), stream_of(mem_state));
  check_rc(rc, "PageAllocator.free");
  mark_written(mem_state);
}

// xor of the 32-bit words of every listed pool page (int32 tensor, one entry per page)
Tensor page_checksums(const Tensor& buffer, const Tensor& loc) {
  SL_CHECK_INPUT(buffer);
  SL_CHECK_INPUT(loc);
  SL_CHECK_INDEX(loc);
  TORCH_CHECK(buffer.dim() >= 1, "buffer must be [pages, ...]");
  const int64_t n_pages = buffer.size(0);
  const int64_t page_bytes = n_pages > 0 ? buffer.numel() / n_pages * buffer.element_size() : 0;
  Tensor out = at::empty({loc.numel()}, loc.options().dtype(at::kInt));
  const int rc = slora_pool_page_checksums(reinterpret_cast<uint32_t*>(out.data_ptr<int32_t>()), buffer.data_ptr(),
                                           loc.data_ptr<int64_t>(), loc.numel(), page_bytes, n_pages, stream_of(buffer));
  check_rc(rc, "page_checksums");
  return out;
}

// buffer[loc[i]] ^= key on every 32-bit word, in place (key 0: a pure read-modify-write)
void page_xor(Tensor& buffer, const Tensor& loc, int64_t key) {
  SL_CHECK_INPUT(buffer);
  SL_CHECK_INPUT(loc);
  SL_CHECK_INDEX(loc);
  TORCH_CHECK(buffer.dim() >= 1, "buffer must be [pages, ...]");
  TORCH_CHECK(key >= 0 && key <= 0xffffffffLL, "key must fit 32 bits");
  const int64_t n_pages = buffer.size(0);
  const int64_t page_bytes = n_pages > 0 ? buffer.numel() / n_pages * buffer.element_size() : 0;
  const int rc = slora_pool_page_xor(buffer.data_ptr(), loc.data_ptr<int64_t>(), loc.numel(), page_bytes, n_pages,
                                     static_cast<uint32_t>(key), stream_of(buffer));
  check_rc(rc, "page_xor");
  mark_written(buffer);
}

Tensor gather_lora_a(const Tensor& key_buffer, const Tensor& a_loc, int64_t first, int64_t rank, int64_t hidden,
                     int64_t out_cols) {
  SL_CHECK_INPUT(key_buffer);
  SL_CHECK_INPUT(a_loc);
  SL_CHECK_INDEX(a_loc);
  TORCH_CHECK(key_buffer.scalar_type() == at::kHalf || key_buffer.scalar_type() == at::kBFloat16,
              "key_buffer must be float16 or bfloat16");
  if (out_cols <= 0) out_cols = rank;
  const int64_t page_elems = key_buffer.size(0) > 0 ? key_buffer.numel() / key_buffer.size(0) : 0;
  Tensor out = at::empty({hidden, out_cols}, key_buffer.options());
  const int rc = slora_pool_gather_a(out.data_ptr(), out_cols, key_buffer.data_ptr(), a_loc.data_ptr<int64_t>(),
                                     a_loc.numel(), first, rank, hidden, page_elems, key_buffer.size(0),
                                     stream_of(key_buffer));
  check_rc(rc, "gather_lora_a");
  return out;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "MI355X-native multi-LoRA batching operators (HIP kernels of libslora_hip.so)";
  py::class_<BgmvPlan, std::shared_ptr<BgmvPlan>>(m, "BgmvPlan")
      .def_readonly("buf", &BgmvPlan::buf)
      .def_readonly("rank_cap", &BgmvPlan::rank_cap)
      .def_readonly("batch", &BgmvPlan::batch)
      .def_readwrite("n_items", &BgmvPlan::n_items)
      .def_readonly("max_rank", &BgmvPlan::max_rank)
      .def_readonly("n_runs", &BgmvPlan::n_runs)
      .def("status", [](const BgmvPlan& pl) { return plan_status_of(pl.buf); },
           "status word of the plan (waits for the current stream): 0, or bit 0 = a launch named another batch "
           "size or rank cap and did nothing, bit 1 = a hand-over of the one-launch LoRA was abandoned");
  py::class_<SgmmPlan, std::shared_ptr<SgmmPlan>>(m, "SgmmPlan")
      .def_readonly("buf", &SgmmPlan::buf)
      .def_readonly("usable", &SgmmPlan::usable)
      .def_readonly("n_requests", &SgmmPlan::n_requests)
      .def_readonly("n_tokens", &SgmmPlan::n_tokens)
      .def_readonly("max_rank", &SgmmPlan::max_rank)
      .def_readonly("max_input_len", &SgmmPlan::max_input_len)
      .def("status", [](const SgmmPlan& pl) { return plan_status_of(pl.buf); },
           "status word of the plan (waits for the current stream): 0, or 1 = a launch of another shape was given "
           "this plan and did nothing");

  m.def("slora_version", [] { return slora_version(); });
  m.def("dispatch_bgmv", &dispatch_bgmv, "dispatch_bgmv", py::arg("y"), py::arg("x"), py::arg("w"),
        py::arg("start_indicies"), py::arg("lora_ranks"), py::arg("loc_indicies"), py::arg("indicies"), py::arg("qkvo"),
        py::arg("lora_scales"), py::arg("plan") = py::none());
  m.def("dispatch_bgmv_qkv_shrink", &dispatch_bgmv_qkv_shrink, py::arg("y_q"), py::arg("y_k"), py::arg("y_v"),
        py::arg("x"), py::arg("w"), py::arg("start_indicies"), py::arg("lora_ranks"), py::arg("loc_indicies"),
        py::arg("indicies"), py::arg("plan") = py::none());
  m.def("dispatch_bgmv_qkv_expand", &dispatch_bgmv_qkv_expand, py::arg("y_q"), py::arg("y_k"), py::arg("y_v"),
        py::arg("x_q"), py::arg("x_k"), py::arg("x_v"), py::arg("w"), py::arg("start_indicies"), py::arg("lora_ranks"),
        py::arg("loc_indicies"), py::arg("indicies"), py::arg("lora_scales"), py::arg("plan") = py::none());
  m.def("dispatch_bgmv_lora", &dispatch_bgmv_lora, py::arg("y"), py::arg("delta"), py::arg("x"), py::arg("w_a"),
        py::arg("w_b"), py::arg("start_indicies"), py::arg("lora_ranks"), py::arg("loc_indicies"), py::arg("indicies"),
        py::arg("qkvo"), py::arg("lora_scales"), py::arg("plan") = py::none());
  m.def("dispatch_bgmv_qkv_lora", &dispatch_bgmv_qkv_lora, py::arg("y_q"), py::arg("y_k"), py::arg("y_v"), py::arg("d_q"),
        py::arg("d_k"), py::arg("d_v"), py::arg("x"), py::arg("w_a"), py::arg("w_b"), py::arg("start_indicies"),
        py::arg("lora_ranks"), py::arg("loc_indicies"), py::arg("indicies"), py::arg("lora_scales"),
        py::arg("plan") = py::none());
  m.def("make_plan", &make_plan, py::arg("start_indicies"), py::arg("lora_ranks"), py::arg("loc_indicies"),
        py::arg("indicies"), py::arg("rank_cap"), py::arg("n_pages"), py::arg("readback") = true);
  m.def("rebuild_plan", &rebuild_plan, py::arg("plan"), py::arg("start_indicies"), py::arg("lora_ranks"),
        py::arg("loc_indicies"), py::arg("indicies"), py::arg("n_pages"));
  m.def("clear_plan_cache", [] { plan_cache().clear(); });
  m.def("clear_prefill_plan_cache", [] { prefill_plan_cache().clear(); });
  m.def("set_plan_cache_enabled", [](bool on) { g_cache_enabled = on; });
  m.def("plan_cache_enabled", [] { return g_cache_enabled; });
  m.def("plan_cache_stats", [](bool reset) {
    py::dict d;
    d["hits"] = plan_cache().hits();
    d["builds"] = plan_cache().builds();
    d["prefill_hits"] = prefill_plan_cache().hits();
    d["prefill_builds"] = prefill_plan_cache().builds();
    if (reset) {
      plan_cache().reset_stats();
      prefill_plan_cache().reset_stats();
    }
    return d;
  }, py::arg("reset") = false);

  m.def("lora_get_qkvo_fwd_shrink", &lora_get_qkvo_fwd_shrink, py::arg("x"), py::arg("w"), py::arg("o"), py::arg("b_loc"),
        py::arg("b_lora_start"), py::arg("b_lora_ranks"), py::arg("b_start_loc"), py::arg("b_seq_len"),
        py::arg("b_indicies"), py::arg("hidden_size"), py::arg("qkvo"), py::arg("max_rank"), py::arg("max_input_len"),
        py::arg("plan") = py::none());
  m.def("lora_get_qkvo_fwd_shrink_qkv", &lora_get_qkvo_fwd_shrink_qkv, py::arg("x"), py::arg("w"), py::arg("o_q"),
        py::arg("o_k"), py::arg("o_v"), py::arg("b_loc"), py::arg("b_lora_start"), py::arg("b_lora_ranks"),
        py::arg("b_start_loc"), py::arg("b_seq_len"), py::arg("b_indicies"), py::arg("hidden_size"), py::arg("max_rank"),
        py::arg("max_input_len"), py::arg("plan") = py::none());
  m.def("lora_get_qkvo_fwd_expand", &lora_get_qkvo_fwd_expand, py::arg("x"), py::arg("w"), py::arg("o"), py::arg("scale"),
        py::arg("b_loc"), py::arg("b_lora_start"), py::arg("b_lora_ranks"), py::arg("b_start_loc"), py::arg("b_seq_len"),
        py::arg("b_indicies"), py::arg("feat_out"), py::arg("qkvo"), py::arg("max_rank"), py::arg("max_input_len"));
  m.def("lora_get_qkvo_fwd_expand_qkv", &lora_get_qkvo_fwd_expand_qkv, py::arg("x_q"), py::arg("x_k"), py::arg("x_v"),
        py::arg("w"), py::arg("o_q"), py::arg("o_k"), py::arg("o_v"), py::arg("scale"), py::arg("b_loc"),
        py::arg("b_lora_start"), py::arg("b_lora_ranks"), py::arg("b_start_loc"), py::arg("b_seq_len"),
        py::arg("b_indicies"), py::arg("feat_out_q"), py::arg("feat_out_kv"), py::arg("max_rank"),
        py::arg("max_input_len"));
  m.def("make_prefill_plan", &make_prefill_plan, py::arg("b_lora_start"), py::arg("b_lora_ranks"), py::arg("b_start_loc"),
        py::arg("b_seq_len"), py::arg("b_indicies"), py::arg("n_tokens"), py::arg("max_rank"), py::arg("max_input_len"));

  m.def("load_rows_into_pool", &load_rows_into_pool, py::arg("buffers"), py::arg("rows"), py::arg("loc"));
  m.def("pack_transposed_into_pool", &pack_transposed_into_pool, py::arg("buffers"), py::arg("mats"), py::arg("first"),
        py::arg("dst_pitch"), py::arg("n_slot"), py::arg("loc"));
  m.def("launch_var_len_copy", &launch_var_len_copy);
  m.def("compact_adapter_tables_raw", &compact_adapter_tables_raw);
  m.def("pool_alloc_workspace_bytes", &pool_alloc_workspace_bytes);
  m.def("pool_alloc", &pool_alloc);
  m.def("pool_alloc_contiguous", &pool_alloc_contiguous, py::arg("mem_state"), py::arg("need"), py::arg("out_index"),
        py::arg("result"), py::arg("work") = py::none());
  m.def("pool_free", &pool_free);
  m.def("page_checksums", &page_checksums, py::arg("buffer"), py::arg("loc"));
  m.def("page_xor", &page_xor, py::arg("buffer"), py::arg("loc"), py::arg("key") = 0);
  m.def("gather_lora_a", &gather_lora_a, py::arg("key_buffer"), py::arg("a_loc"), py::arg("first"), py::arg("rank"),
        py::arg("hidden"), py::arg("out_cols") = 0);
}
