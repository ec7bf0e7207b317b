// Torch binding of libmlora.so: the reference's op entry points under their own signatures, taking
// torch tensors -- what valora/csrc/lora_ops.cc:76-133 (dispatch_bgmv) and
// atmm/valora/csrc/lora_ops.cc:115-193 (dispatch_bgmv, imported as dispatch_sgmm) are in the
// reference, plus the Triton prefill pair valora/models/peft/triton_kernel/lora/lora_prefill.py:105-163.
// Every call checks its operands, finds the plan of the batch and makes ONE call through the C ABI
// (include/mlora.h) with that plan: host time per call is the pybind argument conversion plus one
// kernel launch.
//
// The plan of a batch is kept between calls.  The reference's caller passes the SAME tensors for the
// 8 calls of a layer and for all layers of a forward pass
// (valora/models/peft/lora_unordered_batch_infer.py:946-1063: batch_req_bins, a_start, a_len),
// sometimes as fresh views (output_counts[1:], start_ids[1:], :1006-1008).  A tensor is identified by
// (data_ptr, numel, dtype, version counter); the entry holds a reference to every tensor it was built
// from, which pins their storages: while the entry lives the caching allocator cannot hand the same
// address to another tensor, so an equal key means the same memory, and the version says it has not
// been written through PyTorch since.  Tensors created under inference_mode have no version counter;
// they are cached by address alone unless that is switched off.  Writes that bypass PyTorch (a foreign
// kernel given the raw pointer) are never seen: the cache can be disabled as a whole.
//
// Compiled by the host compiler alone (no device code); links libmlora.so, libtorch and libc10_hip
// (for the current stream).
#include <torch/extension.h>

#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "mlora.h"

namespace py = pybind11;

namespace {

[[noreturn]] void raise(const std::string &msg) { throw std::runtime_error(msg); }

void check_rc(int rc) {
  if (rc == MLORA_OK) return;
  const char *m = mlora_last_error();
  raise((m && *m) ? std::string(m) : "libmlora call failed with status " + std::to_string(rc));
}

// ---- the cache ------------------------------------------------------------------------------------
// Module state without locks: every entry point is called from Python with the GIL held.
constexpr int KEY_TENSORS = 8, KEY_SCALARS = 8;

struct Key {
  struct T {
    const void *ptr;
    int64_t numel;
    int64_t dtype;
    int64_t version;
  } t[KEY_TENSORS];
  int64_t s[KEY_SCALARS];
  int nt = 0, ns = 0;
  bool ok = true;  // false: one of the tensors cannot be identified, nothing is cached for it

  bool operator==(const Key &o) const {
    return nt == o.nt && ns == o.ns && std::memcmp(t, o.t, sizeof(T) * nt) == 0 &&
           std::memcmp(s, o.s, sizeof(int64_t) * ns) == 0;
  }
};

struct Entry {
  Key key;
  std::vector<at::Tensor> pins;
  py::object value;                   // what a Python user of the cache stored
  at::Tensor plan_buf, workspace, ids;  // a plan cut by the ops below
  mlora_plan plan{};
  unsigned long long capture = 0;     // id of the stream capture the plan's build was recorded into, or 0
};

std::vector<std::unique_ptr<Entry>> g_entries;  // most recently used last
size_t g_max_entries = 8;
bool g_enabled = true, g_cache_inference = true;
int64_t g_hits = 0, g_misses = 0;
int g_sgmm_shrink_mode = MLORA_SHRINK_OVERWRITE;

void key_tensor(Key &k, const at::Tensor &t) {
  if (k.nt >= KEY_TENSORS) raise("plan cache: too many tensors in one key");
  int64_t version = -1;
  if (t.is_inference()) {
    if (!g_cache_inference) k.ok = false;
  } else {
    version = (int64_t)t._version();
  }
  Key::T &e = k.t[k.nt++];
  std::memset(&e, 0, sizeof(e));
  e.ptr = t.data_ptr();
  e.numel = t.numel();
  e.dtype = (int64_t)t.scalar_type();
  e.version = version;
}

void key_scalar(Key &k, int64_t v) {
  if (k.ns >= KEY_SCALARS) raise("plan cache: too many scalars in one key");
  k.s[k.ns++] = v;
}

// Id of the capture `stream` is recording into, 0 if it is not capturing.
unsigned long long capture_id(hipStream_t stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  unsigned long long id = 0;
  if (hipStreamGetCaptureInfo(stream, &st, &id) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return st == hipStreamCaptureStatusActive ? (id ? id : ~0ull) : 0;
}

// The entry for `key` that may serve a call on `stream`.  A plan is valid in the context it was built in and in no
// other: one cut eagerly (capture == 0) for eager calls only -- recorded into a capture it would leave the graph
// without a build of its own, and every replay would reuse the tiles of the batch that happened to be in the ids
// tensor at warm-up, whatever the caller has written there since, from buffers this cache is free to drop -- and one
// whose build was only recorded (capture != 0) for calls recorded into the same capture.  A call under capture
// that finds none of its own builds a fresh plan inside the capture (its buffers come from the graph's memory pool
// and live as long as the graph); entries of a capture that is over are dropped when their key comes up again.
Entry *find(const Key &key, hipStream_t stream, bool native) {
  const unsigned long long now = native ? capture_id(stream) : 0;
  for (size_t i = g_entries.size(); i-- > 0;) {
    Entry *e = g_entries[i].get();
    if (!(e->key == key)) continue;
    if (native && e->capture != now) {
      if (e->capture != 0) g_entries.erase(g_entries.begin() + i);  // recorded into another capture: never cut eagerly
      continue;
    }
    if (i + 1 != g_entries.size()) {
      std::unique_ptr<Entry> keep = std::move(g_entries[i]);
      g_entries.erase(g_entries.begin() + i);
      g_entries.push_back(std::move(keep));
    }
    ++g_hits;
    return g_entries.back().get();
  }
  return nullptr;
}

Entry *insert(std::unique_ptr<Entry> e) {
  ++g_misses;
  g_entries.push_back(std::move(e));
  while (g_entries.size() > g_max_entries) g_entries.erase(g_entries.begin());
  return g_entries.back().get();
}

// ---- operand checks shared by the entry points --------------------------------------------------------
mlora_dtype dtype_code(const at::Tensor &t) {
  if (t.scalar_type() == at::kHalf) return MLORA_F16;
  if (t.scalar_type() == at::kBFloat16) return MLORA_BF16;
  return (mlora_dtype)-1;
}

std::string dtype_name(const at::Tensor &t) { return std::string("torch.") + c10::toString(t.scalar_type()); }

[[noreturn]] void no_kernel(int64_t h_in, int64_t h_out, const at::Tensor &x) {
  // valora/csrc/lora_ops.cc:122-125
  raise("No suitable kernel. h_in=" + std::to_string(h_in) + " h_out=" + std::to_string(h_out) + " dtype=" +
        dtype_name(x));
}

void check_input(const at::Tensor &t, const char *name) {
  // CHECK_INPUT = CHECK_CUDA + CHECK_CONTIGUOUS (valora/csrc/lora_ops.cc:27-34)
  if (!t.is_cuda()) raise(std::string(name) + " must be a CUDA tensor");
  if (!t.is_contiguous()) raise(std::string(name) + " must be contiguous");
}

void check_long(const at::Tensor &t, const char *name) {
  // data_ptr<int64_t>() throws on any other type
  if (t.scalar_type() != at::kLong)
    raise(std::string("expected scalar type Long but found ") + c10::toString(t.scalar_type()) + " (" + name + ")");
}

void check_common(const at::Tensor &y, const at::Tensor &x, const at::Tensor &w, const at::Tensor &a_start,
                  const at::Tensor &a_len, const at::Tensor &a_loc, const at::Tensor &ids) {
  check_input(y, "y");
  check_input(x, "x");
  check_input(w, "w");
  check_input(a_start, "start_indicies");
  check_input(a_len, "lora_ranks");
  check_input(a_loc, "loc_indicies");
  check_input(ids, "indicies");
  if (y.dim() != 2) raise("y must be a 2D tensor");
  if (x.dim() != 2) raise("x must be a 2D tensor");
  if (w.dim() != 3) raise("w must be a 3D tensor");
  if (ids.dim() != 1) raise("indicies must be a 1D tensor");
  if (ids.size(0) != x.size(0))
    raise("CHECK_EQ(indicies.size(0), x.size(0)) failed. " + std::to_string(ids.size(0)) + " vs " +
          std::to_string(x.size(0)));
  if (y.size(0) != x.size(0))
    raise("CHECK_EQ(y.size(0), x.size(0)) failed. " + std::to_string(y.size(0)) + " vs " + std::to_string(x.size(0)));
  check_long(a_start, "start_indicies");
  check_long(a_len, "lora_ranks");
  check_long(a_loc, "loc_indicies");
  check_long(ids, "indicies");
}

mlora_pool make_pool(const at::Tensor &w, const at::Tensor &a_start, const at::Tensor &a_len, const at::Tensor &a_loc,
                     int64_t row_width) {
  // w: the pool viewed as rows of row_width elements (the reference passes [rows, heads, head_dim])
  mlora_pool p;
  p.w = w.data_ptr();
  p.w_rows = row_width > 0 ? w.numel() / row_width : 0;
  p.a_start = static_cast<const int64_t *>(a_start.data_ptr());
  p.a_len = static_cast<const int64_t *>(a_len.data_ptr());
  p.a_loc = static_cast<const int64_t *>(a_loc.data_ptr());
  p.n_adapters = a_start.numel();
  p.a_loc_len = a_loc.numel();
  p.n_slots = 4;
  return p;
}

// The stream the call's kernels go to: PyTorch's current stream on the operands' device, which has to be the
// current device (the library launches on the current device; the reference's binding has the same contract).
hipStream_t current_stream(const at::Tensor &t) {
  const auto dev = t.get_device();
  if (dev != c10::hip::current_device())
    raise("operands live on cuda:" + std::to_string(dev) + " but the current device is cuda:" +
          std::to_string(c10::hip::current_device()) + " (use torch.cuda.device)");
  return c10::hip::getCurrentHIPStream(dev).stream();
}

void check_same_device(const at::Tensor &ref, std::initializer_list<const at::Tensor *> ts) {
  for (const at::Tensor *t : ts)
    if (t->defined() && t->is_cuda() && t->get_device() != ref.get_device())
      raise("all operands must live on one device");
}

at::Tensor device_bytes(size_t n, const at::Tensor &like) {
  return at::empty({(int64_t)std::max<size_t>(n, 256)}, like.options().dtype(at::kByte));
}

bool cacheable(int64_t T, int64_t narrow, int64_t wide) {
  // everything else goes to the one-call form, which reports the reference's errors for it
  return g_enabled && T > 0 && narrow > 0 && narrow <= 128 && (narrow % 8) == 0 && narrow < wide;
}

// The plan for `key`: from the cache, or cut now from the ids make_ids() returns (int64[T] on the device;
// the tensor lives as long as the entry).
template <typename MakeIds>
Entry *plan_for(const Key &key, hipStream_t stream, std::initializer_list<at::Tensor> pins, const mlora_pool &pool,
                int64_t T, int64_t narrow, int64_t wide, const at::Tensor &like, MakeIds make_ids) {
  if (Entry *e = find(key, stream, true)) return e;
  auto e = std::make_unique<Entry>();
  e->key = key;
  e->pins.assign(pins.begin(), pins.end());
  e->capture = capture_id(stream);
  mlora_tile_config cfg;
  check_rc(mlora_tile_lookup(T, narrow, wide, pool.n_adapters, &cfg));
  e->ids = make_ids();
  e->plan_buf = device_bytes(mlora_plan_bytes(T, pool.n_adapters), like);
  e->plan.dev = e->plan_buf.data_ptr();
  e->plan.bytes = (size_t)e->plan_buf.numel();
  check_rc(mlora_build_plan(stream, &e->plan, static_cast<const int64_t *>(e->ids.data_ptr()), T, pool.a_start,
                            pool.a_len, pool.n_adapters, pool.n_slots, cfg.bm_shrink, cfg.bm_expand));
  e->workspace = device_bytes(mlora_workspace_bytes(T, pool.n_adapters, narrow), like);
  return insert(std::move(e));
}

const void *scales_ptr(const c10::optional<at::Tensor> &scales, const at::Tensor &x, at::Tensor &keep) {
  if (!scales.has_value() || !scales->defined()) return nullptr;
  if (scales->scalar_type() == x.scalar_type()) return scales->data_ptr();
  keep = scales->to(x.scalar_type());  // the kernel reads scales in the operand type (bgmv_impl.cuh:180)
  return keep.data_ptr();
}

// ---- dispatch_bgmv (valora/csrc/lora_ops.cc:76-126) ---------------------------------------------------
void dispatch_bgmv(const at::Tensor &y, const at::Tensor &x, const at::Tensor &w, const at::Tensor &a_start,
                   const at::Tensor &a_len, const at::Tensor &a_loc, const at::Tensor &ids, int64_t qkvo,
                   const c10::optional<at::Tensor> &lora_scales) {
  check_common(y, x, w, a_start, a_len, a_loc, ids);
  check_same_device(x, {&y, &w, &a_start, &a_len, &a_loc, &ids});
  const int64_t T = x.size(0), h_in = x.size(1), h_out = y.size(1);
  const mlora_dtype code = dtype_code(x);
  if ((int)code < 0 || y.scalar_type() != x.scalar_type() || w.scalar_type() != x.scalar_type() || h_in >= 65536 ||
      h_out >= 65536)
    no_kernel(h_in, h_out, x);
  const int64_t wide = std::max(h_in, h_out), narrow = std::min(h_in, h_out);
  at::Tensor keep;
  const void *scales = scales_ptr(lora_scales, x, keep);
  const mlora_pool pool = make_pool(w, a_start, a_len, a_loc, wide);
  const hipStream_t stream = current_stream(x);
  const int64_t *ids_p = static_cast<const int64_t *>(ids.data_ptr());
  if (cacheable(T, narrow, wide)) {
    Key key;
    key_tensor(key, ids);
    key_tensor(key, a_start);
    key_tensor(key, a_len);
    key_scalar(key, 0);  // which entry point
    key_scalar(key, T);
    key_scalar(key, narrow);
    key_scalar(key, wide);
    key_scalar(key, x.get_device());
    if (key.ok) {
      Entry *e = plan_for(key, stream, {ids, a_start, a_len}, pool, T, narrow, wide, x, [&] { return ids; });
      check_rc(mlora_dispatch_bgmv(stream, y.data_ptr(), x.data_ptr(), &pool, ids_p, qkvo, scales, T, h_in, h_out, code,
                                   e->workspace.data_ptr(), (size_t)e->workspace.numel(), &e->plan));
      return;
    }
  }
  at::Tensor ws = device_bytes(mlora_workspace_bytes(T, pool.n_adapters, narrow), x);
  check_rc(mlora_dispatch_bgmv(stream, y.data_ptr(), x.data_ptr(), &pool, ids_p, qkvo, scales, T, h_in, h_out, code,
                               ws.data_ptr(), (size_t)ws.numel(), nullptr));
}

// ---- dispatch_sgmm (atmm/valora/csrc/lora_ops.cc:115-186) ----------------------------------------------
// Rows of the first num_problems segments [start_ids[i], start_ids[i] + output_counts[i]) are processed, each
// with the adapter its per-token id names; rank_counts, lora_ids and the tile arguments are accepted and
// ignored; tmp_d serves as workspace when it is large enough.
void dispatch_sgmm(const at::Tensor &y, const at::Tensor &x, const at::Tensor &w, const at::Tensor &a_start,
                   const at::Tensor &a_len, const at::Tensor &a_loc, const at::Tensor &ids, int64_t qkvo,
                   const c10::optional<at::Tensor> &lora_scales, const at::Tensor &output_counts,
                   const py::object & /*rank_counts*/, const py::object & /*lora_ids*/, const at::Tensor &start_ids,
                   const c10::optional<at::Tensor> &tmp_d, int64_t num_problems, int64_t, int64_t, int64_t, int64_t,
                   int64_t, int64_t) {
  check_common(y, x, w, a_start, a_len, a_loc, ids);
  check_same_device(x, {&y, &w, &a_start, &a_len, &a_loc, &ids, &output_counts, &start_ids});
  const int64_t T = x.size(0), h_in = x.size(1), h_out = y.size(1);
  const mlora_dtype code = dtype_code(x);
  if ((int)code < 0 || y.scalar_type() != x.scalar_type() || w.scalar_type() != x.scalar_type() || h_in >= 65536 ||
      h_out >= 65536)
    no_kernel(h_in, h_out, x);
  if (!output_counts.is_cuda() || output_counts.scalar_type() != at::kLong)
    raise("expected a CUDA Long tensor (output_counts)");
  if (!start_ids.is_cuda() || start_ids.scalar_type() != at::kLong) raise("expected a CUDA Long tensor (start_ids)");
  const int64_t P = num_problems;
  if (P > output_counts.numel() || P > start_ids.numel())
    raise("num_problems=" + std::to_string(P) + " exceeds the segment tensors");
  const int64_t wide = std::max(h_in, h_out), narrow = std::min(h_in, h_out);
  at::Tensor keep;
  const void *scales = scales_ptr(lora_scales, x, keep);
  const mlora_pool pool = make_pool(w, a_start, a_len, a_loc, wide);
  const hipStream_t stream = current_stream(x);
  const at::Tensor oc = output_counts.contiguous(), st = start_ids.contiguous();
  const int64_t *ids_p = static_cast<const int64_t *>(ids.data_ptr());
  const int64_t *oc_p = static_cast<const int64_t *>(oc.data_ptr()), *st_p = static_cast<const int64_t *>(st.data_ptr());
  if (cacheable(T, narrow, wide)) {
    Key key;
    key_tensor(key, ids);
    key_tensor(key, a_start);
    key_tensor(key, a_len);
    key_tensor(key, oc);
    key_tensor(key, st);
    key_scalar(key, 1);
    key_scalar(key, T);
    key_scalar(key, narrow);
    key_scalar(key, wide);
    key_scalar(key, x.get_device());
    key_scalar(key, P);
    if (key.ok) {
      Entry *e = plan_for(key, stream, {ids, a_start, a_len, oc, st}, pool, T, narrow, wide, x, [&] {
        at::Tensor eff = at::empty({T}, ids.options());
        check_rc(mlora_ids_from_segments(stream, static_cast<int64_t *>(eff.data_ptr()), ids_p, st_p, oc_p, P, T));
        return eff;
      });
      check_rc(mlora_dispatch_sgmm(stream, y.data_ptr(), x.data_ptr(), &pool, ids_p, qkvo, scales, oc_p, st_p, P, T, h_in,
                                   h_out, code, g_sgmm_shrink_mode, e->workspace.data_ptr(), (size_t)e->workspace.numel(),
                                   &e->plan));
      return;
    }
  }
  const size_t need = mlora_workspace_bytes(T, pool.n_adapters, narrow);
  at::Tensor ws;
  if (tmp_d.has_value() && tmp_d->defined() && tmp_d->is_cuda() && tmp_d->is_contiguous() && tmp_d->element_size() == 1 &&
      (size_t)tmp_d->numel() >= need && (reinterpret_cast<uintptr_t>(tmp_d->data_ptr()) % 16) == 0)
    ws = *tmp_d;
  else
    ws = device_bytes(need, x);
  check_rc(mlora_dispatch_sgmm(stream, y.data_ptr(), x.data_ptr(), &pool, ids_p, qkvo, scales, oc_p, st_p, P, T, h_in,
                               h_out, code, g_sgmm_shrink_mode, ws.data_ptr(), (size_t)ws.numel(), nullptr));
}

// ---- the Triton prefill pair (lora_prefill.py:105-163) -------------------------------------------------
struct Requests {
  at::Tensor start, len, idx;  // int32, int32, int64, contiguous (infer_batch.py:77,106 builds them so)
  Requests(const at::Tensor &b_start_loc, const at::Tensor &b_seq_len, const at::Tensor &b_indicies)
      : start(b_start_loc.to(at::kInt).contiguous()), len(b_seq_len.to(at::kInt).contiguous()),
        idx(b_indicies.to(at::kLong).contiguous()) {}
  const int32_t *s() const { return static_cast<const int32_t *>(start.data_ptr()); }
  const int32_t *n() const { return static_cast<const int32_t *>(len.data_ptr()); }
  const int64_t *i() const { return static_cast<const int64_t *>(idx.data_ptr()); }
};

// The plan of a batch given by per-request operands, or nullptr where only the one-call form reports properly.
Entry *request_plan(hipStream_t stream, const at::Tensor &like, const mlora_pool &pool, const at::Tensor &b_lora_start,
                    const at::Tensor &b_lora_ranks, const at::Tensor &b_start_loc, const at::Tensor &b_seq_len,
                    const at::Tensor &b_indicies, int64_t T, int64_t max_rank, int64_t wide, int64_t max_input_len) {
  const int64_t narrow = std::max<int64_t>(8, (max_rank + 7) / 8 * 8);
  if (T <= 0 || b_seq_len.numel() == 0 || max_rank <= 0 || !cacheable(T, narrow, wide)) return nullptr;
  if (b_lora_start.scalar_type() != at::kLong || b_lora_ranks.scalar_type() != at::kLong) return nullptr;
  const int64_t max_rows = (max_input_len + 31) / 32 * 32;  // rows visited per request (lora_prefill.py:147)
  Key key;
  key_tensor(key, b_indicies);
  key_tensor(key, b_lora_start);
  key_tensor(key, b_lora_ranks);
  key_tensor(key, b_start_loc);
  key_tensor(key, b_seq_len);
  key_scalar(key, 2);
  key_scalar(key, T);
  key_scalar(key, narrow);
  key_scalar(key, wide);
  key_scalar(key, like.get_device());
  key_scalar(key, max_rows);
  if (!key.ok) return nullptr;
  return plan_for(key, stream, {b_indicies, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len}, pool, T, narrow, wide,
                  like, [&] {
                    Requests r(b_start_loc, b_seq_len, b_indicies);
                    at::Tensor eff = at::empty({T}, r.idx.options());
                    check_rc(mlora_ids_from_requests(stream, static_cast<int64_t *>(eff.data_ptr()), r.s(), r.n(), r.i(),
                                                     r.len.numel(), T, max_rows));
                    return eff;
                  });
}

void check_requests(const at::Tensor &b_start_loc, const at::Tensor &b_seq_len, const at::Tensor &b_indicies) {
  if (!b_start_loc.is_cuda() || !b_seq_len.is_cuda() || !b_indicies.is_cuda())
    raise("b_start_loc, b_seq_len and b_indicies must be CUDA tensors");
}

void check_index(const at::Tensor &b_loc, const at::Tensor &b_lora_start, const at::Tensor &b_lora_ranks) {
  check_input(b_loc, "b_loc");
  check_input(b_lora_start, "b_lora_start");
  check_input(b_lora_ranks, "b_lora_ranks");
  check_long(b_loc, "b_loc");
  check_long(b_lora_start, "b_lora_start");
  check_long(b_lora_ranks, "b_lora_ranks");
}

// o[t, :max_rank] = x[t] @ A_a.T for the rows of every request; columns >= r are zero-filled, rows past
// max_input_len rounded up to 32 are not visited.
void lora_get_qkvo_fwd_shrink(const at::Tensor &x, const at::Tensor &w, const at::Tensor &o, const at::Tensor &b_loc,
                              const at::Tensor &b_lora_start, const at::Tensor &b_lora_ranks,
                              const at::Tensor &b_start_loc, const at::Tensor &b_seq_len, const at::Tensor &b_indicies,
                              int64_t hidden_size, int64_t qkvo, int64_t max_rank, int64_t max_input_len) {
  const mlora_dtype code = dtype_code(x);
  if ((int)code < 0 || w.scalar_type() != x.scalar_type() || o.scalar_type() != x.scalar_type())
    no_kernel(hidden_size, max_rank, x);
  if (x.dim() != 2 || o.dim() != 2 || x.stride(1) != 1 || o.stride(1) != 1 || x.stride(0) != hidden_size ||
      !w.is_contiguous())
    raise("x rows must be dense, o and w must have unit inner stride");
  if (!x.is_cuda() || !o.is_cuda() || !w.is_cuda()) raise("x, w and o must be CUDA tensors");
  check_index(b_loc, b_lora_start, b_lora_ranks);
  check_requests(b_start_loc, b_seq_len, b_indicies);
  check_same_device(x, {&w, &o, &b_loc, &b_lora_start, &b_lora_ranks, &b_start_loc, &b_seq_len, &b_indicies});
  const int64_t T = x.size(0);
  const mlora_pool pool = make_pool(w, b_lora_start, b_lora_ranks, b_loc, hidden_size);
  const hipStream_t stream = current_stream(x);
  if (Entry *e = request_plan(stream, x, pool, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies, T,
                              max_rank, hidden_size, max_input_len)) {
    check_rc(mlora_prefill_shrink(stream, o.data_ptr(), x.data_ptr(), &pool, nullptr, nullptr, nullptr,
                                  b_seq_len.numel(), T, hidden_size, o.stride(0), qkvo, max_rank, max_input_len, code,
                                  e->workspace.data_ptr(), (size_t)e->workspace.numel(), &e->plan));
    return;
  }
  Requests r(b_start_loc, b_seq_len, b_indicies);
  at::Tensor ws = device_bytes(mlora_workspace_bytes(T, pool.n_adapters, std::max<int64_t>(8, (max_rank + 7) / 8 * 8)), x);
  check_rc(mlora_prefill_shrink(stream, o.data_ptr(), x.data_ptr(), &pool, r.s(), r.n(), r.i(), r.len.numel(), T,
                                hidden_size, o.stride(0), qkvo, max_rank, max_input_len, code, ws.data_ptr(),
                                (size_t)ws.numel(), nullptr));
}

// o[t] += scale_a * x[t, :r] @ B_a for the rows of every request.
void lora_get_qkvo_fwd_expand(const at::Tensor &x, const at::Tensor &w, const at::Tensor &o, const at::Tensor &scale,
                              const at::Tensor &b_loc, const at::Tensor &b_lora_start, const at::Tensor &b_lora_ranks,
                              const at::Tensor &b_start_loc, const at::Tensor &b_seq_len, const at::Tensor &b_indicies,
                              int64_t feat_out, int64_t qkvo, int64_t max_rank, int64_t max_input_len) {
  const mlora_dtype code = dtype_code(x);
  if ((int)code < 0 || w.scalar_type() != x.scalar_type() || o.scalar_type() != x.scalar_type())
    no_kernel(max_rank, feat_out, x);
  if (x.dim() != 2 || o.dim() != 2 || x.stride(1) != 1 || o.stride(1) != 1 || o.stride(0) != feat_out ||
      !w.is_contiguous())
    raise("o rows must be dense, x and w must have unit inner stride");
  if (!x.is_cuda() || !o.is_cuda() || !w.is_cuda() || !scale.is_cuda()) raise("x, w, o and scale must be CUDA tensors");
  check_index(b_loc, b_lora_start, b_lora_ranks);
  check_requests(b_start_loc, b_seq_len, b_indicies);
  check_same_device(x, {&w, &o, &scale, &b_loc, &b_lora_start, &b_lora_ranks, &b_start_loc, &b_seq_len, &b_indicies});
  const int64_t T = o.size(0);
  at::Tensor keep;
  const void *scales = scales_ptr(scale, x, keep);
  const mlora_pool pool = make_pool(w, b_lora_start, b_lora_ranks, b_loc, feat_out);
  const hipStream_t stream = current_stream(x);
  if (Entry *e = request_plan(stream, x, pool, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies, T,
                              max_rank, feat_out, max_input_len)) {
    check_rc(mlora_prefill_expand(stream, o.data_ptr(), x.data_ptr(), &pool, scales, nullptr, nullptr, nullptr,
                                  b_seq_len.numel(), T, x.stride(0), feat_out, qkvo, max_rank, max_input_len, code,
                                  nullptr, 0, &e->plan));
    return;
  }
  Requests r(b_start_loc, b_seq_len, b_indicies);
  at::Tensor ws = device_bytes(mlora_workspace_bytes(T, pool.n_adapters, std::max<int64_t>(8, (max_rank + 7) / 8 * 8)), x);
  check_rc(mlora_prefill_expand(stream, o.data_ptr(), x.data_ptr(), &pool, scales, r.s(), r.n(), r.i(), r.len.numel(), T,
                                x.stride(0), feat_out, qkvo, max_rank, max_input_len, code, ws.data_ptr(),
                                (size_t)ws.numel(), nullptr));
}

// ---- the cache as Python sees it ---------------------------------------------------------------------
Key python_key(const std::vector<at::Tensor> &tensors, const std::vector<int64_t> &scalars) {
  Key key;
  for (const at::Tensor &t : tensors) key_tensor(key, t);
  key_scalar(key, -1);  // never equal to an entry of the ops above
  for (int64_t v : scalars) key_scalar(key, v);
  return key;
}

// The stored value, or None; `identifiable` False means nothing can be cached for these tensors.
py::tuple cache_lookup(const std::vector<at::Tensor> &tensors, const std::vector<int64_t> &scalars) {
  const Key key = python_key(tensors, scalars);
  if (!key.ok || !g_enabled) return py::make_tuple(false, py::none());
  Entry *e = find(key, nullptr, false);
  return py::make_tuple(true, e ? e->value : py::object(py::none()));
}

void cache_insert(const std::vector<at::Tensor> &tensors, const std::vector<int64_t> &scalars, py::object value) {
  const Key key = python_key(tensors, scalars);
  if (!key.ok || !g_enabled) return;
  auto e = std::make_unique<Entry>();
  e->key = key;
  e->pins = tensors;
  e->value = std::move(value);
  insert(std::move(e));
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "torch binding of libmlora.so: the reference's LoRA op entry points";
  m.def("dispatch_bgmv", &dispatch_bgmv, py::arg("y"), py::arg("x"), py::arg("w"), py::arg("start_indicies"),
        py::arg("lora_ranks"), py::arg("loc_indicies"), py::arg("indicies"), py::arg("qkvo"), py::arg("lora_scales"),
        "In place on y.  h_in > h_out: shrink y[t, :r] = x[t] @ A_a.T (columns >= r keep their value); "
        "h_in < h_out: expand y[t] += scale_a * x[t, :r] @ B_a.  lora_ranks holds 4 * r; w is the pool "
        "[rows, heads, head_dim] whose row width is the wide dimension of the call.");
  m.def("dispatch_sgmm", &dispatch_sgmm, py::arg("y"), py::arg("x"), py::arg("w"), py::arg("start_indicies"),
        py::arg("lora_ranks"), py::arg("loc_indicies"), py::arg("indicies"), py::arg("qkvo"), py::arg("lora_scales"),
        py::arg("output_counts"), py::arg("rank_counts"), py::arg("lora_ids"), py::arg("start_ids"), py::arg("tmp_d"),
        py::arg("num_problems"), py::arg("tb_x") = 0, py::arg("tb_y") = 0, py::arg("tb_z") = 0, py::arg("wp_x") = 0,
        py::arg("wp_y") = 0, py::arg("wp_z") = 0,
        "dispatch_bgmv of the segment signature: rows of the first num_problems segments only.");
  m.def("lora_get_qkvo_fwd_shrink", &lora_get_qkvo_fwd_shrink, py::arg("x"), py::arg("w"), py::arg("o"), py::arg("b_loc"),
        py::arg("b_lora_start"), py::arg("b_lora_ranks"), py::arg("b_start_loc"), py::arg("b_seq_len"),
        py::arg("b_indicies"), py::arg("hidden_size"), py::arg("qkvo"), py::arg("max_rank"), py::arg("max_input_len"));
  m.def("lora_get_qkvo_fwd_expand", &lora_get_qkvo_fwd_expand, py::arg("x"), py::arg("w"), py::arg("o"), py::arg("scale"),
        py::arg("b_loc"), py::arg("b_lora_start"), py::arg("b_lora_ranks"), py::arg("b_start_loc"), py::arg("b_seq_len"),
        py::arg("b_indicies"), py::arg("feat_out"), py::arg("qkvo"), py::arg("max_rank"), py::arg("max_input_len"));
  m.def("shrink_accumulate", [](bool on) { g_sgmm_shrink_mode = on ? MLORA_SHRINK_ACCUMULATE : MLORA_SHRINK_OVERWRITE; },
        "True: the segment signature's shrink adds into y (D = X*W + C, atmm/valora/csrc/bgmv/bgmv_impl.cuh:174) "
        "instead of overwriting it.");
  m.def("cache_lookup", &cache_lookup);
  m.def("cache_insert", &cache_insert);
  m.def("cache_clear", [] { g_entries.clear(); });
  m.def("cache_size", [] { return g_entries.size(); });
  m.def("cache_hits", [] { return g_hits; });
  m.def("cache_misses", [] { return g_misses; });
  m.def("cache_enabled", [] { return g_enabled; });
  m.def("cache_set_enabled", [](bool on) {
    g_enabled = on;
    if (!on) g_entries.clear();
  });
  m.def("cache_inference_tensors", [] { return g_cache_inference; });
  m.def("cache_set_inference_tensors", [](bool on) { g_cache_inference = on; });
  m.def("cache_max_entries", [] { return g_max_entries; });
  // the entries hold device tensors and Python objects: let go of them while the interpreter and the HIP
  // runtime are still there
  py::module_::import("atexit").attr("register")(py::cpp_function([] { g_entries.clear(); }));
}
