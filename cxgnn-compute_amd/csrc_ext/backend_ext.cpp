// cxgnncomp_backend._C -- the compiled part of the drop-in for the reference's pybind module
// (src/cpp/python_bindings/binding.cpp:14-130).
//
// A thin host layer over the C ABI of libcxgnn_hip.so (include/cxgnn_hip.h): it checks tensors,
// allocates results through torch, takes the current HIP stream of the tensors' device and calls
// the library.  What the reference implements as torch::autograd::Function in C++ is one here too:
//   SAGEFunction / SAGEEdgeValueFunction   src/cpp/src/aggr.cu:107-303   -> SageFunction
//   EdgeSoftMaxFunction                    src/cpp/src/edge_softmax.cu:97-177 -> EdgeSoftmaxFunction
//   GatherFunction                         src/cpp/src/aggr.cu:395-448   -> GatherFunction
//   AggrRelFunction                        src/cpp/src/rel_spmm.cu:37-136 -> AggrRelFunction
// together with the plain entry points of the SpMM / SDDMM families (spmm_host.cu, sddmm_host.cu)
// and the cache of transposed graphs that their backward passes gather over.  The relational,
// typed-GEMM and scheduling entry points are bound from Python (cxgnncomp_backend/_typed.py,
// _rel.py, _schedule.py) on the same C ABI.
//
// Differences from the reference's module, all deliberate: errors are Python exceptions
// (ValueError for bad arguments, RuntimeError otherwise), not exit(1); autograd contexts keep the
// graph tensors alive instead of raw pointers (aggr.cu:116-117); kernels run on the current
// stream of the tensors' device.
#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <list>
#include <map>
#include <memory>
#include <atomic>
#include <mutex>
#include <string>
#include <tuple>

#include "cxgnn_hip.h"

namespace {

using torch::Tensor;
using OptTensor = c10::optional<Tensor>;
using torch::autograd::AutogradContext;
using torch::autograd::tensor_list;

constexpr unsigned kSpmmMean = CXG_SPMM_MEAN;
constexpr unsigned kSpmmAccumulate = CXG_SPMM_ACCUMULATE;
constexpr unsigned kSpmmExactEdges = CXG_SPMM_HINT_EXACT_EDGES;

// ---------------------------------------------------------------------------------------------
// small helpers
// ---------------------------------------------------------------------------------------------
template <typename... Args>
std::string fmt(const char* f, Args... args) {
  char buf[512];
  snprintf(buf, sizeof(buf), f, args...);
  return std::string(buf);
}

[[noreturn]] void bad(const std::string& msg) { throw py::value_error(msg); }

void check(int status) {
  if (status == 0) return;
  const std::string msg = cxg_last_error();
  if (status == CXG_ERR_ARG) throw py::value_error("cxgnn_hip: " + msg);
  throw std::runtime_error(fmt("cxgnn_hip (status %d): ", status) + msg);
}

const char* dtype_name(at::ScalarType t) { return c10::toString(t); }

// A contiguous device tensor of the given dtype (and, if given, one of the given ranks): the
// kernels index raw memory.
void req(const Tensor& t, const char* name, at::ScalarType dtype, std::initializer_list<int64_t> dims = {}) {
  if (!t.defined()) bad(fmt("%s must be a tensor", name));
  if (!t.is_cuda()) bad(fmt("%s must be a CUDA tensor", name));
  if (t.scalar_type() != dtype) bad(fmt("%s must be %s, got %s", name, dtype_name(dtype), dtype_name(t.scalar_type())));
  if (!t.is_contiguous()) bad(fmt("%s must be contiguous", name));
  if (dims.size() > 0) {
    bool ok = false;
    for (int64_t d : dims) ok = ok || t.dim() == d;
    if (!ok) bad(fmt("%s has %d dims, which this operation does not take", name, (int)t.dim()));
  }
}

void check_graph(const Tensor& ptr, const Tensor& idx, int64_t n_rows, at::ScalarType dtype = at::kLong) {
  req(ptr, "ptr", dtype, {1});
  req(idx, "idx", dtype, {1});
  if (n_rows < 0 || n_rows + 1 > ptr.size(0))
    bad(fmt("num_node=%lld does not fit ptr of length %lld", (long long)n_rows, (long long)ptr.size(0)));
  if (ptr.device() != idx.device()) bad("ptr and idx are on different devices");
}

void* stream_of(const Tensor& t) {
  return reinterpret_cast<void*>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

Tensor workspace(size_t nbytes, const Tensor& like) {
  const int64_t n = nbytes < 256 ? 256 : (int64_t)nbytes;
  return torch::empty({n}, like.options().dtype(at::kByte));
}

const void* ptr_or_null(const Tensor& t) { return t.defined() && t.numel() > 0 ? t.data_ptr() : nullptr; }
const void* ptr_or_null(const OptTensor& t) { return t.has_value() ? ptr_or_null(*t) : nullptr; }

// Scalars arrive as Python ints or 0-d tensors (cxgnncomp/graph_conv.py:41-50).
int64_t as_int(const py::object& v) {
  if (py::hasattr(v, "item")) return py::cast<int64_t>(v.attr("item")());
  return py::cast<int64_t>(v);
}

// ---------------------------------------------------------------------------------------------
// SpMM family
// ---------------------------------------------------------------------------------------------
// out[r] = sum_{e in row r} (val[vrow(e)] *) x[idx[e]] for r < n_rows.  x is [n_src, F] or
// [n_src, H, C]; val (optional) is [E] or [E, H]; val_perm maps edge positions to rows of val;
// bias (with val, without mean) is added to every row as it is stored.
Tensor spmm(const Tensor& ptr, const Tensor& idx, const Tensor& x, int64_t n_rows, bool mean, const OptTensor& val,
            const OptTensor& val_perm, const OptTensor& out_opt, bool accumulate, const OptTensor& bias) {
  const bool int32 = ptr.defined() && ptr.scalar_type() == at::kInt;
  check_graph(ptr, idx, n_rows, int32 ? at::kInt : at::kLong);
  req(x, "x", at::kFloat, {2, 3});
  if (x.device() != ptr.device()) bad("x and ptr are on different devices");
  int64_t heads = 1, channels = x.size(-1);
  if (val.has_value()) {
    req(*val, "val", at::kFloat, {1, 2});
    if (val->dim() == 2) {
      heads = val->size(1);
      if (x.dim() != 3 || x.size(1) != heads) bad(fmt("val has %lld heads but x does not", (long long)heads));
    } else if (x.dim() == 3 && x.size(1) != 1) {
      bad("1-D val needs x of shape [N, F] or [N, 1, F]");
    }
    if (!val_perm.has_value() && val->size(0) < idx.size(0))
      bad(fmt("val has %lld rows, idx has %lld", (long long)val->size(0), (long long)idx.size(0)));
    if (val_perm.has_value()) {
      req(*val_perm, "val_perm", at::kLong, {1});
      if (val_perm->size(0) < idx.size(0)) bad("val_perm shorter than idx");
    }
  } else if (x.dim() == 3) {
    channels = x.size(1) * x.size(2);
  }
  const int64_t row = val.has_value() ? heads * channels : channels;
  std::vector<int64_t> shape = x.sizes().vec();
  shape[0] = n_rows;
  Tensor out;
  if (out_opt.has_value()) {
    out = *out_opt;
    req(out, "out", at::kFloat);
    if (out.sizes().vec() != shape) bad("out does not have the shape of the result");
  } else {
    out = torch::empty(shape, x.options());
  }
  if (n_rows == 0) return out;
  if (bias.has_value() && !val.has_value()) bad("bias needs edge values");
  const int64_t n_cap = idx.size(0);
  Tensor ws = workspace(cxg_spmm_workspace_bytes(n_cap, row), x);
  unsigned flags = (mean ? kSpmmMean : 0u) | (accumulate ? kSpmmAccumulate : 0u);
  if (n_rows == ptr.size(0) - 1) flags |= kSpmmExactEdges;       // all rows of ptr: idx holds exactly their edges
  c10::DeviceGuard guard(x.device());
  void* st = stream_of(x);
  int rc;
  if (!val.has_value()) {
    if (int32)
      rc = cxg_spmm_sum_f32_i32((const int32_t*)ptr.data_ptr(), (const int32_t*)ptr_or_null(idx), (const float*)ptr_or_null(x),
                                row, (float*)out.data_ptr(), row, n_rows, n_cap, (int)row, flags, ws.data_ptr(),
                                (size_t)ws.numel(), st);
    else
      rc = cxg_spmm_sum_f32((const int64_t*)ptr.data_ptr(), (const int64_t*)ptr_or_null(idx), (const float*)ptr_or_null(x), row,
                            (float*)out.data_ptr(), row, n_rows, n_cap, (int)row, flags, ws.data_ptr(),
                            (size_t)ws.numel(), st);
  } else {
    if (int32) bad("weighted SpMM needs int64 ptr/idx");
    if (bias.has_value()) {
      req(*bias, "bias", at::kFloat, {1});
      if (bias->size(0) != row || mean) bad(fmt("bias needs %lld floats and no mean", (long long)row));
      rc = cxg_spmm_weighted_bias_f32((const int64_t*)ptr.data_ptr(), (const int64_t*)ptr_or_null(idx),
                                      (const float*)val->data_ptr(), (const int64_t*)ptr_or_null(val_perm),
                                      (const float*)ptr_or_null(x), row, (const float*)bias->data_ptr(),
                                      (float*)out.data_ptr(), row, n_rows, n_cap, (int)heads, (int)channels, flags,
                                      ws.data_ptr(), (size_t)ws.numel(), st);
    } else {
      rc = cxg_spmm_weighted_f32((const int64_t*)ptr.data_ptr(), (const int64_t*)ptr_or_null(idx),
                                 (const float*)val->data_ptr(), (const int64_t*)ptr_or_null(val_perm),
                                 (const float*)ptr_or_null(x), row, (float*)out.data_ptr(), row, n_rows, n_cap,
                                 (int)heads, (int)channels, flags, ws.data_ptr(), (size_t)ws.numel(), st);
    }
  }
  check(rc);
  return out;
}

Tensor spmm_plain(const Tensor& ptr, const Tensor& idx, const Tensor& x, int64_t n_rows, bool mean = false) {
  return spmm(ptr, idx, x, n_rows, mean, c10::nullopt, c10::nullopt, c10::nullopt, false, c10::nullopt);
}

Tensor head_sum(const Tensor& x) {
  req(x, "x", at::kFloat, {3});
  Tensor out = torch::empty({x.size(0), x.size(2)}, x.options());
  c10::DeviceGuard guard(x.device());
  check(cxg_head_sum_f32((const float*)ptr_or_null(x), (float*)ptr_or_null(out), x.size(0), (int)x.size(1), (int)x.size(2),
                         stream_of(x)));
  return out;
}

Tensor edge_value_degree(const Tensor& ptr, int64_t n_rows, int64_t n_edges) {
  req(ptr, "ptr", at::kLong, {1});
  if (n_rows + 1 > ptr.size(0)) bad(fmt("num_dst=%lld does not fit ptr", (long long)n_rows));
  Tensor out = torch::zeros({n_edges}, ptr.options().dtype(at::kFloat));
  c10::DeviceGuard guard(ptr.device());
  check(cxg_edge_value_degree_f32((const int64_t*)ptr.data_ptr(), n_rows, (float*)ptr_or_null(out), stream_of(ptr)));
  return out;
}

// ---------------------------------------------------------------------------------------------
// SDDMM
// ---------------------------------------------------------------------------------------------
Tensor feat3(const Tensor& t, const char* name) {
  req(t, name, at::kFloat, {2, 3});
  return t.dim() == 3 ? t : t.unsqueeze(1);
}

// 1: dst_feat carries heads (or there is one head), 0: a 2-D dst_feat shared by all heads
int dst_head_mode(const Tensor& a, const Tensor& dst_feat) {
  req(dst_feat, "dst_feat", at::kFloat, {2, 3});
  const int64_t heads = a.size(1), channels = a.size(2);
  if (dst_feat.dim() == 3) {
    if (dst_feat.size(1) != heads || dst_feat.size(2) != channels) bad("dst_feat shape does not match src_feat");
    return 1;
  }
  if (dst_feat.size(1) != channels)
    bad(fmt("dst_feat has %lld channels, src_feat %lld", (long long)dst_feat.size(1), (long long)channels));
  return heads == 1 ? 1 : 0;
}

// out[e,h] = <src_feat[idx[e],h,:], dst_feat[row(e),(h,):]> in CSR edge order, [E, H].
Tensor sddmm_csr(const Tensor& ptr, const Tensor& idx, const Tensor& src_feat, const Tensor& dst_feat, int64_t n_rows,
                 const OptTensor& out_opt) {
  check_graph(ptr, idx, n_rows);
  const Tensor a = feat3(src_feat, "src_feat");
  const int64_t heads = a.size(1), channels = a.size(2);
  const int b_heads = dst_head_mode(a, dst_feat);
  if (dst_feat.size(0) < n_rows) bad("dst_feat has fewer rows than num_node");
  const int64_t n_cap = idx.size(0);
  Tensor out;
  if (out_opt.has_value()) {
    out = *out_opt;
    req(out, "out", at::kFloat);
    if (out.numel() < n_cap * heads) bad("output too small");
  } else {
    out = torch::zeros({n_cap, heads}, a.options());
  }
  c10::DeviceGuard guard(a.device());
  check(cxg_sddmm_csr_f32((const int64_t*)ptr.data_ptr(), (const int64_t*)ptr_or_null(idx), (const float*)a.data_ptr(),
                          (const float*)dst_feat.data_ptr(), (float*)out.data_ptr(), n_rows, n_cap, (int)heads,
                          (int)channels, b_heads, stream_of(a)));
  return out;
}

Tensor sddmm_coo(const Tensor& src, const Tensor& dst, const Tensor& src_feat, const Tensor& dst_feat, Tensor out,
                 int64_t n_edges) {
  req(src, "src", at::kLong, {1});
  req(dst, "dst", at::kLong, {1});
  if (src.size(0) < n_edges || dst.size(0) < n_edges) bad("src/dst shorter than num_edge");
  const Tensor a = feat3(src_feat, "src_feat");
  const int b_heads = dst_head_mode(a, dst_feat);
  req(out, "output", at::kFloat);
  if (out.numel() < n_edges * a.size(1)) bad("output too small");
  c10::DeviceGuard guard(a.device());
  check(cxg_sddmm_coo_f32((const int64_t*)src.data_ptr(), (const int64_t*)dst.data_ptr(), (const float*)a.data_ptr(),
                          (const float*)dst_feat.data_ptr(), (float*)out.data_ptr(), n_edges, (int)a.size(1),
                          (int)a.size(2), b_heads, stream_of(a)));
  return out;
}

// ---------------------------------------------------------------------------------------------
// Transposed graphs: the CSR the backward passes gather over, cached per (ptr, idx, rows, sources)
// ---------------------------------------------------------------------------------------------
struct TransposedGraph {
  Tensor ptr_t, idx_t, perm;        // rows = source nodes, idx_t = destination ids, perm = original edge position
  int64_t n_edges = 0, n_src = 0, n_dst = 0;
  Tensor keep_ptr, keep_idx;        // the tensors the key was made from stay alive while cached
  OptTensor inv_deg_t, rows32, inv_perm;   // filled on first use, under fill_mu (a cached graph is shared between threads)
  std::mutex fill_mu;
};
using GraphPtr = std::shared_ptr<TransposedGraph>;

using GraphId = std::tuple<void*, void*, int64_t, int64_t, int64_t, int64_t, int>;
using GraphKey = std::tuple<GraphId, int64_t, int64_t>;

GraphId graph_id(const Tensor& ptr, const Tensor& idx) {
  return GraphId(ptr.data_ptr(), idx.data_ptr(), ptr.size(0), idx.size(0), (int64_t)ptr._version(),
                 (int64_t)idx._version(), (int)ptr.device().index());
}

struct LayerHint {
  int64_t n_rows, n_src;
  c10::weak_intrusive_ptr<c10::TensorImpl> ptr, idx;   // a hint must not outlive its tensors
};

// Edge counts of row prefixes that the caller knows (a sampled batch carries num_edge_in_layer):
// with them no transposition has to read ptr[n_rows] back from the device.
struct EdgeCounts {
  std::vector<std::pair<int64_t, int64_t>> rows_edges;
  c10::weak_intrusive_ptr<c10::TensorImpl> ptr, idx;
};

struct GraphCache {
  std::mutex mu;
  std::list<std::pair<GraphId, EdgeCounts>> edge_counts;
  size_t capacity = 8;
  std::list<std::pair<GraphKey, GraphPtr>> lru;                      // most recently used last
  std::map<GraphKey, std::list<std::pair<GraphKey, GraphPtr>>::iterator> index;
  std::list<std::pair<GraphId, LayerHint>> hints;
  int64_t sorts = 0, cuts = 0;                                       // transpositions by sort / by compaction

  GraphPtr find(const GraphKey& key) {
    auto it = index.find(key);
    if (it == index.end()) return nullptr;
    lru.splice(lru.end(), lru, it->second);
    return it->second->second;
  }
  void insert(const GraphKey& key, GraphPtr g) {
    if (capacity == 0) return;
    lru.emplace_back(key, std::move(g));
    index[key] = std::prev(lru.end());
    while (lru.size() > capacity) {
      index.erase(lru.front().first);
      lru.pop_front();
    }
  }
  void clear() {
    lru.clear();
    index.clear();
    hints.clear();
    edge_counts.clear();
  }
  // number of edges of rows [0, n_rows) if the caller has announced it, else -1
  int64_t known_edges(const GraphId& gid, const Tensor& ptr, const Tensor& idx, int64_t n_rows) {
    for (auto it = edge_counts.begin(); it != edge_counts.end(); ++it) {
      if (it->first != gid) continue;
      auto p = it->second.ptr.lock(), i = it->second.idx.lock();
      if (p.get() != ptr.unsafeGetTensorImpl() || i.get() != idx.unsafeGetTensorImpl()) {
        edge_counts.erase(it);
        return -1;
      }
      for (const auto& re : it->second.rows_edges)
        if (re.first == n_rows) return re.second;
      return -1;
    }
    return -1;
  }
  const LayerHint* hint(const GraphId& gid, const Tensor& ptr, const Tensor& idx) {
    for (auto it = hints.begin(); it != hints.end(); ++it) {
      if (it->first != gid) continue;
      auto p = it->second.ptr.lock(), i = it->second.idx.lock();
      if (p.get() != ptr.unsafeGetTensorImpl() || i.get() != idx.unsafeGetTensorImpl()) {
        hints.erase(it);
        return nullptr;
      }
      return &it->second;
    }
    return nullptr;
  }
};

// Never destroyed: the cached device tensors must not be released after the runtime they live
// in has shut down at process exit.
GraphCache& cache() {
  static GraphCache* c = new GraphCache;
  return *c;
}

std::atomic<int64_t> g_edge_count_readbacks{0};   // times a transposition had to fetch ptr[n_rows] from the device

// Uncached transposition by a stable sort: (ptr_t, idx_t, perm, n_edges).
// `known_edges` >= 0: the caller vouches for ptr[0] == 0 and ptr[n_rows] == known_edges, and nothing is read back.
std::tuple<Tensor, Tensor, Tensor, int64_t> csr_transpose(const Tensor& ptr, const Tensor& idx, int64_t n_rows, int64_t n_src,
                                                          int64_t known_edges = -1) {
  check_graph(ptr, idx, n_rows);
  int64_t n_edges = known_edges;
  if (n_edges < 0) {
    ++g_edge_count_readbacks;
    const Tensor ends = torch::stack({ptr[0], ptr[n_rows]}).cpu();          // one read-back for both
    n_edges = ends[1].item<int64_t>();
    if (ends[0].item<int64_t>() != 0) bad("ptr[0] must be 0");
  }
  if (n_edges > idx.size(0))
    bad(fmt("ptr[num_node]=%lld exceeds idx length %lld", (long long)n_edges, (long long)idx.size(0)));
  Tensor ptr_t = torch::empty({n_src + 1}, ptr.options());
  Tensor idx_t = torch::empty({n_edges}, ptr.options());
  Tensor perm = torch::empty({n_edges}, ptr.options());
  Tensor ws = workspace(cxg_csr_transpose_workspace_bytes(n_edges, n_src), ptr);
  c10::DeviceGuard guard(ptr.device());
  check(cxg_csr_transpose_i64((const int64_t*)ptr.data_ptr(), (const int64_t*)ptr_or_null(idx), n_rows, n_src, n_edges,
                              (int64_t*)ptr_t.data_ptr(), (int64_t*)ptr_or_null(idx_t), (int64_t*)ptr_or_null(perm),
                              ws.data_ptr(), (size_t)ws.numel(), stream_of(ptr)));
  return std::make_tuple(ptr_t, idx_t, perm, n_edges);
}

// The first n_rows rows of the graph `whole` was built from, as a stable compaction of its entries.
std::tuple<Tensor, Tensor, Tensor, int64_t> csr_transpose_prefix(const TransposedGraph& whole, const Tensor& ptr,
                                                                 int64_t n_rows, int64_t n_src, int64_t known_edges = -1) {
  req(ptr, "ptr", at::kLong, {1});
  if (n_rows < 0 || n_rows + 1 > ptr.size(0)) bad("num_node does not fit ptr");
  if (n_src + 1 > whole.ptr_t.size(0)) bad("the whole graph has fewer sources than the prefix");
  if (known_edges < 0) ++g_edge_count_readbacks;
  const int64_t n_edges = known_edges >= 0 ? known_edges : ptr[n_rows].item<int64_t>();
  if (n_edges > whole.n_edges) bad("the prefix has more edges than the whole graph");
  Tensor ptr_t = torch::empty({n_src + 1}, ptr.options());
  Tensor idx_t = torch::empty({n_edges}, ptr.options());
  Tensor perm = torch::empty({n_edges}, ptr.options());
  Tensor ws = workspace(cxg_csr_transpose_prefix_workspace_bytes(whole.n_edges), ptr);
  c10::DeviceGuard guard(ptr.device());
  check(cxg_csr_transpose_prefix_i64((const int64_t*)whole.ptr_t.data_ptr(), (const int64_t*)ptr_or_null(whole.idx_t),
                                     (const int64_t*)ptr_or_null(whole.perm), whole.n_edges, n_edges, n_src,
                                     (int64_t*)ptr_t.data_ptr(), (int64_t*)ptr_or_null(idx_t), (int64_t*)ptr_or_null(perm),
                                     ws.data_ptr(), (size_t)ws.numel(), stream_of(ptr)));
  return std::make_tuple(ptr_t, idx_t, perm, n_edges);
}

// Tell the cache that a layer aggregates rows [0, n_rows) of (ptr, idx) over n_src sources: the
// layers of a sampled mini-batch work on nested row prefixes of one CSR, and the backward pass,
// which meets the smallest layer first, then sorts the largest once and cuts the others out of it.
void note_layer(const Tensor& ptr, const Tensor& idx, int64_t n_rows, int64_t n_src) {
  GraphCache& c = cache();
  std::lock_guard<std::mutex> lock(c.mu);
  const GraphId gid = graph_id(ptr, idx);
  const LayerHint* seen = c.hint(gid, ptr, idx);
  if (seen && n_rows <= seen->n_rows) return;
  const int64_t src = seen ? std::max(seen->n_src, n_src) : n_src;
  c.hints.remove_if([&](const std::pair<GraphId, LayerHint>& h) { return h.first == gid; });
  c.hints.emplace_back(gid, LayerHint{n_rows, src, c10::weak_intrusive_ptr<c10::TensorImpl>(ptr.getIntrusivePtr()),
                                      c10::weak_intrusive_ptr<c10::TensorImpl>(idx.getIntrusivePtr())});
  while (c.hints.size() > 64) c.hints.pop_front();
}

// The caller knows how many edges the first rows[k] rows hold (Batch.num_node_in_layer /
// num_edge_in_layer of a sampled batch, cxgnncomp/batch.py): transpositions of those row prefixes
// then size their outputs from it instead of reading ptr[rows[k]] back, which made the host wait
// for the GPU once per layer in the first backward pass of every new batch.
void note_edge_counts(const Tensor& ptr, const Tensor& idx, const std::vector<int64_t>& rows,
                      const std::vector<int64_t>& edges) {
  if (rows.size() != edges.size()) bad("note_edge_counts: one edge count per row count");
  std::vector<std::pair<int64_t, int64_t>> rows_edges;
  for (size_t k = 0; k < rows.size(); ++k) {
    if (rows[k] < 0 || rows[k] + 1 > ptr.size(0) || edges[k] < 0 || edges[k] > idx.size(0))
      bad("note_edge_counts: counts do not fit ptr / idx");
    rows_edges.emplace_back(rows[k], edges[k]);
  }
  EdgeCounts ec{std::move(rows_edges), c10::weak_intrusive_ptr<c10::TensorImpl>(ptr.getIntrusivePtr()),
                c10::weak_intrusive_ptr<c10::TensorImpl>(idx.getIntrusivePtr())};
  GraphCache& c = cache();
  std::lock_guard<std::mutex> lock(c.mu);
  const GraphId gid = graph_id(ptr, idx);
  c.edge_counts.remove_if([&](const std::pair<GraphId, EdgeCounts>& h) { return h.first == gid; });
  c.edge_counts.emplace_back(gid, std::move(ec));
  while (c.edge_counts.size() > 64) c.edge_counts.pop_front();
}

GraphPtr transposed(const Tensor& ptr, const Tensor& idx, int64_t n_rows, int64_t n_src) {
  GraphCache& c = cache();
  const GraphId gid = graph_id(ptr, idx);
  const GraphKey key(gid, n_rows, n_src);
  int64_t whole_rows = -1, whole_src = -1, known = -1;
  {
    std::lock_guard<std::mutex> lock(c.mu);
    if (GraphPtr g = c.find(key)) return g;
    known = c.known_edges(gid, ptr, idx, n_rows);
    const LayerHint* h = c.hint(gid, ptr, idx);
    if (h && ptr.is_cuda() && h->n_rows > n_rows && h->n_src >= n_src && c.capacity > 1) {
      whole_rows = h->n_rows;
      whole_src = h->n_src;
    }
  }
  auto g = std::make_shared<TransposedGraph>();
  if (whole_rows >= 0) {
    GraphPtr whole = transposed(ptr, idx, whole_rows, whole_src);
    std::tie(g->ptr_t, g->idx_t, g->perm, g->n_edges) = csr_transpose_prefix(*whole, ptr, n_rows, n_src, known);
    std::lock_guard<std::mutex> lock(c.mu);
    ++c.cuts;
  } else {
    std::tie(g->ptr_t, g->idx_t, g->perm, g->n_edges) = csr_transpose(ptr, idx, n_rows, n_src, known);
    std::lock_guard<std::mutex> lock(c.mu);
    ++c.sorts;
  }
  g->n_src = n_src;
  g->n_dst = n_rows;
  g->keep_ptr = ptr;
  g->keep_idx = idx;
  std::lock_guard<std::mutex> lock(c.mu);
  c.insert(key, g);
  return g;
}

// 1/deg(dst) per edge, in transposed edge order (kept with the graph).
Tensor inv_degree_transposed(TransposedGraph& g, const Tensor& ptr, int64_t n_rows) {
  std::lock_guard<std::mutex> lock(g.fill_mu);
  if (!g.inv_deg_t.has_value()) {
    Tensor inv = edge_value_degree(ptr, n_rows, g.n_edges);
    g.inv_deg_t = g.n_edges > 0 ? inv.index({g.perm}) : inv;
  }
  return *g.inv_deg_t;
}

// Row (source) id of every edge of a transposed graph as int32 (kept with the graph).
Tensor rows32_transposed(TransposedGraph& g) {
  std::lock_guard<std::mutex> lock(g.fill_mu);
  if (!g.rows32.has_value()) {
    Tensor rows = torch::empty({g.n_edges}, g.ptr_t.options().dtype(at::kInt));
    c10::DeviceGuard guard(g.ptr_t.device());
    check(cxg_csr_row_ids_i32((const int64_t*)g.ptr_t.data_ptr(), g.n_src, g.n_edges, (int32_t*)ptr_or_null(rows),
                              stream_of(g.ptr_t)));
    g.rows32 = rows;
  }
  return *g.rows32;
}

// ---------------------------------------------------------------------------------------------
// sum / mean / edge-weighted aggregation with autograd (SAGEFunction, SAGEEdgeValueFunction)
// ---------------------------------------------------------------------------------------------
Tensor inverse_perm_transposed(TransposedGraph& g);
Tensor gather_rows(const Tensor& inp, const Tensor& sel);

struct SageFunction : public torch::autograd::Function<SageFunction> {
  static Tensor forward(AutogradContext* ctx, Tensor x, Tensor ptr, Tensor idx, OptTensor edge_value, int64_t num_node,
                        bool mean) {
    int64_t n = num_node;
    if (n == 0) n = ptr.size(0) - 1;              // aggr.cu:118
    ctx->saved_data["n"] = n;
    ctx->saved_data["mean"] = mean;
    ctx->saved_data["n_src"] = x.size(0);
    ctx->saved_data["x_shape"] = x.sizes().vec();
    ctx->saved_data["weighted"] = edge_value.has_value();
    if (x.requires_grad()) note_layer(ptr, idx, n, x.size(0));
    x = x.contiguous();
    if (!edge_value.has_value()) {
      ctx->save_for_backward({ptr, idx});
      return spmm_plain(ptr, idx, x, n, mean);
    }
    if (mean) bad("DO NOT use mean with edge value");          // aggr.cu:158,163 aborts with this message
    Tensor ev = edge_value->contiguous();
    if (ev.dim() == 2 && x.dim() != 3) bad("multi-head edge_value needs input [N, H, C]");
    ctx->saved_data["ev_needs_grad"] = edge_value->requires_grad();
    ctx->save_for_backward({ptr, idx, x, ev});
    return spmm(ptr, idx, x, n, false, ev, c10::nullopt, c10::nullopt, false, c10::nullopt);
  }

  static tensor_list backward(AutogradContext* ctx, tensor_list grads) {
    Tensor grad_out = grads[0].contiguous();
    const auto saved = ctx->get_saved_variables();
    const Tensor& ptr = saved[0];
    const Tensor& idx = saved[1];
    const int64_t n = ctx->saved_data["n"].toInt(), n_src = ctx->saved_data["n_src"].toInt();
    const bool mean = ctx->saved_data["mean"].toBool();
    const std::vector<int64_t> x_shape = ctx->saved_data["x_shape"].toIntVector();
    GraphPtr g = transposed(ptr, idx, n, n_src);
    Tensor gx, gval;
    if (!ctx->saved_data["weighted"].toBool()) {
      const Tensor go = grad_out.reshape({n, -1});
      if (mean) {
        gx = spmm(g->ptr_t, g->idx_t, go, n_src, false, inv_degree_transposed(*g, ptr, n), c10::nullopt, c10::nullopt,
                  false, c10::nullopt);
      } else {
        gx = spmm_plain(g->ptr_t, g->idx_t, go, n_src);
      }
      return {gx.reshape(x_shape), Tensor(), Tensor(), Tensor(), Tensor(), Tensor()};
    }
    const Tensor& x = saved[2];
    const Tensor& ev = saved[3];
    const bool need_ev = ctx->saved_data["ev_needs_grad"].toBool();
    const int64_t heads = ev.dim() == 2 ? ev.size(1) : 1;
    const int64_t channels = x.size(-1);
    const int64_t row = heads * channels;
    // Rows of 256 * k floats: ONE pass over the reversed graph gathers the rows of grad_out for the
    // input gradient and multiplies them with the source's own row of x for the edge-value
    // gradient (stored at the edge's original position), instead of an aggregation and an SDDMM
    // that each gather every row once.
    if (need_ev && row % 256 == 0 && (channels == 32 || channels == 64 || channels == 128 || channels == 256) &&
        ev.size(0) == idx.size(0) && grad_out.numel() == n * row && n_src > 0 && g->n_edges > 0) {
      // (the products leave the pass in its own edge order -- contiguous stores -- and one row gather
      // through the inverse permutation puts them into the original order: faster than scattering
      // them from the pass, the same bits)
      gx = torch::empty({n_src, row}, x.options());
      Tensor in_pass_order = torch::empty({ev.size(0), heads}, ev.options());
      const int64_t n_cap = g->idx_t.size(0);
      Tensor ws = workspace(cxg_spmm_workspace_bytes(n_cap, row), x);
      c10::DeviceGuard guard(x.device());
      check(cxg_spmm_weighted_dot_f32((const int64_t*)g->ptr_t.data_ptr(), (const int64_t*)ptr_or_null(g->idx_t),
                                      (const float*)ev.data_ptr(), (const int64_t*)ptr_or_null(g->perm),
                                      (const float*)grad_out.data_ptr(), row, (float*)gx.data_ptr(), row,
                                      (const float*)x.data_ptr(), row, (float*)in_pass_order.data_ptr(), n_src, n_cap,
                                      (int)heads, (int)channels, CXG_SPMM_DOT_AT_EDGE, ws.data_ptr(), (size_t)ws.numel(),
                                      stream_of(x)));
      Tensor ordered = gather_rows(in_pass_order, inverse_perm_transposed(*g));       // [n_edges, heads]
      if (g->n_edges == ev.size(0)) {
        gval = ordered;
      } else {
        gval = torch::zeros({ev.size(0), heads}, ev.options());
        gval.narrow(0, 0, g->n_edges).copy_(ordered);
      }
      return {gx.reshape(x_shape), Tensor(), Tensor(), gval.reshape(ev.sizes()), Tensor(), Tensor()};
    }
    gx = spmm(g->ptr_t, g->idx_t, grad_out, n_src, false, ev, g->perm, c10::nullopt, false, c10::nullopt);
    if (need_ev) gval = sddmm_csr(ptr, idx, x, grad_out, n, c10::nullopt).reshape(ev.sizes());
    return {gx.reshape(x_shape), Tensor(), Tensor(), gval, Tensor(), Tensor()};
  }
};

Tensor sage_apply(const Tensor& x, const Tensor& ptr, const Tensor& idx, const OptTensor& ev, const py::object& num_node,
                  bool mean) {
  return SageFunction::apply(x, ptr, idx, ev, as_int(num_node), mean);
}

// ---------------------------------------------------------------------------------------------
// edge attention (EdgeSoftMaxFunction)
// ---------------------------------------------------------------------------------------------
std::tuple<Tensor, Tensor> edge_softmax_fwd(const Tensor& ptr, const Tensor& idx, const Tensor& att_dst,
                                            const Tensor& att_src, int64_t n_edges, double slope) {
  req(att_dst, "att_dst", at::kFloat, {2});
  req(att_src, "att_src", at::kFloat, {2});
  const int64_t n_dst = att_dst.size(0), heads = att_dst.size(1);
  if (att_src.size(1) != heads) bad("att_src/att_dst head mismatch");
  check_graph(ptr, idx, n_dst);
  if (idx.size(0) < n_edges) bad("idx shorter than num_edge");
  Tensor out = torch::empty({n_edges, heads}, att_dst.options());
  Tensor mask = torch::empty({n_edges, heads}, att_dst.options().dtype(at::kBool));
  c10::DeviceGuard guard(att_dst.device());
  check(cxg_edge_softmax_fwd_f32((const int64_t*)ptr.data_ptr(), (const int64_t*)ptr_or_null(idx),
                                 (const float*)att_dst.data_ptr(), (const float*)att_src.data_ptr(),
                                 (float*)ptr_or_null(out), (uint8_t*)ptr_or_null(mask), n_dst, (int)heads, (float)slope,
                                 stream_of(att_dst)));
  return std::make_tuple(out, mask);
}

// (g_dst [n_dst, H], t_edge [E, H]); rows of t_edge at or past ptr[n_dst] are not written.
// grad_pos (optional, int64 per edge): the gradient row of edge k is grad[grad_pos[k]].
std::tuple<Tensor, Tensor> edge_softmax_bwd(const Tensor& ptr, const Tensor& out, const Tensor& mask, const Tensor& grad,
                                            int64_t n_dst, double slope, const OptTensor& grad_pos = c10::nullopt) {
  req(out, "out", at::kFloat, {2});
  req(grad, "grad", at::kFloat, {2});
  req(mask, "mask", at::kBool, {2});
  const int64_t heads = out.size(1);
  Tensor g_dst = torch::empty({n_dst, heads}, out.options());
  Tensor t_edge = torch::empty_like(out);
  if (grad_pos.has_value()) {
    req(*grad_pos, "grad_pos", at::kLong, {1});
    if (n_dst + 1 > ptr.size(0)) bad("num rows does not fit ptr");
  }
  c10::DeviceGuard guard(out.device());
  check(cxg_edge_softmax_bwd_at_f32((const int64_t*)ptr.data_ptr(), (const float*)ptr_or_null(out),
                                    (const uint8_t*)ptr_or_null(mask), (const float*)ptr_or_null(grad),
                                    grad_pos.has_value() ? (const int64_t*)ptr_or_null(*grad_pos) : nullptr,
                                    (float*)ptr_or_null(g_dst), (float*)ptr_or_null(t_edge), n_dst, (int)heads,
                                    (float)slope, stream_of(out)));
  return std::make_tuple(g_dst, t_edge);
}

// Position in the transposed order of every original edge position (the inverse of perm; kept
// with the graph): what a consumer walking the original order needs to read rows that were stored
// in the transposed order.
Tensor inverse_perm_transposed(TransposedGraph& g) {
  std::lock_guard<std::mutex> lock(g.fill_mu);
  if (!g.inv_perm.has_value()) {
    c10::DeviceGuard guard(g.perm.device());
    Tensor inv = torch::empty({g.n_edges}, g.perm.options());
    if (g.n_edges > 0) inv.index_put_({g.perm}, torch::arange(g.n_edges, g.perm.options()));
    g.inv_perm = inv;
  }
  return *g.inv_perm;
}

// out[r,:] = sum_{k in row r} inp[sel[k],:] (sel undefined: inp[k,:]); inp [M] or [M, W].  With
// rows32 (int32 row id per edge, ptr[0] == 0) and W in {1, 2, 4, 8} the edge-parallel kernel runs.
Tensor narrow_gather_sum(const Tensor& ptr, const OptTensor& sel, const Tensor& inp, int64_t n_rows, const OptTensor& rows32) {
  req(ptr, "ptr", at::kLong, {1});
  if (n_rows + 1 > ptr.size(0)) bad("num rows does not fit ptr");
  if (sel.has_value()) req(*sel, "sel", at::kLong, {1});
  req(inp, "input", at::kFloat, {1, 2});
  const int64_t width = inp.dim() == 1 ? 1 : inp.size(1);
  Tensor out = inp.dim() == 1 ? torch::empty({n_rows}, inp.options()) : torch::empty({n_rows, width}, inp.options());
  c10::DeviceGuard guard(inp.device());
  int rc;
  if (rows32.has_value() && (width == 1 || width == 2 || width == 4 || width == 8)) {
    req(*rows32, "rows32", at::kInt, {1});
    const int64_t n_edges = rows32->size(0);
    Tensor ws = workspace(cxg_segment_gather_sum_workspace_bytes(n_edges, (int)width), inp);
    rc = cxg_segment_gather_sum_f32((const int32_t*)ptr_or_null(*rows32), (const int64_t*)ptr.data_ptr(),
                                    (const int64_t*)ptr_or_null(sel), (const float*)ptr_or_null(inp),
                                    (float*)ptr_or_null(out), n_rows, n_edges, (int)width, ws.data_ptr(),
                                    (size_t)ws.numel(), stream_of(inp));
  } else {
    rc = cxg_narrow_gather_sum_f32((const int64_t*)ptr.data_ptr(), (const int64_t*)ptr_or_null(sel),
                                   (const float*)ptr_or_null(inp), (float*)ptr_or_null(out), n_rows, (int)width,
                                   stream_of(inp));
  }
  check(rc);
  return out;
}

struct EdgeSoftmaxFunction : public torch::autograd::Function<EdgeSoftmaxFunction> {
  static Tensor forward(AutogradContext* ctx, Tensor ptr, Tensor idx, Tensor att_dst, Tensor att_src, int64_t num_edge,
                        double relu_l) {
    att_dst = att_dst.contiguous();
    att_src = att_src.contiguous();
    Tensor out, mask;
    std::tie(out, mask) = edge_softmax_fwd(ptr, idx, att_dst, att_src, num_edge, relu_l);
    ctx->save_for_backward({ptr, idx, out, mask});
    ctx->saved_data["n_dst"] = att_dst.size(0);
    ctx->saved_data["n_src"] = att_src.size(0);
    ctx->saved_data["slope"] = relu_l;
    return out;
  }
  static tensor_list backward(AutogradContext* ctx, tensor_list grads) {
    const auto saved = ctx->get_saved_variables();
    const Tensor &ptr = saved[0], &idx = saved[1], &out = saved[2], &mask = saved[3];
    const int64_t n_dst = ctx->saved_data["n_dst"].toInt(), n_src = ctx->saved_data["n_src"].toInt();
    Tensor g_dst, t_edge;
    std::tie(g_dst, t_edge) = edge_softmax_bwd(ptr, out, mask, grads[0].contiguous(), n_dst, ctx->saved_data["slope"].toDouble());
    GraphPtr g = transposed(ptr, idx, n_dst, n_src);
    Tensor g_src = narrow_gather_sum(g->ptr_t, g->perm, t_edge, n_src, rows32_transposed(*g));
    return {Tensor(), Tensor(), g_dst, g_src, Tensor(), Tensor()};
  }
};

// ---------------------------------------------------------------------------------------------
// gather: edge -> node scatter-add (GatherFunction, src/cpp/src/aggr.cu:395-448)
// ---------------------------------------------------------------------------------------------
// The reference adds every edge row to its node with atomics.  Here the edge positions are grouped
// by destination once per destination array (one stable sort, cached) and every node sums its own
// rows with the aggregation kernel: several times faster than fp32 atomics at these widths, and
// reproducible.
struct DestGroups {
  Tensor ptr, perm;     // ptr [n + 1], perm [E]: edge positions in destination order (stable)
  Tensor keep;          // the destination array the key was made from
};
using DestPtr = std::shared_ptr<DestGroups>;
using DestKey = std::tuple<void*, int64_t, int64_t, int64_t, int>;

struct DestCache {
  std::mutex mu;
  std::list<std::pair<DestKey, DestPtr>> lru;
};
DestCache& dest_cache() {
  static DestCache* c = new DestCache;     // never destroyed, like the graph cache
  return *c;
}

DestPtr dest_groups(const Tensor& dest, int64_t n_rows) {
  req(dest, "dest", at::kLong, {1});
  DestCache& c = dest_cache();
  const DestKey key(dest.data_ptr(), dest.size(0), (int64_t)dest._version(), n_rows, (int)dest.device().index());
  {
    std::lock_guard<std::mutex> lock(c.mu);
    for (auto it = c.lru.begin(); it != c.lru.end(); ++it)
      if (it->first == key) {
        c.lru.splice(c.lru.end(), c.lru, it);
        return c.lru.back().second;
      }
  }
  const int64_t e = dest.size(0);
  if (e > 0) {
    const Tensor lim = torch::stack({dest.min(), dest.max()}).cpu();
    if (lim[0].item<int64_t>() < 0 || lim[1].item<int64_t>() >= n_rows)
      bad(fmt("destination ids must lie in [0, %lld)", (long long)n_rows));
  }
  auto g = std::make_shared<DestGroups>();
  g->ptr = torch::empty({n_rows + 1}, dest.options());
  g->perm = torch::empty({e}, dest.options());
  g->keep = dest;
  Tensor idx = torch::empty({e}, dest.options());
  Tensor ws = workspace(cxg_coo_to_csr_workspace_bytes(e, n_rows), dest);
  {
    c10::DeviceGuard guard(dest.device());
    check(cxg_coo_to_csr_i64((const int64_t*)ptr_or_null(dest), (const int64_t*)ptr_or_null(dest), e, n_rows,
                             (int64_t*)g->ptr.data_ptr(), (int64_t*)ptr_or_null(idx), (int64_t*)ptr_or_null(g->perm),
                             ws.data_ptr(), (size_t)ws.numel(), stream_of(dest)));
  }
  std::lock_guard<std::mutex> lock(c.mu);
  const size_t cap = cache().capacity;
  if (cap > 0) {
    c.lru.emplace_back(key, g);
    while (c.lru.size() > cap) c.lru.pop_front();
  }
  return g;
}

// out[e] = inp[sel[e]]
Tensor gather_rows(const Tensor& inp, const Tensor& sel) {
  req(inp, "input", at::kFloat, {2});
  req(sel, "sel", at::kLong, {1});
  Tensor out = torch::empty({sel.size(0), inp.size(1)}, inp.options());
  c10::DeviceGuard guard(inp.device());
  check(cxg_gather_rows_f32((const float*)ptr_or_null(inp), (const int64_t*)ptr_or_null(sel), (float*)ptr_or_null(out),
                            sel.size(0), (int)inp.size(1), stream_of(inp)));
  return out;
}

struct GatherFunction : public torch::autograd::Function<GatherFunction> {
  static Tensor forward(AutogradContext* ctx, Tensor input, Tensor dest, int64_t num_node) {
    if (num_node <= 0) bad("num_node must be > 0");
    ctx->save_for_backward({dest});
    input = input.contiguous();
    if (input.dim() != 2 || input.size(0) != dest.size(0))
      bad("input must be [num_edge, F] with one row per entry of dest");
    if (dest.size(0) == 0) return torch::zeros({num_node, input.size(1)}, input.options());
    DestPtr g = dest_groups(dest, num_node);
    return spmm_plain(g->ptr, g->perm, input, num_node);
  }
  static tensor_list backward(AutogradContext* ctx, tensor_list grads) {
    const auto saved = ctx->get_saved_variables();
    return {gather_rows(grads[0].contiguous(), saved[0]), Tensor(), Tensor()};
  }
};

// ---------------------------------------------------------------------------------------------
// aggr_rel: relational aggregation over pre-transformed features (AggrRelFunction,
// src/cpp/src/rel_spmm.cu:37-136): out[r] = sum_e input[etype[e] * N + idx[e]]
// ---------------------------------------------------------------------------------------------
// The combined row index etype[e] * N + idx[e] of every edge is kept per (idx, etype): with it the
// relational gather is the plain SpMM, and its transposed graph (cached like any other) gives the
// backward pass without the reference's atomics.
struct RelKeys {
  Tensor keys, keep_idx, keep_etype;
};
using RelKeyId = std::tuple<void*, void*, int64_t, int64_t, int64_t, int64_t, int>;
struct RelKeyCache {
  std::mutex mu;
  std::list<std::pair<RelKeyId, std::shared_ptr<RelKeys>>> lru;
};
RelKeyCache& rel_key_cache() {
  static RelKeyCache* c = new RelKeyCache;   // never destroyed, like the graph cache
  return *c;
}

Tensor rel_keys(const Tensor& idx, const Tensor& etype, int64_t n_edges, int64_t stride, int64_t num_rel) {
  req(idx, "idx", at::kLong, {1});
  if (!etype.defined() || !etype.is_cuda() || etype.dim() != 1 ||
      (etype.scalar_type() != at::kInt && etype.scalar_type() != at::kLong))
    bad("etype must be a 1-D int32 or int64 CUDA tensor");
  if (idx.size(0) < n_edges || etype.size(0) < n_edges) bad("idx / etype shorter than the rows' edges");
  RelKeyCache& c = rel_key_cache();
  const RelKeyId id(idx.data_ptr(), etype.data_ptr(), (int64_t)idx._version(), (int64_t)etype._version(), n_edges, stride,
                    (int)idx.device().index());
  {
    std::lock_guard<std::mutex> lock(c.mu);
    for (auto it = c.lru.begin(); it != c.lru.end(); ++it)
      if (it->first == id) {
        c.lru.splice(c.lru.end(), c.lru, it);
        return c.lru.back().second->keys;
      }
  }
  const Tensor rel64 = etype.slice(0, 0, n_edges).to(at::kLong);
  if (n_edges > 0) {
    const Tensor lim = torch::stack({rel64.min(), rel64.max()}).cpu();
    if (lim[0].item<int64_t>() < 0 || lim[1].item<int64_t>() >= num_rel)
      bad(fmt("relation ids must lie in [0, %lld)", (long long)num_rel));
  }
  auto k = std::make_shared<RelKeys>();
  k->keys = rel64 * stride + idx.slice(0, 0, n_edges);
  k->keep_idx = idx;
  k->keep_etype = etype;
  std::lock_guard<std::mutex> lock(c.mu);
  c.lru.emplace_back(id, k);
  while (c.lru.size() > 4) c.lru.pop_front();
  return k->keys;
}

struct AggrRelFunction : public torch::autograd::Function<AggrRelFunction> {
  static Tensor forward(AutogradContext* ctx, Tensor input, Tensor ptr, Tensor idx, Tensor etype, int64_t num_node,
                        int64_t num_rel) {
    int64_t n = num_node;
    if (n == 0) n = ptr.size(0) - 1;
    if (num_rel <= 0 || input.size(0) % num_rel != 0)
      bad(fmt("input rows (%lld) must be num_rel (%lld) x nodes", (long long)input.size(0), (long long)num_rel));
    req(ptr, "ptr", at::kLong, {1});
    if (n < 0 || n + 1 > ptr.size(0)) bad("num_node does not fit ptr");
    const int64_t stride = input.size(0) / num_rel;
    const int64_t n_edges = ptr[n].item<int64_t>();
    const Tensor keys = rel_keys(idx, etype, n_edges, stride, num_rel);
    ctx->save_for_backward({ptr, keys});
    ctx->saved_data["n"] = n;
    ctx->saved_data["rows"] = input.size(0);
    return spmm_plain(ptr, keys, input.contiguous(), n);
  }
  static tensor_list backward(AutogradContext* ctx, tensor_list grads) {
    const auto saved = ctx->get_saved_variables();
    const int64_t n = ctx->saved_data["n"].toInt(), rows = ctx->saved_data["rows"].toInt();
    GraphPtr g = transposed(saved[0], saved[1], n, rows);
    return {spmm_plain(g->ptr_t, g->idx_t, grads[0].contiguous(), rows), Tensor(), Tensor(), Tensor(), Tensor(), Tensor()};
  }
};

// ---------------------------------------------------------------------------------------------
// entry points under the reference's names
// ---------------------------------------------------------------------------------------------
Tensor run_spmm_configurable(const Tensor& ptr, const Tensor& idx, const Tensor& vin, const py::object& num_node,
                             const py::args&) {
  if (vin.dim() != 2) bad("vin must be 2D");
  return spmm_plain(ptr, idx, vin, as_int(num_node));
}

Tensor run_spmm_configurable_bwd(const Tensor& ptr, const Tensor& idx, const Tensor& vin, const Tensor& grad_vout,
                                 const py::object& num_node, const py::args&) {
  if (grad_vout.dim() != 2) bad("grad_vout must be 2D");
  GraphPtr g = transposed(ptr, idx, as_int(num_node), vin.size(0));
  return spmm_plain(g->ptr_t, g->idx_t, grad_vout.contiguous(), vin.size(0));
}

enum class MultiheadSchedule : int { Naive = 0, PreReduce = 1, Optimal = 2 };

Tensor spmm_multihead(const Tensor& ptr, const Tensor& idx, const Tensor& val, const Tensor& vin, const py::object& num_node,
                      MultiheadSchedule schedule, int64_t /*block_size*/) {
  if (vin.dim() != 3) bad("vin must be 3D, [num_node, num_head, feat_len]");
  if (val.dim() != 2) bad("val must be 2D, [num_edge, num_head]");
  if (val.size(1) != vin.size(1)) bad(fmt("num_head mismatch %lld %lld", (long long)vin.size(1), (long long)val.size(1)));
  const int64_t n = as_int(num_node);
  if (schedule != MultiheadSchedule::Naive) {
    // PreReduce / Optimal: out[N, F], summed over the heads inside the aggregation kernel where the
    // row of heads x channels floats is one 64-lane gather; other shapes aggregate per head and sum after
    const int64_t heads = vin.size(1), channels = vin.size(2), row = heads * channels;
    const bool one_gather = heads > 1 && (heads & (heads - 1)) == 0 && (row == 64 || row == 128 || row == 256);
    if (one_gather && n > 0) {
      check_graph(ptr, idx, n);
      req(vin, "vin", at::kFloat, {3});
      req(val, "val", at::kFloat, {2});
      if (vin.device() != ptr.device()) bad("vin and ptr are on different devices");
      if (val.size(0) < idx.size(0)) bad(fmt("val has %lld rows, idx has %lld", (long long)val.size(0), (long long)idx.size(0)));
      Tensor out = torch::empty({n, channels}, vin.options());
      Tensor ws = workspace(cxg_spmm_workspace_bytes(idx.size(0), row), vin);
      c10::DeviceGuard guard(vin.device());
      const int rc = cxg_spmm_prereduce_f32((const int64_t*)ptr.data_ptr(), (const int64_t*)ptr_or_null(idx),
                                            (const float*)val.data_ptr(), nullptr, (const float*)ptr_or_null(vin), row,
                                            (float*)out.data_ptr(), channels, n, idx.size(0), (int)heads, (int)channels,
                                            n == ptr.size(0) - 1 ? kSpmmExactEdges : 0u, ws.data_ptr(), (size_t)ws.numel(),
                                            stream_of(vin));
      if (rc == 0) return out;
      if (rc != CXG_ERR_UNSUPPORTED) check(rc);
    }
  }
  Tensor out = spmm(ptr, idx, vin, n, false, val, c10::nullopt, c10::nullopt, false, c10::nullopt);
  return schedule == MultiheadSchedule::Naive ? out : head_sum(out);
}

void spmm_multihead_bwd(const Tensor& ptr, const Tensor& idx, const Tensor& val, const Tensor& grad_output, Tensor grad_x,
                        const py::object& num_node, MultiheadSchedule, int64_t /*block_size*/) {
  GraphPtr g = transposed(ptr, idx, as_int(num_node), grad_x.size(0));
  spmm(g->ptr_t, g->idx_t, grad_output.contiguous(), grad_x.size(0), false, val, g->perm, grad_x, true, c10::nullopt);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "compiled host layer of cxgnncomp_backend over libcxgnn_hip.so";
  m.def("lib_version", []() { return cxg_version(); });

  py::class_<TransposedGraph, GraphPtr>(m, "TransposedGraph",
                                        "CSR of the reversed graph: rows = source nodes, idx_t = destination ids, "
                                        "perm = position of each transposed edge in the original idx array")
      .def_readonly("ptr_t", &TransposedGraph::ptr_t)
      .def_readonly("idx_t", &TransposedGraph::idx_t)
      .def_readonly("perm", &TransposedGraph::perm)
      .def_readonly("n_edges", &TransposedGraph::n_edges)
      .def_readonly("n_src", &TransposedGraph::n_src)
      .def_readonly("n_dst", &TransposedGraph::n_dst);

  // tensor-level operations (also used by the Python-side operators)
  m.def("spmm", &spmm, py::arg("ptr"), py::arg("idx"), py::arg("x"), py::arg("n_rows"), py::arg("mean") = false,
        py::arg("val") = py::none(), py::arg("val_perm") = py::none(), py::arg("out") = py::none(),
        py::arg("accumulate") = false, py::arg("bias") = py::none());
  m.def("head_sum", &head_sum);
  m.def("edge_value_degree_raw", &edge_value_degree);
  m.def("sddmm_csr", &sddmm_csr, py::arg("ptr"), py::arg("idx"), py::arg("src_feat"), py::arg("dst_feat"),
        py::arg("n_rows"), py::arg("out") = py::none());
  m.def("sddmm_coo", &sddmm_coo);
  m.def("edge_softmax_fwd", &edge_softmax_fwd);
  m.def("edge_softmax_bwd", &edge_softmax_bwd, py::arg("ptr"), py::arg("out"), py::arg("mask"), py::arg("grad"),
        py::arg("n_dst"), py::arg("slope"), py::arg("grad_pos") = py::none());
  m.def("inverse_perm_transposed", [](const GraphPtr& g) { return inverse_perm_transposed(*g); });
  m.def("narrow_gather_sum", &narrow_gather_sum, py::arg("ptr"), py::arg("sel"), py::arg("inp"), py::arg("n_rows"),
        py::arg("rows32") = py::none());
  m.def("csr_transpose", &csr_transpose, py::arg("ptr"), py::arg("idx"), py::arg("n_rows"), py::arg("n_src"),
        py::arg("known_edges") = -1);
  m.def("csr_transpose_prefix",
        [](const GraphPtr& whole, const Tensor& ptr, int64_t n_rows, int64_t n_src, int64_t known_edges) {
          return csr_transpose_prefix(*whole, ptr, n_rows, n_src, known_edges);
        }, py::arg("whole"), py::arg("ptr"), py::arg("n_rows"), py::arg("n_src"), py::arg("known_edges") = -1);
  m.def("note_edge_counts", &note_edge_counts);
  m.def("transposed", &transposed);
  m.def("note_layer", &note_layer);
  m.def("inv_degree_transposed", [](const GraphPtr& g, const Tensor& ptr, int64_t n) { return inv_degree_transposed(*g, ptr, n); });
  m.def("rows32_transposed", [](const GraphPtr& g) { return rows32_transposed(*g); });
  m.def("clear_graph_cache", []() {
    {
      std::lock_guard<std::mutex> lock(cache().mu);
      cache().clear();
    }
    {
      std::lock_guard<std::mutex> lock(dest_cache().mu);
      dest_cache().lru.clear();
    }
    std::lock_guard<std::mutex> lock(rel_key_cache().mu);
    rel_key_cache().lru.clear();
  });
  m.def("gather_rows", &gather_rows);
  m.def("dest_groups", [](const Tensor& dest, int64_t n_rows) {
    DestPtr g = dest_groups(dest, n_rows);
    return std::make_tuple(g->ptr, g->perm);
  });
  m.def("aggr_rel", [](const Tensor& input, const Tensor& ptr, const Tensor& idx, const Tensor& etype,
                       const py::object& num_node, const py::object& num_rel) {
    return AggrRelFunction::apply(input, ptr, idx, etype, as_int(num_node), as_int(num_rel));
  });
  m.def("gather", [](const Tensor& input, const Tensor& dest, const py::object& num_node) {
    return GatherFunction::apply(input, dest, as_int(num_node));
  });
  m.def("set_graph_cache_capacity", [](int64_t n) {
    GraphCache& c = cache();
    std::lock_guard<std::mutex> lock(c.mu);
    c.capacity = n < 0 ? 0 : (size_t)n;
    while (c.lru.size() > c.capacity) {
      c.index.erase(c.lru.front().first);
      c.lru.pop_front();
    }
  });
  m.def("graph_cache_stats", []() {
    GraphCache& c = cache();
    std::lock_guard<std::mutex> lock(c.mu);
    return py::dict(py::arg("graphs") = c.lru.size(), py::arg("sorts") = c.sorts, py::arg("cuts") = c.cuts,
                    py::arg("readbacks") = g_edge_count_readbacks.load());
  });

  // the reference's names (binding.cpp:15-25, 37-41, 58-78)
  m.def("sage_sum_forward", [](const Tensor& x, const Tensor& ptr, const Tensor& idx, const py::object& n) {
    return sage_apply(x, ptr, idx, c10::nullopt, n, false);
  });
  m.def("sage_mean_forward", [](const Tensor& x, const Tensor& ptr, const Tensor& idx, const py::object& n) {
    return sage_apply(x, ptr, idx, c10::nullopt, n, true);
  });
  m.def("sage_sum_forward_edge_value",
        [](const Tensor& x, const Tensor& ptr, const Tensor& idx, const Tensor& ev, const py::object& n) {
          return sage_apply(x, ptr, idx, ev, n, false);
        });
  m.def("sage_mean_forward_edge_value",
        [](const Tensor& x, const Tensor& ptr, const Tensor& idx, const Tensor& ev, const py::object& n) {
          return sage_apply(x, ptr, idx, ev, n, true);
        });
  m.def("edge_attention",
        [](const Tensor& ptr, const Tensor& idx, const Tensor& att_dst, const Tensor& att_src, const py::object& num_edge,
           double relu_l) { return EdgeSoftmaxFunction::apply(ptr, idx, att_dst, att_src, as_int(num_edge), relu_l); },
        py::arg("ptr"), py::arg("idx"), py::arg("att_dst"), py::arg("att_src"), py::arg("num_edge"), py::arg("relu_l"));
  m.def("edge_value_degree", [](const Tensor& ptr, const py::object& num_dst, const py::object& num_edge) {
    return edge_value_degree(ptr, as_int(num_dst), as_int(num_edge));
  });
  m.def("spmv", [](const Tensor& ptr, const Tensor& idx, const Tensor& input, const py::object& num_dst) {
    return narrow_gather_sum(ptr, idx, input, as_int(num_dst), c10::nullopt);
  });
  m.def("run_spmm_configurable", &run_spmm_configurable);
  m.def("run_spmm_configurable_int32", &run_spmm_configurable);
  m.def("run_spmm_configurable_bwd", &run_spmm_configurable_bwd);
  py::enum_<MultiheadSchedule>(m, "SPMM_MULTIHEAD_SCHEDULE")
      .value("Naive", MultiheadSchedule::Naive)
      .value("PreReduce", MultiheadSchedule::PreReduce)
      .value("Optimal", MultiheadSchedule::Optimal)
      .export_values();
  m.def("spmm_multihead", &spmm_multihead, py::arg("ptr"), py::arg("idx"), py::arg("val"), py::arg("vin"),
        py::arg("num_node"), py::arg("schedule") = MultiheadSchedule::Optimal, py::arg("block_size") = 256);
  m.def("spmm_multihead_bwd", &spmm_multihead_bwd, py::arg("ptr"), py::arg("idx"), py::arg("val"), py::arg("grad_output"),
        py::arg("grad_x"), py::arg("num_node"), py::arg("schedule") = MultiheadSchedule::Optimal,
        py::arg("block_size") = 256);
  m.def("run_spmm_multihead_configurable",
        [](const Tensor& ptr, const Tensor& idx, const Tensor& val, const Tensor& vin, const py::object& num_node,
           const py::args&) { return spmm_multihead(ptr, idx, val, vin, num_node, MultiheadSchedule::PreReduce, 256); });
  m.def("run_sddmm", [](const Tensor& src, const Tensor& dst, const Tensor& src_feat, const Tensor& dst_feat, Tensor output,
                        const py::object& num_edge) { sddmm_coo(src, dst, src_feat, dst_feat, output, as_int(num_edge)); });
  m.def("run_sddmm_vertex_centric",
        [](const Tensor& ptr, const Tensor& idx, const Tensor& src_feat, const Tensor& dst_feat, const py::object& num_node,
           const py::args&) { return sddmm_csr(ptr, idx, src_feat, dst_feat, as_int(num_node), c10::nullopt); });
}
