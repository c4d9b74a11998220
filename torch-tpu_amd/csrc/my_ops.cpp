// Operator registration of the MoE path, the way the reference does it: a C++ extension with
//     TORCH_LIBRARY(my_ops, m) { m.def("fused_moe_fused_experts", fused_moe_fused_experts); ... }
// (torch_tpu/csrc/ops/my_ops/myOps.cpp:29-80) - function pointers, schemas inferred, all arguments positional, caller
// allocated outputs, the output alias returned, argument errors through TORCH_CHECK (fusedMoE.cpp:143,148,231).
// Signatures follow torch_tpu/csrc/ops/my_ops/ops.hpp:610-676 and 716-722.
//
// The ops forward to the C ABI of libmoe_hip.so (include/moe_hip.h) on the current HIP stream.  Plain host C++
// against the torch headers; no device code here.  What the common call needs lives here: argument checks, the
// packed copy of the reference-layout weights (made once per weight set, found again through the identity of the
// sources' storages), one workspace per (device, stream).  The rarer forms of the op - bf16 weights, block sizes
// other than 128, ragged sizes, the W8A16 arithmetic - are handed to `my_ops::_fused_experts_general`, which the
// Python package defines on the same C ABI.
#include <ATen/ATen.h>
#include <ATen/core/dispatch/Dispatcher.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>
#include <torch/library.h>

#include <array>
#include <cstdio>
#include <map>
#include <mutex>
#include <optional>
#include <sstream>
#include <string>
#include <vector>

#include "../../include/moe_hip.h"

namespace {

using at::Tensor;
using OptTensor = std::optional<Tensor>;

void check_rc(int rc, const char *what) { TORCH_CHECK(rc == 0, what, ": ", moe_hip_strerror(rc), " (code ", rc, ")"); }

void *stream_of(const Tensor &t) { return (void *)c10::hip::getCurrentHIPStream(t.device().index()).stream(); }

// ---- identity of a weight set ---------------------------------------------------------------------------------
// A packed copy belongs to the STORAGES of the tensors it was made from (not to the Python or C++ wrapper objects,
// which callers re-create freely: `param.data`, views made per call): storage, offset, shape, strides, dtype and the
// version counter.  The entry keeps weak references to the storages; once one of them has been freed the entry is
// dead and is dropped the next time the table is walked, so new weights that land on a recycled address never meet
// an old copy.  An in-place write that does not move the version counter cannot be seen from here
// (my_ops::_invalidate_weight_cache after such an update).
// (three dimensions: the callers of identify() have checked that)
struct SourceId {
  const c10::StorageImpl *storage;
  const void *data;
  int64_t offset;
  uint32_t version;
  c10::ScalarType dtype;
  int64_t sizes[3], strides[3];
  bool operator==(const SourceId &o) const {
    bool same = storage == o.storage && data == o.data && offset == o.offset && version == o.version && dtype == o.dtype;
    for (int i = 0; i < 3; i++) same = same && sizes[i] == o.sizes[i] && strides[i] == o.strides[i];
    return same;
  }
};

SourceId identify(const Tensor &t) {
  SourceId s;
  s.storage = t.unsafeGetTensorImpl()->unsafe_storage().unsafeGetStorageImpl();
  s.data = t.data_ptr();
  s.offset = t.storage_offset();
  s.version = t.is_inference() ? 0u : (uint32_t)t._version();
  s.dtype = t.scalar_type();
  for (int i = 0; i < 3; i++) {
    s.sizes[i] = t.size(i);
    s.strides[i] = t.stride(i);
  }
  return s;
}

struct PackedEntry {
  std::array<SourceId, 6> ids;
  std::vector<c10::weak_intrusive_ptr<c10::StorageImpl>> alive;
  Tensor w13, w13s, w2, w2s;
};

std::mutex g_mutex;
std::vector<PackedEntry> g_packed;
std::map<std::pair<int, void *>, Tensor> g_workspace, g_rw;
int g_numerics = 0;     // 0 = w8a8 (this file), 1 = w8a16 (general path)

// row-major weight bytes -> tile-blocked (moe_pack_weights), out of place
Tensor tile_block(const Tensor &w) {
  Tensor out = at::empty_like(w);
  const int64_t rows = w.numel() / w.size(-1);
  check_rc(moe_pack_weights(stream_of(w), w.data_ptr(), rows, (int)(w.size(-1) * w.element_size()), out.data_ptr()),
           "moe_pack_weights");
  return out;
}

// Reference argument layout (gate [E,I,H], up [E,I,H], down pre-transposed [E,I,H], bf16 scales of the same
// orientation: python/regression/test_llm/test_moe.py:285-288) -> W13 = gate rows then up rows [E,2I,H], W2 = down in
// checkpoint orientation [E,H,I], scales widened to fp32, weight bytes tile-blocked.  Values are untouched.
const PackedEntry &packed_weights(const Tensor &gate, const Tensor &up, const Tensor &down, const Tensor &gs,
                                  const Tensor &us, const Tensor &ds) {
  const Tensor *src[6] = {&gate, &up, &down, &gs, &us, &ds};
  std::array<SourceId, 6> ids;
  for (int i = 0; i < 6; i++) ids[i] = identify(*src[i]);
  for (size_t i = 0; i < g_packed.size();) {
    bool dead = false;
    for (auto &w : g_packed[i].alive) dead = dead || w.expired();
    if (dead) {
      g_packed[i] = std::move(g_packed.back());
      g_packed.pop_back();
      continue;
    }
    if (g_packed[i].ids == ids) return g_packed[i];
    i++;
  }
  PackedEntry e;
  e.ids = ids;
  for (const Tensor *t : src) e.alive.push_back(t->storage().getWeakStorageImpl());
  e.w13 = tile_block(at::cat({gate, up}, 1).contiguous());
  e.w13s = at::cat({gs, us}, 1).to(at::kFloat).contiguous();
  e.w2 = tile_block(down.transpose(1, 2).contiguous());
  e.w2s = ds.transpose(1, 2).to(at::kFloat).contiguous();
  g_packed.push_back(std::move(e));
  return g_packed.back();
}

// one scratch tensor per (device, stream), grown on demand: nothing is allocated once it is large enough
Tensor &scratch(std::map<std::pair<int, void *>, Tensor> &table, const Tensor &like, void *stream, size_t bytes,
                size_t floor_bytes) {
  Tensor &t = table[{(int)like.device().index(), stream}];
  if (!t.defined() || (size_t)t.numel() < bytes)
    t = at::empty({(int64_t)std::max(bytes, floor_bytes)}, like.options().dtype(at::kByte));
  return t;
}

// ---- enable_profile / disable_profile (torch_tpu/csrc/ops/my_ops/profile.cpp:12-44) --------------------------------
// While enabled, every op of this file brackets its work on the stream with a pair of events; disable_profile waits
// for them and reports GPU time per op (count, total, mean, min, max).  At most `max_record_num` calls are recorded.
struct ProfileRecord {
  const char *op;
  hipEvent_t start, stop;
};
bool g_profiling = false;
int64_t g_profile_max = 0, g_profile_mode = 0;
std::vector<ProfileRecord> g_profile;
std::string g_profile_report;

struct ProfileScope {
  hipEvent_t stop = nullptr;
  void *stream = nullptr;
  // call with g_mutex held
  ProfileScope(const char *op, void *st) {
    if (!g_profiling || (int64_t)g_profile.size() >= g_profile_max) return;
    ProfileRecord r{op, nullptr, nullptr};
    if (hipEventCreate(&r.start) != hipSuccess) return;
    if (hipEventCreate(&r.stop) != hipSuccess) {
      (void)hipEventDestroy(r.start);
      return;
    }
    (void)hipEventRecord(r.start, (hipStream_t)st);
    stop = r.stop;
    stream = st;
    g_profile.push_back(r);
  }
  ~ProfileScope() {
    if (stop) (void)hipEventRecord(stop, (hipStream_t)stream);
  }
};

Tensor call_general(const char *name, std::vector<c10::IValue> stack) {
  auto op = c10::Dispatcher::singleton().findSchema({name, ""});
  TORCH_CHECK(op.has_value(), name, " is not defined: this form of the op is implemented by the Python package "
              "(import torch_tpu_amd)");
  op->callBoxed(stack);
  return stack.at(0).toTensor();
}

}  // namespace

namespace at {

Tensor fused_moe_fused_experts(const Tensor &output, const Tensor &input, const OptTensor &output_sample,
                               const OptTensor &input_sample, const Tensor &gate_weights, const Tensor &up_weights,
                               const Tensor &down_weights, const OptTensor &gate_scales, const OptTensor &up_scales,
                               const OptTensor &down_scales, const Tensor &select_experts, const Tensor &routing_weights,
                               const OptTensor &num_select_experts, const OptTensor &select_experts_middle,
                               const OptTensor &routing_weights_middle, int64_t blocksize, int64_t num_experts,
                               int64_t num_experts_per_tok, bool use_grouped_topk, int64_t num_expert_group,
                               int64_t topk_group, const OptTensor &silu, const OptTensor &sigmoid, const OptTensor &m0,
                               bool save_mid_res) {
  TORCH_CHECK(select_experts.scalar_type() == at::kInt, "select_experts must be int32 dtype");
  if (num_select_experts.has_value())
    TORCH_CHECK(num_select_experts->scalar_type() == at::kLong, "num_select_experts must be int64 dtype");
  const std::pair<const char *, const OptTensor *> unpinned[] = {
      {"output_sample", &output_sample}, {"input_sample", &input_sample}, {"num_select_experts", &num_select_experts},
      {"silu", &silu},                   {"sigmoid", &sigmoid},           {"m0", &m0}};
  for (auto &p : unpinned)
    TORCH_CHECK(!p.second->has_value(), p.first, ": the reference never passes this argument and leaves its meaning "
                "undefined; it is not supported");
  TORCH_CHECK(!save_mid_res, "save_mid_res is not supported");

  const bool scaled = gate_scales.has_value() && up_scales.has_value() && down_scales.has_value();
  bool fast = scaled && blocksize == 128 && g_numerics == 0 && input.dim() == 2 && gate_weights.dim() == 3 &&
              select_experts.dim() == 2 && (output.dim() == 2 || output.dim() == 3);
  if (fast) {
    const int64_t I = gate_weights.size(1), H = gate_weights.size(2);
    fast = I % 128 == 0 && H % 128 == 0 && input.size(1) == H && gate_weights.scalar_type() == at::kFloat8_e4m3fn &&
           up_weights.scalar_type() == at::kFloat8_e4m3fn && down_weights.scalar_type() == at::kFloat8_e4m3fn &&
           up_weights.sizes() == gate_weights.sizes() && down_weights.sizes() == gate_weights.sizes() &&
           gate_scales->dim() == 3 && gate_scales->sizes() == up_scales->sizes() &&
           gate_scales->sizes() == down_scales->sizes() && gate_scales->size(1) == I / 128 &&
           gate_scales->size(2) == H / 128;
  }
  if (!fast) {
    return call_general("my_ops::_fused_experts_general",
                        {output, input, output_sample, input_sample, gate_weights, up_weights, down_weights, gate_scales,
                         up_scales, down_scales, select_experts, routing_weights, num_select_experts, select_experts_middle,
                         routing_weights_middle, blocksize, num_experts, num_experts_per_tok, use_grouped_topk,
                         num_expert_group, topk_group, silu, sigmoid, m0, save_mid_res});
  }

  const int64_t T = input.size(0), H = input.size(1), E = gate_weights.size(0), I = gate_weights.size(1);
  const int64_t K = select_experts.size(1);
  TORCH_CHECK(E == num_experts && K == num_experts_per_tok, "num_experts / num_experts_per_tok do not match the tensors");
  for (const Tensor *t : {&output, &input, &gate_weights, &up_weights, &down_weights, &*gate_scales, &*up_scales,
                          &*down_scales, &select_experts})
    TORCH_CHECK(t->is_cuda() && t->is_contiguous(), "tensors must be contiguous and on the GPU");
  TORCH_CHECK(input.scalar_type() == at::kBFloat16 && output.scalar_type() == at::kBFloat16,
              "input and output must be bfloat16");
  TORCH_CHECK(select_experts.size(0) == T, "select_experts must be [T, K]");
  const int out_mode = output.dim() == 2 ? 1 : 0;
  if (out_mode) {
    TORCH_CHECK(output.size(0) == T && output.size(1) == H, "output must be [T,H] or [T,K,H]");
  } else {
    TORCH_CHECK(output.size(0) == T && output.size(1) == K && output.size(2) == H, "output must be [T,H] or [T,K,H]");
  }

  std::lock_guard<std::mutex> lock(g_mutex);
  void *st = stream_of(input);
  ProfileScope prof("fused_moe_fused_experts", st);
  const PackedEntry &w = packed_weights(gate_weights, up_weights, down_weights, *gate_scales, *up_scales, *down_scales);
  const void *rw = nullptr;
  int rw_dtype = MOE_DTYPE_F32;
  if (out_mode) {
    // [T,H] form: the fp32 weighted sum over the slots; the reference's callers hold the weights in bf16, which the
    // library widens inside the sum
    TORCH_CHECK(routing_weights.dim() == 2 && routing_weights.size(0) == T && routing_weights.size(1) == K &&
                routing_weights.is_cuda(), "routing_weights must be [T, K]");
    if (routing_weights.scalar_type() == at::kFloat && routing_weights.is_contiguous()) {
      rw = routing_weights.data_ptr();
    } else if (routing_weights.scalar_type() == at::kBFloat16 && routing_weights.is_contiguous()) {
      rw = routing_weights.data_ptr();
      rw_dtype = MOE_DTYPE_BF16;
    } else {
      Tensor &buf = scratch(g_rw, input, st, (size_t)(T * K) * 4, 16384);
      Tensor view = buf.narrow(0, 0, T * K * 4).view(at::kFloat).view({T, K});
      view.copy_(routing_weights);
      rw = view.data_ptr();
    }
  }
  const size_t need = moe_fused_experts_workspace_bytes((int)T, (int)H, (int)I, (int)E, (int)K, 0);
  Tensor &ws = scratch(g_workspace, input, st, need, (size_t)1 << 20);
  check_rc(moe_fused_experts_fp8_rw(st, input.data_ptr(), (int)T, (int)H, (const uint8_t *)w.w13.data_ptr(),
                                    w.w13s.data_ptr<float>(), (const uint8_t *)w.w2.data_ptr(), w.w2s.data_ptr<float>(),
                                    (int)I, (int)E, select_experts.data_ptr<int32_t>(), rw, rw_dtype, (int)K, nullptr,
                                    nullptr, nullptr, nullptr, 0, output.data_ptr(), out_mode, ws.data_ptr(),
                                    (size_t)ws.numel()),
           "fused_moe_fused_experts");
  return output;
}

// the second implementation of the reference (fusedMoE.cpp:237-318): same result; its scratch tensors are accepted
// and left untouched
Tensor fused_moe_fused_experts_v2(const Tensor &output, const Tensor &input, const OptTensor &output_sample,
                                  const OptTensor &input_sample, const Tensor &gate_weights, const Tensor &up_weights,
                                  const Tensor &down_weights, const OptTensor &gate_scales, const OptTensor &up_scales,
                                  const OptTensor &down_scales, const Tensor &select_experts,
                                  const Tensor &routing_weights, const OptTensor &num_select_experts,
                                  const OptTensor &select_experts_middle, const OptTensor &routing_weights_middle,
                                  const OptTensor &gather_buffer, const OptTensor &scatter_buffer, int64_t blocksize,
                                  int64_t num_experts, int64_t num_experts_per_tok, bool use_grouped_topk,
                                  int64_t num_expert_group, int64_t topk_group, const OptTensor &silu,
                                  const OptTensor &sigmoid, const OptTensor &m0, bool save_mid_res) {
  return fused_moe_fused_experts(output, input, output_sample, input_sample, gate_weights, up_weights, down_weights,
                                 gate_scales, up_scales, down_scales, select_experts, routing_weights, num_select_experts,
                                 select_experts_middle, routing_weights_middle, blocksize, num_experts,
                                 num_experts_per_tok, use_grouped_topk, num_expert_group, topk_group, silu, sigmoid, m0,
                                 save_mid_res);
}

// torch_tpu/csrc/ops/my_ops/NoauxTcTopk.cpp:9-67: group-limited top-k into caller-allocated values / indices
Tensor noaux_tc_topk(const Tensor &values, const Tensor &indices, const Tensor &scores, int64_t n_groups,
                     int64_t topk_groups, int64_t top_k) {
  TORCH_CHECK(scores.dim() == 2, "scores must be 2D tensor");
  TORCH_CHECK(values.scalar_type() == scores.scalar_type(), "values and scores must have the same dtype");
  TORCH_CHECK(indices.scalar_type() == at::kInt, "indices must be int32");
  const int64_t T = scores.size(0), E = scores.size(1);
  TORCH_CHECK(values.dim() == 2 && values.size(0) == T && values.size(1) == top_k, "values shape must be [batch_size, top_k]");
  TORCH_CHECK(indices.dim() == 2 && indices.size(0) == T && indices.size(1) == top_k,
              "indices shape must be [batch_size, top_k]");
  TORCH_CHECK(n_groups > 0 && E % n_groups == 0, "total_size must be divisible by n_groups");
  TORCH_CHECK(topk_groups <= n_groups, "topk_groups must be <= n_groups");
  TORCH_CHECK(top_k > 0, "top_k must be positive");
  TORCH_CHECK(scores.scalar_type() == at::kFloat || scores.scalar_type() == at::kBFloat16,
              "scores must be float32 or bfloat16");
  for (const Tensor *t : {&values, &indices, &scores})
    TORCH_CHECK(t->is_cuda() && t->is_contiguous(), "tensors must be contiguous and on the GPU");
  std::lock_guard<std::mutex> lock(g_mutex);
  ProfileScope prof("noaux_tc_topk", stream_of(scores));
  check_rc(moe_noaux_tc_topk(stream_of(scores), scores.data_ptr(),
                             scores.scalar_type() == at::kFloat ? MOE_DTYPE_F32 : MOE_DTYPE_BF16, (int)T, (int)E,
                             (int)n_groups, (int)topk_groups, (int)top_k, values.data_ptr(), indices.data_ptr<int32_t>()),
           "noaux_tc_topk");
  return values;
}

// torch_tpu/csrc/ops/my_ops/fusedMoE.cpp:82-115: closed, untested and undocumented in the reference
Tensor fused_moe_grouped_topk(const Tensor &, const Tensor &, const Tensor &, const Tensor &, const Tensor &,
                              const Tensor &, const Tensor &, const Tensor &, const Tensor &, const Tensor &) {
  TORCH_CHECK(false, "fused_moe_grouped_topk: the reference's fused router is closed-source, untested and undocumented; "
              "use noaux_tc_topk or torch_tpu_amd.moe_route instead");
}

void enable_profile(std::optional<int64_t> max_record_num, std::optional<int64_t> mode) {
  std::lock_guard<std::mutex> lock(g_mutex);
  for (auto &r : g_profile) {
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  g_profile.clear();
  g_profile_max = max_record_num.value_or(40960);          // the reference's defaults (profile.cpp:17-18)
  g_profile_mode = mode.value_or(1);
  TORCH_CHECK(g_profile_max >= 0, "max_record_num must not be negative");
  g_profiling = true;
}

void disable_profile() {
  std::lock_guard<std::mutex> lock(g_mutex);
  g_profiling = false;
  struct Sum {
    int64_t n = 0;
    double total = 0, lo = 1e300, hi = 0;
  };
  std::map<std::string, Sum> per_op;
  for (auto &r : g_profile) {
    float ms = 0.f;
    if (hipEventSynchronize(r.stop) == hipSuccess && hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
      Sum &s = per_op[r.op];
      s.n++;
      s.total += ms * 1e3;
      s.lo = std::min(s.lo, (double)ms * 1e3);
      s.hi = std::max(s.hi, (double)ms * 1e3);
    }
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  g_profile.clear();
  std::ostringstream os;
  os << "my_ops profile: op, calls, total us, mean us, min us, max us\n";
  for (auto &kv : per_op)
    os << kv.first << ", " << kv.second.n << ", " << kv.second.total << ", " << kv.second.total / kv.second.n << ", "
       << kv.second.lo << ", " << kv.second.hi << "\n";
  g_profile_report = os.str();
  if (g_profile_mode != 0) std::fputs(g_profile_report.c_str(), stdout);
}

std::string _profile_report() {
  std::lock_guard<std::mutex> lock(g_mutex);
  return g_profile_report;
}

// housekeeping for the Python package: the arithmetic switch and the packed-copy table
void _set_expert_numerics(int64_t mode) {
  TORCH_CHECK(mode == 0 || mode == 1, "mode must be 0 (w8a8) or 1 (w8a16)");
  std::lock_guard<std::mutex> lock(g_mutex);
  g_numerics = (int)mode;
}

void _invalidate_weight_cache() {
  std::lock_guard<std::mutex> lock(g_mutex);
  g_packed.clear();
}

int64_t _packed_weight_sets() {
  std::lock_guard<std::mutex> lock(g_mutex);
  return (int64_t)g_packed.size();
}

TORCH_LIBRARY(my_ops, m) {
  m.def("fused_moe_grouped_topk", fused_moe_grouped_topk);
  m.def("fused_moe_fused_experts", fused_moe_fused_experts);
  m.def("fused_moe_fused_experts_v2", fused_moe_fused_experts_v2);
  m.def("noaux_tc_topk", noaux_tc_topk);
  m.def("enable_profile", enable_profile);
  m.def("disable_profile", disable_profile);
  m.def("_profile_report", _profile_report);
  m.def("_set_expert_numerics", _set_expert_numerics);
  m.def("_invalidate_weight_cache", _invalidate_weight_cache);
  m.def("_packed_weight_sets", _packed_weight_sets);
}

}  // namespace at
