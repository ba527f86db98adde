// TorchScript custom classes over the C ABI: the registration surface of the reference
// (src/invariant_message_passing.cpp:73-90, src/spherical_harmonics.cpp:52-69, src/cubic_spline.cpp:54-68,
// src/linear.cpp:105-137, src/symmetric_contraction.cpp:124-158) -- same namespaces, class names, method schemas
// (including the argument spelled `raidal`) and empty pickle state -- built into lib/libcuda_mace.so and loaded with
// torch.classes.load_library, exactly as the reference loads its library (ops/__init__.py:7-15).
//
// Every forward/backward is one or two calls into libcuda_mace_hip.so on torch's current HIP stream; torch only
// allocates the outputs.  Structures that depend only on the neighbour list, the species or the weights (CSR
// offsets, sender-sorted view, nodes grouped by element, folded contraction tables) are kept in a small cache that is
// valid only while the tensors they were derived from are alive and unmodified, so that they are built once per
// neighbour list / model and never outlive their source.
#include <c10/hip/HIPStream.h>
#include <torch/custom_class.h>
#include <torch/script.h>

#include <algorithm>
#include <array>
#include <cmath>
#include <map>
#include <mutex>
#include <tuple>
#include <type_traits>
#include <vector>

#include "cuda_mace_hip.h"

using torch::Tensor;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

namespace {

void *stream_of(const Tensor &t) { return c10::hip::getCurrentHIPStream(t.device().index()).stream(); }

#define CM_CALL(expr) TORCH_CHECK((expr) == 0, cm_last_error())

// Profiler range over one autograd forward or backward, as the reference's PUSH_RANGE / POP_RANGE (include/utils.h:9-21);
// emitted only when tracing is switched on (see cm_trace_push).
struct TraceRange {
  explicit TraceRange(const char *name) { cm_trace_push(name); }
  ~TraceRange() { cm_trace_pop(); }
  TraceRange(const TraceRange &) = delete;
  TraceRange &operator=(const TraceRange &) = delete;
};

void need(const Tensor &t, c10::ScalarType dtype, const char *name) {
  TORCH_CHECK(t.is_cuda(), name, " must live on the GPU (got a ", t.device(), " tensor)");
  TORCH_CHECK(t.scalar_type() == dtype, name, " must be ", dtype, " (got ", t.scalar_type(), ")");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

const float *fptr(const Tensor &t) { return t.numel() ? t.data_ptr<float>() : nullptr; }
template <typename T>
T *ptr(const Tensor &t) {
  return t.defined() && t.numel() ? t.data_ptr<T>() : nullptr;
}

// Message passing, harmonics, spline and contraction take float or double tensors, as the reference's
// AT_DISPATCH_FLOATING_TYPES does (jit_wrappers/src/invariant_message_passing_wrapper.cpp:102 and siblings); the
// linears are float only (linear_wrapper.cpp:67).
c10::ScalarType float_type_of(const Tensor &t, const char *name) {
  TORCH_CHECK(t.scalar_type() == torch::kFloat32 || t.scalar_type() == torch::kFloat64, name,
              " must be float32 or float64 (got ", t.scalar_type(), ")");
  return t.scalar_type();
}

// Calls f with a value of the scalar type that dt names.
template <typename F>
void by_dtype(c10::ScalarType dt, F &&f) {
  if (dt == torch::kFloat64)
    f(double{});
  else
    f(float{});
}

// The fp32 or the fp64 entry point of a pair, by scalar type.
template <typename T, typename A, typename B>
auto pick(A f32, B f64) {
  if constexpr (std::is_same_v<T, double>)
    return f64;
  else
    return f32;
}
const int32_t *iptr(const Tensor &t) { return t.numel() ? t.data_ptr<int32_t>() : nullptr; }

// ---- cache of derived tensors -------------------------------------------------------------------------------
// An entry is valid while every tensor it was derived from is still alive (weak reference to its TensorImpl, so the
// address cannot be recycled under the cache) and unmodified (version counter).
struct Dep {
  c10::weak_intrusive_ptr<c10::TensorImpl> impl;
  uint32_t version;
};

struct Entry {
  std::vector<Dep> deps;
  std::vector<Tensor> value;
  bool valid() const {
    for (const Dep &d : deps) {
      if (d.impl.expired()) return false;
      auto strong = d.impl.lock();
      if (!strong || strong->version_counter().current_version() != d.version) return false;
    }
    return true;
  }
};

class DerivedCache {
 public:
  using Key = std::tuple<int, const void *, int64_t>;  // kind, TensorImpl of the first dependency, extra

  template <typename Build>
  std::vector<Tensor> get(int kind, const std::vector<Tensor> &owners, int64_t extra, Build build) {
    const Key key{kind, owners[0].unsafeGetTensorImpl(), extra};
    {
      std::lock_guard<std::mutex> lock(mutex_);
      auto it = map_.find(key);
      if (it != map_.end() && it->second.deps.size() == owners.size() && it->second.valid()) {
        bool same = true;
        for (size_t i = 0; i < owners.size(); ++i)
          same = same && it->second.deps[i].impl.lock().get() == owners[i].unsafeGetTensorImpl();
        if (same) return it->second.value;
      }
    }
    Entry e;
    e.value = build();
    for (const Tensor &t : owners)
      e.deps.push_back(Dep{c10::weak_intrusive_ptr<c10::TensorImpl>(t.getIntrusivePtr()), t._version()});
    std::lock_guard<std::mutex> lock(mutex_);
    if (map_.size() >= 64) {
      for (auto it = map_.begin(); it != map_.end();) it = it->second.valid() ? std::next(it) : map_.erase(it);
      if (map_.size() >= 64) map_.clear();
    }
    map_[key] = e;
    return e.value;
  }

 private:
  std::mutex mutex_;
  std::map<Key, Entry> map_;
};

DerivedCache &cache() {
  static DerivedCache c;
  return c;
}

enum { kCsr = 1, kSorted = 2, kOneHotGroups = 3, kMonomials = 4, kTables = 5 };

Tensor csr_of(const Tensor &receiver, int64_t nnodes) {
  return cache().get(kCsr, {receiver}, nnodes, [&] {
    Tensor out = torch::empty({2 * nnodes}, receiver.options());
    CM_CALL(cm_first_occurences(iptr(receiver), receiver.numel(), nnodes, out.data_ptr<int32_t>(), stream_of(receiver)));
    return std::vector<Tensor>{out};
  })[0];
}

std::vector<Tensor> sort_by_key(const Tensor &keys, int64_t nkeys) {
  const int64_t n = keys.numel();
  Tensor perm = torch::empty({n}, keys.options());
  Tensor off = torch::empty({nkeys + 1}, keys.options());
  const size_t bytes = cm_stable_key_sort_workspace(n, nkeys);
  Tensor ws = torch::empty({static_cast<int64_t>(std::max<size_t>(bytes, 1))}, keys.options().dtype(torch::kUInt8));
  CM_CALL(cm_stable_key_sort(iptr(keys), n, nkeys, n ? perm.data_ptr<int32_t>() : nullptr, off.data_ptr<int32_t>(),
                             ws.data_ptr(), bytes, stream_of(keys)));
  return {perm, off};
}

std::vector<Tensor> sorted_view_of(const Tensor &keys, int64_t nkeys) {
  return cache().get(kSorted, {keys}, nkeys, [&] { return sort_by_key(keys, nkeys); });
}

// nodes grouped by the column where one_hot == 1; group `ne` collects the rows without such a column
std::vector<Tensor> groups_of_one_hot(const Tensor &one_hot) {
  return cache().get(kOneHotGroups, {one_hot}, 0, [&] {
    const int64_t ne = one_hot.size(1);
    Tensor mask = one_hot == 1;
    Tensor elem = mask.to(torch::kInt8).argmax(1).to(torch::kInt32);
    elem = torch::where(mask.any(1), elem, torch::full_like(elem, ne)).contiguous();
    return sort_by_key(elem, ne + 1);
  });
}

// ---- message passing -------------------------------------------------------------------------------------------
class InvariantMessagePassingTPAutograd : public torch::autograd::Function<InvariantMessagePassingTPAutograd> {
 public:
  static Tensor forward(AutogradContext *ctx, Tensor X, Tensor Y, Tensor radial, Tensor sender_list, Tensor receiver_list,
                        int64_t nnodes) {
    TraceRange range("cuda_mace:message_passing forward");
    X = X.contiguous(), Y = Y.contiguous();
    Tensor R = radial.contiguous();
    const auto dt = float_type_of(X, "X");
    need(X, dt, "X"), need(Y, dt, "Y"), need(R, dt, "radial");
    need(sender_list, torch::kInt32, "sender_list"), need(receiver_list, torch::kInt32, "receiver_list");
    TORCH_CHECK(X.dim() == 2 && X.size(0) == nnodes, "X must be [nnodes, channels]");
    const int64_t E = sender_list.numel(), C = X.size(1);
    TORCH_CHECK(Y.dim() == 2 && Y.size(0) == 16 && Y.size(1) == E, "Y must be [16, nedges]");
    TORCH_CHECK(R.numel() == E * 4 * C, "radial must hold nedges * 4 * channels values");
    Tensor first_occ = csr_of(receiver_list, nnodes);
    Tensor out = torch::empty({nnodes, 16, C}, X.options());
    by_dtype(dt, [&](auto tag) {
      using T = decltype(tag);
      CM_CALL(pick<T>(cm_mp_forward, cm_mp_forward_f64)(ptr<T>(X), ptr<T>(Y), ptr<T>(R), iptr(sender_list), iptr(first_occ),
                                                        nnodes, E, static_cast<int>(C), ptr<T>(out), stream_of(X)));
    });
    if (X.requires_grad() || Y.requires_grad() || radial.requires_grad()) {
      ctx->saved_data["nnodes"] = nnodes;
      ctx->saved_data["radial_sizes"] = radial.sizes().vec();
      ctx->save_for_backward({X, Y, R, sender_list, first_occ});
    }
    return out;
  }

  static variable_list backward(AutogradContext *ctx, variable_list grad_outputs) {
    TraceRange range("cuda_mace:message_passing backward");
    auto saved = ctx->get_saved_variables();
    const Tensor &X = saved[0], &Y = saved[1], &R = saved[2], &sender = saved[3], &first_occ = saved[4];
    const int64_t nnodes = ctx->saved_data["nnodes"].toInt();
    const int64_t E = sender.numel(), C = X.size(1);
    const bool need_x = ctx->needs_input_grad(0), need_y = ctx->needs_input_grad(1), need_r = ctx->needs_input_grad(2);
    Tensor g = grad_outputs[0].contiguous();
    need(g, X.scalar_type(), "grad_output");
    Tensor gX, gY, gR, scratch, perm, off;
    if (need_x) {
      auto view = sorted_view_of(sender, nnodes);
      perm = view[0], off = view[1];
      gX = torch::empty({nnodes, C}, X.options());
      scratch = torch::empty({E, C}, X.options());
    }
    if (need_y) gY = torch::empty({16, E}, X.options());
    if (need_r) gR = torch::empty(ctx->saved_data["radial_sizes"].toIntVector(), X.options());
    by_dtype(X.scalar_type(), [&](auto tag) {
      using T = decltype(tag);
      CM_CALL(pick<T>(cm_mp_backward, cm_mp_backward_f64)(
          ptr<T>(X), ptr<T>(Y), ptr<T>(R), ptr<T>(g), iptr(sender), iptr(first_occ), need_x ? iptr(perm) : nullptr,
          need_x ? iptr(off) : nullptr, nnodes, E, static_cast<int>(C), ptr<T>(gX), ptr<T>(gY), ptr<T>(gR), ptr<T>(scratch),
          stream_of(X)));
    });
    return {gX, gY, gR, Tensor(), Tensor(), Tensor()};
  }
};

// ---- spherical harmonics -------------------------------------------------------------------------------------
class SphericalHarmonicsAutograd : public torch::autograd::Function<SphericalHarmonicsAutograd> {
 public:
  static Tensor forward(AutogradContext *ctx, Tensor xyz) {
    TraceRange range("cuda_mace:spherical_harmonics forward");
    xyz = xyz.contiguous();
    const auto dt = float_type_of(xyz, "xyz");
    need(xyz, dt, "xyz");
    TORCH_CHECK(xyz.dim() == 2 && xyz.size(1) == 3, "xyz must be [nedges, 3]");
    Tensor Y = torch::empty({16, xyz.size(0)}, xyz.options());
    by_dtype(dt, [&](auto tag) {
      using T = decltype(tag);
      CM_CALL(pick<T>(cm_sh_forward, cm_sh_forward_f64)(ptr<T>(xyz), xyz.size(0), ptr<T>(Y), stream_of(xyz)));
    });
    if (xyz.requires_grad()) ctx->save_for_backward({xyz});
    return Y;
  }
  static variable_list backward(AutogradContext *ctx, variable_list grad_outputs) {
    TraceRange range("cuda_mace:spherical_harmonics backward");
    const Tensor xyz = ctx->get_saved_variables()[0];
    Tensor g = grad_outputs[0].contiguous();
    need(g, xyz.scalar_type(), "grad_output");
    Tensor out = torch::empty_like(xyz);
    by_dtype(xyz.scalar_type(), [&](auto tag) {
      using T = decltype(tag);
      CM_CALL(pick<T>(cm_sh_backward, cm_sh_backward_f64)(ptr<T>(xyz), ptr<T>(g), xyz.size(0), ptr<T>(out), stream_of(xyz)));
    });
    return {out};
  }
};

// ---- cubic spline ------------------------------------------------------------------------------------------------
class CubicSplineAutograd : public torch::autograd::Function<CubicSplineAutograd> {
 public:
  static Tensor forward(AutogradContext *ctx, Tensor r, Tensor r_knots, Tensor coeffs, double r_width, double r_max) {
    TraceRange range("cuda_mace:cubic_spline forward");
    Tensor rc = r.contiguous().view({-1});
    const auto dt = float_type_of(rc, "r");
    need(rc, dt, "r"), need(r_knots, dt, "r_knots"), need(coeffs, dt, "coeffs");
    TORCH_CHECK(coeffs.dim() == 3 && coeffs.size(0) == r_knots.numel() - 1 && coeffs.size(1) == 4,
                "coeffs must be [nknots - 1, 4, noutputs]");
    const int64_t E = rc.numel(), J = coeffs.size(2);
    Tensor R = torch::empty({E, J}, rc.options());
    // the reference hands r_width and r_max to its kernels as float in both precisions (cuda/src/cubic_spline_impl.cu:9-10)
    by_dtype(dt, [&](auto tag) {
      using T = decltype(tag);
      CM_CALL(pick<T>(cm_spline_forward, cm_spline_forward_f64)(
          ptr<T>(rc), ptr<T>(r_knots), ptr<T>(coeffs), E, static_cast<int>(r_knots.numel()), static_cast<int>(J),
          static_cast<float>(r_width), static_cast<float>(r_max), ptr<T>(R), static_cast<T *>(nullptr), stream_of(rc)));
    });
    if (r.requires_grad()) {
      ctx->saved_data["r_width"] = r_width;
      ctx->saved_data["r_max"] = r_max;
      ctx->saved_data["r_sizes"] = r.sizes().vec();
      ctx->save_for_backward({rc, r_knots, coeffs});
    }
    return R;
  }
  static variable_list backward(AutogradContext *ctx, variable_list grad_outputs) {
    TraceRange range("cuda_mace:cubic_spline backward");
    auto saved = ctx->get_saved_variables();
    const Tensor &r = saved[0], &knots = saved[1], &coeffs = saved[2];
    Tensor g = grad_outputs[0].contiguous();
    need(g, r.scalar_type(), "grad_output");
    Tensor out = torch::empty({r.numel()}, r.options());
    by_dtype(r.scalar_type(), [&](auto tag) {
      using T = decltype(tag);
      CM_CALL(pick<T>(cm_spline_backward, cm_spline_backward_f64)(
          ptr<T>(r), ptr<T>(knots), ptr<T>(coeffs), ptr<T>(g), r.numel(), static_cast<int>(knots.numel()),
          static_cast<int>(coeffs.size(2)), static_cast<float>(ctx->saved_data["r_width"].toDouble()),
          static_cast<float>(ctx->saved_data["r_max"].toDouble()), ptr<T>(out), stream_of(r)));
    });
    return {out.view(ctx->saved_data["r_sizes"].toIntVector()), Tensor(), Tensor(), Tensor(), Tensor()};
  }
};

// ---- linears ---------------------------------------------------------------------------------------------------------
// X [N, 16, K] (or [N, K]); WT: transposed weight blocks [ngroups, 4 | 1, Nout, K]
Tensor run_linear(const Tensor &X, const Tensor &WT, const Tensor &perm, const Tensor &off, bool zero_last_group, float scale) {
  const bool scalar = X.dim() == 2;
  const int64_t N = X.size(0), K = X.size(-1);
  const int64_t Nout = WT.size(-2);
  const int64_t ngroups = WT.numel() / ((scalar ? 1 : 4) * Nout * K);
  TORCH_CHECK(WT.size(-1) == K, "linear: weights do not match the feature width");
  Tensor out = scalar ? torch::empty({N, Nout}, X.options()) : torch::empty({N, 16, Nout}, X.options());
  const bool grouped = perm.defined();
  CM_CALL(cm_linear(fptr(X), fptr(WT), grouped ? iptr(perm) : nullptr, grouped ? iptr(off) : nullptr, N,
                    static_cast<int>(ngroups + (zero_last_group ? 1 : 0)), zero_last_group ? 1 : 0, scalar ? 1 : 16,
                    static_cast<int>(K), static_cast<int>(Nout), scale, nullptr, nullptr, N ? out.data_ptr<float>() : nullptr,
                    stream_of(X)));
  return out;
}

class LinearAutograd : public torch::autograd::Function<LinearAutograd> {
 public:
  static Tensor forward(AutogradContext *ctx, Tensor X, Tensor W, Tensor W_T) {
    TraceRange range("cuda_mace:linear forward");
    X = X.contiguous();
    need(X, torch::kFloat32, "X"), need(W, torch::kFloat32, "W"), need(W_T, torch::kFloat32, "W_T");
    TORCH_CHECK(X.dim() == 3 && X.size(1) == 16, "X must be [nnodes, 16, K]");
    const float scale = 1.0f / std::sqrt(static_cast<float>(X.size(2)));
    if (X.requires_grad()) {
      ctx->saved_data["scale"] = static_cast<double>(scale);
      ctx->save_for_backward({W});
    }
    return run_linear(X, W_T, Tensor(), Tensor(), false, scale);
  }
  static variable_list backward(AutogradContext *ctx, variable_list grad_outputs) {
    TraceRange range("cuda_mace:linear backward");
    const Tensor W = ctx->get_saved_variables()[0];
    // dX = scale * g . W^T: the operand the kernel wants is the transpose of W^T, i.e. W itself
    Tensor dX = run_linear(grad_outputs[0].contiguous(), W, Tensor(), Tensor(), false,
                           static_cast<float>(ctx->saved_data["scale"].toDouble()));
    return {dX, Tensor(), Tensor()};
  }
};

class ElementalLinearAutograd : public torch::autograd::Function<ElementalLinearAutograd> {
 public:
  static Tensor forward(AutogradContext *ctx, Tensor X, Tensor W, Tensor W_T, Tensor one_hot) {
    TraceRange range("cuda_mace:elemental_linear forward");
    X = X.contiguous();
    need(X, torch::kFloat32, "X"), need(W, torch::kFloat32, "W"), need(W_T, torch::kFloat32, "W_T");
    TORCH_CHECK((X.dim() == 3 && X.size(1) == 16) || X.dim() == 2, "X must be [nnodes, 16, K] or [nnodes, K]");
    TORCH_CHECK(one_hot.dim() == 2 && one_hot.size(1) == W.size(0), "one_hot must be [nnodes, nelements]");
    auto groups = groups_of_one_hot(one_hot);
    const float scale = 1.0f / std::sqrt(static_cast<float>(X.size(-1)));
    if (X.requires_grad()) {
      ctx->saved_data["scale"] = static_cast<double>(scale);
      ctx->save_for_backward({W, groups[0], groups[1]});
    }
    return run_linear(X, W_T, groups[0], groups[1], true, scale);
  }
  static variable_list backward(AutogradContext *ctx, variable_list grad_outputs) {
    TraceRange range("cuda_mace:elemental_linear backward");
    auto saved = ctx->get_saved_variables();
    Tensor dX = run_linear(grad_outputs[0].contiguous(), saved[0], saved[1], saved[2], true,
                           static_cast<float>(ctx->saved_data["scale"].toDouble()));
    return {dX, Tensor(), Tensor(), Tensor()};
  }
};

// ---- symmetric contraction ---------------------------------------------------------------------------------------------
// Host pass over the packed sparse coupling tables (format of ops/symmetric_contraction.py:91-187): groups the entries
// (i, j, k, path, value) by the sorted index triple they multiply.  Returns device tensors
// {mono3, off3, path3, val3, mono2, off2, path2, val2, val3 (fp64), val2 (fp64)} and whether the structure is the one compiled into the library.
struct Monomials {
  std::vector<Tensor> dev;
  bool builtin;
};

template <size_t D>
void pack_terms(const std::map<std::array<int, D>, std::map<int, double>> &terms, std::vector<int32_t> &mono,
                std::vector<int32_t> &off, std::vector<int32_t> &path, std::vector<double> &val) {
  off.push_back(0);
  for (const auto &kv : terms) {
    int32_t word = 0;
    for (size_t d = 0; d < D; ++d) word |= kv.first[d] << (8 * d);
    mono.push_back(word);
    for (const auto &pv : kv.second) {
      path.push_back(pv.first);
      val.push_back(pv.second);
    }
    off.push_back(static_cast<int32_t>(path.size()));
  }
}

Monomials monomials_of(const Tensor &U3_num, const Tensor &U3_idx, const Tensor &U3_val, const Tensor &U2_num,
                       const Tensor &U2_idx, const Tensor &U2_val) {
  std::vector<Tensor> got = cache().get(kMonomials, {U3_idx, U3_num, U3_val, U2_num, U2_idx, U2_val}, 0, [&] {
    Tensor n3 = U3_num.to(torch::kCPU, torch::kInt64).contiguous(), i3 = U3_idx.to(torch::kCPU, torch::kInt64).contiguous();
    Tensor v3 = U3_val.to(torch::kCPU, torch::kFloat64).contiguous();
    Tensor n2 = U2_num.to(torch::kCPU, torch::kInt64).contiguous(), i2 = U2_idx.to(torch::kCPU, torch::kInt64).contiguous();
    Tensor v2 = U2_val.to(torch::kCPU, torch::kFloat64).contiguous();
    std::map<std::array<int, 3>, std::map<int, double>> t3;
    std::map<std::array<int, 2>, std::map<int, double>> t2;
    const int64_t kmax = i3.size(0);
    for (int i = 0; i < 16; ++i)
      for (int j = 0; j < 16; ++j) {
        const int64_t cnt = std::min<int64_t>(n3.data_ptr<int64_t>()[i * 16 + j], kmax);
        for (int64_t t = 0; t < cnt; ++t) {
          const int64_t word = i3.data_ptr<int64_t>()[(t * 16 + i) * 16 + j];
          std::array<int, 3> key{i, j, static_cast<int>((word >> 8) & 0xFF)};
          std::sort(key.begin(), key.end());
          t3[key][static_cast<int>(word & 0xFF)] += v3.data_ptr<double>()[(t * 16 + i) * 16 + j];
        }
        if (n2.data_ptr<int64_t>()[i * 16 + j] > 0) {
          std::array<int, 2> key{std::min(i, j), std::max(i, j)};
          t2[key][static_cast<int>(i2.data_ptr<int64_t>()[i * 16 + j])] += v2.data_ptr<double>()[i * 16 + j];
        }
      }
    std::vector<int32_t> m3, o3, p3, m2, o2, p2;
    std::vector<double> w3, w2;
    pack_terms<3>(t3, m3, o3, p3, w3);
    pack_terms<2>(t2, m2, o2, p2, w2);
    int b3n = 0, b2n = 0;
    cm_symcon_builtin_structure(nullptr, 0, nullptr, 0, &b3n, &b2n);
    std::vector<int32_t> b3(b3n), b2(b2n);
    cm_symcon_builtin_structure(b3.data(), b3n, b2.data(), b2n, nullptr, nullptr);
    const bool builtin = b3 == m3 && b2 == m2;
    auto dev_i = [&](const std::vector<int32_t> &v) { return torch::tensor(v, torch::kInt32).to(U3_idx.device()); };
    auto dev_f = [&](const std::vector<double> &v, c10::ScalarType dt) {
      return torch::tensor(v, torch::kFloat64).to(U3_idx.device(), dt);
    };
    // values in both precisions: [3] / [7] fp32, [8] / [9] fp64
    return std::vector<Tensor>{dev_i(m3), dev_i(o3), dev_i(p3), dev_f(w3, torch::kFloat32), dev_i(m2), dev_i(o2), dev_i(p2),
                               dev_f(w2, torch::kFloat32), dev_f(w3, torch::kFloat64), dev_f(w2, torch::kFloat64),
                               torch::tensor({builtin ? 1 : 0}, torch::kInt32)};
  });
  Monomials m;
  m.builtin = got.back().item<int>() != 0;
  got.pop_back();
  m.dev = got;
  return m;
}

class SymmetricContractionAutograd : public torch::autograd::Function<SymmetricContractionAutograd> {
 public:
  static Tensor forward(AutogradContext *ctx, Tensor X, Tensor atom_types, int64_t U3_max_nonsparse, Tensor U3_num_nonzero,
                        Tensor U3_indices, Tensor U3_values, Tensor U2_num_nonzero, Tensor U2_indices, Tensor U2_values,
                        Tensor U1_num_nonzero, Tensor U1_index, Tensor W3, Tensor W2, Tensor W1, int64_t W3_size, int64_t W2_size,
                        int64_t W1_size) {
    TraceRange range("cuda_mace:symmetric_contraction forward");
    X = X.contiguous();
    const auto dt = float_type_of(X, "X");
    need(X, dt, "X"), need(atom_types, torch::kInt32, "atom_types");
    need(W3, dt, "W3"), need(W2, dt, "W2"), need(W1, dt, "W1");
    const bool f64 = dt == torch::kFloat64;
    TORCH_CHECK(X.dim() == 3 && X.size(1) == 16 && X.size(2) % 32 == 0, "X must be [nnodes, 16, C] with C % 32 == 0");
    const int64_t N = X.size(0), C = X.size(2);
    Monomials mono = monomials_of(U3_num_nonzero, U3_indices, U3_values, U2_num_nonzero, U2_indices, U2_values);
    const auto &d = mono.dev;
    const int n3 = static_cast<int>(d[0].numel()), n2 = static_cast<int>(d[4].numel());

    // weights are [nlout = 1, nelements, npaths, C]; only the scalar output block exists
    const int64_t ne = W3.numel() / (W3.size(-2) * C);
    const int64_t extra = (W3_size << 40) ^ (W2_size << 20) ^ W1_size;
    std::vector<Tensor> tables = cache().get(kTables, {W3, W2, W1, d[0]}, extra, [&] {
      Tensor T3 = torch::empty({ne, n3, C}, X.options()), T2 = torch::empty({ne, n2, C}, X.options());
      Tensor T1 = torch::empty({ne, C}, X.options());
      TORCH_CHECK(W3_size <= W3.size(-2) && W2_size <= W2.size(-2) && W1_size <= W1.size(-2), "weight sizes out of range");
      Tensor w3 = W3.reshape({ne, W3.size(-2), C}).narrow(1, 0, W3_size).contiguous();
      Tensor w2 = W2.reshape({ne, W2.size(-2), C}).narrow(1, 0, W2_size).contiguous();
      Tensor w1 = W1.reshape({ne, W1.size(-2), C}).narrow(1, 0, W1_size).contiguous();
      by_dtype(dt, [&](auto tag) {
        using T = decltype(tag);
        CM_CALL(pick<T>(cm_symcon_tables, cm_symcon_tables_f64)(
            iptr(d[1]), iptr(d[2]), ptr<T>(d[f64 ? 8 : 3]), n3, iptr(d[5]), iptr(d[6]), ptr<T>(d[f64 ? 9 : 7]), n2, ptr<T>(w3),
            ptr<T>(w2), ptr<T>(w1), static_cast<int>(ne), static_cast<int>(W3_size), static_cast<int>(W2_size),
            static_cast<int>(W1_size), static_cast<int>(C), ptr<T>(T3), ptr<T>(T2), ptr<T>(T1), stream_of(X)));
      });
      return std::vector<Tensor>{T3, T2, T1};
    });

    // element indices must lie in [0, nelements), as in the reference; rows of other nodes are left unwritten
    auto groups = sorted_view_of(atom_types, ne);
    const bool want_grad = X.requires_grad();
    Tensor out = torch::empty({N, C}, X.options());
    Tensor grad = want_grad ? torch::empty({N, 16, C}, X.options()) : Tensor();
    by_dtype(dt, [&](auto tag) {
      using T = decltype(tag);
      CM_CALL(pick<T>(cm_symcon_forward, cm_symcon_forward_f64)(
          ptr<T>(X), iptr(groups[0]), iptr(groups[1]), mono.builtin ? nullptr : iptr(d[0]), n3,
          mono.builtin ? nullptr : iptr(d[4]), n2, ptr<T>(tables[0]), ptr<T>(tables[1]), ptr<T>(tables[2]), N,
          static_cast<int>(ne), static_cast<int>(C), ptr<T>(out), ptr<T>(grad), stream_of(X)));
    });
    if (want_grad) ctx->save_for_backward({grad});
    return out.view({N, 1, C});
  }

  static variable_list backward(AutogradContext *ctx, variable_list grad_outputs) {
    TraceRange range("cuda_mace:symmetric_contraction backward");
    const Tensor grad = ctx->get_saved_variables()[0];
    const int64_t N = grad.size(0), C = grad.size(2);
    Tensor g = grad_outputs[0].contiguous().view({N, C});
    need(g, grad.scalar_type(), "grad_output");
    Tensor gX = torch::empty_like(grad);
    by_dtype(grad.scalar_type(), [&](auto tag) {
      using T = decltype(tag);
      CM_CALL(pick<T>(cm_symcon_backward, cm_symcon_backward_f64)(ptr<T>(grad), ptr<T>(g), N, static_cast<int>(C), ptr<T>(gX),
                                                                  stream_of(grad)));
    });
    variable_list out(17);
    out[0] = gX;
    return out;
  }
};

// ---- the classes ---------------------------------------------------------------------------------------------------------
struct Stateless : torch::CustomClassHolder {
  std::vector<Tensor> __getstate__() { return {}; }
  void __setstate__(const std::vector<Tensor> &) {}
};

struct InvariantMessagePassingTP : Stateless {
  Tensor forward(Tensor X, Tensor Y, Tensor radial, Tensor sender_list, Tensor receiver_list, int64_t nnodes) {
    return InvariantMessagePassingTPAutograd::apply(X, Y, radial, sender_list, receiver_list, nnodes);
  }
};
struct SphericalHarmonics : Stateless {
  Tensor forward(Tensor xyz) { return SphericalHarmonicsAutograd::apply(xyz); }
};
struct CubicSpline : Stateless {
  Tensor forward(Tensor r, Tensor r_knots, Tensor coeffs, double r_width, double r_max) {
    return CubicSplineAutograd::apply(r, r_knots, coeffs, r_width, r_max);
  }
};
struct Linear : Stateless {
  Tensor forward(Tensor X, Tensor W, Tensor W_T) { return LinearAutograd::apply(X, W, W_T); }
};
struct ElementalLinear : Stateless {
  Tensor forward(Tensor X, Tensor W, Tensor W_T, Tensor one_hot_encoding) {
    return ElementalLinearAutograd::apply(X, W, W_T, one_hot_encoding);
  }
};
struct SymmetricContraction : Stateless {
  Tensor forward(Tensor X, Tensor atom_types, int64_t U3_max_nonsparse, Tensor U3_num_nonzero, Tensor U3_indices,
                 Tensor U3_values, Tensor U2_num_nonzero, Tensor U2_indices, Tensor U2_values, Tensor U1_num_nonzero,
                 Tensor U1_index, Tensor W3, Tensor W2, Tensor W1, int64_t W3_size, int64_t W2_size, int64_t W1_size) {
    return SymmetricContractionAutograd::apply(X, atom_types, U3_max_nonsparse, U3_num_nonzero, U3_indices, U3_values,
                                               U2_num_nonzero, U2_indices, U2_values, U1_num_nonzero, U1_index, W3, W2, W1,
                                               W3_size, W2_size, W1_size);
  }
};

template <typename T, typename Class>
void with_pickle(Class &cls) {
  cls.def_pickle([](const c10::intrusive_ptr<T> &self) -> std::vector<Tensor> { return self->__getstate__(); },
                 [](const std::vector<Tensor> &state) -> c10::intrusive_ptr<T> {
                   auto obj = c10::make_intrusive<T>();
                   obj->__setstate__(state);
                   return obj;
                 });
}

}  // namespace

TORCH_LIBRARY(inv_message_passing, m) {
  auto cls = m.class_<InvariantMessagePassingTP>("InvariantMessagePassingTP")
                 .def(torch::init<>(), "", {})
                 .def("forward", &InvariantMessagePassingTP::forward, "",
                      {torch::arg("X"), torch::arg("Y"), torch::arg("raidal"), torch::arg("sender_list"),
                       torch::arg("receiver_list"), torch::arg("nnodes")});
  with_pickle<InvariantMessagePassingTP>(cls);
}

TORCH_LIBRARY(spherical_harmonics, m) {
  auto cls = m.class_<SphericalHarmonics>("SphericalHarmonics")
                 .def(torch::init<>(), "", {})
                 .def("forward", &SphericalHarmonics::forward, "", {torch::arg("xyz")});
  with_pickle<SphericalHarmonics>(cls);
}

TORCH_LIBRARY(cubic_spline, m) {
  auto cls = m.class_<CubicSpline>("CubicSpline")
                 .def(torch::init<>(), "", {})
                 .def("forward", &CubicSpline::forward, "",
                      {torch::arg("r"), torch::arg("r_knots"), torch::arg("coeffs"), torch::arg("r_width"), torch::arg("r_max")});
  with_pickle<CubicSpline>(cls);
}

TORCH_LIBRARY(linear_wmma, m) {
  auto lin = m.class_<Linear>("Linear")
                 .def(torch::init<>(), "", {})
                 .def("forward", &Linear::forward, "", {torch::arg("X"), torch::arg("W"), torch::arg("W_T")});
  with_pickle<Linear>(lin);
  auto el = m.class_<ElementalLinear>("ElementalLinear")
                .def(torch::init<>(), "", {})
                .def("forward", &ElementalLinear::forward, "",
                     {torch::arg("X"), torch::arg("W"), torch::arg("W_T"), torch::arg("one_hot_encoding")});
  with_pickle<ElementalLinear>(el);
}

TORCH_LIBRARY(symm_contract, m) {
  auto cls = m.class_<SymmetricContraction>("SymmetricContraction")
                 .def(torch::init<>(), "", {})
                 .def("forward", &SymmetricContraction::forward, "",
                      {torch::arg("X"), torch::arg("atom_types"), torch::arg("U3_max_nonsparse"), torch::arg("U3_num_nonzero"),
                       torch::arg("U3_indices"), torch::arg("U3_values"), torch::arg("U2_num_nonzero"), torch::arg("U2_indices"),
                       torch::arg("U2_values"), torch::arg("U1_num_nonzero"), torch::arg("U1_index"), torch::arg("W3"),
                       torch::arg("W2"), torch::arg("W1"), torch::arg("W3_size"), torch::arg("W2_size"), torch::arg("W1_size")});
  with_pickle<SymmetricContraction>(cls);
}
