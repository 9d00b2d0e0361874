// Torch extension module ascend910a_extras_C: the layer between the Python API and the C-ABI kernel
// library libaops.so.  It takes the place of the reference's pybind module of the same name
// (reference csrc/ffi/bind.cpp:53-61 and csrc/ffi/ops.cpp:13-491): an `ops` submodule with one
// function per operator, plus print_info.  Each function repeats the reference's argument checks
// (same conditions, TORCH_CHECK -> RuntimeError), allocates the outputs with at::empty*, looks up
// torch's current HIP stream and makes one aops_* call with raw device pointers.  Nothing here
// synchronises or reads device data on the host, and there is no CPU path: tensors that are not on
// the GPU are refused.
//
// Host code only (no kernels): compiled with the C++ compiler against the torch headers and linked
// against libaops.so, which sits next to the module.
#include <ATen/ATen.h>
#include <ATen/hip/EmptyTensor.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <c10/hip/HIPStream.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>
#include <torch/csrc/utils/pybind.h>

#include <optional>
#include <string>
#include <tuple>
#include <vector>

#include "aops.h"

namespace py = pybind11;
using at::Tensor;

namespace {

// dtype and device checks (the reference hard-codes ACL_FLOAT16 / ACL_INT32 / ACL_INT64).
struct Arg {
  const char* name;
  const Tensor& t;
  at::ScalarType dtype;
};

const char* dtype_name(at::ScalarType t) {
  switch (t) {
    case at::kHalf: return "torch.float16";
    case at::kFloat: return "torch.float32";
    case at::kInt: return "torch.int32";
    case at::kLong: return "torch.int64";
    default: return c10::toString(t);
  }
}

void require_device(const char* op, std::initializer_list<Arg> args) {
  const Tensor* first = nullptr;
  for (const Arg& a : args) {
    TORCH_CHECK(a.t.scalar_type() == a.dtype, op, ": ", a.name, " must be ", dtype_name(a.dtype), ", got ",
                dtype_name(a.t.scalar_type()));
    TORCH_CHECK(a.t.is_cuda(), op, ": ", a.name, " must be on the GPU device, got ", a.t.device());
    if (!first) {
      first = &a.t;
    } else {
      TORCH_CHECK(a.t.device() == first->device(), op, ": all tensors must be on the same device");
    }
  }
}

// Device address of t (null for an empty tensor).  The kernels move 128 bits per lane, so fp16 data
// must start on a 16-byte boundary; index tensors are read element by element.
void* dev_ptr(const Tensor& t) {
  if (t.numel() == 0) return nullptr;
  void* p = t.data_ptr();
  TORCH_CHECK(t.scalar_type() != at::kHalf || (reinterpret_cast<uintptr_t>(p) & 15) == 0,
              "fp16 tensor data must be 16-byte aligned (a view that starts inside a row is not)");
  return p;
}

void* dev_ptr(const std::optional<Tensor>& t) { return t.has_value() ? dev_ptr(*t) : nullptr; }

// Makes the tensors' device current for the call and hands out torch's current stream on it.
struct Launch {
  c10::hip::HIPGuardMasqueradingAsCUDA guard;
  void* stream;
  explicit Launch(const Tensor& t)
      : guard(t.device()), stream(c10::hip::getCurrentHIPStream(t.device().index()).stream()) {}
};

void status(const char* op, int code) {
  if (code == AOPS_OK) return;
  if (code == AOPS_ERR_LAUNCH)
    TORCH_CHECK(false, op, ": ", aops_strerror(code), " (hipError ", aops_last_hip_error(), ")");
  TORCH_CHECK(false, op, ": ", aops_strerror(code));
}

// Output allocation straight from the caching allocator (what at::empty arrives at after its dispatch):
// the operators of a decode step take a few microseconds, so the host cost per call matters.
Tensor fresh(const Tensor& like, at::IntArrayRef sizes, at::ScalarType dtype) {
  return Tensor(at::detail::empty_cuda(sizes, dtype, like.device(), std::nullopt));
}
Tensor fresh_like(const Tensor& t) { return fresh(t, t.sizes(), t.scalar_type()); }

Tensor scratch(const Tensor& like, size_t bytes) { return fresh(like, {(int64_t)bytes}, at::kByte); }

// ---- the reference's six operators ---------------------------------------------------------------

// reference csrc/ffi/ops.cpp:13-108
std::vector<Tensor> rope(const Tensor& q, const Tensor& k, const Tensor& position_ids,
                         const Tensor& cos_cache, const Tensor& sin_cache) {
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && position_ids.dim() == 1 && cos_cache.dim() == 2 &&
                  sin_cache.dim() == 2,
              "rope: input tensors must be 3D, 3D, 1D, 2D, and 2D, got ", q.dim(), "D, ", k.dim(), "D, ",
              position_ids.dim(), "D, ", cos_cache.dim(), "D, ", sin_cache.dim(), "D");
  TORCH_CHECK(position_ids.size(0) == q.size(0),
              "rope: position_ids must have the same batch size as q, got ", position_ids.size(0), " and ",
              q.size(0));
  TORCH_CHECK(q.is_contiguous() && k.is_contiguous() && position_ids.is_contiguous() &&
                  cos_cache.is_contiguous() && sin_cache.is_contiguous(),
              "rope: all input tensors must be contiguous");
  const int64_t bs = q.size(0), num_heads = q.size(1), head_dim = q.size(2);
  TORCH_CHECK(k.size(0) == bs && k.size(2) == head_dim, "rope: k must match q in batch size and head_dim");
  TORCH_CHECK(head_dim % 16 == 0, "rope: head_dim must be a multiple of 16, got ", head_dim);
  TORCH_CHECK(cos_cache.size(1) == head_dim / 2 && sin_cache.sizes() == cos_cache.sizes(),
              "rope: cos_cache and sin_cache must be [max_position, head_dim/2], got ", cos_cache.sizes(),
              " and ", sin_cache.sizes());
  require_device("rope", {{"q", q, at::kHalf},
                          {"k", k, at::kHalf},
                          {"position_ids", position_ids, at::kInt},
                          {"cos_cache", cos_cache, at::kHalf},
                          {"sin_cache", sin_cache, at::kHalf}});
  Tensor out_q = fresh_like(q);
  Tensor out_k = fresh_like(k);
  Launch l(q);
  status("rope", aops_rope_neox_f16(dev_ptr(q), dev_ptr(k), static_cast<const int32_t*>(dev_ptr(position_ids)),
                                    dev_ptr(cos_cache), dev_ptr(sin_cache), dev_ptr(out_q), dev_ptr(out_k), bs,
                                    num_heads, k.size(1), head_dim, l.stream));
  return {out_q, out_k};
}

// reference csrc/ffi/ops.cpp:110-154
Tensor swiglu(const Tensor& x) {
  TORCH_CHECK(x.dim() == 2, "swiglu: input tensor must be 2D, got ", x.dim(), "D tensor");
  TORCH_CHECK(x.size(-1) >= 64 && x.size(-1) % 64 == 0, "swiglu: last dimension must be a multiple of 64, got ",
              x.size(-1));
  TORCH_CHECK(x.is_contiguous(), "swiglu: input tensor must be contiguous");
  require_device("swiglu", {{"x", x, at::kHalf}});
  Tensor y = fresh(x, {x.size(0), x.size(1) / 2}, x.scalar_type());
  Launch l(x);
  status("swiglu", aops_swiglu_f16(dev_ptr(x), dev_ptr(y), x.size(0), x.size(1) / 2, l.stream));
  return y;
}

// Argument checks of reference csrc/ffi/ops.cpp:158-174 plus dtype, device and packing.
void check_grouped_matmul(const char* name, const Tensor& x, const Tensor& w, const Tensor& group_list) {
  TORCH_CHECK(x.dim() == 2 && w.dim() == 3 && group_list.dim() == 1, name,
              ": input tensors must be 2D and group_list must be 1D");
  const int64_t dim = x.size(1), num_experts = w.size(0), inner_dim = w.size(2);
  TORCH_CHECK(dim == w.size(1), name, ": last dimension of x must match second dimension of w, got ", dim,
              " and ", w.size(1));
  TORCH_CHECK(x.is_contiguous() && group_list.is_contiguous(), name,
              ": x and group_list must be contiguous tensors");
  TORCH_CHECK(w.stride(1) == 1 && w.stride(2) == dim, name, ": w must be K-major order, got strides ",
              w.strides());
  TORCH_CHECK(w.size(1) % 64 == 0 && w.size(2) % 64 == 0, name,
              ": second and third dimensions of w must be multiples of 64, got ", w.size(1), " and ", w.size(2));
  TORCH_CHECK(num_experts <= 1 || w.stride(0) == dim * inner_dim, name,
              ": experts of w must be densely packed, got strides ", w.strides());
  TORCH_CHECK(group_list.size(0) == num_experts, name, ": group_list must have one entry per expert, got ",
              group_list.size(0), " and ", num_experts);
  require_device(name, {{"x", x, at::kHalf}, {"w", w, at::kHalf}, {"group_list", group_list, at::kLong}});
}

// reference csrc/ffi/ops.cpp:157-233; the workspace phase maps onto aops_grouped_matmul_workspace
Tensor grouped_matmul(const Tensor& x, const Tensor& w, const Tensor& group_list) {
  check_grouped_matmul("grouped_matmul", x, w, group_list);
  const int64_t rows = x.size(0), dim = x.size(1), num_experts = w.size(0), inner_dim = w.size(2);
  Tensor y = fresh(x, {rows, inner_dim}, x.scalar_type());
  Launch l(x);
  const size_t ws_bytes = aops_grouped_matmul_workspace(rows, dim, num_experts, inner_dim);
  Tensor ws;
  if (ws_bytes > 0) ws = scratch(x, ws_bytes);
  status("grouped_matmul",
         aops_grouped_matmul_ws_f16(dev_ptr(x), dev_ptr(w), static_cast<const int64_t*>(dev_ptr(group_list)),
                                    dev_ptr(y), ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, rows, dim,
                                    num_experts, inner_dim, l.stream));
  return y;
}

// reference csrc/ffi/ops.cpp:236-333
std::tuple<Tensor, Tensor> add_rms_norm(const Tensor& x, const Tensor& residual, const Tensor& weight,
                                        double epsilon) {
  TORCH_CHECK(x.dim() == 2 && residual.dim() == 2 && weight.dim() == 1,
              "add_rms_norm: x and residual must be 2D, weight must be 1D");
  TORCH_CHECK(x.size(1) == weight.size(0), "add_rms_norm: last dimension of x must match weight size, got ",
              x.size(1), " and ", weight.size(0));
  TORCH_CHECK(x.size(0) == residual.size(0) && x.size(1) == residual.size(1),
              "add_rms_norm: x and residual must have the same shape, got ", x.sizes(), " and ",
              residual.sizes());
  TORCH_CHECK(x.is_contiguous() && residual.is_contiguous() && weight.is_contiguous(),
              "add_rms_norm: all input tensors must be contiguous");
  TORCH_CHECK(x.size(1) % 64 == 0, "add_rms_norm: last dimension must be a multiple of 64, got ", x.size(1));
  require_device("add_rms_norm",
                 {{"x", x, at::kHalf}, {"residual", residual, at::kHalf}, {"weight", weight, at::kHalf}});
  Tensor y = fresh_like(x);
  Tensor residual_output = fresh_like(x);
  Launch l(x);
  status("add_rms_norm",
         aops_add_rms_norm_f16(dev_ptr(x), dev_ptr(residual), dev_ptr(weight), (float)epsilon, dev_ptr(y),
                               dev_ptr(residual_output), x.size(0), x.size(1), l.stream));
  return {y, residual_output};
}

// reference csrc/ffi/ops.cpp:336-405; an empty value / value_cache means "not given"
void reshape_and_cache(const Tensor& key, const Tensor& value, const Tensor& key_cache,
                       const Tensor& value_cache, const Tensor& slot_indices) {
  TORCH_CHECK(key.dim() == 3 && key_cache.dim() == 4 && slot_indices.dim() == 1,
              "reshape_and_cache: key must be 3D, key_cache must be 4D, slot_indices must be 1D");
  TORCH_CHECK(key.is_contiguous() && key_cache.is_contiguous() && slot_indices.is_contiguous(),
              "reshape_and_cache: key, key_cache, slot_indices must be contiguous tensors");
  if (value.numel() > 0)
    TORCH_CHECK(value.dim() == 3 && value.is_contiguous(),
                "reshape_and_cache: value must be 3D and contiguous if not None");
  if (value_cache.numel() > 0)
    TORCH_CHECK(value_cache.dim() == 4 && value_cache.is_contiguous(),
                "reshape_and_cache: value_cache must be 4D and contiguous if not None");
  const int64_t num_tokens = key.size(0), num_kv_heads = key.size(1), head_size = key.size(2);
  const int64_t num_blocks = key_cache.size(0), nh16 = key_cache.size(1), block_size = key_cache.size(2),
                chunk = key_cache.size(3);
  // reference csrc/opdev/op_host/reshape_and_cache_ex.cpp:31-36
  TORCH_CHECK(slot_indices.size(0) == num_tokens, "reshape_and_cache: slot_indices length must equal num_tokens, got ",
              slot_indices.size(0), " and ", num_tokens);
  TORCH_CHECK(chunk == 16 && nh16 * 16 == num_kv_heads * head_size,
              "reshape_and_cache: key_cache must be [num_blocks, num_kv_heads*head_size/16, block_size, 16], got ",
              key_cache.sizes(), " for key ", key.sizes());
  // "None" arrives as an empty 1-D tensor; a batch of zero tokens is an empty 3-D value and still "given".
  // One of the two without the other would silently leave the V cache stale.
  const bool value_given = value.numel() > 0 || value.dim() == 3;
  const bool value_cache_given = value_cache.numel() > 0 || value_cache.dim() == 4;
  TORCH_CHECK(value_given == value_cache_given,
              "reshape_and_cache: value and value_cache must be given together (or both be None)");
  const bool with_value = value_given;
  if (with_value) {
    TORCH_CHECK(value.sizes() == key.sizes(), "reshape_and_cache: value must have the shape of key");
    TORCH_CHECK(value_cache.sizes() == key_cache.sizes(),
                "reshape_and_cache: value_cache must have the shape of key_cache");
    require_device("reshape_and_cache", {{"key", key, at::kHalf},
                                         {"key_cache", key_cache, at::kHalf},
                                         {"slot_indices", slot_indices, at::kInt},
                                         {"value", value, at::kHalf},
                                         {"value_cache", value_cache, at::kHalf}});
  } else {
    require_device("reshape_and_cache", {{"key", key, at::kHalf},
                                         {"key_cache", key_cache, at::kHalf},
                                         {"slot_indices", slot_indices, at::kInt}});
  }
  Launch l(key);
  status("reshape_and_cache",
         aops_reshape_and_cache_f16(dev_ptr(key), with_value ? dev_ptr(value) : nullptr, dev_ptr(key_cache),
                                    with_value ? dev_ptr(value_cache) : nullptr,
                                    static_cast<const int32_t*>(dev_ptr(slot_indices)), num_tokens,
                                    num_kv_heads * head_size, num_blocks, block_size, l.stream));
}

// reference csrc/ffi/ops.cpp:408-482 (which performs no checks; the shapes it assumes are enforced here)
Tensor paged_attention(const Tensor& q, const Tensor& key_cache, const Tensor& value_cache,
                       const Tensor& block_tables, const Tensor& context_lens) {
  TORCH_CHECK(q.dim() == 3 && key_cache.dim() == 4 && value_cache.dim() == 4 && block_tables.dim() == 2 &&
                  context_lens.dim() == 1,
              "paged_attention: q must be 3D, key_cache and value_cache 4D, block_tables 2D, context_lens 1D");
  TORCH_CHECK(q.is_contiguous() && key_cache.is_contiguous() && value_cache.is_contiguous() &&
                  block_tables.is_contiguous() && context_lens.is_contiguous(),
              "paged_attention: all input tensors must be contiguous");
  const int64_t bs = q.size(0), num_heads = q.size(1), head_dim = q.size(2);
  const int64_t num_blocks = key_cache.size(0), nh16 = key_cache.size(1), block_size = key_cache.size(2),
                chunk = key_cache.size(3);
  TORCH_CHECK(chunk == 16, "paged_attention: last dimension of the caches must be 16, got ", chunk);
  TORCH_CHECK(value_cache.sizes() == key_cache.sizes(),
              "paged_attention: key_cache and value_cache must have the same shape");
  TORCH_CHECK(head_dim > 0 && (nh16 * 16) % head_dim == 0 && nh16 * 16 >= head_dim,
              "paged_attention: cache rows (", nh16 * 16, " halfs) must hold whole heads of ", head_dim);
  const int64_t num_kv_heads = nh16 * 16 / head_dim;
  TORCH_CHECK(num_heads % num_kv_heads == 0, "paged_attention: num_heads (", num_heads,
              ") must be a multiple of num_kv_heads (", num_kv_heads, ")");
  TORCH_CHECK(block_tables.size(0) == bs && context_lens.size(0) == bs,
              "paged_attention: block_tables and context_lens must have one row per sequence");
  require_device("paged_attention", {{"q", q, at::kHalf},
                                     {"key_cache", key_cache, at::kHalf},
                                     {"value_cache", value_cache, at::kHalf},
                                     {"block_tables", block_tables, at::kInt},
                                     {"context_lens", context_lens, at::kInt}});
  const int64_t max_blocks = block_tables.size(1);
  Tensor o = fresh_like(q);
  if (bs == 0) return o;
  Launch l(q);
  const size_t ws_bytes =
      aops_paged_attention_workspace(bs, num_heads, num_kv_heads, head_dim, block_size, max_blocks);
  TORCH_CHECK(ws_bytes > 0, "paged_attention: unsupported shape (head_dim=", head_dim, ", block_size=", block_size,
              "); head_dim must be a multiple of 16 up to 256");
  Tensor ws = scratch(q, ws_bytes);
  status("paged_attention",
         aops_paged_attention_f16(dev_ptr(q), dev_ptr(key_cache), dev_ptr(value_cache),
                                  static_cast<const int32_t*>(dev_ptr(block_tables)),
                                  static_cast<const int32_t*>(dev_ptr(context_lens)), dev_ptr(o), ws.data_ptr(),
                                  ws_bytes, bs, num_heads, num_kv_heads, head_dim, block_size, max_blocks,
                                  num_blocks, l.stream));
  return o;
}

// reference csrc/ffi/bind.cpp:26-51
void print_info(int device_id) {
  char buf[1024];
  const int n = aops_device_info(device_id, buf, sizeof(buf));
  status("print_info", n < 0 ? n : 0);
  py::print(std::string(buf, (size_t)n), py::arg("end") = "");
}

// ---- beyond the reference's surface ----------------------------------------------------------------

// y = x @ w.T for x [m, k], w [n, k]: reference legacy tree _csrc/ffi.cpp:408-442
Tensor matmul(const Tensor& x, const Tensor& w) {
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2, "matmul: input tensors must be 2D");
  TORCH_CHECK(x.size(1) == w.size(1), "matmul: last dimension of x must match last dimension of w, got ",
              x.size(1), " and ", w.size(1));
  TORCH_CHECK(x.is_contiguous() && w.is_contiguous(), "matmul: x and w must be contiguous tensors");
  const int64_t m = x.size(0), k = x.size(1), n = w.size(0);
  TORCH_CHECK(k % 64 == 0 && n % 64 == 0, "matmul: k and n must be multiples of 64, got k=", k, " and n=", n);
  require_device("matmul", {{"x", x, at::kHalf}, {"w", w, at::kHalf}});
  Tensor y = fresh(x, {m, n}, x.scalar_type());
  Launch l(x);
  const size_t ws_bytes = m > 0 ? aops_matmul_nt_workspace(m, k, n) : 0;
  Tensor ws;
  if (ws_bytes > 0) ws = scratch(x, ws_bytes);
  status("matmul", aops_matmul_nt_ws_f16(dev_ptr(x), dev_ptr(w), dev_ptr(y), ws_bytes ? ws.data_ptr() : nullptr,
                                         ws_bytes, m, k, n, l.stream));
  return y;
}

// swiglu(grouped_matmul(x, w, group_list)) in one kernel: fuses the chain reference csrc/ffi/ops.cpp:157-233
// -> 110-154 of an expert MLP.
Tensor grouped_matmul_swiglu(const Tensor& x, const Tensor& w, const Tensor& group_list) {
  check_grouped_matmul("grouped_matmul_swiglu", x, w, group_list);
  const int64_t rows = x.size(0), dim = x.size(1), num_experts = w.size(0), inner_dim = w.size(2);
  Tensor y = fresh(x, {rows, inner_dim / 2}, x.scalar_type());
  Launch l(x);
  status("grouped_matmul_swiglu",
         aops_grouped_matmul_swiglu_f16(dev_ptr(x), dev_ptr(w), static_cast<const int64_t*>(dev_ptr(group_list)),
                                        dev_ptr(y), rows, dim, num_experts, inner_dim, l.stream));
  return y;
}

// x_sorted[j] = x[sorted_idx[j] / topk] for the routed rows (later rows are left unwritten)
Tensor moe_gather(const Tensor& x, const Tensor& sorted_idx, const Tensor& group_list, int64_t topk) {
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous() && sorted_idx.dim() == 1 && sorted_idx.is_contiguous() &&
                  group_list.dim() == 1 && group_list.is_contiguous(),
              "moe_gather: x must be 2D, sorted_idx and group_list 1D, all contiguous");
  TORCH_CHECK(topk > 0 && sorted_idx.numel() == x.size(0) * topk,
              "moe_gather: sorted_idx must have tokens*topk entries, got ", sorted_idx.numel(), " for ", x.size(0),
              " tokens, topk ", topk);
  TORCH_CHECK(x.size(1) % 8 == 0, "moe_gather: hidden must be a multiple of 8, got ", x.size(1));
  require_device("moe_gather",
                 {{"x", x, at::kHalf}, {"sorted_idx", sorted_idx, at::kInt}, {"group_list", group_list, at::kLong}});
  const int64_t n = sorted_idx.numel();
  Tensor out = fresh(x, {n, x.size(1)}, x.scalar_type());
  Launch l(x);
  status("moe_gather",
         aops_moe_gather_f16(dev_ptr(x), static_cast<const int32_t*>(dev_ptr(sorted_idx)),
                             static_cast<const int64_t*>(dev_ptr(group_list)), dev_ptr(out), n, topk, x.size(1),
                             group_list.numel(), l.stream));
  return out;
}

// grouped_matmul_swiglu(moe_gather(x, sorted_idx, group_list, topk), w, group_list) without the gathered copy
Tensor grouped_matmul_swiglu_gather(const Tensor& x, const Tensor& sorted_idx, int64_t topk, const Tensor& w,
                                    const Tensor& group_list) {
  const char* name = "grouped_matmul_swiglu_gather";
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous() && sorted_idx.dim() == 1 && sorted_idx.is_contiguous(), name,
              ": x must be 2D, sorted_idx 1D, both contiguous");
  TORCH_CHECK(topk > 0 && sorted_idx.numel() == x.size(0) * topk, name,
              ": sorted_idx must have tokens*topk entries, got ", sorted_idx.numel(), " for ", x.size(0),
              " tokens, topk ", topk);
  const int64_t rows = sorted_idx.numel(), dim = x.size(1);
  if (x.size(0) * dim >= ((int64_t)1 << 32))  // the kernel addresses the rows of x with 32-bit offsets
    return grouped_matmul_swiglu(moe_gather(x, sorted_idx, group_list, topk), w, group_list);
  // the remaining checks are those of grouped_matmul on the (virtual) gathered matrix
  TORCH_CHECK(w.dim() == 3 && group_list.dim() == 1 && group_list.is_contiguous(), name,
              ": w must be 3D, group_list 1D");
  TORCH_CHECK(dim == w.size(1), name, ": last dimension of x must match second dimension of w, got ", dim, " and ",
              w.size(1));
  TORCH_CHECK(w.stride(1) == 1 && w.stride(2) == dim, name, ": w must be K-major order, got strides ", w.strides());
  TORCH_CHECK(w.size(2) % 64 == 0, name, ": third dimension of w must be a multiple of 64, got ", w.size(2));
  const int64_t num_experts = w.size(0), inner_dim = w.size(2);
  TORCH_CHECK(num_experts <= 1 || w.stride(0) == dim * inner_dim, name, ": experts of w must be densely packed");
  TORCH_CHECK(group_list.size(0) == num_experts, name, ": group_list must have one entry per expert");
  require_device(name, {{"x", x, at::kHalf},
                        {"w", w, at::kHalf},
                        {"group_list", group_list, at::kLong},
                        {"sorted_idx", sorted_idx, at::kInt}});
  Tensor y = fresh(x, {rows, inner_dim / 2}, x.scalar_type());
  Launch l(x);
  status(name, aops_grouped_matmul_swiglu_gather_f16(
                   dev_ptr(x), static_cast<const int32_t*>(dev_ptr(sorted_idx)), topk, x.size(0), dev_ptr(w),
                   static_cast<const int64_t*>(dev_ptr(group_list)), dev_ptr(y), rows, dim, num_experts, inner_dim,
                   l.stream));
  return y;
}

// rope -> reshape_and_cache in one kernel (order of reference csrc/ffi/graph.cpp:255-270); with norm weights
// the per-head RMSNorm of reference csrc/ffi/graph.cpp:252-253 runs in front of the rotation.
py::object rope_reshape_and_cache(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& position_ids,
                                  const Tensor& cos_cache, const Tensor& sin_cache, const Tensor& key_cache,
                                  const Tensor& value_cache, const Tensor& slot_indices, bool return_k,
                                  const std::optional<Tensor>& q_norm_weight,
                                  const std::optional<Tensor>& k_norm_weight, double epsilon) {
  const char* name = "rope_reshape_and_cache";
  const bool norm = q_norm_weight.has_value() || k_norm_weight.has_value();
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3 && position_ids.dim() == 1 && cos_cache.dim() == 2 &&
                  sin_cache.dim() == 2 && key_cache.dim() == 4 && value_cache.dim() == 4 && slot_indices.dim() == 1,
              name, ": q, k, v must be 3D, position_ids and slot_indices 1D, cos_cache and sin_cache 2D, caches 4D");
  TORCH_CHECK(q.is_contiguous() && k.is_contiguous() && v.is_contiguous() && position_ids.is_contiguous() &&
                  cos_cache.is_contiguous() && sin_cache.is_contiguous() && key_cache.is_contiguous() &&
                  value_cache.is_contiguous() && slot_indices.is_contiguous(),
              name, ": all input tensors must be contiguous");
  const int64_t bs = q.size(0), num_heads = q.size(1), head_dim = q.size(2), num_kv_heads = k.size(1);
  TORCH_CHECK(k.size(0) == bs && k.size(2) == head_dim && v.sizes() == k.sizes(), name,
              ": k and v must be [bs, num_kv_heads, head_dim] matching q");
  TORCH_CHECK(position_ids.size(0) == bs && slot_indices.size(0) == bs, name,
              ": position_ids and slot_indices must have one entry per token");
  TORCH_CHECK(head_dim % 16 == 0, name, ": head_dim must be a multiple of 16, got ", head_dim);
  TORCH_CHECK(cos_cache.size(1) == head_dim / 2 && sin_cache.sizes() == cos_cache.sizes(), name,
              ": cos_cache and sin_cache must be [max_position, head_dim/2]");
  const int64_t num_blocks = key_cache.size(0), nh16 = key_cache.size(1), block_size = key_cache.size(2),
                chunk = key_cache.size(3);
  TORCH_CHECK(chunk == 16 && nh16 * 16 == num_kv_heads * head_dim && value_cache.sizes() == key_cache.sizes(), name,
              ": caches must be [num_blocks, num_kv_heads*head_dim/16, block_size, 16], got ", key_cache.sizes(),
              " and ", value_cache.sizes());
  require_device(name, {{"q", q, at::kHalf},
                        {"k", k, at::kHalf},
                        {"v", v, at::kHalf},
                        {"position_ids", position_ids, at::kInt},
                        {"cos_cache", cos_cache, at::kHalf},
                        {"sin_cache", sin_cache, at::kHalf},
                        {"key_cache", key_cache, at::kHalf},
                        {"value_cache", value_cache, at::kHalf},
                        {"slot_indices", slot_indices, at::kInt}});
  Tensor out_q = fresh_like(q);
  Tensor out_k;
  if (return_k) out_k = fresh_like(k);
  Launch l(q);
  int code;
  if (norm) {
    TORCH_CHECK(q_norm_weight.has_value() && k_norm_weight.has_value(), name, ": give both norm weights or none");
    TORCH_CHECK(q_norm_weight->dim() == 1 && k_norm_weight->dim() == 1 && q_norm_weight->size(0) == head_dim &&
                    k_norm_weight->size(0) == head_dim && q_norm_weight->is_contiguous() &&
                    k_norm_weight->is_contiguous(),
                name, ": norm weights must be contiguous [head_dim] tensors");
    require_device(name, {{"q_norm_weight", *q_norm_weight, at::kHalf}, {"k_norm_weight", *k_norm_weight, at::kHalf}});
    code = aops_qknorm_rope_reshape_and_cache_f16(
        dev_ptr(q), dev_ptr(k), dev_ptr(v), dev_ptr(q_norm_weight), dev_ptr(k_norm_weight), (float)epsilon,
        static_cast<const int32_t*>(dev_ptr(position_ids)), dev_ptr(cos_cache), dev_ptr(sin_cache), dev_ptr(out_q),
        return_k ? dev_ptr(out_k) : nullptr, dev_ptr(key_cache), dev_ptr(value_cache),
        static_cast<const int32_t*>(dev_ptr(slot_indices)), bs, num_heads, num_kv_heads, head_dim, num_blocks,
        block_size, l.stream);
  } else {
    code = aops_rope_reshape_and_cache_f16(
        dev_ptr(q), dev_ptr(k), dev_ptr(v), static_cast<const int32_t*>(dev_ptr(position_ids)), dev_ptr(cos_cache),
        dev_ptr(sin_cache), dev_ptr(out_q), return_k ? dev_ptr(out_k) : nullptr, dev_ptr(key_cache),
        dev_ptr(value_cache), static_cast<const int32_t*>(dev_ptr(slot_indices)), bs, num_heads, num_kv_heads,
        head_dim, num_blocks, block_size, l.stream);
  }
  status(name, code);
  if (return_k) return py::cast(std::vector<Tensor>{out_q, out_k});
  return py::cast(out_q);
}

// Stable sort of the flattened routing by expert: (sorted_idx, inverse_idx, group_list)
std::tuple<Tensor, Tensor, Tensor> moe_sort(const Tensor& topk_ids, int64_t num_experts) {
  TORCH_CHECK((topk_ids.dim() == 1 || topk_ids.dim() == 2) && topk_ids.is_contiguous(),
              "moe_sort: topk_ids must be a contiguous 1D or 2D tensor");
  TORCH_CHECK(num_experts > 0 && num_experts <= 4095, "moe_sort: num_experts must be in 1..4095, got ", num_experts);
  require_device("moe_sort", {{"topk_ids", topk_ids, at::kInt}});
  const int64_t n = topk_ids.numel();
  Tensor sorted_idx = fresh(topk_ids, {n}, topk_ids.scalar_type());
  Tensor inverse_idx = fresh(topk_ids, {n}, topk_ids.scalar_type());
  Tensor group_list = fresh(topk_ids, {num_experts}, at::kLong);
  Launch l(topk_ids);
  const size_t ws_bytes = aops_moe_sort_workspace(n, num_experts);
  TORCH_CHECK(ws_bytes > 0, "moe_sort: unsupported size n=", n, ", num_experts=", num_experts);
  Tensor ws = scratch(topk_ids, ws_bytes);
  status("moe_sort", aops_moe_sort_i32(static_cast<const int32_t*>(dev_ptr(topk_ids)), n, num_experts,
                                       static_cast<int32_t*>(dev_ptr(sorted_idx)),
                                       static_cast<int32_t*>(dev_ptr(inverse_idx)),
                                       static_cast<int64_t*>(dev_ptr(group_list)), ws.data_ptr(), ws_bytes, l.stream));
  return {sorted_idx, inverse_idx, group_list};
}

// out[t] = sum_k topk_weights[t, k] * y[inverse_idx[t*topk + k]] over the valid expert ids
Tensor moe_combine(const Tensor& y, const Tensor& inverse_idx, const Tensor& topk_weights, const Tensor& topk_ids,
                   int64_t num_experts) {
  TORCH_CHECK(y.dim() == 2 && y.is_contiguous() && topk_weights.dim() == 2 && topk_weights.is_contiguous() &&
                  topk_ids.sizes() == topk_weights.sizes() && topk_ids.is_contiguous() && inverse_idx.is_contiguous(),
              "moe_combine: y must be 2D, topk_weights and topk_ids [tokens, topk], all contiguous");
  const int64_t tokens = topk_weights.size(0), topk = topk_weights.size(1);
  TORCH_CHECK(y.size(0) == tokens * topk && inverse_idx.numel() == tokens * topk,
              "moe_combine: y and inverse_idx must have tokens*topk rows, got ", y.size(0), " and ",
              inverse_idx.numel());
  TORCH_CHECK(y.size(1) % 8 == 0, "moe_combine: hidden must be a multiple of 8, got ", y.size(1));
  require_device("moe_combine", {{"y", y, at::kHalf},
                                 {"inverse_idx", inverse_idx, at::kInt},
                                 {"topk_weights", topk_weights, at::kFloat},
                                 {"topk_ids", topk_ids, at::kInt}});
  Tensor out = fresh(y, {tokens, y.size(1)}, y.scalar_type());
  Launch l(y);
  status("moe_combine",
         aops_moe_combine_f16(dev_ptr(y), static_cast<const int32_t*>(dev_ptr(inverse_idx)),
                              static_cast<const float*>(dev_ptr(topk_weights)),
                              static_cast<const int32_t*>(dev_ptr(topk_ids)), dev_ptr(out), tokens, topk, y.size(1),
                              num_experts, l.stream));
  return out;
}

// The address the kernels would be given for t (0 for an empty tensor); raises for misaligned fp16 data.
uintptr_t tensor_address(const Tensor& t) { return reinterpret_cast<uintptr_t>(dev_ptr(t)); }

void def_reference_ops(py::module_& m) {
  m.def("rope", &rope, py::arg("q"), py::arg("k"), py::arg("position_ids"), py::arg("cos_cache"),
        py::arg("sin_cache"));
  m.def("swiglu", &swiglu, py::arg("x"));
  m.def("grouped_matmul", &grouped_matmul, py::arg("x"), py::arg("w"), py::arg("group_list"));
  m.def("add_rms_norm", &add_rms_norm, py::arg("x"), py::arg("residual"), py::arg("weight"), py::arg("epsilon"));
  m.def("reshape_and_cache", &reshape_and_cache, py::arg("key"), py::arg("value"), py::arg("key_cache"),
        py::arg("value_cache"), py::arg("slot_indices"));
  m.def("paged_attention", &paged_attention, py::arg("q"), py::arg("key_cache"), py::arg("value_cache"),
        py::arg("block_tables"), py::arg("context_lens"));
}

}  // namespace

PYBIND11_MODULE(ascend910a_extras_C, m) {
  m.doc() = "ascend910a_extras operators on MI355X: torch tensors in, one libaops C-ABI call each";
  m.def("print_info", &print_info, py::arg("device_id"));  // reference csrc/ffi/bind.cpp:56-57
  py::module_ ops = m.def_submodule("ops");                // reference csrc/ffi/ops.cpp:484-491
  def_reference_ops(ops);
  def_reference_ops(m);
  m.def("matmul", &matmul, py::arg("x"), py::arg("w"));
  m.def("grouped_matmul_swiglu", &grouped_matmul_swiglu, py::arg("x"), py::arg("w"), py::arg("group_list"));
  m.def("grouped_matmul_swiglu_gather", &grouped_matmul_swiglu_gather, py::arg("x"), py::arg("sorted_idx"),
        py::arg("topk"), py::arg("w"), py::arg("group_list"));
  m.def("rope_reshape_and_cache", &rope_reshape_and_cache, py::arg("q"), py::arg("k"), py::arg("v"),
        py::arg("position_ids"), py::arg("cos_cache"), py::arg("sin_cache"), py::arg("key_cache"),
        py::arg("value_cache"), py::arg("slot_indices"), py::arg("return_k") = false,
        py::arg("q_norm_weight") = py::none(), py::arg("k_norm_weight") = py::none(), py::arg("epsilon") = 1e-6);
  m.def("moe_sort", &moe_sort, py::arg("topk_ids"), py::arg("num_experts"));
  m.def("moe_gather", &moe_gather, py::arg("x"), py::arg("sorted_idx"), py::arg("group_list"), py::arg("topk"));
  m.def("moe_combine", &moe_combine, py::arg("y"), py::arg("inverse_idx"), py::arg("topk_weights"),
        py::arg("topk_ids"), py::arg("num_experts"));
  m.def("tensor_address", &tensor_address, py::arg("t"));
  m.def("library_version", []() { return aops_version(); });
}
