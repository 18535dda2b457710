#include "gpu.h"

#include <dlfcn.h>

#include <algorithm>
#include <sstream>

namespace vosti {

void hip_check(hipError_t e, const char* what) {
  if (e != hipSuccess) throw EngineError(std::string(what) + ": " + hipGetErrorString(e));
}

const char* dtype_name(DType t) { return t == DType::BF16 ? "bfloat16" : (t == DType::F32 ? "float32" : "int32"); }

DeviceBuffer::DeviceBuffer(size_t bytes) : bytes_(bytes) {
  hip_check(hipMalloc(&ptr_, bytes ? bytes : 16), "device allocation");
}
DeviceBuffer::~DeviceBuffer() {
  if (ptr_) (void)hipFree(ptr_);
}

Tensor Tensor::view(std::vector<int64_t> new_shape) const {
  Tensor t = *this;
  t.shape = std::move(new_shape);
  if (t.numel() != numel()) throw EngineError("view of " + describe() + " with another number of elements");
  return t;
}

Tensor Tensor::rows(int64_t first, int64_t count) const {
  if (shape.empty() || first < 0 || count < 0 || first + count > shape[0]) throw EngineError("rows outside " + describe());
  Tensor t = *this;
  const int64_t row = shape[0] ? numel() / shape[0] : 0;
  t.data = static_cast<char*>(data) + (size_t)(first * row) * dtype_bytes(dtype);
  t.shape[0] = count;
  return t;
}

std::string Tensor::describe() const {
  std::ostringstream s;
  s << dtype_name(dtype) << "[";
  for (size_t i = 0; i < shape.size(); ++i) s << (i ? ", " : "") << shape[i];
  s << "]";
  return s.str();
}

// ------------------------------------------------------------------------------------------ arena
void* Arena::take(size_t bytes) {
  bytes = (bytes + 255) & ~(size_t)255;
  if (bytes == 0) bytes = 256;
  while (block_ < blocks_.size()) {
    if (offset_ + bytes <= blocks_[block_]->bytes()) {
      void* p = static_cast<char*>(blocks_[block_]->data()) + offset_;
      offset_ += bytes;
      return p;
    }
    ++block_;
    offset_ = 0;
  }
  if (frozen_) throw EngineError("a step that is being recorded asks for more activation memory than the step before it");
  const size_t min_block = (size_t)64 << 20;
  blocks_.push_back(std::make_unique<DeviceBuffer>(bytes > min_block ? bytes : min_block));
  offset_ = bytes;
  return blocks_.back()->data();
}

size_t Arena::capacity() const {
  size_t n = 0;
  for (const auto& b : blocks_) n += b->bytes();
  return n;
}

// ---------------------------------------------------------------------------------------- kernels
using P = void*;
using CP = const void*;
struct Kernels::Fn {
  const char* (*last_error)();
  int (*abi_version)();
  int (*elem_bytes)();
  int (*embedding)(P, CP, CP, int, int, int, hipStream_t);
  int (*rmsnorm)(P, CP, CP, int, int, int, int, int64_t, int64_t, float, hipStream_t);
  int (*add_rmsnorm)(P, P, CP, CP, int, int, int, float, hipStream_t);
  int (*swiglu)(P, CP, int, int, hipStream_t);
  int (*gather_rows)(P, CP, CP, int, int, hipStream_t);
  int (*cast_to_f32)(P, CP, int64_t, hipStream_t);
  int (*rope_tables)(P, P, CP, int, int, hipStream_t);
  int (*fill_random)(P, int64_t, uint64_t, int, float, float, hipStream_t);
  int (*gemm)(P, CP, CP, int, int, int, int64_t, int64_t, int, hipStream_t);
  int (*gemm_swiglu)(P, CP, CP, int, int, int, int64_t, int64_t, hipStream_t);
  int (*gemm_swiglu_supported)(int, int, int);
  int (*gemm_split)(P, CP, CP, int, int, int, int64_t, int64_t, int, P, int64_t, hipStream_t);
  int64_t (*gemm_split_floats)(int, int, int, int);
  int (*gemm_split_preferred)(int, int, int, int);
  int (*qkv_post)(CP, int64_t, P, P, P, CP, CP, int, CP, CP, int, CP, CP, int, int, int, int, int, float, hipStream_t);
  int (*paged_attention)(P, CP, CP, CP, CP, int, CP, CP, CP, int, int, int, P, int, int, int, int, int, int, float, hipStream_t);
  int (*sample)(P, CP, CP, CP, P, int, int, int64_t, hipStream_t);
  int (*sample_scratch_words)(int);
  int64_t (*attn_scratch_floats)(int, int, int, int);
  int (*attn_segment_keys)();
  int (*attn_item_rows)();
  int (*embed_sinusoid)(P, CP, CP, CP, CP, int, int, int, hipStream_t);
  int (*stream_norm)(P, CP, int, CP, int, int, int, float, float, hipStream_t);
  int (*stream_norm_add)(P, CP, CP, CP, int, int, int, float, float, float, hipStream_t);
  int (*stream_mix)(P, CP, int64_t, CP, int, int, int64_t, hipStream_t);
  int (*gather_rows_f32)(P, CP, CP, int, int, hipStream_t);
  int (*softcap)(P, float, int64_t, hipStream_t);
  int (*qkv_post_bias)(CP, int64_t, P, P, P, CP, CP, int, CP, CP, int, CP, CP, int, int, int, int, int, float, CP, hipStream_t);
  int (*paged_attention_capped)(P, CP, CP, CP, CP, int, CP, CP, CP, int, int, int, P, int, int, int, int, int, int, int, float, float, CP, int,
                                hipStream_t);
  int (*delta_conv)(P, CP, int64_t, CP, P, int64_t, int64_t, CP, CP, CP, CP, int, int, int, int, hipStream_t);
  int (*delta_unit)(P, int64_t, int, int, int, int, float, float, hipStream_t);
  int (*delta_decay)(P, CP, CP, CP, int, int, int, int, hipStream_t);
  int (*delta_prep)(P, int64_t, int, int, int, int, int, int, float, float, P, CP, CP, CP, int, hipStream_t);
  int (*delta_rule)(P, CP, int64_t, int, int, int, CP, CP, int64_t, P, int64_t, CP, CP, CP, int, int, int, int, int, hipStream_t);
  int (*delta_out)(P, int64_t, CP, CP, int64_t, CP, int, int, int, int, float, hipStream_t);
  int (*delta_conv_bias)(P, CP, int64_t, CP, CP, P, int64_t, int64_t, CP, CP, CP, CP, int, int, int, int, hipStream_t);
  int (*paged_attention_blocked)(P, CP, CP, CP, CP, int, CP, CP, CP, int, int, int, P, int, int, int, int, int, int, float, float, CP, int,
                                 hipStream_t);
  int (*qkv_post_angles)(CP, int64_t, P, P, P, CP, float, int, CP, CP, int, int, int, int, int, hipStream_t);
  int (*embed_scaled)(P, CP, CP, int, int, int, float, hipStream_t);
  int (*stream_add)(P, CP, CP, int, CP, int, int64_t, hipStream_t);
  int (*stream_pair_norm)(P, CP, CP, CP, CP, int, int, int, float, float, float, hipStream_t);
  int (*ssm_scan)(P, CP, int64_t, int, int, CP, int64_t, CP, CP, CP, int, P, int64_t, CP, CP, CP, int, int, int, int, int, int, hipStream_t);
  int (*ssm_gate_norm)(P, int64_t, CP, CP, int64_t, CP, int, int, int, int, float, hipStream_t);
  int (*moe_max_tiles)(int, int, int, int);
  int (*gemm_grouped)(P, CP, CP, int, int, int, int64_t, int64_t, CP, int64_t, hipStream_t);
  int (*moe_route)(P, P, P, CP, CP, int, int, int, int, float, hipStream_t);
  int (*moe_plan)(CP, P, P, P, P, P, int, int, int, int, hipStream_t);
  int (*moe_up)(P, int64_t, CP, int64_t, CP, CP, CP, CP, int, int, int, int, int, hipStream_t);
  int (*moe_down)(P, CP, int64_t, CP, CP, CP, int, int, int, int, int, hipStream_t);
  int (*moe_combine)(P, CP, CP, CP, int, int, int, hipStream_t);
  int (*moe_relu_square)(P, int64_t, hipStream_t);
  int (*qkv_post_norm_angles)(CP, int64_t, P, P, P, CP, CP, int, int, float, CP, float, int, CP, CP, int, int, int, int, int, hipStream_t);
  int (*gate_mul)(P, int64_t, CP, int64_t, int, int, int, hipStream_t);
  int (*gla_decay)(P, CP, int64_t, CP, int, int, int, float, hipStream_t);
  int (*gla_rule)(P, CP, int64_t, int, int, int, CP, P, int64_t, CP, CP, CP, int, int, int, int, float, hipStream_t);
  int (*gated_head_norm)(P, int64_t, CP, CP, int64_t, CP, int, int, int, int, float, int, hipStream_t);
  int (*moe_route_bias)(P, P, P, CP, CP, CP, int, int, int, int, int, float, hipStream_t);
  int (*moe_up_plain)(P, int64_t, CP, int64_t, CP, CP, CP, CP, int, int, int, int, int, hipStream_t);
  int (*moe_glu)(P, CP, int64_t, int, float, float, float, hipStream_t);
  int (*moe_combine_add)(P, CP, CP, CP, CP, int, int, int, hipStream_t);
  int (*stream_norm_add_f32)(P, CP, CP, CP, int, int, int, float, float, float, hipStream_t);
  int (*cast_from_f32)(P, CP, int64_t, hipStream_t);
  int (*stream_norm_add_rounded)(P, CP, CP, CP, int, int, int, float, float, float, P, hipStream_t);
  int (*stream_norm_add_f32_rounded)(P, CP, CP, CP, int, int, int, float, float, float, P, hipStream_t);
  int (*moe_route_scored)(P, P, P, CP, CP, CP, int, int, int, int, int, float, int, hipStream_t);
  int (*moe_glu_weighed)(P, CP, int64_t, int, float, float, float, CP, CP, hipStream_t);
  int (*norm_columns)(P, int64_t, CP, int64_t, int, int, CP, int, float, int, hipStream_t);
  int (*gemm_heads)(P, int64_t, int64_t, CP, int64_t, int64_t, CP, int, int, int, int, hipStream_t);
  int (*latent_post)(CP, int64_t, CP, int64_t, int64_t, int, P, P, P, CP, int, float, CP, int, CP, CP, int, int, int, int, int, int, hipStream_t);
  int (*qkv_post_norm_angles_paired)(CP, int64_t, P, P, P, CP, CP, int, int, float, CP, float, int, int, CP, CP, int, int, int, int, int, hipStream_t);
  int (*linear_rule)(P, CP, int64_t, int, int, int, CP, P, int64_t, CP, CP, CP, int, int, int, int, float, hipStream_t);
  int (*side_gate)(P, int64_t, CP, int64_t, CP, int64_t, CP, int, int, int, hipStream_t);
  int (*gated_row_norm)(P, int64_t, CP, CP, int64_t, CP, int, int, int, float, int, hipStream_t);
  int (*silu_columns)(P, int64_t, int64_t, int, int, hipStream_t);
};

static constexpr int KERNEL_ABI = 18;

Kernels::Kernels(const std::string& lib_dir, const std::string& name) : name_(name), fn_(new Fn) {
  if (name == "bf16") dtype_ = DType::BF16;
  else if (name == "f32") dtype_ = DType::F32;
  else throw EngineError("unsupported element type '" + name + "'; use bf16 or f32");
  const std::string path = lib_dir + "/libvosti_" + name + ".so";
  handle_ = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
  if (!handle_) throw EngineError("the kernel library is missing: " + std::string(dlerror()) + " (build it: python -m vosti_amd.kernels.build)");
  auto sym = [&](const char* s) {
    void* p = dlsym(handle_, s);
    if (!p) throw EngineError(path + " lacks " + s + "; rebuild it");
    return p;
  };
#define VK(field, symbol) fn_->field = reinterpret_cast<decltype(fn_->field)>(sym(symbol))
  VK(last_error, "vk_last_error"); VK(abi_version, "vk_abi_version"); VK(elem_bytes, "vk_elem_bytes");
  if (fn_->abi_version() != KERNEL_ABI)
    throw EngineError(path + " has ABI " + std::to_string(fn_->abi_version()) + ", expected " + std::to_string(KERNEL_ABI) + "; rebuild it");
  if (fn_->elem_bytes() != dtype_bytes(dtype_)) throw EngineError(path + " was built for another element type");
  VK(embedding, "vk_embedding"); VK(rmsnorm, "vk_rmsnorm"); VK(add_rmsnorm, "vk_add_rmsnorm"); VK(swiglu, "vk_swiglu");
  VK(gather_rows, "vk_gather_rows"); VK(cast_to_f32, "vk_cast_to_f32"); VK(rope_tables, "vk_rope_tables"); VK(fill_random, "vk_fill_random");
  VK(gemm, "vk_gemm"); VK(gemm_swiglu, "vk_gemm_swiglu"); VK(gemm_swiglu_supported, "vk_gemm_swiglu_supported");
  VK(gemm_split, "vk_gemm_split"); VK(gemm_split_floats, "vk_gemm_split_floats"); VK(gemm_split_preferred, "vk_gemm_split_preferred");
  VK(qkv_post, "vk_qkv_post"); VK(paged_attention, "vk_paged_attention"); VK(sample, "vk_sample");
  VK(sample_scratch_words, "vk_sample_scratch_words"); VK(attn_scratch_floats, "vk_attn_scratch_floats");
  VK(attn_segment_keys, "vk_attn_segment_keys"); VK(attn_item_rows, "vk_attn_item_rows");
  VK(embed_sinusoid, "vk_embed_sinusoid"); VK(stream_norm, "vk_stream_norm"); VK(stream_norm_add, "vk_stream_norm_add");
  VK(stream_mix, "vk_stream_mix"); VK(gather_rows_f32, "vk_gather_rows_f32"); VK(softcap, "vk_softcap");
  VK(qkv_post_bias, "vk_qkv_post_bias"); VK(paged_attention_capped, "vk_paged_attention_capped");
  VK(delta_conv, "vk_delta_conv"); VK(delta_prep, "vk_delta_prep"); VK(delta_unit, "vk_delta_unit"); VK(delta_decay, "vk_delta_decay"); VK(delta_rule, "vk_delta_rule");
  VK(delta_out, "vk_delta_out"); VK(delta_conv_bias, "vk_delta_conv_bias"); VK(paged_attention_blocked, "vk_paged_attention_blocked");
  VK(qkv_post_angles, "vk_qkv_post_angles"); VK(embed_scaled, "vk_embed_scaled"); VK(stream_add, "vk_stream_add");
  VK(stream_pair_norm, "vk_stream_pair_norm"); VK(ssm_scan, "vk_ssm_scan"); VK(ssm_gate_norm, "vk_ssm_gate_norm");
  VK(moe_max_tiles, "vk_moe_max_tiles"); VK(moe_route, "vk_moe_route"); VK(moe_plan, "vk_moe_plan"); VK(moe_up, "vk_moe_up");
  VK(moe_down, "vk_moe_down"); VK(moe_combine, "vk_moe_combine"); VK(moe_relu_square, "vk_moe_relu_square"); VK(gemm_grouped, "vk_gemm_grouped");
  VK(qkv_post_norm_angles, "vk_qkv_post_norm_angles"); VK(gate_mul, "vk_gate_mul"); VK(gla_decay, "vk_gla_decay"); VK(gla_rule, "vk_gla_rule");
  VK(gated_head_norm, "vk_gated_head_norm"); VK(moe_route_bias, "vk_moe_route_bias"); VK(moe_up_plain, "vk_moe_up_plain"); VK(moe_glu, "vk_moe_glu");
  VK(moe_combine_add, "vk_moe_combine_add"); VK(stream_norm_add_f32, "vk_stream_norm_add_f32");
  VK(stream_norm_add_rounded, "vk_stream_norm_add_rounded"); VK(stream_norm_add_f32_rounded, "vk_stream_norm_add_f32_rounded");
  VK(cast_from_f32, "vk_cast_from_f32"); VK(moe_route_scored, "vk_moe_route_scored"); VK(moe_glu_weighed, "vk_moe_glu_weighed");
  VK(norm_columns, "vk_norm_columns"); VK(gemm_heads, "vk_gemm_heads"); VK(latent_post, "vk_latent_post");
  VK(qkv_post_norm_angles_paired, "vk_qkv_post_norm_angles_paired"); VK(linear_rule, "vk_linear_rule"); VK(side_gate, "vk_side_gate");
  VK(gated_row_norm, "vk_gated_row_norm"); VK(silu_columns, "vk_silu_columns");
#undef VK
  segment_keys_ = fn_->attn_segment_keys();
  item_rows_ = fn_->attn_item_rows();
  hip_check(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking), "stream creation");
}

Kernels::~Kernels() {
  if (stream) (void)hipStreamDestroy(stream);
  // The library stays loaded: its code objects are registered with the runtime.
}

void Kernels::call(int rc) const {
  if (rc != 0) throw EngineError(fn_->last_error());
}

void Kernels::expect(const Tensor& t, const char* what, DType dtype, std::vector<int64_t> shape) const {
  if (t.data == nullptr && t.numel() != 0) throw EngineError(std::string(what) + " has no memory");
  if (t.dtype != dtype) throw EngineError(std::string(what) + " has type " + dtype_name(t.dtype) + ", expected " + dtype_name(dtype));
  if (!shape.empty() && t.shape != shape) {
    Tensor want;
    want.dtype = dtype;
    want.shape = shape;
    throw EngineError(std::string(what) + " is " + t.describe() + ", expected " + want.describe());
  }
}

int Kernels::norm_weight(const Tensor& w, const char* what, int64_t n) const {
  // A norm weight may be stored as elements or as float.
  if (w.dtype == DType::F32) {
    expect(w, what, DType::F32, {n});
    return 1;
  }
  expect(w, what, dtype_, {n});
  return 0;
}

Tensor Kernels::empty(std::vector<int64_t> shape, DType t) {
  Tensor out;
  out.dtype = t;
  out.shape = std::move(shape);
  for (int64_t s : out.shape)
    if (s < 0) throw EngineError("a tensor with a negative size");
  out.data = arena.take(out.bytes());
  return out;
}

Tensor Kernels::embedding(const Tensor& table, const Tensor& ids) {
  expect(table, "embedding table", dtype_);
  if (table.shape.size() != 2) throw EngineError("embedding table is " + table.describe());
  const int64_t V = table.dim(0), H = table.dim(1), T = ids.numel();
  expect(ids, "ids", DType::I32, {T});
  Tensor out = empty({T, H});
  call(fn_->embedding(out.data, table.data, ids.data, (int)T, (int)H, (int)V, stream));
  return out;
}

Tensor Kernels::rmsnorm(const Tensor& x, const Tensor& w, float eps) {
  expect(x, "norm input", dtype_);
  const int64_t H = x.dim(-1), rows = H ? x.numel() / H : 0;
  const int wf = norm_weight(w, "norm weight", H);
  Tensor out = empty(x.shape);
  call(fn_->rmsnorm(out.data, x.data, w.data, wf, (int)rows, (int)H, 1, H, H, eps, stream));
  return out;
}

Tensor Kernels::add_rmsnorm(const Tensor& x, Tensor& residual, const Tensor& w, float eps) {
  expect(x, "norm input", dtype_);
  if (x.shape.size() != 2) throw EngineError("norm input is " + x.describe());
  expect(residual, "residual", dtype_, x.shape);
  const int wf = norm_weight(w, "norm weight", x.dim(1));
  Tensor out = empty(x.shape);
  call(fn_->add_rmsnorm(out.data, residual.data, x.data, w.data, wf, (int)x.dim(0), (int)x.dim(1), eps, stream));
  return out;
}

Tensor Kernels::swiglu(const Tensor& gate_up) {
  expect(gate_up, "gate/up tensor", dtype_);
  if (gate_up.shape.size() != 2 || gate_up.dim(1) % 2) throw EngineError("swiglu: gate/up tensor is " + gate_up.describe());
  const int64_t T = gate_up.dim(0), I = gate_up.dim(1) / 2;
  Tensor out = empty({T, I});
  call(fn_->swiglu(out.data, gate_up.data, (int)T, (int)I, stream));
  return out;
}

Tensor Kernels::gather_rows(const Tensor& x, const Tensor& rows) {
  if (x.dtype != DType::F32) expect(x, "rows' source", dtype_);
  if (x.shape.size() != 2) throw EngineError("gather_rows: source is " + x.describe());
  const int64_t R = rows.numel();
  expect(rows, "row numbers", DType::I32, {R});
  Tensor out = empty({R, x.dim(1)}, x.dtype);
  if (x.dtype == DType::F32 && dtype_ != DType::F32) call(fn_->gather_rows_f32(out.data, x.data, rows.data, (int)R, (int)x.dim(1), stream));
  else call(fn_->gather_rows(out.data, x.data, rows.data, (int)R, (int)x.dim(1), stream));
  return out;
}

Tensor Kernels::to_f32(const Tensor& x) {
  expect(x, "cast input", dtype_);
  Tensor out = empty(x.shape, DType::F32);
  call(fn_->cast_to_f32(out.data, x.data, x.numel(), stream));
  return out;
}

Tensor Kernels::to_elements(const Tensor& x) {
  expect(x, "cast input", DType::F32);
  if (dtype_ == DType::F32) return x;
  Tensor out = empty(x.shape);
  call(fn_->cast_from_f32(out.data, x.data, x.numel(), stream));
  return out;
}

void Kernels::copy_columns(Tensor& dst, int64_t dst_first, const Tensor& src, int64_t src_first, int64_t count) {
  if (src.shape.size() != 2 || dst.shape.size() != 2 || src.dim(0) != dst.dim(0) || src.dtype != dst.dtype || count < 0 || src_first < 0 ||
      dst_first < 0 || src_first + count > src.dim(1) || dst_first + count > dst.dim(1))
    throw EngineError("copy_columns: " + std::to_string(count) + " columns from " + std::to_string(src_first) + " of " + src.describe() +
                      " to " + std::to_string(dst_first) + " of " + dst.describe());
  if (count == 0 || src.dim(0) == 0) return;
  const size_t e = (size_t)dtype_bytes(src.dtype);
  hip_check(hipMemcpy2DAsync(static_cast<char*>(dst.data) + (size_t)dst_first * e, (size_t)dst.dim(1) * e,
                             static_cast<const char*>(src.data) + (size_t)src_first * e, (size_t)src.dim(1) * e, (size_t)count * e,
                             (size_t)src.dim(0), hipMemcpyDeviceToDevice, stream),
            "copying columns");
}

Tensor Kernels::columns(const Tensor& x, int64_t first, int64_t count) {
  if (x.shape.size() != 2) throw EngineError("columns of " + x.describe());
  Tensor out = empty({x.dim(0), count}, x.dtype);
  copy_columns(out, 0, x, first, count);
  return out;
}

void Kernels::rope_tables(Tensor& cos, Tensor& sin, const Tensor& inv_freq) {
  const int64_t half = inv_freq.numel();
  expect(inv_freq, "inverse frequencies", DType::F32, {half});
  expect(cos, "cosine table", dtype_);
  if (cos.shape.size() != 2 || cos.dim(1) != half) throw EngineError("cosine table is " + cos.describe());
  expect(sin, "sine table", dtype_, cos.shape);
  call(fn_->rope_tables(cos.data, sin.data, inv_freq.data, (int)cos.dim(0), (int)half, stream));
}

int64_t Kernels::gemm_workspace_floats(int64_t M, int64_t rows, int64_t K, bool swiglu) const {
  if (!fn_->gemm_split_preferred((int)M, (int)rows, (int)K, swiglu ? 1 : 0)) return 0;
  return fn_->gemm_split_floats((int)M, (int)rows, (int)K, swiglu ? 1 : 0);
}

// Runs the product through chunk sums in the workspace if that is the faster route and it fits.
bool Kernels::split(Tensor& out, const Tensor& act, const Tensor& w, bool swiglu, const Tensor* workspace) {
  if (!workspace) return false;
  const int64_t M = act.dim(0), K = act.dim(1), rows = w.dim(0);
  const int64_t need = gemm_workspace_floats(M, rows, K, swiglu);
  if (need == 0 || workspace->dtype != DType::F32 || workspace->numel() < need) return false;
  call(fn_->gemm_split(out.data, act.data, w.data, (int)M, (int)rows, (int)K, K, out.dim(1), swiglu ? 1 : 0, workspace->data,
                       workspace->numel(), stream));
  return true;
}

void Kernels::fill_random(Tensor& out, uint64_t seed, int kind, float p0, float p1) {
  expect(out, "tensor to fill", dtype_);
  call(fn_->fill_random(out.data, out.numel(), seed, kind, p0, p1, stream));
}

Tensor Kernels::gemm(const Tensor& act, const Tensor& w, const Tensor* workspace) {
  expect(act, "activation", dtype_);
  expect(w, "weight", dtype_);
  if (act.shape.size() != 2 || w.shape.size() != 2 || act.dim(1) != w.dim(1))
    throw EngineError("gemm: activation " + act.describe() + " does not fit weight " + w.describe());
  const int64_t M = act.dim(0), K = act.dim(1), N = w.dim(0);
  Tensor out = empty({M, N});
  if (split(out, act, w, false, workspace)) return out;
  call(fn_->gemm(out.data, act.data, w.data, (int)M, (int)N, (int)K, K, N, 0, stream));
  return out;
}

Tensor Kernels::gemm_swiglu(const Tensor& act, const Tensor& w, const Tensor* workspace) {
  expect(act, "activation", dtype_);
  expect(w, "gate/up weight", dtype_);
  if (act.shape.size() != 2 || w.shape.size() != 2 || act.dim(1) != w.dim(1) || w.dim(0) % 2)
    throw EngineError("gemm_swiglu: activation " + act.describe() + " does not fit a gate/up weight " + w.describe());
  const int64_t M = act.dim(0), K = act.dim(1), I = w.dim(0) / 2;
  // One launch where the sizes allow it, else projection and activation one after the other: the same bits.
  if (!fn_->gemm_swiglu_supported((int)M, (int)I, (int)K)) return swiglu(gemm(act, w, workspace));
  Tensor out = empty({M, I});
  if (split(out, act, w, true, workspace)) return out;
  call(fn_->gemm_swiglu(out.data, act.data, w.data, (int)M, (int)I, (int)K, K, I, stream));
  return out;
}

Tensor Kernels::qkv_post(const Tensor& qkv, int nq, int nkv, int d, const Tensor* k_cache, const Tensor* v_cache,
                         int page_size, const Tensor* q_w, const Tensor* k_w, float eps, const Tensor* cos,
                         const Tensor* sin, const Tensor* positions, const Tensor* slots) {
  expect(qkv, "qkv", dtype_);
  const int64_t W = (int64_t)(nq + 2 * nkv) * d;
  if (qkv.shape.size() != 2 || qkv.dim(1) != W) throw EngineError("qkv_post: rows are " + qkv.describe() + ", expected width " + std::to_string(W));
  const int64_t T = qkv.dim(0);
  Tensor q_out;
  if (nq) q_out = empty({T, nq, d});
  int wf = 0;
  if (q_w) wf = norm_weight(*q_w, "q norm weight", d);
  if (k_w) {
    const int wf2 = norm_weight(*k_w, "k norm weight", d);
    if (q_w && wf2 != wf) throw EngineError("qkv_post: q and k norm weights must have the same type");
    wf = wf2;
  }
  int rot_half = 0;
  if (cos) {
    if (!sin || !positions) throw EngineError("qkv_post: a rotation needs cosines, sines and positions");
    expect(*cos, "cosine table", dtype_);
    if (cos->shape.size() != 2 || 2 * cos->dim(1) > d) throw EngineError("qkv_post: cosine table is " + cos->describe());
    expect(*sin, "sine table", dtype_, cos->shape);
    expect(*positions, "positions", DType::I32, {T});
    rot_half = (int)cos->dim(1);
  }
  if (nkv) {
    if (!k_cache || !v_cache || !slots) throw EngineError("qkv_post: a store needs both caches and slots");
    expect(*k_cache, "k cache", dtype_);
    if (k_cache->shape.size() != 4) throw EngineError("k cache is " + k_cache->describe());
    const int64_t pages = k_cache->dim(0);
    expect(*k_cache, "k cache", dtype_, {pages, nkv, page_size, d});
    expect(*v_cache, "v cache", dtype_, {pages, nkv, d, page_size});
    expect(*slots, "slots", DType::I32, {T});
  }
  call(fn_->qkv_post(qkv.data, W, nq ? q_out.data : nullptr, nkv ? k_cache->data : nullptr, nkv ? v_cache->data : nullptr,
                     q_w ? q_w->data : nullptr, k_w ? k_w->data : nullptr, wf, cos ? cos->data : nullptr,
                     cos ? sin->data : nullptr, rot_half, positions ? positions->data : nullptr,
                     slots ? slots->data : nullptr, (int)T, nq, nkv, d, page_size, eps, stream));
  return q_out;
}

int64_t Kernels::attn_scratch_floats(int items, int nq, int d, int nseg) const {
  return fn_->attn_scratch_floats(items, nq, d, nseg);
}

void Kernels::paged_attention(Tensor& out, const Tensor& q, const Tensor& k_cache, const Tensor& v_cache,
                              const Tensor& block_table, const Tensor& cu_q, const Tensor& k_len, const Tensor& items,
                              int mode, float scale, int window, int max_k_len, int nseg, const Tensor* scratch) {
  expect(q, "q", dtype_);
  expect(k_cache, "k cache", dtype_);
  expect(block_table, "block table", DType::I32);
  if (q.shape.size() != 3 || k_cache.shape.size() != 4 || block_table.shape.size() != 2)
    throw EngineError("attention: q " + q.describe() + ", k cache " + k_cache.describe() + ", block table " + block_table.describe());
  const int64_t T = q.dim(0), nq = q.dim(1), d = q.dim(2), pages = k_cache.dim(0), nkv = k_cache.dim(1), P = k_cache.dim(2);
  const int64_t S = block_table.dim(0), W = block_table.dim(1);
  expect(k_cache, "k cache", dtype_, {pages, nkv, P, d});
  expect(v_cache, "v cache", dtype_, {pages, nkv, d, P});
  expect(cu_q, "cu_q", DType::I32, {S + 1});
  expect(k_len, "k_len", DType::I32, {S});
  expect(out, "attention output", dtype_, q.shape);
  if (items.shape.size() != 2 || items.dim(1) != 2) throw EngineError("attention: items are " + items.describe());
  expect(items, "items", DType::I32);
  const int64_t n_items = items.dim(0);
  if (W * P < max_k_len)
    throw EngineError("attention: a block table of " + std::to_string(W) + " pages of " + std::to_string(P) + " does not cover " +
                      std::to_string(max_k_len) + " keys");
  void* sp = nullptr;
  if (mode == 1 || (mode >= 3 && mode <= 5) || mode == 7) {
    if (nseg < (max_k_len + segment_keys_ - 1) / segment_keys_)
      throw EngineError("attention: " + std::to_string(nseg) + " segments do not cover " + std::to_string(max_k_len) + " keys");
    const int64_t need = attn_scratch_floats((int)n_items, (int)nq, (int)d, nseg);
    if (!scratch || scratch->dtype != DType::F32 || scratch->numel() < need)
      throw EngineError("attention: scratch of " + std::to_string(need) + " floats needed");
    sp = scratch->data;
  }
  call(fn_->paged_attention(out.data, q.data, k_cache.data, v_cache.data, block_table.data, (int)W, cu_q.data, k_len.data,
                            items.data, (int)n_items, mode, nseg, sp, (int)T, (int)nq, (int)nkv, (int)d, (int)P, window, scale,
                            stream));
}

// ------------------------------------------------------------------------- the 32-bit residual stream
Tensor Kernels::embed_sinusoid(const Tensor& table, const Tensor& ids, const Tensor& positions, const Tensor& inv_freq) {
  expect(table, "embedding table", dtype_);
  if (table.shape.size() != 2) throw EngineError("embedding table is " + table.describe());
  const int64_t V = table.dim(0), H = table.dim(1), T = ids.numel();
  expect(ids, "ids", DType::I32, {T});
  expect(positions, "positions", DType::I32, {T});
  expect(inv_freq, "inverse frequencies", DType::F32, {H / 2});
  Tensor out = empty({T, H}, DType::F32);
  call(fn_->embed_sinusoid(out.data, table.data, ids.data, positions.data, inv_freq.data, (int)T, (int)H, (int)V, stream));
  return out;
}

Tensor Kernels::stream_norm(const Tensor& x, const Tensor& w, float eps, float offset) {
  if (x.dtype != DType::F32) expect(x, "norm input", dtype_);
  if (x.shape.empty()) throw EngineError("norm input is " + x.describe());
  const int64_t H = x.dim(-1), rows = H ? x.numel() / H : 0;
  const int wf = norm_weight(w, "norm weight", H);
  Tensor out = empty(x.shape);
  call(fn_->stream_norm(out.data, x.data, x.dtype == DType::F32 ? 1 : 0, w.data, wf, (int)rows, (int)H, eps, offset, stream));
  return out;
}

void Kernels::stream_norm_add(Tensor& out, const Tensor& base, const Tensor& y, const Tensor& w, float eps, float offset, float mult, Tensor* rounded) {
  if (y.dtype != DType::F32) expect(y, "norm input", dtype_);
  if (y.shape.size() != 2) throw EngineError("norm input is " + y.describe());
  expect(base, "stream", DType::F32, y.shape);
  expect(out, "stream", DType::F32, y.shape);
  const int wf = norm_weight(w, "norm weight", y.dim(1));
  if (rounded) {
    expect(*rounded, "the stream's rounded rows", dtype_, y.shape);
    auto fn = (y.dtype == DType::F32 && dtype_ != DType::F32) ? fn_->stream_norm_add_f32_rounded : fn_->stream_norm_add_rounded;
    call(fn(out.data, base.data, y.data, w.data, wf, (int)y.dim(0), (int)y.dim(1), eps, offset, mult, rounded->data, stream));
    return;
  }
  // A sublayer's rows may be elements or, where it left them unrounded, floats.
  if (y.dtype == DType::F32 && dtype_ != DType::F32) {
    call(fn_->stream_norm_add_f32(out.data, base.data, y.data, w.data, wf, (int)y.dim(0), (int)y.dim(1), eps, offset, mult, stream));
    return;
  }
  call(fn_->stream_norm_add(out.data, base.data, y.data, w.data, wf, (int)y.dim(0), (int)y.dim(1), eps, offset, mult, stream));
}

Tensor Kernels::stream_mix(const Tensor& states, const Tensor& coef, int n) {
  expect(states, "stream states", DType::F32);
  if (states.shape.size() < 2 || n <= 0 || n > states.dim(0)) throw EngineError("stream mix: " + std::to_string(n) + " of " + states.describe());
  const int cf = norm_weight(coef, "mixing weights", n);
  std::vector<int64_t> shape(states.shape.begin() + 1, states.shape.end());
  Tensor out = empty(shape, DType::F32);
  const int64_t numel = out.numel();
  call(fn_->stream_mix(out.data, states.data, numel, coef.data, cf, n, numel, stream));
  return out;
}

void Kernels::softcap(Tensor& x, float cap) {
  expect(x, "values to cap", dtype_);
  call(fn_->softcap(x.data, cap, x.numel(), stream));
}

Tensor Kernels::gemm_columns(const Tensor& act, int64_t first, const Tensor& w) {
  expect(act, "activation", dtype_);
  expect(w, "weight", dtype_);
  if (act.shape.size() != 2 || w.shape.size() != 2 || first < 0 || first + w.dim(1) > act.dim(1))
    throw EngineError("gemm: columns " + std::to_string(first) + ".. of " + act.describe() + " do not fit weight " + w.describe());
  const int vec = 16 / dtype_bytes(dtype_);
  if (first % vec || act.dim(1) % vec) throw EngineError("gemm: columns must start on a 16-byte boundary");
  const int64_t M = act.dim(0), K = w.dim(1), N = w.dim(0);
  Tensor out = empty({M, N});
  call(fn_->gemm(out.data, static_cast<const char*>(act.data) + (size_t)first * dtype_bytes(dtype_), w.data, (int)M, (int)N, (int)K, act.dim(1), N,
                 0, stream));
  return out;
}

Tensor Kernels::qkv_post_bias(const Tensor& qkv, int nq, int nkv, int d, const Tensor* k_cache, const Tensor* v_cache, int page_size,
                              const Tensor* slots, const Tensor& bias) {
  expect(qkv, "qkv", dtype_);
  const int64_t W = (int64_t)(nq + 2 * nkv) * d;
  if (qkv.shape.size() != 2 || qkv.dim(1) != W) throw EngineError("qkv_post: rows are " + qkv.describe() + ", expected width " + std::to_string(W));
  expect(bias, "qkv bias", dtype_, {W});
  const int64_t T = qkv.dim(0);
  Tensor q_out;
  if (nq) q_out = empty({T, nq, d});
  if (nkv) {
    if (!k_cache || !v_cache || !slots) throw EngineError("qkv_post: a store needs both caches and slots");
    if (k_cache->shape.size() != 4) throw EngineError("k cache is " + k_cache->describe());
    const int64_t pages = k_cache->dim(0);
    expect(*k_cache, "k cache", dtype_, {pages, nkv, page_size, d});
    expect(*v_cache, "v cache", dtype_, {pages, nkv, d, page_size});
    expect(*slots, "slots", DType::I32, {T});
  }
  call(fn_->qkv_post_bias(qkv.data, W, nq ? q_out.data : nullptr, nkv ? k_cache->data : nullptr, nkv ? v_cache->data : nullptr, nullptr, nullptr, 0,
                          nullptr, nullptr, 0, nullptr, nkv ? slots->data : nullptr, (int)T, nq, nkv, d, page_size, 0.f, bias.data, stream));
  return q_out;
}

void Kernels::paged_attention_capped(Tensor& out, const Tensor& q, const Tensor& k_cache, const Tensor& v_cache, const Tensor& block_table,
                                     const Tensor& cu_q, const Tensor& k_len, const Tensor& items, int mode, float scale, int window, int keep,
                                     float softcap, const Tensor* sinks, int max_k_len, int nseg, const Tensor* scratch, int block) {
  expect(q, "q", dtype_);
  expect(block_table, "block table", DType::I32);
  if (block < 0 || (block > 0 && (window != 0 || keep != 0))) throw EngineError("attention: blocks of positions exclude a window");
  if (q.shape.size() != 3 || k_cache.shape.size() != 4 || block_table.shape.size() != 2)
    throw EngineError("attention: q " + q.describe() + ", k cache " + k_cache.describe() + ", block table " + block_table.describe());
  const int64_t T = q.dim(0), nq = q.dim(1), d = q.dim(2), pages = k_cache.dim(0), nkv = k_cache.dim(1), P = k_cache.dim(2);
  const int64_t S = block_table.dim(0), W = block_table.dim(1);
  expect(k_cache, "k cache", dtype_, {pages, nkv, P, d});
  expect(v_cache, "v cache", dtype_, {pages, nkv, d, P});
  expect(cu_q, "cu_q", DType::I32, {S + 1});
  expect(k_len, "k_len", DType::I32, {S});
  expect(out, "attention output", dtype_, q.shape);
  if (items.shape.size() != 2 || items.dim(1) != 2) throw EngineError("attention: items are " + items.describe());
  expect(items, "items", DType::I32);
  if (mode != 0 && mode != 1) throw EngineError("attention with capped scores: mode " + std::to_string(mode));
  if (W * P < max_k_len)
    throw EngineError("attention: a block table of " + std::to_string(W) + " pages of " + std::to_string(P) + " does not cover " +
                      std::to_string(max_k_len) + " keys");
  int sf = 0;
  if (sinks) sf = norm_weight(*sinks, "attention sinks", nq);
  void* sp = nullptr;
  const int64_t n_items = items.dim(0);
  if (mode == 1) {
    if (nseg < (max_k_len + segment_keys_ - 1) / segment_keys_)
      throw EngineError("attention: " + std::to_string(nseg) + " segments do not cover " + std::to_string(max_k_len) + " keys");
    const int64_t need = attn_scratch_floats((int)n_items, (int)nq, (int)d, nseg);
    if (!scratch || scratch->dtype != DType::F32 || scratch->numel() < need)
      throw EngineError("attention: scratch of " + std::to_string(need) + " floats needed");
    sp = scratch->data;
  }
  if (block > 0) {
    call(fn_->paged_attention_blocked(out.data, q.data, k_cache.data, v_cache.data, block_table.data, (int)W, cu_q.data, k_len.data, items.data,
                                      (int)n_items, mode, nseg, sp, (int)T, (int)nq, (int)nkv, (int)d, (int)P, block, scale, softcap,
                                      sinks ? sinks->data : nullptr, sf, stream));
    return;
  }
  call(fn_->paged_attention_capped(out.data, q.data, k_cache.data, v_cache.data, block_table.data, (int)W, cu_q.data, k_len.data, items.data,
                                   (int)n_items, mode, nseg, sp, (int)T, (int)nq, (int)nkv, (int)d, (int)P, window, keep, scale, softcap,
                                   sinks ? sinks->data : nullptr, sf, stream));
}

// ------------------------------------------------------------------------------------- the delta rule
Tensor Kernels::delta_conv(const Tensor& x, const Tensor& taps, Tensor& state, int64_t tail_offset, const Tensor& token_seq, const Tensor& cu_q,
                           const Tensor& positions, const Tensor& slots, int64_t first_col, const Tensor* bias) {
  expect(x, "convolution input", dtype_);
  expect(taps, "convolution taps", dtype_);
  expect(state, "state", DType::F32);
  if (x.shape.size() != 2 || taps.shape.size() != 2 || state.shape.size() != 2 || first_col < 0 || first_col + taps.dim(0) > x.dim(1))
    throw EngineError("short convolution: input " + x.describe() + ", taps " + taps.describe() + ", state " + state.describe());
  const int64_t T = x.dim(0), C = taps.dim(0), K = taps.dim(1), S = slots.numel();
  expect(token_seq, "token sequences", DType::I32, {T});
  expect(positions, "positions", DType::I32, {T});
  expect(cu_q, "cu_q", DType::I32, {S + 1});
  expect(slots, "state slots", DType::I32, {S});
  Tensor y = empty({T, C}, DType::F32);
  const void* x0 = static_cast<const char*>(x.data) + (size_t)first_col * dtype_bytes(dtype_);
  if (bias) {
    expect(*bias, "convolution bias", dtype_, {C});
    call(fn_->delta_conv_bias(y.data, x0, x.dim(1), taps.data, bias->data, state.data, state.dim(1), tail_offset, token_seq.data, cu_q.data,
                              positions.data, slots.data, (int)T, (int)S, (int)C, (int)K, stream));
    return y;
  }
  call(fn_->delta_conv(y.data, x0, x.dim(1), taps.data, state.data, state.dim(1), tail_offset, token_seq.data, cu_q.data, positions.data,
                       slots.data, (int)T, (int)S, (int)C, (int)K, stream));
  return y;
}

void Kernels::delta_unit(Tensor& x, int64_t col0, int heads, int d, float eps, float scale) {
  expect(x, "unit norm input", DType::F32);
  if (x.shape.size() != 2) throw EngineError("unit norm input is " + x.describe());
  call(fn_->delta_unit(x.data, x.dim(1), (int)col0, (int)x.dim(0), heads, d, eps, scale, stream));
}

Tensor Kernels::delta_decay(const Tensor& a, const Tensor& dt_bias, const Tensor& A_log, int H, int d) {
  expect(a, "decay input", dtype_);
  if (a.shape.size() != 2 || a.dim(1) != (int64_t)H * d) throw EngineError("decay input is " + a.describe());
  const int wf = norm_weight(dt_bias, "dt_bias", (int64_t)H * d);
  if (norm_weight(A_log, "A_log", H) != wf) throw EngineError("decay: dt_bias and A_log must have one type");
  Tensor g = empty({a.dim(0), H, d}, DType::F32);
  call(fn_->delta_decay(g.data, a.data, dt_bias.data, A_log.data, wf, (int)a.dim(0), H, d, stream));
  return g;
}

Tensor Kernels::delta_prep(Tensor& x, int64_t q_col, int64_t k_col, int G, int H, int d, float unit_eps, float q_scale, const Tensor& a,
                           const Tensor& dt_bias, const Tensor& A_log) {
  expect(x, "delta rule input", DType::F32);
  expect(a, "decay input", dtype_);
  if (x.shape.size() != 2 || a.shape.size() != 2 || a.dim(0) != x.dim(0) || a.dim(1) != (int64_t)H * d ||
      std::max(q_col, k_col) + (int64_t)G * d > x.dim(1) || q_col < 0 || k_col < 0)
    throw EngineError("delta prep: input " + x.describe() + ", decay input " + a.describe());
  const int wf = norm_weight(dt_bias, "dt_bias", (int64_t)H * d);
  if (norm_weight(A_log, "A_log", H) != wf) throw EngineError("decay: dt_bias and A_log must have one type");
  Tensor g = empty({a.dim(0), H, d}, DType::F32);
  call(fn_->delta_prep(x.data, x.dim(1), (int)q_col, (int)k_col, (int)x.dim(0), G, H, d, unit_eps, q_scale, g.data, a.data, dt_bias.data,
                       A_log.data, wf, stream));
  return g;
}

Tensor Kernels::delta_rule(const Tensor& qkv, int q_col, int k_col, int v_col, const Tensor& decay, const Tensor& b, int64_t b_col, Tensor& state,
                           const Tensor& cu_q, const Tensor& positions, const Tensor& slots, int H, int G, int d, int dv) {
  expect(qkv, "delta rule input", DType::F32);
  expect(b, "beta input", dtype_);
  expect(state, "state", DType::F32);
  if (qkv.shape.size() != 2 || b.shape.size() != 2 || state.shape.size() != 2 || b.dim(0) != qkv.dim(0) || b_col + H > b.dim(1) ||
      std::max(q_col, k_col) + (int64_t)G * d > qkv.dim(1) || v_col + (int64_t)H * dv > qkv.dim(1))
    throw EngineError("delta rule: input " + qkv.describe() + ", beta " + b.describe() + ", state " + state.describe());
  const int64_t T = qkv.dim(0), S = slots.numel();
  expect(decay, "decay", DType::F32, {T, H, d});
  expect(positions, "positions", DType::I32, {T});
  expect(cu_q, "cu_q", DType::I32, {S + 1});
  expect(slots, "state slots", DType::I32, {S});
  Tensor out = empty({T, H, dv}, DType::F32);
  call(fn_->delta_rule(out.data, qkv.data, qkv.dim(1), q_col, k_col, v_col, decay.data,
                       static_cast<const char*>(b.data) + (size_t)b_col * dtype_bytes(dtype_), b.dim(1), state.data, state.dim(1), cu_q.data,
                       positions.data, slots.data, (int)S, H, G, d, dv, stream));
  return out;
}

Tensor Kernels::delta_out(const Tensor& o, const Tensor& gate, const Tensor& w, int H, int dv, float eps, int64_t width) {
  expect(o, "delta read-out", DType::F32);
  expect(gate, "gate", dtype_);
  if (o.shape.size() != 3 || o.dim(1) != H || o.dim(2) != dv || gate.shape.size() != 2 || gate.dim(0) != o.dim(0) || gate.dim(1) != (int64_t)H * dv)
    throw EngineError("delta read-out: " + o.describe() + " with gate " + gate.describe());
  const int wf = norm_weight(w, "read-out norm weight", dv);
  if (width < (int64_t)H * dv) throw EngineError("delta read-out: a row of " + std::to_string(width) + " does not hold the heads");
  Tensor y = empty({o.dim(0), width});
  call(fn_->delta_out(y.data, width, o.data, gate.data, gate.dim(1), w.data, wf, (int)o.dim(0), H, dv, eps, stream));
  return y;
}

// ---------------------------------------------------- scaled embedding, sums and means of branches
Tensor Kernels::embed_scaled(const Tensor& table, const Tensor& ids, float scale) {
  expect(table, "embedding table", dtype_);
  if (table.shape.size() != 2) throw EngineError("embedding table is " + table.describe());
  const int64_t V = table.dim(0), H = table.dim(1), T = ids.numel();
  expect(ids, "ids", DType::I32, {T});
  Tensor out = empty({T, H}, DType::F32);
  call(fn_->embed_scaled(out.data, table.data, ids.data, (int)T, (int)H, (int)V, scale, stream));
  return out;
}

void Kernels::stream_add(Tensor& s, const Tensor& a, const Tensor* b) {
  expect(s, "stream", DType::F32);
  for (const Tensor* t : {&a, b}) {
    if (!t) continue;
    if (t->dtype != DType::F32) expect(*t, "a branch's output", dtype_, s.shape);
    else expect(*t, "a branch's output", DType::F32, s.shape);
  }
  call(fn_->stream_add(s.data, s.data, a.data, a.dtype == DType::F32 ? 1 : 0, b ? b->data : nullptr, b && b->dtype == DType::F32 ? 1 : 0, s.numel(),
                       stream));
}

Tensor Kernels::stream_pair_norm(const Tensor& a, const Tensor& wa, const Tensor& b, const Tensor& wb, float eps, float ca, float cb) {
  expect(a, "first branch", dtype_);
  if (a.shape.size() != 2) throw EngineError("pair norm: the first branch is " + a.describe());
  expect(b, "second branch", dtype_, a.shape);
  const int wf = norm_weight(wa, "first branch's norm weight", a.dim(1));
  if (norm_weight(wb, "second branch's norm weight", a.dim(1)) != wf) throw EngineError("pair norm: the two weights must have one type");
  Tensor out = empty(a.shape, DType::F32);
  call(fn_->stream_pair_norm(out.data, a.data, wa.data, b.data, wb.data, wf, (int)a.dim(0), (int)a.dim(1), eps, ca, cb, stream));
  return out;
}

Tensor Kernels::qkv_post_angles(const Tensor& qkv, int nq, int nkv, int d, const Tensor* k_cache, const Tensor* v_cache, int page_size,
                                const Tensor& inv_freq, float mag, const Tensor& positions, const Tensor* slots) {
  expect(qkv, "qkv", dtype_);
  const int64_t W = (int64_t)(nq + 2 * nkv) * d;
  if (qkv.shape.size() != 2 || qkv.dim(1) != W) throw EngineError("qkv_post: rows are " + qkv.describe() + ", expected width " + std::to_string(W));
  const int64_t T = qkv.dim(0);
  expect(inv_freq, "rotation frequencies", DType::F32);
  if (inv_freq.shape.size() != 1 || inv_freq.dim(0) < 1 || 2 * inv_freq.dim(0) > d)
    throw EngineError("qkv_post: rotation frequencies are " + inv_freq.describe() + " for a head size of " + std::to_string(d));
  expect(positions, "positions", DType::I32, {T});
  Tensor q_out;
  if (nq) q_out = empty({T, nq, d});
  if (nkv) {
    if (!k_cache || !v_cache || !slots) throw EngineError("qkv_post: a store needs both caches and slots");
    if (k_cache->shape.size() != 4) throw EngineError("k cache is " + k_cache->describe());
    const int64_t pages = k_cache->dim(0);
    expect(*k_cache, "k cache", dtype_, {pages, nkv, page_size, d});
    expect(*v_cache, "v cache", dtype_, {pages, nkv, d, page_size});
    expect(*slots, "slots", DType::I32, {T});
  }
  call(fn_->qkv_post_angles(qkv.data, W, nq ? q_out.data : nullptr, nkv ? k_cache->data : nullptr, nkv ? v_cache->data : nullptr, inv_freq.data, mag,
                            (int)inv_freq.dim(0), positions.data, nkv ? slots->data : nullptr, (int)T, nq, nkv, d, page_size, stream));
  return q_out;
}

Tensor Kernels::qkv_post_norm_angles(const Tensor& qkv, int nq, int nkv, int d, const Tensor* k_cache, const Tensor* v_cache, int page_size,
                                     const Tensor* q_w, const Tensor* k_w, int norm_d, float eps, const Tensor& inv_freq, float mag,
                                     const Tensor& positions, const Tensor* slots) {
  expect(qkv, "qkv", dtype_);
  const int64_t W = (int64_t)(nq + 2 * nkv) * d;
  if (qkv.shape.size() != 2 || qkv.dim(1) < W) throw EngineError("qkv_post: rows are " + qkv.describe() + ", expected a width of at least " + std::to_string(W));
  const int64_t T = qkv.dim(0);
  expect(inv_freq, "rotation frequencies", DType::F32);
  if (norm_d < 1 || norm_d > d || inv_freq.shape.size() != 1 || inv_freq.dim(0) < 1 || 2 * inv_freq.dim(0) > norm_d)
    throw EngineError("qkv_post: rotation frequencies are " + inv_freq.describe() + " for a head norm over " + std::to_string(norm_d) + " of " +
                      std::to_string(d));
  int wf = 0;
  if (q_w) wf = norm_weight(*q_w, "q norm weight", norm_d);
  if (k_w) {
    const int wf2 = norm_weight(*k_w, "k norm weight", norm_d);
    if (q_w && wf2 != wf) throw EngineError("qkv_post: q and k norm weights must have the same type");
    wf = wf2;
  }
  expect(positions, "positions", DType::I32, {T});
  Tensor q_out;
  if (nq) q_out = empty({T, nq, d});
  if (nkv) {
    if (!k_cache || !v_cache || !slots) throw EngineError("qkv_post: a store needs both caches and slots");
    if (k_cache->shape.size() != 4) throw EngineError("k cache is " + k_cache->describe());
    const int64_t pages = k_cache->dim(0);
    expect(*k_cache, "k cache", dtype_, {pages, nkv, page_size, d});
    expect(*v_cache, "v cache", dtype_, {pages, nkv, d, page_size});
    expect(*slots, "slots", DType::I32, {T});
  }
  call(fn_->qkv_post_norm_angles(qkv.data, qkv.dim(1), nq ? q_out.data : nullptr, nkv ? k_cache->data : nullptr, nkv ? v_cache->data : nullptr,
                                 q_w ? q_w->data : nullptr, k_w ? k_w->data : nullptr, wf, norm_d, eps, inv_freq.data, mag, (int)inv_freq.dim(0),
                                 positions.data, nkv ? slots->data : nullptr, (int)T, nq, nkv, d, page_size, stream));
  return q_out;
}

void Kernels::gate_mul(Tensor& x, const Tensor& gate, int64_t gate_col, int kind) {
  expect(x, "gated rows", dtype_);
  expect(gate, "gate", dtype_);
  if (x.shape.size() != 2 || gate.shape.size() != 2 || gate.dim(0) != x.dim(0) || gate_col < 0 || gate_col + x.dim(1) > gate.dim(1))
    throw EngineError("gate: rows " + x.describe() + " with the gate's " + gate.describe() + " from column " + std::to_string(gate_col));
  call(fn_->gate_mul(x.data, x.dim(1), static_cast<const char*>(gate.data) + (size_t)gate_col * dtype_bytes(dtype_), gate.dim(1), (int)x.dim(0),
                     (int)x.dim(1), kind, stream));
}

// ------------------------------------------------------------------------- gated linear attention
Tensor Kernels::gla_decay(const Tensor& a, const Tensor& bias, int H, int d, float root) {
  expect(a, "decay input", dtype_);
  if (a.shape.size() != 2 || a.dim(1) != (int64_t)H * d) throw EngineError("linear attention decay: input is " + a.describe());
  const int wf = norm_weight(bias, "decay bias", (int64_t)H * d);
  Tensor g = empty({a.dim(0), H, d}, DType::F32);
  call(fn_->gla_decay(g.data, a.data, a.dim(1), bias.data, wf, (int)a.dim(0), H * d, root, stream));
  return g;
}

Tensor Kernels::gla_rule(const Tensor& x, int64_t q_col, int64_t k_col, int64_t v_col, const Tensor& decay, Tensor& state, const Tensor& cu_q,
                         const Tensor& positions, const Tensor& slots, int H, int d, int dv, float q_scale) {
  expect(x, "linear attention input", dtype_);
  expect(state, "state", DType::F32);
  if (x.shape.size() != 2 || state.shape.size() != 2 || q_col < 0 || k_col < 0 || v_col < 0 || std::max(q_col, k_col) + (int64_t)H * d > x.dim(1) ||
      v_col + (int64_t)H * dv > x.dim(1) || state.dim(1) < (int64_t)H * d * dv)
    throw EngineError("linear attention: input " + x.describe() + ", state " + state.describe());
  const int64_t T = x.dim(0), S = slots.numel();
  expect(decay, "decay", DType::F32, {T, H, d});
  expect(positions, "positions", DType::I32, {T});
  expect(cu_q, "cu_q", DType::I32, {S + 1});
  expect(slots, "state slots", DType::I32, {S});
  Tensor out = empty({T, H, dv}, DType::F32);
  call(fn_->gla_rule(out.data, x.data, x.dim(1), (int)q_col, (int)k_col, (int)v_col, decay.data, state.data, state.dim(1), cu_q.data, positions.data,
                     slots.data, (int)S, H, d, dv, q_scale, stream));
  return out;
}

Tensor Kernels::gated_head_norm(const Tensor& o, const Tensor& gate, int64_t gate_col, const Tensor& w, int H, int dv, float eps, int gate_kind,
                                int64_t width) {
  expect(o, "read-out", DType::F32);
  expect(gate, "gate", dtype_);
  if (o.shape.size() != 3 || o.dim(1) != H || o.dim(2) != dv || gate.shape.size() != 2 || gate.dim(0) != o.dim(0) || gate_col < 0 ||
      gate_col + (int64_t)H * dv > gate.dim(1))
    throw EngineError("gated head norm: " + o.describe() + " with gate " + gate.describe());
  const int wf = norm_weight(w, "read-out norm weight", dv);
  if (width < (int64_t)H * dv) throw EngineError("gated head norm: a row of " + std::to_string(width) + " does not hold the heads");
  Tensor y = empty({o.dim(0), width});
  call(fn_->gated_head_norm(y.data, width, o.data, static_cast<const char*>(gate.data) + (size_t)gate_col * dtype_bytes(dtype_), gate.dim(1), w.data, wf,
                            (int)o.dim(0), H, dv, eps, gate_kind, stream));
  return y;
}

// ---------------------------------------------------------------------------- state-space recurrence
Tensor Kernels::ssm_scan(const Tensor& xbc, int64_t b_col, int64_t c_col, const Tensor& proj, int64_t dt_col, const Tensor& dt_bias,
                         const Tensor& A_log, const Tensor& D, Tensor& state, const Tensor& cu_q, const Tensor& positions, const Tensor& slots, int H,
                         int G, int N, int P) {
  expect(xbc, "state-space input", DType::F32);
  expect(proj, "input projection", dtype_);
  expect(state, "state", DType::F32);
  if (xbc.shape.size() != 2 || proj.shape.size() != 2 || state.shape.size() != 2 || proj.dim(0) != xbc.dim(0) || dt_col < 0 ||
      dt_col + H > proj.dim(1) || b_col < (int64_t)H * P || c_col < 0 || std::max(b_col, c_col) + (int64_t)G * N > xbc.dim(1) ||
      state.dim(1) < (int64_t)H * P * N)
    throw EngineError("state-space scan: input " + xbc.describe() + ", projection " + proj.describe() + ", state " + state.describe());
  const int64_t T = xbc.dim(0), S = slots.numel();
  const int wf = norm_weight(dt_bias, "dt_bias", H);
  if (norm_weight(A_log, "A_log", H) != wf || norm_weight(D, "D", H) != wf) throw EngineError("state-space scan: dt_bias, A_log and D must have one type");
  expect(positions, "positions", DType::I32, {T});
  expect(cu_q, "cu_q", DType::I32, {S + 1});
  expect(slots, "state slots", DType::I32, {S});
  Tensor y = empty({T, H, P}, DType::F32);
  call(fn_->ssm_scan(y.data, xbc.data, xbc.dim(1), (int)b_col, (int)c_col, static_cast<const char*>(proj.data) + (size_t)dt_col * dtype_bytes(dtype_),
                     proj.dim(1), dt_bias.data, A_log.data, D.data, wf, state.data, state.dim(1), cu_q.data, positions.data, slots.data, (int)S, (int)T, H,
                     G, N, P, stream));
  return y;
}

Tensor Kernels::ssm_gate_norm(const Tensor& y, const Tensor& proj, int64_t z_col, const Tensor& w, int parts, float eps, int64_t width) {
  expect(y, "state-space read-out", DType::F32);
  expect(proj, "input projection", dtype_);
  if (y.shape.size() < 2 || proj.shape.size() != 2 || proj.dim(0) != y.dim(0)) throw EngineError("gated norm: " + y.describe() + " with " + proj.describe());
  const int64_t T = y.dim(0), inner = T ? y.numel() / T : 0;
  if (inner <= 0 || parts <= 0 || inner % parts || z_col < 0 || z_col + inner > proj.dim(1) || width < inner)
    throw EngineError("gated norm: rows of " + std::to_string(inner) + " in " + std::to_string(parts) + " parts");
  const int wf = norm_weight(w, "read-out norm weight", inner);
  Tensor out = empty({T, width});
  call(fn_->ssm_gate_norm(out.data, width, y.data, static_cast<const char*>(proj.data) + (size_t)z_col * dtype_bytes(dtype_), proj.dim(1), w.data, wf,
                          (int)T, (int)inner, parts, eps, stream));
  return out;
}

// ------------------------------------------------------------------------------ mixture of experts
Kernels::MoePlan Kernels::moe_route(const Tensor& h, const Tensor& router, int top, float weight_eps, int tile_rows, const Tensor* bias) {
  return moe_route_scored(h, router, top, weight_eps, tile_rows, bias, 0);
}

Kernels::MoePlan Kernels::moe_route_scored(const Tensor& h, const Tensor& router, int top, float weight_eps, int tile_rows, const Tensor* bias,
                                           int score_kind) {
  expect(h, "router input", dtype_);
  expect(router, "router weight", dtype_);
  if (h.shape.size() != 2 || router.shape.size() != 2 || router.dim(1) != h.dim(1) || top < 1 || top > router.dim(0))
    throw EngineError("router: input " + h.describe() + ", weight " + router.describe() + ", top " + std::to_string(top));
  const int64_t T = h.dim(0), E = router.dim(0);
  MoePlan p;
  if (tile_rows != 16 && tile_rows != 128) throw EngineError("router: tiles of " + std::to_string(tile_rows) + " rows");
  p.top = top;
  p.experts = (int)E;
  p.tile_rows = tile_rows;
  const int64_t tiles = fn_->moe_max_tiles((int)T, top, (int)E, tile_rows);
  p.idx = empty({T, top}, DType::I32);
  p.wts = empty({T, top}, DType::F32);
  p.row_pair = empty({tiles * tile_rows}, DType::I32);
  p.row_token = empty({tiles * tile_rows}, DType::I32);
  p.pair_row = empty({T * top}, DType::I32);
  p.tile_expert = empty({tiles}, DType::I32);
  p.expert_start = empty({E + 1}, DType::I32);
  Tensor logits = empty({T, E}, DType::F32);
  if (score_kind != 0) {
    const int bf = bias ? norm_weight(*bias, "router bias", E) : 0;
    call(fn_->moe_route_scored(p.idx.data, p.wts.data, logits.data, h.data, router.data, bias ? bias->data : nullptr, bf, (int)T, (int)h.dim(1), (int)E,
                               top, weight_eps, score_kind, stream));
  } else if (bias) {
    const int bf = norm_weight(*bias, "router bias", E);
    call(fn_->moe_route_bias(p.idx.data, p.wts.data, logits.data, h.data, router.data, bias->data, bf, (int)T, (int)h.dim(1), (int)E, top, weight_eps,
                             stream));
  } else {
    call(fn_->moe_route(p.idx.data, p.wts.data, logits.data, h.data, router.data, (int)T, (int)h.dim(1), (int)E, top, weight_eps, stream));
  }
  call(fn_->moe_plan(p.idx.data, p.row_pair.data, p.row_token.data, p.pair_row.data, p.tile_expert.data, p.expert_start.data, (int)T, top, (int)E,
                     tile_rows, stream));
  return p;
}

Tensor Kernels::moe_up(const Tensor& h, const Tensor& w_up, const MoePlan& plan) {
  expect(h, "experts' input", dtype_);
  expect(w_up, "experts' up weights", dtype_);
  if (h.shape.size() != 2 || w_up.shape.size() != 3 || w_up.dim(0) != plan.experts || w_up.dim(2) != h.dim(1) || plan.idx.dim(0) != h.dim(0) ||
      plan.tile_rows != 16)
    throw EngineError("experts (up): input " + h.describe() + ", weights " + w_up.describe());
  const int64_t T = h.dim(0), N = w_up.dim(1);
  Tensor act = empty({plan.row_pair.dim(0), N});
  call(fn_->moe_up(act.data, N, h.data, h.dim(1), w_up.data, plan.row_pair.data, plan.row_token.data, plan.tile_expert.data, (int)T, plan.top,
                   plan.experts, (int)N, (int)h.dim(1), stream));
  return act;
}

Tensor Kernels::moe_down(const Tensor& act, const Tensor& w_down, const MoePlan& plan) {
  expect(act, "experts' activations", dtype_);
  expect(w_down, "experts' down weights", dtype_);
  if (act.shape.size() != 2 || w_down.shape.size() != 3 || w_down.dim(0) != plan.experts || w_down.dim(2) != act.dim(1) ||
      act.dim(0) != plan.row_pair.dim(0) || plan.tile_rows != 16)
    throw EngineError("experts (down): activations " + act.describe() + ", weights " + w_down.describe());
  const int64_t W = w_down.dim(1), T = plan.idx.dim(0);
  Tensor y = empty({act.dim(0), W});
  call(fn_->moe_down(y.data, act.data, act.dim(1), w_down.data, plan.row_pair.data, plan.tile_expert.data, (int)T, plan.top, plan.experts, (int)W,
                     (int)act.dim(1), stream));
  return y;
}

Tensor Kernels::moe_up_plain(const Tensor& h, const Tensor& w, const MoePlan& plan) {
  expect(h, "experts' input", dtype_);
  expect(w, "experts' weights", dtype_);
  if (h.shape.size() != 2 || w.shape.size() != 3 || w.dim(0) != plan.experts || w.dim(2) != h.dim(1) || plan.idx.dim(0) != h.dim(0) ||
      plan.tile_rows != 16)
    throw EngineError("experts (up): input " + h.describe() + ", weights " + w.describe());
  const int64_t T = h.dim(0), N = w.dim(1);
  Tensor act = empty({plan.row_pair.dim(0), N});
  call(fn_->moe_up_plain(act.data, N, h.data, h.dim(1), w.data, plan.row_pair.data, plan.row_token.data, plan.tile_expert.data, (int)T, plan.top,
                         plan.experts, (int)N, (int)h.dim(1), stream));
  return act;
}

Tensor Kernels::moe_glu(const Tensor& gate_up, float limit, float slope, float shift) {
  expect(gate_up, "gate and up outputs", dtype_);
  if (gate_up.shape.size() != 2 || gate_up.dim(1) % 2) throw EngineError("gated activation: rows are " + gate_up.describe());
  const int64_t F = gate_up.dim(1) / 2;
  Tensor out = empty({gate_up.dim(0), F});
  call(fn_->moe_glu(out.data, gate_up.data, gate_up.dim(0), (int)F, limit, slope, shift, stream));
  return out;
}

Tensor Kernels::moe_glu_weighed(const Tensor& gate_up, float limit, float slope, float shift, const MoePlan& plan) {
  expect(gate_up, "gate and up outputs", dtype_);
  if (gate_up.shape.size() != 2 || gate_up.dim(1) % 2 || gate_up.dim(0) != plan.row_pair.dim(0))
    throw EngineError("gated activation: rows are " + gate_up.describe() + " for a plan of " + std::to_string(plan.row_pair.dim(0)) + " rows");
  const int64_t F = gate_up.dim(1) / 2;
  Tensor out = empty({gate_up.dim(0), F});
  call(fn_->moe_glu_weighed(out.data, gate_up.data, gate_up.dim(0), (int)F, limit, slope, shift, plan.row_pair.data, plan.wts.data, stream));
  return out;
}

Tensor Kernels::moe_sum_unweighed(const Tensor& y, const MoePlan& plan) {
  expect(y, "experts' outputs", dtype_);
  if (y.shape.size() != 2 || y.dim(0) != plan.row_pair.dim(0)) throw EngineError("experts (sum): outputs " + y.describe());
  const int64_t T = plan.idx.dim(0), W = y.dim(1);
  Tensor out = empty({T, W}, DType::F32);
  call(fn_->moe_combine(out.data, y.data, nullptr, plan.pair_row.data, (int)T, (int)W, plan.top, stream));
  return out;
}

// ----------------------------------------------------------------------- attention through a latent
Tensor Kernels::norm_columns(const Tensor& x, int64_t col, int64_t n, const Tensor& w, float eps, int64_t width) {
  expect(x, "norm input", dtype_);
  if (x.shape.size() != 2 || col < 0 || n < 1 || col + n > x.dim(1) || width < n) throw EngineError("norm of columns " + std::to_string(col) + ".. of " + x.describe());
  const int wf = norm_weight(w, "norm weight", n);
  Tensor out = empty({x.dim(0), width});
  call(fn_->norm_columns(out.data, width, x.data, x.dim(1), (int)col, (int)n, w.data, wf, eps, (int)x.dim(0), stream));
  return out;
}

void Kernels::gemm_heads(Tensor& out, int64_t out_stride, const Tensor& x, int64_t x_col, int64_t x_stride, const Tensor& w) {
  expect(out, "heads' outputs", dtype_);
  expect(x, "heads' inputs", dtype_);
  expect(w, "heads' weights", dtype_);
  if (out.shape.size() != 2 || x.shape.size() != 2 || w.shape.size() != 3 || out.dim(0) != x.dim(0) || x_col < 0 || out_stride < 0 || x_stride < 0)
    throw EngineError("product a head: outputs " + out.describe() + ", inputs " + x.describe() + ", weights " + w.describe());
  const int64_t H = w.dim(0), N = w.dim(1), K = w.dim(2);
  const int vec = 16 / dtype_bytes(dtype_);
  if (x_col + (H - 1) * x_stride + K > x.dim(1) || (H - 1) * out_stride + N > out.dim(1) || x_col % vec)
    throw EngineError("product a head: " + std::to_string(H) + " heads of " + std::to_string(K) + " -> " + std::to_string(N) + " do not fit inputs " +
                      x.describe() + " from column " + std::to_string(x_col) + " or outputs " + out.describe());
  call(fn_->gemm_heads(out.data, out.dim(1), out_stride, static_cast<const char*>(x.data) + (size_t)x_col * dtype_bytes(dtype_), x.dim(1), x_stride, w.data,
                       (int)x.dim(0), (int)H, (int)N, (int)K, stream));
}

void Kernels::latent_post(const Tensor& proj, int64_t kv_col, const Tensor& q, int64_t q_stride, int64_t q_first, Tensor& q_abs, const Tensor* k_cache,
                          const Tensor* v_cache, int page_size, const Tensor* norm_w, float eps, const Tensor& inv_freq, bool neighbours,
                          const Tensor& positions, const Tensor* slots, int r, int dr) {
  expect(q, "queries", dtype_);
  expect(q_abs, "queries as the cache meets them", dtype_);
  if (q.shape.size() != 2 || q_abs.shape.size() != 3 || q_abs.dim(0) != q.dim(0) || r < 1 || dr < 2 || q_abs.dim(2) < r + dr)
    throw EngineError("latent attention: queries " + q.describe() + " to " + q_abs.describe());
  const int64_t T = q.dim(0), H = q_abs.dim(1), D = q_abs.dim(2);
  if (q_first < 0 || q_stride < q_first + dr || (H - 1) * q_stride + q_first + dr > q.dim(1))
    throw EngineError("latent attention: " + std::to_string(H) + " heads do not fit queries " + q.describe());
  expect(inv_freq, "rotation frequencies", DType::F32, {(int64_t)dr / 2});
  expect(positions, "positions", DType::I32, {T});
  const bool store = kv_col >= 0;
  int wf = 0;
  if (store) {
    expect(proj, "latent projection", dtype_);
    if (proj.shape.size() != 2 || proj.dim(0) != T || kv_col + r + dr > proj.dim(1)) throw EngineError("latent attention: the projection is " + proj.describe());
    if (!k_cache || !v_cache || !slots || !norm_w) throw EngineError("latent attention: a store needs both caches, slots and the norm's weight");
    if (k_cache->shape.size() != 4) throw EngineError("k cache is " + k_cache->describe());
    const int64_t pages = k_cache->dim(0);
    expect(*k_cache, "k cache", dtype_, {pages, 1, page_size, D});
    expect(*v_cache, "v cache", dtype_, {pages, 1, D, page_size});
    expect(*slots, "slots", DType::I32, {T});
    wf = norm_weight(*norm_w, "latent norm weight", r);
  }
  call(fn_->latent_post(store ? static_cast<const char*>(proj.data) + (size_t)kv_col * dtype_bytes(dtype_) : nullptr, store ? proj.dim(1) : 0, q.data,
                        q.dim(1), q_stride, (int)q_first, q_abs.data, store ? k_cache->data : nullptr, store ? v_cache->data : nullptr,
                        store ? norm_w->data : nullptr, wf, eps, inv_freq.data, neighbours ? 1 : 0, positions.data, store ? slots->data : nullptr, (int)T,
                        (int)H, r, dr, (int)D, page_size, stream));
}

Tensor Kernels::qkv_post_norm_angles_paired(const Tensor& qkv, int nq, int nkv, int d, const Tensor* k_cache, const Tensor* v_cache, int page_size,
                                            const Tensor* q_w, const Tensor* k_w, int norm_d, float eps, const Tensor& inv_freq, float mag,
                                            bool neighbours, const Tensor& positions, const Tensor* slots) {
  expect(qkv, "qkv", dtype_);
  const int64_t W = (int64_t)(nq + 2 * nkv) * d;
  if (qkv.shape.size() != 2 || qkv.dim(1) < W) throw EngineError("qkv_post: rows are " + qkv.describe() + ", expected a width of at least " + std::to_string(W));
  const int64_t T = qkv.dim(0);
  expect(inv_freq, "rotation frequencies", DType::F32);
  if (norm_d < 1 || norm_d > d || inv_freq.shape.size() != 1 || inv_freq.dim(0) < 1 || 2 * inv_freq.dim(0) > norm_d)
    throw EngineError("qkv_post: rotation frequencies are " + inv_freq.describe() + " for a head of " + std::to_string(norm_d) + " in " + std::to_string(d));
  int wf = 0;
  if (q_w) wf = norm_weight(*q_w, "q norm weight", norm_d);
  if (k_w) {
    const int wf2 = norm_weight(*k_w, "k norm weight", norm_d);
    if (q_w && wf2 != wf) throw EngineError("qkv_post: q and k norm weights must have the same type");
    wf = wf2;
  }
  expect(positions, "positions", DType::I32, {T});
  Tensor q_out;
  if (nq) q_out = empty({T, nq, d});
  if (nkv) {
    if (!k_cache || !v_cache || !slots) throw EngineError("qkv_post: a store needs both caches and slots");
    if (k_cache->shape.size() != 4) throw EngineError("k cache is " + k_cache->describe());
    const int64_t pages = k_cache->dim(0);
    expect(*k_cache, "k cache", dtype_, {pages, nkv, page_size, d});
    expect(*v_cache, "v cache", dtype_, {pages, nkv, d, page_size});
    expect(*slots, "slots", DType::I32, {T});
  }
  call(fn_->qkv_post_norm_angles_paired(qkv.data, qkv.dim(1), nq ? q_out.data : nullptr, nkv ? k_cache->data : nullptr, nkv ? v_cache->data : nullptr,
                                        q_w ? q_w->data : nullptr, k_w ? k_w->data : nullptr, wf, norm_d, eps, inv_freq.data, mag, (int)inv_freq.dim(0),
                                        neighbours ? 1 : 0, positions.data, nkv ? slots->data : nullptr, (int)T, nq, nkv, d, page_size, stream));
  return q_out;
}

Tensor Kernels::linear_rule(const Tensor& x, int64_t q_col, int64_t k_col, int64_t v_col, const Tensor& head_decay, Tensor& state,
                            const Tensor& cu_q, const Tensor& positions, const Tensor& slots, int H, int d, int dv, float q_scale) {
  expect(x, "linear attention input", dtype_);
  expect(state, "state", DType::F32);
  if (x.shape.size() != 2 || state.shape.size() != 2 || q_col < 0 || k_col < 0 || v_col < 0 || std::max(q_col, k_col) + (int64_t)H * d > x.dim(1) ||
      v_col + (int64_t)H * dv > x.dim(1) || state.dim(1) < (int64_t)H * d * dv)
    throw EngineError("linear attention: input " + x.describe() + ", state " + state.describe());
  const int64_t T = x.dim(0), S = slots.numel();
  expect(head_decay, "the heads' decays", DType::F32, {(int64_t)H});
  expect(positions, "positions", DType::I32, {T});
  expect(cu_q, "cu_q", DType::I32, {S + 1});
  expect(slots, "state slots", DType::I32, {S});
  Tensor out = empty({T, H, dv}, DType::F32);
  call(fn_->linear_rule(out.data, x.data, x.dim(1), (int)q_col, (int)k_col, (int)v_col, head_decay.data, state.data, state.dim(1),
                        cu_q.data, positions.data, slots.data, (int)S, H, d, dv, q_scale, stream));
  return out;
}

Tensor Kernels::gated_row_norm(const Tensor& o, const Tensor& gate, int64_t gate_col, const Tensor& w, float eps, int gate_kind, int64_t width) {
  expect(o, "read-out", DType::F32);
  expect(gate, "gate", dtype_);
  const int64_t T = o.shape.empty() ? 0 : o.dim(0), n = T ? o.numel() / T : 0;
  if (o.shape.size() < 2 || gate.shape.size() != 2 || gate.dim(0) != T || gate_col < 0 || gate_col + n > gate.dim(1) || width < n || n < 1)
    throw EngineError("gated row norm: " + o.describe() + " with gate " + gate.describe());
  const int wf = norm_weight(w, "read-out norm weight", n);
  Tensor y = empty({T, width});
  call(fn_->gated_row_norm(y.data, width, o.data, static_cast<const char*>(gate.data) + (size_t)gate_col * dtype_bytes(dtype_), gate.dim(1), w.data, wf,
                           (int)T, (int)n, eps, gate_kind, stream));
  return y;
}

void Kernels::silu_columns(Tensor& x, int64_t first, int64_t count) {
  expect(x, "rows to activate", dtype_);
  if (x.shape.size() != 2 || first < 0 || count < 1 || first + count > x.dim(1)) throw EngineError("silu of columns " + std::to_string(first) + ".. of " + x.describe());
  call(fn_->silu_columns(x.data, x.dim(1), first, (int)count, (int)x.dim(0), stream));
}

Tensor Kernels::side_gate(const Tensor& gate, const Tensor& table, const Tensor& ids, int64_t first, int64_t n) {
  expect(gate, "side gate", dtype_);
  expect(table, "side table", dtype_);
  if (gate.shape.size() != 2 || table.shape.size() != 2 || first < 0 || n < 1 || n > gate.dim(1) || first + n > table.dim(1))
    throw EngineError("token side input: gate " + gate.describe() + ", table " + table.describe());
  expect(ids, "ids", DType::I32, {gate.dim(0)});
  Tensor out = empty(gate.shape);
  call(fn_->side_gate(out.data, gate.dim(1), gate.data, gate.dim(1), table.data, table.dim(1), ids.data, (int)first, (int)n, (int)gate.dim(0), stream));
  return out;
}

Tensor Kernels::moe_sum(const Tensor& y, const MoePlan& plan, const Tensor* extra) {
  expect(y, "experts' outputs", dtype_);
  if (y.shape.size() != 2 || y.dim(0) != plan.row_pair.dim(0)) throw EngineError("experts (sum): outputs " + y.describe());
  const int64_t T = plan.idx.dim(0), W = y.dim(1);
  Tensor out = empty({T, W}, DType::F32);
  if (extra) {
    expect(*extra, "the shared expert's output", dtype_, {T, W});
    call(fn_->moe_combine_add(out.data, y.data, plan.wts.data, plan.pair_row.data, extra->data, (int)T, (int)W, plan.top, stream));
    return out;
  }
  call(fn_->moe_combine(out.data, y.data, plan.wts.data, plan.pair_row.data, (int)T, (int)W, plan.top, stream));
  return out;
}

void Kernels::relu_square(Tensor& x) {
  expect(x, "activations", dtype_);
  call(fn_->moe_relu_square(x.data, x.numel(), stream));
}

bool Kernels::gemm_grouped_takes(int64_t K) const { return K % (dtype_ == DType::BF16 ? 64 : 32) == 0; }

Tensor Kernels::gemm_grouped(const Tensor& act, const Tensor& w, const Tensor& block_weights) {
  expect(act, "activation", dtype_);
  expect(w, "weights", dtype_);
  if (act.shape.size() != 2 || w.shape.size() != 3 || act.dim(1) != w.dim(2) || act.dim(0) % 128 || !gemm_grouped_takes(act.dim(1)))
    throw EngineError("grouped gemm: activation " + act.describe() + ", weights " + w.describe());
  expect(block_weights, "the blocks' matrices", DType::I32, {act.dim(0) / 128});
  Tensor out = empty({act.dim(0), w.dim(1)});
  call(fn_->gemm_grouped(out.data, act.data, w.data, (int)act.dim(0), (int)w.dim(1), (int)w.dim(2), act.dim(1), w.dim(1), block_weights.data,
                         w.dim(1) * w.dim(2), stream));
  return out;
}

int Kernels::sample_scratch_words(int rows) const { return fn_->sample_scratch_words(rows); }

void Kernels::sample(Tensor& out, const Tensor& logits, const Tensor* temps, const Tensor* unis, Tensor& scratch) {
  expect(logits, "logits", dtype_);
  if (logits.shape.size() != 2) throw EngineError("logits are " + logits.describe());
  const int64_t R = logits.dim(0), V = logits.dim(1);
  expect(out, "sampled ids", DType::I32, {R});
  if (temps) {
    if (!unis) throw EngineError("sampling at a temperature needs uniform numbers");
    expect(*temps, "temperatures", DType::F32, {R});
    expect(*unis, "uniform numbers", DType::F32, {R});
  }
  if (scratch.dtype != DType::I32 || scratch.numel() < sample_scratch_words((int)R))
    throw EngineError("sampling: scratch of " + std::to_string(sample_scratch_words((int)R)) + " words needed");
  call(fn_->sample(out.data, logits.data, temps ? temps->data : nullptr, temps ? unis->data : nullptr, scratch.data, (int)R,
                   (int)V, V, stream));
}

}  // namespace vosti
